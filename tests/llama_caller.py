"""Test helper: a decoder-style caller of the LLM kernels, forward and backward.

The reference drives its model-level patterns from a transformers attention function that looks up
a per-layer configuration (experiments/llm/llama_intra.py:177-270).  This helper gives the tests
such a caller, built for this repository: a schedule string is expanded into one immutable
`LayerPlan` per decoder layer, and `sparse_attention` - an attention-interface function in the
transformers sense, (module, query, key, value, ...) -> (output, None) on (B, H, S, D) tensors -
runs the plan it finds on the module through intra_llm_attn / intra_llm_attn_func.  It is not part
of the product package; tests/test_llama_caller_gpu.py uses it to exercise the block Scatter and
window-with-sinks kernels and their backward pass the way a model would.
"""
import dataclasses
import itertools

import torch
import torch.nn.functional as F

from intra_amd import intra_llm_attn, intra_llm_attn_func


@dataclasses.dataclass(frozen=True)
class LayerPlan:
    kind: str            # "scatter" | "window" | "dense"
    group_num: int = 1
    block: int = 1       # tokens per Scatter block; 1 = token-level Scatter
    offset: int = 0      # stripe offset of a block Scatter layer
    window: int = 0
    n_sink: int = 0

    def kernel_call(self):
        """(pattern name, keyword arguments) of intra_llm_attn for this layer, or None for dense."""
        if self.kind == "window":
            return "window_sink", dict(window=self.window, n_sink=self.n_sink)
        if self.kind != "scatter":
            return None
        if self.block == 1 and self.n_sink == 0:
            return "scatter", dict(group_num=self.group_num)
        if self.block % 64:
            raise ValueError(f"block Scatter kernels need blocks of a multiple of 64 tokens (got {self.block})")
        if self.n_sink > self.block:
            raise ValueError(f"at most one block of sinks (n_sink={self.n_sink}, block={self.block})")
        return "block_scatter", dict(group_num=self.group_num, block=self.block, offset=self.offset, n_sink=self.n_sink)


_KINDS = {"S": "scatter", "W": "window", "D": "dense"}


def plan_layers(n_layers, schedule, group_num, window, n_sink=0, blocks=(1,), stripe_offsets=1):
    """One LayerPlan per layer: the letters of `schedule` (S, W, D) repeat over the layers; the k-th
    Scatter layer takes blocks[k % len(blocks)] and stripe offset k % stripe_offsets."""
    kinds = itertools.cycle(_KINDS[c] for c in schedule.upper())
    plans, k = [], 0
    for _ in range(n_layers):
        kind = next(kinds)
        if kind == "scatter":
            block, offset = blocks[k % len(blocks)], k % max(stripe_offsets, 1)
            if offset and block % 256:
                raise ValueError(f"a stripe offset needs blocks of a multiple of 256 tokens for the backward kernels (got {block})")
            plans.append(LayerPlan("scatter", group_num=group_num, block=block, offset=offset, n_sink=n_sink))
            k += 1
        elif kind == "window":
            plans.append(LayerPlan("window", window=window, n_sink=n_sink))
        else:
            plans.append(LayerPlan("dense"))
    return plans


def attach_plans(attention_modules, plans):
    for module, plan in zip(attention_modules, plans):
        module.intra_plan = plan
        module.intra_force_dense = False


def force_dense(attention_modules, flag):
    """Every layer dense (the teacher of a distillation run) or back to its plan."""
    for module in attention_modules:
        module.intra_force_dense = bool(flag)


def _sdpa(query, key, value, scaling, **kw):
    return F.scaled_dot_product_attention(query, key, value, scale=scaling, enable_gqa=key.shape[1] != query.shape[1], **kw)


def sparse_attention(module, query, key, value, attention_mask=None, scaling=None, dropout=0.0, **kwargs):
    """query (B, Hq, S, D), key / value (B, Hkv, S, D) -> (output (B, S, Hq, D), None)."""
    if scaling is None:
        scaling = getattr(module, "scaling", None) or query.shape[-1] ** -0.5
    plan = getattr(module, "intra_plan", None)
    call = None if plan is None or getattr(module, "intra_force_dense", False) else plan.kernel_call()
    if query.shape[2] == 1 and key.shape[2] > 1:  # decode: one query against the whole cache
        mask = None if attention_mask is None else attention_mask[..., :key.shape[2]]
        out = _sdpa(query, key, value, scaling, attn_mask=mask)
    elif call is None:
        out = _sdpa(query, key, value, scaling, is_causal=True)
    else:
        pattern, kw = call
        q, k, v = (t.transpose(1, 2) for t in (query, key, value))  # (B, S, H, D) views: the kernels take strides
        if torch.is_grad_enabled() and (q.requires_grad or k.requires_grad or v.requires_grad):
            return intra_llm_attn_func(q, k, v, pattern, softmax_scale=scaling, **kw).contiguous(), None
        with torch.no_grad():
            return intra_llm_attn(q, k, v, pattern, softmax_scale=scaling, **kw).contiguous(), None
    return out.transpose(1, 2).contiguous(), None
