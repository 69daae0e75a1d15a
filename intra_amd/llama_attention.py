"""INTRA attention for LLaMA / Qwen style decoders on the HIP kernels, forward and backward.

Counterpart of the reference's model integration (experiments/llm/llama_intra.py:177-221,
232-270): the same attention-interface function and per-layer configuration, with the Scatter and
window branches - which the reference runs through gathered SDPA or FlexAttention - on
intra_llm_attn / intra_llm_attn_func.  The branches that are not sparse (single-token decode,
dense layers, the dense teacher toggle) stay on torch SDPA exactly as in the reference.

    install_intra_llama(model, num_groups=2, window=575, n_sink=64, scatter_blocks=(256,),
                        layer_pattern="SWWWWWWW", scatter_stripe=True, scatter_n_offsets=2)

stamps `module._intra` on every `layer.self_attn`; `intra_attention_forward` is the function to
register as the model's attention implementation (with transformers installed:
`AttentionInterface.register("intra", intra_attention_forward)`, done by `register()`).
"""
import torch
import torch.nn.functional as F

from .interface import intra_llm_attn, intra_llm_attn_func

HEAD_DIM = 128  # the kernels' head dimension


def _sparse(pattern, query, key, value, scaling, **kw):
    """One sparse layer on (B, H, S, D) tensors; returns (B, H, S, D) like the branches of the
    reference (llama_intra.py:124-168)."""
    q, k, v = (t.transpose(1, 2) for t in (query, key, value))  # views: the kernels take strides
    if torch.is_grad_enabled() and any(t.requires_grad for t in (q, k, v)):
        out = intra_llm_attn_func(q, k, v, pattern, softmax_scale=scaling, **kw)
    else:
        with torch.no_grad():
            out = intra_llm_attn(q, k, v, pattern, softmax_scale=scaling, **kw)
    return out.transpose(1, 2)


def _dense_causal(query, key, value, scaling):
    return F.scaled_dot_product_attention(query, key, value, is_causal=True, scale=scaling,
                                          enable_gqa=key.shape[1] != query.shape[1])


def intra_attention_forward(module, query, key, value, attention_mask=None, scaling=None, dropout=0.0, **kwargs):
    """Attention-interface function: query (B, Hq, S, D), key / value (B, Hkv, S, D); returns
    (output (B, S, Hq, D), None).  Routing by the dict `module._intra` as in the reference
    (llama_intra.py:177-221): 'S' block Scatter (groups, block, stripe offset, sinks), 'W' causal
    window (with sinks), 'D' or no config: dense causal; a single query against a longer cache
    (decode) attends densely to the whole cache."""
    cfg = getattr(module, "_intra", None)
    if scaling is None:
        scaling = getattr(module, "scaling", None) or query.shape[-1] ** -0.5
    decode = query.shape[2] == 1 and key.shape[2] > 1
    if decode:
        mask = None if attention_mask is None else attention_mask[:, :, :, :key.shape[2]]
        out = F.scaled_dot_product_attention(query, key, value, attn_mask=mask, scale=scaling, is_causal=False,
                                             enable_gqa=key.shape[1] != query.shape[1])
    elif cfg is None or cfg.get("dense_debug", False) or cfg["kind"] not in ("S", "W"):
        out = _dense_causal(query, key, value, scaling)
    elif query.shape[-1] != HEAD_DIM or query.dtype != torch.bfloat16:
        raise ValueError("the INTRA kernels need bfloat16 and head_dim 128")
    elif cfg["kind"] == "S":
        block = cfg.get("scatter_block", 1)
        if block == 1 and not cfg.get("n_sink", 0):
            # token-level Scatter (the reference's default scatter_blocks=(1,)): the plain Scatter kernel
            out = _sparse("scatter", query, key, value, scaling, group_num=cfg["num_groups"])
            return out.transpose(1, 2).contiguous(), None
        if block % 64:
            raise ValueError(f"block Scatter kernels need blocks of a multiple of 64 tokens (got {block})")
        if cfg.get("n_sink", 0) > block:
            raise ValueError(f"block Scatter kernels keep at most one block of sinks (n_sink={cfg['n_sink']}, block={block})")
        out = _sparse("block_scatter", query, key, value, scaling, group_num=cfg["num_groups"], block=block,
                      offset=cfg.get("scatter_offset", 0), n_sink=cfg.get("n_sink", 0))
    else:
        out = _sparse("window_sink", query, key, value, scaling, window=cfg["window"], n_sink=cfg.get("n_sink", 0))
    return out.transpose(1, 2).contiguous(), None


def _decoder_layers(model):
    """LLaMA / Qwen causal-LM wrappers keep the decoder under `.model`; a bare decoder has `.layers`."""
    inner = getattr(model, "model", model)
    return inner.layers


def install_intra_llama(model, num_groups=8, window=512, dense_debug=False, n_sink=0, scatter_blocks=(1,),
                        layer_pattern="SSWW", scatter_stripe=False, scatter_n_offsets=0):
    """Give every decoder layer its branch: the letters of `layer_pattern` ('S' Scatter, 'W' window,
    'D' dense) are cycled over the layers, `scatter_blocks` over the Scatter layers, and with
    `scatter_stripe` the s-th Scatter layer gets offset s % n_offsets (n_offsets =
    scatter_n_offsets or num_groups).  Same meaning as llama_intra.py:232-270; the arguments that
    choose between the reference's SDPA / FlexAttention code paths have no counterpart.  Returns
    the numbers of (Scatter, window, dense) layers."""
    layers = _decoder_layers(model)
    blocks = list(scatter_blocks) or [1]
    letters = [c for c in layer_pattern.upper() if c in "SWD"] or ["S", "S", "W", "W"]
    n_off = max(scatter_n_offsets, 0) or num_groups
    count = {"S": 0, "W": 0, "D": 0}
    for index, layer in enumerate(layers):
        kind = letters[index % len(letters)]
        block = blocks[count["S"] % len(blocks)] if kind == "S" else 1
        offset = count["S"] % n_off if (kind == "S" and scatter_stripe) else 0
        if kind == "S" and offset and block % 256:
            raise ValueError(f"a stripe offset needs blocks of a multiple of 256 tokens for the backward kernels (got {block})")
        layer.self_attn._intra = dict(num_groups=num_groups, window=window, layer_idx=index, kind=kind,
                                      dense_debug=dense_debug, n_sink=n_sink, scatter_block=block,
                                      scatter_offset=offset)
        count[kind] += 1
    return count["S"], count["W"], count["D"]


def set_dense_debug(model, flag):
    """Teacher / student toggle of the reference (llama_intra.py:273-278): every layer dense."""
    for layer in _decoder_layers(model):
        cfg = getattr(layer.self_attn, "_intra", None)
        if cfg is not None:
            cfg["dense_debug"] = bool(flag)


def register(name="intra"):
    """Register intra_attention_forward with transformers under `name` (llama_intra.py:224-230)."""
    try:
        from transformers import AttentionInterface
        AttentionInterface.register(name, intra_attention_forward)
    except ImportError:
        from transformers.modeling_utils import ALL_ATTENTION_FUNCTIONS
        ALL_ATTENTION_FUNCTIONS[name] = intra_attention_forward
