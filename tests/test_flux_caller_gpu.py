"""The kernels seen from their one real caller: a FLUX-style joint-attention layer.

Counterpart of the reference's experiments/flux/intra_processor.py:54-169 without model weights:
random projections, per-head RMS norm of q and k, text tokens concatenated in front of the image
tokens along the sequence axis of (B, H, S, D) tensors, the attention called on
`x.transpose(1, 2)` views of those tensors (head stride S*128, token stride 128) with an explicit
softmax scale, and the pattern schedule Scatter, Scatter, Gather 0, Gather 0 over the layers
(intra_processor.py:162-169).  Every layer is run twice on identical inputs: through the kernels
and through the masked-SDPA fallback branch of the same processor (intra_processor.py:138-142),
whose mask comes from the oracle here.

Tolerance: the attention outputs are bf16; 1.6e-2 max-abs as for the other parity tests.  The
layer outputs go through one more bf16 projection, checked at 4e-2.
"""
import math

import pytest
import torch
import torch.nn.functional as F

import oracle
from intra_amd import intra_image_attn, intra_image_attn_func

pytestmark = pytest.mark.gpu
DEV = "cuda"
TEXT = 512


class JointAttention(torch.nn.Module):
    """Stand-in for diffusers' Attention module of a FLUX double-stream block (random weights)."""

    def __init__(self, dim, heads, seed):
        super().__init__()
        g = torch.Generator().manual_seed(seed)
        self.heads = heads

        def lin():
            layer = torch.nn.Linear(dim, dim, bias=True)
            with torch.no_grad():
                layer.weight.copy_(torch.randn(dim, dim, generator=g) / math.sqrt(dim))
                layer.bias.copy_(torch.randn(dim, generator=g) * 0.02)
            return layer

        self.to_q, self.to_k, self.to_v = lin(), lin(), lin()
        self.add_q_proj, self.add_k_proj, self.add_v_proj = lin(), lin(), lin()
        self.to_out, self.to_add_out = lin(), lin()
        self.norm_w = torch.nn.Parameter(1.0 + 0.1 * torch.randn(4, dim // heads, generator=g))

    def rms(self, x, i):
        xf = x.float()
        return (xf * torch.rsqrt(xf.pow(2).mean(-1, keepdim=True) + 1e-6) * self.norm_w[i].float()).to(x.dtype)


def joint_layer(attn, hidden, text, pattern, width, use_kernel):
    B = hidden.shape[0]
    H, D = attn.heads, hidden.shape[-1] // attn.heads

    def heads(x):
        return x.view(B, -1, H, D).transpose(1, 2)  # (B, H, S, D) view of (B, S, H*D)

    q, k, v = heads(attn.to_q(hidden)), heads(attn.to_k(hidden)), heads(attn.to_v(hidden))
    q, k = attn.rms(q, 0), attn.rms(k, 1)
    tq, tk, tv = heads(attn.add_q_proj(text)), heads(attn.add_k_proj(text)), heads(attn.add_v_proj(text))
    tq, tk = attn.rms(tq, 2), attn.rms(tk, 3)
    q, k, v = (torch.cat([a, b], dim=2) for a, b in ((tq, q), (tk, k), (tv, v)))  # text first
    scale = math.sqrt(1 / D)
    if use_kernel:
        qv, kv, vv = q.transpose(1, 2), k.transpose(1, 2), v.transpose(1, 2)
        assert qv.stride(2) == q.shape[2] * D and qv.stride(1) == D  # (B, H, S, D) storage
        attend = intra_image_attn_func if torch.is_grad_enabled() else intra_image_attn  # training / inference
        a = attend(qv, kv, vv, pattern=pattern, width=width, softmax_scale=scale).transpose(1, 2)
    else:
        mask = oracle.mask_rows(f"image/{pattern}", q.shape[2], device=q.device, width=width)
        a = F.scaled_dot_product_attention(q.float(), k.float(), v.float(), attn_mask=mask, scale=scale).to(q.dtype)
    flat = a.transpose(1, 2).reshape(B, -1, H * D)
    return attn.to_add_out(flat[:, :TEXT]), attn.to_out(flat[:, TEXT:]), a


@pytest.mark.parametrize("width,heads,batch", [(64, 4, 2), (128, 2, 1)])
def test_flux_style_layers_kernel_equals_masked_sdpa(width, heads, batch):
    dim = heads * 128
    g = torch.Generator().manual_seed(100 + width)
    hidden = torch.randn(batch, width * width, dim, generator=g).to(torch.bfloat16).to(DEV)
    text = torch.randn(batch, TEXT, dim, generator=g).to(torch.bfloat16).to(DEV)
    with torch.no_grad():
        for idx in range(4):
            pattern = "gather0" if idx % 4 in (2, 3) else "scatter"
            attn = JointAttention(dim, heads, seed=idx).to(DEV).to(torch.bfloat16)
            t_k, h_k, a_k = joint_layer(attn, hidden, text, pattern, width, use_kernel=True)
            t_r, h_r, a_r = joint_layer(attn, hidden, text, pattern, width, use_kernel=False)
            assert bool(torch.isfinite(a_k).all())
            err = (a_k.float() - a_r.float()).abs().max().item()
            assert err <= 1.6e-2, f"layer {idx} ({pattern}): attention max|err|={err:.3e}"
            for got, ref in ((t_k, t_r), (h_k, h_r)):
                e2 = (got.float() - ref.float()).abs().max().item()
                assert e2 <= 4e-2, f"layer {idx} ({pattern}): layer output max|err|={e2:.3e}"
            # feed the kernel path's result forward, as the model would (residual + normalise)
            hidden = F.layer_norm((hidden.float() + h_k.float()), (dim,)).to(torch.bfloat16)
            text = F.layer_norm((text.float() + t_k.float()), (dim,)).to(torch.bfloat16)


@pytest.mark.parametrize("pattern", ["scatter", "gather0"])
def test_flux_style_layer_trains_through_the_kernels(pattern):
    """The branch of the processor that needs gradients (intra_processor.py:138-142, masked SDPA in
    the reference) on the backward kernels: gradients of the layer's weights and inputs against
    the masked-SDPA path, for the distillation-style loss the reference trains with (a mean squared
    error on the layer outputs).  Tolerance: relative l2 error 3e-2 per tensor (the SDPA path runs
    its attention in fp32, the kernels in bf16 with fp32 accumulation)."""
    width, heads, batch = 64, 2, 1
    dim = heads * 128
    g = torch.Generator().manual_seed(7)
    hidden0 = torch.randn(batch, width * width, dim, generator=g).to(torch.bfloat16).to(DEV)
    text0 = torch.randn(batch, TEXT, dim, generator=g).to(torch.bfloat16).to(DEV)
    attn = JointAttention(dim, heads, seed=3).to(DEV).to(torch.bfloat16)
    results = []
    for use_kernel in (True, False):
        hidden, text = hidden0.clone().requires_grad_(True), text0.clone().requires_grad_(True)
        attn.zero_grad(set_to_none=True)
        t_out, h_out, _ = joint_layer(attn, hidden, text, pattern, width, use_kernel=use_kernel)
        (t_out.float().square().mean() + h_out.float().square().mean()).backward()
        results.append([hidden.grad, text.grad] + [p.grad.clone() for p in attn.parameters()])
    for i, (a, b) in enumerate(zip(*results)):
        rel = ((a.float() - b.float()).norm() / b.float().norm()).item()
        assert torch.isfinite(a).all() and rel <= 3e-2, (i, rel)
