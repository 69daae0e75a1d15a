"""Parity of the image backward kernels (intra_image_bwd of the C ABI) against the gradients of the
fp32 dense-mask oracle.  The reference has no backward kernels; its FLUX training differentiates
the dense-mask attention the oracle restates (experiments/flux/intra_processor.py:138-142).
Tolerances as in test_backward_gpu.py; the grid keys' rows of Gather 0 are written by two passes
(query patches, then the text queries' share added in bf16), which stays inside the same bounds."""
import pytest
import torch

import oracle
from intra_amd import _lib, intra_image_attn, intra_image_attn_bwd, intra_image_attn_func
from test_backward_gpu import compare

pytestmark = pytest.mark.gpu
DEV = "cuda"


def make(B, S, H, Hkv, seed):
    g = torch.Generator(device="cpu").manual_seed(seed)
    mk = lambda h: torch.randn(B, S, h, 128, generator=g, dtype=torch.float32).to(torch.bfloat16).to(DEV)
    return mk(H), mk(Hkv), mk(Hkv), mk(H)


@pytest.mark.parametrize("pattern", ["scatter", "gather0"])
@pytest.mark.parametrize("B,H,Hkv", [(1, 4, 4), (2, 2, 1), (1, 8, 2)])
def test_flux_1024_grads(pattern, B, H, Hkv):
    S = 512 + 64 * 64
    q, k, v, dout = make(B, S, H, Hkv, seed=H)
    with torch.no_grad():
        out, lse = intra_image_attn(q, k, v, pattern, 64, return_lse=True)
        got = intra_image_attn_bwd(q, k, v, out, lse, dout, pattern, 64)
    mask = oracle.mask_rows(f"image/{pattern}", S, device=DEV, width=64)
    compare(got, oracle.masked_attention_grads(q, k, v, dout, mask), f"image/{pattern} H={H}/{Hkv}")


@pytest.mark.parametrize("pattern", ["scatter", "gather0"])
def test_flux_2048_grads(pattern):
    S = 512 + 128 * 128
    q, k, v, dout = make(1, S, 2, 2, seed=7)
    with torch.no_grad():
        out, lse = intra_image_attn(q, k, v, pattern, 128, softmax_scale=0.07, return_lse=True)
        got = intra_image_attn_bwd(q, k, v, out, lse, dout, pattern, 128, softmax_scale=0.07)
    mask = oracle.mask_rows(f"image/{pattern}", S, device=DEV, width=128)
    compare(got, oracle.masked_attention_grads(q, k, v, dout, mask, softmax_scale=0.07), f"image/{pattern} 2048")


@pytest.mark.parametrize("width,text_len,H,Hkv", [(24, 72, 4, 4), (40, 8, 8, 2), (16, 200, 2, 1), (32, 96, 4, 1), (48, 64, 3, 3)])
@pytest.mark.parametrize("pattern,pid", [("scatter", 0), ("gather0", 4)])
def test_other_widths_and_text_lengths_through_the_c_abi(width, text_len, H, Hkv, pattern, pid):
    lib = _lib.load()
    B, S = 2, text_len + width * width
    q, k, v, dout = make(B, S, H, Hkv, seed=width)
    out = torch.empty_like(q)
    lse = torch.empty(B, H, S, dtype=torch.float32, device=DEV)
    stream = torch.cuda.current_stream().cuda_stream
    rc = lib.intra_image_fwd_lse(q.data_ptr(), k.data_ptr(), v.data_ptr(), out.data_ptr(), B, S, H, Hkv,
                                 _lib.strides3(q), _lib.strides3(k), _lib.strides3(v), _lib.strides3(out),
                                 pid, width, text_len, 128 ** -0.5, stream, lse.data_ptr(), _lib.strides3(lse))
    assert rc == 0, _lib.last_error()
    n = lib.intra_image_bwd_workspace(B, S, H, Hkv, pid, width, text_len)
    assert n >= B * H * S
    work = torch.full((n + 64,), float("nan"), dtype=torch.float32, device=DEV)
    dq, dk, dv = (torch.full_like(t, float("nan")) for t in (q, k, v))
    rc = lib.intra_image_bwd(q.data_ptr(), k.data_ptr(), v.data_ptr(), out.data_ptr(), lse.data_ptr(), dout.data_ptr(),
                             dq.data_ptr(), dk.data_ptr(), dv.data_ptr(), work.data_ptr(), B, S, H, Hkv,
                             _lib.strides3(q), _lib.strides3(k), _lib.strides3(v), _lib.strides3(out), _lib.strides3(dout),
                             _lib.strides3(dq), _lib.strides3(dk), _lib.strides3(dv), _lib.strides3(lse),
                             pid, width, text_len, 128 ** -0.5, stream)
    assert rc == 0, _lib.last_error()
    torch.cuda.synchronize()
    assert bool(torch.isnan(work[n:]).all()), "wrote past the workspace"
    mask = oracle.mask_rows(f"image/{pattern}", S, device=DEV, width=width, text_len=text_len)
    compare((dq, dk, dv), oracle.masked_attention_grads(q, k, v, dout, mask), f"image/{pattern} W={width} T={text_len}")


def test_autograd_function_and_reruns():
    S = 512 + 64 * 64
    q, k, v, dout = make(1, S, 2, 2, seed=11)
    q, k, v = (t.requires_grad_(True) for t in (q, k, v))
    out = intra_image_attn_func(q, k, v, "gather0", 64)
    out.backward(dout)
    mask = oracle.mask_rows("image/gather0", S, device=DEV, width=64)
    compare((q.grad, k.grad, v.grad), oracle.masked_attention_grads(q, k, v, dout, mask), "autograd gather0")
    with torch.no_grad():
        o2, lse = intra_image_attn(q, k, v, "gather0", 64, return_lse=True)
        again = intra_image_attn_bwd(q, k, v, o2, lse, dout, "gather0", 64)
    for a, b in zip(again, (q.grad, k.grad, v.grad)):
        assert torch.equal(a, b), "not bit-identical between calls"
