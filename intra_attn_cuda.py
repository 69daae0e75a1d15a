"""Stand-in for the reference's compiled extension module `intra_attn_cuda` on MI355X.

The reference's Python layer (`intra_attn/interface.py:10,43-44,64-65`) and its FLUX processor
(`experiments/flux/intra_processor.py:25-29`) import a pybind11 module of this name and call
`fwd_llm` / `fwd` with the 16 positional arguments of `mha_fwd_llm` / `mha_fwd`
(`csrc/flash_attn/flash_api.cpp:355-371,556-574,1766-1770`).  With this file on the import path
those files run unchanged: the two functions take the same arguments, reject what the reference's
build rejects (dropout, ALiBi, softcap, returned softmax; `flash_api.cpp:105,129,338,474`) with
RuntimeError like TORCH_CHECK does, launch the HIP kernels through the C ABI of libintra_hip.so
and return `[out, softmax_lse, None, None]`.  `softmax_lse` is (batch, heads, seqlen) fp32 indexed
by token position (the reference indexes it by in-group row; its callers use only `[0]`).
"""
import torch

from intra_amd import _lib

_C = _lib.load()


def _fail(msg):
    raise RuntimeError(msg)


def _common(q, k, v, out_, alibi_slopes_, p_dropout, softcap, return_softmax):
    for name, x in (("q", q), ("k", k), ("v", v)):
        if not x.is_cuda:
            _fail(f"{name} must be on the GPU")
        if x.stride(-1) != 1:
            _fail("Input tensor must have contiguous last dimension")
    if q.dtype != torch.bfloat16:
        _fail("this build only supports bfloat16")
    if k.dtype != q.dtype:
        _fail("query and key must have the same dtype")
    if v.dtype != q.dtype:
        _fail("query and value must have the same dtype")
    if q.dim() != 4 or k.dim() != 4 or v.shape != k.shape or k.shape[:2] != q.shape[:2] or k.shape[3] != q.shape[3]:
        _fail("q must have shape (batch, seqlen, heads, head_size) and k, v (batch, seqlen, heads_k, head_size)")
    if q.shape[0] <= 0:
        _fail("batch size must be positive")
    if q.shape[3] != 128:
        _fail("this build only supports head dimension 128")
    if q.shape[2] % k.shape[2]:
        _fail("Number of heads in key/value must divide number of heads in query")
    if alibi_slopes_ is not None:
        _fail("This flash attention build does not support alibi.")
    if p_dropout != 0.0:
        _fail("This flash attention build does not support dropout.")
    if softcap > 0.0:
        _fail("This flash attention build does not support softcap.")
    if return_softmax:
        _fail("return_softmax is only supported when p_dropout > 0.0")
    if out_ is None:
        return torch.empty(q.shape, dtype=q.dtype, device=q.device)
    if out_.dtype != q.dtype:
        _fail("Output must have the same dtype as inputs")
    if not out_.is_cuda or out_.shape != q.shape:
        _fail("out must be on the GPU and have the shape of q")
    if out_.stride(-1) != 1:
        _fail("Output tensor must have contiguous last dimension")
    return out_


def _launch(fn, q, k, v, out, pattern, a0, a1, softmax_scale):
    if any(t.data_ptr() % 16 or any(s % 8 for s in t.stride()[:3]) for t in (q, k, v, out)):
        _fail("q, k, v and out rows must be 16-byte aligned")
    B, S, H, _ = q.shape
    lse = torch.empty(B, H, S, dtype=torch.float32, device=q.device)
    with torch.cuda.device(q.device):
        rc = fn(q.data_ptr(), k.data_ptr(), v.data_ptr(), out.data_ptr(), B, S, H, k.shape[2], _lib.strides3(q),
                _lib.strides3(k), _lib.strides3(v), _lib.strides3(out), int(pattern), int(a0), int(a1),
                float(softmax_scale), torch.cuda.current_stream(q.device).cuda_stream, lse.data_ptr(), _lib.strides3(lse))
    if rc != _lib.INTRA_OK:
        _fail(_lib.last_error())
    return [out, lse, None, None]


def fwd_llm(q, k, v, out_, alibi_slopes_, p_dropout, softmax_scale, is_causal, window_size_left, window_size_right,
            softcap, return_softmax, gen_, mask, group_num, window):
    """mha_fwd_llm: mask 0 Scatter, 1 Gather 1 (group_num groups), 4 window of `window` keys."""
    out = _common(q, k, v, out_, alibi_slopes_, p_dropout, softcap, return_softmax)
    if mask == 1 and q.shape[1] % (group_num * group_num):
        _fail("Gather 1 needs a sequence length that is a multiple of group_num * group_num")  # flash_api.cpp:709
    return _launch(_C.intra_llm_fwd_lse, q, k, v, out, mask, group_num, window, softmax_scale)


def fwd(q, k, v, out_, alibi_slopes_, p_dropout, softmax_scale, is_causal, window_size_left, window_size_right,
        softcap, return_softmax, gen_, mask, width, length):
    """mha_fwd (image): mask 0 Scatter, 4 Gather 0 on 512 text tokens + a width x width grid."""
    out = _common(q, k, v, out_, alibi_slopes_, p_dropout, softcap, return_softmax)
    return _launch(_C.intra_image_fwd_lse, q, k, v, out, mask, width, 512, softmax_scale)
