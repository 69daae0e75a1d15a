"""Python entry points of the MI355X INTRA kernels: the reference's two forward calls, and a
backward pass with autograd wrappers that the reference does not have.

Same surface as the reference's intra_attn/interface.py:12-66: `intra_llm_attn` and
`intra_image_attn` take q, k, v of shape (batch, seqlen, heads, 128) in bfloat16 on the GPU and
return the attention output in q's layout; k/v may have fewer heads than q (GQA) as long as they
divide the query heads.  Pattern names, arguments, defaults and exception types are the
reference's.  The work is done by libintra_hip.so through its C ABI (include/intra_hip.h); there
is no fallback path, a missing library is an ImportError.
"""
import contextlib

import torch

from . import _lib

_C = _lib.load()

LLM_PATTERNS = {"scatter": 0, "gather1": 1, "window": 4}
IMAGE_PATTERNS = {"scatter": 0, "gather0": 4}
# Patterns of the reference's LLaMA / Qwen integration that its kernels do not have
# (experiments/llm/llama_intra.py:57-72,93-110); they run through intra_llm_fwd_ex.
EXTRA_LLM_PATTERNS = {"block_scatter": 8, "window_sink": 9}
TEXT_LEN = 512


def _aligned(x):
    if x.data_ptr() % 16:
        return False
    if x.is_contiguous():  # the usual case, and the cheap test: rows of 128 bf16 are 256 bytes
        return True
    st = x.stride()
    return st[-1] == 1 and st[0] % 8 == 0 and st[1] % 8 == 0 and st[2] % 8 == 0


# INTRA_SOFTMAX_* of include/intra_hip.h ("fast" is the older name of "folded")
SOFTMAX_MODES = {"auto": 0, "exact": 1, "folded": 2, "scaled": 3, "fast": 2}
_SOFTMAX_NAMES = {0: "auto", 1: "exact", 2: "folded", 3: "scaled"}


def set_softmax_mode(mode):
    """Softmax arithmetic that calls without a `softmax=` argument get, process-wide.  "exact" scales
    the fp32 scores after the first product and keeps a running reference like the reference
    (csrc/flash_attn/src/softmax.h:65-91); "scaled" scales them the same way but keeps no running
    maximum and recomputes, exactly, the queries whose weight sum leaves the safe exponent range;
    "folded" multiplies the scale into the bf16 queries instead (about 2 % faster, error grows with
    the magnitude of q and k); "auto" (default) is scaled up to four times the default
    softmax_scale, exact beyond.  Meant for experiments: pass `softmax=` per call otherwise."""
    if _C.intra_set_softmax_mode(SOFTMAX_MODES[mode]) != _lib.INTRA_OK:
        raise RuntimeError(f"intra_hip: {_lib.last_error()}")


def get_softmax_mode():
    return _SOFTMAX_NAMES[_C.intra_get_softmax_mode()]


_BF16 = torch.bfloat16


def _check(q, k, v, forward_call=True):
    # reference: intra_attn/interface.py:17-23 (same conditions, same exception types and texts);
    # written flat because this runs in front of kernels that take a few tens of microseconds
    qs, ks, vs = q.shape, k.shape, v.shape
    if not (q.is_cuda and k.is_cuda and v.is_cuda and q.dtype is _BF16 and k.dtype is _BF16 and v.dtype is _BF16
            and qs[-1] == 128 and ks[-1] == 128 and vs[-1] == 128):
        raise ValueError("INTRA kernels need CUDA bfloat16 tensors with head_dim 128")
    # the plain forward calls record no graph (intra_llm_attn_func / intra_image_attn_func do)
    if forward_call and (q.requires_grad or k.requires_grad or v.requires_grad) and torch.is_grad_enabled():
        raise RuntimeError("INTRA kernels are forward-only; call them under torch.no_grad()")
    if len(qs) != 4 or len(ks) != 4 or len(vs) != 4:
        raise ValueError("q, k, v must be (batch, seqlen, heads, 128)")
    if ks != vs or ks[0] != qs[0] or ks[1] != qs[1] or qs[2] % ks[2]:
        raise RuntimeError(f"q {tuple(qs)} and k/v {tuple(ks)}/{tuple(vs)} do not "
                           "match: need equal batch and seqlen, and query heads divisible by kv heads")
    # The kernels honour arbitrary batch/token/head strides; only rows that are not contiguous
    # or not 16-byte aligned are copied.
    return (q if _aligned(q) else q.contiguous(), k if _aligned(k) else k.contiguous(),
            v if _aligned(v) else v.contiguous())


def _scale(q, softmax_scale):
    return q.shape[-1] ** -0.5 if softmax_scale is None else softmax_scale


def _stream_on(device):
    """(context that makes `device` current, handle of its current stream).  Switching devices is
    only paid for when the tensors live on another GPU than the current one."""
    index = device.index
    if index == torch.cuda.current_device():
        return _NO_GUARD, _raw_stream(index)
    return torch.cuda.device(device), _raw_stream(index)


_NO_GUARD = contextlib.nullcontext()
# handle of the current stream of a device without building a torch.cuda.Stream object per call
_raw_stream = getattr(torch._C, "_cuda_getCurrentRawStream", None) or (lambda i: torch.cuda.current_stream(i).cuda_stream)


def _launch(fn, fn_lse, q, k, v, pattern_id, arg0, arg1, scale, return_lse=False):
    out = torch.empty_like(q)
    if not _aligned(out):
        out = torch.empty(q.shape, dtype=q.dtype, device=q.device)
    B, S, H, _ = q.shape
    guard, stream = _stream_on(q.device)
    with guard:
        if return_lse:
            lse = torch.empty(B, H, S, dtype=torch.float32, device=q.device)
            rc = fn_lse(q.data_ptr(), k.data_ptr(), v.data_ptr(), out.data_ptr(), B, S, H, k.shape[2],
                        _lib.strides3(q), _lib.strides3(k), _lib.strides3(v), _lib.strides3(out),
                        pattern_id, arg0, arg1, float(scale), stream, lse.data_ptr(), _lib.strides3(lse))
        else:
            rc = fn(q.data_ptr(), k.data_ptr(), v.data_ptr(), out.data_ptr(), B, S, H, k.shape[2],
                    _lib.strides3(q), _lib.strides3(k), _lib.strides3(v), _lib.strides3(out),
                    pattern_id, arg0, arg1, float(scale), stream)
    if rc != _lib.INTRA_OK:
        raise RuntimeError(f"intra_hip: {_lib.last_error()}")
    return (out, lse) if return_lse else out


def _launch_ex(q, k, v, pattern_id, group_num, window, block, offset, n_sink, scale, return_lse, softmax=None):
    flags = 0 if softmax is None else SOFTMAX_MODES[softmax]
    out = torch.empty_like(q)
    if not _aligned(out):
        out = torch.empty(q.shape, dtype=q.dtype, device=q.device)
    B, S, H, _ = q.shape
    lse = torch.empty(B, H, S, dtype=torch.float32, device=q.device) if return_lse else None
    guard, stream = _stream_on(q.device)
    with guard:
        rc = _C.intra_llm_fwd_ex(q.data_ptr(), k.data_ptr(), v.data_ptr(), out.data_ptr(), B, S, H, k.shape[2],
                                 _lib.strides3(q), _lib.strides3(k), _lib.strides3(v), _lib.strides3(out),
                                 pattern_id, group_num, window, block, offset, n_sink, float(scale), stream,
                                 lse.data_ptr() if return_lse else None,
                                 _lib.strides3(lse) if return_lse else None, flags)
    if rc != _lib.INTRA_OK:
        raise RuntimeError(f"intra_hip: {_lib.last_error()}")
    return (out, lse) if return_lse else out


def _launch_image_ex(q, k, v, pattern_id, width, text_len, scale, return_lse, softmax):
    out = torch.empty_like(q)
    if not _aligned(out):
        out = torch.empty(q.shape, dtype=q.dtype, device=q.device)
    B, S, H, _ = q.shape
    lse = torch.empty(B, H, S, dtype=torch.float32, device=q.device) if return_lse else None
    guard, stream = _stream_on(q.device)
    with guard:
        rc = _C.intra_image_fwd_ex(q.data_ptr(), k.data_ptr(), v.data_ptr(), out.data_ptr(), B, S, H, k.shape[2],
                                   _lib.strides3(q), _lib.strides3(k), _lib.strides3(v), _lib.strides3(out),
                                   pattern_id, width, text_len, float(scale), stream,
                                   lse.data_ptr() if return_lse else None,
                                   _lib.strides3(lse) if return_lse else None, SOFTMAX_MODES[softmax])
    if rc != _lib.INTRA_OK:
        raise RuntimeError(f"intra_hip: {_lib.last_error()}")
    return (out, lse) if return_lse else out


def intra_llm_attn(q, k, v, pattern="scatter", group_num=8, window=576, softmax_scale=None, return_lse=False,
                   block=256, offset=0, n_sink=0, softmax=None):
    """Causal prefill attention for language models.

    pattern="scatter": token i attends to earlier tokens j with j % group_num == i % group_num.
    pattern="gather1": groups are segments of group_num tokens, segment s in group s % group_num.
    pattern="window":  each 64-query block attends to itself and the preceding window - 64 tokens.

    Any seqlen works for scatter and window; gather1 keeps the reference's contract of
    group_num=8 and seqlen % 64 == 0 (intra_attn/interface.py:41-42).

    Not in the reference's signature:
    return_lse=True also returns the (batch, heads, seqlen) fp32 log-sum-exp of the scaled scores
    of every query, as `(out, lse)`.
    softmax="exact" | "scaled" | "folded" names the kernel's softmax arithmetic for this call (see
    set_softmax_mode); None takes the process default.
    pattern="block_scatter": tokens form blocks of `block` (a multiple of 64), block b in group
        b % group_num; a query block qb reads the earlier blocks of group (qb + offset) % group_num
        and itself where it is in that group or offset != 0, plus the first n_sink tokens.
    pattern="window_sink": query i sees keys j <= i with i - j < window or j < n_sink.
    These two are the Scatter and window layers of the reference's model integration
    (experiments/llm/llama_intra.py; its LLaMA setting is group_num=2, block=256, offset 0 / 1,
    window=575, n_sink=64).
    """
    q, k, v = _check(q, k, v)
    if pattern == "gather1" and (group_num != 8 or q.shape[1] % (group_num * group_num)):
        raise ValueError(f"gather1 needs group_num=8 and seqlen % 64 == 0, got G={group_num}, S={q.shape[1]}")
    if pattern in EXTRA_LLM_PATTERNS or softmax is not None:
        ids = EXTRA_LLM_PATTERNS if pattern in EXTRA_LLM_PATTERNS else LLM_PATTERNS
        return _launch_ex(q, k, v, ids[pattern], int(group_num), int(window), int(block),
                          int(offset), int(n_sink), _scale(q, softmax_scale), return_lse, softmax)
    return _launch(_C.intra_llm_fwd, _C.intra_llm_fwd_lse, q, k, v, LLM_PATTERNS[pattern], int(group_num),
                   int(window), _scale(q, softmax_scale), return_lse)


def intra_llm_attn_bwd(q, k, v, out, lse, dout, pattern="scatter", group_num=8, window=576, softmax_scale=None,
                       block=256, offset=0, n_sink=0):
    """Gradients (dq, dk, dv) of intra_llm_attn for any of its patterns, given the forward results
    `out`, `lse` (return_lse=True) and the gradient `dout` of `out`; the pattern arguments are those
    of the forward call.  block_scatter with offset != 0 needs block % 256 == 0.  The reference has
    no backward kernels (its training runs differentiate masked SDPA,
    experiments/llm/llama_intra.py:26)."""
    q, k, v = _check(q, k, v, forward_call=False)
    ids = dict(LLM_PATTERNS, **EXTRA_LLM_PATTERNS)
    if pattern not in ids:
        raise ValueError(f"unknown pattern {pattern!r}")
    if pattern == "gather1" and (group_num != 8 or q.shape[1] % (group_num * group_num)):
        raise ValueError(f"gather1 needs group_num=8 and seqlen % 64 == 0, got G={group_num}, S={q.shape[1]}")
    B, S, H, _ = q.shape
    args = (ids[pattern], int(group_num), int(window), int(block), int(offset), int(n_sink))
    n_work = _C.intra_llm_bwd_workspace(B, S, H, k.shape[2], *args)
    return _bwd_call(_C.intra_llm_bwd, n_work, q, k, v, out, lse, dout, args, _scale(q, softmax_scale))


class _LlmAttnFunction(torch.autograd.Function):
    @staticmethod
    def forward(ctx, q, k, v, pattern, group_num, window, softmax_scale, block, offset, n_sink):
        out, lse = intra_llm_attn(q, k, v, pattern, group_num, window, softmax_scale, return_lse=True, block=block,
                                  offset=offset, n_sink=n_sink)
        ctx.save_for_backward(q, k, v, out, lse)
        ctx.args = (pattern, group_num, window, softmax_scale, block, offset, n_sink)
        return out

    @staticmethod
    def backward(ctx, dout):
        q, k, v, out, lse = ctx.saved_tensors
        dq, dk, dv = intra_llm_attn_bwd(q, k, v, out, lse, dout, *ctx.args)
        return (dq, dk, dv) + (None,) * 7


def intra_llm_attn_func(q, k, v, pattern="scatter", group_num=8, window=576, softmax_scale=None, block=256, offset=0,
                        n_sink=0):
    """intra_llm_attn as a differentiable function (torch.autograd): forward and backward kernels."""
    return _LlmAttnFunction.apply(q, k, v, pattern, group_num, window, softmax_scale, block, offset, n_sink)


def _bwd_call(fn, n_work, q, k, v, out, lse, dout, args, scale):
    """Shared part of the backward wrappers: checks, allocation of the results and the workspace, the call."""
    fix = lambda t: t if (t.stride(-1) == 1 and _aligned(t)) else t.contiguous()
    out, dout = fix(out), fix(dout)
    if out.shape != q.shape or dout.shape != q.shape or out.dtype != q.dtype or dout.dtype != q.dtype:
        raise ValueError("out and dout must have the shape and dtype of q")
    B, S, H, _ = q.shape
    if lse.shape != (B, H, S) or lse.dtype != torch.float32:
        raise ValueError("lse must be the (batch, heads, seqlen) fp32 tensor of the forward call")
    if n_work < 0:
        raise RuntimeError(f"intra_hip: {_lib.last_error()}")
    dq, dk, dv = (torch.empty(t.shape, dtype=t.dtype, device=t.device) for t in (q, k, v))
    work = torch.empty(n_work, dtype=torch.float32, device=q.device)
    guard, stream = _stream_on(q.device)
    with guard:
        rc = fn(q.data_ptr(), k.data_ptr(), v.data_ptr(), out.data_ptr(), lse.data_ptr(), dout.data_ptr(),
                dq.data_ptr(), dk.data_ptr(), dv.data_ptr(), work.data_ptr(), B, S, H, k.shape[2],
                _lib.strides3(q), _lib.strides3(k), _lib.strides3(v), _lib.strides3(out), _lib.strides3(dout),
                _lib.strides3(dq), _lib.strides3(dk), _lib.strides3(dv), _lib.strides3(lse), *args, float(scale), stream)
    if rc != _lib.INTRA_OK:
        raise RuntimeError(f"intra_hip: {_lib.last_error()}")
    return dq, dk, dv


def intra_image_attn_bwd(q, k, v, out, lse, dout, pattern="scatter", width=64, softmax_scale=None):
    """Gradients (dq, dk, dv) of intra_image_attn, given the forward results `out`, `lse`
    (return_lse=True) and the gradient `dout` of `out`.  The reference has no backward kernels (its
    FLUX training differentiates masked SDPA, experiments/flux/intra_processor.py:138-142)."""
    q, k, v = _check(q, k, v, forward_call=False)
    if width not in (64, 128):
        raise ValueError("image kernels are compiled for width 64 and 128")
    if q.shape[1] != TEXT_LEN + width * width:
        raise ValueError(f"expected {TEXT_LEN} text + {width}x{width} image tokens, got {q.shape[1]}")
    B, S, H, _ = q.shape
    args = (IMAGE_PATTERNS[pattern], int(width), TEXT_LEN)
    n_work = _C.intra_image_bwd_workspace(B, S, H, k.shape[2], *args)
    return _bwd_call(_C.intra_image_bwd, n_work, q, k, v, out, lse, dout, args, _scale(q, softmax_scale))


class _ImageAttnFunction(torch.autograd.Function):
    @staticmethod
    def forward(ctx, q, k, v, pattern, width, softmax_scale):
        out, lse = intra_image_attn(q, k, v, pattern, width, softmax_scale, return_lse=True)
        ctx.save_for_backward(q, k, v, out, lse)
        ctx.args = (pattern, width, softmax_scale)
        return out

    @staticmethod
    def backward(ctx, dout):
        q, k, v, out, lse = ctx.saved_tensors
        return intra_image_attn_bwd(q, k, v, out, lse, dout, *ctx.args) + (None,) * 3


def intra_image_attn_func(q, k, v, pattern="scatter", width=64, softmax_scale=None):
    """intra_image_attn as a differentiable function (torch.autograd): forward and backward kernels."""
    return _ImageAttnFunction.apply(q, k, v, pattern, width, softmax_scale)


def intra_image_attn(q, k, v, pattern="scatter", width=64, softmax_scale=None, return_lse=False, softmax=None):
    """Bidirectional attention for FLUX-style sequences: 512 text tokens followed by a
    width x width grid of image tokens.

    pattern="scatter": 8 groups, image token (r, c) in group (r % 2) * 4 + c % 4; text chunks of
                       64 tokens ride with groups 0..7; all text keys are always visible.
    pattern="gather0": each 8 x 8 image patch attends to a 16 x 16 window around it plus all text.

    Width 64 (1024 x 1024 FLUX images) and 128 (2048 x 2048), as in the reference
    (intra_attn/interface.py:59-63).  return_lse and softmax as for intra_llm_attn.
    """
    q, k, v = _check(q, k, v)
    if width not in (64, 128):
        raise ValueError("image kernels are compiled for width 64 and 128")
    if q.shape[1] != TEXT_LEN + width * width:
        raise ValueError(f"expected {TEXT_LEN} text + {width}x{width} image tokens, got {q.shape[1]}")
    if softmax is not None:
        return _launch_image_ex(q, k, v, IMAGE_PATTERNS[pattern], int(width), TEXT_LEN, _scale(q, softmax_scale),
                                return_lse, softmax)
    return _launch(_C.intra_image_fwd, _C.intra_image_fwd_lse, q, k, v, IMAGE_PATTERNS[pattern], int(width),
                   TEXT_LEN, _scale(q, softmax_scale), return_lse)
