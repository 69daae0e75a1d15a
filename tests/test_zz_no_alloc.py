"""intra_llm_bwd_noalloc - the backward entry point that allocates nothing and keeps its workspace
in an array of the library's own device image - against intra_llm_bwd on the same inputs, through
the C ABI.  The kernels are the same and deterministic, so the results have to be bit-identical.
Two calls in a row share the built-in array; the second is smaller and must not be disturbed by
what the first left behind.  Requests beyond the built-in size are refused with a clear message."""
import ctypes

import pytest
import torch

from intra_amd import _lib, intra_llm_attn

pytestmark = pytest.mark.gpu
DEV = "cuda"
IDS = {"scatter": 0, "gather1": 1, "window": 4, "block_scatter": 8, "window_sink": 9}


def make(B, S, H, Hkv, seed):
    g = torch.Generator(device="cpu").manual_seed(seed)
    mk = lambda h: torch.randn(B, S, h, 128, generator=g, dtype=torch.float32).to(torch.bfloat16).to(DEV)
    return mk(H), mk(Hkv), mk(Hkv), mk(H)


def both_ways(lib, B, S, H, Hkv, pattern, seed, group_num=8, window=576, block=256, offset=0, n_sink=0):
    q, k, v, dout = make(B, S, H, Hkv, seed)
    with torch.no_grad():
        out, lse = intra_llm_attn(q, k, v, pattern, group_num=group_num, window=window, return_lse=True, block=block,
                                  offset=offset, n_sink=n_sink)
    pat = (IDS[pattern], group_num, window, block, offset, n_sink)
    st = _lib.strides3
    stream = torch.cuda.current_stream().cuda_stream
    scale = 128 ** -0.5

    def call(fn, *work):
        grads = [torch.full_like(t, float("nan")) for t in (q, k, v)]
        rc = fn(q.data_ptr(), k.data_ptr(), v.data_ptr(), out.data_ptr(), lse.data_ptr(), dout.data_ptr(),
                *(g.data_ptr() for g in grads), *work, B, S, H, Hkv, st(q), st(k), st(v), st(out), st(dout),
                *(st(g) for g in grads), st(lse), *pat, scale, stream)
        assert rc == 0, _lib.last_error()
        torch.cuda.synchronize()
        return grads

    n_work = lib.intra_llm_bwd_workspace(B, S, H, Hkv, *pat)
    assert 0 < n_work <= 4 * 1024 * 1024
    work = torch.full((n_work,), float("nan"), dtype=torch.float32, device=DEV)
    want = call(lib.intra_llm_bwd, work.data_ptr())
    got = call(lib.intra_llm_bwd_noalloc)
    for name, g, w in zip(("dq", "dk", "dv"), got, want):
        assert bool(torch.isfinite(g).all()), name
        assert torch.equal(g, w), f"{pattern} S={S}: {name} differs from intra_llm_bwd"


def test_no_alloc_backward_matches_the_workspace_entry_point(lib):
    # a call with sink keys (both parts of the workspace in use), then a smaller one right after it
    both_ways(lib, 2, 2048, 8, 2, "block_scatter", seed=1, group_num=2, block=256, offset=1, n_sink=64)
    both_ways(lib, 1, 1000, 4, 4, "scatter", seed=2, group_num=3)
    both_ways(lib, 1, 640, 4, 1, "window_sink", seed=3, window=63, n_sink=5)


def test_no_alloc_backward_refuses_what_does_not_fit(lib):
    ptr = 1 << 20  # never dereferenced: the size check comes before any launch
    st = (ctypes.c_int64 * 3)(128 * 32 * 128, 32 * 128, 128)
    B, S, H = 8, 32768, 32  # B * H * S floats = 8 Mi > 4 Mi
    assert lib.intra_llm_bwd_workspace(B, S, H, 8, 0, 8, 576, 256, 0, 0) > 4 * 1024 * 1024
    rc = lib.intra_llm_bwd_noalloc(ptr, ptr, ptr, ptr, ptr, ptr, ptr, ptr, ptr, B, S, H, 8, st, st, st, st, st, st, st, st,
                                   st, 0, 8, 576, 256, 0, 0, 0.1, None)
    assert rc == _lib.INTRA_ERR_UNSUPPORTED and "built-in one holds" in _lib.last_error()
