"""Randomised shapes for the host walk of the kernel's decomposition (the same index maps, block
tests and per-element bounds as the device code): it must reproduce the oracle's mask, every
visible pair exactly once, for any sequence length and pattern parameters the C ABI accepts."""
import ctypes

import numpy as np
import pytest
import torch
from hypothesis import HealthCheck, given, settings
from hypothesis import strategies as st

import oracle
from intra_amd import _lib


@pytest.fixture(scope="module")
def lib():
    return _lib.load()


def _walk(lib, pattern, S, hp, group_num=8, window=576, block=256, offset=0, n_sink=0):
    count = np.zeros((S, S), dtype=np.uint8)
    rc = lib.intra_model_mask_llm_ex(pattern, S, group_num, window, block, offset, n_sink, hp, count.ctypes.data)
    return rc, torch.from_numpy(count)


COMMON = dict(max_examples=150, deadline=None, suppress_health_check=[HealthCheck.function_scoped_fixture])


@settings(**COMMON)
@given(S=st.integers(1, 1400), G=st.integers(1, 40), hp=st.sampled_from([1, 2, 4]), gather=st.booleans())
def test_scatter_and_gather1(lib, S, G, hp, gather):
    rc, count = _walk(lib, 1 if gather else 0, S, hp, group_num=G)
    assert rc == 0, _lib.last_error()
    kind = "llm/gather1" if gather else "llm/scatter"
    assert torch.equal(count, oracle.mask_rows(kind, S, group_num=G).to(torch.uint8))


@settings(**COMMON)
@given(S=st.integers(1, 1400), G=st.integers(1, 40), W=st.integers(64, 3000), hp=st.sampled_from([1, 2, 4]),
       pattern=st.sampled_from([0, 1, 4]))
def test_half_size_workgroups(lib, S, G, W, hp, pattern):
    """The same walks with row blocks of 4 wavefronts (128 / hp queries)."""
    count = np.zeros((S, S), dtype=np.uint8)
    rc = lib.intra_model_mask(0, pattern, S, G, W, hp, 4, count.ctypes.data)
    assert rc == 0, _lib.last_error()
    kind = {0: "llm/scatter", 1: "llm/gather1", 4: "llm/window"}[pattern]
    kw = dict(window=W) if pattern == 4 else dict(group_num=G)
    assert torch.equal(torch.from_numpy(count), oracle.mask_rows(kind, S, **kw).to(torch.uint8))


@settings(**COMMON)
@given(S=st.integers(1, 1400), W=st.integers(64, 3000), hp=st.sampled_from([1, 2, 4]))
def test_aligned_window(lib, S, W, hp):
    rc, count = _walk(lib, 4, S, hp, window=W)
    assert rc == 0, _lib.last_error()
    assert torch.equal(count, oracle.mask_rows("llm/window", S, window=W).to(torch.uint8))


@settings(**COMMON)
@given(S=st.integers(1, 1400), W=st.integers(1, 2000), ns=st.integers(0, 1500), hp=st.sampled_from([1, 2, 4]))
def test_window_with_sinks(lib, S, W, ns, hp):
    rc, count = _walk(lib, 9, S, hp, window=W, n_sink=ns)
    assert rc == 0, _lib.last_error()
    assert torch.equal(count, oracle.mask_rows("llm/window_sink", S, window=W, n_sink=ns).to(torch.uint8))


@settings(**COMMON)
@given(S=st.integers(1, 1400), G=st.integers(1, 6), blk64=st.integers(1, 8), off=st.integers(0, 5),
       ns_frac=st.floats(0, 1), hp=st.sampled_from([1, 2, 4]))
def test_block_scatter(lib, S, G, blk64, off, ns_frac, hp):
    blk, off = 64 * blk64, off % G
    ns = int(ns_frac * blk)
    rc, count = _walk(lib, 8, S, hp, group_num=G, block=blk, offset=off, n_sink=ns)
    if off and blk % (256 // hp):
        assert rc == _lib.INTRA_ERR_UNSUPPORTED
        return
    assert rc == 0, _lib.last_error()
    want = oracle.mask_rows("llm/block_scatter", S, group_num=G, block=blk, offset=off, n_sink=ns)
    assert torch.equal(count, want.to(torch.uint8))


@settings(max_examples=40, deadline=None, suppress_health_check=[HealthCheck.function_scoped_fixture])
@given(w8=st.integers(2, 7), t8=st.integers(1, 40), hp=st.sampled_from([1, 2, 4]), gather0=st.booleans(),
       waves=st.sampled_from([8, 4]))
def test_image_patterns(lib, w8, t8, hp, gather0, waves):
    W, T = 8 * w8, 8 * t8
    S = T + W * W
    count = np.zeros((S, S), dtype=np.uint8)
    rc = lib.intra_model_mask(1, 4 if gather0 else 0, S, W, T, hp, waves, count.ctypes.data)
    if gather0 and waves * 32 // hp < 64:  # a row block holds whole 8x8 patches
        assert rc == _lib.INTRA_ERR_UNSUPPORTED
        return
    assert rc == 0, _lib.last_error()
    kind = "image/gather0" if gather0 else "image/scatter"
    want = oracle.mask_rows(kind, S, width=W, text_len=T)
    assert torch.equal(torch.from_numpy(count), want.to(torch.uint8))


# ---------------------------------------------------------------------------- backward (dk / dv launches)
def _walk_bwd(lib, pattern, S, group_num=8, window=576, block=256, offset=0, n_sink=0):
    count = np.zeros((S, S), dtype=np.uint8)
    rc = lib.intra_model_mask_llm_bwd(pattern, S, group_num, window, block, offset, n_sink, count.ctypes.data)
    return rc, torch.from_numpy(count)


@settings(**COMMON)
@given(S=st.integers(1, 1400), G=st.integers(1, 40), gather=st.booleans())
def test_backward_scatter_and_gather1(lib, S, G, gather):
    rc, count = _walk_bwd(lib, 1 if gather else 0, S, group_num=G)
    assert rc == 0, _lib.last_error()
    kind = "llm/gather1" if gather else "llm/scatter"
    assert torch.equal(count, oracle.mask_rows(kind, S, group_num=G).to(torch.uint8))


@settings(**COMMON)
@given(S=st.integers(1, 1400), W=st.integers(64, 3000))
def test_backward_aligned_window(lib, S, W):
    rc, count = _walk_bwd(lib, 4, S, window=W)
    assert rc == 0, _lib.last_error()
    assert torch.equal(count, oracle.mask_rows("llm/window", S, window=W).to(torch.uint8))


@settings(**COMMON)
@given(S=st.integers(1, 2600), W=st.integers(1, 2000), ns=st.integers(0, 1500))
def test_backward_window_with_sinks(lib, S, W, ns):
    rc, count = _walk_bwd(lib, 9, S, window=W, n_sink=ns)
    assert rc == 0, _lib.last_error()
    assert torch.equal(count, oracle.mask_rows("llm/window_sink", S, window=W, n_sink=ns).to(torch.uint8))


@settings(**COMMON)
@given(S=st.integers(1, 2600), G=st.integers(1, 6), blk64=st.integers(1, 8), off=st.integers(0, 5), ns_frac=st.floats(0, 1))
def test_backward_block_scatter(lib, S, G, blk64, off, ns_frac):
    blk, off = 64 * blk64, off % G
    if off != 0:
        blk = 256 * ((blk64 + 1) // 2)  # a stripe offset needs 256-key row blocks inside one block
    ns = int(ns_frac * blk)
    rc, count = _walk_bwd(lib, 8, S, group_num=G, block=blk, offset=off, n_sink=ns)
    assert rc == 0, _lib.last_error()
    want = oracle.mask_rows("llm/block_scatter", S, group_num=G, block=blk, offset=off, n_sink=ns)
    assert torch.equal(count, want.to(torch.uint8))


@settings(max_examples=60, deadline=None, suppress_health_check=[HealthCheck.function_scoped_fixture])
@given(w8=st.integers(2, 9), t8=st.integers(1, 50), gather=st.booleans())
def test_backward_image_patterns(lib, w8, t8, gather):
    W, T = 8 * w8, 8 * t8
    S = T + W * W
    count = np.zeros((S, S), dtype=np.uint8)
    rc = lib.intra_model_mask_image_bwd(4 if gather else 0, S, W, T, count.ctypes.data)
    assert rc == 0, _lib.last_error()
    kind = "image/gather0" if gather else "image/scatter"
    assert torch.equal(torch.from_numpy(count), oracle.mask_rows(kind, S, width=W, text_len=T).to(torch.uint8))
