"""CPU-side checks of libintra_hip.so: it loads, exports every symbol of include/intra_hip.h,
validates arguments without touching a GPU, plans launches, and its host walk of the kernel's
set / row-block / wavefront / key-block decomposition reproduces the oracle masks exactly."""
import ctypes
import os
import re

import numpy as np
import pytest
import torch

import oracle
from intra_amd import _lib

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))


def test_exports_every_declared_symbol(lib):
    header = open(os.path.join(ROOT, "include", "intra_hip.h")).read()
    declared = set(re.findall(r"^\s*(?:const\s+char\*|int|int64_t)\s+(intra_\w+)\s*\(", header, re.M))
    assert declared == set(_lib.SYMBOLS), (declared, set(_lib.SYMBOLS))
    for name in declared:
        assert getattr(lib, name) is not None
    assert lib.intra_version() >= 100


def _plan(lib, domain, pattern, B, S, H, Hkv, a0, a1):
    p = _lib.IntraPlan()
    rc = lib.intra_plan(domain, pattern, B, S, H, Hkv, a0, a1, ctypes.byref(p))
    return rc, p


def test_plan_headline(lib):
    rc, p = _plan(lib, 0, 0, 1, 32768, 32, 8, 8, 576)
    assert rc == 0
    assert (p.heads_per_block, p.waves, p.pos_per_block) == (4, 8, 64)
    assert (p.n_sets, p.n_mblocks, p.work_items, p.grid) == (8, 64, 4096, 4096)
    assert p.pairs_per_head == 67125248 and 0 < p.lds_bytes <= 160 * 1024


def test_plan_gather0_sets(lib):
    # one launch: sets of text rows (the 64 text queries of 1 or 2 scatter groups each), then sets of
    # 2 / 1 / 1 neighbouring 8x8 patches.  At 2048 x 2048 a merged text item would be much longer than
    # a patch item, so the chunks stay apart; so they do in the half-size row blocks at 1024 x 1024.
    # Workgroups of 4 wavefronts where a row block then still holds a whole patch.
    for H, Hkv, hp, waves, pg in ((24, 24, 1, 4, 2), (16, 8, 2, 4, 1), (32, 8, 4, 8, 1)):
        rc, p = _plan(lib, 1, 4, 1, 16896, H, Hkv, 128, 512)
        assert rc == 0 and p.launches == 1
        assert (p.heads_per_block, p.waves, p.pos_per_block) == (hp, waves, waves * 32 // hp)
        assert (p.n_sets, p.n_mblocks) == (8 + 16 * 16 // pg, 1)
        assert p.work_items == 8 * -(-Hkv * p.n_sets // 8) * (H // Hkv // hp)
    rc, p = _plan(lib, 1, 4, 1, 4608, 24, 24, 64, 512)
    assert rc == 0 and (p.n_sets, p.n_mblocks) == (8 + 8 * 8 // 2, 1)
    # image scatter: 576 queries per set; at 1024 x 1024 the row blocks of 256 queries would be 2.25 per
    # CU of a 256-CU device, so the launch takes half-size ones; at 2048 x 2048 it keeps the large ones
    rc, p = _plan(lib, 1, 0, 1, 4608, 24, 24, 64, 512)
    assert rc == 0 and (p.n_sets, p.n_mblocks, p.waves) == (8, 5, 4)
    rc, p = _plan(lib, 1, 0, 1, 16896, 24, 24, 128, 512)
    assert rc == 0 and p.launches == 1 and (p.n_sets, p.n_mblocks, p.waves) == (8, 9, 8)


@pytest.mark.parametrize("domain,pattern,kind,S,a0,a1", [
    (0, 0, "llm/scatter", 1000, 3, 576), (0, 1, "llm/gather1", 3000, 8, 576),
    (0, 4, "llm/window", 3000, 8, 1000), (1, 0, "image/scatter", 4608, 64, 512),
    (1, 4, "image/gather0", 16896, 128, 512)])
def test_plan_pair_counts(lib, domain, pattern, kind, S, a0, a1):
    rc, p = _plan(lib, domain, pattern, 1, S, 8, 8, a0, a1)
    assert rc == 0
    kw = dict(group_num=a0, window=a1) if domain == 0 else dict(width=a0, text_len=a1)
    assert p.pairs_per_head == oracle.pairs_per_head(kind, S, **kw)


BAD = [  # domain, pattern, B, S, H, Hkv, a0, a1, text in the message
    (0, 7, 1, 128, 4, 4, 8, 576, "unknown LLM pattern"),
    (0, 0, 1, 128, 4, 3, 8, 576, "multiple of kv heads"),
    (0, 0, 0, 128, 4, 4, 8, 576, "must be positive"),
    (0, 0, 1, 128, 4, 4, 0, 576, "group_num must be >= 1"),
    (0, 4, 1, 128, 4, 4, 8, 32, "window must be >= 64"),
    (1, 1, 1, 4608, 4, 4, 64, 512, "unknown image pattern"),
    (1, 0, 1, 4600, 4, 4, 64, 512, "expected 512 text + 64x64"),
    (1, 0, 1, 512 + 100, 4, 4, 10, 512, "width must be a multiple of 8"),
    (1, 4, 1, 500 + 4096, 4, 4, 64, 500, "text_len must be a positive multiple of 8"),
    (2, 0, 1, 128, 4, 4, 8, 576, "unknown domain"),
]


@pytest.mark.parametrize("case", BAD)
def test_plan_rejects_bad_requests(lib, case):
    *args, text = case
    rc, _ = _plan(lib, *args)
    assert rc == _lib.INTRA_ERR_INVALID
    assert text in _lib.last_error()


def test_fwd_validates_before_touching_the_gpu(lib):
    st = (ctypes.c_int64 * 3)(128 * 4 * 128, 4 * 128, 128)
    bad = (ctypes.c_int64 * 3)(128 * 4 * 128, 4 * 128 + 4, 128)
    ptr = 1 << 20  # never dereferenced: every call below fails validation first
    call = lambda *a: lib.intra_llm_fwd(*a)
    assert call(None, ptr, ptr, ptr, 1, 128, 4, 4, st, st, st, st, 0, 8, 576, 0.1, None) == 1
    assert "non-null" in _lib.last_error()
    assert call(ptr + 2, ptr, ptr, ptr, 1, 128, 4, 4, st, st, st, st, 0, 8, 576, 0.1, None) == 1
    assert "16-byte aligned" in _lib.last_error()
    assert call(ptr, ptr, ptr, ptr, 1, 128, 4, 4, st, bad, st, st, 0, 8, 576, 0.1, None) == 1
    assert "k stride 1" in _lib.last_error()
    assert call(ptr, ptr, ptr, ptr, 1, 128, 4, 4, st, st, st, None, 0, 8, 576, 0.1, None) == 1
    assert "o strides pointer is null" in _lib.last_error()
    assert call(ptr, ptr, ptr, ptr, 1, 128, 4, 4, st, st, st, st, 0, 8, 576, float("nan"), None) == 1
    assert "finite" in _lib.last_error()
    assert call(ptr, ptr, ptr, ptr, 1, 128, 4, 4, st, st, st, st, 9, 8, 576, 0.1, None) == 1
    assert lib.intra_image_fwd(ptr, ptr, ptr, ptr, 1, 128, 4, 4, st, st, st, st, 0, 64, 512, 0.1, None) == 1
    assert "expected 512 text" in _lib.last_error()


def test_zero_strides_are_for_inputs_only(lib):
    # expanded (stride 0) views are fine where the kernels only read; outputs may not alias
    st = (ctypes.c_int64 * 3)(128 * 4 * 128, 4 * 128, 128)
    tok0 = (ctypes.c_int64 * 3)(128 * 4 * 128, 0, 128)
    head0 = (ctypes.c_int64 * 3)(128 * 4 * 128, 4 * 128, 0)
    ptr = 1 << 20  # never dereferenced: the NaN scale fails validation after the stride checks
    nan = float("nan")
    for inputs in ((tok0, st, st), (st, head0, st), (st, st, head0), (tok0, tok0, tok0)):
        assert lib.intra_llm_fwd(ptr, ptr, ptr, ptr, 1, 128, 4, 4, *inputs, st, 0, 8, 576, nan, None) == 1
        assert "finite" in _lib.last_error()
    for out in (tok0, head0):
        assert lib.intra_llm_fwd(ptr, ptr, ptr, ptr, 1, 128, 4, 4, st, st, st, out, 0, 8, 576, nan, None) == 1
        assert "o has a zero stride" in _lib.last_error()


def test_version_and_softmax_mode(lib):
    import intra_amd
    major, minor, patch = (int(x) for x in intra_amd.__version__.split("."))
    assert lib.intra_version() == major * 10000 + minor * 100 + patch
    start = lib.intra_get_softmax_mode()
    try:
        for mode in (1, 2, 3, 0):
            assert lib.intra_set_softmax_mode(mode) == 0 and lib.intra_get_softmax_mode() == mode
        assert lib.intra_set_softmax_mode(4) == 1 and "softmax mode" in _lib.last_error()
        assert lib.intra_set_softmax_mode(-1) == 1
        assert lib.intra_get_softmax_mode() == 0
        for name in ("exact", "scaled", "folded", "auto"):
            intra_amd.set_softmax_mode(name)
            assert intra_amd.get_softmax_mode() == name
        intra_amd.set_softmax_mode("fast")  # the older name of folded
        assert intra_amd.get_softmax_mode() == "folded"
    finally:
        lib.intra_set_softmax_mode(start)


def test_lse_entry_points_validate_their_extra_arguments(lib):
    st = (ctypes.c_int64 * 3)(128 * 4 * 128, 4 * 128, 128)
    ls = (ctypes.c_int64 * 3)(4 * 128, 128, 1)
    zero = (ctypes.c_int64 * 3)(4 * 128, 0, 1)
    ptr = 1 << 20  # never dereferenced
    for fn, a0, a1, S in ((lib.intra_llm_fwd_lse, 8, 576, 128), (lib.intra_image_fwd_lse, 16, 8, 264)):
        common = (ptr, ptr, ptr, ptr, 1, S, 4, 4, st, st, st, st, 0, a0, a1, 0.1, None)
        assert fn(*common, None, ls) == 1 and "lse must be a non-null" in _lib.last_error()
        assert fn(*common, ptr + 2, ls) == 1 and "4-byte aligned" in _lib.last_error()
        assert fn(*common, ptr, None) == 1 and "lse strides pointer is null" in _lib.last_error()
        assert fn(*common, ptr, zero) == 1 and "zero stride" in _lib.last_error()
    # the shared checks still come first
    assert lib.intra_llm_fwd_lse(None, ptr, ptr, ptr, 1, 128, 4, 4, st, st, st, st, 0, 8, 576, 0.1, None, ptr, ls) == 1
    assert "q, k, v and o must be non-null" in _lib.last_error()


def _model(lib, domain, pattern, S, a0, a1, hp=0, nw=0):
    count = np.zeros((S, S), dtype=np.uint8)
    rc = lib.intra_model_mask(domain, pattern, S, a0, a1, hp, nw, count.ctypes.data)
    assert rc == 0, _lib.last_error()
    return torch.from_numpy(count)


LLM_CASES = [(S, "llm/scatter", 0, dict(group_num=G)) for S in (1, 5, 63, 64, 65, 257, 1000) for G in (1, 2, 3, 8, 16)] + \
            [(S, "llm/gather1", 1, dict(group_num=G)) for S in (64, 128, 1000, 1024) for G in (8, 3)] + \
            [(S, "llm/window", 4, dict(window=W)) for S in (1, 64, 100, 1000, 1300) for W in (64, 65, 96, 576, 1000, 5000)]


@pytest.mark.parametrize("S,kind,pattern,kw", LLM_CASES)
@pytest.mark.parametrize("hp", [1, 2, 4])
def test_kernel_decomposition_equals_mask_llm(lib, S, kind, pattern, kw, hp):
    count = _model(lib, 0, pattern, S, kw.get("group_num", 8), kw.get("window", 576), hp, 8)
    want = oracle.mask_rows(kind, S, **kw)
    assert count.max() <= 1, "a score is computed more than once"
    assert torch.equal(count.bool(), want)


IMG_CASES = [(16, 64), (24, 16), (32, 512), (64, 512), (40, 8)]


@pytest.mark.parametrize("W,T", IMG_CASES)
@pytest.mark.parametrize("kind,pattern", [("image/scatter", 0), ("image/gather0", 4)])
@pytest.mark.parametrize("hp", [1, 2, 4])
def test_kernel_decomposition_equals_mask_image(lib, W, T, kind, pattern, hp):
    S = T + W * W
    count = _model(lib, 1, pattern, S, W, T, hp, 8)
    want = oracle.mask_rows(kind, S, width=W, text_len=T)
    assert count.max() <= 1
    assert torch.equal(count.bool(), want)


def test_model_rejects_unknown_shape(lib):
    count = np.zeros((64, 64), dtype=np.uint8)
    assert lib.intra_model_mask(0, 0, 64, 8, 576, 3, 8, count.ctypes.data) == 1
    assert "no kernel" in _lib.last_error()


# ------------------------------------------------------------------ block scatter / window with sinks
EX_CASES = \
    [(S, "llm/block_scatter", 8, dict(group_num=G, block=blk, offset=off, n_sink=ns))
     for S in (1, 64, 200, 1000, 1537) for (G, blk, off, ns) in
     ((2, 256, 0, 0), (2, 256, 1, 64), (2, 256, 0, 64), (3, 64, 2, 10), (3, 128, 1, 128), (4, 64, 0, 33),
      (1, 64, 0, 0), (2, 512, 1, 0))] + \
    [(S, "llm/window_sink", 9, dict(window=W, n_sink=ns))
     for S in (1, 63, 200, 1000, 1300) for (W, ns) in
     ((575, 64), (575, 0), (1, 0), (1, 5), (64, 64), (100, 37), (5000, 64), (300, 700))]


def _model_ex(lib, pattern, S, hp, group_num=2, window=575, block=256, offset=0, n_sink=0):
    count = np.zeros((S, S), dtype=np.uint8)
    rc = lib.intra_model_mask_llm_ex(pattern, S, group_num, window, block, offset, n_sink, hp, count.ctypes.data)
    return rc, torch.from_numpy(count)


@pytest.mark.parametrize("S,kind,pattern,kw", EX_CASES)
@pytest.mark.parametrize("hp", [1, 2, 4])
def test_kernel_decomposition_equals_mask_llm_ex(lib, S, kind, pattern, kw, hp):
    rc, count = _model_ex(lib, pattern, S, hp, **kw)
    if kw.get("offset", 0) and kw["block"] % (256 // hp):  # row blocks would straddle query blocks
        assert rc == _lib.INTRA_ERR_UNSUPPORTED
        return
    assert rc == 0, _lib.last_error()
    want = oracle.mask_rows(kind, S, **kw)
    assert torch.equal(count, want.to(torch.uint8)), f"{kind} {kw} hp={hp}: kernel walk differs from the mask"


@pytest.mark.parametrize("S,kind,pattern,kw", EX_CASES[::3])
def test_plan_ex_pair_counts(lib, S, kind, pattern, kw):
    p = _lib.IntraPlan()
    rc = lib.intra_plan_llm_ex(pattern, 1, S, 8, 2, kw.get("group_num", 2), kw.get("window", 575),
                               kw.get("block", 256), kw.get("offset", 0), kw.get("n_sink", 0), ctypes.byref(p))
    assert rc == 0, _lib.last_error()
    assert p.pairs_per_head == oracle.pairs_per_head(kind, S, **kw) == int(oracle.mask_rows(kind, S, **kw).sum())


def test_ex_argument_checks(lib):
    p = _lib.IntraPlan()
    bad = [((8, 1, 512, 4, 4, 2, 575, 100, 0, 0), "block must be a positive multiple of 64"),
           ((8, 1, 512, 4, 4, 2, 575, 256, 2, 0), "offset must be in [0, group_num)"),
           ((8, 1, 512, 4, 4, 2, 575, 256, 0, 300), "n_sink must be in [0, block]"),
           ((9, 1, 512, 4, 4, 2, 0, 256, 0, 0), "window must be >= 1"),
           ((9, 1, 512, 4, 4, 2, 575, 256, 0, -1), "n_sink must be >= 0"),
           ((7, 1, 512, 4, 4, 2, 575, 256, 0, 0), "unknown LLM pattern")]
    for args, text in bad:
        assert lib.intra_plan_llm_ex(*args, ctypes.byref(p)) == _lib.INTRA_ERR_INVALID
        assert text in _lib.last_error()
    # a stripe offset needs row blocks inside one query block: with 1 q head per kv head the smallest
    # row block has 128 queries, which 64-token blocks cannot hold
    assert lib.intra_plan_llm_ex(8, 1, 512, 4, 4, 2, 575, 64, 1, 0, ctypes.byref(p)) == _lib.INTRA_ERR_UNSUPPORTED
    assert lib.intra_plan_llm_ex(8, 1, 512, 16, 4, 2, 575, 64, 1, 0, ctypes.byref(p)) == 0
    assert (p.heads_per_block, p.pos_per_block) == (4, p.waves * 32 // 4)  # (so few row blocks: half-size workgroups)
    assert lib.intra_plan_llm_ex(8, 1, 512, 8, 4, 2, 575, 128, 1, 0, ctypes.byref(p)) == 0
    assert (p.heads_per_block, p.pos_per_block) == (2, p.waves * 32 // 2)
    assert lib.intra_plan_llm_ex(8, 1, 512, 4, 4, 2, 575, 128, 1, 0, ctypes.byref(p)) == 0  # (only the half-size row blocks fit)
    assert (p.heads_per_block, p.waves, p.pos_per_block) == (1, 4, 128)
    # the old patterns pass through and ignore the extra arguments
    q = _lib.IntraPlan()
    assert lib.intra_plan_llm_ex(0, 1, 32768, 32, 8, 8, 576, 0, 0, 0, ctypes.byref(p)) == 0
    assert lib.intra_plan(0, 0, 1, 32768, 32, 8, 8, 576, ctypes.byref(q)) == 0
    assert (p.work_items, p.pairs_per_head) == (q.work_items, q.pairs_per_head)


def test_bwd_validates_before_touching_the_gpu(lib):
    st = _lib._i64x3(512 * 4 * 128, 4 * 128, 128)
    ls = _lib._i64x3(4 * 512, 512, 1)
    P = 0x1000  # never dereferenced: every call below fails validation first

    def call(ptrs=(P,) * 10, B=1, S=512, H=4, Hkv=4, strides=(st,) * 8, lse_strides=ls, pattern=0, G=2, window=576,
             block=256, offset=0, n_sink=0, scale=0.1):
        return lib.intra_llm_bwd(*ptrs, B, S, H, Hkv, *strides, lse_strides, pattern, G, window, block, offset, n_sink,
                                 scale, None)

    for i in range(10):  # q, k, v, o, lse, dout, dq, dk, dv, workspace
        assert call(ptrs=tuple(None if j == i else P for j in range(10))) == _lib.INTRA_ERR_INVALID
        assert "non-null" in _lib.last_error()
    assert call(ptrs=(P + 8,) + (P,) * 9) == _lib.INTRA_ERR_INVALID and "16-byte aligned" in _lib.last_error()
    assert call(ptrs=(P,) * 4 + (P + 2,) + (P,) * 5) == _lib.INTRA_ERR_INVALID and "4-byte aligned" in _lib.last_error()
    odd = _lib._i64x3(512 * 4 * 128, 4 * 128 + 4, 128)
    assert call(strides=(st,) * 4 + (odd,) + (st,) * 3) == _lib.INTRA_ERR_INVALID and "dout" in _lib.last_error()
    assert call(scale=float("nan")) == _lib.INTRA_ERR_INVALID
    assert call(lse_strides=_lib._i64x3(4 * 512, -512, 1)) == _lib.INTRA_ERR_INVALID and "lse stride" in _lib.last_error()
    assert call(H=6, Hkv=4) == _lib.INTRA_ERR_INVALID
    assert call(pattern=7) == _lib.INTRA_ERR_INVALID
    assert call(scale=0.0) == _lib.INTRA_ERR_UNSUPPORTED
    # a stripe offset needs key row blocks inside one block
    assert call(pattern=8, offset=1, block=128) == _lib.INTRA_ERR_UNSUPPORTED
    assert "backward" in _lib.last_error()
    assert call(ptrs=(P,) * 9 + (P + 4,)) == _lib.INTRA_ERR_INVALID and "workspace" in _lib.last_error()


def _leading_chunks(S, B, Hkv, ns, cus=320):
    """The library's rule for the pass over leading keys: about one workgroup per CU (the workspace
    is sized for a device of 320 CUs, whatever device is current), chunks of at least 128 queries and
    a multiple of 64."""
    row_wgs = B * Hkv * -(-ns // 256)
    chunks = min(max(1, cus // row_wgs), max(1, S // 128))
    chunk = 64 * -(-S // (64 * chunks))
    return -(-S // chunk)


def test_bwd_workspace_size(lib):
    # two values per (batch, head, token): -rowsum(dO o O) and lse * log2(e)
    assert lib.intra_llm_bwd_workspace(1, 1000, 8, 2, 0, 8, 576, 256, 0, 0) == 2 * 8000
    assert lib.intra_llm_bwd_workspace(2, 1001, 3, 3, 4, 8, 576, 256, 0, 0) == 2 * 6008  # each rounded up to 4
    # sinks: chunks x B x Hkv x n_sink x 128 more
    assert _leading_chunks(3000, 1, 2, 64) == 16 and _leading_chunks(65536, 1, 8, 64) == 40
    assert lib.intra_llm_bwd_workspace(1, 3000, 8, 2, 9, 2, 575, 256, 0, 64) == 2 * 24000 + 16 * 2 * 64 * 128
    assert lib.intra_llm_bwd_workspace(1, 65536, 32, 8, 9, 2, 575, 256, 0, 64) == 2 * 65536 * 32 + 40 * 8 * 64 * 128
    assert lib.intra_llm_bwd_workspace(1, 3000, 8, 2, 8, 2, 575, 256, 1, 0) == 2 * 24000
    assert lib.intra_llm_bwd_workspace(1, 3000, 8, 2, 8, 2, 575, 128, 1, 0) == -1
    assert lib.intra_llm_bwd_workspace(1, 3000, 8, 3, 0, 8, 576, 256, 0, 0) == -1
    # image patterns: the 512 text keys are the leading keys
    S = 512 + 64 * 64
    assert lib.intra_image_bwd_workspace(1, S, 24, 24, 0, 64, 512) == 2 * S * 24 + _leading_chunks(S, 1, 24, 512) * 24 * 512 * 128
    assert lib.intra_image_bwd_workspace(1, S, 24, 24, 4, 64, 511) == -1


BWD_CASES = [
    (0, "llm/scatter", 1000, dict(group_num=3)), (0, "llm/scatter", 63, dict(group_num=8)),
    (1, "llm/gather1", 1024, dict(group_num=8)), (4, "llm/window", 1000, dict(window=192)),
    (4, "llm/window", 300, dict(window=64)),
    (8, "llm/block_scatter", 1500, dict(group_num=2, block=256)),
    (8, "llm/block_scatter", 1111, dict(group_num=3, block=64, n_sink=40)),
    (8, "llm/block_scatter", 2000, dict(group_num=2, block=256, offset=1, n_sink=64)),
    (8, "llm/block_scatter", 2100, dict(group_num=4, block=256, offset=3)),
    (8, "llm/block_scatter", 1300, dict(group_num=3, block=512, offset=2, n_sink=512)),
    (8, "llm/block_scatter", 200, dict(group_num=2, block=256, offset=1, n_sink=64)),
    (9, "llm/window_sink", 1500, dict(window=575, n_sink=64)), (9, "llm/window_sink", 700, dict(window=1, n_sink=3)),
    (9, "llm/window_sink", 600, dict(window=100, n_sink=300)), (9, "llm/window_sink", 500, dict(window=5000, n_sink=0)),
]


@pytest.mark.parametrize("pattern,kind,S,kw", BWD_CASES)
def test_backward_key_row_maps_equal_mask(lib, pattern, kind, S, kw):
    """Every (query, key) pair of the mask is multiplied exactly once by the dk / dv launches
    (inverse index maps, unsaved sink rows, sink pass)."""
    count = np.zeros((S, S), dtype=np.uint8)
    rc = lib.intra_model_mask_llm_bwd(pattern, S, kw.get("group_num", 2), kw.get("window", 575), kw.get("block", 256),
                                      kw.get("offset", 0), kw.get("n_sink", 0), count.ctypes.data)
    assert rc == 0, _lib.last_error()
    want = oracle.mask_rows(kind, S, **kw).numpy().astype(np.uint8)
    assert np.array_equal(count, want), np.argwhere(count != want)[:5]


@pytest.mark.parametrize("W,T", [(64, 512), (16, 8), (24, 72), (40, 200), (32, 96), (48, 64)])
@pytest.mark.parametrize("kind,pattern", [("image/scatter", 0), ("image/gather0", 4)])
def test_backward_key_row_maps_equal_mask_image(lib, W, T, kind, pattern):
    """The dk / dv passes of the image patterns (grid keys by group or by window, text queries'
    share, text keys against all queries) multiply every pair of the mask exactly once."""
    S = T + W * W
    count = np.zeros((S, S), dtype=np.uint8)
    rc = lib.intra_model_mask_image_bwd(pattern, S, W, T, count.ctypes.data)
    assert rc == 0, _lib.last_error()
    want = oracle.mask_rows(kind, S, width=W, text_len=T).numpy().astype(np.uint8)
    assert np.array_equal(count, want), np.argwhere(count != want)[:5]


def test_flags_of_the_ex_entry_points_are_checked_before_any_launch(lib):
    """Unknown bits in `flags` are refused during argument validation (no GPU needed); the known
    values get past it and fail later, on the null pointers."""
    st = (ctypes.c_int64 * 3)(128 * 4 * 128, 4 * 128, 128)
    for flags, text in ((4, "unknown bits in flags"), (0x80000000, "unknown bits in flags")):
        assert lib.intra_llm_fwd_ex(None, None, None, None, 1, 128, 4, 4, st, st, st, st, 0, 8, 576, 256, 0, 0,
                                    0.1, None, None, None, flags) == _lib.INTRA_ERR_INVALID
        assert text in _lib.last_error()
        assert lib.intra_image_fwd_ex(None, None, None, None, 1, 512 + 256, 4, 4, st, st, st, st, 0, 16, 512,
                                      0.1, None, None, None, flags) == _lib.INTRA_ERR_INVALID
        assert text in _lib.last_error()
    for flags in (0, 1, 2, 3):
        assert lib.intra_llm_fwd_ex(None, None, None, None, 1, 128, 4, 4, st, st, st, st, 0, 8, 576, 256, 0, 0,
                                    0.1, None, None, None, flags) == _lib.INTRA_ERR_INVALID
        assert "non-null device pointers" in _lib.last_error()


def test_production_library_carries_no_ablation(lib, tmp_path):
    """The library tests and callers load computes every ingredient of the kernel's step; the
    ablations of the measurement builds do not compile without the timers."""
    import subprocess
    from intra_amd import build
    assert lib.intra_diag_ablation() == 0
    assert lib.intra_diag_set_buffer(None, 0) == _lib.INTRA_ERR_UNSUPPORTED  # no timers either
    res = subprocess.run([build.hipcc_path(), "--offload-arch=gfx950", "-std=c++17", "-fsyntax-only", "--cuda-device-only",
                          "-DINTRA_ABLATE=1", "-x", "hip", os.path.join(ROOT, "intra_amd", "csrc", "intra_kernel.hip.h")],
                         stdout=subprocess.PIPE, stderr=subprocess.STDOUT, text=True, cwd=tmp_path)
    assert res.returncode != 0 and "INTRA_ABLATE belongs to measurement builds" in res.stdout
