"""Both workgroup sizes of the forward kernels on the same inputs.  A plain call picks the size by
pattern and problem size (half-size workgroups for image gather0 and for launches with few row
blocks); the environment variable INTRA_WAVES, which the library reads at every call, names one for
measurements.  Every pattern has to meet the oracle with either size - also at sizes where the
other one is the default - and the patterns whose row blocks number their keys the same way whatever
their size (all but the per-token window with sinks, whose key list starts where the row block's
first query's window starts, and image gather0, whose runs of patches differ) have to agree bit for
bit: the same keys then meet in the same 32-key blocks and the sums are formed in the same order."""
import os

import pytest
import torch

import oracle
from intra_amd import _lib, intra_image_attn, intra_llm_attn
from parity_util import DEV, check, make_qkv

pytestmark = pytest.mark.gpu

LLM = [("scatter", dict(group_num=8)), ("scatter", dict(group_num=2)), ("gather1", dict(group_num=8)),
       ("window", dict(window=576)), ("block_scatter", dict(group_num=2, block=256, offset=1, n_sink=64)),
       ("window_sink", dict(window=575, n_sink=64))]


@pytest.fixture()
def waves():
    saved = os.environ.pop("INTRA_WAVES", None)

    def choose(n):
        if n is None:
            os.environ.pop("INTRA_WAVES", None)
        else:
            os.environ["INTRA_WAVES"] = str(n)
    yield choose
    os.environ.pop("INTRA_WAVES", None)
    if saved is not None:
        os.environ["INTRA_WAVES"] = saved


@pytest.mark.parametrize("pattern,kw", LLM)
@pytest.mark.parametrize("S,H,Hkv", [(8192, 32, 8), (3000 + 8 * 64, 6, 2), (640, 4, 4)])
def test_llm_patterns_with_either_size(waves, pattern, kw, S, H, Hkv):
    if pattern == "gather1" and S % 64:
        S -= S % 64
    q, k, v = make_qkv(1, S, H, Hkv, seed=S + H)
    rows = torch.unique(torch.cat([torch.randperm(S, generator=torch.Generator().manual_seed(S))[:384],
                                   torch.tensor([0, 1, 63, 64, 127, 128, S - 1])])).to(DEV)
    outs = {}
    for n in (8, 4):
        waves(n)
        with torch.no_grad():
            outs[n] = intra_llm_attn(q, k, v, pattern, **kw)
        check(outs[n], q, k, v, "llm/" + pattern, rows, None, True, f"{pattern} S={S} waves={n}", **kw)
    if pattern != "window_sink":
        assert torch.equal(outs[8], outs[4])
    waves(None)
    with torch.no_grad():
        plain = intra_llm_attn(q, k, v, pattern, **kw)
    assert torch.equal(plain, outs[8]) or torch.equal(plain, outs[4])


def _random_cases(n, seed):
    """Random shapes, patterns, head ratios (1 - 8 query heads per kv head) and scales; the arguments
    stay inside what both workgroup sizes accept (a striped block pattern with an offset needs blocks
    of 128 tokens per odd head ratio for the half-size kernel, of 256 for the other)."""
    import random
    rnd = random.Random(seed)
    heads = [(4, 4), (4, 2), (8, 2), (4, 1), (16, 4), (3, 3), (6, 3), (32, 8), (5, 1), (12, 2), (2, 2), (1, 1)]
    cases = []
    for _ in range(n):
        H, Hkv = rnd.choice(heads)
        S = rnd.choice([rnd.randint(1, 300), rnd.randint(300, 3000), 64 * rnd.randint(1, 40), rnd.randint(3000, 6000)])
        B = 1 if S * H > 48000 else rnd.choice([1, 2, 3])
        kind = rnd.choice(["scatter", "gather1", "window", "block_scatter", "window_sink"])
        if kind == "scatter":
            kw = dict(group_num=rnd.choice([1, 2, 3, 4, 5, 7, 8, 13, 16]))
        elif kind == "gather1":
            S = 64 * max(1, S // 64)
            kw = dict(group_num=8)
        elif kind == "window":
            kw = dict(window=rnd.choice([64, 65, 128, 576, 1000, 4000, rnd.randint(64, 3000)]))
        elif kind == "block_scatter":
            G = rnd.choice([1, 2, 3, 4])
            off = rnd.randrange(G)
            blk = 256 * rnd.choice([1, 1, 2]) if (off or (H // Hkv) % 4) else 64 * rnd.choice([1, 2, 4, 8])
            kw = dict(group_num=G, block=blk, offset=off, n_sink=rnd.choice([0, 1, 64, blk, rnd.randint(0, blk)]))
        else:
            kw = dict(window=rnd.choice([1, 2, 63, 64, 575, 2000, rnd.randint(1, 1500)]),
                      n_sink=rnd.choice([0, 1, 64, 100, 700, rnd.randint(0, 500)]))
        cases.append((kind, B, S, H, Hkv, kw, rnd.choice([None, None, 0.05, -0.11, 0.2])))
    return cases


@pytest.mark.parametrize("case", _random_cases(120, seed=5), ids=lambda c: f"{c[0]}-S{c[2]}-H{c[3]}/{c[4]}")
def test_random_shapes_with_either_size(waves, case):
    """Whole outputs and log-sum-exps against the oracle, for a plain call and for each size by name."""
    kind, B, S, H, Hkv, kw, scale = case
    q, k, v = make_qkv(B, S, H, Hkv, seed=S + 7 * H)
    ref = oracle.masked_lse_rows(q, k, oracle.mask_rows(f"llm/{kind}", S, device=DEV, **kw), softmax_scale=scale)
    for n in (None, 4, 8):
        waves(n)
        with torch.no_grad():
            out, lse = intra_llm_attn(q, k, v, kind, softmax_scale=scale, return_lse=True, **kw)
        check(out, q, k, v, f"llm/{kind}", None, scale, True, f"{kind} S={S} H={H}/{Hkv} waves={n}", **kw)
        assert (lse - ref).abs().max().item() <= 5e-3


@pytest.mark.parametrize("width", [64, 128])
@pytest.mark.parametrize("pattern", ["scatter", "gather0"])
def test_image_patterns_with_either_size(waves, pattern, width):
    S = 512 + width * width
    q, k, v = make_qkv(1, S, 6, 6, seed=width)
    rows = torch.unique(torch.cat([torch.randperm(S, generator=torch.Generator().manual_seed(width))[:512],
                                   torch.arange(0, 520, 7), torch.tensor([S - 1])])).to(DEV)
    outs = {}
    for n in (8, 4):
        waves(n)
        with torch.no_grad():
            outs[n] = intra_image_attn(q, k, v, pattern, width)
        check(outs[n], q, k, v, "image/" + pattern, rows, None, True, f"{pattern} {width} waves={n}", width=width)
    if pattern == "scatter":
        assert torch.equal(outs[8], outs[4])


def _random_image_cases(n, seed):
    import random
    rnd = random.Random(seed)
    heads = [(4, 4), (4, 2), (8, 2), (4, 1), (3, 3), (6, 3), (24, 24), (5, 1), (2, 2), (1, 1), (6, 1)]
    cases = []
    for _ in range(n):
        H, Hkv = rnd.choice(heads)
        width = 8 * rnd.choice([2, 3, 4, 5, 6, 7, 8, 8, 9, 10, 12])
        text_len = 8 * rnd.choice([1, 2, 4, 8, 9, 12, 25, 32, 64, 64, 33, 100])
        cases.append((rnd.choice([("scatter", 0), ("gather0", 4)]), width, text_len, rnd.choice([1, 2]), H, Hkv,
                      rnd.choice([128 ** -0.5, 0.05, -0.11])))
    return cases


@pytest.mark.parametrize("case", _random_image_cases(40, seed=6), ids=lambda c: f"{c[0][0]}-W{c[1]}-T{c[2]}-H{c[4]}/{c[5]}")
def test_random_image_shapes_with_either_size_and_their_gradients(waves, case):
    """Grids of 16 - 96 tokens a side and 8 - 800 text tokens through the C ABI: outputs and
    log-sum-exps of each size against the oracle, then the backward of the plain call's result."""
    from test_backward_gpu import compare
    (pattern, pid), width, text_len, B, H, Hkv, scale = case
    lib = _lib.load()
    S = text_len + width * width
    g = torch.Generator(device="cpu").manual_seed(S + H)
    mk = lambda h: torch.randn(B, S, h, 128, generator=g, dtype=torch.float32).to(torch.bfloat16).to(DEV)
    q, k, v, dout = mk(H), mk(Hkv), mk(Hkv), mk(H)
    stream = torch.cuda.current_stream().cuda_stream
    mask = oracle.mask_rows(f"image/{pattern}", S, device=DEV, width=width, text_len=text_len)
    ref_lse = oracle.masked_lse_rows(q, k, mask, softmax_scale=scale)
    for n in (8, 4, None):
        waves(n)
        out = torch.full_like(q, float("nan"))
        lse = torch.full((B, H, S), float("nan"), dtype=torch.float32, device=DEV)
        rc = lib.intra_image_fwd_lse(q.data_ptr(), k.data_ptr(), v.data_ptr(), out.data_ptr(), B, S, H, Hkv,
                                     _lib.strides3(q), _lib.strides3(k), _lib.strides3(v), _lib.strides3(out),
                                     pid, width, text_len, scale, stream, lse.data_ptr(), _lib.strides3(lse))
        assert rc == 0, _lib.last_error()
        torch.cuda.synchronize()
        check(out, q, k, v, f"image/{pattern}", None, scale, True, f"{pattern} W={width} T={text_len} waves={n}",
              width=width, text_len=text_len)
        assert (lse - ref_lse).abs().max().item() <= 5e-3
    nws = lib.intra_image_bwd_workspace(B, S, H, Hkv, pid, width, text_len)
    work = torch.full((nws + 64,), float("nan"), dtype=torch.float32, device=DEV)
    dq, dk, dv = (torch.full_like(t, float("nan")) for t in (q, k, v))
    rc = lib.intra_image_bwd(q.data_ptr(), k.data_ptr(), v.data_ptr(), out.data_ptr(), lse.data_ptr(), dout.data_ptr(),
                             dq.data_ptr(), dk.data_ptr(), dv.data_ptr(), work.data_ptr(), B, S, H, Hkv,
                             _lib.strides3(q), _lib.strides3(k), _lib.strides3(v), _lib.strides3(out), _lib.strides3(dout),
                             _lib.strides3(dq), _lib.strides3(dk), _lib.strides3(dv), _lib.strides3(lse),
                             pid, width, text_len, scale, stream)
    assert rc == 0, _lib.last_error()
    torch.cuda.synchronize()
    assert bool(torch.isnan(work[nws:]).all()), "wrote past the workspace"
    compare((dq, dk, dv), oracle.masked_attention_grads(q, k, v, dout, mask, softmax_scale=scale),
            f"image/{pattern} W={width} T={text_len}")


def test_the_plan_names_what_a_plain_call_runs(waves):
    lib = _lib.load()
    plan = _lib.IntraPlan()
    waves(None)
    assert lib.intra_plan(1, 4, 1, 4608, 24, 24, 64, 512, plan) == 0 and plan.waves == 4   # image gather0
    assert lib.intra_plan(0, 0, 1, 32768, 32, 8, 8, 576, plan) == 0 and plan.waves == 8   # the headline shape
    assert lib.intra_plan(0, 0, 1, 1024, 32, 8, 8, 576, plan) == 0 and plan.waves == 4    # 128 row blocks of 64 positions
    waves(8)
    assert lib.intra_plan(1, 4, 1, 4608, 24, 24, 64, 512, plan) == 0 and plan.waves == 8
    waves(4)
    assert lib.intra_plan(0, 0, 1, 32768, 32, 8, 8, 576, plan) == 0 and plan.waves == 4
