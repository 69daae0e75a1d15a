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
