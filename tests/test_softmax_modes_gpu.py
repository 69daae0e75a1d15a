"""The two softmax arithmetics of the forward kernels (EXACT: fp32 scaling and a watched running
maximum, the reference's csrc/flash_attn/src/softmax.h:65-91; FAST: scale folded into bf16 Q, no
maximum, out-of-range queries recomputed exactly) against the fp32 dense-mask oracle:

* on both sides of the scale gate of the automatic mode,
* on inputs whose scores leave the +-60 exponent band that both modes treat specially: whole
  blocks far below it before anything was accumulated, blocks far above it later on, for queries
  whose two half-wavefront lanes see different numbers of keys (windows with window % 32 in 1..4,
  0 or 1 sink tokens), with the log-sum-exp checked as well.

Tolerance: the parity bar of the reference, max-abs 1.6e-2 on bf16 outputs; lse within 1e-2 + 2e-3
relative (it sums bf16-rounded weights).  The inputs built to leave the band give rows that one key
dominates, so outputs are single V rows of magnitude up to 5, where one bf16 ulp is 3.1e-2: those
tests allow one ulp (2^-7 relative) on top, since kernel and oracle round their results separately."""
import pytest
import torch

import oracle
import intra_amd
from intra_amd import intra_image_attn, intra_llm_attn

pytestmark = pytest.mark.gpu
ATOL = 1.6e-2
DEV = "cuda"


@pytest.fixture(autouse=True)
def _restore_mode():
    start = intra_amd.get_softmax_mode()
    yield
    intra_amd.set_softmax_mode(start)


def make_qkv(B, S, H, Hkv, seed=0):
    g = torch.Generator(device="cpu").manual_seed(seed)
    mk = lambda h: torch.randn(B, S, h, 128, generator=g, dtype=torch.float32)
    return mk(H), mk(Hkv), mk(Hkv)


def to_dev(*ts):
    return [t.to(torch.bfloat16).to(DEV) for t in ts]


def run(kind, q, k, v, scale, **kw):
    with torch.no_grad():
        if kind.startswith("image/"):
            return intra_image_attn(q, k, v, kind.split("/")[1], kw["width"], softmax_scale=scale, return_lse=True)
        return intra_llm_attn(q, k, v, kind.split("/")[1], softmax_scale=scale, return_lse=True, **kw)


def check(kind, q, k, v, scale=None, tag="", rtol=0.0, **kw):
    out, lse = run(kind, q, k, v, scale, **kw)
    S = q.shape[1]
    mask = oracle.mask_rows(kind, S, device=DEV, **kw)
    ref = oracle.masked_attention_rows(q, k, v, mask, None, softmax_scale=scale)
    assert bool(torch.isfinite(out).all()), f"{tag} {kind} {kw}: non-finite output"
    diff = (out.float() - ref.float()).abs()
    err = diff.max().item()
    assert bool((diff <= ATOL + rtol * ref.float().abs()).all()), f"{tag} {kind} {kw} scale={scale}: max|err|={err:.3e}"
    want = oracle.masked_lse_rows(q, k, mask, None, softmax_scale=scale)
    lerr = (lse - want).abs()
    assert bool((lerr <= 1e-2 + 2e-3 * want.abs()).all()), f"{tag} {kind} {kw}: lse err {lerr.max().item():.3e}"
    return err


CASES = [("llm/scatter", dict(group_num=8), 2048, 8, 2), ("llm/scatter", dict(group_num=3), 1000, 4, 4),
         ("llm/gather1", dict(group_num=8), 1024, 4, 1), ("llm/window", dict(window=576), 2048, 8, 2),
         ("llm/window", dict(window=100), 1000, 2, 1),
         ("llm/window_sink", dict(window=63, n_sink=0), 1000, 4, 2), ("llm/window_sink", dict(window=63, n_sink=1), 1000, 4, 2),
         ("llm/window_sink", dict(window=575, n_sink=64), 2048, 4, 1),
         ("llm/block_scatter", dict(group_num=2, block=256, offset=1, n_sink=64), 2048, 4, 1),
         ("image/scatter", dict(width=64), 4608, 4, 4), ("image/gather0", dict(width=64), 4608, 4, 2)]


@pytest.mark.parametrize("scale", [None, 0.3, -0.07, 0.17, 0.18, 0.0])
@pytest.mark.parametrize("kind,kw,S,H,Hkv", CASES)
def test_auto_mode_on_both_sides_of_the_scale_gate(kind, kw, S, H, Hkv, scale):
    q, k, v = to_dev(*make_qkv(1, S, H, Hkv, seed=S + H))
    check(kind, q, k, v, scale, **kw)


def banded_inputs(S, H, Hkv, seed):
    """N(0,1) inputs plus a shared +-1 direction u: queries of a subset of rows carry +3u, keys of
    some position ranges carry -3u or +3u.  For a marked query, scaled scores are about -147 (in
    powers of two) on the first kind of key, +147 on the second and of ordinary size elsewhere:
    early keys sit far below the band, later ones far above it, and rows that only see the first
    kind have all their weights below 2^-100."""
    q, k, v = make_qkv(2, S, H, Hkv, seed)
    g = torch.Generator(device="cpu").manual_seed(seed + 1)
    u = (torch.randint(0, 2, (128,), generator=g).float() * 2 - 1)
    pos = torch.arange(S)
    k_lo = (pos < 40) | ((pos % 256 >= 100) & (pos % 256 < 108))
    k_hi = (pos % 512 >= 300) & (pos % 512 < 305)
    q_mark = (pos % 7 == 3) | (pos < 12)
    k[:, k_lo] -= 3 * u
    k[:, k_hi] += 3 * u
    q[:, q_mark] += 3 * u
    q[:, :, 1::2] *= -1  # every other head: the signs of its scores flipped
    return to_dev(q, k, v)


@pytest.mark.parametrize("mode", ["exact", "fast", "auto"])
@pytest.mark.parametrize("kind,kw,S,H,Hkv", CASES)
def test_scores_far_outside_the_exponent_band(kind, kw, S, H, Hkv, mode):
    intra_amd.set_softmax_mode(mode)
    q, k, v = banded_inputs(S, H, Hkv, seed=S)
    check(kind, q, k, v, None, tag=mode, rtol=2.0 ** -7, **kw)


@pytest.mark.parametrize("mode", ["exact", "fast"])
@pytest.mark.parametrize("kind,kw", [("llm/window", dict(window=100)), ("llm/window_sink", dict(window=63, n_sink=1)),
                                     ("llm/scatter", dict(group_num=8)), ("image/gather0", dict(width=64))])
def test_large_scale_on_plain_inputs(kind, kw, mode):
    # softmax_scale 4 on N(0,1) inputs: scores of +-45 nats, most rows cross the band somewhere.
    # FAST is forced far outside its gate here: what it recomputes must be exact, and what it keeps
    # carries the score noise of the folded scale (about 1e-3 * |score|), hence the wider bound.
    intra_amd.set_softmax_mode(mode)
    S = 4608 if kind.startswith("image") else 1000
    q, k, v = to_dev(*make_qkv(1, S, 4, 2, seed=7))
    out, lse = run(kind, q, k, v, 4.0, **kw)
    mask = oracle.mask_rows(kind, S, device=DEV, **kw)
    ref = oracle.masked_attention_rows(q, k, v, mask, None, softmax_scale=4.0)
    assert bool(torch.isfinite(out).all()) and bool(torch.isfinite(lse).all())
    err = (out.float() - ref.float()).abs().max().item()
    assert err <= (ATOL if mode == "exact" else 0.25), f"{mode} {kind}: {err:.3e}"
    want = oracle.masked_lse_rows(q, k, mask, None, softmax_scale=4.0)
    assert bool(((lse - want).abs() <= (1e-2 if mode == "exact" else 0.3) + 2e-3 * want.abs()).all())


def test_fast_and_exact_agree_at_the_headline_scale():
    q, k, v = to_dev(*make_qkv(1, 4096, 32, 8, seed=3))
    outs = {}
    for mode in ("exact", "fast"):
        intra_amd.set_softmax_mode(mode)
        outs[mode] = run("llm/scatter", q, k, v, None, group_num=8)
    d = (outs["exact"][0].float() - outs["fast"][0].float()).abs().max().item()
    assert d <= ATOL, d
    assert (outs["exact"][1] - outs["fast"][1]).abs().max().item() <= 1e-2
