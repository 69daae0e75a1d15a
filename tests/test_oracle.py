"""Pins the CPU oracle (oracle/) without the reference on the path.

Each check is independent of the oracle's own formulas: loop constructions written from the
prose description of a pattern, the known answers and invariants that the reference's self-check
holds (intra_attn/reference.py:86-103), the mask densities its FLUX mask test prints
(experiments/flux/test_masks.py:126-134: 22.2 % / 17.3 %), a float64 triple loop, and torch's
scaled_dot_product_attention, which is the library routine the reference's oracle consists of.
"""
import math

import pytest
import torch
import torch.nn.functional as F

import oracle
from oracle import masks, pairs


# ------------------------------------------------------------------ LLM masks
@pytest.mark.parametrize("S,G", [(32, 4), (37, 3), (64, 8), (100, 8), (5, 8), (50, 1), (33, 2)])
def test_llm_scatter_bruteforce(S, G):
    m = masks.llm_scatter_mask(S, G)
    for a in range(S):
        for b in range(S):
            assert bool(m[a, b]) == (b <= a and a % G == b % G)


@pytest.mark.parametrize("S,G", [(257, 8), (100, 3), (64, 2), (9, 16), (40, 1)])
def test_llm_scatter_by_dealing(S, G):
    # built from the prose, without the predicate: deal the tokens round-robin into G piles, in
    # order; a token attends to the tokens that lie below it in its own pile and to itself.  Row
    # counts follow: token i has i // G tokens below it.
    piles = [[] for _ in range(G)]
    want = torch.zeros(S, S, dtype=torch.bool)
    for token in range(S):
        pile = piles[token % len(piles)]
        pile.append(token)
        want[token, pile] = True
    m = masks.llm_scatter_mask(S, G)
    assert torch.equal(m, want)
    assert m.sum(1).tolist() == [i // G + 1 for i in range(S)]
    assert not bool(torch.triu(m, 1).any())                       # causal
    assert int(m.sum()) == sum(len(p) * (len(p) + 1) // 2 for p in piles)
    # Gather 1 with segments of one token is the same dealing
    if G > 1:
        assert torch.equal(masks.llm_block_scatter_mask(S, G, 1, 0, 0), want)


@pytest.mark.parametrize("S,G", [(32, 4), (128, 8), (64, 8), (70, 3), (200, 8)])
def test_llm_gather1_bruteforce(S, G):
    m = masks.llm_gather1_mask(S, G)
    for a in range(S):
        for b in range(S):
            assert bool(m[a, b]) == (b <= a and (a // G) % G == (b // G) % G)


def test_llm_gather1_by_segments():
    # built from the prose: cut the sequence into segments of G tokens, deal segments to groups
    # round-robin, attend causally inside a group
    S, G = 256, 8
    group_of = []
    for seg in range(math.ceil(S / G)):
        group_of += [seg % G] * G
    m = masks.llm_gather1_mask(S, G)
    for a in range(S):
        for b in range(S):
            assert bool(m[a, b]) == (b <= a and group_of[a] == group_of[b])


def test_llm_window_known_answers():
    # reference.py:93-94
    m = masks.llm_window_mask(200, window=96, block=64)
    assert m[130, 128 - 32] and not m[130, 128 - 33] and m[63, 0] and not m[10, 11]


@pytest.mark.parametrize("S,W", [(200, 96), (1000, 576), (700, 64), (300, 1000), (640, 130)])
def test_llm_window_by_blocks(S, W):
    # prose: a block of 64 queries sees itself (causally) and the W - 64 tokens before the block
    want = torch.zeros(S, S, dtype=torch.bool)
    for b0 in range(0, S, 64):
        first = max(b0 - (W - 64), 0)
        for i in range(b0, min(b0 + 64, S)):
            want[i, first:i + 1] = True
    assert torch.equal(masks.llm_window_mask(S, W), want)


def test_llm_window_key_counts():
    # rows far enough in see between W-63 and W keys
    S, W = 4096, 576
    cnt = masks.llm_window_mask(S, W).sum(1)
    assert cnt[W:].min() == W - 63 and cnt.max() == W
    assert cnt[0] == 1 and cnt[63] == 64


# ------------------------------------------------------------------ image masks
def _loop_image_scatter(W, T):
    S = T + W * W
    grp = [t // (T // 8) for t in range(T)]
    for r in range(W):
        for c in range(W):
            grp.append((r % 2) * 4 + c % 4)
    want = torch.zeros(S, S, dtype=torch.bool)
    members = [[p for p in range(T, S) if grp[p] == g] for g in range(8)]
    for i in range(S):
        want[i, :T] = True
        want[i, members[grp[i]]] = True
    return want


def _loop_image_gather0(W, T):
    S = T + W * W
    want = _loop_image_scatter(W, T)
    n = W // 8
    for R in range(n):
        for C in range(n):
            def first(idx):
                if idx == 0:
                    return 0
                if idx == n - 1:
                    return 8 * idx - 8
                return 8 * idx - 4
            r0, c0 = first(R), first(C)
            keys = [T + r * W + c for r in range(r0, r0 + 16) for c in range(c0, c0 + 16)]
            for r in range(8 * R, 8 * R + 8):
                for c in range(8 * C, 8 * C + 8):
                    i = T + r * W + c
                    want[i] = False
                    want[i, :T] = True
                    want[i, keys] = True
    return want


@pytest.mark.parametrize("W,T", [(16, 64), (32, 512), (24, 16)])
def test_image_masks_by_loops_small(W, T):
    assert torch.equal(masks.image_scatter_mask(W, T), _loop_image_scatter(W, T))
    assert torch.equal(masks.image_gather0_mask(W, T), _loop_image_gather0(W, T))


def test_image_masks_by_loops_flux_1024():
    assert torch.equal(masks.image_scatter_mask(64), _loop_image_scatter(64, 512))
    assert torch.equal(masks.image_gather0_mask(64), _loop_image_gather0(64, 512))


def test_image_invariants_reference_selfcheck():
    # reference.py:95-102
    W, T = 64, masks.TEXT_LEN
    m = masks.image_scatter_mask(W)
    assert m.shape == (T + W * W,) * 2 and m[:, :T].all()
    assert m[T:, T:].sum(1).eq(W * W // 8).all()
    m = masks.image_gather0_mask(W)
    assert m[T:, T:].sum(1).eq(256).all()
    q = T + 9 * W + 9  # patch (1, 1) -> window rows/cols 4..19
    assert m[q, T + 4 * W + 4] and not m[q, T + 3 * W + 4] and m[q, T + 19 * W + 19]
    assert not m[q, T + 20 * W + 19] and not m[q, T + 4 * W + 3]


def test_image_densities_published():
    # experiments/flux/test_masks.py prints density 0.2222 (scatter) and 0.1728 (gather0) at W=64
    assert abs(masks.image_scatter_mask(64).float().mean().item() - 0.2222) < 5e-5
    assert abs(masks.image_gather0_mask(64).float().mean().item() - 0.1728) < 5e-5


def test_image_w128_invariants():
    W, T = 128, 512
    rows = torch.cat([torch.arange(0, T, 37), T + torch.arange(0, W * W, 251)])
    ms = masks.image_scatter_mask(W, rows=rows)
    assert ms[:, :T].all() and ms[:, T:].sum(1).eq(W * W // 8).all()
    mg = masks.image_gather0_mask(W, rows=rows)
    is_text = rows < T
    assert mg[is_text][:, T:].sum(1).eq(W * W // 8).all()
    assert mg[~is_text][:, T:].sum(1).eq(256).all()
    # last patch (15, 15): window rows/cols 112..127
    q = T + 127 * W + 127
    row = masks.image_gather0_mask(W, rows=torch.tensor([q]))[0]
    assert row[T + 112 * W + 112] and not row[T + 111 * W + 112] and row[T + 127 * W + 127]


@pytest.mark.parametrize("kind,S,kw", [
    ("llm/scatter", 1000, dict(group_num=3)), ("llm/gather1", 1024, dict(group_num=8)),
    ("llm/window", 1000, dict(window=576)), ("image/scatter", 64 + 256, dict(width=16, text_len=64)),
    ("image/gather0", 512 + 1024, dict(width=32))])
def test_row_subset_equals_full(kind, S, kw):
    full = masks.mask_rows(kind, S, **kw)
    rows = torch.tensor([0, 1, 63, 64, S // 2, S - 2, S - 1])
    assert torch.equal(masks.mask_rows(kind, S, rows=rows, **kw), full[rows])


# ------------------------------------------------------------------ pair counts
@pytest.mark.parametrize("kind,S,kw", [
    ("llm/scatter", 1000, dict(group_num=3)), ("llm/scatter", 2048, dict(group_num=8)),
    ("llm/gather1", 1024, dict(group_num=8)), ("llm/gather1", 1000, dict(group_num=8)),
    ("llm/window", 1000, dict(window=576)), ("llm/window", 3000, dict(window=1000)),
    ("image/scatter", 4608, dict(width=64)), ("image/gather0", 4608, dict(width=64))])
def test_pair_counts_equal_mask_sums(kind, S, kw):
    assert pairs.pairs_per_head(kind, S, **kw) == int(masks.mask_rows(kind, S, **kw).sum())


def test_pair_counts_headline():
    assert pairs.pairs_per_head("llm/scatter", 32768, group_num=8) == 8 * (4096 * 4097 // 2) == 67125248
    assert pairs.pairs_per_head("image/scatter", 16896, width=128) == 16896 * (512 + 2048)


# ------------------------------------------------------------------ attention
def _rand(B, S, H, Hkv, D, seed):
    g = torch.Generator().manual_seed(seed)
    q = torch.randn(B, S, H, D, generator=g).to(torch.bfloat16)
    k = torch.randn(B, S, Hkv, D, generator=g).to(torch.bfloat16)
    v = torch.randn(B, S, Hkv, D, generator=g).to(torch.bfloat16)
    return q, k, v


def test_attention_vs_float64_loops():
    B, S, H, Hkv, D = 1, 24, 4, 2, 8
    q, k, v = _rand(B, S, H, Hkv, D, 1)
    q, k, v = q.float(), k.float(), v.float()
    mask = masks.llm_scatter_mask(S, 3)
    got = oracle.masked_attention(q, k, v, mask, softmax_scale=0.3)
    for h in range(H):
        kh = h // (H // Hkv)
        for i in range(S):
            js = [j for j in range(S) if mask[i, j]]
            sc = [0.3 * sum(float(q[0, i, h, d]) * float(k[0, j, kh, d]) for d in range(D)) for j in js]
            mx = max(sc)
            w = [math.exp(s - mx) for s in sc]
            z = sum(w)
            for d in range(D):
                want = sum(wi * float(v[0, j, kh, d]) for wi, j in zip(w, js)) / z
                assert abs(float(got[0, i, h, d]) - want) < 1e-5


@pytest.mark.parametrize("B,S,H,Hkv,kind,kw", [
    (1, 1024, 4, 1, "llm/scatter", dict(group_num=8)),   # the reference's CPU-runnable configuration
    (2, 300, 6, 2, "llm/window", dict(window=100)),
    (1, 320, 3, 3, "image/gather0", dict(width=16, text_len=64))])
def test_attention_vs_torch_sdpa(B, S, H, Hkv, kind, kw):
    # same call shape as reference.py:78-83
    q, k, v = _rand(B, S, H, Hkv, 128, 0)
    mask = masks.mask_rows(kind, S, **kw)
    got = oracle.masked_attention(q, k, v, mask)
    qf, kf, vf = (x.float().transpose(1, 2) for x in (q, k, v))
    ref = F.scaled_dot_product_attention(qf, kf, vf, attn_mask=mask, enable_gqa=H != Hkv)
    ref = ref.transpose(1, 2).to(q.dtype)
    assert got.dtype == q.dtype and got.shape == q.shape
    assert (got.float() - ref.float()).abs().max().item() <= 2 ** -8  # one bf16 ulp at |x| < 1


def test_attention_rows_subset_and_scale():
    q, k, v = _rand(1, 200, 4, 2, 128, 3)
    mask = masks.llm_scatter_mask(200, 2)
    full = oracle.masked_attention(q, k, v, mask, softmax_scale=0.05)
    rows = torch.tensor([0, 7, 64, 199])
    sub = oracle.masked_attention_rows(q, k, v, mask[rows], rows, softmax_scale=0.05)
    assert torch.equal(sub, full[:, rows])
    assert not torch.equal(full, oracle.masked_attention(q, k, v, mask))


def test_lse_is_the_log_of_the_softmax_denominator():
    # float64 loop on a tiny case: lse_i = log sum_j exp(scale * q_i.k_j) over visible j, and
    # softmax weights rebuilt from it reproduce masked_attention
    g = torch.Generator().manual_seed(5)
    B, S, H, Hkv, D = 1, 40, 4, 2, 128
    q = torch.randn(B, S, H, D, generator=g)
    k = torch.randn(B, S, Hkv, D, generator=g)
    v = torch.randn(B, S, Hkv, D, generator=g)
    mask = oracle.llm_scatter_mask(S, 3)
    lse = oracle.masked_lse_rows(q, k, mask, softmax_scale=0.11)
    assert lse.shape == (B, H, S) and lse.dtype == torch.float32
    out = oracle.masked_attention(q, k, v, mask, softmax_scale=0.11)
    for h in range(H):
        for i in (0, 1, 7, 39):
            acc, o = 0.0, torch.zeros(D, dtype=torch.float64)
            for j in range(S):
                if mask[i, j]:
                    w = math.exp(0.11 * float(q[0, i, h].double() @ k[0, j, h // 2].double()))
                    acc += w
                    o += w * v[0, j, h // 2].double()
            assert abs(math.log(acc) - lse[0, h, i].item()) < 1e-4
            assert (o / acc - out[0, i, h].double()).abs().max() < 1e-4
    rows = torch.tensor([3, 17])
    sub = oracle.masked_lse_rows(q, k, mask[rows], rows, softmax_scale=0.11)
    assert torch.allclose(sub, lse[:, :, rows])


# ------------------------------------------------------------------ block scatter / window with sinks
def _loop_block_scatter(S, G, blk, off, ns):
    m = torch.zeros(S, S, dtype=torch.bool)
    for i in range(S):
        for j in range(i + 1):
            same_class = (j // blk) % G == ((i // blk) + off) % G
            m[i, j] = same_class or (off != 0 and j // blk == i // blk) or j < ns
    return m


@pytest.mark.parametrize("S,G,blk,off,ns", [(70, 2, 16, 0, 0), (70, 2, 16, 1, 5), (90, 3, 8, 2, 8), (50, 4, 4, 0, 3)])
def test_block_scatter_mask_brute_force(S, G, blk, off, ns):
    assert torch.equal(masks.llm_block_scatter_mask(S, G, blk, off, ns), _loop_block_scatter(S, G, blk, off, ns))


def test_block_scatter_reduces_to_scatter_and_gather1():
    for S, G in ((100, 2), (257, 3), (1000, 8)):
        assert torch.equal(masks.llm_block_scatter_mask(S, G, 1, 0, 0), masks.llm_scatter_mask(S, G))
        assert torch.equal(masks.llm_block_scatter_mask(S, G, G, 0, 0), masks.llm_gather1_mask(S, G))
    assert torch.equal(masks.llm_block_scatter_mask(300, 1, 64, 0, 0), torch.ones(300, 300).tril().bool())


def test_block_scatter_offsets_partition_the_earlier_blocks():
    # every key block in front of a query block is read at exactly one offset; the own block is read
    # at every offset; sinks add nothing once block 0 is visible
    S, G, blk = 640, 4, 64
    ms = [masks.llm_block_scatter_mask(S, G, blk, off, 0) for off in range(G)]
    total = sum(m.to(torch.int32) for m in ms)
    qb = torch.arange(S)[:, None] // blk
    kb = torch.arange(S)[None, :] // blk
    causal = torch.ones(S, S).tril().bool()
    assert torch.equal(total[(kb < qb)], torch.ones_like(total[(kb < qb)]))
    assert torch.equal(total[(kb == qb) & causal], torch.full_like(total[(kb == qb) & causal], G))
    assert int(total[~causal].sum()) == 0
    for off in range(G):
        with_sinks = masks.llm_block_scatter_mask(S, G, blk, off, 48)
        extra = with_sinks & ~ms[off]
        assert bool((extra.nonzero()[:, 1] < 48).all()) and torch.equal(with_sinks | ms[off], with_sinks)
        assert bool(with_sinks.any(dim=1).all())  # no empty row


def test_block_scatter_equals_gathered_group_attention_with_sinks():
    """The reference builds the same layer a second way (llama_intra.py:124-165): per group, gather
    the group's tokens, put the sink tokens in front of the key list (dropping them from the
    group's own part) and run causal attention in original positions.  Restated here with plain
    softmax; it must agree with masked attention under llm_block_scatter_mask at offset 0."""
    g = torch.Generator().manual_seed(9)
    B, S, H, Hkv, D, G, blk, ns = 1, 300, 2, 1, 128, 2, 64, 20
    q = torch.randn(B, S, H, D, generator=g)
    k = torch.randn(B, S, Hkv, D, generator=g)
    v = torch.randn(B, S, Hkv, D, generator=g)
    ref = oracle.masked_attention(q, k, v, masks.llm_block_scatter_mask(S, G, blk, 0, ns), softmax_scale=0.1)
    out = torch.zeros_like(q)
    pos = torch.arange(S)
    gid = (pos // blk) % G
    for grp in range(G):
        idx = pos[gid == grp]
        kv = torch.cat([pos[:ns], idx[idx >= ns]])
        allowed = kv[None, :] <= idx[:, None]
        for h in range(H):
            s = (q[0, idx, h].double() @ k[0, kv, 0].double().T) * 0.1
            s = s.masked_fill(~allowed, float("-inf"))
            out[0, idx, h] = (torch.softmax(s, -1) @ v[0, kv, 0].double()).float()
    assert (out - ref).abs().max() < 1e-5


def test_window_sink_mask_special_cases_and_counts():
    S = 300
    tril = torch.ones(S, S).tril().bool()
    assert torch.equal(masks.llm_window_sink_mask(S, S, 0), tril)
    assert torch.equal(masks.llm_window_sink_mask(S, 5000, 7), tril)
    assert torch.equal(masks.llm_window_sink_mask(S, 1, 0), torch.eye(S).bool())
    for W, ns in ((575, 64), (100, 37), (64, 64), (1, 5), (17, 0)):
        m = masks.llm_window_sink_mask(S, W, ns)
        assert not bool((m & ~tril).any())
        rows = m.sum(1)
        want = torch.tensor([min(i + 1, W) + max(0, min(ns, i + 1 - W)) for i in range(S)])
        assert torch.equal(rows, want)
        # the window part is a band, the rest sits in the first ns columns
        i = torch.arange(S)[:, None]
        j = torch.arange(S)[None, :]
        band = (j <= i) & (j > i - W)
        assert torch.equal(m & band, band) and bool(((m & ~band).nonzero()[:, 1] < ns).all())
    m = masks.llm_window_sink_mask(200, 96, 4)
    assert m[130, 35] and not m[130, 34] and m[130, 3] and not m[130, 4] and m[2, 2] and not m[2, 3]


def test_new_pair_counts_match_masks():
    for S in (1, 100, 777):
        for kw in (dict(group_num=2, block=64, offset=0, n_sink=0), dict(group_num=2, block=64, offset=1, n_sink=20),
                   dict(group_num=3, block=128, offset=2, n_sink=128), dict(group_num=4, block=64, offset=0, n_sink=9)):
            assert pairs.pairs_per_head("llm/block_scatter", S, **kw) == int(oracle.mask_rows("llm/block_scatter", S, **kw).sum())
        for kw in (dict(window=575, n_sink=64), dict(window=10, n_sink=3), dict(window=1, n_sink=0)):
            assert pairs.pairs_per_head("llm/window_sink", S, **kw) == int(oracle.mask_rows("llm/window_sink", S, **kw).sum())
    rows = torch.tensor([0, 5, 99])
    assert torch.equal(oracle.mask_rows("llm/window_sink", 100, rows=rows, window=10, n_sink=3),
                       masks.llm_window_sink_mask(100, 10, 3)[rows])


def test_reference_known_answers():
    """tests/golden/reference_known_answers.json: every point, count and density the reference
    asserts or prints about its own masks."""
    import json
    import os
    path = os.path.join(os.path.dirname(__file__), "golden", "reference_known_answers.json")
    data = json.load(open(path))
    for entry in data["masks"]:
        m = oracle.mask_rows(entry["kind"], entry["S"], **entry["args"])
        for q, k in entry.get("true", []):
            assert bool(m[q, k]), (entry["source"], q, k)
        for q, k in entry.get("false", []):
            assert not bool(m[q, k]), (entry["source"], q, k)
        if "all_true_columns_below" in entry:
            assert bool(m[:, :entry["all_true_columns_below"]].all())
        if "grid_keys_per_grid_row" in entry:
            T = oracle.TEXT_LEN
            assert bool(m[T:, T:].sum(1).eq(entry["grid_keys_per_grid_row"]).all())
        if "density_percent" in entry:
            assert round(100.0 * m.float().mean().item(), 2) == entry["density_percent"]
    for entry in data["brute_force"]:
        S, G = entry["S"], entry["args"]["group_num"]
        m = oracle.mask_rows(entry["kind"], S, **entry["args"])
        for q in range(S):
            for k in range(S):
                assert bool(m[q, k]) == bool(eval(entry["rule"], {"q": q, "k": k, "G": G}))
    for entry in data["pairs"]:
        assert pairs.pairs_per_head(entry["kind"], entry["S"], **entry["args"]) == entry["pairs_per_head"]


# ---------------------------------------------------------------------------- gradients
def _tiny_problem(seed, S=12, H=4, Hkv=2, D=8):
    g = torch.Generator().manual_seed(seed)
    mk = lambda h: torch.randn(1, S, h, D, generator=g, dtype=torch.float64)
    return mk(H), mk(Hkv), mk(Hkv), mk(H)


def test_grads_match_finite_differences():
    # central differences of the scalar sum(O * dout) in float64, every input element
    q, k, v, dout = _tiny_problem(3, S=6, H=2, Hkv=1, D=4)
    mask = masks.llm_scatter_mask(6, 2)
    grads = oracle.masked_attention_grads(q, k, v, dout, mask, dtype=torch.float64)
    sdpa = lambda a, b, c: F.scaled_dot_product_attention(a.transpose(1, 2), b.transpose(1, 2), c.transpose(1, 2),
                                                          attn_mask=mask, enable_gqa=True).transpose(1, 2)
    f = lambda a, b, c: (sdpa(a, b, c) * dout).sum().item()  # the library routine, in float64
    eps = 1e-5
    for which, (x, gx) in enumerate(zip((q, k, v), grads)):
        flat = x.reshape(-1)
        for i in range(flat.numel()):
            old = flat[i].item()
            flat[i] = old + eps
            up = f(q, k, v)
            flat[i] = old - eps
            dn = f(q, k, v)
            flat[i] = old
            assert abs((up - dn) / (2 * eps) - gx.reshape(-1)[i].item()) < 1e-6, (which, i)


def test_grads_match_the_softmax_jacobian_formulas():
    # dV = P^T dO, dS = P o (dP - rowsum(dO o O)), dQ = scale dS K, dK = scale dS^T Q, in plain loops
    q, k, v, dout = _tiny_problem(5)
    S, H, Hkv, D = 12, 4, 2, 8
    mask = masks.llm_window_mask(S, 4) | torch.eye(S, dtype=torch.bool)
    scale = 0.3
    dq, dk, dv = oracle.masked_attention_grads(q, k, v, dout, mask, softmax_scale=scale, dtype=torch.float64)
    eq, ek, ev = torch.zeros_like(q), torch.zeros_like(k), torch.zeros_like(v)
    for h in range(H):
        kv = h // (H // Hkv)
        for i in range(S):
            js = [j for j in range(S) if mask[i, j]]
            s = torch.tensor([scale * float(q[0, i, h] @ k[0, j, kv]) for j in js], dtype=torch.float64)
            p = torch.exp(s - torch.logsumexp(s, 0))
            o = sum(p[n] * v[0, j, kv] for n, j in enumerate(js))
            dsum = float(dout[0, i, h] @ o)
            for n, j in enumerate(js):
                ev[0, j, kv] += p[n] * dout[0, i, h]
                ds = p[n] * (float(dout[0, i, h] @ v[0, j, kv]) - dsum)
                eq[0, i, h] += scale * ds * k[0, j, kv]
                ek[0, j, kv] += scale * ds * q[0, i, h]
    for got, want in ((dq, eq), (dk, ek), (dv, ev)):
        assert (got - want).abs().max().item() < 1e-10


def test_grads_of_one_key_rows_have_a_closed_form():
    # a query that sees a single key has P = 1: dV gets dO, dQ and dK get nothing
    q, k, v, dout = _tiny_problem(7, H=2, Hkv=2)
    mask = torch.eye(12, dtype=torch.bool)
    dq, dk, dv = oracle.masked_attention_grads(q, k, v, dout, mask, dtype=torch.float64)
    assert dq.abs().max().item() < 1e-12 and dk.abs().max().item() < 1e-12
    assert (dv - dout).abs().max().item() < 1e-12
