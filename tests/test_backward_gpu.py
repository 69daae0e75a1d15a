"""Parity of the backward kernels (dq, dk, dv through intra_llm_bwd of the C ABI) against the
gradients of the fp32 dense-mask oracle.  The reference has no backward kernels; what it
differentiates in training is the dense-mask attention the oracle restates
(experiments/llm/llama_intra.py:26), so that is the specification.

Tolerance, on bf16 results, per tensor with m = max|want|:
  every element  |got - want| <= m / 64 + |want| / 64
  whole tensor   ||got - want||_2 <= ||want||_2 / 128
(plus 1e-4 per element in both, for gradients that are exactly zero)
The kernels round the softmax weights and their derivatives to bf16 before the second product
(2^-9 relative each), use the forward pass's log-sum-exp (within 2^-8 of exact), form
D = dout . out from the bf16 output, and round the results to bf16 (2^-9).  The terms that add up
to one gradient element partly cancel, so an element's error scales with the tensor, not with the
element: hence the m / 64.  The norm bound is the sharp one: a dropped term, a wrong scale or a
missed key block moves it by orders of magnitude.
Observed over all comparisons of this file, test_backward_image_gpu.py and test_llama_caller_gpu.py
(477 tensors): the worst element is at (m + |want|) / 169, the worst tensor at ||want||_2 / 212, so
the two bounds sit at 2.6 and 1.7 times what occurs."""
import pytest
import torch

import oracle
from intra_amd import intra_llm_attn, intra_llm_attn_bwd, intra_llm_attn_func

pytestmark = pytest.mark.gpu
RTOL, NORM_RTOL = 1.0 / 64, 1.0 / 128
ABS_FLOOR = 1e-4  # gradients that vanish exactly (one-key rows) come out as fp32 rounding noise of dP - D
DEV = "cuda"


def make(B, S, H, Hkv, seed=0):
    g = torch.Generator(device="cpu").manual_seed(seed)
    mk = lambda h: torch.randn(B, S, h, 128, generator=g, dtype=torch.float32).to(torch.bfloat16).to(DEV)
    return mk(H), mk(Hkv), mk(Hkv), mk(H)


def kernel_grads(q, k, v, dout, pattern, scale=None, **kw):
    with torch.no_grad():
        out, lse = intra_llm_attn(q, k, v, pattern, softmax_scale=scale, return_lse=True, **kw)
        return intra_llm_attn_bwd(q, k, v, out, lse, dout, pattern, softmax_scale=scale, **kw)


def compare(got, want, what):
    for name, g, w in zip(("dq", "dk", "dv"), got, want):
        assert g.dtype == torch.bfloat16 and g.shape == w.shape
        assert bool(torch.isfinite(g).all()), f"{what} {name} not finite"
        w = w.float()
        diff = (g.float() - w).abs()
        m = w.abs().max().item()
        ok = diff <= RTOL * m + RTOL * w.abs() + ABS_FLOOR
        assert bool(ok.all()), f"{what} {name}: max|err|={diff.max().item():.3e}, max|want|={m:.3e}"
        bound = NORM_RTOL * w.norm().item() + ABS_FLOOR * w.numel() ** 0.5
        assert diff.norm().item() <= bound, f"{what} {name}: l2 error {diff.norm().item():.3e} > {bound:.3e}"


def run_case(kind, pattern, B, S, H, Hkv, seed=0, scale=None, mask_kw=None, **kw):
    q, k, v, dout = make(B, S, H, Hkv, seed)
    got = kernel_grads(q, k, v, dout, pattern, scale, **kw)
    mask = oracle.mask_rows(kind, S, device=DEV, **(mask_kw if mask_kw is not None else kw))
    want = oracle.masked_attention_grads(q, k, v, dout, mask, softmax_scale=scale)
    compare(got, want, f"{kind} S={S} H={H}/{Hkv} {kw}")


@pytest.mark.parametrize("S", [63, 777, 1024, 4096])
@pytest.mark.parametrize("G", [2, 3, 8])
@pytest.mark.parametrize("B,H,Hkv", [(1, 8, 2), (2, 4, 4), (1, 6, 3)])
def test_scatter_grads(S, G, B, H, Hkv):
    run_case("llm/scatter", "scatter", B, S, H, Hkv, group_num=G)


@pytest.mark.parametrize("S", [64, 1024, 2112])
@pytest.mark.parametrize("B,H,Hkv", [(1, 8, 2), (2, 4, 4)])
def test_gather1_grads(S, B, H, Hkv):
    run_case("llm/gather1", "gather1", B, S, H, Hkv, group_num=8)


@pytest.mark.parametrize("S,W", [(300, 64), (2000, 576), (3000, 1000), (1000, 4096)])
@pytest.mark.parametrize("B,H,Hkv", [(1, 8, 2), (2, 2, 2)])
def test_window_grads(S, W, B, H, Hkv):
    run_case("llm/window", "window", B, S, H, Hkv, window=W)


@pytest.mark.parametrize("S,G,block", [(1500, 2, 256), (1111, 3, 64), (4096, 2, 256), (700, 4, 128)])
@pytest.mark.parametrize("B,H,Hkv", [(1, 8, 2), (1, 4, 1)])
def test_block_scatter_grads(S, G, block, B, H, Hkv):
    run_case("llm/block_scatter", "block_scatter", B, S, H, Hkv, group_num=G, block=block)


def test_headline_heads_at_8k():
    run_case("llm/scatter", "scatter", 1, 8192, 32, 8, group_num=8)


def test_other_scale():
    run_case("llm/scatter", "scatter", 1, 1000, 8, 2, scale=0.05, group_num=4)


def test_strided_inputs_and_packed_qkv():
    # q, k, v as slices of one packed projection output; dout a transposed view
    B, S, H, Hkv = 1, 1024, 8, 2
    g = torch.Generator(device="cpu").manual_seed(4)
    qkv = torch.randn(B, S, H + 2 * Hkv, 128, generator=g).to(torch.bfloat16).to(DEV)
    q, k, v = qkv[:, :, :H], qkv[:, :, H:H + Hkv], qkv[:, :, H + Hkv:]
    dout = torch.randn(B, H, S, 128, generator=g).to(torch.bfloat16).to(DEV).transpose(1, 2)
    got = kernel_grads(q, k, v, dout, "scatter", group_num=8)
    want = oracle.masked_attention_grads(q, k, v, dout, oracle.llm_scatter_mask(S, 8, DEV))
    compare(got, want, "packed qkv")


def test_full_length_properties():
    """At S = 32768 (headline shape) the dense oracle is out of reach; properties that hold for
    any size: the gradients are linear in dout; dv of an all-ones dout sums the weights (every
    query's weights add to one, so the sum over keys of dv is the number of queries per kv head);
    the first token of each group sees only itself, so its weight is 1 and its dq vanishes (up to
    the fp32 rounding of dP - D, both of which equal dout . v there)."""
    B, S, H, Hkv, G = 1, 32768, 32, 8, 8
    q, k, v, dout = make(B, S, H, Hkv, seed=9)
    with torch.no_grad():
        out, lse = intra_llm_attn(q, k, v, "scatter", group_num=G, return_lse=True)
        d1 = intra_llm_attn_bwd(q, k, v, out, lse, dout, "scatter", group_num=G)
        d2 = intra_llm_attn_bwd(q, k, v, out, lse, dout * 2, "scatter", group_num=G)  # exact in bf16
        for a, b in zip(d1, d2):
            assert torch.equal(a.float() * 2, b.float())
        ones = torch.ones_like(dout)
        dq1, dk1, dv1 = intra_llm_attn_bwd(q, k, v, out, lse, ones, "scatter", group_num=G)
        total = dv1.float().sum(dim=1)  # (B, Hkv, 128): sum over keys
        assert (total / (S * H // Hkv) - 1).abs().max().item() < 4e-3
        assert d1[0][:, :G].float().abs().max().item() < 1e-3
        assert bool(torch.isfinite(dk1).all()) and bool(torch.isfinite(dq1).all())


def test_autograd_function_matches_dense_autograd():
    B, S, H, Hkv = 1, 1024, 8, 2
    q, k, v, _ = make(B, S, H, Hkv, seed=2)
    q, k, v = (t.requires_grad_(True) for t in (q, k, v))
    out = intra_llm_attn_func(q, k, v, "scatter", 8)
    w = torch.linspace(-1, 1, 128, device=DEV)
    (out.float() * w).sum().backward()
    dout = w.expand_as(out).to(torch.bfloat16)
    want = oracle.masked_attention_grads(q, k, v, dout, oracle.llm_scatter_mask(S, 8, DEV))
    compare((q.grad, k.grad, v.grad), want, "autograd")


@pytest.mark.parametrize("S,kw", [
    (2000, dict(group_num=2, block=256, offset=1, n_sink=64)),   # the LLaMA setting of the reference's model code
    (2000, dict(group_num=2, block=256, offset=0, n_sink=64)),
    (2100, dict(group_num=4, block=256, offset=3, n_sink=0)),
    (1300, dict(group_num=3, block=512, offset=2, n_sink=100)),
    (1111, dict(group_num=3, block=64, offset=0, n_sink=40)),
    (200, dict(group_num=2, block=256, offset=1, n_sink=64)),
    (4096, dict(group_num=2, block=256, offset=1, n_sink=256)),
])
@pytest.mark.parametrize("B,H,Hkv", [(1, 8, 2), (2, 2, 2)])
def test_block_scatter_offsets_and_sinks_grads(S, kw, B, H, Hkv):
    run_case("llm/block_scatter", "block_scatter", B, S, H, Hkv, **kw)


@pytest.mark.parametrize("S,kw", [
    (1500, dict(window=575, n_sink=64)), (700, dict(window=1, n_sink=3)), (600, dict(window=100, n_sink=300)),
    (500, dict(window=5000, n_sink=0)), (3000, dict(window=64, n_sink=0)), (2500, dict(window=300, n_sink=17)),
])
@pytest.mark.parametrize("B,H,Hkv", [(1, 8, 2), (2, 3, 3)])
def test_window_sink_grads(S, kw, B, H, Hkv):
    run_case("llm/window_sink", "window_sink", B, S, H, Hkv, **kw)


def test_model_setting_at_16k():
    run_case("llm/block_scatter", "block_scatter", 1, 16384, 8, 2, group_num=2, block=256, offset=1, n_sink=64)
    run_case("llm/window_sink", "window_sink", 1, 16384, 8, 2, window=575, n_sink=64)


def test_autograd_function_with_sinks():
    B, S, H, Hkv = 1, 1024, 4, 2
    q, k, v, _ = make(B, S, H, Hkv, seed=3)
    q, k, v = (t.requires_grad_(True) for t in (q, k, v))
    out = intra_llm_attn_func(q, k, v, "window_sink", window=200, n_sink=16)
    w = torch.linspace(-1, 1, 128, device=DEV)
    (out.float() * w).sum().backward()
    dout = w.expand_as(out).to(torch.bfloat16)
    mask = oracle.mask_rows("llm/window_sink", S, device=DEV, window=200, n_sink=16)
    compare((q.grad, k.grad, v.grad), oracle.masked_attention_grads(q, k, v, dout, mask), "autograd with sinks")


def test_unsupported_requests_raise():
    q, k, v, dout = make(1, 512, 8, 4)  # two query heads per kv head: the forward takes 128-token blocks
    with torch.no_grad():
        out, lse = intra_llm_attn(q, k, v, "block_scatter", group_num=2, block=128, offset=1, return_lse=True)
    with pytest.raises(RuntimeError, match="block % 256"):
        intra_llm_attn_bwd(q, k, v, out, lse, dout, "block_scatter", group_num=2, block=128, offset=1)
    with pytest.raises(ValueError):
        intra_llm_attn_bwd(q, k, v, out, lse, dout, "gather0")


def test_c_abi_with_packed_gradient_buffer_and_strided_lse():
    """The C ABI directly: dq, dk, dv written into slices of one packed (B, S, H + 2 Hkv, 128)
    gradient buffer, lse passed with (batch, head, token) strides of a (B, S, H) tensor, and a
    workspace of exactly the size the library asks for."""
    from intra_amd import _lib
    lib = _lib.load()
    B, S, H, Hkv = 2, 1000, 8, 2
    q, k, v, dout = make(B, S, H, Hkv, seed=11)
    kw = dict(window=200, n_sink=24)
    with torch.no_grad():
        out, lse = intra_llm_attn(q, k, v, "window_sink", return_lse=True, **kw)
    lse_t = lse.transpose(1, 2).contiguous()  # (B, S, H) storage
    lse_st = _lib._i64x3(lse_t.stride(0), lse_t.stride(2), lse_t.stride(1))
    grads = torch.full((B, S, H + 2 * Hkv, 128), float("nan"), dtype=torch.bfloat16, device=DEV)
    dq, dk, dv = grads[:, :, :H], grads[:, :, H:H + Hkv], grads[:, :, H + Hkv:]
    n = lib.intra_llm_bwd_workspace(B, S, H, Hkv, 9, 2, 200, 256, 0, 24)
    assert n > B * H * S  # the partial sums of the sink pass follow rowsum(dout * out)
    work = torch.full((n + 64,), float("nan"), dtype=torch.float32, device=DEV)  # NaN: contents must not matter
    rc = lib.intra_llm_bwd(q.data_ptr(), k.data_ptr(), v.data_ptr(), out.data_ptr(), lse_t.data_ptr(), dout.data_ptr(),
                           dq.data_ptr(), dk.data_ptr(), dv.data_ptr(), work.data_ptr(), B, S, H, Hkv,
                           _lib.strides3(q), _lib.strides3(k), _lib.strides3(v), _lib.strides3(out), _lib.strides3(dout),
                           _lib.strides3(dq), _lib.strides3(dk), _lib.strides3(dv), lse_st, 9, 2, 200, 256, 0, 24,
                           128 ** -0.5, torch.cuda.current_stream().cuda_stream)
    assert rc == 0, _lib.last_error()
    torch.cuda.synchronize()
    assert bool(torch.isnan(work[n:]).all()), "wrote past the workspace"
    mask = oracle.mask_rows("llm/window_sink", S, device=DEV, **kw)
    compare((dq, dk, dv), oracle.masked_attention_grads(q, k, v, dout, mask), "packed gradients")


def test_results_do_not_change_between_calls():
    """No atomics anywhere (the sink rows are summed in a fixed order): bit-identical reruns."""
    q, k, v, dout = make(1, 3000, 8, 2, seed=5)
    kw = dict(group_num=2, block=256, offset=1, n_sink=64)
    a = kernel_grads(q, k, v, dout, "block_scatter", **kw)
    b = kernel_grads(q, k, v, dout, "block_scatter", **kw)
    for x, y in zip(a, b):
        assert torch.equal(x, y)


def test_backward_can_be_captured_in_a_graph_and_replayed():
    """Forward + backward allocate only through torch and record no memset, so they can go into a
    HIP graph; every replay, with fresh inputs copied into the captured tensors and eager work in
    between, must equal the eager result."""
    B, S, H, Hkv = 1, 1024, 8, 2
    kw = dict(window=300, n_sink=32)
    sq, sk, sv, sd = make(B, S, H, Hkv, seed=20)
    stream = torch.cuda.Stream()
    stream.wait_stream(torch.cuda.current_stream())
    with torch.cuda.stream(stream), torch.no_grad():
        for _ in range(2):  # warm-up outside the capture
            o, l = intra_llm_attn(sq, sk, sv, "window_sink", return_lse=True, **kw)
            intra_llm_attn_bwd(sq, sk, sv, o, l, sd, "window_sink", **kw)
    torch.cuda.current_stream().wait_stream(stream)
    torch.cuda.synchronize()
    graph = torch.cuda.CUDAGraph()
    with torch.cuda.graph(graph), torch.no_grad():
        o, l = intra_llm_attn(sq, sk, sv, "window_sink", return_lse=True, **kw)
        gq, gk, gv = intra_llm_attn_bwd(sq, sk, sv, o, l, sd, "window_sink", **kw)
    for seed in (21, 22, 23):
        nq, nk, nv, nd = make(B, S, H, Hkv, seed=seed)
        for dst, src in ((sq, nq), (sk, nk), (sv, nv), (sd, nd)):
            dst.copy_(src)
        graph.replay()
        torch.cuda.synchronize()
        eager = kernel_grads(nq, nk, nv, nd, "window_sink", **kw)
        torch.cuda.synchronize()
        for x, y in zip((gq, gk, gv), eager):
            assert torch.equal(x, y), f"replay with seed {seed} differs from the eager call"


def _random_cases(n, seed):
    import random
    rnd = random.Random(seed)
    heads = [(4, 4), (4, 2), (8, 2), (4, 1), (16, 4), (3, 3), (6, 3)]
    cases = []
    for _ in range(n):
        H, Hkv = rnd.choice(heads)
        B = rnd.choice([1, 1, 2])
        S = rnd.choice([rnd.randint(1, 300), rnd.randint(300, 2500), 64 * rnd.randint(1, 36)])
        kind = rnd.choice(["scatter", "gather1", "window", "block_scatter", "window_sink"])
        if kind == "scatter":
            kw = dict(group_num=rnd.choice([1, 2, 3, 5, 8, 13]))
        elif kind == "gather1":
            S = 64 * max(1, S // 64)
            kw = dict(group_num=8)
        elif kind == "window":
            kw = dict(window=rnd.choice([64, 65, 128, 576, 1000, 4000]))
        elif kind == "block_scatter":
            G = rnd.choice([1, 2, 3, 4])
            off = rnd.randrange(G)
            blk = 256 * rnd.choice([1, 1, 2]) if (off or (H // Hkv) % 4) else 64 * rnd.choice([1, 2, 4, 8])
            kw = dict(group_num=G, block=blk, offset=off, n_sink=rnd.choice([0, 1, 64, blk]))
        else:
            kw = dict(window=rnd.choice([1, 2, 63, 64, 575, 2000]), n_sink=rnd.choice([0, 1, 64, 100, 700]))
        cases.append((kind, B, S, H, Hkv, kw, rnd.choice([None, None, 0.05, -0.11])))
    return cases


@pytest.mark.parametrize("case", _random_cases(40, seed=77) + _random_cases(80, seed=78), ids=lambda c: f"{c[0]}-S{c[2]}-H{c[3]}/{c[4]}")
def test_random_shapes(case):
    kind, B, S, H, Hkv, kw, scale = case
    run_case(f"llm/{kind}", kind, B, S, H, Hkv, seed=S + H, scale=scale, **kw)


@pytest.mark.parametrize("H,Hkv", [(8, 1), (6, 2), (16, 2), (5, 1)])
def test_other_head_ratios(H, Hkv):
    """8, 3 and 5 query heads per kv head: several head groups per kv head in dQ, more streams in dK / dV."""
    run_case("llm/scatter", "scatter", 1, 900, H, Hkv, seed=H, group_num=3)
    run_case("llm/window_sink", "window_sink", 1, 900, H, Hkv, seed=H + 1, window=130, n_sink=40)
