"""The call pattern of the reference's LLaMA / Qwen integration (experiments/llm/llama_intra.py:
177-221, 232-270) without model weights: a small decoder stack with random projections whose
attention goes through the test helper llama_caller.sparse_attention, forward and backward,
against the same stack on masked SDPA with the oracle's masks (what the reference trains with,
llama_intra.py:26).  Inputs reach the kernels as transposed (B, H, S, D) views of the projection
outputs, with GQA, an explicit scaling and the "g2s4" layer schedule: Scatter layers with stripe
offsets 0 / 1 and window layers, all with sinks.

Tolerance: both stacks compute in bf16; outputs and every gradient agree to a relative l2 error of
3e-2 (observed about 1e-2, the level of two bf16 implementations of the same layer stack)."""
import types

import pytest
import torch
import torch.nn.functional as F

import oracle
from llama_caller import attach_plans, force_dense, plan_layers, sparse_attention

pytestmark = pytest.mark.gpu
DEV = "cuda"
HQ, HKV, D = 4, 2, 128
HIDDEN = HQ * D


def make_model(n_layers, seed):
    g = torch.Generator(device="cpu").manual_seed(seed)
    w = lambda o, i: (torch.randn(o, i, generator=g) * i ** -0.5).to(torch.bfloat16).to(DEV).requires_grad_(True)
    layers = []
    for _ in range(n_layers):
        attn = types.SimpleNamespace(scaling=D ** -0.5, wq=w(HQ * D, HIDDEN), wk=w(HKV * D, HIDDEN),
                                     wv=w(HKV * D, HIDDEN), wo=w(HIDDEN, HQ * D))
        layers.append(types.SimpleNamespace(self_attn=attn))
    return types.SimpleNamespace(layers=layers)


def masked_sdpa_forward(module, query, key, value, attention_mask=None, scaling=None, dropout=0.0, **kwargs):
    """The same interface on dense-mask SDPA, masks from the oracle."""
    plan, S = module.intra_plan, query.shape[2]
    if plan.kind == "scatter":
        mask = oracle.mask_rows("llm/block_scatter", S, device=DEV, group_num=plan.group_num, block=plan.block,
                                offset=plan.offset, n_sink=plan.n_sink)
    elif plan.kind == "window":
        mask = oracle.mask_rows("llm/window_sink", S, device=DEV, window=plan.window, n_sink=plan.n_sink)
    else:
        mask = torch.ones(S, S, dtype=torch.bool, device=DEV).tril()
    out = F.scaled_dot_product_attention(query, key, value, attn_mask=mask, scale=scaling, enable_gqa=True)
    return out.transpose(1, 2).contiguous(), None


def run_stack(model, x, attention):
    B, S, _ = x.shape
    for layer in model.layers:
        a = layer.self_attn
        h = F.rms_norm(x, (HIDDEN,))
        q = (h @ a.wq.T).view(B, S, HQ, D).transpose(1, 2)   # (B, H, S, D) views, as transformers passes them
        k = (h @ a.wk.T).view(B, S, HKV, D).transpose(1, 2)
        v = (h @ a.wv.T).view(B, S, HKV, D).transpose(1, 2)
        out, _ = attention(a, q, k, v, attention_mask=None, scaling=a.scaling, dropout=0.0)
        assert out.shape == (B, S, HQ, D) and out.is_contiguous()
        x = x + out.reshape(B, S, HIDDEN) @ a.wo.T
    return x


def params(model):
    return [w for layer in model.layers for w in (layer.self_attn.wq, layer.self_attn.wk, layer.self_attn.wv, layer.self_attn.wo)]


def rel(a, b):
    return ((a.float() - b.float()).norm() / b.float().norm()).item()


@pytest.mark.parametrize("S", [1024, 1300])
def test_g2s4_stack_forward_and_backward(S):
    B = 2
    model = make_model(8, seed=1)
    plans = plan_layers(8, "SWWW", group_num=2, window=200, n_sink=64, blocks=(256,), stripe_offsets=2)
    attach_plans([l.self_attn for l in model.layers], plans)
    assert [p.kind for p in plans].count("scatter") == 2 and [p.kind for p in plans].count("window") == 6
    assert [p.offset for p in plans if p.kind == "scatter"] == [0, 1]
    g = torch.Generator(device="cpu").manual_seed(2)
    x0 = torch.randn(B, S, HIDDEN, generator=g).to(torch.bfloat16).to(DEV)
    results = []
    for attention in (sparse_attention, masked_sdpa_forward):
        x = x0.clone().requires_grad_(True)
        for w in params(model):
            w.grad = None
        y = run_stack(model, x, attention)
        y.float().square().mean().backward()
        results.append((y.detach(), x.grad, [w.grad.clone() for w in params(model)]))
    (y1, gx1, gw1), (y2, gx2, gw2) = results
    assert rel(y1, y2) <= 3e-2, rel(y1, y2)
    assert rel(gx1, gx2) <= 3e-2, rel(gx1, gx2)
    for i, (a, b) in enumerate(zip(gw1, gw2)):
        assert torch.isfinite(a).all() and rel(a, b) <= 3e-2, (i, rel(a, b))


def test_inference_decode_and_dense_branches():
    model = make_model(2, seed=3)
    attach_plans([l.self_attn for l in model.layers],
                 plan_layers(2, "SD", group_num=2, window=128, n_sink=16, blocks=(64,)))
    attn_s, attn_d = model.layers[0].self_attn, model.layers[1].self_attn
    g = torch.Generator(device="cpu").manual_seed(4)
    mk = lambda h, s: torch.randn(1, h, s, D, generator=g).to(torch.bfloat16).to(DEV)
    q, k, v = mk(HQ, 700), mk(HKV, 700), mk(HKV, 700)
    with torch.no_grad():
        out, _ = sparse_attention(attn_s, q, k, v, scaling=0.07)          # prefill, Scatter layer
        ref, _ = masked_sdpa_forward(attn_s, q, k, v, scaling=0.07)
        assert (out.float() - ref.float()).abs().max().item() <= 1.6e-2
        out, _ = sparse_attention(attn_d, q, k, v)                        # dense layer
        ref = F.scaled_dot_product_attention(q, k, v, is_causal=True, scale=D ** -0.5, enable_gqa=True).transpose(1, 2)
        assert torch.equal(out, ref.contiguous())
        out, _ = sparse_attention(attn_s, q[:, :, -1:], k, v)             # decode: one query, whole cache
        ref = F.scaled_dot_product_attention(q[:, :, -1:], k, v, scale=D ** -0.5, enable_gqa=True).transpose(1, 2)
        assert out.shape == (1, 1, HQ, D) and torch.equal(out, ref.contiguous())
        force_dense([l.self_attn for l in model.layers], True)                   # teacher toggle
        out, _ = sparse_attention(attn_s, q, k, v)
        ref = F.scaled_dot_product_attention(q, k, v, is_causal=True, scale=D ** -0.5, enable_gqa=True).transpose(1, 2)
        assert torch.equal(out, ref.contiguous())


def test_configuration_errors():
    model = make_model(2, seed=5)
    with pytest.raises(ValueError, match="256"):
        plan_layers(2, "S", group_num=2, window=0, blocks=(128,), stripe_offsets=2)
    attach_plans([l.self_attn for l in model.layers], plan_layers(2, "S", group_num=2, window=0, blocks=(100,)))
    q = torch.zeros(1, HQ, 256, D, dtype=torch.bfloat16, device=DEV)
    k = torch.zeros(1, HKV, 256, D, dtype=torch.bfloat16, device=DEV)
    with pytest.raises(ValueError, match="multiple of 64"):
        sparse_attention(model.layers[0].self_attn, q, k, k)


@pytest.mark.timeout(600)  # the first import of transformers on a fresh machine takes a while
def test_transformers_llama_model_trains_through_the_kernels():
    """A randomly initialised transformers LLaMA (tiny: 4 layers, 4 query / 2 kv heads of dim 128,
    rotary embeddings, RMSNorm, MLP - the real modelling code) with attn_implementation="intra":
    logits and parameter gradients against the same weights with the masked-SDPA function."""
    transformers = pytest.importorskip("transformers")
    from transformers import AttentionInterface, LlamaConfig, LlamaForCausalLM

    AttentionInterface.register("intra", sparse_attention)
    AttentionInterface.register("intra_masked_sdpa", masked_sdpa_forward)
    cfg = LlamaConfig(hidden_size=HIDDEN, num_attention_heads=HQ, num_key_value_heads=HKV, head_dim=D, num_hidden_layers=4,
                      intermediate_size=1024, vocab_size=512, max_position_embeddings=4096)
    cfg._attn_implementation = "intra"
    torch.manual_seed(0)
    model = LlamaForCausalLM(cfg).to(torch.bfloat16).to(DEV)
    plans = plan_layers(4, "SW", group_num=2, window=300, n_sink=64, blocks=(256,), stripe_offsets=2)
    attach_plans([layer.self_attn for layer in model.model.layers], plans)
    assert [p.kind for p in plans] == ["scatter", "window", "scatter", "window"]
    ids = torch.randint(0, 512, (2, 1536), generator=torch.Generator().manual_seed(1)).to(DEV)
    results = []
    for impl in ("intra", "intra_masked_sdpa"):
        model.config._attn_implementation = impl
        for layer in model.model.layers:
            layer.self_attn.config._attn_implementation = impl
        model.zero_grad(set_to_none=True)
        out = model(input_ids=ids, labels=ids, use_cache=False)
        out.loss.backward()
        results.append((out.logits.detach().float(), out.loss.item(),
                        {n: p.grad.detach().float().clone() for n, p in model.named_parameters()}))
    (l1, loss1, g1), (l2, loss2, g2) = results
    assert not torch.equal(l1, l2), "both runs took the same attention function"
    assert abs(loss1 - loss2) <= 2e-2 * abs(loss2), (loss1, loss2)
    assert rel(l1, l2) <= 3e-2, rel(l1, l2)
    worst = max((rel(g1[n], g2[n]), n) for n in g1)
    assert worst[0] <= 5e-2, worst
