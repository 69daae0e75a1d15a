"""`intra_attn_cuda.fwd_llm` / `fwd` called exactly as the reference's Python layer calls its
compiled extension (intra_attn/interface.py:43-44,64-65): 16 positional arguments, result `[0]`."""
import pytest
import torch

import oracle

pytestmark = pytest.mark.gpu
DEV = "cuda"


def make(B, S, H, Hkv, seed):
    g = torch.Generator(device="cpu").manual_seed(seed)
    mk = lambda h: torch.randn(B, S, h, 128, generator=g).to(torch.bfloat16).to(DEV)
    return mk(H), mk(Hkv), mk(Hkv)


@pytest.mark.parametrize("mask_id,kind,kw", [(0, "llm/scatter", dict(group_num=8)), (1, "llm/gather1", dict(group_num=8)),
                                              (4, "llm/window", dict(window=576))])
def test_fwd_llm_like_the_reference_calls_it(mask_id, kind, kw):
    import intra_attn_cuda as _C
    q, k, v = make(1, 2048, 8, 2, seed=mask_id)
    scale = 128 ** -0.5
    res = _C.fwd_llm(q, k, v, None, None, 0.0, scale, True, -1, -1, 0.0, False, None, mask_id, kw.get("group_num", 8),
                     kw.get("window", 576))
    assert len(res) == 4 and res[2] is None and res[3] is None
    mask = oracle.mask_rows(kind, 2048, device=DEV, **kw)
    assert (res[0].float() - oracle.masked_attention(q, k, v, mask).float()).abs().max().item() <= 1.6e-2
    assert (res[1] - oracle.masked_lse_rows(q, k, mask)).abs().max().item() <= 5e-3  # ln(1 + 2^-8): the sum runs over bf16-rounded weights


@pytest.mark.parametrize("mask_id,kind", [(0, "image/scatter"), (4, "image/gather0")])
def test_fwd_image_like_the_reference_calls_it(mask_id, kind):
    import intra_attn_cuda as _C
    S = 512 + 64 * 64
    q, k, v = make(1, S, 4, 4, seed=10 + mask_id)
    out_ = torch.empty_like(q)
    res = _C.fwd(q, k, v, out_, None, 0.0, 0.1, False, -1, -1, 0.0, False, None, mask_id, 64, 64)
    assert res[0] is out_
    mask = oracle.mask_rows(kind, S, device=DEV, width=64)
    assert (out_.float() - oracle.masked_attention(q, k, v, mask, softmax_scale=0.1).float()).abs().max().item() <= 1.6e-2


def test_rejections_raise_runtime_error():
    import intra_attn_cuda as _C
    q, k, v = make(1, 256, 4, 2, seed=3)
    args = lambda **o: [o.get("q", q), k, v, None, o.get("alibi"), o.get("p", 0.0), 0.1, True, -1, -1, o.get("softcap", 0.0),
                        o.get("rs", False), None, o.get("mask", 0), 8, 576]
    for bad, text in ((dict(p=0.1), "dropout"), (dict(alibi=torch.ones(4, device=DEV)), "alibi"), (dict(softcap=1.0), "softcap"),
                      (dict(rs=True), "return_softmax"), (dict(q=q.float()), "bfloat16"), (dict(q=q[..., ::2]), "contiguous"),
                      (dict(mask=7), "unknown LLM pattern")):
        with pytest.raises(RuntimeError, match=text):
            _C.fwd_llm(*args(**bad))
    q2, k2, v2 = make(1, 200, 4, 2, seed=4)  # 200 is not a multiple of 8 * 8
    with pytest.raises(RuntimeError, match="multiple of group_num"):
        _C.fwd_llm(q2, k2, v2, None, None, 0.0, 0.1, True, -1, -1, 0.0, False, None, 1, 8, 576)
