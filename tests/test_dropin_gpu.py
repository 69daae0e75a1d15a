"""The reference's own parity loop (tests/test_kernel.py:19-51: same run() shape, same case
matrix, its 2e-2 bound) driven through the names a user of the reference imports -
`intra_attn.intra_llm_attn`, `intra_attn.intra_image_attn` and the masks and masked_attention of
`intra_attn.reference` - with this repository in place of the reference package.  The longest
sequences of that matrix (S = 16384) are covered against the chunked oracle in test_parity_gpu.py;
here the dense S x S specification is used as the reference uses it, up to S = 8192."""
import pytest
import torch

from intra_attn import intra_image_attn, intra_llm_attn
from intra_attn.reference import (TEXT_LEN, image_gather0_mask, image_scatter_mask, llm_gather1_mask,
                                  llm_scatter_mask, llm_window_mask, masked_attention)

pytestmark = pytest.mark.gpu
ATOL = 2e-2  # tests/test_kernel.py:13


def run(fn, mask, B, S, H, Hkv):
    g = torch.Generator(device="cpu").manual_seed(S + H)
    q = torch.randn(B, S, H, 128, generator=g).to(torch.bfloat16).cuda()
    k = torch.randn(B, S, Hkv, 128, generator=g).to(torch.bfloat16).cuda()
    v = torch.randn(B, S, Hkv, 128, generator=g).to(torch.bfloat16).cuda()
    with torch.no_grad():
        out = fn(q, k, v)
        ref = masked_attention(q, k, v, mask)
    err = (out.float() - ref.float()).abs().max().item()
    return bool(torch.isfinite(out).all()) and err < ATOL, err


@pytest.mark.parametrize("S", [1000, 2048, 3000, 4096, 8192])
@pytest.mark.parametrize("B,H,Hkv", [(1, 32, 8), (2, 32, 32)])
def test_llm_cases_of_the_reference_test(S, B, H, Hkv):
    dev = "cuda"
    for G in (2, 3, 8):
        ok, err = run(lambda q, k, v: intra_llm_attn(q, k, v, "scatter", group_num=G), llm_scatter_mask(S, G, dev), B, S, H, Hkv)
        assert ok, f"llm scatter G={G}: {err}"
    if S % 64 == 0:
        ok, err = run(lambda q, k, v: intra_llm_attn(q, k, v, "gather1", group_num=8), llm_gather1_mask(S, 8, dev), B, S, H, Hkv)
        assert ok, f"llm gather1: {err}"
    for W in (576, 1000):
        ok, err = run(lambda q, k, v: intra_llm_attn(q, k, v, "window", window=W), llm_window_mask(S, W, device=dev), B, S, H, Hkv)
        assert ok, f"llm window W={W}: {err}"


@pytest.mark.parametrize("width,H", [(64, 24), (128, 8)])
@pytest.mark.parametrize("B", [1, 2])
def test_image_cases_of_the_reference_test(width, H, B):
    S = TEXT_LEN + width * width
    ok, err = run(lambda q, k, v: intra_image_attn(q, k, v, "scatter", width), image_scatter_mask(width, device="cuda"), B, S, H, H)
    assert ok, f"image scatter: {err}"
    ok, err = run(lambda q, k, v: intra_image_attn(q, k, v, "gather0", width), image_gather0_mask(width, device="cuda"), B, S, H, H)
    assert ok, f"image gather0: {err}"
