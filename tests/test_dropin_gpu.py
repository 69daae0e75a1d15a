"""The reference's parity matrix (tests/test_kernel.py:33-51) driven through the names a user of
the reference imports - `intra_attn.intra_llm_attn`, `intra_attn.intra_image_attn` and the masks and
masked_attention of `intra_attn.reference` - with this repository in place of the reference
package.  Only the import lines and the case matrix are the reference's; every case is one pytest
item, checked at this repository's bound (1.6e-2, finite outputs) against the dense S x S
specification as the reference uses it.  The longest sequences of the matrix (S = 16384) are
covered against the chunked oracle in test_parity_gpu.py; here S goes up to 8192."""
import pytest
import torch

from intra_attn import intra_image_attn, intra_llm_attn
from intra_attn.reference import (TEXT_LEN, image_gather0_mask, image_scatter_mask, llm_gather1_mask,
                                  llm_scatter_mask, llm_window_mask, masked_attention)
from parity_util import ATOL, make_qkv

pytestmark = pytest.mark.gpu

LLM_CASES = [("scatter", dict(group_num=G), lambda S, dev, G=G: llm_scatter_mask(S, G, dev)) for G in (2, 3, 8)]
LLM_CASES += [("gather1", dict(group_num=8), lambda S, dev: llm_gather1_mask(S, 8, dev))]
LLM_CASES += [("window", dict(window=W), lambda S, dev, W=W: llm_window_mask(S, W, device=dev)) for W in (576, 1000)]
IMAGE_CASES = [("scatter", image_scatter_mask), ("gather0", image_gather0_mask)]


def assert_matches_dense_specification(out, q, k, v, mask, what):
    assert out.shape == q.shape and out.dtype == q.dtype, what
    assert bool(torch.isfinite(out).all()), f"{what}: non-finite output"
    with torch.no_grad():
        want = masked_attention(q, k, v, mask)
    err = (out.float() - want.float()).abs().max().item()
    assert err <= ATOL, f"{what}: max|err| = {err:.3e}"


@pytest.mark.parametrize("S", [1000, 2048, 3000, 4096, 8192])
@pytest.mark.parametrize("B,H,Hkv", [(1, 32, 8), (2, 32, 32)])
@pytest.mark.parametrize("pattern,kw,mask_of", LLM_CASES, ids=lambda c: c if isinstance(c, str) else None)
def test_llm_cases_of_the_reference_test(S, B, H, Hkv, pattern, kw, mask_of):
    if pattern == "gather1" and S % 64:
        pytest.skip("gather1 needs seqlen % 64 == 0, as in the reference's loop")
    q, k, v = make_qkv(B, S, H, Hkv, seed=S + H)
    with torch.no_grad():
        out = intra_llm_attn(q, k, v, pattern, **kw)
    assert_matches_dense_specification(out, q, k, v, mask_of(S, "cuda"), f"llm {pattern} {kw} S={S} B={B} H={H}/{Hkv}")


@pytest.mark.parametrize("width,H", [(64, 24), (128, 8)])
@pytest.mark.parametrize("B", [1, 2])
@pytest.mark.parametrize("pattern,mask_of", IMAGE_CASES, ids=lambda c: c if isinstance(c, str) else None)
def test_image_cases_of_the_reference_test(width, H, B, pattern, mask_of):
    q, k, v = make_qkv(B, TEXT_LEN + width * width, H, H, seed=width + H)
    with torch.no_grad():
        out = intra_image_attn(q, k, v, pattern, width)
    assert_matches_dense_specification(out, q, k, v, mask_of(width, device="cuda"), f"image {pattern} W={width} B={B} H={H}")
