"""Image Gather 0 deals its text queries as sets of their own (two scatter groups per row block at
1024 x 1024) and numbers text rows and patch runs in separate sections of work items.  Head counts
that are not multiples of 8 put both kinds of sets into one slot of pairs, grouped query heads
change the rows per block: every such launch against the dense-mask oracle."""
import pytest
import torch

import oracle
from intra_amd import intra_image_attn

pytestmark = pytest.mark.gpu


@pytest.mark.parametrize("H,Hkv,B", [(1, 1, 1), (3, 3, 1), (5, 5, 2), (7, 7, 1), (12, 12, 3), (4, 2, 1), (8, 2, 2), (6, 3, 1)])
@pytest.mark.parametrize("pattern", ["gather0", "scatter"])
def test_head_layouts(pattern, H, Hkv, B):
    width, dev = 64, "cuda:0"
    S = 512 + width * width
    g = torch.Generator().manual_seed(1000 * H + 10 * Hkv + B)
    mk = lambda h: torch.randn(B, S, h, 128, generator=g).to(torch.bfloat16).to(dev)
    q, k, v = mk(H), mk(Hkv), mk(Hkv)
    with torch.no_grad():
        out = intra_image_attn(q, k, v, pattern, width)
    ref = oracle.masked_attention(q, k, v, oracle.mask_rows("image/" + pattern, S, device=dev, width=width))
    assert torch.isfinite(out).all()
    assert (out.float() - ref.float()).abs().max().item() <= 1.6e-2  # bf16 output, as in the parity matrix
