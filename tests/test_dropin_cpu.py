"""The repository as a drop-in for the reference package: with only the repository root on
sys.path, the import lines of the reference's own callers resolve -
tests/test_kernel.py:9-11, benchmarks/bench_kernel.py:19-20 and
experiments/flux/intra_processor.py:23-27 of the reference - and intra_attn.reference is the
dense-mask specification under the reference's names and signatures (intra_attn/reference.py:10-83).
intra_attn.reference is written independently of oracle/ (the product may not import the checker),
so comparing the two is a check of both."""
import inspect
import os
import subprocess
import sys

import pytest
import torch

import oracle

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))

IMPORTS = """
import sys
sys.path[:] = [p for p in sys.path if p and 'reference' not in p]   # nothing of the reference tree
sys.path.insert(0, {root!r})
# tests/test_kernel.py:9-11
from intra_attn import intra_image_attn, intra_llm_attn
from intra_attn.reference import (TEXT_LEN, image_gather0_mask, image_scatter_mask, llm_gather1_mask,
                                  llm_scatter_mask, llm_window_mask, masked_attention)
# benchmarks/bench_kernel.py:19-20
from intra_attn import intra_image_attn, intra_llm_attn
from intra_attn.reference import TEXT_LEN
# experiments/flux/intra_processor.py:23-27
from intra_attn.reference import TEXT_LEN, image_gather0_mask, image_scatter_mask
try:
    import intra_attn_cuda  # noqa: F401
    from intra_attn import intra_image_attn
except ImportError:
    intra_image_attn = None
import intra_attn, intra_attn.reference as ref, os
assert os.path.dirname(intra_attn.__file__) == os.path.join({root!r}, 'intra_attn'), intra_attn.__file__
assert intra_image_attn is not None and callable(intra_llm_attn)
assert hasattr(intra_attn_cuda, 'fwd_llm') and hasattr(intra_attn_cuda, 'fwd')
assert TEXT_LEN == 512 and intra_attn.__version__
# nothing on the product side pulls in the checker
assert 'oracle' not in sys.modules, 'the drop-in package imported oracle'
print('imports ok')
"""


def test_reference_callers_import_lines_resolve():
    res = subprocess.run([sys.executable, "-c", IMPORTS.format(root=ROOT)], cwd="/", capture_output=True, text=True,
                         env={k: v for k, v in os.environ.items() if k != "PYTHONPATH"})
    assert res.returncode == 0 and "imports ok" in res.stdout, res.stdout + res.stderr


def test_signatures_are_the_reference_ones():
    from intra_attn import reference as ref
    sig = lambda f: [(n, p.default) for n, p in inspect.signature(f).parameters.items()]
    E = inspect.Parameter.empty
    assert sig(ref.llm_scatter_mask) == [("S", E), ("group_num", 8), ("device", None)]
    assert sig(ref.llm_gather1_mask) == [("S", E), ("group_num", 8), ("device", None)]
    assert sig(ref.llm_window_mask) == [("S", E), ("window", 576), ("block", 64), ("device", None)]
    assert sig(ref.image_scatter_mask) == [("width", E), ("text_len", 512), ("device", None)]
    assert sig(ref.image_gather0_mask) == [("width", E), ("text_len", 512), ("patch", 8), ("window", 16), ("device", None)]
    assert sig(ref.masked_attention) == [("q", E), ("k", E), ("v", E), ("mask", E), ("softmax_scale", None)]


@pytest.mark.parametrize("S", [1, 63, 200, 1000])
@pytest.mark.parametrize("G", [1, 2, 3, 8])
def test_llm_masks_equal_the_oracle(S, G):
    from intra_attn import reference as ref
    assert torch.equal(ref.llm_scatter_mask(S, G), oracle.llm_scatter_mask(S, G))
    assert torch.equal(ref.llm_gather1_mask(S, G), oracle.llm_gather1_mask(S, G))
    for W in (64, 96, 576, 1000):
        assert torch.equal(ref.llm_window_mask(S, W), oracle.llm_window_mask(S, W))


def test_reference_known_answers():
    # the reference's own self-check (intra_attn/reference.py:86-103) on this module
    from intra_attn import reference as ref
    m = ref.llm_window_mask(200, window=96, block=64)
    assert m[130, 96] and not m[130, 95] and m[63, 0] and not m[10, 11]
    W, T = 64, ref.TEXT_LEN
    m = ref.image_scatter_mask(W)
    assert m.shape == (T + W * W,) * 2 and bool(m[:, :T].all())
    assert bool(m[T:, T:].sum(1).eq(W * W // 8).all())
    m = ref.image_gather0_mask(W)
    assert bool(m[T:, T:].sum(1).eq(256).all())
    q = T + 9 * W + 9
    assert m[q, T + 4 * W + 4] and not m[q, T + 3 * W + 4] and m[q, T + 19 * W + 19]


@pytest.mark.parametrize("width", [16, 24, 64])
def test_image_masks_equal_the_oracle(width):
    from intra_attn import reference as ref
    assert torch.equal(ref.image_scatter_mask(width), oracle.image_scatter_mask(width))
    assert torch.equal(ref.image_gather0_mask(width), oracle.image_gather0_mask(width))
    assert torch.equal(ref.image_scatter_mask(width, 64), oracle.image_scatter_mask(width, 64))
    assert torch.equal(ref.image_gather0_mask(width, 64), oracle.image_gather0_mask(width, 64))


def test_masked_attention_equals_the_oracle():
    from intra_attn import reference as ref
    g = torch.Generator().manual_seed(0)
    q = torch.randn(2, 96, 4, 128, generator=g).to(torch.bfloat16)
    k, v = (torch.randn(2, 96, 2, 128, generator=g).to(torch.bfloat16) for _ in range(2))
    mask = ref.llm_scatter_mask(96, 3)
    for scale in (None, 0.3):
        a = ref.masked_attention(q, k, v, mask, scale)
        b = oracle.masked_attention(q, k, v, mask, scale)
        assert a.dtype == torch.bfloat16 and a.shape == q.shape
        assert (a.float() - b.float()).abs().max().item() <= 2 ** -7
