"""Distribution of the default mode's error, not only its maximum: a seeded sweep over shapes (it
stops at the first failure) that compares a row subset of every output with the oracle's fp32 result
and histograms the element errors, in absolute terms and in bf16 steps of the result.  The headline
shape (Scatter G=8, S=32768, 32 query / 8 kv heads) comes first.

What must hold: every element inside the derived bound of parity_util.py (1.6e-2 + half a bf16
step); at most 1 element in 1000 beyond half of the plain bound; at least 90 % of the elements
within one bf16 step of the fp32 result.  Observed on the headline shape (4.2 M elements): maximum
7.3e-3; 93.9 % of the errors below 2.5e-4, 99.7 % below 1e-3, 2 in 100 000 above 4e-3, none above
8e-3; 81 % within half a bf16 step of the fp32 result (what the output rounding alone would give),
97 % within one step.  The histogram itself is printed and, where the scratch directory of a GPU run
exists, written to gpurun_out/error_histogram.json."""
import json
import os

import pytest
import torch

import oracle
from intra_amd import intra_image_attn, intra_llm_attn
from parity_util import ATOL, DEV, half_step_bf16, make_qkv

pytestmark = pytest.mark.gpu
ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))

ABS_EDGES = [0, 2.5e-4, 5e-4, 1e-3, 2e-3, 4e-3, 8e-3, 1.6e-2, float("inf")]
STEP_EDGES = [0, 0.25, 0.5, 1.0, 2.0, 4.0, float("inf")]

SWEEP = [
    ("llm/scatter", dict(group_num=8), 32768, 32, 8, 1.0),      # the headline shape
    ("llm/scatter", dict(group_num=8), 32768, 32, 8, 2.0),      # the same with q, k twice as large
    ("llm/scatter", dict(group_num=2), 16384, 32, 8, 1.0),
    ("llm/gather1", dict(group_num=8), 32768, 32, 8, 1.0),
    ("llm/window", dict(window=576), 32768, 32, 8, 1.0),
    ("llm/window", dict(window=576), 8192, 32, 8, 3.0),
    ("llm/block_scatter", dict(group_num=2, block=256, offset=1, n_sink=64), 16384, 32, 8, 1.0),
    ("llm/window_sink", dict(window=575, n_sink=64), 16384, 32, 8, 1.0),
    ("image/scatter", dict(width=64), 4608, 24, 24, 1.0),
    ("image/gather0", dict(width=64), 4608, 24, 24, 1.0),
    ("image/scatter", dict(width=128), 16896, 24, 24, 1.0),
    ("image/gather0", dict(width=128), 16896, 24, 24, 2.0),
]


def histogram(values, edges):
    counts = torch.histogram(values.flatten().cpu().double(), torch.tensor(edges[:-1] + [1e30], dtype=torch.float64)).hist
    return [int(c) for c in counts]


def test_error_distribution_of_the_default_mode():
    report = []
    for index, (kind, kw, S, H, Hkv, sigma) in enumerate(SWEEP):
        q, k, v = make_qkv(1, S, H, Hkv, seed=1000 + index, sigma=sigma)
        g = torch.Generator().manual_seed(index)
        rows = torch.unique(torch.cat([torch.randperm(S, generator=g)[:1024], torch.tensor([0, 1, 63, 64, S - 1])])).to(DEV)
        with torch.no_grad():
            if kind.startswith("image/"):
                out = intra_image_attn(q, k, v, kind.split("/")[1], kw["width"])
            else:
                out = intra_llm_attn(q, k, v, kind.split("/")[1], **kw)
        mask = oracle.mask_rows(kind, S, rows=rows, device=DEV, **kw)
        ref = oracle.masked_attention_rows(q, k, v, mask, rows, out_dtype=torch.float32)
        err = (out[:, rows].float() - ref).abs()
        steps = err / (2 * half_step_bf16(ref))
        entry = {"kind": kind, "args": kw, "S": S, "heads": [H, Hkv], "sigma": sigma, "elements": err.numel(),
                 "max_abs": err.max().item(), "max_steps": steps.max().item(),
                 "abs_edges": ABS_EDGES[:-1], "abs_counts": histogram(err, ABS_EDGES),
                 "step_edges": STEP_EDGES[:-1], "step_counts": histogram(steps, STEP_EDGES)}
        report.append(entry)
        print(json.dumps(entry), flush=True)
        n = err.numel()
        assert bool((err <= ATOL + half_step_bf16(ref)).all()), entry
        assert (err > ATOL / 2).sum().item() <= n / 1000, entry
        assert (steps <= 1.0).sum().item() >= 0.90 * n, entry
        del q, k, v, out, ref, err, steps
    scratch = os.path.join(ROOT, "gpurun_out")
    if os.path.isdir(scratch):
        with open(os.path.join(scratch, "error_histogram.json"), "w") as f:
            json.dump(report, f, indent=1)
