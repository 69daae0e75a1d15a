"""Shared pieces of the GPU parity tests: seeded inputs and the two error bounds.

Plain bound: max-abs error <= 1.6e-2 between the kernel's bf16 output and the oracle's bf16 output
(the reference's statement, README.md:68-69; its tests/test_kernel.py:13 uses 2e-2).

Derived bound, for results that are not small: kernel and oracle round their fp32 results to bf16
separately, and for |out| >= 2 one bf16 step (2^-6 and up) exceeds the plain bound, so a kernel whose
fp32 result is well inside 1.6e-2 of the oracle's can still land a step away from the oracle's
rounded value.  The honest comparison is with the oracle's result BEFORE its rounding
(masked_attention_rows(..., out_dtype=torch.float32)), allowing the kernel's own rounding on top:
|out_bf16 - ref_fp32| <= 1.6e-2 + half a bf16 step at that magnitude.
"""
import torch

import oracle

ATOL = 1.6e-2
DEV = "cuda"


def make_qkv(B, S, H, Hkv, seed=0, sigma=1.0, device=DEV):
    """q, k ~ sigma * N(0,1), v ~ N(0,1), drawn on the CPU from a fixed seed, rounded to bf16, then moved."""
    g = torch.Generator(device="cpu").manual_seed(seed)
    q = (sigma * torch.randn(B, S, H, 128, generator=g, dtype=torch.float32)).to(torch.bfloat16)
    k = (sigma * torch.randn(B, S, Hkv, 128, generator=g, dtype=torch.float32)).to(torch.bfloat16)
    v = torch.randn(B, S, Hkv, 128, generator=g, dtype=torch.float32).to(torch.bfloat16)
    return q.to(device), k.to(device), v.to(device)


def half_step_bf16(x):
    """Half the spacing of bf16 numbers around |x| (taken at |x| + ATOL, so that a kernel result just
    across a power of two from the oracle's gets the spacing of its own side): 2^(e-9) for
    |x| + ATOL in [2^(e-1), 2^e)."""
    _, e = torch.frexp(x.abs() + ATOL)
    return torch.ldexp(torch.ones_like(x), e - 9)


def errors(out, q, k, v, kind, rows=None, scale=None, derived=False, **kw):
    """(elementwise |error|, elementwise bound) of a kernel output against the oracle on the same inputs."""
    S = q.shape[1]
    assert out.shape == q.shape and out.dtype == torch.bfloat16
    assert bool(torch.isfinite(out).all()), f"{kind} {kw}: non-finite output"
    mask = oracle.mask_rows(kind, S, rows=rows, device=q.device, **kw)
    got = (out if rows is None else out[:, rows]).float()
    if derived:
        ref = oracle.masked_attention_rows(q, k, v, mask, rows, softmax_scale=scale, out_dtype=torch.float32)
        return (got - ref).abs(), ATOL + half_step_bf16(ref)
    ref = oracle.masked_attention_rows(q, k, v, mask, rows, softmax_scale=scale).float()
    return (got - ref).abs(), torch.full_like(ref, ATOL)


def check(out, q, k, v, kind, rows=None, scale=None, derived=False, tag="", **kw):
    """Assert the bound (plain, or derived=True: against the fp32 oracle plus the kernel's own
    output rounding); returns the largest error."""
    diff, bound = errors(out, q, k, v, kind, rows, scale, derived, **kw)
    err = diff.max().item()
    worst = (diff - bound).max().item()
    assert worst <= 0, f"{tag} {kind} {kw} S={q.shape[1]} scale={scale}: max|err|={err:.3e}, {worst:.3e} over the bound"
    return err
