"""Builds libintra_hip.so for gfx950 with hipcc (no torch or CUDA-compat headers involved).

    python -m intra_amd.build            # intra_amd/libintra_hip.so
    python -m intra_amd.build --diag     # intra_amd/libintra_hip_diag.so, with in-kernel phase timers
    python -m intra_amd.build --ablate N # intra_amd/libintra_hip_ablate<N>.so: the timers plus ablation N of the
                                         # forward kernel's inner step (wrong results on purpose; see intra_hip.h)

Takes the place of the reference's CUDAExtension build (setup.py:28-68).
"""
import os
import shutil
import subprocess
import sys

HERE = os.path.dirname(os.path.abspath(__file__))
SRC = os.path.join(HERE, "csrc", "intra_api.hip")
LIB = os.path.join(HERE, "libintra_hip.so")

# -packed-fp32-ops off: plain v_add/v_mul/v_fma only, no v_pk_*_f32 forms.
HIPCC_FLAGS = [
    "--offload-arch=gfx950", "-O3", "-std=c++17", "-shared", "-fPIC",
    "-Xclang", "-target-feature", "-Xclang", "-packed-fp32-ops",
    # inputs are finite by contract; -inf is used for masking, so infinities stay honoured
    "-fno-honor-nans",
    # MFMA results may live in ordinary registers also where a kernel needs more than 256 of them (the
    # fused dK / dV kernel, one wavefront per SIMD): only pure accumulators then go to the other half of
    # the register file.  Kernels below that size compile to the same code with and without it.
    "-mllvm", "-amdgpu-mfma-vgpr-form",
]


def hipcc_path():
    for cand in (os.environ.get("HIPCC"), shutil.which("hipcc"), "/opt/rocm/bin/hipcc"):
        if cand and os.path.exists(cand):
            return cand
    raise RuntimeError("hipcc not found; set HIPCC or install ROCm")


DIAG_LIB = os.path.join(HERE, "libintra_hip_diag.so")


def build(verbose=False, extra_flags=(), diag=False, ablate=0):
    """Compile the library in-tree and return its path.  diag=True builds the measurement variant
    libintra_hip_diag.so (same sources with the in-kernel phase timers compiled in) instead;
    ablate=N that variant with ablation N of the forward kernel (libintra_hip_ablate<N>.so)."""
    lib = DIAG_LIB if diag else LIB
    if ablate:
        lib = os.path.join(HERE, f"libintra_hip_ablate{int(ablate)}.so")
        extra_flags = ("-DINTRA_DIAG_TIMERS", f"-DINTRA_ABLATE={int(ablate)}", *extra_flags)
    elif diag:
        extra_flags = ("-DINTRA_DIAG_TIMERS", *extra_flags)
    cmd = [hipcc_path(), *HIPCC_FLAGS, *extra_flags, SRC, "-o", lib + ".tmp"]
    if verbose:
        print(" ".join(cmd), flush=True)
    res = subprocess.run(cmd, stdout=subprocess.PIPE, stderr=subprocess.STDOUT, text=True)
    out = "\n".join(l for l in res.stdout.splitlines() if "not a recognized feature" not in l)
    if res.returncode != 0:
        raise RuntimeError(f"hipcc failed ({res.returncode}):\n{out}")
    if verbose and out.strip():
        print(out)
    os.replace(lib + ".tmp", lib)
    return lib


if __name__ == "__main__":
    args = sys.argv[1:]
    n_ablate = 0
    if "--ablate" in args:
        at = args.index("--ablate")
        n_ablate = int(args[at + 1])
        del args[at:at + 2]
    print(build(verbose=True, extra_flags=[a for a in args if a != "--diag"], diag="--diag" in args, ablate=n_ablate))
