"""Headline benchmark: LLM causal Scatter G=8 at S=32768 (B=1, 32 query / 8 kv heads, d=128,
bf16) on one MI355X.  A step is one call of intra_llm_attn on inputs already resident in HBM.

    python bench.py [--gpus 1] [--steps K] [--warmup W] [--seqlen S] [--settle N] [--no-cpu]

Prints ONE JSON line.  `value` is effective TFLOP/s (flops of unmasked query-key pairs only,
4*128 per pair and head) over the wall-clock of the K timed steps; `roofline` is the same
algorithmic work over the kernel's own average duration (HIP events on the launch stream);
`cpu_baseline` is the fp32 dense-mask oracle on the host cores for a bounded sample of query rows
of the same problem.

Order of the run: the oracle's rows for the parity check, then N = --settle correctness launches
(the first is the one checked against the oracle, all N must be bit-identical; each is timed with
HIP events and the series is reported as `settle.ms`), then without a gap the W warm-up steps and
the K timed steps.  The correctness launches stand where they do on purpose: after any pause of a
few milliseconds the board's power management runs the next two dozen launches of this kernel up
to 30 % slower (the series shows it), which says nothing about the kernel; --settle 0 gives the
figure that includes that transient.
"""
import argparse
import json
import os
import sys
import time

ROOT = os.path.dirname(os.path.abspath(__file__))
if ROOT not in sys.path:
    sys.path.insert(0, ROOT)

PEAK_BF16_TFLOPS = 2516.6  # 256 CU x 2.4 GHz x 4096 flop/clk/CU; AMD publishes it as 2.5 PFLOP/s dense
# HBM bytes per launch from rocprofv3 --pmc FETCH_SIZE / WRITE_SIZE, written by
# `python -m intra_amd.rocprof_summary traffic` together with a hash of the kernel sources
TRAFFIC_FILE = os.path.join(ROOT, "profiles", "hbm_traffic.json")


def measured_traffic(seqlen):
    """Bytes per launch if they were measured for exactly this kernel source and workload, else None."""
    try:
        from intra_amd.rocprof_summary import source_hash
        rec = json.load(open(TRAFFIC_FILE))
        if rec.get("source_sha256_16") == source_hash() and rec.get("seqlen") == seqlen:
            return rec["hbm_bytes_per_launch"]
    except (OSError, ValueError, KeyError):
        pass
    return None


def main():
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=50)
    ap.add_argument("--warmup", type=int, default=10)
    ap.add_argument("--seqlen", type=int, default=32768)
    ap.add_argument("--settle", type=int, default=60,
                    help="correctness launches (parity, bit-identical repeats) in front of the warm-up steps")
    ap.add_argument("--no-cpu", action="store_true", help="skip the cpu_baseline leg")
    ap.add_argument("--softmax", choices=["auto", "exact", "scaled", "folded"], default="auto",
                    help="softmax arithmetic of the kernel (auto: what a plain call gets)")
    ap.add_argument("--copy-calib", action="store_true",
                    help="also run three plain 1 GiB device copies, the known-size kernel that scales "
                         "FETCH_SIZE / WRITE_SIZE readings of a counter run")
    args = ap.parse_args()
    if args.gpus != 1:
        sys.exit("bench.py measures one GPU: the kernels are single-GPU and this build launches nothing "
                 "across GPUs; run with --gpus 1")

    import torch

    import oracle
    import intra_amd
    from intra_amd import _lib, intra_llm_attn

    assert torch.cuda.is_available(), "bench.py needs a GPU"
    assert os.path.exists(_lib.LIB_PATH), "libintra_hip.so is not built"
    intra_amd.set_softmax_mode(args.softmax)
    dev = torch.device("cuda:0")
    B, S, H, Hkv, G = 1, args.seqlen, 32, 8, 8
    g = torch.Generator(device="cpu").manual_seed(0)
    mk = lambda h: torch.randn(B, S, h, 128, generator=g, dtype=torch.float32).to(torch.bfloat16)
    q_cpu, k_cpu, v_cpu = mk(H), mk(Hkv), mk(Hkv)
    q, k, v = q_cpu.to(dev), k_cpu.to(dev), v_cpu.to(dev)
    pairs = oracle.pairs_per_head("llm/scatter", S, group_num=G)
    flop = 4.0 * 128 * pairs * H * B

    if args.copy_calib:
        src = torch.empty(1 << 30, dtype=torch.uint8, device=dev).fill_(1)
        dst = torch.empty_like(src)
        for _ in range(3):
            dst.copy_(src)
        torch.cuda.synchronize()
        del src, dst

    step = lambda: intra_llm_attn(q, k, v, "scatter", group_num=G)
    timed_event = lambda: (torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True))
    with torch.no_grad():
        # what the parity spot check will compare with: the oracle on a row subset
        rows = torch.unique(torch.cat([torch.randperm(S, generator=g)[:256], torch.tensor([0, S - 1])])).to(dev)
        ref = oracle.masked_attention_rows(q, k, v, oracle.llm_scatter_mask(S, G, dev, rows), rows)
        torch.cuda.synchronize()
        # correctness launches, each kept; checked after the timed region, before anything is printed
        n_settle = max(1, args.settle)
        settle_ev, settle_out = [timed_event() for _ in range(n_settle)], []
        for a, b in settle_ev:
            a.record()
            settle_out.append(step())
            b.record()
        for _ in range(args.warmup):
            out = step()
        torch.cuda.synchronize()
        t0 = time.perf_counter()
        for _ in range(args.steps):
            out = step()
        torch.cuda.synchronize()
        wall_ms = (time.perf_counter() - t0) * 1e3 / args.steps

        # per-launch kernel duration: HIP events on the stream the kernel is launched on
        evs = [timed_event() for _ in range(args.steps)]
        for a, b in evs:
            a.record()
            step()
            b.record()
        torch.cuda.synchronize()
        kern_ms = sorted(a.elapsed_time(b) for a, b in evs)
        settle_ms = [round(a.elapsed_time(b), 4) for a, b in settle_ev]
    kern_avg = sum(kern_ms) / len(kern_ms)

    # a wrong kernel posts nothing: parity of the first launch, every other launch bit-identical to it
    checked = settle_out[0]
    err = (checked[:, rows].float() - ref.float()).abs().max().item()
    assert err <= 1.6e-2, f"parity failed in bench: {err}"
    assert all(torch.equal(checked, o) for o in settle_out[1:]), "repeated launches differ"
    assert torch.equal(checked, out), "the timed launches produced another output than the checked one"
    del settle_out, ref

    tflops = flop / (wall_ms * 1e-3) / 1e12
    achieved = flop / (kern_avg * 1e-3) / 1e12
    res = {
        "metric": "Scatter G=8 32K ms/call + effective TFLOP/s (% bf16 MFMA peak), 1 MI355X",
        "value": round(tflops, 2), "unit": "effective TFLOP/s (unmasked pairs only)",
        "n_gpus": 1, "steps": args.steps, "warmup": args.warmup, "ms_per_step": round(wall_ms, 4),
        "higher_is_better": True, "scaling": "weak", "vs_baseline": None, "dtype": "bf16",
        "data": "synthetic: i.i.d. N(0,1) from CPU seed 0, rounded to bf16",
        "config": {"workload": f"LLM causal Scatter G={G}, B={B}, S={S}, {H} query / {Hkv} kv heads, d=128",
                   "pairs_per_head": pairs, "tflop_per_call": round(flop / 1e12, 6)},
        "ms_per_call": round(wall_ms, 4), "pct_of_peak": round(100 * tflops / PEAK_BF16_TFLOPS, 2),
        "kernel_ms": {"avg": round(kern_avg, 4), "median": round(kern_ms[len(kern_ms) // 2], 4),
                      "min": round(kern_ms[0], 4), "p90": round(kern_ms[int(0.9 * (len(kern_ms) - 1))], 4)},
        "parity_max_abs_err": err, "softmax": args.softmax,
        "settle": {"launches": n_settle, "ms": settle_ms,
                   "what": "correctness launches in front of the warm-up steps (parity on the first, the rest "
                           "bit-identical), HIP-event time of each in launch order"},
        "roofline": {"bound": "mfma", "achieved": round(achieved, 2), "peak": PEAK_BF16_TFLOPS,
                     "unit": "TFLOP/s", "frac": round(achieved / PEAK_BF16_TFLOPS, 4),
                     "traffic": measured_traffic(S)},
        "device": torch.cuda.get_device_name(0),
        "cu_count": torch.cuda.get_device_properties(0).multi_processor_count,
    }

    if not args.no_cpu:
        # Bounded sample of the same problem: evenly spaced query rows of all heads against all
        # keys through the dense-mask fp32 path, on the host cores.
        n_rows = 4096 if S >= 8192 else S  # about 10 s on 16 host cores
        rows_c = torch.arange(0, S, S // n_rows)[:n_rows]
        mask_c = oracle.llm_scatter_mask(S, G, rows=rows_c)
        cores = torch.get_num_threads()
        oracle.masked_attention_rows(q_cpu, k_cpu, v_cpu, mask_c[:64], rows_c[:64], chunk=64)  # warm-up
        t0 = time.perf_counter()
        oracle.masked_attention_rows(q_cpu, k_cpu, v_cpu, mask_c, rows_c, chunk=128)
        dt = time.perf_counter() - t0
        eff = 4.0 * 128 * int(mask_c.sum()) * H * B
        res["cpu_baseline"] = {
            "value": round(eff / dt / 1e12, 6), "unit": "effective TFLOP/s (unmasked pairs only)",
            "cores": cores, "kind": "port",
            "sample": f"{n_rows} evenly spaced query rows x {H} heads of the same S={S} problem, dense-mask fp32 "
                      f"oracle, {dt:.2f} s; dense work {4.0 * 128 * n_rows * S * H / dt / 1e12:.4f} TFLOP/s",
        }
        # the reference's CPU-runnable case beside it, whole problem on both sides: Scatter G=8,
        # S=1024, 4 query / 1 kv heads (median of 5 runs after a warm-up)
        qs, ks, vs = (t[:, :1024, :n].contiguous() for t, n in ((q_cpu, 4), (k_cpu, 1), (v_cpu, 1)))
        mask_s = oracle.llm_scatter_mask(1024, G)
        cpu_ms = []
        for _ in range(6):
            t0 = time.perf_counter()
            oracle.masked_attention(qs, ks, vs, mask_s)
            cpu_ms.append((time.perf_counter() - t0) * 1e3)
        qg, kg, vg = qs.to(dev), ks.to(dev), vs.to(dev)
        small_gpu_ms = []
        with torch.no_grad():
            for i in range(8):
                a, b = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
                a.record()
                intra_llm_attn(qg, kg, vg, "scatter", group_num=G)
                b.record()
                torch.cuda.synchronize()
                small_gpu_ms.append(a.elapsed_time(b))
        # like for like: the whole problem at the headline's head layout (32 query / 8 kv heads) at the
        # largest length the dense-mask path handles in seconds, CPU and GPU on the same inputs
        Sw = min(S, 8192)
        qw, kw_, vw = (t[:, :Sw].contiguous() for t in (q_cpu, k_cpu, v_cpu))
        mask_w = oracle.llm_scatter_mask(Sw, G)
        t0 = time.perf_counter()
        oracle.masked_attention(qw, kw_, vw, mask_w, chunk=512)
        cpu_s = time.perf_counter() - t0
        qg, kg, vg = qw.to(dev), kw_.to(dev), vw.to(dev)
        gpu_ms = []
        with torch.no_grad():
            for i in range(13):
                a, b = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
                a.record()
                intra_llm_attn(qg, kg, vg, "scatter", group_num=G)
                b.record()
                torch.cuda.synchronize()
                gpu_ms.append(a.elapsed_time(b))
        eff_w = 4.0 * 128 * oracle.pairs_per_head("llm/scatter", Sw, group_num=G) * H * B
        res["cpu_baseline"]["whole_problem"] = {
            "workload": f"LLM causal Scatter G={G}, B=1, S={Sw}, {H} query / {Hkv} kv heads",
            "cpu_ms": round(cpu_s * 1e3, 1), "cpu_tflops_effective": round(eff_w / cpu_s / 1e12, 6),
            "gpu_ms": round(sorted(gpu_ms[3:])[5], 4)}
        res["cpu_baseline"]["small_case"] = {
            "workload": f"LLM causal Scatter G={G}, B=1, S=1024, 4 query / 1 kv heads",
            "cpu_ms": round(sorted(cpu_ms[1:])[2], 3), "gpu_ms": round(sorted(small_gpu_ms[3:])[2], 4)}
    print(json.dumps(res), flush=True)


if __name__ == "__main__":
    main()
