"""Per-pattern latency table of the INTRA kernels on MI355X, and two measurement modes.

`llm` and `image`: protocol and CLI of the reference's benchmarks/bench_kernel.py:23-34,91-111
(median of --iters event-timed calls after --warmup calls), rows with the reference's keys and the
latency in ms as value (benchmarks/results/*.json), extended by `<key>_tflops` (unmasked pairs
only), `<key>_pct_peak` (of the bf16 dense MFMA peak), the `*_run` stacks and, with --cpu, the
dense-mask specification timed on the host cores (`<key>_cpu_ms`, `cpu_cores`).

    python -m intra_amd.bench_kernel llm   --seqlens 4096,8192,16384,32768,65536
    python -m intra_amd.bench_kernel image

`phases`: where a workgroup's time goes, from timers inside the kernel.  Needs the measurement
build of the library (python -m intra_amd.build --diag), selected through INTRA_HIP_LIB:

    INTRA_HIP_LIB=intra_amd/libintra_hip_diag.so python -m intra_amd.bench_kernel phases \
        --pattern scatter --seqlen 32768 [--softmax exact]

The same mode prices the ingredients of the kernel's inner step on an ablation build
(python -m intra_amd.build --ablate N; the row reports N as "ablation"):

    INTRA_HIP_LIB=intra_amd/libintra_hip_ablate1.so python -m intra_amd.bench_kernel phases --pattern scatter

`series`: the HIP-event time of every launch of the headline kernel, in launch order, behind a pause
without GPU work (the board's power management answers a pause of a few milliseconds with two dozen
slow launches):

    python -m intra_amd.bench_kernel series --pauses-ms 500,50,5,0 --launches 40

`ceiling`: what the matrix cores sustain with nothing else running, per MFMA shape (16x16x32 and
32x32x16), with constant and with random operand bits, and the clock they run at (the board is
power-limited):

    python -m intra_amd.bench_kernel ceiling
"""
import argparse
import ctypes
import json
import time

import torch
import torch.nn.functional as F

import intra_amd
from intra_amd import _lib, intra_image_attn, intra_image_attn_bwd, intra_llm_attn, intra_llm_attn_bwd
from intra_amd.interface import TEXT_LEN

PEAK_BF16_TFLOPS = 2516.6


def median_ms(fn, warmup, iters):
    """Median latency of fn() in ms.  After `warmup` untimed calls, each of `iters` calls sits
    between two events on the current stream and has finished before the next one is issued."""
    for _ in range(warmup):
        fn()
    samples = []
    while len(samples) < iters:
        tic, toc = (torch.cuda.Event(enable_timing=True) for _ in range(2))
        tic.record()
        fn()
        toc.record()
        toc.synchronize()
        samples.append(tic.elapsed_time(toc))
    samples.sort()
    return samples[iters // 2]


def cpu_spec_ms(q, k, v, mask_fn):
    """The dense-mask specification (masked fp32 attention over an S x S boolean mask, what the
    reference's intra_attn/reference.py:78-83 defines) on the host cores: one warm-up, median of 3."""
    from intra_attn.reference import masked_attention
    qc, kc, vc = (x.cpu() for x in (q, k, v))
    mask = mask_fn()
    times = []
    for _ in range(4):
        t0 = time.perf_counter()
        masked_attention(qc, kc, vc, mask)
        times.append((time.perf_counter() - t0) * 1e3)
    return round(sorted(times[1:])[1], 2)


def pairs(domain, pattern, B, S, H, Hkv, a0, a1):
    plan = _lib.IntraPlan()
    rc = _lib.load().intra_plan(domain, pattern, B, S, H, Hkv, a0, a1, ctypes.byref(plan))
    assert rc == 0, _lib.last_error()
    return plan.pairs_per_head


def pairs_ex(pattern, B, S, H, Hkv, group_num, window, block, offset, n_sink):
    plan = _lib.IntraPlan()
    rc = _lib.load().intra_plan_llm_ex(pattern, B, S, H, Hkv, group_num, window, block, offset, n_sink,
                                       ctypes.byref(plan))
    assert rc == 0, _lib.last_error()
    return plan.pairs_per_head


def dense_sdpa(q, k, v, causal):
    q, k, v = (x.transpose(1, 2) for x in (q, k, v))
    return F.scaled_dot_product_attention(q, k, v, is_causal=causal, enable_gqa=q.shape[1] != k.shape[1])


def qkv(B, S, H, Hkv, seed=0):
    g = torch.Generator(device="cpu").manual_seed(seed)
    mk = lambda h: torch.randn(B, S, h, 128, generator=g).to(torch.bfloat16).cuda()
    return mk(H), mk(Hkv), mk(Hkv)


def put(row, key, ms, npairs, B, H):
    """row[key] is the latency in ms, as in the reference's result files; the effective TFLOP/s
    (unmasked pairs only) and the fraction of the bf16 MFMA peak go beside it."""
    tf = 4 * 128 * npairs * H * B / (ms * 1e-3) / 1e12
    row[key] = round(ms, 4)
    row[key + "_tflops"] = round(tf, 1)
    row[key + "_pct_peak"] = round(100 * tf / PEAK_BF16_TFLOPS, 1)


@torch.no_grad()
def bench_llm(args):
    rows = []
    B, H, Hkv = args.batch, args.heads, args.kv_heads
    for S in args.seqlens:
        q, k, v = qkv(B, S, H, Hkv)
        r = {"seqlen": S}
        if args.dense:
            ms = median_ms(lambda: dense_sdpa(q, k, v, True), args.warmup, args.iters)
            put(r, "dense", ms, S * (S + 1) // 2, B, H)
        cpu = args.cpu and S <= 8192
        if cpu:
            from intra_attn import reference as spec
            r["cpu_cores"] = torch.get_num_threads()
        for G in args.groups:
            ms = median_ms(lambda: intra_llm_attn(q, k, v, "scatter", group_num=G), args.warmup, args.iters)
            put(r, f"scatter_g{G}", ms, pairs(0, 0, B, S, H, Hkv, G, 576), B, H)
            if cpu:
                r[f"scatter_g{G}_cpu_ms"] = cpu_spec_ms(q, k, v, lambda: spec.llm_scatter_mask(S, G))
        if S % 64 == 0:
            ms = median_ms(lambda: intra_llm_attn(q, k, v, "gather1", group_num=8), args.warmup, args.iters)
            put(r, "gather1_g8", ms, pairs(0, 1, B, S, H, Hkv, 8, 576), B, H)
            if cpu:
                r["gather1_g8_cpu_ms"] = cpu_spec_ms(q, k, v, lambda: spec.llm_gather1_mask(S, 8))
        ms = median_ms(lambda: intra_llm_attn(q, k, v, "window", window=576), args.warmup, args.iters)
        put(r, "window576", ms, pairs(0, 4, B, S, H, Hkv, 8, 576), B, H)
        if cpu:
            r["window576_cpu_ms"] = cpu_spec_ms(q, k, v, lambda: spec.llm_window_mask(S, 576))
        if "scatter_g2" in r:
            # the reference's arithmetic for the 32-layer g2s4 schedule (bench_kernel.py:66-68) ...
            r["g2s4_32layer"] = round(4 * r["scatter_g2"] + 28 * r["window576"], 3)
            if "dense" in r:
                r["dense_32layer"] = round(32 * r["dense"], 3)
            # ... and the same stack actually run back to back with fresh inputs per layer
            layers = [qkv(B, S, H, Hkv, seed=i) for i in range(4)]

            def stack():
                for i in range(32):
                    ql, kl, vl = layers[i % 4]
                    if i % 8 == 0:
                        intra_llm_attn(ql, kl, vl, "scatter", group_num=2)
                    else:
                        intra_llm_attn(ql, kl, vl, "window", window=576)
            r["g2s4_32layer_run"] = round(median_ms(stack, 2, max(3, args.iters // 10)), 3)
        if args.backward:
            # dq, dk, dv of the same calls (three launches); flops counted as 5 products per pair
            # (S, dP, dV, dQ, dK), i.e. 2.5 x the forward's, whatever the kernels recompute
            dout = qkv(B, S, H, Hkv, seed=1)[0]
            cases = [(f"scatter_g{G}", "scatter", dict(group_num=G), pairs(0, 0, B, S, H, Hkv, G, 576)) for G in args.groups]
            if S % 64 == 0:
                cases.append(("gather1_g8", "gather1", dict(group_num=8), pairs(0, 1, B, S, H, Hkv, 8, 576)))
            cases.append(("window576", "window", dict(window=576), pairs(0, 4, B, S, H, Hkv, 8, 576)))
            if args.model_patterns:
                for off in (0, 1):
                    cases.append((f"block_scatter_g2_b256_off{off}_sink64", "block_scatter",
                                  dict(group_num=2, block=256, offset=off, n_sink=64),
                                  pairs_ex(8, B, S, H, Hkv, 2, 575, 256, off, 64)))
                cases.append(("window575_sink64", "window_sink", dict(window=575, n_sink=64),
                              pairs_ex(9, B, S, H, Hkv, 2, 575, 256, 0, 64)))
            for key, pattern, kw, npairs in cases:
                out, lse = intra_llm_attn(q, k, v, pattern, return_lse=True, **kw)
                ms = median_ms(lambda: intra_llm_attn_bwd(q, k, v, out, lse, dout, pattern, **kw), args.warmup, args.iters)
                tf = 10 * 128 * npairs * H * B / (ms * 1e-3) / 1e12
                r[key + "_bwd"] = round(ms, 4)
                r[key + "_bwd_tflops"] = round(tf, 1)
                r[key + "_bwd_pct_peak"] = round(100 * tf / PEAK_BF16_TFLOPS, 1)
        if args.model_patterns:
            # the layers the reference's model integration really runs in its g2s4 LLaMA setting
            # (experiments/llm/llama_intra.py:16-18): block Scatter with 2 groups of 256-token
            # blocks, stripe offset 0 / 1, 64 sink tokens; per-token window 575 with 64 sinks
            for off in (0, 1):
                kw = dict(group_num=2, block=256, offset=off, n_sink=64)
                ms = median_ms(lambda: intra_llm_attn(q, k, v, "block_scatter", **kw), args.warmup, args.iters)
                put(r, f"block_scatter_g2_b256_off{off}_sink64", ms, pairs_ex(8, B, S, H, Hkv, 2, 575, 256, off, 64), B, H)
            ms = median_ms(lambda: intra_llm_attn(q, k, v, "window_sink", window=575, n_sink=64), args.warmup, args.iters)
            put(r, "window575_sink64", ms, pairs_ex(9, B, S, H, Hkv, 2, 575, 256, 0, 64), B, H)
            layers = [qkv(B, S, H, Hkv, seed=i) for i in range(4)]

            def model_stack():
                for i in range(32):
                    ql, kl, vl = layers[i % 4]
                    if i % 8 == 0:
                        intra_llm_attn(ql, kl, vl, "block_scatter", group_num=2, block=256, offset=(i // 8) % 2, n_sink=64)
                    else:
                        intra_llm_attn(ql, kl, vl, "window_sink", window=575, n_sink=64)
            r["g2s4_model_32layer_run"] = round(median_ms(model_stack, 2, max(3, args.iters // 10)), 3)
            if args.backward:
                # the same 32 layers forward (with log-sum-exp) and backward: the attention part of a training step
                douts = [qkv(B, S, H, Hkv, seed=10 + i)[0] for i in range(2)]

                def model_train_stack():
                    for i in range(32):
                        ql, kl, vl = layers[i % 4]
                        if i % 8 == 0:
                            name, kw = "block_scatter", dict(group_num=2, block=256, offset=(i // 8) % 2, n_sink=64)
                        else:
                            name, kw = "window_sink", dict(window=575, n_sink=64)
                        out, lse = intra_llm_attn(ql, kl, vl, name, return_lse=True, **kw)
                        intra_llm_attn_bwd(ql, kl, vl, out, lse, douts[i % 2], name, **kw)
                r["g2s4_model_32layer_fwd_bwd_run"] = round(median_ms(model_train_stack, 1, max(3, args.iters // 10)), 3)
        rows.append(r)
        print(json.dumps(r), flush=True)
    return rows


@torch.no_grad()
def bench_image(args):
    rows = []
    B, H = args.batch, args.image_heads
    for width in args.widths:
        S = TEXT_LEN + width * width
        q, k, v = qkv(B, S, H, H)
        r = {"width": width, "seqlen": S}
        if args.dense:
            put(r, "dense", median_ms(lambda: dense_sdpa(q, k, v, False), args.warmup, args.iters), S * S, B, H)
        for pattern, pid in (("scatter", 0), ("gather0", 4)):
            ms = median_ms(lambda: intra_image_attn(q, k, v, pattern, width), args.warmup, args.iters)
            put(r, pattern, ms, pairs(1, pid, B, S, H, H, width, TEXT_LEN), B, H)
            if args.cpu and S <= 8192:
                from intra_attn import reference as spec
                mask_fn = spec.image_scatter_mask if pattern == "scatter" else spec.image_gather0_mask
                r[pattern + "_cpu_ms"] = cpu_spec_ms(q, k, v, lambda: mask_fn(width))
                r["cpu_cores"] = torch.get_num_threads()
        r["interleaved_mean"] = round((r["scatter"] + r["gather0"]) / 2, 4)  # layers alternate the two patterns
        if args.backward:
            dout = qkv(B, S, H, H, seed=1)[0]
            for pattern, pid in (("scatter", 0), ("gather0", 4)):
                out, lse = intra_image_attn(q, k, v, pattern, width, return_lse=True)
                ms = median_ms(lambda: intra_image_attn_bwd(q, k, v, out, lse, dout, pattern, width), args.warmup, args.iters)
                tf = 10 * 128 * pairs(1, pid, B, S, H, H, width, TEXT_LEN) * H * B / (ms * 1e-3) / 1e12
                r[pattern + "_bwd"] = round(ms, 4)
                r[pattern + "_bwd_tflops"] = round(tf, 1)
                r[pattern + "_bwd_pct_peak"] = round(100 * tf / PEAK_BF16_TFLOPS, 1)
        rows.append(r)
        print(json.dumps(r), flush=True)
    return rows


PHASES = ["item set-up", "first barrier", "first key block", "tile loop", "next item, Q request, normalise, store"]
DIAG_SLOTS = 16  # values per workgroup (csrc/intra_kernel.hip.h)
BARRIERS = ["in front of the Q slots", "in front of the first key block", "opening tile 0", "between tiles (per tile)"]


def placement(raw, iters):
    """Half-size workgroups: which share a CU, and the busy time of the one in the CU's first wavefront
    slot against the one in its second (HW_ID of wavefront 0, written over - not added to - slot 8)."""
    raw = raw[raw[:, 5] > 0]
    hw = raw[:, 8]
    cu = (((hw >> 32) & 0xF) << 12) | (((hw >> 13) & 7) << 8) | (((hw >> 12) & 1) << 4) | ((hw >> 8) & 0xF)  # XCC, SE, SH, CU
    slot = hw & 0xF
    busy = raw[:, :5].sum(1).double() / 100 / iters
    per_cu = {}
    for i in range(raw.shape[0]):
        per_cu.setdefault(int(cu[i]), []).append(i)
    sizes = sorted({len(v) for v in per_cu.values()})
    first = [busy[i].item() for v in per_cu.values() for i in v if slot[i] == 0]
    second = [busy[i].item() for v in per_cu.values() for i in v if slot[i] != 0]
    return {"cus": len(per_cu), "workgroups_per_cu": sizes,
            "busy_us_first_slot": round(sum(first) / max(1, len(first)), 1),
            "busy_us_second_slot": round(sum(second) / max(1, len(second)), 1)}


@torch.no_grad()
def bench_phases(args):
    """Sum over a launch of the in-kernel phase timers (see include/intra_hip.h, intra_diag_set_buffer)."""
    lib = _lib.load()
    n_wg = 4096
    buf = torch.zeros(n_wg * DIAG_SLOTS, dtype=torch.int64, device="cuda")
    if lib.intra_diag_set_buffer(buf.data_ptr(), buf.numel()) != 0:
        raise SystemExit(f"{_lib.last_error()}; run with INTRA_HIP_LIB={_lib.DIAG_LIB_PATH}")
    intra_amd.set_softmax_mode(args.softmax)
    S = TEXT_LEN + args.width ** 2 if args.pattern.startswith("image") else args.seqlen
    if args.pattern.startswith("image"):
        q, k, v = qkv(args.batch, S, args.image_heads, args.image_heads)
        call = lambda: intra_image_attn(q, k, v, args.pattern.split("_")[1], args.width)
    else:
        q, k, v = qkv(args.batch, S, args.heads, args.kv_heads)
        kw = {"scatter": dict(group_num=args.groups[-1]), "gather1": dict(group_num=8), "window": dict(window=576)}[args.pattern]
        call = lambda: intra_llm_attn(q, k, v, args.pattern, **kw)
    for _ in range(args.warmup):
        call()
    torch.cuda.synchronize()
    buf.zero_()
    for _ in range(args.iters):
        call()
    torch.cuda.synchronize()
    lib.intra_diag_set_buffer(None, 0)
    d = buf.view(-1, DIAG_SLOTS).double().cpu()
    d = d[d[:, 5] > 0] / args.iters
    items, tiles = d[:, 5].mean().item(), d[:, 6].mean().item()
    res = {"pattern": args.pattern, "seqlen": S, "softmax": args.softmax, "ablation": lib.intra_diag_ablation(),
           "workgroups": d.shape[0],
           "items_per_workgroup": round(items, 2), "tiles_per_item": round(tiles / items, 2), "us_per_item": {}}
    for i, name in enumerate(PHASES):
        res["us_per_item"][name] = round(d[:, i].mean().item() / 100 / items, 3)  # 100 MHz ticks
    loop_us = d[:, 3].mean().item() / 100
    res["us_per_tile"] = round(loop_us / tiles, 4)
    res["cycles_per_tile"] = round(d[:, 7].mean().item() / tiles, 1)
    res["shader_clock_mhz"] = round(d[:, 7].mean().item() / loop_us, 1)
    res["us_per_workgroup"] = {"mean": round(d[:, :5].sum(1).mean().item() / 100, 1),
                               "max": round(d[:, :5].sum(1).max().item() / 100, 1)}
    res["share_outside_tile_loop"] = round(1 - d[:, 3].sum().item() / d[:, :5].sum().item(), 4)
    # shader cycles -> us with the clock of the tile loops; [own requests and LDS reads, other wavefronts]
    mhz = d[:, 7].mean().item() / loop_us
    res["waves"] = 4 if d.shape[0] > torch.cuda.get_device_properties(0).multi_processor_count else 8
    res["barrier_wait_us"] = {}
    for i, name in enumerate(BARRIERS):
        if res["waves"] == 4 and i < 3:
            continue  # half-size workgroups have no barriers at the item boundary (slots 8 .. 11 hold the placement)
        per = tiles if i == 3 else items
        res["barrier_wait_us"][name] = [round(d[:, 8 + 2 * i + j].mean().item() / mhz / per, 3) for j in range(2)]
    if res["waves"] == 4:
        res["placement"] = placement(buf.view(-1, DIAG_SLOTS).cpu(), args.iters)
    print(json.dumps(res), flush=True)
    return [res]


@torch.no_grad()
def bench_series(args):
    """Per-launch times of Scatter G=8 at --seqlen behind pauses of --pauses-ms (in that order; 0 = none)."""
    q, k, v = qkv(args.batch, args.seqlen, args.heads, args.kv_heads)
    call = lambda: intra_llm_attn(q, k, v, "scatter", group_num=8)
    call()
    torch.cuda.synchronize()
    rows = []
    for pause in args.pauses_ms:
        time.sleep(pause / 1e3)
        evs = [(torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)) for _ in range(args.launches)]
        for a, b in evs:
            a.record()
            call()
            b.record()
        torch.cuda.synchronize()
        ms = [round(a.elapsed_time(b), 4) for a, b in evs]
        row = {"pattern": "scatter_g8", "seqlen": args.seqlen, "pause_ms": pause, "ms": ms,
               "mean_first_20": round(sum(ms[:20]) / len(ms[:20]), 4), "mean_rest": round(sum(ms[20:]) / max(1, len(ms[20:])), 4)}
        rows.append(row)
        print(json.dumps(row), flush=True)
    return rows


def bench_ceiling(args):
    """MFMA-only launches (8 wavefronts per CU on every CU, nothing but v_mfma_f32_16x16x32_bf16, the
    kernels' instruction, or v_mfma_f32_32x32x16_bf16, the alternative shape) with constant
    and with random operand bits: TFLOP/s and the shader clock each ran at."""
    lib = _lib.load()
    n_wg = torch.cuda.get_device_properties(0).multi_processor_count
    iters = 20000
    sink = torch.empty(n_wg * 512, dtype=torch.float32, device="cuda")
    clocks = torch.zeros(n_wg * 2, dtype=torch.int64, device="cuda")
    g = torch.Generator().manual_seed(1)
    tables = {"constant 1.0": torch.full((65536,), 1.0).to(torch.bfloat16),
              "random N(0,1)": torch.randn(65536, generator=g).to(torch.bfloat16)}
    rows = []
    for shape, name, host in [(sh, n, h) for sh in (16, 32) for n, h in tables.items()]:
        table = host.cuda()
        stream = torch.cuda.current_stream().cuda_stream
        best = None
        for rep in range(4):
            tic, toc = (torch.cuda.Event(enable_timing=True) for _ in range(2))
            tic.record()
            rc = lib.intra_diag_mfma_ceiling(table.data_ptr(), sink.data_ptr(), clocks.data_ptr(), n_wg, iters, shape, stream)
            assert rc == 0, _lib.last_error()
            toc.record()
            toc.synchronize()
            ms = tic.elapsed_time(toc)
            c = clocks.view(-1, 2).double().cpu()
            row = {"mfma": "16x16x32" if shape == 16 else "32x32x16", "operands": name, "workgroups": n_wg, "ms": round(ms, 3),
                   "tflops": round(n_wg * 8 * iters * 16 * 32768 / (ms * 1e-3) / 1e12, 1),
                   "shader_clock_mhz": round((c[:, 0] / c[:, 1]).mean().item() * 100, 1)}
            if rep > 0 and (best is None or row["ms"] < best["ms"]):  # first launch: clock still ramping
                best = row
        best["pct_peak"] = round(100 * best["tflops"] / PEAK_BF16_TFLOPS, 1)
        rows.append(best)
        print(json.dumps(best), flush=True)
    return rows


def main():
    p = argparse.ArgumentParser()
    p.add_argument("mode", choices=["llm", "image", "phases", "ceiling", "series"])
    p.add_argument("--seqlens", default="4096,8192,16384,32768,65536")
    p.add_argument("--groups", default="2,8")
    p.add_argument("--batch", type=int, default=1)
    p.add_argument("--heads", type=int, default=32)
    p.add_argument("--kv-heads", type=int, default=8)
    p.add_argument("--image-heads", type=int, default=24)
    p.add_argument("--widths", default="64,128", help="image: latent grid sides (64: 1024 x 1024, 128: 2048 x 2048)")
    p.add_argument("--warmup", type=int, default=10)
    p.add_argument("--iters", type=int, default=50)
    p.add_argument("--no-dense", dest="dense", action="store_false",
                   help="skip torch SDPA on the dense problem (the reference's `dense` column)")
    p.add_argument("--cpu", action="store_true",
                   help="also time the dense-mask fp32 specification on the host cores (S <= 8192)")
    p.add_argument("--model-patterns", action="store_true",
                   help="llm: also time block Scatter and window-with-sinks layers (g2s4 model setting)")
    p.add_argument("--backward", action="store_true", help="also time the backward pass (dq, dk, dv) of each pattern")
    p.add_argument("--pattern", default="scatter",
                   choices=["scatter", "gather1", "window", "image_scatter", "image_gather0"], help="phases: which kernel")
    p.add_argument("--seqlen", type=int, default=32768, help="phases: LLM sequence length")
    p.add_argument("--width", type=int, default=64, help="phases: image grid side")
    p.add_argument("--softmax", default="auto", choices=["auto", "exact", "scaled", "folded"], help="phases: softmax arithmetic")
    p.add_argument("--pauses-ms", default="500,50,5,0", help="series: pauses in front of each run of launches")
    p.add_argument("--launches", type=int, default=40, help="series: launches per run")
    p.add_argument("--out", help="optional JSON output path")
    args = p.parse_args()
    args.seqlens = [int(x) for x in args.seqlens.split(",")]
    args.widths = [int(x) for x in args.widths.split(",")]
    args.groups = [int(x) for x in args.groups.split(",")]
    print(f"device: {torch.cuda.get_device_name()}  torch {torch.__version__}  peak {PEAK_BF16_TFLOPS} TFLOP/s")
    args.pauses_ms = [float(x) for x in args.pauses_ms.split(",")]
    rows = {"llm": bench_llm, "image": bench_image, "phases": bench_phases, "ceiling": bench_ceiling,
            "series": bench_series}[args.mode](args)
    if args.out:
        json.dump({"device": torch.cuda.get_device_name(), "torch": torch.__version__,
                   "args": {k: v for k, v in vars(args).items() if k != "out"}, "rows": rows},
                  open(args.out, "w"), indent=1)


if __name__ == "__main__":
    main()
