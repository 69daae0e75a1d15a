"""Per-pattern latency table of the INTRA kernels on MI355X.

Same protocol and CLI as the reference's benchmarks/bench_kernel.py:23-34,91-111 (median of
--iters event-timed calls after --warmup calls; `llm` and `image` modes), with the rows extended
by effective TFLOP/s (unmasked pairs only) and the fraction of the bf16 dense MFMA peak.  The rows
keep the reference's keys with the latency in ms as value (benchmarks/results/*.json); the
additions are `<key>_tflops`, `<key>_pct_peak` and the `*_run` stacks.

    python -m intra_amd.bench_kernel llm   --seqlens 4096,8192,16384,32768,65536
    python -m intra_amd.bench_kernel image
"""
import argparse
import json

import torch
import torch.nn.functional as F

from intra_amd import _lib, intra_image_attn, intra_image_attn_bwd, intra_llm_attn, intra_llm_attn_bwd
from intra_amd.interface import TEXT_LEN

PEAK_BF16_TFLOPS = 2516.6


def median_ms(fn, warmup, iters):
    for _ in range(warmup):
        fn()
    times = []
    for _ in range(iters):
        start, end = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
        start.record()
        fn()
        end.record()
        torch.cuda.synchronize()
        times.append(start.elapsed_time(end))
    return sorted(times)[len(times) // 2]


def pairs(domain, pattern, B, S, H, Hkv, a0, a1):
    import ctypes
    plan = _lib.IntraPlan()
    rc = _lib.load().intra_plan(domain, pattern, B, S, H, Hkv, a0, a1, ctypes.byref(plan))
    assert rc == 0, _lib.last_error()
    return plan.pairs_per_head


def pairs_ex(pattern, B, S, H, Hkv, group_num, window, block, offset, n_sink):
    import ctypes
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
        if args.cpu and S <= 8192:
            # torch SDPA on the host cores for the dense causal problem, fp32: the scale of a CPU run
            # beside the GPU rows (one warm-up, median of 3)
            import time
            qc, kc, vc = (x.float().cpu() for x in (q, k, v))
            times = []
            for _ in range(4):
                t0 = time.perf_counter()
                dense_sdpa(qc, kc, vc, True)
                times.append((time.perf_counter() - t0) * 1e3)
            r["dense_cpu_ms"] = round(sorted(times[1:])[1], 2)
            r["cpu_cores"] = torch.get_num_threads()
        for G in args.groups:
            ms = median_ms(lambda: intra_llm_attn(q, k, v, "scatter", group_num=G), args.warmup, args.iters)
            put(r, f"scatter_g{G}", ms, pairs(0, 0, B, S, H, Hkv, G, 576), B, H)
        if S % 64 == 0:
            ms = median_ms(lambda: intra_llm_attn(q, k, v, "gather1", group_num=8), args.warmup, args.iters)
            put(r, "gather1_g8", ms, pairs(0, 1, B, S, H, Hkv, 8, 576), B, H)
        ms = median_ms(lambda: intra_llm_attn(q, k, v, "window", window=576), args.warmup, args.iters)
        put(r, "window576", ms, pairs(0, 4, B, S, H, Hkv, 8, 576), B, H)
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


def main():
    p = argparse.ArgumentParser()
    p.add_argument("mode", choices=["llm", "image"])
    p.add_argument("--seqlens", default="4096,8192,16384,32768,65536")
    p.add_argument("--groups", default="2,8")
    p.add_argument("--batch", type=int, default=1)
    p.add_argument("--heads", type=int, default=32)
    p.add_argument("--kv-heads", type=int, default=8)
    p.add_argument("--image-heads", type=int, default=24)
    p.add_argument("--widths", default="64,128", help="image: latent grid sides (64: 1024 x 1024, 128: 2048 x 2048)")
    p.add_argument("--warmup", type=int, default=10)
    p.add_argument("--iters", type=int, default=50)
    p.add_argument("--dense", action="store_true", help="also time torch SDPA on the dense problem")
    p.add_argument("--cpu", action="store_true", help="llm: also time dense causal SDPA on the host CPU (S <= 8192)")
    p.add_argument("--model-patterns", action="store_true",
                   help="llm: also time block Scatter and window-with-sinks layers (g2s4 model setting)")
    p.add_argument("--backward", action="store_true", help="also time the backward pass (dq, dk, dv) of each pattern")
    p.add_argument("--out", help="optional JSON output path")
    args = p.parse_args()
    args.seqlens = [int(x) for x in args.seqlens.split(",")]
    args.widths = [int(x) for x in args.widths.split(",")]
    args.groups = [int(x) for x in args.groups.split(",")]
    print(f"device: {torch.cuda.get_device_name()}  torch {torch.__version__}  peak {PEAK_BF16_TFLOPS} TFLOP/s")
    rows = bench_llm(args) if args.mode == "llm" else bench_image(args)
    if args.out:
        json.dump({"device": torch.cuda.get_device_name(), "torch": torch.__version__,
                   "args": {k: v for k, v in vars(args).items() if k != "out"}, "rows": rows},
                  open(args.out, "w"), indent=1)


if __name__ == "__main__":
    main()
