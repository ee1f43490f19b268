#!/usr/bin/env python3
"""Benchmark of the block-FP8 W8A8 linear path on one MI355X.

One "step" is one pass of the path over one batch of synthetic input: per_token_group_quant_fp8 of the
bf16 activations followed by w8a8_block_fp8_matmul against block-quantized weights, everything resident
in HBM.  The headline workload is the DeepSeek-V3-shaped prefill gate_up linear (M=4096, N=36864, K=7168),
the configuration the FP8-MFMA target is stated on; the other shapes of the benchmark plan (decode-size M,
the standalone quantizer, the routed-expert grouped GEMM) are timed too and reported under "others".

Prints ONE JSON line.  Runs on one GPU only.
"""
import argparse
import json
import os
import sys
import time

ROOT = os.path.dirname(os.path.abspath(__file__))
sys.path.insert(0, ROOT)

FP8_MFMA_PEAK_TFLOPS = 5033.0  # 256 CU x 4 SIMD x 2048 flop/clk x 2.4 GHz, dense
HBM_PEAK_GBS = 8000.0


def _events(n):
    import torch

    return [torch.cuda.Event(enable_timing=True) for _ in range(n)]


def _time_calls(fn, iters, warm, batches=7):
    """Duration of `fn` in microseconds: the median over `batches` back-to-back batches of `iters` calls, each
    batch bracketed by HIP events on torch's current stream (the launch stream)."""
    import torch

    # sustained load first: the clocks need tens of milliseconds to settle after an idle gap
    t_settle = time.perf_counter()
    while time.perf_counter() - t_settle < 0.08:
        for _ in range(5):
            fn()
        torch.cuda.synchronize()
    for _ in range(warm):
        fn()
    torch.cuda.synchronize()
    ev = _events(batches + 1)
    ev[0].record()
    for b in range(batches):
        for _ in range(iters):
            fn()
        ev[b + 1].record()
    torch.cuda.synchronize()
    per_call = sorted(ev[b].elapsed_time(ev[b + 1]) * 1e3 / iters for b in range(batches))
    return per_call[batches // 2]


def _rotating(items):
    """Calls see `items` round-robin, so that a bandwidth-bound launch never finds its input in the 256 MB
    memory-side cache left there by the previous launch."""
    state = [0]

    def nxt():
        it = items[state[0] % len(items)]
        state[0] += 1
        return it

    return nxt


def roofline_us(flops, nbytes):
    return max(nbytes / HBM_PEAK_GBS / 1e3, flops / FP8_MFMA_PEAK_TFLOPS / 1e6)


def gemm_bytes(M, N, K):
    return M * K + N * K + 2 * M * N + 4 * M * (K // 128) + 4 * ((N + 127) // 128) * (K // 128)


def quant_bytes(M, K):
    return M * K * 3 + 4 * M * (K // 128)


def make_weight(N, K, seed, device):
    """~N(0, 0.02) bf16 weight, block-quantized by the library's own load-time quantizer."""
    import torch

    from lightllm_amd.quantization import mm_weight_quant

    g = torch.Generator(device=device).manual_seed(seed)
    w = (torch.randn((N, K), generator=g, device=device, dtype=torch.float32) * 0.02).to(torch.bfloat16)
    q, s = mm_weight_quant(w)
    return q, s


def make_act(M, K, seed, device, outliers=False):
    import torch

    g = torch.Generator(device=device).manual_seed(seed)
    x = torch.randn((M, K), generator=g, device=device, dtype=torch.float32)
    if outliers:
        x = torch.where(torch.rand((M, K), generator=g, device=device) < 0.01, x * 50.0, x)
        x[0] = 0.0
    return x.to(torch.bfloat16)


def measured_traffic(key):
    """Bytes per launch from profiles/traffic.json (written when the rocprofv3 counter passes of a kernel are
    summarised into profiles/): fetched + written, or None."""
    try:
        with open(os.path.join(ROOT, "profiles", "traffic.json")) as f:
            entry = json.load(f)[key]
        return float(entry["fetch_bytes"]) + float(entry["write_bytes"])
    except (OSError, KeyError, ValueError, TypeError):
        return None


def cpu_baseline(M_sample, N, K):
    """The reference's torch dequant+matmul form in fp32 plus its CPU quantizer, timed on the host cores
    on a row sample of the headline workload (full N and K, M_sample of the 4096 rows)."""
    import torch

    from oracle import torch_ref as tr

    g = torch.Generator().manual_seed(0)
    x = torch.randn((M_sample, K), generator=g).to(torch.bfloat16)
    w = (torch.randn((N, K), generator=g) * 0.02).to(torch.bfloat16)
    wq, ws = tr.block_weight_quant(w)
    del w

    def step():
        xq, xs = tr.group_quant(x)
        return tr.dequant_matmul(xq, xs, wq, ws)

    step()
    times = []
    t_end = time.perf_counter() + 20.0
    while len(times) < 3 or (time.perf_counter() < t_end and len(times) < 10):
        t0 = time.perf_counter()
        step()
        times.append(time.perf_counter() - t0)
    times.sort()
    med = times[len(times) // 2]
    return {
        "value": round(2.0 * M_sample * N * K / med / 1e12, 4),
        "unit": "TFLOP/s",
        "cores": torch.get_num_threads(),
        "kind": "port",
        "sample": f"rows 0..{M_sample - 1} of the M=4096 activations, full N={N} K={K}; torch CPU fp32 "
                  f"quant + dequant + matmul, median of {len(times)} runs ({med:.2f} s each), os.cpu_count()={os.cpu_count()}",
    }


def main():
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=20)
    ap.add_argument("--warmup", type=int, default=5)
    ap.add_argument("--no-cpu-baseline", action="store_true")
    ap.add_argument("--no-others", action="store_true")
    ap.add_argument("--only", default=None, help="run just one leg: headline|quant|decode|prefill|grouped|moe|ceiling|copy (for profiling)")
    ap.add_argument("--shape", default=None,
                    help="with --only decode / prefill: just the weight of that name (decode: gate_up, down, lm_head, "
                         "deepseek-v3-gate_up; prefill: gate_up, down, q_a+kv_a, q_b), so that a kernel trace of the "
                         "run averages one shape's launches only")
    ap.add_argument("--rows", default=None, help="with --shape: comma-separated M values instead of the leg's own list")
    args = ap.parse_args()
    if args.gpus != 1:
        print("bench.py measures one GPU's share of the path; this build has no multi-GPU leg (--gpus must be 1)",
              file=sys.stderr)
        sys.exit(2)

    import torch

    from lightllm_amd import _lib
    from lightllm_amd.fused_moe import grouped_matmul, moe_align_fused
    from lightllm_amd.quantization import (lightllm_per_token_group_quant_fp8, per_token_group_quant_fp8,
                                           w8a8_block_fp8_matmul)

    _lib.lib()  # fail loudly if the HIP library is not built
    dev = torch.device("cuda", 0)
    torch.cuda.set_device(dev)
    info = _lib.device_info()
    derived_peak = info["compute_units"] * 4 * 2048 * info["clock_khz"] * 1e3 / 1e12

    M, N, K = 4096, 36864, 7168
    run_all = args.only is None
    rows_only = [int(v) for v in args.rows.split(",")] if args.rows else None
    result = {}
    others = []

    if run_all or args.only == "headline":
        x = make_act(M, K, 0, dev)
        wq, ws = make_weight(N, K, 1, dev)
        xq = torch.empty((M, K), dtype=torch.float8_e4m3fn, device=dev)
        xs = torch.empty((M, K // 128), dtype=torch.float32, device=dev)
        out = torch.empty((M, N), dtype=torch.bfloat16, device=dev)
        wq_t, ws_t = wq.t(), ws.t()

        def step():
            lightllm_per_token_group_quant_fp8(x, 128, xq, xs)
            w8a8_block_fp8_matmul(xq, wq_t, xs, ws_t, out, [128, 128], dtype=torch.bfloat16)

        # The part needs some tens of milliseconds of sustained load before its clocks settle (launch time falls
        # from ~1.1 ms to its steady value over the first ~40 launches), so the measured steps are preceded by an
        # untimed settling run of the same step, then by the W warm-up steps that were asked for.
        settle = 0
        t_settle = time.perf_counter()
        while settle < 200 and time.perf_counter() - t_settle < 0.25:
            for _ in range(10):
                step()
            torch.cuda.synchronize()
            settle += 10
        for _ in range(args.warmup):
            step()
        torch.cuda.synchronize()
        t0 = time.perf_counter()
        ev = _events(2 * args.steps)
        for i in range(args.steps):
            lightllm_per_token_group_quant_fp8(x, 128, xq, xs)
            ev[2 * i].record()          # brackets only the GEMM kernel, on the stream it is launched on
            w8a8_block_fp8_matmul(xq, wq_t, xs, ws_t, out, [128, 128], dtype=torch.bfloat16)
            ev[2 * i + 1].record()
        torch.cuda.synchronize()
        elapsed = time.perf_counter() - t0
        ms_per_step = elapsed * 1e3 / args.steps
        gemm_all = sorted(ev[2 * i].elapsed_time(ev[2 * i + 1]) * 1e3 for i in range(args.steps))
        gemm_us = gemm_all[len(gemm_all) // 2]   # median launch duration
        flops = 2.0 * M * N * K
        value = flops / (ms_per_step * 1e-3) / 1e12
        achieved = flops / (gemm_us * 1e-6) / 1e12
        result = {
            "metric": "block-FP8 GEMM TFLOP/s (% FP8 MFMA peak); quant GB/s (% HBM peak), 1 GPU",
            "value": round(value, 1),
            "unit": "TFLOP/s",
            "n_gpus": 1,
            "steps": args.steps,
            "warmup": args.warmup,
            "ms_per_step": round(ms_per_step, 4),
            "higher_is_better": True,
            "scaling": "weak",
            "vs_baseline": None,
            "dtype": "fp8_e4m3 x fp8_e4m3 -> f32 accumulate -> bf16",
            "data": "synthetic (seeded N(0,1) bf16 activations; N(0,0.02) weights block-quantized 128x128)",
            "config": {
                "workload": "DeepSeek-V3-shaped prefill gate_up linear: per_token_group_quant_fp8([4096,7168] bf16) "
                            "+ w8a8_block_fp8_matmul(M=4096, N=36864, K=7168), bf16 out",
                "M": M, "N": N, "K": K, "block": [128, 128], "clock_settle_steps": settle,
            },
            "roofline": {
                "bound": "mfma",
                "kernel": "block_fp8_gemm_pp_kernel<false,false,true,false,false> (dense 256x256 ping-pong tile, persistent)",
                "achieved": round(achieved, 1),
                "peak": FP8_MFMA_PEAK_TFLOPS,
                "unit": "TFLOP/s",
                "frac": round(achieved / FP8_MFMA_PEAK_TFLOPS, 4),
                # bytes per GEMM launch that cross the L2 (rocprofv3 --pmc FETCH_SIZE and WRITE_SIZE, each scaled by
                # what the same counter reads for a 1 GiB device copy), as the last profile of this kernel recorded
                # them in profiles/traffic.json; null when that file has no entry for the kernel
                "traffic": measured_traffic("gemm_pp_deepseek_gate_up_M4096"),
                "algorithmic_bytes_per_launch": gemm_bytes(M, N, K),
                "launch_us": round(gemm_us, 2),
                "launch_us_min_max": [round(gemm_all[0], 2), round(gemm_all[-1], 2)],
                "algorithmic_flops_per_launch": flops,
                "peak_derived_from_device": round(derived_peak, 1),
            },
        }
        del x, wq, ws, xq, xs, out, wq_t, ws_t
        torch.cuda.empty_cache()

    if (run_all and not args.no_others) or args.only == "quant":
        # standalone quantizer bandwidth test: [16384,7168] with 1% x50 outliers and an all-zero row; the input
        # rotates through 4 distinct tensors (940 MB) and the outputs through 4 more
        Mq, Kq = 16384, 7168
        sets = []
        for c in range(4):
            sets.append((make_act(Mq, Kq, 4 + c, dev, outliers=True),
                         torch.empty((Mq, Kq), dtype=torch.float8_e4m3fn, device=dev),
                         torch.empty((Mq, Kq // 128), dtype=torch.float32, device=dev)))
        nxt = _rotating(sets)

        def call():
            x, xq, xs = nxt()
            lightllm_per_token_group_quant_fp8(x, 128, xq, xs)

        us = _time_calls(call, 20, 5)
        gbs = quant_bytes(Mq, Kq) / us / 1e3
        others.append({"name": "per_token_group_quant_fp8 [16384,7168]", "us": round(us, 2), "GB/s": round(gbs, 1),
                       "frac_hbm": round(gbs / HBM_PEAK_GBS, 4), "rotated_MB": round(4 * Mq * Kq * 2 / 1e6)})
        del sets, nxt
        torch.cuda.empty_cache()
        # the load-time weight quantizer (bf16 -> e4m3fn + one fp32 scale per 128x128 block) and its inverse on the
        # gate_up weight; three sources rotate (1.6 GB); each call also allocates its outputs, as the operator does
        from lightllm_amd.quantization import mm_weight_quant
        from lightllm_amd.quantization.weight_dequant import weight_dequant

        Nw, Kw = 36864, 7168
        srcs = [make_act(Nw, Kw, 60 + c, dev) for c in range(3)]
        nxt = _rotating(srcs)
        us = _time_calls(lambda: mm_weight_quant(nxt()), 6, 3, batches=5)
        byts = Nw * Kw * 3 + (Nw // 128) * (Kw // 128) * 4
        others.append({"name": f"block weight quant [{Nw},{Kw}]", "us": round(us, 1), "GB/s": round(byts / us / 1e3, 1),
                       "frac_hbm": round(byts / us / 1e3 / HBM_PEAK_GBS, 4)})
        wq8, ws8 = mm_weight_quant(srcs[0])
        del srcs, nxt
        us = _time_calls(lambda: weight_dequant(wq8, ws8), 6, 3, batches=5)
        others.append({"name": f"block weight dequant [{Nw},{Kw}]", "us": round(us, 1), "GB/s": round(byts / us / 1e3, 1),
                       "frac_hbm": round(byts / us / 1e3 / HBM_PEAK_GBS, 4)})
        del wq8, ws8
        torch.cuda.empty_cache()

    if (run_all and not args.no_others) or args.only == "decode":
        # Llama-3-8B decode linears (and the DeepSeek-V3 dense gate_up, 264 MB); the weights rotate through enough
        # copies (> 600 MB) that no launch finds them in the 256 MB memory-side cache
        for (Nd, Kd, name) in [(28672, 4096, "gate_up"), (4096, 14336, "down"), (128256, 4096, "lm_head"),
                               (36864, 7168, "deepseek-v3 gate_up")]:
            if args.shape and args.shape != name.replace(" ", "-"):
                continue
            ncopies = -(-640_000_000 // (Nd * Kd))
            copies = [make_weight(Nd, Kd, 10 + c, dev) for c in range(ncopies)]
            views = [(q.t(), s.t()) for q, s in copies]
            for Md in rows_only or (1, 8, 32, 64, 128):
                xq, xs = per_token_group_quant_fp8(make_act(Md, Kd, 20 + Md, dev), 128)
                out = torch.empty((Md, Nd), dtype=torch.bfloat16, device=dev)
                nxt = _rotating(views)

                def call():
                    q_t, s_t = nxt()
                    w8a8_block_fp8_matmul(xq, q_t, xs, s_t, out, [128, 128])

                us = _time_calls(call, 2 * ncopies, ncopies)
                gbs = gemm_bytes(Md, Nd, Kd) / us / 1e3
                model = "" if name.startswith("deepseek") else "llama3-8b "
                others.append({"name": f"{model}{name} M={Md} N={Nd} K={Kd}", "us": round(us, 2),
                               "GB/s": round(gbs, 1), "frac_hbm": round(gbs / HBM_PEAK_GBS, 4),
                               "TFLOP/s": round(2.0 * Md * Nd * Kd / us / 1e6, 2),
                               "rotated_MB": round(ncopies * Nd * Kd / 1e6)})
            del copies, views
            torch.cuda.empty_cache()

    if (run_all and not args.no_others) or args.only == "prefill":
        # the three DeepSeek-V3 prefill linears over M (the shape -> variant table has two thresholds), and one K
        # that is not a multiple of 1024 (q_b: K=1536); each row against its own roofline
        # max(bytes / 8 TB/s, flops / 5.03 PFLOP/s)
        shapes = [(36864, 7168, "gate_up"), (7168, 18432, "down"), (2112, 7168, "q_a+kv_a"), (24576, 1536, "q_b")]
        for (Np, Kp, name) in shapes:
            if args.shape and args.shape != name:
                continue
            # a row whose roofline is its byte term is a stream over the weight: like the decode leg it rotates
            # through enough copies (> 640 MB) that no launch finds the weight in the 256 MB memory-side cache;
            # the compute-bound rows keep one copy
            ncopies = -(-640_000_000 // (Np * Kp))
            copies = [make_weight(Np, Kp, 30 + c, dev) for c in range(ncopies)]
            views = [(q.t(), s.t()) for q, s in copies]
            for Mp in rows_only or (128, 192, 256, 512, 1024, 2048, 4096):
                if name == "gate_up" and Mp == 4096 and not args.shape:
                    continue  # the headline
                flops = 2.0 * Mp * Np * Kp
                nbytes = gemm_bytes(Mp, Np, Kp)
                byte_bound = nbytes / HBM_PEAK_GBS / 1e3 > flops / FP8_MFMA_PEAK_TFLOPS / 1e6
                xq, xs = per_token_group_quant_fp8(make_act(Mp, Kp, 31, dev), 128)
                out = torch.empty((Mp, Np), dtype=torch.bfloat16, device=dev)
                nxt = _rotating(views if byte_bound else views[:1])

                def call():
                    q_t, s_t = nxt()
                    w8a8_block_fp8_matmul(xq, q_t, xs, s_t, out, [128, 128])

                us = _time_calls(call, max(10, 2 * ncopies) if byte_bound else 10, 3, batches=5)
                tf = flops / us / 1e6
                roof = roofline_us(flops, nbytes)
                others.append({"name": f"deepseek-v3 {name} M={Mp} N={Np} K={Kp}", "us": round(us, 2),
                               "TFLOP/s": round(tf, 1), "frac_mfma": round(tf / FP8_MFMA_PEAK_TFLOPS, 4),
                               "roofline_us": round(roof, 2), "frac_roofline": round(roof / us, 4),
                               "bound": "hbm" if byte_bound else "mfma",
                               "rotated_MB": round((ncopies if byte_bound else 1) * Np * Kp / 1e6)})
                del xq, xs, out
            del copies, views
            torch.cuda.empty_cache()

    if (run_all and not args.no_others) or args.only == "grouped":
        # routed experts: 4096 tokens x top-8 over 256 experts, Zipf(1.1) popularity; weights ~N(0, 0.02) bf16,
        # block-quantized expert by expert by the library's load-time quantizer (11.3 GB of e4m3 bytes)
        T, E, topk = 4096, 256, 8
        g = torch.Generator(device=dev).manual_seed(5)
        perm = torch.randperm(E, generator=g, device=dev)
        p = torch.zeros(E, device=dev)
        p[perm] = 1.0 / torch.arange(1, E + 1, device=dev, dtype=torch.float32) ** 1.1
        ids = torch.multinomial((p / p.sum()).expand(T, E), topk, replacement=False, generator=g).to(torch.int32)
        tw = torch.softmax(torch.randn((T, topk), generator=g, device=dev), dim=-1)
        P = T * topk
        e2t = torch.empty((E, P), dtype=torch.int32, device=dev)
        e2w = torch.empty((E, P), dtype=torch.float32, device=dev)
        cnt = torch.empty((E,), dtype=torch.int32, device=dev)
        moe_align_fused(e2t, e2w, cnt, ids, tw)
        experts_hit = int((cnt > 0).sum())

        def expert_weights(Ng, Kg):
            from lightllm_amd.quantization import mm_weight_quant

            w = torch.empty((E, Ng, Kg), dtype=torch.float8_e4m3fn, device=dev)
            sc = torch.empty((E, Ng // 128, Kg // 128), dtype=torch.float32, device=dev)
            for e in range(E):
                wb = (torch.randn((Ng, Kg), generator=g, device=dev, dtype=torch.float32) * 0.02).to(torch.bfloat16)
                w[e], sc[e] = mm_weight_quant(wb)
            return w, sc

        kept = {}
        for (Ng, Kg, tk, mulw, name) in [(4096, 7168, topk, False, "gate_up"), (7168, 2048, 1, True, "down")]:
            w, wscale = expert_weights(Ng, Kg)
            kept[name] = (w, wscale)
            rows = T if tk == topk else P
            xq, xs = per_token_group_quant_fp8(make_act(rows, Kg, 40, dev), 128)
            out = torch.empty((P, Ng), dtype=torch.bfloat16, device=dev)
            us = _time_calls(lambda: grouped_matmul(P, xq, xs, cnt, e2t, e2w, w, wscale, tk, out, mulw, True), 5, 3,
                             batches=5)
            flops = 2.0 * P * Ng * Kg
            byts = experts_hit * Ng * Kg + rows * Kg + 2 * P * Ng
            roof = roofline_us(flops, byts)
            others.append({"name": f"deepseek-v3 routed experts {name}: {P} rows, E={E}, N={Ng} K={Kg}",
                           "us": round(us, 1), "TFLOP/s": round(flops / us / 1e6, 1), "GB/s": round(byts / us / 1e3, 1),
                           "roofline_us": round(roof, 1), "frac_roofline": round(roof / us, 4),
                           "experts_hit": experts_hit})
            del w, wscale, xq, xs, out
            torch.cuda.empty_cache()
        # the whole routed-expert FFN of the layer on the same batch: routing tables, quantizer, gate/up GEMM,
        # fused SiLU-mul + quantizer, down GEMM with the routed weight, sum over the top-k slots
        from lightllm_amd.fused_moe import fused_experts_impl

        hidden = make_act(T, 7168, 41, dev)
        (w1, s1), (w2, s2) = kept["gate_up"], kept["down"]
        us = _time_calls(lambda: fused_experts_impl(hidden, w1, w2, tw, ids, use_fp8_w8a8=True, w1_scale=s1, w2_scale=s2),
                         3, 2, batches=5)
        flops = 2.0 * P * (4096 * 7168 + 7168 * 2048)
        others.append({"name": f"deepseek-v3 routed-expert FFN end to end (fused_experts_impl): {T} tokens, top-{topk} of {E}",
                       "us": round(us, 1), "TFLOP/s": round(flops / us / 1e6, 1)})
        del kept, hidden, w1, s1, w2, s2
        torch.cuda.empty_cache()

    if (run_all and not args.no_others) or args.only == "moe":
        # the element-wise steps of the routed-expert FFN at the same size (32768 rows, intermediate 2048,
        # hidden 7168)
        from lightllm_amd.fused_moe import moe_sum_reduce, silu_and_mul_fwd, silu_and_mul_post_quant_fwd

        Pm, Im, Hm, topk_m = 32768, 2048, 7168, 8
        h1 = make_act(Pm, 2 * Im, 50, dev)
        act = torch.empty((Pm, Im), dtype=torch.bfloat16, device=dev)
        aq = torch.empty((Pm, Im), dtype=torch.float8_e4m3fn, device=dev)
        asc = torch.empty((Pm, Im // 128), dtype=torch.float32, device=dev)
        us = _time_calls(lambda: silu_and_mul_fwd(h1, act), 10, 5)
        byts = Pm * Im * 6
        others.append({"name": f"silu_and_mul [{Pm},{2 * Im}]", "us": round(us, 2), "GB/s": round(byts / us / 1e3, 1),
                       "frac_hbm": round(byts / us / 1e3 / HBM_PEAK_GBS, 4)})
        us = _time_calls(lambda: silu_and_mul_post_quant_fwd(h1, aq, asc), 10, 5)
        byts = Pm * Im * 5 + Pm * (Im // 128) * 4
        others.append({"name": f"silu_and_mul + group quant fused [{Pm},{2 * Im}]", "us": round(us, 2),
                       "GB/s": round(byts / us / 1e3, 1), "frac_hbm": round(byts / us / 1e3 / HBM_PEAK_GBS, 4)})
        del h1, act, aq, asc
        h3 = make_act(Pm, Hm, 51, dev).view(Pm // topk_m, topk_m, Hm)
        red = torch.empty((Pm // topk_m, Hm), dtype=torch.bfloat16, device=dev)
        us = _time_calls(lambda: moe_sum_reduce(h3, red), 10, 5)
        byts = (Pm + Pm // topk_m) * Hm * 2
        others.append({"name": f"moe_sum_reduce [{Pm // topk_m},{topk_m},{Hm}]", "us": round(us, 2),
                       "GB/s": round(byts / us / 1e3, 1), "frac_hbm": round(byts / us / 1e3 / HBM_PEAK_GBS, 4)})
        del h3, red
        torch.cuda.empty_cache()

    if (run_all and not args.no_others) or args.only == "ceiling":
        # What the matrix cores give the path's inner arithmetic at most: the 32 fp8 products of a K step per wave on
        # register-resident operands, accumulated in the matrix core or folded with fp32 scales as the kernels must,
        # on zero and on random e4m3 operands (the part lowers its clock under load, more so on random data).
        gen = torch.Generator(device=dev).manual_seed(7)
        rnd = torch.randint(0, 256, (1 << 17,), generator=gen, device=dev, dtype=torch.uint8)
        rnd = torch.where((rnd & 0x7F) == 0x7F, rnd ^ 1, rnd)   # no NaN codes
        zero = torch.zeros_like(rnd)
        sink = torch.empty((info["compute_units"] * 512,), dtype=torch.float32, device=dev)
        lib = _lib.lib()
        iters = 2000
        for data, dname in ((zero, "zero"), (rnd, "random e4m3")):
            for fold in (0, 1):
                def call():
                    _lib.check(lib.mi355_probe_mfma(data.data_ptr(), sink.data_ptr(), fold, 8, iters,
                                                    _lib.stream_ptr(dev)), "mi355_probe_mfma")
                us = _time_calls(call, 3, 2, batches=5)
                tf = info["compute_units"] * 8 * iters * 32 * 65536.0 / us / 1e6
                others.append({"name": f"ceiling: fp8 MFMA 16x16x128 {'+ fp32 scale fold' if fold else 'accumulating'}, "
                                       f"registers only, {dname} operands", "us": round(us, 1), "TFLOP/s": round(tf, 1),
                               "frac_mfma": round(tf / FP8_MFMA_PEAK_TFLOPS, 4)})
                if fold and data is rnd and result.get("roofline"):
                    # the headline kernel against what its own instruction mix sustains on this box in this run
                    # (the data-sheet fraction moves with the box's clock under load; this ratio does not)
                    result["roofline"]["register_only_mix_TFLOPs"] = round(tf, 1)
                    result["roofline"]["frac_of_register_only_mix"] = round(result["roofline"]["achieved"] / tf, 4)
        del rnd, zero, sink

    if args.only == "copy":
        # calibration for the FETCH_SIZE / WRITE_SIZE counters: a plain device copy of known size
        src = torch.empty(1 << 28, dtype=torch.float32, device=dev).normal_()
        dst = torch.empty_like(src)
        us = _time_calls(lambda: dst.copy_(src), 5, 2, batches=3)
        others.append({"name": "copy 1 GiB (reads 2^30 B, writes 2^30 B per launch)", "us": round(us, 1),
                       "GB/s": round(2 * (1 << 30) / us / 1e3, 1)})

    if not result:
        result = {"metric": "partial run (--only)", "n_gpus": 1}
    if others:
        result["others"] = others
    if run_all and not args.no_cpu_baseline:
        result["cpu_baseline"] = cpu_baseline(2048, N, K)
    print(json.dumps(result))


if __name__ == "__main__":
    main()
