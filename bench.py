#!/usr/bin/env python3
"""Benchmark of the quantized-weight matmul path on one MI355X.

Default workload = BASELINE.json configs[1]: GGUF GEMV at batch 1 and 8 over Llama-8B MLP shapes
(4096->14336 and 14336->4096) in Q8_0 and Q4_K. One step = the eight matmuls of that set, each on
the next of a rotating pool of distinct weight copies (>= 1.5 GB per format and shape) so the 256 MB
Infinity Cache cannot serve them; activations are quantized on the device before the timed region
(the kernels measured are the dequant-fused GEMVs). value = algorithmic bytes of a step / time.

Prints ONE JSON line: metric / value / unit / ms_per_step and the run's parameters, `roofline` (the dominant
kernel's algorithmic bytes or flops per launch over its mean duration by HIP events, against the published peak, and
its measured HBM traffic) and `cpu_baseline` (the CPU restatement on the host cores, a bounded sample). `--workload`
selects other configurations for profiling runs; the default workload is the headline one.
"""
import argparse
import json
import os
import sys
import time

import numpy as np

ROOT = os.path.dirname(os.path.abspath(__file__))
if ROOT not in sys.path:
    sys.path.insert(0, ROOT)

METRIC = "quant GEMV GB/s (% of 8 TB/s); quant GEMM TFLOPS (% MFMA peak); vs CPU"
HBM_PEAK_GBS = 8000.0
POOL_BYTES = 1.5e9

Q8_0, Q4_K, Q6_K = 8, 12, 14
ROW_BYTES = {Q8_0: (32, 34), Q4_K: (256, 144), Q6_K: (256, 210)}
FMT_NAME = {Q8_0: "Q8_0", Q4_K: "Q4_K", Q6_K: "Q6_K"}
KERNEL_FMT = {Q8_0: 1, Q4_K: 2, Q6_K: 3}  # template argument in the kernel symbol
# HBM bytes per launch of the dominant kernel, from rocprofv3 --pmc FETCH_SIZE and WRITE_SIZE runs of this
# benchmark (KiB per dispatch, FETCH_SIZE scaled by 2.000 and WRITE_SIZE by 1.000: what a 256 MiB device copy
# reads on the same counters); the summaries of those runs are kept under profiles/.
TRAFFIC_BYTES = {"decode_batch_kernel": 391571276, "decode_batch_kernel/q6k": 200196474}


def weight_bytes(kind, n_out, n_in):
    bs, ts = ROW_BYTES[kind]
    return n_out * (n_in // bs) * ts


def algorithmic_bytes(kind, n_out, n_in, t):
    """Format-native weight bytes + the quantized activations read (int8 + f32 scale per 32, + f32 half sums
    and int32 sums per 16 where the format uses them) + the f32 outputs written, each counted once."""
    act = t * (n_in + n_in // 32 * 4)
    if kind == Q4_K:
        act += t * (n_in // 16) * 8
    elif kind == Q6_K:
        act += t * (n_in // 16) * 4
    return weight_bytes(kind, n_out, n_in) + act + t * n_out * 4


def gemv_cases(kinds):
    cases = []
    for kind in kinds:
        for n_in, n_out in ((4096, 14336), (14336, 4096)):
            for t in (1, 8):
                cases.append(dict(kind=kind, n_out=n_out, n_in=n_in, t=t,
                                  name=f"{FMT_NAME[kind]}_{n_in}x{n_out}_t{t}",
                                  bytes=algorithmic_bytes(kind, n_out, n_in, t)))
    return cases


def cpu_baseline(cases, gens, seconds=20.0):
    """The oracle's AVX2 restatement of the reference's x86 decode kernels, scheduled like
    matmul_quant_multi_at over all host cores, on the same eight matmuls: best of 5 per case over rotating
    weight copies (so the caches do not help). Tokens up to 8 take the int-dot kernels, as with
    set_decode_max_tokens(8) in the reference's kernel_bench."""
    from oracle import oxref
    from oxinfer_amd import synth
    threads = oxref.hw_threads()
    total_bytes, total_s, per = 0, 0.0, {}
    t_start = time.time()
    host = {}
    for c in cases:
        key = (c["kind"], c["n_out"], c["n_in"])
        if key not in host:
            raw = gens[c["kind"]](c["n_out"], c["n_in"], 1)
            ncopies = max(2, int(np.ceil(4.0e8 / raw.size)))  # 0.4 GB per shape: well past the host caches
            host[key] = [raw] + [raw.copy() for _ in range(ncopies - 1)]
        x = synth.activations(c["t"], c["n_in"], 5)
        best = float("inf")
        copies = host[key]
        reps = 0
        while reps < 5 or (reps < 50 and time.time() - t_start < seconds * 0.1):
            raw = copies[reps % len(copies)]
            t0 = time.perf_counter()
            oxref.gguf_decode(c["kind"], raw, c["n_out"], c["n_in"], x, c["t"], avx2=True, threads=threads)
            best = min(best, time.perf_counter() - t0)
            reps += 1
        per[c["name"]] = round(weight_bytes(c["kind"], c["n_out"], c["n_in"]) / best / 1e9, 2)
        total_bytes += c["bytes"]
        total_s += best
    return {"value": round(total_bytes / total_s / 1e9, 2), "unit": "GB/s", "cores": threads, "kind": "port",
            "sample": "the 8 matmuls of one step, best of >=5 runs each over rotating weight copies; C++ AVX2 "
                      "restatement of kernels_ggml_x86 (int8 dot path, decode_max_tokens >= 8), activation "
                      "quantization included",
            "per_case_weight_GBs": per}


MFMA_PEAK = {"bf16": 2500.0, "i8": 5000.0, "fp8": 5000.0}


def timed_steps(torch, step, steps, warmup):
    """W untimed steps, then K steps between synchronizations: (wall seconds, mean milliseconds between the CUDA/HIP
    events recorded around each step on the launch stream)."""
    for i in range(warmup):
        step(i)
    torch.cuda.synchronize()
    ev = [(torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)) for _ in range(steps)]
    t0 = time.perf_counter()
    for i in range(steps):
        ev[i][0].record()
        step(warmup + i)
        ev[i][1].record()
    torch.cuda.synchronize()
    wall = time.perf_counter() - t0
    return wall, float(np.mean([a.elapsed_time(b) for a, b in ev]))


def other_workload(args, be, torch, synth):
    """The other configurations of BASELINE.json, one JSON line each (profiling and per-config numbers; the default
    workload is the headline one). Weights rotate over >= pool-gb of distinct copies where HBM bounds."""
    base = {"metric": METRIC, "n_gpus": 1, "steps": args.steps, "warmup": args.warmup, "higher_is_better": True,
            "scaling": "weak", "vs_baseline": None, "data": "synthetic"}

    def pool(make, nbytes):
        return [make() for _ in range(max(2, int(np.ceil(args.pool_gb * 1e9 / nbytes))))]

    if args.workload == "mlx_gemv":                      # configs[0]: N = K = 4096, T = 1
        n = k = 4096
        wq, sc, bi = synth.mlx_q4(n, k, 1)
        ws = pool(lambda: be.upload_mlx_q4(wq, sc, bi, 64, n, k), n * k * 0.5625)
        xa = be.quantize_act(torch.from_numpy(synth.activations(1, k, 2)).cuda())
        y = torch.empty((1, n), dtype=torch.float32, device="cuda")
        nbytes = int(n * k * 0.5625) + k * (1 + 4 / 32 + 8 / 32) + n * 4
        # the library's own events: for a single launch they ride on the dispatch (its start and end on the device)
        # (on every fourth step: an event pair costs the host more than this launch takes)
        evs = [(be.event(), be.event()) if i % 4 == 0 else (None, None) for i in range(args.steps)]
        warm = [be.decode_jobs([(ws[i % len(ws)], xa, None, 1, y, None, None)]) for i in range(args.warmup)]
        timed = [be.decode_jobs([(ws[(args.warmup + i) % len(ws)], xa, None, 1, y, evs[i][0], evs[i][1])]) for i in range(args.steps)]
        for arr in warm:
            be.decode_batch(arr)
        torch.cuda.synchronize()
        t0 = time.perf_counter()
        for arr in timed:
            be.decode_batch(arr)
        torch.cuda.synchronize()
        wall = time.perf_counter() - t0
        ms = float(np.mean([be.elapsed_ms(a, b) for a, b in evs if a is not None]))
        ach = nbytes / (ms * 1e-3) / 1e9
        return dict(base, value=round(nbytes * args.steps / wall / 1e9, 2), unit="GB/s", ms_per_step=round(wall / args.steps * 1e3, 5),
                    dtype="int8", config={"workload": "configs[0]: MLX 4-bit g64 GEMV 4096 -> 4096, T = 1", "bytes_per_step": nbytes,
                                          "events": "carried by the launch itself, on every fourth step"},
                    roofline={"bound": "hbm", "achieved": round(ach, 1), "peak": HBM_PEAK_GBS, "unit": "GB/s",
                              "frac": round(ach / HBM_PEAK_GBS, 4), "traffic": None, "kernel": "decode_mfma_kernel<6, 1, ...>",
                              "bytes_per_launch": nbytes, "avg_launch_us": round(ms * 1e3, 2)})

    if args.workload == "mlx_gemm":                      # configs[2]: M = 512, both shapes, variant (a) or (b)
        variant = {"bf16": 0, "i8": 1}[args.variant]
        shapes = [(14336, 4096), (4096, 14336)]
        ws, xs = [], []
        for n, k in shapes:
            wq, sc, bi = synth.mlx_q4(n, k, 3)
            ws.append([be.upload_mlx_q4(wq, sc, bi, 64, n, k) for _ in range(4)])
            xs.append(torch.from_numpy(synth.activations(512, k, 4, bf16=True)).cuda().to(torch.bfloat16))
        flops = sum(2 * 512 * n * k for n, k in shapes)

        def step(i):
            for j in range(2):
                be.gemm(ws[j][i % 4], xs[j], variant=variant)
        wall, ms = timed_steps(torch, step, args.steps, args.warmup)
        ach = flops / (ms * 1e-3) / 1e12
        peak = MFMA_PEAK[args.variant]
        return dict(base, value=round(flops * args.steps / wall / 1e12, 2), unit="TFLOP/s", ms_per_step=round(wall / args.steps * 1e3, 5),
                    dtype="bf16" if variant == 0 else "int8",
                    config={"workload": f"configs[2]: MLX 4-bit g64 prefill GEMM, M = 512, 4096 -> 14336 and 14336 -> 4096, variant {args.variant}",
                            "flops_per_step": flops, "events": "around the two calls of a step (activation packing + GEMM (+ K-slice sum))"},
                    roofline={"bound": "mfma", "achieved": round(ach, 1), "peak": peak, "unit": "TFLOP/s", "frac": round(ach / peak, 4),
                              "traffic": None, "kernel": "gemm_bf16_kernel<6, false, 4>" if variant == 0 else "gemm_i8_q4m_kernel",
                              "flops_per_launch": flops / 2, "avg_launch_us": round(ms * 1e3 / 2, 2)})

    if args.workload == "gguf_gemm":                     # configs[1]'s weights at configs[2]'s token count: M = 512, both shapes
        kind, gen = {"q8_0": (Q8_0, synth.gguf_q8_0), "q4_k": (Q4_K, synth.gguf_q4_k), "q6_k": (Q6_K, synth.gguf_q6_k)}[args.format]
        shapes = [(14336, 4096), (4096, 14336)]
        ws, xs = [], []
        for n, k in shapes:
            raw = gen(n, k, 3)
            ws.append([be.upload_gguf(kind, raw, n, k) for _ in range(4)])
            xs.append(torch.from_numpy(synth.activations(512, k, 4, bf16=True)).cuda().to(torch.bfloat16))
        flops = sum(2 * 512 * n * k for n, k in shapes)

        def step(i):
            for j in range(2):
                be.gemm(ws[j][i % 4], xs[j])
        wall, ms = timed_steps(torch, step, args.steps, args.warmup)
        ach = flops / (ms * 1e-3) / 1e12
        return dict(base, value=round(flops * args.steps / wall / 1e12, 2), unit="TFLOP/s", ms_per_step=round(wall / args.steps * 1e3, 5), dtype="bf16",
                    config={"workload": f"GGUF {args.format.upper()} prefill GEMM, M = 512, 4096 -> 14336 and 14336 -> 4096 (bf16 matrix cores)",
                            "flops_per_step": flops, "events": "around the two calls of a step (activation packing + GEMM (+ K-slice sum))"},
                    roofline={"bound": "mfma", "achieved": round(ach, 1), "peak": MFMA_PEAK["bf16"], "unit": "TFLOP/s", "frac": round(ach / MFMA_PEAK["bf16"], 4),
                              "traffic": None, "kernel": f"gemm_bf16_kernel<{ {'q8_0': 1, 'q4_k': 2, 'q6_k': 3}[args.format]}, false, 4>",
                              "flops_per_launch": flops / 2, "avg_launch_us": round(ms * 1e3 / 2, 2)})

    if args.workload == "moe":                           # configs[3]: 128 experts, top-8, h = 2048, inter = 768
        ne, k, h, inter = 128, 8, 2048, 768
        t = args.tokens or 1
        gu = [synth.mlx_q4(2 * inter, h, 100 + e) for e in range(ne)]
        dn = [synth.mlx_q4(h, inter, 300 + e) for e in range(ne)]
        expert_bytes = int((2 * inter * h + h * inter) * 0.5625)
        devs = pool(lambda: be.upload_moe([be.desc_mlx_q4(*g, 64, 2 * inter, h) for g in gu],
                                          [be.desc_mlx_q4(*d, 64, h, inter) for d in dn], h, inter), ne * expert_bytes)
        x = torch.from_numpy(synth.activations(t, h, 5, bf16=True)).cuda()
        logits = torch.from_numpy(synth.router_logits(t, ne, 6)).cuda()
        idx, w = be.route_top_k(logits, k)
        touched = len(set(idx.cpu().numpy().reshape(-1).tolist()))
        y = torch.zeros((t, h), dtype=torch.float32, device="cuda")
        nbytes = touched * expert_bytes
        flops = 2 * t * k * (2 * inter * h + h * inter)
        # six or more routed rows per expert: the library takes the bf16 form of the grouped matmuls (the reference's prefill form)
        prefill_form = (t * k) // ne >= 6 and os.environ.get("OXHIP_MOE_INT8") != "1"

        def step(i):
            be.route_top_k(logits, k)
            be.dev_moe(devs[i % len(devs)], x, idx, w, y)
        wall, ms = timed_steps(torch, step, args.steps, args.warmup)
        ach = nbytes / (ms * 1e-3) / 1e9
        return dict(base, value=round(nbytes * args.steps / wall / 1e9, 2), unit="GB/s", ms_per_step=round(wall / args.steps * 1e3, 5),
                    dtype="int8" if prefill_form is False else "bf16",
                    config={"workload": f"configs[3]: MoE 128 experts top-8, h 2048, inter 768, MLX 4-bit g64, T = {t}",
                            "experts_touched": touched, "bytes_per_step": nbytes, "flops_per_step": flops,
                            "events": "around routing + the MoE call (" + ("plan + quantize, grouped gate_up, activation + quantize, grouped down, combine)"
                                                                           if not prefill_form else "plan, bf16 fragments of x, grouped gate_up, activation as bf16 fragments, grouped down, combine)")},
                    roofline={"bound": "hbm", "achieved": round(ach, 1), "peak": HBM_PEAK_GBS, "unit": "GB/s",
                              "frac": round(ach / HBM_PEAK_GBS, 4), "traffic": None, "kernel": "moe_bf16_kernel<4> (grouped)" if prefill_form else "decode_mfma_kernel<6, *, false, true, true> (grouped)",
                              "bytes_per_launch": nbytes, "avg_launch_us": round(ms * 1e3, 2)},
                    tflops=round(flops / (ms * 1e-3) / 1e12, 2))

    # configs[4]: FP8 E4M3 [7168, 18432] with 128 x 128 block scales, bf16 activations, bf16 out
    n, k = 7168, 18432
    m = args.tokens or 1024
    data, scales = synth.fp8_e4m3(n, k, 7)
    ws = pool(lambda: be.upload_fp8(data, scales, n, k), n * k)
    x32 = torch.from_numpy(synth.activations(m, k, 8, bf16=True)).cuda()
    xb = x32.to(torch.bfloat16)
    variant = {"bf16": 0, "fp8": 2}.get(args.variant, 0)
    if m <= 16:
        step = lambda i: be.decode(ws[i % len(ws)], x=x32)
        kern = "skinny_fp8_kernel<*, 1, 2, *, false> (+ pack_skinny_kernel)"
    else:
        step = lambda i: be.gemm(ws[i % len(ws)], xb, variant=variant, out_bf16=True)
        kern = ("skinny_fp8_kernel<4, 2, 1, 16, true> (+ pack_skinny_kernel, gemm_reduce_kernel)" if m <= 32 else "gemm_bf16_kernel<4, true, 4>") if variant == 0 else "gemm_fp8_kernel<true>"
    wall, ms = timed_steps(torch, step, args.steps, args.warmup)
    flops, nbytes = 2 * m * n * k, n * k + scales.size * 4 + m * k * 2 + m * n * 2
    hbm = m <= 64
    ach = nbytes / (ms * 1e-3) / 1e9 if hbm else flops / (ms * 1e-3) / 1e12
    peak = HBM_PEAK_GBS if hbm else MFMA_PEAK["bf16" if variant == 0 else "fp8"]
    return dict(base, value=round((nbytes / 1e9 if hbm else flops / 1e12) * args.steps / wall, 2), unit="GB/s" if hbm else "TFLOP/s",
                ms_per_step=round(wall / args.steps * 1e3, 5), dtype="fp8 weights, " + ("f32" if m <= 16 else ("bf16" if variant == 0 else "fp8")) + " activations",
                config={"workload": f"configs[4]: FP8 E4M3 block-scaled GEMM [7168, 18432], M = {m}, variant {args.variant if m > 16 else 'decode'}",
                        "bytes_per_step": nbytes, "flops_per_step": flops},
                roofline={"bound": "hbm" if hbm else "mfma", "achieved": round(ach, 1), "peak": peak, "unit": "GB/s" if hbm else "TFLOP/s",
                          "frac": round(ach / peak, 4), "traffic": None, "kernel": kern, "avg_launch_us": round(ms * 1e3, 2)})


def main():
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=200)
    ap.add_argument("--warmup", type=int, default=20)
    ap.add_argument("--workload", default="gguf_gemv", choices=["gguf_gemv", "gguf_gemv_q6k", "gguf_stream", "gguf_gemm", "mlx_gemv", "mlx_gemm", "moe", "fp8", "copy"],
                    help="copy = a plain 256 MiB device copy, the known-size kernel that scales the HBM traffic counters; "
                         "gguf_stream = every GGUF case alone as a steady stream of 192 matmuls handed over in one call")
    ap.add_argument("--no-cpu", action="store_true", help="skip the CPU baseline leg")
    ap.add_argument("--event-every", type=int, default=1,
                    help="gguf_gemv: the launch of every n-th timed step carries the timing events (with n > 1 the launches run closer "
                         "together: the whole-job figure rises ~3 %, and a timed launch shares the device with its predecessor's tail)")
    ap.add_argument("--pool-gb", type=float, default=POOL_BYTES / 1e9)
    ap.add_argument("--variant", default="bf16", choices=["bf16", "i8", "fp8"], help="GEMM variant of mlx_gemm / fp8")
    ap.add_argument("--format", default="q4_k", choices=["q8_0", "q4_k", "q6_k"], help="weight format of the gguf_gemm workload")
    ap.add_argument("--tokens", type=int, default=0, help="tokens of the moe (1 or 256) and fp8 (1, 32, 1024) workloads")
    args = ap.parse_args()
    if args.gpus != 1:
        print("bench.py: this build measures one GPU; --gpus must be 1 (nothing here uses a second device)", file=sys.stderr)
        sys.exit(2)

    import torch
    from oxinfer_amd import HipBackend, synth
    if not torch.cuda.is_available():
        print("bench.py: no GPU visible; the HIP path has no CPU fallback", file=sys.stderr)
        sys.exit(1)
    torch.cuda.set_device(0)
    if args.workload == "copy":
        n = 256 << 20
        src = torch.full((n,), 3, dtype=torch.uint8, device="cuda")
        dst = torch.empty_like(src)
        for _ in range(args.warmup + args.steps):
            dst.copy_(src)
        torch.cuda.synchronize()
        print(json.dumps({"workload": "copy", "bytes_read": n, "bytes_written": n, "launches": args.warmup + args.steps}))
        return
    be = HipBackend(0)
    if args.workload in ("mlx_gemv", "mlx_gemm", "gguf_gemm", "moe", "fp8"):
        print(json.dumps(other_workload(args, be, torch, synth)))
        be.close()
        return
    gens = {Q8_0: synth.gguf_q8_0, Q4_K: synth.gguf_q4_k, Q6_K: synth.gguf_q6_k}
    kinds = [Q8_0, Q4_K] if args.workload == "gguf_gemv" else [Q6_K] if args.workload == "gguf_gemv_q6k" else [Q8_0, Q4_K, Q6_K]
    cases = gemv_cases(kinds)

    # rotating pools of distinct device copies per (format, shape)
    pools = {}
    for c in cases:
        key = (c["kind"], c["n_out"], c["n_in"])
        if key in pools:
            continue
        raw = gens[c["kind"]](c["n_out"], c["n_in"], 1)
        n = max(2, int(np.ceil(args.pool_gb * 1e9 / raw.size)))
        pools[key] = []
        for _ in range(n):
            w = be.upload_gguf(c["kind"], raw, c["n_out"], c["n_in"])
            if w is None:
                raise RuntimeError(be.last_error())
            pools[key].append(w)
    for c in cases:
        x = torch.from_numpy(synth.activations(c["t"], c["n_in"], 5)).cuda()
        c["xa"] = be.quantize_act(x)
        c["y"] = torch.empty((c["t"], c["n_out"]), dtype=torch.float32, device="cuda")
        c["pool"] = pools[(c["kind"], c["n_out"], c["n_in"])]
    torch.cuda.synchronize()

    if args.workload == "gguf_stream":
        # Each case alone, 192 matmuls over rotating weight copies in one call (launches of 16, back to back): what the
        # kernel streams at when no launch boundary, ramp or tail is in the way. One JSON line; `value` is the mean.
        detail, tot_b, tot_s = {}, 0.0, 0.0
        for c in cases:
            pool = c["pool"]
            arr = be.decode_jobs([(pool[i % len(pool)], c["xa"], None, c["t"], c["y"], None, None) for i in range(192)])
            be.decode_batch(arr)
            torch.cuda.synchronize()
            e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
            e0.record()
            be.decode_batch(arr)
            e1.record()
            torch.cuda.synchronize()
            us = e0.elapsed_time(e1) * 1e3 / 192
            detail[c["name"]] = {"us": round(us, 2), "GBs": round(c["bytes"] / us / 1e3, 1), "frac_hbm": round(c["bytes"] / us / 1e3 / HBM_PEAK_GBS, 4)}
            tot_b += c["bytes"]
            tot_s += us * 1e-6
        print(json.dumps({"metric": METRIC, "value": round(tot_b / tot_s / 1e9, 2), "unit": "GB/s", "n_gpus": 1, "higher_is_better": True,
                          "vs_baseline": None, "dtype": "int8", "data": "synthetic",
                          "config": {"workload": "GGUF GEMV cases of configs[1] (and Q6_K), each as a steady stream of 192 matmuls in one call"},
                          "detail": detail}))
        be.close()
        return

    # The dominant kernel. The jobs of one call share one launch (decode_batch_kernel): that launch is the step, and
    # its events bracket it. (Formats the shared launch does not take would launch one by one: then the largest
    # matmul at the larger batch is timed.)
    shared = all(k in (Q8_0, Q4_K, Q6_K) for k in kinds)
    dom_kind = kinds[0]
    for c in cases:
        c["dom"] = shared or (c["kind"] == dom_kind and c["t"] == 8)
    dom = [c for c in cases if c["dom"]]
    per_step = 1 if shared else len(dom)
    dom_symbol = "decode_batch_kernel"

    # One call per step: the job arrays (one per rotation phase) are built once; the dominant launches of every
    # `--event-every`-th step (default: every step) carry HIP events recorded by the library on the launch stream. An
    # event pair on a launch leaves a gap of a few microseconds before the next one; without it a launch starts in the
    # tail of its predecessor, so its own duration reads longer.
    every = max(1, args.event_every)
    n_timed = (args.steps + every - 1) // every
    n_ev = n_timed * per_step
    ev = [(be.event(), be.event()) for _ in range(min(n_ev, 4096))]

    def jobs_for(i, timed_slot=None):
        jobs, k = [], 0
        for n, c in enumerate(cases):
            w = c["pool"][(2 * i + (c["t"] > 1)) % len(c["pool"])]
            e0 = e1 = None
            if timed_slot is not None and shared:
                pair = ev[timed_slot % len(ev)]
                e0 = pair[0] if n == 0 else None
                e1 = pair[1] if n == len(cases) - 1 else None
            elif timed_slot is not None and c["dom"]:
                e0, e1 = ev[(timed_slot * per_step + k) % len(ev)]
                k += 1
            jobs.append((w, c["xa"], None, c["t"], c["y"], e0, e1))
        return be.decode_jobs(jobs)

    warm = [jobs_for(i) for i in range(args.warmup)]
    timed = [jobs_for(args.warmup + i, i // every if i % every == 0 else None) for i in range(args.steps)]
    for arr in warm:
        be.decode_batch(arr)
    torch.cuda.synchronize()
    t0 = time.perf_counter()
    for arr in timed:
        be.decode_batch(arr)
    torch.cuda.synchronize()
    elapsed = time.perf_counter() - t0
    used = min(n_ev, len(ev))
    dom_ms = [be.elapsed_ms(a, b) for a, b in ev[:used]]

    step_bytes = sum(c["bytes"] for c in cases)
    value = step_bytes * args.steps / elapsed / 1e9
    dom_avg_s = float(np.mean(dom_ms)) / 1e3
    dom_bytes = float(step_bytes) if shared else float(np.mean([c["bytes"] for c in dom]))
    achieved = dom_bytes / dom_avg_s / 1e9

    # per-case detail (untimed pass, one event pair per launch)
    detail = {}
    for c in cases:
        ms = []
        for i in range(30):
            w = c["pool"][i % len(c["pool"])]
            arr = be.decode_jobs([(w, c["xa"], None, c["t"], c["y"], ev[0][0], ev[0][1])])
            be.decode_batch(arr)
            ms.append(be.elapsed_ms(ev[0][0], ev[0][1]))
        us = float(np.median(ms)) * 1e3
        detail[c["name"]] = {"us": round(us, 2), "GBs": round(c["bytes"] / us / 1e3, 1),
                             "frac_hbm": round(c["bytes"] / us / 1e3 / HBM_PEAK_GBS, 4)}

    out = {
        "metric": METRIC, "value": round(value, 2), "unit": "GB/s", "n_gpus": 1, "steps": args.steps,
        "warmup": args.warmup, "ms_per_step": round(elapsed / args.steps * 1e3, 5), "higher_is_better": True,
        "scaling": "weak", "vs_baseline": None, "dtype": "int8", "data": "synthetic",
        "config": {"workload": "configs[1]: GGUF GEMV batch 1 and 8, Llama-8B MLP shapes 4096->14336 and 14336->4096, "
                               + " + ".join(FMT_NAME[k] for k in kinds),
                   "matmuls_per_step": len(cases), "launches_per_step": 1 if shared else len(cases), "bytes_per_step": step_bytes,
                   "weight_pool_GB_per_shape": args.pool_gb, "activations": "int8 per 32 (quantize_act), resident in HBM",
                   "events": f"on the launch of every {every}. step ({min(n_ev, len(ev))} timed launches)"},
        "roofline": {"bound": "hbm", "achieved": round(achieved, 1), "peak": HBM_PEAK_GBS, "unit": "GB/s",
                     "frac": round(achieved / HBM_PEAK_GBS, 4), "traffic": TRAFFIC_BYTES.get(dom_symbol if all(k in (Q8_0, Q4_K) for k in kinds) else dom_symbol + "/q6k"), "kernel": dom_symbol,
                     "bytes_per_launch": dom_bytes, "avg_launch_us": round(dom_avg_s * 1e6, 2)},
        "frac_of_hbm_peak": round(value / HBM_PEAK_GBS, 4),
        "detail": detail,
    }
    if not args.no_cpu:
        out["cpu_baseline"] = cpu_baseline(cases, gens)
    print(json.dumps(out))
    be.close()


if __name__ == "__main__":
    main()
