#!/usr/bin/env python3
"""Benchmark of the quantized-weight matmul path on one MI355X.

Headline workload = BASELINE.json configs[1]: GGUF GEMV at batch 1 and 8 over Llama-8B MLP shapes
(4096->14336 and 14336->4096) in Q8_0 and Q4_K. One step = the activation quantization of the four inputs (one
launch) and the eight matmuls of that set (one launch), each matmul on the next of a rotating pool of distinct
weight copies (>= 1.5 GB per format and shape) so the 256 MB Infinity Cache cannot serve them; the f32 inputs are
resident in HBM when the timed region starts. value = algorithmic bytes of a step / wall time per step.

Prints ONE JSON line: metric / value / unit / ms_per_step and the run's parameters, `roofline` (the dominant
kernel's algorithmic bytes per launch over its mean duration by HIP events, against the published peak, and its
measured HBM traffic from the kept profile), `cpu_baseline` (the CPU restatement on the host cores, a bounded
sample) and `per_config`: every other configuration of BASELINE.json measured in the same run (value, dominant
kernel, mean time, roofline fraction, and its own CPU baseline). `--workload` runs one configuration alone (for
profiling runs) and prints that configuration's full line.
"""
import argparse
import json
import os
import re
import sys
import time

import numpy as np

ROOT = os.path.dirname(os.path.abspath(__file__))
if ROOT not in sys.path:
    sys.path.insert(0, ROOT)

METRIC = "quant GEMV GB/s (% of 8 TB/s); quant GEMM TFLOPS (% MFMA peak); vs CPU"
HBM_PEAK_GBS = 8000.0
MFMA_PEAK = {"bf16": 2500.0, "i8": 5000.0, "fp8": 5000.0}
POOL_BYTES = 1.5e9

Q8_0, Q4_K, Q6_K = 8, 12, 14
ROW_BYTES = {Q8_0: (32, 34), Q4_K: (256, 144), Q6_K: (256, 210)}
FMT_NAME = {Q8_0: "Q8_0", Q4_K: "Q4_K", Q6_K: "Q6_K"}


def profile_traffic(profile):
    """HBM bytes per launch of a roofline figure's kernel(s) from the kept rocprofv3 summary `profiles/<profile>`: its
    "Roofline traffic:" line (FETCH_SIZE + WRITE_SIZE per dispatch, each scaled by what the counter reads for a plain
    device copy of known size, summed over the launches the figure's time covers); None when the summary or the line
    is missing."""
    try:
        text = open(os.path.join(ROOT, "profiles", profile or "-")).read()
    except OSError:
        return None
    m = re.search(r"^Roofline traffic: (\d+) bytes", text, re.M)
    return int(m.group(1)) if m else None


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


def best_of(fn, min_reps, seconds):
    """Best wall time of fn(i) over at least min_reps runs and about `seconds` of them."""
    best, reps, t_start = float("inf"), 0, time.time()
    while reps < min_reps or (reps < 200 and time.time() - t_start < seconds):
        t0 = time.perf_counter()
        fn(reps)
        best = min(best, time.perf_counter() - t0)
        reps += 1
    return best, reps


# ---------------------------------------------------------------------------------------------------------------
# CPU baselines: the oracle's C++ restatement of the reference's x86 kernels, on all host cores (kind "port": the
# reference is Rust and cannot be built here). Each is a bounded sample of its configuration.
# ---------------------------------------------------------------------------------------------------------------
def cpu_gguf_gemv(cases, gens, seconds=16.0):
    """The AVX2 restatement of kernels_ggml_x86 scheduled like matmul_quant_multi_at over all host cores, on the same
    eight matmuls: best of >= 5 per case over rotating weight copies (so the caches do not help). Tokens up to 8 take
    the int-dot kernels, as with set_decode_max_tokens(8) in the reference's kernel_bench."""
    from oracle import oxref
    from oxinfer_amd import synth
    threads = oxref.hw_threads()
    total_bytes, total_s, per, host = 0, 0.0, {}, {}
    for c in cases:
        key = (c["kind"], c["n_out"], c["n_in"])
        if key not in host:
            raw = gens[c["kind"]](c["n_out"], c["n_in"], 1)
            ncopies = max(2, int(np.ceil(4.0e8 / raw.size)))  # 0.4 GB per shape: well past the host caches
            host[key] = [raw] + [raw.copy() for _ in range(ncopies - 1)]
        x = synth.activations(c["t"], c["n_in"], 5)
        copies = host[key]
        best, _ = best_of(lambda i: oxref.gguf_decode(c["kind"], copies[i % len(copies)], c["n_out"], c["n_in"], x, c["t"], avx2=True, threads=threads),
                          5, seconds / len(cases))
        per[c["name"]] = round(weight_bytes(c["kind"], c["n_out"], c["n_in"]) / best / 1e9, 2)
        total_bytes += c["bytes"]
        total_s += best
    return {"value": round(total_bytes / total_s / 1e9, 2), "unit": "GB/s", "cores": threads, "kind": "port",
            "sample": "the 8 matmuls of one step, best of >= 5 runs each over rotating weight copies; C++ AVX2 "
                      "restatement of kernels_ggml_x86 (int8 dot path, decode_max_tokens >= 8), activation "
                      "quantization included",
            "per_case_weight_GBs": per}


def cpu_mlx_gemv(seconds=3.0):
    from oracle import oxref
    from oxinfer_amd import synth
    n = k = 4096
    q, s16, off = oxref.from_mlx_q4(*synth.mlx_q4(n, k, 1), n, k, 64)
    copies = [(q.copy(), s16.copy(), off.copy()) for _ in range(40)]  # 0.4 GB
    x = synth.activations(1, k, 2)
    threads = oxref.hw_threads()
    best, reps = best_of(lambda i: oxref.q4_decode(*copies[i % len(copies)], 64, n, k, x, 1, avx2=True, threads=threads), 20, seconds)
    nbytes = int(n * k * 0.5625) + k * 4 + n * 4
    return {"value": round(nbytes / best / 1e9, 2), "unit": "GB/s", "cores": threads, "kind": "port",
            "sample": f"the whole matmul, best of {reps} runs over 40 rotating weight copies; AVX2 restatement of q4_dot_rows_tc_avx2 + add_offsets "
                      "(src/kernels_x86.rs:476-519), activation quantization included"}


def cpu_mlx_gemm(seconds=6.0):
    """The x86 prefill path (dequantize 8 rows, f32 FMA GEMM; src/kernels.rs:1998-2038) over both shapes; the reference's
    int8 GEMM is aarch64-only, so on these host cores this is the CPU path of both variants."""
    from oracle import oxref
    from oxinfer_amd import synth
    threads = oxref.hw_threads()
    total_f, total_s = 0.0, 0.0
    for n, k in ((14336, 4096), (4096, 14336)):
        q, s16, off = oxref.from_mlx_q4(*synth.mlx_q4(n, k, 3), n, k, 64)
        x = synth.activations(512, k, 4, bf16=True)
        best, _ = best_of(lambda i: oxref.gemm_quant(-1, q, s16, off, n, k, x, 512, threads=threads), 2, seconds / 2)
        total_f += 2.0 * 512 * n * k
        total_s += best
    return {"value": round(total_f / total_s / 1e12, 3), "unit": "TFLOP/s", "cores": threads, "kind": "port",
            "sample": "both shapes whole, best of >= 2 runs each; restatement of matmul_quant_block_prefill + gemm_8x8_avx2 "
                      "(dequantize 8 rows to f32, one fma chain per output)"}


def cpu_moe(t, experts, seconds=4.0):
    from oracle import oxref
    from oxinfer_amd import synth
    ne, k, h, inter = 128, 8, 2048, 768
    q_gu = [oxref.from_mlx_q4(*g, 2 * inter, h, 64) for g in experts[0]]
    q_dn = [oxref.from_mlx_q4(*d, h, inter, 64) for d in experts[1]]
    x = synth.activations(t, h, 5, bf16=True)
    logits = synth.router_logits(t, ne, 6)
    idx = np.zeros((t, k), np.uint32)
    w = np.zeros((t, k), np.float32)
    for i in range(t):
        idx[i], w[i] = oxref.route_top_k(logits[i], k)
    y0 = np.zeros((t, h), np.float32)
    threads = oxref.hw_threads()
    touched = len(set(idx.reshape(-1).tolist()))
    if t < 8:
        fn = lambda i: oxref.moe_q4(q_gu, q_dn, 64, h, inter, x, t, idx, w, y0, decode_path=True, avx2=True, threads=threads)
        what = "the whole pass (8 experts stay in the host caches), AVX2 int8 decode kernels in one parallel region per projection (forward_batched + matmul_quant_batch)"
    else:
        fn = lambda i: oxref.moe_q4(q_gu, q_dn, 64, h, inter, x, t, idx, w, y0, decode_path=False)
        what = "the whole pass, grouped f32 path (dequantize + f32 FMA GEMM per expert, Act::scalar), experts in parallel"
    best, reps = best_of(fn, 3, seconds)
    nbytes = touched * int((2 * inter * h + h * inter) * 0.5625)
    return {"value": round(nbytes / best / 1e9, 2), "unit": "GB/s", "cores": threads, "kind": "port",
            "sample": f"{what}; best of {reps} runs", "tflops": round(2 * t * k * (2 * inter * h + h * inter) / best / 1e12, 4)}


def cpu_fp8(m, data, scales, seconds=6.0):
    """dequantize_rows + the f32 GEMM (float-stored matrices take the f32 path at every M, src/kernels.rs:1802). At
    M = 1024 a quarter of the rows is timed (the work is uniform over rows) and scaled."""
    from oracle import oxref
    from oxinfer_amd import synth
    n, k = data.shape
    rows = n if m < 1024 else n // 4
    x = synth.activations(m, k, 8, bf16=True)
    threads = oxref.hw_threads()
    sub = np.ascontiguousarray(data[:rows])
    best, reps = best_of(lambda i: oxref.gemm_quant(oxref.F8E4M3, sub, scales, None, rows, k, x, m, threads=threads), 2, seconds)
    flops = 2.0 * m * rows * k
    hbm = m <= 64
    val = (rows * k + m * k * 4 + m * rows * 4) / best / 1e9 if hbm else flops / best / 1e12
    return {"value": round(val, 3), "unit": "GB/s" if hbm else "TFLOP/s", "cores": threads, "kind": "port",
            "sample": f"rows 0..{rows} of {n} (all columns), best of {reps} runs; restatement of dequantize_rows (e4m3 x block scale) + gemm_8x8_avx2"}


# ---------------------------------------------------------------------------------------------------------------
# GPU legs. Each returns the configuration's full line.
# ---------------------------------------------------------------------------------------------------------------
def base_line(steps, warmup):
    return {"metric": METRIC, "n_gpus": 1, "steps": steps, "warmup": warmup, "higher_is_better": True,
            "scaling": "weak", "vs_baseline": None, "data": "synthetic"}


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


def timed_gemm_steps(be, torch, calls, steps, warmup):
    """calls(i) -> the step's GEMM calls as (weight, x, kwargs). Two passes of W untimed and K timed steps: a plain one
    for the wall time and the whole step by events around it, then one in which the library records events right
    before and after each call's matrix kernel (their recording costs the stream a few microseconds per call, which is
    why the first pass does without). Returns (wall seconds, mean milliseconds of a step, mean milliseconds of one
    call's matrix kernel)."""
    def step(i):
        for w, x, kw in calls(i):
            be.gemm(w, x, **kw)
    wall, step_ms = timed_steps(torch, step, steps, warmup)
    n = len(calls(0))
    kev = [[(be.event(), be.event()) for _ in range(n)] for _ in range(steps)]
    for i in range(steps):
        for (w, x, kw), e in zip(calls(warmup + i), kev[i]):
            be.gemm(w, x, events=e, **kw)
    torch.cuda.synchronize()
    kern_ms = float(np.mean([be.elapsed_ms(a, b) for row in kev for a, b in row]))
    for row in kev:
        for a, b in row:
            be.lib.oxhip_event_destroy(a)
            be.lib.oxhip_event_destroy(b)
    return wall, step_ms, kern_ms


GEMM_EVENTS = ("recorded by the library right before and after each call's matrix kernel (oxhip_dev_gemm_timed) in a second pass; "
               "value, ms_per_step and call_us are the first pass's whole calls: activation packing or quantization + that kernel (+ K-slice sum)")


def make_pool(make, nbytes, pool_gb):
    return [make() for _ in range(max(2, int(np.ceil(pool_gb * 1e9 / nbytes))))]


def bench_mlx_gemv(be, torch, synth, steps, warmup, pool_gb):
    """configs[0]: N = K = 4096, T = 1. Three figures: the single launch over rotating copies (cold HBM; `value` and
    `roofline`), the shared launch of a layer's four 4096 x 4096 matmuls (q/k/v/o) over rotating copies, and the
    single launch on one copy (cache-resident)."""
    n = k = 4096
    wq, sc, bi = synth.mlx_q4(n, k, 1)
    ws = make_pool(lambda: be.upload_mlx_q4(wq, sc, bi, 64, n, k), n * k * 0.5625, pool_gb)
    x = torch.from_numpy(synth.activations(1, k, 2)).cuda()
    xa = be.quantize_act(x)
    ys = [torch.empty((1, n), dtype=torch.float32, device="cuda") for _ in range(4)]
    nbytes = int(n * k * 0.5625) + k * (1 + 4 / 32 + 8 / 32) + n * 4

    def run(jobs_of, per_call):
        # the library's own events ride on the dispatch (its start and end on the device), on every fourth step: an
        # event pair costs the host more than this launch takes
        evs = [(be.event(), be.event()) if i % 4 == 0 else (None, None) for i in range(steps)]
        warm = [be.decode_jobs(jobs_of(i, None, None)) for i in range(warmup)]
        timed = [be.decode_jobs(jobs_of(warmup + i, *evs[i])) for i in range(steps)]
        for arr in warm:
            be.decode_batch(arr)
        torch.cuda.synchronize()
        t0 = time.perf_counter()
        for arr in timed:
            be.decode_batch(arr)
        torch.cuda.synchronize()
        wall = time.perf_counter() - t0
        ms = float(np.mean([be.elapsed_ms(a, b) for a, b in evs if a is not None]))
        return wall, ms

    single = lambda i, e0, e1: [(ws[i % len(ws)], xa, None, 1, ys[0], e0, e1)]
    four = lambda i, e0, e1: [(ws[(4 * i + j) % len(ws)], xa, None, 1, ys[j], e0 if j == 0 else None, e1 if j == 3 else None) for j in range(4)]
    hot = lambda i, e0, e1: [(ws[0], xa, None, 1, ys[0], e0, e1)]
    wall, ms = run(single, 1)
    _, ms4 = run(four, 4)
    _, msh = run(hot, 1)
    # a steady stream: 192 matmuls over rotating copies handed over in one call (shared launches of 16, back to back)
    arr = be.decode_jobs([(ws[i % len(ws)], xa, None, 1, ys[i % 4], None, None) for i in range(192)])
    be.decode_batch(arr)
    torch.cuda.synchronize()
    e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
    e0.record()
    be.decode_batch(arr)
    e1.record()
    torch.cuda.synchronize()
    us_stream = e0.elapsed_time(e1) * 1e3 / 192
    ach = nbytes / (ms * 1e-3) / 1e9
    line = dict(base_line(steps, warmup), value=round(nbytes * steps / wall / 1e9, 2), unit="GB/s", ms_per_step=round(wall / steps * 1e3, 5),
                dtype="int8", config={"workload": "configs[0]: MLX 4-bit g64 GEMV 4096 -> 4096, T = 1", "bytes_per_step": nbytes,
                                      "events": "carried by the launch itself, on every fourth step"},
                roofline={"bound": "hbm", "achieved": round(ach, 1), "peak": HBM_PEAK_GBS, "unit": "GB/s",
                          "frac": round(ach / HBM_PEAK_GBS, 4), "traffic": profile_traffic("decode_mfma_kernel_mlx_gemv.md"), "kernel": "decode_mfma_kernel<6, 1, ...>",
                          "bytes_per_launch": nbytes, "avg_launch_us": round(ms * 1e3, 2)})
    line["shared_launch_of_4"] = {"what": "a layer's four 4096 x 4096 matmuls (q, k, v, o) in one oxhip_dev_decode_batch launch, rotating copies (cold HBM)",
                                  "kernel": "decode_batch_kernel", "avg_launch_us": round(ms4 * 1e3, 2), "GBs": round(4 * nbytes / (ms4 * 1e-3) / 1e9, 1),
                                  "frac_hbm": round(4 * nbytes / (ms4 * 1e-3) / 1e9 / HBM_PEAK_GBS, 4)}
    line["steady_stream"] = {"what": "192 matmuls over rotating copies in one call (launches of 16 back to back): what the kernel streams at without launch boundaries",
                             "us_per_matmul": round(us_stream, 2), "GBs": round(nbytes / us_stream / 1e3, 1),
                             "frac_hbm": round(nbytes / us_stream / 1e3 / HBM_PEAK_GBS, 4)}
    line["cache_resident"] = {"what": "the single launch on one weight copy (9.4 MB stays in the 256 MB Infinity Cache)",
                              "avg_launch_us": round(msh * 1e3, 2), "GBs": round(nbytes / (msh * 1e-3) / 1e9, 1)}
    return line


def bench_mlx_gemm(be, torch, synth, steps, warmup, variant_name):
    """configs[2]: M = 512, both shapes, variant (a) bf16 or (b) i8."""
    variant = {"bf16": 0, "i8": 1}[variant_name]
    shapes = [(14336, 4096), (4096, 14336)]
    ws, xs = [], []
    for n, k in shapes:
        wq, sc, bi = synth.mlx_q4(n, k, 3)
        ws.append([be.upload_mlx_q4(wq, sc, bi, 64, n, k) for _ in range(4)])
        xs.append(torch.from_numpy(synth.activations(512, k, 4, bf16=True)).cuda().to(torch.bfloat16))
    flops = sum(2 * 512 * n * k for n, k in shapes)

    calls = lambda i: [(ws[j][i % 4], xs[j], {"variant": variant}) for j in range(2)]
    wall, step_ms, ms = timed_gemm_steps(be, torch, calls, steps, warmup)
    ach = flops / 2 / (ms * 1e-3) / 1e12
    peak = MFMA_PEAK[variant_name]
    roof = {"bound": "mfma", "achieved": round(ach, 1), "peak": peak, "unit": "TFLOP/s", "frac": round(ach / peak, 4),
            "traffic": profile_traffic("gemm_bf16_kernel_mlx_prefill.md" if variant == 0 else "gemm_i8_q4m_kernel_mlx_prefill.md"),
            "kernel": "gemm_bf16_kernel<6, false, 2, 8, 7|8>" if variant == 0 else "gemm_i8_q4m_kernel",
            "flops_per_launch": flops / 2, "avg_launch_us": round(ms * 1e3, 2), "call_us": round(step_ms * 1e3 / 2, 2)}
    if variant == 1:
        # one activation scale per token and block of 32: every int8 matrix instruction (16 x 16 x 32) is followed by a
        # conversion and a multiply-add per accumulator and the scale products, >= 8 VALU cycles-worth next to its 8:
        # the variant's semantics bound it near a fifth of the int8 peak
        roof["ceiling"] = {"frac_of_peak": 0.2, "why": "per-(token, 32-block) f32 rescale: >= 8 VALU instructions per mfma_i32_16x16x32_i8"}
    return dict(base_line(steps, warmup), value=round(flops * steps / wall / 1e12, 2), unit="TFLOP/s", ms_per_step=round(wall / steps * 1e3, 5),
                dtype="bf16" if variant == 0 else "int8",
                config={"workload": f"configs[2]: MLX 4-bit g64 prefill GEMM, M = 512, 4096 -> 14336 and 14336 -> 4096, variant {variant_name}",
                        "flops_per_step": flops, "events": GEMM_EVENTS},
                roofline=roof)


def bench_gguf_gemm(be, torch, synth, steps, warmup, fmt):
    """configs[1]'s weights at configs[2]'s token count: M = 512, both shapes."""
    kind, gen = {"q8_0": (Q8_0, synth.gguf_q8_0), "q4_k": (Q4_K, synth.gguf_q4_k), "q6_k": (Q6_K, synth.gguf_q6_k)}[fmt]
    shapes = [(14336, 4096), (4096, 14336)]
    ws, xs = [], []
    for n, k in shapes:
        raw = gen(n, k, 3)
        ws.append([be.upload_gguf(kind, raw, n, k) for _ in range(4)])
        xs.append(torch.from_numpy(synth.activations(512, k, 4, bf16=True)).cuda().to(torch.bfloat16))
    flops = sum(2 * 512 * n * k for n, k in shapes)

    calls = lambda i: [(ws[j][i % 4], xs[j], {}) for j in range(2)]
    wall, step_ms, ms = timed_gemm_steps(be, torch, calls, steps, warmup)
    ach = flops / 2 / (ms * 1e-3) / 1e12
    return dict(base_line(steps, warmup), value=round(flops * steps / wall / 1e12, 2), unit="TFLOP/s", ms_per_step=round(wall / steps * 1e3, 5), dtype="bf16",
                config={"workload": f"GGUF {fmt.upper()} prefill GEMM, M = 512, 4096 -> 14336 and 14336 -> 4096 (bf16 matrix cores)",
                        "flops_per_step": flops, "events": GEMM_EVENTS},
                roofline={"bound": "mfma", "achieved": round(ach, 1), "peak": MFMA_PEAK["bf16"], "unit": "TFLOP/s", "frac": round(ach / MFMA_PEAK["bf16"], 4),
                          "traffic": profile_traffic(f"gemm_bf16_kernel_gguf_{fmt}_prefill.md"),
                          "kernel": f"gemm_bf16_kernel<{ {'q8_0': 1, 'q4_k': 2, 'q6_k': 3}[fmt]}, false, 2, 8, 7|8>",
                          "flops_per_launch": flops / 2, "avg_launch_us": round(ms * 1e3, 2), "call_us": round(step_ms * 1e3 / 2, 2)})


def bench_gguf_layer(be, torch, synth, steps, warmup, t, gens):
    """Beyond BASELINE.json's configurations: the seven matmuls of one Llama-8B layer as a Q4_K_M file stores them
    (Q4_K q, k, o, gate, up; Q6_K v, down) handed over as one oxhip_dev_decode_batch call: Q8_0, Q4_K and Q6_K share a kernel,
    so the seven run as one launch. Weights rotate over copies larger than the Infinity Cache."""
    spec = [(Q4_K, 4096, 4096), (Q4_K, 1024, 4096), (Q6_K, 1024, 4096), (Q4_K, 4096, 4096), (Q4_K, 14336, 4096), (Q4_K, 14336, 4096),
            (Q6_K, 4096, 14336)]
    nbytes = sum(algorithmic_bytes(k, n, kk, t) for k, n, kk in spec)
    copies = max(2, int(np.ceil(0.6e9 / nbytes)))
    ws = [[be.upload_gguf(k, gens[k](n, kk, 11 + j), n, kk) for j, (k, n, kk) in enumerate(spec)] for _ in range(copies)]
    xa = {kk: be.quantize_act(torch.from_numpy(synth.activations(t, kk, 3)).cuda()) for kk in (4096, 14336)}
    ys = [torch.empty((t, n), dtype=torch.float32, device="cuda") for _, n, _ in spec]
    arrs = [be.decode_jobs([(ws[c][j], xa[spec[j][2]], None, t, ys[j], None, None) for j in range(len(spec))]) for c in range(copies)]
    wall, ms = timed_steps(torch, lambda i: be.decode_batch(arrs[i % copies]), steps, warmup)
    ach = nbytes / (ms * 1e-3) / 1e9
    return dict(base_line(steps, warmup), value=round(nbytes * steps / wall / 1e9, 2), unit="GB/s", ms_per_step=round(wall / steps * 1e3, 5), dtype="int8",
                config={"workload": f"a Q4_K_M layer's seven matmuls (Q4_K q, k, o, gate, up; Q6_K v, down; Llama-8B shapes) in one batch call, T = {t}",
                        "bytes_per_step": nbytes, "events": "around the call (one launch)"},
                roofline={"bound": "hbm", "achieved": round(ach, 1), "peak": HBM_PEAK_GBS, "unit": "GB/s", "frac": round(ach / HBM_PEAK_GBS, 4),
                          "traffic": profile_traffic("decode_batch_kernel_q4_k_m_layer.md") if t == 1 else None,
                          "kernel": "decode_batch_kernel<Q8_0 | Q4_K | Q6_K>", "bytes_per_launch": nbytes,
                          "avg_launch_us": round(ms * 1e3, 2)})


def moe_experts(synth):
    ne, h, inter = 128, 2048, 768
    return ([synth.mlx_q4(2 * inter, h, 100 + e) for e in range(ne)], [synth.mlx_q4(h, inter, 300 + e) for e in range(ne)])


def bench_moe(be, torch, synth, steps, warmup, pool_gb, t, experts, int8=False):
    """configs[3]: 128 experts, top-8, h = 2048, inter = 768; a step = routing + the MoE pass."""
    from oxinfer_amd import hip
    ne, k, h, inter = 128, 8, 2048, 768
    gu, dn = experts
    expert_bytes = int((2 * inter * h + h * inter) * 0.5625)
    devs = make_pool(lambda: be.upload_moe([be.desc_mlx_q4(*g, 64, 2 * inter, h) for g in gu],
                                           [be.desc_mlx_q4(*d, 64, h, inter) for d in dn], h, inter), ne * expert_bytes, pool_gb)
    if int8:
        for d in devs:
            d.set_mode(hip.MOE_INT8)
    x = torch.from_numpy(synth.activations(t, h, 5, bf16=True)).cuda()
    logits = torch.from_numpy(synth.router_logits(t, ne, 6)).cuda()
    idx, w = be.route_top_k(logits, k)
    touched = len(set(idx.cpu().numpy().reshape(-1).tolist()))
    y = torch.zeros((t, h), dtype=torch.float32, device="cuda")
    nbytes = touched * expert_bytes
    flops = 2 * t * k * (2 * inter * h + h * inter)
    # six or more routed rows per expert: the library takes the bf16 form of the grouped matmuls (the reference's prefill form)
    prefill_form = (t * k) // ne >= 6 and not int8

    sel = torch.empty((2, t, k), dtype=torch.int32, device="cuda")

    def step(i):  # routing (top-k of the logits) and the experts, one library call
        be.moe_routed(devs[i % len(devs)], x, logits, k, y, sel=sel)
    wall, ms = timed_steps(torch, step, steps, warmup)
    ach = nbytes / (ms * 1e-3) / 1e9
    replayed = None
    if t == 1:
        # the same pass recorded once per weight copy (oxhip_plan_*) and replayed: one host call submits its launches
        side = torch.cuda.Stream()
        with torch.cuda.stream(side):
            plans = []
            for d in devs:
                be.moe_routed(d, x, logits, k, y, sel=sel)
                plans.append(be.plan_record(lambda d=d: be.moe_routed(d, x, logits, k, y, sel=sel)))
            pwall, pms = timed_steps(torch, lambda i: plans[i % len(plans)].replay(), steps, warmup)
            side.synchronize()
        replayed = {"what": "the same pass as a recorded plan (oxhip_plan_replay: one submission for its launches)", "launches": int(plans[0].launches),
                    "ms_per_step": round(pwall / steps * 1e3, 5), "value": round(nbytes * steps / pwall / 1e9, 2), "avg_us_by_events": round(pms * 1e3, 2)}
        del plans
    return dict(base_line(steps, warmup), value=round(nbytes * steps / wall / 1e9, 2), unit="GB/s", ms_per_step=round(wall / steps * 1e3, 5),
                dtype="bf16" if prefill_form else "int8", **({"plan_replay": replayed} if replayed else {}),
                config={"workload": f"configs[3]: MoE 128 experts top-8, h 2048, inter 768, MLX 4-bit g64, T = {t}",
                        "experts_touched": touched, "bytes_per_step": nbytes, "flops_per_step": flops,
                        "events": "around routing + the MoE call"},
                roofline={"bound": "hbm", "achieved": round(ach, 1), "peak": HBM_PEAK_GBS, "unit": "GB/s",
                          "frac": round(ach / HBM_PEAK_GBS, 4),
                          "traffic": profile_traffic(f"moe_t{t}.md") if t in (1, 256) and not int8 else None,
                          "kernel": "moe_bf16_kernel<4> (grouped)" if prefill_form else "decode_mfma_kernel<6, *, false, true, true> (grouped)",
                          "bytes_per_launch": nbytes, "avg_launch_us": round(ms * 1e3, 2)},
                tflops=round(flops / (ms * 1e-3) / 1e12, 2))


FP8_PROFILE = {(1, 0): "fp8_m1_skinny_fp8_kernel.md", (32, 0): "fp8_m32_skinny_fp8_kernel.md",
               (1024, 0): "fp8_m1024_gemm_bf16_kernel.md", (1024, 2): "fp8_m1024_gemm_fp8_kernel.md"}


def fp8_weights(synth):
    return synth.fp8_e4m3(7168, 18432, 7)


def bench_fp8(be, torch, synth, steps, warmup, pool_gb, m, variant_name, weights):
    """configs[4]: FP8 E4M3 [7168, 18432] with 128 x 128 block scales, bf16 activations, bf16 out."""
    n, k = 7168, 18432
    data, scales = weights
    ws = make_pool(lambda: be.upload_fp8(data, scales, n, k), n * k, pool_gb)
    x32 = torch.from_numpy(synth.activations(m, k, 8, bf16=True)).cuda()
    xb = x32.to(torch.bfloat16)
    variant = {"bf16": 0, "fp8": 2}.get(variant_name, 0)
    call_ms = None
    if m <= 16:
        step = lambda i: be.decode(ws[i % len(ws)], x=x32)
        kern = "skinny_fp8_kernel<*, 1, 2, *, false> (+ pack_skinny_kernel)"
        wall, ms = timed_steps(torch, step, steps, warmup)
    elif m <= 32 and variant == 0:
        step = lambda i: be.gemm(ws[i % len(ws)], xb, variant=variant, out_bf16=True)
        kern = "skinny_fp8_kernel<4, 2, 1, 16, true> (+ pack_skinny_kernel, gemm_reduce_kernel)"
        wall, ms = timed_steps(torch, step, steps, warmup)
    else:
        kern = "gemm_bf16_kernel<4, true, 2, 8, 7>" if variant == 0 else "gemm_fp8_kernel<true>"
        calls = lambda i: [(ws[i % len(ws)], xb, {"variant": variant, "out_bf16": True})]
        wall, call_ms, ms = timed_gemm_steps(be, torch, calls, steps, warmup)
    flops, nbytes = 2 * m * n * k, n * k + scales.size * 4 + m * k * 2 + m * n * 2
    hbm = m <= 64
    ach = nbytes / (ms * 1e-3) / 1e9 if hbm else flops / (ms * 1e-3) / 1e12
    peak = HBM_PEAK_GBS if hbm else MFMA_PEAK["bf16" if variant == 0 else "fp8"]
    return dict(base_line(steps, warmup), value=round((nbytes / 1e9 if hbm else flops / 1e12) * steps / wall, 2), unit="GB/s" if hbm else "TFLOP/s",
                ms_per_step=round(wall / steps * 1e3, 5), dtype="fp8 weights, " + ("f32" if m <= 16 else ("bf16" if variant == 0 else "fp8")) + " activations",
                config={"workload": f"configs[4]: FP8 E4M3 block-scaled GEMM [7168, 18432], M = {m}, variant {variant_name if m > 16 else 'decode'}",
                        "bytes_per_step": nbytes, "flops_per_step": flops, **({"events": GEMM_EVENTS} if call_ms is not None else {})},
                roofline={"bound": "hbm" if hbm else "mfma", "achieved": round(ach, 1), "peak": peak, "unit": "GB/s" if hbm else "TFLOP/s",
                          "frac": round(ach / peak, 4), "traffic": profile_traffic(FP8_PROFILE.get((m, variant))), "kernel": kern,
                          "avg_launch_us": round(ms * 1e3, 2),
                          **({"call_us": round(call_ms * 1e3, 2)} if call_ms is not None else {})})


def bench_gguf_gemv(args, be, torch, synth, kinds, gens):
    """configs[1] (or its Q6_K counterpart): the headline line, without the CPU leg."""
    from oxinfer_amd.hip import QAct
    cases = gemv_cases(kinds)
    pools = {}
    for c in cases:
        key = (c["kind"], c["n_out"], c["n_in"])
        if key in pools:
            continue
        raw = gens[c["kind"]](c["n_out"], c["n_in"], 1)
        pools[key] = []
        for _ in range(max(2, int(np.ceil(args.pool_gb * 1e9 / raw.size)))):
            w = be.upload_gguf(c["kind"], raw, c["n_out"], c["n_in"])
            if w is None:
                raise RuntimeError(be.last_error())
            pools[key].append(w)
    # the step's inputs: one f32 matrix per (batch, width), shared by the formats like a layer's gate and up share theirs
    inputs = {}
    for c in cases:
        key = (c["t"], c["n_in"])
        if key not in inputs:
            x = torch.from_numpy(synth.activations(c["t"], c["n_in"], 5)).cuda()
            inputs[key] = (x, QAct(c["t"], c["n_in"], x.device))
        c["xa"] = inputs[key][1]
        c["y"] = torch.empty((c["t"], c["n_out"]), dtype=torch.float32, device="cuda")
        c["pool"] = pools[(c["kind"], c["n_out"], c["n_in"])]
    qjobs = be.quantize_jobs(list(inputs.values()))
    be.quantize_act_batch(qjobs)
    torch.cuda.synchronize()

    if args.workload == "gguf_stream":
        # Each case alone, 192 matmuls over rotating weight copies in one call (launches of 16, back to back): what the
        # kernel streams at when no launch boundary, ramp or tail is in the way. `value` is the mean.
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
        return {"metric": METRIC, "value": round(tot_b / tot_s / 1e9, 2), "unit": "GB/s", "n_gpus": 1, "higher_is_better": True,
                "vs_baseline": None, "dtype": "int8", "data": "synthetic",
                "config": {"workload": "GGUF GEMV cases of configs[1] (and Q6_K), each as a steady stream of 192 matmuls in one call"},
                "detail": detail}, cases

    # The dominant kernel: the jobs of one call share one launch (decode_batch_kernel); that launch carries HIP events
    # recorded by the library on the launch stream, on every `--event-every`-th step (default: every fourth; an event pair on every launch keeps consecutive
    # launches a few microseconds apart, which costs the whole-step figure 5 %). An event
    # pair on a launch leaves a gap of a few microseconds before the next one; without it a launch starts in the tail of
    # its predecessor, so its own duration reads longer.
    dom_symbol = "decode_batch_kernel"
    every = max(1, args.event_every)
    # the event figure comes from a pass of its own of at least EV_STEPS steps whatever --steps says (a handful of
    # launches right after the warm-up see clocks that have not settled); `value` and `ms_per_step` are the K timed steps
    EV_STEPS = 400
    ev_steps = max(args.steps, EV_STEPS)
    ev = [(be.event(), be.event()) for _ in range(min((ev_steps + every - 1) // every, 4096))]

    def jobs_for(i, timed_slot=None):
        jobs = []
        for n, c in enumerate(cases):
            w = c["pool"][(2 * i + (c["t"] > 1)) % len(c["pool"])]
            e0 = e1 = None
            if timed_slot is not None:
                pair = ev[timed_slot % len(ev)]
                e0 = pair[0] if n == 0 else None
                e1 = pair[1] if n == len(cases) - 1 else None
            jobs.append((w, c["xa"], None, c["t"], c["y"], e0, e1))
        return be.decode_jobs(jobs)

    def run(with_quantize, steps, events=True):
        n_ev = min((steps + every - 1) // every, len(ev)) if events else 0
        warm = [jobs_for(i) for i in range(args.warmup)]
        timed = [jobs_for(args.warmup + i, i // every if events and i % every == 0 and i // every < n_ev else None) for i in range(steps)]
        for arr in warm:
            if with_quantize:
                be.quantize_act_batch(qjobs)
            be.decode_batch(arr)
        torch.cuda.synchronize()
        t0 = time.perf_counter()
        for arr in timed:
            if with_quantize:
                be.quantize_act_batch(qjobs)
            be.decode_batch(arr)
        torch.cuda.synchronize()
        elapsed = time.perf_counter() - t0
        return elapsed, [be.elapsed_ms(a, b) for a, b in ev[:n_ev]]

    elapsed_k, _ = run(False, args.steps)      # the matmul launches alone (activations quantized beforehand)
    elapsed, dom_ms = run(True, args.steps)    # the whole step: quantize the four inputs, then the eight matmuls
    if ev_steps > args.steps:
        _, dom_ms = run(True, ev_steps)        # the same steps again, longer: the dominant kernel's event figure
    step_bytes = sum(c["bytes"] for c in cases) + sum(x.numel() * 4 for x, _ in inputs.values())
    dom_bytes = float(sum(c["bytes"] for c in cases))
    value = step_bytes * args.steps / elapsed / 1e9
    dom_avg_s = float(np.mean(dom_ms)) / 1e3
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

    q6k = kinds == [Q6_K]
    traffic = profile_traffic("decode_batch_kernel_q6k_gemv.md" if q6k else "decode_batch_kernel_gguf_gemv.md") if kinds in ([Q8_0, Q4_K], [Q6_K]) else None
    out = dict(base_line(args.steps, args.warmup), value=round(value, 2), unit="GB/s", ms_per_step=round(elapsed / args.steps * 1e3, 5), dtype="int8",
               config={"workload": "configs[1]: GGUF GEMV batch 1 and 8, Llama-8B MLP shapes 4096->14336 and 14336->4096, "
                                   + " + ".join(FMT_NAME[k] for k in kinds),
                       "matmuls_per_step": len(cases), "launches_per_step": 2, "bytes_per_step": step_bytes,
                       "weight_pool_GB_per_shape": args.pool_gb,
                       "activations": "f32 in HBM; quantize_act (int8 per 32) of the step's four inputs is one launch inside the timed step",
                       "events": f"on the matmul launch of every {every}. step of a pass of {ev_steps} steps ({len(dom_ms)} timed launches)"},
               roofline={"bound": "hbm", "achieved": round(achieved, 1), "peak": HBM_PEAK_GBS, "unit": "GB/s",
                         "frac": round(achieved / HBM_PEAK_GBS, 4), "traffic": traffic, "kernel": dom_symbol,
                         "bytes_per_launch": dom_bytes, "avg_launch_us": round(dom_avg_s * 1e6, 2)},
               frac_of_hbm_peak=round(value / HBM_PEAK_GBS, 4),
               matmul_launches_only={"what": "the same steps with the activations quantized beforehand (the matmul launches back to back)",
                                     "value": round(dom_bytes * args.steps / elapsed_k / 1e9, 2), "unit": "GB/s",
                                     "ms_per_step": round(elapsed_k / args.steps * 1e3, 5)},
               detail=detail)
    return out, cases


def summary(line, cpu):
    """A configuration's entry of `per_config`."""
    r = line["roofline"]
    e = {"workload": line["config"]["workload"], "value": line["value"], "unit": line["unit"], "ms_per_step": line["ms_per_step"],
         "dtype": line["dtype"], "kernel": r["kernel"], "avg_us": r["avg_launch_us"], "bound": r["bound"],
         "roofline_frac": r["frac"], "achieved": r["achieved"], "peak": r["peak"], "traffic": r["traffic"], "steps": line["steps"]}
    for k in ("ceiling",):
        if k in r:
            e[k] = r[k]
    for k in ("shared_launch_of_4", "steady_stream", "cache_resident", "tflops", "plan_replay"):
        if k in line:
            e[k] = line[k]
    e["cpu_baseline"] = cpu
    if cpu and cpu["unit"] == line["unit"] and cpu["value"]:
        e["gpu_over_cpu"] = round(r["achieved"] / cpu["value"], 1)
    return e


def main():
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=200)
    ap.add_argument("--warmup", type=int, default=20)
    ap.add_argument("--workload", default="all", choices=["all", "gguf_gemv", "gguf_gemv_q6k", "gguf_stream", "gguf_gemm", "gguf_layer", "mlx_gemv", "mlx_gemm", "moe", "fp8", "copy"],
                    help="all (default) = the headline configs[1] line with every other configuration in per_config; gguf_gemv = the headline alone; "
                         "copy = a plain 256 MiB device copy, the known-size kernel that scales the HBM traffic counters; "
                         "gguf_stream = every GGUF case alone as a steady stream of 192 matmuls handed over in one call")
    ap.add_argument("--no-cpu", action="store_true", help="skip the CPU baseline legs")
    ap.add_argument("--event-every", type=int, default=4,
                    help="gguf_gemv: the launch of every n-th timed step carries the timing events (with n > 1 the launches run closer "
                         "together, and a timed launch shares the device with its predecessor's tail)")
    ap.add_argument("--pool-gb", type=float, default=POOL_BYTES / 1e9)
    ap.add_argument("--variant", default="bf16", choices=["bf16", "i8", "fp8"], help="GEMM variant of mlx_gemm / fp8")
    ap.add_argument("--format", default="q4_k", choices=["q8_0", "q4_k", "q6_k"], help="weight format of the gguf_gemm workload")
    ap.add_argument("--tokens", type=int, default=0, help="tokens of the moe (1 or 256) and fp8 (1, 32, 1024) workloads")
    ap.add_argument("--moe-int8", action="store_true", help="moe: keep the integer kernels at every size (oxhip_moe_set_mode)")
    ap.add_argument("--config-steps", type=int, default=200, help="all: timed steps of each per_config entry")
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
    cpu = not args.no_cpu
    gens = {Q8_0: synth.gguf_q8_0, Q4_K: synth.gguf_q4_k, Q6_K: synth.gguf_q6_k}
    w = args.workload
    if w == "mlx_gemv":
        line = bench_mlx_gemv(be, torch, synth, args.steps, args.warmup, args.pool_gb)
        if cpu:
            line["cpu_baseline"] = cpu_mlx_gemv()
    elif w == "mlx_gemm":
        line = bench_mlx_gemm(be, torch, synth, args.steps, args.warmup, args.variant)
        if cpu:
            line["cpu_baseline"] = cpu_mlx_gemm()
    elif w == "gguf_gemm":
        line = bench_gguf_gemm(be, torch, synth, args.steps, args.warmup, args.format)
    elif w == "gguf_layer":
        line = bench_gguf_layer(be, torch, synth, args.steps, args.warmup, args.tokens or 1, gens)
    elif w == "moe":
        ex = moe_experts(synth)
        line = bench_moe(be, torch, synth, args.steps, args.warmup, args.pool_gb, args.tokens or 1, ex, args.moe_int8)
        if cpu:
            line["cpu_baseline"] = cpu_moe(args.tokens or 1, ex)
    elif w == "fp8":
        wts = fp8_weights(synth)
        line = bench_fp8(be, torch, synth, args.steps, args.warmup, args.pool_gb, args.tokens or 1024, args.variant, wts)
        if cpu:
            line["cpu_baseline"] = cpu_fp8(args.tokens or 1024, *wts)
    else:
        kinds = [Q6_K] if w == "gguf_gemv_q6k" else [Q8_0, Q4_K, Q6_K] if w == "gguf_stream" else [Q8_0, Q4_K]
        line, cases = bench_gguf_gemv(args, be, torch, synth, kinds, gens)
        if cpu and w != "gguf_stream":
            line["cpu_baseline"] = cpu_gguf_gemv(cases, gens)
        if w == "all":
            # every other configuration, measured in this same run (GPU leg, then its CPU leg)
            ks, kw = args.config_steps, max(3, args.config_steps // 8)
            per = {}
            l = bench_mlx_gemv(be, torch, synth, 4 * ks, 4 * kw, args.pool_gb)
            per["configs[0] MLX GEMV T=1"] = summary(l, cpu_mlx_gemv() if cpu else None)
            cg = cpu_mlx_gemm() if cpu else None
            per["configs[2a] MLX GEMM M=512 bf16 MFMA"] = summary(bench_mlx_gemm(be, torch, synth, ks, kw, "bf16"), cg)
            per["configs[2b] MLX GEMM M=512 int8 MFMA"] = summary(bench_mlx_gemm(be, torch, synth, ks, kw, "i8"), cg)
            ex = moe_experts(synth)
            per["configs[3] MoE T=1"] = summary(bench_moe(be, torch, synth, 2 * ks, 2 * kw, args.pool_gb, 1, ex), cpu_moe(1, ex) if cpu else None)
            per["configs[3] MoE T=256"] = summary(bench_moe(be, torch, synth, ks, kw, args.pool_gb, 256, ex), cpu_moe(256, ex) if cpu else None)
            del ex
            wts = fp8_weights(synth)
            for m in (1, 32, 1024):
                per[f"configs[4] FP8 M={m}"] = summary(bench_fp8(be, torch, synth, ks, kw, args.pool_gb, m, "bf16", wts), cpu_fp8(m, *wts) if cpu else None)
            per["configs[4] FP8 M=1024 fp8 MFMA"] = summary(bench_fp8(be, torch, synth, ks, kw, args.pool_gb, 1024, "fp8", wts), per["configs[4] FP8 M=1024"]["cpu_baseline"])
            for t in (1, 8):
                per[f"beyond configs: Q4_K_M layer (Q4_K + Q6_K jobs in one call) T={t}"] = summary(bench_gguf_layer(be, torch, synth, ks, kw, t, gens), None)
            line["per_config"] = per
    print(json.dumps(line))
    be.close()


if __name__ == "__main__":
    main()
