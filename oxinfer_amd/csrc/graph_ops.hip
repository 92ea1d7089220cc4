// Kernels of the single-token decode graph around the matmuls (the reference's Op list, src/gpu_decode.rs:52-340):
// the output modes of a linear for the formats whose decode kernels only store, the gate / up pair as an elementwise
// op (Op::Glu), the router's logits (Op::Route before its top-k), and RMSNorm fused with the activation quantization
// that the next matmul reads (Op::Norm feeding Op::Linear; rmsnorm, src/kernels.rs:2107-2123, then quantize_act,
// src/quant.rs:243-343).
#include "act_body.hpp"
#include "internal.hpp"

namespace oxhip {

__global__ __launch_bounds__(256) void epilogue_kernel(const float* __restrict__ v, uint32_t n, size_t total, float* __restrict__ y, Epi epi) {
    const size_t i = (size_t)blockIdx.x * blockDim.x + threadIdx.x;
    if (i >= total) return;
    const float x = v[i];
    if (epi.mode == EPI_STORE) y[i] = x;
    else if (epi.mode == EPI_ADD) y[i] = y[i] + x;
    else y[i] = y[i] + (1.0f / (1.0f + expf(-epi.gate[i / n]))) * x;
}

hipError_t launch_epilogue(const float* v, size_t t, size_t n, float* y, const Epi& epi, hipStream_t s) {
    const size_t total = t * n;
    if (!total) return hipSuccess;
    epilogue_kernel<<<(unsigned)((total + 255) / 256), 256, 0, s>>>(v, (uint32_t)n, total, y, epi);
    return hipGetLastError();
}

// y = silu(g) * u or gelu_tanh(g) * u (silu_mul / gelu_mul, src/kernels.rs:2188-2198, :2234-2257: both through fast_exp).
__global__ __launch_bounds__(256) void glu_kernel(const float* __restrict__ g, const float* __restrict__ u, size_t n, uint32_t kind,
                                                  float* __restrict__ y) {
    const size_t i = (size_t)blockIdx.x * blockDim.x + threadIdx.x;
    if (i < n) y[i] = gated_act(g[i], u[i], kind, 0.0f);
}

hipError_t launch_glu(const float* g, const float* u, size_t n, bool gelu, float* y, hipStream_t s) {
    if (!n) return hipSuccess;
    glu_kernel<<<(unsigned)((n + 255) / 256), 256, 0, s>>>(g, u, n, gelu ? 1u : 0u, y);
    return hipGetLastError();
}

// logits[tok][e] = router[e] . x[tok] for e < n_exp, and with `gate` one more logit gate . x[tok] behind them
// (Op::Route, src/gpu_decode.rs:154-172). One wavefront per logit: f32 rows read as whole lines, f32 accumulation.
__global__ __launch_bounds__(512) void router_logits_kernel(const float* __restrict__ x, const float* __restrict__ router,
                                                            const float* __restrict__ gate, uint32_t n_exp, uint32_t h,
                                                            float* __restrict__ logits) {
    const uint32_t lane = threadIdx.x & 63, row = blockIdx.x * 8 + (threadIdx.x >> 6), tok = blockIdx.y;
    const uint32_t rows = n_exp + (gate ? 1u : 0u);
    if (row >= rows) return;
    const float* w = row < n_exp ? router + (size_t)row * h : gate;
    const float* xr = x + (size_t)tok * h;
    float acc = 0.0f;
    if (h % 4 == 0) {
        for (uint32_t i = 4 * lane; i < h; i += 256) {
            const float4 a = *reinterpret_cast<const float4*>(w + i), b = *reinterpret_cast<const float4*>(xr + i);
            acc = fmaf(a.x, b.x, acc);
            acc = fmaf(a.y, b.y, acc);
            acc = fmaf(a.z, b.z, acc);
            acc = fmaf(a.w, b.w, acc);
        }
    } else {
        for (uint32_t i = lane; i < h; i += 64) acc = fmaf(w[i], xr[i], acc);
    }
    acc = wave_sum(acc);
    if (lane == 0) logits[(size_t)tok * rows + row] = acc;
}

hipError_t launch_router_logits(const float* x, const float* router, const float* gate, size_t t, size_t n_exp, size_t h, float* logits,
                                hipStream_t s) {
    const size_t rows = n_exp + (gate ? 1 : 0);
    if (!t || !rows) return hipSuccess;
    router_logits_kernel<<<dim3((unsigned)((rows + 7) / 8), (unsigned)t), 512, 0, s>>>(x, router, gate, (uint32_t)n_exp, (uint32_t)h, logits);
    return hipGetLastError();
}

// RMSNorm of one row per workgroup, then quantize_act of the normed row without a round trip through memory:
//   r = (sum x^2 / n + eps)^(-1/2);  v = (x * r) * w  (or x * r);  v -> `out` (optional) and, per block of 32, the QAct.
// The reference sums the squares one after the other in f32 (src/kernels.rs:2109), which no parallel machine can
// repeat bit for bit in useful time: here the squares are exact in f64 and summed in f64 (a fixed order), the mean and
// eps added in f32 as the reference does, and r is the correctly rounded power. The quantization of v is quantize_act's,
// bit for bit (the same code on the same values).
__global__ __launch_bounds__(256) void rmsnorm_quantize_kernel(const float* __restrict__ x, const float* __restrict__ w_f32,
                                                               const uint16_t* __restrict__ w_bf16, float eps, uint32_t n,
                                                               float* __restrict__ out, int8_t* __restrict__ q, float* __restrict__ scales,
                                                               int32_t* __restrict__ sums, float* __restrict__ fsums,
                                                               float* __restrict__ hsums, int32_t* __restrict__ sums16) {
    __shared__ double part[4];
    __shared__ float r_s;
    const uint32_t tok = blockIdx.x, lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
    const float* xr = x + (size_t)tok * n;
    double ss = 0.0;
    for (uint32_t i = 4 * threadIdx.x; i < n; i += 1024) {  // n is a multiple of 32
        const float4 v = *reinterpret_cast<const float4*>(xr + i);
        ss += (double)v.x * v.x;
        ss += (double)v.y * v.y;
        ss += (double)v.z * v.z;
        ss += (double)v.w * v.w;
    }
    for (int off = 32; off >= 1; off >>= 1) ss += __shfl_xor(ss, off);
    if (lane == 0) part[wave] = ss;
    __syncthreads();
    if (threadIdx.x == 0) {
        const double total = ((part[0] + part[1]) + part[2]) + part[3];
        const float m = (float)total / (float)n + eps;
        r_s = (float)(1.0 / sqrt((double)m));
    }
    __syncthreads();
    const float r = r_s;
    const uint32_t nblocks = n / 32;
    for (uint32_t b = threadIdx.x; b < nblocks; b += 256) {
        float v[32];
#pragma unroll
        for (int i = 0; i < 8; i++) {
            const float4 f = *reinterpret_cast<const float4*>(xr + 32 * b + 4 * i);
            v[4 * i] = f.x * r;
            v[4 * i + 1] = f.y * r;
            v[4 * i + 2] = f.z * r;
            v[4 * i + 3] = f.w * r;
        }
        if (w_f32) {
#pragma unroll
            for (int i = 0; i < 32; i++) v[i] = v[i] * w_f32[32 * b + i];
        } else if (w_bf16) {
#pragma unroll
            for (int i = 0; i < 32; i++) v[i] = v[i] * bf16_bits_to_f32(w_bf16[32 * b + i]);
        }
        const size_t gb = (size_t)tok * nblocks + b;
        if (out) {
#pragma unroll
            for (int i = 0; i < 8; i++)
                *reinterpret_cast<float4*>(out + gb * 32 + 4 * i) = make_float4(v[4 * i], v[4 * i + 1], v[4 * i + 2], v[4 * i + 3]);
        }
        if (q) quantize_act_values(v, gb, q, scales, sums, fsums, hsums, sums16);
    }
}

hipError_t launch_rmsnorm_quantize(const float* x, const float* w_f32, const uint16_t* w_bf16, float eps, size_t t, size_t n, float* out,
                                   const oxhip_qact* qa, hipStream_t s) {
    if (!t || !n) return hipSuccess;
    if (n % 32) return hipErrorInvalidValue;
    rmsnorm_quantize_kernel<<<(unsigned)t, 256, 0, s>>>(x, w_f32, w_bf16, eps, (uint32_t)n, out, qa ? qa->q : nullptr, qa ? qa->scales : nullptr,
                                                       qa ? qa->sums : nullptr, qa ? qa->fsums : nullptr, qa ? qa->hsums : nullptr,
                                                       qa ? qa->sums16 : nullptr);
    return hipGetLastError();
}

}  // namespace oxhip
