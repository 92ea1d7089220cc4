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

// RMSNorm of one row per workgroup (Op::Norm, src/gpu_decode.rs:53-66), then quantize_act of the row that was written,
// without a round trip through memory:
//   x' = x * pre;  r = (sum x'^2 / n + eps)^(-1/2);  v = (x' * r) * w  (or x' * r);  out = v, or out += v with `add`;
//   what `out` then holds goes, per block of 32, to the QAct (optional).
// The reference sums the squares one after the other in f32 (src/kernels.rs:2109), which no parallel machine can
// repeat bit for bit in useful time: here the squares are exact in f64 and summed in f64 (a fixed order), the mean and
// eps added in f32 as the reference does, and r is the correctly rounded power. The quantization of v is quantize_act's,
// bit for bit (the same code on the same values). VEC: rows of x, out and w start on 16-byte boundaries (float4 access);
// otherwise every access is one float.
template <bool VEC>
__global__ __launch_bounds__(256) void rmsnorm_quantize_kernel(const float* __restrict__ x, const float* __restrict__ w_f32,
                                                               const uint16_t* __restrict__ w_bf16, float eps, float pre, uint32_t add,
                                                               uint32_t n, size_t x_stride, size_t out_stride,
                                                               float* __restrict__ out, int8_t* __restrict__ q, float* __restrict__ scales,
                                                               int32_t* __restrict__ sums, float* __restrict__ fsums,
                                                               float* __restrict__ hsums, int32_t* __restrict__ sums16) {
    __shared__ double part[4];
    __shared__ float r_s;
    const uint32_t tok = blockIdx.x, lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
    const float* xr = x + (size_t)tok * x_stride;
    auto load4 = [&](const float* p, float* v) {
        if constexpr (VEC) {
            const float4 f = *reinterpret_cast<const float4*>(p);
            v[0] = f.x; v[1] = f.y; v[2] = f.z; v[3] = f.w;
        } else {
            v[0] = p[0]; v[1] = p[1]; v[2] = p[2]; v[3] = p[3];
        }
    };
    double ss = 0.0;
    for (uint32_t i = 4 * threadIdx.x; i < n; i += 1024) {  // n is a multiple of 32
        float v[4];
        load4(xr + i, v);
#pragma unroll
        for (int j = 0; j < 4; j++) {
            const float p = v[j] * pre;
            ss += (double)p * p;
        }
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
            float f[4];
            load4(xr + 32 * b + 4 * i, f);
#pragma unroll
            for (int j = 0; j < 4; j++) v[4 * i + j] = (f[j] * pre) * r;
        }
        if (w_f32) {
#pragma unroll
            for (int i = 0; i < 32; i++) v[i] = v[i] * w_f32[32 * b + i];
        } else if (w_bf16) {
#pragma unroll
            for (int i = 0; i < 32; i++) v[i] = v[i] * bf16_bits_to_f32(w_bf16[32 * b + i]);
        }
        const size_t gb = (size_t)tok * nblocks + b;
        float* orow = out ? out + (size_t)tok * out_stride + 32 * b : nullptr;
        if (out && add) {
#pragma unroll
            for (int i = 0; i < 8; i++) {
                float f[4];
                load4(orow + 4 * i, f);
#pragma unroll
                for (int j = 0; j < 4; j++) v[4 * i + j] = f[j] + v[4 * i + j];
            }
        }
        if (out) {
#pragma unroll
            for (int i = 0; i < 8; i++) {
                if constexpr (VEC) {
                    *reinterpret_cast<float4*>(orow + 4 * i) = make_float4(v[4 * i], v[4 * i + 1], v[4 * i + 2], v[4 * i + 3]);
                } else {
#pragma unroll
                    for (int j = 0; j < 4; j++) orow[4 * i + j] = v[4 * i + j];
                }
            }
        }
        if (q) quantize_act_values(v, gb, q, scales, sums, fsums, hsums, sums16);
    }
}

hipError_t launch_rmsnorm_quantize(const float* x, const float* w_f32, const uint16_t* w_bf16, float eps, size_t t, size_t n, float* out,
                                   const oxhip_qact* qa, hipStream_t s, float pre, bool add, size_t x_stride, size_t out_stride) {
    if (!t || !n) return hipSuccess;
    if (n % 32) return hipErrorInvalidValue;
    if (!x_stride) x_stride = n;
    if (!out_stride) out_stride = n;
    auto al = [](const void* p) { return reinterpret_cast<uintptr_t>(p) % 16 == 0; };
    const bool vec = al(x) && al(out) && al(w_f32) && x_stride % 4 == 0 && out_stride % 4 == 0;
    auto go = [&](auto kern) {
        kern<<<(unsigned)t, 256, 0, s>>>(x, w_f32, w_bf16, eps, pre, add ? 1u : 0u, (uint32_t)n, x_stride, out_stride, out, qa ? qa->q : nullptr,
                                        qa ? qa->scales : nullptr, qa ? qa->sums : nullptr, qa ? qa->fsums : nullptr, qa ? qa->hsums : nullptr,
                                        qa ? qa->sums16 : nullptr);
    };
    if (vec) go(rmsnorm_quantize_kernel<true>);
    else go(rmsnorm_quantize_kernel<false>);
    return hipGetLastError();
}

}  // namespace oxhip
