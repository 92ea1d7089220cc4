// The kernels around the grouped expert matmuls of an MoE layer (moe::Experts::forward and
// forward_batched, src/moe.rs:438-617 and :625-828 of the reference; route_top_k, :180-193):
// routing, the plan that groups (token, expert) pairs by expert, the gated activation with the
// re-quantization of its output, and the weighted combination in route order.
#include "internal.hpp"

namespace oxhip {

// route_top_k: the k largest logits (ties to the lower index, total order on the float bits like
// f32::total_cmp), weights exp(l - max) / sum over the k. One wavefront per token; n <= 1024.
__global__ __launch_bounds__(64) void route_top_k_kernel(const float* __restrict__ logits, uint32_t n, uint32_t k,
                                                         uint32_t* __restrict__ idx, float* __restrict__ wts) {
    const uint32_t tok = blockIdx.x, lane = threadIdx.x;
    const float* l = logits + (size_t)tok * n;
    constexpr int PER = 16;  // logits per lane
    int key[PER];
    bool live[PER];
#pragma unroll
    for (int i = 0; i < PER; i++) {
        const uint32_t j = lane + 64 * i;
        live[i] = j < n;
        const int b = live[i] ? __float_as_int(l[j]) : 0;
        key[i] = b ^ (int)(((uint32_t)(b >> 31)) >> 1);  // f32::total_cmp's order as a signed compare
    }
    float sel[32];
    uint32_t seli[32];
    for (uint32_t r = 0; r < k && r < 32; r++) {
        // this lane's best remaining logit (its indices ascend, so ties keep the lower one)
        int bk = 0;
        uint32_t bj = 0xFFFFFFFFu;
#pragma unroll
        for (int i = 0; i < PER; i++)
            if (live[i] && (bj == 0xFFFFFFFFu || key[i] > bk)) {
                bk = key[i];
                bj = lane + 64 * i;
            }
        for (int off = 32; off >= 1; off >>= 1) {
            const int ok = __shfl_xor(bk, off);
            const uint32_t oj = __shfl_xor(bj, off);
            if (oj != 0xFFFFFFFFu && (bj == 0xFFFFFFFFu || ok > bk || (ok == bk && oj < bj))) {
                bk = ok;
                bj = oj;
            }
        }
        seli[r] = bj;
        sel[r] = l[bj];
#pragma unroll
        for (int i = 0; i < PER; i++)
            if (lane + 64 * i == bj) live[i] = false;
    }
    if (lane == 0) {
        const float m = sel[0];
        float e[32];
        float s = -0.0f;
        for (uint32_t r = 0; r < k; r++) {
            e[r] = expf(sel[r] - m);
            s += e[r];
        }
        for (uint32_t r = 0; r < k; r++) {
            idx[(size_t)tok * k + r] = seli[r];
            wts[(size_t)tok * k + r] = e[r] / s;
        }
    }
}

hipError_t launch_route_top_k(const float* logits, size_t t, size_t n, size_t k, uint32_t* idx, float* w, hipStream_t s) {
    if (!t) return hipSuccess;
    route_top_k_kernel<<<(unsigned)t, 64, 0, s>>>(logits, (uint32_t)n, (uint32_t)k, idx, w);
    return hipGetLastError();
}

// The plan of one pass: pairs (token i, slot j) -> gathered row, grouped by expert in (token, slot)
// order, cut into chunks of at most 8 rows. One workgroup; thread e owns expert e.
//   row_of[i * k + j]  gathered row of the pair
//   src[row]           token of a gathered row
//   chunks[c]          {expert, first row, rows, 0}; *nchunks
__global__ __launch_bounds__(1024) void moe_plan_kernel(const uint32_t* __restrict__ route_idx, uint32_t pairs, uint32_t k,
                                                        uint32_t n_exp, int* __restrict__ row_of, int* __restrict__ src,
                                                        int4* __restrict__ chunks, int* __restrict__ nchunks) {
    extern __shared__ int sh[];
    int* cnt = sh;               // [n_exp]
    int* start = sh + n_exp;     // [n_exp]
    int* cstart = sh + 2 * n_exp;  // [n_exp]
    for (uint32_t e = threadIdx.x; e < n_exp; e += blockDim.x) cnt[e] = 0;
    __syncthreads();
    for (uint32_t i = threadIdx.x; i < pairs; i += blockDim.x) atomicAdd(&cnt[route_idx[i]], 1);
    __syncthreads();
    if (threadIdx.x == 0) {
        int r = 0, c = 0;
        for (uint32_t e = 0; e < n_exp; e++) {
            start[e] = r;
            cstart[e] = c;
            r += cnt[e];
            c += (cnt[e] + 7) / 8;
        }
        *nchunks = c;
    }
    __syncthreads();
    for (uint32_t e = threadIdx.x; e < n_exp; e += blockDim.x) {
        const int n = cnt[e];
        if (!n) continue;
        int pos = start[e];
        for (uint32_t i = 0; i < pairs && pos < start[e] + n; i++) {
            if (route_idx[i] == e) {
                row_of[i] = pos;
                src[pos] = (int)(i / k);
                pos++;
            }
        }
        for (int c = 0; c < (n + 7) / 8; c++) chunks[cstart[e] + c] = make_int4((int)e, start[e] + 8 * c, min(8, n - 8 * c), 0);
    }
}

hipError_t launch_moe_plan(const uint32_t* route_idx, size_t pairs, size_t k, size_t n_exp, int* row_of, int* src, int4* chunks,
                           int* nchunks, hipStream_t s) {
    unsigned threads = (unsigned)(n_exp < 64 ? 64 : (n_exp > 1024 ? 1024 : (n_exp + 63) / 64 * 64));
    moe_plan_kernel<<<1, threads, 3 * n_exp * sizeof(int), s>>>(route_idx, (uint32_t)pairs, (uint32_t)k, (uint32_t)n_exp, row_of, src,
                                                               chunks, nchunks);
    return hipGetLastError();
}

// fast_exp of the reference (src/kernels.rs:2225-2231): clamp, Cody-Waite reduction, degree-6 polynomial,
// scale by 2^fx through the exponent bits; every operation unfused as written there.
__device__ __forceinline__ float fast_exp(float x) {
    x = fminf(fmaxf(x, -87.0f), 88.0f);
    const float fx = roundf(x * 1.44269504088896340736f);
    const float r = (x - fx * 0.693359375f) - fx * -2.12194440e-4f;
    const float p = 1.0f + r * (1.0f + r * (0.5f + r * (0.16666667f + r * (0.041666668f + r * (0.008333334f + r * 0.0013888889f)))));
    return __int_as_float(((int)fx + 127) << 23) * p;
}

// Act::apply on gathered rows: a = act(g) * u as f32 [rows][inter], with g and u rows `stride` apart (fused
// gate/up outputs: g = gu, u = gu + inter, stride 2 * inter). kind: 0 SiLU, 1 GELU-tanh, 2 SiLU with clamp
// `param` (src/moe.rs:18-37, silu_mul / gelu_mul).
__global__ __launch_bounds__(256) void moe_act_kernel(const float* __restrict__ gp, const float* __restrict__ up, size_t stride,
                                                      size_t rows, uint32_t inter, uint32_t kind, float param, float* __restrict__ a) {
    size_t i = (size_t)blockIdx.x * blockDim.x + threadIdx.x;
    if (i >= rows * inter) return;
    size_t r = i / inter, j = i % inter;
    float g = gp[r * stride + j], u = up[r * stride + j];
    float v;
    if (kind == 1) {
        const float K2 = 2.0f * 0.7978846f;
        const float uu = K2 * (g + 0.044715f * g * g * g);
        v = g / (1.0f + fast_exp(-uu)) * u;
    } else {
        if (kind == 2) {
            g = fminf(g, param);
            u = fminf(fmaxf(u, -param), param);
        }
        v = g / (1.0f + fast_exp(-g)) * u;
    }
    a[i] = v;
}

hipError_t launch_moe_act(const float* g, const float* u, size_t stride, size_t rows, size_t inter, uint32_t kind, float param,
                          float* a, hipStream_t s) {
    size_t total = rows * inter;
    if (!total) return hipSuccess;
    moe_act_kernel<<<(unsigned)((total + 255) / 256), 256, 0, s>>>(g, u, stride, rows, (uint32_t)inter, kind, param, a);
    return hipGetLastError();
}

// y[i] += w_j * o[row_of(i, j)] for j in route order: axpy per expert, multiply then add (src/moe.rs:608-615).
__global__ __launch_bounds__(256) void moe_combine_kernel(const float* __restrict__ o, const int* __restrict__ row_of,
                                                          const float* __restrict__ route_w, uint32_t t, uint32_t k, uint32_t h,
                                                          float* __restrict__ y) {
    size_t i = (size_t)blockIdx.x * blockDim.x + threadIdx.x;
    if (i >= (size_t)t * h) return;
    uint32_t tok = i / h, c = i % h;
    float acc = y[i];
    for (uint32_t j = 0; j < k; j++) {
        const float w = route_w[(size_t)tok * k + j];
        acc = acc + w * o[(size_t)row_of[(size_t)tok * k + j] * h + c];
    }
    y[i] = acc;
}

hipError_t launch_moe_combine(const float* o, const int* row_of, const float* route_w, size_t t, size_t k, size_t h, float* y,
                              hipStream_t s) {
    size_t total = t * h;
    if (!total) return hipSuccess;
    moe_combine_kernel<<<(unsigned)((total + 255) / 256), 256, 0, s>>>(o, row_of, route_w, (uint32_t)t, (uint32_t)k, (uint32_t)h, y);
    return hipGetLastError();
}

}  // namespace oxhip
