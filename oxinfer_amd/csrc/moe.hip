// The kernels around the grouped expert matmuls of an MoE layer (moe::Experts::forward and
// forward_batched, src/moe.rs:438-617 and :625-828 of the reference; route_top_k, :180-193):
// routing, the plan that groups (token, expert) pairs by expert, the gated activation with the
// re-quantization of its output, and the weighted combination in route order.
#include "act_body.hpp"
#include "internal.hpp"

namespace oxhip {

// route_top_k: the k largest logits (ties to the lower index, total order on the float bits like
// f32::total_cmp), weights exp(l - max) / sum over the k. One wavefront per token; n <= 1024, k <= 64.
//
// PER: logits per lane (n <= 64 PER). Up to 256 experts an element's place in the sorted order is counted directly
// (how many elements beat it: every element is broadcast from its lane in turn, n * PER compares per lane, no
// dependent lane-to-lane round trips); beyond that k rounds of a wave-wide argmax cost less.
__device__ __forceinline__ int order_key(float v) {
    const int b = __float_as_int(v);
    return b ^ (int)(((uint32_t)(b >> 31)) >> 1);  // f32::total_cmp's order as a signed compare; its own inverse
}

// NW waves per token. A lone wave issues an instruction every five to eight cycles, so the counting loop is split
// over the waves (each broadcasts 64 / NW lanes of every register) and the counts meet in LDS; wave 0 finishes.
template <int PER, int NW>
__device__ __forceinline__ void route_top_k_body(const float* __restrict__ logits, uint32_t stride, uint32_t n, uint32_t k,
                                                 uint32_t* __restrict__ idx, float* __restrict__ wts,
                                                 const float* __restrict__ expert_scale, uint32_t tok) {
    const uint32_t lane = threadIdx.x & 63, wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
    const float* l = logits + (size_t)tok * stride;
    int key[PER];
    bool live[PER];
#pragma unroll
    for (int i = 0; i < PER; i++) {
        const uint32_t j = lane + 64 * i;
        live[i] = j < n;
        key[i] = order_key(live[i] ? l[j] : 0.0f);
    }
    // round r's winner ends up in lane r
    float mysel = 0.0f;
    uint32_t myidx = 0;
    if constexpr (PER <= 4) {
        __shared__ uint32_t rank_s[PER * 64];
        __shared__ int sel_key[64];
        __shared__ uint32_t sel_idx[64];
        if (NW > 1) {
            for (uint32_t i = threadIdx.x; i < PER * 64; i += 64 * NW) rank_s[i] = 0;
            __syncthreads();
        }
        uint32_t rank[PER];
#pragma unroll
        for (int i = 0; i < PER; i++) rank[i] = 0;
        // element j = src + 64 i2 beats element (lane, i) when its key is larger, or equal with a lower index
        constexpr uint32_t SPAN = 64 / NW;
#pragma unroll
        for (int i2 = 0; i2 < PER; i2++) {
            const uint32_t cnt = min(64u, n > 64u * i2 ? n - 64u * i2 : 0u);  // live lanes of register i2 (uniform)
            const uint32_t s1 = min(cnt, (wave + 1) * SPAN);
            for (uint32_t src = wave * SPAN; src < s1; src++) {
                const int ok = __builtin_amdgcn_readlane(key[i2], (int)src);
#pragma unroll
                for (int i = 0; i < PER; i++) {
                    const bool lower = i2 < i || (i2 == i && src < lane);
                    rank[i] += (ok > key[i] || (ok == key[i] && lower)) ? 1u : 0u;
                }
            }
        }
        if (NW > 1) {
#pragma unroll
            for (int i = 0; i < PER; i++)
                if (rank[i]) atomicAdd(&rank_s[64 * i + lane], rank[i]);
            __syncthreads();
            if (wave) return;
#pragma unroll
            for (int i = 0; i < PER; i++) rank[i] = rank_s[64 * i + lane];
        }
#pragma unroll
        for (int i = 0; i < PER; i++)
            if (live[i] && rank[i] < k && rank[i] < 64) {
                sel_key[rank[i]] = key[i];
                sel_idx[rank[i]] = lane + 64 * i;
            }
        __builtin_amdgcn_s_waitcnt(0xc07f);  // lgkmcnt(0): wave 0's LDS writes before its reads below
        __builtin_amdgcn_wave_barrier();
        if (lane < k && lane < n) {
            mysel = __int_as_float(order_key(__int_as_float(sel_key[lane])));
            myidx = sel_idx[lane];
        }
    } else {
        for (uint32_t r = 0; r < k && r < 64; r++) {
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
            if (lane == r) {
                myidx = bj;
                mysel = __int_as_float(order_key(__int_as_float(bk)));
            }
#pragma unroll
            for (int i = 0; i < PER; i++)
                if (lane + 64 * i == bj) live[i] = false;
        }
    }
    // weights: exp(l - max) over the k, summed in rank order from -0.0 as the reference does
    const float m = __int_as_float(__builtin_amdgcn_readfirstlane(__float_as_int(mysel)));
    const float e = lane < k ? expf(mysel - m) : 0.0f;
    float sum = -0.0f;
    for (uint32_t r = 0; r < k && r < 64; r++) sum += __int_as_float(__builtin_amdgcn_readlane(__float_as_int(e), (int)r));
    if (lane < k) {
        idx[(size_t)tok * k + lane] = myidx;
        // (per-expert factors multiply the weights after the softmax, src/gpu_decode.rs:167-168)
        wts[(size_t)tok * k + lane] = expert_scale ? e / sum * expert_scale[myidx] : e / sum;
    }
}

template <int PER, int NW>
__global__ __launch_bounds__(64 * NW) void route_top_k_kernel(const float* __restrict__ logits, uint32_t stride, uint32_t n, uint32_t k,
                                                              uint32_t* __restrict__ idx, float* __restrict__ wts,
                                                              const float* __restrict__ expert_scale) {
    route_top_k_body<PER, NW>(logits, stride, n, k, idx, wts, expert_scale, blockIdx.x);
}

// Workgroups 0 .. t - 1 route a token each; the others quantize one block of 32 of x per lane.
template <int PER>
__global__ __launch_bounds__(512) void route_quantize_kernel(const float* __restrict__ logits, uint32_t stride, uint32_t n, uint32_t k,
                                                             uint32_t* __restrict__ idx, float* __restrict__ wts,
                                                             const float* __restrict__ expert_scale, uint32_t t, const float* __restrict__ x,
                                                             size_t nblocks, int8_t* __restrict__ q, float* __restrict__ scales,
                                                             int32_t* __restrict__ sums, float* __restrict__ fsums, float* __restrict__ hsums,
                                                             int32_t* __restrict__ sums16) {
    if (blockIdx.x < t) {
        route_top_k_body<PER, 8>(logits, stride, n, k, idx, wts, expert_scale, blockIdx.x);
        return;
    }
    const size_t b = (size_t)(blockIdx.x - t) * blockDim.x + threadIdx.x;
    if (b < nblocks) quantize_act_block(x, b, q, scales, sums, fsums, hsums, sums16);
}

hipError_t launch_route_quantize(const float* logits, size_t t, size_t n, size_t k, uint32_t* idx, float* w, size_t stride,
                                 const float* expert_scale, const float* x, size_t h, const oxhip_qact& o, hipStream_t s) {
    if (!t) return hipSuccess;
    if (n > 256) return hipErrorInvalidValue;
    const uint32_t st = (uint32_t)(stride ? stride : n);
    const size_t nblocks = t * h / 32;
    const unsigned grid = (unsigned)(t + (nblocks + 511) / 512);
    if (n <= 128)
        route_quantize_kernel<2><<<grid, 512, 0, s>>>(logits, st, (uint32_t)n, (uint32_t)k, idx, w, expert_scale, (uint32_t)t, x, nblocks, o.q, o.scales,
                                                     o.sums, o.fsums, o.hsums, o.sums16);
    else
        route_quantize_kernel<4><<<grid, 512, 0, s>>>(logits, st, (uint32_t)n, (uint32_t)k, idx, w, expert_scale, (uint32_t)t, x, nblocks, o.q, o.scales,
                                                     o.sums, o.fsums, o.hsums, o.sums16);
    return hipGetLastError();
}

// `stride`: floats between the logit rows of consecutive tokens (>= n; the decode graph keeps one more logit behind them).
hipError_t launch_route_top_k(const float* logits, size_t t, size_t n, size_t k, uint32_t* idx, float* w, hipStream_t s, size_t stride,
                              const float* expert_scale) {
    if (!t) return hipSuccess;
    const uint32_t st = (uint32_t)(stride ? stride : n);
    if (n <= 128) route_top_k_kernel<2, 8><<<(unsigned)t, 512, 0, s>>>(logits, st, (uint32_t)n, (uint32_t)k, idx, w, expert_scale);
    else if (n <= 256) route_top_k_kernel<4, 8><<<(unsigned)t, 512, 0, s>>>(logits, st, (uint32_t)n, (uint32_t)k, idx, w, expert_scale);
    else route_top_k_kernel<16, 1><<<(unsigned)t, 64, 0, s>>>(logits, st, (uint32_t)n, (uint32_t)k, idx, w, expert_scale);
    return hipGetLastError();
}

// The plan of one pass: pairs (token i, slot j) -> gathered row, grouped by expert in (token, slot)
// order, cut into chunks of at most `cr` rows (8, 16 or 32). One workgroup: counts per expert, prefix sums, then each
// pair takes the next free row of its expert (LDS counters; the route list is staged in LDS when it fits).
//   row_of[i * k + j]  gathered row of the pair
//   src[row]           token of a gathered row
//   chunks[c]          {expert, first row, rows, 0}; *nchunks
constexpr uint32_t PLAN_LDS_PAIRS = 24 * 1024;  // route entries kept in LDS (96 KiB); longer lists are read from L2
__device__ __forceinline__ void moe_plan_body(int* sh, const uint32_t* __restrict__ route_idx, uint32_t pairs, uint32_t k, uint32_t n_exp, int cr,
                                              int* __restrict__ row_of, int* __restrict__ src, int4* __restrict__ chunks,
                                              int* __restrict__ nchunks) {
    int* cnt = sh;                 // [n_exp]
    int* start = sh + n_exp;       // [n_exp]
    int* cstart = sh + 2 * n_exp;  // [n_exp]
    int* fill = sh + 3 * n_exp;    // [n_exp]
    uint32_t* routes = reinterpret_cast<uint32_t*>(sh + 4 * n_exp);
    const bool staged = pairs <= PLAN_LDS_PAIRS;
    const uint32_t lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
    for (uint32_t e = threadIdx.x; e < n_exp; e += blockDim.x) cnt[e] = fill[e] = 0;
    __syncthreads();
    for (uint32_t i = threadIdx.x; i < pairs; i += blockDim.x) {
        const uint32_t e = route_idx[i];
        if (staged) routes[i] = e;
        atomicAdd(&cnt[e], 1);
    }
    __syncthreads();
    if (wave == 0) {  // exclusive prefix sums over the experts: each lane owns a run of experts, the runs meet by a wave scan
        const uint32_t per = (n_exp + 63) / 64, e0 = lane * per, e1 = min(n_exp, e0 + per);
        int r = 0, c = 0;
        for (uint32_t e = e0; e < e1; e++) {
            r += cnt[e];
            c += (cnt[e] + cr - 1) / cr;
        }
        int rs = r, cs = c;  // inclusive scan over lanes
        for (int d = 1; d < 64; d <<= 1) {
            const int ro = __shfl_up(rs, d), co = __shfl_up(cs, d);
            if ((int)lane >= d) {
                rs += ro;
                cs += co;
            }
        }
        int rb = rs - r, cb = cs - c;
        for (uint32_t e = e0; e < e1; e++) {
            start[e] = rb;
            cstart[e] = cb;
            rb += cnt[e];
            cb += (cnt[e] + cr - 1) / cr;
        }
        if (lane == 63) *nchunks = cs;
    }
    __syncthreads();
    // a pair's place inside its expert's run is the order of arrival: which rows share a chunk varies from run to run,
    // but a row's result does not depend on its chunk (every (token, row) sum is formed on its own, in a fixed order)
    for (uint32_t i = threadIdx.x; i < pairs; i += blockDim.x) {
        const uint32_t e = staged ? routes[i] : route_idx[i];
        const int r = start[e] + atomicAdd(&fill[e], 1);
        row_of[i] = r;
        src[r] = (int)(i / k);
    }
    for (uint32_t e = threadIdx.x; e < n_exp; e += blockDim.x) {
        const int n = cnt[e];
        for (int c = 0; c < (n + cr - 1) / cr; c++) chunks[cstart[e] + c] = make_int4((int)e, start[e] + cr * c, min(cr, n - cr * c), 0);
    }
}

__global__ __launch_bounds__(1024) void moe_plan_kernel(const uint32_t* __restrict__ route_idx, uint32_t pairs, uint32_t k,
                                                        uint32_t n_exp, int cr, int* __restrict__ row_of, int* __restrict__ src,
                                                        int4* __restrict__ chunks, int* __restrict__ nchunks) {
    extern __shared__ int sh[];
    moe_plan_body(sh, route_idx, pairs, k, n_exp, cr, row_of, src, chunks, nchunks);
}

// The plan and the quantization of the layer's input depend only on the layer's arguments, and each is a few
// microseconds of latency: one launch runs both (workgroup 0 plans, the others quantize one block of 32 per lane).
__global__ __launch_bounds__(1024) void moe_front_kernel(const uint32_t* __restrict__ route_idx, uint32_t pairs, uint32_t k, uint32_t n_exp,
                                                         int cr, int* __restrict__ row_of, int* __restrict__ src, int4* __restrict__ chunks,
                                                         int* __restrict__ nchunks, const float* __restrict__ x, size_t nblocks,
                                                         int8_t* __restrict__ q, float* __restrict__ scales, int32_t* __restrict__ sums,
                                                         float* __restrict__ fsums, float* __restrict__ hsums, int32_t* __restrict__ sums16) {
    extern __shared__ int sh[];
    if (blockIdx.x == 0) {
        moe_plan_body(sh, route_idx, pairs, k, n_exp, cr, row_of, src, chunks, nchunks);
        return;
    }
    const size_t b = (size_t)(blockIdx.x - 1) * blockDim.x + threadIdx.x;
    if (b < nblocks) quantize_act_block(x, b, q, scales, sums, fsums, hsums, sums16);
}

hipError_t launch_moe_plan(const uint32_t* route_idx, size_t pairs, size_t k, size_t n_exp, uint32_t chunk_rows, int* row_of, int* src,
                           int4* chunks, int* nchunks, hipStream_t s) {
    const size_t lds = 4 * n_exp * sizeof(int) + (pairs <= PLAN_LDS_PAIRS ? pairs * sizeof(uint32_t) : 0);
    if (lds > 48 * 1024) {  // once per pass: not worth caching per device
        hipError_t e = hipFuncSetAttribute(reinterpret_cast<const void*>(moe_plan_kernel), hipFuncAttributeMaxDynamicSharedMemorySize, 128 * 1024);
        if (e != hipSuccess) return e;
    }
    moe_plan_kernel<<<1, 1024, lds, s>>>(route_idx, (uint32_t)pairs, (uint32_t)k, (uint32_t)n_exp, (int)chunk_rows, row_of, src, chunks, nchunks);
    return hipGetLastError();
}

// Plan + quantize_act(x [t][h]) in one launch when the plan's LDS is small (it is allocated to every workgroup);
// else two launches.
hipError_t launch_moe_front(const uint32_t* route_idx, size_t pairs, size_t k, size_t n_exp, uint32_t chunk_rows, int* row_of, int* src,
                            int4* chunks, int* nchunks, const float* x, size_t t, size_t h, const oxhip_qact& o, hipStream_t s) {
    const size_t lds = 4 * n_exp * sizeof(int) + pairs * sizeof(uint32_t), nblocks = t * h / 32;
    if (pairs > 4096 || lds > 32 * 1024 || !nblocks) {
        hipError_t e = launch_moe_plan(route_idx, pairs, k, n_exp, chunk_rows, row_of, src, chunks, nchunks, s);
        return e != hipSuccess ? e : launch_quantize_act(x, t, h, o, s);
    }
    moe_front_kernel<<<1 + (unsigned)((nblocks + 1023) / 1024), 1024, lds, s>>>(route_idx, (uint32_t)pairs, (uint32_t)k, (uint32_t)n_exp,
                                                                              (int)chunk_rows, row_of, src, chunks, nchunks, x, nblocks, o.q, o.scales,
                                                                              o.sums, o.fsums, o.hsums, o.sums16);
    return hipGetLastError();
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

// The same, followed by quantize_act on the result (src/quant.rs:267-292) without the round trip through memory;
// bit-identical to moe_act_kernel + quantize_act_kernel. A workgroup of 256 threads takes 32 blocks of 32: eight
// neighbouring lanes read one block's gate and up values as whole lines and apply the activation (four values each);
// the values meet in LDS and one lane per block forms the sums in the reference's order and the int8 codes.
__global__ __launch_bounds__(256) void moe_act_quantize_kernel(const float* __restrict__ gp, const float* __restrict__ up, size_t stride,
                                                              size_t rows, uint32_t inter, uint32_t kind, float param,
                                                              int8_t* __restrict__ q, float* __restrict__ scales, int32_t* __restrict__ sums,
                                                              float* __restrict__ fsums, float* __restrict__ hsums,
                                                              int32_t* __restrict__ sums16) {
    __shared__ float vals[32][36];  // rows padded: the finishing lanes read their blocks 36 words apart
    const size_t bpr = inter / 32, nblocks = rows * bpr;
    const size_t b0 = (size_t)blockIdx.x * 32;
    {
        const uint32_t lb = threadIdx.x >> 3, part = threadIdx.x & 7;
        const size_t b = b0 + lb;
        if (b < nblocks) {
            const size_t r = b / bpr, j0 = (b % bpr) * 32 + 4 * part;
            const float4 gg = *reinterpret_cast<const float4*>(gp + r * stride + j0);
            const float4 uu = *reinterpret_cast<const float4*>(up + r * stride + j0);
            const float gs[4] = {gg.x, gg.y, gg.z, gg.w}, us[4] = {uu.x, uu.y, uu.z, uu.w};
#pragma unroll
            for (int e = 0; e < 4; e++) {
                float g = gs[e], u = us[e], v;
                if (kind == 1) {
                    const float K2 = 2.0f * 0.7978846f;
                    const float t = K2 * (g + 0.044715f * g * g * g);
                    v = g / (1.0f + fast_exp(-t)) * u;
                } else {
                    if (kind == 2) {
                        g = fminf(g, param);
                        u = fminf(fmaxf(u, -param), param);
                    }
                    v = g / (1.0f + fast_exp(-g)) * u;
                }
                vals[lb][4 * part + e] = v;
            }
        }
    }
    __syncthreads();
    const size_t b = b0 + threadIdx.x;
    if (threadIdx.x >= 32 || b >= nblocks) return;
    float v[32];
#pragma unroll
    for (int i = 0; i < 8; i++) {
        const float4 f = *reinterpret_cast<const float4*>(&vals[threadIdx.x][4 * i]);
        v[4 * i] = f.x;
        v[4 * i + 1] = f.y;
        v[4 * i + 2] = f.z;
        v[4 * i + 3] = f.w;
    }
    float amax = 0.0f;
#pragma unroll
    for (int i = 0; i < 32; i++) amax = fmaxf(amax, fabsf(v[i]));
    const float inv = amax > 0.0f ? 127.0f / amax : 0.0f;
    float h0 = -0.0f, h1 = -0.0f, f = -0.0f;
#pragma unroll
    for (int i = 0; i < 16; i++) h0 += v[i];
#pragma unroll
    for (int i = 16; i < 32; i++) h1 += v[i];
#pragma unroll
    for (int i = 0; i < 32; i++) f += v[i];
    int s0 = 0, s1 = 0;
    uint32_t packed[8];
#pragma unroll
    for (int i = 0; i < 8; i++) {
        uint32_t wv = 0;
#pragma unroll
        for (int e = 0; e < 4; e++) {
            const float rr = roundf(v[4 * i + e] * inv);
            const int iv = rr != rr ? 0 : (int)fminf(fmaxf(rr, -128.0f), 127.0f);
            if (i < 4) s0 += iv; else s1 += iv;
            wv |= ((uint32_t)iv & 0xFF) << (8 * e);
        }
        packed[i] = wv;
    }
    uint4* dst = reinterpret_cast<uint4*>(q + b * 32);
    dst[0] = make_uint4(packed[0], packed[1], packed[2], packed[3]);
    dst[1] = make_uint4(packed[4], packed[5], packed[6], packed[7]);
    scales[b] = amax / 127.0f;
    sums[b] = s0 + s1;
    fsums[b] = f;
    hsums[2 * b] = h0;
    hsums[2 * b + 1] = h1;
    sums16[2 * b] = s0;
    sums16[2 * b + 1] = s1;
}

hipError_t launch_moe_act_quantize(const float* g, const float* u, size_t stride, size_t rows, size_t inter, uint32_t kind, float param,
                                   const oxhip_qact& o, hipStream_t s) {
    const size_t blocks = rows * (inter / 32);
    if (!blocks) return hipSuccess;
    moe_act_quantize_kernel<<<(unsigned)((blocks + 31) / 32), 256, 0, s>>>(g, u, stride, rows, (uint32_t)inter, kind, param, o.q, o.scales, o.sums,
                                                                        o.fsums, o.hsums, o.sums16);
    return hipGetLastError();
}

// y[i] += w_j * o[row_of(i, j)] for j in route order: axpy per expert, multiply then add (src/moe.rs:608-615).
__global__ __launch_bounds__(256) void moe_combine_kernel(const float* __restrict__ o, const int* __restrict__ row_of,
                                                          const float* __restrict__ route_w, uint32_t t, uint32_t k, uint32_t h,
                                                          float* __restrict__ y, bool add) {
    size_t i = (size_t)blockIdx.x * blockDim.x + threadIdx.x;
    if (i >= (size_t)t * h) return;
    uint32_t tok = i / h, c = i % h;
    float acc = add ? y[i] : 0.0f;
    // eight routes at a time: their row numbers, then their values, are all requested before the first is added (one after
    // the other, every route costs two dependent round trips to memory)
    for (uint32_t j0 = 0; j0 < k; j0 += 8) {
        uint32_t row[8];
        float w[8], v[8];
#pragma unroll
        for (int e = 0; e < 8; e++) {
            const uint32_t j = min(j0 + e, k - 1);
            row[e] = (uint32_t)row_of[(size_t)tok * k + j];
            w[e] = route_w[(size_t)tok * k + j];
        }
#pragma unroll
        for (int e = 0; e < 8; e++) v[e] = o[(size_t)row[e] * h + c];
#pragma unroll
        for (int e = 0; e < 8; e++)
            if (j0 + e < k) acc = acc + w[e] * v[e];
    }
    y[i] = acc;
}

hipError_t launch_moe_combine(const float* o, const int* row_of, const float* route_w, size_t t, size_t k, size_t h, float* y,
                              hipStream_t s, bool add) {
    size_t total = t * h;
    if (!total) return hipSuccess;
    moe_combine_kernel<<<(unsigned)((total + 255) / 256), 256, 0, s>>>(o, row_of, route_w, (uint32_t)t, (uint32_t)k, (uint32_t)h, y, add);
    return hipGetLastError();
}

}  // namespace oxhip
