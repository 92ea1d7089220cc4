// Decode kernels on the vector ALUs (v_dot4_i32_i8) for the planar Q4 format (per-32 scales, any offset
// group) and for float-stored weights: dequant-fused GEMV / skinny GEMM, one wavefront per group of R
// weight rows. Q8_0, Q4_K, Q6_K and MLX Q4 run on the matrix cores (decode_mfma.hip).
//
// What they compute is what the reference's CPU decode kernels compute (QMat::rows_t1 / rows_tc,
// src/kernels.rs:1339-1369; dot_row_generic, src/ggml.rs:1288-1315; q4_dot_rows_tc_scalar,
// src/kernels_x86.rs:447-474): exact int32 dot products of the unpacked int8 weights with the int8
// activations per 32 elements, scaled in f32 by weight scale x activation scale,
// plus offset terms over the exact f32 activation sums. Only the order of the f32 additions
// differs (lanes, then a DPP tree).
//
// Shape of the kernel: a "unit" is one aligned 16-byte chunk of packed weights. Lane l of a wave
// takes units l, l+64, ... of a row, so a wave-wide load reads 1 KiB of consecutive bytes. The
// activations of a unit are loaded once per token and reused for the R rows of the wave; packed
// nibbles are split in registers and multiplied with v_dot4_i32_i8; the bias of the unsigned
// nibble codes is folded through the per-16 integer sums of the activations, so no
// per-element subtraction is needed.
#include "internal.hpp"
#include "layout.hpp"

namespace oxhip {

// One group of 16 activations of one token.
struct ActG {
    uint4 xq;
    float xs;   // scale of the enclosing block of 32
    float hs;   // exact f32 sum of the 16 values
    int s16;    // integer sum of the 16 int8 values
};

template <bool MIN, bool S16>
__device__ __forceinline__ void load_act(const QActView& xa, size_t tok_off16, uint32_t g, ActG& a) {
    // tok_off16 = token * n_in / 16
    a.xq = *reinterpret_cast<const uint4*>(xa.q + (tok_off16 + g) * 16);
    a.xs = xa.scales[(tok_off16 >> 1) + (g >> 1)];
    if (MIN) a.hs = xa.hsums[tok_off16 + g];
    if (S16) a.s16 = xa.sums16[tok_off16 + g];
}

__device__ __forceinline__ int dot16(const uint4& w, const uint4& x) {
    int s = dot4(w.x, x.x, 0);
    s = dot4(w.y, x.y, s);
    s = dot4(w.z, x.z, s);
    return dot4(w.w, x.w, s);
}
__device__ __forceinline__ uint4 lo_nibbles(const uint4& v) {
    return make_uint4(v.x & 0x0F0F0F0Fu, v.y & 0x0F0F0F0Fu, v.z & 0x0F0F0F0Fu, v.w & 0x0F0F0F0Fu);
}
__device__ __forceinline__ uint4 hi_nibbles(const uint4& v) {
    return make_uint4((v.x >> 4) & 0x0F0F0F0Fu, (v.y >> 4) & 0x0F0F0F0Fu, (v.z >> 4) & 0x0F0F0F0Fu, (v.w >> 4) & 0x0F0F0F0Fu);
}

template <int FMT>
struct F;

// ---- Q4 (Q4_0 layout, optional bf16 offsets): unit = one block of 32 ------------------------------
template <>
struct F<FMT_Q4> {
    static constexpr int NG = 2;
    static constexpr bool MIN = false, S16 = true;
    static constexpr int ISUMS_PER_UNIT = 1;
    struct W {
        uint4 lo, hi;
        float d;
    };
    __device__ static uint32_t units(const WeightView& w) { return w.n_in / 32; }
    __device__ static uint32_t group(uint32_t u, int g) { return 2 * u + g; }
    __device__ static void load(const WeightView& w, uint32_t r, uint32_t u, W& o) {
        uint4 v = *reinterpret_cast<const uint4*>(w.p0 + ((size_t)r * (w.n_in / 32) + u) * 16);
        o.lo = lo_nibbles(v);
        o.hi = hi_nibbles(v);
        o.d = f16_bits_to_f32(reinterpret_cast<const uint16_t*>(w.p1)[(size_t)r * (w.n_in / w.sgroup) + (u * 32) / w.sgroup]);
    }
    __device__ static void isums(const W& w, const ActG* a, int* out) {
        out[0] = dot16(w.lo, a[0].xq) + dot16(w.hi, a[1].xq) - 8 * (a[0].s16 + a[1].s16);
    }
    __device__ static float dot(const W& w, const ActG* a) {
        int i;
        isums(w, a, &i);
        return ((float)i * w.d) * a[0].xs;
    }
};

template <int FMT, int T, int R>
__global__ __launch_bounds__(256) void decode_kernel(WeightView w, QActView xa, float* __restrict__ y) {
    using Fm = F<FMT>;
    const uint32_t lane = threadIdx.x & 63;
    const uint32_t wave = blockIdx.x * (blockDim.x >> 6) + (threadIdx.x >> 6);
    const uint32_t nwaves = gridDim.x * (blockDim.x >> 6);
    const uint32_t units = Fm::units(w);
    const size_t tok16 = w.n_in / 16;
    for (uint32_t rg = wave; (size_t)rg * R < w.n_out; rg += nwaves) {
        const uint32_t r0 = rg * R;
        float acc[R][T];
#pragma unroll
        for (int r = 0; r < R; r++)
#pragma unroll
            for (int c = 0; c < T; c++) acc[r][c] = 0.0f;
        for (uint32_t u = lane; u < units; u += 64) {
            typename Fm::W wt[R];
#pragma unroll
            for (int r = 0; r < R; r++) Fm::load(w, min(r0 + r, w.n_out - 1), u, wt[r]);
#pragma unroll
            for (int c = 0; c < T; c++) {
                ActG a[Fm::NG];
#pragma unroll
                for (int g = 0; g < Fm::NG; g++) load_act<Fm::MIN, Fm::S16>(xa, c * tok16, Fm::group(u, g), a[g]);
#pragma unroll
                for (int r = 0; r < R; r++) acc[r][c] += Fm::dot(wt[r], a);
            }
        }
        if (FMT == FMT_Q4 && w.group) {
            // add_offsets (src/kernels.rs:1287-1297): sum_g offset[r][g] * (sum of x over group g)
            const uint32_t gpr = w.n_in / w.group, k = w.group / 32;
            const uint16_t* off = reinterpret_cast<const uint16_t*>(w.p2);
            for (uint32_t g = lane; g < gpr; g += 64) {
#pragma unroll
                for (int c = 0; c < T; c++) {
                    float gs = -0.0f;
                    for (uint32_t i = 0; i < k; i++) gs += xa.fsums[c * (w.n_in / 32) + g * k + i];
#pragma unroll
                    for (int r = 0; r < R; r++)
                        acc[r][c] += bf16_bits_to_f32(off[(size_t)min(r0 + r, w.n_out - 1) * gpr + g]) * gs;
                }
            }
        }
#pragma unroll
        for (int r = 0; r < R; r++)
#pragma unroll
            for (int c = 0; c < T; c++) {
                float v = wave_sum(acc[r][c]);
                if (lane == (uint32_t)(r * T + c) % 64 && r0 + r < w.n_out) y[(size_t)c * w.n_out + r0 + r] = v;
            }
    }
}

// ---- float-stored weights (FP8 with block scales, bf16): f32 activations, f32 FMA -----------------
// The reference multiplies the dequantized f32 weight (e4m3 * block scale) with the f32 activation
// (src/ggml.rs:433-444 + src/kernels.rs:1998-2038); here the block scale multiplies the partial sum
// of its 16 columns instead, which differs in rounding only.
template <int FMT, int T, int R>
__global__ __launch_bounds__(256) void decode_dense_kernel(WeightView w, const float* __restrict__ x, float* __restrict__ y) {
    const uint32_t lane = threadIdx.x & 63;
    const uint32_t wave = blockIdx.x * (blockDim.x >> 6) + (threadIdx.x >> 6);
    const uint32_t nwaves = gridDim.x * (blockDim.x >> 6);
    constexpr uint32_t EPU = FMT == FMT_FP8 ? 16 : 8;  // elements per 16-byte unit
    const uint32_t units = w.n_in / EPU;
    const uint32_t ncb = FMT == FMT_FP8 ? (w.n_in + w.bc - 1) / w.bc : 0;
    const float* bs = reinterpret_cast<const float*>(w.p1);
    for (uint32_t rg = wave; (size_t)rg * R < w.n_out; rg += nwaves) {
        const uint32_t r0 = rg * R;
        float acc[R][T];
#pragma unroll
        for (int r = 0; r < R; r++)
#pragma unroll
            for (int c = 0; c < T; c++) acc[r][c] = 0.0f;
        for (uint32_t u = lane; u < units; u += 64) {
            float wf[R][EPU];
            float sc[R];
#pragma unroll
            for (int r = 0; r < R; r++) {
                uint32_t row = min(r0 + r, w.n_out - 1);
                uint4 v = *reinterpret_cast<const uint4*>(w.p0 + (FMT == FMT_FP8 ? fp8_offset(w, row, (size_t)u * 16) : ((size_t)row * units + u) * 16));
                uint32_t d[4] = {v.x, v.y, v.z, v.w};
                if (FMT == FMT_FP8) {
#pragma unroll
                    for (int i = 0; i < 16; i++) wf[r][i] = e4m3_to_f32((d[i >> 2] >> (8 * (i & 3))) & 0xFF);
                    sc[r] = bs[(size_t)(row / w.br) * ncb + (u * 16) / w.bc];
                } else {
#pragma unroll
                    for (int i = 0; i < 8; i++) wf[r][i] = __uint_as_float(((d[i >> 1] >> (16 * (i & 1))) & 0xFFFF) << 16);
                    sc[r] = 1.0f;
                }
            }
#pragma unroll
            for (int c = 0; c < T; c++) {
                float xv[EPU];
                const float4* xp = reinterpret_cast<const float4*>(x + (size_t)c * w.n_in + (size_t)u * EPU);
#pragma unroll
                for (int i = 0; i < (int)EPU / 4; i++) {
                    float4 f = xp[i];
                    xv[4 * i] = f.x;
                    xv[4 * i + 1] = f.y;
                    xv[4 * i + 2] = f.z;
                    xv[4 * i + 3] = f.w;
                }
#pragma unroll
                for (int r = 0; r < R; r++) {
                    float p = 0.0f;
#pragma unroll
                    for (int i = 0; i < (int)EPU; i++) p = __builtin_fmaf(wf[r][i], xv[i], p);
                    acc[r][c] = __builtin_fmaf(sc[r], p, acc[r][c]);
                }
            }
        }
#pragma unroll
        for (int r = 0; r < R; r++)
#pragma unroll
            for (int c = 0; c < T; c++) {
                float v = wave_sum(acc[r][c]);
                if (lane == (uint32_t)(r * T + c) % 64 && r0 + r < w.n_out) y[(size_t)c * w.n_out + r0 + r] = v;
            }
    }
}

// ---- NVFP4 (float-stored: f32 activations, src/ggml.rs:219-224) from its tile records --------------------------------
// A workgroup of 8 waves owns a row tile and splits its K-steps; lane 16 kq + n of a wave owns row n's 32 weights of
// the step that its 16 bytes hold (layout.hpp), dequantized as the reference does ((scale / 2) * doubled value, then the
// matrix's scale) and multiplied with the f32 activations in f32. T tokens per pass.
template <int T>
__global__ __launch_bounds__(512) void decode_nvfp4_kernel(WeightView w, const float* __restrict__ x, float* __restrict__ y) {
    __shared__ float red[8][T][16];
    const uint32_t lane = threadIdx.x & 63, wave = threadIdx.x >> 6, n = lane & 15, kq = lane >> 4;
    const uint32_t nsteps = t4m_steps(w.n_in), tile = blockIdx.x, row = tile * 16 + n;
    const uint8_t* base = w.p0 + (size_t)tile * nsteps * T4N_REC;
    const float* bs = reinterpret_cast<const float*>(w.p1);
    const uint32_t ncb = w.br ? (w.n_in + w.bc - 1) / w.bc : 0;
    float acc[T];
#pragma unroll
    for (int c = 0; c < T; c++) acc[c] = 0.0f;
    for (uint32_t s = wave; s < nsteps; s += 8) {
        const uint8_t* rec = base + (size_t)s * T4N_REC;
        const uint4 cv = *reinterpret_cast<const uint4*>(rec + 16 * lane);
        const uint2 sv = *reinterpret_cast<const uint2*>(rec + 1024 + 8 * n);
        const uint32_t cw[4] = {cv.x, cv.y, cv.z, cv.w};
        const float g = w.br ? bs[(size_t)(min(row, w.n_out - 1) / w.br) * ncb + (128 * s) / w.bc] : 1.0f;
#pragma unroll
        for (int b = 0; b < 4; b++) {
            if (128 * s + 32 * b >= w.n_in) break;  // a row's last step may hold fewer than four groups of 32 (uniform)
            const uint32_t sw = b < 2 ? sv.x : sv.y;
            const float d[2] = {ue4m3_half(sw >> (16 * (b & 1))), ue4m3_half(sw >> (16 * (b & 1) + 8))};
#pragma unroll
            for (int h = 0; h < 2; h++) {  // the low nibbles: columns 32 b + 4 kq + j; the high ones: + 16
                const uint32_t kv4 = mxfp4_values<0>((cw[b] >> (4 * h)) & 0x0F0F0F0Fu);
                float wf[4];
#pragma unroll
                for (int j = 0; j < 4; j++) {
                    wf[j] = d[h] * (float)(int)(int8_t)((kv4 >> (8 * j)) & 0xFF);
                    if (w.br) wf[j] *= g;
                }
                const size_t col = (size_t)128 * s + 32 * b + 16 * h + 4 * kq;
#pragma unroll
                for (int c = 0; c < T; c++) {
                    const float4 xv = *reinterpret_cast<const float4*>(x + (size_t)c * w.n_in + col);
                    acc[c] = __builtin_fmaf(wf[0], xv.x, acc[c]);
                    acc[c] = __builtin_fmaf(wf[1], xv.y, acc[c]);
                    acc[c] = __builtin_fmaf(wf[2], xv.z, acc[c]);
                    acc[c] = __builtin_fmaf(wf[3], xv.w, acc[c]);
                }
            }
        }
    }
#pragma unroll
    for (int c = 0; c < T; c++) {
        float v = acc[c];
        v += __shfl_xor(v, 16);
        v += __shfl_xor(v, 32);
        if (kq == 0) red[wave][c][n] = v;
    }
    __syncthreads();
    if (threadIdx.x < 16 * T) {
        const uint32_t c = threadIdx.x / 16, nn = threadIdx.x % 16;
        float v = 0.0f;
#pragma unroll
        for (int k = 0; k < 8; k++) v += red[k][c][nn];
        if (tile * 16 + nn < w.n_out) y[(size_t)c * w.n_out + tile * 16 + nn] = v;
    }
}

hipError_t launch_decode_nvfp4(const WeightView& w, const float* x, size_t t, float* y, hipStream_t s) {
    if (w.fmt != FMT_NVFP4 || !x || reinterpret_cast<uintptr_t>(x) % 16) return hipErrorInvalidValue;  // (rows are multiples of 64 floats)
    const unsigned grid = row_tiles(w.n_out);
    size_t c0 = 0;
    while (c0 < t) {
        const size_t tc = t - c0 < 4 ? t - c0 : 4;
        const float* xi = x + c0 * w.n_in;
        float* yo = y + c0 * w.n_out;
        switch (tc) {
            case 1: decode_nvfp4_kernel<1><<<grid, 512, 0, s>>>(w, xi, yo); break;
            case 2: decode_nvfp4_kernel<2><<<grid, 512, 0, s>>>(w, xi, yo); break;
            case 3: decode_nvfp4_kernel<3><<<grid, 512, 0, s>>>(w, xi, yo); break;
            default: decode_nvfp4_kernel<4><<<grid, 512, 0, s>>>(w, xi, yo); break;
        }
        hipError_t e = hipGetLastError();
        if (e != hipSuccess) return e;
        c0 += tc;
    }
    return hipSuccess;
}

// ---- exact integer accumulators (parity checks): one thread per (token, row, unit) ---------------
template <int FMT>
__global__ __launch_bounds__(256) void isums_kernel(WeightView w, QActView xa, uint32_t t, int32_t* __restrict__ out) {
    using Fm = F<FMT>;
    const uint32_t units = Fm::units(w);
    size_t idx = (size_t)blockIdx.x * blockDim.x + threadIdx.x;
    size_t total = (size_t)t * w.n_out * units;
    if (idx >= total) return;
    uint32_t u = idx % units;
    uint32_t r = (idx / units) % w.n_out;
    uint32_t c = idx / ((size_t)units * w.n_out);
    typename Fm::W wt;
    Fm::load(w, r, u, wt);
    ActG a[Fm::NG];
    for (int g = 0; g < Fm::NG; g++) load_act<Fm::MIN, Fm::S16>(xa, (size_t)c * (w.n_in / 16), Fm::group(u, g), a[g]);
    int v[2];
    Fm::isums(wt, a, v);
    if (FMT == FMT_Q4) {
        out[((size_t)c * w.n_out + r) * (w.n_in / 32) + u] = v[0];
    } else {
        size_t base = ((size_t)c * w.n_out + r) * (w.n_in / 16);
        for (int g = 0; g < Fm::ISUMS_PER_UNIT; g++) out[base + Fm::group(u, g)] = v[g];
    }
}

namespace {

unsigned grid_for(size_t row_groups) {
    // enough workgroups of 4 waves to cover every row group once, capped at 16 waves per CU
    size_t blocks = (row_groups + 3) / 4;
    size_t cap = 256 * 4 * 4;  // 256 CUs x 4 workgroups of 4 waves
    return (unsigned)(blocks < cap ? (blocks ? blocks : 1) : cap);
}

template <int FMT, int R>
hipError_t decode_t(const WeightView& w, const QActView& xa, size_t t, float* y, hipStream_t s) {
    unsigned grid = grid_for((w.n_out + R - 1) / R);
    // tokens in chunks of up to 8 (the weights are re-read per chunk)
    size_t c0 = 0;
    while (c0 < t) {
        size_t tc = t - c0 < 8 ? t - c0 : 8;
        QActView v = xa;
        v.q += c0 * w.n_in;
        v.scales += c0 * (w.n_in / 32);
        v.sums += c0 * (w.n_in / 32);
        v.fsums += c0 * (w.n_in / 32);
        v.hsums += c0 * (w.n_in / 16);
        v.sums16 += c0 * (w.n_in / 16);
        float* yo = y + c0 * w.n_out;
        switch (tc) {
            case 1: decode_kernel<FMT, 1, R><<<grid, 256, 0, s>>>(w, v, yo); break;
            case 2: decode_kernel<FMT, 2, R><<<grid, 256, 0, s>>>(w, v, yo); break;
            case 3: decode_kernel<FMT, 3, R><<<grid, 256, 0, s>>>(w, v, yo); break;
            case 4: decode_kernel<FMT, 4, R><<<grid, 256, 0, s>>>(w, v, yo); break;
            case 5: decode_kernel<FMT, 5, R><<<grid, 256, 0, s>>>(w, v, yo); break;
            case 6: decode_kernel<FMT, 6, R><<<grid, 256, 0, s>>>(w, v, yo); break;
            case 7: decode_kernel<FMT, 7, R><<<grid, 256, 0, s>>>(w, v, yo); break;
            default: decode_kernel<FMT, 8, R><<<grid, 256, 0, s>>>(w, v, yo); break;
        }
        hipError_t e = hipGetLastError();
        if (e != hipSuccess) return e;
        c0 += tc;
    }
    return hipSuccess;
}

template <int FMT, int R>
hipError_t decode_dense_t(const WeightView& w, const float* x, size_t t, float* y, hipStream_t s) {
    unsigned grid = grid_for((w.n_out + R - 1) / R);
    size_t c0 = 0;
    while (c0 < t) {
        size_t tc = t - c0 < 4 ? t - c0 : 4;
        const float* xi = x + c0 * w.n_in;
        float* yo = y + c0 * w.n_out;
        switch (tc) {
            case 1: decode_dense_kernel<FMT, 1, R><<<grid, 256, 0, s>>>(w, xi, yo); break;
            case 2: decode_dense_kernel<FMT, 2, R><<<grid, 256, 0, s>>>(w, xi, yo); break;
            case 3: decode_dense_kernel<FMT, 3, R><<<grid, 256, 0, s>>>(w, xi, yo); break;
            default: decode_dense_kernel<FMT, 4, R><<<grid, 256, 0, s>>>(w, xi, yo); break;
        }
        hipError_t e = hipGetLastError();
        if (e != hipSuccess) return e;
        c0 += tc;
    }
    return hipSuccess;
}

}  // namespace

static hipError_t launch_decode_plain(const WeightView& w, const QActView& xa, const float* x, size_t t, float* y, hipStream_t s,
                                      const DecodeScratch& sc) {
    switch (w.fmt) {
        case FMT_Q4: return decode_t<FMT_Q4, 4>(w, xa, t, y, s);
        case FMT_FP8:
            // the matrix-core kernel when the block scales allow it and the caller's scratch holds the packed activations
            if (skinny_fp8_ok(w, t) && sc.partial && skinny_fp8_pack_bytes(w, t, 2) <= sc.partial_floats * 4)
                return launch_skinny_fp8(w, x, false, true, t, y, false, sc.partial, s);
            return decode_dense_t<FMT_FP8, 4>(w, x, t, y, s);
        case FMT_BF16: return decode_dense_t<FMT_BF16, 4>(w, x, t, y, s);
        case FMT_NVFP4: return launch_decode_nvfp4(w, x, t, y, s);
        default: return hipErrorInvalidValue;
    }
}

hipError_t launch_decode(const WeightView& w, const QActView& xa, const float* x, size_t t, float* y, hipStream_t s,
                         const DecodeScratch& sc, hipEvent_t ev_start, hipEvent_t ev_stop) {
    if (mfma_decode_format(w.fmt)) return launch_decode_mfma(w, xa, t, y, sc, s, ev_start, ev_stop);
    hipError_t e = ev_start ? hipEventRecord(ev_start, s) : hipSuccess;
    if (e == hipSuccess) e = launch_decode_plain(w, xa, x, t, y, s, sc);
    if (e == hipSuccess && ev_stop) e = hipEventRecord(ev_stop, s);
    return e;
}

hipError_t launch_isums(const WeightView& w, const QActView& xa, size_t t, int32_t* out, hipStream_t s) {
    if (mfma_decode_format(w.fmt)) return launch_isums_mfma(w, xa, t, nullptr, out, s);
    size_t units = w.n_in / 32;
    size_t total = t * w.n_out * units;
    unsigned grid = (unsigned)((total + 255) / 256);
    switch (w.fmt) {
        case FMT_Q4: isums_kernel<FMT_Q4><<<grid, 256, 0, s>>>(w, xa, (uint32_t)t, out); break;
        default: return hipErrorInvalidValue;
    }
    return hipGetLastError();
}

}  // namespace oxhip
