// FP8 block-scaled GEMM on the fp8 matrix cores: y[t][n_out] = x[t][n_in] * W^T with W e4m3 bytes and one f32
// scale per 128 x 128 block (GgufMatrix::fp8, src/ggml.rs:325-341 of the reference).
//
// The reference multiplies the dequantized f32 weights (e4m3 * block scale, src/ggml.rs:433-444) with f32
// activations (its float-stored path, src/kernels.rs:1802); its only GPU FP8 path converts to half
// (src/metal.rs:805-812). Here the activations are quantized on the device to e4m3 per token and 128-column tile
// (scale = amax / 448, round to nearest even, saturating), one v_mfma_f32_16x16x128_f8f6f4 forms the f32 product of
// a whole scale block, and the two scales multiply that partial sum on its way into the f32 accumulator. Results
// agree with the CPU to fp8-activation precision (the 2e-2 bar), not bit for bit.
//
// Work split as in gemm.hip: a workgroup of 4 waves owns 256 tokens x 128 rows (one row of scale blocks); per
// K-block of 128 the four waves copy the 8 row tiles' bytes (2 KiB each, two tiles per wave) into LDS as MFMA
// fragments (lane = 16 kq + n holds row n's bytes 32 kq .. 32 kq + 31, which are contiguous in the row-major
// weights, so no repacking at upload) and every wave reads all 8; activation fragments come packed from global
// memory. K may be split over workgroups (gridDim.z) when the output is narrow.
#include <type_traits>

#include "internal.hpp"
#include "layout.hpp"

namespace oxhip {

typedef int v8i __attribute__((ext_vector_type(8)));
typedef float f32x4 __attribute__((ext_vector_type(4)));

// x [t][n_in] (f32 or bf16) -> e4m3 fragments [mtile][kblock][lane][32 B] (lane = 16 kq + m: token 16 mtile + m,
// columns 128 kb + 32 kq .. + 31) and scales sx [kblock][mtiles * 16]. One wave per (token tile, K-block): the
// four lanes of a token share its amax through two shuffles.
template <bool SRC_BF16>
__global__ __launch_bounds__(64) void quantize_act_fp8_kernel(const void* __restrict__ x, uint32_t t, uint32_t n_in, uint32_t mtiles,
                                                              uint32_t kblocks, uint4* __restrict__ out, float* __restrict__ sx) {
    const uint32_t lane = threadIdx.x, m = lane & 15, kq = lane >> 4;
    const uint32_t kb = blockIdx.x % kblocks, mt = blockIdx.x / kblocks;
    const uint32_t tok = mt * 16 + m;
    float v[32];
#pragma unroll
    for (int j = 0; j < 32; j++) {
        const uint32_t k = 128 * kb + 32 * kq + j;
        float f = 0.0f;
        if (tok < t && k < n_in) {
            if (SRC_BF16) f = bf16_bits_to_f32(reinterpret_cast<const uint16_t*>(x)[(size_t)tok * n_in + k]);
            else f = reinterpret_cast<const float*>(x)[(size_t)tok * n_in + k];
        }
        v[j] = f;
    }
    float amax = 0.0f;
#pragma unroll
    for (int j = 0; j < 32; j++) amax = fmaxf(amax, fabsf(v[j]));
    amax = fmaxf(amax, __shfl_xor(amax, 16));
    amax = fmaxf(amax, __shfl_xor(amax, 32));
    const float scale = amax / 448.0f;
    const float inv = amax > 0.0f ? 448.0f / amax : 0.0f;
    uint32_t w[8];
#pragma unroll
    for (int j = 0; j < 8; j++) {
        int p = 0;
        p = __builtin_amdgcn_cvt_pk_fp8_f32(fminf(fmaxf(v[4 * j] * inv, -448.0f), 448.0f), fminf(fmaxf(v[4 * j + 1] * inv, -448.0f), 448.0f), p, false);
        p = __builtin_amdgcn_cvt_pk_fp8_f32(fminf(fmaxf(v[4 * j + 2] * inv, -448.0f), 448.0f), fminf(fmaxf(v[4 * j + 3] * inv, -448.0f), 448.0f), p, true);
        w[j] = (uint32_t)p;
    }
    uint4* dst = out + ((size_t)(mt * kblocks + kb) * 64 + lane) * 2;
    dst[0] = make_uint4(w[0], w[1], w[2], w[3]);
    dst[1] = make_uint4(w[4], w[5], w[6], w[7]);
    if (kq == 0) sx[(size_t)kb * mtiles * 16 + tok] = scale;
}

hipError_t launch_quantize_act_fp8(const void* x, bool src_bf16, size_t t, size_t n_in, size_t mtiles, size_t kblocks, void* out,
                                   float* sx, hipStream_t s) {
    const size_t blocks = mtiles * kblocks;
    if (!blocks) return hipSuccess;
    if (src_bf16) quantize_act_fp8_kernel<true><<<(unsigned)blocks, 64, 0, s>>>(x, (uint32_t)t, (uint32_t)n_in, (uint32_t)mtiles, (uint32_t)kblocks, static_cast<uint4*>(out), sx);
    else quantize_act_fp8_kernel<false><<<(unsigned)blocks, 64, 0, s>>>(x, (uint32_t)t, (uint32_t)n_in, (uint32_t)mtiles, (uint32_t)kblocks, static_cast<uint4*>(out), sx);
    return hipGetLastError();
}

namespace {
constexpr int F8_MT = 16;  // token tiles per workgroup (4 per wave)
constexpr int F8_NT = 8;   // row tiles per workgroup (128 rows = one scale block row)
}  // namespace

template <bool OUT_BF16>
__global__ __launch_bounds__(256) void gemm_fp8_kernel(WeightView w, const uint4* __restrict__ apk, const float* __restrict__ sx,
                                                       uint32_t t, uint32_t mtiles, void* __restrict__ yv) {
    extern __shared__ uint4 bfrag[];  // [2][8 row tiles][64 lanes][2]
    const uint32_t lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
    const uint32_t n = lane & 15, kq = lane >> 4;
    const uint32_t all_kb = (w.n_in + 127) / 128;
    const uint32_t per_z = (all_kb + gridDim.z - 1) / gridDim.z;
    const uint32_t kb0 = blockIdx.z * per_z;
    const uint32_t nkb = min(all_kb, kb0 + per_z) - kb0;
    const uint32_t nt0 = blockIdx.x * F8_NT;
    const uint32_t mt0 = blockIdx.y * F8_MT + wave * 4;
    const uint32_t ncb = (w.n_in + w.bc - 1) / w.bc;
    const float* bs = reinterpret_cast<const float*>(w.p1);

    // the two row tiles whose bytes this wave copies: row pointers of this lane (rows past the end repeat the last)
    const uint8_t* wrow[2];
#pragma unroll
    for (int i = 0; i < 2; i++) wrow[i] = w.p0 + fp8_offset(w, min((nt0 + 2 * wave + i) * 16 + n, w.n_out - 1), 32 * kq);
    const uint32_t wstep = w.group == 1 ? 2048 : 128;  // bytes between a lane's chunks of consecutive 128-column steps
    const uint4* abase[4];
#pragma unroll
    for (int i = 0; i < 4; i++) abase[i] = apk + ((size_t)min(mt0 + i, mtiles - 1) * all_kb * 64 + lane) * 2;
    const uint32_t srow = min(nt0 * 16, w.n_out - 1) / w.br;  // the workgroup's 128 rows lie in one scale block row

    f32x4 acc[4][F8_NT];
#pragma unroll
    for (int i = 0; i < 4; i++)
#pragma unroll
        for (int j = 0; j < F8_NT; j++) acc[i][j] = f32x4{0.0f, 0.0f, 0.0f, 0.0f};

    auto load_w = [&](uint4 (*r)[2], uint32_t kb) {
        const size_t col = (size_t)wstep * kb;
#pragma unroll
        for (int i = 0; i < 2; i++) {
            r[i][0] = *reinterpret_cast<const uint4*>(wrow[i] + col);
            r[i][1] = *reinterpret_cast<const uint4*>(wrow[i] + col + 16);
        }
    };
    auto store_w = [&](const uint4 (*r)[2], uint32_t buf) {
#pragma unroll
        for (int i = 0; i < 2; i++) {
            bfrag[((buf * F8_NT + 2 * wave + i) * 64 + lane) * 2] = r[i][0];
            bfrag[((buf * F8_NT + 2 * wave + i) * 64 + lane) * 2 + 1] = r[i][1];
        }
    };
    auto read_a = [&](uint4 (*dst)[2], uint32_t kb) {
#pragma unroll
        for (int i = 0; i < 4; i++) {
            dst[i][0] = abase[i][(size_t)kb * 128];
            dst[i][1] = abase[i][(size_t)kb * 128 + 1];
        }
    };
    // per token-tile: s_w * s_x for the 4 tokens this lane's registers hold
    auto read_f = [&](f32x4* f, uint32_t kb) {
        const float sw = bs[(size_t)srow * ncb + (128 * kb) / w.bc];
#pragma unroll
        for (int i = 0; i < 4; i++) {
            const float4 v = *reinterpret_cast<const float4*>(sx + (size_t)kb * mtiles * 16 + min(mt0 + i, mtiles - 1) * 16 + 4 * kq);
            f[i] = f32x4{v.x * sw, v.y * sw, v.z * sw, v.w * sw};
        }
    };
    auto lds_barrier = [] { asm volatile("s_waitcnt lgkmcnt(0)\n\ts_barrier" ::: "memory"); };

    uint4 wr[2][2], a_cur[4][2], a_nxt[4][2];
    f32x4 f_cur[4], f_nxt[4];
    load_w(wr, kb0);
    read_a(a_cur, kb0);
    read_f(f_cur, kb0);
    store_w(wr, 0);
    if (nkb > 1) load_w(wr, kb0 + 1);
    lds_barrier();
    auto block = [&](uint32_t i_kb, auto more_c) {
        constexpr bool MORE = decltype(more_c)::value;
        const uint32_t buf = i_kb & 1, kb = kb0 + i_kb;
        if (MORE) {
            read_a(a_nxt, kb + 1);
            read_f(f_nxt, kb + 1);
            store_w(wr, buf ^ 1);  // the other buffer was last read two blocks ago, before the previous barrier
        }
#pragma unroll
        for (int j = 0; j < F8_NT; j++) {
            const uint4 b0 = bfrag[((buf * F8_NT + j) * 64 + lane) * 2], b1 = bfrag[((buf * F8_NT + j) * 64 + lane) * 2 + 1];
            const v8i bb = {(int)b0.x, (int)b0.y, (int)b0.z, (int)b0.w, (int)b1.x, (int)b1.y, (int)b1.z, (int)b1.w};
#pragma unroll
            for (int i = 0; i < 4; i++) {
                const v8i aa = {(int)a_cur[i][0].x, (int)a_cur[i][0].y, (int)a_cur[i][0].z, (int)a_cur[i][0].w,
                                (int)a_cur[i][1].x, (int)a_cur[i][1].y, (int)a_cur[i][1].z, (int)a_cur[i][1].w};
                const f32x4 z = {0.0f, 0.0f, 0.0f, 0.0f};
                const f32x4 d = __builtin_amdgcn_mfma_scale_f32_16x16x128_f8f6f4(aa, bb, z, 0, 0, 0, 127, 0, 127);
#pragma unroll
                for (int r = 0; r < 4; r++) acc[i][j][r] = __builtin_fmaf(f_cur[i][r], d[r], acc[i][j][r]);
            }
        }
        if (MORE) {
            if (i_kb + 2 < nkb) load_w(wr, kb + 2);
            lds_barrier();
#pragma unroll
            for (int i = 0; i < 4; i++) {
                a_cur[i][0] = a_nxt[i][0];
                a_cur[i][1] = a_nxt[i][1];
                f_cur[i] = f_nxt[i];
            }
        }
    };
    using T_ = std::integral_constant<bool, true>;
    using F_ = std::integral_constant<bool, false>;
    uint32_t i_kb = 0;
    for (; i_kb + 1 < nkb; i_kb++) block(i_kb, T_{});
    block(i_kb, F_{});

    if (gridDim.z > 1) yv = reinterpret_cast<float*>(yv) + (size_t)blockIdx.z * t * w.n_out;
#pragma unroll
    for (int i = 0; i < 4; i++) {
#pragma unroll
        for (int j = 0; j < F8_NT; j++) {
            const uint32_t row = (nt0 + j) * 16 + n;
#pragma unroll
            for (int r = 0; r < 4; r++) {
                const uint32_t tok = (mt0 + i) * 16 + 4 * kq + r;
                if (tok < t && row < w.n_out && mt0 + i < mtiles) {
                    if (OUT_BF16) reinterpret_cast<uint16_t*>(yv)[(size_t)tok * w.n_out + row] = f32_to_bf16_bits(acc[i][j][r]);
                    else reinterpret_cast<float*>(yv)[(size_t)tok * w.n_out + row] = acc[i][j][r];
                }
            }
        }
    }
}

template <bool OUT_BF16>
__global__ __launch_bounds__(256) void gemm_fp8_reduce_kernel(const float* __restrict__ p, size_t n, uint32_t slices, void* __restrict__ yv) {
    size_t i = (size_t)blockIdx.x * blockDim.x + threadIdx.x;
    if (i >= n) return;
    float v = p[i];
    for (uint32_t z = 1; z < slices; z++) v += p[(size_t)z * n + i];
    if (OUT_BF16) reinterpret_cast<uint16_t*>(yv)[i] = f32_to_bf16_bits(v);
    else reinterpret_cast<float*>(yv)[i] = v;
}

uint32_t gemm_fp8_k_slices(const WeightView& w, size_t mtiles) {
    const uint32_t wgs = ((row_tiles(w.n_out) + F8_NT - 1) / F8_NT) * (uint32_t)((mtiles + F8_MT - 1) / F8_MT);
    const uint32_t kbs = (w.n_in + 127) / 128;
    uint32_t z = 1;
    while (z < 8 && wgs * z * 2 <= 256 && kbs / (z * 2) >= 8) z *= 2;
    return z;
}

hipError_t launch_gemm_fp8(const WeightView& w, const void* apk, const float* sx, size_t t, size_t mtiles, void* y, bool out_bf16,
                           float* partial, hipStream_t s) {
    if (w.fmt != FMT_FP8 || w.br != 128 || w.bc != 128 || w.n_in % 128) return hipErrorInvalidValue;
    const uint32_t slices = gemm_fp8_k_slices(w, mtiles);
    dim3 grid((row_tiles(w.n_out) + F8_NT - 1) / F8_NT, (unsigned)((mtiles + F8_MT - 1) / F8_MT), slices);
    const size_t lds = 2 * F8_NT * 64 * 32;  // 32 KiB
    const bool direct_bf16 = out_bf16 && slices == 1;
    void* dst = slices > 1 ? static_cast<void*>(partial) : y;
    if (direct_bf16) gemm_fp8_kernel<true><<<grid, 256, lds, s>>>(w, static_cast<const uint4*>(apk), sx, (uint32_t)t, (uint32_t)mtiles, dst);
    else gemm_fp8_kernel<false><<<grid, 256, lds, s>>>(w, static_cast<const uint4*>(apk), sx, (uint32_t)t, (uint32_t)mtiles, dst);
    hipError_t e = hipGetLastError();
    if (e != hipSuccess || slices == 1) return e;
    const size_t n = t * (size_t)w.n_out;
    if (out_bf16) gemm_fp8_reduce_kernel<true><<<(unsigned)((n + 255) / 256), 256, 0, s>>>(partial, n, slices, y);
    else gemm_fp8_reduce_kernel<false><<<(unsigned)((n + 255) / 256), 256, 0, s>>>(partial, n, slices, y);
    return hipGetLastError();
}

}  // namespace oxhip
