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
// Work split as in gemm.hip: a workgroup of 8 waves owns 256 tokens x 128 rows (one row of scale blocks), each wave
// two token tiles and all the rows; per
// K-block of 128 the waves copy the 8 row tiles' bytes (2 KiB each, one tile per wave) into LDS as MFMA
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
    const uint32_t k0 = 128 * kb + 32 * kq;
    if (tok < t && k0 + 32 <= n_in && n_in % 8 == 0 && reinterpret_cast<uintptr_t>(x) % 16 == 0) {  // the lane's 32 columns as whole 16-byte reads
        if (SRC_BF16) {
            const uint4* src = reinterpret_cast<const uint4*>(reinterpret_cast<const uint16_t*>(x) + (size_t)tok * n_in + k0);
#pragma unroll
            for (int q = 0; q < 4; q++) {
                const uint4 u = src[q];
                const uint32_t d[4] = {u.x, u.y, u.z, u.w};
#pragma unroll
                for (int e = 0; e < 4; e++) {
                    v[8 * q + 2 * e] = __uint_as_float(d[e] << 16);
                    v[8 * q + 2 * e + 1] = __uint_as_float(d[e] & 0xFFFF0000u);
                }
            }
        } else {
            const float4* src = reinterpret_cast<const float4*>(reinterpret_cast<const float*>(x) + (size_t)tok * n_in + k0);
#pragma unroll
            for (int q = 0; q < 8; q++) {
                const float4 f = src[q];
                v[4 * q] = f.x;
                v[4 * q + 1] = f.y;
                v[4 * q + 2] = f.z;
                v[4 * q + 3] = f.w;
            }
        }
    } else {
#pragma unroll
        for (int j = 0; j < 32; j++) {
            const uint32_t k = k0 + j;
            float f = 0.0f;
            if (tok < t && k < n_in) {
                if (SRC_BF16) f = bf16_bits_to_f32(reinterpret_cast<const uint16_t*>(x)[(size_t)tok * n_in + k]);
                else f = reinterpret_cast<const float*>(x)[(size_t)tok * n_in + k];
            }
            v[j] = f;
        }
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
constexpr int F8_MT = 16;  // token tiles per workgroup
constexpr int F8_NT = 8;   // row tiles per workgroup (128 rows = one scale block row)
constexpr int F8_WAVES = 8;              // waves per workgroup: two per SIMD, so that one issues matrix instructions while the other scales and accumulates
constexpr int F8_TW = F8_MT / F8_WAVES;  // token tiles per wave
constexpr int F8_RW = F8_NT / F8_WAVES;  // row tiles whose bytes a wave copies
}  // namespace

template <bool OUT_BF16>
__global__ __launch_bounds__(64 * F8_WAVES) void gemm_fp8_kernel(WeightView w, const uint4* __restrict__ apk, const float* __restrict__ sx,
                                                       uint32_t t, uint32_t mtiles, void* __restrict__ yv) {
    extern __shared__ uint4 bfrag[];  // [2][8 row tiles][2 halves][64 lanes]: a lane's two 16-byte halves lie a plane apart (no bank conflicts)
    const uint32_t lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
    const uint32_t n = lane & 15, kq = lane >> 4;
    const uint32_t all_kb = (w.n_in + 127) / 128;
    const uint32_t per_z = (all_kb + gridDim.z - 1) / gridDim.z;
    const uint32_t kb0 = blockIdx.z * per_z;
    const uint32_t nkb = min(all_kb, kb0 + per_z) - kb0;
    const uint32_t nt0 = blockIdx.x * F8_NT;
    const uint32_t mt0 = blockIdx.y * F8_MT + wave * F8_TW;
    const uint32_t ncb = (w.n_in + w.bc - 1) / w.bc;
    const float* bs = reinterpret_cast<const float*>(w.p1);

    // the two row tiles whose bytes this wave copies: row pointers of this lane (rows past the end repeat the last)
    const uint8_t* wrow[F8_RW];
#pragma unroll
    for (int i = 0; i < F8_RW; i++) wrow[i] = w.p0 + fp8_offset(w, min((nt0 + F8_RW * wave + i) * 16 + n, w.n_out - 1), 32 * kq);
    const uint32_t wstep = w.group == 1 ? 2048 : 128;  // bytes between a lane's chunks of consecutive 128-column steps
    const uint32_t whi = fp8_second_chunk(w);
    const uint4* abase[F8_TW];
#pragma unroll
    for (int i = 0; i < F8_TW; i++) abase[i] = apk + ((size_t)min(mt0 + i, mtiles - 1) * all_kb * 64 + lane) * 2;
    const uint32_t srow = min(nt0 * 16, w.n_out - 1) / w.br;  // the workgroup's 128 rows lie in one scale block row

    f32x4 acc[F8_TW][F8_NT];
#pragma unroll
    for (int i = 0; i < F8_TW; i++)
#pragma unroll
        for (int j = 0; j < F8_NT; j++) acc[i][j] = f32x4{0.0f, 0.0f, 0.0f, 0.0f};

    // Register sets are structs of vector-extension values, indexed only by compile-time constants: HIP's uint4 under
    // a condition, or a set reached through a pointer, ends up in scratch memory.
    typedef uint32_t u32x4 __attribute__((ext_vector_type(4)));
    struct WRegs {
        u32x4 v[F8_RW][2];
    };
    struct ARegs {
        u32x4 v[F8_TW][2];
        f32x4 sx[F8_TW];  // the activation scales of the lane's four tokens per tile
        float sw;     // the weight block's scale
    };
    // every request is unconditional and clamped to the last block: a request under a condition makes the compiler
    // wait for all outstanding ones
    auto load_w = [&](WRegs& r, uint32_t i_kb) {
        const size_t col = (size_t)wstep * (kb0 + min(i_kb, nkb - 1));
#pragma unroll
        for (int i = 0; i < F8_RW; i++) {
            r.v[i][0] = *reinterpret_cast<const u32x4*>(wrow[i] + col);
            r.v[i][1] = *reinterpret_cast<const u32x4*>(wrow[i] + col + whi);
        }
    };
    auto store_w = [&](const WRegs& r, uint32_t buf) {
#pragma unroll
        for (int i = 0; i < F8_RW; i++) {
            u32x4* dst = reinterpret_cast<u32x4*>(bfrag + (size_t)(buf * F8_NT + F8_RW * wave + i) * 128 + lane);
            dst[0] = r.v[i][0];
            dst[64] = r.v[i][1];
        }
    };
    auto read_a = [&](ARegs& dst, uint32_t i_kb) {
        const uint32_t kb = kb0 + min(i_kb, nkb - 1);
#pragma unroll
        for (int i = 0; i < F8_TW; i++) {
            const u32x4* src = reinterpret_cast<const u32x4*>(abase[i] + (size_t)kb * 128);
            dst.v[i][0] = src[0];
            dst.v[i][1] = src[1];
            dst.sx[i] = *reinterpret_cast<const f32x4*>(sx + (size_t)kb * mtiles * 16 + min(mt0 + i, mtiles - 1) * 16 + 4 * kq);
        }
        dst.sw = bs[(size_t)srow * ncb + (128 * kb) / w.bc];
    };
    auto lds_barrier = [] { asm volatile("s_waitcnt lgkmcnt(0)\n\ts_barrier" ::: "memory"); };

    // Software pipeline, three blocks deep in registers. At block
    // i (ring position P = i % 3): the weights of block i + 1 go from registers to the other LDS buffer and their
    // registers take the request for block i + 4; the matrix instructions run on activation set P and LDS buffer
    // i & 1; then set P takes the request for block i + 3.
    WRegs W[3];
    ARegs A[3];
    load_w(W[0], 0);
    read_a(A[0], 0);
    load_w(W[1], 1);
    read_a(A[1], 1);
    load_w(W[2], 2);
    read_a(A[2], 2);
    store_w(W[0], 0);
    load_w(W[0], 3);
    lds_barrier();
    auto block = [&](uint32_t i_kb, auto pos) {
        constexpr int P = decltype(pos)::value, P1 = (P + 1) % 3;
        const uint32_t buf = i_kb & 1;
        store_w(W[P1], buf ^ 1);  // the other buffer was last read a block ago, before the previous barrier
        load_w(W[P1], i_kb + 4);
        float f[F8_TW][4];
#pragma unroll
        for (int i = 0; i < F8_TW; i++)
#pragma unroll
            for (int r = 0; r < 4; r++) f[i][r] = A[P].sx[i][r] * A[P].sw;
        // the matrix instruction of tile pair k + 1 is issued before the four multiply-adds that take tile pair k's
        // result into the accumulators: next to each other they would run one after the other
        f32x4 dprev = {0.0f, 0.0f, 0.0f, 0.0f};
        u32x4 bq[2][2];  // the row tiles' fragments, read from LDS a tile ahead
        auto read_b = [&](int j) {
            const u32x4* bp = reinterpret_cast<const u32x4*>(bfrag + (size_t)(buf * F8_NT + j) * 128 + lane);
            bq[j & 1][0] = bp[0];
            bq[j & 1][1] = bp[64];
        };
        read_b(0);
#pragma unroll
        for (int k = 0; k <= F8_TW * F8_NT; k++) {
            const int j = k / F8_TW, i = k % F8_TW;
            f32x4 d = {0.0f, 0.0f, 0.0f, 0.0f};
            if (k < F8_TW * F8_NT) {
                if (i == 0 && j + 1 < F8_NT) read_b(j + 1);
                const u32x4 b0 = bq[j & 1][0], b1 = bq[j & 1][1];
                const v8i bb = {(int)b0.x, (int)b0.y, (int)b0.z, (int)b0.w, (int)b1.x, (int)b1.y, (int)b1.z, (int)b1.w};
                const u32x4 a0 = A[P].v[i][0], a1 = A[P].v[i][1];
                const v8i aa = {(int)a0.x, (int)a0.y, (int)a0.z, (int)a0.w, (int)a1.x, (int)a1.y, (int)a1.z, (int)a1.w};
                const f32x4 z = {0.0f, 0.0f, 0.0f, 0.0f};
                d = __builtin_amdgcn_mfma_scale_f32_16x16x128_f8f6f4(aa, bb, z, 0, 0, 0, 127, 0, 127);
            }
            if (k > 0) {
                const int jp = (k - 1) / F8_TW, ip = (k - 1) % F8_TW;
#pragma unroll
                for (int r = 0; r < 4; r++) acc[ip][jp][r] = __builtin_fmaf(f[ip][r], dprev[r], acc[ip][jp][r]);
            }
            dprev = d;
        }
        read_a(A[P], i_kb + 3);
        lds_barrier();
    };
    using P0 = std::integral_constant<int, 0>;
    using P1_ = std::integral_constant<int, 1>;
    using P2 = std::integral_constant<int, 2>;
    uint32_t i_kb = 0;
    for (; i_kb + 3 <= nkb; i_kb += 3) {
        block(i_kb, P0{});
        block(i_kb + 1, P1_{});
        block(i_kb + 2, P2{});
    }
    if (i_kb < nkb) block(i_kb, P0{});
    if (i_kb + 1 < nkb) block(i_kb + 1, P1_{});

    if (gridDim.z > 1) yv = reinterpret_cast<float*>(yv) + (size_t)blockIdx.z * t * w.n_out;
#pragma unroll
    for (int i = 0; i < F8_TW; i++) {
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
    span_start(s);
    if (direct_bf16) gemm_fp8_kernel<true><<<grid, 64 * F8_WAVES, lds, s>>>(w, static_cast<const uint4*>(apk), sx, (uint32_t)t, (uint32_t)mtiles, dst);
    else gemm_fp8_kernel<false><<<grid, 64 * F8_WAVES, lds, s>>>(w, static_cast<const uint4*>(apk), sx, (uint32_t)t, (uint32_t)mtiles, dst);
    hipError_t e = hipGetLastError();
    span_stop(s);
    if (e != hipSuccess || slices == 1) return e;
    return launch_gemm_reduce(partial, t * (size_t)w.n_out, slices, y, out_bf16, s);  // (the slices in order, as gemm.hip's)
}

}  // namespace oxhip
