// Prefill GEMM, variant (a): weights dequantized to bf16 on the way to the matrix cores, bf16 MFMA with f32
// accumulation. y[t][n_out] = x[t][n_in] * W^T for the tile-packed MLX 4-bit, Q8_0 / Q8, Q4_K and Q6_K formats (and
// FP8 bytes with block scales).
//
// The CPU computes this product from the f32-dequantized rows with one fused multiply-add chain per output
// (matmul_quant_block_prefill + gemm_8x8, src/kernels.rs:1998-2038, src/kernels_x86.rs:296-324 of the reference);
// here weights and activations are rounded to bf16 first, so results agree to bf16 precision, not bit for bit.
//
// Work split: a workgroup of 8 waves (two per SIMD) owns 256 tokens x 128 weight rows; wave v owns the token tiles v
// and v + 8 of the workgroup's sixteen and all 128 rows (2 x 8 MFMA tiles of 16 x 16, 64 accumulator registers). One
// wave per SIMD issues a matrix instruction about every 30 cycles with this loop's vector, LDS and memory
// instructions between them; a second wave fills the pipe while the first dequantizes, provided the two do not
// dequantize at the same time: the waves 0-3 do so in a step's first block, the waves 4-7 in its second. Sharing the
// token dimension keeps the activation requests at one per fragment and workgroup (sharing the rows instead would
// request every fragment twice and run into the vector memory path's 64 bytes per cycle and CU). A
// launch of at most 64 tokens runs 4 waves with one token tile each (64 tokens x 128 rows per workgroup), one of 65 to
// 128 tokens 8 waves with one tile each (34 -> 27 us on the Llama-8B MLP shapes against two tiles per wave).
//   B (weights): each K-step of 128 the waves dequantize the step's 8 row tiles (one each; two each with 4 waves) from the packed
//     records into bf16 MFMA fragments in LDS (double-buffered, one barrier per step); every wave then reads all
//     8 x 4 fragments with ds_read_b128. A weight is dequantized once per workgroup: (code - 8) * d + offset in
//     f32 as one fma(code, d, offset - 8 d), rounded to bf16. The GGUF formats likewise, from their own records:
//     Q8_0 q * d, Q4_K (d * sc) * nibble - dmin * mn, Q6_K (d * sc) * (code - 32) (dequantize_row, src/ggml.rs:707-793
//     of the reference), each as one fma over the unsigned code.
//   A (activations): packed beforehand (pack_a_kernel) into MFMA fragments, one 1 KiB record per (16 tokens,
//     block of 32) in the K order the weight fragments use, so a wave fetches its fragment with one coalesced
//     16-byte-per-lane load straight from global memory / L2, a block ahead of its use.
#include <type_traits>

#include "internal.hpp"
#include "layout.hpp"

namespace oxhip {

typedef __bf16 bf16x8 __attribute__((ext_vector_type(8)));
typedef float f32x4 __attribute__((ext_vector_type(4)));

// Activations [t][n_in] (f32 or bf16) -> fragments [mtile][block][lane][8 bf16]; lane = 16 kq + m holds token
// 16 mtile + m at K positions 32 b + 4 kq + {0..3} then 32 b + 16 + 4 kq + {0..3} (SPLIT, the order of the
// nibble pairs of Q4 bytes) or 32 b + 8 kq + {0..7}. Tokens past t and columns past n_in are zero.
// MODE 2 (FP8 weights read 32 row bytes per lane): block kb = 4 s + b of step s holds columns 128 s + 32 kq + 8 b + j.
// MODE 3 (Q6_K records: a lane owns 16 consecutive columns of each half step): block kb = 4 s + 2 h + e holds columns
// 128 s + 64 h + 16 kq + 8 e + j.
template <int MODE, bool SRC_BF16>
__global__ __launch_bounds__(256) void pack_a_kernel(const void* __restrict__ x, uint32_t t, uint32_t n_in, uint32_t mtiles,
                                                     uint32_t kblocks, uint4* __restrict__ out) {
    size_t idx = (size_t)blockIdx.x * blockDim.x + threadIdx.x;
    if (idx >= (size_t)mtiles * kblocks * 64) return;
    const uint32_t lane = idx & 63, m = lane & 15, kq = lane >> 4;
    const uint32_t b = (idx >> 6) % kblocks, mt = (idx >> 6) / kblocks;
    const uint32_t tok = mt * 16 + m;
    uint32_t pk[4] = {0, 0, 0, 0};
    if (tok < t) {
        // the lane's 8 values are two runs of 4 consecutive columns (SPLIT) or one run of 8: whole runs are fetched with
        // one 8- or 16-byte request each (rows are multiples of 8 columns here), a ragged tail value by value
        const uint32_t k0 = MODE == 1   ? 32 * b + 4 * kq
                            : MODE == 2 ? 128 * (b >> 2) + 32 * kq + 8 * (b & 3)
                            : MODE == 3 ? 128 * (b >> 2) + 64 * ((b >> 1) & 1) + 16 * kq + 8 * (b & 1)
                                        : 32 * b + 8 * kq;
        const uint32_t k1 = MODE == 1 ? k0 + 16 : k0 + 4;  // first column of the second run of 4
        const size_t row = (size_t)tok * n_in;
        if (k1 + 4 <= n_in && n_in % 8 == 0) {
            if (SRC_BF16) {
                const uint16_t* xs = reinterpret_cast<const uint16_t*>(x) + row;
                const uint2 a = *reinterpret_cast<const uint2*>(xs + k0), c = *reinterpret_cast<const uint2*>(xs + k1);
                pk[0] = a.x;
                pk[1] = a.y;
                pk[2] = c.x;
                pk[3] = c.y;
            } else {
                const float* xs = reinterpret_cast<const float*>(x) + row;
                const float4 a = *reinterpret_cast<const float4*>(xs + k0), c = *reinterpret_cast<const float4*>(xs + k1);
                pk[0] = f32_to_bf16_bits(a.x) | ((uint32_t)f32_to_bf16_bits(a.y) << 16);
                pk[1] = f32_to_bf16_bits(a.z) | ((uint32_t)f32_to_bf16_bits(a.w) << 16);
                pk[2] = f32_to_bf16_bits(c.x) | ((uint32_t)f32_to_bf16_bits(c.y) << 16);
                pk[3] = f32_to_bf16_bits(c.z) | ((uint32_t)f32_to_bf16_bits(c.w) << 16);
            }
        } else {
#pragma unroll
            for (int j = 0; j < 8; j++) {
                const uint32_t k = (j < 4 ? k0 : k1 - 4) + j;
                uint16_t h = 0;
                if (k < n_in) {
                    if (SRC_BF16) h = reinterpret_cast<const uint16_t*>(x)[row + k];
                    else h = f32_to_bf16_bits(reinterpret_cast<const float*>(x)[row + k]);
                }
                pk[j >> 1] |= (uint32_t)h << (16 * (j & 1));
            }
        }
    }
    out[idx] = make_uint4(pk[0], pk[1], pk[2], pk[3]);
}

hipError_t launch_pack_a(const void* x, bool src_bf16, int mode, size_t t, size_t n_in, size_t mtiles, size_t kblocks, void* out,
                         hipStream_t s) {
    size_t total = mtiles * kblocks * 64;
    if (!total) return hipSuccess;
    unsigned grid = (unsigned)((total + 255) / 256);
    uint4* o = static_cast<uint4*>(out);
    const uint32_t tt = (uint32_t)t, kk = (uint32_t)n_in, mt = (uint32_t)mtiles, kb = (uint32_t)kblocks;
    if (mode == 1) {
        if (src_bf16) pack_a_kernel<1, true><<<grid, 256, 0, s>>>(x, tt, kk, mt, kb, o);
        else pack_a_kernel<1, false><<<grid, 256, 0, s>>>(x, tt, kk, mt, kb, o);
    } else if (mode == 2) {
        if (src_bf16) pack_a_kernel<2, true><<<grid, 256, 0, s>>>(x, tt, kk, mt, kb, o);
        else pack_a_kernel<2, false><<<grid, 256, 0, s>>>(x, tt, kk, mt, kb, o);
    } else if (mode == 3) {
        if (src_bf16) pack_a_kernel<3, true><<<grid, 256, 0, s>>>(x, tt, kk, mt, kb, o);
        else pack_a_kernel<3, false><<<grid, 256, 0, s>>>(x, tt, kk, mt, kb, o);
    } else {
        if (src_bf16) pack_a_kernel<0, true><<<grid, 256, 0, s>>>(x, tt, kk, mt, kb, o);
        else pack_a_kernel<0, false><<<grid, 256, 0, s>>>(x, tt, kk, mt, kb, o);
    }
    return hipGetLastError();
}

#ifndef OXHIP_GEMM_EARLY_RAW
#define OXHIP_GEMM_EARLY_RAW 1
#endif

namespace {

// the formats in the T4M code geometry (NVFP4's records too: float-stored, so not one of the int8 decode formats)
__host__ __device__ constexpr bool t4_geometry(int f) { return t4m_format(f) || f == FMT_NVFP4; }

typedef uint32_t u32x4g __attribute__((ext_vector_type(4)));
constexpr int WG_NT = 8;   // row tiles per workgroup (128 rows), or 7 where that fills more CUs (gemm_row_tiles)
constexpr int AR = 4;      // blocks of A fragments held ahead (a whole K-step: two starve the FP8 shapes, whose activations do not stay in L2)

typedef __bf16 bf16x2 __attribute__((ext_vector_type(2)));
typedef float f32x2 __attribute__((ext_vector_type(2)));
// Two f32 -> packed bf16 (round to nearest even) with the hardware conversion, one instruction, no branches.
__device__ __forceinline__ uint32_t pack_bf16(float a, float b) {
    return __builtin_bit_cast(uint32_t, __builtin_convertvector(f32x2{a, b}, bf16x2));
}

// Eight unsigned byte codes (the bytes of lo, then of hi) -> 8 bf16 of code * d + c.
template <int K>
__device__ __forceinline__ float byte_f32(uint32_t x) {  // byte K of x as f32: one conversion that selects the byte itself
    float f;
    if constexpr (K == 0) asm("v_cvt_f32_ubyte0_e32 %0, %1" : "=v"(f) : "v"(x));
    else if constexpr (K == 1) asm("v_cvt_f32_ubyte1_e32 %0, %1" : "=v"(f) : "v"(x));
    else if constexpr (K == 2) asm("v_cvt_f32_ubyte2_e32 %0, %1" : "=v"(f) : "v"(x));
    else asm("v_cvt_f32_ubyte3_e32 %0, %1" : "=v"(f) : "v"(x));
    return f;
}
__device__ __forceinline__ uint4 dequant_u8x8(uint32_t lo, uint32_t hi, float d, float c) {
    float f[8];
    f[0] = __builtin_fmaf(byte_f32<0>(lo), d, c);
    f[1] = __builtin_fmaf(byte_f32<1>(lo), d, c);
    f[2] = __builtin_fmaf(byte_f32<2>(lo), d, c);
    f[3] = __builtin_fmaf(byte_f32<3>(lo), d, c);
    f[4] = __builtin_fmaf(byte_f32<0>(hi), d, c);
    f[5] = __builtin_fmaf(byte_f32<1>(hi), d, c);
    f[6] = __builtin_fmaf(byte_f32<2>(hi), d, c);
    f[7] = __builtin_fmaf(byte_f32<3>(hi), d, c);
    return make_uint4(pack_bf16(f[0], f[1]), pack_bf16(f[2], f[3]), pack_bf16(f[4], f[5]), pack_bf16(f[6], f[7]));
}
// One dword of a T4M chunk (4 bytes of one block: low nibbles = elements 4 kq + i, high = 16 + 4 kq + i) -> the
// lane's 8 bf16 of that block.
__device__ __forceinline__ uint4 dequant_q4m(uint32_t w, float d, float c) {
    return dequant_u8x8(w & 0x0F0F0F0Fu, (w >> 4) & 0x0F0F0F0Fu, d, c);
}

}  // namespace

// grid: (row groups of 128, token groups of 256). apk: packed activations [mtiles][kblocks][64][16 B] with
// kblocks = 4 * steps. OUT_BF16: y is bf16 [t][n_out], else f32.
// With gridDim.z > 1 the K-steps are split over z and each slice writes its partial sums as f32 to
// yv + z * t * n_out (a second kernel adds the slices in order).
// FMT: FMT_Q4M (tile-packed MLX 4-bit), FMT_Q8_0 / FMT_Q8F / FMT_Q4_K / FMT_Q6_K (their tile records) or FMT_FP8 (e4m3 bytes with 128 x 128 block scales: the bytes are
// exact in bf16, the block scale multiplies in f32 before the rounding, and a lane takes 32 consecutive row bytes
// per step, which pack_a's mode 2 mirrors on the activation side).
template <int FMT, bool OUT_BF16, int NV, int WAVES, int NT>
__global__ __launch_bounds__(64 * WAVES) void gemm_bf16_kernel(WeightView w, const uint4* __restrict__ apk, uint32_t t, uint32_t mtiles,
                                                        void* __restrict__ yv) {
    extern __shared__ uint4 bfrag[];  // [2][4 blocks][NT row tiles][64 lanes]
    const uint32_t lane = threadIdx.x & 63, wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
    const uint32_t n = lane & 15;
    constexpr int DT = (NT + WAVES - 1) / WAVES;  // row tiles a wave dequantizes (with NT = 7 the last wave has one fewer)
    const uint32_t all_steps = (w.n_in + 127) / 128, kblocks = 4 * all_steps;  // == t4m_steps(n_in)
    const uint32_t per_z = (all_steps + gridDim.z - 1) / gridDim.z;
    const uint32_t step0 = blockIdx.z * per_z;              // this slice's K-steps: step0 .. step0 + nsteps
    const uint32_t nsteps = min(all_steps, step0 + per_z) - step0;
    const uint32_t ntiles = row_tiles(w.n_out);
    const uint32_t nt0 = blockIdx.x * NT;               // first row tile of the workgroup
    // the wave's token tiles: mt0, mt0 + WAVES, ... (NV of them: 2, or 1 when the whole launch has at most 64 tokens per
    // workgroup row, so that a few tokens do not pay for 256)
    const uint32_t mt0 = blockIdx.y * (WAVES * NV) + wave;

    // the row tiles this wave dequantizes
    const uint8_t* wbase[2];
    const float* sbase[2] = {nullptr, nullptr};  // FP8: the block scales of the tile's rows
#pragma unroll
    for (int i = 0; i < DT; i++) {
        const uint32_t tile = min(nt0 + DT * wave + i, ntiles - 1);
        if (t4_geometry(FMT)) {
            wbase[i] = w.p0 + ((size_t)tile * all_steps + step0) * (FMT == FMT_MXFP4 ? T4X_REC : T4M_REC);  // (T4N_REC == T4M_REC)
        } else if (q8_format(FMT)) {  // the tile's records; load_raw indexes them from the matrix's first step
            wbase[i] = w.p0 + (size_t)tile * t8_steps(w.n_in) * (FMT == FMT_Q8F ? T8F_REC : T8_REC);
        } else if (k45_format(FMT)) {
            wbase[i] = w.p0 + (size_t)tile * tk4_sbs(w.n_in) * (FMT == FMT_Q5_K ? TK5_REC : TK4_REC);
        } else if (FMT == FMT_Q6_K) {
            wbase[i] = w.p0 + (size_t)tile * t6k_steps(w.n_in) * T6K_REC;
        } else {
            const uint32_t row = min(tile * 16 + n, w.n_out - 1);
            wbase[i] = w.p0 + fp8_offset(w, row, 128 * (size_t)step0 + 32 * (lane >> 4));
            sbase[i] = reinterpret_cast<const float*>(w.p1) + (size_t)(tile * 16 / w.br) * ((w.n_in + w.bc - 1) / w.bc);  // indexed by the absolute column block
        }
    }
    // A fragments of the wave's token tiles (tiles past the end repeat the last one; their rows are not stored)
    const uint4* abase[NV];
#pragma unroll
    for (int i = 0; i < NV; i++) abase[i] = apk + ((size_t)min(mt0 + WAVES * i, mtiles - 1) * kblocks + 4 * step0) * 64;  // (the same in every lane)

    f32x4 acc[NV][NT];
#pragma unroll
    for (int i = 0; i < NV; i++)
#pragma unroll
        for (int j = 0; j < NT; j++) acc[i][j] = f32x4{0.0f, 0.0f, 0.0f, 0.0f};

    struct Raw {
        uint4 c, c2;    // Q4M, Q4_K: one chunk; Q8: the chunks of the step's two records; Q6_K: low nibbles, high bit pairs; FP8: 32 row bytes
        uint32_t m[4];  // the row's scale words (Q4M: scales, offsets; FP8: the block scale's bits)
    };
    auto load_raw_tile = [&](Raw* r, int i, uint32_t s) {  // the records of the wave's row tile i at step s
        if (NT % WAVES == 0 || DT * wave + i < NT) {  // (with NT = 7 the eighth wave has no tile)
            if (FMT == FMT_NVFP4) {  // the row's eight sub-block scale bytes, and the matrix's scale of this step's columns
                const uint8_t* rec = wbase[i] + (size_t)s * T4N_REC;
                r[i].c = *reinterpret_cast<const uint4*>(rec + 16 * lane);
                const uint2 sv = *reinterpret_cast<const uint2*>(rec + 1024 + 8 * n);
                r[i].m[0] = sv.x;
                r[i].m[1] = sv.y;
                const uint32_t tile = min(nt0 + DT * wave + i, ntiles - 1);
                r[i].m[2] = w.br ? __float_as_uint(reinterpret_cast<const float*>(w.p1)[(size_t)(min(tile * 16 + n, w.n_out - 1) / w.br) * ((w.n_in + w.bc - 1) / w.bc) +
                                                                                    (128 * (step0 + s)) / w.bc])
                                 : 0x3F800000u;
            } else if (t4m_format(FMT)) {
                const uint8_t* rec = wbase[i] + (size_t)s * (FMT == FMT_MXFP4 ? T4X_REC : T4M_REC);
                r[i].c = *reinterpret_cast<const uint4*>(rec + 16 * lane);
                r[i].m[0] = *reinterpret_cast<const uint32_t*>(rec + 1024 + 4 * n);
                if (FMT != FMT_MXFP4) r[i].m[1] = *reinterpret_cast<const uint32_t*>(rec + 1088 + 4 * n);
            } else if (q8_format(FMT)) {  // a step of 128 columns is two records of 64 (past the row's last record: that one again,
                                          // which dequant_tile zeroes: nothing here may depend on a loaded value, or the request
                                          // would be waited for where it is made)
                constexpr uint32_t REC = FMT == FMT_Q8F ? T8F_REC : T8_REC;
                const uint32_t nrec = t8_steps(w.n_in);
#pragma unroll
                for (int h = 0; h < 2; h++) {
                    const uint8_t* rec = wbase[i] + (size_t)min(2 * (step0 + s) + h, nrec - 1) * REC;
                    const uint4 v = *reinterpret_cast<const uint4*>(rec + 16 * lane);
                    if (h) r[i].c2 = v;
                    else r[i].c = v;
                    if (FMT == FMT_Q8F) {
                        const uint2 sc = *reinterpret_cast<const uint2*>(rec + 1024 + 8 * n);
                        r[i].m[2 * h] = sc.x;
                        r[i].m[2 * h + 1] = sc.y;
                    } else {
                        r[i].m[h] = *reinterpret_cast<const uint32_t*>(rec + 1024 + 4 * n);
                    }
                }
            } else if (k45_format(FMT)) {  // half a super-block record: sub-blocks 4 (sa & 1) .. + 3
                const uint32_t sa = step0 + s;
                const uint8_t* rec = wbase[i] + (size_t)(sa >> 1) * (FMT == FMT_Q5_K ? TK5_REC : TK4_REC);
                r[i].c = *reinterpret_cast<const uint4*>(rec + (sa & 1) * 1024 + 16 * lane);
                if (FMT == FMT_Q5_K) r[i].c2.x = *reinterpret_cast<const uint32_t*>(rec + TK4_REC + (sa & 1) * 256 + 4 * lane);
                r[i].m[0] = *reinterpret_cast<const uint32_t*>(rec + 2048 + 16 * n + 4 * (sa & 1));
                r[i].m[1] = *reinterpret_cast<const uint32_t*>(rec + 2048 + 16 * n + 8 + 4 * (sa & 1));
                r[i].m[2] = *reinterpret_cast<const uint32_t*>(rec + 2304 + 4 * n);
            } else if (FMT == FMT_Q6_K) {
                const uint8_t* rec = wbase[i] + (size_t)(step0 + s) * T6K_REC;
                r[i].c = *reinterpret_cast<const uint4*>(rec + 16 * lane);
                const uint2 hb = *reinterpret_cast<const uint2*>(rec + 1024 + 8 * lane);
                r[i].c2.x = hb.x;
                r[i].c2.y = hb.y;
                const uint2 sc = *reinterpret_cast<const uint2*>(rec + 1536 + 8 * n);
                r[i].m[0] = sc.x;
                r[i].m[1] = sc.y;
                r[i].m[2] = *reinterpret_cast<const uint16_t*>(rec + 1664 + 2 * n);
            } else {
                const uint8_t* p = wbase[i] + (w.group == 1 ? 2048 : 128) * (size_t)s;
                r[i].c = *reinterpret_cast<const uint4*>(p);
                r[i].c2 = *reinterpret_cast<const uint4*>(p + fp8_second_chunk(w));
                r[i].m[0] = __float_as_uint(sbase[i][(128 * (step0 + s)) / w.bc]);
            }
        }
    };
    auto load_raw = [&](Raw* r, uint32_t s) {
        load_raw_tile(r, 0, s);
        if (DT == 2) load_raw_tile(r, 1, s);
    };
    // `s`: the step the records belong to (of this slice)
    auto dequant_tile = [&](const Raw& r, int i, uint32_t buf, uint32_t s) {  // one of the wave's row tiles, 4 blocks
        if (NT % WAVES != 0 && DT * wave + i >= NT) return;
        uint4* dst = bfrag + ((size_t)(buf * 4) * NT + DT * wave + i) * 64 + lane;  // block b: + b * NT * 64
        if (FMT == FMT_NVFP4) {  // as MXFP4 below with a scale per 16: the low nibbles' sub-block 2 b, the high nibbles' 2 b + 1
            const uint32_t cw[4] = {r.c.x, r.c.y, r.c.z, r.c.w};
            const float g = __uint_as_float(r.m[2]);
#pragma unroll
            for (int b = 0; b < 4; b++) {
                const uint32_t sw = r.m[b >> 1] >> (16 * (b & 1));
                const float d0 = ue4m3_half(sw) * g, d1 = ue4m3_half(sw >> 8) * g;
                const uint32_t lo = mxfp4_values<12>(cw[b] & 0x0F0F0F0Fu), hi = mxfp4_values<12>((cw[b] >> 4) & 0x0F0F0F0Fu);
                const float c0 = -12.0f * d0, c1 = -12.0f * d1;
                dst[b * NT * 64] = make_uint4(pack_bf16(__builtin_fmaf(byte_f32<0>(lo), d0, c0), __builtin_fmaf(byte_f32<1>(lo), d0, c0)),
                                              pack_bf16(__builtin_fmaf(byte_f32<2>(lo), d0, c0), __builtin_fmaf(byte_f32<3>(lo), d0, c0)),
                                              pack_bf16(__builtin_fmaf(byte_f32<0>(hi), d1, c1), __builtin_fmaf(byte_f32<1>(hi), d1, c1)),
                                              pack_bf16(__builtin_fmaf(byte_f32<2>(hi), d1, c1), __builtin_fmaf(byte_f32<3>(hi), d1, c1)));
            }
        } else if (FMT == FMT_MXFP4) {  // the code's doubled value + 12 as an unsigned byte, times the block's power of two: exact in bf16
            const uint32_t cw[4] = {r.c.x, r.c.y, r.c.z, r.c.w};
#pragma unroll
            for (int b = 0; b < 4; b++) {
                const float d = e8m0_half((r.m[0] >> (8 * b)) & 0xFF);
                dst[b * NT * 64] = dequant_u8x8(mxfp4_values<12>(cw[b] & 0x0F0F0F0Fu), mxfp4_values<12>((cw[b] >> 4) & 0x0F0F0F0Fu), d, -12.0f * d);
            }
        } else if (FMT == FMT_Q40) {  // the block's own scale: word b / 2, half b % 2; (nib - 8) * d
            const uint32_t cw[4] = {r.c.x, r.c.y, r.c.z, r.c.w};
#pragma unroll
            for (int b = 0; b < 4; b++) {
                const float d = f16_bits_to_f32((uint16_t)((b & 1) ? r.m[b >> 1] >> 16 : r.m[b >> 1] & 0xFFFF));
                dst[b * NT * 64] = dequant_q4m(cw[b], d, -8.0f * d);
            }
        } else if (FMT == FMT_Q4M) {
            const uint32_t cw[4] = {r.c.x, r.c.y, r.c.z, r.c.w};
#pragma unroll
            for (int b = 0; b < 4; b++) {
                const int g = b >> 1;
                const float d = f16_bits_to_f32((uint16_t)(g ? r.m[0] >> 16 : r.m[0] & 0xFFFF));
                const float off = bf16_bits_to_f32((uint16_t)(g ? r.m[1] >> 16 : r.m[1] & 0xFFFF));
                dst[b * NT * 64] = dequant_q4m(cw[b], d, off - 8.0f * d);
            }
        } else if (q8_format(FMT)) {  // block b = 2 h + e: codes 8 kq .. + 7 of block e of record h; q * d as (q + 128) * d - 128 d
            const uint32_t cw[8] = {r.c.x, r.c.y, r.c.z, r.c.w, r.c2.x, r.c2.y, r.c2.z, r.c2.w};
            const bool past = 2 * (step0 + s) + 1 >= t8_steps(w.n_in);  // the step's second record lies past the row
#pragma unroll
            for (int b = 0; b < 4; b++) {
                const int h = b >> 1, e = b & 1;
                float d = FMT == FMT_Q8F ? __uint_as_float(r.m[b]) : f16_bits_to_f32((uint16_t)(e ? r.m[h] >> 16 : r.m[h] & 0xFFFF));
                if (h && past) d = 0.0f;
                dst[b * NT * 64] = dequant_u8x8(cw[2 * b] ^ 0x80808080u, cw[2 * b + 1] ^ 0x80808080u, d, -128.0f * d);
            }
        } else if (k45_format(FMT)) {  // block b = 2 jj + e: the low (e = 0) or high nibbles of the chunk's byte pair jj
            const float d = f16_bits_to_f32((uint16_t)(r.m[2] & 0xFFFF)), dmin = f16_bits_to_f32((uint16_t)(r.m[2] >> 16));
#pragma unroll
            for (int b = 0; b < 4; b++) {
                const int jj = b >> 1, e = b & 1;
                const uint32_t lo = jj ? r.c.z : r.c.x, hi = jj ? r.c.w : r.c.y;
                const float sc = (float)((r.m[0] >> (8 * b)) & 0xFF), mn = (float)((r.m[1] >> (8 * b)) & 0xFF);
                uint32_t w0 = (lo >> (4 * e)) & 0x0F0F0F0Fu, w1 = (hi >> (4 * e)) & 0x0F0F0F0Fu;
                if (FMT == FMT_Q5_K) {  // the fifth bits of the block's two dwords: bits 8 k + 2 b and 8 k + 2 b + 1 of the plane
                    w0 |= ((r.c2.x >> (2 * b)) & 0x01010101u) << 4;
                    w1 |= ((r.c2.x >> (2 * b + 1)) & 0x01010101u) << 4;
                }
                dst[b * NT * 64] = dequant_u8x8(w0, w1, d * sc, -(dmin * mn));
            }
        } else if (FMT == FMT_Q6_K) {  // block b = 2 h + e: codes 8 e .. + 7 of the lane's 16 columns of half h
            const float d = f16_bits_to_f32((uint16_t)(r.m[2] & 0xFFFF));
            const uint32_t kq = lane >> 4;
#pragma unroll
            for (int b = 0; b < 4; b++) {
                const int h = b >> 1, e = b & 1;
                const uint32_t src = e ? (h ? r.c.w : r.c.y) : (h ? r.c.z : r.c.x), hh = (h ? r.c2.y : r.c2.x) >> (4 * e);
                const uint32_t w0 = (src & 0x0F0F0F0Fu) | ((hh & 0x03030303u) << 4);
                const uint32_t w1 = ((src >> 4) & 0x0F0F0F0Fu) | (((hh >> 2) & 0x03030303u) << 4);
                const float dsc = d * (float)(int)(int8_t)((r.m[h] >> (8 * kq)) & 0xFF);
                dst[b * NT * 64] = dequant_u8x8(w0, w1, dsc, -32.0f * dsc);
            }
        } else {
            const uint32_t cw[8] = {r.c.x, r.c.y, r.c.z, r.c.w, r.c2.x, r.c2.y, r.c2.z, r.c2.w};
            const float sc = __uint_as_float(r.m[0]);
#pragma unroll
            for (int b = 0; b < 4; b++) {  // bytes 8 b .. 8 b + 7 of the lane's 32
                const f32x2 v0 = __builtin_amdgcn_cvt_pk_f32_fp8((int)cw[2 * b], false);
                const f32x2 v1 = __builtin_amdgcn_cvt_pk_f32_fp8((int)cw[2 * b], true);
                const f32x2 v2 = __builtin_amdgcn_cvt_pk_f32_fp8((int)cw[2 * b + 1], false);
                const f32x2 v3 = __builtin_amdgcn_cvt_pk_f32_fp8((int)cw[2 * b + 1], true);
                const uint32_t o[4] = {pack_bf16(v0.x * sc, v0.y * sc), pack_bf16(v1.x * sc, v1.y * sc),
                                       pack_bf16(v2.x * sc, v2.y * sc), pack_bf16(v3.x * sc, v3.y * sc)};
                dst[b * NT * 64] = make_uint4(o[0], o[1], o[2], o[3]);
            }
        }
    };
    auto read_b = [&](uint4* dst, uint32_t buf, uint32_t b) {
#pragma unroll
        for (int j = 0; j < NT; j++) dst[j] = bfrag[((buf * 4 + b) * NT + j) * 64 + lane];
    };
    auto read_a = [&](uint4* dst, uint32_t blk) {  // the A fragments of block `blk` of this slice
#pragma unroll
        for (int i = 0; i < NV; i++) {
            // the block's base is the same in every lane: kept in scalar registers, the request takes it with the lane's 32-bit offset
            const uint64_t pa = reinterpret_cast<uint64_t>(abase[i] + (size_t)blk * 64);
            const uint32_t lo = __builtin_amdgcn_readfirstlane((uint32_t)pa), hi = __builtin_amdgcn_readfirstlane((uint32_t)(pa >> 32));
            dst[i] = __builtin_bit_cast(uint4, reinterpret_cast<const __attribute__((address_space(1))) u32x4g*>(((uint64_t)hi << 32) | lo)[lane]);
        }
    };
    // LDS traffic only: outstanding global loads (the prefetches) stay in flight across the barrier
    auto lds_barrier = [] { asm volatile("s_waitcnt lgkmcnt(0)\n\ts_barrier" ::: "memory"); };

    // B fragments are read from LDS one block ahead of the MFMAs that consume them; A fragments come from global
    // memory a whole K-step (four blocks, ~2000 MFMA cycles) ahead; the packed records of the next step two blocks
    // before they are dequantized into the other LDS buffer. Each fragment has one home, refilled in place right after
    // its last use.
    constexpr bool EARLY_RAW = OXHIP_GEMM_EARLY_RAW;
    Raw raw[DT];
    load_raw(raw, 0);
    uint4 a_cur[AR][NV], b_cur[NT];
    const uint32_t last = nsteps - 1, last_blk = 4 * nsteps - 1;
#pragma unroll
    for (int b = 0; b < AR; b++) read_a(a_cur[b], min((uint32_t)b, last_blk));
    dequant_tile(raw[0], 0, 0, 0);
    if (DT == 2) dequant_tile(raw[DT - 1], 1, 0, 0);
    load_raw(raw, min(1u, last));
    lds_barrier();
    read_b(b_cur, 0, 0);
    // One K-step; every step does the same work, so that the loop is one body whose accumulators stay in place: the
    // records of the next step are dequantized into the other LDS buffer during blocks 0 and 1 (with 8 waves: block 0
    // by the waves 0-3, block 1 by the waves 4-7, which share their SIMDs with them), block 3 refills from
    // that buffer after the barrier, and the step after next is requested during block 2. Past the end the indices
    // repeat the last step: a little work that nobody reads, instead of separate loop tails.
    for (uint32_t s = 0; s < nsteps; s++) {
        const uint32_t buf = s & 1;
#pragma unroll
        for (int b = 0; b < 4; b++) {
            if (b == 3) lds_barrier();  // the other buffer is complete, and nobody still reads this one
#pragma unroll
            for (int j = 0; j < NT; j++) {
                const bf16x8 bb = __builtin_bit_cast(bf16x8, b_cur[j]);
#pragma unroll
                for (int i = 0; i < NV; i++)
                    acc[i][j] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(__builtin_bit_cast(bf16x8, a_cur[b % AR][i]), bb, acc[i][j], 0, 0, 0);
                if (b < 3) b_cur[j] = bfrag[((buf * 4 + b + 1) * NT + j) * 64 + lane];
                else b_cur[j] = bfrag[(((buf ^ 1) * 4) * NT + j) * 64 + lane];
            }
            read_a(a_cur[b % AR], min(4 * s + b + AR, last_blk));
            if (DT == 1) {
                if (b == (int)(wave >> 2)) {
                    dequant_tile(raw[0], 0, buf ^ 1, min(s + 1, last));
                    load_raw_tile(raw, 0, min(s + 2, last));
                }
            } else if (EARLY_RAW) {  // a tile's records of the step after next are requested as soon as its registers are free
                if (b < 2) {
                    dequant_tile(raw[b < DT ? b : 0], b, buf ^ 1, min(s + 1, last));
                    load_raw_tile(raw, b, min(s + 2, last));
                }
            } else {
                if (b == 0) dequant_tile(raw[0], 0, buf ^ 1, min(s + 1, last));
                if (b == 1) dequant_tile(raw[DT - 1], 1, buf ^ 1, min(s + 1, last));
                if (b == 2) load_raw(raw, min(s + 2, last));
            }
        }
    }
    // D[token 4 kq + r][row n] per tile
    const uint32_t kq = lane >> 4;
    if (gridDim.z > 1) yv = reinterpret_cast<float*>(yv) + (size_t)blockIdx.z * t * w.n_out;
#pragma unroll
    for (int i = 0; i < NV; i++) {
#pragma unroll
        for (int j = 0; j < NT; j++) {
            const uint32_t row = (nt0 + j) * 16 + n;
#pragma unroll
            for (int r = 0; r < 4; r++) {
                const uint32_t tok = (mt0 + WAVES * i) * 16 + 4 * kq + r;
                if (tok < t && row < w.n_out && mt0 + WAVES * i < mtiles) {
                    if (OUT_BF16) reinterpret_cast<uint16_t*>(yv)[(size_t)tok * w.n_out + row] = f32_to_bf16_bits(acc[i][j][r]);
                    else reinterpret_cast<float*>(yv)[(size_t)tok * w.n_out + row] = acc[i][j][r];
                }
            }
        }
    }
}

// Adds the K slices in order: y = p[0] + p[1] + ... (f32 or bf16 out). VEC outputs per thread (4 when n is a multiple of 4 and
// the buffers are 16-byte aligned).
template <bool OUT_BF16, int VEC>
__global__ __launch_bounds__(256) void gemm_reduce_kernel(const float* __restrict__ p, size_t n, uint32_t slices, void* __restrict__ yv) {
    const size_t i = ((size_t)blockIdx.x * blockDim.x + threadIdx.x) * VEC;
    if (i >= n) return;
    float v[VEC];
    if (VEC == 4) {
        const float4 a = *reinterpret_cast<const float4*>(p + i);
        v[0] = a.x; v[1 % VEC] = a.y; v[2 % VEC] = a.z; v[3 % VEC] = a.w;
        for (uint32_t z = 1; z < slices; z++) {
            const float4 b = *reinterpret_cast<const float4*>(p + (size_t)z * n + i);
            v[0] += b.x; v[1 % VEC] += b.y; v[2 % VEC] += b.z; v[3 % VEC] += b.w;
        }
        if (OUT_BF16) {
            *reinterpret_cast<uint2*>(reinterpret_cast<uint16_t*>(yv) + i) =
                make_uint2(f32_to_bf16_bits(v[0]) | ((uint32_t)f32_to_bf16_bits(v[1 % VEC]) << 16),
                           f32_to_bf16_bits(v[2 % VEC]) | ((uint32_t)f32_to_bf16_bits(v[3 % VEC]) << 16));
        } else {
            *reinterpret_cast<float4*>(reinterpret_cast<float*>(yv) + i) = make_float4(v[0], v[1 % VEC], v[2 % VEC], v[3 % VEC]);
        }
    } else {
        v[0] = p[i];
        for (uint32_t z = 1; z < slices; z++) v[0] += p[(size_t)z * n + i];
        if (OUT_BF16) reinterpret_cast<uint16_t*>(yv)[i] = f32_to_bf16_bits(v[0]);
        else reinterpret_cast<float*>(yv)[i] = v[0];
    }
}

static void run_gemm_reduce(const float* partial, size_t n, uint32_t slices, void* y, bool out_bf16, hipStream_t s) {
    const bool wide = n % 4 == 0 && reinterpret_cast<uintptr_t>(partial) % 16 == 0 && reinterpret_cast<uintptr_t>(y) % 16 == 0;
    if (wide) {
        const unsigned grid = (unsigned)((n / 4 + 255) / 256);
        if (out_bf16) gemm_reduce_kernel<true, 4><<<grid, 256, 0, s>>>(partial, n, slices, y);
        else gemm_reduce_kernel<false, 4><<<grid, 256, 0, s>>>(partial, n, slices, y);
    } else {
        const unsigned grid = (unsigned)((n + 255) / 256);
        if (out_bf16) gemm_reduce_kernel<true, 1><<<grid, 256, 0, s>>>(partial, n, slices, y);
        else gemm_reduce_kernel<false, 1><<<grid, 256, 0, s>>>(partial, n, slices, y);
    }
}

// K slices for a launch: enough workgroups to cover the CUs while each keeps at least 8 steps.
// Token tiles per wave and waves per workgroup: one tile and four waves when the launch has at most four tiles (64 tokens),
// one tile and eight waves up to eight tiles (128 tokens), else two tiles and eight waves.
static int gemm_nv(size_t mtiles) { return mtiles <= 8 ? 1 : 2; }
static int gemm_waves(size_t mtiles) { return mtiles <= 4 ? 4 : 8; }  // (5 to 8 token tiles: eight waves of one tile each)

static uint32_t k_slices_for(const WeightView& w, size_t mtiles, uint32_t nt) {
    const uint32_t per_wg = gemm_waves(mtiles) * gemm_nv(mtiles);
    const uint32_t wgs = ((row_tiles(w.n_out) + nt - 1) / nt) * (uint32_t)((mtiles + per_wg - 1) / per_wg);
    const uint32_t steps = (w.n_in + 127) / 128;
    uint32_t z = 1;
    // (one token tile per wave: a K-step is short, two workgroups fit a CU, and what counts is requests in flight)
    const uint32_t places = gemm_nv(mtiles) == 1 ? 512 : 256, min_steps = gemm_nv(mtiles) == 1 ? 4 : 8;
    while (z < 8 && wgs * z * 2 <= places && steps / (z * 2) >= min_steps) {
        // every slice must own a step: the kernel gives slice i the steps from i * ceil(steps / z) (33 steps in 8 slices
        // of 5 would start the last one past the end)
        const uint32_t z2 = z * 2, per = (steps + z2 - 1) / z2;
        if ((z2 - 1) * per >= steps) break;
        z = z2;
    }
    return z;
}

// Row tiles per workgroup: 8, or 7 where that costs less by this count: rounds of workgroups over the 256 CUs x row tiles
// per workgroup x K-steps per slice (14336 rows x 512 tokens: one round of 256 workgroups of 112 rows instead of 224 of 128,
// 63 -> 60 us; x 1024 tokens: two full rounds of 256 instead of 256 + 192).
static int gemm_row_tiles(const WeightView& w, size_t mtiles) {
    if (gemm_nv(mtiles) == 1) return WG_NT;
    const uint32_t per_wg = gemm_waves(mtiles) * gemm_nv(mtiles), cols = (uint32_t)((mtiles + per_wg - 1) / per_wg);
    const uint32_t steps = (w.n_in + 127) / 128;
    auto cost = [&](uint32_t nt) {
        const uint32_t z = k_slices_for(w, mtiles, nt), wgs = ((row_tiles(w.n_out) + nt - 1) / nt) * cols * z;
        return (uint64_t)((wgs + 255) / 256) * nt * ((steps + z - 1) / z);
    };
    return cost(7) < cost(8) ? 7 : WG_NT;
}

uint32_t gemm_k_slices(const WeightView& w, size_t mtiles) { return k_slices_for(w, mtiles, (uint32_t)gemm_row_tiles(w, mtiles)); }

namespace {
template <int FMT, int NV, int NT, int WAVES = (NV == 1 ? 4 : 8)>
hipError_t run_gemm_bf16_nv(const WeightView& w, const void* apk, size_t t, size_t mtiles, void* y, bool out_bf16, float* partial,
                         hipStream_t s) {
    const uint32_t slices = gemm_k_slices(w, mtiles);
    dim3 grid((row_tiles(w.n_out) + NT - 1) / NT, (unsigned)((mtiles + WAVES * NV - 1) / (WAVES * NV)), slices);
    const size_t lds = 2 * 4 * NT * 64 * 16;  // 64 KiB with 8 row tiles
    const bool direct_bf16 = out_bf16 && slices == 1;
    void* dst = slices > 1 ? static_cast<void*>(partial) : y;
    hipError_t e;
    span_start(s);
    if (direct_bf16) {
        e = hipFuncSetAttribute(reinterpret_cast<const void*>(gemm_bf16_kernel<FMT, true, NV, WAVES, NT>), hipFuncAttributeMaxDynamicSharedMemorySize, (int)lds);
        if (e != hipSuccess) return e;
        gemm_bf16_kernel<FMT, true, NV, WAVES, NT><<<grid, 64 * WAVES, lds, s>>>(w, static_cast<const uint4*>(apk), (uint32_t)t, (uint32_t)mtiles, dst);
    } else {
        e = hipFuncSetAttribute(reinterpret_cast<const void*>(gemm_bf16_kernel<FMT, false, NV, WAVES, NT>), hipFuncAttributeMaxDynamicSharedMemorySize, (int)lds);
        if (e != hipSuccess) return e;
        gemm_bf16_kernel<FMT, false, NV, WAVES, NT><<<grid, 64 * WAVES, lds, s>>>(w, static_cast<const uint4*>(apk), (uint32_t)t, (uint32_t)mtiles, dst);
    }
    e = hipGetLastError();
    span_stop(s);
    if (e != hipSuccess || slices == 1) return e;
    run_gemm_reduce(partial, t * (size_t)w.n_out, slices, y, out_bf16, s);
    return hipGetLastError();
}
template <int FMT>
hipError_t run_gemm_bf16(const WeightView& w, const void* apk, size_t t, size_t mtiles, void* y, bool out_bf16, float* partial,
                         hipStream_t s) {
    if (gemm_nv(mtiles) == 1 && gemm_waves(mtiles) == 4) return run_gemm_bf16_nv<FMT, 1, WG_NT>(w, apk, t, mtiles, y, out_bf16, partial, s);
    if (gemm_nv(mtiles) == 1) return run_gemm_bf16_nv<FMT, 1, WG_NT, 8>(w, apk, t, mtiles, y, out_bf16, partial, s);
    if (gemm_row_tiles(w, mtiles) == 7) return run_gemm_bf16_nv<FMT, 2, 7>(w, apk, t, mtiles, y, out_bf16, partial, s);
    return run_gemm_bf16_nv<FMT, 2, WG_NT>(w, apk, t, mtiles, y, out_bf16, partial, s);
}
}  // namespace

hipError_t launch_gemm_reduce(const float* partial, size_t n, uint32_t slices, void* y, bool out_bf16, hipStream_t s) {
    if (!n) return hipSuccess;
    run_gemm_reduce(partial, n, slices, y, out_bf16, s);
    return hipGetLastError();
}

// `partial`: scratch of slices * t * n_out floats when gemm_k_slices() > 1.
// The formats the kernel dequantizes: tile-packed MLX 4-bit and Q4_0, Q8_0 / Q8, Q4_K, Q6_K, and FP8 rows of whole 128-column
// steps with scale blocks of 16 k rows x 128 k columns.
bool gemm_bf16_ok(const WeightView& w) {
    if (t4_geometry(w.fmt) || q8_format(w.fmt)) return true;
    if (k45_format(w.fmt) || w.fmt == FMT_Q6_K) return w.n_in % 256 == 0;
    return w.fmt == FMT_FP8 && w.br % 16 == 0 && w.bc % 128 == 0 && w.n_in % 128 == 0;
}
// pack_a's MODE for the format's fragments
int gemm_bf16_pack_mode(const WeightView& w) { return t4_geometry(w.fmt) ? 1 : w.fmt == FMT_FP8 ? 2 : w.fmt == FMT_Q6_K ? 3 : 0; }

hipError_t launch_gemm_bf16(const WeightView& w, const void* apk, size_t t, size_t mtiles, void* y, bool out_bf16, float* partial,
                            hipStream_t s) {
    if (!gemm_bf16_ok(w)) return hipErrorInvalidValue;
    switch (w.fmt) {
        case FMT_Q4M: return run_gemm_bf16<FMT_Q4M>(w, apk, t, mtiles, y, out_bf16, partial, s);
        case FMT_Q40: return run_gemm_bf16<FMT_Q40>(w, apk, t, mtiles, y, out_bf16, partial, s);
        case FMT_MXFP4: return run_gemm_bf16<FMT_MXFP4>(w, apk, t, mtiles, y, out_bf16, partial, s);
        case FMT_NVFP4: return run_gemm_bf16<FMT_NVFP4>(w, apk, t, mtiles, y, out_bf16, partial, s);
        case FMT_Q8_0: return run_gemm_bf16<FMT_Q8_0>(w, apk, t, mtiles, y, out_bf16, partial, s);
        case FMT_Q8F: return run_gemm_bf16<FMT_Q8F>(w, apk, t, mtiles, y, out_bf16, partial, s);
        case FMT_Q4_K: return run_gemm_bf16<FMT_Q4_K>(w, apk, t, mtiles, y, out_bf16, partial, s);
        case FMT_Q5_K: return run_gemm_bf16<FMT_Q5_K>(w, apk, t, mtiles, y, out_bf16, partial, s);
        case FMT_Q6_K: return run_gemm_bf16<FMT_Q6_K>(w, apk, t, mtiles, y, out_bf16, partial, s);
        default: return run_gemm_bf16<FMT_FP8>(w, apk, t, mtiles, y, out_bf16, partial, s);
    }
}

}  // namespace oxhip
