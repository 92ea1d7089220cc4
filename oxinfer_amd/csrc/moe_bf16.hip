// Grouped expert matmuls of an MoE prefill pass on the bf16 matrix cores (the experts' forward_batched of the
// reference, src/moe.rs:625-828, over MLX 4-bit weights repacked as Q4 blocks, src/quant.rs:518-606).
//
// With a dozen or more routed tokens per expert the integer path (int8 activations, one scale per token and block of
// 32) spends a conversion and two to three multiply-adds per (row, token, block), and those, not the weights' bytes,
// bound it. Here the routed tokens of a chunk (up to 16 rows of one expert) go in as bf16 and a weight is the bf16
// value 128 + nibble, made by one byte permute per two weights (0x4300 | nibble); per group of 64 columns the matrix
// cores form D = sum (128 + nib) x and E = sum x exactly in f32, and
//     y += d D + (off - 136 d) E          (the group's weights are d (nib - 8) + off)
// costs two multiply-adds per (row, token, group). The other formats in the same record geometry run the same way with a
// scale per block of 32: GGUF Q4_0 (d (nib - 8): y += d (D - 136 E) per block) and MXFP4 (2^(e - 128) times the doubled
// E2M1 value kv: the weight goes in as 128 + 12 + kv, y += d (D - 140 E)). This is the reference's own prefill form: from 8 rows on its
// experts run a grouped f32 GEMM over exact activations with Act::scalar between the two (src/moe.rs:735-827,
// matmul_quant_grouped, src/kernels.rs:195-279); the results here differ from it by the bf16 rounding of the
// activations. The integer path stays the one for decode, where the reference quantizes the activations too.
#include "act_body.hpp"
#include "internal.hpp"
#include "layout.hpp"

#include <cstdio>
#include <cstdlib>

namespace oxhip {

namespace {

typedef __bf16 bf16x8 __attribute__((ext_vector_type(8)));
typedef float f32x4 __attribute__((ext_vector_type(4)));
typedef uint32_t u32x4 __attribute__((ext_vector_type(4)));

// Fragments of a chunk's rows in operand order: [chunk][step of 128 columns][block b of 32][lane] x 8 bf16. Lane
// 16 kq + n holds row first + n of the chunk (zeros past its rows) at columns 128 s + 32 b + {4 kq .. + 3, 16 + 4 kq .. + 3}:
// the positions whose nibbles lane (kq, row) of a weight record holds in its dword b.
// ACT: the source is act(g) * u of the gathered rows (g, u rows `ld` floats apart); else row rowmap[first + n] of x.
// STD (the consumer's records are Q8_0's or Q4_K's, whose lane (kq, row) holds eight consecutive columns of a block): the
// lane's columns are 128 s + 32 b + 8 kq + {0 .. 7}.
template <bool ACT, bool STD>
__global__ __launch_bounds__(256) void moe_pack_bf16_kernel(const float* __restrict__ x, const float* __restrict__ up, size_t ld,
                                                           const int* __restrict__ rowmap, const int4* __restrict__ chunks,
                                                           const int* __restrict__ nchunks, uint32_t nsteps, uint32_t kind, float param,
                                                           uint4* __restrict__ out) {
    const uint32_t c = blockIdx.y, s = blockIdx.x;
    if (c >= (uint32_t)*nchunks) return;
    const int4 ch = chunks[c];
    const uint32_t lane = threadIdx.x & 63, b = threadIdx.x >> 6, n = lane & 15, kq = lane >> 4;
    uint32_t pk[4] = {0, 0, 0, 0};
    if (n < (uint32_t)ch.z) {
        const size_t r = ACT ? (size_t)(ch.y + n) : (size_t)(rowmap ? rowmap[ch.y + n] : ch.y + (int)n);
        const size_t col = 128 * (size_t)s + 32 * b + (STD ? 8 : 4) * kq;
        float v[8];
#pragma unroll
        for (int h = 0; h < 2; h++) {
            const float4 a = *reinterpret_cast<const float4*>(x + r * ld + col + (STD ? 4 : 16) * h);
            v[4 * h] = a.x; v[4 * h + 1] = a.y; v[4 * h + 2] = a.z; v[4 * h + 3] = a.w;
            if (ACT) {
                const float4 u = *reinterpret_cast<const float4*>(up + r * ld + col + (STD ? 4 : 16) * h);
                v[4 * h] = gated_act_scalar(a.x, u.x, kind, param);
                v[4 * h + 1] = gated_act_scalar(a.y, u.y, kind, param);
                v[4 * h + 2] = gated_act_scalar(a.z, u.z, kind, param);
                v[4 * h + 3] = gated_act_scalar(a.w, u.w, kind, param);
            }
        }
#pragma unroll
        for (int j = 0; j < 4; j++) pk[j] = (uint32_t)f32_to_bf16_bits(v[2 * j]) | ((uint32_t)f32_to_bf16_bits(v[2 * j + 1]) << 16);
    }
    out[(((size_t)c * nsteps + s) * 4 + b) * 64 + lane] = make_uint4(pk[0], pk[1], pk[2], pk[3]);
}

// Fused gate / up experts with the activation in the output stage: the workgroup's waves 0..3 take RT tiles each of the gate
// rows [64 RT gx, 64 RT (gx + 1)), waves 4..7 the up tiles of the same rows, and instead of the products the workgroup writes
// act(gate) * up of its rows as the down projection's fragments (what moe_pack_bf16_kernel<ACT> makes of the stored
// products, value for value: the same f32 sums go through the same gated_act_scalar and the same rounding).
struct MoeGlu {
    uint32_t inter = 0;      // 0: plain products to `out`
    uint32_t kind = 0;
    float param = 0.0f;
    uint32_t std_out = 0;    // the down projection's records hold consecutive columns per lane (Q8_0, Q4_K)
    uint4* frag = nullptr;   // [chunk][inter / 128][4][64] x 16 B
};
template <int RT>
__device__ __forceinline__ void moe_glu_store(const float* red, const MoeGlu& glu, uint32_t gx, uint32_t c, uint32_t rows) {
    constexpr uint32_t STEPS = 64 * RT / 128 ? 64 * RT / 128 : 1;  // steps of 128 columns the workgroup's rows make
    static_assert(64 * RT % 128 == 0, "whole steps per workgroup");
    for (uint32_t idx = threadIdx.x; idx < STEPS * 256; idx += blockDim.x) {
        const uint32_t l = idx & 63, b = (idx >> 6) & 3, sl = idx >> 8, n = l & 15, kq = l >> 4;
        uint32_t pk[4] = {0, 0, 0, 0};
        if (n < rows) {
            float v[8];
#pragma unroll
            for (int j = 0; j < 8; j++) {
                const uint32_t col = 128 * sl + 32 * b + (glu.std_out ? 8 * kq + j : 4 * kq + (j & 3) + 16 * (j >> 2));
                const uint32_t t = col >> 4, wv = t / RT, r = t % RT;
                const size_t at = (((size_t)wv * RT + r) * 64 + 16 * (n >> 2) + (col & 15)) * 4 + (n & 3);
                v[j] = gated_act_scalar(red[at], red[at + (size_t)4 * RT * 64 * 4], glu.kind, glu.param);
            }
#pragma unroll
            for (int j = 0; j < 4; j++) pk[j] = (uint32_t)f32_to_bf16_bits(v[2 * j]) | ((uint32_t)f32_to_bf16_bits(v[2 * j + 1]) << 16);
        }
        glu.frag[(((size_t)c * (glu.inter / 128) + gx * STEPS + sl) * 4 + b) * 64 + l] = make_uint4(pk[0], pk[1], pk[2], pk[3]);
    }
}

// Which (run of row tiles gx, chunk c) a workgroup of the one-dimensional grid takes. Workgroups go to the 8 XCDs in turn
// (linear id mod 8), and each XCD has an L2 of its own; an expert with more than 16 routed rows has several chunks, each
// of which streams the expert's rows again. Items are numbered (gx, c) with c fastest, so that the chunks of one expert
// are neighbours, and XCD k takes the k-th eighth of them in order: workgroups that read the same weights start
// together on the same XCD, and all but the first find them in its L2 instead of asking HBM again. False: no item.
__device__ __forceinline__ bool moe_bf16_item(uint32_t nx, uint32_t nch, uint32_t* gx, uint32_t* c) {
    const uint32_t total = nx * nch, per = (total + 7) >> 3;
    const uint32_t xcd = blockIdx.x & 7, q = blockIdx.x >> 3, v = xcd * per + q;
    if (q >= per || v >= total) return false;
    *gx = v / nch;
    *c = v - *gx * nch;
    return true;
}

// Workgroup: 8 waves = 8 / kw groups of RT row tiles x kw waves that split the K steps (wave v takes steps v, v + kw, ...)
// and meet in LDS in wave order. A workgroup's item (moe_bf16_item): a run of (8 / kw) RT row tiles of a chunk {expert, first row, rows <= 16}.
// The chunk's fragments (4 KiB per step) are staged into LDS once per workgroup: all eight waves multiply the same
// rows (each wave asking memory for them costs more than the weights). out [gathered row][n_out] f32.
template <int RT, int FMT>
__global__ __launch_bounds__(512, 4) void moe_bf16_kernel(WeightView w, const uint8_t* const* __restrict__ bases, const int4* __restrict__ chunks,
                                                          const int* __restrict__ nchunks, const uint4* __restrict__ afrag, uint32_t kw, uint32_t nx, MoeGlu glu,
                                                          float* __restrict__ out) {
    extern __shared__ __align__(16) float lds[];  // fragments [step][4][64] x 16 B; then the waves' sums [wave][RT][64][4]
    uint32_t gx, c;
    if (!moe_bf16_item(nx, (uint32_t)*nchunks, &gx, &c)) return;  // uniform over the workgroup
    const int4 ch = chunks[c];
    const uint32_t first = (uint32_t)ch.y, rows = (uint32_t)ch.z;
    const uint32_t lane = threadIdx.x & 63, wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
    const uint32_t n = lane & 15;
    const uint32_t nsteps = w.n_in / 128, ntiles = row_tiles(w.n_out);
    const uint32_t ng = 8 / kw, rg = wave / kw, kwave = wave % kw;
    // (with the activation fused: waves 0..3 the gate tiles of the workgroup's rows, waves 4..7 the up tiles; kw = 1)
    const uint32_t tile0 = glu.inter ? (rg < 4 ? (gx * 4 + rg) * RT : glu.inter / 16 + (gx * 4 + rg - 4) * RT) : (gx * ng + rg) * RT;
    const gbytes base = as_global(bases[ch.x]);
    gbytes wp[RT];
    constexpr uint32_t REC = FMT == FMT_MXFP4 ? T4X_REC : T4M_REC;
    constexpr bool PER32 = FMT != FMT_Q4M;  // a scale per block of 32 (Q4_0, MXFP4) instead of a scale and an offset per 64
#pragma unroll
    for (int r = 0; r < RT; r++) wp[r] = base + (size_t)min(tile0 + r, ntiles - 1) * t4m_steps(w.n_in) * REC;
    const uint32_t cnt = (nsteps - kwave + kw - 1) / kw, ilast = cnt - 1;  // kw <= nsteps

    struct St {
        u32x4 w[RT];
    };
    // every request is unconditional (past the end the last step again): the compiler then knows how many are in flight
    auto load = [&](St& st, uint32_t i) {
        const uint32_t s = kwave + kw * min(i, ilast);
#pragma unroll
        for (int r = 0; r < RT; r++) st.w[r] = gload<u32x4>(wp[r] + (size_t)s * REC + 16 * lane);
    };
    // A record's scale words (per row: the two groups' f16 scales at +1024, their bf16 offsets at +1088): a request costs
    // the memory pipeline the same for 64 bytes as for 1 KiB, so one request per row tile serves two steps: lane group kq
    // asks for word kq & 1 of step i + (kq >> 1), and at each step every lane takes its row's two words from those lanes.
    const uint32_t kq = lane >> 4;
    auto load_scales = [&](uint32_t* sc, uint32_t i) {
        const uint32_t s = kwave + kw * min(i + (kq >> 1), ilast);
#pragma unroll
        // (Q4_0: the same two words hold the row's four f16 block scales; MXFP4: one word of four E8M0 bytes)
        for (int r = 0; r < RT; r++) sc[r] = gload<uint32_t>(wp[r] + (size_t)s * REC + 1024 + (FMT == FMT_MXFP4 ? 0 : 64 * (kq & 1)) + 4 * n);
    };
    // the fragments first (L2 hits, needed by every step), then the first weight records, then the fragments go to LDS
    // while the weights are still on their way
    const u32x4* src = reinterpret_cast<const u32x4*>(afrag) + (size_t)c * nsteps * 256;
    u32x4* lf = reinterpret_cast<u32x4*>(lds);
    constexpr int SG = 8;  // 16-byte pieces a thread holds at a time (2048 columns of 16 rows in one batch)
    const uint32_t total = nsteps * 256;
    constexpr int PF = RT > 2 ? 2 : 4;  // steps on request (an even number: scales go by pairs of steps)
    St ring[PF];
    uint32_t scl[PF / 2][RT];
    for (uint32_t i0 = 0; i0 < total; i0 += 512 * SG) {
        u32x4 t[SG];
#pragma unroll
        for (int k = 0; k < SG; k++) t[k] = src[min(i0 + 512 * k + threadIdx.x, total - 1)];
        if (i0 == 0) {
#pragma unroll
            for (int p = 0; p < PF; p++) {
                if (p % 2 == 0) load_scales(scl[p / 2], (uint32_t)p);
                load(ring[p], (uint32_t)p);
            }
        }
#pragma unroll
        for (int k = 0; k < SG; k++)
            if (i0 + 512 * k + threadIdx.x < total) lf[i0 + 512 * k + threadIdx.x] = t[k];
    }
    __syncthreads();

    f32x4 acc[RT];
#pragma unroll
    for (int r = 0; r < RT; r++) acc[r] = f32x4{0.0f, 0.0f, 0.0f, 0.0f};
    const u32x4 one4 = {0x3F803F80u, 0x3F803F80u, 0x3F803F80u, 0x3F803F80u};
    const bf16x8 ones = __builtin_bit_cast(bf16x8, one4);
    auto compute = [&](const St& st, const uint32_t* sc, int odd, uint32_t i) {
        const uint32_t s = kwave + kw * i;
        bf16x8 a[4];
#pragma unroll
        for (int b = 0; b < 4; b++) a[b] = __builtin_bit_cast(bf16x8, lf[(s * 4 + b) * 64 + lane]);
        // E: the sum of activations per token over a group of 64 (every row's offset multiplies it), or over each block of 32
        constexpr int NE = PER32 ? 4 : 2;
        f32x4 E[NE];
#pragma unroll
        for (int g = 0; g < NE; g++) {
            E[g] = f32x4{0.0f, 0.0f, 0.0f, 0.0f};
            if (PER32) {
                E[g] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(a[g], ones, E[g], 0, 0, 0);
            } else {
                E[g] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(a[2 * g], ones, E[g], 0, 0, 0);
                E[g] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(a[2 * g + 1], ones, E[g], 0, 0, 0);
            }
        }
#pragma unroll
        for (int r = 0; r < RT; r++) {
            f32x4 D[NE];
#pragma unroll
            for (int g = 0; g < NE; g++) D[g] = f32x4{0.0f, 0.0f, 0.0f, 0.0f};
#pragma unroll
            for (int b = 0; b < 4; b++) {
                // byte j of the dword: low nibble = position 4 kq + j, high nibble = position 16 + 4 kq + j; bf16 0x43nn = 128 + nn
                const uint32_t wd = st.w[r][b];
                uint32_t lo = wd & 0x0F0F0F0Fu, hi = (wd >> 4) & 0x0F0F0F0Fu;
                if (FMT == FMT_MXFP4) {  // table codes -> their doubled values + 12 (0 .. 24)
                    lo = mxfp4_values<12>(lo);
                    hi = mxfp4_values<12>(hi);
                }
                const u32x4 wb = {__builtin_amdgcn_perm(0x43434343u, lo, 0x04010400u), __builtin_amdgcn_perm(0x43434343u, lo, 0x04030402u),
                                  __builtin_amdgcn_perm(0x43434343u, hi, 0x04010400u), __builtin_amdgcn_perm(0x43434343u, hi, 0x04030402u)};
                D[PER32 ? b : b >> 1] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(a[b], __builtin_bit_cast(bf16x8, wb), D[PER32 ? b : b >> 1], 0, 0, 0);
            }
            const uint32_t dw = (uint32_t)__builtin_amdgcn_ds_bpermute((int)(4 * (32 * odd + n)), (int)sc[r]);
            const uint32_t ow = FMT == FMT_MXFP4 ? 0u : (uint32_t)__builtin_amdgcn_ds_bpermute((int)(4 * (32 * odd + 16 + n)), (int)sc[r]);
            if (PER32) {
#pragma unroll
                for (int b = 0; b < 4; b++) {
                    float d;
                    if (FMT == FMT_MXFP4) d = e8m0_half((dw >> (8 * b)) & 0xFF);
                    else d = f16_bits_to_f32((uint16_t)(((b < 2 ? dw : ow) >> (16 * (b & 1))) & 0xFFFF));
                    const float cc = (FMT == FMT_MXFP4 ? -140.0f : -136.0f) * d;
#pragma unroll
                    for (int i2 = 0; i2 < 4; i2++) acc[r][i2] = fmaf(cc, E[b][i2], fmaf(d, D[b][i2], acc[r][i2]));
                }
            } else {
#pragma unroll
                for (int g = 0; g < 2; g++) {
                    const float d = f16_bits_to_f32((uint16_t)(g ? dw >> 16 : dw & 0xFFFF));
                    const float off = bf16_bits_to_f32((uint16_t)(g ? ow >> 16 : ow & 0xFFFF));
                    const float cc = off - 136.0f * d;
#pragma unroll
                    for (int i2 = 0; i2 < 4; i2++) acc[r][i2] = fmaf(cc, E[g][i2], fmaf(d, D[g][i2], acc[r][i2]));
                }
            }
        }
    };
    for (uint32_t ib = 0; ib < cnt; ib += PF) {
#pragma unroll
        for (int p = 0; p < PF; p++) {
            if (ib + p < cnt) compute(ring[p], scl[p / 2], p % 2, ib + p);
            load(ring[p], ib + PF + p);
            if (p % 2 == 1) load_scales(scl[p / 2], ib + PF + p - 1);  // both steps of the pair are done with the old words
        }
    }
    __syncthreads();  // the sums overwrite the fragments
    float* red = lds;
#pragma unroll
    for (int r = 0; r < RT; r++) *reinterpret_cast<f32x4*>(red + (((size_t)wave * RT + r) * 64 + lane) * 4) = acc[r];
    __syncthreads();
    if (glu.inter) {  // uniform over the launch
        moe_glu_store<RT>(red, glu, gx, c, rows);
        return;
    }
    // D[token 4 kq + i][row n]: thread (group, r, lane) adds the group's waves in order and stores its four tokens
    for (uint32_t idx = threadIdx.x; idx < ng * RT * 64; idx += blockDim.x) {
        const uint32_t l = idx & 63, r = (idx >> 6) % RT, g = (idx >> 6) / RT;
        const uint32_t tile = (gx * ng + g) * RT + r, row = tile * 16 + (l & 15);
        if (tile >= ntiles || row >= w.n_out) continue;
        f32x4 sum = *reinterpret_cast<const f32x4*>(red + (((size_t)(g * kw) * RT + r) * 64 + l) * 4);
        for (uint32_t k = 1; k < kw; k++) {
            const f32x4 v = *reinterpret_cast<const f32x4*>(red + (((size_t)(g * kw + k) * RT + r) * 64 + l) * 4);
#pragma unroll
            for (int i = 0; i < 4; i++) sum[i] += v[i];
        }
#pragma unroll
        for (int i = 0; i < 4; i++) {
            const uint32_t tok = 4 * (l >> 4) + i;
            if (tok < rows) out[(size_t)(first + tok) * w.n_out + row] = sum[i];
        }
    }
}

// The same for experts in GGUF Q8_0 or Q4_K records, whose lane (kq, row) holds a block's eight consecutive columns
// 8 kq .. 8 kq + 7 (the fragments come packed in that order, moe_pack_bf16_kernel's STD form):
//   Q4_K  a nibble goes in as 128 + nib; per block of 32 y += (d sc) (D - 128 E) - (dmin mn) E   (dequantize_row's
//         (d sc) nib - dmin mn, src/ggml.rs:750-773)
//   Q8_0  the code q as the byte m = q + 128 = 16 H + L, both nibbles as 128 + nibble in two matrix instructions:
//         sum q x = 16 D_H + D_L - 2304 E, y += d (that) per block of 32   (q d, src/ggml.rs:707-712)
// Every product and sum is exact up to the f32 rounding of the matrix cores' accumulation.
template <int RT, int FMT>
__global__ __launch_bounds__(512, 4) void moe_bf16_std_kernel(WeightView w, const uint8_t* const* __restrict__ bases, const int4* __restrict__ chunks,
                                                              const int* __restrict__ nchunks, const uint4* __restrict__ afrag, uint32_t kw, uint32_t nx, MoeGlu glu,
                                                              float* __restrict__ out) {
    static_assert(FMT == FMT_Q8_0 || FMT == FMT_Q4_K, "the formats whose records hold consecutive columns per lane");
    constexpr bool Q8 = FMT == FMT_Q8_0;
    extern __shared__ __align__(16) float lds[];  // fragments [step][4][64] x 16 B; then the waves' sums [wave][RT][64][4]
    uint32_t gx, c;
    if (!moe_bf16_item(nx, (uint32_t)*nchunks, &gx, &c)) return;  // uniform over the workgroup
    const int4 ch = chunks[c];
    const uint32_t first = (uint32_t)ch.y, rows = (uint32_t)ch.z;
    const uint32_t lane = threadIdx.x & 63, wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
    const uint32_t n = lane & 15, kq = lane >> 4;
    const uint32_t nsteps = w.n_in / 128, ntiles = row_tiles(w.n_out);
    const uint32_t ng = 8 / kw, rg = wave / kw, kwave = wave % kw;
    // (with the activation fused: waves 0..3 the gate tiles of the workgroup's rows, waves 4..7 the up tiles; kw = 1)
    const uint32_t tile0 = glu.inter ? (rg < 4 ? (gx * 4 + rg) * RT : glu.inter / 16 + (gx * 4 + rg - 4) * RT) : (gx * ng + rg) * RT;
    const gbytes base = as_global(bases[ch.x]);
    gbytes wp[RT];
#pragma unroll
    for (int r = 0; r < RT; r++)
        wp[r] = base + (size_t)min(tile0 + r, ntiles - 1) * (Q8 ? (size_t)t8_steps(w.n_in) * T8_REC : (size_t)tk4_sbs(w.n_in) * TK4_REC);
    const uint32_t cnt = (nsteps - kwave + kw - 1) / kw, ilast = cnt - 1;  // kw <= nsteps

    struct St {
        u32x4 w[RT];
        u32x4 w2[Q8 ? RT : 1];  // Q8_0: the step's second record of 64 columns
        uint32_t sc[RT];         // the row's scale words of the step, one kind per lane group (see below)
    };
    // every request is unconditional (past the end the last step again): the compiler then knows how many are in flight.
    // Scale words: lane group kq asks for Q8_0 {d of blocks 0-1, d of blocks 2-3, .., ..}, Q4_K {four scales, four mins,
    // (d, dmin), ..} of row n; at the step every lane takes its row's words from lanes n, 16 + n, 32 + n.
    auto load = [&](St& st, uint32_t i) {
        const uint32_t s = kwave + kw * min(i, ilast);
#pragma unroll
        for (int r = 0; r < RT; r++) {
            if (Q8) {
                const gbytes rec = wp[r] + (size_t)(2 * s) * T8_REC;
                st.w[r] = gload<u32x4>(rec + 16 * lane);
                st.w2[r] = gload<u32x4>(rec + T8_REC + 16 * lane);
                st.sc[r] = gload<uint32_t>(rec + (kq & 1) * T8_REC + 1024 + 4 * n);
            } else {
                const gbytes rec = wp[r] + (size_t)(s >> 1) * TK4_REC;
                st.w[r] = gload<u32x4>(rec + (s & 1) * 1024 + 16 * lane);
                st.sc[r] = gload<uint32_t>(rec + (kq == 0 ? 2048 + 16 * n + 4 * (s & 1) : kq == 1 ? 2048 + 16 * n + 8 + 4 * (s & 1) : 2304 + 4 * n));
            }
        }
    };
    const u32x4* src = reinterpret_cast<const u32x4*>(afrag) + (size_t)c * nsteps * 256;
    u32x4* lf = reinterpret_cast<u32x4*>(lds);
    constexpr int SG = 8;
    const uint32_t total = nsteps * 256;
    constexpr int PF = 2;
    St ring[PF];
    for (uint32_t i0 = 0; i0 < total; i0 += 512 * SG) {
        u32x4 t[SG];
#pragma unroll
        for (int k = 0; k < SG; k++) t[k] = src[min(i0 + 512 * k + threadIdx.x, total - 1)];
        if (i0 == 0) {
#pragma unroll
            for (int p = 0; p < PF; p++) load(ring[p], (uint32_t)p);
        }
#pragma unroll
        for (int k = 0; k < SG; k++)
            if (i0 + 512 * k + threadIdx.x < total) lf[i0 + 512 * k + threadIdx.x] = t[k];
    }
    __syncthreads();

    f32x4 acc[RT];
#pragma unroll
    for (int r = 0; r < RT; r++) acc[r] = f32x4{0.0f, 0.0f, 0.0f, 0.0f};
    const u32x4 one4 = {0x3F803F80u, 0x3F803F80u, 0x3F803F80u, 0x3F803F80u};
    const bf16x8 ones = __builtin_bit_cast(bf16x8, one4);
    auto nib_bf16 = [](uint32_t n0, uint32_t n1) {  // eight nibbles (one per byte of n0, n1) -> eight bf16 of 128 + nibble
        const u32x4 wb = {__builtin_amdgcn_perm(0x43434343u, n0, 0x04010400u), __builtin_amdgcn_perm(0x43434343u, n0, 0x04030402u),
                          __builtin_amdgcn_perm(0x43434343u, n1, 0x04010400u), __builtin_amdgcn_perm(0x43434343u, n1, 0x04030402u)};
        return __builtin_bit_cast(bf16x8, wb);
    };
    auto compute = [&](const St& st, uint32_t i) {
        const uint32_t s = kwave + kw * i;
        bf16x8 a[4];
        f32x4 E[4];
#pragma unroll
        for (int b = 0; b < 4; b++) {
            a[b] = __builtin_bit_cast(bf16x8, lf[(s * 4 + b) * 64 + lane]);
            E[b] = f32x4{0.0f, 0.0f, 0.0f, 0.0f};
            E[b] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(a[b], ones, E[b], 0, 0, 0);
        }
#pragma unroll
        for (int r = 0; r < RT; r++) {
            const uint32_t w0 = (uint32_t)__builtin_amdgcn_ds_bpermute((int)(4 * n), (int)st.sc[r]);
            const uint32_t w1 = (uint32_t)__builtin_amdgcn_ds_bpermute((int)(4 * (16 + n)), (int)st.sc[r]);
            const uint32_t w2 = Q8 ? 0u : (uint32_t)__builtin_amdgcn_ds_bpermute((int)(4 * (32 + n)), (int)st.sc[r]);
            const float zero4[4] = {0.0f, 0.0f, 0.0f, 0.0f};
            (void)zero4;
#pragma unroll
            for (int b = 0; b < 4; b++) {
                const f32x4 z = f32x4{0.0f, 0.0f, 0.0f, 0.0f};
                if (Q8) {
                    const int h = b >> 1, e = b & 1;
                    const uint32_t c0 = (h ? st.w2[r][2 * e] : st.w[r][2 * e]) ^ 0x80808080u, c1 = (h ? st.w2[r][2 * e + 1] : st.w[r][2 * e + 1]) ^ 0x80808080u;
                    const f32x4 DH = __builtin_amdgcn_mfma_f32_16x16x32_bf16(a[b], nib_bf16((c0 >> 4) & 0x0F0F0F0Fu, (c1 >> 4) & 0x0F0F0F0Fu), z, 0, 0, 0);
                    const f32x4 DL = __builtin_amdgcn_mfma_f32_16x16x32_bf16(a[b], nib_bf16(c0 & 0x0F0F0F0Fu, c1 & 0x0F0F0F0Fu), z, 0, 0, 0);
                    const float d = f16_bits_to_f32((uint16_t)(((h ? w1 : w0) >> (16 * e)) & 0xFFFF));
                    const float cc = -2304.0f * d;
#pragma unroll
                    for (int i2 = 0; i2 < 4; i2++) acc[r][i2] = fmaf(cc, E[b][i2], fmaf(d, fmaf(16.0f, DH[i2], DL[i2]), acc[r][i2]));
                } else {
                    const int jj = b >> 1, hi = b & 1;
                    const uint32_t c0 = ((jj ? st.w[r][2] : st.w[r][0]) >> (4 * hi)) & 0x0F0F0F0Fu, c1 = ((jj ? st.w[r][3] : st.w[r][1]) >> (4 * hi)) & 0x0F0F0F0Fu;
                    const f32x4 D = __builtin_amdgcn_mfma_f32_16x16x32_bf16(a[b], nib_bf16(c0, c1), z, 0, 0, 0);
                    const float d = f16_bits_to_f32((uint16_t)(w2 & 0xFFFF)), dmin = f16_bits_to_f32((uint16_t)(w2 >> 16));
                    const float dsc = d * (float)((w0 >> (8 * b)) & 0xFF), m1 = dmin * (float)((w1 >> (8 * b)) & 0xFF);
                    const float cc = fmaf(-128.0f, dsc, -m1);
#pragma unroll
                    for (int i2 = 0; i2 < 4; i2++) acc[r][i2] = fmaf(cc, E[b][i2], fmaf(dsc, D[i2], acc[r][i2]));
                }
            }
        }
    };
    for (uint32_t ib = 0; ib < cnt; ib += PF) {
#pragma unroll
        for (int p = 0; p < PF; p++) {
            if (ib + p < cnt) compute(ring[p], ib + p);
            load(ring[p], ib + PF + p);
        }
    }
    __syncthreads();  // the sums overwrite the fragments
    float* red = lds;
#pragma unroll
    for (int r = 0; r < RT; r++) *reinterpret_cast<f32x4*>(red + (((size_t)wave * RT + r) * 64 + lane) * 4) = acc[r];
    __syncthreads();
    if (glu.inter) {  // uniform over the launch
        moe_glu_store<RT>(red, glu, gx, c, rows);
        return;
    }
    for (uint32_t idx = threadIdx.x; idx < ng * RT * 64; idx += blockDim.x) {
        const uint32_t l = idx & 63, r = (idx >> 6) % RT, g = (idx >> 6) / RT;
        const uint32_t tile = (gx * ng + g) * RT + r, row = tile * 16 + (l & 15);
        if (tile >= ntiles || row >= w.n_out) continue;
        f32x4 sum = *reinterpret_cast<const f32x4*>(red + (((size_t)(g * kw) * RT + r) * 64 + l) * 4);
        for (uint32_t k = 1; k < kw; k++) {
            const f32x4 v = *reinterpret_cast<const f32x4*>(red + (((size_t)(g * kw + k) * RT + r) * 64 + l) * 4);
#pragma unroll
            for (int i = 0; i < 4; i++) sum[i] += v[i];
        }
#pragma unroll
        for (int i = 0; i < 4; i++) {
            const uint32_t tok = 4 * (l >> 4) + i;
            if (tok < rows) out[(size_t)(first + tok) * w.n_out + row] = sum[i];
        }
    }
}

}  // namespace

// (the fragments of a chunk, 32 bytes per column, must fit the LDS)
bool moe_bf16_ok(const WeightView& w) {
    if (w.n_in % 128 || w.n_in < 128 || w.n_in > 4096) return false;
    return t4m_format(w.fmt) || w.fmt == FMT_Q8_0 || (w.fmt == FMT_Q4_K && w.n_in % 256 == 0);
}
// The order of a block's columns in the fragments that the format's kernel reads (launch_moe_pack_bf16's `std_geometry`).
bool moe_bf16_std_geometry(const WeightView& w) { return w.fmt == FMT_Q8_0 || w.fmt == FMT_Q4_K; }

size_t moe_bf16_frag_bytes(size_t max_chunks, size_t n_in) { return max_chunks * (n_in / 128) * 4 * 64 * 16; }

// Fragments of x rows (rowmap: gathered row -> row of x; ld = n_in) for chunks of at most 16 rows.
hipError_t launch_moe_pack_bf16(const float* x, size_t n_in, const int* rowmap, const int4* chunks, const int* nchunks, uint32_t max_chunks,
                                void* frag, hipStream_t s, bool std_geometry) {
    if (!max_chunks) return hipSuccess;
    const dim3 grid((unsigned)(n_in / 128), max_chunks);
    if (std_geometry) moe_pack_bf16_kernel<false, true><<<grid, 256, 0, s>>>(x, nullptr, n_in, rowmap, chunks, nchunks, (uint32_t)(n_in / 128), 0, 0.0f, static_cast<uint4*>(frag));
    else moe_pack_bf16_kernel<false, false><<<grid, 256, 0, s>>>(x, nullptr, n_in, rowmap, chunks, nchunks, (uint32_t)(n_in / 128), 0, 0.0f, static_cast<uint4*>(frag));
    return hipGetLastError();
}

// Fragments of act(g) * u over the gathered rows (g, u rows `stride` floats apart).
hipError_t launch_moe_act_pack_bf16(const float* g, const float* u, size_t stride, size_t inter, uint32_t kind, float param, const int4* chunks,
                                    const int* nchunks, uint32_t max_chunks, void* frag, hipStream_t s, bool std_geometry) {
    if (!max_chunks) return hipSuccess;
    const dim3 grid((unsigned)(inter / 128), max_chunks);
    if (std_geometry) moe_pack_bf16_kernel<true, true><<<grid, 256, 0, s>>>(g, u, stride, nullptr, chunks, nchunks, (uint32_t)(inter / 128), kind, param, static_cast<uint4*>(frag));
    else moe_pack_bf16_kernel<true, false><<<grid, 256, 0, s>>>(g, u, stride, nullptr, chunks, nchunks, (uint32_t)(inter / 128), kind, param, static_cast<uint4*>(frag));
    return hipGetLastError();
}

// Whether the gate / up launch over fused experts `w` ([2 inter, h]) can apply the activation itself and write the down
// projection's fragments (launch_moe_bf16 with glu_inter): whole workgroups of gate rows, and the plain one-wave-per-row shape.
bool moe_bf16_glu_ok(const WeightView& w, size_t inter, uint32_t max_chunks) {
    if (!moe_bf16_ok(w) || w.n_out != 2 * inter || inter % 128) return false;
    const uint32_t rt = w.fmt == FMT_Q8_0 ? 2 : 4, nsteps = w.n_in / 128, ntiles = row_tiles(w.n_out);
    if (inter % (64 * rt)) return false;
    return !(nsteps / 2 >= 4 && (uint64_t)((ntiles + 8 * rt - 1) / (8 * rt)) * max_chunks < 512);  // (the launcher would split K over waves)
}

// glu_inter != 0 (moe_bf16_glu_ok): `out_frag` receives the fragments of act(gate) * up for a down projection whose records
// are in `std_out` geometry or not; else `out` receives the products' rows.
hipError_t launch_moe_bf16(const WeightView& w, const GroupView& g, uint32_t max_chunks, const void* frag, float* out, hipStream_t s,
                           size_t glu_inter, uint32_t act_kind, float act_param, bool std_out, void* out_frag) {
    if (!moe_bf16_ok(w)) return hipErrorInvalidValue;
    if (!max_chunks) return hipSuccess;
    const uint32_t nsteps = w.n_in / 128, ntiles = row_tiles(w.n_out);
    // a wave streams a whole row of records (kw = 1) unless that leaves fewer workgroups than two per CU
    uint32_t rt = w.fmt == FMT_Q8_0 ? 2 : 4, kw = 1;  // (Q8_0: a step is two records per row tile)
    while (kw < 4 && nsteps / (2 * kw) >= 4 && (uint64_t)((ntiles + (8 / kw) * rt - 1) / ((8 / kw) * rt)) * max_chunks < 512) kw *= 2;
    MoeGlu glu{};
    if (glu_inter) {
        if (!moe_bf16_glu_ok(w, glu_inter, max_chunks) || kw != 1 || !out_frag) return hipErrorInvalidValue;
        glu = MoeGlu{(uint32_t)glu_inter, act_kind, act_param, std_out ? 1u : 0u, static_cast<uint4*>(out_frag)};
    }
#ifdef OXHIP_TUNING  // tuning builds only: "rt,kw" in OXHIP_MOE_BF16
    if (const char* e = getenv("OXHIP_MOE_BF16")) {
        unsigned a = 0, b = 0;
        if (sscanf(e, "%u,%u", &a, &b) == 2 && (a == 2 || a == 4) && (b == 1 || b == 2 || b == 4 || b == 8) && b <= nsteps) {
            rt = a;
            kw = b;
        }
    }
#endif
    const uint32_t ng = 8 / kw;
    const size_t red = (size_t)8 * rt * 64 * 16, fr = (size_t)nsteps * 4096, lds = fr > red ? fr : red;
    const uint32_t nx = glu_inter ? (uint32_t)(glu_inter / (64 * rt)) : (ntiles + ng * rt - 1) / (ng * rt);
    const dim3 grid((nx * max_chunks + 7) / 8 * 8);  // every XCD's share of the items (moe_bf16_item), whatever the chunk count turns out to be
    hipError_t e = hipSuccess;
    auto go = [&](auto kern) {
        if (lds > 48 * 1024) e = hipFuncSetAttribute(reinterpret_cast<const void*>(kern), hipFuncAttributeMaxDynamicSharedMemorySize, (int)lds);
        if (e == hipSuccess) kern<<<grid, 512, lds, s>>>(w, g.bases, g.chunks, g.nchunks, static_cast<const uint4*>(frag), kw, nx, glu, out);
    };
    if (w.fmt == FMT_Q8_0) go(moe_bf16_std_kernel<2, FMT_Q8_0>);
    else if (w.fmt == FMT_Q4_K) rt == 2 ? go(moe_bf16_std_kernel<2, FMT_Q4_K>) : go(moe_bf16_std_kernel<4, FMT_Q4_K>);
    else if (w.fmt == FMT_Q40) rt == 2 ? go(moe_bf16_kernel<2, FMT_Q40>) : go(moe_bf16_kernel<4, FMT_Q40>);
    else if (w.fmt == FMT_MXFP4) rt == 2 ? go(moe_bf16_kernel<2, FMT_MXFP4>) : go(moe_bf16_kernel<4, FMT_MXFP4>);
    else rt == 2 ? go(moe_bf16_kernel<2, FMT_Q4M>) : go(moe_bf16_kernel<4, FMT_Q4M>);
    return e != hipSuccess ? e : hipGetLastError();
}

}  // namespace oxhip
