// Prefill GEMM on the int8 matrix cores over tile-packed MLX 4-bit weights: the semantics of the reference's int8
// GEMM (src/kernels_i8gemm.rs:160-315, one activation plane). Activations are quantized per token and block of 32
// exactly as quantize_act does (src/quant.rs:267-292: q = round_half_away(x * 127 / amax), scale = amax / 127,
// f = sum of x); per weight row, token and block the int32 sum I = sum (nib - 8) * q is exact, and
//     y[t][r] = sum_b I_b * (d_b * xs_b) + sum_g off_g * F_g          (F_g = f of the group's two blocks)
// in f32. One v_mfma_i32_16x16x32_i8 yields a block's sums for 16 rows x 16 tokens; the weights are the A operand,
// so a lane's four results are rows 4 kq + i of the tile for token n: its row scales come from one 16-byte load of
// the record and its token's activation scales are its own.
#include "internal.hpp"
#include "layout.hpp"

#include <cstdlib>

namespace oxhip {

namespace {

typedef int v4i __attribute__((ext_vector_type(4)));

// Four nibbles (one per byte, 0..15) -> four int8 codes nib - 8: flip bit 3, then extend it into bits 4..7.
__device__ __forceinline__ uint32_t center4(uint32_t nib) {
    const uint32_t s = nib ^ 0x08080808u;
    return s | ((s & 0x08080808u) * 0x1Eu);
}

__device__ __forceinline__ long pack64(uint32_t lo, uint32_t hi) { return (long)(((uint64_t)hi << 32) | lo); }

// One thread per (token slot, group of 64 columns). Writes, for token tile tt = slot / 16 and group g:
//   frag[(tt * ngrp + g) * 64 + 16 kq + slot % 16] = {blk0 cols 4kq.., blk0 cols 16+4kq.., blk1 cols 4kq.., blk1 cols 16+4kq..}
//   xs[(tt * ngrp + g) * 16 + slot % 16] = the two block scales;  fs[...] = f_0 + f_1
// Slots past t and groups past n_in / 64 hold zeros.
template <bool SRC_BF16>
__global__ __launch_bounds__(256) void quantize_pack_i8_kernel(const void* __restrict__ xv, uint32_t t, uint32_t n_in, uint32_t slots,
                                                               uint32_t ngrp, uint4* __restrict__ frag, float2* __restrict__ xs,
                                                               float* __restrict__ fs) {
    const size_t idx = (size_t)blockIdx.x * blockDim.x + threadIdx.x;
    if (idx >= (size_t)slots * ngrp) return;
    const uint32_t g = (uint32_t)(idx % ngrp), slot = (uint32_t)(idx / ngrp);
    const uint32_t tt = slot >> 4, n = slot & 15;
    uint32_t word[2][8];
    float scale[2] = {0.0f, 0.0f}, fsum[2] = {0.0f, 0.0f};
#pragma unroll
    for (int h = 0; h < 2; h++)
#pragma unroll
        for (int i = 0; i < 8; i++) word[h][i] = 0;
    if (slot < t && g < n_in / 64) {
#pragma unroll
        for (int h = 0; h < 2; h++) {
            float v[32];
            const size_t at = (size_t)slot * n_in + 64 * (size_t)g + 32 * h;
            if (SRC_BF16) {
                const uint4* src = reinterpret_cast<const uint4*>(static_cast<const uint16_t*>(xv) + at);
#pragma unroll
                for (int i = 0; i < 4; i++) {
                    const uint4 u = src[i];
                    const uint32_t d[4] = {u.x, u.y, u.z, u.w};
#pragma unroll
                    for (int k = 0; k < 4; k++) {
                        v[8 * i + 2 * k] = __uint_as_float(d[k] << 16);
                        v[8 * i + 2 * k + 1] = __uint_as_float(d[k] & 0xFFFF0000u);
                    }
                }
            } else {
                const float4* src = reinterpret_cast<const float4*>(static_cast<const float*>(xv) + at);
#pragma unroll
                for (int i = 0; i < 8; i++) {
                    const float4 f = src[i];
                    v[4 * i] = f.x; v[4 * i + 1] = f.y; v[4 * i + 2] = f.z; v[4 * i + 3] = f.w;
                }
            }
            float amax = 0.0f;
#pragma unroll
            for (int i = 0; i < 32; i++) amax = fmaxf(amax, fabsf(v[i]));
            const float inv = amax > 0.0f ? 127.0f / amax : 0.0f;
            float f = -0.0f;
#pragma unroll
            for (int i = 0; i < 32; i++) f += v[i];
#pragma unroll
            for (int i = 0; i < 8; i++) {
                uint32_t wv = 0;
#pragma unroll
                for (int k = 0; k < 4; k++) {
                    const float r = roundf(v[4 * i + k] * inv);
                    const int iv = r != r ? 0 : (int)fminf(fmaxf(r, -128.0f), 127.0f);
                    wv |= ((uint32_t)iv & 0xFF) << (8 * k);
                }
                word[h][i] = wv;
            }
            scale[h] = amax / 127.0f;
            fsum[h] = f;
        }
    }
    const size_t base = (size_t)tt * ngrp + g;
#pragma unroll
    for (int kq = 0; kq < 4; kq++) frag[base * 64 + 16 * kq + n] = make_uint4(word[0][kq], word[0][4 + kq], word[1][kq], word[1][4 + kq]);
    xs[base * 16 + n] = make_float2(scale[0], scale[1]);
    fs[base * 16 + n] = fsum[0] + fsum[1];
}

// Workgroup: 4 waves, each RT row tiles (16 RT rows) x TT token tiles (16 TT tokens) over one K slice; no LDS and no
// barrier: every operand a lane needs is its own (weights, row scales) or its token's (activation fragments, scales).
// A group of 64 columns is worked in PH phases of TT / PH token tiles, each phase's activation operands requested one
// phase ahead. Two waves per SIMD keep the matrix-core results in ordinary registers.
// DUMP also stores the exact block sums to dump[(token * n_out + row) * (n_in / 32) + block].
template <int RT, int TT, int PH, bool DUMP>
__global__ __launch_bounds__(256, 2) void gemm_i8_q4m_kernel(WeightView w, const uint4* __restrict__ afrag, const float2* __restrict__ axs,
                                                             const float* __restrict__ afs, uint32_t t, uint32_t ngrp,
                                                             float* __restrict__ y, int32_t* __restrict__ dump) {
    constexpr int TH = TT / PH;
    const uint32_t lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
    const uint32_t n = lane & 15, kq = lane >> 4;
    const uint32_t ntiles = row_tiles(w.n_out), all_steps = t4m_steps(w.n_in), nblk = w.n_in / 32;
    const uint32_t rt0 = (blockIdx.x * 4 + wave) * RT;
    if (rt0 >= ntiles) return;
    const uint32_t tt0 = blockIdx.y * TT;
    const uint32_t per = (all_steps + gridDim.z - 1) / gridDim.z;
    const uint32_t s0 = blockIdx.z * per, s1 = min(all_steps, s0 + per);
    y += (size_t)blockIdx.z * t * w.n_out;

    const uint8_t* wbase[RT];
#pragma unroll
    for (int i = 0; i < RT; i++) wbase[i] = w.p0 + (size_t)min(rt0 + i, ntiles - 1) * all_steps * T4M_REC;
    float acc[RT][TT][4];
#pragma unroll
    for (int i = 0; i < RT; i++)
#pragma unroll
        for (int tt = 0; tt < TT; tt++)
#pragma unroll
            for (int e = 0; e < 4; e++) acc[i][tt][e] = 0.0f;

    struct Act {
        uint4 f[TH];
        float2 xs[TH];
        float fs[TH];
    };
    auto load_codes = [&](uint4* c, uint32_t s) {
#pragma unroll
        for (int i = 0; i < RT; i++) c[i] = *reinterpret_cast<const uint4*>(wbase[i] + (size_t)s * T4M_REC + 16 * lane);
    };
    auto load_scales = [&](uint4* dd, uint4* oo, uint32_t s) {
#pragma unroll
        for (int i = 0; i < RT; i++) {
            const uint8_t* rec = wbase[i] + (size_t)s * T4M_REC;
            dd[i] = *reinterpret_cast<const uint4*>(rec + 1024 + 16 * kq);
            oo[i] = *reinterpret_cast<const uint4*>(rec + 1088 + 16 * kq);
        }
    };
    // phase p = PH * group + part
    const uint4* fb = afrag + (size_t)tt0 * ngrp * 64 + lane;
    const float2* xb = axs + (size_t)tt0 * ngrp * 16 + n;
    const float* sb = afs + (size_t)tt0 * ngrp * 16 + n;
    auto load_act = [&](Act& a, uint32_t p) {
        const uint32_t grp = p / PH, h = p % PH;
#pragma unroll
        for (int tt = 0; tt < TH; tt++) {
            const size_t at = (size_t)(h * TH + tt) * ngrp + grp;
            a.f[tt] = fb[at * 64];
            a.xs[tt] = xb[at * 16];
            a.fs[tt] = sb[at * 16];
        }
    };
    auto compute = [&](const uint4* c, const uint4* dv, const uint4* ov, const Act& a, uint32_t grp, int g, int h) {
        long wa[RT][2];
        float ds[RT][4], off[RT][4];
#pragma unroll
        for (int i = 0; i < RT; i++) {
            const uint32_t w0 = g ? c[i].z : c[i].x, w1 = g ? c[i].w : c[i].y;
            wa[i][0] = pack64(center4(w0 & 0x0F0F0F0Fu), center4((w0 >> 4) & 0x0F0F0F0Fu));
            wa[i][1] = pack64(center4(w1 & 0x0F0F0F0Fu), center4((w1 >> 4) & 0x0F0F0F0Fu));
            const uint32_t dd[4] = {dv[i].x, dv[i].y, dv[i].z, dv[i].w};
            const uint32_t oo[4] = {ov[i].x, ov[i].y, ov[i].z, ov[i].w};
#pragma unroll
            for (int e = 0; e < 4; e++) {
                ds[i][e] = f16_bits_to_f32((uint16_t)(g ? dd[e] >> 16 : dd[e] & 0xFFFF));
                off[i][e] = bf16_bits_to_f32((uint16_t)(g ? oo[e] >> 16 : oo[e] & 0xFFFF));
            }
        }
#pragma unroll
        for (int tt = 0; tt < TH; tt++) {
            const long b0 = pack64(a.f[tt].x, a.f[tt].y), b1 = pack64(a.f[tt].z, a.f[tt].w);
#pragma unroll
            for (int i = 0; i < RT; i++) {
                const v4i z = {0, 0, 0, 0};
                const v4i d0 = __builtin_amdgcn_mfma_i32_16x16x32_i8(wa[i][0], b0, z, 0, 0, 0);
                const v4i d1 = __builtin_amdgcn_mfma_i32_16x16x32_i8(wa[i][1], b1, z, 0, 0, 0);
                float* ac = acc[i][h * TH + tt];
#pragma unroll
                for (int e = 0; e < 4; e++) {
                    float u = (float)d0[e] * a.xs[tt].x;
                    u = fmaf((float)d1[e], a.xs[tt].y, u);
                    ac[e] = fmaf(u, ds[i][e], ac[e]);
                    ac[e] = fmaf(off[i][e], a.fs[tt], ac[e]);
                }
                if (DUMP) {
                    const uint32_t tok = 16 * (tt0 + h * TH + tt) + n;
#pragma unroll
                    for (int e = 0; e < 4; e++) {
                        const uint32_t row = 16 * (rt0 + i) + 4 * kq + e;
                        if (tok < t && row < w.n_out) {
                            if (2 * grp < nblk) dump[((size_t)tok * w.n_out + row) * nblk + 2 * grp] = d0[e];
                            if (2 * grp + 1 < nblk) dump[((size_t)tok * w.n_out + row) * nblk + 2 * grp + 1] = d1[e];
                        }
                    }
                }
            }
        }
    };

    if (s0 < s1) {
        // The next step's record is requested a step ahead and each phase's activation operands a phase ahead; past
        // the end the requests repeat the last valid address and are dropped.
        const uint32_t plast = 2 * PH * s1 - 1;
        uint4 c[RT], cnext[RT], dd[RT], oo[RT], dnext[RT], onext[RT];
        Act cur, nxt;
        load_codes(c, s0);
        load_scales(dd, oo, s0);
        load_act(cur, 2 * PH * s0);
        for (uint32_t s = s0; s < s1; s++) {
            load_codes(cnext, min(s + 1, s1 - 1));
            load_scales(dnext, onext, min(s + 1, s1 - 1));
#pragma unroll
            for (int ph = 0; ph < 2 * PH; ph++) {
                load_act(nxt, min(2 * PH * s + ph + 1, plast));
                compute(c, dd, oo, cur, 2 * s + ph / PH, ph / PH, ph % PH);
                cur = nxt;
            }
#pragma unroll
            for (int i = 0; i < RT; i++) {
                c[i] = cnext[i];
                dd[i] = dnext[i];
                oo[i] = onext[i];
            }
        }
    }

#pragma unroll
    for (int i = 0; i < RT; i++) {
        if (rt0 + i >= ntiles) continue;
#pragma unroll
        for (int tt = 0; tt < TT; tt++) {
            const uint32_t tok = 16 * (tt0 + tt) + n;
            if (tok >= t) continue;
#pragma unroll
            for (int e = 0; e < 4; e++) {
                const uint32_t row = 16 * (rt0 + i) + 4 * kq + e;
                if (row < w.n_out) y[(size_t)tok * w.n_out + row] = acc[i][tt][e];
            }
        }
    }
}

// Wave tiles on offer: {row tiles, token tiles, phases}. The pick spreads the (row tile, token tile) pairs evenly
// over the 1024 SIMDs at two waves each: time goes as the pairs the busiest SIMD works through; smaller tiles win ties
// (2 x 2 runs four waves per SIMD: 147 us per M = 512 shape against 160 with 2 x 8 and 168 with 2 x 4). Four row tiles per wave
// measured 1.6 to 2.5 times slower than two, one row tile 1.2 to 1.3 times, and are not offered.
struct Tile {
    uint32_t rt, tt, ph;
};
constexpr Tile TILES[] = {{2, 8, 2}, {2, 4, 1}, {2, 2, 1}};
constexpr int NTILES = sizeof(TILES) / sizeof(TILES[0]);

int pick_tile(uint32_t ntiles, uint32_t ttiles) {
#ifdef OXHIP_TUNING  // tuning builds only: tile index in OXHIP_I8_TILE
    if (const char* e = getenv("OXHIP_I8_TILE")) {
        const int v = atoi(e);
        if (v >= 0 && v < NTILES) return v;
    }
#endif
    int best = 0;
    uint64_t best_cost = ~0ull;
    for (int i = 0; i < NTILES; i++) {
        const Tile& c = TILES[i];
        const uint64_t waves = (uint64_t)((ntiles + c.rt - 1) / c.rt) * ((ttiles + c.tt - 1) / c.tt);
        const uint64_t cost = ((waves + 2047) / 2048) * c.rt * c.tt;
        if (cost <= best_cost) {  // ties go to the smaller tile: four waves per SIMD hide the operand requests' latency better than fewer loads do
            best_cost = cost;
            best = i;
        }
    }
    return best;
}

template <int RT, int TT, int PH>
void launch_tile(dim3 grid, hipStream_t s, const WeightView& w, const uint4* f, const float2* x2, const float* f1, uint32_t t, uint32_t ngrp,
                 float* y, int32_t* dump) {
    if (dump) gemm_i8_q4m_kernel<RT, TT, PH, true><<<grid, 256, 0, s>>>(w, f, x2, f1, t, ngrp, y, dump);
    else gemm_i8_q4m_kernel<RT, TT, PH, false><<<grid, 256, 0, s>>>(w, f, x2, f1, t, ngrp, y, dump);
}

}  // namespace

// Token slots (a multiple of the picked tile's tokens) and column groups the packed activations hold.
void gemm_i8_geometry(const WeightView& w, size_t t, size_t* slots, size_t* ngrp) {
    const uint32_t ttiles = (uint32_t)((t + 15) / 16);
    const Tile& c = TILES[pick_tile(row_tiles(w.n_out), ttiles)];
    *slots = (size_t)((ttiles + c.tt - 1) / c.tt) * c.tt * 16;
    *ngrp = 2 * (size_t)t4m_steps(w.n_in);
}

uint32_t gemm_i8_k_slices(const WeightView& w, size_t t) {
    const uint32_t ttiles = (uint32_t)((t + 15) / 16);
    const Tile& c = TILES[pick_tile(row_tiles(w.n_out), ttiles)];
    const size_t waves = (size_t)((row_tiles(w.n_out) + c.rt - 1) / c.rt) * ((ttiles + c.tt - 1) / c.tt);
    const uint32_t steps = t4m_steps(w.n_in);
    uint32_t z = 1;
    while (z < 8 && waves * z < 1024 && steps / (z * 2) >= 4) z *= 2;
    return z;
}

hipError_t launch_quantize_pack_i8(const void* x, bool src_bf16, size_t t, const WeightView& w, void* frag, void* xs, void* fs,
                                   hipStream_t s) {
    size_t slots, ngrp;
    gemm_i8_geometry(w, t, &slots, &ngrp);
    const size_t total = slots * ngrp;
    const unsigned grid = (unsigned)((total + 255) / 256);
    if (src_bf16)
        quantize_pack_i8_kernel<true><<<grid, 256, 0, s>>>(x, (uint32_t)t, w.n_in, (uint32_t)slots, (uint32_t)ngrp, static_cast<uint4*>(frag),
                                                           static_cast<float2*>(xs), static_cast<float*>(fs));
    else
        quantize_pack_i8_kernel<false><<<grid, 256, 0, s>>>(x, (uint32_t)t, w.n_in, (uint32_t)slots, (uint32_t)ngrp, static_cast<uint4*>(frag),
                                                            static_cast<float2*>(xs), static_cast<float*>(fs));
    return hipGetLastError();
}

// `y` receives gemm_i8_k_slices() partial results of t * n_out floats each (one when there is one slice);
// `dump` (optional) the exact block sums.
hipError_t launch_gemm_i8(const WeightView& w, const void* frag, const void* xs, const void* fs, size_t t, float* y, int32_t* dump,
                          hipStream_t s) {
    if (w.fmt != FMT_Q4M) return hipErrorInvalidValue;
    size_t slots, ngrp;
    gemm_i8_geometry(w, t, &slots, &ngrp);
    const uint32_t ttiles = (uint32_t)((t + 15) / 16);
    const int pick = pick_tile(row_tiles(w.n_out), ttiles);
    const Tile& c = TILES[pick];
    const uint32_t wrt = (row_tiles(w.n_out) + c.rt - 1) / c.rt;
    dim3 grid((wrt + 3) / 4, (unsigned)(slots / 16 / c.tt), gemm_i8_k_slices(w, t));
    const uint4* f = static_cast<const uint4*>(frag);
    const float2* x2 = static_cast<const float2*>(xs);
    const float* f1 = static_cast<const float*>(fs);
    const uint32_t tt = (uint32_t)t, ng = (uint32_t)ngrp;
    span_start(s);
    switch (pick) {
        case 0: launch_tile<2, 8, 2>(grid, s, w, f, x2, f1, tt, ng, y, dump); break;
        case 1: launch_tile<2, 4, 1>(grid, s, w, f, x2, f1, tt, ng, y, dump); break;
        default: launch_tile<2, 2, 1>(grid, s, w, f, x2, f1, tt, ng, y, dump); break;
    }
    span_stop(s);
    return hipGetLastError();
}

}  // namespace oxhip
