// Grouped expert matmuls of an MoE prefill pass on the bf16 matrix cores (the experts' forward_batched of the
// reference, src/moe.rs:625-828, over MLX 4-bit weights repacked as Q4 blocks, src/quant.rs:518-606).
//
// With a dozen or more routed tokens per expert the integer path (int8 activations, one scale per token and block of
// 32) spends a conversion and two to three multiply-adds per (row, token, block), and those, not the weights' bytes,
// bound it. Here the routed tokens of a chunk (up to 16 rows of one expert) go in as bf16 and a weight is the bf16
// value 128 + nibble, made by one byte permute per two weights (0x4300 | nibble); per group of 64 columns the matrix
// cores form D = sum (128 + nib) x and E = sum x exactly in f32, and
//     y += d D + (off - 136 d) E          (the group's weights are d (nib - 8) + off)
// costs two multiply-adds per (row, token, group). This is the reference's own prefill form: from 8 rows on its
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
template <bool ACT>
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
        const size_t col = 128 * (size_t)s + 32 * b + 4 * kq;
        float v[8];
#pragma unroll
        for (int h = 0; h < 2; h++) {
            const float4 a = *reinterpret_cast<const float4*>(x + r * ld + col + 16 * h);
            v[4 * h] = a.x; v[4 * h + 1] = a.y; v[4 * h + 2] = a.z; v[4 * h + 3] = a.w;
            if (ACT) {
                const float4 u = *reinterpret_cast<const float4*>(up + r * ld + col + 16 * h);
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

// Workgroup: 8 waves = 8 / kw groups of RT row tiles x kw waves that split the K steps (wave v takes steps v, v + kw, ...)
// and meet in LDS in wave order. grid x: runs of (8 / kw) RT row tiles; grid y: chunks {expert, first row, rows <= 16}.
// The chunk's fragments (4 KiB per step) are staged into LDS once per workgroup: all eight waves multiply the same
// rows (each wave asking memory for them costs more than the weights). out [gathered row][n_out] f32.
template <int RT>
__global__ __launch_bounds__(512, 4) void moe_bf16_kernel(WeightView w, const uint8_t* const* __restrict__ bases, const int4* __restrict__ chunks,
                                                          const int* __restrict__ nchunks, const uint4* __restrict__ afrag, uint32_t kw,
                                                          float* __restrict__ out) {
    extern __shared__ __align__(16) float lds[];  // fragments [step][4][64] x 16 B; then the waves' sums [wave][RT][64][4]
    const uint32_t c = blockIdx.y;
    if (c >= (uint32_t)*nchunks) return;  // uniform over the workgroup
    const int4 ch = chunks[c];
    const uint32_t first = (uint32_t)ch.y, rows = (uint32_t)ch.z;
    const uint32_t lane = threadIdx.x & 63, wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
    const uint32_t n = lane & 15;
    const uint32_t nsteps = w.n_in / 128, ntiles = row_tiles(w.n_out);
    const uint32_t ng = 8 / kw, rg = wave / kw, kwave = wave % kw;
    const uint32_t tile0 = (blockIdx.x * ng + rg) * RT;
    const gbytes base = as_global(bases[ch.x]);
    gbytes wp[RT];
#pragma unroll
    for (int r = 0; r < RT; r++) wp[r] = base + (size_t)min(tile0 + r, ntiles - 1) * t4m_steps(w.n_in) * T4M_REC;
    const uint32_t cnt = (nsteps - kwave + kw - 1) / kw, ilast = cnt - 1;  // kw <= nsteps

    struct St {
        u32x4 w[RT];
    };
    // every request is unconditional (past the end the last step again): the compiler then knows how many are in flight
    auto load = [&](St& st, uint32_t i) {
        const uint32_t s = kwave + kw * min(i, ilast);
#pragma unroll
        for (int r = 0; r < RT; r++) st.w[r] = gload<u32x4>(wp[r] + (size_t)s * T4M_REC + 16 * lane);
    };
    // A record's scale words (per row: the two groups' f16 scales at +1024, their bf16 offsets at +1088): a request costs
    // the memory pipeline the same for 64 bytes as for 1 KiB, so one request per row tile serves two steps: lane group kq
    // asks for word kq & 1 of step i + (kq >> 1), and at each step every lane takes its row's two words from those lanes.
    const uint32_t kq = lane >> 4;
    auto load_scales = [&](uint32_t* sc, uint32_t i) {
        const uint32_t s = kwave + kw * min(i + (kq >> 1), ilast);
#pragma unroll
        for (int r = 0; r < RT; r++) sc[r] = gload<uint32_t>(wp[r] + (size_t)s * T4M_REC + 1024 + 64 * (kq & 1) + 4 * n);
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
        // E[g]: the group's sum of activations per token (every row's offset multiplies it)
        f32x4 E[2];
#pragma unroll
        for (int g = 0; g < 2; g++) {
            E[g] = f32x4{0.0f, 0.0f, 0.0f, 0.0f};
            E[g] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(a[2 * g], ones, E[g], 0, 0, 0);
            E[g] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(a[2 * g + 1], ones, E[g], 0, 0, 0);
        }
#pragma unroll
        for (int r = 0; r < RT; r++) {
            f32x4 D[2] = {f32x4{0.0f, 0.0f, 0.0f, 0.0f}, f32x4{0.0f, 0.0f, 0.0f, 0.0f}};
#pragma unroll
            for (int b = 0; b < 4; b++) {
                // byte j of the dword: low nibble = position 4 kq + j, high nibble = position 16 + 4 kq + j; bf16 0x43nn = 128 + nn
                const uint32_t wd = st.w[r][b], lo = wd & 0x0F0F0F0Fu, hi = (wd >> 4) & 0x0F0F0F0Fu;
                const u32x4 wb = {__builtin_amdgcn_perm(0x43434343u, lo, 0x04010400u), __builtin_amdgcn_perm(0x43434343u, lo, 0x04030402u),
                                  __builtin_amdgcn_perm(0x43434343u, hi, 0x04010400u), __builtin_amdgcn_perm(0x43434343u, hi, 0x04030402u)};
                D[b >> 1] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(a[b], __builtin_bit_cast(bf16x8, wb), D[b >> 1], 0, 0, 0);
            }
            const uint32_t dw = (uint32_t)__builtin_amdgcn_ds_bpermute((int)(4 * (32 * odd + n)), (int)sc[r]);
            const uint32_t ow = (uint32_t)__builtin_amdgcn_ds_bpermute((int)(4 * (32 * odd + 16 + n)), (int)sc[r]);
#pragma unroll
            for (int g = 0; g < 2; g++) {
                const float d = f16_bits_to_f32((uint16_t)(g ? dw >> 16 : dw & 0xFFFF));
                const float off = bf16_bits_to_f32((uint16_t)(g ? ow >> 16 : ow & 0xFFFF));
                const float cc = off - 136.0f * d;
#pragma unroll
                for (int i2 = 0; i2 < 4; i2++) acc[r][i2] = fmaf(cc, E[g][i2], fmaf(d, D[g][i2], acc[r][i2]));
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
    // D[token 4 kq + i][row n]: thread (group, r, lane) adds the group's waves in order and stores its four tokens
    for (uint32_t idx = threadIdx.x; idx < ng * RT * 64; idx += blockDim.x) {
        const uint32_t l = idx & 63, r = (idx >> 6) % RT, g = (idx >> 6) / RT;
        const uint32_t tile = (blockIdx.x * ng + g) * RT + r, row = tile * 16 + (l & 15);
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
bool moe_bf16_ok(const WeightView& w) { return w.fmt == FMT_Q4M && w.n_in % 128 == 0 && w.n_in >= 128 && w.n_in <= 4096; }

size_t moe_bf16_frag_bytes(size_t max_chunks, size_t n_in) { return max_chunks * (n_in / 128) * 4 * 64 * 16; }

// Fragments of x rows (rowmap: gathered row -> row of x; ld = n_in) for chunks of at most 16 rows.
hipError_t launch_moe_pack_bf16(const float* x, size_t n_in, const int* rowmap, const int4* chunks, const int* nchunks, uint32_t max_chunks,
                                void* frag, hipStream_t s) {
    if (!max_chunks) return hipSuccess;
    moe_pack_bf16_kernel<false><<<dim3((unsigned)(n_in / 128), max_chunks), 256, 0, s>>>(x, nullptr, n_in, rowmap, chunks, nchunks,
                                                                                       (uint32_t)(n_in / 128), 0, 0.0f, static_cast<uint4*>(frag));
    return hipGetLastError();
}

// Fragments of act(g) * u over the gathered rows (g, u rows `stride` floats apart).
hipError_t launch_moe_act_pack_bf16(const float* g, const float* u, size_t stride, size_t inter, uint32_t kind, float param, const int4* chunks,
                                    const int* nchunks, uint32_t max_chunks, void* frag, hipStream_t s) {
    if (!max_chunks) return hipSuccess;
    moe_pack_bf16_kernel<true><<<dim3((unsigned)(inter / 128), max_chunks), 256, 0, s>>>(g, u, stride, nullptr, chunks, nchunks,
                                                                                      (uint32_t)(inter / 128), kind, param, static_cast<uint4*>(frag));
    return hipGetLastError();
}

hipError_t launch_moe_bf16(const WeightView& w, const GroupView& g, uint32_t max_chunks, const void* frag, float* out, hipStream_t s) {
    if (!moe_bf16_ok(w)) return hipErrorInvalidValue;
    if (!max_chunks) return hipSuccess;
    const uint32_t nsteps = w.n_in / 128, ntiles = row_tiles(w.n_out);
    // a wave streams a whole row of records (kw = 1) unless that leaves fewer workgroups than two per CU
    uint32_t rt = 4, kw = 1;
    while (kw < 4 && nsteps / (2 * kw) >= 4 && (uint64_t)((ntiles + (8 / kw) * rt - 1) / ((8 / kw) * rt)) * max_chunks < 512) kw *= 2;
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
    const dim3 grid((ntiles + ng * rt - 1) / (ng * rt), max_chunks);
    hipError_t e = hipSuccess;
    auto go = [&](auto kern) {
        if (lds > 48 * 1024) e = hipFuncSetAttribute(reinterpret_cast<const void*>(kern), hipFuncAttributeMaxDynamicSharedMemorySize, (int)lds);
        if (e == hipSuccess) kern<<<grid, 512, lds, s>>>(w, g.bases, g.chunks, g.nchunks, static_cast<const uint4*>(frag), kw, out);
    };
    if (rt == 2) go(moe_bf16_kernel<2>);
    else go(moe_bf16_kernel<4>);
    return e != hipSuccess ? e : hipGetLastError();
}

}  // namespace oxhip
