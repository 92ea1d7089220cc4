// Decode (1..8 tokens) on the matrix cores: a dequant-fused skinny GEMM over int8 activations.
//
// The arithmetic is the CPU decode kernels' (QMat::rows_t1 / rows_tc, src/kernels.rs:1339-1369;
// dot_row_generic, src/ggml.rs:1288-1315 of the reference): exact int32 sums of int8 weight codes
// times int8 activations per block of 32, scaled in f32 by weight scale x activation scale, plus
// the min / offset terms over the exact f32 activation sums. Each (token, row) result depends on
// that token alone and is summed in a fixed order, so a token's row is bit-identical whatever
// the batch (the reference's batch invariance, src/ggml.rs:1829-1848).
//
// Mapping onto v_mfma_i32_16x16x64_i8 (D[m][n] += sum_k A[m][k] B[k][n], lane l = 16 kq + idx
// supplies 16 K-bytes of row idx of A and of column idx of B, and receives D[4 kq + i][idx]):
//   B = weights: column n is row n of a 16-row tile; a lane's bytes 0-7 are 8 codes of one block of
//       32 and bytes 8-15 the 8 codes of the next block at the same positions;
//   A = activations: row m = 8 half + token carries token's int8 values of block `half` of the pair
//       in the matching byte half and zeros in the other, so that D[8 half + token][n] is the
//       integer dot product of one whole block: one instruction yields 2 blocks x 8 tokens x 16
//       rows of exact block sums, and every output lane is useful at 8 tokens.
// Weights stream from HBM through a register ring (several 1 KiB records in flight per wave, see
// layout.hpp). The activations are staged once per workgroup into LDS: the int8 values in A-operand
// order (one conflict-free ds_read_b64 per instruction; reading them from global memory per record
// instead costs three times the weights' L2 requests and doubles the kernel's time), the per-block
// scales and sums transposed so that a lane reads the four tokens it owns with one ds_read_b128.
// Rows too long for LDS fall back to reading the int8 values from L2.
//
// A workgroup owns `rt` row tiles and splits K over `kw` waves per tile; the partial sums meet in
// LDS in a fixed order. No atomics, no second launch.
#include <cstdlib>

#include "internal.hpp"
#include "layout.hpp"

namespace oxhip {

typedef int v4i __attribute__((ext_vector_type(4)));

namespace {

// Records a wave keeps in flight. HBM delivers about 8 TB/s at about 2 us of loaded latency, so some 16 MB must be
// on request across the chip at any moment: about 4000 resident waves x PF KiB.
template <int FMT, int NT>
constexpr int pf_for() { return FMT == FMT_Q4_K ? 6 : 8; }

struct Meta4 {
    float xs[4];
    float c[4];
    float fs[4];
    int su[4];
};

// The kernels evaluate a block's contribution with the fewest f32 operations per (row, token):
//   Q8_0:  d * (xs * I)
//   Q4_K:  d * sc * (xs * U + c) - dmin * mn * fs,   c = 8 * (fs - xs * su)      [U = sum of unsigned nibbles * q]
//   MLX:   d * (xs * U + c) + off * fs,              c = -8 * xs * su
// which equal the reference's (s * xs) * (U - 8 su) + m * fs (src/ggml.rs:1288-1315, src/kernels.rs:1287-1297)
// up to f32 rounding; the integer sums U - 8 su themselves are exact (and are what the DUMP variant writes).
// LDS: xs | c | fs | su, each [nblk][TPAD] (c, fs only for the formats with sums; su only for DUMP)
template <int FMT, int TPAD, bool SUMS, bool DUMP, class RowOf>
__device__ __forceinline__ void stage_meta(const QActView& xa, uint32_t t, uint32_t nblk, float* lds, RowOf row_of) {
    float* xs = lds;
    float* cc = lds + (size_t)nblk * TPAD;
    float* fs = lds + (size_t)2 * nblk * TPAD;
    int* su = reinterpret_cast<int*>(lds + (size_t)3 * nblk * TPAD);
    for (uint32_t i = threadIdx.x; i < nblk * TPAD; i += blockDim.x) {
        uint32_t tok = i / nblk, b = i % nblk;  // consecutive threads read consecutive blocks of one token
        bool live = tok < t;
        size_t src = (live ? row_of(tok) : 0) * nblk + b;
        const float x = live ? xa.scales[src] : 0.0f;
        xs[b * TPAD + tok] = x;
        if (SUMS) {
            const int sq = live ? xa.sums[src] : 0;
            const float f = live ? xa.fsums[src] : 0.0f;
            cc[b * TPAD + tok] = FMT == FMT_Q4_K ? 8.0f * (f - x * (float)sq) : -8.0f * (x * (float)sq);
            fs[b * TPAD + tok] = f;
            if (DUMP) su[b * TPAD + tok] = sq;
        }
    }
}

template <int TPAD, bool SUMS, bool DUMP>
__device__ __forceinline__ void load_meta(const float* lds, uint32_t nblk, uint32_t b, uint32_t tok0, Meta4& m) {
    const float4 x = *reinterpret_cast<const float4*>(lds + (size_t)b * TPAD + tok0);
    m.xs[0] = x.x; m.xs[1] = x.y; m.xs[2] = x.z; m.xs[3] = x.w;
    if (SUMS) {
        const float4 c = *reinterpret_cast<const float4*>(lds + (size_t)nblk * TPAD + (size_t)b * TPAD + tok0);
        const float4 f = *reinterpret_cast<const float4*>(lds + (size_t)2 * nblk * TPAD + (size_t)b * TPAD + tok0);
        m.c[0] = c.x; m.c[1] = c.y; m.c[2] = c.z; m.c[3] = c.w;
        m.fs[0] = f.x; m.fs[1] = f.y; m.fs[2] = f.z; m.fs[3] = f.w;
        if (DUMP) {
            const int4 q = *reinterpret_cast<const int4*>(lds + (size_t)3 * nblk * TPAD + (size_t)b * TPAD + tok0);
            m.su[0] = q.x; m.su[1] = q.y; m.su[2] = q.z; m.su[3] = q.w;
        }
    }
}

}  // namespace

// Everything one K-step needs from global memory, loaded a ring-length ahead of its use: the
// record's 16 bytes of codes for this lane, the scales of its row, and the int8 activations this
// lane feeds to the A operand (two dwords per MFMA).
template <int FMT>
struct Step;
template <>
struct Step<FMT_Q8_0> {
    uint4 w;
    uint32_t dd;
    uint32_t a[2];
};
template <>
struct Step<FMT_Q4_K> {
    uint4 w;
    uint32_t sc4, mn4, dd;
    uint32_t a[4];
};
template <>
struct Step<FMT_Q4M> {
    uint4 w;
    uint32_t dd, oo;
    uint32_t a[4];
};

// FMT: FMT_Q8_0 / FMT_Q4_K / FMT_Q4M. NT: tokens handled (1, 2, 4 or 8). DUMP: also write the exact
// integer block sums to `dump` ([t][n_out][n_in/32]) for parity checks.
// GROUPED: blockIdx.y walks the chunks of a grouped launch (MoE experts over their routed tokens): chunk c is
// {expert, first row, rows (<= 8)}; the weights are expert's, activation row i of the chunk is row
// rowmap[first + i] of xa (or first + i without a map), and its output is row first + i of y.
// ALDS: the int8 activations are staged into LDS in operand order (the launcher checks that they fit).
template <int FMT, int NT, bool DUMP, bool GROUPED, bool ALDS>
__global__ __launch_bounds__(1024) void decode_mfma_kernel(WeightView w, QActView xa, uint32_t t, uint32_t rt, uint32_t kw,
                                                           float* __restrict__ y, int32_t* __restrict__ dump, GroupView grp) {
    constexpr int TPAD = NT <= 4 ? 4 : 8;
    constexpr int NI = NT < 4 ? NT : 4;          // accumulator registers that hold live tokens
    constexpr bool SUMS = FMT != FMT_Q8_0;
    extern __shared__ float lds_all[];
    const uint32_t lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
    const uint32_t n = lane & 15, kq = lane >> 4;  // B / D role: row n of the tile; A role: slot n
    const uint32_t nblk = w.n_in / 32;
    const uint32_t r = wave / kw, ks = wave % kw;
    const uint32_t tile = blockIdx.x * rt + r;
    const uint32_t ntiles = row_tiles(w.n_out);
    // LDS: [operand-order activations: 512 B per pair of blocks] [scales, sums] [partial sums]; with ALDS the
    // partial sums reuse the activations' space once every wave is done with them
    const uint32_t nmf = (nblk + 1) / 2;
    uint2* afr = reinterpret_cast<uint2*>(lds_all);
    float* lds = lds_all + (ALDS ? (size_t)nmf * 128 : 0);
    float* red = ALDS ? lds_all : lds + (size_t)(SUMS ? (DUMP ? 4 : 3) : 1) * nblk * TPAD;  // [rt * kw][TPAD][16]
    uint32_t row0 = 0;  // first activation / output row of this launch unit
    if (GROUPED) {
        if (blockIdx.y >= (uint32_t)*grp.nchunks) return;  // uniform over the workgroup
        const int4 ch = grp.chunks[blockIdx.y];
        w.p0 = grp.bases[ch.x];
        row0 = (uint32_t)ch.y;
        t = (uint32_t)ch.z;
        y += (size_t)row0 * w.n_out;
    }
    auto src_row = [&](uint32_t i) -> size_t { return GROUPED && grp.rowmap ? (size_t)grp.rowmap[row0 + i] : (size_t)row0 + i; };

    // A role: slot n of this lane = (half, token); tokens past t read token t - 1 (their sums are dropped)
    const uint32_t a_half = n >> 3, a_tok = min(n & 7u, t - 1);
    const int8_t* xrow = xa.q + src_row(a_tok) * w.n_in;
    const uint32_t amask0 = a_half ? 0u : 0xFFFFFFFFu, amask1 = ~amask0;
    // D role: this lane's registers are tokens 4 (kq & 1) + i of block parity kq >> 1
    const uint32_t d_half = kq >> 1, d_tok0 = 4 * (kq & 1);

    const uint32_t nsteps = FMT == FMT_Q8_0 ? t8_steps(w.n_in) : (FMT == FMT_Q4_K ? 2 * tk4_sbs(w.n_in) : t4m_steps(w.n_in));
    const uint32_t per = (nsteps + kw - 1) / kw;
    const uint32_t s0 = ks * per;
    const uint32_t s1 = tile < ntiles ? min(nsteps, s0 + per) : 0;  // a tile past the matrix streams nothing
    const uint8_t* base = w.p0 + (size_t)min(tile, ntiles - 1) * (FMT == FMT_Q8_0   ? (size_t)nsteps * T8_REC
                                                                  : FMT == FMT_Q4_K ? (size_t)(nsteps / 2) * TK4_REC
                                                                                    : (size_t)nsteps * T4M_REC);

    auto act2 = [&](uint32_t b, uint32_t pos, uint32_t* out) {  // 8 consecutive activations of block b
        const uint2 v = *reinterpret_cast<const uint2*>(xrow + min(b, nblk - 1) * 32 + pos);
        out[0] = v.x;
        out[1] = v.y;
    };
    auto load_step = [&](Step<FMT>& st, uint32_t s) {
        if constexpr (FMT == FMT_Q8_0) {
            const uint8_t* rec = base + (size_t)s * T8_REC;
            st.w = *reinterpret_cast<const uint4*>(rec + 16 * lane);
            st.dd = *reinterpret_cast<const uint32_t*>(rec + 1024 + 4 * n);
            if (!ALDS) act2(2 * s + a_half, 8 * kq, st.a);
        } else if constexpr (FMT == FMT_Q4_K) {
            const uint8_t* rec = base + (size_t)(s >> 1) * TK4_REC;
            st.w = *reinterpret_cast<const uint4*>(rec + (s & 1) * 1024 + 16 * lane);
            // this step's four sub-blocks are 4 (s & 1) .. + 3 of the super-block
            st.sc4 = *reinterpret_cast<const uint32_t*>(rec + 2048 + 16 * n + 4 * (s & 1));
            st.mn4 = *reinterpret_cast<const uint32_t*>(rec + 2048 + 16 * n + 8 + 4 * (s & 1));
            st.dd = *reinterpret_cast<const uint32_t*>(rec + 2304 + 4 * n);
            if (!ALDS) {
                act2(4 * s + a_half, 8 * kq, st.a);
                act2(4 * s + 2 + a_half, 8 * kq, st.a + 2);
            }
        } else {
            const uint8_t* rec = base + (size_t)s * T4M_REC;
            st.w = *reinterpret_cast<const uint4*>(rec + 16 * lane);
            st.dd = *reinterpret_cast<const uint32_t*>(rec + 1024 + 4 * n);
            st.oo = *reinterpret_cast<const uint32_t*>(rec + 1088 + 4 * n);
            if (!ALDS) {
#pragma unroll
                for (int g = 0; g < 2; g++) {  // positions 4 kq.. and 16 + 4 kq.. of block 4 s + 2 g + half
                    const int8_t* xb = xrow + min(4 * s + 2 * g + a_half, nblk - 1) * 32;
                    st.a[2 * g] = *reinterpret_cast<const uint32_t*>(xb + 4 * kq);
                    st.a[2 * g + 1] = *reinterpret_cast<const uint32_t*>(xb + 16 + 4 * kq);
                }
            }
        }
    };

    float acc[4] = {0.0f, 0.0f, 0.0f, 0.0f};
    // `m`: index of the instruction along K (pair of blocks 2 m, 2 m + 1); with ALDS its operand comes from LDS
    auto mfma = [&](v4i bw, uint32_t m, uint32_t d0, uint32_t d1) -> v4i {
        if (ALDS) {
            const uint2 av = afr[(size_t)m * 64 + lane];
            d0 = av.x;
            d1 = av.y;
        }
        v4i a = {(int)(d0 & amask0), (int)(d1 & amask0), (int)(d0 & amask1), (int)(d1 & amask1)};
        v4i c = {0, 0, 0, 0};
        return __builtin_amdgcn_mfma_i32_16x16x64_i8(a, bw, c, 0, 0, 0);
    };
    auto dump_block = [&](uint32_t b, const int* isum) {
        if (!DUMP) return;
        const uint32_t row = tile * 16 + n;
        if (b >= nblk || row >= w.n_out) return;
#pragma unroll
        for (int i = 0; i < 4; i++)
            if (d_tok0 + i < t) dump[((size_t)(d_tok0 + i) * w.n_out + row) * nblk + b] = isum[i];
    };
    auto compute_step = [&](const Step<FMT>& st, uint32_t s) {
        const uint4 c = st.w;
        if constexpr (FMT == FMT_Q8_0) {
            const float d = f16_bits_to_f32((uint16_t)(d_half ? st.dd >> 16 : st.dd & 0xFFFF));
            v4i bw = {(int)c.x, (int)c.y, (int)c.z, (int)c.w};
            v4i D = mfma(bw, s, st.a[0], st.a[1]);
            const uint32_t b = 2 * s + d_half;
            Meta4 m;
            load_meta<TPAD, SUMS, DUMP>(lds, nblk, min(b, nblk - 1), d_tok0, m);
            int isum[4] = {D.x, D.y, D.z, D.w};
#pragma unroll
            for (int i = 0; i < NI; i++) acc[i] = fmaf(d, m.xs[i] * (float)isum[i], acc[i]);
            dump_block(b, isum);
        } else if constexpr (FMT == FMT_Q4_K) {
            const float d = f16_bits_to_f32((uint16_t)(st.dd & 0xFFFF)), ndmin = -f16_bits_to_f32((uint16_t)(st.dd >> 16));
            float P[4] = {0.0f, 0.0f, 0.0f, 0.0f}, Q[4] = {0.0f, 0.0f, 0.0f, 0.0f};
#pragma unroll
            for (int pr = 0; pr < 2; pr++) {  // the two byte pairs of the lane's chunk
                const uint32_t lo = pr ? c.z : c.x, hi = pr ? c.w : c.y;
                v4i bw = {(int)(lo & 0x0F0F0F0Fu), (int)(hi & 0x0F0F0F0Fu), (int)((lo >> 4) & 0x0F0F0F0Fu),
                          (int)((hi >> 4) & 0x0F0F0F0Fu)};
                v4i D = mfma(bw, 2 * s + pr, st.a[2 * pr], st.a[2 * pr + 1]);
                const uint32_t b = 4 * s + 2 * pr + d_half;  // global index of this lane's block of 32
                const uint32_t q = 2 * pr + d_half;
                const float sc = (float)((st.sc4 >> (8 * q)) & 0xFF), mn = (float)((st.mn4 >> (8 * q)) & 0xFF);
                Meta4 m;
                load_meta<TPAD, SUMS, DUMP>(lds, nblk, b, d_tok0, m);
                const int U[4] = {D.x, D.y, D.z, D.w};
#pragma unroll
                for (int i = 0; i < NI; i++) {
                    P[i] = fmaf(sc, fmaf(m.xs[i], (float)U[i], m.c[i]), P[i]);
                    Q[i] = fmaf(mn, m.fs[i], Q[i]);
                }
                if (DUMP) {
                    int isum[4] = {U[0] - 8 * m.su[0], U[1] - 8 * m.su[1], U[2] - 8 * m.su[2], U[3] - 8 * m.su[3]};
                    dump_block(b, isum);
                }
            }
#pragma unroll
            for (int i = 0; i < NI; i++) acc[i] = fmaf(ndmin, Q[i], fmaf(d, P[i], acc[i]));
        } else {
#pragma unroll
            for (int g = 0; g < 2; g++) {  // the two groups of 64 of the step
                const uint32_t w0 = g ? c.z : c.x, w1 = g ? c.w : c.y;  // blocks 2 g, 2 g + 1
                v4i bw = {(int)(w0 & 0x0F0F0F0Fu), (int)((w0 >> 4) & 0x0F0F0F0Fu), (int)(w1 & 0x0F0F0F0Fu),
                          (int)((w1 >> 4) & 0x0F0F0F0Fu)};
                v4i D = mfma(bw, 2 * s + g, st.a[2 * g], st.a[2 * g + 1]);
                const uint32_t b = 4 * s + 2 * g + d_half;
                const float d = f16_bits_to_f32((uint16_t)(g ? st.dd >> 16 : st.dd & 0xFFFF));
                const float off = bf16_bits_to_f32((uint16_t)(g ? st.oo >> 16 : st.oo & 0xFFFF));
                Meta4 m;
                load_meta<TPAD, SUMS, DUMP>(lds, nblk, min(b, nblk - 1), d_tok0, m);
                const int U[4] = {D.x, D.y, D.z, D.w};
                if (b < nblk) {  // padding blocks hold zero codes and zero scales, but their staged sums are a real block's
#pragma unroll
                    for (int i = 0; i < NI; i++) acc[i] = fmaf(off, m.fs[i], fmaf(d, fmaf(m.xs[i], (float)U[i], m.c[i]), acc[i]));
                }
                if (DUMP) {
                    int isum[4] = {U[0] - 8 * m.su[0], U[1] - 8 * m.su[1], U[2] - 8 * m.su[2], U[3] - 8 * m.su[3]};
                    dump_block(b, isum);
                }
            }
        }
    };

    // The first ring of records is requested before anything else, so that HBM latency overlaps the
    // staging of the activation scales.
    constexpr int PF = pf_for<FMT, NT>();
    Step<FMT> ring[PF];
#pragma unroll
    for (int p = 0; p < PF; p++)
        if (s0 + p < s1) load_step(ring[p], s0 + p);
    stage_meta<FMT, TPAD, SUMS, DUMP>(xa, t, nblk, lds, src_row);
    if (ALDS) {
        // slot (m, lane) of the operand array: lane = 16 kq + 8 half + token holds the 8 values of block 2 m + half
        // that the weights' lane group kq pairs with (Q4: positions 4 kq.. and 16 + 4 kq..; else 8 kq..). A thread
        // moves 16 (Q4: 32) consecutive bytes of one token's row, so the global reads are whole lines. Absent tokens
        // and a padding block keep whatever LDS holds: those products meet zero weights or are dropped.
        if (FMT == FMT_Q4M) {
            for (uint32_t i = threadIdx.x; i < t * nblk; i += blockDim.x) {
                const uint32_t tok = i / nblk, b = i % nblk;
                const uint4* xb = reinterpret_cast<const uint4*>(xa.q + src_row(tok) * w.n_in + (size_t)b * 32);
                const uint4 lo = xb[0], hi = xb[1];
                uint2* dst = afr + (size_t)(b >> 1) * 64 + 8 * (b & 1) + tok;
                dst[0] = make_uint2(lo.x, hi.x);
                dst[16] = make_uint2(lo.y, hi.y);
                dst[32] = make_uint2(lo.z, hi.z);
                dst[48] = make_uint2(lo.w, hi.w);
            }
        } else {
            for (uint32_t i = threadIdx.x; i < t * 2 * nblk; i += blockDim.x) {
                const uint32_t tok = i / (2 * nblk), c = i % (2 * nblk), b = c >> 1;
                const uint4 v = *reinterpret_cast<const uint4*>(xa.q + src_row(tok) * w.n_in + (size_t)c * 16);
                uint2* dst = afr + (size_t)(b >> 1) * 64 + 32 * (c & 1) + 8 * (b & 1) + tok;
                dst[0] = make_uint2(v.x, v.y);
                dst[16] = make_uint2(v.z, v.w);
            }
        }
    }
    __syncthreads();
    // each slot is refilled as soon as its record has been consumed, so PF - 1 records stay on request
    for (uint32_t sb = s0; sb < s1; sb += PF) {
#pragma unroll
        for (int p = 0; p < PF; p++) {
            if (sb + p < s1) compute_step(ring[p], sb + p);
            if (sb + PF + p < s1) load_step(ring[p], sb + PF + p);
        }
    }
    // the two block parities of a token meet across lane groups kq and kq ^ 2
#pragma unroll
    for (int i = 0; i < 4; i++) acc[i] += __shfl_xor(acc[i], 32);
    if (ALDS) __syncthreads();  // the partial sums overwrite the staged activations
    if (kq < 2) {
#pragma unroll
        for (int i = 0; i < 4; i++)
            if (d_tok0 + i < (uint32_t)TPAD) red[((size_t)wave * TPAD + d_tok0 + i) * 16 + n] = acc[i];
    }
    __syncthreads();
    // K-slices in order
    for (uint32_t idx = threadIdx.x; idx < rt * TPAD * 16; idx += blockDim.x) {
        const uint32_t rr = idx / (TPAD * 16), tok = (idx / 16) % TPAD, nn = idx % 16;
        const uint32_t row = (blockIdx.x * rt + rr) * 16 + nn;
        if (tok >= t || row >= w.n_out || !y) continue;
        float sum = 0.0f;
        for (uint32_t k = 0; k < kw; k++) sum += red[((size_t)(rr * kw + k) * TPAD + tok) * 16 + nn];
        y[(size_t)tok * w.n_out + row] = sum;
    }
}

namespace {

struct Shape {
    uint32_t rt, kw;
};

// Waves per workgroup (rt row tiles x kw K slices, 16 waves when the matrix allows) and how they split. A function
// of the weight's shape only, so a row's sum is associated the same way whatever the batch or launch kind.
// K is split as far as each wave keeps about four records; then row tiles are added per workgroup until the
// workgroups fit the chip at once (256 CUs, one 16-wave workgroup each), so that the whole matrix is on request
// from the first microsecond instead of in successive generations of workgroups.
Shape shape_for(uint32_t ntiles, uint32_t nsteps) {
    uint32_t kw = 1;
    while (kw < 16 && nsteps / (kw * 2) >= 4) kw *= 2;
    uint32_t rt = 16 / kw;
    while (kw > 1 && (ntiles + rt - 1) / rt > 256) {
        kw /= 2;
        rt *= 2;
    }
    if (const char* e = getenv("OXHIP_DECODE_KW")) {  // developer override for tuning runs
        uint32_t v = (uint32_t)atoi(e);
        if (v == 1 || v == 2 || v == 4 || v == 8 || v == 16) {
            kw = v;
            rt = 16 / kw;
        }
    }
    return Shape{rt, kw};
}

constexpr size_t LDS_MAX = 160 * 1024;

// Dynamic LDS of a launch; `alds` comes back false when the operand-order activations do not fit.
size_t lds_bytes(bool sums, bool dump, uint32_t nblk, int tpad, const Shape& sh, bool* alds) {
    const size_t meta = (size_t)(sums ? (dump ? 4 : 3) : 1) * nblk * tpad * 4, red = (size_t)sh.rt * sh.kw * tpad * 16 * 4;
    const size_t act = (size_t)((nblk + 1) / 2) * 512;
    const size_t with = act + meta > red ? act + meta : red;  // the partial sums reuse the activations' space
    *alds = with <= LDS_MAX && act >= red;
    return *alds ? with : meta + red;
}

template <int FMT, int NT, bool DUMP, bool GROUPED>
hipError_t launch_one(bool alds, dim3 grid, dim3 block, size_t lds, hipStream_t s, const WeightView& w, const QActView& v, uint32_t t,
                      const Shape& sh, float* y, int32_t* dump, const GroupView& g) {
    hipError_t e = hipSuccess;
    auto go = [&](auto kern) {
        if (lds > 48 * 1024) e = hipFuncSetAttribute(reinterpret_cast<const void*>(kern), hipFuncAttributeMaxDynamicSharedMemorySize, (int)lds);
        if (e == hipSuccess) kern<<<grid, block, lds, s>>>(w, v, t, sh.rt, sh.kw, y, dump, g);
    };
    if (alds) go(decode_mfma_kernel<FMT, NT, DUMP, GROUPED, true>);
    else go(decode_mfma_kernel<FMT, NT, DUMP, GROUPED, false>);
    return e != hipSuccess ? e : hipGetLastError();
}

template <int FMT, bool DUMP>
hipError_t run(const WeightView& w, const QActView& xa, size_t t, float* y, int32_t* dump, hipStream_t s) {
    const uint32_t ntiles = row_tiles(w.n_out);
    const uint32_t nsteps = FMT == FMT_Q8_0 ? t8_steps(w.n_in) : (FMT == FMT_Q4_K ? 2 * tk4_sbs(w.n_in) : t4m_steps(w.n_in));
    const Shape sh = shape_for(ntiles, nsteps);
    const uint32_t nblk = w.n_in / 32;
    dim3 grid((ntiles + sh.rt - 1) / sh.rt), block(64 * sh.rt * sh.kw);
    size_t c0 = 0;
    while (c0 < t) {
        const size_t tc = t - c0 < 8 ? t - c0 : 8;
        QActView v = xa;
        v.q += c0 * w.n_in;
        v.scales += c0 * nblk;
        v.sums += c0 * nblk;
        v.fsums += c0 * nblk;
        float* yo = y ? y + c0 * w.n_out : nullptr;  // no output rows when only the block sums are wanted
        int32_t* du = dump ? dump + c0 * (size_t)w.n_out * nblk : nullptr;
        const int tpad = tc <= 4 ? 4 : 8;
        bool alds;
        const size_t lds = lds_bytes(FMT != FMT_Q8_0, DUMP, nblk, tpad, sh, &alds);
        if (lds > LDS_MAX) return hipErrorInvalidValue;  // rows too long for the staged activation scales
        const uint32_t tt = (uint32_t)tc;
        hipError_t e;
        if (tc == 1) e = launch_one<FMT, 1, DUMP, false>(alds, grid, block, lds, s, w, v, tt, sh, yo, du, GroupView{});
        else if (tc == 2) e = launch_one<FMT, 2, DUMP, false>(alds, grid, block, lds, s, w, v, tt, sh, yo, du, GroupView{});
        else if (tc <= 4) e = launch_one<FMT, 4, DUMP, false>(alds, grid, block, lds, s, w, v, tt, sh, yo, du, GroupView{});
        else e = launch_one<FMT, 8, DUMP, false>(alds, grid, block, lds, s, w, v, tt, sh, yo, du, GroupView{});
        if (e != hipSuccess) return e;
        c0 += tc;
    }
    return hipSuccess;
}

template <int FMT>
hipError_t run_grouped(const WeightView& w, const QActView& xa, const GroupView& g, uint32_t max_chunks, uint32_t max_rows,
                       float* y, hipStream_t s) {
    const uint32_t ntiles = row_tiles(w.n_out);
    const uint32_t nsteps = FMT == FMT_Q8_0 ? t8_steps(w.n_in) : (FMT == FMT_Q4_K ? 2 * tk4_sbs(w.n_in) : t4m_steps(w.n_in));
    // the same K split as a plain launch on this matrix, so that a row's sum is associated the same way
    // (and is bit-identical) whether its expert runs alone or in a group
    const Shape sh = shape_for(ntiles, nsteps);
    const uint32_t nblk = w.n_in / 32;
    dim3 grid((ntiles + sh.rt - 1) / sh.rt, max_chunks), block(64 * sh.rt * sh.kw);
    const int tpad = max_rows <= 4 ? 4 : 8;
    bool alds;
    const size_t lds = lds_bytes(FMT != FMT_Q8_0, false, nblk, tpad, sh, &alds);
    if (lds > LDS_MAX) return hipErrorInvalidValue;
    if (max_rows == 1) return launch_one<FMT, 1, false, true>(alds, grid, block, lds, s, w, xa, 0u, sh, y, nullptr, g);
    if (max_rows <= 4) return launch_one<FMT, 4, false, true>(alds, grid, block, lds, s, w, xa, 0u, sh, y, nullptr, g);
    return launch_one<FMT, 8, false, true>(alds, grid, block, lds, s, w, xa, 0u, sh, y, nullptr, g);
}

}  // namespace

hipError_t launch_decode_mfma_grouped(const WeightView& w, const QActView& xa, const GroupView& g, uint32_t max_chunks,
                                      uint32_t max_rows_per_chunk, float* y, hipStream_t s) {
    if (!max_chunks) return hipSuccess;
    switch (w.fmt) {
        case FMT_Q8_0: return run_grouped<FMT_Q8_0>(w, xa, g, max_chunks, max_rows_per_chunk, y, s);
        case FMT_Q4_K: return run_grouped<FMT_Q4_K>(w, xa, g, max_chunks, max_rows_per_chunk, y, s);
        case FMT_Q4M: return run_grouped<FMT_Q4M>(w, xa, g, max_chunks, max_rows_per_chunk, y, s);
        default: return hipErrorInvalidValue;
    }
}

hipError_t launch_decode_mfma(const WeightView& w, const QActView& xa, size_t t, float* y, hipStream_t s) {
    switch (w.fmt) {
        case FMT_Q8_0: return run<FMT_Q8_0, false>(w, xa, t, y, nullptr, s);
        case FMT_Q4_K: return run<FMT_Q4_K, false>(w, xa, t, y, nullptr, s);
        case FMT_Q4M: return run<FMT_Q4M, false>(w, xa, t, y, nullptr, s);
        default: return hipErrorInvalidValue;
    }
}

// The integer block sums the kernel forms ([t][n_out][n_in/32]); y is scratch of [t][n_out].
hipError_t launch_isums_mfma(const WeightView& w, const QActView& xa, size_t t, float* y, int32_t* out, hipStream_t s) {
    switch (w.fmt) {
        case FMT_Q8_0: return run<FMT_Q8_0, true>(w, xa, t, y, out, s);
        case FMT_Q4_K: return run<FMT_Q4_K, true>(w, xa, t, y, out, s);
        case FMT_Q4M: return run<FMT_Q4M, true>(w, xa, t, y, out, s);
        default: return hipErrorInvalidValue;
    }
}

}  // namespace oxhip
