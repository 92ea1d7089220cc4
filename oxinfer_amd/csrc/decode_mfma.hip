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
// A workgroup owns `rt` row tiles over one of `ksplit` slices of K (grid y) and splits its slice over `kw` waves
// per tile; the waves' partial sums meet in LDS in a fixed order. With more than one slice each workgroup leaves
// its partial rows in global scratch and the last one to arrive (a counter per row group) adds the slices in slice
// order: the association of a row's sum depends on the weight's shape only, never on arrival order, and there is
// no second launch. A workgroup stages only its slice of the activations. (That is the plain mapping of a launch of one
// matmul; a shared launch with enough work gives a workgroup several slices and a wave several waves' shares, each summed
// apart as before: see decode_body's Mapping and place_job.)
#include <algorithm>
#include <atomic>
#include <cstdio>
#include <cstdlib>
#include <cstring>
#include <map>
#include <mutex>
#include <vector>

#include <hip/hip_ext.h>

#include "act_body.hpp"
#include "internal.hpp"
#include "layout.hpp"

namespace oxhip {

typedef int v4i __attribute__((ext_vector_type(4)));
typedef float v4f __attribute__((ext_vector_type(4)));

// Where slot `slot` (0..63) of row `row` of the LDS operand array sits: the staging stores of a token's consecutive chunks
// differ only in the row and in slot bits 3 and 5, which alone would put 64 lanes into two bank pairs; mixing the row's
// low bits into slot bits 0..2 and 4 spreads them over all banks, and a row's 64 slots stay a permutation of the row.
__device__ __forceinline__ uint32_t opslot(uint32_t row, uint32_t slot) { return slot ^ (row & 7u) ^ ((row & 8u) << 1); }

namespace {

// Records a wave keeps in flight. HBM delivers about 8 TB/s at about 2 us of loaded latency, so some 16 MB must be
// on request across the chip at any moment: about 4000 resident waves x PF KiB.
template <int FMT, int NT>
constexpr int pf_for() { return FMT == FMT_Q6_K ? 4 : 8; }  // Q6_K records are 1.7 KiB and its step needs the registers

// The kernels evaluate a block's contribution as the reference does (src/ggml.rs:1288-1315, src/kernels.rs:1287-1297):
//   Q8_0:        d * (xs * I)                                  I = sum of codes * activation codes (exact)
//   4-bit:       (s / 16) * (xs * I16) + m * fs                I16 = 16 * sum of (nibble - 8) * activation codes (exact)
//                Q4_K: s = d * sc, m = 8 s - dmin * mn (decode_i8's s and m);  MLX: s = d, m = the group's offset
// up to the order of the f32 operations. The centred nibbles go to the matrix cores as the int8 values 16 * (nibble - 8)
// (a nibble moved to the top of its byte with its top bit flipped), so the integer sum needs no correction by the
// activations' own sums; the DUMP variant writes I16 / 16. The m * fs terms of a step's four blocks are one more
// matrix instruction (f32, 16 x 16 x 4: rows = tokens, K = the four blocks), straight into the accumulators.
// LDS metadata: xs [nbl][TPAD], and for the formats with mins or offsets fs [nbl][TPAD], over the workgroup's nbl
// blocks from b0. Q6_K keeps its own three arrays (see its step).
// `at`: index of the lane's first token in its block's row
__device__ __forceinline__ void load_xs(const float* lds, uint32_t at, float* xs) {
    const float4 x = *reinterpret_cast<const float4*>(lds + at);
    xs[0] = x.x; xs[1] = x.y; xs[2] = x.z; xs[3] = x.w;
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
    uint32_t a[2];
};
template <>
struct Step<FMT_Q8F> {
    uint4 w;
    uint32_t a[2];
};
template <>
struct Step<FMT_Q4_K> {
    uint4 w;
    uint32_t a[4];
};
template <>
struct Step<FMT_Q5_K> {
    uint4 w;
    uint32_t h;  // the fifth bits of the lane's 32 codes
    uint32_t a[4];
};
template <>
struct Step<FMT_Q4M> {
    uint4 w;
    uint32_t a[4];
};
template <>
struct Step<FMT_Q40> {
    uint4 w;
    uint32_t a[4];
};
template <>
struct Step<FMT_MXFP4> {
    uint4 w;
    uint32_t a[4];
};
template <>
struct Step<FMT_Q6_K> {
    uint4 w;   // low nibbles
    uint2 h;   // high bit pairs
    uint32_t a[1];
};

// FMT: FMT_Q8_0 / FMT_Q8F (the same codes with f32 scales) / FMT_Q4_K / FMT_Q6_K / FMT_Q4M. NT: tokens handled (1, 2, 4 or 8). DUMP: also write the exact
// integer block sums to `dump` ([t][n_out][n_in/32]) for parity checks.
// GROUPED: blockIdx.y walks the chunks of a grouped launch (MoE experts over their routed tokens): chunk c is
// {expert, first row, rows (<= 8 NG)}; the weights are expert's, activation row i of the chunk is row
// rowmap[first + i] of xa (or first + i without a map), and its output is row first + i of y.
// ALDS: the int8 activations are staged into LDS in operand order (the launcher checks that they fit).
// `bx`, `by`: the workgroup's place in its launch unit (row group; K slice or chunk); `nthr` threads take
// part (a launch may hold more: those waves have left before the first barrier); `lds_all`: the dynamic LDS.
// `kw` and `ksplit` say how a row's sum is associated: K is cut into ksplit slices of kw runs each, a run is summed
// step by step, a slice's runs are added in order, and the slices in order. Who sums a run is a separate matter
// (Mapping): in the plain mapping a wave has one run and a workgroup one slice (64 rt kw threads); a dense launch may
// instead give a workgroup `fs` consecutive slices and a tile `kwp` waves, each of which then streams fs kw / kwp
// consecutive runs in one go, leaving every run's sums apart. The bits are the same; the workgroups are fewer and fatter.
// NG (grouped launches of 8 tokens per group): a chunk holds up to 8 NG rows; every weight record is used for NG
// instructions, one per group of 8 tokens, before the next is touched.
struct Mapping {
    uint32_t kwp = 0;  // waves per tile (0: kw, one run per wave)
    uint32_t fs = 0;   // K slices per workgroup (0: one)
};

template <int FMT, int NT, bool DUMP, bool GROUPED, bool ALDS, int NG = 1, bool REMAP = false>
__device__ __forceinline__ void decode_body(WeightView w, QActView xa, uint32_t t, uint32_t rt, uint32_t kw, float* __restrict__ y,
                                            int32_t* __restrict__ dump, GroupView grp, uint32_t ksplit, float* __restrict__ partial,
                                            uint32_t* __restrict__ counters, uint32_t bx, uint32_t by, uint32_t nthr,
                                            float* __restrict__ lds_all, Epi epi = Epi{}, Mapping map = Mapping{}) {
    static_assert(NG == 1 || (GROUPED && ALDS && !DUMP && NT == 8), "token groups are for grouped launches");
    static_assert(!REMAP || (!GROUPED && !DUMP && ALDS && NG == 1), "other mappings are for dense launches over staged activations");
    constexpr int TPAD = NT <= 4 ? 4 : 8;
    // the swizzled operand array pays at 8 tokens (where the staging stores are many); at fewer its address math costs more
    constexpr bool SWZ = NT >= 8;
    constexpr int NI = NT < 4 ? NT : 4;          // accumulator registers that hold live tokens
    constexpr bool MINS = k45_format(FMT) || FMT == FMT_Q4M;   // m * fs terms (Q4_0 has none)
    constexpr int NARR = q8_format(FMT) || FMT == FMT_Q40 || FMT == FMT_MXFP4 ? 1 : FMT == FMT_Q6_K ? (DUMP ? 4 : 3) : 2;  // metadata arrays
    // the wave index and everything derived from it (tile, K range) live in scalar registers: branches on them are
    // scalar, and the load counters the compiler keeps stay exact across them
    const uint32_t lane = threadIdx.x & 63, wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
    const uint32_t n = lane & 15, kq = lane >> 4;  // B / D role: row n of the tile; A role: slot n
    const uint32_t nblk = w.n_in / 32;
    // kw and the number of K slices are powers of two (the launchers see to it): shifts, where a division by a value only
    // known at run time costs some twenty instructions even when it is the same for the whole wave
    const uint32_t kwsh = (uint32_t)__builtin_ctz(kw), kssh = (uint32_t)__builtin_ctz(ksplit);
    // the mapping: kwp waves per tile and fs slices per workgroup (both powers of two); runs of a tile in the workgroup, runs
    // per wave. Launchers only leave the plain mapping when every run has the same number of steps.
    const uint32_t kwp = REMAP && map.kwp ? map.kwp : kw, fs = REMAP && map.fs ? map.fs : 1u;
    const uint32_t runs = fs << kwsh, rpw = runs >> __builtin_ctz(kwp);
    const uint32_t r = wave >> __builtin_ctz(kwp), kj = wave & (kwp - 1);
    // (fused gate / up experts: the first rt / 2 tiles of the workgroup are gate tiles, the others the up tiles of the same rows;
    // a gate / up pair of two matrices likewise: the first rt / 2 waves' tiles come from `w`, the others' from epi.pair_p0)
    const bool glu = GROUPED && grp.glu_inter != 0;
    const bool pair = !GROUPED && !DUMP && epi.pair_p0 != nullptr;
    const uint32_t ghalf = rt >> 1, gtiles = grp.glu_inter / 16;
    const uint32_t tile = glu    ? (r < ghalf ? bx * ghalf + r : gtiles + bx * ghalf + (r - ghalf))
                          : pair ? bx * ghalf + (r < ghalf ? r : r - ghalf)
                                 : bx * rt + r;
    const uint32_t ntiles = glu && r < ghalf ? gtiles : row_tiles(w.n_out);
    // this workgroup's slice of K: steps [S0, S1), blocks [B0, B0 + nbl) (a multiple of 4 blocks)
    constexpr uint32_t BPS = q8_format(FMT) ? 2 : 4;  // blocks of 32 per step
    constexpr uint32_t K45_REC = FMT == FMT_Q5_K ? TK5_REC : TK4_REC, T4_REC = FMT == FMT_MXFP4 ? T4X_REC : T4M_REC;
    const uint32_t nsteps = q8_format(FMT)    ? t8_steps(w.n_in)
                            : k45_format(FMT) ? 2 * tk4_sbs(w.n_in)
                            : FMT == FMT_Q6_K ? t6k_steps(w.n_in)
                                              : t4m_steps(w.n_in);
    const uint32_t slice = GROUPED ? 0 : by;
    const uint32_t sl = (nsteps + ksplit - 1) >> kssh;
    const uint32_t S0 = min(nsteps, slice * fs * sl), S1 = min(nsteps, S0 + fs * sl);  // (the workgroup's fs slices)
    const uint32_t B0 = BPS * S0, nbl = BPS * fs * sl, M0 = B0 / 2;
    // LDS: [operand-order activations: 512 B per pair of blocks] [scales, sums] [partial sums]; with ALDS the
    // partial sums reuse the activations' space once every wave is done with them
    uint2* afr = reinterpret_cast<uint2*>(lds_all);  // [NG][nbl / 2][64]
    float* lds = lds_all + (ALDS ? (size_t)NG * (nbl / 2) * 128 : 0);
    const uint32_t nm = nbl * TPAD, as = NG * nm;  // scale entries of a token group; floats per array
    float* red = ALDS ? lds_all : lds + (size_t)NARR * as;  // [rt][runs][NG][TPAD][16]
    uint32_t row0 = 0;  // first activation / output row of this launch unit
    if (GROUPED) {
        if (grp.direct) {
            if (by >= grp.direct_n) return;  // uniform over the workgroup
            w.p0 = grp.bases[grp.direct[by]];
            row0 = by;
            t = 1;
        } else {
            if (by >= (uint32_t)*grp.nchunks) return;  // uniform over the workgroup
            const int4 ch = grp.chunks[by];
            w.p0 = grp.bases[ch.x];
            row0 = (uint32_t)ch.y;
            t = (uint32_t)ch.z;
        }
        y += (size_t)row0 * w.n_out;
    }
    auto src_row = [&](uint32_t i) -> size_t {
        if (GROUPED && grp.direct && grp.direct_x0) return 0;
        return GROUPED && grp.rowmap ? (size_t)grp.rowmap[row0 + i] : (size_t)row0 + i;
    };

    // A role: slot n of this lane = (half, token); tokens past t read token t - 1 (their sums are dropped)
    const uint32_t a_half = n >> 3, a_tok = min(n & 7u, t - 1);
    const int8_t* xrow = xa.q + src_row(a_tok) * w.n_in;
    const uint32_t amask0 = a_half ? 0u : 0xFFFFFFFFu, amask1 = ~amask0;
    // D role: this lane's registers are tokens 4 (kq & 1) + i of block parity kq >> 1
    const uint32_t d_half = kq >> 1, d_tok0 = 4 * (kq & 1);
    // Q4_K: the bytes this lane takes from a step's {scales, mins} words (v_perm_b32: 0..3 = the scales, 4..7 = the mins)
    const uint32_t q4k_sel = d_half | ((2 + d_half) << 8) | (kq << 16) | ((4 + kq) << 24);

    const uint32_t per = fs == 1 && rpw == 1 ? (S1 - S0 + kw - 1) >> kwsh : sl >> kwsh;  // steps of a run
    const uint32_t s0 = S0 + kj * rpw * per;
    const uint32_t s1 = tile < ntiles ? min(S1, s0 + rpw * per) : 0;  // a tile past the matrix streams nothing
    // (typed as global memory: a grouped launch reads w.p0 from the table of expert bases)
    const gbytes base = as_global(pair && r >= ghalf ? epi.pair_p0 : w.p0) + (size_t)min(tile, ntiles - 1) * (FMT == FMT_Q8_0   ? (size_t)nsteps * T8_REC
                                                                  : FMT == FMT_Q8F  ? (size_t)nsteps * T8F_REC
                                                                  : k45_format(FMT) ? (size_t)(nsteps / 2) * K45_REC
                                                                  : FMT == FMT_Q6_K ? (size_t)nsteps * T6K_REC
                                                                                    : (size_t)nsteps * T4_REC);

    auto act2 = [&](uint32_t b, uint32_t pos, uint32_t* out) {  // 8 consecutive activations of block b
        const uint2 v = *reinterpret_cast<const uint2*>(xrow + min(b, nblk - 1) * 32 + pos);
        out[0] = v.x;
        out[1] = v.y;
    };
    auto load_step = [&](Step<FMT>& st, uint32_t s) {
        if constexpr (q8_format(FMT)) {
            const gbytes rec = base + (size_t)s * (FMT == FMT_Q8F ? T8F_REC : T8_REC);
            st.w = gload_once<uint4>(rec + 16 * lane);
            if (!ALDS) act2(2 * s + a_half, 8 * kq, st.a);
        } else if constexpr (k45_format(FMT)) {
            const gbytes rec = base + (size_t)(s >> 1) * K45_REC;
            st.w = gload_once<uint4>(rec + (s & 1) * 1024 + 16 * lane);
            if constexpr (FMT == FMT_Q5_K) st.h = gload_once<uint32_t>(rec + TK4_REC + (s & 1) * 256 + 4 * lane);
            if (!ALDS) {
                act2(4 * s + a_half, 8 * kq, st.a);
                act2(4 * s + 2 + a_half, 8 * kq, st.a + 2);
            }
        } else if constexpr (FMT == FMT_Q6_K) {
            static_assert(FMT != FMT_Q6_K || ALDS, "Q6_K takes its activations from LDS");
            const gbytes rec = base + (size_t)s * T6K_REC;
            st.w = gload_once<uint4>(rec + 16 * lane);
            st.h = gload_once<uint2>(rec + 1024 + 8 * lane);
        } else {
            const gbytes rec = base + (size_t)s * T4_REC;
            st.w = gload_once<uint4>(rec + 16 * lane);
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

    // The records' scales: a request costs the memory pipeline the same for 64 bytes as for 1 KiB, and one per step
    // and scale word (1 to 3) would cost more than the weights themselves. So one request serves four steps: lane group
    // kq asks for the words of step `first + kq` (row n of it), and at step first + q every lane takes them from lane
    // 16 q + n. Q8_0: {d of the two blocks}; Q4_K: {four sub-block scales, four mins, (d, dmin)}: this step's four
    // sub-blocks are 4 (s & 1) .. + 3 of the super-block; MLX: {d of the two groups, offsets of the two groups}.
    // (The scale words are ordinary loads, not read-once ones like the codes: a record is not a whole number of cache lines,
    // so its scales share a line with the next record's first codes, and a line that came in as read-once is gone again
    // before its other half is asked for: Q6_K's launch fetched 7.5 % more than its records hold, one line per record.)
    constexpr int NM = FMT == FMT_Q8_0 || FMT == FMT_MXFP4 ? 1 : (k45_format(FMT) || FMT == FMT_Q6_K) ? 3 : 2;  // (Q8F: the two f32 scales)
    uint32_t slast = max(s1, 1u) - 1;
    // (Q6_K: with the clamp's bound opaque the compiler keeps 111 registers instead of 141 and a fourth wave per SIMD fits: the
    // shared launch of four Q6_K matmuls 47.9 -> 45.6 us. The other formats' kernels do not gain, Q4_0's loses.)
    if constexpr (FMT == FMT_Q6_K) asm volatile("" : "+v"(slast));
    auto load_scales = [&](uint32_t* m, uint32_t first) {
        const uint32_t s = min(first + kq, slast);
        if constexpr (FMT == FMT_Q8F) {
            m[0] = gload<uint32_t>(base + (size_t)s * T8F_REC + 1024 + 8 * n);
            m[1] = gload<uint32_t>(base + (size_t)s * T8F_REC + 1028 + 8 * n);
        } else if constexpr (FMT == FMT_Q8_0) {
            m[0] = gload<uint32_t>(base + (size_t)s * T8_REC + 1024 + 4 * n);
        } else if constexpr (k45_format(FMT)) {
            const gbytes rec = base + (size_t)(s >> 1) * K45_REC;
            m[0] = gload<uint32_t>(rec + 2048 + 16 * n + 4 * (s & 1));
            m[1] = gload<uint32_t>(rec + 2048 + 16 * n + 8 + 4 * (s & 1));
            m[2] = gload<uint32_t>(rec + 2304 + 4 * n);
        } else if constexpr (FMT == FMT_Q6_K) {  // {scales of sub-blocks 0..3, of 4..7, d}
            const gbytes rec = base + (size_t)s * T6K_REC;
            m[0] = gload<uint32_t>(rec + 1536 + 8 * n);
            m[1] = gload<uint32_t>(rec + 1540 + 8 * n);
            m[2] = gload<uint16_t>(rec + 1664 + 2 * n);
        } else if constexpr (FMT == FMT_MXFP4) {  // the four scale bytes of row n's blocks
            m[0] = gload<uint32_t>(base + (size_t)s * T4X_REC + 1024 + 4 * n);
        } else {
            const gbytes rec = base + (size_t)s * T4M_REC;
            m[0] = gload<uint32_t>(rec + 1024 + 4 * n);
            m[1] = gload<uint32_t>(rec + 1088 + 4 * n);
        }
    };
    const int take0 = (int)(4 * n);  // byte index of lane n for the lane-to-lane read; + 64 q: lane 16 q + n
    auto scales_of = [&](const uint32_t* grp, int q, uint32_t* m) {
#pragma unroll
        for (int j = 0; j < NM; j++) m[j] = (uint32_t)__builtin_amdgcn_ds_bpermute(take0 + 64 * q, (int)grp[j]);
    };

    float acc[NG][4];
#pragma unroll
    for (int g = 0; g < NG; g++)
#pragma unroll
        for (int i = 0; i < 4; i++) acc[g][i] = 0.0f;
    // the m * fs terms accumulate on their own (a chain of matrix instructions that depends on nothing else) and join at the end
    v4f macc[MINS ? NG : 1];
#pragma unroll
    for (int g = 0; g < (MINS ? NG : 1); g++) macc[g] = v4f{0.0f, 0.0f, 0.0f, 0.0f};
    // Q6_K: every lane group sums its own 16-column sub-block for tokens 4 tg + i
    float acc6a[4] = {0.0f, 0.0f, 0.0f, 0.0f}, acc6b[4] = {0.0f, 0.0f, 0.0f, 0.0f};  // tg = 0, 1
    // `m`: index of the instruction along K (pair of blocks 2 m, 2 m + 1); with ALDS its operand comes from LDS
    auto mfma = [&](v4i bw, uint32_t m, int tg, uint32_t d0, uint32_t d1) -> v4i {
        v4i c = {0, 0, 0, 0};
        if (ALDS) {
            const uint2 av = afr[((size_t)tg * (nbl / 2) + (m - M0)) * 64 + (SWZ ? opslot(m - M0, lane) : lane)];
            d0 = av.x;
            d1 = av.y;
        }
        v4i a = {(int)(d0 & amask0), (int)(d1 & amask0), (int)(d0 & amask1), (int)(d1 & amask1)};
        return __builtin_amdgcn_mfma_i32_16x16x64_i8(a, bw, c, 0, 0, 0);
    };
    // The m * fs terms of the step's four blocks (blocks b4 .. b4 + 3): rows = tokens (8 .. 15: none), K = the blocks;
    // this lane supplies fs of (token n, block b4 + kq) and `mk`, row n's m of block b4 + kq. D[4 kq + i][n]: the lane
    // groups 0 and 1 receive the tokens their accumulators hold, the others zeros.
    auto mins = [&](uint32_t b4, float mk) {
        if constexpr (MINS) {
            // (a block past the row lies inside the slice's arrays all the same, staged as zero)
            const uint32_t at = (b4 + kq - B0) * TPAD + min(n, (uint32_t)TPAD - 1);
#pragma unroll
            for (int tg = 0; tg < NG; tg++) {
                const float f = lds[(size_t)as + tg * nm + at];
                macc[tg] = __builtin_amdgcn_mfma_f32_16x16x4f32(n < (uint32_t)TPAD ? f : 0.0f, mk, macc[tg], 0, 0, 0);
            }
        }
    };
    // a nibble moved to the top of its byte with its top bit flipped: one three-input bit operation per operand dword
    // (plus the shift for the low nibbles)
    constexpr uint32_t TOPB = 0x80808080u, TOPN = 0xF0F0F0F0u;
    auto centre_lo = [](uint32_t x) { return (int)(((x << 4) & TOPN) ^ TOPB); };
    auto centre_hi = [](uint32_t x) { return (int)((x & TOPN) ^ TOPB); };
    auto dump_block = [&](uint32_t b, const int* isum) {
        if (!DUMP) return;
        const uint32_t row = tile * 16 + n;
        if (b >= nblk || row >= w.n_out) return;
#pragma unroll
        for (int i = 0; i < 4; i++)
            if (d_tok0 + i < t) dump[((size_t)(d_tok0 + i) * w.n_out + row) * nblk + b] = isum[i];
    };
    auto compute_step = [&](const Step<FMT>& st, const uint32_t* sw, uint32_t s) {
        const uint4 c = st.w;
        if constexpr (q8_format(FMT)) {
            const float d = FMT == FMT_Q8F ? __uint_as_float(d_half ? sw[NM - 1] : sw[0]) : f16_bits_to_f32((uint16_t)(d_half ? sw[0] >> 16 : sw[0] & 0xFFFF));
            v4i bw = {(int)c.x, (int)c.y, (int)c.z, (int)c.w};
            const uint32_t b = 2 * s + d_half;
#pragma unroll
            for (int tg = 0; tg < NG; tg++) {
                v4i D = mfma(bw, s, tg, st.a[0], st.a[1]);
                float xs[4];
                load_xs(lds, tg * nm + (min(b, nblk - 1) - B0) * TPAD + d_tok0, xs);
                int isum[4] = {D.x, D.y, D.z, D.w};
#pragma unroll
                for (int i = 0; i < NI; i++) acc[tg][i] = fmaf(d, xs[i] * (float)isum[i], acc[tg][i]);
                dump_block(b, isum);
            }
        } else if constexpr (k45_format(FMT)) {
            // sw[0]: the step's four sub-block scales, sw[1]: its four mins (bytes), sw[2]: (d, dmin). One byte permute
            // gathers this lane's four: the scales of its two blocks (sub-blocks d_half and 2 + d_half of the step) and,
            // for the mins' matrix instruction, the scale and min of sub-block kq.
            const float d = f16_bits_to_f32((uint16_t)(sw[2] & 0xFFFF)), dmin = f16_bits_to_f32((uint16_t)(sw[2] >> 16));
            const uint32_t pk = __builtin_amdgcn_perm(sw[1], sw[0], q4k_sel);
            // Q5_K: the codes centre on 16 and go to the matrix cores as 8 (code - 16): the nibble in bits 3..6 of its
            // byte, the inverted fifth bit on top
            constexpr bool FIVE = FMT == FMT_Q5_K;
            const float d16 = d * (FIVE ? 0.125f : 0.0625f);
            const float dsc[2] = {d16 * (float)(pk & 0xFF), d16 * (float)((pk >> 8) & 0xFF)};
            // decode_i8's m of sub-block kq: 8 s - dmin * mn, 16 s for Q5_K (src/ggml.rs:1046-1073)
            const float mk = fmaf((FIVE ? 16.0f : 8.0f) * d, (float)((pk >> 16) & 0xFF), -(dmin * (float)(pk >> 24)));
#pragma unroll
            for (int pr = 0; pr < 2; pr++) {  // the two byte pairs of the lane's chunk
                v4i bw;
                if constexpr (FIVE) {
                    constexpr uint32_t NIB = 0x78787878u, TOP = 0x80808080u;
                    const uint32_t x0 = pr ? c.z : c.x, x1 = pr ? c.w : c.y, hb = ~st.h;
                    bw = v4i{(int)(((x0 << 3) & NIB) | ((hb << (7 - 4 * pr)) & TOP)), (int)(((x1 << 3) & NIB) | ((hb << (6 - 4 * pr)) & TOP)),
                             (int)(((x0 >> 1) & NIB) | ((hb << (5 - 4 * pr)) & TOP)), (int)(((x1 >> 1) & NIB) | ((hb << (4 - 4 * pr)) & TOP))};
                } else {
                    const uint32_t x0 = pr ? c.z : c.x, x1 = pr ? c.w : c.y;
                    bw = v4i{centre_lo(x0), centre_lo(x1), centre_hi(x0), centre_hi(x1)};
                }
                const uint32_t b = 4 * s + 2 * pr + d_half;  // global index of this lane's block of 32
#pragma unroll
                for (int tg = 0; tg < NG; tg++) {
                    v4i D = mfma(bw, 2 * s + pr, tg, st.a[2 * pr], st.a[2 * pr + 1]);
                    float xs[4];
                    load_xs(lds, tg * nm + (b - B0) * TPAD + d_tok0, xs);
                    const int I[4] = {D.x, D.y, D.z, D.w};
#pragma unroll
                    for (int i = 0; i < NI; i++) acc[tg][i] = fmaf(dsc[pr], xs[i] * (float)I[i], acc[tg][i]);
                    if (DUMP) {
                        constexpr int SH = FIVE ? 3 : 4;
                        int isum[4] = {I[0] >> SH, I[1] >> SH, I[2] >> SH, I[3] >> SH};
                        dump_block(b, isum);
                    }
                }
            }
            mins(4 * s, mk);
        } else if constexpr (FMT == FMT_Q6_K) {
            // Scales go per 16 columns, so an instruction's 16 operand slots are (sub-block sb, token t4): lane group kq
            // supplies sub-block kq's 16 activations of token t4 in the slots with sb = kq and zeros elsewhere, and lane
            // (kq, n) receives sub-block kq's exact sums for tokens 4 tg + i of row n. Eight tokens take two instructions.
            const float d = f16_bits_to_f32((uint16_t)(sw[2] & 0xFFFF));
            const uint32_t hq[2] = {st.h.x, st.h.y};
            const bool on = (n >> 2) == kq;
            const uint4* afr6 = reinterpret_cast<const uint4*>(afr);  // [64-column group][8 tokens][kq]
#pragma unroll
            for (int h = 0; h < 2; h++) {  // the step's two groups of 64 columns
                const uint32_t lo = h ? c.z : c.x, hi = h ? c.w : c.y, hh = hq[h];
                const v4i bw = {(int)((lo & 0x0F0F0F0Fu) | ((hh & 0x03030303u) << 4)), (int)(((lo >> 4) & 0x0F0F0F0Fu) | (((hh >> 2) & 0x03030303u) << 4)),
                                (int)((hi & 0x0F0F0F0Fu) | (((hh >> 4) & 0x03030303u) << 4)), (int)(((hi >> 4) & 0x0F0F0F0Fu) | (((hh >> 6) & 0x03030303u) << 4))};
                const float dsc = d * (float)(int)(int8_t)((sw[h] >> (8 * kq)) & 0xFF);
                const uint32_t m64 = 2 * s + h, b = 2 * m64 + (kq >> 1);  // the lane's 32-block (its scale's) and its half
                const uint32_t at = (min(b, nblk - 1) - B0) * TPAD;
#pragma unroll
                for (int tg = 0; tg < (NT > 4 ? 2 : 1); tg++) {
                    const uint4 av = afr6[((size_t)(m64 - M0) * 8 + 4 * tg + (n & 3)) * 4 + kq];
                    const v4i a = {on ? (int)av.x : 0, on ? (int)av.y : 0, on ? (int)av.z : 0, on ? (int)av.w : 0};
                    const v4i z = {0, 0, 0, 0};
                    const v4i D = __builtin_amdgcn_mfma_i32_16x16x64_i8(a, bw, z, 0, 0, 0);
                    const float4 xs = *reinterpret_cast<const float4*>(lds + at + 4 * tg);
                    const float4 cc = *reinterpret_cast<const float4*>(lds + (size_t)(1 + (kq & 1)) * as + at + 4 * tg);
                    const float xv[4] = {xs.x, xs.y, xs.z, xs.w}, cv[4] = {cc.x, cc.y, cc.z, cc.w};
                    const int U[4] = {D.x, D.y, D.z, D.w};
#pragma unroll
                    for (int i = 0; i < NI; i++) {
                        const float v = fmaf(xv[i], (float)U[i], cv[i]);
                        if (tg == 0) acc6a[i] = fmaf(dsc, v, acc6a[i]);
                        else acc6b[i] = fmaf(dsc, v, acc6b[i]);
                    }
                    if (DUMP) {
                        const int4 sp = *reinterpret_cast<const int4*>(lds + (size_t)3 * as + at + 4 * tg);
                        const int su[4] = {sp.x, sp.y, sp.z, sp.w};
                        const uint32_t row = tile * 16 + n;
#pragma unroll
                        for (int i = 0; i < 4; i++) {
                            const int s16 = (kq & 1) ? (su[i] >> 16) : (int)(int16_t)(su[i] & 0xFFFF);
                            if (4 * tg + i < (int)t && row < w.n_out && b < nblk)
                                dump[((size_t)(4 * tg + i) * w.n_out + row) * (w.n_in / 16) + 4 * m64 + kq] = U[i] - 32 * s16;
                        }
                    }
                }
            }
        } else {
#pragma unroll
            for (int g = 0; g < 2; g++) {  // the two groups of 64 of the step
                const uint32_t x0 = g ? c.z : c.x, x1 = g ? c.w : c.y;  // blocks 2 g, 2 g + 1
                constexpr bool MX = FMT == FMT_MXFP4;  // table codes: the int8 operand is the code's doubled value itself
                constexpr uint32_t NIB = 0x0F0F0F0Fu;
                v4i bw = MX ? v4i{(int)mxfp4_values<0>(x0 & NIB), (int)mxfp4_values<0>((x0 >> 4) & NIB), (int)mxfp4_values<0>(x1 & NIB),
                                  (int)mxfp4_values<0>((x1 >> 4) & NIB)}
                            : v4i{centre_lo(x0), centre_hi(x0), centre_lo(x1), centre_hi(x1)};
                const uint32_t b = 4 * s + 2 * g + d_half;
                // MLX: the group's scale; Q4_0: the lane's block's own scale (word g, half d_half); MXFP4: its scale byte
                float d;
                if constexpr (MX) d = e8m0_half((sw[0] >> (8 * (2 * g + d_half))) & 0xFF);
                else if constexpr (FMT == FMT_Q40) d = f16_bits_to_f32((uint16_t)(d_half ? sw[g] >> 16 : sw[g] & 0xFFFF));
                else d = f16_bits_to_f32((uint16_t)(g ? sw[0] >> 16 : sw[0] & 0xFFFF));
                // padding blocks hold zero codes (which centre to -8) and zero scales: they add zeros (as a select, not a
                // branch: a divergent branch here makes every step wait for all requests)
                const float dz = b < nblk ? (MX ? d : d * 0.0625f) : 0.0f;
#pragma unroll
                for (int tg = 0; tg < NG; tg++) {
                    v4i D = mfma(bw, 2 * s + g, tg, st.a[2 * g], st.a[2 * g + 1]);
                    float xs[4];
                    load_xs(lds, tg * nm + (min(b, nblk - 1) - B0) * TPAD + d_tok0, xs);
                    const int I[4] = {D.x, D.y, D.z, D.w};
#pragma unroll
                    for (int i = 0; i < NI; i++) acc[tg][i] = fmaf(dz, xs[i] * (float)I[i], acc[tg][i]);
                    if (DUMP) {
                        constexpr int SH = MX ? 0 : 4;
                        int isum[4] = {I[0] >> SH, I[1] >> SH, I[2] >> SH, I[3] >> SH};
                        dump_block(b, isum);
                    }
                }
            }
            if constexpr (FMT == FMT_Q4M) {  // the offset of block kq's group of 64, times the block's exact activation sum
                const float off = bf16_bits_to_f32((uint16_t)(kq >> 1 ? sw[1] >> 16 : sw[1] & 0xFFFF));
                mins(4 * s, 4 * s + kq < nblk ? off : 0.0f);
            }
        }
    };

    // Order of the requests: a wave's loads return in order, so the activations and their scales (L2 hits, needed by
    // every step) are requested first, into registers; then the first ring of weight records (HBM); then the staged
    // values go to LDS while the weights are still on their way. Requested after the weights, the activations would
    // only arrive behind them and no step could start before the whole ring had landed.
    constexpr int PF = pf_for<FMT, NT>();
    // 16-byte activation chunks / scale entries a thread holds in registers (more go later): every one is a request of
    // every wave whether or not it has a unit to fetch, so few tokens get few
    constexpr int SA = NG > 1 ? 8 : NT == 1 ? 2 : NT <= 4 ? 4 : 8, SM = NT <= 4 && NG == 1 ? 2 : 4;
    const uint32_t nb = min(nblk, B0 + nbl) - min(nblk, B0);  // real blocks of the slice
    // slot (m, lane) of the operand array: lane = 16 kq + 8 half + token holds the 8 values of block 2 m + half that
    // the weights' lane group kq pairs with (Q4: positions 4 kq.. and 16 + 4 kq..; else 8 kq..). A thread moves 16
    // (Q4: 32) consecutive bytes of one token's row, so the global reads are whole lines. Absent tokens and a padding
    // block keep whatever LDS holds: those products meet zero weights or are dropped.
    constexpr int AU = t4m_format(FMT) ? 2 : 1;  // 16-byte loads per unit of staging work
    // Unit i of the staging work is (token i / adiv, chunk i % adiv); a thread takes units tid, tid + nthr, ...: one
    // division for its first unit, then carries (a division per unit would be most of the instructions of a wave that
    // only streams some fifteen records).
    const uint32_t adiv = max(t4m_format(FMT) ? nb : 2 * nb, 1u);
    auto advance = [](uint32_t& q, uint32_t& r, uint32_t dq, uint32_t dr, uint32_t dv) {
        r += dr;
        q += dq;
        if (r >= dv) {
            r -= dv;
            q++;
        }
    };
    const uint32_t a_dq = nthr / adiv, a_dr = nthr - a_dq * adiv;
    auto act_load = [&](uint32_t tok, uint32_t c, uint4* v) {  // tok < t; c: chunk (Q4M: block) within the slice
        if (t4m_format(FMT)) {
            const uint4* xb = reinterpret_cast<const uint4*>(xa.q + src_row(tok) * w.n_in + (size_t)(B0 + c) * 32);
            v[0] = xb[0];
            v[1] = xb[1];
        } else {
            v[0] = *reinterpret_cast<const uint4*>(xa.q + src_row(tok) * w.n_in + (size_t)B0 * 32 + (size_t)c * 16);
        }
    };
    auto act_store = [&](uint32_t tok, uint32_t c, const uint4* v) {
        if (t4m_format(FMT)) {
            const uint32_t b = c;
            uint2* dst = afr + ((size_t)(tok >> 3) * (nbl / 2) + (b >> 1)) * 64;
            const uint32_t s0 = SWZ ? opslot(b >> 1, 8 * (b & 1) + (tok & 7)) : 8 * (b & 1) + (tok & 7);
            dst[s0] = make_uint2(v[0].x, v[1].x);
            dst[s0 ^ 16] = make_uint2(v[0].y, v[1].y);
            dst[s0 ^ 32] = make_uint2(v[0].z, v[1].z);
            dst[s0 ^ 48] = make_uint2(v[0].w, v[1].w);
        } else if (FMT == FMT_Q6_K) {  // chunk c = columns 16 c ..: sub-block c % 4 of 64-column group c / 4
            reinterpret_cast<uint4*>(afr)[((size_t)(c >> 2) * 8 + (tok & 7)) * 4 + (c & 3)] = make_uint4(v[0].x, v[0].y, v[0].z, v[0].w);
        } else {
            const uint32_t b = c >> 1;
            uint2* dst = afr + ((size_t)(tok >> 3) * (nbl / 2) + (b >> 1)) * 64;
            const uint32_t s0 = SWZ ? opslot(b >> 1, 32 * (c & 1) + 8 * (b & 1) + (tok & 7)) : 32 * (c & 1) + 8 * (b & 1) + (tok & 7);
            dst[s0] = make_uint2(v[0].x, v[0].y);
            dst[s0 ^ 16] = make_uint2(v[0].z, v[0].w);
        }
    };
    // scales and sums: unit i = (q = i / nbl, block i % nbl of the slice) with q = TPAD group + token of the group
    struct MetaReg {
        float x, f;
        int sq, sq2;  // Q6_K: the sums of the block's two halves
    };
    const uint32_t m_dq = nthr / nbl, m_dr = nthr - m_dq * nbl;
    auto meta_load = [&](uint32_t q, uint32_t b, MetaReg& r) {
        const uint32_t tok = 8 * (q / TPAD) + q % TPAD;
        const bool live = tok < t && B0 + b < nblk;
        const size_t src = (live ? src_row(tok) : 0) * nblk + B0 + (live ? b : 0);
        r.x = live ? xa.scales[src] : 0.0f;
        if (FMT == FMT_Q6_K) {
            r.sq = live ? xa.sums16[2 * src] : 0;
            r.sq2 = live ? xa.sums16[2 * src + 1] : 0;
            r.f = 0.0f;
        } else {
            r.sq = r.sq2 = 0;
            r.f = MINS && live ? xa.fsums[src] : 0.0f;
        }
    };
    auto meta_store = [&](uint32_t q, uint32_t b, const MetaReg& r) {
        const uint32_t at = (q / TPAD) * nm + b * TPAD + q % TPAD;
        lds[at] = r.x;
        if (FMT == FMT_Q6_K) {  // the codes are unsigned (0..63): -32 x the half's activation sum, scaled like the dot
            lds[(size_t)as + at] = -32.0f * (r.x * (float)r.sq);
            lds[(size_t)2 * as + at] = -32.0f * (r.x * (float)r.sq2);
            if (DUMP) reinterpret_cast<int*>(lds)[(size_t)3 * as + at] = (r.sq & 0xFFFF) | (r.sq2 << 16);
        } else if (MINS) {
            lds[(size_t)as + at] = r.f;
        }
    };
    uint4 sa[SA];
    MetaReg smr[SM];
    // (every request below is issued by every lane, with its unit clamped into range, so that the waits can be
    // counted exactly; the extra requests hit lines that are being fetched anyway)
    const uint32_t aq0 = threadIdx.x / adiv, ar0 = threadIdx.x - aq0 * adiv;
    const uint32_t mq0 = threadIdx.x / nbl, mr0 = threadIdx.x - mq0 * nbl;
    uint32_t aq = aq0, ar = ar0, mq = mq0, mr = mr0;
    if (ALDS) {
#pragma unroll
        for (int j = 0; j < SA / AU; j++) {
            act_load(min(aq, t - 1), ar, sa + AU * j);
            advance(aq, ar, a_dq, a_dr, adiv);
        }
    }
#pragma unroll
    for (int j = 0; j < SM; j++) {
        meta_load(mq, mr, smr[j]);
        advance(mq, mr, m_dq, m_dr, nbl);
    }
    // the ring's requests go out in the order in which the loop below renews them (the barriers keep the compiler from
    // regrouping them): its waits are counted against that order
    static_assert(PF % 4 == 0, "a request for scales serves four steps");
    Step<FMT> ring[PF];
    uint32_t snext[PF / 4][NM], scur[NM];
#pragma unroll
    for (int p = 0; p < PF; p++) {
        if (p % 4 == 0) {
            load_scales(snext[p / 4], s0 + p);
            __builtin_amdgcn_sched_barrier(0);
        }
        load_step(ring[p], min(s0 + p, slast));
        __builtin_amdgcn_sched_barrier(0);
    }
    aq = aq0, ar = ar0, mq = mq0, mr = mr0;
    if (ALDS) {
#pragma unroll
        for (int j = 0; j < SA / AU; j++) {
            if (aq < t) act_store(aq, ar, sa + AU * j);
            advance(aq, ar, a_dq, a_dr, adiv);
        }
    }
#pragma unroll
    for (int j = 0; j < SM; j++) {
        if (mq < NG * TPAD) meta_store(mq, mr, smr[j]);
        advance(mq, mr, m_dq, m_dr, nbl);
    }
    // what did not fit the registers (long rows, small workgroups) follows behind the weights
    if (ALDS) {
        for (; aq < t; advance(aq, ar, a_dq, a_dr, adiv)) {
            uint4 v[AU];
            act_load(aq, ar, v);
            act_store(aq, ar, v);
        }
    }
    for (; mq < NG * TPAD; advance(mq, mr, m_dq, m_dr, nbl)) {
        MetaReg r;
        meta_load(mq, mr, r);
        meta_store(mq, mr, r);
    }
    __syncthreads();
    // Each slot is refilled as soon as its record has been consumed, so PF - 1 records stay on request. No request sits
    // under a condition: the compiler counts the requests in flight to place its waits, and where a path may or may not
    // have issued one it waits for (nearly) all of them, which empties the ring at every step. So a generation that has
    // a successor refills every slot (past the wave's last step: with that step again, a hit), and the last one none.
    // The end of a run: its sums as a wave of its own leaves them ...
    auto close_run = [&]() {
        if constexpr (FMT == FMT_Q6_K) {
            // the four sub-blocks of a token meet across the lane groups; group 0 then holds tokens 0..3, group 1 tokens 4..7
#pragma unroll
            for (int i = 0; i < 4; i++) {
                float a = acc6a[i], b = acc6b[i];
                a += __shfl_xor(a, 16);
                a += __shfl_xor(a, 32);
                b += __shfl_xor(b, 16);
                b += __shfl_xor(b, 32);
                acc[0][i] = (kq & 1) ? b : a;
            }
        } else {
            if constexpr (MINS) {
#pragma unroll
                for (int g = 0; g < NG; g++)
#pragma unroll
                    for (int i = 0; i < 4; i++) acc[g][i] += macc[g][i];
            }
            // the two block parities of a token meet across lane groups kq and kq ^ 2
#pragma unroll
            for (int g = 0; g < NG; g++)
#pragma unroll
                for (int i = 0; i < 4; i++) acc[g][i] += __shfl_xor(acc[g][i], 32);
        }
    };
    // ... go to the run's place among its tile's partial sums ...
    auto store_run = [&](uint32_t run) {
        if (kq < 2) {
#pragma unroll
            for (int g = 0; g < NG; g++)
#pragma unroll
                for (int i = 0; i < 4; i++)
                    if (d_tok0 + i < (uint32_t)TPAD) red[((((size_t)r * runs + run) * NG + g) * TPAD + d_tok0 + i) * 16 + n] = acc[g][i];
        }
    };
    // A wave with further runs (up to MAXRUNS in all) keeps the closed run's sums in registers (the partial sums' place in
    // LDS still holds the activations) and starts the next run from zero. `left`: steps to the end of the run in hand.
    constexpr int MAXRUNS = 4;
    float held[REMAP ? MAXRUNS - 1 : 1][4] = {};
    uint32_t nrun = 0, left = per;  // runs closed so far
    auto step_done = [&]() {
        if constexpr (REMAP) {
            if (rpw > 1 && --left == 0 && nrun + 1 < rpw) {  // uniform over the wave
                close_run();
#pragma unroll
                for (int h = 0; h < MAXRUNS - 1; h++)
#pragma unroll
                    for (int i = 0; i < 4; i++) held[h][i] = nrun == (uint32_t)h ? acc[0][i] : held[h][i];
                nrun++;
                left = per;
#pragma unroll
                for (int i = 0; i < 4; i++) acc[0][i] = acc6a[i] = acc6b[i] = 0.0f;
                macc[0] = v4f{0.0f, 0.0f, 0.0f, 0.0f};
            }
        }
    };
    uint32_t sb = s0;
    for (; sb + PF < s1; sb += PF) {
#pragma unroll
        for (int p = 0; p < PF; p++) {
            if (p % 4 == 0) {
#pragma unroll
                for (int j = 0; j < NM; j++) scur[j] = snext[p / 4][j];
                load_scales(snext[p / 4], sb + PF + p);
            }
            uint32_t sw[NM];
            scales_of(scur, p % 4, sw);
            compute_step(ring[p], sw, sb + p);
            load_step(ring[p], min(sb + PF + p, slast));
            step_done();
        }
    }
#pragma unroll
    for (int p = 0; p < PF; p++) {
        if (p % 4 == 0) {
#pragma unroll
            for (int j = 0; j < NM; j++) scur[j] = snext[p / 4][j];
        }
        if (sb + p < s1) {
            uint32_t sw[NM];
            scales_of(scur, p % 4, sw);
            compute_step(ring[p], sw, sb + p);
            step_done();
        }
    }
    close_run();
    if (ALDS) __syncthreads();  // the partial sums overwrite the staged activations
    if constexpr (REMAP) {
        if (rpw > 1 && kq < 2) {  // the runs closed on the way
#pragma unroll
            for (int h = 0; h < MAXRUNS - 1; h++)
                if ((uint32_t)h < rpw - 1) {
#pragma unroll
                    for (int i = 0; i < 4; i++)
                        if (d_tok0 + i < (uint32_t)TPAD) red[(((size_t)r * runs + kj * rpw + h) * TPAD + d_tok0 + i) * 16 + n] = held[h][i];
                }
        }
    }
    store_run(kj * rpw + rpw - 1);
    __syncthreads();
    // how a finished sum goes out (uniform branches)
    auto emit = [&](float* dst, float v, uint32_t tok) {
        if (epi.mode == EPI_STORE) *dst = v;
        else if (epi.mode == EPI_ADD) *dst = *dst + v;
        else *dst = *dst + (1.0f / (1.0f + expf(-epi.gate[tok]))) * v;
    };
    if constexpr (GROUPED && !DUMP) {
        if (glu) {
            // a [token][rt / 2 * 16 rows of inter] = act(gate) * up behind the partial sums in LDS, then one lane per (token,
            // block of 32) quantizes its block exactly as quantize_act does (sequential sums in element order)
            float* aval = red + (size_t)rt * kw * NG * TPAD * 16;  // [NG * TPAD][ghalf * 16]
            const uint32_t cols = ghalf * 16;
            for (uint32_t idx = threadIdx.x; idx < ghalf * NG * TPAD * 16; idx += nthr) {
                const uint32_t rr = idx / (NG * TPAD * 16), gt = (idx / 16) % (NG * TPAD), nn = idx % 16;
                const uint32_t g = gt / TPAD, tl = gt % TPAD;
                float gs = 0.0f, us = 0.0f;
                for (uint32_t k = 0; k < kw; k++) {
                    gs += red[((((size_t)rr * kw + k) * NG + g) * TPAD + tl) * 16 + nn];
                    us += red[((((size_t)(ghalf + rr) * kw + k) * NG + g) * TPAD + tl) * 16 + nn];
                }
                aval[(size_t)gt * cols + rr * 16 + nn] = gated_act(gs, us, grp.act_kind, grp.act_param);
            }
            __syncthreads();
            // quantize_act's arithmetic (act_body.hpp) with 32 lanes per block: the maximum, the codes and the integer sums do
            // not depend on the order; the f32 sums do, and lane 0 (block and first half) and lane 16 (second half) of a block
            // form them one element after the other as the reference does. (A lone lane walking the whole block is a
            // microsecond and a half of dependent instructions at the end of every workgroup.)
            const uint32_t bpw = cols / 32, bpr = grp.glu_inter / 32;  // blocks of the workgroup; blocks of a row
            for (uint32_t idx = threadIdx.x; idx < NG * TPAD * bpw * 32; idx += nthr) {
                const uint32_t e = idx & 31, u = idx >> 5, gt = u / bpw, bl = u % bpw, tok = 8 * (gt / TPAD) + gt % TPAD;
                const uint32_t blk = bx * bpw + bl;
                const bool live = tok < t && blk < bpr;  // uniform over the 32 lanes of a block
                const float* src = aval + (size_t)gt * cols + bl * 32;
                const float v = src[e];
                float amax = fabsf(v);
#pragma unroll
                for (int off = 16; off >= 1; off >>= 1) amax = fmaxf(amax, __shfl_xor(amax, off));
                const float inv = amax > 0.0f ? 127.0f / amax : 0.0f;
                const float rr = roundf(v * inv);  // half away from zero
                const int iv = rr != rr ? 0 : (int)fminf(fmaxf(rr, -128.0f), 127.0f);
                int s16 = iv;  // the integer sum of the lane's half of the block
#pragma unroll
                for (int off = 8; off >= 1; off >>= 1) s16 += __shfl_xor(s16, off);
                const int s_other = __shfl_xor(s16, 16);
                float fsum = -0.0f, h0 = -0.0f;  // Rust's iter().sum() starts from -0.0
                if ((e & 15) == 0) {
                    if (e == 0) {
#pragma unroll
                        for (int i = 0; i < 16; i++) fsum += src[i];
                        h0 = fsum;
#pragma unroll
                        for (int i = 16; i < 32; i++) fsum += src[i];
                    } else {
#pragma unroll
                        for (int i = 16; i < 32; i++) h0 += src[i];
                    }
                }
                if (!live) continue;
                const size_t gb = (size_t)(row0 + tok) * bpr + blk;
                grp.aq_q[gb * 32 + e] = (int8_t)iv;
                if (e == 0) {
                    grp.aq_scales[gb] = amax / 127.0f;
                    grp.aq_sums[gb] = s16 + s_other;
                    grp.aq_fsums[gb] = fsum;
                    grp.aq_hsums[2 * gb] = h0;
                    grp.aq_sums16[2 * gb] = s16;
                } else if (e == 16) {
                    grp.aq_hsums[2 * gb + 1] = h0;
                    grp.aq_sums16[2 * gb + 1] = s16;
                }
            }
            return;
        }
    }
    const bool combine = GROUPED && grp.comb_y != nullptr;
    if (pair && ksplit == 1) {
        // act(gate) * up of the workgroup's rt / 2 row tiles: each product summed over its waves in order, as a launch of its own would
        for (uint32_t idx = threadIdx.x; idx < ghalf * TPAD * 16; idx += nthr) {
            const uint32_t rr = idx / (TPAD * 16), tok = (idx / 16) % TPAD, nn = idx % 16;
            const uint32_t row = (bx * ghalf + rr) * 16 + nn;
            if (tok >= t || row >= w.n_out) continue;
            float gs = 0.0f, us = 0.0f;
            for (uint32_t k = 0; k < kw; k++) {
                gs += red[(((size_t)rr * kw + k) * TPAD + tok) * 16 + nn];
                us += red[(((size_t)(ghalf + rr) * kw + k) * TPAD + tok) * 16 + nn];
            }
            y[(size_t)tok * w.n_out + row] = gated_act(gs, us, epi.pair_act, 0.0f);
        }
        return;
    }
    // the waves of a tile in order; with one slice that is the result, else this slice's partial rows (a pair's partial rows are
    // 2 n_out wide: the first matrix's, then the second's)
    const uint32_t prow = pair ? 2 * w.n_out : w.n_out;
    for (uint32_t zl = 0; zl < fs; zl++) {  // the workgroup's slices, each with a partial row of its own
        float* out = ksplit > 1 ? partial + (size_t)(slice * fs + zl) * t * prow : y;
        for (uint32_t idx = threadIdx.x; idx < rt * NG * TPAD * 16; idx += nthr) {
            const uint32_t rr = idx / (NG * TPAD * 16), g = (idx / (TPAD * 16)) % NG, tok = 8 * g + (idx / 16) % TPAD, nn = idx % 16;
            const uint32_t row = pair ? (bx * ghalf + (rr < ghalf ? rr : rr - ghalf)) * 16 + nn : (bx * rt + rr) * 16 + nn;
            if (tok >= t || row >= w.n_out || !y) continue;
            float sum = 0.0f;
            for (uint32_t k = 0; k < kw; k++) sum += red[((((size_t)rr * runs + (zl << kwsh) + k) * NG + g) * TPAD + (idx / 16) % TPAD) * 16 + nn];
            // partial rows go out as device-scope stores (written through to memory, where the other XCDs' L2s see them)
            if (ksplit > 1 || combine) __hip_atomic_store(out + (size_t)tok * prow + (pair && rr >= ghalf ? w.n_out : 0u) + row, sum, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
            else emit(out + (size_t)tok * w.n_out + row, sum, tok);
        }
    }
    if constexpr (GROUPED) {
        if (!combine) return;
        // The chunks of a row group meet like K slices do (below): the last workgroup to arrive, of all the launch's chunks,
        // adds every token's routed rows in route order (multiply, then add: src/moe.rs:608-615).
        __shared__ uint32_t last_chunk;
        asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
        __syncthreads();
        if (threadIdx.x == 0) {
            const uint32_t total = grp.direct ? grp.direct_n : (uint32_t)*grp.nchunks;
            const uint32_t seen = __hip_atomic_fetch_add(&grp.comb_counters[(size_t)bx * CTR_STRIDE], 1u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
            last_chunk = seen == total - 1;
            if (seen == total - 1) __hip_atomic_store(&grp.comb_counters[(size_t)bx * CTR_STRIDE], 0u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
        }
        __syncthreads();
        if (!last_chunk) return;
        const float* o = y - (size_t)row0 * w.n_out;  // the gathered rows from row 0
        for (uint32_t idx = threadIdx.x; idx < rt * 16 * grp.comb_t; idx += nthr) {
            const uint32_t tok = idx / (rt * 16), row = bx * rt * 16 + idx % (rt * 16);
            if (row >= w.n_out) continue;
            float acc_y = grp.comb_add ? grp.comb_y[(size_t)tok * w.n_out + row] : 0.0f;
            for (uint32_t j0 = 0; j0 < grp.comb_k; j0 += 4) {  // four routes per round trip, added in route order
                float v[4], wt[4];
#pragma unroll
                for (uint32_t i = 0; i < 4; i++) {
                    const uint32_t j = min(j0 + i, grp.comb_k - 1);
                    const int rw = grp.row_of ? grp.row_of[(size_t)tok * grp.comb_k + j] : (int)j;
                    wt[i] = grp.route_w[(size_t)tok * grp.comb_k + j];
                    v[i] = __hip_atomic_load(o + (size_t)rw * w.n_out + row, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
                }
#pragma unroll
                for (uint32_t i = 0; i < 4; i++)
                    if (j0 + i < grp.comb_k) acc_y = acc_y + wt[i] * v[i];
            }
            grp.comb_y[(size_t)tok * w.n_out + row] = acc_y;
        }
        return;
    }
    if (ksplit == 1 || !y) return;  // uniform over the workgroup
    // The last workgroup of this row group to get here adds the slices in slice order; the counter returns to zero
    // for the next launch. Every access to the partial rows and the counter is a device-scope atomic access, and each
    // thread waits for its stores to complete before the workgroup's arrival is counted, so no cache-wide write-back
    // or invalidation is needed (a device-scope fence here costs tens of microseconds per launch).
    __shared__ uint32_t is_last;
    asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
    __syncthreads();
    if (threadIdx.x == 0) {
        const uint32_t seen = __hip_atomic_fetch_add(&counters[(size_t)bx * CTR_STRIDE], 1u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
        const uint32_t arrivals = ksplit >> __builtin_ctz(fs);  // workgroups of this row group
        is_last = seen == arrivals - 1;
        if (seen == arrivals - 1) __hip_atomic_store(&counters[(size_t)bx * CTR_STRIDE], 0u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
    }
    __syncthreads();
    if (!is_last) return;
    // four slices per round trip (a loop of one load per slice waits for each in turn); still added in slice order
    auto slice_sum = [&](const float* p) {
        float sum = 0.0f;
        for (uint32_t z0 = 0; z0 < ksplit; z0 += 4) {
            float v[4];
#pragma unroll
            for (uint32_t i = 0; i < 4; i++)
                v[i] = __hip_atomic_load(p + (size_t)min(z0 + i, ksplit - 1) * t * prow, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
#pragma unroll
            for (uint32_t i = 0; i < 4; i++) sum = z0 + i == 0 ? v[i] : z0 + i < ksplit ? sum + v[i] : sum;
        }
        return sum;
    };
    const uint32_t wrows = (pair ? ghalf : rt) * 16;  // output rows of the workgroup
    for (uint32_t idx = threadIdx.x; idx < wrows * t; idx += nthr) {
        const uint32_t tok = idx / wrows, row = bx * wrows + idx % wrows;
        if (row >= w.n_out) continue;
        const float* p = partial + (size_t)tok * prow + row;
        if (pair) y[(size_t)tok * w.n_out + row] = gated_act(slice_sum(p), slice_sum(p + w.n_out), epi.pair_act, 0.0f);
        else emit(y + (size_t)tok * w.n_out + row, slice_sum(p), tok);
    }
}


// Dynamic LDS is declared 16-byte aligned whatever static LDS a kernel also holds: the 8- and 16-byte LDS reads are split
// into dwords (and the kernel runs two to three times longer) when the array starts at an odd dword.
// (Grouped launches keep to 8 waves, which leaves them 256 registers for the accumulators of their token groups.)
// (Q6_K: bounded at 8 waves like its shared-launch kernel, see decode_batch_kernel)
template <int FMT, int NT, bool DUMP, bool GROUPED, bool ALDS, int NG>
__global__ __launch_bounds__(GROUPED || FMT == FMT_Q6_K ? 512 : 1024) void decode_mfma_kernel(WeightView w, QActView xa, uint32_t t, uint32_t rt,
                                                                           uint32_t kw, float* __restrict__ y,
                                                                           int32_t* __restrict__ dump, GroupView grp, uint32_t ksplit,
                                                                           float* __restrict__ partial,
                                                                           uint32_t* __restrict__ counters, Epi epi) {
    extern __shared__ __align__(16) float lds_dyn[];
    decode_body<FMT, NT, DUMP, GROUPED, ALDS, NG>(w, xa, t, rt, kw, y, dump, grp, ksplit, partial, counters, blockIdx.x, blockIdx.y,
                                                  blockDim.x, lds_dyn, epi);
}

// Several independent matmuls in one launch (the jobs of one Backend::matmul call, src/gpu.rs:160: Q/K/V, gate/up ...):
// job j owns workgroups [wg0_j, wg0_{j+1}); each workgroup runs its job exactly as a launch of that job alone would
// (same shape, same order of sums), so the results are bit-identical to separate launches. What the single launch
// buys is time: a decode matmul is a chain of dependent latencies (stage activations, stream weights, reduce, store:
// about 6 us before the first byte of bandwidth counts), and here the chains of neighbouring jobs overlap instead of
// queueing behind kernel boundaries.
constexpr int BATCH_MAX = 16;
struct BatchJob {
    WeightView w;
    QActView xa;
    float* y;
    float* partial;      // this job's share of the scratch (K slices across workgroups)
    uint32_t* counters;
    uint32_t t, rt, kw, ks, wg0;
    Mapping map;  // (ks / fs slices across workgroups, 64 rt kwp threads)
    Epi epi;
};
struct BatchArgs {
    uint32_t njobs, nwg;
    BatchJob j[BATCH_MAX];
};

template <int FMT, bool FAT>
__device__ __forceinline__ void batch_dispatch(const BatchJob& jb, uint32_t bid, float* lds) {
    const uint32_t nthr = 64 * jb.rt * jb.map.kwp;
    if (threadIdx.x >= nthr) return;  // whole waves (nthr is a multiple of 64), before any barrier
    const GroupView none{};
    const uint32_t ksp = jb.ks >> __builtin_ctz(jb.map.fs);  // slices across workgroups
    const uint32_t bx = bid >> __builtin_ctz(ksp), by = bid & (ksp - 1);  // the slices of a row group are neighbours in launch order (a power of two)
    if (jb.t == 1) decode_body<FMT, 1, false, false, true, 1, FAT>(jb.w, jb.xa, jb.t, jb.rt, jb.kw, jb.y, nullptr, none, jb.ks, jb.partial, jb.counters, bx, by, nthr, lds, jb.epi, jb.map);
    else if (jb.t == 2 && !t4m_format(FMT)) decode_body<FMT, 2, false, false, true, 1, FAT>(  // (MLX at 2 tokens: the 4-token body, which fits the registers)
        jb.w, jb.xa, jb.t, jb.rt, jb.kw, jb.y, nullptr, none, jb.ks, jb.partial, jb.counters, bx, by, nthr, lds, jb.epi, jb.map);
    else if (jb.t <= 4) decode_body<FMT, 4, false, false, true, 1, FAT>(jb.w, jb.xa, jb.t, jb.rt, jb.kw, jb.y, nullptr, none, jb.ks, jb.partial, jb.counters, bx, by, nthr, lds, jb.epi, jb.map);
    else decode_body<FMT, 8, false, false, true, 1, FAT>(jb.w, jb.xa, jb.t, jb.rt, jb.kw, jb.y, nullptr, none, jb.ks, jb.partial, jb.counters, bx, by, nthr, lds, jb.epi, jb.map);
}

// FSET: the formats compiled in, one bit per Fmt. The compiler allocates registers over the whole kernel, so every
// format in it costs the others (a seventh format made the common GGUF ones 15 % slower, and one kernel of all formats
// spilled 480 registers): the formats are split into
// the sets below, and a call whose jobs span several sets becomes one launch per set, back to back on the stream.
constexpr uint32_t fbit(int f) { return 1u << f; }
constexpr uint32_t FSET_GGUF = fbit(FMT_Q8_0) | fbit(FMT_Q4_K) | fbit(FMT_Q6_K), FSET_MLX = fbit(FMT_Q4M),
                   FSET_K5 = fbit(FMT_Q5_K) | fbit(FMT_Q4_K) | fbit(FMT_Q6_K), FSET_Q40 = fbit(FMT_Q40), FSET_MX4 = fbit(FMT_MXFP4), FSET_Q8F = fbit(FMT_Q8F);
// The sets in launch order: more instruction work per byte first, so that the call's tail is made of the lightest jobs.
constexpr uint32_t FSETS[] = {FSET_K5, FSET_Q40, FSET_MX4, FSET_MLX, FSET_GGUF, FSET_Q8F};
constexpr int NSETS = sizeof(FSETS) / sizeof(FSETS[0]);
// The set a job of format `fmt` goes out with, given the formats present in the call (`mask`). Q4_K and Q6_K are in two sets:
// with Q8_0 (the formats a Q4_K_M file mixes) and with Q5_K (a Q5_K_M file's), whose step needs a few registers more; they
// take the second only when the call has Q5_K jobs, so that its layers' matmuls share one launch too.
inline int set_of(int fmt, uint32_t mask) {
    const uint32_t both = fbit(FMT_Q4_K) | fbit(FMT_Q6_K);
    for (int i = 0; i < NSETS; i++) {
        if (!(FSETS[i] & fbit(fmt))) continue;
        if ((fbit(fmt) & both) && FSETS[i] == FSET_K5 && !(mask & fbit(FMT_Q5_K))) continue;
        if ((fbit(fmt) & both) && FSETS[i] == FSET_GGUF && (mask & fbit(FMT_Q5_K))) continue;
        return i;
    }
    return -1;
}
// (Q6_K shares the kernel of Q8_0 and Q4_K since its step keeps 111 registers: a Q4_K_M file's layers mix the three, and their
// matmuls go out in one launch. Q4_0's kernel is bounded at 512 threads, which saves it nine spilled registers; its shapes
// never exceed 8 waves.)
// FAT: the launch's jobs use the fat mapping (see place_job); the plain kernels do without its bookkeeping.
template <uint32_t FSET, bool FAT>
__global__ __launch_bounds__(FSET == (1u << FMT_Q40) ? 512 : 1024) void decode_batch_kernel(BatchArgs a) {
    extern __shared__ __align__(16) float lds_dyn[];
    uint32_t j = 0;
    while (j + 1 < a.njobs && blockIdx.x >= a.j[j + 1].wg0) j++;  // uniform
    const BatchJob& jb = a.j[j];
    const uint32_t bx = blockIdx.x - jb.wg0;
    switch (jb.w.fmt) {
        case FMT_Q8_0: if constexpr (FSET & fbit(FMT_Q8_0)) batch_dispatch<FMT_Q8_0, FAT>(jb, bx, lds_dyn); break;
        case FMT_Q8F: if constexpr (FSET & fbit(FMT_Q8F)) batch_dispatch<FMT_Q8F, FAT>(jb, bx, lds_dyn); break;
        case FMT_Q4_K: if constexpr (FSET & fbit(FMT_Q4_K)) batch_dispatch<FMT_Q4_K, FAT>(jb, bx, lds_dyn); break;
        case FMT_Q5_K: if constexpr (FSET & fbit(FMT_Q5_K)) batch_dispatch<FMT_Q5_K, FAT>(jb, bx, lds_dyn); break;
        case FMT_Q6_K: if constexpr (FSET & fbit(FMT_Q6_K)) batch_dispatch<FMT_Q6_K, FAT>(jb, bx, lds_dyn); break;
        case FMT_Q4M: if constexpr (FSET & fbit(FMT_Q4M)) batch_dispatch<FMT_Q4M, FAT>(jb, bx, lds_dyn); break;
        case FMT_Q40: if constexpr (FSET & fbit(FMT_Q40)) batch_dispatch<FMT_Q40, FAT>(jb, bx, lds_dyn); break;
        case FMT_MXFP4: if constexpr (FSET & fbit(FMT_MXFP4)) batch_dispatch<FMT_MXFP4, FAT>(jb, bx, lds_dyn); break;
        default: break;
    }
}

namespace {

struct Shape {
    uint32_t rt, kw, ks;
};

constexpr uint32_t NCU = 256;

// Workgroup shape (rt row tiles x kw waves per tile) and the number of K slices across workgroups (ks): a function of
// the weight's shape and format only, so a row's sum is associated the same way whatever the batch or the kind of
// launch. A cost model fitted to measurements of the Llama-8B MLP shapes (steady streams of launches, single
// launches and the shared launch of eight):
//  * A matmul at these sizes is a chain of dependent latencies (stage activations, stream weights, reduce, store)
//    and only overlaps them when a CU holds two workgroups in different phases (the registers allow no more):
//    workgroups have at most 8 waves, and K is sliced until two workgroups' staged activations (11 bytes per column
//    at 8 tokens) fit a CU's 160 KiB. Twice as many slices are also tried: they buy more, smaller workgroups.
//  * Every further slice costs: its partial rows meet through memory (store, wait, count, and the last one reads
//    them all), two to three round trips during which the workgroup holds its place and does nothing.
//  * Among the (rt, kw) left, the pick minimizes the records that pass through the busiest CU when workgroups are
//    dealt round-robin, and prefers a few records per wave, four or more waves, enough workgroups for every CU, and
//    little restaging (every workgroup stages its slice of the activations: 11 bytes per column next to the
//    rt * bytes-per-column of weights it streams).
Shape search_shape(uint32_t ntiles, uint32_t nsteps, uint32_t cols_per_step, double weight_bytes_per_col) {
    uint32_t ks0 = 1;
    while (ks0 < 32 && (size_t)nsteps * cols_per_step * 11 / ks0 > 80 * 1024 && nsteps / (ks0 * 2) >= 4) ks0 *= 2;
    while (ks0 > 1 && (nsteps + ks0 - 1) / ks0 * (ks0 - 1) >= nsteps) ks0 /= 2;  // no empty slice
    Shape best{1, 1, ks0};
    double best_cost = 1e300;
    for (uint32_t ks = ks0; ks <= (ks0 > 1 ? 2 * ks0 : 1u); ks *= 2) {
        if (ks > ks0 && (ks > 32 || nsteps / ks < 4 || (nsteps + ks - 1) / ks * (ks - 1) >= nsteps)) break;
        const uint32_t sl = (nsteps + ks - 1) / ks;
        double slices = 1.0;
        for (uint32_t k = 1; k < ks; k *= 2) slices *= 1.06;
        for (uint32_t kw = 1; kw <= 8; kw *= 2)
            for (uint32_t rt = 1; rt * kw <= 8; rt++) {
                const uint32_t per = (sl + kw - 1) / kw;
                const uint64_t wgs = (uint64_t)((ntiles + rt - 1) / rt) * ks;
                double cost = (double)((wgs + NCU - 1) / NCU) * rt * per * kw;  // records through the busiest CU
                if (rt * kw < 4) cost *= 1.0 + 0.10 * (4 - rt * kw);
                if (per < 8) cost *= 1.0 + 0.03 * (8 - per);     // short streams: the latency chain dominates
                if (per > 16) cost *= 1.0 + 0.001 * (per - 16);  // long streams: fewer waves to keep HBM busy
                if (wgs < NCU) cost *= 1.05;
                cost *= 1.0 + 0.25 * 11.0 / (weight_bytes_per_col * rt) + 0.002 * kw;
                cost *= slices;
                if (cost < best_cost) {
                    best_cost = cost;
                    best = Shape{rt, kw, ks};
                }
            }
    }
#ifdef OXHIP_TUNING  // tuning builds only (never the shipped library): "tiles:steps=rt,kw,ks;..." in OXHIP_DECODE_SHAPE
    if (const char* e = getenv("OXHIP_DECODE_SHAPE")) {
        for (const char* p = e; p && *p;) {
            unsigned nt = 0, ns = 0, a = 0, b = 0, c = 0;
            if (sscanf(p, "%u:%u=%u,%u,%u", &nt, &ns, &a, &b, &c) == 5 && nt == ntiles && ns == nsteps && a >= 1 && b >= 1 && c >= 1 &&
                (b & (b - 1)) == 0 && (c & (c - 1)) == 0 && a * b <= 16 && c <= 32 && (nsteps + c - 1) / c * (c - 1) < nsteps)  // kw, ks: powers of two; no empty slice
                best = Shape{a, b, c};
            p = strchr(p, ';');
            if (p) p++;
        }
    }
#endif
    return best;
}

// The search runs once per shape: a decode launch is a few microseconds of GPU time and must not spend as long on
// the host. Without scratch for the slices (allow_slices false) K stays inside a workgroup.
Shape shape_for(uint32_t ntiles, uint32_t nsteps, bool allow_slices, int fmt) {
    const uint32_t cols_per_step = q8_format(fmt) ? 64 : 128;
    // weight bytes per column of a row tile, as the restaging term of the cost sees them: the 8-bit records, and the
    // 4-bit ones for the 4- and 6-bit formats alike (the 6-bit records are larger but cost as many instructions more)
    const double bytes_per_col = q8_format(fmt) ? (double)T8_REC / 64 : fmt == FMT_Q5_K ? (double)TK5_REC / 256 : (double)TK4_REC / 256;
    static std::mutex mu;
    static std::map<uint64_t, Shape> cache;
    // ntiles and nsteps are below 2^27 (n_out, n_in < 2^31): 27 + 27 + 8 bits of format + 1
    static_assert(FMT_MXFP4 < 256, "the key keeps 8 bits of the format");
    const uint64_t key = ((uint64_t)ntiles << 36) | ((uint64_t)nsteps << 9) | ((uint64_t)(fmt & 0xFF) << 1) | (allow_slices ? 1u : 0u);
    std::lock_guard<std::mutex> g(mu);
    auto it = cache.find(key);
    if (it != cache.end()) return it->second;
    Shape sh = search_shape(ntiles, nsteps, cols_per_step, bytes_per_col);
    if (!allow_slices) sh.ks = 1;
    cache.emplace(key, sh);
    return sh;
}

// A gate / up pair: a workgroup holds the tiles of the same rows of both matrices, so its tile count is even; kw and ks (the
// order of a row's sum) stay what the weight's shape alone gives, which keeps each product's bits those of a launch of its own.
Shape pair_shape(Shape sh) {
    if (sh.rt % 2) sh.rt = (sh.rt + 1) * sh.kw <= 8 ? sh.rt + 1 : sh.rt > 1 ? sh.rt - 1 : 2;  // (rt = 1 with kw = 8: 16 waves)
    return sh;
}
uint32_t pair_tiles(const Shape& sh, bool pair) { return pair ? pair_shape(sh).rt / 2 : sh.rt; }

constexpr size_t LDS_MAX = 160 * 1024 - 256;  // dynamic LDS on offer (the kernel also holds a static word)

// Dynamic LDS of a launch; `alds` comes back false when the operand-order activations do not fit (they are then read
// from L2 per record).
// `map`: the workgroup's fs slices (see decode_body); zeros for the plain mapping.
size_t lds_bytes(int fmt, bool dump, uint32_t nsteps, int tpad, const Shape& sh, bool* alds, uint32_t ng = 1, Mapping map = Mapping{}) {
    const uint32_t bps = q8_format(fmt) ? 2 : 4;
    const uint32_t fs = map.fs ? map.fs : 1;
    const uint32_t nbl = bps * fs * ((nsteps + sh.ks - 1) / sh.ks);  // blocks of the workgroup's slices
    const uint32_t narr = q8_format(fmt) || fmt == FMT_Q40 || fmt == FMT_MXFP4 ? 1 : fmt == FMT_Q6_K ? (dump ? 4 : 3) : 2;  // metadata arrays
    const size_t meta = (size_t)narr * ng * nbl * tpad * 4, red = (size_t)sh.rt * fs * sh.kw * ng * tpad * 16 * 4;
    const size_t act = (size_t)ng * (nbl / 2) * 512;
    const size_t with = act + meta > red ? act + meta : red;  // the partial sums reuse the activations' space
    *alds = with <= LDS_MAX;
    return *alds ? with : meta + red;
}

template <int FMT, int NT, bool DUMP, bool GROUPED, int NG = 1>
hipError_t launch_one(bool alds, dim3 grid, dim3 block, size_t lds, hipStream_t s, const WeightView& w, const QActView& v, uint32_t t,
                      const Shape& sh, float* y, int32_t* dump, const GroupView& g, const DecodeScratch& sc, hipEvent_t ev_start = nullptr,
                      hipEvent_t ev_stop = nullptr, const Epi& epi = Epi{}) {
    hipError_t e = hipSuccess;
    auto go = [&](auto kern) {
        // once per kernel and device: allow the whole LDS
        static std::atomic<uint64_t> allowed[4];  // one bit per device
        int dev = 0;
        (void)hipGetDevice(&dev);
        const uint64_t bit = 1ull << (dev & 63);
        if (lds > 48 * 1024 && !(allowed[(dev >> 6) & 3].load(std::memory_order_acquire) & bit)) {
            e = hipFuncSetAttribute(reinterpret_cast<const void*>(kern), hipFuncAttributeMaxDynamicSharedMemorySize, (int)LDS_MAX);
            if (e == hipSuccess) allowed[(dev >> 6) & 3].fetch_or(bit, std::memory_order_release);
        }
        if (e != hipSuccess) return;
        // timing events ride on the dispatch: its start and end as the device saw them
        if (ev_start || ev_stop)
            hipExtLaunchKernelGGL(kern, grid, block, (uint32_t)lds, s, ev_start, ev_stop, 0, w, v, t, sh.rt, sh.kw, y, dump, g, sh.ks, sc.partial, sc.counters, epi);
        else kern<<<grid, block, lds, s>>>(w, v, t, sh.rt, sh.kw, y, dump, g, sh.ks, sc.partial, sc.counters, epi);
    };
    if (alds) go(decode_mfma_kernel<FMT, NT, DUMP, GROUPED, true, NG>);
    else if constexpr (NG == 1 && FMT != FMT_Q6_K) go(decode_mfma_kernel<FMT, NT, DUMP, GROUPED, false, 1>);
    else e = hipErrorInvalidValue;  // token groups and Q6_K need the staged activations
    return e != hipSuccess ? e : hipGetLastError();
}

template <int FMT>
constexpr uint32_t steps_of(uint32_t n_in) {
    return q8_format(FMT) ? t8_steps(n_in) : k45_format(FMT) ? 2 * tk4_sbs(n_in) : FMT == FMT_Q6_K ? t6k_steps(n_in) : t4m_steps(n_in);
}

template <int FMT, bool DUMP>
hipError_t run(const WeightView& w, const QActView& xa, size_t t, float* y, int32_t* dump, const DecodeScratch& sc, hipStream_t s,
               hipEvent_t ev_start = nullptr, hipEvent_t ev_stop = nullptr, const Epi& epi0 = Epi{}) {
    const uint32_t ntiles = row_tiles(w.n_out), nsteps = steps_of<FMT>(w.n_in);
    const bool pair = !DUMP && epi0.pair_p0 != nullptr;
    Shape sh = shape_for(ntiles, nsteps, true, FMT);
    // slices need scratch: 8 token rows per slice (of both matrices of a pair) and a counter per row group
    auto scratch_ok = [&](const Shape& h) {
        const uint32_t groups = (ntiles + pair_tiles(h, pair) - 1) / pair_tiles(h, pair);
        return h.ks == 1 || (sc.partial && sc.counters && sc.partial_floats >= (size_t)h.ks * 8 * w.n_out * (pair ? 2 : 1) && sc.ncounters >= (size_t)groups * CTR_STRIDE);
    };
    if (!scratch_ok(sh)) sh = shape_for(ntiles, nsteps, false, FMT);
    if (pair) sh = pair_shape(sh);
    const uint32_t nblk = w.n_in / 32;
    const uint32_t per_wg = pair ? sh.rt / 2 : sh.rt;  // row tiles of the output per workgroup
    dim3 grid((ntiles + per_wg - 1) / per_wg, sh.ks), block(64 * sh.rt * sh.kw);
    // timing events: one launch carries them itself; around several they are recorded on the stream
    const bool ride = t <= 8;
    if (!ride && ev_start) {
        hipError_t e = hipEventRecord(ev_start, s);
        if (e != hipSuccess) return e;
    }
    hipEvent_t e0 = ride ? ev_start : nullptr, e1 = ride ? ev_stop : nullptr;
    size_t c0 = 0;
    while (c0 < t) {
        const size_t tc = t - c0 < 8 ? t - c0 : 8;
        QActView v = xa;
        v.q += c0 * w.n_in;
        v.scales += c0 * nblk;
        v.sums += c0 * nblk;
        v.fsums += c0 * nblk;
        if (v.hsums) v.hsums += c0 * 2 * nblk;
        if (v.sums16) v.sums16 += c0 * 2 * nblk;
        float* yo = y ? y + c0 * w.n_out : nullptr;  // no output rows when only the block sums are wanted
        int32_t* du = dump ? dump + c0 * (size_t)w.n_out * nblk * (FMT == FMT_Q6_K ? 2 : 1) : nullptr;
        const int tpad = tc <= 4 ? 4 : 8;
        bool alds;
        const size_t lds = lds_bytes(FMT, DUMP, nsteps, tpad, sh, &alds);
        if (lds > LDS_MAX) return hipErrorInvalidValue;  // rows too long for the staged activation scales
        const uint32_t tt = (uint32_t)tc;
        Epi epi = epi0;
        if (epi.gate) epi.gate += c0;
        hipError_t e;
        if (tc == 1) e = launch_one<FMT, 1, DUMP, false>(alds, grid, block, lds, s, w, v, tt, sh, yo, du, GroupView{}, sc, e0, e1, epi);
        else if (tc == 2 && !t4m_format(FMT)) e = launch_one<FMT, 2, DUMP, false>(alds, grid, block, lds, s, w, v, tt, sh, yo, du, GroupView{}, sc, e0, e1, epi);
        else if (tc <= 4) e = launch_one<FMT, 4, DUMP, false>(alds, grid, block, lds, s, w, v, tt, sh, yo, du, GroupView{}, sc, e0, e1, epi);
        else e = launch_one<FMT, 8, DUMP, false>(alds, grid, block, lds, s, w, v, tt, sh, yo, du, GroupView{}, sc, e0, e1, epi);
        if (e != hipSuccess) return e;
        c0 += tc;
    }
    if (!ride && ev_stop) return hipEventRecord(ev_stop, s);
    return hipSuccess;
}

// The workgroup of a grouped launch: rows are split over up to eight waves of 16 records or more (kw: a function of the
// weight alone, since it fixes the order of a row's sum), and a workgroup takes as many row tiles as eight waves allow,
// because every workgroup stages its chunk's activations. Decode-sized passes (chunks of at most 8 rows: little to stage,
// few chunks) take at most four tiles: smaller workgroups spread a pass of 8 experts over more CUs (24.8 -> 23.0 us).
Shape grouped_shape(uint32_t nsteps, uint32_t max_rows) {
    uint32_t gkw = 1;
    while (gkw < 8 && nsteps / (gkw * 2) >= 16) gkw *= 2;
    const uint32_t rt = 8 / gkw;
    return Shape{max_rows <= 8 && rt > 4 ? 4u : rt, gkw, 1};
}

template <int FMT>
hipError_t run_grouped(const WeightView& w, const QActView& xa, const GroupView& g, uint32_t max_chunks, uint32_t max_rows,
                       float* y, hipStream_t s) {
    const uint32_t ntiles = row_tiles(w.n_out), nsteps = steps_of<FMT>(w.n_in);
    // grid y walks the chunks (no K slices across workgroups). Every workgroup stages its chunk's activations, so it
    // takes as many row tiles as 8 waves allow, each wave keeping 16 records or more where K is long enough. The shape depends on the
    // weight alone, so a token's row is bit-identical whatever else is in the group.
    Shape sh = grouped_shape(nsteps, max_rows);
#ifdef OXHIP_TUNING  // tuning builds only: "rt,kw" in OXHIP_GROUPED_SHAPE
    if (const char* e = getenv("OXHIP_GROUPED_SHAPE")) {
        unsigned a = 0, b = 0;
        if (sscanf(e, "%u,%u", &a, &b) == 2 && a >= 1 && b >= 1 && (b & (b - 1)) == 0 && a * b <= 8) sh = Shape{a, b, 1};
    }
#endif
    dim3 grid((ntiles + sh.rt - 1) / sh.rt, max_chunks), block(64 * sh.rt * sh.kw);
    const int tpad = max_rows <= 4 ? 4 : 8;
    const uint32_t ng = max_rows <= 8 ? 1 : (max_rows <= 16 ? 2 : 4);
    if (max_rows > 32) return hipErrorInvalidValue;
    bool alds;
    size_t lds = lds_bytes(FMT, false, nsteps, tpad, sh, &alds, ng);
    if (g.glu_inter) {
        // gate and up tiles in pairs, whole blocks of 32 rows per workgroup; act(gate) * up sits behind the partial sums
        if (sh.rt % 4 || g.glu_inter % 32 || w.n_out != 2 * g.glu_inter) return hipErrorInvalidValue;
        grid.x = (g.glu_inter / 16 + sh.rt / 2 - 1) / (sh.rt / 2);
        const size_t red = (size_t)sh.rt * sh.kw * ng * tpad * 16 * 4, aval = (size_t)ng * tpad * (sh.rt / 2) * 16 * 4;
        if (alds) lds = std::max(lds, red + aval);
        else lds += aval;
    }
    if (lds > LDS_MAX || (ng > 1 && !alds)) return hipErrorInvalidValue;
    const DecodeScratch none{};
    if (max_rows == 1) return launch_one<FMT, 1, false, true>(alds, grid, block, lds, s, w, xa, 0u, sh, y, nullptr, g, none);
    if (max_rows <= 4) return launch_one<FMT, 4, false, true>(alds, grid, block, lds, s, w, xa, 0u, sh, y, nullptr, g, none);
    if (ng == 1) return launch_one<FMT, 8, false, true>(alds, grid, block, lds, s, w, xa, 0u, sh, y, nullptr, g, none);
    if (ng == 2) return launch_one<FMT, 8, false, true, 2>(alds, grid, block, lds, s, w, xa, 0u, sh, y, nullptr, g, none);
    return launch_one<FMT, 8, false, true, 4>(alds, grid, block, lds, s, w, xa, 0u, sh, y, nullptr, g, none);
}

}  // namespace

namespace {
uint32_t steps_rt(const WeightView& w) {
    return q8_format(w.fmt)    ? steps_of<FMT_Q8_0>(w.n_in)
           : k45_format(w.fmt) ? steps_of<FMT_Q4_K>(w.n_in)
           : w.fmt == FMT_Q6_K ? steps_of<FMT_Q6_K>(w.n_in)
                               : steps_of<FMT_Q4M>(w.n_in);
}
}  // namespace

// Whether a gate / up pair of this weight's shape and format runs as one launch (its workgroup of paired tiles fits the
// kernel's bound: Q6_K's kernels take at most 8 waves).
bool decode_pair_ok(const WeightView& w) {
    if (!mfma_decode_format(w.fmt)) return false;
    const Shape sh = pair_shape(shape_for(row_tiles(w.n_out), steps_rt(w), true, w.fmt));
    return sh.rt * sh.kw <= (w.fmt == FMT_Q6_K || w.fmt == FMT_Q40 ? 8u : 16u);  // (their shared-launch kernels are bounded at 8 waves)
}

bool decode_batchable(const WeightView& w, size_t t) {
    if (!mfma_decode_format(w.fmt)) return false;
    if (t < 1 || t > 8) return false;
    const Shape sh = shape_for(row_tiles(w.n_out), steps_rt(w), true, w.fmt);  // as a launch of its own: same bits
    bool alds;
    const size_t lds = lds_bytes(w.fmt, false, steps_rt(w), t <= 4 ? 4 : 8, sh, &alds);
    return alds && lds <= LDS_MAX;
}

// Scratch a launch of this weight alone takes when its shape slices K across workgroups (floats of partial rows,
// arrival counters); both zero when K stays inside a workgroup.
void decode_scratch_need(const WeightView& w, size_t* partial_floats, size_t* ncounters, bool pair) {
    *partial_floats = *ncounters = 0;
    if (!mfma_decode_format(w.fmt)) return;
    const uint32_t ntiles = row_tiles(w.n_out);
    const Shape sh = shape_for(ntiles, steps_rt(w), true, w.fmt);
    if (sh.ks <= 1) return;
    const uint32_t per_wg = pair_tiles(sh, pair);
    *partial_floats = (size_t)sh.ks * 8 * w.n_out * (pair ? 2 : 1);
    *ncounters = (size_t)((ntiles + per_wg - 1) / per_wg) * CTR_STRIDE;
}

// Every item must be decode_batchable. Items go out in launches of up to BATCH_MAX jobs; jobs whose shape slices K
// across workgroups take their partial rows and counters from `sc` (hipErrorOutOfMemory when it is too small:
// nothing has been launched then and the caller launches the jobs one by one).
// A job's workgroups in a shared launch: row tiles per workgroup and the mapping of runs to waves (decode_body).
struct Placed {
    uint32_t rt;
    Mapping map;
    uint32_t wgs;
    size_t lds;
};
// Plain: the shape's own workgroups, as a launch of the job alone has them.
// Fat (for launches that still fill seven eighths of the chip's two places per CU that way): a workgroup takes as many of the shape's slices as
// keep two workgroups' staging within a CU's LDS, a wave streams about FAT_STEPS steps, and the workgroup has
// eight waves' worth of tiles. Fewer, fatter workgroups stage less, start and finish less often and keep longer
// streams: the shared launch of eight GGUF matmuls runs 5 % faster with them, every row's bits unchanged. A launch of a
// job alone needs the many small workgroups to cover the chip, which is why the shape keeps describing those.
constexpr uint32_t FAT_STEPS = 32, FAT_STEPS_Q6K = 24;  // (Q6_K's records are 1.7 KiB, the others' 1 to 1.2 KiB)
Placed place_job(const DecodeBatchItem& it, bool fat, uint32_t fat_steps) {
    if (it.w.fmt == FMT_Q6_K && fat_steps == FAT_STEPS) fat_steps = FAT_STEPS_Q6K;
    const uint32_t ntiles = row_tiles(it.w.n_out), nsteps = steps_rt(it.w);
    const bool pair = it.epi.pair_p0 != nullptr;
    Shape sh = shape_for(ntiles, nsteps, true, it.w.fmt);
    if (pair) sh = pair_shape(sh);
    const int tpad = it.t <= 4 ? 4 : 8;
    Placed pl{sh.rt, Mapping{sh.kw, 1}, 0, 0};
    bool alds = false;
    if (fat && nsteps % (sh.ks * sh.kw) == 0) {  // (every run has the same number of steps)
        const uint32_t sl = nsteps / sh.ks;
        uint32_t fs = sh.ks;
        Shape probe = sh;
        probe.rt = 8;
        while (fs > 1 && lds_bytes(it.w.fmt, false, nsteps, tpad, probe, &alds, 1, Mapping{1, fs}) > 80 * 1024) fs /= 2;
        uint32_t kwp = 1;
        while (kwp * 2 <= fs * sh.kw && kwp * 2 <= 8 && (fs * sl / (kwp * 2) >= fat_steps || fs * sh.kw / kwp > 4)) kwp *= 2;  // (a wave holds four runs at most)
        if (pair && kwp == 8) kwp = 4;  // (a pair's workgroup holds an even number of tiles)
        uint32_t rt = 8 / kwp;
        const uint32_t cap = pair ? 2 * ntiles : ntiles;
        while (rt > 1 && rt / 2 >= cap) rt /= 2;
        probe.rt = rt;
        const size_t l = lds_bytes(it.w.fmt, false, nsteps, tpad, probe, &alds, 1, Mapping{kwp, fs});
        if (alds && l <= LDS_MAX && (!pair || rt % 2 == 0)) {
            pl.rt = rt;
            pl.map = Mapping{kwp, fs};
            pl.lds = l;
        }
    }
#ifdef OXHIP_TUNING  // tuning builds only: "tiles:steps:tokens=rt,kwp,fs;..." in OXHIP_MAP overrides a job's mapping (tokens: 4 or 8 = its padding)
    if (const char* e = getenv("OXHIP_MAP")) {
        for (const char* p = e; fat && p && *p;) {
            unsigned nt = 0, ns = 0, tp = 0, a = 0, b = 0, c = 0;
            if (sscanf(p, "%u:%u:%u=%u,%u,%u", &nt, &ns, &tp, &a, &b, &c) == 6 && nt == ntiles && ns == nsteps && (int)tp == tpad && a >= 1 && b >= 1 && c >= 1 &&
                a * b <= 8 && sh.ks % c == 0 && (c * sh.kw) % b == 0 && c * sh.kw / b <= 4 && nsteps % (sh.ks * sh.kw) == 0 && (!pair || a % 2 == 0)) {
                Shape probe = sh;
                probe.rt = a;
                const size_t l = lds_bytes(it.w.fmt, false, nsteps, tpad, probe, &alds, 1, Mapping{b, c});
                if (alds && l <= LDS_MAX) {
                    pl.rt = a;
                    pl.map = Mapping{b, c};
                    pl.lds = l;
                }
            }
            p = strchr(p, ';');
            if (p) p++;
        }
        if (getenv("OXHIP_MAP_PRINT"))
            fprintf(stderr, "job fmt %d tiles %u steps %u tpad %d: shape (%u,%u,%u) -> rt %u kwp %u fs %u lds %zu\n", it.w.fmt, ntiles, nsteps, tpad, sh.rt, sh.kw, sh.ks, pl.rt,
                    pl.map.kwp, pl.map.fs, pl.lds);
    }
#endif
    if (!pl.lds) {
        pl.lds = lds_bytes(it.w.fmt, false, nsteps, tpad, sh, &alds);
        if (!alds) pl.lds = LDS_MAX + 1;  // (refused by the caller)
    }
    const uint32_t per_wg = pair ? pl.rt / 2 : pl.rt;
    pl.wgs = (ntiles + per_wg - 1) / per_wg * (sh.ks / pl.map.fs);
    return pl;
}

hipError_t launch_decode_mfma_batch(const DecodeBatchItem* items, size_t n, const DecodeScratch& sc, hipStream_t s, hipEvent_t ev_start,
                                    hipEvent_t ev_stop) {
    static std::atomic<uint64_t> allowed[4];  // whole LDS allowed, one bit per device
    int dev = 0;
    (void)hipGetDevice(&dev);
    const uint64_t bit = 1ull << (dev & 63);
    if (!(allowed[(dev >> 6) & 3].load(std::memory_order_acquire) & bit)) {
#define OXHIP_BATCH_KERNELS(F) reinterpret_cast<const void*>(decode_batch_kernel<F, false>), reinterpret_cast<const void*>(decode_batch_kernel<F, true>)
        for (const void* k : {OXHIP_BATCH_KERNELS(FSET_GGUF), OXHIP_BATCH_KERNELS(FSET_MLX), OXHIP_BATCH_KERNELS(FSET_K5),
                              OXHIP_BATCH_KERNELS(FSET_Q40), OXHIP_BATCH_KERNELS(FSET_MX4), OXHIP_BATCH_KERNELS(FSET_Q8F)}) {
#undef OXHIP_BATCH_KERNELS
            hipError_t e = hipFuncSetAttribute(k, hipFuncAttributeMaxDynamicSharedMemorySize, (int)LDS_MAX);
            if (e != hipSuccess) return e;
        }
        allowed[(dev >> 6) & 3].fetch_or(bit, std::memory_order_release);
    }
    std::vector<BatchArgs> launches;
    std::vector<size_t> ldss;
    std::vector<uint32_t> threadss;
    std::vector<bool> fats;
    // the jobs by format set (the caller's order within a set), then launches of up to BATCH_MAX jobs of one set
    std::vector<const DecodeBatchItem*> sorted;
    std::vector<std::pair<size_t, size_t>> runs;  // [first, count) into `sorted`
    sorted.reserve(n);
    uint32_t call_mask = 0;
    for (size_t i = 0; i < n; i++) call_mask |= fbit(items[i].w.fmt);
    for (int set = 0; set < NSETS; set++) {
        const size_t first = sorted.size();
        for (size_t i = 0; i < n; i++) {
            const int so = set_of(items[i].w.fmt, call_mask);
            if (so < 0) return hipErrorInvalidValue;
            if (so == set) sorted.push_back(&items[i]);
        }
        for (size_t i0 = first; i0 < sorted.size(); i0 += BATCH_MAX) runs.emplace_back(i0, std::min(sorted.size() - i0, (size_t)BATCH_MAX));
    }
    for (const auto& run : runs) {
        const DecodeBatchItem* const* items_of = sorted.data() + run.first;
        BatchArgs a{};
        a.njobs = (uint32_t)run.second;
        size_t lds = 0, pf = 0, nc = 0;  // scratch is shared by the jobs of one launch, reused by the next launch
        uint32_t wg = 0, threads = 64;
        // Block order within the launch. Workgroups start in block order, so the last jobs make the tail of the launch,
        // when the CUs run dry one after the other: it is shortest when its workgroups do little work per byte and
        // have no slices to combine. Formats with more instruction work per byte go first (4-bit, 6-bit, 8-bit; the
        // caller's order within a format), and in the last format present the jobs that slice K go before the others.
        uint32_t order[BATCH_MAX];
        {
            auto cls = [](int fmt) { return q8_format(fmt) ? 2 : fmt == FMT_Q6_K ? 1 : 0; };
            auto sliced = [](const WeightView& w) {
                return shape_for(row_tiles(w.n_out), steps_rt(w), true, w.fmt).ks > 1;
            };
            int last = 0;
            for (uint32_t j = 0; j < a.njobs; j++) last = std::max(last, cls(items_of[j]->w.fmt));
            uint32_t key[BATCH_MAX];
            for (uint32_t j = 0; j < a.njobs; j++) {
                const WeightView& w = items_of[j]->w;
                key[j] = 2 * cls(w.fmt) + (cls(w.fmt) == last && !sliced(w) ? 1 : 0);
                order[j] = j;
            }
            std::stable_sort(order, order + a.njobs, [&](uint32_t x, uint32_t y) { return key[x] < key[y]; });
        }
        // fat workgroups when they still fill most of the chip
        // (measured: 1056 and 480 fat workgroups beat the plain mapping by 4 to 5 %, 512 are even, 296 lose 40 %)
        uint32_t fat_steps = FAT_STEPS, fat_min = 7 * NCU / 4;
#ifdef OXHIP_TUNING  // tuning builds only: "steps a wave streams, least number of workgroups" in OXHIP_FAT
        if (const char* e = getenv("OXHIP_FAT")) {
            unsigned x = 0, y = 0;
            if (sscanf(e, "%u,%u", &x, &y) == 2 && x >= 1) {
                fat_steps = x;
                fat_min = y;
            }
        }
#endif
        uint64_t fat_wgs = 0;
        for (uint32_t j = 0; j < a.njobs; j++) fat_wgs += place_job(*items_of[j], true, fat_steps).wgs;
        const bool fat = fat_wgs >= fat_min;
        for (uint32_t j = 0; j < a.njobs; j++) {
            const DecodeBatchItem& it = *items_of[order[j]];
            const uint32_t ntiles = row_tiles(it.w.n_out), nsteps = steps_rt(it.w);
            const bool pair = it.epi.pair_p0 != nullptr;
            Shape sh = shape_for(ntiles, nsteps, true, it.w.fmt);
            if (pair) sh = pair_shape(sh);
            const Placed pl = place_job(it, fat, fat_steps);
            const size_t l = pl.lds;
            if (l > LDS_MAX || it.t < 1 || it.t > 8) return hipErrorInvalidValue;
            sh.rt = pl.rt;
            const uint32_t per_wg = pair ? sh.rt / 2 : sh.rt;
            const uint32_t groups = (ntiles + per_wg - 1) / per_wg;
            float* partial = nullptr;
            uint32_t* counters = nullptr;
            if (sh.ks > 1) {
                const size_t need = (size_t)sh.ks * it.t * it.w.n_out * (pair ? 2 : 1);
                if (!sc.partial || !sc.counters || pf + need > sc.partial_floats || nc + (size_t)groups * CTR_STRIDE > sc.ncounters) return hipErrorOutOfMemory;
                partial = sc.partial + pf;
                counters = sc.counters + nc;
                pf += (need + 63) / 64 * 64;
                nc += (size_t)groups * CTR_STRIDE;
            }
            lds = l > lds ? l : lds;
            threads = 64 * sh.rt * pl.map.kwp > threads ? 64 * sh.rt * pl.map.kwp : threads;
            a.j[j] = BatchJob{it.w, it.xa, it.y, partial, counters, it.t, sh.rt, sh.kw, sh.ks, wg, pl.map, it.epi};
            wg += groups * (sh.ks / pl.map.fs);
        }
        a.nwg = wg;
        launches.push_back(a);
        fats.push_back(fat);
        ldss.push_back(lds);
        threadss.push_back(threads);
    }
    // Timing events: with one launch they ride on the dispatch itself (its start and end as the device saw them, and no
    // barrier packets on the stream, which would keep neighbouring launches from overlapping); with several they are
    // recorded on the stream before the first and after the last.
    const bool ride = launches.size() == 1 && launches[0].nwg && (ev_start || ev_stop);
    if (!ride && ev_start) {
        hipError_t e = hipEventRecord(ev_start, s);
        if (e != hipSuccess) return e;
    }
    for (size_t i = 0; i < launches.size(); i++) {
        if (!launches[i].nwg) continue;
        uint32_t fset = 0;
        for (uint32_t j = 0; j < launches[i].njobs; j++) fset |= fbit(launches[i].j[j].w.fmt);
        if (threadss[i] > (fset == FSET_Q40 ? 512u : 1024u)) return hipErrorInvalidValue;  // (the kernels' launch bounds)
        auto go = [&](auto kern) {
            if (ride) hipExtLaunchKernelGGL(kern, dim3(launches[i].nwg), dim3(threadss[i]), (uint32_t)ldss[i], s, ev_start, ev_stop, 0, launches[i]);
            else kern<<<launches[i].nwg, threadss[i], ldss[i], s>>>(launches[i]);
        };
        const bool fat = fats[i];
#define OXHIP_GO(F) (fat ? go(decode_batch_kernel<F, true>) : go(decode_batch_kernel<F, false>))
        if (!(fset & ~FSET_GGUF)) OXHIP_GO(FSET_GGUF);
        else if (!(fset & ~FSET_MLX)) OXHIP_GO(FSET_MLX);
        else if (!(fset & ~FSET_K5)) OXHIP_GO(FSET_K5);
        else if (!(fset & ~FSET_Q40)) OXHIP_GO(FSET_Q40);
        else if (!(fset & ~FSET_MX4)) OXHIP_GO(FSET_MX4);
        else if (!(fset & ~FSET_Q8F)) OXHIP_GO(FSET_Q8F);
#undef OXHIP_GO
        else return hipErrorInvalidValue;
        hipError_t e = hipGetLastError();
        if (e != hipSuccess) return e;
    }
    if (!ride && ev_stop) return hipEventRecord(ev_stop, s);
    return hipSuccess;
}

// Whether the grouped launch of fused gate / up experts can pair its gate and up tiles per workgroup (and so apply the
// activation and the quantization itself): its shape gives a workgroup a multiple of four row tiles.
bool decode_grouped_glu_ok(const WeightView& w, size_t inter) {
    if (!mfma_decode_format(w.fmt) || w.fmt == FMT_Q6_K || inter % 32 || w.n_out != 2 * inter) return false;
    return grouped_shape(steps_rt(w), 8).rt % 4 == 0 && grouped_shape(steps_rt(w), 32).rt % 4 == 0;
}

// Whether a grouped launch with chunks of up to max_rows rows fits this weight's staged activations into LDS.
bool decode_grouped_fits(const WeightView& w, uint32_t max_rows) {
    if (!mfma_decode_format(w.fmt) || max_rows < 1 || max_rows > 32) return false;
    const uint32_t nsteps = steps_rt(w);
    const Shape sh = grouped_shape(nsteps, max_rows);
    const uint32_t ng = max_rows <= 8 ? 1 : (max_rows <= 16 ? 2 : 4);
    bool alds;
    const size_t lds = lds_bytes(w.fmt, false, nsteps, max_rows <= 4 ? 4 : 8, sh, &alds, ng);
    return lds <= LDS_MAX && (alds || (ng == 1 && w.fmt != FMT_Q6_K));
}

hipError_t launch_decode_mfma_grouped(const WeightView& w, const QActView& xa, const GroupView& g, uint32_t max_chunks,
                                      uint32_t max_rows_per_chunk, float* y, hipStream_t s) {
    if (!max_chunks) return hipSuccess;
    switch (w.fmt) {
        case FMT_Q8_0: return run_grouped<FMT_Q8_0>(w, xa, g, max_chunks, max_rows_per_chunk, y, s);
        case FMT_Q4_K: return run_grouped<FMT_Q4_K>(w, xa, g, max_chunks, max_rows_per_chunk, y, s);
        case FMT_Q4M: return run_grouped<FMT_Q4M>(w, xa, g, max_chunks, max_rows_per_chunk, y, s);
        case FMT_Q40: return run_grouped<FMT_Q40>(w, xa, g, max_chunks, max_rows_per_chunk, y, s);
        case FMT_MXFP4: return run_grouped<FMT_MXFP4>(w, xa, g, max_chunks, max_rows_per_chunk, y, s);
        default: return hipErrorInvalidValue;
    }
}

hipError_t launch_decode_mfma(const WeightView& w, const QActView& xa, size_t t, float* y, const DecodeScratch& sc, hipStream_t s,
                              hipEvent_t ev_start, hipEvent_t ev_stop, const Epi& epi) {
    switch (w.fmt) {
        case FMT_Q8_0: return run<FMT_Q8_0, false>(w, xa, t, y, nullptr, sc, s, ev_start, ev_stop, epi);
        case FMT_Q8F: return run<FMT_Q8F, false>(w, xa, t, y, nullptr, sc, s, ev_start, ev_stop, epi);
        case FMT_Q4_K: return run<FMT_Q4_K, false>(w, xa, t, y, nullptr, sc, s, ev_start, ev_stop, epi);
        case FMT_Q5_K: return run<FMT_Q5_K, false>(w, xa, t, y, nullptr, sc, s, ev_start, ev_stop, epi);
        case FMT_Q6_K: return run<FMT_Q6_K, false>(w, xa, t, y, nullptr, sc, s, ev_start, ev_stop, epi);
        case FMT_Q4M: return run<FMT_Q4M, false>(w, xa, t, y, nullptr, sc, s, ev_start, ev_stop, epi);
        case FMT_Q40: return run<FMT_Q40, false>(w, xa, t, y, nullptr, sc, s, ev_start, ev_stop, epi);
        case FMT_MXFP4: return run<FMT_MXFP4, false>(w, xa, t, y, nullptr, sc, s, ev_start, ev_stop, epi);
        default: return hipErrorInvalidValue;
    }
}

// The integer block sums the kernel forms ([t][n_out][n_in/32]; Q6_K: per 16, [t][n_out][n_in/16]); y is scratch of [t][n_out].
hipError_t launch_isums_mfma(const WeightView& w, const QActView& xa, size_t t, float* y, int32_t* out, hipStream_t s) {
    switch (w.fmt) {
        case FMT_Q8_0: return run<FMT_Q8_0, true>(w, xa, t, y, out, DecodeScratch{}, s);
        case FMT_Q8F: return run<FMT_Q8F, true>(w, xa, t, y, out, DecodeScratch{}, s);
        case FMT_Q4_K: return run<FMT_Q4_K, true>(w, xa, t, y, out, DecodeScratch{}, s);
        case FMT_Q5_K: return run<FMT_Q5_K, true>(w, xa, t, y, out, DecodeScratch{}, s);
        case FMT_Q6_K: return run<FMT_Q6_K, true>(w, xa, t, y, out, DecodeScratch{}, s);
        case FMT_Q4M: return run<FMT_Q4M, true>(w, xa, t, y, out, DecodeScratch{}, s);
        case FMT_Q40: return run<FMT_Q40, true>(w, xa, t, y, out, DecodeScratch{}, s);
        case FMT_MXFP4: return run<FMT_MXFP4, true>(w, xa, t, y, out, DecodeScratch{}, s);
        default: return hipErrorInvalidValue;
    }
}

}  // namespace oxhip
