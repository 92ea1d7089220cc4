// FP8 E4M3 block-scaled weights at up to 32 tokens: a bandwidth-bound skinny GEMM on the bf16 matrix cores.
//
// The reference runs float-stored matrices through its f32 path at every token count (src/kernels.rs:1802):
// w[r][c] = e4m3(byte) * s[r / 128][c / 128] (src/ggml.rs:259-293, :433-444), y = x W^T in f32. Here the e4m3 bytes
// become bf16 exactly (one conversion instruction per two weights), the activations are bf16 (bf16 inputs, or f32
// inputs split into a bf16 value and a bf16 residual: two planes, exact to 2^-17), the products accumulate in f32 per
// 128-column block, and the block scale multiplies the block's sum once: the same value as scaling every weight, in
// 1/32 of the multiplies.
//
// A wave streams 16 RT rows x its slice of K: a lane (kq, n) owns 32 consecutive bytes of row n per 128-column step
// (the weights are tile-packed at upload so that a wave's 64 lanes read one contiguous 2 KiB record), through a register ring; the activation fragments come packed in operand order from
// a small buffer that stays in L2. Rows are bit-identical whatever the batch (one fixed order per (token, row)).
#include "internal.hpp"

#include <cstdlib>
#include <type_traits>

namespace oxhip {

namespace {

typedef __bf16 bf16x8 __attribute__((ext_vector_type(8)));
typedef __bf16 bf16x2 __attribute__((ext_vector_type(2)));
typedef float f32x4 __attribute__((ext_vector_type(4)));
typedef float f32x2 __attribute__((ext_vector_type(2)));

// Requests to memory cost the same whether 4 or 64 of a wave's lanes take part, and at a few tokens they, not the bytes
// of the weights, would bound the kernel. So a token tile's fragments are packed for the smallest TS in {4, 8, 16} that
// holds its tokens: one 16-byte request of lane 16 kq + n brings token n % TS its 8 columns 32 kq + 8 b + j of a step, with
// b = n / TS + (16 / TS) i for request i of TS / 4; the lanes of the 16 token rows of the matrix cores then take their four
// blocks b from lanes n + TS (b % (16 / TS)) with a row shift.
//
// x [t][n_in] -> [ttile][plane][step][request i][lane][8 bf16]. Plane 0 is bf16(x), plane 1 (f32 sources) bf16(x - plane 0).
// Tokens past t are zero.
template <bool SRC_BF16>
__global__ __launch_bounds__(256) void pack_skinny_kernel(const void* __restrict__ x, uint32_t t, uint32_t n_in, uint32_t ttiles,
                                                        uint32_t planes, uint32_t nsteps, uint32_t ts, uint4* __restrict__ out) {
    const size_t idx = (size_t)blockIdx.x * blockDim.x + threadIdx.x;
    const uint32_t cnt = ts / 4;
    if (idx >= (size_t)ttiles * planes * nsteps * cnt * 64) return;
    const uint32_t lane = idx & 63, n = lane & 15, kq = lane >> 4;
    size_t q = idx >> 6;
    const uint32_t i = (uint32_t)(q % cnt);
    q /= cnt;
    const uint32_t st = (uint32_t)(q % nsteps);
    q /= nsteps;
    const uint32_t pl = (uint32_t)(q % planes), tt = (uint32_t)(q / planes);
    const uint32_t tok = tt * 16 + n % ts, b = n / ts + (16 / ts) * i;
    uint32_t pk[4] = {0, 0, 0, 0};
    if (tok < t) {
#pragma unroll
        for (int j = 0; j < 8; j++) {
            const uint32_t k = 128 * st + 32 * kq + 8 * b + j;
            uint16_t h;
            if (SRC_BF16) {
                h = pl ? 0 : reinterpret_cast<const uint16_t*>(x)[(size_t)tok * n_in + k];
            } else {
                const float v = reinterpret_cast<const float*>(x)[(size_t)tok * n_in + k];
                const uint16_t hi = f32_to_bf16_bits(v);
                h = pl ? f32_to_bf16_bits(v - bf16_bits_to_f32(hi)) : hi;
            }
            pk[j >> 1] |= (uint32_t)h << (16 * (j & 1));
        }
    }
    out[idx] = make_uint4(pk[0], pk[1], pk[2], pk[3]);
}

// lane i of each row of 16 takes the value of lane i + SH of the row (zero past the row's end)
template <int SH>
__device__ inline uint4 row_take(const uint4& v) {
    if (SH == 0) return v;
    constexpr int ctrl = 0x100 + (SH ? SH : 1);  // row_shl:SH
    return make_uint4((uint32_t)__builtin_amdgcn_update_dpp(0, (int)v.x, ctrl, 0xf, 0xf, true),
                      (uint32_t)__builtin_amdgcn_update_dpp(0, (int)v.y, ctrl, 0xf, 0xf, true),
                      (uint32_t)__builtin_amdgcn_update_dpp(0, (int)v.z, ctrl, 0xf, 0xf, true),
                      (uint32_t)__builtin_amdgcn_update_dpp(0, (int)v.w, ctrl, 0xf, 0xf, true));
}

// DIRECT (at most 4 tokens, f32 activations kept exact): `apk` is x itself, [t][n_in] f32: lane 16 kq + n reads the 8
// columns of token n % 4 and block n / 4 (32 bytes; a token's 16 lanes cover a step's 512 bytes) and splits them into
// the bf16 value and residual planes in registers; no packing kernel and no scratch.
// grid x: groups of RT row tiles; grid y: K slices; the workgroup's `kw` waves split the slice's steps and meet in LDS in
// wave order; with more than one slice the sums go out as f32 partial rows [slice][t][n_out] that a second kernel adds.
// PF: 128-column steps a wave keeps on request. A step's activation fragments (L2 hits) are requested together with its
// weights: loads complete in issue order, so fragments asked for any later would make the wave wait for every weight
// request issued before them and cut the depth of the ring.
template <int RT, int NTT, int NP, int TS, bool OUT_BF16, bool DIRECT = false>
__global__ __launch_bounds__(512) void skinny_fp8_kernel(WeightView w, const uint4* __restrict__ apk, uint32_t t, uint32_t kw,
                                                         void* __restrict__ yv, float* __restrict__ partial) {
    constexpr int CNT = TS / 4, PER = 16 / TS;  // requests per step and plane; blocks b in a request
    constexpr int PF = 2 * RT + NTT * NP * CNT > 12 ? 2 : 4;
    extern __shared__ __align__(16) float red[];  // [kw][RT][NTT][64][4]
    const uint32_t lane = threadIdx.x & 63, wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
    const uint32_t n = lane & 15, kq = lane >> 4;
    const uint32_t nsteps = w.n_in / 128, ntiles = (w.n_out + 15) / 16;
    // wave v of slice z takes steps z kw + v, + kw slices, ...: at any moment the workgroups of a row group read one
    // contiguous window of its records
    const uint32_t gw = blockIdx.y * kw + wave, stride = kw * gridDim.y;  // kw * slices <= nsteps
    const uint32_t cnt = (nsteps - gw + stride - 1) / stride, ilast = cnt - 1;
    const uint8_t* wp[RT];
    const float* sp[RT];
    const uint32_t scols = (w.n_in + w.bc - 1) / w.bc;
    const uint32_t wstep = w.group == 1 ? 2048 : 128;  // bytes between a lane's chunks of consecutive steps
    const uint32_t whi = fp8_second_chunk(w);
#pragma unroll
    for (int r = 0; r < RT; r++) {
        const uint32_t tile = min(blockIdx.x * RT + r, ntiles - 1), row = min(tile * 16 + n, w.n_out - 1);
        wp[r] = w.p0 + fp8_offset(w, row, 32 * kq);
        sp[r] = reinterpret_cast<const float*>(w.p1) + (size_t)(tile * 16 / w.br) * scols;
    }
    static_assert(!DIRECT || (TS == 4 && NP == 2 && NTT == 1), "direct f32 activations: up to 4 tokens, two planes");
    const uint4* ap = apk + lane;
    // DIRECT: the lane's 8 columns of a step start at xd + 128 s (absent tokens read token t - 1 and are zeroed)
    const float* xd = reinterpret_cast<const float*>(apk) + (size_t)min(n & 3u, t - 1) * w.n_in + 32 * kq + 8 * (n >> 2);
    const bool xlive = (n & 3u) < t;
    struct St {
        uint4 lo[RT], hi[RT];
        float sc[RT];
        uint4 a[NTT][NP][CNT];  // DIRECT: a[0][0][0], a[0][1][0] hold the 8 f32 values until they are split
    };
    auto load = [&](St& st, uint32_t s) {  // s: a step of the matrix
#pragma unroll
        for (int r = 0; r < RT; r++) {
            const uint8_t* p = wp[r] + wstep * (size_t)s;
            // (the one-to-four-token variant marks its weight bytes as read once, -4 % at one token; the 32-token variant
            // with its four row tiles per wave lost 5 % with the same hint)
            st.lo[r] = DIRECT ? gload_once<uint4>(as_global(p)) : gload<uint4>(as_global(p));
            st.hi[r] = DIRECT ? gload_once<uint4>(as_global(p + whi)) : gload<uint4>(as_global(p + whi));
            st.sc[r] = sp[r][(128 * s) / w.bc];
        }
        if (DIRECT) {
            const uint4* p = reinterpret_cast<const uint4*>(xd + 128 * (size_t)s);
            st.a[0][0][0] = p[0];
            st.a[0][NP - 1][0] = p[1];
        } else {
#pragma unroll
            for (int tt = 0; tt < NTT; tt++)
#pragma unroll
                for (int pl = 0; pl < NP; pl++)
#pragma unroll
                    for (int i = 0; i < CNT; i++) st.a[tt][pl][i] = ap[((((size_t)tt * NP + pl) * nsteps + s) * CNT + i) * 64];
        }
    };
    // DIRECT: 8 f32 -> the two bf16 planes (round to nearest even; the residual x - bf16(x) is exact in f32)
    auto split = [&](const St& st, uint4& hi, uint4& lo) {
        const uint32_t raw[8] = {st.a[0][0][0].x, st.a[0][0][0].y, st.a[0][0][0].z, st.a[0][0][0].w,
                                 st.a[0][NP - 1][0].x, st.a[0][NP - 1][0].y, st.a[0][NP - 1][0].z, st.a[0][NP - 1][0].w};
        uint32_t h[4], l[4];
#pragma unroll
        for (int j = 0; j < 4; j++) {
            const float x0 = xlive ? __uint_as_float(raw[2 * j]) : 0.0f, x1 = xlive ? __uint_as_float(raw[2 * j + 1]) : 0.0f;
            const uint32_t hp = __builtin_bit_cast(uint32_t, __builtin_convertvector(f32x2{x0, x1}, bf16x2));
            const float r0 = x0 - __uint_as_float(hp << 16), r1 = x1 - __uint_as_float(hp & 0xFFFF0000u);
            h[j] = hp;
            l[j] = __builtin_bit_cast(uint32_t, __builtin_convertvector(f32x2{r0, r1}, bf16x2));
        }
        hi = make_uint4(h[0], h[1], h[2], h[3]);
        lo = make_uint4(l[0], l[1], l[2], l[3]);
    };
    f32x4 acc[RT][NTT];
#pragma unroll
    for (int r = 0; r < RT; r++)
#pragma unroll
        for (int tt = 0; tt < NTT; tt++) acc[r][tt] = f32x4{0.0f, 0.0f, 0.0f, 0.0f};

    St ring[PF];
#pragma unroll
    for (int p = 0; p < PF; p++) load(ring[p], gw + stride * min((uint32_t)p, ilast));
    auto frag = [&](const St& st, const uint4* dp, int tt, int pl, int b) -> uint4 {
        const uint4& v = DIRECT ? dp[pl] : st.a[tt][pl][b / PER];
        switch (TS * (b % PER)) {
            case 4: return row_take<4>(v);
            case 8: return row_take<8>(v);
            case 12: return row_take<12>(v);
            default: return v;
        }
    };
    auto compute = [&](const St& st) {
        uint4 dp[2];
        if (DIRECT) split(st, dp[0], dp[1]);
#pragma unroll
        for (int r = 0; r < RT; r++) {
            const uint32_t d[8] = {st.lo[r].x, st.lo[r].y, st.lo[r].z, st.lo[r].w, st.hi[r].x, st.hi[r].y, st.hi[r].z, st.hi[r].w};
            f32x4 D[NTT];
#pragma unroll
            for (int tt = 0; tt < NTT; tt++) D[tt] = f32x4{0.0f, 0.0f, 0.0f, 0.0f};
#pragma unroll
            for (int b = 0; b < 4; b++) {  // bytes 8 b .. 8 b + 7 of the lane's 32: one 32-column block of the matrix cores
                const bf16x2 w0 = __builtin_amdgcn_cvt_scalef32_pk_bf16_fp8((int)d[2 * b], 1.0f, false);
                const bf16x2 w1 = __builtin_amdgcn_cvt_scalef32_pk_bf16_fp8((int)d[2 * b], 1.0f, true);
                const bf16x2 w2 = __builtin_amdgcn_cvt_scalef32_pk_bf16_fp8((int)d[2 * b + 1], 1.0f, false);
                const bf16x2 w3 = __builtin_amdgcn_cvt_scalef32_pk_bf16_fp8((int)d[2 * b + 1], 1.0f, true);
                const bf16x8 wb = {w0.x, w0.y, w1.x, w1.y, w2.x, w2.y, w3.x, w3.y};
#pragma unroll
                for (int tt = 0; tt < NTT; tt++)
#pragma unroll
                    for (int pl = 0; pl < NP; pl++)
                        D[tt] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(__builtin_bit_cast(bf16x8, frag(st, dp, tt, pl, b)), wb, D[tt], 0, 0, 0);
            }
#pragma unroll
            for (int tt = 0; tt < NTT; tt++)
#pragma unroll
                for (int i = 0; i < 4; i++) acc[r][tt][i] = fmaf(st.sc[r], D[tt][i], acc[r][tt][i]);
        }
    };
    // refills ask for a clamped step unconditionally (the last ones repeat the wave's last step), which keeps the number
    // of requests in flight known at every wait
    for (uint32_t ib = 0; ib < cnt; ib += PF) {
#pragma unroll
        for (int p = 0; p < PF; p++) {
            if (ib + p < cnt) compute(ring[p]);
            load(ring[p], gw + stride * min(ib + PF + p, ilast));
        }
    }
#pragma unroll
    for (int r = 0; r < RT; r++)
#pragma unroll
        for (int tt = 0; tt < NTT; tt++)
            *reinterpret_cast<f32x4*>(red + ((((size_t)wave * RT + r) * NTT + tt) * 64 + lane) * 4) = acc[r][tt];
    __syncthreads();
    // D[token 4 kq + i][row n]: thread (r, tt, lane) adds the waves in order and stores its four tokens
    for (uint32_t idx = threadIdx.x; idx < RT * NTT * 64; idx += blockDim.x) {
        const uint32_t l = idx & 63, tt = (idx >> 6) % NTT, r = (idx >> 6) / NTT;
        const uint32_t row = (blockIdx.x * RT + r) * 16 + (l & 15);
        if (row >= w.n_out || blockIdx.x * RT + r >= ntiles) continue;
        f32x4 sum = *reinterpret_cast<const f32x4*>(red + (((size_t)r * NTT + tt) * 64 + l) * 4);
        for (uint32_t k = 1; k < kw; k++) {
            const f32x4 v = *reinterpret_cast<const f32x4*>(red + ((((size_t)k * RT + r) * NTT + tt) * 64 + l) * 4);
#pragma unroll
            for (int i = 0; i < 4; i++) sum[i] += v[i];
        }
#pragma unroll
        for (int i = 0; i < 4; i++) {
            const uint32_t tok = 16 * tt + 4 * (l >> 4) + i;
            if (tok >= t) continue;
            if (gridDim.y > 1) partial[((size_t)blockIdx.y * t + tok) * w.n_out + row] = sum[i];
            else if (OUT_BF16) reinterpret_cast<uint16_t*>(yv)[(size_t)tok * w.n_out + row] = f32_to_bf16_bits(sum[i]);
            else reinterpret_cast<float*>(yv)[(size_t)tok * w.n_out + row] = sum[i];
        }
    }
}

}  // namespace

bool skinny_fp8_ok(const WeightView& w, size_t t) {
    return w.fmt == FMT_FP8 && t >= 1 && t <= 32 && w.n_in % 128 == 0 && w.bc % 128 == 0 && w.br % 16 == 0;
}

// More than 16 tokens: four row tiles per wave (a step's 8 fragment requests then serve 4 records, not 2), and K in two
// slices so that the 112 row groups of a 7168-row matrix still cover the chip.
constexpr uint32_t WIDE_RT = 4, WIDE_SLICES = 2;

static size_t frag_bytes(const WeightView& w, size_t t, int planes) { return (size_t)((t + 15) / 16) * planes * (w.n_in / 32) * 64 * 16; }

// Scratch for t tokens at most (`planes`: 2 for f32 sources kept exact, else 1): the packed fragments, then the partial
// rows of the K slices.
size_t skinny_fp8_pack_bytes(const WeightView& w, size_t t, int planes) {
    return frag_bytes(w, t, planes) + (t > 16 ? (size_t)WIDE_SLICES * t * w.n_out * 4 : 0);
}

// y [t][n_out] (f32 or bf16) = x W^T; `pack` holds skinny_fp8_pack_bytes(). exact_f32: f32 sources go in as two bf16
// planes (value + residual); otherwise they are rounded to bf16 as the prefill GEMM does.
hipError_t launch_skinny_fp8(const WeightView& w, const void* x, bool x_bf16, bool exact_f32, size_t t, void* y, bool y_bf16, void* pack,
                             hipStream_t s) {
    if (!skinny_fp8_ok(w, t)) return hipErrorInvalidValue;
    const uint32_t ttiles = (uint32_t)((t + 15) / 16), planes = (!x_bf16 && exact_f32) ? 2 : 1, nsteps = w.n_in / 128;
    const uint32_t ts = t <= 4 ? 4 : t <= 8 ? 8 : 16;
    // up to 4 tokens of exact f32 activations: the kernel reads x itself (rows of whole 16-byte runs)
    const bool direct = ts == 4 && planes == 2 && w.n_in % 4 == 0 && reinterpret_cast<uintptr_t>(x) % 16 == 0;
    const size_t total = direct ? 0 : (size_t)ttiles * planes * nsteps * (ts / 4) * 64;
    const unsigned pgrid = (unsigned)((total + 255) / 256);
    if (!total) {
    } else if (x_bf16) pack_skinny_kernel<true><<<pgrid, 256, 0, s>>>(x, (uint32_t)t, w.n_in, ttiles, planes, nsteps, ts, static_cast<uint4*>(pack));
    else pack_skinny_kernel<false><<<pgrid, 256, 0, s>>>(x, (uint32_t)t, w.n_in, ttiles, planes, nsteps, ts, static_cast<uint4*>(pack));
    hipError_t e = hipGetLastError();
    if (e != hipSuccess) return e;
    const uint32_t ntiles = (w.n_out + 15) / 16;
    const uint4* a = direct ? static_cast<const uint4*>(x) : static_cast<const uint4*>(pack);
    float* partial = reinterpret_cast<float*>(static_cast<uint8_t*>(pack) + frag_bytes(w, t, (int)planes));
    uint32_t slices = 1;
    auto go = [&](auto kern, uint32_t rt, uint32_t ntt) {
        uint32_t kw = 4;  // (four waves of 36 steps stream [7168, 18432] 5 % faster than eight of 18; two: 45 % slower)
#ifdef OXHIP_TUNING  // tuning builds only: waves per workgroup in OXHIP_FP8_KW
        if (const char* e = getenv("OXHIP_FP8_KW")) kw = (uint32_t)atoi(e);
#endif
        while (kw > 1 && nsteps / (kw * slices) < 4) kw /= 2;
        const size_t lds = (size_t)kw * rt * ntt * 64 * 16;
        if (lds > 48 * 1024) {
            e = hipFuncSetAttribute(reinterpret_cast<const void*>(kern), hipFuncAttributeMaxDynamicSharedMemorySize, (int)lds);
            if (e != hipSuccess) return;
        }
        kern<<<dim3((ntiles + rt - 1) / rt, slices), 64 * kw, lds, s>>>(w, a, (uint32_t)t, kw, y, partial);
    };
    using one = std::integral_constant<int, 1>;
    using two = std::integral_constant<int, 2>;
    auto pick = [&](auto np, auto out) {
        constexpr int NP = decltype(np)::value;
        constexpr bool OB = decltype(out)::value;
        if (ts == 4 && NP == 2 && direct) go(skinny_fp8_kernel<1, 1, 2, 4, OB, true>, 1, 1);
        else if (ts == 4) go(skinny_fp8_kernel<1, 1, NP, 4, OB>, 1, 1);
        else if (ts == 8) go(skinny_fp8_kernel<1, 1, NP, 8, OB>, 1, 1);
        else if (ttiles == 1) go(skinny_fp8_kernel<2, 1, NP, 16, OB>, 2, 1);
        else {
            slices = nsteps >= 8 * WIDE_SLICES ? WIDE_SLICES : 1;
            go(skinny_fp8_kernel<WIDE_RT, 2, NP, 16, OB>, WIDE_RT, 2);
        }
    };
    if (planes == 2) y_bf16 ? pick(two{}, std::true_type{}) : pick(two{}, std::false_type{});
    else y_bf16 ? pick(one{}, std::true_type{}) : pick(one{}, std::false_type{});
    if (e != hipSuccess) return e;
    e = hipGetLastError();
    if (e != hipSuccess || slices == 1) return e;
    return launch_gemm_reduce(partial, t * (size_t)w.n_out, slices, y, y_bf16, s);
}

}  // namespace oxhip
