// Shared declarations of liboxinfer_hip: device layouts, launchers, small device helpers.
#pragma once
#include <hip/hip_runtime.h>
#include <stddef.h>
#include <stdint.h>

#include <mutex>
#include <string>

#include "../../include/oxhip.h"

namespace oxhip {

// ------------------------------------------------------------------------------------------------
// Device layouts. Uploads repack every format so that each lane of a wavefront reads one aligned
// 16-byte chunk and consecutive lanes read consecutive chunks. The bytes are those of the source
// format, only rearranged. Q8_0, Q4_K and Q4 with one scale and offset per 64 (MLX) are stored
// tile-packed for the matrix cores (layout.hpp: all in p0); the others in planes:
//
//   Q4    p0 q   [n_out][n_in/2]      byte j of a 32-block: element j (low nibble), j+16 (high)
//         p1 sc  [n_out][n_in/sgroup] f16 scale; sgroup = 32, or the offset group when every block
//                                     of a group carries the same scale
//         p2 off [n_out][n_in/group]  bf16 offsets, optional
//   Q6_K  p0      T6K records (layout.hpp)
//   Q5_K  p0      TK5 records (layout.hpp)
//   MXFP4 p0      T4X records (layout.hpp)
//   Q40   p0      T4M records of GGUF Q4_0: the four f16 block scales of a row where MLX keeps two scales and two offsets
//   Q8F   p0      T8F records: QMatrix, int8 codes with one f32 scale per 32
//   FP8   p0 q   [n_out][n_in]        e4m3 bytes (row-major, or tile-packed when group == 1: fp8_offset below);
//         p1 bs f32 [ceil(n_out/br)][ceil(n_in/bc)]
//   BF16  p0 q   [n_out][n_in]        bf16
//   NVFP4 p0      T4N records (layout.hpp); p1 f32 scales on top of the decoded values [ceil(n_out/br)][ceil(n_in/bc)],
//                 or none (br == 0). Float-stored like FP8: f32 activations at decode sizes.
// ------------------------------------------------------------------------------------------------
enum Fmt : int { FMT_Q4 = 0, FMT_Q8_0 = 1, FMT_Q4_K = 2, FMT_Q6_K = 3, FMT_FP8 = 4, FMT_BF16 = 5, FMT_Q4M = 6, FMT_Q8F = 7, FMT_Q40 = 8, FMT_Q5_K = 9, FMT_MXFP4 = 10, FMT_NVFP4 = 11 };
// the formats of the matrix-core decode kernels (decode_mfma.hip); the two Q8 kinds carry no sums or offsets
inline bool mfma_decode_format(int f) { return f == FMT_Q8_0 || f == FMT_Q8F || f == FMT_Q4_K || f == FMT_Q6_K || f == FMT_Q4M || f == FMT_Q40 || f == FMT_Q5_K || f == FMT_MXFP4; }
// the two 4-bit formats in T4M records (MLX: a scale and an offset per 64; GGUF Q4_0: a scale per 32)
// (and MXFP4 in the same geometry: 4-bit table codes with a power-of-two scale byte per 32)
__host__ __device__ constexpr bool t4m_format(int f) { return f == FMT_Q4M || f == FMT_Q40 || f == FMT_MXFP4; }
__host__ __device__ constexpr bool q8_format(int f) { return f == FMT_Q8_0 || f == FMT_Q8F; }
// the K-quants in super-block records with 6-bit scales and mins (Q5_K: the Q4_K record and a plane of fifth bits)
__host__ __device__ constexpr bool k45_format(int f) { return f == FMT_Q4_K || f == FMT_Q5_K; }

struct WeightView {
    int fmt;
    uint32_t n_out, n_in;
    const uint8_t* p0;
    const uint8_t* p1;
    const uint8_t* p2;
    const uint8_t* p3;
    uint32_t sgroup;  // Q4: elements per scale
    uint32_t group;   // Q4: elements per offset (0: none)
    uint32_t br, bc;  // FP8 block scale geometry; planar Q4: br = 1 marks GGUF Q4_0 blocks (dequantized without an offset term)
};

struct QActView {
    const int8_t* q;
    const float* scales;
    const int32_t* sums;
    const float* fsums;
    const float* hsums;
    const int32_t* sums16;
};

// How a decode matmul writes its rows (LinMode of the reference's decode graph, src/gpu_decode.rs:37-50): y = v,
// y += v (a residual), or y += sigmoid(gate[token]) * v (a gated shared expert).
enum : uint32_t { EPI_STORE = 0, EPI_ADD = 1, EPI_ADD_GATED = 2 };
struct Epi {
    uint32_t mode = EPI_STORE;
    const float* gate = nullptr;  // EPI_ADD_GATED: one f32 per token
    // A gate / up pair in one launch (LinMode::SiluPair / GeluPair, src/gpu_decode.rs:43-46; the CUDA kernels' modes 2 and
    // 3, src/cuda_decode.cu:131-167): pair_p0 != nullptr is the second matrix's records (same shape and format as the
    // first). A workgroup streams the tiles of the same rows of both matrices and stores act(W x) * (W2 x); each product's
    // sum is formed exactly as a launch of its own forms it, so the result is gated_act of the two separate products, bit
    // for bit. pair_act: 0 SiLU, 1 GELU-tanh. Stores only (mode EPI_STORE).
    const uint8_t* pair_p0 = nullptr;
    uint32_t pair_act = 0;
};

// A grouped launch (MoE): chunk c = {expert, first row, rows (<= 8), 0}; see decode_mfma.hip.
struct GroupView {
    const uint8_t* const* bases;  // per expert: tile-packed weights
    const int4* chunks;
    const int* nchunks;           // device scalar: chunks in use (the grid covers the worst case)
    const int* rowmap;            // optional: activation row of each gathered row
    // Fused gate / up experts ([2 inter, n_in]: gate rows, then up rows), glu_inter = inter != 0: a workgroup's row tiles
    // are rt / 2 gate tiles and the up tiles of the same rows; instead of the products it writes act(gate) * up, quantized
    // as quantize_act quantizes it, into the QAct `aq` ([gathered rows][inter]) -- the input of the down projection.
    uint32_t glu_inter = 0;
    uint32_t act_kind = 0;
    float act_param = 0.0f;
    int8_t* aq_q = nullptr;
    float* aq_scales = nullptr;
    int32_t* aq_sums = nullptr;
    float* aq_fsums = nullptr;
    float* aq_hsums = nullptr;
    int32_t* aq_sums16 = nullptr;
    // The down projection with the combination inside (comb_y != nullptr): the products go to the gathered rows `y` as
    // always; the last workgroup of a row group to finish (arrival counter per row group, zero between launches) then
    // adds them into comb_y [comb_t, n_out] in route order: comb_y[i] (+)= sum_j route_w[i k + j] * y[row_of[i k + j]].
    float* comb_y = nullptr;
    const int* row_of = nullptr;
    const float* route_w = nullptr;
    uint32_t comb_t = 0, comb_k = 0;
    uint32_t comb_add = 1;
    uint32_t* comb_counters = nullptr;
    // A one-token pass needs no plan: with direct != nullptr chunk c is {expert direct[c], gathered row c, one row} for
    // c < direct_n, every gathered row of the gate / up launch reads token 0 (direct_x0), and route j's row is row j.
    const uint32_t* direct = nullptr;
    uint32_t direct_n = 0;
    uint32_t direct_x0 = 0;
};

// Launchers (each returns hipSuccess or the launch error).
hipError_t launch_quantize_act(const float* x, size_t t, size_t n_in, const oxhip_qact& out, hipStream_t s);
constexpr int QUANT_BATCH_MAX = 16;  // matrices per launch of the batched form
hipError_t launch_quantize_act_batch(const float* const* x, const size_t* t, const size_t* n_in, const oxhip_qact* o, size_t n, hipStream_t s);
hipError_t launch_dequantize(const WeightView& w, size_t r0, size_t r1, float* out, hipStream_t s);
// FP8 weights are tile-packed (WeightView::group == 1) when their rows are whole 128-column steps and the scale blocks
// are multiples of 16 rows x 128 columns: record (tile of 16 rows, step of 128 columns) is 2048 contiguous bytes, lane
// 16 kq + n of a wave owning the 32 bytes of row n at columns 32 kq .. 32 kq + 31 of the step, the first 16 of them at
// byte 16 lane of the record and the other 16 at byte 1024 + 16 lane: each of a wave's two requests per record reads one
// contiguous KiB. Otherwise the bytes stay row-major. Byte offset of (row, col) either way:
__host__ __device__ inline size_t fp8_offset(const WeightView& w, size_t row, size_t col) {
    if (w.group != 1) return row * w.n_in + col;
    const size_t nsteps = w.n_in / 128;
    return ((row / 16) * nsteps + col / 128) * 2048 + 1024 * ((col % 32) / 16) + 16 * (((col % 128) / 32) * 16 + row % 16) + col % 16;
}
// Bytes from the first to the second 16-byte chunk of a lane's 32 bytes of a step.
__host__ __device__ inline uint32_t fp8_second_chunk(const WeightView& w) { return w.group == 1 ? 1024 : 16; }
inline bool fp8_tileable(size_t n_in, uint32_t br, uint32_t bc) { return n_in % 128 == 0 && bc % 128 == 0 && br % 16 == 0; }
hipError_t launch_pack_q8f(const int8_t* q, const float* scales, size_t n_out, size_t n_in, uint8_t* dst, hipStream_t s);
hipError_t launch_pack_fp8(const uint8_t* raw, size_t n_out, size_t n_in, uint8_t* dst, hipStream_t s);
// NVFP4: half the value of an unsigned E4M3 scale byte (src/ggml.rs:477-490: 0 and 0x7f decode to 0, bit 7 is ignored);
// every value is exact in f32.
__host__ __device__ inline float ue4m3_half(uint32_t x) {
    x &= 0xFF;
    if (x == 0 || x == 0x7F) return 0.0f;
    const uint32_t e = (x >> 3) & 0xF, m = x & 7;
    // (1 + m / 8) 2^(e - 7) / 2 = (1 + m / 8) 2^(e - 8): exponent field e - 8 + 127; subnormals m 2^-9 / 2 = m 2^-10
    const uint32_t bits = e == 0 ? 0u : ((e + 119u) << 23) | (m << 20);
    union { uint32_t u; float f; } v;
    v.u = bits;
    return e == 0 ? (float)m * (1.0f / 1024.0f) : v.f;
}
// decode.hip: NVFP4 weights at up to 16 tokens, f32 activations (float-stored, like FP8)
hipError_t launch_decode_nvfp4(const WeightView& w, const float* x, size_t t, float* y, hipStream_t s);

// Global scratch of the decode kernels that split K across workgroups: `partial` holds slices x 8 token rows of
// n_out floats, `counters` (zero between launches) one entry per group of row tiles. Launches that share a scratch
// must be ordered on one stream. Without scratch the kernels keep K inside a workgroup.
// Arrival counters of the K slices sit one per 128 bytes: atomics on one line take their turn, and neighbouring row
// groups finish at about the same time.
constexpr uint32_t CTR_STRIDE = 32;
struct DecodeScratch {
    float* partial = nullptr;
    uint32_t* counters = nullptr;
    size_t partial_floats = 0, ncounters = 0;
};
// ev_start / ev_stop (optional): timing events around the launches (carried by the launch itself where there is one).
hipError_t launch_decode(const WeightView& w, const QActView& xa, const float* x, size_t t, float* y, hipStream_t s,
                         const DecodeScratch& sc = DecodeScratch{}, hipEvent_t ev_start = nullptr, hipEvent_t ev_stop = nullptr);
// y <- epi(y, v) over n values of t tokens ([t][n], v likewise): the epilogue as a kernel of its own, for the formats whose
// decode kernels only store.
hipError_t launch_epilogue(const float* v, size_t t, size_t n, float* y, const Epi& epi, hipStream_t s);
hipError_t launch_isums(const WeightView& w, const QActView& xa, size_t t, int32_t* out, hipStream_t s);
// Independent matmuls that may share one launch (decode_mfma.hip): each 1..8 tokens over a tile-packed weight.
struct DecodeBatchItem {
    WeightView w;
    QActView xa;
    float* y;
    uint32_t t;
    Epi epi{};
};
void decode_scratch_need(const WeightView& w, size_t* partial_floats, size_t* ncounters, bool pair = false);  // of a launch that slices K; else zeros (a pair launch: twice the floats)
bool decode_pair_ok(const WeightView& w);  // a gate / up pair of this shape and format runs as one launch (Epi::pair_p0)
bool decode_batchable(const WeightView& w, size_t t);  // the kernel takes it and its activations fit LDS
// ev_start / ev_stop (optional): timing events around the launches.
hipError_t launch_decode_mfma_batch(const DecodeBatchItem* items, size_t n, const DecodeScratch& sc, hipStream_t s, hipEvent_t ev_start = nullptr,
                                    hipEvent_t ev_stop = nullptr);
hipError_t launch_decode_mfma(const WeightView& w, const QActView& xa, size_t t, float* y, const DecodeScratch& sc, hipStream_t s,
                              hipEvent_t ev_start = nullptr, hipEvent_t ev_stop = nullptr, const Epi& epi = Epi{});
hipError_t launch_decode_mfma_grouped(const WeightView& w, const QActView& xa, const GroupView& g, uint32_t max_chunks,
                                      uint32_t max_rows_per_chunk, float* y, hipStream_t s);
bool decode_grouped_fits(const WeightView& w, uint32_t max_rows_per_chunk);
bool decode_grouped_glu_ok(const WeightView& w, size_t inter);  // the grouped launch can apply act(gate) * up and quantize it itself  // LDS holds a chunk's staged activations
hipError_t launch_isums_mfma(const WeightView& w, const QActView& xa, size_t t, float* y, int32_t* out, hipStream_t s);
hipError_t launch_repack_gguf(int fmt, const uint8_t* raw, size_t n_out, size_t n_in, const WeightView& dst, hipStream_t s);
// off == nullptr: `sc` holds one scale per 32 (Q4_0) and the record keeps all four of a row's step
hipError_t launch_pack_q4m(const uint8_t* q, const uint16_t* sc, const uint16_t* off, size_t n_out, size_t n_in, uint8_t* dst,
                           hipStream_t s);
hipError_t launch_repack_mlx_q4(const uint32_t* w, const uint16_t* scales, const uint16_t* biases, size_t n_out,
                                size_t n_in, size_t group, const WeightView& dst, hipStream_t s);
hipError_t launch_q4_scale_groups(const uint16_t* sc32, size_t n_out, size_t n_in, size_t sgroup, uint16_t* dst,
                                  int* mismatch, hipStream_t s);

hipError_t launch_pack_a(const void* x, bool src_bf16, int mode, size_t t, size_t n_in, size_t mtiles, size_t kblocks, void* out,
                         hipStream_t s);
uint32_t gemm_k_slices(const WeightView& w, size_t mtiles);
bool gemm_bf16_ok(const WeightView& w);        // the bf16 matrix-core GEMM dequantizes this weight's format and shape
int gemm_bf16_pack_mode(const WeightView& w);  // launch_pack_a's mode for its activation fragments
// decode_fp8.hip: FP8 weights at up to 32 tokens on the bf16 matrix cores
bool skinny_fp8_ok(const WeightView& w, size_t t);
size_t skinny_fp8_pack_bytes(const WeightView& w, size_t t, int planes);
hipError_t launch_skinny_fp8(const WeightView& w, const void* x, bool x_bf16, bool exact_f32, size_t t, void* y, bool y_bf16, void* pack,
                             hipStream_t s);
hipError_t launch_gemm_reduce(const float* partial, size_t n, uint32_t slices, void* y, bool out_bf16, hipStream_t s);
// Events a caller wants around the matrix kernel of the GEMM it is about to launch on this thread (oxhip_dev_gemm_timed): the
// launchers record them right before and right after that kernel, inside the activation packing and the K-slice sum.
struct KernelSpan {
    hipEvent_t start = nullptr, stop = nullptr;
};
extern thread_local KernelSpan g_kernel_span;
inline void span_start(hipStream_t s) {
    if (g_kernel_span.start) (void)hipEventRecord(g_kernel_span.start, s);
}
inline void span_stop(hipStream_t s) {
    if (g_kernel_span.stop) (void)hipEventRecord(g_kernel_span.stop, s);
}
void gemm_i8_geometry(const WeightView& w, size_t t, size_t* slots, size_t* ngrp);
uint32_t gemm_i8_k_slices(const WeightView& w, size_t t);
hipError_t launch_quantize_pack_i8(const void* x, bool src_bf16, size_t t, const WeightView& w, void* frag, void* xs, void* fs, hipStream_t s);
hipError_t launch_gemm_i8(const WeightView& w, const void* frag, const void* xs, const void* fs, size_t t, float* y, int32_t* dump, hipStream_t s);
hipError_t launch_gemm_bf16(const WeightView& w, const void* apk, size_t t, size_t mtiles, void* y, bool out_bf16, float* partial,
                            hipStream_t s);
hipError_t launch_quantize_act_fp8(const void* x, bool src_bf16, size_t t, size_t n_in, size_t mtiles, size_t kblocks, void* out,
                                   float* sx, hipStream_t s);
uint32_t gemm_fp8_k_slices(const WeightView& w, size_t mtiles);
hipError_t launch_gemm_fp8(const WeightView& w, const void* apk, const float* sx, size_t t, size_t mtiles, void* y, bool out_bf16,
                           float* partial, hipStream_t s);
hipError_t launch_route_top_k(const float* logits, size_t t, size_t n, size_t k, uint32_t* idx, float* w, hipStream_t s, size_t stride = 0,
                              const float* expert_scale = nullptr);
// route_top_k of t rows of logits and quantize_act of x [t][h] in one launch (the two are independent and each is a few
// microseconds of latency); n <= 256.
hipError_t launch_route_quantize(const float* logits, size_t t, size_t n, size_t k, uint32_t* idx, float* w, size_t stride,
                                 const float* expert_scale, const float* x, size_t h, const oxhip_qact& o, hipStream_t s);
hipError_t launch_moe_plan(const uint32_t* route_idx, size_t pairs, size_t k, size_t n_exp, uint32_t chunk_rows, int* row_of, int* src,
                           int4* chunks, int* nchunks, hipStream_t s);
hipError_t launch_moe_front(const uint32_t* route_idx, size_t pairs, size_t k, size_t n_exp, uint32_t chunk_rows, int* row_of, int* src,
                            int4* chunks, int* nchunks, const float* x, size_t t, size_t h, const oxhip_qact& o, hipStream_t s);
hipError_t launch_moe_act(const float* g, const float* u, size_t stride, size_t rows, size_t inter, uint32_t kind, float param,
                          float* a, hipStream_t s);
hipError_t launch_moe_act_quantize(const float* g, const float* u, size_t stride, size_t rows, size_t inter, uint32_t kind, float param,
                                   const oxhip_qact& o, hipStream_t s);
hipError_t launch_moe_combine(const float* o, const int* row_of, const float* route_w, size_t t, size_t k, size_t h, float* y,
                              hipStream_t s, bool add = true);
// decode-graph kernels (graph_ops.hip)
hipError_t launch_glu(const float* g, const float* u, size_t n, bool gelu, float* y, hipStream_t s);
hipError_t launch_router_logits(const float* x, const float* router, const float* gate, size_t t, size_t n_exp, size_t h, float* logits,
                                hipStream_t s);
// x_stride / out_stride: floats between rows (0 = n); pre: x is scaled by it first; add: out += instead of out =
hipError_t launch_rmsnorm_quantize(const float* x, const float* w_f32, const uint16_t* w_bf16, float eps, size_t t, size_t n, float* out,
                                   const oxhip_qact* q, hipStream_t s, float pre = 1.0f, bool add = false, size_t x_stride = 0,
                                   size_t out_stride = 0);
// The bf16 form of the grouped expert matmuls for prefill passes (moe_bf16.hip): MLX 4-bit weights, chunks of <= 16 rows.
bool moe_bf16_ok(const WeightView& w);
bool moe_bf16_std_geometry(const WeightView& w);  // its fragments hold a block's columns as 8 kq + j (Q8_0, Q4_K), not as T4M records do
size_t moe_bf16_frag_bytes(size_t max_chunks, size_t n_in);
hipError_t launch_moe_pack_bf16(const float* x, size_t n_in, const int* rowmap, const int4* chunks, const int* nchunks, uint32_t max_chunks,
                                void* frag, hipStream_t s, bool std_geometry = false);
hipError_t launch_moe_act_pack_bf16(const float* g, const float* u, size_t stride, size_t inter, uint32_t kind, float param, const int4* chunks,
                                    const int* nchunks, uint32_t max_chunks, void* frag, hipStream_t s, bool std_geometry = false);
bool moe_bf16_glu_ok(const WeightView& w, size_t inter, uint32_t max_chunks);  // the gate / up launch can apply the activation and write the down projection's fragments
hipError_t launch_moe_bf16(const WeightView& w, const GroupView& g, uint32_t max_chunks, const void* frag, float* out, hipStream_t s,
                           size_t glu_inter = 0, uint32_t act_kind = 0, float act_param = 0.0f, bool std_out = false, void* out_frag = nullptr);

hipError_t launch_fill_zero(uint32_t* p, size_t n, hipStream_t s);  // n dwords, by a kernel on `s`

void set_error(const std::string& msg);

// ------------------------------------------------------------------------------------------------
// Device helpers
// ------------------------------------------------------------------------------------------------
// A pointer that a kernel reads from memory (a table of per-expert bases) carries no address space, and loads through
// it would be flat: those count as LDS traffic as well as memory traffic, so every wait for an LDS read would also wait
// for all the weight records in flight. Weight streams therefore go through pointers typed as global memory.
typedef const __attribute__((address_space(1))) uint8_t* gbytes;
__device__ __forceinline__ gbytes as_global(const uint8_t* p) { return (gbytes)p; }
template <int BYTES>
struct GWord;
template <>
struct GWord<2> {
    typedef uint16_t type;
};
template <>
struct GWord<4> {
    typedef uint32_t type;
};
template <>
struct GWord<8> {
    typedef uint32_t type __attribute__((ext_vector_type(2)));
};
template <>
struct GWord<16> {
    typedef uint32_t type __attribute__((ext_vector_type(4)));
};
template <class T>
__device__ __forceinline__ T gload(gbytes p) {  // one request of sizeof(T) bytes
    typedef typename GWord<sizeof(T)>::type W;
    const W v = *reinterpret_cast<const __attribute__((address_space(1))) W*>(p);
    return __builtin_bit_cast(T, v);
}
// The same for bytes that are read once (weight records): marked non-temporal, they pass through the L2 without displacing
// what is read again and again (activations, partial sums). On the 8-matmul decode launch: 71.4 -> 68.9 us.
template <class T>
__device__ __forceinline__ T gload_once(gbytes p) {
    typedef typename GWord<sizeof(T)>::type W;
    const W v = __builtin_nontemporal_load(reinterpret_cast<const __attribute__((address_space(1))) W*>(p));
    return __builtin_bit_cast(T, v);
}
__device__ __forceinline__ float f16_bits_to_f32(uint16_t h) {
    return (float)__builtin_bit_cast(_Float16, h);  // exact
}
__device__ __forceinline__ float bf16_bits_to_f32(uint16_t h) { return __uint_as_float((uint32_t)h << 16); }

// IEEE round-to-nearest-even f32 -> bf16 bits (NaN quieted), as half::bf16::from_f32.
__device__ __forceinline__ uint16_t f32_to_bf16_bits(float x) {
    uint32_t b = __float_as_uint(x);
    if ((b & 0x7FFFFFFFu) > 0x7F800000u) return (uint16_t)((b >> 16) | 0x0040);
    return (uint16_t)((b + 0x7FFFu + ((b >> 16) & 1)) >> 16);
}
// IEEE round-to-nearest-even f32 -> f16 bits (the hardware conversion is RNE, denormals kept).
__device__ __forceinline__ uint16_t f32_to_f16_bits(float x) {
    _Float16 h = (_Float16)x;
    return __builtin_bit_cast(uint16_t, h);
}

// OCP e4m3 (float8_e4m3fn) byte -> f32 from the bits: (1 + m/8) 2^(e-7), subnormals m 2^-9,
// 0x7f / 0xff NaN.
__device__ __forceinline__ float e4m3_to_f32(uint32_t b) {
    uint32_t e = (b >> 3) & 0xF, m = b & 7;
    uint32_t normal = ((e + 120) << 23) | (m << 20);
    uint32_t sub = __float_as_uint((float)(int)m * (1.0f / 512.0f));
    uint32_t mag = e == 0 ? sub : normal;
    mag = (b & 0x7F) == 0x7F ? 0x7FC00000u : mag;
    return __uint_as_float(mag | ((b & 0x80) << 24));
}

// Scale and min `i` (0..8) of a Q4_K block from its 12 packed bytes held as three dwords.
__device__ __forceinline__ void scale_min_k4(uint32_t i, uint32_t d0, uint32_t d1, uint32_t d2, uint32_t& sc, uint32_t& mn) {
    uint32_t sh = 8 * (i & 3);
    uint32_t a = (d0 >> sh) & 0xFF, b = (d1 >> sh) & 0xFF, c = (d2 >> sh) & 0xFF;
    if (i < 4) {
        sc = a & 63;
        mn = b & 63;
    } else {
        sc = (c & 15) | ((a >> 6) << 4);
        mn = (c >> 4) | ((b >> 6) << 4);
    }
}

// MXFP4: four E2M1 codes (one per byte, 0..15) -> their doubled values {0, 1, 2, 3, 4, 6, 8, 12} with the sign of bit 3
// (src/ggml_tables.rs:1896) plus BIAS, as four bytes: a byte permute per sign over an 8-byte table, then a select.
template <int BIAS>
__device__ __forceinline__ uint32_t mxfp4_values(uint32_t codes) {
    constexpr uint32_t B4 = (uint32_t)(BIAS & 0xFF) * 0x01010101u;
    constexpr uint32_t PLO = 0x03020100u + B4, PHI = 0x0C080604u + B4;                    // BIAS + {0, 1, 2, 3}, {4, 6, 8, 12}
    constexpr uint32_t NLO = (B4 - 0x03020100u) & 0xFFFFFFFFu, NHI = B4 - 0x0C080604u;  // BIAS - ..., bytewise when BIAS >= 12
    constexpr uint32_t NLO0 = 0xFDFEFF00u, NHI0 = 0xF4F8FAFCu;                            // BIAS 0: {0, -1, -2, -3}, {-4, -6, -8, -12} as int8
    const uint32_t sel = codes & 0x07070707u;
    const uint32_t pos = __builtin_amdgcn_perm(PHI, PLO, sel);
    const uint32_t neg = __builtin_amdgcn_perm(BIAS ? NHI : NHI0, BIAS ? NLO : NLO0, sel);
    const uint32_t m = ((codes >> 3) & 0x01010101u) * 0xFFu;
    return (pos & ~m) | (neg & m);
}
// Half the value of an E8M0 scale byte, 2^(e - 128) (src/ggml.rs:466-475; exact for every e, subnormal for e < 2).
__device__ __forceinline__ float e8m0_half(uint32_t e) { return ldexpf(1.0f, (int)e - 128); }

__device__ __forceinline__ int dot4(uint32_t a, uint32_t b, int c) { return __builtin_amdgcn_sdot4((int)a, (int)b, c, false); }

template <int CTRL, int ROW_MASK = 0xF>
__device__ __forceinline__ float dpp_f32(float v) {
    return __int_as_float(__builtin_amdgcn_update_dpp(0, __float_as_int(v), CTRL, ROW_MASK, 0xF, true));
}
// Sum over the 64 lanes of a wavefront, result in every lane: DPP inside rows of 16, then the
// cross-row exchanges.
__device__ __forceinline__ float wave_sum(float v) {
    v += dpp_f32<0xB1>(v);   // quad_perm [1,0,3,2]
    v += dpp_f32<0x4E>(v);   // quad_perm [2,3,0,1]
    v += dpp_f32<0x141>(v);  // row_half_mirror
    v += dpp_f32<0x140>(v);  // row_mirror
    v += __shfl_xor(v, 16);
    v += __shfl_xor(v, 32);
    return v;
}

}  // namespace oxhip
