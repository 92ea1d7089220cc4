/* liboxinfer_hip: MI355X (gfx950) quantized-weight matmuls behind oxinfer's accelerator surface.
 *
 * A C ABI (plain pointers and sizes) that an `impl Backend for HipBackend` on the Rust side binds at
 * run time with dlsym, the way src/cuda.rs:31-86 binds libcuda. Each entry point names the
 * reference interface it stands behind (paths relative to the oxinfer tree).
 *
 * Conventions (those of `trait Backend`, src/gpu.rs:151-294):
 *   - functions returning int: 1 = done, 0 = declined and NOTHING was written; the caller then runs
 *     its CPU path (src/gpu.rs:158-160, src/model.rs:877-882). Handle-returning calls give NULL.
 *   - oxhip_last_error() holds the reason of the calling thread's last decline.
 *   - every call may come from any thread, concurrently (src/cuda.rs:2047-2077, :2410-2438).
 *   - matrices are [n_out, n_in] row-major, outputs y[t][n_out] f32 (src/kernels.rs:54-57).
 *
 * Two layers:
 *   1. the Backend surface: host pointers in, host pointers out (the library owns staging);
 *   2. device-pointer entry points (oxhip_dev_*): the same kernels on buffers already in HBM, on a
 *      caller-chosen stream, for callers that keep activations resident and for measurement.
 */
#ifndef OXHIP_H
#define OXHIP_H
#include <stddef.h>
#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

typedef struct oxhip_ctx oxhip_ctx;       /* one per device: `HipBackend` (cf. CudaBackend, src/cuda.rs:404-446) */
typedef struct oxhip_weight oxhip_weight; /* `DeviceWeight` of one matrix (src/gpu.rs:57) */
typedef struct oxhip_moe oxhip_moe;       /* `DeviceWeight` of one MoE layer's experts (src/gpu.rs:206-216) */

/* `WeightRef` (src/gpu.rs:15-21) plus the MLX triplet before `from_mlx_q4` (src/quant.rs:518). */
enum {
    OXHIP_W_BF16 = 0,   /* data: u16 bf16 [n_out, n_in] */
    OXHIP_W_Q8 = 1,     /* QMatrix: data i8 [n_out, n_in], scales f32 [n_out, n_in/32] (src/quant.rs) */
    OXHIP_W_Q4 = 2,     /* Q4Matrix: data nibbles [n_out, n_in/2], scales f16 [n_out, n_in/32],
                           offsets bf16 [n_out, n_in/group] or NULL (src/quant.rs:427-440) */
    OXHIP_W_GGUF = 3,   /* GgufMatrix: raw blocks of ggml_type; F8E4M3 with block_scales (src/ggml.rs:240-256) */
    OXHIP_W_MLX_Q4 = 4  /* MLX affine 4-bit: data u32 [n_out, n_in/8], scales / offsets(=biases) bf16
                           [n_out, n_in/group]; repacked on the device exactly as from_mlx_q4 does */
};

/* GGUF type ids handled (src/ggml.rs:42-93). */
enum { OXHIP_GGML_Q4_0 = 2, OXHIP_GGML_Q8_0 = 8, OXHIP_GGML_Q4_K = 12, OXHIP_GGML_Q5_K = 13, OXHIP_GGML_Q6_K = 14, OXHIP_GGML_MXFP4 = 39, OXHIP_GGML_NVFP4 = 40, OXHIP_GGML_F8E4M3 = 0x1000 };

typedef struct {
    uint32_t kind;            /* OXHIP_W_* */
    uint32_t ggml_type;       /* OXHIP_GGML_* when kind == OXHIP_W_GGUF */
    size_t n_out, n_in;
    const void* data;
    const void* scales;
    const void* offsets;
    uint32_t group;           /* elements per offset (Q4) / per scale and bias (MLX) */
    const float* block_scales;/* FP8: [ceil(n_out/bs_rows), ceil(n_in/bs_cols)]; NVFP4: the same, optional (its global scale:
                                 one block spanning the matrix, src/model.rs:550-557), on top of the decoded values */
    uint32_t bs_rows, bs_cols;
} oxhip_weight_desc;

/* `Job` (src/gpu.rs:60-65). */
typedef struct {
    const oxhip_weight* w;
    size_t n_out;
    float* y; /* host, [t, n_out] */
} oxhip_job;

/* `RowsJob` (src/gpu.rs:69-75): y = W x, or with `up`: y = silu(W x) * (U x). */
typedef struct {
    const oxhip_weight* w;
    const oxhip_weight* up; /* NULL for a plain product */
    size_t n_out;
    float* y;
} oxhip_rows_job;

/* `MoeAct` (src/gpu.rs:35-54); the CPU-only kinds are declined like the reference's backends do. */
enum { OXHIP_ACT_SILU = 0, OXHIP_ACT_GELU_TANH = 1, OXHIP_ACT_SILU_CLAMP = 2 };

/* ---- detection --------------------------------------------------------------------------- */
/* platform::gpu::cuda::probe (src/platform.rs:446-482) for HIP devices, the source of a `GpuInfo { kind: GpuKind::Hip, .. }`
 * (src/platform.rs:25-34): fills up to `cap` entries and returns the number of devices the runtime reports (0 without a
 * driver or a device; never an error). `usable`: this library holds code for the device's architecture (gfx950);
 * oxhip_open declines the others. */
typedef struct {
    int index;
    char name[256];        /* marketing name */
    char arch[64];         /* e.g. "gfx950" */
    uint64_t memory_bytes; /* device-local memory */
    char driver[64];       /* runtime version, architecture, CU count */
    int usable;
} oxhip_gpu_info;
int oxhip_probe(oxhip_gpu_info* out, int cap);

/* ---- life cycle -------------------------------------------------------------------------- */
/* CudaBackend::new (src/cuda.rs:448-570). 1 on success; 0 when the device cannot start. */
int oxhip_open(int device, oxhip_ctx** out);
void oxhip_close(oxhip_ctx* ctx);
/* Backend::name (src/gpu.rs:152), e.g. "hip (gfx950)". */
const char* oxhip_name(const oxhip_ctx* ctx);
const char* oxhip_last_error(void);
/* Backend::stats (src/gpu.rs:291): cumulative copy-in / gpu / copy-out ms; returns bytes written. */
size_t oxhip_stats(oxhip_ctx* ctx, char* buf, size_t len);

/* ---- Backend surface (host pointers) ------------------------------------------------------ */
/* Backend::wants (src/gpu.rs:155; CUDA's policy src/cuda.rs:1134-1136). */
int oxhip_wants(const oxhip_ctx* ctx, size_t n_out, size_t n_in, size_t t);
/* Backend::upload (src/gpu.rs:157; src/cuda.rs:640-699). NULL when declined (unsupported format
 * or shape, memory short under a 512 MiB reserve). */
oxhip_weight* oxhip_upload(oxhip_ctx* ctx, const oxhip_weight_desc* desc);
/* Dropping a DeviceWeight. */
void oxhip_free_weight(oxhip_ctx* ctx, oxhip_weight* w);
/* Bytes the weight occupies in HBM. */
size_t oxhip_weight_bytes(const oxhip_weight* w);
/* Backend::matmul (src/gpu.rs:160; src/cuda.rs:1428-1493): all jobs share x [t, n_in] (host f32);
 * computes every job or none. Routing as matmul_quant_multi_at's (src/kernels.rs:1731-1879): up to 8 tokens the
 * Q8 / Q8_0 / Q4_K / Q5_K / Q6_K / MXFP4 / MLX 4-bit jobs share one launch of the int8 decode kernel (the CPU's decode semantics,
 * src/kernels.rs:1908-1928); more than 16 tokens over MLX 4-bit, Q8, Q8_0, Q4_K, Q5_K, Q6_K, MXFP4, NVFP4 or FP8 (128-column
 * blocks) weights run the bf16 matrix-core GEMM; everything else runs the decode kernels over 16 tokens at a time. */
int oxhip_matmul(oxhip_ctx* ctx, const float* x, size_t t, size_t n_in, oxhip_job* jobs, size_t n_jobs);
/* Backend::matvec_rows (src/gpu.rs:165): t in 1..=4. The jobs over the matrix-core formats share one launch, a gate / up
 * job as a pair (see oxhip_dev_linear). */
int oxhip_matvec_rows(oxhip_ctx* ctx, const float* x, size_t t, size_t n_in, oxhip_rows_job* jobs, size_t n_jobs);

/* Backend::upload_moe (src/gpu.rs:206-216): expert e has gate_up[e] ([2*inter, h] fused, or [inter, h] when `up` is
 * given) and down[e] ([h, inter]). Backend::upload_moe_transient (src/gpu.rs:221-231: experts uploaded for one pass and
 * dropped after it) is this call followed by oxhip_free_moe once the pass has returned: uploads here never share or
 * cache device memory between calls, so a transient layer costs exactly its upload and nothing stays behind. */
oxhip_moe* oxhip_upload_moe(oxhip_ctx* ctx, const oxhip_weight_desc* gate_up, const oxhip_weight_desc* up,
                            const oxhip_weight_desc* down, size_t n_experts, size_t h, size_t inter,
                            uint32_t act_kind, float act_param);
void oxhip_free_moe(oxhip_ctx* ctx, oxhip_moe* m);
/* The arithmetic of prefill-sized passes (a property of the layer, as `act` is; the reference picks by token count
 * alone, src/moe.rs:625-640): OXHIP_MOE_AUTO follows the reference's split (decode-sized passes on int8 activations,
 * passes with six or more routed rows per expert over MLX 4-bit experts on the exact rows, bf16 matrix cores);
 * OXHIP_MOE_INT8 keeps the integer kernels (int8 activations, exact int32 block sums) at every size. Must not overlap
 * a pass over the same oxhip_moe. */
enum { OXHIP_MOE_AUTO = 0, OXHIP_MOE_INT8 = 1 };
int oxhip_moe_set_mode(oxhip_moe* m, uint32_t mode);
/* Backend::moe (src/gpu.rs:237-248) with `routes` flattened as CUDA's moe_run does
 * (src/cuda.rs:802-838): token i goes through experts route_idx[i*k .. i*k+k] with weights
 * route_w[...]; y[i] += sum_j w_j * down(act(gate x) * up x), in route order. */
int oxhip_moe_forward(oxhip_ctx* ctx, const float* x, size_t t, size_t h, size_t inter, const uint32_t* route_idx,
                      const float* route_w, size_t k, oxhip_moe* m, float* y);

/* ---- device-pointer entry points ---------------------------------------------------------- */
/* `QAct` (src/quant.rs:222-238) in HBM, plus sums16: the integer sum of each 16 int8 values (what
 * the centred nibble formats fold their offset through; the CPU derives it from `sums`). */
typedef struct {
    int8_t* q;        /* [t, n_in] */
    float* scales;    /* [t, n_in/32] */
    int32_t* sums;    /* [t, n_in/32] */
    float* fsums;     /* [t, n_in/32] */
    float* hsums;     /* [t, n_in/16] */
    int32_t* sums16;  /* [t, n_in/16] */
    size_t t, n_in;
} oxhip_qact;

/* quant::quantize_act (src/quant.rs:294-343) on device rows x [t, n_in] f32. */
int oxhip_dev_quantize_act(oxhip_ctx* ctx, const float* x, size_t t, size_t n_in, const oxhip_qact* out, void* stream);
/* The same for several activation matrices in one launch (a decode step quantizes the input of each group of matmuls:
 * QAct::new per input, src/quant.rs:294-343; every launch costs its latency whatever its size). */
typedef struct {
    const float* x; /* device, [t, n_in] f32 */
    size_t t, n_in;
    const oxhip_qact* out;
} oxhip_quant_job;
int oxhip_dev_quantize_act_batch(oxhip_ctx* ctx, const oxhip_quant_job* jobs, size_t n_jobs, void* stream);
/* QMat::dequantize_rows (src/kernels.rs:1336, src/ggml.rs:409-459): rows r0..r1 as f32 [r1-r0, n_in]. */
int oxhip_dev_dequantize(oxhip_ctx* ctx, const oxhip_weight* w, size_t r0, size_t r1, float* out, void* stream);
/* The decode kernels (QMat::rows_t1 / rows_tc, src/kernels.rs:1339-1369, src/ggml.rs:1319-1354):
 * y [t, n_out] f32 from quantized activations, t <= 16. FP8 / bf16 weights are float-stored
 * (`dense`, src/ggml.rs:1370): they take f32 rows `x` instead and `xa` may be NULL. */
int oxhip_dev_decode(oxhip_ctx* ctx, const oxhip_weight* w, const oxhip_qact* xa, const float* x, size_t t, float* y,
                     void* stream);
/* oxhip_dev_decode for callers that cannot allocate device memory (code under HIP graph capture, tight serving
 * loops, harnesses that forbid hipMalloc); it has no counterpart in the reference. The same kernels and the same
 * bits as oxhip_dev_decode over the quantized formats of the matrix-core decode kernel (Q8, Q8_0, Q4_0, Q4_K, Q5_K, Q6_K,
 * MXFP4, MLX 4-bit; 1 <= t <= 16), but the partial rows and arrival counters of shapes that slice K live in an array the
 * library holds statically on every GPU (4 MiB + 256 KiB, kept until the process ends), and the call allocates and
 * frees nothing on the device. Declined (0, nothing written) when the weight needs more than that: K slices x 8 x
 * n_out floats of partial rows beyond 4 MiB, or more than 2048 row groups. All calls on one GPU share the array:
 * calls that overlap on one GPU (other streams, other threads, other contexts) race; order them. */
int oxhip_dev_decode_noalloc(oxhip_ctx* ctx, const oxhip_weight* w, const oxhip_qact* xa, size_t t, float* y, void* stream);
/* Several independent decode matmuls in one call (a decode step issues many small matmuls; what
 * matmul_quant_batch does for the CPU, src/kernels.rs:1937-1994). The jobs must not depend on one another: runs of
 * consecutive jobs of at most 8 tokens over Q8 / Q8_0 / Q4_K / Q5_K / Q6_K / Q4_0 / MXFP4 / MLX 4-bit weights share launches: one per
 * kernel among them (Q8_0, Q4_K and Q6_K share one, Q5_K takes Q4_K and Q6_K jobs into its own, each other format has its own), up to 16 jobs each; their latency chains
 * overlap, and every job's rows are bit-identical to a launch of its own. The others launch one by one, in order, on
 * `stream` (inside a shared launch the library orders the jobs itself). ev_start / ev_stop (from oxhip_event_create, or
 * NULL) are recorded before / after the launch that holds the job; for jobs that share a launch the first start and the
 * last stop event take the shared launch's own start and end as the device saw them.
 * The device-pointer entry points keep their scratch (partial rows of K slices, packed GEMM activations) per calling
 * stream: calls on one stream are ordered and share it, calls on different streams may overlap one another and the
 * host-pointer surface. A stream's scratch is allocated when a call first needs it (hipMalloc: such a call cannot run
 * under stream capture and may wait for the device): 16 MiB of partial rows + 2 MiB of counters with the stream's first
 * decode launch whose shape slices K across workgroups (cleared by a kernel on that stream), the GEMMs' packed
 * activations with its first GEMM. It stays until oxhip_stream_release or oxhip_close. */
typedef struct {
    const oxhip_weight* w;
    const oxhip_qact* xa; /* quantized weights */
    const float* x;       /* float-stored weights */
    size_t t;
    float* y;
    void* ev_start;
    void* ev_stop;
} oxhip_decode_job;
int oxhip_dev_decode_batch(oxhip_ctx* ctx, const oxhip_decode_job* jobs, size_t n_jobs, void* stream);
/* Frees the scratch the device-pointer entry points hold for `stream` (after waiting for the stream's work); a later call
 * on that stream allocates it again. For callers that create and destroy streams: the scratch of a destroyed stream is
 * otherwise kept until oxhip_close. No counterpart in the reference (its backends serialize on one stream). */
int oxhip_stream_release(oxhip_ctx* ctx, void* stream);
/* HIP events for timing launches on a stream (Backend::stats-style measurement without a profiler). */
void* oxhip_event_create(void);
void oxhip_event_destroy(void* ev);
/* Milliseconds between two recorded events; waits for `stop`. Negative on error. */
float oxhip_event_elapsed_ms(void* start, void* stop);
/* Prefill: y [t, n_out] = x [t, n_in] W^T on the matrix cores (what matmul_quant_multi's GEMM paths compute,
 * src/kernels.rs:1774-1847). x_dtype / y_dtype: OXHIP_F32 or OXHIP_BF16. variant:
 *   OXHIP_GEMM_BF16  weights dequantized to bf16 (through LDS), bf16 MFMA, f32 accumulation (the x86 CPU's
 *                    f32 GEMM rounded to bf16 operands); MLX 4-bit, Q8, Q8_0, Q4_K, Q5_K and Q6_K weights (the rows
 *                    that dequantize_row yields, src/ggml.rs:630-793, rounded to bf16);
 *                    also FP8 weights whose rows are multiples of 128 (e4m3 x block scale rounded to bf16);
 *   OXHIP_GEMM_I8    MLX 4-bit weights on the int8 matrix cores: activations quantized per token and block of 32
 *                    as quantize_act does, exact int32 block sums, f32 rescale by the block and activation scales,
 *                    offsets times the exact activation sums (the reference's int8 GEMM, one activation plane,
 *                    src/kernels_i8gemm.rs:160-315);
 *   OXHIP_GEMM_FP8   FP8 weights with 128 x 128 block scales: activations quantized on the device to e4m3 per token
 *                    and 128 columns (scale amax / 448), fp8 MFMA, the two scales applied to each block's f32
 *                    partial sum (the reference has no activation-FP8 path: parity is against its f32 product);
 * Packed activations live in the calling stream's scratch (grown on first use). */
enum { OXHIP_F32 = 0, OXHIP_BF16 = 1 };
enum { OXHIP_GEMM_BF16 = 0, OXHIP_GEMM_I8 = 1, OXHIP_GEMM_FP8 = 2 };
int oxhip_dev_gemm(oxhip_ctx* ctx, const oxhip_weight* w, const void* x, int x_dtype, size_t t, void* y, int y_dtype, int variant,
                   void* stream);
/* oxhip_dev_gemm with two events (from oxhip_event_create; either may be NULL) recorded on `stream` right before and right
 * after the variant's matrix kernel, i.e. after the activation packing or quantization launch and before the K-slice sum: the
 * kernel's own duration as the device saw it, for measurement without a profiler (Backend::stats-style; no counterpart in
 * the reference's trait). The FP8 skinny path (up to 32 tokens) counts its packing launch and its kernel as one. */
int oxhip_dev_gemm_timed(oxhip_ctx* ctx, const oxhip_weight* w, const void* x, int x_dtype, size_t t, void* y, int y_dtype, int variant,
                         void* stream, void* ev_start, void* ev_stop);
/* The exact int32 block sums of the OXHIP_GEMM_I8 variant, [t, n_out, n_in/32], written by the GEMM kernel itself
 * (kernels_i8gemm's `block` accumulators, src/kernels_i8gemm.rs:249-334). For parity checks. */
int oxhip_dev_gemm_isums(oxhip_ctx* ctx, const oxhip_weight* w, const void* x, int x_dtype, size_t t, int32_t* out, void* stream);
/* moe::route_top_k (src/moe.rs:180-193) for t rows of n_experts logits (n_experts <= 1024, k <= 32):
 * idx / w [t, k], sorted by descending logit, ties to the lower index, w = softmax over the k. */
int oxhip_dev_route_top_k(oxhip_ctx* ctx, const float* logits, size_t t, size_t n_experts, size_t k, uint32_t* idx, float* w,
                          void* stream);
/* Backend::moe on device buffers: x [t, h] f32, route_idx / route_w [t, k], y [t, h] f32 (added to).
 * One grouped launch per projection over the routed token lists. Decode-sized passes run the integer kernels on
 * int8 activations (Experts::forward / forward_batched, src/moe.rs:438-617; within 1e-3 of them); passes with six
 * or more routed rows per expert over MLX 4-bit experts run the grouped matmuls on the bf16 matrix cores over the
 * exact rows with Act::scalar between them, which is the reference's grouped prefill form (src/moe.rs:735-827;
 * within 2e-2 of it: the rows and the activation's output are rounded to bf16); oxhip_moe_set_mode(m, OXHIP_MOE_INT8)
 * keeps the integer kernels at every size. The scratch it needs lives in
 * `m` and grows on first use (a call with a larger t * k than any before synchronizes and
 * reallocates); calls on one oxhip_moe must not overlap. */
int oxhip_dev_moe(oxhip_ctx* ctx, oxhip_moe* m, const float* x, size_t t, const uint32_t* route_idx, const float* route_w,
                  size_t k, float* y, void* stream);
/* ---- device-resident ops of the single-token decode graph (src/gpu_decode.rs:52-340) ---------------------------
 * What a `DecodePlan` (src/gpu_decode.rs:572-587) runs between the embedding lookup and the logits, on buffers that
 * stay in HBM: a plan built on these issues a token's linears and its MoE layer back to back on one stream, with no
 * host round trip (the reference measured that per-matmul offload of decode loses, docs/platforms.md:115-117). */
/* The arena of a plan (src/cuda_decode.rs:1044-1049: one zeroed device allocation; `View`s are offsets into it,
 * src/gpu_decode.rs:17-33). buf_write / buf_read copy between host memory and the arena and wait for the copy. */
void* oxhip_buf_alloc(oxhip_ctx* ctx, size_t bytes);
void oxhip_buf_free(oxhip_ctx* ctx, void* buf);
int oxhip_buf_write(oxhip_ctx* ctx, void* dst, const void* src_host, size_t bytes, void* stream);
int oxhip_buf_read(oxhip_ctx* ctx, void* dst_host, const void* src, size_t bytes, void* stream);
/* Op::Norm feeding a linear (src/gpu_decode.rs:53-66; rmsnorm, src/kernels.rs:2107-2123, then QAct::new,
 * src/quant.rs:294-343): v = (x * r) * w with r = (mean(x^2) + eps)^(-1/2), weights f32 (`w_f32`), bf16 (`w_bf16`) or
 * none; v goes to `out` ([t, n] f32, optional) and, quantized exactly as quantize_act quantizes it, to `q` (optional).
 * The squares are summed in f64 in a fixed order (the CPU's one-after-the-other f32 sum cannot be repeated in
 * parallel): r is within an ulp or two of the CPU's, the quantization of v is bit-exact. */
int oxhip_dev_rmsnorm_quantize(oxhip_ctx* ctx, const float* x, const float* w_f32, const uint16_t* w_bf16, float eps, size_t t, size_t n,
                               float* out, const oxhip_qact* q, void* stream);
/* Op::Norm with all its fields (src/gpu_decode.rs:53-66; the CUDA form, src/cuda_decode.cu:314-327): `rows` rows of n
 * values, x_stride / out_stride floats apart (0 = n): x' = x * pre, v = (x' * r) * w with r = (mean(x'^2) + eps)^(-1/2),
 * out = v or, with `add`, out += v; what `out` then holds is also quantized into `q` (optional; rows of q are dense).
 * oxhip_dev_rmsnorm_quantize is this call with pre = 1, no add and dense rows. Pointers and strides that are multiples
 * of 16 bytes take 16-byte accesses, any others (`View`s are float offsets into the arena) one float at a time. */
int oxhip_dev_norm(oxhip_ctx* ctx, const float* x, float* out, const float* w_f32, const uint16_t* w_bf16, float pre, size_t n, size_t rows,
                   size_t x_stride, size_t out_stride, float eps, int add, const oxhip_qact* q, void* stream);
/* Op::Linear with its LinMode (src/gpu_decode.rs:37-50, :67-77): y [t, n_out] f32 on the device, t <= 16.
 *   STORE      y  = W x
 *   ADD        y += W x                        (residual)
 *   SILU_PAIR  y  = silu(W x) * (W2 x)         (silu_mul, src/kernels.rs:2188-2198)
 *   GELU_PAIR  y  = gelu_tanh(W x) * (W2 x)    (gelu_mul, src/kernels.rs:2234-2257)
 *   ADD_GATED  y += sigmoid(gate[token]) * W x (a gated shared expert; `gate` one f32 per token on the device)
 * Inputs as oxhip_dev_decode's: `xa` for quantized weights, f32 rows `x` for float-stored ones. The matrices of a
 * pair share shape and format (pairable, src/gpu_decode.rs:340-349). The store / add / gated modes are the decode
 * kernels' own output stage. A pair over the matrix-core formats (Q8, Q8_0, Q4_0, Q4_K, Q5_K, Q6_K, MXFP4, MLX 4-bit) is ONE
 * launch: a workgroup streams the tiles of the same rows of both matrices and stores act(W x) * (W2 x) itself (the CUDA
 * kernels' modes 2 and 3, src/cuda_decode.cu:131-167), bit-identical to the two products followed by oxhip_dev_glu; the
 * other formats run the two products and the gate as launches of their own. */
enum { OXHIP_LIN_STORE = 0, OXHIP_LIN_ADD = 1, OXHIP_LIN_SILU_PAIR = 2, OXHIP_LIN_GELU_PAIR = 3, OXHIP_LIN_ADD_GATED = 4 };
int oxhip_dev_linear(oxhip_ctx* ctx, const oxhip_weight* w, const oxhip_weight* w2, const oxhip_qact* xa, const float* x, size_t t,
                     float* y, uint32_t mode, const float* gate, void* stream);
/* Op::Glu (src/gpu_decode.rs:231-239): y = silu(g) * u or gelu_tanh(g) * u over n values, for pairs of different formats. */
int oxhip_dev_glu(oxhip_ctx* ctx, const float* g, const float* u, size_t n, int gelu, float* y, void* stream);
/* Op::Route (src/gpu_decode.rs:154-172): logits [t, n_exp (+1)] = router [n_exp, h] (f32) . x, with `gate` ([h]) one
 * more logit behind them; then route_top_k over the first n_exp (ties to the lower index) into `sel`: the k expert
 * ids of every token ([t, k] u32), then their k softmax weights ([t, k] f32 bits) -- for one token "k ids then k
 * weights" -- times expert_scale[id] when given. All pointers on the device. */
int oxhip_dev_route(oxhip_ctx* ctx, const float* x, const float* router, const float* gate, size_t t, size_t n_exp, size_t h, size_t k,
                    float* logits, uint32_t* sel, const float* expert_scale, void* stream);
/* Op::Experts (src/gpu_decode.rs:318-337): the routed experts chosen in `sel` (as oxhip_dev_route writes it) over
 * x [t, h]: y += (add) or y = the weighted sum of down_e(act(gate_e x) * up_e x), in route order. The activation
 * (SiLU / GELU-tanh) is the layer's (oxhip_upload_moe). k <= 32. The expert ids in `sel` are read on the device and
 * cannot be checked by this call: every id must be below the layer's n_experts (oxhip_dev_route and
 * oxhip_dev_moe_routed write only such ids). */
int oxhip_dev_experts(oxhip_ctx* ctx, oxhip_moe* m, const float* x, size_t t, const uint32_t* sel, size_t k, float* y, int add, void* stream);

/* Op::Route's top-k and Op::Experts in one call, for plans that keep the router's logits on the device: `logits`
 * [t] rows of n_experts (rows `logit_stride` floats apart; 0 = n_experts), as oxhip_dev_route leaves them; `sel`
 * receives the routes (ids [t, k], then weights [t, k]) and y the experts' weighted sum (added or stored). For one
 * token over fused gate / up experts the pass is three launches: routing + input quantization; gate / up with the
 * activation and its quantization in the launch's output stage; down with the route-order combination done by the last
 * workgroup of each row group to finish. */
int oxhip_dev_moe_routed(oxhip_ctx* ctx, oxhip_moe* m, const float* x, size_t t, const float* logits, size_t logit_stride, size_t k,
                         const float* expert_scale, uint32_t* sel, float* y, int add, void* stream);

/* ---- a recorded chain of device-pointer ops, replayed as one submission ---------------------------------------------
 * The matmul side of DecodePlan::step (src/gpu_decode.rs:572-587; CUDA's per-graph launch list, src/cuda_decode.rs:1044-1049):
 * a token's ops (norm + quantize, linears, route, experts, ...) are issued once between oxhip_plan_begin and
 * oxhip_plan_end on `stream` (a stream of the caller's, not the null stream), where they are recorded instead of run; every
 * oxhip_plan_replay then submits the whole chain with one call. The recorded launches read and write the same device
 * buffers every time (the plan's arena, oxhip_buf_alloc): a new token is new contents in those buffers. Results are those
 * of the same calls issued one by one, bit for bit.
 * Before recording, run the chain once on the same stream: scratch that grows on first use (K-slice rows of the stream, an
 * MoE layer's pass buffers) must exist, since a recorded call can neither allocate nor wait; one that would have to makes
 * oxhip_plan_end fail (0, nothing replayable). Calls with timing events (oxhip_dev_decode_batch's ev_start / ev_stop,
 * oxhip_dev_gemm_timed) and the host-pointer surface cannot be recorded. While a plan records on a stream, no other
 * thread may use that stream. A plan holds no buffers of its own: free the weights and buffers it names after the plan. */
typedef struct oxhip_plan oxhip_plan;
oxhip_plan* oxhip_plan_begin(oxhip_ctx* ctx, void* stream);
int oxhip_plan_end(oxhip_plan* plan);
/* Launches the plan holds (0 before oxhip_plan_end succeeded). */
size_t oxhip_plan_launches(const oxhip_plan* plan);
/* Submits the recorded chain on `stream` (NULL: the stream it was recorded on). */
int oxhip_plan_replay(oxhip_plan* plan, void* stream);
/* Also abandons a recording in progress. */
void oxhip_plan_free(oxhip_plan* plan);

/* The exact integer accumulators of the decode kernels, written by the kernels themselves: per
 * block of 32 ([t, n_out, n_in/32]) for Q4, Q8, Q8_0, Q4_K and Q5_K, per 16 ([t, n_out, n_in/16]) for Q6_K.
 * For parity checks (the CPU's per-16 sums add up to the per-32 ones exactly). */
int oxhip_dev_isums(oxhip_ctx* ctx, const oxhip_weight* w, const oxhip_qact* xa, int32_t* out, void* stream);

#ifdef __cplusplus
}
#endif
#endif
