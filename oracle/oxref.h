/* CPU oracle for the quantized-weight matmul path: TEST INFRASTRUCTURE ONLY.
 *
 * A C++ restatement of the algorithms of oxinfer's CPU kernels for this path, written from
 * the Rust sources (each function cites the reference file:line it follows). Only tests, the
 * smoke check and the benchmark's CPU-baseline leg may load this library; the product library
 * (liboxinfer_hip.so) never does.
 *
 * Pinning status (what fixes each function without running the reference):
 *   f16/bf16 conversions ........ exhaustive against numpy float16 / torch bfloat16
 *   random_blocks + dequantize .. the reference's REF_HASHES (src/ggml.rs:1547-1577), produced
 *                                 by gguf-py / ggml C, for every type restated here
 *   decode_i8 ................... invariant s*q+m == dequantize_row within 1e-6 (src/ggml.rs:1663-1681)
 *   e4m3 ........................ closed form + torch.float8_e4m3fn over all 256 bytes
 *   NVFP4 ....................... every (scale byte, code) pair against torch.float8_e4m3fn and the E2M1 definition
 *   quantize_act ................ scalar definition (src/quant.rs:645-656), special cases
 *   from_mlx_q4 ................. invariant against mlx_dequant_row, exact where representable
 *   integer dot products ........ brute force; power-of-two scales make the f32 math exact
 *   decode / prefill / MoE ...... f64 definitions (src/ggml.rs:1712-1747, src/cuda.rs:2145-2179)
 *   route_top_k ................. equals full softmax -> top-k -> renormalize
 *   act_apply / act_scalar ...... torch's silu, gelu(approximate="tanh") and clamp in f64 (to fast_exp's 3e-7)
 * Parity unpinned (only running the reference could fix these bit for bit; the parity contract
 * does not need them): the f32 summation order of the AVX2 Q4 kernel and of dot_bf16 inside
 * add_offsets, fast_exp's exact output bits, libm expf.
 */
#ifndef OXREF_H
#define OXREF_H
#include <stddef.h>
#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

/* GGUF type ids (src/ggml.rs:42-93). */
enum {
    OXREF_F32 = 0, OXREF_F16 = 1, OXREF_Q4_0 = 2, OXREF_Q4_1 = 3, OXREF_Q5_0 = 6, OXREF_Q5_1 = 7,
    OXREF_Q8_0 = 8, OXREF_Q2_K = 10, OXREF_Q3_K = 11, OXREF_Q4_K = 12, OXREF_Q5_K = 13,
    OXREF_Q6_K = 14, OXREF_BF16 = 30, OXREF_MXFP4 = 39, OXREF_NVFP4 = 40, OXREF_F8E4M3 = 0x1000
};

/* conversions (half crate 2.7.1 semantics: IEEE RNE) */
float    oxref_f16_to_f32(uint16_t h);
uint16_t oxref_f32_to_f16(float x);
uint16_t oxref_f32_to_bf16(float x);
float    oxref_bf16_to_f32(uint16_t h);

/* type geometry; 0 for a type this oracle does not restate */
size_t oxref_block_size(uint32_t kind);
size_t oxref_type_size(uint32_t kind);
size_t oxref_row_bytes(uint32_t kind, size_t n);

uint64_t oxref_lcg(uint64_t* seed);
void     oxref_random_blocks(uint32_t kind, size_t nb, uint64_t* seed, uint8_t* out);
uint64_t oxref_fnv1a_f32(const float* v, size_t n);

void oxref_dequantize_row(uint32_t kind, const uint8_t* src, size_t n, float* out);
int  oxref_decode_i8(uint32_t kind, const uint8_t* blk, int8_t* q, float* s, float* m);

/* NVFP4 (src/ggml.rs:79-83, :477-490, :936-947): half an unsigned E4M3 scale byte; rows with the matrix's scales on top. */
float oxref_ue4m3_half(uint8_t x);
void  oxref_gguf_dequant_rows_scaled(uint32_t kind, const uint8_t* data, const float* scales, size_t n_in, size_t brows, size_t bcols,
                                     size_t r0, size_t r1, float* out);

float oxref_e4m3_to_f32(uint8_t b);
void  oxref_e4m3_scaled(const uint8_t* src, size_t n, float s, float* out);
void  oxref_fp8_dequant_rows(const uint8_t* data, const float* scales, size_t n_out, size_t n_in,
                             size_t brows, size_t bcols, size_t r0, size_t r1, float* out);

void oxref_quantize_act(const float* x, size_t t, size_t n_in, int8_t* q, float* scales,
                        int32_t* sums, float* fsums, float* hsums);

void oxref_from_mlx_q4(const uint32_t* w, const uint16_t* scales, const uint16_t* biases,
                       size_t n_out, size_t n_in, size_t group, uint8_t* q, uint16_t* sc, uint16_t* off);
void oxref_mlx_dequant_row(const uint32_t* w, const uint16_t* scales, const uint16_t* biases,
                           size_t bits, size_t group, size_t n, float* out);
void oxref_dequant_rows_q4(const uint8_t* q, const uint16_t* sc, const uint16_t* off, size_t group,
                           size_t n_in, size_t r0, size_t r1, float* out);

/* Decode (int8 activations).  y is [t][n_out].  isums (optional) receives the exact integer
 * accumulators: Q4 per block of 32 [t][n_out][n_in/32]; GGUF per 16 [t][n_out][n_in/16]. */
/* Q8 (QMatrix, src/quant.rs:128-133): dequantize_rows (src/quant.rs:405-419) and the portable rows_t1 (src/kernels.rs:1156-1167). */
void oxref_q8_dequant_rows(const int8_t* q, const float* scales, size_t n_in, size_t r0, size_t r1, float* out);
void oxref_q8_decode(const int8_t* q, const float* scales, size_t n_out, size_t n_in, const float* x, size_t t, float* y, int32_t* isums);
void oxref_q4_decode(const uint8_t* q, const uint16_t* sc, const uint16_t* off, size_t group,
                     size_t n_out, size_t n_in, const float* x, size_t t, float* y, int32_t* isums);
void oxref_q4_decode_avx2(const uint8_t* q, const uint16_t* sc, const uint16_t* off, size_t group,
                          size_t n_out, size_t n_in, const float* x, size_t t, float* y, int threads);
void oxref_gguf_decode(uint32_t kind, const uint8_t* data, size_t n_out, size_t n_in,
                       const float* x, size_t t, float* y, int32_t* isums);
void oxref_gguf_decode_avx2(uint32_t kind, const uint8_t* data, size_t n_out, size_t n_in,
                            const float* x, size_t t, float* y, int threads);

/* Prefill on x86: dequantized f32 rows, one fma chain per output, k ascending. w is [n_out][n_in]. */
void oxref_gemm_f32(const float* w, size_t n_out, size_t n_in, const float* x, size_t t, float* y, int threads);
/* The same through a dequantizer, 8 rows at a time (what the CPU baseline times). kind:
 * a GGUF id, or -1 for Q4 (data=q, aux0=scales f16, aux1=offsets bf16, group), or F8E4M3
 * (aux0 = f32 block scales, brows/bcols). */
void oxref_gemm_quant(int64_t kind, const void* data, const void* aux0, const void* aux1, size_t group,
                      size_t brows, size_t bcols, size_t n_out, size_t n_in, const float* x, size_t t,
                      float* y, int threads);

/* int8 prefill GEMM semantics of kernels_i8gemm (one plane) for a Q4 matrix.
 * isums (optional): [t][n_out][n_in/32]. */
void oxref_i8gemm_q4(const uint8_t* q, const uint16_t* sc, const uint16_t* off, size_t group,
                     size_t n_out, size_t n_in, const float* x, size_t t, float* y, int32_t* isums);

float oxref_fast_exp(float x);
void  oxref_silu_mul(float* a, const float* b, size_t n);
void  oxref_route_top_k(const float* logits, size_t n, size_t k, uint32_t* idx, float* w);

/* MoE over MLX-4bit (repacked Q4) experts.  gate_up: [ne] pointers per plane.  y += ... */
typedef struct {
    const uint8_t*  q;
    const uint16_t* sc;
    const uint16_t* off;
} oxref_q4_ref;
void oxref_moe_q4(const oxref_q4_ref* gate_up, const oxref_q4_ref* down, size_t ne, size_t group,
                  size_t h, size_t inter, const float* x, size_t t, const uint32_t* route_idx,
                  const float* route_w, size_t k, float* y, int decode_path);

/* Act::apply (src/moe.rs:18-37) in place over n pairs, and Act::scalar (src/moe.rs:39-46). kind: 0 SiLU, 1 GELU-tanh,
 * 2 SiLU with the clamp `param`. */
void  oxref_act_apply(uint32_t kind, float param, float* g, const float* u, size_t n);
float oxref_act_scalar(uint32_t kind, float param, float g, float u);
/* oxref_moe_q4 with the layer's activation and, with `up` != NULL, split gate / up experts (gate_up[e] = the gate
 * [inter, h], up[e] = [inter, h]; src/gpu.rs:206-216). */
void oxref_moe_q4_act(const oxref_q4_ref* gate_up, const oxref_q4_ref* up, const oxref_q4_ref* down, size_t ne, size_t group,
                      size_t h, size_t inter, const float* x, size_t t, const uint32_t* route_idx,
                      const float* route_w, size_t k, float* y, int decode_path, uint32_t act_kind, float act_param);

/* The decode-sized pass scheduled and vectorized as the x86 CPU does it (timed baseline). */
void oxref_moe_q4_avx2(const oxref_q4_ref* gate_up, const oxref_q4_ref* down, size_t ne, size_t group,
                       size_t h, size_t inter, const float* x, size_t t, const uint32_t* route_idx,
                       const float* route_w, size_t k, float* y, int threads);

int oxref_hw_threads(void);

#ifdef __cplusplus
}
#endif
#endif
