/*
 * CPU oracle for the GGUF quantized-matmul path.  TEST INFRASTRUCTURE ONLY:
 * nothing in the shipped library links, loads or calls this file.  Only the
 * tests, the smoke check and the bench's cpu_baseline leg may use it, and
 * there only as the checker / the timed CPU baseline.
 *
 * Every function restates one function of the reference in plain C and cites
 * the reference file:line it follows.  The functions marked "own" have no
 * counterpart in the reference (it ships no encoder for those formats); they
 * only produce test inputs.
 *
 * Parity status (what pins each function is in tests/test_oracle_*.py):
 *   pinned: orc_f16_to_f32, orc_f32_to_f16, orc_runner_f16_to_f32,
 *           orc_get_scale_min_k4, orc_dequant_q8_0/q4_0/q4_k/q6_k,
 *           orc_quantize_rows_q8_0, orc_requantize_q4k_to_affine,
 *           orc_split_q8_0/q4_0, orc_matmul_sep_*, orc_matmul_gguf_*,
 *           orc_transpose_q4_nibble, orc_quantize_act_q8,
 *           orc_matmul_q8_i8
 *   no function here is "parity unpinned".
 */
#ifndef CUT_ORACLE_H
#define CUT_ORACLE_H

#include <stddef.h>
#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

/* Block formats (interface/loader/gguf/gguf_types.hpp:109-142). The numeric
 * values are the library's own format codes (see include/cut_hip.h). */
enum { ORC_Q8_0 = 0, ORC_Q4_0 = 1, ORC_Q4_K = 2, ORC_Q6_K = 3 };

size_t orc_block_elems(int fmt);
size_t orc_block_bytes(int fmt);

/* gguf_reader.cpp:515-539 */
float orc_f16_to_f32(uint16_t h);
/* llama.cpp:445-482 */
uint16_t orc_f32_to_f16(float v);
/* llama.cpp:512-542 */
float orc_runner_f16_to_f32(uint16_t h);
/* OpRefs.h:164-177 (truncating test helper) */
uint16_t orc_harness_f32_to_f16(float v);
/* array forms of the three conversions above (for exhaustive tests) */
void orc_f16_to_f32_array(const uint16_t *h, size_t n, float *out);
void orc_f32_to_f16_array(const float *v, size_t n, uint16_t *out);
void orc_runner_f16_to_f32_array(const uint16_t *h, size_t n, float *out);
/* gguf_reader.cpp:668-676 and llama.cpp:547-555 */
void orc_get_scale_min_k4(int j, const uint8_t *q, uint8_t *sc, uint8_t *m);

/* gguf_reader.cpp:826-850, 541-572, 678-724, 774-824 */
void orc_dequant_q8_0(const uint8_t *data, float *out, size_t n);
void orc_dequant_q4_0(const uint8_t *data, float *out, size_t n);
void orc_dequant_q4_k(const uint8_t *data, float *out, size_t n);
void orc_dequant_q6_k(const uint8_t *data, float *out, size_t n);
/* gguf_reader.cpp:326-387 (type switch); returns 0, or -1 for a bad format */
int orc_dequant(int fmt, const uint8_t *data, float *out, size_t n);
/* dequant followed by the host narrowing of llama.cpp:805-811, 922-928 */
int orc_dequant_f16(int fmt, const uint8_t *data, uint16_t *out, size_t n);

/* llama.cpp:488-505; values [n], scales [n/32] */
void orc_quantize_rows_q8_0(const float *x, size_t n, int8_t *values,
                            uint16_t *scales);
/* values+scales -> GGUF Q8_0 blocks (inverse of gguf_reader.cpp:389-444) */
void orc_pack_q8_0(const int8_t *values, const uint16_t *scales, size_t n,
                   uint8_t *blocks);
/* gguf_reader.cpp:389-444 / 446-501: split blocks into values and scales */
void orc_split_q8_0(const uint8_t *blocks, uint32_t rows, uint32_t cols,
                    int8_t *values, uint16_t *scales);
void orc_split_q4_0(const uint8_t *blocks, uint32_t rows, uint32_t cols,
                    uint8_t *packed, uint16_t *scales);
/* llama.cpp:573-619; returns 1 on success, 0 if the shape is refused */
int orc_requantize_q4k_to_affine(const uint8_t *raw, size_t raw_bytes,
                                 uint32_t N, uint32_t K, uint8_t *packedT,
                                 uint16_t *scalesT);
/* decode of the affine layout, llama.cpp:712-720 */
void orc_decode_affine_q4(const uint8_t *packedT, const uint16_t *scalesT,
                          uint32_t N, uint32_t K, float *out /* [N,K] */);
/* TransposeQ4Nibble.cu:36-61 semantics: GGML Q4_0 packed [N,K/2] (block-local
 * low/high halves) -> [K,N/2], even n in the low nibble */
void orc_transpose_q4_nibble(const uint8_t *packed, uint32_t N, uint32_t K,
                             uint8_t *packedT);

/* Reference-layout ("separated") matmul, OpRegistry.h:2043-2051, 2107-2112:
 * C[m,n] = sum_k A[m,k] * float(q[k,n]) * S[k/32,n], fp32 sequential.
 * q4: nibble-8 (+ min when affine). scales are fp32 here (the harness uses
 * the float values); *_f16s variants take stored fp16 bits. */
void orc_matmul_sep_q8_f32(const float *A, const int8_t *B, const float *S,
                           uint32_t M, uint32_t K, uint32_t N, float *C);
void orc_matmul_sep_q4_f32(const float *A, const uint8_t *Bp, const float *S,
                           uint32_t M, uint32_t K, uint32_t N, int affine,
                           float *C);
/* RuntimeTests.cpp:2907-2920: double accumulation */
void orc_matmul_sep_q8_f64(const float *A, const int8_t *B, const float *S,
                           uint32_t M, uint32_t K, uint32_t N, float *C);

/* Native-block matmul: C[m,n] = sum_k A[m,k] * dequant(W)[n,k]; W is N rows
 * of K/blk GGUF blocks.  Semantics "A . dequant_cpu(W)^T" with the harness's
 * fp32 sequential accumulation (OpRegistry.h:2043-2051) resp. the double
 * accumulation of RuntimeTests.cpp:2907-2920. */
int orc_matmul_gguf_f32(int fmt, const uint8_t *W, const float *A, uint32_t M,
                        uint32_t K, uint32_t N, float *C);
int orc_matmul_gguf_f64(int fmt, const uint8_t *W, const float *A, uint32_t M,
                        uint32_t K, uint32_t N, double *C);
/* same over an already dequantized fp32 W [N,K] */
void orc_matmul_dense_f32(const float *Wf, const float *A, uint32_t M,
                          uint32_t K, uint32_t N, float *C);

/* MatMulQ8GemvDot.cu:60-64: per-32 activation quantizer, a_scale = amax/127,
 * q = clamp(round-half-away(a*127/amax), -127, 127) */
void orc_quantize_act_q8(const float *a, size_t n, int8_t *q, float *scale);
int orc_matmul_q8_i8(const uint8_t *W, const float *A, uint32_t M, uint32_t K,
                     uint32_t N, float *C32, double *C64);

/* own encoders (test inputs only; the reference has none for these) */
void orc_quantize_q4_0(const float *x, size_t n, uint8_t *blocks);
void orc_quantize_q4_k(const float *x, size_t n, uint8_t *blocks);
void orc_quantize_q6_k(const float *x, size_t n, uint8_t *blocks);
int orc_quantize(int fmt, const float *x, size_t n, uint8_t *blocks);

/* ---- operators between the matmuls of a decode step (fp32, as the reference kernels compute) ---- */
/* RMSNorm.cu:15-37: out = x * rsqrt(sum(x^2)/dim + eps) * weight, per row */
void orc_rmsnorm(const float *x, const float *weight, uint32_t rows, uint32_t dim,
                 float eps, float *out);
/* FusedRoPEKVWrite.cu:27-80: half-split rotation of q and k at `pos` with
 * tables [pos][head_dim/2]; k (rotated) and v go to cache row pos as fp16 bits
 * (host narrowing = round to nearest even here, as __float2half). */
void orc_rope_kv_write(const float *q, const float *k, const float *v, uint32_t pos,
                       const float *cos_t, const float *sin_t, uint32_t q_dim,
                       uint32_t kv_dim, uint32_t head_dim, uint32_t aligned_kv_dim,
                       float *q_out, uint16_t *k_cache, uint16_t *v_cache);
/* Attention.cu:35-106: per head, scores = scale * q.K over seq_len cache rows,
 * softmax, weighted sum of V; GQA: kv head = h / (n_heads / n_kv_heads) */
void orc_attention_decode(const float *q, const uint16_t *k_cache, const uint16_t *v_cache,
                          uint32_t seq_len, uint32_t n_heads, uint32_t n_kv_heads,
                          uint32_t head_dim, uint32_t aligned_kv_dim, float scale, float *out);
/* llama.cpp:1832-1857: silu(gate) * up on a fused [gate | up] vector */
void orc_silu_mul(const float *gate_up, uint32_t n, float *out);

#ifdef __cplusplus
}
#endif
#endif
