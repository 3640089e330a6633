/*
 * cut_hip.h -- C ABI of the MI355X (gfx950) backend for CUT's GGUF
 * quantized-matmul path: block dequantization, the batch-1..8 quantized GEMV
 * of decode and the dequant-to-LDS MFMA GEMM of prefill.
 *
 * Plain pointers and sizes only; every pointer named "device" is a HIP device
 * address owned by the caller.  No entry point below allocates device memory
 * unless its comment says so.  All functions return 0 on success and a
 * negative cuthip_status otherwise; cuthip_last_error() then holds a message
 * (thread-local).  A C++ caller maps non-zero to std::runtime_error, which is
 * how the reference reports failures (core/api/src/ComputeCommon.cpp:48-52).
 *
 * Precedent in the reference for "HIP behind a C ABI so host .cpp files need
 * no HIP header": benchmarks/vendor/amd/rocblas_wrappers.hip:1-120.
 */
#ifndef CUT_HIP_H
#define CUT_HIP_H

#include <stddef.h>
#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

typedef enum {
  CUTHIP_OK = 0,
  CUTHIP_ERR_INVALID = -1,   /* bad argument / unsupported shape */
  CUTHIP_ERR_HIP = -2,       /* a HIP runtime call failed */
  CUTHIP_ERR_NO_DEVICE = -3, /* no gfx950 device */
  CUTHIP_ERR_UNKNOWN_VARIANT = -4
} cuthip_status;

/* GGUF block formats (interface/loader/gguf/gguf_types.hpp:109-142):
 * Q8_0 34 B / 32, Q4_0 18 B / 32, Q4_K 144 B / 256, Q6_K 210 B / 256. */
typedef enum { CUTHIP_Q8_0 = 0, CUTHIP_Q4_0 = 1, CUTHIP_Q4_K = 2, CUTHIP_Q6_K = 3 } cuthip_format;
typedef enum { CUTHIP_F32 = 0, CUTHIP_F16 = 1 } cuthip_dtype;

/* Operator families with variant tables (the shape of
 * operators/impl/matmul/MatMulQ4Variants.generated.h:11-29). */
typedef enum { CUTHIP_OP_DEQUANT = 0, CUTHIP_OP_MATMUL_GGUF = 1, CUTHIP_OP_MATMUL_Q8 = 2, CUTHIP_OP_MATMUL_Q4 = 3 } cuthip_op;

/* Fused epilogues of the matmul (operators/impl/matmul/MatMulQ8Common.cuh:58-109;
 * MatMulOp.h:14 "MatMulFusion { None, Unary, Binary }"). */
typedef enum {
  CUTHIP_EPI_NONE = 0,
  CUTHIP_EPI_UNARY = 1,
  CUTHIP_EPI_BINARY = 2,
  /* SwiGLU over interleaved rows: weight rows 2i and 2i+1 are gate_i and up_i, C is [M, N/2] with
   * C[m, i] = silu(A . gate_i) * (A . up_i): the fused gate+up matmul, SiLU and BinaryMul of the runner
   * (interface/runner/llama/llama.cpp:1832-1857) in one launch.  M <= 8 only (the 8-row GEMV), N even;
   * strideC counts the N/2 outputs; epilogue_op and D unused. */
  CUTHIP_EPI_SWIGLU_PAIRS = 3
} cuthip_epilogue;
typedef enum { CUTHIP_UNARY_SILU = 0, CUTHIP_UNARY_RELU = 1, CUTHIP_UNARY_GELU_TANH = 2, CUTHIP_UNARY_SIGMOID = 3, CUTHIP_UNARY_TANH = 4, CUTHIP_UNARY_NEG = 5 } cuthip_unary_op;
typedef enum { CUTHIP_BINARY_ADD = 0, CUTHIP_BINARY_SUB = 1, CUTHIP_BINARY_MUL = 2, CUTHIP_BINARY_DIV = 3, CUTHIP_BINARY_MIN = 4, CUTHIP_BINARY_MAX = 5 } cuthip_binary_op;

/* Prologues on the activations of cuthip_matmul_gguf_pro. */
typedef enum { CUTHIP_PRO_NONE = 0, CUTHIP_PRO_RMSNORM = 1, CUTHIP_PRO_SWIGLU = 2 } cuthip_prologue;

typedef struct {
  char name[64];
  char arch[32];
  int compute_units;
  int wave_size;
  int lds_bytes_per_workgroup;
  int clock_khz;
  int memory_clock_khz;
  int memory_bus_bits;
  size_t hbm_bytes;
  size_t l2_bytes;
} cuthip_device_info_t;

/* One row of a variant table: MatMulQ4VariantInfo{name,wgX,wgY,effTileM,
 * effTileN,description} (MatMulQ4Variants.generated.h:11-18). Indices are ABI
 * and never renumbered (MatMulOp.cpp:353-356). */
typedef struct {
  const char *name;
  uint32_t wgX, wgY;
  uint32_t effTileM, effTileN;
  const char *description;
} cuthip_variant_info_t;

/* ---- library / device -------------------------------------------------- */

/* Selects the device and checks that it is gfx950.  Replaces the backend
 * constructor's device pick-up (core/backends/cuda/CudaCompute.cpp:60-100). */
int cuthip_init(int device);
const char *cuthip_last_error(void);
/* DeviceCaps + DeviceInfo of the reference (core/api/include/ComputeCommon.h:92-97). */
int cuthip_device_info(cuthip_device_info_t *info);

/* ---- memory, streams, events (ComputeInterface::createBuffer /
 * copyDataToBuffer / copyDataFromBuffer, core/api/include/ComputeInterface.h:45-120;
 * stream and event use of core/backends/cuda/CudaCommandBuffer.cpp:128-360).
 * cuthip_malloc is the ONLY call in this header that allocates device memory. */
int cuthip_malloc(void **device_ptr, size_t bytes);
int cuthip_free(void *device_ptr);
int cuthip_memcpy_h2d(void *device_dst, const void *host_src, size_t bytes, void *stream);
int cuthip_memcpy_d2h(void *host_dst, const void *device_src, size_t bytes, void *stream);
int cuthip_memcpy_d2d(void *device_dst, const void *device_src, size_t bytes, void *stream);
int cuthip_memset(void *device_dst, int value, size_t bytes, void *stream);
int cuthip_stream_create(void **stream);
int cuthip_stream_destroy(void *stream);
int cuthip_stream_sync(void *stream); /* NULL = the default stream */
int cuthip_event_create(void **event);
int cuthip_event_destroy(void *event);
int cuthip_event_record(void *event, void *stream);
int cuthip_event_sync(void *event);
int cuthip_event_elapsed_ms(void *start, void *stop, float *ms);

/* ---- variant tables ---------------------------------------------------- */
int cuthip_variant_count(int op);
int cuthip_variant_default(int op);
int cuthip_variant_info(int op, int index, cuthip_variant_info_t *info);
/* Index of a variant by name, or CUTHIP_ERR_UNKNOWN_VARIANT: an unknown name is
 * a hard error, never a silently skipped dispatch (the hazard described in
 * core/backends/cuda/CudaCommandBuffer.cpp:146-162). */
int cuthip_variant_lookup(int op, const char *name);

/* ---- dequantization ----------------------------------------------------
 * Replaces Operations::dequantize(raw, fmt, rows, cols) / DequantOpNode
 * (runtime/Operations.cpp:1354-1361, operators/impl/dequant/DequantOp.cpp:7-67;
 * kernels DequantQ4K.cu:6-50, DequantQ6K.cu:6-64) and the host loops
 * GGUFReader::dequantize_* (interface/loader/gguf/gguf_reader.cpp:541-850).
 *
 * blocks : device, rows x (cols/blk) GGUF blocks, row-major, 2-byte aligned
 * out    : device, [rows, out_stride] elements of out_dtype; the reference
 *          uses out_stride = (cols+3)&~3 (DequantOp.cpp:15)
 * fp32 output is bit-identical to the reference's CPU dequantizers; fp16
 * output is bit-identical to that followed by the host narrowing f32ToF16
 * (interface/runner/llama/llama.cpp:445-482, used at :805-811 and :922-928).
 * cols must be a multiple of the block size (32 or 256). */
int cuthip_dequant(int fmt, const void *blocks, void *out, int out_dtype, uint32_t rows, uint32_t cols,
                   uint32_t out_stride, void *stream);

/* ---- quantized matmul on native GGUF blocks ------------------------------
 * C[m,n] (op)= sum_k A[m,k] * dequant(W)[n,k]   ("A . dequant_cpu(W)^T")
 *
 * The op-level call behind Operations::matmul(a, packedB, scales)
 * (runtime/Operations.cpp:226-231 -> MatMulOpNode 3-input constructor,
 * operators/impl/matmul/MatMulOp.cpp:271-383) for weights kept as GGUF blocks:
 * it supersedes MatMulQ{4,8}GemvKPar8.cu (M == 1 decode default,
 * MatMulOp.cpp:336-356) and MatMulQ{4,8}CoopMatTiled.cu (M > 1 default,
 * MatMulOp.cpp:363-374).
 *
 * W      : device, N rows of K/blk GGUF blocks (the file layout: GGUF dims
 *          [K, N], gguf_reader.cpp:404-406); the base must be 16-byte aligned
 *          and every row must start 2-byte aligned (always true)
 * A      : device, [M, strideA] of a_dtype (fp32 as in the reference, or fp16)
 * C      : device, [M, strideC] of c_dtype
 * D      : device, [M, strideC] of c_dtype, second operand of a BINARY
 *          epilogue (residual add etc.), else NULL
 * K must be a multiple of the block size; fp32 accumulation throughout.
 * variant: index into the CUTHIP_OP_MATMUL_GGUF table, or -1 = choose by shape
 *          (M <= 8 -> streaming GEMV, 9..40 -> passes of 8 rows through it, else the
 *          LDS-tiled MFMA GEMM); variant 4 needs
 *          cuthip_matmul_gguf_ws. */
int cuthip_matmul_gguf(int fmt, const void *W, const void *A, int a_dtype, void *C, int c_dtype, uint32_t M, uint32_t K,
                       uint32_t N, uint32_t strideA, uint32_t strideC, int epilogue, int epilogue_op, const void *D,
                       int variant, void *stream);

/* The same matmul with a caller-provided device workspace, which opens variant 4
 * (MatMulGgufDequantGemm) for large M: the weight tensor is dequantized once to
 * fp16 in the workspace (cuthip_dequant's kernel) and multiplied by a dense fp16
 * MFMA GEMM, two launches on `stream`, no allocation.  It replaces the M > 1
 * default MatMulQ{4,8}CoopMatTiled.cu (MatMulOp.cpp:363-374), which re-decodes
 * the weights for every tile of activations.
 * workspace: device, 256-byte aligned, at least
 *            cuthip_matmul_gguf_workspace_bytes(fmt, M, K, N, a_dtype) bytes
 *            (N*K fp16, plus M*K fp16 when A is fp32, plus the larger of the fp32
 *            partial products of a split K and 32 MiB of scratch for the vendor
 *            GEMM); contents are scratch.
 * variant  : 4 = the two-pass path (an error if K is not a multiple of 128, the
 *            rows of A are not 16-byte aligned or the workspace is too small);
 *            5 = MatMulGgufDequantBlasLt: the same dequantization, then hipBLASLt's
 *            dense fp16 GEMM (the weights are plain fp16 by then, so it is a library
 *            GEMM; the library is opened with dlopen by cuthip_init and its handle is
 *            created then (outside any stream capture), the only allocation this
 *            library ever causes; the first matmul of a new shape asks the library's
 *            heuristic for a kernel, on the host; an error if
 *            the library is absent or an epilogue is asked for; CUT_HIP_NO_BLASLT=1 in
 *            the environment keeps it closed);
 *            -1 = choose by shape: the two-pass path (variant 5 where hipBLASLt is
 *            present, has a kernel for the shape and no epilogue is fused, else
 *            variant 4) when it applies and M >= 1024 (or, with so
 *            few output tiles that the single-launch GEMM would leave most of the chip
 *            idle, from M = 256, and from M = 41 when K >= 8192; K is then split and
 *            the partial products summed), else
 *            as cuthip_matmul_gguf; 0..3 = as cuthip_matmul_gguf (workspace unused).
 * With variant -1 the workspace also serves batch 3-8 on long rows (K >= 8192) of few (N < 12288): the 8-row GEMV
 * then splits K across workgroups, writes fp32 partial products to the workspace and sums them in a second launch
 * (the unsplit kernel would have to stage all of the activations in every workgroup).
 * Other arguments and numerics as cuthip_matmul_gguf. */
size_t cuthip_matmul_gguf_workspace_bytes(int fmt, uint32_t M, uint32_t K, uint32_t N, int a_dtype);
int cuthip_matmul_gguf_ws(int fmt, const void *W, const void *A, int a_dtype, void *C, int c_dtype, uint32_t M, uint32_t K,
                          uint32_t N, uint32_t strideA, uint32_t strideC, int epilogue, int epilogue_op, const void *D,
                          int variant, void *workspace, size_t workspace_bytes, void *stream);

/* Prefill matmul on weights that are kept dequantized: W16 = fp16 [N][K], written once per tensor by
 * cuthip_dequant(fmt, blocks, W16, CUTHIP_F16, N, K, K, stream) (bit-exact against the reference's CPU dequant +
 * f32ToF16, gguf_reader.cpp:515-850, llama.cpp:445-482, 805-811).  The reference's runner does the same for its
 * float path (it uploads dequantized fp16 weights, llama.cpp:800-815); here the GGUF blocks stay resident for the
 * decode GEMV, which is bound by bytes, and the fp16 copy (2 bytes per weight: 16 GB for an 8B model of the 288 GB)
 * serves prefill, which is bound by the matrix core, so no prefill call pays for a dequantization.
 * C[M,N] = A[M,K] . W16^T with fp32 accumulation; the GEMM is hipBLASLt's where that library is present and no
 * epilogue is fused, else this library's dense fp16 MFMA kernel.  K a multiple of 128; W16 256-byte aligned;
 * workspace: device, 256-byte aligned, cuthip_matmul_dense_f16_workspace_bytes bytes (converted activations when A is
 * fp32, split-K partial products, GEMM scratch).  Epilogues: none, unary, binary as in cuthip_matmul_gguf. */
size_t cuthip_matmul_dense_f16_workspace_bytes(uint32_t M, uint32_t K, uint32_t N, int a_dtype);
int cuthip_matmul_dense_f16(const void *W16, const void *A, int a_dtype, void *C, int c_dtype, uint32_t M, uint32_t K, uint32_t N,
                            uint32_t strideA, uint32_t strideC, int epilogue, int epilogue_op, const void *D, void *workspace,
                            size_t workspace_bytes, void *stream);

/* Fields of an RMSNorm carried across batch-1 matmuls (cuthip_matmul_gguf_carry). */
typedef struct {
  const float *sumsq_parts;      /* consumer: device [ceil(K/8)], partial sums of squares of the un-normalised activations */
  float eps;
  const float *next_norm_weight; /* producer: weight [N] of the norm that follows this matmul */
  void *next_x16;                /* producer: fp16 [N] out */
  float *next_sumsq_parts;       /* producer: device [ceil(N/8)] out, sum of C^2 over each group of 8 outputs */
} cuthip_norm_carry_t;

/* RoPE and KV-cache append in the epilogue of cuthip_matmul_gguf_pair, which then is the whole of
 * "q, k, v projections + FusedRoPEKVWrite" (operators/impl/attention/FusedRoPEKVWrite.cu:12-81) in one launch:
 * tensor A holds the rows [q heads | k heads], inside every head interleaved as d = 0, head_dim/2, 1,
 * head_dim/2 + 1, ... (a row permutation done once at load) so that the two partners of the half-split rotation
 * are neighbouring rows; tensor B holds the v rows.  Rotated q goes to q_out [q_dim] in natural order, rotated k and
 * v as fp16 to row runtime_params[0] of the caches.  Ca and Cb are not written (may be NULL). */
typedef struct {
  const uint32_t *runtime_params;   /* device uint32[2]: {position, sequence length} */
  const float *cos_table, *sin_table; /* [position][head_dim / 2] */
  void *q_out;
  int q_out_dtype;
  void *k_cache, *v_cache;          /* fp16 [max_ctx][aligned_kv_dim] */
  uint32_t q_dim, head_dim, aligned_kv_dim;
} cuthip_rope_append_t;

/* Two batch-1 matmuls on the same activations in one launch:
 *   Ca[Na] = A . dequant(Wa)^T,  Cb[Nb] = A . dequant(Wb)^T,  A [K].
 * For the q/k and v projections of a decode step, whose weights differ in format
 * (Q4_K and Q6_K in the common GGUF mixes) and so cannot be concatenated like
 * gate and up; the reference fuses wqkv only when the loader could concatenate
 * them and otherwise issues one matmul per projection
 * (interface/runner/llama/llama.cpp:1710-1756).  One launch for the K-quant
 * formats at decode shapes, otherwise the same two products as two launches.
 * No epilogue; dtypes and alignment as cuthip_matmul_gguf. */
int cuthip_matmul_gguf_pair(int fmt_a, const void *Wa, uint32_t Na, void *Ca, int fmt_b, const void *Wb, uint32_t Nb,
                            void *Cb, const void *A, int a_dtype, int c_dtype, uint32_t K,
                            const cuthip_norm_carry_t *carry /* consumer fields only, or NULL */,
                            const cuthip_rope_append_t *rope /* or NULL */, void *stream);

/* Batch-1 matmul that takes part in an RMSNorm carried across matmuls, which removes
 * the RMSNorm launches of a decode step (the reference fuses RMSNorm into its
 * consumers, runtime/graph/GraphOptimizer.cpp:46-70; here the work is split between
 * producer and consumer so that neither repeats it per workgroup):
 *   producer (the matmul whose epilogue forms the residual stream, C = A.W^T + D):
 *     also stores next_x16[n] = fp16(C[n] * next_norm_weight[n]) and the sum of
 *     C[n]^2 over each group of 8 outputs in next_sumsq_parts[n / 8];
 *   consumer (the matmul that reads next_x16 as its activations, so its K is the
 *     producer's N): multiplies its result by rsqrt(sum(sumsq_parts) / K + eps)
 *     before the epilogue, i.e. computes RMSNorm(x) . W^T with the rounding to fp16
 *     taken before the scaling.
 * The partial sums are added in a fixed order (no atomics): results are
 * reproducible from run to run.
 * Any field group may be NULL.  M = 1, the 8-row GEMV only; other arguments as
 * cuthip_matmul_gguf (strideA = K, strideC = N, or N/2 with CUTHIP_EPI_SWIGLU_PAIRS). */
int cuthip_matmul_gguf_carry(int fmt, const void *W, const void *A, int a_dtype, void *C, int c_dtype, uint32_t K, uint32_t N,
                             int epilogue, int epilogue_op, const void *D, const cuthip_norm_carry_t *carry, void *stream);

/* The same matmul at batch 1 with the operator in front of it fused into the
 * staging of the activations, which saves a launch per use in a decode step
 * (the reference fuses RMSNorm into its consumers in ExtendedRMSNormFusion /
 * RMSNormFusion, runtime/graph/GraphOptimizer.cpp:46-70):
 *   CUTHIP_PRO_RMSNORM: A = x [K]; C = (x * rsqrt(mean(x^2) + eps) * norm_weight) . dequant(W)^T
 *                       (RMSNorm.cu:15-37 followed by the matmul; norm_weight fp32 [K], 16-byte aligned)
 *   CUTHIP_PRO_SWIGLU : A = [gate(K) | up(K)] fp16; C = (silu(gate) * up) . dequant(W)^T
 *                       (llama.cpp:1832-1860: SiLU, BinaryMul, then w_down)
 * M must be 1 and the activations must fit the 8-row GEMV's LDS budget (K <= ~40k);
 * other arguments as cuthip_matmul_gguf (no variant choice: always the 8-row GEMV). */
int cuthip_matmul_gguf_pro(int fmt, const void *W, const void *A, int a_dtype, void *C, int c_dtype, uint32_t K, uint32_t N,
                           int epilogue, int epilogue_op, const void *D, int prologue, const float *norm_weight, float eps,
                           void *stream);

/* ---- quantized matmul on the reference's separated weight layout ----------
 * Drop-in for the 3-input MatMulOpNode (operators/impl/matmul/MatMulOp.cpp:271-383)
 * on the tensors the reference's loader produces (read_tensor_q8_separated /
 * read_tensor_q4_separated, gguf_reader.cpp:389-501; affine Q4 from
 * requantizeQ4KToAffine, llama.cpp:573-619); arguments are its PushConstants
 * {M, K, N, strideA, strideB, strideC, scaleStride} (MatMulOp.cpp:514-541):
 *   Q8: B int8 [K, strideB], scales fp16 [K/32, scaleStride]
 *   Q4: packedB bytes [K, strideBNpacked], even column in the low nibble,
 *       value nibble - 8; affine != 0: minima in rows [K/32, 2K/32) of scales
 *       (MatMulQ4Common.cuh:126-153)
 * A [M, strideA], C and D [M, strideC] are fp32; K must be a multiple of 32.
 * epilogue / epilogue_op / D as in cuthip_matmul_gguf (MatMulFusion).
 * workspace: device scratch of cuthip_matmul_sep_workspace_bytes(M, K, N)
 * bytes, 256-byte aligned (may be NULL when that is 0).  Below 32 rows of A
 * (or when K is not a multiple of 128) the weights are streamed once per 4 rows
 * and the workspace holds split-K partial sums; from 32 rows on the tensors are
 * first dequantized to fp16 [N][K] in the workspace (one launch) and multiplied
 * by the dense GEMM of cuthip_matmul_dense_f16 (fp16 operands, fp32 accumulate:
 * within 1e-3 of the fp32 loop). */
size_t cuthip_matmul_sep_workspace_bytes(uint32_t M, uint32_t K, uint32_t N);
int cuthip_matmul_q8_sep(const float *A, const int8_t *B, const uint16_t *scales, const float *D, float *C, uint32_t M,
                         uint32_t K, uint32_t N, uint32_t strideA, uint32_t strideB, uint32_t strideC, uint32_t scaleStride,
                         int epilogue, int epilogue_op, void *workspace, size_t workspace_bytes, void *stream);
int cuthip_matmul_q4_sep(const float *A, const uint8_t *packedB, const uint16_t *scales, const float *D, float *C, uint32_t M,
                         uint32_t K, uint32_t N, uint32_t strideA, uint32_t strideBNpacked, uint32_t strideC,
                         uint32_t scaleStride, int epilogue, int epilogue_op, int affine, void *workspace,
                         size_t workspace_bytes, void *stream);

/* ---- Q8_0 weights x int8 activations on the int8 matrix core -----------------
 * The arithmetic of the reference's int8 dot-product GEMV (MatMulQ8GemvDot.cu:60-85)
 * for prefill-sized M: A is quantized per 32 elements (a_scale = amax / 127,
 * q = clamp(round(a * (127 / amax)), -127, 127)) and
 *   C[m,n] = sum_b float(sum_{k in b} qa[m,k] * qw[n,k]) * a_scale[m,b] * d_w[n,b]
 * with W in GGUF Q8_0 blocks [N][K/32].  The 8-bit activations put the result
 * about 5e-3 (normwise) from the fp32 path, so this is its own entry point and
 * cuthip_matmul_gguf never selects it.  workspace: device scratch of
 * cuthip_matmul_q8_i8_workspace_bytes(M, K) bytes (the quantized activations),
 * 16-byte aligned.  A: fp32 or fp16, aligned to 4 elements, strideA a multiple
 * of 4; epilogue / epilogue_op / D as in cuthip_matmul_gguf (none, unary, binary). */
size_t cuthip_matmul_q8_i8_workspace_bytes(uint32_t M, uint32_t K);
int cuthip_matmul_q8_i8(const void *W, const void *A, int a_dtype, void *C, int c_dtype, uint32_t M, uint32_t K, uint32_t N,
                        uint32_t strideA, uint32_t strideC, int epilogue, int epilogue_op, const void *D, void *workspace,
                        size_t workspace_bytes, void *stream);

/* ---- load-time preparation of the separated layout, on the device ----------
 * cuthip_prepare_sep: GGUF blocks (row n = K/blk consecutive blocks, as in the
 * file) -> the tensors cuthip_matmul_q8_sep / cuthip_matmul_q4_sep take, in one
 * launch.  Replaces the host split of read_tensor_q8_separated /
 * read_tensor_q4_separated (gguf_reader.cpp:389-501) followed by the GPU
 * transposes of uploadQ4 / uploadQ8 (llama.cpp:940-965, TransposeQ4Nibble.cu:17-61),
 * and, for fmt = CUTHIP_Q4_K, requantizeQ4KToAffine (llama.cpp:573-619):
 *   Q8_0: B int8 [K, strideB],        scales fp16 [K/32, scaleStride]
 *   Q4_0: B nibbles [K, strideB bytes], even row n in the low nibble; scales as Q8_0
 *   Q4_K: B nibbles as Q4_0; scales fp16 [2K/32, scaleStride]: rows [0, K/32) hold
 *         f16(d*sc), rows [K/32, 2K/32) hold f16(8*(d*sc) - dmin*m); decode
 *         (nibble - 8) * scale + min (pass affine = 1 to cuthip_matmul_q4_sep)
 * N must be even for the nibble formats (the reference throws otherwise), K a
 * multiple of the block size; B must be 4-byte aligned.  Bit-exact against the
 * reference's host code for finite block scales. */
int cuthip_prepare_sep(int fmt, const void *blocks, uint32_t N, uint32_t K, void *B, uint32_t strideB, uint16_t *scales,
                       uint32_t scaleStride, void *stream);

/* TransposeQ4NibbleOpNode (operators/impl/q4transpose/TransposeQ4NibbleOp.cpp:7-23,
 * TransposeQ4Nibble.cu:17-61): packed [N, strideInHalf bytes] in GGML Q4_0 nibble
 * order (low nibble of byte j of a 16-byte block = element j, high = j + 16) ->
 * packedT [K, strideOutHalf bytes], even n in the low nibble.  N even, K a
 * multiple of 32, strideInHalf even. */
int cuthip_transpose_q4_nibble(const void *packed, void *packedT, uint32_t N, uint32_t K, uint32_t strideInHalf,
                               uint32_t strideOutHalf, void *stream);

/* quantizeRowsQ8_0 (llama.cpp:488-505): fp32 x[n] -> n/32 Q8_0 blocks (34 bytes:
 * fp16 scale, 32 int8).  d = absmax/127, q = lroundf(x * (1/d)) from the
 * unrounded d, stored scale = f32ToF16(d).  The reference returns values and
 * scales as two vectors; the blocks written here hold the same numbers in GGUF
 * order, ready for cuthip_matmul_gguf or cuthip_prepare_sep.  x 16-byte aligned. */
int cuthip_quantize_rows_q8_0(const float *x, uint64_t n, void *blocks, void *stream);

/* ---- the operators between the matmuls of a decode step --------------------
 * What the runner chains around the quantized matmuls for one token
 * (interface/runner/llama/llama.cpp, runLayer / decode graph).  All take
 * fp32 or fp16 activations (cuthip_dtype) and compute in fp32.
 * runtime_params: device uint32[2] = {position of this token, sequence
 * length including it}, the reference's runtimeParams buffer: read on the
 * device so that a captured graph can be replayed for the next token. */

/* out[r,c] = x[r,c] * rsqrt(mean_c(x[r,:]^2) + eps) * weight[c]
 * (operators/impl/rmsnorm/RMSNorm.cu:15-37). stride: elements between rows. */
int cuthip_rmsnorm(const void *x, int x_dtype, const float *weight, void *out, int out_dtype, uint32_t rows, uint32_t dim,
                   uint32_t stride, float eps, void *stream);

/* Half-split RoPE on q [q_dim] and k [kv_dim] with tables [pos][head_dim/2];
 * k (rotated) and v are stored as fp16 to cache row `position`
 * (rows of aligned_kv_dim elements); q (rotated) goes to q_out
 * (operators/impl/attention/FusedRoPEKVWrite.cu:12-81). */
int cuthip_rope_kv_write(const void *q, const void *k, const void *v, int in_dtype, const uint32_t *runtime_params,
                         const float *cos_table, const float *sin_table, void *k_cache, void *v_cache, void *q_out,
                         int q_out_dtype, uint32_t q_dim, uint32_t kv_dim, uint32_t head_dim, uint32_t aligned_kv_dim,
                         void *stream);

/* Scaled dot-product attention of one token over an fp16 KV cache with GQA:
 * out[h,:] = softmax(scale * q[h,:] . K[0:seq, h/nRep, :]) . V[0:seq, h/nRep, :]
 * (operators/impl/attention/Attention.cu:35-106; head_dim <= 128 as there).
 * workspace: device scratch of cuthip_attn_decode_workspace_bytes(); the
 * call allocates nothing.  max_seq_len sizes the launch (cache capacity). */
size_t cuthip_attn_decode_workspace_bytes(uint32_t n_heads, uint32_t head_dim, uint32_t max_seq_len);
int cuthip_attn_decode(const void *q, int q_dtype, const void *k_cache, const void *v_cache, const uint32_t *runtime_params,
                       void *out, int out_dtype, uint32_t n_heads, uint32_t n_kv_heads, uint32_t head_dim,
                       uint32_t aligned_kv_dim, float scale, uint32_t max_seq_len, void *workspace, size_t workspace_bytes,
                       void *stream);

/* cuthip_attn_decode without a caller workspace.  It has no counterpart in the reference; it exists for callers that
 * cannot allocate device memory or carry a workspace around (code under HIP graph capture, tight serving loops,
 * harnesses that forbid hipMalloc): the partial results of the context splits live in a device array inside this
 * library, cuthip_attn_decode_static_max_bytes() = 4 MiB on every GPU the library runs on, held until the process
 * ends.  The call allocates nothing; its device address is looked up by cuthip_init (or on the first call on a
 * device).  Shapes whose partial results exceed the array (cuthip_attn_decode_workspace_bytes(n_heads, head_dim,
 * max_seq_len) > 4 MiB, e.g. 32 heads of dimension 128 beyond a capacity of 16,128) are rejected with
 * CUTHIP_ERR_INVALID.  All calls on one GPU share the array: calls that overlap on one GPU (two streams, two
 * threads) race; serialise them or give the others a workspace through cuthip_attn_decode.  Results are identical
 * to cuthip_attn_decode (same kernels). */
size_t cuthip_attn_decode_static_max_bytes(void);
int cuthip_attn_decode_static(const void *q, int q_dtype, const void *k_cache, const void *v_cache,
                              const uint32_t *runtime_params, void *out, int out_dtype, uint32_t n_heads, uint32_t n_kv_heads,
                              uint32_t head_dim, uint32_t aligned_kv_dim, float scale, uint32_t max_seq_len, void *stream);

/* out[i] = silu(gate_up[i]) * gate_up[n + i]: the SwiGLU combine after a fused
 * gate+up matmul (llama.cpp:1832-1857: unary SiLU, then BinaryMul). */
int cuthip_silu_mul(const void *gate_up, int in_dtype, void *out, int out_dtype, uint32_t n, void *stream);

/* Index of the first maximum of x[0:n] (greedy sampling), written to device memory. */
int cuthip_argmax(const void *x, int x_dtype, uint32_t n, uint32_t *out_index, void *stream);

#ifdef __cplusplus
}
#endif
#endif /* CUT_HIP_H */
