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
/* epilogue_op of a fused epilogue: the reference's operator codes themselves (OP_UNARY_* / OP_BINARY_* of
 * operators/runtime/ComputeOpsShared.h:22-40, 118-167, the value of its FUSION_OP specialization constant), so a
 * caller passes what MatMulOpNode::setFusion received.  The set is what cut_writeOutput implements
 * (operators/impl/matmul/MatMulQ8Common.cuh:58-109: 21 unary and 9 binary operators) with the same formulas; any
 * other code is refused with CUTHIP_ERR_INVALID (the reference's shader would silently store the unfused value).
 * NEG, TANH, RELU, SIGMOID, GELU, SILU and ADD, SUB, MUL, DIV, MIN, MAX (what the runner's graphs fuse) run inside the
 * matmul kernels; the others are applied by a second, elementwise launch on the same stream (inlined at every store
 * of the tiled GEMMs the whole set costs those kernels their register allocation): same
 * result up to the rounding of C to its dtype in between, and for MOD, POW, FLOOR_DIV D must not alias C. */
typedef enum {
  CUTHIP_UNARY_NEG = 100, CUTHIP_UNARY_ABS = 101, CUTHIP_UNARY_SQRT = 102, CUTHIP_UNARY_SQUARE = 103,
  CUTHIP_UNARY_RECIPROCAL = 104, CUTHIP_UNARY_EXP = 106, CUTHIP_UNARY_LOG = 109, CUTHIP_UNARY_TANH = 121,
  CUTHIP_UNARY_FLOOR = 122, CUTHIP_UNARY_CEIL = 123, CUTHIP_UNARY_ROUND = 124, CUTHIP_UNARY_RELU = 130,
  CUTHIP_UNARY_SIGMOID = 131, CUTHIP_UNARY_GELU = 132, CUTHIP_UNARY_GELU_TANH = 132, CUTHIP_UNARY_SILU = 133,
  CUTHIP_UNARY_SOFTPLUS = 134, CUTHIP_UNARY_RELU6 = 137, CUTHIP_UNARY_MISH = 141, CUTHIP_UNARY_HARDSWISH = 142,
  CUTHIP_UNARY_HARDSIGMOID = 143, CUTHIP_UNARY_RSQRT = 148
} cuthip_unary_op;
typedef enum {
  CUTHIP_BINARY_ADD = 0, CUTHIP_BINARY_SUB = 1, CUTHIP_BINARY_MUL = 2, CUTHIP_BINARY_DIV = 3, CUTHIP_BINARY_MOD = 4,
  CUTHIP_BINARY_POW = 5, CUTHIP_BINARY_FLOOR_DIV = 6, CUTHIP_BINARY_MIN = 13, CUTHIP_BINARY_MAX = 14
} cuthip_binary_op;
/* 1 if `op` is an operator the given epilogue kind implements, else 0. */
int cuthip_epilogue_op_supported(int epilogue, int op);

/* Prologues on the activations of cuthip_matmul_gguf_pro. */
/* (CUTHIP_PRO_ATTN_MERGE is the prologue of cuthip_matmul_gguf_attn_merge; cuthip_matmul_gguf_pro refuses it.) */
typedef enum { CUTHIP_PRO_NONE = 0, CUTHIP_PRO_RMSNORM = 1, CUTHIP_PRO_SWIGLU = 2, CUTHIP_PRO_ATTN_MERGE = 3 } cuthip_prologue;

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
 * constructor's device pick-up (core/backends/cuda/CudaCompute.cpp:60-100).
 * Also takes over, once, the launch-shape overrides of the environment (CUT_HIP_ROWS8_SHAPE, CUT_HIP_GEMV_SHAPE,
 * CUT_HIP_GEMM_KSPLIT, CUT_HIP_DENSE_TILE, CUT_HIP_DENSE_MFMA16, CUT_HIP_DENSE_PF: the values cuthip_set_tuning takes);
 * no launch reads the environment. */
int cuthip_init(int device);
const char *cuthip_last_error(void);
/* Forces a launch shape for tests and tuning sweeps, process-wide, until changed; value NULL or "" restores the
 * library's own choice.  Keys: "rows8_shape" = "rwg,kw" (8-row GEMV: row groups per workgroup, K ranges 1/2/4/8),
 * "gemv_shape" = "kp,waves" (fallback GEMV), "gemm_ksplit" = "n" (K ranges of the single-launch GEMM, 1..16),
 * "dense_tile" = "bm,bn[,ksplit]" (256,224 / 128,448 / 128,256 / 256,256), "dense_mfma16" = "0" | "1",
 * "dense_pf" = prefetch distance in slices.  Not synchronised with launches in flight on other threads.  The
 * reference's counterpart is the per-operator `spec` argument that its tests and op_bench pass
 * (operators/impl/matmul/MatMulOp.cpp:336-374); an unknown key or a malformed value is CUTHIP_ERR_INVALID. */
int cuthip_set_tuning(const char *key, const char *value);
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
/* hipMemsetAsync; CUTHIP_ERR_INVALID while `stream` is capturing (memset nodes are kept out of graphs). */
int cuthip_memset(void *device_dst, int value, size_t bytes, void *stream);
int cuthip_stream_create(void **stream);
int cuthip_stream_destroy(void *stream);
int cuthip_stream_sync(void *stream); /* NULL = the default stream */
int cuthip_event_create(void **event);
int cuthip_event_destroy(void *event);
int cuthip_event_record(void *event, void *stream);
int cuthip_event_sync(void *event);
int cuthip_event_elapsed_ms(void *start, void *stop, float *ms);

/* Capture and replay of a launch sequence: what the reference's reusable command buffers do on its CUDA backend
 * (core/backends/cuda/CudaCommandBuffer.cpp:261-285: cuStreamBeginCapture, the dispatches, cuStreamEndCapture,
 * cuGraphInstantiate once, then cuGraphLaunch per token).  Between begin and end every cuthip_* launch on `stream`
 * (a stream from cuthip_stream_create, not the default one) is recorded instead of run; no entry point of this
 * library allocates, so all of them may be captured (cuthip_memset is the exception and refuses a capturing stream:
 * clear memory before the capture or with a kernel of the sequence).  Values that change between replays (position, sequence length, token ids,
 * penalty lists) are read from device memory by the kernels, so the host updates those buffers and launches the same
 * graph again.  The handle owns both the graph and its executable form. */
int cuthip_graph_begin_capture(void *stream);
int cuthip_graph_end_capture(void *stream, void **graph);
int cuthip_graph_launch(void *graph, void *stream);
int cuthip_graph_destroy(void *graph);

/* Measurement aid (no counterpart in the reference): one launch that only reads `bytes` of device memory with
 * 16-byte loads (the tail below 16 bytes is ignored) and stores one dword per wave into sink (65,536 dwords).  Its
 * duration is what a launch of that size can reach on the part when it does nothing but load, the yardstick the
 * streaming kernels are held against (bench.py --calibrate-read). */
int cuthip_read_probe(const void *src, size_t bytes, uint32_t *sink, void *stream);
/* Test hook (no counterpart in the reference): fills the LDS of every CU with `pattern`.  LDS keeps what the last
 * workgroup left there, so an operator that read a location it had not written would return results that depend on
 * what ran before it; the tests run the operators behind different patterns and ask for identical bits. */
int cuthip_debug_fill_lds(uint32_t pattern, void *stream);

/* ---- variant tables ---------------------------------------------------- */
int cuthip_variant_count(int op);
/* Default index of a table: the reference's kMatMulQ8DefaultVariant = 2 / kMatMulQ4DefaultVariant = 0 for the
 * separated-layout tables; 0 for CUTHIP_OP_MATMUL_GGUF, whose entry 0 is valid for every M (it is the streaming GEMV
 * up to 8 rows of A and the library's choice by shape beyond), so that the reference's idiom
 * `spec ? *spec : kDefaultVariant` (MatMulOp.cpp:244-246) never yields an index the shape rejects. */
int cuthip_variant_default(int op);
/* 1 if the variant can run in this process, 0 if not (MatMulGgufDequantBlasLt without hipBLASLt), < 0 = no such
 * variant.  A tuning rule that names an unavailable variant is to be skipped by the caller. */
int cuthip_variant_available(int op, int index);
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
 *          (M <= 8 -> streaming GEMV; 9..16 rows of Q4_K with K <= 4096 -> variant 6, the
 *          streaming MFMA kernel; other 9..40 -> passes of 8 rows through the GEMV; else
 *          the LDS-tiled MFMA GEMM); variants 4 and 5 need cuthip_matmul_gguf_ws, which
 *          also gives variants 2 and 6 the scratch memory they split K through. */
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
 *            GEMM; the library is opened with dlopen, and its handle created, by the first
 *            cuthip_variant_available(CUTHIP_OP_MATMUL_GGUF, 5) or the first call with this index:
 *            a caller that captures streams does one of these before it captures; it is the
 *            only allocation this library ever causes; the first matmul of a new shape asks the
 *            library's heuristic for a kernel, on the host; an error if the library is absent or
 *            an epilogue is asked for; CUT_HIP_NO_BLASLT=1 in the environment keeps it closed).
 *            Variant 5 runs only when this index is passed: no automatic choice takes it;
 *            -1 = choose by shape among the hand-written kernels: the two-pass path (variant 4)
 *            when it applies and M >= 1024 (or, with so
 *            few output tiles that the single-launch GEMM would leave most of the chip
 *            idle, from M = 256, and from M = 41 when K >= 8192; K is then split and
 *            the partial products summed), else
 *            as cuthip_matmul_gguf; 0, 1, 3 = as cuthip_matmul_gguf (workspace unused);
 *            2 = the single-launch GEMM, which with a workspace at hand splits K over
 *            workgroups where its tiles alone would not fill the chip (up to 256 rows:
 *            fp32 partial products in the workspace, summed in a second launch);
 *            6 = MatMulGgufStreamMfma (Q4_K, M <= 32, 16-byte aligned rows of A, else an
 *            error): the weights stay packed until they are multiplied (integer-scaled
 *            nibbles as fp16 subnormals into 16x16x32 MFMAs: the products are exact and
 *            the result differs from fp32 FMAs only by the order of the fp32 sums, given
 *            fp16 activations; fp32 activations are rounded to fp16, nearest even, when they
 *            are staged - 2^-11 relative per element, |a| > 65504 becomes inf - as on the 8-row
 *            GEMV and the GEMMs); K above 4096 (2048 beyond 16 rows) is split over
 *            workgroups through the workspace, an error without one.  With variant -1
 *            it is what runs for 9..32 rows of Q4_K.
 * With variant -1 the workspace also serves batch 2-8 (Q6_K: 3-8) on long rows (K >= 8192) of few (N < 12288): the 8-row GEMV
 * then splits K across workgroups, writes fp32 partial products to the workspace and sums them in a second launch
 * (the unsplit kernel would have to stage all of the activations in every workgroup).  The same for any N where the
 * batch rows times K exceed the 96 KB of LDS the unsplit kernel stages them in (8 rows of K >= 8192, 4 of K >= 16384): K
 * is split into as many parts as that takes (28672 x 8192 at 8 rows: Q4_K 47 us against 80 without a workspace, Q6_K 77
 * against 123, Q8_0 80 against 119).  Without a workspace such shapes run as passes over fewer rows where those fit
 * (all formats but Q4_K), else on the 32-row fallback kernel.
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
  void *k_cache, *v_cache;          /* fp16 [max_positions][aligned_kv_dim] */
  uint32_t q_dim, head_dim, aligned_kv_dim;
  uint32_t max_positions;           /* rows of the caches and of the tables: a position at or beyond it writes nothing */
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
 * reproducible from run to run.  next_x16 holds the un-normalised C[n] * weight[n]:
 * the carry is exact to fp16 rounding while |C[n] * weight[n]| <= 65504 (larger
 * products store as infinity; the plain RMSNorm kernel has no such limit).
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
 * within 1e-3 of the fp32 loop, normwise).  That path rounds the fp32 activations
 * and the products q * scale to fp16 once each, where the reference's kernels
 * keep fmaf(a, q * scale, acc) in fp32: activations beyond the fp16 range
 * (|a| > 65504) become infinite there; the GEMV variants (Q8 1, Q4 1) take any fp32.
 * variant: the MatMulOpNode `spec` argument, an index into the CUTHIP_OP_MATMUL_Q8 / CUTHIP_OP_MATMUL_Q4 tables,
 * which hold the reference's variant names at the reference's indices (MatMulQ8Variants.generated.h:20-32, default 2;
 * MatMulQ4Variants.generated.h:20-29, default 0; "indices are ABI", MatMulOp.cpp:353-356), or -1 = choose by shape.
 * The reference's shaders collapse onto two kernels here: its tiled shaders (Q8 0, 2, 6; Q4 0) choose by shape as -1
 * does; its GEMV shaders (Q8 1, 3, 4, 5; Q4 1, 2, 3) stream the weights once per 4 rows whatever M is; its
 * cooperative-matrix shaders (Q8 7; Q4 4) dequantize to fp16 and run the dense MFMA GEMM whatever M is (an error if
 * K is not a multiple of 128 or the workspace is too small).  The int8-activation shaders of the reference (Q8 5, 6)
 * run with unquantized activations here.  Any other index: CUTHIP_ERR_UNKNOWN_VARIANT.
 * cuthip_matmul_sep_workspace_bytes sizes the workspace for variant -1 and the table defaults,
 * cuthip_matmul_sep_workspace_bytes_for(op, variant, ...) for an explicit index. */
size_t cuthip_matmul_sep_workspace_bytes(uint32_t M, uint32_t K, uint32_t N);
size_t cuthip_matmul_sep_workspace_bytes_for(int op, int variant, uint32_t M, uint32_t K, uint32_t N);
int cuthip_matmul_q8_sep(const float *A, const int8_t *B, const uint16_t *scales, const float *D, float *C, uint32_t M,
                         uint32_t K, uint32_t N, uint32_t strideA, uint32_t strideB, uint32_t strideC, uint32_t scaleStride,
                         int epilogue, int epilogue_op, int variant, void *workspace, size_t workspace_bytes, void *stream);
int cuthip_matmul_q4_sep(const float *A, const uint8_t *packedB, const uint16_t *scales, const float *D, float *C, uint32_t M,
                         uint32_t K, uint32_t N, uint32_t strideA, uint32_t strideBNpacked, uint32_t strideC,
                         uint32_t scaleStride, int epilogue, int epilogue_op, int affine, int variant, void *workspace,
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
 * (operators/impl/attention/FusedRoPEKVWrite.cu:12-81).  max_positions: rows of the caches and of the tables; the
 * position is read on the device, so it cannot be refused here: a position at or beyond max_positions writes
 * nothing at all (the reference would write past the cache). */
int cuthip_rope_kv_write(const void *q, const void *k, const void *v, int in_dtype, const uint32_t *runtime_params,
                         const float *cos_table, const float *sin_table, void *k_cache, void *v_cache, void *q_out,
                         int q_out_dtype, uint32_t q_dim, uint32_t kv_dim, uint32_t head_dim, uint32_t aligned_kv_dim,
                         uint32_t max_positions, void *stream);

/* Scaled dot-product attention of one token over an fp16 KV cache with GQA:
 * out[h,:] = softmax(scale * q[h,:] . K[0:seq, h/nRep, :]) . V[0:seq, h/nRep, :]
 * (operators/impl/attention/Attention.cu:35-106; head_dim <= 128 as there).
 * workspace: device scratch of cuthip_attn_decode_workspace_bytes(); the call allocates nothing.
 * max_seq_len bounds the launch: any value from the current sequence length up to the cache capacity (at most
 *   65,536).  The call reads max_seq_len positions of K and V whatever runtime_params[1] says (its loads do not wait
 *   for that value: waiting puts a second memory round trip in front of every workgroup, measured + 1.7 us per
 *   launch), so a caller that knows the length on the host passes it rounded up, and a caller that replays a captured
 *   graph captures one per context bucket; a sequence length beyond max_seq_len is attended up to max_seq_len only. */
size_t cuthip_attn_decode_workspace_bytes(uint32_t n_heads, uint32_t head_dim, uint32_t max_seq_len);
int cuthip_attn_decode(const void *q, int q_dtype, const void *k_cache, const void *v_cache, const uint32_t *runtime_params,
                       void *out, int out_dtype, uint32_t n_heads, uint32_t n_kv_heads, uint32_t head_dim,
                       uint32_t aligned_kv_dim, float scale, uint32_t max_seq_len, void *workspace, size_t workspace_bytes,
                       void *stream);

/* The same attention in two halves, so that the second half can ride in the matmul that consumes the attention output
 * (the attention output projection `wo` of interface/runner/llama/llama.cpp:1790-1795) and a decode step has one launch
 * per layer fewer.  cuthip_attn_decode_partial leaves, per query head, cuthip_attn_partial_splits(max_seq_len) <= 8
 * records [max, sum, o[head_dim]] (fp32; o un-normalised: softmax numerators times V over the positions of the split)
 * in `records` (cuthip_attn_partial_bytes() bytes, 8-byte aligned); head_dim must be 128 (CUTHIP_ERR_INVALID
 * otherwise: use cuthip_attn_decode).  cuthip_attn_merge folds such records into out[h,:] (what cuthip_attn_decode
 * does with its own, narrower records); cuthip_matmul_gguf_attn_merge does the same fold while it stages its
 * activations: C = merge(records) . dequant(W)^T with K = n_heads * head_dim, the merged activations rounded to fp16
 * as the attention output of the unfused chain is.  M = 1, the 8-row GEMV only; epilogue, D and the producer fields
 * of `carry` as in cuthip_matmul_gguf_carry (its consumer field sumsq_parts must be NULL: the activations are not a
 * carried norm).  Other arguments as cuthip_attn_decode / cuthip_matmul_gguf. */
uint32_t cuthip_attn_partial_splits(uint32_t max_seq_len);
size_t cuthip_attn_partial_bytes(uint32_t n_heads, uint32_t head_dim, uint32_t max_seq_len);
int cuthip_attn_decode_partial(const void *q, int q_dtype, const void *k_cache, const void *v_cache,
                               const uint32_t *runtime_params, uint32_t n_heads, uint32_t n_kv_heads, uint32_t head_dim,
                               uint32_t aligned_kv_dim, float scale, uint32_t max_seq_len, void *records, size_t records_bytes,
                               void *stream);
int cuthip_attn_merge(const void *records, uint32_t nsplit, uint32_t n_heads, uint32_t head_dim, void *out, int out_dtype,
                      void *stream);
int cuthip_matmul_gguf_attn_merge(int fmt, const void *W, const void *records, uint32_t nsplit, uint32_t n_heads,
                                  uint32_t head_dim, void *C, int c_dtype, uint32_t N, int epilogue, int epilogue_op,
                                  const void *D, const cuthip_norm_carry_t *carry, void *stream);

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

/* RepetitionPenaltyOpNode (operators/impl/sampling/RepetitionPenaltyOp.cpp:9-66, RepetitionPenalty.cu:19-41) on the
 * dense factor vector the runner uploads per token: out[i] = logits[i] > 0 ? logits[i] / factors[i] : logits[i] *
 * factors[i]; all fp32 [n]; out may be logits. */
int cuthip_repetition_penalty(const float *logits, const float *factors, float *out, uint32_t n, void *stream);

/* The runner's "penalty, then arg-max" (interface/runner/llama/llama.cpp:2145-2152) without the dense factor vector:
 * pen_tokens / pen_factors (device, n_pen <= 1024 entries) list the penalised tokens, i.e. the entries of the runner's
 * factor vector that are not 1 (llama.cpp:2566-2592: the recent window at `repeat_penalty`, then end-of-sequence
 * tokens at 1e9); as there, a token listed several times is penalised once, with the factor of its last entry, and
 * ids outside [0, n) are ignored.  The listed logits are rewritten in place (the penalised logits), the index of the
 * first maximum of the result goes to out_index (device).  One workgroup; n_pen = 0 is a plain arg-max. */
int cuthip_argmax_penalized(void *logits, int x_dtype, uint32_t n, const int32_t *pen_tokens, const float *pen_factors,
                            uint32_t n_pen, uint32_t *out_index, void *stream);

/* The output head of a decode step with the sampling folded in: logits[N] = A[K] . dequant(W)^T (batch 1; carry: the
 * consumer side of a carried RMSNorm or NULL), then the penalty and arg-max of cuthip_argmax_penalized.  The matmul's
 * epilogue leaves the winner of every 8 vocabulary rows in the workspace, so the second launch reduces N / 8 pairs
 * instead of scanning N logits (the reference runs LM head, RepetitionPenalty and ReduceArgmax as three dispatches,
 * llama.cpp:2145-2152).  workspace: device, 8-byte aligned, cuthip_matmul_gguf_argmax_workspace_bytes(N) bytes, scratch
 * (without it, or where the matmul's shape does not allow the epilogue, the logits are scanned instead: same result). */
size_t cuthip_matmul_gguf_argmax_workspace_bytes(uint32_t N);
int cuthip_matmul_gguf_argmax(int fmt, const void *W, const void *A, int a_dtype, void *logits, int c_dtype, uint32_t K, uint32_t N,
                              const cuthip_norm_carry_t *carry, const int32_t *pen_tokens, const float *pen_factors,
                              uint32_t n_pen, void *workspace, size_t workspace_bytes, uint32_t *out_index, void *stream);

/* Embedding lookup on a table kept as GGUF blocks (row t = the embedding of token t, as in the file):
 * out[i, 0:dim] = dequant(row token_ids[i]), i < n_ids; token_ids on the device, so a captured graph follows the
 * token it sampled itself.  Bit-identical to cuthip_dequant of that row (fp32, or fp16 with the reference's
 * narrowing); an id >= n_rows yields a zero row.  Replaces Operations::embedding on the dequantized table
 * (interface/runner/llama/llama.cpp:1037-1046) without ever materialising that table. */
int cuthip_embedding_rows(int fmt, const void *blocks, const uint32_t *token_ids, uint32_t n_ids, uint32_t n_rows,
                          uint32_t dim, void *out, int out_dtype, uint32_t out_stride, void *stream);

/* EmbeddingColOpNode (operators/impl/memory/EmbeddingCol.cu:16-44) on the loader's column-wise tables, arguments
 * are its push constants: value of (token t, dim d) at matrix[d * vocab_stride + t]; format 0: fp16 table, format 1:
 * int8 table with fp16 scales[(d >> 5) * scale_stride + t] (the separated Q8_0 tensors of cuthip_prepare_sep).  out
 * fp32 [num_indices, out_stride].  vocab bounds the indices (an index >= vocab yields zeros; the reference reads
 * out of bounds). */
int cuthip_embedding_col(const uint32_t *indices, const void *matrix, const uint16_t *scales, float *out, uint32_t num_indices,
                         uint32_t emb_dim, uint32_t vocab_stride, uint32_t scale_stride, uint32_t out_stride, uint32_t vocab,
                         int format, void *stream);

#ifdef __cplusplus
}
#endif
#endif /* CUT_HIP_H */
