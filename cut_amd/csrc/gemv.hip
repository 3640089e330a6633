// Entry point and launch heuristics of the quantized matmul on GGUF blocks.
// The kernels live in gemv_kernel.hpp and are instantiated per format in
// gemv_q8_0.hip, gemv_q4_0.hip, gemv_q4_k.hip and gemv_q6_k.hip.
#include <cstdio>
#include <cstdlib>

#include "gemv_kernel.hpp"
#include "gemv_rows8.hpp"

namespace cuthip {

extern template int launch_fmt<CUTHIP_Q8_0>(GemvParams, hipStream_t);
extern template int launch_fmt<CUTHIP_Q4_0>(GemvParams, hipStream_t);
extern template int launch_fmt<CUTHIP_Q4_K>(GemvParams, hipStream_t);
extern template int launch_fmt<CUTHIP_Q6_K>(GemvParams, hipStream_t);

#define CUTHIP_EXTERN_ROWS8(F) \
  extern template int launch_rows8_fmt<F>(const GemvParams &, hipStream_t); \
  extern template bool rows8_fits<F>(const GemvParams &);
CUTHIP_EXTERN_ROWS8(CUTHIP_Q8_0)
CUTHIP_EXTERN_ROWS8(CUTHIP_Q4_0)
CUTHIP_EXTERN_ROWS8(CUTHIP_Q4_K)
CUTHIP_EXTERN_ROWS8(CUTHIP_Q6_K)
#undef CUTHIP_EXTERN_ROWS8

// Workgroup shape of the rows8 GEMV: split K (kw step ranges per 8-row group)
// while the grid has fewer than ~6 waves per CU and each wave keeps >= 2 steps.
Rows8Shape pick_rows8_shape(int fmt, uint32_t M, uint32_t N, uint32_t nsteps) {
  if (g_tuning.rows8_kw) return Rows8Shape{g_tuning.rows8_rwg, g_tuning.rows8_kw};   // forced by a test or a sweep
  uint32_t groups = (N + 7) / 8;
  int kw = 1;
  if (M > 4) {
    // 5-8 batch rows: every workgroup stages all eight rows of activations (72-80 KB at K = 4096, two workgroups per
    // CU), so fewer, larger workgroups win earlier than at batch 1.  Measured at K = 4096, batch 8, us with
    // (row groups, K ranges) = (1,8) / (1,4) / (2,2) / (8,1):
    //   1024 rows  Q4_K  6.0 /  8.5 /  9.5 / 10.8    Q6_K  8.1 /  9.2 / 10.8 / 15.8    Q8_0  8.1 /  9.2 / 10.2 / 16.9
    //   2048 rows  Q4_K  6.6 /  9.1 /  9.7 / 11.2    Q6_K  8.5 /  9.9 / 11.0 / 15.9    Q8_0  8.5 /  9.6 / 10.3 / 16.9
    //   4096 rows  Q4_K 11.0 / 10.4 / 10.0 / 11.2    Q6_K 14.7 / 12.1 / 11.6 / 15.9    Q8_0 14.7 / 11.9 / 10.7 / 16.9
    //   6144 rows  Q4_K 15.1 / 16.5 / 11.5 / 11.3    Q6_K 20.8 / 18.6 / 14.1 / 16.0    Q8_0 20.6 / 18.8 / 13.3 / 17.0
    //   8192 rows  Q4_K 19.6 / 18.6 / 12.0 / 11.6    Q6_K 26.9 / 21.1 / 14.8 / 16.3    Q8_0 27.6 / 22.3 / 14.7 / 17.7
    //  14336 rows  Q4_K 32.3 / 32.4 / 21.2 / 12.7    Q6_K 49.7 / 39.8 / 27.1 / 19.7    Q8_0 46.9 / 40.5 / 25.7 / 18.8
    const int want = groups <= 256 ? 8 : groups < 512 ? 4 : groups < 1536 ? 2 : 1;
    while (kw < want && nsteps / (uint32_t)(2 * kw) >= 2u) kw *= 2;
    return Rows8Shape{kw == 1 ? 8 : kw == 2 ? 2 : 1, kw};
  }
  // 1536 waves exactly (the q | k | v pair of an 8B model: 6144 rows, split once) still gain from a second split:
  // 5.8 us against 6.2 us for 6144 x 4096
  // (the split into eight only while a wave keeps four steps: 1024 x 4096 Q6_K 4.8 us with four ranges, 6.2 with eight)
  while (kw < 8 && (uint64_t)groups * kw < (kw == 1 ? 1536u : 1537u) && nsteps / (uint32_t)(2 * kw) >= (kw < 4 ? 2u : 4u)) kw *= 2;
  // rows split four ways: two row groups per workgroup share one staging of x (28 KB at K = 14336, which every
  // workgroup reads from L2): 9.8 us against 10.7 us for 4096 x 14336; 4096 x 4096 (16 steps) 5.2 us against 5.4, and
  // 1.3 us per layer of an 8B decode step, whose attention output projection has that shape (batch 1 only: the
  // launch keeps one row group per workgroup for more batch rows); from 4096 rows on: 1024 x 4096 is faster with
  // one row group per workgroup (Q6_K 4.8 us against 5.5)
  // (5120 and 6144 rows again with one: Q8_0 8.7 us against 9.8, Q6_K 7.3 against 8.1, Q4_K 6.2 against 6.3)
  if (kw == 4) return Rows8Shape{groups >= 512 && groups < 640 ? 2 : 1, 4};
  // Q8_0, whose rows are twice as long in bytes, gains from two K ranges on very many rows as well (batch 1, 28672 x
  // 4096: 27.7 us against 30.4 with eight row groups and one range; 128256 x 4096: 105 against 108)
  if (fmt == CUTHIP_Q8_0 && M <= 1 && groups >= 3584) return Rows8Shape{2, 2};
  // eight row groups per workgroup from 28672 rows on (fused gate + up of an 8B model: 15.6 us against 16.0-16.2 us)
  return Rows8Shape{groups >= 3584 ? 8 : 4, kw};
}

#define CUTHIP_EXTERN_KSPLIT(F) \
  extern template int launch_rows8_ksplit<F>(const GemvParams &, float *, uint32_t *, hipStream_t);
CUTHIP_EXTERN_KSPLIT(CUTHIP_Q8_0)
CUTHIP_EXTERN_KSPLIT(CUTHIP_Q4_0)
CUTHIP_EXTERN_KSPLIT(CUTHIP_Q4_K)
CUTHIP_EXTERN_KSPLIT(CUTHIP_Q6_K)
#undef CUTHIP_EXTERN_KSPLIT

// defined with the two-pass GEMM: C = epilogue(sum of the fp32 partial products)
int launch_splitk_reduce(const float *partial, uint32_t ksplit, uint32_t M, uint32_t N, void *C, uint32_t strideC, Epilogue epi,
                         int c_f16, hipStream_t stream);

// The split across workgroups pays where one row group per workgroup would re-stage long activations for few rows:
// batch 2-8, rows of at least 32 steps, and not enough row groups to fill the chip without splitting K.
static bool ksplit_gemv_preferred(int fmt, uint32_t M, uint32_t K, uint32_t N) {
  if (M < 2 || M > 8) return false;
  // whatever the number of weight rows where the unsplit kernel cannot hold the activations in LDS (8 rows of K >= 8192):
  // what would run otherwise is the 32-row fallback
  if (rows8_lds_bytes_rt(fmt, (K + 255) / 256, rows8_batch_class(M)) > kRows8LdsBudget) return true;
  // from 2 batch rows on (4096 x 14336 at two rows: Q4_K 11.6 us against 12.6 unsplit, Q8_0 18.2 against 19.6); Q6_K
  // from 3: its two rows run the dot-product path, unsplit 17.4 us against 18.2
  return M >= (fmt == CUTHIP_Q6_K ? 3u : 2u) && K >= 8192 && (N + 7) / 8 < 1536;
}
static size_t ksplit_gemv_workspace(int fmt, uint32_t M, uint32_t K, uint32_t N) {
  return (size_t)rows8_ksplit_parts(fmt, M, N, (K + 255) / 256) * M * N * sizeof(float);
}

#define CUTHIP_EXTERN_PAIR(FA, FB) \
  extern template bool launch_rows8_pair_fmt<FA, FB>(const GemvParams &, const GemvParams &, hipStream_t, int *);
CUTHIP_EXTERN_PAIR(CUTHIP_Q4_K, CUTHIP_Q4_K)
CUTHIP_EXTERN_PAIR(CUTHIP_Q4_K, CUTHIP_Q6_K)
CUTHIP_EXTERN_PAIR(CUTHIP_Q6_K, CUTHIP_Q4_K)
CUTHIP_EXTERN_PAIR(CUTHIP_Q6_K, CUTHIP_Q6_K)
#undef CUTHIP_EXTERN_PAIR

static int launch_rows8_any(int fmt, const GemvParams &p, hipStream_t stream, bool *taken) {
  *taken = true;
  switch (fmt) {
  case CUTHIP_Q8_0: if (rows8_fits<CUTHIP_Q8_0>(p)) return launch_rows8_fmt<CUTHIP_Q8_0>(p, stream); break;
  case CUTHIP_Q4_0: if (rows8_fits<CUTHIP_Q4_0>(p)) return launch_rows8_fmt<CUTHIP_Q4_0>(p, stream); break;
  case CUTHIP_Q4_K: if (rows8_fits<CUTHIP_Q4_K>(p)) return launch_rows8_fmt<CUTHIP_Q4_K>(p, stream); break;
  default: if (rows8_fits<CUTHIP_Q6_K>(p)) return launch_rows8_fmt<CUTHIP_Q6_K>(p, stream); break;
  }
  *taken = false;
  return CUTHIP_OK;
}

GemvShape pick_gemv_shape(uint32_t N, uint32_t nsteps, int mt) {
  if (g_tuning.gemv_waves) return GemvShape{mt > 8 ? 1 : g_tuning.gemv_kp, g_tuning.gemv_waves};   // forced by a test or a sweep
  // Measured on MI355X at the projection shapes of an 8B model: two parts per
  // wave (16 weight rows per workgroup) win for M <= 2 unless N is huge, and
  // K is split over as many waves as keep >= 2 steps of 256 per part.
  const uint32_t tiles32 = (N + 31) / 32;
  int kp = (mt <= 2 && tiles32 < 1024 && nsteps >= 4) ? 2 : 1;
  const int w_max = mt * kp > 16 ? 4 : 8;
  int w = 1;
  while (w < w_max && nsteps / (uint32_t)(2 * w * kp) >= 2) w *= 2;
  return GemvShape{kp, w};
}

int launch_gemm(int fmt, const void *W, const void *A, int a_f16, void *C, int c_f16, uint32_t M, uint32_t K, uint32_t N,
                uint32_t strideA, uint32_t strideC, Epilogue epi, hipStream_t stream, void *scratch, size_t scratch_bytes);

bool dense_gemm_fits(uint32_t M, uint32_t K, uint32_t N, uint32_t strideA, int a_f16, const void *A);
size_t dense_gemm_workspace(uint32_t M, uint32_t K, uint32_t N, int a_f16);
double dense_cost_us(int fmt, uint32_t M, uint32_t K, uint32_t N);
double single_launch_rows_cost_us(int fmt, uint32_t M, uint32_t K, uint32_t N);
int launch_dense_gemm(int fmt, const void *W, const void *A, int a_f16, void *C, int c_f16, uint32_t M, uint32_t K,
                      uint32_t N, uint32_t strideA, uint32_t strideC, Epilogue epi, void *workspace, hipStream_t stream,
                      int use_blaslt);
uint32_t tiled_gemm_ksplit(uint32_t M, uint32_t K, uint32_t N, size_t scratch_bytes);
bool stream_gemm_fits(int fmt, uint32_t M, uint32_t K, uint32_t N, uint32_t strideA, int a_f16, const void *A);
size_t stream_gemm_scratch(uint32_t M, uint32_t K, uint32_t N);
int launch_stream_gemm(const void *W, const void *A, int a_f16, void *C, int c_f16, uint32_t M, uint32_t K, uint32_t N,
                       uint32_t strideA, uint32_t strideC, Epilogue epi, void *scratch, size_t scratch_bytes, hipStream_t stream);
bool blaslt_available();
size_t dense_f16_workspace(uint32_t M, uint32_t K, uint32_t N, int a_f16);

static int launch_gemv(int fmt, const GemvParams &p, hipStream_t stream) {
  switch (fmt) {
  case CUTHIP_Q8_0: return launch_fmt<CUTHIP_Q8_0>(p, stream);
  case CUTHIP_Q4_0: return launch_fmt<CUTHIP_Q4_0>(p, stream);
  case CUTHIP_Q4_K: return launch_fmt<CUTHIP_Q4_K>(p, stream);
  default: return launch_fmt<CUTHIP_Q6_K>(p, stream);
  }
}

}  // namespace cuthip

// Launch parameters of the GEMV kernels for C[M, strideC] = A[M, strideA] . dequant(W)^T.
static cuthip::GemvParams gemv_params(int fmt, const void *W, const void *A, int a_dtype, void *C, int c_dtype, uint32_t M,
                                      uint32_t K, uint32_t N, uint32_t strideA, uint32_t strideC, const cuthip::Epilogue &epi) {
  using namespace cuthip;
  GemvParams p;
  p.W = reinterpret_cast<const uint8_t *>(W);
  p.A = A;
  p.C = C;
  p.epi = epi;
  p.M = M; p.K = K; p.N = N; p.strideA = strideA; p.strideC = strideC;
  p.nsteps = (K + 255) / 256;
  p.row_bytes = (uint32_t)((uint64_t)(K / fmt_elems(fmt)) * fmt_bytes(fmt));
  p.a_f16 = a_dtype == CUTHIP_F16;
  p.c_f16 = c_dtype == CUTHIP_F16;
  return p;
}

constexpr uint32_t kPassesMaxRows = 40;   // up to here 8-row passes of the decode kernels can beat one tiled GEMM launch

// Costs in microseconds fitted to a sweep over the weight shapes of an 8B model (HIP-graph replay, MI355X): an 8-row
// pass of the decode kernels 6.5 + weight bytes / 4.3 MB (x 1.45 on rows of K >= 8192, x 1.05 for Q6_K: 14336 x 4096 18.6 us,
// 28672 x 4096 34.4; x 1.55 for both), one launch of
// the tiled GEMM on the blocks 62 + weight bytes / 7 MB (its cost is the decode of the whole matrix whatever M is; on
// rows of K >= 8192 it has too few tiles and is never the better one).
static double weight_bytes(int fmt, uint32_t K, uint32_t N) { return (double)N * K / cuthip::fmt_elems(fmt) * cuthip::fmt_bytes(fmt); }
static double passes_cost_us(int fmt, uint32_t M, uint32_t K, uint32_t N) {
  const double f = K >= 8192 ? (fmt == CUTHIP_Q6_K ? 1.55 : 1.45) : (fmt == CUTHIP_Q6_K ? 1.05 : 1.0);
  return ((M + 7) / 8) * (6.5 + weight_bytes(fmt, K, N) / 4.3e6) * f;
}
// The tiled GEMM with its K split over workgroups (scratch memory at hand, so few 128 x 128 tiles that the launch rule
// of gemm.hip splits): 9.5 us for the two launches + 0.66 us (Q4_K; Q6_K x 1.84, Q8_0 x 1.31) per slice of 64 that a
// CU walks (x 0.85 with the 64-row tiles of up to 64 rows) + the partial products written and read back at 6 MB/us.
// 14336 x 4096 Q4_K: 27 us at 32 rows, 29 at 64, 38 at 128, 62 at 256 (unsplit 65 at every M up to 128; 216 on
// K = 14336); 4096 x 1024: 19 at 256 rows, 20 at 512, 28 at 1024.
// Beyond 256 rows only for matrices of fewer than 32 M weights: on 4096 x 14336 at 512 rows the model says 89 us and
// the launch takes 102, against 93 for the two-pass path.
static bool tiled_split_applies(uint32_t M, uint32_t K, uint32_t N, const void *scratch, size_t scratch_bytes) {
  return scratch && (uintptr_t)scratch % 16 == 0 && M > 8 && (M <= 256 || (uint64_t)N * K < 32000000ull) &&
         cuthip::tiled_gemm_ksplit(M, K, N, scratch_bytes) > 1;
}
static double tiled_split_cost_us(int fmt, uint32_t M, uint32_t K, uint32_t N, size_t scratch_bytes) {
  const double f = fmt == CUTHIP_Q6_K ? 1.84 : fmt == CUTHIP_Q8_0 ? 1.31 : fmt == CUTHIP_Q4_0 ? 1.1 : 1.0;
  const double tiles = (double)((M + 127) / 128) * ((N + 127) / 128), slices = (K + 63) / 64;
  const uint32_t ks = cuthip::tiled_gemm_ksplit(M, K, N, scratch_bytes);
  const double tile_rows = M <= 64 ? 0.85 : 1.0;   // 64-row tiles: half the matrix-core work per slice
  return 9.5 + 0.66 * f * tile_rows * tiles * slices / 256.0 + (double)ks * M * N * 8.0 / 6e6;
}
// split: bytes of scratch the tiled GEMM may split K through, 0 = none (or the launch would not split)
static double single_launch_cost_us(int fmt, uint32_t M, uint32_t K, uint32_t N, size_t split) {
  return split ? tiled_split_cost_us(fmt, M, K, N, split) : 62.0 + weight_bytes(fmt, K, N) / 7e6;
}
static bool passes_preferred(int fmt, uint32_t M, uint32_t K, uint32_t N, size_t split) {
  return M > 8 && M <= kPassesMaxRows &&
         ((K >= 8192 && !split) || passes_cost_us(fmt, M, K, N) <= single_launch_cost_us(fmt, M, K, N, split));
}

// Argument checks shared by the matmul entry points: 0 = go on, 1 = empty problem (success), < 0 = error.
static int check_matmul_args(int fmt, const void *W, const void *A, int a_dtype, const void *C, int c_dtype, uint32_t M,
                             uint32_t K, uint32_t N, uint32_t strideA, uint32_t strideC, int epilogue, const void *D) {
  using namespace cuthip;
  if (fmt < CUTHIP_Q8_0 || fmt > CUTHIP_Q6_K) {
    set_error("cuthip_matmul_gguf: unknown format %d", fmt);
    return CUTHIP_ERR_INVALID;
  }
  if ((a_dtype != CUTHIP_F32 && a_dtype != CUTHIP_F16) || (c_dtype != CUTHIP_F32 && c_dtype != CUTHIP_F16)) {
    set_error("cuthip_matmul_gguf: unsupported dtype (a %d, c %d)", a_dtype, c_dtype);
    return CUTHIP_ERR_INVALID;
  }
  if (M == 0 || N == 0) return 1;  // nothing to do
  if (K == 0 || K % fmt_elems(fmt) != 0) {
    set_error("cuthip_matmul_gguf: K (%u) must be a positive multiple of the block size %d", K, fmt_elems(fmt));
    return CUTHIP_ERR_INVALID;
  }
  if (!W || !A || !C) {
    set_error("cuthip_matmul_gguf: null device pointer");
    return CUTHIP_ERR_INVALID;
  }
  if (epilogue < CUTHIP_EPI_NONE || epilogue > CUTHIP_EPI_SWIGLU_PAIRS) {
    set_error("cuthip_matmul_gguf: unknown epilogue %d", epilogue);
    return CUTHIP_ERR_INVALID;
  }
  const uint32_t n_out = epilogue == CUTHIP_EPI_SWIGLU_PAIRS ? N / 2 : N;
  if (strideA < K || strideC < n_out) {
    set_error("cuthip_matmul_gguf: strideA (%u) < K (%u) or strideC (%u) < N (%u)", strideA, K, strideC, n_out);
    return CUTHIP_ERR_INVALID;
  }
  if (epilogue == CUTHIP_EPI_SWIGLU_PAIRS && (N % 2 != 0 || M > 8)) {
    set_error("cuthip_matmul_gguf: the SwiGLU row-pair epilogue needs an even N and M <= 8 (N %u, M %u)", N, M);
    return CUTHIP_ERR_INVALID;
  }
  if (epilogue == CUTHIP_EPI_BINARY && !D) {
    set_error("cuthip_matmul_gguf: binary epilogue needs the operand D");
    return CUTHIP_ERR_INVALID;
  }
  if ((uintptr_t)W % 2 != 0 || (uintptr_t)A % (a_dtype == CUTHIP_F16 ? 2 : 4) != 0) {
    set_error("cuthip_matmul_gguf: misaligned W or A pointer");
    return CUTHIP_ERR_INVALID;
  }
  return 0;
}

static bool stream_preferred(int fmt, uint32_t M, uint32_t K, uint32_t N, uint32_t strideA, int a_f16, const void *A,
                             const void *scratch, size_t scratch_bytes) {
  // (few weight rows: too few workgroups for it; 1024 x 4096 at 16-32 rows 11.6-13.3 us against 10.6-11.2 for the tiled GEMM)
  if (M < 9 || M > 32 || N < 2048 || !cuthip::stream_gemm_fits(fmt, M, K, N, strideA, a_f16, A)) return false;
  const size_t need = cuthip::stream_gemm_scratch(M, K, N);
  return need == 0 || (scratch && (uintptr_t)scratch % 16 == 0 && scratch_bytes >= need);
}

// cuthip_matmul_gguf with optional scratch memory (the workspace of cuthip_matmul_gguf_ws, or none): the tiled GEMM
// splits K through it where it has too few tiles for the chip
static int matmul_gguf_scratch(int fmt, const void *W, const void *A, int a_dtype, void *C, int c_dtype, uint32_t M,
                               uint32_t K, uint32_t N, uint32_t strideA, uint32_t strideC, int epilogue,
                               int epilogue_op, const void *D, int variant, void *stream, void *scratch, size_t scratch_bytes) {
  using namespace cuthip;
  if (int rc = check_matmul_args(fmt, W, A, a_dtype, C, c_dtype, M, K, N, strideA, strideC, epilogue, D))
    return rc > 0 ? CUTHIP_OK : rc;
  if (int rc = check_epilogue_op("cuthip_matmul_gguf", epilogue, epilogue_op)) return rc;
  if (epilogue_op_long(epilogue, epilogue_op)) {   // unfused matmul, then the operator as an elementwise launch
    if (int rc = check_long_epilogue_alias(epilogue, epilogue_op, C, D)) return rc;   // before anything is written
    if (int rc = matmul_gguf_scratch(fmt, W, A, a_dtype, C, c_dtype, M, K, N, strideA, strideC, CUTHIP_EPI_NONE, 0, nullptr,
                                     variant, stream, scratch, scratch_bytes))
      return rc;
    return launch_long_epilogue(C, c_dtype == CUTHIP_F16, M, N, strideC, epilogue, epilogue_op, D,
                                reinterpret_cast<hipStream_t>(stream));
  }
  int nvar = cuthip_variant_count(CUTHIP_OP_MATMUL_GGUF);
  if (variant < -1 || variant >= nvar) {
    set_error("cuthip_matmul_gguf: unknown variant index %d (table has %d)", variant, nvar);
    return CUTHIP_ERR_UNKNOWN_VARIANT;
  }
  uint64_t row_bytes = (uint64_t)(K / fmt_elems(fmt)) * fmt_bytes(fmt);
  if (row_bytes > 0xFFFFFFFFull) {
    set_error("cuthip_matmul_gguf: K too large");
    return CUTHIP_ERR_INVALID;
  }
  // variant table: 0 streaming GEMV (M <= 8; beyond, as -1), 1 skinny passes of 32 rows, 2 LDS-tiled GEMM,
  // 3 the 8-row GEMV, 4 / 5 dequantize + dense GEMM (workspace entry point only), 6 the streaming MFMA kernel (Q4_K, M <= 32)
  Epilogue epi{epilogue, epilogue_op, epilogue == CUTHIP_EPI_BINARY ? D : nullptr};
  if (epilogue == CUTHIP_EPI_SWIGLU_PAIRS && variant != -1 && variant != 3) {
    set_error("cuthip_matmul_gguf: the SwiGLU row-pair epilogue exists in variant 3 only (got variant %d)", variant);
    return CUTHIP_ERR_INVALID;
  }
  if (variant == 4 || variant == 5) {
    set_error("cuthip_matmul_gguf: variants 4 and 5 (dequantize, then dense GEMM) need a workspace: call cuthip_matmul_gguf_ws");
    return CUTHIP_ERR_INVALID;
  }
  // the table's default entry is valid for every M: beyond the 8 rows its GEMV takes it is the choice by shape
  if (variant == 0 && M > 8) variant = -1;
  // 9-32 rows on Q4_K: the streaming MFMA kernel (9-16 rows of 14336 x 4096: 15.8 us against 25 for two 8-row
  // passes; 17-32 rows: 21 us against 30 for the tiled GEMM with K split), wherever the scratch memory it needs
  // for long rows or two activation tiles is at hand
  if (variant == -1 && stream_preferred(fmt, M, K, N, strideA, a_dtype == CUTHIP_F16, A, scratch, scratch_bytes)) variant = 6;
  // variant 6: the streaming MFMA kernel (Q4_K, up to 32 rows); scratch only where K has to be split over workgroups
  if (variant == 6) {
    if (!stream_gemm_fits(fmt, M, K, N, strideA, a_dtype == CUTHIP_F16, A)) {
      set_error("cuthip_matmul_gguf: variant 6 takes Q4_K, M <= 32 and 16-byte aligned rows of A (fmt %d, M %u, K %u)", fmt, M, K);
      return CUTHIP_ERR_INVALID;
    }
    return launch_stream_gemm(W, A, a_dtype == CUTHIP_F16, C, c_dtype == CUTHIP_F16, M, K, N, strideA, strideC, epi, scratch,
                              scratch_bytes, reinterpret_cast<hipStream_t>(stream));
  }
  // 9-40 rows, automatic choice: passes of 8 rows through the decode kernels.  Measured on 14336 x 4096: 14 us per
  // pass, against 69-87 us for the 32-row skinny kernel and 73-80 us for one launch of the tiled GEMM, whose cost
  // is the decode of the whole weight matrix whatever M is.
  if (variant == -1 && passes_preferred(fmt, M, K, N, tiled_split_applies(M, K, N, scratch, scratch_bytes) ? scratch_bytes : 0)) {
    const size_t asz = a_dtype == CUTHIP_F16 ? 2 : 4, csz = c_dtype == CUTHIP_F16 ? 2 : 4;
    for (uint32_t m0 = 0; m0 < M; m0 += 8) {
      const uint8_t *a = reinterpret_cast<const uint8_t *>(A) + (size_t)m0 * strideA * asz;
      uint8_t *c = reinterpret_cast<uint8_t *>(C) + (size_t)m0 * strideC * csz;
      const uint8_t *d = D ? reinterpret_cast<const uint8_t *>(D) + (size_t)m0 * strideC * csz : nullptr;
      if (int rc = matmul_gguf_scratch(fmt, W, a, a_dtype, c, c_dtype, min(8u, M - m0), K, N, strideA, strideC, epilogue,
                                       epilogue_op, d, -1, stream, nullptr, 0))
        return rc;
    }
    return CUTHIP_OK;
  }
  if (variant == 2 || (variant == -1 && M > 8)) {   // 9..40 rows come here when one tiled launch beats the passes
    if ((uint64_t)N * row_bytes > 0xFFFFFFFFFFFFull) {
      set_error("cuthip_matmul_gguf: weight matrix too large");
      return CUTHIP_ERR_INVALID;
    }
    return launch_gemm(fmt, W, A, a_dtype == CUTHIP_F16, C, c_dtype == CUTHIP_F16, M, K, N, strideA, strideC, epi,
                       reinterpret_cast<hipStream_t>(stream), scratch, scratch_bytes);
  }
  GemvParams p = gemv_params(fmt, W, A, a_dtype, C, c_dtype, M, K, N, strideA, strideC, epi);
  // variant 3 (and the automatic choice for M <= 8): 8 rows x 128-byte runs per wave instruction
  if (variant == 3 || (variant == -1 && M <= 8)) {
    bool taken = false;
    int rc = launch_rows8_any(fmt, p, reinterpret_cast<hipStream_t>(stream), &taken);
    if (taken) return rc;
    if (variant == 3 || epilogue == CUTHIP_EPI_SWIGLU_PAIRS) {
      set_error("cuthip_matmul_gguf: variant 3 needs M <= 8 and the activations to fit in LDS (M = %u, K = %u)", M, K);
      return CUTHIP_ERR_INVALID;
    }
    // The batch rows do not fit the 8-row GEMV's LDS budget together (8 rows of K = 8192, 3 of K = 14336) and no scratch
    // memory is at hand for its K split: passes over fewer rows at a time where those beat the 32-row fallback kernel,
    // which is slow on every format but Q4_K.  Measured, us, fallback against passes: 28672 x 8192 at 8 rows Q6_K 248 / 123,
    // Q8_0 196 / 119, Q4_0 125 / 88; 4096 x 14336 at 4 rows Q6_K 80 / 30, Q8_0 61 / 36, at 8 rows Q6_K 87 / 58,
    // Q8_0 70 / 75; Q4_K 4096 x 14336 at 4 rows 21 / 25: its fallback stays.
    if (fmt != CUTHIP_Q4_K) {
      uint32_t rows = 4;
      while (rows >= 1 && (rows >= M || rows8_lds_bytes_rt(fmt, (K + 255) / 256, (int)rows) > kRows8LdsBudget)) rows /= 2;
      if (rows >= 1 && (M + rows - 1) / rows <= (fmt == CUTHIP_Q6_K ? 4u : 2u)) {
        const size_t asz = a_dtype == CUTHIP_F16 ? 2 : 4, csz = c_dtype == CUTHIP_F16 ? 2 : 4;
        for (uint32_t m0 = 0; m0 < M; m0 += rows) {
          const uint8_t *a = reinterpret_cast<const uint8_t *>(A) + (size_t)m0 * strideA * asz;
          uint8_t *c = reinterpret_cast<uint8_t *>(C) + (size_t)m0 * strideC * csz;
          const uint8_t *d = D ? reinterpret_cast<const uint8_t *>(D) + (size_t)m0 * strideC * csz : nullptr;
          if (int rc2 = matmul_gguf_scratch(fmt, W, a, a_dtype, c, c_dtype, min(rows, M - m0), K, N, strideA, strideC, epilogue,
                                            epilogue_op, d, -1, stream, nullptr, 0))
            return rc2;
        }
        return CUTHIP_OK;
      }
    }
  }
  if (epilogue == CUTHIP_EPI_SWIGLU_PAIRS) {
    set_error("cuthip_matmul_gguf: the SwiGLU row-pair epilogue exists in variant 3 only (got variant %d)", variant);
    return CUTHIP_ERR_INVALID;
  }
  return launch_gemv(fmt, p, reinterpret_cast<hipStream_t>(stream));
}

extern "C" int cuthip_matmul_gguf(int fmt, const void *W, const void *A, int a_dtype, void *C, int c_dtype, uint32_t M,
                                  uint32_t K, uint32_t N, uint32_t strideA, uint32_t strideC, int epilogue,
                                  int epilogue_op, const void *D, int variant, void *stream) {
  return matmul_gguf_scratch(fmt, W, A, a_dtype, C, c_dtype, M, K, N, strideA, strideC, epilogue, epilogue_op, D, variant,
                             stream, nullptr, 0);
}
extern "C" {

// Copies the consumer / producer fields of a carried RMSNorm into the launch parameters; false = malformed.
static bool apply_carry(cuthip::GemvParams &p, const cuthip_norm_carry_t *carry, bool producer_allowed) {
  if (!carry) return true;
  const bool producer = carry->next_norm_weight || carry->next_x16 || carry->next_sumsq_parts;
  if (producer && !(producer_allowed && carry->next_norm_weight && carry->next_x16 && carry->next_sumsq_parts)) return false;
  if ((uintptr_t)carry->next_x16 % 2 != 0) return false;
  p.sumsq_parts = carry->sumsq_parts;
  p.eps = carry->eps;
  p.next_norm_w = carry->next_norm_weight;
  p.next_x16 = reinterpret_cast<cuthip::half_t *>(carry->next_x16);
  p.next_sumsq_parts = carry->next_sumsq_parts;
  return true;
}

int cuthip_matmul_gguf_carry(int fmt, const void *W, const void *A, int a_dtype, void *C, int c_dtype, uint32_t K, uint32_t N,
                             int epilogue, int epilogue_op, const void *D, const cuthip_norm_carry_t *carry, void *stream) {
  using namespace cuthip;
  const uint32_t n_out = epilogue == CUTHIP_EPI_SWIGLU_PAIRS ? N / 2 : N;
  if (int rc = check_matmul_args(fmt, W, A, a_dtype, C, c_dtype, 1, K, N, K, n_out, epilogue, D)) return rc > 0 ? CUTHIP_OK : rc;
  if (int rc = check_epilogue_op("cuthip_matmul_gguf_carry", epilogue, epilogue_op)) return rc;
  if (epilogue_op_long(epilogue, epilogue_op)) {
    if (int rc = check_long_epilogue_alias(epilogue, epilogue_op, C, D)) return rc;   // before anything is written
    if (carry && (carry->next_norm_weight || carry->next_x16 || carry->next_sumsq_parts)) {
      set_error("cuthip_matmul_gguf_carry: operator %d runs as a launch of its own after the matmul and cannot feed the "
                "producer side of a carried RMSNorm", epilogue_op);
      return CUTHIP_ERR_INVALID;
    }
    if (int rc = cuthip_matmul_gguf_carry(fmt, W, A, a_dtype, C, c_dtype, K, N, CUTHIP_EPI_NONE, 0, nullptr, carry, stream))
      return rc;
    return launch_long_epilogue(C, c_dtype == CUTHIP_F16, 1, N, N, epilogue, epilogue_op, D, reinterpret_cast<hipStream_t>(stream));
  }
  GemvParams p = gemv_params(fmt, W, A, a_dtype, C, c_dtype, 1, K, N, K, n_out,
                             Epilogue{epilogue, epilogue_op, epilogue == CUTHIP_EPI_BINARY ? D : nullptr});
  if (!apply_carry(p, carry, epilogue != CUTHIP_EPI_SWIGLU_PAIRS)) {
    set_error("cuthip_matmul_gguf_carry: the producer fields (next_norm_weight, next_x16, next_sumsq_parts) come together, "
              "next_x16 2-byte aligned, and not with the SwiGLU row-pair epilogue");
    return CUTHIP_ERR_INVALID;
  }
  bool taken = false;
  int rc = launch_rows8_any(fmt, p, reinterpret_cast<hipStream_t>(stream), &taken);
  if (!taken) {
    set_error("cuthip_matmul_gguf_carry: K = %u does not fit the LDS budget of the 8-row GEMV", K);
    return CUTHIP_ERR_INVALID;
  }
  return rc;
}

int cuthip_matmul_gguf_attn_merge(int fmt, const void *W, const void *records, uint32_t nsplit, uint32_t n_heads,
                                  uint32_t head_dim, void *C, int c_dtype, uint32_t N, int epilogue, int epilogue_op,
                                  const void *D, const cuthip_norm_carry_t *carry, void *stream) {
  using namespace cuthip;
  const uint64_t K64 = (uint64_t)n_heads * head_dim;
  if (fmt < CUTHIP_Q8_0 || fmt > CUTHIP_Q6_K || (c_dtype != CUTHIP_F32 && c_dtype != CUTHIP_F16) || !W || !records || !C ||
      N == 0 || K64 == 0 || K64 > 0xFFFFFFFFull || K64 % fmt_elems(fmt) != 0 || head_dim % 8 != 0 || nsplit == 0 ||
      nsplit > (uint32_t)kMergeMax || (uintptr_t)records % 8 != 0 || (uintptr_t)W % 2 != 0 || epilogue < CUTHIP_EPI_NONE ||
      epilogue > CUTHIP_EPI_BINARY || (epilogue == CUTHIP_EPI_BINARY && !D)) {
    set_error("cuthip_matmul_gguf_attn_merge: bad argument (format %d, heads %u x %u, splits %u (<= %d), N %u, epilogue %d)", fmt,
              n_heads, head_dim, nsplit, kMergeMax, N, epilogue);
    return CUTHIP_ERR_INVALID;
  }
  const uint32_t K = (uint32_t)K64;
  if (int rc = check_epilogue_op("cuthip_matmul_gguf_attn_merge", epilogue, epilogue_op)) return rc;
  if (epilogue_op_long(epilogue, epilogue_op)) {
    set_error("cuthip_matmul_gguf_attn_merge: operator %d runs as a launch of its own after a matmul; not offered here", epilogue_op);
    return CUTHIP_ERR_INVALID;
  }
  if (carry && carry->sumsq_parts) {
    set_error("cuthip_matmul_gguf_attn_merge: the activations are attention records, not a carried RMSNorm (sumsq_parts must be NULL)");
    return CUTHIP_ERR_INVALID;
  }
  GemvParams p = gemv_params(fmt, W, records, CUTHIP_F32, C, c_dtype, 1, K, N, K, N,
                             Epilogue{epilogue, epilogue_op, epilogue == CUTHIP_EPI_BINARY ? D : nullptr});
  if (!apply_carry(p, carry, true)) {
    set_error("cuthip_matmul_gguf_attn_merge: the producer fields (next_norm_weight, next_x16, next_sumsq_parts) come together, "
              "next_x16 2-byte aligned");
    return CUTHIP_ERR_INVALID;
  }
  p.pro = CUTHIP_PRO_ATTN_MERGE;
  p.mrg_nsplit = nsplit;
  p.mrg_head_dim = head_dim;
  bool taken = false;
  int rc = launch_rows8_any(fmt, p, reinterpret_cast<hipStream_t>(stream), &taken);
  if (!taken) {
    set_error("cuthip_matmul_gguf_attn_merge: K = %u does not fit the LDS budget of the 8-row GEMV", K);
    return CUTHIP_ERR_INVALID;
  }
  return rc;
}

}  // extern "C"

namespace cuthip {
int launch_argmax_finish(const ArgmaxPart *parts, void *logits, int x_f16, uint32_t n, const int32_t *pen_tokens,
                         const float *pen_factors, uint32_t n_pen, uint32_t *out_index, hipStream_t stream);
uint32_t max_penalized();
}

extern "C" {

size_t cuthip_matmul_gguf_argmax_workspace_bytes(uint32_t N) { return (size_t)((N + 7) / 8) * sizeof(cuthip::ArgmaxPart); }

int cuthip_matmul_gguf_argmax(int fmt, const void *W, const void *A, int a_dtype, void *logits, int c_dtype, uint32_t K, uint32_t N,
                              const cuthip_norm_carry_t *carry, const int32_t *pen_tokens, const float *pen_factors,
                              uint32_t n_pen, void *workspace, size_t workspace_bytes, uint32_t *out_index, void *stream) {
  using namespace cuthip;
  if (int rc = check_matmul_args(fmt, W, A, a_dtype, logits, c_dtype, 1, K, N, K, N, CUTHIP_EPI_NONE, nullptr)) {
    if (rc > 0) {
      set_error("cuthip_matmul_gguf_argmax: empty vocabulary");
      return CUTHIP_ERR_INVALID;
    }
    return rc;
  }
  if (!out_index || n_pen > max_penalized() || (n_pen && (!pen_tokens || !pen_factors))) {
    set_error("cuthip_matmul_gguf_argmax: out_index missing, or %u penalised tokens without their arrays / beyond %u", n_pen,
              max_penalized());
    return CUTHIP_ERR_INVALID;
  }
  if (carry && (carry->next_norm_weight || carry->next_x16 || carry->next_sumsq_parts)) {
    set_error("cuthip_matmul_gguf_argmax: only the consumer fields of the carried RMSNorm apply here");
    return CUTHIP_ERR_INVALID;
  }
  hipStream_t s = reinterpret_cast<hipStream_t>(stream);
  GemvParams p = gemv_params(fmt, W, A, a_dtype, logits, c_dtype, 1, K, N, K, N, Epilogue{CUTHIP_EPI_NONE, 0, nullptr});
  apply_carry(p, carry, false);
  // the arg-max rides in the matmul's epilogue where the 8-row GEMV runs one K range per wave (any vocabulary-sized N)
  // and the caller brought room for the per-group winners; otherwise the logits are scanned by the second launch
  const bool fused = pick_rows8_shape(fmt, 1, N, p.nsteps).kw == 1 && workspace && (uintptr_t)workspace % 8 == 0 &&
                     workspace_bytes >= cuthip_matmul_gguf_argmax_workspace_bytes(N);
  if (fused) p.argmax_parts = reinterpret_cast<ArgmaxPart *>(workspace);
  bool taken = false;
  int rc = launch_rows8_any(fmt, p, s, &taken);
  if (rc) return rc;
  if (!taken) {   // activations beyond the LDS budget of the 8-row GEMV: the fallback kernel, no carried norm
    if (carry && carry->sumsq_parts) {
      set_error("cuthip_matmul_gguf_argmax: K = %u does not fit the LDS budget of the 8-row GEMV (needed for the carried norm)", K);
      return CUTHIP_ERR_INVALID;
    }
    p.argmax_parts = nullptr;
    if (int rc2 = launch_gemv(fmt, p, s)) return rc2;
  }
  return launch_argmax_finish(p.argmax_parts, logits, c_dtype == CUTHIP_F16, N, pen_tokens, pen_factors, n_pen, out_index, s);
}

int cuthip_matmul_gguf_pair(int fmt_a, const void *Wa, uint32_t Na, void *Ca, int fmt_b, const void *Wb, uint32_t Nb,
                            void *Cb, const void *A, int a_dtype, int c_dtype, uint32_t K,
                            const cuthip_norm_carry_t *carry, const cuthip_rope_append_t *rope, void *stream) {
  using namespace cuthip;
  RopeAppend ra, rb;
  if (rope) {
    const uint32_t hd = rope->head_dim;
    if (!rope->runtime_params || !rope->cos_table || !rope->sin_table || !rope->q_out || !rope->k_cache || !rope->v_cache ||
        hd == 0 || hd % 2 || rope->q_dim == 0 || rope->q_dim % hd || Na <= rope->q_dim || (Na - rope->q_dim) % hd ||
        Nb != Na - rope->q_dim || rope->aligned_kv_dim < Nb ||
        (rope->q_out_dtype != CUTHIP_F32 && rope->q_out_dtype != CUTHIP_F16)) {
      set_error("cuthip_matmul_gguf_pair: bad RoPE / cache-append arguments (q_dim %u, head_dim %u, Na %u, Nb %u)",
                rope ? rope->q_dim : 0u, hd, Na, Nb);
      return CUTHIP_ERR_INVALID;
    }
    ra.mode = 1;
    ra.params = rope->runtime_params;
    ra.cosT = rope->cos_table;
    ra.sinT = rope->sin_table;
    ra.q_out = rope->q_out;
    ra.q_out_f16 = rope->q_out_dtype == CUTHIP_F16;
    ra.k_cache = reinterpret_cast<half_t *>(rope->k_cache);
    ra.v_cache = reinterpret_cast<half_t *>(rope->v_cache);
    ra.q_dim = rope->q_dim;
    ra.head_dim = hd;
    ra.kv_stride = rope->aligned_kv_dim;
    ra.max_pos = rope->max_positions;
    rb = ra;
    rb.mode = 2;
    if (!Ca) Ca = rope->q_out;   // the plain outputs are not written in this mode
    if (!Cb) Cb = rope->q_out;
  }
  if (carry && (carry->next_norm_weight || carry->next_x16 || carry->next_sumsq_parts)) {
    set_error("cuthip_matmul_gguf_pair: only the consumer fields of the carried RMSNorm apply here");
    return CUTHIP_ERR_INVALID;
  }
  if (int rc = check_matmul_args(fmt_a, Wa, A, a_dtype, Ca, c_dtype, 1, K, Na, K, Na, CUTHIP_EPI_NONE, nullptr))
    return rc > 0 ? cuthip_matmul_gguf(fmt_b, Wb, A, a_dtype, Cb, c_dtype, 1, K, Nb, K, Nb, 0, 0, nullptr, -1, stream) : rc;
  if (int rc = check_matmul_args(fmt_b, Wb, A, a_dtype, Cb, c_dtype, 1, K, Nb, K, Nb, CUTHIP_EPI_NONE, nullptr))
    return rc > 0 ? cuthip_matmul_gguf(fmt_a, Wa, A, a_dtype, Ca, c_dtype, 1, K, Na, K, Na, 0, 0, nullptr, -1, stream) : rc;
  auto params = [&](int fmt, const void *W, uint32_t N, void *C, const RopeAppend &r) {
    GemvParams p = gemv_params(fmt, W, A, a_dtype, C, c_dtype, 1, K, N, K, N, Epilogue{CUTHIP_EPI_NONE, 0, nullptr});
    p.rope = r;
    apply_carry(p, carry, false);
    return p;
  };
  if ((uint64_t)(K / fmt_elems(fmt_a)) * fmt_bytes(fmt_a) <= 0xFFFFFFFFull && (uint64_t)Na + Nb <= 0x7FFFFFFFull) {
    const GemvParams pa = params(fmt_a, Wa, Na, Ca, ra), pb = params(fmt_b, Wb, Nb, Cb, rb);
    hipStream_t s = reinterpret_cast<hipStream_t>(stream);
    int rc = CUTHIP_OK;
    bool taken = false;
    if (fmt_a == CUTHIP_Q4_K && fmt_b == CUTHIP_Q4_K) taken = launch_rows8_pair_fmt<CUTHIP_Q4_K, CUTHIP_Q4_K>(pa, pb, s, &rc);
    else if (fmt_a == CUTHIP_Q4_K && fmt_b == CUTHIP_Q6_K) taken = launch_rows8_pair_fmt<CUTHIP_Q4_K, CUTHIP_Q6_K>(pa, pb, s, &rc);
    else if (fmt_a == CUTHIP_Q6_K && fmt_b == CUTHIP_Q4_K) taken = launch_rows8_pair_fmt<CUTHIP_Q6_K, CUTHIP_Q4_K>(pa, pb, s, &rc);
    else if (fmt_a == CUTHIP_Q6_K && fmt_b == CUTHIP_Q6_K) taken = launch_rows8_pair_fmt<CUTHIP_Q6_K, CUTHIP_Q6_K>(pa, pb, s, &rc);
    if (taken) return rc;
  }
  // other formats or shapes: the same two products as two launches
  if (rope) {
    hipStream_t s = reinterpret_cast<hipStream_t>(stream);
    const GemvParams pa = params(fmt_a, Wa, Na, Ca, ra), pb = params(fmt_b, Wb, Nb, Cb, rb);
    bool taken = false;
    int rc = launch_rows8_any(fmt_a, pa, s, &taken);
    if (taken && rc == CUTHIP_OK) rc = launch_rows8_any(fmt_b, pb, s, &taken);
    if (!taken) {
      set_error("cuthip_matmul_gguf_pair: K = %u does not fit the LDS budget of the 8-row GEMV", K);
      return CUTHIP_ERR_INVALID;
    }
    return rc;
  }
  if (carry) {
    if (int rc = cuthip_matmul_gguf_carry(fmt_a, Wa, A, a_dtype, Ca, c_dtype, K, Na, 0, 0, nullptr, carry, stream)) return rc;
    return cuthip_matmul_gguf_carry(fmt_b, Wb, A, a_dtype, Cb, c_dtype, K, Nb, 0, 0, nullptr, carry, stream);
  }
  if (int rc = cuthip_matmul_gguf(fmt_a, Wa, A, a_dtype, Ca, c_dtype, 1, K, Na, K, Na, 0, 0, nullptr, -1, stream)) return rc;
  return cuthip_matmul_gguf(fmt_b, Wb, A, a_dtype, Cb, c_dtype, 1, K, Nb, K, Nb, 0, 0, nullptr, -1, stream);
}

size_t cuthip_matmul_gguf_workspace_bytes(int fmt, uint32_t M, uint32_t K, uint32_t N, int a_dtype) {
  (void)fmt;
  if (cuthip::ksplit_gemv_preferred(fmt, M, K, N)) return cuthip::ksplit_gemv_workspace(fmt, M, K, N);
  return cuthip::dense_gemm_workspace(M, K, N, a_dtype == CUTHIP_F16);
}

int cuthip_matmul_gguf_ws(int fmt, const void *W, const void *A, int a_dtype, void *C, int c_dtype, uint32_t M, uint32_t K,
                          uint32_t N, uint32_t strideA, uint32_t strideC, int epilogue, int epilogue_op, const void *D,
                          int variant, void *workspace, size_t workspace_bytes, void *stream) {
  using namespace cuthip;
  if ((variant != 4 && variant != 5 && variant != -1) || epilogue == CUTHIP_EPI_SWIGLU_PAIRS)
    return matmul_gguf_scratch(fmt, W, A, a_dtype, C, c_dtype, M, K, N, strideA, strideC, epilogue, epilogue_op, D, variant,
                               stream, workspace, workspace ? workspace_bytes : 0);
  if (int rc = check_matmul_args(fmt, W, A, a_dtype, C, c_dtype, M, K, N, strideA, strideC, epilogue, D))
    return rc > 0 ? CUTHIP_OK : rc;
  if (int rc = check_epilogue_op("cuthip_matmul_gguf_ws", epilogue, epilogue_op)) return rc;
  if (epilogue_op_long(epilogue, epilogue_op)) {
    if (int rc = check_long_epilogue_alias(epilogue, epilogue_op, C, D)) return rc;   // before anything is written
    if (int rc = cuthip_matmul_gguf_ws(fmt, W, A, a_dtype, C, c_dtype, M, K, N, strideA, strideC, CUTHIP_EPI_NONE, 0, nullptr,
                                       variant, workspace, workspace_bytes, stream))
      return rc;
    return launch_long_epilogue(C, c_dtype == CUTHIP_F16, M, N, strideC, epilogue, epilogue_op, D,
                                reinterpret_cast<hipStream_t>(stream));
  }
  const int a_f16 = a_dtype == CUTHIP_F16;
  if (variant == -1 && stream_preferred(fmt, M, K, N, strideA, a_f16, A, workspace, workspace ? workspace_bytes : 0))
    return matmul_gguf_scratch(fmt, W, A, a_dtype, C, c_dtype, M, K, N, strideA, strideC, epilogue, epilogue_op, D, 6, stream,
                               workspace, workspace_bytes);
  // Beyond 8 rows, with a workspace at hand: dequantize + dense GEMM where its modelled cost is below that of what
  // would run otherwise (8-row passes up to 40 rows where those beat the single-launch GEMM, else that GEMM); against
  // either only by a margin (a tenth, a twentieth): the models are rough.  From 1024 rows always.
  const bool fits = dense_gemm_fits(M, K, N, strideA, a_f16, A);
  const size_t need = dense_gemm_workspace(M, K, N, a_f16);
  const bool ws_ok = workspace && (uintptr_t)workspace % 256 == 0 && workspace_bytes >= need;
  const size_t split = tiled_split_applies(M, K, N, workspace, workspace ? workspace_bytes : 0) ? workspace_bytes : 0;
  bool dense_first = false;
  if (variant == -1 && M > 8 && fits && ws_ok) {
    const double t4 = dense_cost_us(fmt, M, K, N);
    const double tiled = split ? tiled_split_cost_us(fmt, M, K, N, split) : single_launch_rows_cost_us(fmt, M, K, N);
    dense_first = (M >= 1024 && !split) || (passes_preferred(fmt, M, K, N, split) ? t4 < 0.9 * passes_cost_us(fmt, M, K, N) : t4 < 0.95 * tiled);
  }
  if (variant == -1 && !dense_first && passes_preferred(fmt, M, K, N, split)) {   // 8-row passes, each with the workspace (K split on long rows)
    const size_t asz = a_f16 ? 2 : 4, csz = c_dtype == CUTHIP_F16 ? 2 : 4;
    for (uint32_t m0 = 0; m0 < M; m0 += 8) {
      const uint8_t *a = reinterpret_cast<const uint8_t *>(A) + (size_t)m0 * strideA * asz;
      uint8_t *c = reinterpret_cast<uint8_t *>(C) + (size_t)m0 * strideC * csz;
      const uint8_t *d = D ? reinterpret_cast<const uint8_t *>(D) + (size_t)m0 * strideC * csz : nullptr;
      if (int rc = cuthip_matmul_gguf_ws(fmt, W, a, a_dtype, c, c_dtype, min(8u, M - m0), K, N, strideA, strideC, epilogue,
                                         epilogue_op, d, -1, workspace, workspace_bytes, stream))
        return rc;
    }
    return CUTHIP_OK;
  }
  // batch 3-8 on long rows: the 8-row GEMV with K split across workgroups, partial products in the workspace
  if (variant == -1 && !dense_first && ksplit_gemv_preferred(fmt, M, K, N) && workspace && (uintptr_t)workspace % 16 == 0 &&
      workspace_bytes >= ksplit_gemv_workspace(fmt, M, K, N) && (uintptr_t)A % 16 == 0 && (strideA * (a_f16 ? 2 : 4)) % 16 == 0) {
    const GemvParams p = gemv_params(fmt, W, A, a_dtype, C, c_dtype, M, K, N, strideA, strideC,
                                     Epilogue{CUTHIP_EPI_NONE, 0, nullptr});
    hipStream_t s = reinterpret_cast<hipStream_t>(stream);
    float *partial = reinterpret_cast<float *>(workspace);
    uint32_t parts = 0;
    int rc;
    switch (fmt) {
    case CUTHIP_Q8_0: rc = launch_rows8_ksplit<CUTHIP_Q8_0>(p, partial, &parts, s); break;
    case CUTHIP_Q4_0: rc = launch_rows8_ksplit<CUTHIP_Q4_0>(p, partial, &parts, s); break;
    case CUTHIP_Q4_K: rc = launch_rows8_ksplit<CUTHIP_Q4_K>(p, partial, &parts, s); break;
    default: rc = launch_rows8_ksplit<CUTHIP_Q6_K>(p, partial, &parts, s); break;
    }
    if (rc) return rc;
    Epilogue epi{epilogue, epilogue_op, epilogue == CUTHIP_EPI_BINARY ? D : nullptr};
    return launch_splitk_reduce(partial, parts, M, N, C, strideC, epi, c_dtype == CUTHIP_F16, s);
  }
  if (variant == -1 && !(dense_first && fits && ws_ok))
    return matmul_gguf_scratch(fmt, W, A, a_dtype, C, c_dtype, M, K, N, strideA, strideC, epilogue, epilogue_op, D, -1,
                               stream, workspace, workspace ? workspace_bytes : 0);
  if (!fits) {
    set_error("cuthip_matmul_gguf_ws: variants 4 and 5 need K a multiple of 128, 16-byte aligned rows of A and operands "
              "below 4 GiB (M %u, K %u, N %u, strideA %u)", M, K, N, strideA);
    return CUTHIP_ERR_INVALID;
  }
  if (!ws_ok) {
    set_error("cuthip_matmul_gguf_ws: variants 4 and 5 need a 256-byte aligned workspace of %zu bytes, got %zu", need,
              workspace ? workspace_bytes : (size_t)0);
    return CUTHIP_ERR_INVALID;
  }
  if (variant == 5 && epilogue != CUTHIP_EPI_NONE) {
    set_error("cuthip_matmul_gguf_ws: variant 5 (dequantize, then the vendor GEMM) has no fused epilogue: use variant 4");
    return CUTHIP_ERR_INVALID;
  }
  // the vendor GEMM runs for variant 5 only; the automatic choice never takes it
  const int use_blaslt = variant == 5 ? 1 : 0;
  Epilogue epi{epilogue, epilogue_op, epilogue == CUTHIP_EPI_BINARY ? D : nullptr};
  return launch_dense_gemm(fmt, W, A, a_f16, C, c_dtype == CUTHIP_F16, M, K, N, strideA, strideC, epi, workspace,
                           reinterpret_cast<hipStream_t>(stream), use_blaslt);
}

size_t cuthip_matmul_dense_f16_workspace_bytes(uint32_t M, uint32_t K, uint32_t N, int a_dtype) {
  return cuthip::dense_f16_workspace(M, K, N, a_dtype == CUTHIP_F16);
}

int cuthip_matmul_dense_f16(const void *W16, const void *A, int a_dtype, void *C, int c_dtype, uint32_t M, uint32_t K, uint32_t N,
                            uint32_t strideA, uint32_t strideC, int epilogue, int epilogue_op, const void *D, void *workspace,
                            size_t workspace_bytes, void *stream) {
  using namespace cuthip;
  if (M == 0 || N == 0) return CUTHIP_OK;
  if (!W16 || !A || !C || (a_dtype != CUTHIP_F32 && a_dtype != CUTHIP_F16) || (c_dtype != CUTHIP_F32 && c_dtype != CUTHIP_F16) ||
      strideA < K || strideC < N) {
    set_error("cuthip_matmul_dense_f16: bad argument (null pointer, dtype, or a stride shorter than its row)");
    return CUTHIP_ERR_INVALID;
  }
  if (epilogue != CUTHIP_EPI_NONE && epilogue != CUTHIP_EPI_UNARY && epilogue != CUTHIP_EPI_BINARY) {
    set_error("cuthip_matmul_dense_f16: epilogue %d is not supported here", epilogue);
    return CUTHIP_ERR_INVALID;
  }
  if (epilogue == CUTHIP_EPI_BINARY && !D) {
    set_error("cuthip_matmul_dense_f16: binary epilogue without D");
    return CUTHIP_ERR_INVALID;
  }
  if (int rc = check_epilogue_op("cuthip_matmul_dense_f16", epilogue, epilogue_op)) return rc;
  if (epilogue_op_long(epilogue, epilogue_op)) {
    if (int rc = check_long_epilogue_alias(epilogue, epilogue_op, C, D)) return rc;   // before anything is written
    if (int rc = cuthip_matmul_dense_f16(W16, A, a_dtype, C, c_dtype, M, K, N, strideA, strideC, CUTHIP_EPI_NONE, 0, nullptr,
                                         workspace, workspace_bytes, stream))
      return rc;
    return launch_long_epilogue(C, c_dtype == CUTHIP_F16, M, N, strideC, epilogue, epilogue_op, D,
                                reinterpret_cast<hipStream_t>(stream));
  }
  const int a_f16 = a_dtype == CUTHIP_F16;
  if (!dense_gemm_fits(M, K, N, strideA, a_f16, A) || (uintptr_t)W16 % 256 != 0) {
    set_error("cuthip_matmul_dense_f16: needs K a multiple of 128, 256-byte aligned weights, 16-byte aligned rows of A and "
              "operands below 4 GiB (M %u, K %u, N %u, strideA %u)", M, K, N, strideA);
    return CUTHIP_ERR_INVALID;
  }
  const size_t need = dense_f16_workspace(M, K, N, a_f16);
  if (!workspace || (uintptr_t)workspace % 256 != 0 || workspace_bytes < need) {
    set_error("cuthip_matmul_dense_f16: needs a 256-byte aligned workspace of %zu bytes, got %zu", need,
              workspace ? workspace_bytes : (size_t)0);
    return CUTHIP_ERR_INVALID;
  }
  Epilogue epi{epilogue, epilogue_op, epilogue == CUTHIP_EPI_BINARY ? D : nullptr};
  return launch_dense_gemm(-1, W16, A, a_f16, C, c_dtype == CUTHIP_F16, M, K, N, strideA, strideC, epi, workspace,
                           reinterpret_cast<hipStream_t>(stream), 0);
}

int cuthip_matmul_gguf_pro(int fmt, const void *W, const void *A, int a_dtype, void *C, int c_dtype, uint32_t K, uint32_t N,
                           int epilogue, int epilogue_op, const void *D, int prologue, const float *norm_weight, float eps,
                           void *stream) {
  using namespace cuthip;
  if (prologue == CUTHIP_PRO_NONE)
    return cuthip_matmul_gguf(fmt, W, A, a_dtype, C, c_dtype, 1, K, N, K, N, epilogue, epilogue_op, D, 3, stream);
  if (fmt < CUTHIP_Q8_0 || fmt > CUTHIP_Q6_K || (a_dtype != CUTHIP_F32 && a_dtype != CUTHIP_F16) ||
      (c_dtype != CUTHIP_F32 && c_dtype != CUTHIP_F16) || !W || !A || !C || N == 0 || K == 0 || K % fmt_elems(fmt) != 0 ||
      epilogue < CUTHIP_EPI_NONE || epilogue > CUTHIP_EPI_BINARY || (epilogue == CUTHIP_EPI_BINARY && !D)) {
    set_error("cuthip_matmul_gguf_pro: bad argument (format %d, K %u, N %u, epilogue %d)", fmt, K, N, epilogue);
    return CUTHIP_ERR_INVALID;
  }
  if (int rc = check_epilogue_op("cuthip_matmul_gguf_pro", epilogue, epilogue_op)) return rc;
  if (epilogue_op_long(epilogue, epilogue_op)) {
    if (int rc = check_long_epilogue_alias(epilogue, epilogue_op, C, D)) return rc;   // before anything is written
    if (int rc = cuthip_matmul_gguf_pro(fmt, W, A, a_dtype, C, c_dtype, K, N, CUTHIP_EPI_NONE, 0, nullptr, prologue, norm_weight,
                                        eps, stream))
      return rc;
    return launch_long_epilogue(C, c_dtype == CUTHIP_F16, 1, N, N, epilogue, epilogue_op, D, reinterpret_cast<hipStream_t>(stream));
  }
  if (prologue == CUTHIP_PRO_RMSNORM) {
    if (!norm_weight || (uintptr_t)norm_weight % 16 != 0 || K % 8 != 0 || (uintptr_t)A % 16 != 0) {
      set_error("cuthip_matmul_gguf_pro: the RMSNorm prologue needs a 16-byte aligned fp32 norm_weight[K] and A");
      return CUTHIP_ERR_INVALID;
    }
  } else if (prologue == CUTHIP_PRO_SWIGLU) {
    if (a_dtype != CUTHIP_F16 || K % 8 != 0 || (uintptr_t)A % 16 != 0) {
      set_error("cuthip_matmul_gguf_pro: the SwiGLU prologue takes 16-byte aligned fp16 [gate | up] with K a multiple of 8");
      return CUTHIP_ERR_INVALID;
    }
  } else {
    set_error("cuthip_matmul_gguf_pro: unknown prologue %d", prologue);
    return CUTHIP_ERR_INVALID;
  }
  GemvParams p = gemv_params(fmt, W, A, a_dtype, C, c_dtype, 1, K, N, K, N, Epilogue{epilogue, epilogue_op, D});
  p.pro = prologue;
  p.norm_w = norm_weight;
  p.eps = eps;
  bool taken = false;
  int rc = launch_rows8_any(fmt, p, reinterpret_cast<hipStream_t>(stream), &taken);
  if (!taken) {
    set_error("cuthip_matmul_gguf_pro: K = %u does not fit the LDS budget of the 8-row GEMV", K);
    return CUTHIP_ERR_INVALID;
  }
  return rc;
}

}  // extern "C"

