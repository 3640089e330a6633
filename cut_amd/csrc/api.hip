// Library plumbing behind the C ABI: error reporting, device selection,
// memory / stream / event wrappers and the variant tables.
#include <cstdarg>
#include <cstdio>
#include <cstring>

#include "common.hpp"

namespace cuthip {

static thread_local char g_error[512] = "";

void set_error(const char *fmt, ...) {
  va_list ap;
  va_start(ap, fmt);
  vsnprintf(g_error, sizeof(g_error), fmt, ap);
  va_end(ap);
}

int check_hip(hipError_t e, const char *what) {
  if (e == hipSuccess) return CUTHIP_OK;
  set_error("%s: %s", what, hipGetErrorString(e));
  return CUTHIP_ERR_HIP;
}

int check_epilogue_op(const char *who, int epilogue, int op) {
  if (epilogue_op_known(epilogue, op)) return CUTHIP_OK;
  set_error("%s: operator code %d is not one the %s epilogue implements (the reference's OP_%s_* codes of its "
            "cut_writeOutput)", who, op, epilogue == CUTHIP_EPI_UNARY ? "unary" : "binary",
            epilogue == CUTHIP_EPI_UNARY ? "UNARY" : "BINARY");
  return CUTHIP_ERR_INVALID;
}

__global__ void __launch_bounds__(256) long_epilogue_kernel(void *C, int c_f16, uint32_t M, uint32_t N, uint32_t strideC,
                                                            int epilogue, int op, const void *D) {
  const uint64_t i = (uint64_t)blockIdx.x * 256 + threadIdx.x;
  if (i >= (uint64_t)M * N) return;
  const size_t idx = (size_t)(i / N) * strideC + (size_t)(i % N);
  float v = c_f16 ? (float)reinterpret_cast<const half_t *>(C)[idx] : reinterpret_cast<const float *>(C)[idx];
  if (epilogue == CUTHIP_EPI_UNARY) {
    v = apply_unary_long(op, v);
  } else {
    const float d = c_f16 ? (float)reinterpret_cast<const half_t *>(D)[idx] : reinterpret_cast<const float *>(D)[idx];
    v = apply_binary_long(op, v, d);
  }
  store_plain(C, c_f16, idx, v);
}

int check_long_epilogue_alias(int epilogue, int op, const void *C, const void *D) {
  if (epilogue == CUTHIP_EPI_BINARY && D == C) {
    set_error("binary operator %d is applied after the matmul, in a launch of its own: D must not alias C", op);
    return CUTHIP_ERR_INVALID;
  }
  return CUTHIP_OK;
}

int launch_long_epilogue(void *C, int c_f16, uint32_t M, uint32_t N, uint32_t strideC, int epilogue, int op, const void *D,
                         hipStream_t stream) {
  const uint64_t total = (uint64_t)M * N;
  if (total == 0) return CUTHIP_OK;
  if (int rc = check_long_epilogue_alias(epilogue, op, C, D)) return rc;   // (the entry points check before the matmul)
  hipLaunchKernelGGL(long_epilogue_kernel, dim3((uint32_t)((total + 255) / 256)), dim3(256), 0, stream, C, c_f16, M, N,
                     strideC, epilogue, op, D);
  return check_hip(hipGetLastError(), "epilogue launch");
}

// Variant tables, one per operator family; the index of a row is ABI.
static const cuthip_variant_info_t kDequantVariants[] = {
    {"DequantGguf8", 256, 1, 1, 2048, "GGUF block dequant, 8 outputs per lane, 16-byte coalesced stores"},
};
static const cuthip_variant_info_t kMatMulGgufVariants[] = {
    {"MatMulGgufGemvMfma", 64, 4, 8, 32,
     "streaming GEMV / skinny GEMM (M <= 8): 32 weight rows per workgroup, split-K over the waves, "
     "in-register unpack feeding 32x32x16 f16 MFMA, fp32 per-sub-block scaling; beyond 8 rows of A the choice by shape"},
    {"MatMulGgufSkinnyMfma", 64, 4, 32, 32, "same pipeline with a 32-row activation tile (8 < M <= 32 per pass)"},
    {"MatMulGgufGemmLds", 256, 1, 128, 128,
     "prefill GEMM: weights dequantized to fp16 tiles in LDS, 32x32x16 f16 MFMA, fp32 accumulate"},
    {"MatMulGgufGemvRows8", 64, 4, 8, 8,
     "decode GEMV (M <= 8): 8 weight rows x 128-byte runs per wave instruction, four 64-element pieces per row as "
     "MFMA columns, register ring of loads, no cross-wave reduction unless K is split"},
    {"MatMulGgufDequantGemm", 256, 1, 256, 256,
     "large-M prefill in two launches: the weights are dequantized once to an fp16 workspace, then a dense fp16 MFMA GEMM "
     "with LDS-direct loads and 128x128 accumulators per wave (needs cuthip_matmul_gguf_ws)"},
    {"MatMulGgufDequantBlasLt", 256, 1, 256, 256,
     "large-M prefill in two launches: the weights are dequantized once to an fp16 workspace, then hipBLASLt's dense fp16 "
     "GEMM (opened at run time; no fused epilogue; needs cuthip_matmul_gguf_ws)"},
    {"MatMulGgufStreamMfma", 256, 1, 16, 64,
     "5..32 rows of A on Q4_K: 16 weight rows per wave, nibbles and 6-bit scales multiplied as integers into fp16 "
     "subnormals, 16x16x32 f16 MFMA chains per super-block, activations staged once per workgroup (long K split over "
     "workgroups through the workspace of cuthip_matmul_gguf_ws)"},
};

// Separated-layout matmuls: the reference's tables, name for name and index for index
// (operators/impl/matmul/MatMulQ8Variants.generated.h:20-32, MatMulQ4Variants.generated.h:20-29); the last column
// says which of this library's two code paths serves the entry.
static const cuthip_variant_info_t kMatMulQ8Variants[] = {
    {"MatMulQ8T16R4x4", 16, 16, 64, 64, "Q8 T16 R4x4 -> choice by shape (streaming kernel below 32 rows, dequant + MFMA GEMM from 32)"},
    {"MatMulQ8Gemv", 256, 1, 1, 256, "Q8 GEMV (M=1 vector) -> column-major streaming kernel"},
    {"MatMulQ8VecT16R4x4", 16, 16, 64, 64, "Q8 Vec4 T16 R4x4 -> choice by shape"},
    {"MatMulQ8GemvKPar", 32, 1, 1, 4, "Q8 GEMV K-parallel -> column-major streaming kernel"},
    {"MatMulQ8GemvKPar8", 32, 8, 1, 8, "Q8 GEMV (M=1, 8 cols/WG, split-K over 8 waves) -> column-major streaming kernel"},
    {"MatMulQ8GemvDot", 32, 1, 1, 4, "Q8 GEMV dotPacked4x8EXT -> column-major streaming kernel, activations not quantized"},
    {"MatMulQ8TiledDot", 256, 1, 32, 64, "Q8 TiledDot dotPacked4x8EXT -> choice by shape, activations not quantized"},
    {"MatMulQ8CoopMatTiled", 128, 1, 32, 32, "Q8 CoopMat 2x2 Tiled -> dequant to fp16, then the dense MFMA GEMM"},
};
static const cuthip_variant_info_t kMatMulQ4Variants[] = {
    {"MatMulQ4T16R4x4", 16, 16, 64, 64, "Q4 T16 R4x4 -> choice by shape (streaming kernel below 32 rows, dequant + MFMA GEMM from 32)"},
    {"MatMulQ4Gemv", 256, 1, 1, 256, "Q4 GEMV (M=1 vector) -> column-major streaming kernel"},
    {"MatMulQ4GemvKPar", 32, 1, 1, 4, "Q4 GEMV K-parallel -> column-major streaming kernel"},
    {"MatMulQ4GemvKPar8", 32, 8, 1, 8, "Q4 GEMV (M=1, 8 cols/WG, split-K over 8 waves) -> column-major streaming kernel"},
    {"MatMulQ4CoopMatTiled", 128, 1, 32, 32, "Q4 CoopMat 2x2 Tiled -> dequant to fp16, then the dense MFMA GEMM"},
};

static const cuthip_variant_info_t *table(int op, int *count) {
  switch (op) {
  case CUTHIP_OP_DEQUANT: *count = 1; return kDequantVariants;
  case CUTHIP_OP_MATMUL_GGUF:
    *count = (int)(sizeof(kMatMulGgufVariants) / sizeof(kMatMulGgufVariants[0]));
    return kMatMulGgufVariants;
  case CUTHIP_OP_MATMUL_Q8:
    *count = (int)(sizeof(kMatMulQ8Variants) / sizeof(kMatMulQ8Variants[0]));
    return kMatMulQ8Variants;
  case CUTHIP_OP_MATMUL_Q4:
    *count = (int)(sizeof(kMatMulQ4Variants) / sizeof(kMatMulQ4Variants[0]));
    return kMatMulQ4Variants;
  }
  *count = 0;
  return nullptr;
}

// A launch that only loads: every thread xors 16-byte loads (four in flight), one dword per workgroup is stored so
// that the loads cannot be dropped.  The measuring stick for what a launch of a given size can reach when it does
// nothing but read (cuthip_read_probe).
__global__ void __launch_bounds__(256) read_probe_kernel(const u32x4 *src, size_t nvec, uint32_t *sink) {
  const size_t stride = (size_t)gridDim.x * 256 * 4;
  u32x4 acc{0, 0, 0, 0};
  for (size_t i = (size_t)blockIdx.x * 1024 + threadIdx.x; i < nvec; i += stride) {
    u32x4 v[4];
#pragma unroll
    for (int u = 0; u < 4; ++u) v[u] = __builtin_nontemporal_load(src + (i + u * 256 < nvec ? i + u * 256 : i));
#pragma unroll
    for (int u = 0; u < 4; ++u) acc ^= v[u];
  }
  uint32_t r = acc.x ^ acc.y ^ acc.z ^ acc.w;
#pragma unroll
  for (int o = 32; o > 0; o >>= 1) r ^= __shfl_xor(r, o);
  if ((threadIdx.x & 63) == 0) sink[(blockIdx.x * 4 + threadIdx.x / 64) & 0xFFFF] = r;
}

// Fills the LDS of every CU with a pattern (cuthip_debug_fill_lds): LDS keeps what the last workgroup left in it, so
// a kernel that reads a location it never wrote gives results that depend on what ran before; the tests run every
// operator behind different patterns and ask for identical bits.
__global__ void __launch_bounds__(1024) fill_lds_kernel(uint32_t pattern, uint32_t ndw, uint32_t *sink) {
  extern __shared__ uint32_t fill_lds[];
  for (uint32_t i = threadIdx.x; i < ndw; i += 1024) fill_lds[i] = pattern;
  __syncthreads();
  if (fill_lds[(threadIdx.x * 37u) % ndw] != pattern && sink) sink[0] = 1;   // never true: keeps the stores
}

}  // namespace cuthip

namespace cuthip {
bool blaslt_available();
int attn_static_setup();
Tuning g_tuning;

// One key of the launch-shape overrides; value nullptr or "" restores the library's own choice for that key.
static int set_tuning_key(const char *key, const char *value) {
  const bool clear = !value || !value[0];
  int a = 0, b = 0, c = 1;
  if (!strcmp(key, "rows8_shape")) {
    if (clear) { g_tuning.rows8_rwg = g_tuning.rows8_kw = 0; return CUTHIP_OK; }
    if (sscanf(value, "%d,%d", &a, &b) == 2 && a >= 1 && (b == 1 || b == 2 || b == 4 || b == 8)) {
      g_tuning.rows8_rwg = a; g_tuning.rows8_kw = b; return CUTHIP_OK;
    }
  } else if (!strcmp(key, "gemv_shape")) {
    if (clear) { g_tuning.gemv_kp = g_tuning.gemv_waves = 0; return CUTHIP_OK; }
    if (sscanf(value, "%d,%d", &a, &b) == 2 && (a == 1 || a == 2) && (b == 1 || b == 2 || b == 4 || b == 8)) {
      g_tuning.gemv_kp = a; g_tuning.gemv_waves = b; return CUTHIP_OK;
    }
  } else if (!strcmp(key, "gemm_ksplit")) {
    if (clear) { g_tuning.gemm_ksplit = 0; return CUTHIP_OK; }
    if (sscanf(value, "%d", &a) == 1 && a >= 1 && a <= 16) { g_tuning.gemm_ksplit = a; return CUTHIP_OK; }
  } else if (!strcmp(key, "dense_tile")) {
    if (clear) { g_tuning.dense_bm = g_tuning.dense_bn = 0; g_tuning.dense_ks = 1; return CUTHIP_OK; }
    const int got = sscanf(value, "%d,%d,%d", &a, &b, &c);
    if (got >= 2 && ((b == 256 && (a == 256 || a == 128)) || (b == 448 && a == 128) || (b == 224 && a == 256)) &&
        (c == 1 || c == 2 || c == 4 || c == 8)) {
      g_tuning.dense_bm = a; g_tuning.dense_bn = b; g_tuning.dense_ks = c; return CUTHIP_OK;
    }
  } else if (!strcmp(key, "dense_mfma16")) {
    if (clear) { g_tuning.dense_mfma16 = 1; return CUTHIP_OK; }
    if (sscanf(value, "%d", &a) == 1) { g_tuning.dense_mfma16 = a != 0; return CUTHIP_OK; }
  } else if (!strcmp(key, "dense_pf")) {
    if (clear) { g_tuning.dense_pf = -1; return CUTHIP_OK; }
    if (sscanf(value, "%d", &a) == 1 && a >= 0) { g_tuning.dense_pf = a; return CUTHIP_OK; }
  } else {
    set_error("cuthip_set_tuning: unknown key '%s' (rows8_shape, gemv_shape, gemm_ksplit, dense_tile, dense_mfma16, dense_pf)", key);
    return CUTHIP_ERR_INVALID;
  }
  set_error("cuthip_set_tuning: value '%s' is not valid for key '%s'", value, key);
  return CUTHIP_ERR_INVALID;
}
}
using namespace cuthip;

extern "C" {

const char *cuthip_last_error(void) { return g_error; }

int cuthip_init(int device) {
  int n = 0;
  hipError_t e = hipGetDeviceCount(&n);
  if (e != hipSuccess || n <= 0) {
    set_error("cuthip_init: no HIP device (%s)", e == hipSuccess ? "count is 0" : hipGetErrorString(e));
    return CUTHIP_ERR_NO_DEVICE;
  }
  if (device < 0 || device >= n) {
    set_error("cuthip_init: device %d out of range (have %d)", device, n);
    return CUTHIP_ERR_INVALID;
  }
  if (int rc = check_hip(hipSetDevice(device), "hipSetDevice")) return rc;
  hipDeviceProp_t p;
  if (int rc = check_hip(hipGetDeviceProperties(&p, device), "hipGetDeviceProperties")) return rc;
  if (strncmp(p.gcnArchName, "gfx950", 6) != 0) {
    set_error("cuthip_init: device %d is %s; this library is built for gfx950 only", device, p.gcnArchName);
    return CUTHIP_ERR_NO_DEVICE;
  }
  // the launch-shape overrides of the environment are taken over here, once: no launcher calls getenv.  A value that
  // does not parse is ignored, as an unset variable is.
  static const struct { const char *env, *key; } kEnv[] = {
      {"CUT_HIP_ROWS8_SHAPE", "rows8_shape"}, {"CUT_HIP_GEMV_SHAPE", "gemv_shape"},   {"CUT_HIP_GEMM_KSPLIT", "gemm_ksplit"},
      {"CUT_HIP_DENSE_TILE", "dense_tile"},   {"CUT_HIP_DENSE_MFMA16", "dense_mfma16"}, {"CUT_HIP_DENSE_PF", "dense_pf"}};
  for (const auto &e : kEnv)
    if (const char *v = getenv(e.env)) (void)set_tuning_key(e.key, v);
  // device address of the built-in attention scratch on this device (cuthip_attn_decode_static)
  return cuthip::attn_static_setup();
}

int cuthip_device_info(cuthip_device_info_t *info) {
  if (!info) {
    set_error("cuthip_device_info: null argument");
    return CUTHIP_ERR_INVALID;
  }
  int dev = 0;
  if (int rc = check_hip(hipGetDevice(&dev), "hipGetDevice")) return rc;
  hipDeviceProp_t p;
  if (int rc = check_hip(hipGetDeviceProperties(&p, dev), "hipGetDeviceProperties")) return rc;
  memset(info, 0, sizeof(*info));
  snprintf(info->name, sizeof(info->name), "%s", p.name);
  snprintf(info->arch, sizeof(info->arch), "%s", p.gcnArchName);
  info->compute_units = p.multiProcessorCount;
  info->wave_size = p.warpSize;
  info->lds_bytes_per_workgroup = (int)p.sharedMemPerBlock;
  info->clock_khz = p.clockRate;
  info->memory_clock_khz = p.memoryClockRate;
  info->memory_bus_bits = p.memoryBusWidth;
  info->hbm_bytes = p.totalGlobalMem;
  info->l2_bytes = (size_t)p.l2CacheSize;
  return CUTHIP_OK;
}

int cuthip_malloc(void **device_ptr, size_t bytes) {
  if (!device_ptr) {
    set_error("cuthip_malloc: null argument");
    return CUTHIP_ERR_INVALID;
  }
  return check_hip(hipMalloc(device_ptr, bytes), "hipMalloc");
}
int cuthip_free(void *device_ptr) { return check_hip(hipFree(device_ptr), "hipFree"); }

int cuthip_memcpy_h2d(void *dst, const void *src, size_t bytes, void *stream) {
  if (!stream) return check_hip(hipMemcpy(dst, src, bytes, hipMemcpyHostToDevice), "hipMemcpy h2d");
  return check_hip(hipMemcpyAsync(dst, src, bytes, hipMemcpyHostToDevice, (hipStream_t)stream), "hipMemcpyAsync h2d");
}
int cuthip_memcpy_d2h(void *dst, const void *src, size_t bytes, void *stream) {
  if (!stream) return check_hip(hipMemcpy(dst, src, bytes, hipMemcpyDeviceToHost), "hipMemcpy d2h");
  return check_hip(hipMemcpyAsync(dst, src, bytes, hipMemcpyDeviceToHost, (hipStream_t)stream), "hipMemcpyAsync d2h");
}
int cuthip_memcpy_d2d(void *dst, const void *src, size_t bytes, void *stream) {
  return check_hip(hipMemcpyAsync(dst, src, bytes, hipMemcpyDeviceToDevice, (hipStream_t)stream), "hipMemcpyAsync d2d");
}
int cuthip_memset(void *dst, int value, size_t bytes, void *stream) {
  // not under capture: memset nodes have given wrong results on replays of a graph on this part
  hipStreamCaptureStatus st = hipStreamCaptureStatusNone;
  if (stream && hipStreamIsCapturing((hipStream_t)stream, &st) == hipSuccess && st != hipStreamCaptureStatusNone) {
    set_error("cuthip_memset: the stream is capturing; clear the memory before the capture or with a kernel of the sequence");
    return CUTHIP_ERR_INVALID;
  }
  return check_hip(hipMemsetAsync(dst, value, bytes, (hipStream_t)stream), "hipMemsetAsync");
}

int cuthip_set_tuning(const char *key, const char *value) {
  if (!key) {
    set_error("cuthip_set_tuning: null key");
    return CUTHIP_ERR_INVALID;
  }
  return set_tuning_key(key, value);
}

int cuthip_stream_create(void **stream) {
  if (!stream) {
    set_error("cuthip_stream_create: null argument");
    return CUTHIP_ERR_INVALID;
  }
  hipStream_t s;
  int rc = check_hip(hipStreamCreate(&s), "hipStreamCreate");  // default priority
  *stream = rc ? nullptr : (void *)s;
  return rc;
}
int cuthip_stream_destroy(void *stream) { return check_hip(hipStreamDestroy((hipStream_t)stream), "hipStreamDestroy"); }
int cuthip_stream_sync(void *stream) { return check_hip(hipStreamSynchronize((hipStream_t)stream), "hipStreamSynchronize"); }

int cuthip_event_create(void **event) {
  if (!event) {
    set_error("cuthip_event_create: null argument");
    return CUTHIP_ERR_INVALID;
  }
  hipEvent_t e;
  int rc = check_hip(hipEventCreate(&e), "hipEventCreate");
  *event = rc ? nullptr : (void *)e;
  return rc;
}
int cuthip_event_destroy(void *event) { return check_hip(hipEventDestroy((hipEvent_t)event), "hipEventDestroy"); }
int cuthip_event_record(void *event, void *stream) {
  return check_hip(hipEventRecord((hipEvent_t)event, (hipStream_t)stream), "hipEventRecord");
}
int cuthip_event_sync(void *event) { return check_hip(hipEventSynchronize((hipEvent_t)event), "hipEventSynchronize"); }
int cuthip_event_elapsed_ms(void *start, void *stop, float *ms) {
  return check_hip(hipEventElapsedTime(ms, (hipEvent_t)start, (hipEvent_t)stop), "hipEventElapsedTime");
}

int cuthip_read_probe(const void *src, size_t bytes, uint32_t *sink, void *stream) {
  if (!src || !sink || bytes < 16 || (uintptr_t)src % 16 != 0) {
    set_error("cuthip_read_probe: needs a 16-byte aligned buffer of at least 16 bytes and a sink of 65,536 dwords");
    return CUTHIP_ERR_INVALID;
  }
  const size_t nvec = bytes / 16;
  size_t blocks = (nvec + 1023) / 1024;
  if (blocks > 256 * 16) blocks = 256 * 16;   // 16 workgroups per CU walk the rest
  hipLaunchKernelGGL(read_probe_kernel, dim3((uint32_t)blocks), dim3(256), 0, (hipStream_t)stream,
                     reinterpret_cast<const u32x4 *>(src), nvec, sink);
  return check_hip(hipGetLastError(), "read probe launch");
}

int cuthip_debug_fill_lds(uint32_t pattern, void *stream) {
  constexpr uint32_t kBytes = 160 * 1024;
  static bool attr = false;   // (single-threaded callers, as everywhere in this library)
  if (!attr) {
    if (int rc = check_hip(hipFuncSetAttribute(reinterpret_cast<const void *>(fill_lds_kernel),
                                               hipFuncAttributeMaxDynamicSharedMemorySize, kBytes), "hipFuncSetAttribute"))
      return rc;
    attr = true;
  }
  // one workgroup fills the whole LDS of the CU it lands on; four rounds over the 256 CUs
  hipLaunchKernelGGL(fill_lds_kernel, dim3(1024), dim3(1024), kBytes, (hipStream_t)stream, pattern, kBytes / 4, (uint32_t *)nullptr);
  return check_hip(hipGetLastError(), "fill lds launch");
}

// ---- capture and replay of a launch sequence (the reusable command buffer of the reference, CudaCommandBuffer.cpp:261-285)
struct CapturedGraph {
  hipGraph_t graph = nullptr;
  hipGraphExec_t exec = nullptr;
};

int cuthip_graph_begin_capture(void *stream) {
  if (!stream) {
    set_error("cuthip_graph_begin_capture: capture needs a stream of its own (not the default stream)");
    return CUTHIP_ERR_INVALID;
  }
  return check_hip(hipStreamBeginCapture((hipStream_t)stream, hipStreamCaptureModeThreadLocal), "hipStreamBeginCapture");
}

int cuthip_graph_end_capture(void *stream, void **graph) {
  if (!stream || !graph) {
    set_error("cuthip_graph_end_capture: null argument");
    return CUTHIP_ERR_INVALID;
  }
  *graph = nullptr;
  CapturedGraph g;
  if (int rc = check_hip(hipStreamEndCapture((hipStream_t)stream, &g.graph), "hipStreamEndCapture")) return rc;
  if (!g.graph) {
    set_error("cuthip_graph_end_capture: the capture was invalidated (a call that is not allowed under capture was made)");
    return CUTHIP_ERR_HIP;
  }
  if (int rc = check_hip(hipGraphInstantiate(&g.exec, g.graph, nullptr, nullptr, 0), "hipGraphInstantiate")) {
    (void)hipGraphDestroy(g.graph);
    return rc;
  }
  *graph = new CapturedGraph(g);
  return CUTHIP_OK;
}

int cuthip_graph_launch(void *graph, void *stream) {
  if (!graph) {
    set_error("cuthip_graph_launch: null graph");
    return CUTHIP_ERR_INVALID;
  }
  return check_hip(hipGraphLaunch(static_cast<CapturedGraph *>(graph)->exec, (hipStream_t)stream), "hipGraphLaunch");
}

int cuthip_graph_destroy(void *graph) {
  if (!graph) return CUTHIP_OK;
  CapturedGraph *g = static_cast<CapturedGraph *>(graph);
  int rc = check_hip(hipGraphExecDestroy(g->exec), "hipGraphExecDestroy");
  int rc2 = check_hip(hipGraphDestroy(g->graph), "hipGraphDestroy");
  delete g;
  return rc ? rc : rc2;
}

int cuthip_epilogue_op_supported(int epilogue, int op) {
  return (epilogue == CUTHIP_EPI_UNARY || epilogue == CUTHIP_EPI_BINARY) && epilogue_op_known(epilogue, op) ? 1 : 0;
}

int cuthip_variant_count(int op) {
  int n;
  table(op, &n);
  return n;
}
int cuthip_variant_default(int op) {
  switch (op) {
  case CUTHIP_OP_DEQUANT: case CUTHIP_OP_MATMUL_GGUF: case CUTHIP_OP_MATMUL_Q4: return 0;   // kMatMulQ4DefaultVariant = 0
  case CUTHIP_OP_MATMUL_Q8: return 2;                                                         // kMatMulQ8DefaultVariant = 2
  }
  set_error("cuthip_variant_default: no operator family %d", op);
  return CUTHIP_ERR_INVALID;
}
int cuthip_variant_available(int op, int index) {
  int n;
  if (!table(op, &n) || index < 0 || index >= n) {
    set_error("cuthip_variant_available: no variant %d in operator family %d", index, op);
    return CUTHIP_ERR_UNKNOWN_VARIANT;
  }
  if (op == CUTHIP_OP_MATMUL_GGUF && index == 5) return blaslt_available() ? 1 : 0;
  return 1;
}
int cuthip_variant_info(int op, int index, cuthip_variant_info_t *info) {
  int n;
  const cuthip_variant_info_t *t = table(op, &n);
  if (!t || !info || index < 0 || index >= n) {
    set_error("cuthip_variant_info: no variant %d in operator family %d", index, op);
    return CUTHIP_ERR_UNKNOWN_VARIANT;
  }
  *info = t[index];
  return CUTHIP_OK;
}
int cuthip_variant_lookup(int op, const char *name) {
  int n;
  const cuthip_variant_info_t *t = table(op, &n);
  for (int i = 0; t && name && i < n; ++i)
    if (strcmp(t[i].name, name) == 0) return i;
  set_error("cuthip_variant_lookup: unknown variant '%s' in operator family %d", name ? name : "(null)", op);
  return CUTHIP_ERR_UNKNOWN_VARIANT;
}

}  // extern "C"
