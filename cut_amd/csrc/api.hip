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

// Variant tables, one per operator family; the index of a row is ABI.
static const cuthip_variant_info_t kDequantVariants[] = {
    {"DequantGguf8", 256, 1, 1, 2048, "GGUF block dequant, 8 outputs per lane, 16-byte coalesced stores"},
};
static const cuthip_variant_info_t kMatMulGgufVariants[] = {
    {"MatMulGgufGemvMfma", 64, 4, 8, 32,
     "streaming GEMV / skinny GEMM (M <= 8): 32 weight rows per workgroup, split-K over the waves, "
     "in-register unpack feeding 32x32x16 f16 MFMA, fp32 per-sub-block scaling"},
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
};

static const cuthip_variant_info_t *table(int op, int *count) {
  switch (op) {
  case CUTHIP_OP_DEQUANT: *count = 1; return kDequantVariants;
  case CUTHIP_OP_MATMUL_GGUF:
    *count = (int)(sizeof(kMatMulGgufVariants) / sizeof(kMatMulGgufVariants[0]));
    return kMatMulGgufVariants;
  }
  *count = 0;
  return nullptr;
}

}  // namespace cuthip

namespace cuthip {
bool blaslt_available();
int attn_static_setup();
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
  // open hipBLASLt (variant 5 of the prefill matmul) now: its handle must not be created inside a stream capture,
  // where the first matmul of a caller may well run; absence of the library is not an error
  (void)cuthip::blaslt_available();
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
  return check_hip(hipMemsetAsync(dst, value, bytes, (hipStream_t)stream), "hipMemsetAsync");
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

int cuthip_variant_count(int op) {
  int n;
  table(op, &n);
  return n;
}
int cuthip_variant_default(int op) { return op == CUTHIP_OP_DEQUANT || op == CUTHIP_OP_MATMUL_GGUF ? 0 : CUTHIP_ERR_INVALID; }
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
