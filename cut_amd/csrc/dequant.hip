// Block dequantization Q8_0 / Q4_0 / Q4_K / Q6_K -> fp32 or fp16 on gfx950.
//
// Supersedes the reference's one-thread-per-element DequantQ4K.cu / DequantQ6K.cu
// (operators/impl/dequant) and the host loops of gguf_reader.cpp:541-850.
// Each lane produces 8 consecutive output elements: one 8-byte load of quants
// (plus the block header, shared through the L1 by the lanes of a block),
// unpack in registers, one 16-byte (fp16) or two 16-byte (fp32) coalesced
// non-temporal stores.  The kernel is HBM-bound and write-dominated:
// 2 B (fp16) or 4 B (fp32) out per element against 0.56 - 1.06 B in.
//
// Bit-exactness against the CPU reference rests on evaluating the same
// expressions in the same order: Q8_0/Q4_0 one exact product, Q6_K two exact
// products (d*sc)*q, Q4_K two exact products and one rounded subtraction
// (an FMA contraction of d1*q - dm1 rounds identically because d1*q is exact).
#include "common.hpp"

namespace cuthip {

template <int FMT> struct Deq8;

// Q8_0: [d:f16][q:32 x i8]; out = float(q) * d  (gguf_reader.cpp:826-850)
template <> struct Deq8<CUTHIP_Q8_0> {
  __device__ static bool run(const uint8_t *row, uint32_t col, float o[8]) {
    const uint8_t *blk = row + (size_t)(col >> 5) * 34;
    uint32_t dh = ld_u16(blk);
    float d = f16bits_to_f32(dh);
    u32x2 w = ld_u32x2(blk + 2 + (col & 31));
#pragma unroll
    for (int i = 0; i < 8; ++i) {
      uint32_t word = i < 4 ? w.x : w.y;
      int q = (int)(int8_t)((word >> (8 * (i & 3))) & 0xFF);
      o[i] = (float)q * d;
    }
    return f16bits_finite(dh);
  }
};

// Q4_0: [d:f16][qs:16]; element j<16 low nibble of qs[j], j>=16 high nibble of
// qs[j-16]; out = float(nib - 8) * d  (gguf_reader.cpp:541-572)
template <> struct Deq8<CUTHIP_Q4_0> {
  __device__ static bool run(const uint8_t *row, uint32_t col, float o[8]) {
    const uint8_t *blk = row + (size_t)(col >> 5) * 18;
    uint32_t dh = ld_u16(blk);
    float d = f16bits_to_f32(dh);
    uint32_t e = col & 31;
    u32x2 w = ld_u32x2(blk + 2 + (e & 15));
    uint32_t sh = (e >> 4) * 4;
#pragma unroll
    for (int i = 0; i < 8; ++i) {
      uint32_t word = i < 4 ? w.x : w.y;
      int q = (int)((word >> (8 * (i & 3) + sh)) & 15) - 8;
      o[i] = (float)q * d;
    }
    return f16bits_finite(dh);
  }
};

// Q4_K: [d][dmin][scales:12][qs:128]; out = (d*sc)*nib - dmin*m
// (gguf_reader.cpp:678-724)
template <> struct Deq8<CUTHIP_Q4_K> {
  __device__ static bool run(const uint8_t *row, uint32_t col, float o[8]) {
    const uint8_t *blk = row + (size_t)(col >> 8) * 144;
    u32x4 hdr = ld_u32x4(blk);
    uint32_t e = col & 255, g = e >> 6, r = e & 63, hi = r >> 5, l = r & 31;
    float d = f16bits_to_f32(hdr.x & 0xFFFF), dmin = f16bits_to_f32(hdr.x >> 16);
    uint32_t sc_lo, sc_hi, m_lo, m_hi;
    q4k_scales(hdr.y, hdr.z, hdr.w, sc_lo, sc_hi, m_lo, m_hi);
    uint32_t j = 2 * g + hi, bsh = 8 * (j & 3);
    uint32_t sc = ((j < 4 ? sc_lo : sc_hi) >> bsh) & 0xFF;
    uint32_t mn = ((j < 4 ? m_lo : m_hi) >> bsh) & 0xFF;
    float d1 = d * (float)sc, dm1 = dmin * (float)mn;
    u32x2 w = ld_u32x2(blk + 16 + 32 * g + l);
    uint32_t sh = hi * 4;
#pragma unroll
    for (int i = 0; i < 8; ++i) {
      uint32_t word = i < 4 ? w.x : w.y;
      uint32_t q = (word >> (8 * (i & 3) + sh)) & 15;
      o[i] = d1 * (float)q - dm1;
    }
    return f16bits_finite(hdr.x) && f16bits_finite(hdr.x >> 16);
  }
};

// Q6_K: [ql:128][qh:64][sc:16 x i8][d]; halves of 128, quarters s of 32:
// q = (ql nibble | qh 2 bits << 4) - 32; out = (d*sc)*q  (gguf_reader.cpp:774-824)
template <> struct Deq8<CUTHIP_Q6_K> {
  __device__ static bool run(const uint8_t *row, uint32_t col, float o[8]) {
    const uint8_t *blk = row + (size_t)(col >> 8) * 210;
    uint32_t e = col & 255, H = e >> 7, p = e & 127, s = p >> 5, l = p & 31;
    u32x2 ql = ld_u32x2(blk + 64 * H + 32 * (s & 1) + l);
    u32x2 qh = ld_u32x2(blk + 128 + 32 * H + l);
    uint32_t scb = blk[192 + 8 * H + 2 * s + (l >> 4)];
    uint32_t dh = ld_u16(blk + 208);
    float dsc = f16bits_to_f32(dh) * (float)(int)(int8_t)scb;
    uint32_t lsh = (s >> 1) * 4, hsh = 2 * s;
#pragma unroll
    for (int i = 0; i < 8; ++i) {
      uint32_t wl = i < 4 ? ql.x : ql.y, wh = i < 4 ? qh.x : qh.y;
      uint32_t lo = (wl >> (8 * (i & 3) + lsh)) & 15;
      uint32_t h2 = (wh >> (8 * (i & 3) + hsh)) & 3;
      int q = (int)(lo | (h2 << 4)) - 32;
      o[i] = dsc * (float)q;
    }
    return f16bits_finite(dh);
  }
};

// Runs of 2048 elements per workgroup.  With two, a thread takes the same 8-element slot of both runs (every load and
// store instruction still covers contiguous memory) and each wave keeps two independent groups of loads in flight:
// measured on 256 Mi elements to fp16, one / two runs: Q8_0 6.15 / 6.34, Q4_K 6.99 / 7.11, Q6_K 6.59 / 7.27 TB/s, but
// Q4_0 7.39 / 7.11, which therefore stays at one.
template <int FMT> constexpr int kDeqRuns = FMT == CUTHIP_Q4_0 ? 1 : 2;

template <int FMT, bool F16OUT, bool VEC, bool KEEP>
__device__ __forceinline__ void dequant_slot(const uint8_t *__restrict__ blocks, void *__restrict__ out, uint32_t row,
                                             uint32_t col, uint32_t out_stride, size_t row_bytes);

template <int FMT, bool F16OUT, bool VEC, bool KEEP = false>
__global__ void __launch_bounds__(256)
dequant_kernel(const uint8_t *__restrict__ blocks, void *__restrict__ out, uint32_t cols, uint32_t out_stride,
               uint32_t chunks_per_row, size_t row_bytes) {
  uint32_t row = blockIdx.x / chunks_per_row;
  uint32_t chunk = blockIdx.x - row * chunks_per_row;
  if constexpr (kDeqRuns<FMT> == 1) {
    uint32_t col = (chunk * 256u + threadIdx.x) * 8u;
    if (col >= cols) return;
    dequant_slot<FMT, F16OUT, VEC, KEEP>(blocks, out, row, col, out_stride, row_bytes);
  } else {
#pragma unroll
    for (int u = 0; u < kDeqRuns<FMT>; ++u) {
      uint32_t col = ((chunk * kDeqRuns<FMT> + u) * 256u + threadIdx.x) * 8u;
      if (col >= cols) return;
      dequant_slot<FMT, F16OUT, VEC, KEEP>(blocks, out, row, col, out_stride, row_bytes);
    }
  }
}

template <int FMT, bool F16OUT, bool VEC, bool KEEP>
__device__ __forceinline__ void dequant_slot(const uint8_t *__restrict__ blocks, void *__restrict__ out, uint32_t row,
                                             uint32_t col, uint32_t out_stride, size_t row_bytes) {
  float o[8];
  bool finite = Deq8<FMT>::run(blocks + (size_t)row * row_bytes, col, o);
  size_t idx = (size_t)row * out_stride + col;
  if (F16OUT) {
    uint32_t h[8];
    if (finite) {
#pragma unroll
      for (int i = 0; i < 8; ++i) h[i] = f32_to_f16bits_finite(o[i]);
    } else {
#pragma unroll
      for (int i = 0; i < 8; ++i) h[i] = f32_to_f16bits_any(o[i]);
    }
    uint16_t *dst = reinterpret_cast<uint16_t *>(out) + idx;
    if (VEC) {
      u32x4 v{h[0] | (h[1] << 16), h[2] | (h[3] << 16), h[4] | (h[5] << 16), h[6] | (h[7] << 16)};
      // streaming stores for a tensor that leaves the GPU's caches alone; plain stores when the next kernel on
      // the stream reads the output back (the fp16 workspace of the two-pass matmul fits the last-level cache)
      if (KEEP)
        *reinterpret_cast<u32x4 *>(dst) = v;
      else
        __builtin_nontemporal_store(v, reinterpret_cast<u32x4 *>(dst));
    } else {
#pragma unroll
      for (int i = 0; i < 8; ++i) dst[i] = (uint16_t)h[i];
    }
  } else {
    float *dst = reinterpret_cast<float *>(out) + idx;
    if (VEC) {
      __builtin_nontemporal_store(f32x4{o[0], o[1], o[2], o[3]}, reinterpret_cast<f32x4 *>(dst));
      __builtin_nontemporal_store(f32x4{o[4], o[5], o[6], o[7]}, reinterpret_cast<f32x4 *>(dst + 4));
    } else {
#pragma unroll
      for (int i = 0; i < 8; ++i) dst[i] = o[i];
    }
  }
}

// Embedding gather on GGUF blocks: out[i, :] = dequant(row token_ids[i]); a workgroup covers 2048 elements of one
// gathered row.  A token id past the table yields a zero row.
template <int FMT, bool F16OUT, bool VEC>
__global__ void __launch_bounds__(256)
embedding_rows_kernel(const uint8_t *__restrict__ blocks, const uint32_t *__restrict__ token_ids, void *__restrict__ out,
                      uint32_t n_rows, uint32_t cols, uint32_t out_stride, uint32_t chunks_per_row, size_t row_bytes) {
  const uint32_t i = blockIdx.x / chunks_per_row, chunk = blockIdx.x - i * chunks_per_row;
  const uint32_t col = (chunk * 256u + threadIdx.x) * 8u;
  if (col >= cols) return;
  const uint32_t tok = token_ids[i];
  uint8_t *dst_row = reinterpret_cast<uint8_t *>(out) + (size_t)i * out_stride * (F16OUT ? 2 : 4);
  if (tok >= n_rows) {
    for (int e = 0; e < 8; ++e) {
      if (F16OUT) reinterpret_cast<uint16_t *>(dst_row)[col + e] = 0;
      else reinterpret_cast<float *>(dst_row)[col + e] = 0.0f;
    }
    return;
  }
  dequant_slot<FMT, F16OUT, VEC, true>(blocks + (size_t)tok * row_bytes, dst_row, 0, col, out_stride, row_bytes);
}

template <int FMT>
static int launch_embedding(const void *blocks, const uint32_t *token_ids, void *out, int out_dtype, uint32_t n_ids,
                            uint32_t n_rows, uint32_t cols, uint32_t out_stride, hipStream_t stream) {
  const size_t row_bytes = (size_t)(cols / Fmt<FMT>::elems) * Fmt<FMT>::bytes;
  const uint32_t chunks = (cols / 8 + 255) / 256;
  const uint64_t grid = (uint64_t)n_ids * chunks;
  if (grid > 0x7FFFFFFFull) {
    set_error("cuthip_embedding_rows: too many rows for one launch");
    return CUTHIP_ERR_INVALID;
  }
  const bool f16 = out_dtype == CUTHIP_F16;
  const bool vec = ((uintptr_t)out % 16 == 0) && ((out_stride * (f16 ? 2 : 4)) % 16 == 0);
  const uint8_t *src = reinterpret_cast<const uint8_t *>(blocks);
  dim3 g((uint32_t)grid), b(256);
#define CUTHIP_LAUNCH(F16, VEC) \
  hipLaunchKernelGGL((embedding_rows_kernel<FMT, F16, VEC>), g, b, 0, stream, src, token_ids, out, n_rows, cols, out_stride, chunks, row_bytes)
  if (f16) {
    if (vec) CUTHIP_LAUNCH(true, true); else CUTHIP_LAUNCH(true, false);
  } else {
    if (vec) CUTHIP_LAUNCH(false, true); else CUTHIP_LAUNCH(false, false);
  }
#undef CUTHIP_LAUNCH
  return check_hip(hipGetLastError(), "embedding launch");
}

template <int FMT>
static int launch_dequant(const void *blocks, void *out, int out_dtype, uint32_t rows, uint32_t cols,
                          uint32_t out_stride, hipStream_t stream, int keep_cached = 0) {
  size_t row_bytes = (size_t)(cols / Fmt<FMT>::elems) * Fmt<FMT>::bytes;
  // A contiguous output is one long row: no partially filled workgroups.
  if (out_stride == cols && (uint64_t)rows * cols < (1ull << 32)) {
    cols = rows * cols;
    out_stride = cols;
    rows = 1;
  }
  uint32_t chunks = (cols / 8 + 256 * kDeqRuns<FMT> - 1) / (256 * kDeqRuns<FMT>);
  uint64_t grid = (uint64_t)rows * chunks;
  if (grid == 0) return CUTHIP_OK;
  if (grid > 0x7FFFFFFFull) {
    set_error("cuthip_dequant: tensor too large for one launch (%llu workgroups)", (unsigned long long)grid);
    return CUTHIP_ERR_INVALID;
  }
  bool f16 = out_dtype == CUTHIP_F16;
  size_t esz = f16 ? 2 : 4;
  bool vec = ((uintptr_t)out % 16 == 0) && ((out_stride * esz) % 16 == 0);
  dim3 g((uint32_t)grid), b(256);
  const uint8_t *src = reinterpret_cast<const uint8_t *>(blocks);
#define CUTHIP_LAUNCH(F16, VEC) \
  hipLaunchKernelGGL((dequant_kernel<FMT, F16, VEC>), g, b, 0, stream, src, out, cols, out_stride, chunks, row_bytes)
  if (f16 && vec && keep_cached) {
    hipLaunchKernelGGL((dequant_kernel<FMT, true, true, true>), g, b, 0, stream, src, out, cols, out_stride, chunks, row_bytes);
  } else if (f16) {
    if (vec) CUTHIP_LAUNCH(true, true); else CUTHIP_LAUNCH(true, false);
  } else {
    if (vec) CUTHIP_LAUNCH(false, true); else CUTHIP_LAUNCH(false, false);
  }
#undef CUTHIP_LAUNCH
  return check_hip(hipGetLastError(), "dequant launch");
}

// Internal entry for other translation units (the two-pass prefill matmul): arguments already validated; the
// output is written with plain stores because the caller reads it back at once.
int launch_dequant_any(int fmt, const void *blocks, void *out, int out_dtype, uint32_t rows, uint32_t cols,
                       uint32_t out_stride, hipStream_t stream) {
  switch (fmt) {
  case CUTHIP_Q8_0: return launch_dequant<CUTHIP_Q8_0>(blocks, out, out_dtype, rows, cols, out_stride, stream, 1);
  case CUTHIP_Q4_0: return launch_dequant<CUTHIP_Q4_0>(blocks, out, out_dtype, rows, cols, out_stride, stream, 1);
  case CUTHIP_Q4_K: return launch_dequant<CUTHIP_Q4_K>(blocks, out, out_dtype, rows, cols, out_stride, stream, 1);
  default: return launch_dequant<CUTHIP_Q6_K>(blocks, out, out_dtype, rows, cols, out_stride, stream, 1);
  }
}

}  // namespace cuthip

extern "C" int cuthip_dequant(int fmt, const void *blocks, void *out, int out_dtype, uint32_t rows, uint32_t cols,
                              uint32_t out_stride, void *stream) {
  using namespace cuthip;
  if (fmt < CUTHIP_Q8_0 || fmt > CUTHIP_Q6_K) {
    set_error("cuthip_dequant: unknown format %d", fmt);
    return CUTHIP_ERR_INVALID;
  }
  if (out_dtype != CUTHIP_F32 && out_dtype != CUTHIP_F16) {
    set_error("cuthip_dequant: unknown output dtype %d", out_dtype);
    return CUTHIP_ERR_INVALID;
  }
  if (rows == 0 || cols == 0) return CUTHIP_OK;
  if (!blocks || !out) {
    set_error("cuthip_dequant: null device pointer");
    return CUTHIP_ERR_INVALID;
  }
  if (cols % fmt_elems(fmt) != 0) {
    set_error("cuthip_dequant: cols (%u) must be a multiple of the block size %d", cols, fmt_elems(fmt));
    return CUTHIP_ERR_INVALID;
  }
  if (out_stride < cols) {
    set_error("cuthip_dequant: out_stride (%u) smaller than cols (%u)", out_stride, cols);
    return CUTHIP_ERR_INVALID;
  }
  if ((uintptr_t)blocks % 2 != 0) {
    set_error("cuthip_dequant: block pointer must be 2-byte aligned");
    return CUTHIP_ERR_INVALID;
  }
  hipStream_t s = reinterpret_cast<hipStream_t>(stream);
  switch (fmt) {
  case CUTHIP_Q8_0: return launch_dequant<CUTHIP_Q8_0>(blocks, out, out_dtype, rows, cols, out_stride, s);
  case CUTHIP_Q4_0: return launch_dequant<CUTHIP_Q4_0>(blocks, out, out_dtype, rows, cols, out_stride, s);
  case CUTHIP_Q4_K: return launch_dequant<CUTHIP_Q4_K>(blocks, out, out_dtype, rows, cols, out_stride, s);
  default: return launch_dequant<CUTHIP_Q6_K>(blocks, out, out_dtype, rows, cols, out_stride, s);
  }
}

extern "C" int cuthip_embedding_rows(int fmt, const void *blocks, const uint32_t *token_ids, uint32_t n_ids, uint32_t n_rows,
                                     uint32_t dim, void *out, int out_dtype, uint32_t out_stride, void *stream) {
  using namespace cuthip;
  if (fmt < CUTHIP_Q8_0 || fmt > CUTHIP_Q6_K || (out_dtype != CUTHIP_F32 && out_dtype != CUTHIP_F16)) {
    set_error("cuthip_embedding_rows: unknown format %d or output dtype %d", fmt, out_dtype);
    return CUTHIP_ERR_INVALID;
  }
  if (n_ids == 0 || dim == 0) return CUTHIP_OK;
  if (!blocks || !token_ids || !out || dim % fmt_elems(fmt) != 0 || out_stride < dim || (uintptr_t)blocks % 2 != 0) {
    set_error("cuthip_embedding_rows: bad argument (dim %u must be a multiple of the block size %d, out_stride %u >= dim)", dim,
              fmt_elems(fmt), out_stride);
    return CUTHIP_ERR_INVALID;
  }
  hipStream_t s = reinterpret_cast<hipStream_t>(stream);
  switch (fmt) {
  case CUTHIP_Q8_0: return launch_embedding<CUTHIP_Q8_0>(blocks, token_ids, out, out_dtype, n_ids, n_rows, dim, out_stride, s);
  case CUTHIP_Q4_0: return launch_embedding<CUTHIP_Q4_0>(blocks, token_ids, out, out_dtype, n_ids, n_rows, dim, out_stride, s);
  case CUTHIP_Q4_K: return launch_embedding<CUTHIP_Q4_K>(blocks, token_ids, out, out_dtype, n_ids, n_rows, dim, out_stride, s);
  default: return launch_embedding<CUTHIP_Q6_K>(blocks, token_ids, out, out_dtype, n_ids, n_rows, dim, out_stride, s);
  }
}
