// Quantized matmul on the reference's own ("separated") weight layout, for
// callers that keep the tensors the reference's loader produced:
//   Q8: values int8 [K, strideB] (row k holds the N columns), scales fp16 [K/32, scaleStride]
//   Q4: nibbles [K, strideB bytes], even column in the low nibble, value nibble - 8;
//       scales fp16 [K/32, scaleStride]; affine: per-block minima appended as rows
//       [K/32 .. 2K/32) of the scale tensor, value (nibble - 8) * scale + min
//   C[m,n] = sum_k A[m,k] * w[k,n]          (MatMulQ8Common.cuh / MatMulQ4Common.cuh:126-153)
// A, C, D are fp32 as in the reference.
//
// The layout is column-major in n, so a wave streams whole k-rows: each lane
// owns 16 consecutive columns (one 16-byte load of int8, or 8 bytes of
// nibbles), a wave 1024 columns, and the k range is split over the four waves
// of a workgroup and over workgroups (grid.y).  Per 32-row block a lane
// accumulates sum(x * q) per column and applies the block's scale once; the
// "- 8" and the affine minimum become multiples of the block's sum(x).  The
// waves of a workgroup are reduced through LDS; if the k range is split over
// several workgroups the partial sums go to a caller-provided workspace and a
// second kernel adds them and applies the epilogue.
#include <cstdint>
#include <type_traits>

#include "common.hpp"

namespace cuthip {

constexpr int kSepCols = 16;            // columns per lane
constexpr int kSepTile = 64 * kSepCols; // columns per wave
constexpr int kSepKC = 32;              // k-rows per wave (one quantization block)
constexpr int kSepWaves = 4;

struct SepParams {
  const float *A;
  const uint8_t *B;
  const uint16_t *S;
  float *C;         // output, or the workspace [nsplit][M][N] when nsplit > 1
  Epilogue epi;
  uint32_t M, K, N, strideA, strideB, strideC, scaleStride;
  uint32_t m0;      // first row of A handled by this launch
  uint32_t nsplit;
  int affine;
};

// RAGGED: N is not a multiple of 16, so the last lane of a row holds fewer columns and reads them byte by byte; the
// instance for whole lanes carries none of that code (32 rows x a divergent byte loop each made the kernel 10,000
// instructions long, more than the instruction cache holds).
template <bool Q4, int MT, bool RAGGED>
__global__ void __launch_bounds__(64 * kSepWaves, 2) sep_gemv_kernel(SepParams p) {
  // activations of the workgroup's k range, [MT][128] floats, rounded up to one slot per thread and load
  constexpr int XL = (MT * kSepWaves * kSepKC + 64 * kSepWaves - 1) / (64 * kSepWaves);
  __shared__ float xs[XL * 64 * kSepWaves];
  __shared__ f32x4 red[kSepWaves - 1][MT][kSepCols / 4][64];   // lane-contiguous 16-byte slots: no bank conflicts
  const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
  const uint32_t c0 = blockIdx.x * kSepTile + lane * kSepCols;
  const uint32_t kwg = blockIdx.y * (kSepWaves * kSepKC);   // first k-row of this workgroup
  const uint32_t k0 = kwg + wave * kSepKC;                  // this wave's block
  const uint32_t blocksK = p.K / 32;
  const uint32_t ncols = c0 < p.N ? min((uint32_t)kSepCols, p.N - c0) : 0u;
  const bool work = k0 < p.K && ncols;
  // The instance for whole lanes issues every load unconditionally (lanes and waves without work read column 0 of
  // block 0 and drop it): with loads under a condition the compiler waits for all of them at the first use of any.
  const uint32_t cb = (RAGGED || work) ? c0 : 0u, kb = (RAGGED || work) ? k0 : 0u;

  // One k-row of this lane's 16 columns: 16 bytes of int8 or 8 bytes of nibbles.
  using Row = typename std::conditional<Q4, u32x2, u32x4>::type;
  auto load_row = [&](uint32_t k) -> Row {
    Row w{};
    if (Q4) {
      const uint8_t *src = p.B + (size_t)k * p.strideB + cb / 2;
      if (!RAGGED || ncols == kSepCols) {
        const u32x2 v = ld_u32x2(src);
        w[0] = v.x;
        w[1] = v.y;
      } else {   // last lane of a ragged row: byte loads inside the row
        for (uint32_t b = 0; b < (ncols + 1) / 2; ++b) w[b >> 2] |= (uint32_t)src[b] << (8 * (b & 3));
      }
    } else {
      const uint8_t *src = p.B + (size_t)k * p.strideB + cb;
      if (!RAGGED || ncols == kSepCols) {
        const u32x4 v = ld_u32x4(src);
        w[0] = v.x; w[1] = v.y; w[2] = v.z; w[3] = v.w;
      } else {
        for (uint32_t b = 0; b < ncols; ++b) w[b >> 2] |= (uint32_t)src[b] << (8 * (b & 3));
      }
    }
    return w;
  };

  // Every load of the wave's block is requested before anything is used: G rows per lane in flight (all 32 where the
  // registers allow), then the block's scales (and minima), then the activations of the workgroup's k range.  With
  // four groups of eight rows, each used right after the next was requested, the kernel waited for four memory round
  // trips in turn and took 20 us for 14336 x 4096 whatever the format.
  // The activations of the workgroup's k range are requested first and unconditionally (threads without an element
  // read element 0 and drop it), so that they arrive ahead of the weights and the wait for them leaves the weight
  // loads in flight: memory returns in issue order.
  float xv[XL];
#pragma unroll
  for (int u = 0; u < XL; ++u) {
    const int i = tid + u * 64 * kSepWaves, m = i / (kSepWaves * kSepKC), kk = i % (kSepWaves * kSepKC);
    const uint32_t row = p.m0 + m, k = kwg + kk;
    const bool ok = m < MT && row < p.M && k < p.K;
    xv[u] = p.A[ok ? (size_t)row * p.strideA + k : (size_t)0];
    if (!ok) xv[u] = 0.0f;
  }
  __builtin_amdgcn_sched_barrier(0);   // the requests above stay ahead of the weight loads
  constexpr int G = MT <= 2 ? kSepKC : kSepKC / 4;   // four batch rows leave registers for eight weight rows in flight
  Row wbuf[G];
  if (!RAGGED || work) {
#pragma unroll
    for (int j = 0; j < G; ++j) wbuf[j] = load_row(kb + j);
  }
  const uint32_t blk = kb / 32;
  const uint16_t *srow = p.S + (size_t)blk * p.scaleStride + cb;
  // without minima the second pair of loads repeats the scales (dropped later): no condition around a load
  const uint16_t *mrow = p.S + (size_t)((Q4 && p.affine ? blocksK : 0u) + blk) * p.scaleStride + cb;
  // whole lanes: the launcher has checked that every lane's scales are 16-byte aligned
  const bool svec = !RAGGED || (work && ncols == kSepCols && ((uintptr_t)srow & 15u) == 0 && ((uintptr_t)mrow & 15u) == 0);
  u32x4 sraw[2] = {u32x4{0, 0, 0, 0}, u32x4{0, 0, 0, 0}}, mraw[2] = {u32x4{0, 0, 0, 0}, u32x4{0, 0, 0, 0}};
  if (svec) {
    sraw[0] = ld_u32x4(reinterpret_cast<const uint8_t *>(srow));
    sraw[1] = ld_u32x4(reinterpret_cast<const uint8_t *>(srow) + 16);
    if (Q4 && (!RAGGED || p.affine)) {
      mraw[0] = ld_u32x4(reinterpret_cast<const uint8_t *>(mrow));
      mraw[1] = ld_u32x4(reinterpret_cast<const uint8_t *>(mrow) + 16);
    }
  }
  // every thread stores (slots beyond [MT][128] are never read): a store under a condition would take its load along
#pragma unroll
  for (int u = 0; u < XL; ++u) xs[tid + u * 64 * kSepWaves] = xv[u];
  __syncthreads();

  // a wave handles exactly one quantization block of k, so the per-block sums become the result in place
  float bs[MT][kSepCols], sx[MT];
#pragma unroll
  for (int m = 0; m < MT; ++m) {
    sx[m] = 0.0f;
#pragma unroll
    for (int c = 0; c < kSepCols; ++c) bs[m][c] = 0.0f;
  }

  if (work) {
    const float *xw = &xs[wave * kSepKC];
    auto row_fma = [&](const Row &w, int kk) {
      float q[kSepCols];
      if constexpr (Q4) {
        // low and high nibbles of four bytes at a time (one mask, one shift + mask), then a byte-to-float conversion each
#pragma unroll
        for (int h = 0; h < 2; ++h) {
          uint32_t lo = w[h] & 0x0F0F0F0Fu, hi = (w[h] >> 4) & 0x0F0F0F0Fu;
          asm volatile("" : "+v"(lo), "+v"(hi));   // known bits would turn every conversion into a bit-field extract + convert
          q[8 * h + 0] = cvt_ubyte0(lo); q[8 * h + 1] = cvt_ubyte0(hi);
          q[8 * h + 2] = cvt_ubyte1(lo); q[8 * h + 3] = cvt_ubyte1(hi);
          q[8 * h + 4] = cvt_ubyte2(lo); q[8 * h + 5] = cvt_ubyte2(hi);
          q[8 * h + 6] = cvt_ubyte3(lo); q[8 * h + 7] = cvt_ubyte3(hi);
        }
      } else {
#pragma unroll
        for (int c = 0; c < kSepCols; ++c) q[c] = (float)(int)(int8_t)((w[c >> 2] >> (8 * (c & 3))) & 0xFF);
      }
#pragma unroll
      for (int m = 0; m < MT; ++m) {
        float x = xw[m * (kSepWaves * kSepKC) + kk];
        sx[m] += x;
#pragma unroll
        for (int c = 0; c < kSepCols; ++c) bs[m][c] = fmaf(x, q[c], bs[m][c]);
      }
    };
#pragma unroll
    for (int j = 0; j < kSepKC; ++j) {
      row_fma(wbuf[j % G], j);
      if (j + G < kSepKC) wbuf[j % G] = load_row(kb + j + G);   // G < 32: the slot is refilled as soon as it is used
      if constexpr (G < kSepKC) __builtin_amdgcn_sched_barrier(0);   // keeps the refills from being hoisted into spills
    }
#pragma unroll
    for (int c = 0; c < kSepCols; ++c) {
      if (!RAGGED || (uint32_t)c < ncols) {
        float s, mn = 0.0f;
        if (svec) {
          s = f16bits_to_f32((sraw[c >> 3][(c >> 1) & 3] >> (16 * (c & 1))) & 0xFFFFu);
          if (Q4 && p.affine) mn = f16bits_to_f32((mraw[c >> 3][(c >> 1) & 3] >> (16 * (c & 1))) & 0xFFFFu);
        } else {
          s = f16bits_to_f32(srow[c]);
          if (Q4 && p.affine) mn = f16bits_to_f32(mrow[c]);
        }
#pragma unroll
        for (int m = 0; m < MT; ++m) {
          float v = Q4 ? fmaf(-8.0f, sx[m], bs[m][c]) : bs[m][c];
          bs[m][c] = fmaf(v, s, mn * sx[m]);
        }
      }
    }
  }

  // fold the four waves (k blocks) of the workgroup into wave 0: one trip through LDS, added in wave order
  if (wave > 0) {
#pragma unroll
    for (int m = 0; m < MT; ++m)
#pragma unroll
      for (int c4 = 0; c4 < kSepCols / 4; ++c4)
        red[wave - 1][m][c4][lane] = f32x4{bs[m][4 * c4], bs[m][4 * c4 + 1], bs[m][4 * c4 + 2], bs[m][4 * c4 + 3]};
  }
  __syncthreads();
  if (wave == 0 && ncols) {
#pragma unroll
    for (int w = 0; w < kSepWaves - 1; ++w)
#pragma unroll
      for (int m = 0; m < MT; ++m)
#pragma unroll
        for (int c4 = 0; c4 < kSepCols / 4; ++c4) {
          const f32x4 v = red[w][m][c4][lane];
          bs[m][4 * c4] += v.x; bs[m][4 * c4 + 1] += v.y; bs[m][4 * c4 + 2] += v.z; bs[m][4 * c4 + 3] += v.w;
        }
#pragma unroll
    for (int m = 0; m < MT; ++m) {
      const uint32_t row = p.m0 + m;
      if (row >= p.M) continue;
      if (p.nsplit > 1) {   // workspace [split][M][N]
        float *dst = p.C + ((size_t)blockIdx.y * p.M + row) * p.N + c0;
        if ((!RAGGED || ncols == kSepCols) && ((uintptr_t)dst & 15u) == 0) {
#pragma unroll
          for (int c4 = 0; c4 < kSepCols / 4; ++c4)
            reinterpret_cast<f32x4 *>(dst)[c4] = f32x4{bs[m][4 * c4], bs[m][4 * c4 + 1], bs[m][4 * c4 + 2], bs[m][4 * c4 + 3]};
        } else {
#pragma unroll
          for (int c = 0; c < kSepCols; ++c)
            if (!RAGGED || (uint32_t)c < ncols) dst[c] = bs[m][c];
        }
      } else {
#pragma unroll
        for (int c = 0; c < kSepCols; ++c)
          if (!RAGGED || (uint32_t)c < ncols) store_out(p.C, p.epi, 0, (size_t)row * p.strideC + c0 + c, bs[m][c]);
      }
    }
  }
}

__global__ void __launch_bounds__(256) sep_reduce_kernel(const float *ws, float *C, Epilogue epi, uint32_t M, uint32_t N,
                                                         uint32_t strideC, uint32_t m0, uint32_t mcount, uint32_t nsplit) {
  uint32_t i = blockIdx.x * 256 + threadIdx.x;
  if (i >= mcount * N) return;
  uint32_t row = m0 + i / N, n = i % N;
  float v = 0.0f;
#pragma unroll 8
  for (uint32_t s = 0; s < nsplit; ++s) v += ws[((size_t)s * M + row) * N + n];
  store_out(C, epi, 0, (size_t)row * strideC + n, v);
}

// The same for four consecutive columns per thread (N a multiple of 4, 16-byte aligned workspace): 16 partial sums
// requested at a time instead of eight single floats, added in the same order.
__global__ void __launch_bounds__(256) sep_reduce4_kernel(const float *ws, float *C, Epilogue epi, uint32_t M, uint32_t N,
                                                          uint32_t strideC, uint32_t m0, uint32_t mcount, uint32_t nsplit) {
  const uint32_t n4 = N / 4, i = blockIdx.x * 256 + threadIdx.x;
  if (i >= mcount * n4) return;
  const uint32_t row = m0 + i / n4, n = (i % n4) * 4;
  const float *src = ws + (size_t)row * N + n;
  const size_t step = (size_t)M * N;
  f32x4 v = {0.0f, 0.0f, 0.0f, 0.0f};
  uint32_t s = 0;
  for (; s + 16 <= nsplit; s += 16) {
    f32x4 t[16];
#pragma unroll
    for (int u = 0; u < 16; ++u) t[u] = *reinterpret_cast<const f32x4 *>(src + (s + u) * step);
#pragma unroll
    for (int u = 0; u < 16; ++u) v += t[u];
  }
  for (; s < nsplit; ++s) v += *reinterpret_cast<const f32x4 *>(src + s * step);
#pragma unroll
  for (int c = 0; c < 4; ++c) store_out(C, epi, 0, (size_t)row * strideC + n + c, v[c]);
}

template <bool Q4, int MT> static int launch_sep(SepParams p, uint32_t mcount, float *C, void *workspace, hipStream_t stream) {
  dim3 grid((p.N + kSepTile - 1) / kSepTile, p.nsplit);
  float *out = p.nsplit == 1 ? C : reinterpret_cast<float *>(workspace);
  p.C = out;
  // whole lanes: every lane holds 16 columns and its scales are 16-byte aligned
  if (p.N % kSepCols == 0 && (uintptr_t)p.S % 16 == 0 && p.scaleStride % 8 == 0)
    hipLaunchKernelGGL((sep_gemv_kernel<Q4, MT, false>), grid, dim3(64 * kSepWaves), 0, stream, p);
  else hipLaunchKernelGGL((sep_gemv_kernel<Q4, MT, true>), grid, dim3(64 * kSepWaves), 0, stream, p);
  if (int rc = check_hip(hipGetLastError(), "separated-layout matmul launch")) return rc;
  if (p.nsplit > 1) {
    if (p.N % 4 == 0 && (uintptr_t)workspace % 16 == 0)
      hipLaunchKernelGGL(sep_reduce4_kernel, dim3((mcount * (p.N / 4) + 255) / 256), dim3(256), 0, stream,
                         reinterpret_cast<const float *>(workspace), C, p.epi, p.M, p.N, p.strideC, p.m0, mcount, p.nsplit);
    else
      hipLaunchKernelGGL(sep_reduce_kernel, dim3((mcount * p.N + 255) / 256), dim3(256), 0, stream,
                         reinterpret_cast<const float *>(workspace), C, p.epi, p.M, p.N, p.strideC, p.m0, mcount, p.nsplit);
    return check_hip(hipGetLastError(), "separated-layout reduce launch");
  }
  return CUTHIP_OK;
}

// ---- prefill on the separated layout: dequantize to fp16 [N][K], then the dense GEMM ------------------------------
// The GEMV above streams the weights once per 4 rows of A; from kSepDenseRows rows on the tensors are turned into the
// fp16 [N][K] operand of the dense GEMM first (one launch: value = float(q) * scale (+ min), rounded to nearest even,
// 64 x 64 tiles transposed through LDS so that both the reads along n and the writes along k are contiguous) and the
// product goes through the same GEMM as cuthip_matmul_dense_f16 (hipBLASLt without an epilogue, else the hand-written one).
constexpr uint32_t kSepDenseRows = 32;

bool dense_gemm_fits(uint32_t M, uint32_t K, uint32_t N, uint32_t strideA, int a_f16, const void *A);
size_t dense_f16_workspace(uint32_t M, uint32_t K, uint32_t N, int a_f16);
int launch_dense_gemm(int fmt, const void *W, const void *A, int a_f16, void *C, int c_f16, uint32_t M, uint32_t K,
                      uint32_t N, uint32_t strideA, uint32_t strideC, Epilogue epi, void *workspace, hipStream_t stream,
                      int use_blaslt);

static size_t sep_w16_bytes(uint32_t K, uint32_t N) { return ((size_t)N * K * 2 + 255) & ~(size_t)255; }
static bool sep_dense_fits(uint32_t K, uint32_t N, uint32_t M) {
  return K % 128 == 0 && (uint64_t)N * K * 2 < (1ull << 32) && (uint64_t)M * K * 2 < (1ull << 32);
}
static bool sep_dense_applies(uint32_t M, uint32_t K, uint32_t N) { return M >= kSepDenseRows && sep_dense_fits(K, N, M); }

template <bool Q4>
__global__ void __launch_bounds__(256) sep_dequant_kernel(const uint8_t *B, const uint16_t *S, half_t *W16, uint32_t K, uint32_t N,
                                                          uint32_t strideB, uint32_t scaleStride, int affine) {
  __shared__ half_t tile[64][64 + 2];   // [n][k], rows 33 dwords apart
  const uint32_t tid = threadIdx.x, n0 = blockIdx.x * 64, k0 = blockIdx.y * 64;
  {
    const uint32_t k = k0 + tid / 4, nseg = (tid & 3) * 16;   // 16 columns of one k-row
    if (k < K) {
      const uint32_t blk = k / 32, blocksK = K / 32;
      uint32_t q[4] = {0, 0, 0, 0};
      const uint32_t n = n0 + nseg;
      // whole, aligned segments take one vector load for the values and two for the scales
      const bool fast = n + 16 <= N && (scaleStride & 7u) == 0 && ((uintptr_t)S & 15u) == 0 &&
                        (strideB & (Q4 ? 7u : 15u)) == 0 && ((uintptr_t)B & (Q4 ? 7u : 15u)) == 0;
      uint32_t sraw[8], mraw[8];
      if (fast) {
        const u32x4 s0 = *reinterpret_cast<const u32x4 *>(S + (size_t)blk * scaleStride + n);
        const u32x4 s1 = *reinterpret_cast<const u32x4 *>(S + (size_t)blk * scaleStride + n + 8);
        sraw[0] = s0.x; sraw[1] = s0.y; sraw[2] = s0.z; sraw[3] = s0.w; sraw[4] = s1.x; sraw[5] = s1.y; sraw[6] = s1.z; sraw[7] = s1.w;
        if (Q4 && affine) {
          const u32x4 m0 = *reinterpret_cast<const u32x4 *>(S + (size_t)(blocksK + blk) * scaleStride + n);
          const u32x4 m1 = *reinterpret_cast<const u32x4 *>(S + (size_t)(blocksK + blk) * scaleStride + n + 8);
          mraw[0] = m0.x; mraw[1] = m0.y; mraw[2] = m0.z; mraw[3] = m0.w; mraw[4] = m1.x; mraw[5] = m1.y; mraw[6] = m1.z; mraw[7] = m1.w;
        }
        if (Q4) {
          const u32x2 b = *reinterpret_cast<const u32x2 *>(B + (size_t)k * strideB + n / 2);
          const uint32_t w[2] = {b.x, b.y};
#pragma unroll
          for (int j = 0; j < 8; ++j) {
            const uint32_t byte = (w[j / 4] >> (8 * (j & 3))) & 0xFFu;
            q[j / 2] |= ((byte & 15u) | ((byte >> 4) << 8)) << (16 * (j & 1));
          }
        } else {
          const u32x4 b = *reinterpret_cast<const u32x4 *>(B + (size_t)k * strideB + n);
          q[0] = b.x; q[1] = b.y; q[2] = b.z; q[3] = b.w;
        }
#pragma unroll
        for (int j = 0; j < 16; ++j) {
          const float sc = f16bits_to_f32((sraw[j / 2] >> (16 * (j & 1))) & 0xFFFFu);
          const uint32_t byte = (q[j / 4] >> (8 * (j & 3))) & 0xFFu;
          float v;
          if (Q4) {
            v = (float)((int)byte - 8) * sc;
            if (affine) v += f16bits_to_f32((mraw[j / 2] >> (16 * (j & 1))) & 0xFFFFu);
          } else {
            v = (float)(int)(int8_t)byte * sc;
          }
          tile[nseg + j][tid / 4] = (half_t)v;
        }
      } else {
      if (Q4) {   // 8 bytes = 16 nibbles, even column in the low nibble
        for (uint32_t j = 0; j < 8 && n + 2 * j < N; ++j) {
          const uint32_t b = B[(size_t)k * strideB + n / 2 + j];
          q[j / 2] |= ((b & 15u) | ((b >> 4) << 8)) << (16 * (j & 1));   // two columns per byte -> two bytes
        }
      } else {
        for (uint32_t j = 0; j < 16 && n + j < N; ++j) q[j / 4] |= (uint32_t)B[(size_t)k * strideB + n + j] << (8 * (j & 3));
      }
#pragma unroll
      for (int j = 0; j < 16; ++j) {
        float v = 0.0f;
        if (n + j < N) {
          const float sc = f16bits_to_f32(S[(size_t)blk * scaleStride + n + j]);
          const uint32_t byte = (q[j / 4] >> (8 * (j & 3))) & 0xFFu;
          if (Q4) {
            v = (float)((int)byte - 8) * sc;
            if (affine) v += f16bits_to_f32(S[(size_t)(blocksK + blk) * scaleStride + n + j]);
          } else {
            v = (float)(int)(int8_t)byte * sc;
          }
        }
        tile[nseg + j][tid / 4] = (half_t)v;
      }
      }
    }
  }
  __syncthreads();
  {
    const uint32_t n = n0 + tid / 4, kseg = (tid & 3) * 16;   // 16 consecutive k of one weight row
    if (n < N) {
      half_t *dst = W16 + (size_t)n * K + k0 + kseg;
      if (k0 + kseg + 16 <= K && (K & 7u) == 0) {   // W16 is 256-byte aligned and K a multiple of 8: 16-byte stores
        uint32_t w[8];
#pragma unroll
        for (int j = 0; j < 8; ++j) {
          const uint16_t lo = __builtin_bit_cast(uint16_t, tile[tid / 4][kseg + 2 * j]);
          const uint16_t hi = __builtin_bit_cast(uint16_t, tile[tid / 4][kseg + 2 * j + 1]);
          w[j] = (uint32_t)lo | ((uint32_t)hi << 16);
        }
        *reinterpret_cast<u32x4 *>(dst) = u32x4{w[0], w[1], w[2], w[3]};
        *reinterpret_cast<u32x4 *>(dst + 8) = u32x4{w[4], w[5], w[6], w[7]};
      } else {
        for (uint32_t j = 0; j < 16 && k0 + kseg + j < K; ++j) dst[j] = tile[tid / 4][kseg + j];
      }
    }
  }
}

// Which of the two code paths a variant index of the reference's tables asks for.  The tables hold the reference's
// names at the reference's indices (MatMulQ8Variants.generated.h:20-32, MatMulQ4Variants.generated.h:20-29); its
// eight / five shaders collapse onto the two kernels here:
//   tiled shaders (Q8 0, 2, 6; Q4 0) and -1            -> the choice by shape the reference's own default makes
//   GEMV shaders (Q8 1, 3, 4, 5; Q4 1, 2, 3)            -> the streaming kernel, whatever M is
//   cooperative-matrix shaders (Q8 7; Q4 4)            -> dequantize to fp16, then the dense MFMA GEMM
// The reference's int8-activation shaders (Q8 5 GemvDot, 6 TiledDot) run here with fp32 / fp16 activations, i.e.
// closer to the fp32 loop than the reference's own result for those indices.
enum SepRoute { kSepAuto = 0, kSepStream = 1, kSepDense = 2 };
static int sep_route(bool q4, int variant) {
  if (variant == -1) return kSepAuto;
  if (q4) {
    switch (variant) {
    case 0: return kSepAuto;
    case 1: case 2: case 3: return kSepStream;
    case 4: return kSepDense;
    }
  } else {
    switch (variant) {
    case 0: case 2: case 6: return kSepAuto;
    case 1: case 3: case 4: case 5: return kSepStream;
    case 7: return kSepDense;
    }
  }
  return -1;
}
static size_t sep_stream_bytes(uint32_t M, uint32_t K, uint32_t N) {
  size_t nsplit = (K + kSepWaves * kSepKC - 1) / (kSepWaves * kSepKC);
  return nsplit > 1 ? nsplit * M * N * sizeof(float) : 0;
}

static int matmul_sep(bool q4, const float *A, const void *B, const void *S, const float *D, float *C, uint32_t M, uint32_t K,
                      uint32_t N, uint32_t strideA, uint32_t strideB, uint32_t strideC, uint32_t scaleStride, int epilogue,
                      int epilogue_op, int affine, int variant, void *workspace, size_t workspace_bytes, hipStream_t stream) {
  const char *who = q4 ? "cuthip_matmul_q4_sep" : "cuthip_matmul_q8_sep";
  const int route = sep_route(q4, variant);
  if (route < 0) {
    set_error("%s: unknown variant index %d (table has %d)", who, variant,
              cuthip_variant_count(q4 ? CUTHIP_OP_MATMUL_Q4 : CUTHIP_OP_MATMUL_Q8));
    return CUTHIP_ERR_UNKNOWN_VARIANT;
  }
  if (!A || !B || !S || !C || M == 0 || K == 0 || N == 0 || K % 32 || strideA < K || strideC < N || scaleStride < N ||
      strideB < (q4 ? (N + 1) / 2 : N) || (q4 && (N & 1))) {
    set_error("%s: bad argument (M %u, K %u (multiple of 32), N %u%s, strides %u %u %u %u)", who, M, K, N,
              q4 ? " (even)" : "", strideA, strideB, strideC, scaleStride);
    return CUTHIP_ERR_INVALID;
  }
  if (epilogue < CUTHIP_EPI_NONE || epilogue > CUTHIP_EPI_BINARY || (epilogue == CUTHIP_EPI_BINARY && !D)) {
    set_error("%s: bad epilogue %d (a binary epilogue needs D)", who, epilogue);
    return CUTHIP_ERR_INVALID;
  }
  if (int rc = check_epilogue_op(who, epilogue, epilogue_op)) return rc;
  if (epilogue_op_long(epilogue, epilogue_op)) {   // unfused matmul, then the operator as an elementwise launch
    if (int rc = check_long_epilogue_alias(epilogue, epilogue_op, C, D)) return rc;   // before anything is written
    if (int rc = matmul_sep(q4, A, B, S, nullptr, C, M, K, N, strideA, strideB, strideC, scaleStride, CUTHIP_EPI_NONE, 0, affine,
                            variant, workspace, workspace_bytes, stream))
      return rc;
    return launch_long_epilogue(C, 0, M, N, strideC, epilogue, epilogue_op, D, stream);
  }
  const bool dense_ok = sep_dense_fits(K, N, M) && dense_gemm_fits(M, K, N, strideA, 0, A) && workspace &&
                        (uintptr_t)workspace % 256 == 0 && workspace_bytes >= sep_w16_bytes(K, N) + dense_f16_workspace(M, K, N, 0);
  if (route == kSepDense && !dense_ok) {
    set_error("%s: variant %d (dequantize, then the MFMA GEMM) needs K a multiple of 128, 16-byte aligned rows of A and a "
              "256-byte aligned workspace of %zu bytes (K %u, strideA %u, workspace %zu)", who, variant,
              sep_w16_bytes(K, N) + dense_f16_workspace(M, K, N, 0), K, strideA, workspace ? workspace_bytes : (size_t)0);
    return CUTHIP_ERR_INVALID;
  }
  if (dense_ok && (route == kSepDense || (route == kSepAuto && M >= kSepDenseRows))) {
    half_t *w16 = reinterpret_cast<half_t *>(workspace);
    dim3 grid((N + 63) / 64, (K + 63) / 64);
    if (q4)
      hipLaunchKernelGGL(sep_dequant_kernel<true>, grid, dim3(256), 0, stream, reinterpret_cast<const uint8_t *>(B),
                         reinterpret_cast<const uint16_t *>(S), w16, K, N, strideB, scaleStride, affine);
    else
      hipLaunchKernelGGL(sep_dequant_kernel<false>, grid, dim3(256), 0, stream, reinterpret_cast<const uint8_t *>(B),
                         reinterpret_cast<const uint16_t *>(S), w16, K, N, strideB, scaleStride, 0);
    if (int rc = check_hip(hipGetLastError(), "separated-layout dequant launch")) return rc;
    Epilogue epi{epilogue, epilogue_op, epilogue == CUTHIP_EPI_BINARY ? D : nullptr};
    return launch_dense_gemm(-1, w16, A, 0, C, 0, M, K, N, strideA, strideC, epi,
                             reinterpret_cast<uint8_t *>(workspace) + sep_w16_bytes(K, N), stream,
                             0);
  }
  SepParams p;
  p.A = A;
  p.B = reinterpret_cast<const uint8_t *>(B);
  p.S = reinterpret_cast<const uint16_t *>(S);
  p.C = C;
  p.epi = Epilogue{epilogue, epilogue_op, D};
  p.M = M; p.K = K; p.N = N; p.strideA = strideA; p.strideB = strideB; p.strideC = strideC; p.scaleStride = scaleStride;
  p.affine = affine;
  p.nsplit = (K + kSepWaves * kSepKC - 1) / (kSepWaves * kSepKC);
  if (p.nsplit > 1 && (!workspace || workspace_bytes < (size_t)p.nsplit * M * N * sizeof(float))) {
    set_error("%s: workspace of %zu bytes, need %zu", who, workspace_bytes, (size_t)p.nsplit * M * N * sizeof(float));
    return CUTHIP_ERR_INVALID;
  }
  // passes of up to 4 rows of A (each pass streams the weights once; 8 rows would spill registers)
  for (uint32_t m0 = 0; m0 < M; m0 += 4) {
    uint32_t mc = min(4u, M - m0);
    p.m0 = m0;
    int rc;
    if (q4) {
      rc = mc == 1 ? launch_sep<true, 1>(p, mc, C, workspace, stream) : mc == 2 ? launch_sep<true, 2>(p, mc, C, workspace, stream)
                                                                                 : launch_sep<true, 4>(p, mc, C, workspace, stream);
    } else {
      rc = mc == 1 ? launch_sep<false, 1>(p, mc, C, workspace, stream) : mc == 2 ? launch_sep<false, 2>(p, mc, C, workspace, stream)
                                                                                  : launch_sep<false, 4>(p, mc, C, workspace, stream);
    }
    if (rc) return rc;
  }
  return CUTHIP_OK;
}

}  // namespace cuthip

using namespace cuthip;

extern "C" {

size_t cuthip_matmul_sep_workspace_bytes(uint32_t M, uint32_t K, uint32_t N) {
  if (sep_dense_applies(M, K, N)) return sep_w16_bytes(K, N) + dense_f16_workspace(M, K, N, 0);   // prefill route
  return sep_stream_bytes(M, K, N);
}

size_t cuthip_matmul_sep_workspace_bytes_for(int op, int variant, uint32_t M, uint32_t K, uint32_t N) {
  const int route = sep_route(op == CUTHIP_OP_MATMUL_Q4, variant);
  if (route == kSepStream) return sep_stream_bytes(M, K, N);
  if (route == kSepDense) return sep_w16_bytes(K, N) + dense_f16_workspace(M, K, N, 0);
  return cuthip_matmul_sep_workspace_bytes(M, K, N);
}

int cuthip_matmul_q8_sep(const float *A, const int8_t *B, const uint16_t *scales, const float *D, float *C, uint32_t M,
                         uint32_t K, uint32_t N, uint32_t strideA, uint32_t strideB, uint32_t strideC, uint32_t scaleStride,
                         int epilogue, int epilogue_op, int variant, void *workspace, size_t workspace_bytes, void *stream) {
  return matmul_sep(false, A, B, scales, D, C, M, K, N, strideA, strideB, strideC, scaleStride, epilogue, epilogue_op, 0,
                    variant, workspace, workspace_bytes, (hipStream_t)stream);
}

int cuthip_matmul_q4_sep(const float *A, const uint8_t *packedB, const uint16_t *scales, const float *D, float *C, uint32_t M,
                         uint32_t K, uint32_t N, uint32_t strideA, uint32_t strideBNpacked, uint32_t strideC,
                         uint32_t scaleStride, int epilogue, int epilogue_op, int affine, int variant, void *workspace,
                         size_t workspace_bytes, void *stream) {
  return matmul_sep(true, A, packedB, scales, D, C, M, K, N, strideA, strideBNpacked, strideC, scaleStride, epilogue,
                    epilogue_op, affine, variant, workspace, workspace_bytes, (hipStream_t)stream);
}

}  // extern "C"
