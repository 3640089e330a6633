// Q8_0 prefill GEMM with int8 activations on the int8 matrix core of gfx950:
//   C[m,n] = sum over 32-element blocks b of
//            float(sum_k qa[m,k] * qw[n,k]) * a_scale[m,b] * d_w[n,b]
// Activations are quantized per block of 32 exactly as the reference's int8
// dot-product GEMV does it (MatMulQ8GemvDot.cu:60-64: a_scale = amax / 127,
// q = clamp(round(a * (127 / amax)), -127, 127)) and the block sums are folded
// as there (:85, acc += float(dot) * a_scale * b_scale).  The reference runs
// that arithmetic for M = 1 on dp4a; here it feeds prefill tiles to
// v_mfma_i32_32x32x32_i8, whose K of 32 is exactly one Q8_0 block, so every
// MFMA yields the integer dot products of one block for a 32 x 32 tile.
//
// Numerics differ from the fp16-activation kernels on purpose: rounding the
// activations to 8 bits per block moves the result about 5e-3 (normwise) from
// the fp32 path, so this variant is opt-in (its own entry point), never chosen
// automatically, and is checked against the same arithmetic on the CPU.
//
// Two launches: quantize_act_kernel writes qa (int8 [M][K]) and a_scale (fp32
// [M][K/32]) to the caller's workspace; gemm_q8_i8_kernel owns a 128 x 128
// tile of C per workgroup (four waves, 64 x 64 each = 2 x 2 MFMA tiles) and
// walks K in slices of 128.  The weight tile needs no decode at all: the int8
// payload of the GGUF blocks is copied to LDS as it is, the fp16 block scales
// become an fp32 side table.  What bounds the kernel is the scaling after the
// MFMA: 16 integer results per lane and MFMA each need a convert, a multiply
// by a_scale (per row) and an FMA with d_w (per column): 48 VALU instructions
// (192 cycles) against 32 cycles of matrix core.
#include <cstdint>

#include "common.hpp"
#include "gemm_store.hpp"

namespace cuthip {

typedef int i32x4 __attribute__((ext_vector_type(4)));
typedef int i32x16 __attribute__((ext_vector_type(16)));
typedef __attribute__((address_space(3))) uint8_t lds_u8i;

constexpr int kI8BM = 128, kI8BN = 128, kI8BK = 128, kI8Blocks = kI8BK / 32;
constexpr int kI8Pitch = kI8BK + 16;   // bytes per LDS row: 16-byte aligned, rows 36 dwords apart

struct I8Params {
  const uint8_t *W;       // Q8_0 blocks [N][K/32]
  const int8_t *qa;       // [M][K]
  const float *sa;        // [M][K/32]
  void *C;
  Epilogue epi;
  uint32_t M, K, N, strideC, row_bytes, nblk;
  uint32_t mtiles, ntiles;
  int c_f16;
  int vec_store;   // C (and a binary epilogue's operand) allow 16-byte accesses
};

// 8 lanes per block of 32 activations (MatMulQ8GemvDot.cu:60-64)
template <bool AF16>
__global__ void __launch_bounds__(256) quantize_act_kernel(const void *A, uint32_t M, uint32_t K, uint32_t strideA, int8_t *qa,
                                                           float *sa) {
  const uint32_t nblk = K / 32;
  const uint64_t t = (uint64_t)blockIdx.x * 256u + threadIdx.x, b = t >> 3;
  const uint32_t i = (uint32_t)t & 7u;
  const bool ok = b < (uint64_t)M * nblk;
  const uint32_t m = ok ? (uint32_t)(b / nblk) : 0u, kb = ok ? (uint32_t)(b % nblk) : 0u;
  float v[4] = {0.0f, 0.0f, 0.0f, 0.0f};
  if (ok) {
    const size_t off = (size_t)m * strideA + kb * 32u + i * 4u;
    if (AF16) {
      const half_t *h = reinterpret_cast<const half_t *>(A) + off;
#pragma unroll
      for (int j = 0; j < 4; ++j) v[j] = (float)h[j];
    } else {
      const float *f = reinterpret_cast<const float *>(A) + off;
#pragma unroll
      for (int j = 0; j < 4; ++j) v[j] = f[j];
    }
  }
  float amax = fmaxf(fmaxf(fabsf(v[0]), fabsf(v[1])), fmaxf(fabsf(v[2]), fabsf(v[3])));
  amax = fmaxf(amax, __shfl_xor(amax, 1));
  amax = fmaxf(amax, __shfl_xor(amax, 2));
  amax = fmaxf(amax, __shfl_xor(amax, 4));
  const float a_scale = amax / 127.0f;
  const float inv = amax > 0.0f ? 127.0f / amax : 0.0f;
  uint32_t word = 0;
#pragma unroll
  for (int j = 0; j < 4; ++j) {
    int q = (int)roundf(v[j] * inv);
    q = max(-127, min(127, q));
    word |= ((uint32_t)q & 0xFFu) << (8 * j);
  }
  if (!ok) return;
  *reinterpret_cast<uint32_t *>(qa + (size_t)m * K + kb * 32u + i * 4u) = word;
  if (i == 0) sa[(size_t)m * nblk + kb] = a_scale;
}

__global__ void __launch_bounds__(256, 2) gemm_q8_i8_kernel(I8Params p) {
  __shared__ __attribute__((aligned(16))) uint8_t ab_s[(kI8BM + kI8BN) * kI8Pitch];   // the operand tiles, then the output staging
  uint8_t *const As = ab_s, *const Bs = ab_s + kI8BM * kI8Pitch;
  __shared__ __attribute__((aligned(16))) float sa_s[kI8Blocks][kI8BM];
  __shared__ __attribute__((aligned(16))) float sw_s[kI8Blocks][kI8BN];

  // workgroups id, id + 8, ... share an XCD: give them the M-tiles of the same weight panel
  uint32_t id = blockIdx.x, mt, nt;
  if (p.ntiles % 8 == 0) {
    const uint32_t xcd = id & 7, slot = id >> 3;
    nt = (slot / p.mtiles) * 8 + xcd;
    mt = slot % p.mtiles;
  } else {
    nt = id / p.mtiles;
    mt = id % p.mtiles;
  }
  const uint32_t m0 = mt * kI8BM, n0 = nt * kI8BN;
  const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
  const int wm = wave >> 1, wn = wave & 1;

  // staging assignment
  //   A: 128 rows x 8 vectors of 16 bytes = 1024 vectors, 4 per thread (row = idx >> 3, vector = idx & 7)
  //   B: 128 rows x 4 blocks = 512 blocks, 2 per thread (row = idx >> 2, block = idx & 3): 2 x 16 bytes + scale each
  //   a_scale: threads 0-127 take the four floats of one row
  i32x4 araw[4], braw[2][2];
  uint32_t bd[2], bkeep[2];
  f32x4 sraw = {0.0f, 0.0f, 0.0f, 0.0f};

  auto load_slice = [&](uint32_t kb0) {   // kb0: first block of the slice
#pragma unroll
    for (int v = 0; v < 4; ++v) {
      const int idx = v * 256 + tid;
      const uint32_t r = min(m0 + (uint32_t)(idx >> 3), p.M - 1);
      const uint32_t k = min(kb0 * 32u + (uint32_t)(idx & 7) * 16u, p.K - 16u);
      araw[v] = *reinterpret_cast<const i32x4 *>(p.qa + (size_t)r * p.K + k);
    }
#pragma unroll
    for (int v = 0; v < 2; ++v) {
      const int idx = v * 256 + tid;
      const uint32_t r = min(n0 + (uint32_t)(idx >> 2), p.N - 1);
      const uint32_t kb = kb0 + (uint32_t)(idx & 3);
      const uint8_t *blk = p.W + (size_t)r * p.row_bytes + (size_t)min(kb, p.nblk - 1) * 34;
      bd[v] = ld_u16(blk);
      // blocks past K get a zero scale (whatever the matrix core sums for them counts nothing): a mask applied where the
      // scale is used, since a select here would wait for the load, and every load before it, ahead of the MFMAs of
      // the slice that is meant to hide them
      bkeep[v] = kb < p.nblk ? 0xFFFFu : 0u;
      braw[v][0] = __builtin_bit_cast(i32x4, ld_u32x4(blk + 2));
      braw[v][1] = __builtin_bit_cast(i32x4, ld_u32x4(blk + 18));
    }
    if (tid < kI8BM) {
      const uint32_t r = min(m0 + (uint32_t)tid, p.M - 1);
      const float *s = p.sa + (size_t)r * p.nblk;
#pragma unroll
      for (int j = 0; j < kI8Blocks; ++j) sraw[j] = s[min(kb0 + (uint32_t)j, p.nblk - 1)];
    }
  };
  auto store_slice = [&]() {
#pragma unroll
    for (int v = 0; v < 4; ++v) {
      const int idx = v * 256 + tid;
      *reinterpret_cast<i32x4 *>(As + (idx >> 3) * kI8Pitch + (idx & 7) * 16) = araw[v];
    }
#pragma unroll
    for (int v = 0; v < 2; ++v) {
      const int idx = v * 256 + tid, row = idx >> 2, blk = idx & 3;
      *reinterpret_cast<i32x4 *>(Bs + row * kI8Pitch + blk * 32) = braw[v][0];
      *reinterpret_cast<i32x4 *>(Bs + row * kI8Pitch + blk * 32 + 16) = braw[v][1];
      sw_s[blk][row] = f16bits_to_f32(bd[v] & bkeep[v]);
    }
    if (tid < kI8BM) {
#pragma unroll
      for (int j = 0; j < kI8Blocks; ++j) sa_s[j][tid] = sraw[j];
    }
  };

  float acc[2][2][16];
#pragma unroll
  for (int i = 0; i < 2; ++i)
#pragma unroll
    for (int j = 0; j < 2; ++j)
#pragma unroll
      for (int r = 0; r < 16; ++r) acc[i][j][r] = 0.0f;

  // Operand layout of v_mfma_i32_32x32x32_i8: lane l supplies 16 consecutive k of row (column) l & 31, the half
  // l >> 5 of the 32.  A and B use the same map, and a block is summed whole by one MFMA, so only that matters.
  // Result register r of lane l: row 8 * (r / 4) + 4 * (l >> 5) + r % 4, column l & 31.
  auto mma_slice = [&]() {
    const uint8_t *a_base = As + (wm * 64 + (lane & 31)) * kI8Pitch + 16 * (lane >> 5);
    const uint8_t *b_base = Bs + (wn * 64 + (lane & 31)) * kI8Pitch + 16 * (lane >> 5);
#pragma unroll
    for (int b = 0; b < kI8Blocks; ++b) {
      i32x4 af[2], bf[2];
      float swj[2];
      f32x4 sar[2][4];
#pragma unroll
      for (int i = 0; i < 2; ++i) {
        af[i] = *reinterpret_cast<const i32x4 *>(a_base + 32 * i * kI8Pitch + 32 * b);
        bf[i] = *reinterpret_cast<const i32x4 *>(b_base + 32 * i * kI8Pitch + 32 * b);
        swj[i] = sw_s[b][wn * 64 + 32 * i + (lane & 31)];
#pragma unroll
        for (int q = 0; q < 4; ++q)
          sar[i][q] = *reinterpret_cast<const f32x4 *>(&sa_s[b][wm * 64 + 32 * i + 8 * q + 4 * (lane >> 5)]);
      }
#pragma unroll
      for (int i = 0; i < 2; ++i)
#pragma unroll
        for (int j = 0; j < 2; ++j) {
          const i32x16 zero = {0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0};
          const i32x16 d = __builtin_amdgcn_mfma_i32_32x32x32_i8(af[i], bf[j], zero, 0, 0, 0);
#pragma unroll
          for (int r = 0; r < 16; ++r)
            acc[i][j][r] = fmaf((float)d[r] * sar[i][r >> 2][r & 3], swj[j], acc[i][j][r]);
        }
    }
  };

  const uint32_t nslices = (p.nblk + kI8Blocks - 1) / kI8Blocks;
  load_slice(0);
  for (uint32_t t = 0; t < nslices; ++t) {
    __syncthreads();   // everyone is done reading the previous slice
    store_slice();
    __syncthreads();
    if (t + 1 < nslices) load_slice((t + 1) * kI8Blocks);
    mma_slice();
  }

  // C tile through LDS, a 32-row stripe of the wave's sub-tile at a time (gemm_store.hpp); the operand tiles are free
  // once every wave has multiplied the last slice
  static_assert(4 * stripe_floats<2>() * 4 <= (kI8BM + kI8BN) * kI8Pitch, "the output staging reuses the operand tiles");
  __syncthreads();
  lds_f32 *stage = (lds_f32 *)(lds_u8i *)(ab_s) + wave * stripe_floats<2>();
  const Epilogue epi = p.epi;
  const uint32_t Mrows = p.M, Ncols = p.N, ldc = p.strideC;
  void *const cbase = p.C;
  const int c_f16 = p.c_f16;
  const bool vec = p.vec_store != 0;
  // the common cases get the short store loops: no operator, or the residual add
  const int fast = !(vec && c_f16) ? 0 : epi.kind == CUTHIP_EPI_NONE ? 1
                   : (epi.kind == CUTHIP_EPI_BINARY && epi.op == CUTHIP_BINARY_ADD) ? 2 : 0;
  static_for<2>([&](auto ii) __attribute__((always_inline)) {
    constexpr int i = decltype(ii)::value;
    static_for<2>([&](auto jj) __attribute__((always_inline)) {
      constexpr int j = decltype(jj)::value;
      f32x16 t;
      static_for<16>([&](auto rr) __attribute__((always_inline)) { t[decltype(rr)::value] = acc[i][j][decltype(rr)::value]; });
      stage_tile32<2>(stage, j, t, lane);
    });
    if (fast == 1) store_staged32<2, 1>(stage, m0 + wm * 64 + 32 * i, n0 + wn * 64, Mrows, Ncols, cbase, ldc, c_f16, epi, vec, lane);
    else if (fast == 2) store_staged32<2, 2>(stage, m0 + wm * 64 + 32 * i, n0 + wn * 64, Mrows, Ncols, cbase, ldc, c_f16, epi, vec, lane);
    else store_staged32<2, 0>(stage, m0 + wm * 64 + 32 * i, n0 + wn * 64, Mrows, Ncols, cbase, ldc, c_f16, epi, vec, lane);
  });
}

static size_t q8_i8_qa_bytes(uint32_t M, uint32_t K) { return ((size_t)M * K + 255) & ~(size_t)255; }

}  // namespace cuthip

using namespace cuthip;

extern "C" {

size_t cuthip_matmul_q8_i8_workspace_bytes(uint32_t M, uint32_t K) {
  return q8_i8_qa_bytes(M, K) + (size_t)M * (K / 32) * sizeof(float);
}

int cuthip_matmul_q8_i8(const void *W, const void *A, int a_dtype, void *C, int c_dtype, uint32_t M, uint32_t K, uint32_t N,
                        uint32_t strideA, uint32_t strideC, int epilogue, int epilogue_op, const void *D, void *workspace,
                        size_t workspace_bytes, void *stream) {
  if (M == 0 || N == 0) return CUTHIP_OK;
  if (!W || !A || !C) {
    set_error("cuthip_matmul_q8_i8: null pointer");
    return CUTHIP_ERR_INVALID;
  }
  if ((a_dtype != CUTHIP_F32 && a_dtype != CUTHIP_F16) || (c_dtype != CUTHIP_F32 && c_dtype != CUTHIP_F16)) {
    set_error("cuthip_matmul_q8_i8: dtypes must be fp32 or fp16");
    return CUTHIP_ERR_INVALID;
  }
  if (K == 0 || K % 32 != 0 || strideA < K || strideC < N) {
    set_error("cuthip_matmul_q8_i8: K = %u must be a positive multiple of 32 (the Q8_0 block), strideA >= K, strideC >= N", K);
    return CUTHIP_ERR_INVALID;
  }
  if (epilogue != CUTHIP_EPI_NONE && epilogue != CUTHIP_EPI_UNARY && epilogue != CUTHIP_EPI_BINARY) {
    set_error("cuthip_matmul_q8_i8: epilogue %d is not supported here", epilogue);
    return CUTHIP_ERR_INVALID;
  }
  if (epilogue == CUTHIP_EPI_BINARY && !D) {
    set_error("cuthip_matmul_q8_i8: binary epilogue without D");
    return CUTHIP_ERR_INVALID;
  }
  if (int rc = check_epilogue_op("cuthip_matmul_q8_i8", epilogue, epilogue_op)) return rc;
  if (epilogue_op_long(epilogue, epilogue_op)) {
    if (int rc = check_long_epilogue_alias(epilogue, epilogue_op, C, D)) return rc;   // before anything is written
    if (int rc = cuthip_matmul_q8_i8(W, A, a_dtype, C, c_dtype, M, K, N, strideA, strideC, CUTHIP_EPI_NONE, 0, nullptr, workspace,
                                     workspace_bytes, stream))
      return rc;
    return launch_long_epilogue(C, c_dtype == CUTHIP_F16, M, N, strideC, epilogue, epilogue_op, D, (hipStream_t)stream);
  }
  const size_t need = cuthip_matmul_q8_i8_workspace_bytes(M, K);
  if (!workspace || workspace_bytes < need || (reinterpret_cast<uintptr_t>(workspace) & 15u)) {
    set_error("cuthip_matmul_q8_i8: workspace of %zu bytes (16-byte aligned) needed, got %zu", need, workspace_bytes);
    return CUTHIP_ERR_INVALID;
  }
  const size_t a_align = a_dtype == CUTHIP_F16 ? 8 : 16;   // 4 elements per lane
  if ((reinterpret_cast<uintptr_t>(A) & (a_align - 1)) || (strideA & 3u)) {
    set_error("cuthip_matmul_q8_i8: A must be aligned to 4 elements and strideA a multiple of 4");
    return CUTHIP_ERR_INVALID;
  }
  hipStream_t s = (hipStream_t)stream;
  int8_t *qa = reinterpret_cast<int8_t *>(workspace);
  float *sa = reinterpret_cast<float *>(reinterpret_cast<uint8_t *>(workspace) + q8_i8_qa_bytes(M, K));
  const uint64_t lanes = (uint64_t)M * (K / 32) * 8, wgs = (lanes + 255) / 256;
  const uint64_t tiles = (uint64_t)((M + kI8BM - 1) / kI8BM) * ((N + kI8BN - 1) / kI8BN);
  if (wgs > 0x7FFFFFFFull || tiles > 0x7FFFFFFFull) {
    set_error("cuthip_matmul_q8_i8: problem too large for one launch");
    return CUTHIP_ERR_INVALID;
  }
  if (a_dtype == CUTHIP_F16)
    hipLaunchKernelGGL(quantize_act_kernel<true>, dim3((uint32_t)wgs), dim3(256), 0, s, A, M, K, strideA, qa, sa);
  else
    hipLaunchKernelGGL(quantize_act_kernel<false>, dim3((uint32_t)wgs), dim3(256), 0, s, A, M, K, strideA, qa, sa);
  if (int rc = check_hip(hipGetLastError(), "activation quantizer launch")) return rc;
  I8Params p;
  p.W = reinterpret_cast<const uint8_t *>(W);
  p.qa = qa;
  p.sa = sa;
  p.C = C;
  p.epi = Epilogue{epilogue, epilogue_op, D};
  p.M = M; p.K = K; p.N = N; p.strideC = strideC;
  p.nblk = K / 32;
  p.row_bytes = p.nblk * 34;
  p.mtiles = (M + kI8BM - 1) / kI8BM;
  p.ntiles = (N + kI8BN - 1) / kI8BN;
  p.c_f16 = c_dtype == CUTHIP_F16;
  p.vec_store = store8_aligned(C, strideC, p.c_f16, p.epi) ? 1 : 0;
  hipLaunchKernelGGL(gemm_q8_i8_kernel, dim3((uint32_t)tiles), dim3(256), 0, s, p);
  return check_hip(hipGetLastError(), "int8 gemm launch");
}

}  // extern "C"
