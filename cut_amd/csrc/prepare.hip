// Load-time weight preparation on the GPU, for callers that keep the reference's
// separated [K, N] weight layout (cuthip_matmul_q8_sep / cuthip_matmul_q4_sep):
//   * GGUF blocks -> transposed separated tensors in one launch.  The reference
//     splits the blocks on the host (read_tensor_q8_separated / _q4_separated,
//     gguf_reader.cpp:389-501), uploads them and transposes on the GPU
//     (TransposeQ4Nibble.cu:17-61 for the nibbles, a generic transpose for the
//     int8 values and the scales; llama.cpp:940-965).
//   * Q4_K -> affine Q4 (requantizeQ4KToAffine, llama.cpp:573-619): per 32
//     elements scale = f16(d * sc), min = f16(8 * (d * sc) - dmin * m) (from the
//     unrounded scale), nibbles kept, written in the [K, N/2] orientation.
//   * fp32 rows -> Q8_0 blocks (quantizeRowsQ8_0, llama.cpp:488-505).
//
// All of it is byte shuffling bound by HBM.  A workgroup copies the block runs
// of 128 weight rows into LDS with coalesced 2-byte loads (GGUF blocks are only
// 2-byte aligned; the LDS image pads every block so that its quants are dword
// aligned), then every thread reads one dword (four consecutive k) of 4 (int8)
// or 8 (nibble) neighbouring rows, transposes the 4 x 4 bytes with v_perm_b32
// and writes four dwords, so the transposed rows are written in runs of 128
// (64) bytes.
#include <cstdint>

#include "common.hpp"

namespace cuthip {

constexpr int kPrepRows = 128;      // weight rows per tile
constexpr int kPrepThreads = 256;

enum PrepMode { PREP_Q8_0 = 0, PREP_Q4_0 = 1, PREP_Q4_K_AFFINE = 2, PREP_NIBBLES = 3 };

// k extent of a tile and the bytes one weight row contributes to it
template <int MODE> struct PrepGeom;
template <> struct PrepGeom<PREP_Q8_0> { static constexpr int KT = 128, RUN = 4 * 34, PITCH = 4 * 36 + 4; };
template <> struct PrepGeom<PREP_Q4_0> { static constexpr int KT = 256, RUN = 8 * 18, PITCH = 8 * 20 + 4; };
template <> struct PrepGeom<PREP_Q4_K_AFFINE> { static constexpr int KT = 256, RUN = 144, PITCH = RUN; };
template <> struct PrepGeom<PREP_NIBBLES> { static constexpr int KT = 256, RUN = 128, PITCH = RUN + 4; };

struct PrepParams {
  const uint8_t *src;
  uint8_t *B;
  uint16_t *S;
  uint32_t N, K, strideB, scaleStride;
  uint32_t src_row_bytes;
};

// Where the quant byte of element k (a multiple of 4) of a row sits in its LDS image, and the shift that brings its
// nibble down.  Q4_K: piece g = k / 64, low nibbles are its first 32 elements, high nibbles the rest.  GGML Q4_0 order
// (also the packed tensor of the separated reader): low nibble of byte j of a block is element j, high nibble element
// j + 16.  The Q4_0 image keeps each block at 20 bytes ([d][2 bytes unused][qs:16]) so that the quants are dword aligned.
template <int MODE> __device__ inline uint32_t prep_quant_offset(uint32_t k) {
  if (MODE == PREP_Q4_K_AFFINE) return 16 + 32 * (k >> 6) + (k & 31);
  if (MODE == PREP_Q4_0) return (k >> 5) * 20 + 4 + (k & 15);
  return (k >> 5) * 16 + (k & 15);
}
template <int MODE> __device__ inline uint32_t prep_quant_shift(uint32_t k) {
  return MODE == PREP_Q4_K_AFFINE ? ((k & 32) ? 4u : 0u) : ((k & 16) ? 4u : 0u);
}

template <int MODE> __global__ void __launch_bounds__(kPrepThreads) prepare_sep_kernel(PrepParams p) {
  using G = PrepGeom<MODE>;
  __shared__ __attribute__((aligned(16))) uint8_t raw[kPrepRows * G::PITCH];
  const uint32_t tid = threadIdx.x;
  const uint32_t n0 = blockIdx.x * kPrepRows, k0 = blockIdx.y * G::KT;
  const uint32_t run_off = blockIdx.y * G::RUN;
  const uint32_t valid = min((uint32_t)G::RUN, p.src_row_bytes - run_off);   // the last tile of a row may be short
  constexpr uint32_t W = G::RUN / 2;
  for (uint32_t i = tid; i < kPrepRows * W; i += kPrepThreads) {
    const uint32_t row = i / W, w = i - row * W, n = n0 + row;
    uint16_t v = 0;
    if (n < p.N && 2 * w < valid) v = (uint16_t)ld_u16(p.src + (size_t)n * p.src_row_bytes + run_off + 2 * w);
    uint32_t dst = 2 * w;
    if (MODE == PREP_Q4_0) dst = (w / 9) * 20 + ((w % 9) ? 2 * (w % 9) + 2 : 0);   // scale at 0, quants from byte 4
    if (MODE == PREP_Q8_0) dst = (w / 17) * 36 + ((w % 17) ? 2 * (w % 17) + 2 : 0);  // [d][2 bytes unused][q:32]
    *reinterpret_cast<uint16_t *>(raw + row * G::PITCH + dst) = v;
  }
  __syncthreads();
  const uint32_t kt = min((uint32_t)G::KT, p.K - k0);

  if constexpr (MODE == PREP_Q8_0) {
    // item = (4 consecutive k, 4 rows): one dword of LDS per row (the image keeps every block at 36 bytes so that the
    // quants are dword aligned), a 4 x 4 byte transpose, four dwords B[k + i, n .. n+3]
    const bool words = (p.strideB & 3u) == 0;
    for (uint32_t i = tid; i < (uint32_t)(G::KT / 4) * (kPrepRows / 4); i += kPrepThreads) {
      const uint32_t k = (i / (kPrepRows / 4)) * 4, r4 = (i % (kPrepRows / 4)) * 4, n = n0 + r4;
      if (k >= kt || n >= p.N) continue;
      const uint32_t off = (k >> 5) * 36 + 4 + (k & 31);
      uint32_t pr[4];
#pragma unroll
      for (int j = 0; j < 4; ++j) pr[j] = *reinterpret_cast<const uint32_t *>(raw + (r4 + j) * G::PITCH + off);
      const uint32_t t0 = __builtin_amdgcn_perm(pr[1], pr[0], 0x05010400u), t1 = __builtin_amdgcn_perm(pr[3], pr[2], 0x05010400u);
      const uint32_t t2 = __builtin_amdgcn_perm(pr[1], pr[0], 0x07030602u), t3 = __builtin_amdgcn_perm(pr[3], pr[2], 0x07030602u);
      const uint32_t out[4] = {__builtin_amdgcn_perm(t1, t0, 0x05040100u), __builtin_amdgcn_perm(t1, t0, 0x07060302u),
                               __builtin_amdgcn_perm(t3, t2, 0x05040100u), __builtin_amdgcn_perm(t3, t2, 0x07060302u)};
#pragma unroll
      for (uint32_t e = 0; e < 4; ++e) {
        if (k + e >= kt) break;
        uint8_t *dst = p.B + (size_t)(k0 + k + e) * p.strideB + n;
        if (words && n + 3 < p.N) {
          *reinterpret_cast<uint32_t *>(dst) = out[e];
        } else {
          for (uint32_t j = 0; j < 4 && n + j < p.N; ++j) dst[j] = (uint8_t)(out[e] >> (8 * j));
        }
      }
    }
    for (uint32_t i = tid; i < (G::KT / 32) * kPrepRows; i += kPrepThreads) {
      const uint32_t blk = i / kPrepRows, row = i % kPrepRows, n = n0 + row;
      if (n < p.N && blk * 32 < kt)
        p.S[(size_t)(k0 / 32 + blk) * p.scaleStride + n] = *reinterpret_cast<const uint16_t *>(raw + row * G::PITCH + blk * 36);
    }
  } else {
    // item = (4 consecutive k, 8 rows): one dword of LDS per row holds the four quants (k .. k+3 share a nibble half
    // and four neighbouring bytes), row pairs are merged into bytes (even row in the low nibble) and a 4 x 4 byte
    // transpose (v_perm_b32) turns [row pair][k] into the four output dwords B[k + i, n/2 .. n/2+3]
    const bool words = (p.strideB & 3u) == 0;
    for (uint32_t i = tid; i < (uint32_t)(G::KT / 4) * (kPrepRows / 8); i += kPrepThreads) {
      const uint32_t k = (i / (kPrepRows / 8)) * 4, r8 = (i % (kPrepRows / 8)) * 8, n = n0 + r8;
      if (k >= kt || n >= p.N) continue;
      const uint32_t off = prep_quant_offset<MODE>(k), sh = prep_quant_shift<MODE>(k);
      uint32_t pr[4];
#pragma unroll
      for (int j = 0; j < 4; ++j) {
        const uint32_t lo = (*reinterpret_cast<const uint32_t *>(raw + (r8 + 2 * j) * G::PITCH + off) >> sh) & 0x0F0F0F0Fu;
        const uint32_t hi = (*reinterpret_cast<const uint32_t *>(raw + (r8 + 2 * j + 1) * G::PITCH + off) >> sh) & 0x0F0F0F0Fu;
        pr[j] = lo | (hi << 4);   // byte i: rows (r8 + 2j, r8 + 2j + 1) at k + i; rows past N are zero
      }
      const uint32_t t0 = __builtin_amdgcn_perm(pr[1], pr[0], 0x05010400u), t1 = __builtin_amdgcn_perm(pr[3], pr[2], 0x05010400u);
      const uint32_t t2 = __builtin_amdgcn_perm(pr[1], pr[0], 0x07030602u), t3 = __builtin_amdgcn_perm(pr[3], pr[2], 0x07030602u);
      const uint32_t out[4] = {__builtin_amdgcn_perm(t1, t0, 0x05040100u), __builtin_amdgcn_perm(t1, t0, 0x07060302u),
                               __builtin_amdgcn_perm(t3, t2, 0x05040100u), __builtin_amdgcn_perm(t3, t2, 0x07060302u)};
#pragma unroll
      for (uint32_t e = 0; e < 4; ++e) {
        if (k + e >= kt) break;
        uint8_t *dst = p.B + (size_t)(k0 + k + e) * p.strideB + n / 2;
        if (words && n + 7 < p.N) {
          *reinterpret_cast<uint32_t *>(dst) = out[e];
        } else {
          for (uint32_t j = 0; j < 4 && n + 2 * j < p.N; ++j) dst[j] = (uint8_t)(out[e] >> (8 * j));
        }
      }
    }
    if constexpr (MODE == PREP_Q4_0) {
      for (uint32_t i = tid; i < (G::KT / 32) * kPrepRows; i += kPrepThreads) {
        const uint32_t blk = i / kPrepRows, row = i % kPrepRows, n = n0 + row;
        if (n < p.N && blk * 32 < kt)
          p.S[(size_t)(k0 / 32 + blk) * p.scaleStride + n] = *reinterpret_cast<const uint16_t *>(raw + row * G::PITCH + blk * 20);
      }
    }
    if constexpr (MODE == PREP_Q4_K_AFFINE) {
      const uint32_t blocksK = p.K / 32;
      for (uint32_t i = tid; i < 8 * kPrepRows; i += kPrepThreads) {
        const uint32_t j = i / kPrepRows, row = i % kPrepRows, n = n0 + row;
        if (n >= p.N) continue;
        const uint8_t *r = raw + row * G::PITCH, *q = r + 4;
        const float d = f16bits_to_f32(*reinterpret_cast<const uint16_t *>(r));
        const float dmin = f16bits_to_f32(*reinterpret_cast<const uint16_t *>(r + 2));
        uint32_t sc, m;   // get_scale_min_k4 (llama.cpp:547-555)
        if (j < 4) {
          sc = q[j] & 63u;
          m = q[j + 4] & 63u;
        } else {
          sc = (q[j + 4] & 15u) | ((uint32_t)(q[j - 4] >> 6) << 4);
          m = (uint32_t)(q[j + 4] >> 4) | ((uint32_t)(q[j] >> 6) << 4);
        }
        // both products are exact in fp32 (11 x 6 bits), so the subtraction is the only rounding whether or not it is fused
        const float scale = d * (float)sc;
        const float minv = 8.0f * scale - dmin * (float)m;
        const size_t b = k0 / 32 + j;
        p.S[b * p.scaleStride + n] = (uint16_t)f32_to_f16bits_any(scale);
        p.S[(blocksK + b) * p.scaleStride + n] = (uint16_t)f32_to_f16bits_any(minv);
      }
    }
  }
}

template <int MODE> static int launch_prepare(const PrepParams &p, hipStream_t stream) {
  using G = PrepGeom<MODE>;
  dim3 grid((p.N + kPrepRows - 1) / kPrepRows, (p.K + G::KT - 1) / G::KT);
  if (grid.y > 65535u) {
    set_error("prepare: K = %u is too long for one launch", p.K);
    return CUTHIP_ERR_INVALID;
  }
  hipLaunchKernelGGL(prepare_sep_kernel<MODE>, grid, dim3(kPrepThreads), 0, stream, p);
  return check_hip(hipGetLastError(), "prepare launch");
}

// 8 lanes per block of 32 values: 16-byte loads, absmax folded over the 8 lanes, one dword of int8 per lane
__global__ void __launch_bounds__(256) quantize_q8_0_kernel(const float *x, uint64_t nblocks, uint8_t *blocks) {
  const uint64_t t = (uint64_t)blockIdx.x * 256u + threadIdx.x, b = t >> 3;
  const uint32_t i = (uint32_t)t & 7u;
  const bool ok = b < nblocks;
  f32x4 v = {0.0f, 0.0f, 0.0f, 0.0f};
  if (ok) v = *reinterpret_cast<const f32x4 *>(x + b * 32 + i * 4);
  float amax = fmaxf(fmaxf(fabsf(v.x), fabsf(v.y)), fmaxf(fabsf(v.z), fabsf(v.w)));
  amax = fmaxf(amax, __shfl_xor(amax, 1));
  amax = fmaxf(amax, __shfl_xor(amax, 2));
  amax = fmaxf(amax, __shfl_xor(amax, 4));
  const float d = amax / 127.0f;                      // correctly rounded fp32 division, as on the host
  const float id = d != 0.0f ? 1.0f / d : 0.0f;
  // lroundf: half away from zero; |x * id| <= 127 * (1 + 2^-22), so the cast cannot overflow int8
  const uint32_t q0 = (uint32_t)(int)roundf(v.x * id) & 0xFFu, q1 = (uint32_t)(int)roundf(v.y * id) & 0xFFu;
  const uint32_t q2 = (uint32_t)(int)roundf(v.z * id) & 0xFFu, q3 = (uint32_t)(int)roundf(v.w * id) & 0xFFu;
  if (!ok) return;
  uint8_t *blk = blocks + b * 34;
  uint16_t *dst = reinterpret_cast<uint16_t *>(blk + 2 + 4 * i);   // blocks are 2-byte aligned
  dst[0] = (uint16_t)(q0 | (q1 << 8));
  dst[1] = (uint16_t)(q2 | (q3 << 8));
  if (i == 0) *reinterpret_cast<uint16_t *>(blk) = (uint16_t)f32_to_f16bits_any(d);
}

}  // namespace cuthip

using namespace cuthip;

extern "C" {

int cuthip_prepare_sep(int fmt, const void *blocks, uint32_t N, uint32_t K, void *B, uint32_t strideB, uint16_t *scales,
                       uint32_t scaleStride, void *stream) {
  if (!blocks || !B || !scales) {
    set_error("cuthip_prepare_sep: null pointer");
    return CUTHIP_ERR_INVALID;
  }
  if (fmt != CUTHIP_Q8_0 && fmt != CUTHIP_Q4_0 && fmt != CUTHIP_Q4_K) {
    set_error("cuthip_prepare_sep: format %d has no separated layout (Q8_0, Q4_0 and Q4_K -> affine Q4 do)", fmt);
    return CUTHIP_ERR_INVALID;
  }
  if (N == 0 || K == 0 || K % (uint32_t)fmt_elems(fmt) != 0) {
    set_error("cuthip_prepare_sep: K = %u must be a positive multiple of %d, N = %u positive", K, fmt_elems(fmt), N);
    return CUTHIP_ERR_INVALID;
  }
  const bool q4 = fmt != CUTHIP_Q8_0;
  if (q4 && (N & 1u)) {   // TransposeQ4NibbleOp.cpp:13-15, llama.cpp:576
    set_error("cuthip_prepare_sep: N = %u must be even for packed nibbles", N);
    return CUTHIP_ERR_INVALID;
  }
  if (strideB < (q4 ? N / 2 : N) || scaleStride < N) {
    set_error("cuthip_prepare_sep: strideB = %u / scaleStride = %u shorter than a row of N = %u", strideB, scaleStride, N);
    return CUTHIP_ERR_INVALID;
  }
  if ((reinterpret_cast<uintptr_t>(B) & 3u) || (reinterpret_cast<uintptr_t>(scales) & 1u) ||
      (reinterpret_cast<uintptr_t>(blocks) & 1u)) {
    set_error("cuthip_prepare_sep: B must be 4-byte aligned, blocks and scales 2-byte aligned");
    return CUTHIP_ERR_INVALID;
  }
  PrepParams p;
  p.src = reinterpret_cast<const uint8_t *>(blocks);
  p.B = reinterpret_cast<uint8_t *>(B);
  p.S = scales;
  p.N = N; p.K = K; p.strideB = strideB; p.scaleStride = scaleStride;
  p.src_row_bytes = K / (uint32_t)fmt_elems(fmt) * (uint32_t)fmt_bytes(fmt);
  if (fmt == CUTHIP_Q8_0) return launch_prepare<PREP_Q8_0>(p, (hipStream_t)stream);
  if (fmt == CUTHIP_Q4_0) return launch_prepare<PREP_Q4_0>(p, (hipStream_t)stream);
  return launch_prepare<PREP_Q4_K_AFFINE>(p, (hipStream_t)stream);
}

int cuthip_transpose_q4_nibble(const void *packed, void *packedT, uint32_t N, uint32_t K, uint32_t strideInHalf,
                               uint32_t strideOutHalf, void *stream) {
  if (!packed || !packedT) {
    set_error("cuthip_transpose_q4_nibble: null pointer");
    return CUTHIP_ERR_INVALID;
  }
  if (N == 0 || (N & 1u)) {
    set_error("TransposeQ4: N must be even");
    return CUTHIP_ERR_INVALID;
  }
  if (K == 0 || K % 32 != 0) {
    set_error("TransposeQ4: K must be a multiple of 32");
    return CUTHIP_ERR_INVALID;
  }
  if (strideInHalf < K / 2 || (strideInHalf & 1u) || strideOutHalf < N / 2) {
    set_error("cuthip_transpose_q4_nibble: strideInHalf = %u (even, >= K/2) / strideOutHalf = %u (>= N/2) do not fit", strideInHalf,
              strideOutHalf);
    return CUTHIP_ERR_INVALID;
  }
  if ((reinterpret_cast<uintptr_t>(packedT) & 3u) || (reinterpret_cast<uintptr_t>(packed) & 1u)) {
    set_error("cuthip_transpose_q4_nibble: output must be 4-byte aligned, input 2-byte aligned");
    return CUTHIP_ERR_INVALID;
  }
  PrepParams p;
  p.src = reinterpret_cast<const uint8_t *>(packed);
  p.B = reinterpret_cast<uint8_t *>(packedT);
  p.S = nullptr;
  p.N = N; p.K = K; p.strideB = strideOutHalf; p.scaleStride = 0;
  p.src_row_bytes = strideInHalf;
  // a tile reads 128 bytes of each row; only K / 2 of a padded row are nibbles, the kernel stops at K
  return launch_prepare<PREP_NIBBLES>(p, (hipStream_t)stream);
}

int cuthip_quantize_rows_q8_0(const float *x, uint64_t n, void *blocks, void *stream) {
  if (!x || !blocks) {
    set_error("cuthip_quantize_rows_q8_0: null pointer");
    return CUTHIP_ERR_INVALID;
  }
  if (n == 0 || n % 32 != 0) {
    set_error("cuthip_quantize_rows_q8_0: n = %llu must be a positive multiple of 32", (unsigned long long)n);
    return CUTHIP_ERR_INVALID;
  }
  if ((reinterpret_cast<uintptr_t>(x) & 15u) || (reinterpret_cast<uintptr_t>(blocks) & 1u)) {
    set_error("cuthip_quantize_rows_q8_0: x must be 16-byte aligned, blocks 2-byte aligned");
    return CUTHIP_ERR_INVALID;
  }
  const uint64_t nblocks = n / 32, wgs = (nblocks * 8 + 255) / 256;
  if (wgs > 0x7FFFFFFFull) {
    set_error("cuthip_quantize_rows_q8_0: n = %llu is too large for one launch", (unsigned long long)n);
    return CUTHIP_ERR_INVALID;
  }
  hipLaunchKernelGGL(quantize_q8_0_kernel, dim3((uint32_t)wgs), dim3(256), 0, (hipStream_t)stream, x, nblocks,
                     reinterpret_cast<uint8_t *>(blocks));
  return check_hip(hipGetLastError(), "quantize launch");
}

}  // extern "C"
