/*
 * CPU oracle for the GGUF quantized-matmul path -- TEST INFRASTRUCTURE ONLY.
 * See cut_oracle.h for the rules of use and the parity status of every
 * function.  Build: gcc -O2 -ffp-contract=off (the reference is built -O3
 * for baseline x86-64, i.e. separate multiply and add; CMakeLists.txt:29-30).
 */
#include "cut_oracle.h"

#include <math.h>
#include <stdlib.h>
#include <string.h>

size_t orc_block_elems(int fmt) {
  switch (fmt) {
  case ORC_Q8_0:
  case ORC_Q4_0:
    return 32;
  case ORC_Q4_K:
  case ORC_Q6_K:
    return 256;
  }
  return 0;
}

size_t orc_block_bytes(int fmt) {
  switch (fmt) { /* gguf_types.hpp:109-142 */
  case ORC_Q8_0:
    return 34;
  case ORC_Q4_0:
    return 18;
  case ORC_Q4_K:
    return 144;
  case ORC_Q6_K:
    return 210;
  }
  return 0;
}

/* ---- half conversions -------------------------------------------------- */

/* gguf_reader.cpp:515-539.  Subnormals are mant * 2^-24 (exact), Inf kept,
 * every NaN becomes the canonical NAN constant. */
float orc_f16_to_f32(uint16_t h) {
  uint32_t sign = (uint32_t)(h & 0x8000u) << 16;
  uint32_t exponent = (h & 0x7C00u) >> 10;
  uint32_t mantissa = (uint32_t)(h & 0x03FFu) << 13;
  float result;
  if (exponent == 0) {
    if (mantissa == 0) {
      memcpy(&result, &sign, sizeof(result));
      return result;
    }
    result = (float)(h & 0x03FF) * 5.960464477539063e-08f;
    return (h & 0x8000) ? -result : result;
  }
  if (exponent == 31)
    return mantissa ? NAN : ((h & 0x8000) ? -INFINITY : INFINITY);
  uint32_t bits = sign | ((exponent + 112u) << 23) | mantissa;
  memcpy(&result, &bits, sizeof(result));
  return result;
}

/* llama.cpp:445-482.  Round half up in magnitude on the dropped bits,
 * subnormals encoded, overflow and NaN clamp to +-Inf. */
uint16_t orc_f32_to_f16(float v) {
  uint32_t u;
  memcpy(&u, &v, sizeof(u));
  uint32_t sign = (u >> 16) & 0x8000u;
  int32_t exp = (int32_t)((u >> 23) & 0xffu) - 127 + 15;
  uint32_t mantissa = u & 0x7fffffu;
  if (exp <= 0) {
    uint32_t shift = (uint32_t)(14 - exp);
    if (shift > 24)
      return (uint16_t)sign;
    uint32_t significand = 0x800000u | mantissa;
    uint32_t half = significand >> shift;
    if ((significand >> (shift - 1)) & 1u)
      ++half;
    return (uint16_t)(sign | half);
  }
  if (exp >= 31)
    return (uint16_t)(sign | 0x7c00u);
  uint32_t m = mantissa >> 13;
  if (mantissa & 0x1000u) {
    ++m;
    if (m == 0x400u) {
      m = 0;
      ++exp;
      if (exp >= 31)
        return (uint16_t)(sign | 0x7c00u);
    }
  }
  return (uint16_t)(sign | ((uint32_t)exp << 10) | m);
}

/* llama.cpp:512-542.  Same values as orc_f16_to_f32 on non-NaN inputs; NaN
 * payload and sign are carried through. */
float orc_runner_f16_to_f32(uint16_t h) {
  uint32_t sign = (uint32_t)(h & 0x8000u) << 16;
  uint32_t exp = (h >> 10) & 0x1Fu;
  uint32_t man = h & 0x03FFu;
  uint32_t bits;
  if (exp == 0) {
    if (man == 0) {
      bits = sign;
    } else {
      uint32_t e = 113;
      while ((man & 0x0400u) == 0) {
        man <<= 1;
        --e;
      }
      man &= 0x03FFu;
      bits = sign | (e << 23) | (man << 13);
    }
  } else if (exp == 31) {
    bits = sign | 0x7F800000u | (man << 13);
  } else {
    bits = sign | ((exp + 112u) << 23) | (man << 13);
  }
  float out;
  memcpy(&out, &bits, sizeof(out));
  return out;
}

/* OpRefs.h:164-177: truncates the mantissa, flushes subnormals. */
uint16_t orc_harness_f32_to_f16(float value) {
  uint32_t f32;
  memcpy(&f32, &value, sizeof(f32));
  uint32_t sign = (f32 >> 16) & 0x8000;
  int32_t exponent = (int32_t)((f32 >> 23) & 0xFF) - 127 + 15;
  uint32_t mantissa = (f32 >> 13) & 0x03FF;
  if (exponent <= 0)
    return (uint16_t)sign;
  if (exponent >= 31)
    return (uint16_t)(sign | 0x7C00);
  return (uint16_t)(sign | ((uint32_t)exponent << 10) | mantissa);
}

void orc_f16_to_f32_array(const uint16_t *h, size_t n, float *out) {
  for (size_t i = 0; i < n; ++i)
    out[i] = orc_f16_to_f32(h[i]);
}
void orc_f32_to_f16_array(const float *v, size_t n, uint16_t *out) {
  for (size_t i = 0; i < n; ++i)
    out[i] = orc_f32_to_f16(v[i]);
}
void orc_runner_f16_to_f32_array(const uint16_t *h, size_t n, float *out) {
  for (size_t i = 0; i < n; ++i)
    out[i] = orc_runner_f16_to_f32(h[i]);
}

/* gguf_reader.cpp:668-676 (and llama.cpp:547-555, the same map). */
void orc_get_scale_min_k4(int j, const uint8_t *q, uint8_t *sc, uint8_t *m) {
  if (j < 4) {
    *sc = q[j] & 63;
    *m = q[j + 4] & 63;
  } else {
    *sc = (uint8_t)((q[j + 4] & 0xF) | ((q[j - 4] >> 6) << 4));
    *m = (uint8_t)((q[j + 4] >> 4) | ((q[j] >> 6) << 4));
  }
}

/* ---- dequantizers ------------------------------------------------------ */

/* gguf_reader.cpp:826-850 */
void orc_dequant_q8_0(const uint8_t *data, float *out, size_t n) {
  size_t n_blocks = (n + 31) / 32, offset = 0, o = 0;
  for (size_t i = 0; i < n_blocks && o < n; ++i) {
    uint16_t bits;
    memcpy(&bits, data + offset, 2);
    offset += 2;
    float scale = orc_f16_to_f32(bits);
    for (size_t j = 0; j < 32 && o < n; ++j) {
      int8_t val = (int8_t)data[offset + j];
      out[o++] = (float)val * scale;
    }
    offset += 32;
  }
}

/* gguf_reader.cpp:541-572: low nibbles -> first half, high -> second half. */
void orc_dequant_q4_0(const uint8_t *data, float *out, size_t n) {
  size_t n_blocks = (n + 31) / 32, offset = 0;
  for (size_t i = 0; i < n_blocks; ++i) {
    uint16_t bits;
    memcpy(&bits, data + offset, 2);
    offset += 2;
    float scale = orc_f16_to_f32(bits);
    size_t base = i * 32;
    for (size_t j = 0; j < 16; ++j) {
      uint8_t byte = data[offset + j];
      int x0 = (byte & 0x0F) - 8;
      int x1 = ((byte >> 4) & 0x0F) - 8;
      if (base + j < n)
        out[base + j] = (float)x0 * scale;
      if (base + j + 16 < n)
        out[base + j + 16] = (float)x1 * scale;
    }
    offset += 16;
  }
}

/* gguf_reader.cpp:678-724: [d][dmin][scales:12][qs:128]; per 64-element pair
 * two exact products and one subtraction. */
void orc_dequant_q4_k(const uint8_t *data, float *out, size_t n) {
  size_t n_blocks = (n + 255) / 256, o = 0;
  for (size_t i = 0; i < n_blocks && o < n; ++i) {
    const uint8_t *block = data + i * 144;
    uint16_t d_bits, dmin_bits;
    memcpy(&d_bits, block, 2);
    memcpy(&dmin_bits, block + 2, 2);
    float d = orc_f16_to_f32(d_bits);
    float dmin = orc_f16_to_f32(dmin_bits);
    const uint8_t *scales = block + 4;
    const uint8_t *qs = block + 16;
    int is = 0;
    for (int j = 0; j < 256 && o < n; j += 64) {
      uint8_t sc1, m1, sc2, m2;
      orc_get_scale_min_k4(is, scales, &sc1, &m1);
      float d1 = d * sc1;
      float dm1 = dmin * m1;
      orc_get_scale_min_k4(is + 1, scales, &sc2, &m2);
      float d2 = d * sc2;
      float dm2 = dmin * m2;
      for (int l = 0; l < 32 && o < n; ++l)
        out[o++] = d1 * (qs[l] & 0xF) - dm1;
      for (int l = 0; l < 32 && o < n; ++l)
        out[o++] = d2 * ((qs[l] >> 4) & 0xF) - dm2;
      qs += 32;
      is += 2;
    }
  }
}

/* gguf_reader.cpp:774-824: [ql:128][qh:64][sc:16 x i8][d]; two halves of 128,
 * each 32 columns x 4 quarters; product order (d * sc) * q. */
void orc_dequant_q6_k(const uint8_t *data, float *out, size_t n) {
  size_t n_blocks = (n + 255) / 256, o = 0;
  for (size_t i = 0; i < n_blocks && o < n; ++i) {
    const uint8_t *block = data + i * 210;
    const uint8_t *ql = block;
    const uint8_t *qh = block + 128;
    const int8_t *sc = (const int8_t *)(block + 192);
    uint16_t d_bits;
    memcpy(&d_bits, block + 208, 2);
    float d = orc_f16_to_f32(d_bits);
    for (int h = 0; h < 256 && o < n; h += 128) {
      for (int l = 0; l < 32 && o + 96 + (size_t)l <= n; ++l) {
        int is = l / 16;
        int8_t q1 = (int8_t)((int8_t)((ql[l] & 0xF) | (((qh[l] >> 0) & 3) << 4)) - 32);
        int8_t q2 = (int8_t)((int8_t)((ql[l + 32] & 0xF) | (((qh[l] >> 2) & 3) << 4)) - 32);
        int8_t q3 = (int8_t)((int8_t)((ql[l] >> 4) | (((qh[l] >> 4) & 3) << 4)) - 32);
        int8_t q4 = (int8_t)((int8_t)((ql[l + 32] >> 4) | (((qh[l] >> 6) & 3) << 4)) - 32);
        out[o + l] = d * sc[is + 0] * q1;
        out[o + l + 32] = d * sc[is + 2] * q2;
        out[o + l + 64] = d * sc[is + 4] * q3;
        out[o + l + 96] = d * sc[is + 6] * q4;
      }
      o += 128;
      ql += 64;
      qh += 32;
      sc += 8;
    }
  }
}

/* gguf_reader.cpp:326-387 */
int orc_dequant(int fmt, const uint8_t *data, float *out, size_t n) {
  switch (fmt) {
  case ORC_Q8_0:
    orc_dequant_q8_0(data, out, n);
    return 0;
  case ORC_Q4_0:
    orc_dequant_q4_0(data, out, n);
    return 0;
  case ORC_Q4_K:
    orc_dequant_q4_k(data, out, n);
    return 0;
  case ORC_Q6_K:
    orc_dequant_q6_k(data, out, n);
    return 0;
  }
  return -1;
}

/* llama.cpp:805-811, 922-928: dequantize to fp32, narrow each element. */
int orc_dequant_f16(int fmt, const uint8_t *data, uint16_t *out, size_t n) {
  const size_t chunk = 1u << 16; /* multiple of every block size */
  float *tmp = (float *)malloc(chunk * sizeof(float));
  if (!tmp)
    return -2;
  size_t be = orc_block_elems(fmt), bb = orc_block_bytes(fmt);
  if (!be) {
    free(tmp);
    return -1;
  }
  for (size_t o = 0; o < n; o += chunk) {
    size_t c = n - o < chunk ? n - o : chunk;
    orc_dequant(fmt, data + (o / be) * bb, tmp, c);
    for (size_t i = 0; i < c; ++i)
      out[o + i] = orc_f32_to_f16(tmp[i]);
  }
  free(tmp);
  return 0;
}

/* ---- reference weight preparation -------------------------------------- */

/* llama.cpp:488-505.  q uses the unrounded d; the stored scale is rounded. */
void orc_quantize_rows_q8_0(const float *f32, size_t n, int8_t *values,
                            uint16_t *scales) {
  size_t nb = n / 32;
  for (size_t b = 0; b < nb; ++b) {
    const float *x = f32 + b * 32;
    float amax = 0.0f;
    for (int i = 0; i < 32; ++i) {
      float a = fabsf(x[i]);
      amax = amax < a ? a : amax; /* std::max(amax, |x|) */
    }
    float d = amax / 127.0f;
    float id = d != 0.0f ? 1.0f / d : 0.0f;
    scales[b] = orc_f32_to_f16(d);
    for (int i = 0; i < 32; ++i)
      values[b * 32 + i] = (int8_t)lroundf(x[i] * id);
  }
}

void orc_pack_q8_0(const int8_t *values, const uint16_t *scales, size_t n,
                   uint8_t *blocks) {
  for (size_t b = 0; b < n / 32; ++b) {
    memcpy(blocks + b * 34, &scales[b], 2);
    memcpy(blocks + b * 34 + 2, values + b * 32, 32);
  }
}

/* gguf_reader.cpp:389-444 */
void orc_split_q8_0(const uint8_t *blocks, uint32_t rows, uint32_t cols,
                    int8_t *values, uint16_t *scales) {
  size_t bpr = cols / 32, total = (size_t)rows * bpr;
  for (size_t b = 0; b < total; ++b) {
    const uint8_t *p = blocks + b * 34;
    memcpy(&scales[b], p, 2);
    size_t row = b / bpr, bir = b % bpr;
    memcpy(values + row * cols + bir * 32, p + 2, 32);
  }
}

/* gguf_reader.cpp:446-501 */
void orc_split_q4_0(const uint8_t *blocks, uint32_t rows, uint32_t cols,
                    uint8_t *packed, uint16_t *scales) {
  size_t bpr = cols / 32, total = (size_t)rows * bpr;
  for (size_t b = 0; b < total; ++b) {
    const uint8_t *p = blocks + b * 18;
    memcpy(&scales[b], p, 2);
    size_t row = b / bpr, bir = b % bpr;
    memcpy(packed + row * (cols / 2) + bir * 16, p + 2, 16);
  }
}

/* llama.cpp:573-619 */
int orc_requantize_q4k_to_affine(const uint8_t *raw, size_t raw_bytes,
                                 uint32_t N, uint32_t K, uint8_t *packedT,
                                 uint16_t *scalesT) {
  if (K % 256 != 0 || N % 2 != 0)
    return 0;
  const uint32_t blocksK = K / 32;
  const size_t superPerRow = K / 256;
  if (raw_bytes < (size_t)N * superPerRow * 144)
    return 0;
  memset(packedT, 0, (size_t)K * (N / 2));
  memset(scalesT, 0, (size_t)2 * blocksK * N * sizeof(uint16_t));
  for (uint32_t n = 0; n < N; ++n) {
    for (uint32_t s = 0; s < superPerRow; ++s) {
      const uint8_t *block = raw + ((size_t)n * superPerRow + s) * 144;
      uint16_t d, dmin;
      memcpy(&d, block, 2);
      memcpy(&dmin, block + 2, 2);
      const float fd = orc_runner_f16_to_f32(d);
      const float fdmin = orc_runner_f16_to_f32(dmin);
      const uint8_t *scales = block + 4;
      const uint8_t *qs = block + 16;
      for (int g = 0; g < 4; ++g) {
        for (int h = 0; h < 2; ++h) {
          uint8_t sc, mm;
          orc_get_scale_min_k4(2 * g + h, scales, &sc, &mm);
          const float scale = fd * sc;
          const float minv = 8.0f * scale - fdmin * mm;
          const uint32_t e0 = s * 256 + (uint32_t)g * 64 + (uint32_t)h * 32;
          const uint32_t b = e0 / 32;
          scalesT[(size_t)b * N + n] = orc_f32_to_f16(scale);
          scalesT[((size_t)blocksK + b) * N + n] = orc_f32_to_f16(minv);
          for (uint32_t l = 0; l < 32; ++l) {
            const uint8_t byte = qs[g * 32 + l];
            const uint8_t q = (h == 0) ? (byte & 0xF) : (byte >> 4);
            const uint32_t k = e0 + l;
            packedT[(size_t)k * (N / 2) + (n >> 1)] |=
                (uint8_t)(q << ((n & 1) * 4));
          }
        }
      }
    }
  }
  return 1;
}

/* llama.cpp:712-720 */
void orc_decode_affine_q4(const uint8_t *packedT, const uint16_t *scalesT,
                          uint32_t N, uint32_t K, float *out) {
  const uint32_t blocksK = K / 32;
  for (uint32_t n = 0; n < N; ++n)
    for (uint32_t k = 0; k < K; ++k) {
      const uint8_t byte = packedT[(size_t)k * (N / 2) + (n >> 1)];
      const int nib = (n & 1) ? (byte >> 4) : (byte & 0xF);
      const uint32_t b = k / 32;
      const float scale = orc_runner_f16_to_f32(scalesT[(size_t)b * N + n]);
      const float minv =
          orc_runner_f16_to_f32(scalesT[((size_t)blocksK + b) * N + n]);
      out[(size_t)n * K + k] = ((float)nib - 8.0f) * scale + minv;
    }
}

/* TransposeQ4Nibble.cu:17-61 with tight strides. */
void orc_transpose_q4_nibble(const uint8_t *packed, uint32_t N, uint32_t K,
                             uint8_t *packedT) {
  uint32_t halfN = N / 2;
  for (uint32_t k = 0; k < K; ++k)
    for (uint32_t bn = 0; bn < halfN; ++bn) {
      uint8_t v = 0;
      for (int s = 0; s < 2; ++s) {
        uint32_t n = bn * 2 + (uint32_t)s;
        uint32_t blk = k / 32, e = k % 32;
        uint32_t j = e < 16 ? e : e - 16, hi = e < 16 ? 0 : 1;
        uint8_t byte = packed[(size_t)n * (K / 2) + blk * 16 + j];
        uint8_t nib = (uint8_t)((byte >> (hi * 4)) & 0xF);
        v |= (uint8_t)(nib << (s * 4));
      }
      packedT[(size_t)k * halfN + bn] = v;
    }
}

/* ---- reference matmul loops -------------------------------------------- */

/* OpRegistry.h:2043-2051: fp32, sequential over k, term (a*q)*s. */
void orc_matmul_sep_q8_f32(const float *A, const int8_t *B, const float *S,
                           uint32_t M, uint32_t K, uint32_t N, float *C) {
  for (uint32_t m = 0; m < M; ++m)
    for (uint32_t n = 0; n < N; ++n) {
      float e = 0.0f;
      for (uint32_t k = 0; k < K; ++k)
        e += A[(size_t)m * K + k] * (float)B[(size_t)k * N + n] *
             S[(size_t)(k / 32) * N + n];
      C[(size_t)m * N + n] = e;
    }
}

/* OpRegistry.h:2107-2112; affine adds the min row block (MatMulQ4Common.cuh
 * decode "(nib-8)*scale + min", llama.cpp:719). */
void orc_matmul_sep_q4_f32(const float *A, const uint8_t *Bp, const float *S,
                           uint32_t M, uint32_t K, uint32_t N, int affine,
                           float *C) {
  uint32_t blocksK = (K + 31) / 32;
  for (uint32_t m = 0; m < M; ++m)
    for (uint32_t n = 0; n < N; ++n) {
      float e = 0.0f;
      for (uint32_t k = 0; k < K; ++k) {
        uint8_t byte = Bp[(size_t)k * (N / 2) + (n >> 1)];
        int nib = (n & 1) ? (byte >> 4) : (byte & 0xF);
        float s = S[(size_t)(k / 32) * N + n];
        if (affine) {
          float w = (float)(nib - 8) * s + S[(size_t)(blocksK + k / 32) * N + n];
          e += A[(size_t)m * K + k] * w;
        } else {
          e += A[(size_t)m * K + k] * (float)(nib - 8) * s;
        }
      }
      C[(size_t)m * N + n] = e;
    }
}

/* RuntimeTests.cpp:2907-2920 */
void orc_matmul_sep_q8_f64(const float *A, const int8_t *B, const float *S,
                           uint32_t M, uint32_t K, uint32_t N, float *C) {
  for (uint32_t m = 0; m < M; ++m)
    for (uint32_t n = 0; n < N; ++n) {
      double sum = 0.0;
      for (uint32_t k = 0; k < K; ++k) {
        double a = A[(size_t)m * K + k];
        double b = (double)B[(size_t)k * N + n];
        double s = S[(size_t)(k / 32) * N + n];
        sum += a * b * s;
      }
      C[(size_t)m * N + n] = (float)sum;
    }
}

void orc_matmul_dense_f32(const float *Wf, const float *A, uint32_t M,
                          uint32_t K, uint32_t N, float *C) {
  for (uint32_t m = 0; m < M; ++m)
    for (uint32_t n = 0; n < N; ++n) {
      float e = 0.0f;
      const float *w = Wf + (size_t)n * K, *a = A + (size_t)m * K;
      for (uint32_t k = 0; k < K; ++k)
        e += a[k] * w[k];
      C[(size_t)m * N + n] = e;
    }
}

/* A . dequant_cpu(W)^T, row by row (one dequantized row at a time). */
int orc_matmul_gguf_f32(int fmt, const uint8_t *W, const float *A, uint32_t M,
                        uint32_t K, uint32_t N, float *C) {
  size_t be = orc_block_elems(fmt), bb = orc_block_bytes(fmt);
  if (!be || K % be)
    return -1;
  size_t row_bytes = (K / be) * bb;
  float *w = (float *)malloc((size_t)K * sizeof(float));
  if (!w)
    return -2;
  for (uint32_t n = 0; n < N; ++n) {
    orc_dequant(fmt, W + (size_t)n * row_bytes, w, K);
    for (uint32_t m = 0; m < M; ++m) {
      float e = 0.0f;
      const float *a = A + (size_t)m * K;
      for (uint32_t k = 0; k < K; ++k)
        e += a[k] * w[k];
      C[(size_t)m * N + n] = e;
    }
  }
  free(w);
  return 0;
}

int orc_matmul_gguf_f64(int fmt, const uint8_t *W, const float *A, uint32_t M,
                        uint32_t K, uint32_t N, double *C) {
  size_t be = orc_block_elems(fmt), bb = orc_block_bytes(fmt);
  if (!be || K % be)
    return -1;
  size_t row_bytes = (K / be) * bb;
  float *w = (float *)malloc((size_t)K * sizeof(float));
  if (!w)
    return -2;
  for (uint32_t n = 0; n < N; ++n) {
    orc_dequant(fmt, W + (size_t)n * row_bytes, w, K);
    for (uint32_t m = 0; m < M; ++m) {
      double e = 0.0;
      const float *a = A + (size_t)m * K;
      for (uint32_t k = 0; k < K; ++k)
        e += (double)a[k] * (double)w[k];
      C[(size_t)m * N + n] = e;
    }
  }
  free(w);
  return 0;
}

/* MatMulQ8GemvDot.cu:60-64; CUDA round() = half away from zero = roundf. */
void orc_quantize_act_q8(const float *a, size_t n, int8_t *q, float *scale) {
  for (size_t b = 0; b < n / 32; ++b) {
    float amax = 0.0f;
    for (int i = 0; i < 32; ++i) {
      float v = fabsf(a[b * 32 + i]);
      amax = v > amax ? v : amax;
    }
    float a_scale = amax / 127.0f;
    float inv = amax > 0.0f ? 127.0f / amax : 0.0f;
    scale[b] = a_scale;
    for (int i = 0; i < 32; ++i) {
      int v = (int)roundf(a[b * 32 + i] * inv);
      v = v < -127 ? -127 : (v > 127 ? 127 : v);
      q[b * 32 + i] = (int8_t)v;
    }
  }
}

/* MatMulQ8GemvDot.cu:60-85 on GGUF Q8_0 blocks W [N][K/32]: activations
 * quantized per 32 (orc_quantize_act_q8), integer dot per block, then
 * acc += (float)dot * a_scale * b_scale in fp32, blocks in order.  C64 (may be
 * NULL) receives the same sum with the scaling and the accumulation in double:
 * the two differ by fp32 rounding only. */
int orc_matmul_q8_i8(const uint8_t *W, const float *A, uint32_t M, uint32_t K,
                     uint32_t N, float *C32, double *C64) {
  if (K % 32 != 0)
    return -1;
  uint32_t nb = K / 32;
  int8_t *qa = (int8_t *)malloc((size_t)M * K);
  float *sa = (float *)malloc((size_t)M * nb * sizeof(float));
  if (!qa || !sa) {
    free(qa);
    free(sa);
    return -2;
  }
  for (uint32_t m = 0; m < M; ++m)
    orc_quantize_act_q8(A + (size_t)m * K, K, qa + (size_t)m * K,
                        sa + (size_t)m * nb);
  for (uint32_t m = 0; m < M; ++m)
    for (uint32_t n = 0; n < N; ++n) {
      float acc = 0.0f;
      double acc64 = 0.0;
      for (uint32_t b = 0; b < nb; ++b) {
        const uint8_t *blk = W + ((size_t)n * nb + b) * 34;
        uint16_t dbits;
        memcpy(&dbits, blk, 2);
        float d = orc_f16_to_f32(dbits);
        const int8_t *qw = (const int8_t *)(blk + 2);
        const int8_t *x = qa + (size_t)m * K + (size_t)b * 32;
        int dot = 0;
        for (int i = 0; i < 32; ++i)
          dot += (int)x[i] * (int)qw[i];
        float a_scale = sa[(size_t)m * nb + b];
        acc += (float)dot * a_scale * d;
        acc64 += (double)dot * (double)a_scale * (double)d;
      }
      if (C32)
        C32[(size_t)m * N + n] = acc;
      if (C64)
        C64[(size_t)m * N + n] = acc64;
    }
  free(qa);
  free(sa);
  return 0;
}

/* ---- own encoders (test inputs only) ----------------------------------- */

static inline int nearest_int(float f) { return (int)lrintf(f); }

/* Textbook Q4_0: d = (signed value of largest magnitude) / -8. */
void orc_quantize_q4_0(const float *x, size_t n, uint8_t *blocks) {
  for (size_t b = 0; b < n / 32; ++b) {
    const float *p = x + b * 32;
    float amax = 0.0f, mx = 0.0f;
    for (int i = 0; i < 32; ++i)
      if (fabsf(p[i]) > amax) {
        amax = fabsf(p[i]);
        mx = p[i];
      }
    float d = mx / -8.0f;
    uint16_t dh = orc_f32_to_f16(d);
    float id = d != 0.0f ? 1.0f / d : 0.0f;
    uint8_t *o = blocks + b * 18;
    memcpy(o, &dh, 2);
    for (int j = 0; j < 16; ++j) {
      int q0 = (int)(p[j] * id + 8.5f), q1 = (int)(p[j + 16] * id + 8.5f);
      q0 = q0 < 0 ? 0 : (q0 > 15 ? 15 : q0);
      q1 = q1 < 0 ? 0 : (q1 > 15 ? 15 : q1);
      o[2 + j] = (uint8_t)(q0 | (q1 << 4));
    }
  }
}

/* Q4_K: per 32-element sub-block an affine min/max fit, then 6-bit
 * quantization of the sub-block scales and mins against the super-block
 * maxima.  Simple and valid; not the iterative search of production encoders. */
void orc_quantize_q4_k(const float *x, size_t n, uint8_t *blocks) {
  for (size_t b = 0; b < n / 256; ++b) {
    const float *p = x + b * 256;
    float scales[8], mins[8], max_scale = 0.0f, max_min = 0.0f;
    for (int j = 0; j < 8; ++j) {
      float lo = p[32 * j], hi = p[32 * j];
      for (int l = 1; l < 32; ++l) {
        float v = p[32 * j + l];
        lo = v < lo ? v : lo;
        hi = v > hi ? v : hi;
      }
      if (lo > 0.0f)
        lo = 0.0f;
      scales[j] = (hi - lo) / 15.0f;
      mins[j] = -lo;
      if (scales[j] > max_scale)
        max_scale = scales[j];
      if (mins[j] > max_min)
        max_min = mins[j];
    }
    float inv_scale = max_scale > 0.0f ? 63.0f / max_scale : 0.0f;
    float inv_min = max_min > 0.0f ? 63.0f / max_min : 0.0f;
    uint8_t *o = blocks + b * 144;
    uint16_t dh = orc_f32_to_f16(max_scale / 63.0f);
    uint16_t dmh = orc_f32_to_f16(max_min / 63.0f);
    memcpy(o, &dh, 2);
    memcpy(o + 2, &dmh, 2);
    uint8_t *sc12 = o + 4;
    memset(sc12, 0, 12);
    uint8_t ls[8], lm[8];
    for (int j = 0; j < 8; ++j) {
      int a = nearest_int(inv_scale * scales[j]);
      int m = nearest_int(inv_min * mins[j]);
      ls[j] = (uint8_t)(a > 63 ? 63 : a);
      lm[j] = (uint8_t)(m > 63 ? 63 : m);
      if (j < 4) {
        sc12[j] = ls[j];
        sc12[j + 4] = lm[j];
      } else {
        sc12[j + 4] = (uint8_t)((ls[j] & 0xF) | ((lm[j] & 0xF) << 4));
        sc12[j - 4] |= (uint8_t)((ls[j] >> 4) << 6);
        sc12[j] |= (uint8_t)((lm[j] >> 4) << 6);
      }
    }
    float d = orc_f16_to_f32(dh), dmin = orc_f16_to_f32(dmh);
    uint8_t L[256];
    for (int j = 0; j < 8; ++j) {
      float dj = d * ls[j], mj = dmin * lm[j];
      for (int l = 0; l < 32; ++l) {
        int q = dj != 0.0f ? nearest_int((p[32 * j + l] + mj) / dj) : 0;
        L[32 * j + l] = (uint8_t)(q < 0 ? 0 : (q > 15 ? 15 : q));
      }
    }
    uint8_t *qs = o + 16;
    for (int g = 0; g < 4; ++g)
      for (int l = 0; l < 32; ++l)
        qs[32 * g + l] = (uint8_t)(L[64 * g + l] | (L[64 * g + 32 + l] << 4));
  }
}

/* Q6_K: 16 sub-blocks of 16 with symmetric scales amax/32 quantized to int8
 * against the super-block maximum. */
void orc_quantize_q6_k(const float *x, size_t n, uint8_t *blocks) {
  for (size_t b = 0; b < n / 256; ++b) {
    const float *p = x + b * 256;
    float scales[16], max_abs_scale = 0.0f, max_scale = 0.0f;
    for (int j = 0; j < 16; ++j) {
      float amax = 0.0f, mx = 0.0f;
      for (int l = 0; l < 16; ++l)
        if (fabsf(p[16 * j + l]) > amax) {
          amax = fabsf(p[16 * j + l]);
          mx = p[16 * j + l];
        }
      scales[j] = mx / -32.0f;
      if (fabsf(scales[j]) > max_abs_scale) {
        max_abs_scale = fabsf(scales[j]);
        max_scale = scales[j];
      }
    }
    uint8_t *o = blocks + b * 210;
    memset(o, 0, 210);
    float iscale = max_abs_scale > 0.0f ? -128.0f / max_scale : 0.0f;
    uint16_t dh = orc_f32_to_f16(iscale != 0.0f ? 1.0f / iscale : 0.0f);
    memcpy(o + 208, &dh, 2);
    int8_t *sc = (int8_t *)(o + 192);
    for (int j = 0; j < 16; ++j) {
      int v = nearest_int(iscale * scales[j]);
      sc[j] = (int8_t)(v > 127 ? 127 : (v < -128 ? -128 : v));
    }
    float d = orc_f16_to_f32(dh);
    uint8_t L[256];
    for (int j = 0; j < 16; ++j) {
      float dj = d * sc[j];
      for (int l = 0; l < 16; ++l) {
        int q = dj != 0.0f ? nearest_int(p[16 * j + l] / dj) : 0;
        q = q < -32 ? -32 : (q > 31 ? 31 : q);
        L[16 * j + l] = (uint8_t)(q + 32);
      }
    }
    uint8_t *ql = o, *qh = o + 128;
    for (int h = 0; h < 2; ++h) {
      const uint8_t *Lh = L + 128 * h;
      for (int l = 0; l < 32; ++l) {
        uint8_t q1 = Lh[l], q2 = Lh[l + 32], q3 = Lh[l + 64], q4 = Lh[l + 96];
        ql[64 * h + l] = (uint8_t)((q1 & 0xF) | ((q3 & 0xF) << 4));
        ql[64 * h + l + 32] = (uint8_t)((q2 & 0xF) | ((q4 & 0xF) << 4));
        qh[32 * h + l] = (uint8_t)((q1 >> 4) | ((q2 >> 4) << 2) |
                                   ((q3 >> 4) << 4) | ((q4 >> 4) << 6));
      }
    }
  }
}

int orc_quantize(int fmt, const float *x, size_t n, uint8_t *blocks) {
  switch (fmt) {
  case ORC_Q8_0: {
    int8_t *v = (int8_t *)malloc(n);
    uint16_t *s = (uint16_t *)malloc((n / 32) * 2);
    if (!v || !s) {
      free(v);
      free(s);
      return -2;
    }
    orc_quantize_rows_q8_0(x, n, v, s);
    orc_pack_q8_0(v, s, n, blocks);
    free(v);
    free(s);
    return 0;
  }
  case ORC_Q4_0:
    orc_quantize_q4_0(x, n, blocks);
    return 0;
  case ORC_Q4_K:
    orc_quantize_q4_k(x, n, blocks);
    return 0;
  case ORC_Q6_K:
    orc_quantize_q6_k(x, n, blocks);
    return 0;
  }
  return -1;
}

/* ---- operators between the matmuls of a decode step ------------------------ */

/* operators/impl/rmsnorm/RMSNorm.cu:15-37 */
void orc_rmsnorm(const float *x, const float *weight, uint32_t rows, uint32_t dim,
                 float eps, float *out) {
  for (uint32_t r = 0; r < rows; ++r) {
    const float *xr = x + (size_t)r * dim;
    double ss = 0.0; /* the kernel sums in fp32 over 256 strided lanes; double is the order-free anchor */
    for (uint32_t i = 0; i < dim; ++i)
      ss += (double)xr[i] * xr[i];
    float scale = (float)(1.0 / sqrt(ss / dim + (double)eps));
    for (uint32_t i = 0; i < dim; ++i)
      out[(size_t)r * dim + i] = xr[i] * scale * weight[i];
  }
}

/* fp32 -> fp16 bits, round to nearest even (what __float2half does; the KV
 * cache store of AttentionCommon.cuh:17).  Built on the exact f16->f32 map. */
static uint16_t f32_to_f16_rne(float v) {
  uint16_t up = orc_f32_to_f16(v); /* round-half-away: differs from RNE only on exact ties */
  uint32_t b;
  memcpy(&b, &v, 4);
  if ((b & 0x7F800000u) == 0x7F800000u)
    return up;
  uint16_t dn = (uint16_t)(up - 1);
  float fu = orc_f16_to_f32(up), fd = orc_f16_to_f32(dn);
  /* a tie: v is exactly halfway between dn and up (same sign) -> pick the even one */
  if ((up & 0x7FFF) != 0 && (double)fu - (double)v == (double)v - (double)fd && (up & 1))
    return dn;
  return up;
}

/* operators/impl/attention/FusedRoPEKVWrite.cu:27-80 */
void orc_rope_kv_write(const float *q, const float *k, const float *v, uint32_t pos,
                       const float *cos_t, const float *sin_t, uint32_t q_dim,
                       uint32_t kv_dim, uint32_t head_dim, uint32_t aligned_kv_dim,
                       float *q_out, uint16_t *k_cache, uint16_t *v_cache) {
  uint32_t half = head_dim / 2;
  const float *c = cos_t + (size_t)pos * half, *s = sin_t + (size_t)pos * half;
  for (uint32_t i = 0; i < q_dim; ++i) {
    uint32_t d = i % head_dim;
    q_out[i] = d < half ? q[i] * c[d] - q[i + half] * s[d]
                        : q[i - half] * s[d - half] + q[i] * c[d - half];
  }
  for (uint32_t i = 0; i < kv_dim; ++i) {
    uint32_t d = i % head_dim;
    float r = d < half ? k[i] * c[d] - k[i + half] * s[d]
                       : k[i - half] * s[d - half] + k[i] * c[d - half];
    k_cache[(size_t)pos * aligned_kv_dim + i] = f32_to_f16_rne(r);
    v_cache[(size_t)pos * aligned_kv_dim + i] = f32_to_f16_rne(v[i]);
  }
}

/* operators/impl/attention/Attention.cu:35-106 */
void orc_attention_decode(const float *q, const uint16_t *k_cache, const uint16_t *v_cache,
                          uint32_t seq_len, uint32_t n_heads, uint32_t n_kv_heads,
                          uint32_t head_dim, uint32_t aligned_kv_dim, float scale, float *out) {
  uint32_t n_rep = n_heads / n_kv_heads;
  double *sc = (double *)malloc(sizeof(double) * (seq_len ? seq_len : 1));
  for (uint32_t h = 0; h < n_heads; ++h) {
    uint32_t kvh = h / n_rep;
    double mx = -1e300;
    for (uint32_t t = 0; t < seq_len; ++t) {
      double dot = 0.0;
      for (uint32_t d = 0; d < head_dim; ++d)
        dot += (double)q[(size_t)h * head_dim + d] *
               orc_f16_to_f32(k_cache[(size_t)t * aligned_kv_dim + kvh * head_dim + d]);
      sc[t] = dot * scale;
      if (sc[t] > mx)
        mx = sc[t];
    }
    double sum = 0.0;
    for (uint32_t t = 0; t < seq_len; ++t) {
      sc[t] = exp(sc[t] - mx);
      sum += sc[t];
    }
    for (uint32_t d = 0; d < head_dim; ++d) {
      double acc = 0.0;
      for (uint32_t t = 0; t < seq_len; ++t)
        acc += sc[t] / sum * orc_f16_to_f32(v_cache[(size_t)t * aligned_kv_dim + kvh * head_dim + d]);
      out[(size_t)h * head_dim + d] = (float)acc;
    }
  }
  free(sc);
}

/* interface/runner/llama/llama.cpp:1832-1857 (unary SiLU then BinaryMul) */
void orc_silu_mul(const float *gate_up, uint32_t n, float *out) {
  for (uint32_t i = 0; i < n; ++i) {
    float g = gate_up[i];
    out[i] = (float)(g / (1.0 + exp(-(double)g))) * gate_up[(size_t)n + i];
  }
}

/* operators/impl/memory/EmbeddingCol.cu:16-44: gather of embedding rows from a table kept column-wise,
 * value of (token t, dim d) at index d * vocabStride + t.  format 0: fp16 table; format 1: int8 table with fp16
 * scales per 32 dims, scale of (d, t) at (d >> 5) * scaleStride + t (the separated Q8_0 layout of the loader). */
void orc_embedding_col(const uint32_t *indices, const void *matrix, const uint16_t *scales,
                       uint32_t num_indices, uint32_t emb_dim, uint32_t vocab_stride,
                       uint32_t scale_stride, uint32_t out_stride, int format, float *out) {
  for (uint32_t i = 0; i < num_indices; ++i) {
    uint32_t t = indices[i];
    for (uint32_t d = 0; d < emb_dim; ++d) {
      size_t idx = (size_t)d * vocab_stride + t;
      float v;
      if (format == 0) {
        v = orc_runner_f16_to_f32(((const uint16_t *)matrix)[idx]); /* __half2float: IEEE, NaN payload kept */
      } else {
        int b = ((const int8_t *)matrix)[idx];
        float sc = orc_runner_f16_to_f32(scales[(size_t)(d >> 5) * scale_stride + t]);
        v = (float)b * sc;
      }
      out[(size_t)i * out_stride + d] = v;
    }
  }
}

/* operators/impl/sampling/RepetitionPenalty.cu:19-41: logit > 0 ? logit / factor : logit * factor
 * (factor 1 for tokens that are not penalised). */
void orc_repetition_penalty(const float *logits, const float *factors, uint32_t n, float *out) {
  for (uint32_t i = 0; i < n; ++i)
    out[i] = logits[i] > 0.0f ? logits[i] / factors[i] : logits[i] * factors[i];
}

/* The dense factor vector the runner builds before every token (interface/runner/llama/llama.cpp:2566-2592):
 * factor[token] = penalty for every token of the recent window (once, however often it occurs), 1 elsewhere. */
void orc_penalty_factors(const int32_t *recent, uint32_t n_recent, float penalty, uint32_t vocab, float *factors) {
  for (uint32_t i = 0; i < vocab; ++i)
    factors[i] = 1.0f;
  for (uint32_t i = 0; i < n_recent; ++i)
    if (recent[i] >= 0 && (uint32_t)recent[i] < vocab)
      factors[recent[i]] = penalty;
}
