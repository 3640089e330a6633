// Shared device helpers for the gfx950 GGUF kernels.
#pragma once

#include <hip/hip_runtime.h>
#include <stdint.h>

#include "../../include/cut_hip.h"

namespace cuthip {

typedef _Float16 half_t;
typedef _Float16 half2_t __attribute__((ext_vector_type(2)));
typedef _Float16 half8_t __attribute__((ext_vector_type(8)));
typedef float f32x4 __attribute__((ext_vector_type(4)));
typedef float f32x16 __attribute__((ext_vector_type(16)));
typedef uint32_t u32x2 __attribute__((ext_vector_type(2)));
typedef uint32_t u32x4 __attribute__((ext_vector_type(4)));

constexpr int kWave = 64;

// Block geometry (interface/loader/gguf/gguf_types.hpp:109-142).
template <int FMT> struct Fmt;
template <> struct Fmt<CUTHIP_Q8_0> { static constexpr int elems = 32, bytes = 34; };
template <> struct Fmt<CUTHIP_Q4_0> { static constexpr int elems = 32, bytes = 18; };
template <> struct Fmt<CUTHIP_Q4_K> { static constexpr int elems = 256, bytes = 144; };
template <> struct Fmt<CUTHIP_Q6_K> { static constexpr int elems = 256, bytes = 210; };

__host__ __device__ inline int fmt_elems(int fmt) { return (fmt == CUTHIP_Q8_0 || fmt == CUTHIP_Q4_0) ? 32 : 256; }
__host__ __device__ inline int fmt_bytes(int fmt) {
  return fmt == CUTHIP_Q8_0 ? 34 : fmt == CUTHIP_Q4_0 ? 18 : fmt == CUTHIP_Q4_K ? 144 : 210;
}

// GGUF blocks are only 2-byte aligned (34, 18 and 210 byte strides); gfx950
// serves unaligned vector loads from global memory, so wide loads go through
// packed views and the compiler still emits global_load_dwordx2/x4.
struct __attribute__((packed, aligned(2))) U16x1 { uint16_t v; };
struct __attribute__((packed, aligned(2))) U32x1p { uint32_t v; };
struct __attribute__((packed, aligned(2))) U32x2p { uint32_t v[2]; };
struct __attribute__((packed, aligned(2))) U32x4p { uint32_t v[4]; };

__device__ inline uint32_t ld_u16(const uint8_t *p) { return reinterpret_cast<const U16x1 *>(p)->v; }
__device__ inline uint32_t ld_u32(const uint8_t *p) { return reinterpret_cast<const U32x1p *>(p)->v; }
__device__ inline u32x2 ld_u32x2(const uint8_t *p) {
  U32x2p t = *reinterpret_cast<const U32x2p *>(p);
  return u32x2{t.v[0], t.v[1]};
}
__device__ inline u32x4 ld_u32x4(const uint8_t *p) {
  U32x4p t = *reinterpret_cast<const U32x4p *>(p);
  return u32x4{t.v[0], t.v[1], t.v[2], t.v[3]};
}

__device__ inline float f16bits_to_f32(uint32_t h) {
  uint16_t b = (uint16_t)h;
  return (float)__builtin_bit_cast(half_t, b);  // exact, subnormals included
}
__device__ inline bool f16bits_finite(uint32_t h) { return (h & 0x7C00u) != 0x7C00u; }

// fp32 -> fp16 bits with the reference's host narrowing (llama.cpp:445-482):
// round half away from zero, subnormals kept, overflow and NaN -> +-Inf.
// Setting the lowest fp32 mantissa bit turns every exact tie into "just above
// the tie" and moves no other value across a rounding boundary, so the
// hardware's round-to-nearest-even conversion then gives the same bits.
// Valid for finite inputs only (an Inf would become a NaN).
__device__ inline uint32_t f32_to_f16bits_finite(float v) {
  uint32_t u = __builtin_bit_cast(uint32_t, v) | 1u;
  half_t h = (half_t)__builtin_bit_cast(float, u);
  return (uint32_t)__builtin_bit_cast(uint16_t, h);
}
// Any input, bit for bit the reference's algorithm.
__device__ inline uint32_t f32_to_f16bits_any(float v) {
  uint32_t u = __builtin_bit_cast(uint32_t, v);
  uint32_t sign = (u >> 16) & 0x8000u;
  if ((u & 0x7F800000u) == 0x7F800000u) return sign | 0x7C00u;
  return f32_to_f16bits_finite(v);
}

__device__ inline float cvt_ubyte0(uint32_t v) { return (float)(v & 0xFFu); }
__device__ inline float cvt_ubyte1(uint32_t v) { return (float)((v >> 8) & 0xFFu); }
__device__ inline float cvt_ubyte2(uint32_t v) { return (float)((v >> 16) & 0xFFu); }
__device__ inline float cvt_ubyte3(uint32_t v) { return (float)(v >> 24); }

// Q4_K: the eight 6-bit (scale, min) pairs of a super-block from its 12 packed
// bytes s0|s1|s2, four per dword (get_scale_min_k4, gguf_reader.cpp:668-676).
__device__ inline void q4k_scales(uint32_t s0, uint32_t s1, uint32_t s2, uint32_t &sc_lo, uint32_t &sc_hi,
                                  uint32_t &m_lo, uint32_t &m_hi) {
  sc_lo = s0 & 0x3F3F3F3Fu;                                    // j = 0..3
  m_lo = s1 & 0x3F3F3F3Fu;
  sc_hi = (s2 & 0x0F0F0F0Fu) | ((s0 >> 2) & 0x30303030u);      // j = 4..7
  m_hi = ((s2 >> 4) & 0x0F0F0F0Fu) | ((s1 >> 2) & 0x30303030u);
}

// Unary / binary epilogues of the matmul: the operator set and the formulas of cut_writeOutput
// (operators/impl/matmul/MatMulQ8Common.cuh:58-109), selected by the reference's operator codes.
// Only six unary (NEG, TANH, RELU, SIGMOID, GELU, SILU) and six binary (ADD, SUB, MUL, DIV, MIN, MAX) operators are part
// of the matmul kernels' epilogues.  The tiled GEMMs store 128 and more accumulators per lane through fully unrolled
// loops; with the whole operator set inlined at every store those loops no longer unroll, and the accumulator arrays
// they index leave the registers (measured: 710 -> 39 TFLOP/s).  The entry points run such a
// matmul unfused and apply the operator in a second, elementwise launch (launch_long_epilogue).
__device__ inline float apply_unary_long(int op, float x) {
  switch (op) {
  case CUTHIP_UNARY_ABS: return fabsf(x);
  case CUTHIP_UNARY_SQRT: return sqrtf(x);
  case CUTHIP_UNARY_SQUARE: return x * x;
  case CUTHIP_UNARY_RECIPROCAL: return 1.0f / x;
  case CUTHIP_UNARY_FLOOR: return floorf(x);
  case CUTHIP_UNARY_CEIL: return ceilf(x);
  case CUTHIP_UNARY_RELU6: return fminf(fmaxf(x, 0.0f), 6.0f);
  case CUTHIP_UNARY_EXP: return expf(x);
  case CUTHIP_UNARY_LOG: return logf(x);
  case CUTHIP_UNARY_ROUND: return roundf(x);
  case CUTHIP_UNARY_SOFTPLUS: return logf(1.0f + expf(x));
  case CUTHIP_UNARY_MISH: return x * tanhf(logf(1.0f + expf(x)));
  case CUTHIP_UNARY_HARDSWISH: return x * fminf(fmaxf(x / 6.0f + 0.5f, 0.0f), 1.0f);
  case CUTHIP_UNARY_HARDSIGMOID: return fminf(fmaxf(x / 6.0f + 0.5f, 0.0f), 1.0f);
  case CUTHIP_UNARY_RSQRT: return 1.0f / sqrtf(x);
  }
  return x;
}
__device__ inline float apply_binary_long(int op, float a, float b) {
  switch (op) {
  case CUTHIP_BINARY_MOD: return a - b * floorf(a / b);
  case CUTHIP_BINARY_POW: return powf(a, b);
  case CUTHIP_BINARY_FLOOR_DIV: return floorf(a / b);
  }
  return a;
}
inline bool epilogue_op_long(int epilogue, int op) {
  if (epilogue == CUTHIP_EPI_UNARY) {
    switch (op) {
    case CUTHIP_UNARY_NEG: case CUTHIP_UNARY_TANH: case CUTHIP_UNARY_RELU: case CUTHIP_UNARY_SIGMOID: case CUTHIP_UNARY_GELU:
    case CUTHIP_UNARY_SILU: return false;   // the six of the kernel epilogues
    }
    return true;
  }
  if (epilogue == CUTHIP_EPI_BINARY) return op == CUTHIP_BINARY_MOD || op == CUTHIP_BINARY_POW || op == CUTHIP_BINARY_FLOOR_DIV;
  return false;
}
// The operators inside the matmul kernels' epilogues.
__device__ inline float apply_unary(int op, float x) {
  switch (op) {
  case CUTHIP_UNARY_NEG: return -x;
  case CUTHIP_UNARY_TANH: return tanhf(x);
  case CUTHIP_UNARY_RELU: return fmaxf(0.0f, x);
  case CUTHIP_UNARY_SIGMOID: return 1.0f / (1.0f + __expf(-x));
  case CUTHIP_UNARY_GELU: {
    float t = 0.7978845608028654f * (x + 0.044715f * x * x * x);   // sqrt(2 / pi)
    return x * 0.5f * (1.0f + tanhf(t));
  }
  case CUTHIP_UNARY_SILU: return x / (1.0f + __expf(-x));
  }
  return x;   // the long operators never reach a kernel epilogue (epilogue_op_long)
}
__device__ inline float apply_binary(int op, float a, float b) {
  switch (op) {
  case CUTHIP_BINARY_ADD: return a + b;
  case CUTHIP_BINARY_SUB: return a - b;
  case CUTHIP_BINARY_MUL: return a * b;
  case CUTHIP_BINARY_DIV: return a / b;
  case CUTHIP_BINARY_MIN: return fminf(a, b);
  case CUTHIP_BINARY_MAX: return fmaxf(a, b);
  }
  return a;   // the long operators never reach a kernel epilogue (epilogue_op_long)
}
inline bool epilogue_op_known(int epilogue, int op) {
  if (epilogue == CUTHIP_EPI_UNARY) {
    switch (op) {
    case CUTHIP_UNARY_NEG: case CUTHIP_UNARY_ABS: case CUTHIP_UNARY_SQRT: case CUTHIP_UNARY_SQUARE:
    case CUTHIP_UNARY_RECIPROCAL: case CUTHIP_UNARY_EXP: case CUTHIP_UNARY_LOG: case CUTHIP_UNARY_TANH:
    case CUTHIP_UNARY_FLOOR: case CUTHIP_UNARY_CEIL: case CUTHIP_UNARY_ROUND: case CUTHIP_UNARY_RELU:
    case CUTHIP_UNARY_SIGMOID: case CUTHIP_UNARY_GELU: case CUTHIP_UNARY_SILU: case CUTHIP_UNARY_SOFTPLUS:
    case CUTHIP_UNARY_RELU6: case CUTHIP_UNARY_MISH: case CUTHIP_UNARY_HARDSWISH: case CUTHIP_UNARY_HARDSIGMOID:
    case CUTHIP_UNARY_RSQRT: return true;
    }
    return false;
  }
  if (epilogue == CUTHIP_EPI_BINARY) {
    switch (op) {
    case CUTHIP_BINARY_ADD: case CUTHIP_BINARY_SUB: case CUTHIP_BINARY_MUL: case CUTHIP_BINARY_DIV: case CUTHIP_BINARY_MOD:
    case CUTHIP_BINARY_POW: case CUTHIP_BINARY_FLOOR_DIV: case CUTHIP_BINARY_MIN: case CUTHIP_BINARY_MAX: return true;
    }
    return false;
  }
  return true;   // no operator to check
}

struct Epilogue {
  int kind;  // cuthip_epilogue
  int op;
  const void *D;
};

// Stores one output element with the fused epilogue applied.
__device__ inline void store_out(void *C, const Epilogue &e, int c_f16, size_t idx, float v) {
  if (e.kind == CUTHIP_EPI_UNARY) {
    v = apply_unary(e.op, v);
  } else if (e.kind == CUTHIP_EPI_BINARY) {
    float d = c_f16 ? (float)reinterpret_cast<const half_t *>(e.D)[idx] : reinterpret_cast<const float *>(e.D)[idx];
    v = apply_binary(e.op, v, d);
  }
  if (c_f16)
    reinterpret_cast<half_t *>(C)[idx] = (half_t)v;
  else
    reinterpret_cast<float *>(C)[idx] = v;
}

// store_out that also returns the fp32 value it stored (before any narrowing to fp16)
__device__ inline float store_out_value(void *C, const Epilogue &e, int c_f16, size_t idx, float v) {
  if (e.kind == CUTHIP_EPI_UNARY) {
    v = apply_unary(e.op, v);
  } else if (e.kind == CUTHIP_EPI_BINARY) {
    float d = c_f16 ? (float)reinterpret_cast<const half_t *>(e.D)[idx] : reinterpret_cast<const float *>(e.D)[idx];
    v = apply_binary(e.op, v, d);
  }
  if (c_f16)
    reinterpret_cast<half_t *>(C)[idx] = (half_t)v;
  else
    reinterpret_cast<float *>(C)[idx] = v;
  return v;
}

__device__ inline void store_plain(void *C, int c_f16, size_t idx, float v) {
  if (c_f16)
    reinterpret_cast<half_t *>(C)[idx] = (half_t)v;
  else
    reinterpret_cast<float *>(C)[idx] = v;
}

void set_error(const char *fmt, ...);
int check_hip(hipError_t e, const char *what);
// CUTHIP_OK, or CUTHIP_ERR_INVALID with the error set when `op` is not an operator the epilogue kind implements
int check_epilogue_op(const char *who, int epilogue, int op);
// C[m, n] = op(C[m, n]) or op(C[m, n], D[m, n]) in place, for the operators of epilogue_op_long: the second launch of a
// matmul whose fused operator is one of those (C and D are [M, strideC] of fp16 or fp32)
int launch_long_epilogue(void *C, int c_f16, uint32_t M, uint32_t N, uint32_t strideC, int epilogue, int op, const void *D,
                         hipStream_t stream);
// CUTHIP_ERR_INVALID (error set) when a binary operator that runs as a launch of its own would find its operand D
// already overwritten by the matmul (D == C); checked by the entry points before the unfused matmul is launched
int check_long_epilogue_alias(int epilogue, int op, const void *C, const void *D);

// Launch-shape overrides for tests and tuning sweeps.  Written by cuthip_set_tuning and, once, by cuthip_init from the
// CUT_HIP_* environment variables; the launchers only read this struct (no getenv on a launch path).  0 / -1 = unset.
struct Tuning {
  int rows8_rwg = 0, rows8_kw = 0;               // "rows8_shape"  = "rwg,kw"
  int gemv_kp = 0, gemv_waves = 0;               // "gemv_shape"   = "kp,waves"
  int gemm_ksplit = 0;                           // "gemm_ksplit"  = "n"
  int dense_bm = 0, dense_bn = 0, dense_ks = 1;  // "dense_tile"   = "bm,bn[,ksplit]"
  int dense_mfma16 = 1;                          // "dense_mfma16" = "0" | "1"
  int dense_pf = -1;                             // "dense_pf"     = prefetch distance in slices
};
extern Tuning g_tuning;

}  // namespace cuthip
