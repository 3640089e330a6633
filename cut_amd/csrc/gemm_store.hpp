// Output side of the MFMA GEMM kernels: a wave's accumulators go through LDS so that the global stores are 16 bytes per
// lane on whole row segments.
//
// A 32 x 32 accumulator tile of v_mfma_f32_32x32x* keeps column l & 31 in lane l and four consecutive ROWS in
// consecutive registers, so a store straight from the registers writes 2 bytes per lane (fp16 C), 64 contiguous bytes
// per half-wave, 16 store instructions per tile.  On the 2048 x 14336 prefill matmul those stores took a third of the
// kernel's time (115 of 335 us: measured by leaving them out).  Staged, a 32-row stripe of NJ tiles is written to LDS
// once (fp32) and read back row-wise: 8 consecutive columns per lane, one 16-byte store each (two for fp32 C).
#pragma once
#include <type_traits>
#include <utility>

#include "common.hpp"

namespace cuthip {

template <int... Is, class F> __device__ __forceinline__ void static_for_impl(std::integer_sequence<int, Is...>, F &&f) {
  (f(std::integral_constant<int, Is>{}), ...);
}
template <int N, class F> __device__ __forceinline__ void static_for(F &&f) {
  static_for_impl(std::make_integer_sequence<int, N>{}, static_cast<F &&>(f));
}

typedef __attribute__((address_space(3))) float lds_f32;
typedef __attribute__((address_space(3))) f32x4 lds_f32x4;

// floats per staged row of a stripe of NJ tiles: 4 rows apart is 32 banks apart (the two half-waves of a tile write)
template <int NJ> constexpr int stripe_ld() { return 32 * NJ + 8; }
template <int NJ> constexpr int stripe_floats() { return 32 * stripe_ld<NJ>(); }

// true when store_out8 may use its 16-byte path on C (and on the operand D of a binary epilogue)
inline bool store8_aligned(const void *C, uint32_t strideC, int c_f16, const Epilogue &e) {
  const uint32_t per16 = c_f16 ? 8 : 4;
  if ((uintptr_t)C % 16 != 0 || strideC % per16 != 0) return false;
  if (e.kind == CUTHIP_EPI_BINARY && (uintptr_t)e.D % 16 != 0) return false;
  return true;
}

// Eight consecutive outputs (lo, hi) of one row with the fused epilogue: idx = row * strideC + col, col a multiple of 8.
// vec: the operands pass store8_aligned.  Same arithmetic per element as store_out.  Every element index is a
// compile-time constant: an indexed copy of the values would live in scratch memory.
__device__ __forceinline__ void store_out8(void *C, const Epilogue &e, int c_f16, size_t idx, f32x4 lo, f32x4 hi, uint32_t col,
                                           uint32_t N, bool vec) {
  if (vec && col + 8 <= N) {
    if (e.kind == CUTHIP_EPI_UNARY) {
      static_for<4>([&](auto ii) __attribute__((always_inline)) {
        constexpr int i = decltype(ii)::value;
        lo[i] = apply_unary(e.op, lo[i]);
        hi[i] = apply_unary(e.op, hi[i]);
      });
    } else if (e.kind == CUTHIP_EPI_BINARY) {
      f32x4 d0, d1;
      if (c_f16) {
        const half8_t d = *reinterpret_cast<const half8_t *>(reinterpret_cast<const half_t *>(e.D) + idx);
        d0 = f32x4{(float)d[0], (float)d[1], (float)d[2], (float)d[3]};
        d1 = f32x4{(float)d[4], (float)d[5], (float)d[6], (float)d[7]};
      } else {
        const f32x4 *dp = reinterpret_cast<const f32x4 *>(reinterpret_cast<const float *>(e.D) + idx);
        d0 = dp[0];
        d1 = dp[1];
      }
      static_for<4>([&](auto ii) __attribute__((always_inline)) {
        constexpr int i = decltype(ii)::value;
        lo[i] = apply_binary(e.op, lo[i], d0[i]);
        hi[i] = apply_binary(e.op, hi[i], d1[i]);
      });
    }
    if (c_f16) {
      const half8_t o{(half_t)lo[0], (half_t)lo[1], (half_t)lo[2], (half_t)lo[3],
                      (half_t)hi[0], (half_t)hi[1], (half_t)hi[2], (half_t)hi[3]};
      *reinterpret_cast<half8_t *>(reinterpret_cast<half_t *>(C) + idx) = o;
    } else {
      f32x4 *cp = reinterpret_cast<f32x4 *>(reinterpret_cast<float *>(C) + idx);
      cp[0] = lo;
      cp[1] = hi;
    }
  } else {
    static_for<4>([&](auto ii) __attribute__((always_inline)) {
      constexpr int i = decltype(ii)::value;
      if (col + i < N) store_out(C, e, c_f16, idx + i, lo[i]);
    });
    static_for<4>([&](auto ii) __attribute__((always_inline)) {
      constexpr int i = decltype(ii)::value;
      if (col + 4 + i < N) store_out(C, e, c_f16, idx + 4 + i, hi[i]);
    });
  }
}

// A stripe = rows row0 .. row0 + 31, columns col0 .. col0 + 32 NJ - 1 of C, from NJ accumulator tiles of one wave.
// stage: stripe_floats<NJ>() floats of LDS that only this wave touches (LDS operations of one wave complete in
// order, so the next stripe may overwrite this one without a barrier).  stage_tile32 once per tile (the accumulator
// by value, from a compile-time position of the caller's array: passed by reference the array would live in scratch
// memory), then store_staged32.
template <int NJ> __device__ __forceinline__ void stage_tile32(lds_f32 *stage, int j, f32x16 a, int lane) {
  // register r of lane l: row 8 (r / 4) + 4 (l >> 5) + r % 4, column l & 31 of the tile
  lds_f32 *wr = stage + (4 * (lane >> 5)) * stripe_ld<NJ>() + 32 * j + (lane & 31);
  static_for<16>([&](auto rr) __attribute__((always_inline)) {
    constexpr int r = decltype(rr)::value;
    wr[(8 * (r >> 2) + (r & 3)) * stripe_ld<NJ>()] = a[r];
  });
}
// FAST: 0 = any epilogue and output type; 1 = the caller has checked that there is no epilogue operator, C is fp16 and
// 16-byte stores are allowed; 2 = the same with the binary operator ADD (the residual of a transformer block, D fp16);
// 3 = no operator, fp32 C (the partial products of a K split).
// The fast loops are a read, a conversion (an add) and a store; the general form carries every operator of the epilogue
// in each iteration and waits for its loads of D and its stores one iteration at a time.
template <int NJ, int FAST = 0>
__device__ __forceinline__ void store_staged32(const lds_f32 *stage, uint32_t row0, uint32_t col0, uint32_t M, uint32_t N, void *C,
                                               uint32_t strideC, int c_f16, const Epilogue &e, bool vec, int lane) {
  constexpr int LD = stripe_ld<NJ>(), CH = 4 * NJ;   // CH chunks of 8 columns per row
  // the fast loops are unrolled (a dozen instructions per iteration); the general one stays a loop: unrolled, its
  // operator switches made the kernels several times larger for nothing
#pragma unroll FAST != 0 ? 32 * CH / 64 : 1
  for (int it = 0; it < 32 * CH / 64; ++it) {
    const int c = it * 64 + lane, row = c / CH, c8 = c % CH;
    const lds_f32x4 *src = reinterpret_cast<const lds_f32x4 *>(stage + row * LD + 8 * c8);
    const f32x4 lo = src[0], hi = src[1];
    const uint32_t grow = row0 + row, gcol = col0 + 8 * c8;
    if constexpr (FAST == 3) {
      if (grow < M && gcol + 8 <= N) {
        f32x4 *cp = reinterpret_cast<f32x4 *>(reinterpret_cast<float *>(C) + (size_t)grow * strideC + gcol);
        cp[0] = lo;
        cp[1] = hi;
      } else if (grow < M && gcol < N) {
        float *cp = reinterpret_cast<float *>(C) + (size_t)grow * strideC + gcol;
        static_for<8>([&](auto kk) __attribute__((always_inline)) {
          constexpr int k = decltype(kk)::value;
          if (gcol + k < N) cp[k] = k < 4 ? lo[k & 3] : hi[k & 3];
        });
      }
    } else if constexpr (FAST != 0) {
      if (grow < M && gcol + 8 <= N) {
        const size_t idx = (size_t)grow * strideC + gcol;
        f32x4 a = lo, b = hi;
        if constexpr (FAST == 2) {
          const half8_t d = *reinterpret_cast<const half8_t *>(reinterpret_cast<const half_t *>(e.D) + idx);
          a += f32x4{(float)d[0], (float)d[1], (float)d[2], (float)d[3]};
          b += f32x4{(float)d[4], (float)d[5], (float)d[6], (float)d[7]};
        }
        const half8_t o{(half_t)a[0], (half_t)a[1], (half_t)a[2], (half_t)a[3],
                        (half_t)b[0], (half_t)b[1], (half_t)b[2], (half_t)b[3]};
        *reinterpret_cast<half8_t *>(reinterpret_cast<half_t *>(C) + idx) = o;
      } else if (grow < M && gcol < N) {   // the ragged right edge, element by element
        const size_t idx = (size_t)grow * strideC + gcol;
        half_t *cp = reinterpret_cast<half_t *>(C) + idx;
        const half_t *dp = reinterpret_cast<const half_t *>(e.D) + idx;
        static_for<8>([&](auto kk) __attribute__((always_inline)) {
          constexpr int k = decltype(kk)::value;
          if (gcol + k < N) {
            float v = k < 4 ? lo[k & 3] : hi[k & 3];
            if constexpr (FAST == 2) v += (float)dp[k];
            cp[k] = (half_t)v;
          }
        });
      }
    } else {
      if (grow < M && gcol < N) store_out8(C, e, c_f16, (size_t)grow * strideC + gcol, lo, hi, gcol, N, vec);
    }
  }
}

}  // namespace cuthip
