// Block formats of the streaming GEMV: per-format register image of one
// 256-element step, its loads and its MFMA/scale arithmetic.  See
// gemv_kernel.hpp for the kernel that drives them.
#pragma once
#include "common.hpp"

namespace cuthip {

// RoPE and KV-cache append in the epilogue of a batch-1 matmul (the q | k and v projections of a decode step).
// mode 1: the weight rows are [q heads | k heads], inside each head interleaved as d = 0, half, 1, half + 1, ... so
// that the two partners of the half-split rotation are neighbouring rows; rotated q goes to q_out, rotated k as
// fp16 to cache row params[0].  mode 2: the rows are v and go to the cache row as fp16.  mode 0: off.
struct RopeAppend {
  int mode = 0;
  const uint32_t *params = nullptr;
  const float *cosT = nullptr, *sinT = nullptr;   // [position][head_dim / 2]
  void *q_out = nullptr;
  int q_out_f16 = 0;
  half_t *k_cache = nullptr, *v_cache = nullptr;
  uint32_t q_dim = 0, head_dim = 0, kv_stride = 0;
  uint32_t max_pos = 0;   // rows of the caches and tables; a position at or beyond it writes nothing
  // set by a kernel that has read params[0] itself, ahead of everything else (the host leaves them 0)
  uint32_t pos = 0;
  int pos_read = 0;
};

struct ArgmaxPart {
  float value;      // -inf if the group holds no row
  uint32_t index;   // row of the first maximum of the group
};

struct GemvParams {
  const uint8_t *W;
  const void *A;
  void *C;
  Epilogue epi;
  uint32_t M, K, N, strideA, strideC;
  uint32_t nsteps;   // ceil(K / 256)
  uint32_t row_bytes;
  int a_f16, c_f16;
  // prologue on the activations (8-row GEMV, batch 1): CUTHIP_PRO_RMSNORM: A is x, the product is taken with
  // x * norm_w and scaled by rsqrt(mean(x^2) + eps); CUTHIP_PRO_SWIGLU: A is [gate(K) | up(K)], input silu(gate) * up
  int pro = 0;
  const float *norm_w = nullptr;
  float eps = 0.0f;
  // RMSNorm carried across matmuls (8-row GEMV, batch 1).  Producer side, after the epilogue: next_x16[n] =
  // fp16(C[n] * next_norm_w[n]) and the sum of C[n]^2 over each group of 8 rows goes to next_sumsq_parts[n / 8].
  // Consumer side (the activations are such a next_x16): the result is multiplied by
  // rsqrt(sum(sumsq_parts[0 .. K/8)) / K + eps).  Fixed summation order, no atomics.
  RopeAppend rope;
  const float *sumsq_parts = nullptr;
  const float *next_norm_w = nullptr;
  half_t *next_x16 = nullptr;
  float *next_sumsq_parts = nullptr;
  // Greedy sampling folded into the matmul that produces the logits (8-row GEMV, batch 1, one K range per wave):
  // every wave also stores the largest of its 8 outputs (as stored in C) and its row index to argmax_parts[n / 8];
  // a one-workgroup kernel finishes the reduction.
  ArgmaxPart *argmax_parts = nullptr;
  uint32_t mrg_nsplit = 0, mrg_head_dim = 0;   // CUTHIP_PRO_ATTN_MERGE: records per head in A, and the head dimension
  uint32_t hot = 0;   // 8-row kernel: flag word of its leading kernel arguments (which optional pointers are set)
};

// ---- per-tile configuration -------------------------------------------------
template <int MT, int KP> struct TileCfg {
  static constexpr int ROWS = MT * KP;                                        // MFMA A rows in use
  static constexpr int R = ROWS <= 4 ? ROWS : (ROWS <= 8 ? 4 : (ROWS <= 16 ? 8 : 16));  // accumulators per lane
  // Few staged rows: the activations of the next tile travel through registers while the
  // current tile is consumed (their loads are issued ahead of the weight loads, so waiting
  // for them never waits for weights).  Otherwise the tile is staged in place.
  static constexpr bool PIPE = ROWS <= 2;
  static constexpr int TB = PIPE ? 8 / ROWS : (ROWS <= 4 ? 8 : (ROWS <= 8 ? 4 : (ROWS <= 16 ? 2 : 1)));  // steps per LDS tile
  static constexpr int D = TB < 4 ? TB : 4;                                   // steps of loads in flight
  static constexpr int XI = ROWS * TB * 32 / 64;                              // 8-element groups per lane per tile
  static constexpr int XROW = TB * 256 + 8;  // halfs per staged row (+16 B against bank conflicts)
};

// row of C held in accumulator register r of a lane in half `half` (32x32 MFMA)
__device__ inline int acc_row(int r, int half) { return (r >> 2) * 8 + half * 4 + (r & 3); }

__device__ inline half8_t as_half8(uint32_t a, uint32_t b, uint32_t c, uint32_t d) {
  return __builtin_bit_cast(half8_t, u32x4{a, b, c, d});
}
__device__ inline f32x16 mfma(half8_t a, half8_t b, f32x16 c) {
  return __builtin_amdgcn_mfma_f32_32x32x16_f16(a, b, c, 0, 0, 0);
}
__device__ inline f32x16 zero16() {
  return f32x16{0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0};
}
template <int R> __device__ inline void fma_acc(float (&acc)[R], const f32x16 &p, float s) {
#pragma unroll
  for (int r = 0; r < R; ++r) acc[r] = fmaf(p[r], s, acc[r]);
}

constexpr uint32_t kNibLo = 0x000F000Fu;  // q * 2^-24
constexpr uint32_t kNibHi = 0x00F000F0u;  // q * 2^-20
constexpr float kTwo24 = 16777216.0f, kTwo20 = 1048576.0f;

// ---- formats ----------------------------------------------------------------
// Each format provides: NSUB (sub-block sums of x per 256-element step), a Raw
// register image of one step of one row-half, load() and compute().
// compute(): x = this lane's staged activation row at the step, sx = the
// wave's sub-block sums at the step ([row][SXROW] floats), nrows = valid rows
// of both, valid = whether the step lies inside the lane's part (else the
// contribution is forced to zero by zeroing the block scale).

template <int FMT> struct Step;

// Q4_K: 144 B = [d][dmin][scales:12][qs:128].  Lane (n, kg) loads the header
// and, for each 64-element group g, the 16 bytes qs[32g+16kg .. +15]: low
// nibbles are elements 64g+16kg+i of sub-block 2g, high nibbles elements
// 64g+32+16kg+i of sub-block 2g+1.
template <> struct Step<CUTHIP_Q4_K> {
  static constexpr int NSUB = 8, SUBK = 32;
  struct Raw { u32x4 hdr; u32x4 q[4]; };
  __device__ static void load(Raw &r, const uint8_t *row, uint32_t step, int kg, uint32_t /*K*/) {
    const uint8_t *p = row + (size_t)step * 144;
    r.hdr = ld_u32x4(p);
#pragma unroll
    for (int g = 0; g < 4; ++g) r.q[g] = ld_u32x4(p + 16 + 32 * g + 16 * kg);
  }
  template <int R, int SXROW>
  __device__ static void compute(const Raw &r, const half_t *x, const float *sx, int kg, int nrows, bool valid,
                                 float (&acc)[R]) {
    uint32_t dd = valid ? r.hdr.x : 0u;
    float d = f16bits_to_f32(dd & 0xFFFF), dmin = f16bits_to_f32(dd >> 16);
    uint32_t sc_lo, sc_hi, m_lo, m_hi;
    q4k_scales(r.hdr.y, r.hdr.z, r.hdr.w, sc_lo, sc_hi, m_lo, m_hi);
    float dl = d * kTwo24, dh = d * kTwo20;
    // even sub-blocks come from low nibbles (2^-24), odd ones from high nibbles (2^-20)
    float ds[8] = {dl * cvt_ubyte0(sc_lo), dh * cvt_ubyte1(sc_lo), dl * cvt_ubyte2(sc_lo), dh * cvt_ubyte3(sc_lo),
                   dl * cvt_ubyte0(sc_hi), dh * cvt_ubyte1(sc_hi), dl * cvt_ubyte2(sc_hi), dh * cvt_ubyte3(sc_hi)};
    float dm[8] = {dmin * cvt_ubyte0(m_lo), dmin * cvt_ubyte1(m_lo), dmin * cvt_ubyte2(m_lo), dmin * cvt_ubyte3(m_lo),
                   dmin * cvt_ubyte0(m_hi), dmin * cvt_ubyte1(m_hi), dmin * cvt_ubyte2(m_hi), dmin * cvt_ubyte3(m_hi)};
    const half8_t *xa = reinterpret_cast<const half8_t *>(x + 16 * kg);
#pragma unroll
    for (int g = 0; g < 4; ++g) {
      u32x4 w = r.q[g];
      half8_t lo_a = as_half8(w.x & kNibLo, (w.x >> 8) & kNibLo, w.y & kNibLo, (w.y >> 8) & kNibLo);
      half8_t lo_b = as_half8(w.z & kNibLo, (w.z >> 8) & kNibLo, w.w & kNibLo, (w.w >> 8) & kNibLo);
      half8_t hi_a = as_half8(w.x & kNibHi, (w.x >> 8) & kNibHi, w.y & kNibHi, (w.y >> 8) & kNibHi);
      half8_t hi_b = as_half8(w.z & kNibHi, (w.z >> 8) & kNibHi, w.w & kNibHi, (w.w >> 8) & kNibHi);
      // x chunks (8 halfs each): 64g + 16kg + {0, 8} and 64g + 32 + 16kg + {0, 8}
      f32x16 p = mfma(xa[8 * g + 0], lo_a, zero16());
      f32x16 q = mfma(xa[8 * g + 4], hi_a, zero16());
      p = mfma(xa[8 * g + 1], lo_b, p);
      q = mfma(xa[8 * g + 5], hi_b, q);
      fma_acc<R>(acc, p, ds[2 * g]);
      fma_acc<R>(acc, q, ds[2 * g + 1]);
    }
#pragma unroll
    for (int r_ = 0; r_ < R; ++r_) {
      int row = min(acc_row(r_, kg), nrows - 1);
      const f32x4 *s = reinterpret_cast<const f32x4 *>(sx + row * SXROW);
      f32x4 s0 = s[0], s1 = s[1];
      float a = acc[r_];
      a = fmaf(-dm[0], s0.x, a); a = fmaf(-dm[1], s0.y, a); a = fmaf(-dm[2], s0.z, a); a = fmaf(-dm[3], s0.w, a);
      a = fmaf(-dm[4], s1.x, a); a = fmaf(-dm[5], s1.y, a); a = fmaf(-dm[6], s1.z, a); a = fmaf(-dm[7], s1.w, a);
      acc[r_] = a;
    }
  }
};

// Q6_K: 210 B = [ql:128][qh:64][sc:16 x i8][d].  Element (H, s, l) of half H,
// quarter s: q = (nibble s>>1 of ql[64H+32(s&1)+l] | bits 2s..2s+1 of
// qh[32H+l] << 4) - 32, scale sc[8H+2s+l/16].  A 16-element sub-block is one
// MFMA: lane kg takes l = 16*lam + 8kg .. +7 for lam = l/16.
template <> struct Step<CUTHIP_Q6_K> {
  static constexpr int NSUB = 16, SUBK = 16;
  struct Raw { u32x2 ql[2][2][2]; u32x2 qh[2][2]; u32x4 sc; uint32_t d; };  // [H][lam][sigma]
  __device__ static void load(Raw &r, const uint8_t *row, uint32_t step, int kg, uint32_t /*K*/) {
    const uint8_t *p = row + (size_t)step * 210;
#pragma unroll
    for (int H = 0; H < 2; ++H)
#pragma unroll
      for (int lam = 0; lam < 2; ++lam) {
        r.ql[H][lam][0] = ld_u32x2(p + 64 * H + 16 * lam + 8 * kg);
        r.ql[H][lam][1] = ld_u32x2(p + 64 * H + 32 + 16 * lam + 8 * kg);
        r.qh[H][lam] = ld_u32x2(p + 128 + 32 * H + 16 * lam + 8 * kg);
      }
    r.sc = ld_u32x4(p + 192);
    r.d = ld_u16(p + 208);
  }
  __device__ static float sc_at(const u32x4 &sc, int j) {
    uint32_t w = j < 4 ? sc.x : j < 8 ? sc.y : j < 12 ? sc.z : sc.w;
    return (float)(int)(int8_t)((w >> (8 * (j & 3))) & 0xFF);
  }
  template <int R, int SXROW>
  __device__ static void compute(const Raw &r, const half_t *x, const float *sx, int kg, int nrows, bool valid,
                                 float (&acc)[R]) {
    float d = f16bits_to_f32(valid ? r.d : 0u);
    const half8_t *xa = reinterpret_cast<const half8_t *>(x + 8 * kg);
    constexpr uint32_t kH45 = 0x00300030u, kH89 = 0x03000300u;
    const float *sxr[R];
#pragma unroll
    for (int r_ = 0; r_ < R; ++r_) sxr[r_] = sx + min(acc_row(r_, kg), nrows - 1) * SXROW;
#pragma unroll
    for (int H = 0; H < 2; ++H)
#pragma unroll
      for (int lam = 0; lam < 2; ++lam) {
        u32x2 wa = r.ql[H][lam][0], wb = r.ql[H][lam][1], h = r.qh[H][lam];
        // s = 0: low nibbles of wa | qh bits 0-1 -> value bits 0-5 (2^-24)
        // s = 1: low nibbles of wb | qh bits 2-3
        // s = 2: high nibbles of wa | qh bits 4-5 -> value bits 4-9 (2^-20)
        // s = 3: high nibbles of wb | qh bits 6-7
        half8_t b[4];
        uint32_t v[4][4];
#pragma unroll
        for (int c = 0; c < 2; ++c) {
          uint32_t a0 = c ? wa.y : wa.x, b0 = c ? wb.y : wb.x, h0 = c ? h.y : h.x;
          uint32_t a8 = a0 >> 8, b8 = b0 >> 8;
          uint32_t hl4 = h0 << 4, hl2 = h0 << 2, hr4 = h0 >> 4, hr6 = h0 >> 6;
          v[0][2 * c + 0] = (a0 & kNibLo) | (hl4 & kH45);
          v[0][2 * c + 1] = (a8 & kNibLo) | (hr4 & kH45);
          v[1][2 * c + 0] = (b0 & kNibLo) | (hl2 & kH45);
          v[1][2 * c + 1] = (b8 & kNibLo) | (hr6 & kH45);
          v[2][2 * c + 0] = (a0 & kNibHi) | (hl4 & kH89);
          v[2][2 * c + 1] = (a8 & kNibHi) | (hr4 & kH89);
          v[3][2 * c + 0] = (b0 & kNibHi) | (hl2 & kH89);
          v[3][2 * c + 1] = (b8 & kNibHi) | (hr6 & kH89);
        }
#pragma unroll
        for (int s = 0; s < 4; ++s) b[s] = as_half8(v[s][0], v[s][1], v[s][2], v[s][3]);
#pragma unroll
        for (int s = 0; s < 4; ++s) {
          int j = 8 * H + 2 * s + lam;                       // sub-block (16 elements)
          // elements 128H + 32s + 16lam + 8kg + i  -> x chunk index (halfs / 8), kg folded into xa
          f32x16 p = mfma(xa[(128 * H + 32 * s + 16 * lam) / 8], b[s], zero16());
          float dsc = d * sc_at(r.sc, j);
          float two = s < 2 ? kTwo24 : kTwo20;
#pragma unroll
          for (int r_ = 0; r_ < R; ++r_) {
            float t = fmaf(p[r_], two, -32.0f * sxr[r_][j]);   // sum((q6 - 32) * x), exact products
            acc[r_] = fmaf(dsc, t, acc[r_]);
          }
        }
      }
  }
};

// Q8_0: 34 B = [d][q:32 x i8], eight blocks per 256-element step.  Lane kg takes
// bytes 16kg .. 16kg+15 of each block; q + 128 (one XOR) is an unsigned byte,
// i.e. the fp16 subnormal (q + 128) * 2^-24, and the +128 goes to the sum term.
template <> struct Step<CUTHIP_Q8_0> {
  static constexpr int NSUB = 8, SUBK = 32;
  // keep: bit i set if block i of the step lies inside K (blocks past K contribute zero: their scale is dropped where
  // it is used; a select or a condition around the load here would make the loads of a step wait for each other)
  struct Raw { u32x4 q[8]; uint32_t d[8]; uint32_t keep; };
  __device__ static void load(Raw &r, const uint8_t *row, uint32_t step, int kg, uint32_t K) {
    uint32_t nblk = K / 32, b0 = step * 8;
    r.keep = b0 + 8 <= nblk ? 0xFFu : (b0 < nblk ? (1u << (nblk - b0)) - 1u : 0u);
#pragma unroll
    for (int i = 0; i < 8; ++i) {
      uint32_t b = min(b0 + i, nblk - 1);
      const uint8_t *p = row + (size_t)b * 34;
      r.q[i] = ld_u32x4(p + 2 + 16 * kg);
      r.d[i] = ld_u16(p);
    }
  }
  template <int R, int SXROW>
  __device__ static void compute(const Raw &r, const half_t *x, const float *sx, int kg, int nrows, bool valid,
                                 float (&acc)[R]) {
    const half8_t *xa = reinterpret_cast<const half8_t *>(x + 16 * kg);
    constexpr uint32_t kByte = 0x00FF00FFu;
    const float *sxr[R];
#pragma unroll
    for (int r_ = 0; r_ < R; ++r_) sxr[r_] = sx + min(acc_row(r_, kg), nrows - 1) * SXROW;
#pragma unroll
    for (int i = 0; i < 8; ++i) {
      u32x4 w = r.q[i] ^ u32x4{0x80808080u, 0x80808080u, 0x80808080u, 0x80808080u};
      half8_t ba = as_half8(w.x & kByte, (w.x >> 8) & kByte, w.y & kByte, (w.y >> 8) & kByte);
      half8_t bb = as_half8(w.z & kByte, (w.z >> 8) & kByte, w.w & kByte, (w.w >> 8) & kByte);
      f32x16 p = mfma(xa[4 * i + 0], ba, zero16());
      p = mfma(xa[4 * i + 1], bb, p);
      float d = f16bits_to_f32((valid && ((r.keep >> i) & 1u)) ? r.d[i] : 0u);
#pragma unroll
      for (int r_ = 0; r_ < R; ++r_) {
        float t = fmaf(p[r_], kTwo24, -128.0f * sxr[r_][i]);
        acc[r_] = fmaf(d, t, acc[r_]);
      }
    }
  }
};

// Q4_0: 18 B = [d][qs:16], low nibble of qs[j] is element j, high nibble element
// j+16, value (nib - 8) * d.  Lane kg takes bytes 8kg .. 8kg+7 of each block.
template <> struct Step<CUTHIP_Q4_0> {
  static constexpr int NSUB = 8, SUBK = 32;
  struct Raw { u32x2 q[8]; uint32_t d[8]; uint32_t keep; };   // keep: as for Q8_0
  __device__ static void load(Raw &r, const uint8_t *row, uint32_t step, int kg, uint32_t K) {
    uint32_t nblk = K / 32, b0 = step * 8;
    r.keep = b0 + 8 <= nblk ? 0xFFu : (b0 < nblk ? (1u << (nblk - b0)) - 1u : 0u);
#pragma unroll
    for (int i = 0; i < 8; ++i) {
      uint32_t b = min(b0 + i, nblk - 1);
      const uint8_t *p = row + (size_t)b * 18;
      r.q[i] = ld_u32x2(p + 2 + 8 * kg);
      r.d[i] = ld_u16(p);
    }
  }
  template <int R, int SXROW>
  __device__ static void compute(const Raw &r, const half_t *x, const float *sx, int kg, int nrows, bool valid,
                                 float (&acc)[R]) {
    const half8_t *xa = reinterpret_cast<const half8_t *>(x + 8 * kg);
    const float *sxr[R];
#pragma unroll
    for (int r_ = 0; r_ < R; ++r_) sxr[r_] = sx + min(acc_row(r_, kg), nrows - 1) * SXROW;
#pragma unroll
    for (int i = 0; i < 8; ++i) {
      u32x2 w = r.q[i];
      uint32_t x4 = w.x >> 4, y4 = w.y >> 4;
      half8_t lo = as_half8(w.x & kNibLo, (w.x >> 8) & kNibLo, w.y & kNibLo, (w.y >> 8) & kNibLo);
      half8_t hi = as_half8(x4 & kNibLo, (x4 >> 8) & kNibLo, y4 & kNibLo, (y4 >> 8) & kNibLo);
      // elements 32i + 8kg + j (low) and 32i + 16 + 8kg + j (high)
      f32x16 p = mfma(xa[4 * i + 0], lo, zero16());
      p = mfma(xa[4 * i + 2], hi, p);
      float d = f16bits_to_f32((valid && ((r.keep >> i) & 1u)) ? r.d[i] : 0u);
#pragma unroll
      for (int r_ = 0; r_ < R; ++r_) {
        float t = fmaf(p[r_], kTwo24, -8.0f * sxr[r_][i]);
        acc[r_] = fmaf(d, t, acc[r_]);
      }
    }
  }
};

}  // namespace cuthip
