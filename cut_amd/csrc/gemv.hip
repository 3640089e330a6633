// Streaming quantized GEMV / skinny GEMM on native GGUF blocks for gfx950:
//   C[m,n] = sum_k A[m,k] * dequant(W)[n,k],  M <= 32 per pass.
//
// Supersedes MatMulQ{4,8}GemvKPar8.cu (operators/impl/matmul), whose lanes
// gather 4 bytes at a stride of N across k; here the weights stay in the GGUF
// file layout (row n = K/blk consecutive blocks) and are streamed once with
// 8- and 16-byte loads.
//
// Work decomposition.  A workgroup owns 32 consecutive weight rows and the
// whole K range; its WAVES waves split K in steps of 256 elements and their
// partial sums are folded through LDS at the end.  Inside a wave, lane l owns
// row n0 + (l & 31) and the half kg = l >> 5 of every 16-element k-slice, the
// operand layout of v_mfma_f32_32x32x16_f16 (A: activations, row m = l & 31;
// B: weights, column n = l & 31; both hold k = 8*kg .. 8*kg+7).
//
// Arithmetic.  The packed quants are turned into fp16 *subnormals* with one
// AND per pair of weights: a nibble left in bits 0-3 of a 16-bit lane is the
// fp16 number q * 2^-24 (bits 4-7: q * 2^-20), exact, and the matrix core
// multiplies subnormals exactly.  One MFMA chain therefore yields the exact
// integer dot product sum(q * x) of one quantization sub-block for 32 rows,
// which is scaled in fp32 by that row's d*sc (times 2^24 or 2^20); the
// "- min" / "- 8" / "- 32" / "+ 128" offsets become -dm * sum(x), with the
// per-sub-block sums of x precomputed once per wave next to the staged
// activations.  Products are exact and accumulation is fp32, so the result is
// at least as accurate as the reference's sequential fp32 loop.  Activations
// are consumed as fp16 (fp32 inputs are rounded to nearest-even fp16 first).
//
// The activations of a K tile are staged per wave into LDS as fp16 with each
// group of 8 stored in the order (0,2,1,3,4,6,5,7): ANDing a dword of packed
// quants with 0x000F000F pairs bytes (0,2) and, after a shift by 8, (1,3).
#include "common.hpp"

namespace cuthip {

struct GemvParams {
  const uint8_t *W;
  const void *A;
  void *C;
  Epilogue epi;
  uint32_t M, K, N, strideA, strideC;
  uint32_t nsteps;   // ceil(K / 256)
  uint32_t row_bytes;
  int a_f16, c_f16;
};

// ---- per-tile configuration -------------------------------------------------
template <int MT> struct TileCfg {
  static constexpr int R = MT <= 4 ? MT : (MT <= 8 ? 4 : 16);     // accumulator registers per lane
  static constexpr int TB = MT <= 2 ? 8 : (MT <= 4 ? 4 : (MT <= 8 ? 2 : 1));  // 256-element steps per LDS tile
  static constexpr int XROW = TB * 256 + 8;                       // halfs per staged row (+16 B against bank conflicts)
};

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
  __device__ static void compute(const Raw &r, const half_t *x, const float *sx, int kg, int half, int M,
                                 float (&acc)[R]) {
    float d = f16bits_to_f32(r.hdr.x & 0xFFFF), dmin = f16bits_to_f32(r.hdr.x >> 16);
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
      int row = min(acc_row(r_, half), M - 1);
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
  __device__ static void compute(const Raw &r, const half_t *x, const float *sx, int kg, int half, int M,
                                 float (&acc)[R]) {
    float d = f16bits_to_f32(r.d);
    const half8_t *xa = reinterpret_cast<const half8_t *>(x + 8 * kg);
    constexpr uint32_t kH45 = 0x00300030u, kH89 = 0x03000300u;
    const float *sxr[R];
#pragma unroll
    for (int r_ = 0; r_ < R; ++r_) sxr[r_] = sx + min(acc_row(r_, half), M - 1) * SXROW;
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
  struct Raw { u32x4 q[8]; uint32_t d[8]; };
  __device__ static void load(Raw &r, const uint8_t *row, uint32_t step, int kg, uint32_t K) {
    uint32_t nblk = K / 32, b0 = step * 8;
#pragma unroll
    for (int i = 0; i < 8; ++i) {
      uint32_t b = min(b0 + i, nblk - 1);
      const uint8_t *p = row + (size_t)b * 34;
      r.q[i] = ld_u32x4(p + 2 + 16 * kg);
      r.d[i] = (b0 + i < nblk) ? ld_u16(p) : 0u;   // blocks past K contribute zero
    }
  }
  template <int R, int SXROW>
  __device__ static void compute(const Raw &r, const half_t *x, const float *sx, int kg, int half, int M,
                                 float (&acc)[R]) {
    const half8_t *xa = reinterpret_cast<const half8_t *>(x + 16 * kg);
    constexpr uint32_t kByte = 0x00FF00FFu;
    const float *sxr[R];
#pragma unroll
    for (int r_ = 0; r_ < R; ++r_) sxr[r_] = sx + min(acc_row(r_, half), M - 1) * SXROW;
#pragma unroll
    for (int i = 0; i < 8; ++i) {
      u32x4 w = r.q[i] ^ u32x4{0x80808080u, 0x80808080u, 0x80808080u, 0x80808080u};
      half8_t ba = as_half8(w.x & kByte, (w.x >> 8) & kByte, w.y & kByte, (w.y >> 8) & kByte);
      half8_t bb = as_half8(w.z & kByte, (w.z >> 8) & kByte, w.w & kByte, (w.w >> 8) & kByte);
      f32x16 p = mfma(xa[4 * i + 0], ba, zero16());
      p = mfma(xa[4 * i + 1], bb, p);
      float d = f16bits_to_f32(r.d[i]);
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
  struct Raw { u32x2 q[8]; uint32_t d[8]; };
  __device__ static void load(Raw &r, const uint8_t *row, uint32_t step, int kg, uint32_t K) {
    uint32_t nblk = K / 32, b0 = step * 8;
#pragma unroll
    for (int i = 0; i < 8; ++i) {
      uint32_t b = min(b0 + i, nblk - 1);
      const uint8_t *p = row + (size_t)b * 18;
      r.q[i] = ld_u32x2(p + 2 + 8 * kg);
      r.d[i] = (b0 + i < nblk) ? ld_u16(p) : 0u;
    }
  }
  template <int R, int SXROW>
  __device__ static void compute(const Raw &r, const half_t *x, const float *sx, int kg, int half, int M,
                                 float (&acc)[R]) {
    const half8_t *xa = reinterpret_cast<const half8_t *>(x + 8 * kg);
    const float *sxr[R];
#pragma unroll
    for (int r_ = 0; r_ < R; ++r_) sxr[r_] = sx + min(acc_row(r_, half), M - 1) * SXROW;
#pragma unroll
    for (int i = 0; i < 8; ++i) {
      u32x2 w = r.q[i];
      uint32_t x4 = w.x >> 4, y4 = w.y >> 4;
      half8_t lo = as_half8(w.x & kNibLo, (w.x >> 8) & kNibLo, w.y & kNibLo, (w.y >> 8) & kNibLo);
      half8_t hi = as_half8(x4 & kNibLo, (x4 >> 8) & kNibLo, y4 & kNibLo, (y4 >> 8) & kNibLo);
      // elements 32i + 8kg + j (low) and 32i + 16 + 8kg + j (high)
      f32x16 p = mfma(xa[4 * i + 0], lo, zero16());
      p = mfma(xa[4 * i + 2], hi, p);
      float d = f16bits_to_f32(r.d[i]);
#pragma unroll
      for (int r_ = 0; r_ < R; ++r_) {
        float t = fmaf(p[r_], kTwo24, -8.0f * sxr[r_][i]);
        acc[r_] = fmaf(d, t, acc[r_]);
      }
    }
  }
};

// ---- staging of the activations -----------------------------------------------
// Copies rows [0, M) x elements [k0, k0 + steps*256) of A into the wave's LDS
// tile as fp16 in the (0,2,1,3,4,6,5,7) order and writes the sums of every
// SUBK consecutive (rounded) elements.  Elements past K are zero.
template <int SUBK, int XROW, int SXROW>
__device__ inline void stage_x(const GemvParams &p, uint32_t k0, int steps, half_t *xs, float *sxs, int lane) {
  const int groups_per_row = steps * 32;  // 8-element groups
  const int total = (int)p.M * groups_per_row;
  for (int t0 = 0; t0 < total; t0 += kWave) {
    int t = t0 + lane;
    bool active = t < total;
    int m = active ? t / groups_per_row : 0;
    int gi = active ? t - m * groups_per_row : 0;
    uint32_t k = k0 + (uint32_t)gi * 8;
    float v[8];
    if (active && k < p.K) {
      size_t off = (size_t)m * p.strideA + k;
      if (p.a_f16) {
        u32x4 raw = ld_u32x4(reinterpret_cast<const uint8_t *>(p.A) + off * 2);
        half8_t h = __builtin_bit_cast(half8_t, raw);
#pragma unroll
        for (int i = 0; i < 8; ++i) v[i] = (float)h[i];
      } else {
        const float *src = reinterpret_cast<const float *>(p.A) + off;
#pragma unroll
        for (int i = 0; i < 8; ++i) v[i] = src[i];
      }
    } else {
#pragma unroll
      for (int i = 0; i < 8; ++i) v[i] = 0.0f;
    }
    half_t h[8];
#pragma unroll
    for (int i = 0; i < 8; ++i) h[i] = (half_t)v[i];
    float s = 0.0f;
#pragma unroll
    for (int i = 0; i < 8; ++i) s += (float)h[i];
    s += __shfl_xor(s, 1);
    if (SUBK == 32) s += __shfl_xor(s, 2);
    if (active) {
      half8_t o{h[0], h[2], h[1], h[3], h[4], h[6], h[5], h[7]};
      *reinterpret_cast<half8_t *>(xs + m * XROW + gi * 8) = o;
      constexpr int per = SUBK / 8;
      if ((gi & (per - 1)) == 0) sxs[m * SXROW + gi / per] = s;
    }
  }
}

// ---- the kernel -----------------------------------------------------------------
template <int FMT, int MT, int WAVES>
__global__ void __launch_bounds__(64 * WAVES) gemv_kernel(GemvParams p) {
  using S = Step<FMT>;
  using T = TileCfg<MT>;
  constexpr int R = T::R, TB = T::TB, XROW = T::XROW, SXROW = TB * S::NSUB;
  constexpr int WAVE_LDS = MT * (XROW * 2 + SXROW * 4);  // bytes per wave
  extern __shared__ __attribute__((aligned(16))) uint8_t lds[];

  const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
  const int kg = lane >> 5, col = lane & 31;
  const uint32_t n0 = blockIdx.x * 32u;
  const uint32_t n = min(n0 + (uint32_t)col, p.N - 1);
  const uint8_t *row = p.W + (size_t)n * p.row_bytes;

  half_t *xs = reinterpret_cast<half_t *>(lds + wave * WAVE_LDS);
  float *sxs = reinterpret_cast<float *>(lds + wave * WAVE_LDS + MT * XROW * 2);
  const int mrow = min(col, (int)p.M - 1);

  const uint32_t s_begin = (uint32_t)(((uint64_t)p.nsteps * wave) / WAVES);
  const uint32_t s_end = (uint32_t)(((uint64_t)p.nsteps * (wave + 1)) / WAVES);

  float acc[R];
#pragma unroll
  for (int r = 0; r < R; ++r) acc[r] = 0.0f;

  typename S::Raw cur, nxt;
  if (s_begin < s_end) S::load(cur, row, s_begin, kg, p.K);
  for (uint32_t ts = s_begin; ts < s_end; ts += TB) {
    int tb = (int)min((uint32_t)TB, s_end - ts);
    __builtin_amdgcn_fence(__ATOMIC_ACQ_REL, "wavefront");
    stage_x<S::SUBK, XROW, SXROW>(p, ts * 256u, tb, xs, sxs, lane);
    __builtin_amdgcn_fence(__ATOMIC_ACQ_REL, "wavefront");
    __builtin_amdgcn_wave_barrier();
    for (int b = 0; b < tb; ++b) {
      uint32_t step = ts + b;
      if (step + 1 < s_end) S::load(nxt, row, step + 1, kg, p.K);
      S::template compute<R, SXROW>(cur, xs + mrow * XROW + b * 256, sxs + b * S::NSUB, kg, kg, (int)p.M, acc);
      cur = nxt;
    }
  }

  // Fold the waves' partial sums and write C with the fused epilogue.
  __syncthreads();
  float *red = reinterpret_cast<float *>(lds);  // [WAVES][MT][32], reuses the staging area
#pragma unroll
  for (int r = 0; r < R; ++r) {
    int m = acc_row(r, kg);
    if (m < (int)p.M) red[(wave * MT + m) * 32 + col] = acc[r];
  }
  __syncthreads();
  for (int t = threadIdx.x; t < (int)p.M * 32; t += 64 * WAVES) {
    int m = t >> 5, c = t & 31;
    uint32_t nn = n0 + c;
    if (nn >= p.N) continue;
    float v = 0.0f;
#pragma unroll
    for (int w = 0; w < WAVES; ++w) v += red[(w * MT + m) * 32 + c];
    store_out(p.C, p.epi, p.c_f16, (size_t)m * p.strideC + nn, v);
  }
}

template <int FMT, int MT, int WAVES> static size_t gemv_lds_bytes() {
  using S = Step<FMT>;
  using T = TileCfg<MT>;
  size_t per_wave = (size_t)MT * (T::XROW * 2 + T::TB * S::NSUB * 4);
  size_t red = (size_t)WAVES * MT * 32 * 4;
  size_t a = per_wave * WAVES;
  return a > red ? a : red;
}

template <int FMT, int MT, int WAVES> static int launch_one(const GemvParams &p, hipStream_t stream) {
  size_t lds = gemv_lds_bytes<FMT, MT, WAVES>();
  auto kern = gemv_kernel<FMT, MT, WAVES>;
  if (lds > 64 * 1024) {
    if (int rc = check_hip(hipFuncSetAttribute(reinterpret_cast<const void *>(kern),
                                               hipFuncAttributeMaxDynamicSharedMemorySize, (int)lds),
                           "hipFuncSetAttribute"))
      return rc;
  }
  dim3 grid((p.N + 31) / 32), block(64 * WAVES);
  hipLaunchKernelGGL(kern, grid, block, lds, stream, p);
  return check_hip(hipGetLastError(), "gemv launch");
}

template <int FMT, int MT> static int launch_waves(const GemvParams &p, int waves, hipStream_t stream) {
  switch (waves) {
  case 1: return launch_one<FMT, MT, 1>(p, stream);
  case 2: return launch_one<FMT, MT, 2>(p, stream);
  case 4: return launch_one<FMT, MT, 4>(p, stream);
  default:
    // the 32-row activation tile keeps 16 accumulators per lane: at most 4 waves
    if constexpr (MT > 8) return launch_one<FMT, MT, 4>(p, stream);
    else return launch_one<FMT, MT, 8>(p, stream);
  }
}

// Waves per workgroup: split K while every wave keeps >= 4 steps of 256, and
// further (down to 1 step) while the grid has fewer than 4 waves per CU.
static int pick_waves(uint32_t N, uint32_t nsteps, int mt) {
  uint32_t tiles = (N + 31) / 32;
  int max_waves = mt > 8 ? 4 : 8;
  int w = 1;
  while (w < max_waves) {
    uint32_t per_wave = nsteps / (uint32_t)(2 * w);  // steps per wave after doubling
    bool plenty = per_wave >= 4;
    bool starved = (uint64_t)tiles * w < 1024 && per_wave >= 1;  // < 4 waves per CU
    if (!plenty && !starved) break;
    w *= 2;
  }
  return w;
}

template <int FMT> static int launch_fmt(GemvParams p, hipStream_t stream) {
  // M <= 8 in one pass; larger M in passes of up to 32 activation rows.
  if (p.M <= 8) {
    int mt = p.M <= 1 ? 1 : p.M <= 2 ? 2 : p.M <= 4 ? 4 : 8;
    int w = pick_waves(p.N, p.nsteps, mt);
    switch (mt) {
    case 1: return launch_waves<FMT, 1>(p, w, stream);
    case 2: return launch_waves<FMT, 2>(p, w, stream);
    case 4: return launch_waves<FMT, 4>(p, w, stream);
    default: return launch_waves<FMT, 8>(p, w, stream);
    }
  }
  uint32_t M = p.M;
  size_t a_es = p.a_f16 ? 2 : 4, c_es = p.c_f16 ? 2 : 4;
  for (uint32_t m0 = 0; m0 < M; m0 += 32) {
    GemvParams q = p;
    q.M = min(32u, M - m0);
    q.A = reinterpret_cast<const uint8_t *>(p.A) + (size_t)m0 * p.strideA * a_es;
    q.C = reinterpret_cast<uint8_t *>(p.C) + (size_t)m0 * p.strideC * c_es;
    if (p.epi.D) q.epi.D = reinterpret_cast<const uint8_t *>(p.epi.D) + (size_t)m0 * p.strideC * c_es;
    int w = pick_waves(p.N, p.nsteps, 32);
    if (int rc = launch_waves<FMT, 32>(q, w, stream)) return rc;
  }
  return CUTHIP_OK;
}

int launch_gemv(int fmt, const GemvParams &p, hipStream_t stream) {
  switch (fmt) {
  case CUTHIP_Q8_0: return launch_fmt<CUTHIP_Q8_0>(p, stream);
  case CUTHIP_Q4_0: return launch_fmt<CUTHIP_Q4_0>(p, stream);
  case CUTHIP_Q4_K: return launch_fmt<CUTHIP_Q4_K>(p, stream);
  default: return launch_fmt<CUTHIP_Q6_K>(p, stream);
  }
}

}  // namespace cuthip

extern "C" int cuthip_matmul_gguf(int fmt, const void *W, const void *A, int a_dtype, void *C, int c_dtype, uint32_t M,
                                  uint32_t K, uint32_t N, uint32_t strideA, uint32_t strideC, int epilogue,
                                  int epilogue_op, const void *D, int variant, void *stream) {
  using namespace cuthip;
  if (fmt < CUTHIP_Q8_0 || fmt > CUTHIP_Q6_K) {
    set_error("cuthip_matmul_gguf: unknown format %d", fmt);
    return CUTHIP_ERR_INVALID;
  }
  if ((a_dtype != CUTHIP_F32 && a_dtype != CUTHIP_F16) || (c_dtype != CUTHIP_F32 && c_dtype != CUTHIP_F16)) {
    set_error("cuthip_matmul_gguf: unsupported dtype (a %d, c %d)", a_dtype, c_dtype);
    return CUTHIP_ERR_INVALID;
  }
  if (M == 0 || N == 0) return CUTHIP_OK;
  if (K == 0 || K % fmt_elems(fmt) != 0) {
    set_error("cuthip_matmul_gguf: K (%u) must be a positive multiple of the block size %d", K, fmt_elems(fmt));
    return CUTHIP_ERR_INVALID;
  }
  if (!W || !A || !C) {
    set_error("cuthip_matmul_gguf: null device pointer");
    return CUTHIP_ERR_INVALID;
  }
  if (strideA < K || strideC < N) {
    set_error("cuthip_matmul_gguf: strideA (%u) < K (%u) or strideC (%u) < N (%u)", strideA, K, strideC, N);
    return CUTHIP_ERR_INVALID;
  }
  if (epilogue < CUTHIP_EPI_NONE || epilogue > CUTHIP_EPI_BINARY) {
    set_error("cuthip_matmul_gguf: unknown epilogue %d", epilogue);
    return CUTHIP_ERR_INVALID;
  }
  if (epilogue == CUTHIP_EPI_BINARY && !D) {
    set_error("cuthip_matmul_gguf: binary epilogue needs the operand D");
    return CUTHIP_ERR_INVALID;
  }
  if ((uintptr_t)W % 2 != 0 || (uintptr_t)A % (a_dtype == CUTHIP_F16 ? 2 : 4) != 0) {
    set_error("cuthip_matmul_gguf: misaligned W or A pointer");
    return CUTHIP_ERR_INVALID;
  }
  int nvar = cuthip_variant_count(CUTHIP_OP_MATMUL_GGUF);
  if (variant < -1 || variant >= nvar) {
    set_error("cuthip_matmul_gguf: unknown variant index %d (table has %d)", variant, nvar);
    return CUTHIP_ERR_UNKNOWN_VARIANT;
  }
  uint64_t row_bytes = (uint64_t)(K / fmt_elems(fmt)) * fmt_bytes(fmt);
  if (row_bytes > 0xFFFFFFFFull) {
    set_error("cuthip_matmul_gguf: K too large");
    return CUTHIP_ERR_INVALID;
  }
  GemvParams p;
  p.W = reinterpret_cast<const uint8_t *>(W);
  p.A = A;
  p.C = C;
  p.epi = Epilogue{epilogue, epilogue_op, epilogue == CUTHIP_EPI_BINARY ? D : nullptr};
  p.M = M; p.K = K; p.N = N; p.strideA = strideA; p.strideC = strideC;
  p.nsteps = (K + 255) / 256;
  p.row_bytes = (uint32_t)row_bytes;
  p.a_f16 = a_dtype == CUTHIP_F16;
  p.c_f16 = c_dtype == CUTHIP_F16;
  return launch_gemv(fmt, p, reinterpret_cast<hipStream_t>(stream));
}
