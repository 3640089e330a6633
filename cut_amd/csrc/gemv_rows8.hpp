// Streaming quantized GEMV on native GGUF blocks for gfx950, batch 1..4:
//   C[m,n] = sum_k A[m,k] * dequant(W)[n,k]
//
// Supersedes MatMulQ{4,8}GemvKPar8.cu (operators/impl/matmul), whose lanes
// gather 4 bytes at a stride of N across k.  Here the weights stay in the GGUF
// file layout (row n = K/blk consecutive blocks) and every wave instruction
// reads 8 rows x 128 contiguous bytes (16 bytes per lane), which is what the
// memory system streams best; nothing is read twice from HBM.
//
// Work decomposition.  K is cut in steps of 256 elements.  One wave owns 8
// consecutive weight rows and a contiguous range of steps; a workgroup is RWG
// row groups x KW step ranges.  Inside a wave the 32 B-columns of
// v_mfma_f32_32x32x16_f16 are (row r, piece g) pairs, column j = 4r + g: the
// four pieces of a row cover the four 64-element quarters of the step, so the
// eight lanes (4 pieces x 2 k-halves) of a row load one contiguous run.  The
// MFMA A-row j carries the activations of batch row j/4 for the same quarter
// j%4, hence C[j][j'] is a valid partial sum when j%4 == j'%4; every lane
// scales all its accumulator registers with its own column's scales and the
// valid one is picked once at the end, followed by a 4-lane sum over pieces.
//
// Arithmetic.  Quants become fp16 subnormals with one AND per pair of weights
// (a nibble in bits 0-3 of a 16-bit lane is q * 2^-24, in bits 4-7 q * 2^-20;
// the matrix core multiplies subnormals exactly), so an MFMA chain gives the
// exact integer dot product sum(q * x) of one quantization sub-block, which is
// scaled in fp32 by d*sc; the "- min" / "- 8" / "- 32" / "+ 128" offsets become
// -(offset scale) * sum(x) with per-sub-block sums of x kept next to the
// staged activations.  Formats whose sub-block is spread over both k-halves of
// a column (Q6_K, Q8_0, Q4_0) first exchange 8-byte halves between lane l and
// lane l+32 (v_permlane32_swap), so that one MFMA always sees one sub-block.
// Activations are consumed as fp16 (fp32 inputs are rounded to nearest even).
//
// Pipeline.  The workgroup stages the activations once: fp16, each group of 8
// in the order (0,2,1,3,4,6,5,7) (the order AND/shift unpacking produces), 64
// elements per 144-byte LDS group so the four pieces hit different banks.
// Each lane then keeps D steps of weight loads in flight in a register ring;
// the loop body is branch-free, so every step waits only for its own loads.
#pragma once
#include "gemv_formats.hpp"

namespace cuthip {

#ifndef CUTHIP_ROWS8_DOTMAX
#define CUTHIP_ROWS8_DOTMAX 1
#endif
constexpr int kRows8DotMax = CUTHIP_ROWS8_DOTMAX;   // batch rows up to which the dot-product path is taken
// Q6_K keeps the dot-product path for two rows (14336 x 4096: 15.3 us either way, 28672 x 4096 25.4 against 26.0) and
// takes the matrix core from three (3 / 4 rows: 15.6 / 15.8 us against 17.2 / 17.3; before that path's ring of loads
// was repaired it lost up to four rows, 18.9 / 20.2 against 15.1 / 18.0); Q4_K and Q8_0 at 2 rows are faster through
// the matrix core: 9.4 against 11.3 us, 17.0 against 17.3
#ifndef CUTHIP_ROWS8_DOTMAX_Q6K
#define CUTHIP_ROWS8_DOTMAX_Q6K 2
#endif
template <int FMT> constexpr int rows8_dot_max() { return FMT == CUTHIP_Q6_K ? CUTHIP_ROWS8_DOTMAX_Q6K : kRows8DotMax; }
constexpr int kXGroup = 72;             // halfs per staged 64-element group (64 + 8 pad)
constexpr int kXStep = 4 * kXGroup;     // halfs per 256-element step

__device__ inline void swap_halves(uint32_t &lo, uint32_t &hi) {
  // lanes 0-31: hi <- partner's lo ; lanes 32-63: lo <- partner's hi  (partner = lane ^ 32)
  auto r = __builtin_amdgcn_permlane32_swap(lo, hi, false, false);
  lo = r[0];
  hi = r[1];
}

typedef _Float16 half2_t __attribute__((ext_vector_type(2)));
__device__ inline float dot2(uint32_t a, uint32_t b, float c) {   // v_dot2_f32_f16; exact for subnormal a
  return __builtin_amdgcn_fdot2(__builtin_bit_cast(half2_t, a), __builtin_bit_cast(half2_t, b), c, false);
}
// 8 products: the bytes of (u0, u1) masked to fp16 subnormals against 8 staged activations
__device__ inline float dot_pairs(uint32_t u0, uint32_t u1, const u32x4 &x, uint32_t mask, float s) {
  s = dot2(u0 & mask, x.x, s);
  s = dot2((u0 >> 8) & mask, x.y, s);
  s = dot2(u1 & mask, x.z, s);
  return dot2((u1 >> 8) & mask, x.w, s);
}

struct LaneCtx {
  int g, kg;            // piece (64-element quarter of the step) and k-half
  uint32_t c0, c1, c2, c3;  // per-lane constants of the format
};

// Sums across lanes without the LDS crossbar (a ds_bpermute round trip is about a hundred cycles, and these sit on
// the tail of every wave).  Every lane of the wave must be active.  add_xor4 / add_xor8 mirror 8 / 16 lanes, which is
// the xor exchange once the smaller groups hold equal sums, so they are used in that order only.
template <int CTRL> __device__ __forceinline__ float dpp_move(float v) {
  return __builtin_bit_cast(float, __builtin_amdgcn_update_dpp(0, __builtin_bit_cast(int, v), CTRL, 0xF, 0xF, true));
}
__device__ __forceinline__ float add_xor1(float v) { return v + dpp_move<0xB1>(v); }    // quad_perm (1 0 3 2)
__device__ __forceinline__ float add_xor2(float v) { return v + dpp_move<0x4E>(v); }    // quad_perm (2 3 0 1)
__device__ __forceinline__ float add_xor4(float v) { return v + dpp_move<0x141>(v); }   // row_half_mirror
__device__ __forceinline__ float add_xor8(float v) { return v + dpp_move<0x140>(v); }   // row_mirror
// (the swaps exchange the odd rows / upper half of the first operand with the even rows / lower half of the second.
// The elements of the result are read into scalars first: __builtin_bit_cast applied to a vector element expression
// reads element 0 whatever the index, with this compiler)
__device__ __forceinline__ float add_xor16(float v) {
  const auto r = __builtin_amdgcn_permlane16_swap(__builtin_bit_cast(uint32_t, v), __builtin_bit_cast(uint32_t, v), false, false);
  const uint32_t mine = r[0], other = r[1];
  return __builtin_bit_cast(float, mine) + __builtin_bit_cast(float, other);
}
__device__ __forceinline__ float add_xor32(float v) {
  const auto r = __builtin_amdgcn_permlane32_swap(__builtin_bit_cast(uint32_t, v), __builtin_bit_cast(uint32_t, v), false, false);
  const uint32_t mine = r[0], other = r[1];
  return __builtin_bit_cast(float, mine) + __builtin_bit_cast(float, other);
}
__device__ inline float wave_sum_all(float v) {
  return add_xor32(add_xor16(add_xor8(add_xor4(add_xor2(add_xor1(v))))));
}

// One output row of a matmul with the RoPE / cache-append epilogue: v = this row's product, partner = the
// neighbouring row's (row ^ 1), cs / sn = the table entries of the pair at the current position.
__device__ inline void rope_store(const RopeAppend &r, uint32_t row, float v, float partner, float cs, float sn, uint32_t pos) {
  if (pos >= r.max_pos) return;
  if (r.mode == 2) {
    r.v_cache[(size_t)pos * r.kv_stride + row] = (half_t)v;
    return;
  }
  const uint32_t hd = r.head_dim, w = row % hd, b = w & 1u, d = (w >> 1) + b * (hd / 2);
  const float x0 = b ? partner : v, x1 = b ? v : partner;   // elements d and d + half of the head, un-rotated
  const float o = b ? x0 * sn + x1 * cs : x0 * cs - x1 * sn;
  if (row < r.q_dim) {
    const size_t i = (size_t)(row - w) + d;
    if (r.q_out_f16) reinterpret_cast<half_t *>(r.q_out)[i] = (half_t)o;
    else reinterpret_cast<float *>(r.q_out)[i] = o;
  } else {
    r.k_cache[(size_t)pos * r.kv_stride + (row - r.q_dim - w) + d] = (half_t)o;
  }
}

template <int FMT> struct Rows8;

// ---- Q4_K -------------------------------------------------------------------
// 144 B = [d][dmin][scales:12][qs:128]; piece g = qs[32g..32g+31]: low nibbles
// are sub-block 2g, high nibbles sub-block 2g+1; lane kg takes bytes 16kg..+15.
template <> struct Rows8<CUTHIP_Q4_K> {
  static constexpr int NSUB = 8, SUBK = 32;
  struct Raw { u32x4 hdr, q; };
  __device__ static void init(LaneCtx &c) {
    c.c0 = 16u * (c.g & 1);                 // bit offset of this piece's byte pair inside a scale dword
    c.c1 = c.g < 2 ? 0x3F3Fu : 0u;          // 6-bit fields of sub-blocks 0-3
    c.c2 = c.g < 2 ? 0u : 0x0F0Fu;          // low 4 bits of sub-blocks 4-7
    c.c3 = c.g < 2 ? 0u : 0x3030u;          // their upper 2 bits, taken from bits 6-7 of dword 0 / 1
  }
  __device__ static void load(Raw &r, const uint8_t *row, uint32_t step, const LaneCtx &c, uint32_t) {
    const uint8_t *p = row + (size_t)step * 144;
    r.hdr = ld_u32x4(p);
    r.q = ld_u32x4(p + 16 + 32 * c.g + 16 * c.kg);
  }
  // xa: staged x of this lane's A-row at (step, piece, kg); sx: sums of x for (batch row of acc quad q, step, piece)
  template <int R>
  __device__ static void compute(const Raw &r, const half_t *xa, const float *const *sx, const LaneCtx &c,
                                 float (&acc)[R], float (&cacc)[(R + 3) / 4]) {
    float d = f16bits_to_f32(r.hdr.x & 0xFFFF), dmin = f16bits_to_f32(r.hdr.x >> 16);
    uint32_t a0 = r.hdr.y >> c.c0, a1 = r.hdr.z >> c.c0, a2 = r.hdr.w >> c.c0;
    uint32_t scp = (a0 & c.c1) | (a2 & c.c2) | ((a0 >> 2) & c.c3);          // (sc[2g], sc[2g+1]) in bytes 0, 1
    uint32_t mp = (a1 & c.c1) | ((a2 >> 4) & c.c2) | ((a1 >> 2) & c.c3);   // (m[2g], m[2g+1])
    float ds0 = d * kTwo24 * cvt_ubyte0(scp), ds1 = d * kTwo20 * cvt_ubyte1(scp);
    float dm0 = dmin * cvt_ubyte0(mp), dm1 = dmin * cvt_ubyte1(mp);
    u32x4 w = r.q;
    half8_t lo_a = as_half8(w.x & kNibLo, (w.x >> 8) & kNibLo, w.y & kNibLo, (w.y >> 8) & kNibLo);
    half8_t lo_b = as_half8(w.z & kNibLo, (w.z >> 8) & kNibLo, w.w & kNibLo, (w.w >> 8) & kNibLo);
    half8_t hi_a = as_half8(w.x & kNibHi, (w.x >> 8) & kNibHi, w.y & kNibHi, (w.y >> 8) & kNibHi);
    half8_t hi_b = as_half8(w.z & kNibHi, (w.z >> 8) & kNibHi, w.w & kNibHi, (w.w >> 8) & kNibHi);
    const half8_t *x8 = reinterpret_cast<const half8_t *>(xa);   // elements 64g + 16kg + {0, 8, 32, 40}
    f32x16 p = mfma(x8[0], lo_a, zero16());
    f32x16 q = mfma(x8[4], hi_a, zero16());
    p = mfma(x8[1], lo_b, p);
    q = mfma(x8[5], hi_b, q);
    fma_acc<R>(acc, p, ds0);
    fma_acc<R>(acc, q, ds1);
#pragma unroll
    for (int qd = 0; qd < (R + 3) / 4; ++qd) {
      const float *s = sx[qd] + 2 * c.g;
      cacc[qd] = fmaf(dm0, s[0], cacc[qd]);
      cacc[qd] = fmaf(dm1, s[1], cacc[qd]);
    }
  }
  __device__ static float finish(float acc, float cacc) { return acc - cacc; }

  // Batch 1 without the matrix core: the lane's 16 low and 16 high nibbles against its own 32 activations.
  // Both k-halves of a piece add half of the "- min" term, so that their sum carries it once.
  __device__ static int x_offset(const LaneCtx &c) { return c.g * kXGroup + 16 * c.kg; }
  __device__ static void init_dot(LaneCtx &c) { init(c); }
  __device__ static int x_offset_dot(const LaneCtx &c) { return c.g * kXGroup + 16 * c.kg; }
  template <int MT>
  __device__ static void dot(const Raw &r, const half_t *xa, int xrow, const float *sx, int sxrow, const LaneCtx &c,
                             float (&acc)[MT], float (&cacc)[MT]) {
    float d = f16bits_to_f32(r.hdr.x & 0xFFFF), dmin = f16bits_to_f32(r.hdr.x >> 16);
    uint32_t a0 = r.hdr.y >> c.c0, a1 = r.hdr.z >> c.c0, a2 = r.hdr.w >> c.c0;
    uint32_t scp = (a0 & c.c1) | (a2 & c.c2) | ((a0 >> 2) & c.c3);
    uint32_t mp = (a1 & c.c1) | ((a2 >> 4) & c.c2) | ((a1 >> 2) & c.c3);
    float ds0 = d * kTwo24 * cvt_ubyte0(scp), ds1 = d * kTwo20 * cvt_ubyte1(scp);
    float dm0 = dmin * cvt_ubyte0(mp), dm1 = dmin * cvt_ubyte1(mp);
#pragma unroll
    for (int m = 0; m < MT; ++m) {
      const u32x4 *x4 = reinterpret_cast<const u32x4 *>(xa + m * xrow);   // elements 64g + 16kg + {0, 8, 32, 40}
      u32x4 xl0 = x4[0], xl1 = x4[1], xh0 = x4[4], xh1 = x4[5];
      float pl = dot_pairs(r.q.x, r.q.y, xl0, kNibLo, 0.0f), ph = dot_pairs(r.q.x, r.q.y, xh0, kNibHi, 0.0f);
      pl = dot_pairs(r.q.z, r.q.w, xl1, kNibLo, pl);
      ph = dot_pairs(r.q.z, r.q.w, xh1, kNibHi, ph);
      acc[m] = fmaf(pl, ds0, acc[m]);
      acc[m] = fmaf(ph, ds1, acc[m]);
      cacc[m] = fmaf(dm0, sx[m * sxrow + 2 * c.g], cacc[m]);
      cacc[m] = fmaf(dm1, sx[m * sxrow + 2 * c.g + 1], cacc[m]);
    }
  }
  __device__ static float finish_dot(float acc, float cacc) { return fmaf(-0.5f, cacc, acc); }
};

// ---- Q6_K -------------------------------------------------------------------
// 210 B = [ql:128][qh:64][sc:16 x i8][d].  Piece g = (H = g>>1, sigma = g&1)
// owns ql[64H+32sigma .. +31]: low nibbles are quarter s = sigma, high nibbles
// quarter s = sigma+2 of half H; qh[32H + l] holds bits 4-5 of all four
// quarters.  Sub-blocks are 16 elements (lam = l>>4).  Lane kg loads the 16
// bytes of lam = kg and swaps halves with its partner, after which both hold
// bytes 8kg..8kg+7 of lam = 0 (registers 0-1) and lam = 1 (registers 2-3).
template <> struct Rows8<CUTHIP_Q6_K> {
  static constexpr int NSUB = 16, SUBK = 16;
  // sc: the 8 scale bytes of this lane's half H (dwords 2H and 2H + 1 of the 16): an 8-byte load.  Loading all 16
  // (one 16-byte load per lane, the same address for the 8 lanes of a row, 2-byte aligned) cost a tenth of the kernel:
  // 128256 x 4096 at batch 1 102.6 us with the 16-byte load, 94.3 with this one, 104.9 with two 2-byte loads of just
  // the byte pairs a lane uses (an instruction more), 78 without any scale load.
  // qh: this lane's half (8 bytes: sigma picks which) of the 16 high-bit bytes that it shares with its neighbour of the
  // other sigma; the two halves are exchanged with DPP moves inside the quad where they are used
  // sd: one dword.  In the kg = 0 lane scale dword 2H + sigma (the neighbour of the other sigma holds the other one of
  // the half), in the kg = 1 lane bytes 206-209 of the block (d in the upper half); the two lanes exchange them where
  // they are used, one load per lane and step less than with d loaded by every lane.
  struct Raw { u32x4 ql; u32x2 qh; uint32_t sd; };
  __device__ static void high_bits(const u32x2 &h, uint32_t (&qh)[4]) {
    const int a = (int)h.x, b = (int)h.y;
    qh[0] = (uint32_t)__builtin_amdgcn_mov_dpp(a, 0xA0, 0xF, 0xF, true);   // quad_perm [0,0,2,2]: the sigma = 0 lane's half
    qh[1] = (uint32_t)__builtin_amdgcn_mov_dpp(b, 0xA0, 0xF, 0xF, true);
    qh[2] = (uint32_t)__builtin_amdgcn_mov_dpp(a, 0xF5, 0xF, 0xF, true);   // quad_perm [1,1,3,3]: the sigma = 1 lane's half
    qh[3] = (uint32_t)__builtin_amdgcn_mov_dpp(b, 0xF5, 0xF, 0xF, true);
  }
  __device__ static void init(LaneCtx &c) {
    c.c0 = 2u * (c.g & 1);        // qh bit offset of quarter sigma
    c.c1 = 16u * (c.g & 1);       // bit offset of scale byte pair (2 sigma, 2 sigma + 1) inside its dword
    c.c2 = (uint32_t)(c.g >> 1);  // H
    c.c3 = c.kg ? 206u : 192u + 8u * c.c2 + 2u * c.c0;   // byte offset of this lane's dword sd
  }
  // both lanes of a pair: the scale dword of its kg = 0 lane and d from its kg = 1 lane
  __device__ static void scales_and_d(uint32_t sd, uint32_t &sc, float &d) {
    uint32_t a = sd, b = sd;
    swap_halves(a, b);
    sc = a;
    d = f16bits_to_f32(b >> 16);
  }
  __device__ static void load(Raw &r, const uint8_t *row, uint32_t step, const LaneCtx &c, uint32_t) {
    const uint8_t *p = row + (size_t)step * 210;
    r.ql = ld_u32x4(p + 32 * c.g + 16 * c.kg);
    r.qh = ld_u32x2(p + 128 + 32 * (c.g >> 1) + 16 * c.kg + 8 * (c.g & 1));
    r.sd = ld_u32(p + c.c3);
  }
  template <int R>
  __device__ static void compute(const Raw &r, const half_t *xa, const float *const *sx, const LaneCtx &c,
                                 float (&acc)[R], float (&cacc)[(R + 3) / 4]) {
    constexpr uint32_t kH45 = 0x00300030u, kH89 = 0x03000300u;
    // The swaps below work in place on single registers.  The ring's 16-byte values pass through this pin as whole
    // tuples: without it the compiler keeps their halves in separate registers across the loop and copies them out
    // of a load's destination right behind the load, i.e. it waits for loads it has just issued (s_waitcnt vmcnt(3)
    // with four steps in flight) and the ring runs one step at a time.
    u32x4 tql = r.ql;
    u32x2 tqh = r.qh;
    asm volatile("" : "+v"(tql), "+v"(tqh));
    uint32_t ql[4] = {tql.x, tql.y, tql.z, tql.w}, qh[4];
    high_bits(tqh, qh);
    swap_halves(ql[0], ql[2]); swap_halves(ql[1], ql[3]);
    swap_halves(qh[0], qh[2]); swap_halves(qh[1], qh[3]);
    float d;
    uint32_t sc;
    scales_and_d(r.sd, sc, d);
    uint32_t wlo = (uint32_t)__builtin_amdgcn_mov_dpp((int)sc, 0xA0, 0xF, 0xF, true);   // dword 2H (quarter sigma), from the sigma = 0 lane
    uint32_t whi = (uint32_t)__builtin_amdgcn_mov_dpp((int)sc, 0xF5, 0xF, 0xF, true);   // dword 2H+1 (quarter sigma+2), from the sigma = 1 lane
    const half8_t *x8 = reinterpret_cast<const half8_t *>(xa);
    // x8 offsets (in 8-half chunks): quarter sigma, lam: 2*lam ; quarter sigma+2, lam: 9 + 2*lam  (72 halfs = 9 chunks)
#pragma unroll
    for (int lam = 0; lam < 2; ++lam) {
      uint32_t v_lo[4], v_hi[4];
#pragma unroll
      for (int k = 0; k < 2; ++k) {
        uint32_t w = ql[2 * lam + k], hs = qh[2 * lam + k] >> c.c0;
        uint32_t w8 = w >> 8, hl = hs << 4, hr = hs >> 4;
        v_lo[2 * k + 0] = (w & kNibLo) | (hl & kH45);
        v_lo[2 * k + 1] = (w8 & kNibLo) | (hr & kH45);
        v_hi[2 * k + 0] = (w & kNibHi) | (hl & kH89);
        v_hi[2 * k + 1] = (w8 & kNibHi) | (hr & kH89);
      }
      f32x16 p = mfma(x8[2 * lam], as_half8(v_lo[0], v_lo[1], v_lo[2], v_lo[3]), zero16());
      f32x16 q = mfma(x8[9 + 2 * lam], as_half8(v_hi[0], v_hi[1], v_hi[2], v_hi[3]), zero16());
      float s_lo = (float)(int)__builtin_amdgcn_sbfe((int)wlo, c.c1 + 8 * lam, 8);
      float s_hi = (float)(int)__builtin_amdgcn_sbfe((int)whi, c.c1 + 8 * lam, 8);
      float dlo = d * s_lo, dhi = d * s_hi;
      fma_acc<R>(acc, p, dlo * kTwo24);
      fma_acc<R>(acc, q, dhi * kTwo20);
      int j_lo = 8 * (c.g >> 1) + 2 * (c.g & 1) + lam;   // sub-block of (H, s = sigma, lam); s = sigma+2 is 4 further
#pragma unroll
      for (int qd = 0; qd < (R + 3) / 4; ++qd) {
        cacc[qd] = fmaf(dlo, sx[qd][j_lo], cacc[qd]);
        cacc[qd] = fmaf(dhi, sx[qd][j_lo + 4], cacc[qd]);
      }
    }
  }
  __device__ static float finish(float acc, float cacc) { return fmaf(-32.0f, cacc, acc); }

  // Batch 1 without the matrix core: lane kg owns the 16-element sub-blocks lam = kg of quarters sigma and sigma+2.
  __device__ static void init_dot(LaneCtx &c) {
    init(c);
    c.c1 += 8u * c.kg;   // bit offset of scale byte 2 sigma + kg
  }
  __device__ static int x_offset(const LaneCtx &c) { return 2 * (c.g >> 1) * kXGroup + 32 * (c.g & 1) + 8 * c.kg; }
  __device__ static int x_offset_dot(const LaneCtx &c) { return 2 * (c.g >> 1) * kXGroup + 32 * (c.g & 1) + 16 * c.kg; }
  template <int MT>
  __device__ static void dot(const Raw &r, const half_t *xa, int xrow, const float *sx, int sxrow, const LaneCtx &c,
                             float (&acc)[MT], float (&cacc)[MT]) {
    constexpr uint32_t kH45 = 0x00300030u, kH89 = 0x03000300u;
    const uint32_t ql[4] = {r.ql.x, r.ql.y, r.ql.z, r.ql.w};
    uint32_t qh[4];
    high_bits(r.qh, qh);
    uint32_t vl[8], vh[8];   // 6-bit quants as fp16 subnormals: q * 2^-24 (quarter sigma) and q * 2^-20 (quarter sigma+2)
#pragma unroll
    for (int k = 0; k < 4; ++k) {
      uint32_t w = ql[k], hs = qh[k] >> c.c0;
      uint32_t w8 = w >> 8, hl = hs << 4, hr = hs >> 4;
      vl[2 * k] = (w & kNibLo) | (hl & kH45);
      vl[2 * k + 1] = (w8 & kNibLo) | (hr & kH45);
      vh[2 * k] = (w & kNibHi) | (hl & kH89);
      vh[2 * k + 1] = (w8 & kNibHi) | (hr & kH89);
    }
    float d;
    uint32_t sc;
    scales_and_d(r.sd, sc, d);
    uint32_t wlo = (uint32_t)__builtin_amdgcn_mov_dpp((int)sc, 0xA0, 0xF, 0xF, true);
    uint32_t whi = (uint32_t)__builtin_amdgcn_mov_dpp((int)sc, 0xF5, 0xF, 0xF, true);
    float dlo = d * (float)(int)__builtin_amdgcn_sbfe((int)wlo, c.c1, 8);
    float dhi = d * (float)(int)__builtin_amdgcn_sbfe((int)whi, c.c1, 8);
    const int j_lo = 8 * (c.g >> 1) + 2 * (c.g & 1) + c.kg;
#pragma unroll
    for (int m = 0; m < MT; ++m) {
      const u32x4 *x4 = reinterpret_cast<const u32x4 *>(xa + m * xrow);   // quarter sigma: chunks 0, 1 ; sigma+2: 9, 10
      const u32x4 xl0 = x4[0], xl1 = x4[1], xh0 = x4[9], xh1 = x4[10];
      float pl = dot2(vl[0], xl0.x, 0.0f), ph = dot2(vh[0], xh0.x, 0.0f);
      pl = dot2(vl[1], xl0.y, pl); ph = dot2(vh[1], xh0.y, ph);
      pl = dot2(vl[2], xl0.z, pl); ph = dot2(vh[2], xh0.z, ph);
      pl = dot2(vl[3], xl0.w, pl); ph = dot2(vh[3], xh0.w, ph);
      pl = dot2(vl[4], xl1.x, pl); ph = dot2(vh[4], xh1.x, ph);
      pl = dot2(vl[5], xl1.y, pl); ph = dot2(vh[5], xh1.y, ph);
      pl = dot2(vl[6], xl1.z, pl); ph = dot2(vh[6], xh1.z, ph);
      pl = dot2(vl[7], xl1.w, pl); ph = dot2(vh[7], xh1.w, ph);
      acc[m] = fmaf(pl, dlo * kTwo24, acc[m]);
      acc[m] = fmaf(ph, dhi * kTwo20, acc[m]);
      cacc[m] = fmaf(dlo, sx[m * sxrow + j_lo], cacc[m]);
      cacc[m] = fmaf(dhi, sx[m * sxrow + j_lo + 4], cacc[m]);
    }
  }
  __device__ static float finish_dot(float acc, float cacc) { return fmaf(-32.0f, cacc, acc); }
};

// ---- Q8_0 -------------------------------------------------------------------
// 34 B = [d][q:32 x i8]; a step is 8 blocks, piece g = blocks 2g and 2g+1.
// Lane kg loads block 2g+kg; after the swap registers (0,1) / (4,5) hold bytes
// 8kg..+7 / 16+8kg..+7 of block 2g and (2,3) / (6,7) those of block 2g+1.
template <> struct Rows8<CUTHIP_Q8_0> {
  static constexpr int NSUB = 8, SUBK = 32;
  // keep: 0xFFFF, or 0 for a block past K (its scale is masked to zero where it is used: touching the loaded value
  // here would make the load wait for itself and every load before it, and the ring of steps would run in turn)
  struct Raw { u32x4 q0, q1; uint32_t d, keep; };
  __device__ static void init(LaneCtx &c) { c.c0 = c.c1 = c.c2 = c.c3 = 0; }
  __device__ static void load(Raw &r, const uint8_t *row, uint32_t step, const LaneCtx &c, uint32_t K) {
    uint32_t nblk = K / 32, b = step * 8 + 2 * c.g + c.kg;
    const uint8_t *p = row + (size_t)min(b, nblk - 1) * 34;
    r.q0 = ld_u32x4(p + 2);
    r.q1 = ld_u32x4(p + 18);
    r.d = ld_u16(p);
    r.keep = b < nblk ? 0xFFFFu : 0u;   // blocks past K contribute zero
  }
  template <int R>
  __device__ static void compute(const Raw &r, const half_t *xa, const float *const *sx, const LaneCtx &c,
                                 float (&acc)[R], float (&cacc)[(R + 3) / 4]) {
    constexpr uint32_t kByte = 0x00FF00FFu, kFlip = 0x80808080u;
    uint32_t w[8] = {r.q0.x ^ kFlip, r.q0.y ^ kFlip, r.q0.z ^ kFlip, r.q0.w ^ kFlip,
                     r.q1.x ^ kFlip, r.q1.y ^ kFlip, r.q1.z ^ kFlip, r.q1.w ^ kFlip};
    swap_halves(w[0], w[2]); swap_halves(w[1], w[3]);
    swap_halves(w[4], w[6]); swap_halves(w[5], w[7]);
    uint32_t da = r.d & r.keep, db = da;
    swap_halves(da, db);   // lanes 0-31: (own, partner) ; lanes 32-63: (partner, own) = (block 2g, block 2g+1)
    float d_a = f16bits_to_f32(da), d_b = f16bits_to_f32(db);
    const half8_t *x8 = reinterpret_cast<const half8_t *>(xa);   // elements 64g + 8kg + {0, 16, 32, 48}
    auto op = [&](uint32_t u0, uint32_t u1) { return as_half8(u0 & kByte, (u0 >> 8) & kByte, u1 & kByte, (u1 >> 8) & kByte); };
    f32x16 p = mfma(x8[0], op(w[0], w[1]), zero16());
    f32x16 q = mfma(x8[4], op(w[2], w[3]), zero16());
    p = mfma(x8[2], op(w[4], w[5]), p);
    q = mfma(x8[6], op(w[6], w[7]), q);
    fma_acc<R>(acc, p, d_a * kTwo24);
    fma_acc<R>(acc, q, d_b * kTwo24);
#pragma unroll
    for (int qd = 0; qd < (R + 3) / 4; ++qd) {
      const float *s = sx[qd] + 2 * c.g;
      cacc[qd] = fmaf(d_a, s[0], cacc[qd]);
      cacc[qd] = fmaf(d_b, s[1], cacc[qd]);
    }
  }
  __device__ static float finish(float acc, float cacc) { return fmaf(-128.0f, cacc, acc); }

  // Batch 1 without the matrix core: lane kg owns block 2g+kg.
  __device__ static void init_dot(LaneCtx &c) { init(c); }
  __device__ static int x_offset(const LaneCtx &c) { return c.g * kXGroup + 8 * c.kg; }
  __device__ static int x_offset_dot(const LaneCtx &c) { return c.g * kXGroup + 32 * c.kg; }
  template <int MT>
  __device__ static void dot(const Raw &r, const half_t *xa, int xrow, const float *sx, int sxrow, const LaneCtx &c,
                             float (&acc)[MT], float (&cacc)[MT]) {
    constexpr uint32_t kByte = 0x00FF00FFu, kFlip = 0x80808080u;
    const uint32_t w[8] = {r.q0.x ^ kFlip, r.q0.y ^ kFlip, r.q0.z ^ kFlip, r.q0.w ^ kFlip,
                           r.q1.x ^ kFlip, r.q1.y ^ kFlip, r.q1.z ^ kFlip, r.q1.w ^ kFlip};
    float d = f16bits_to_f32(r.d & r.keep);
#pragma unroll
    for (int m = 0; m < MT; ++m) {
      const u32x4 *x4 = reinterpret_cast<const u32x4 *>(xa + m * xrow);
      u32x4 x0 = x4[0], x1 = x4[1], x2 = x4[2], x3 = x4[3];
      float p0 = dot_pairs(w[0], w[1], x0, kByte, 0.0f), p1 = dot_pairs(w[2], w[3], x1, kByte, 0.0f);
      p0 = dot_pairs(w[4], w[5], x2, kByte, p0);
      p1 = dot_pairs(w[6], w[7], x3, kByte, p1);
      acc[m] = fmaf(p0 + p1, d * kTwo24, acc[m]);
      cacc[m] = fmaf(d, sx[m * sxrow + 2 * c.g + c.kg], cacc[m]);
    }
  }
  __device__ static float finish_dot(float acc, float cacc) { return fmaf(-128.0f, cacc, acc); }
};

// ---- Q4_0 -------------------------------------------------------------------
// 18 B = [d][qs:16]: low nibble of qs[i] is element i, high nibble element i+16.
// Lane kg loads block 2g+kg; after the swap registers (0,1) hold bytes 8kg..+7
// of block 2g and (2,3) those of block 2g+1.
template <> struct Rows8<CUTHIP_Q4_0> {
  static constexpr int NSUB = 8, SUBK = 32;
  struct Raw { u32x4 q; uint32_t d, keep; };   // keep: as for Q8_0
  __device__ static void init(LaneCtx &c) { c.c0 = c.c1 = c.c2 = c.c3 = 0; }
  __device__ static void load(Raw &r, const uint8_t *row, uint32_t step, const LaneCtx &c, uint32_t K) {
    uint32_t nblk = K / 32, b = step * 8 + 2 * c.g + c.kg;
    const uint8_t *p = row + (size_t)min(b, nblk - 1) * 18;
    r.q = ld_u32x4(p + 2);
    r.d = ld_u16(p);
    r.keep = b < nblk ? 0xFFFFu : 0u;
  }
  template <int R>
  __device__ static void compute(const Raw &r, const half_t *xa, const float *const *sx, const LaneCtx &c,
                                 float (&acc)[R], float (&cacc)[(R + 3) / 4]) {
    u32x4 tq = r.q;
    asm volatile("" : "+v"(tq));   // the ring's value as a whole tuple up to here (see the Q6_K path)
    uint32_t w[4] = {tq.x, tq.y, tq.z, tq.w};
    swap_halves(w[0], w[2]); swap_halves(w[1], w[3]);
    uint32_t da = r.d & r.keep, db = da;
    swap_halves(da, db);
    float d_a = f16bits_to_f32(da), d_b = f16bits_to_f32(db);
    const half8_t *x8 = reinterpret_cast<const half8_t *>(xa);   // elements 64g + 8kg + {0, 16, 32, 48}
    auto lo = [&](uint32_t u0, uint32_t u1) { return as_half8(u0 & kNibLo, (u0 >> 8) & kNibLo, u1 & kNibLo, (u1 >> 8) & kNibLo); };
    auto hi = [&](uint32_t u0, uint32_t u1) { return as_half8(u0 & kNibHi, (u0 >> 8) & kNibHi, u1 & kNibHi, (u1 >> 8) & kNibHi); };
    f32x16 p0 = mfma(x8[0], lo(w[0], w[1]), zero16());   // block 2g, elements 0-15
    f32x16 p1 = mfma(x8[2], hi(w[0], w[1]), zero16());   // block 2g, elements 16-31 (x 2^-20)
    f32x16 q0 = mfma(x8[4], lo(w[2], w[3]), zero16());
    f32x16 q1 = mfma(x8[6], hi(w[2], w[3]), zero16());
    fma_acc<R>(acc, p0, d_a * kTwo24);
    fma_acc<R>(acc, p1, d_a * kTwo20);
    fma_acc<R>(acc, q0, d_b * kTwo24);
    fma_acc<R>(acc, q1, d_b * kTwo20);
#pragma unroll
    for (int qd = 0; qd < (R + 3) / 4; ++qd) {
      const float *s = sx[qd] + 2 * c.g;
      cacc[qd] = fmaf(d_a, s[0], cacc[qd]);
      cacc[qd] = fmaf(d_b, s[1], cacc[qd]);
    }
  }
  __device__ static float finish(float acc, float cacc) { return fmaf(-8.0f, cacc, acc); }

  // Batch 1 without the matrix core: lane kg owns block 2g+kg.
  __device__ static void init_dot(LaneCtx &c) { init(c); }
  __device__ static int x_offset(const LaneCtx &c) { return c.g * kXGroup + 8 * c.kg; }
  __device__ static int x_offset_dot(const LaneCtx &c) { return c.g * kXGroup + 32 * c.kg; }
  template <int MT>
  __device__ static void dot(const Raw &r, const half_t *xa, int xrow, const float *sx, int sxrow, const LaneCtx &c,
                             float (&acc)[MT], float (&cacc)[MT]) {
    float d = f16bits_to_f32(r.d & r.keep);
#pragma unroll
    for (int m = 0; m < MT; ++m) {
      const u32x4 *x4 = reinterpret_cast<const u32x4 *>(xa + m * xrow);
      u32x4 x0 = x4[0], x1 = x4[1], x2 = x4[2], x3 = x4[3];
      float pl = dot_pairs(r.q.x, r.q.y, x0, kNibLo, 0.0f), ph = dot_pairs(r.q.x, r.q.y, x2, kNibHi, 0.0f);
      pl = dot_pairs(r.q.z, r.q.w, x1, kNibLo, pl);
      ph = dot_pairs(r.q.z, r.q.w, x3, kNibHi, ph);
      acc[m] = fmaf(pl, d * kTwo24, acc[m]);
      acc[m] = fmaf(ph, d * kTwo20, acc[m]);
      cacc[m] = fmaf(d, sx[m * sxrow + 2 * c.g + c.kg], cacc[m]);
    }
  }
  __device__ static float finish_dot(float acc, float cacc) { return fmaf(-8.0f, cacc, acc); }
};

// ---- activations -> LDS ---------------------------------------------------------
// xs[m][(K/64) groups of 72 halfs], sxs[m][K/SUBK]; elements past K are zero.
// A thread handles XR groups of 8 elements of each of the MT batch rows per
// batch; the loads of a batch are issued together (XStage::load) and converted
// / stored later (XStage::store), so the caller can put the weight loads in
// between: memory returns in issue order, hence the wait for the activations
// leaves the weight loads in flight.
// PRO: the kernel instance also implements the activation prologues (RMSNorm, SiLU(gate) * up): extra
// registers for the norm weights and the sum of squares, so only batch-1 decode kernels are built with it.
// One group of 8 converted activations into LDS (group gi of batch row m) and, from the first lane of a sub-block, the
// sub-block's sum.  Every lane of the wave calls it (the sums meet through lane shuffles); ok = the group lies inside K,
// active = inside the padded row.
template <int SUBK>
__device__ __forceinline__ void stage_put(half_t (&h)[8], bool ok, bool active, uint32_t m, uint32_t gi, half_t *xs, float *sxs,
                                          int xrow, int sxrow) {
  float s = 0.0f;
#pragma unroll
  for (int i = 0; i < 8; ++i) {
    h[i] = ok ? h[i] : (half_t)0.0f;
    s += (float)h[i];
  }
  s += __shfl_xor(s, 1);
  if (SUBK == 32) s += __shfl_xor(s, 2);
  if (active) {
    half8_t o{h[0], h[2], h[1], h[3], h[4], h[6], h[5], h[7]};
    *reinterpret_cast<half8_t *>(xs + m * xrow + (gi >> 3) * kXGroup + (gi & 7) * 8) = o;
    constexpr uint32_t per = SUBK / 8;
    if ((gi & (per - 1)) == 0) sxs[m * sxrow + gi / per] = s;
  }
}

template <int SUBK, int THREADS, int MT, int XR, bool PRO> struct XStage {
  u32x4 ra[MT * XR], rb[MT * XR];
  u32x4 wa[PRO ? MT * XR : 1], wb[PRO ? MT * XR : 1];   // norm weights of the group (fp32 x 8)
  float ssq[MT];                                        // this thread's share of sum(x^2) per batch row
  __device__ void init() {
#pragma unroll
    for (int m = 0; m < MT; ++m) ssq[m] = 0.0f;
  }
  // base: first group (of a row) of this batch; gpr: groups per padded row
  __device__ void load(const GemvParams &p, uint32_t base, int tid, uint32_t gpr) {
    const uint32_t esz = p.a_f16 ? 2u : 4u;
#pragma unroll
    for (int u = 0; u < MT * XR; ++u) {
      const uint32_t m = u / XR, gi = base + (u % XR) * THREADS + tid, k = gi * 8;
      // lanes without a group issue nothing (the unused slots of a batch cost no traffic); store() masks them
      if (m < p.M && k < p.K) {
        const uint8_t *src = reinterpret_cast<const uint8_t *>(p.A) + ((size_t)m * p.strideA + k) * esz;
        ra[u] = ld_u32x4(src);
        // one load site per register array (a branch per source would let the compiler merge the stores of different
        // arrays into one with a run-time slot, which moves the arrays to scratch memory)
        const bool swiglu = PRO && p.pro == CUTHIP_PRO_SWIGLU;
        // second half of the group: the "up" half of [gate | up] (fp16 only), or elements 4..7 of an fp32 group
        if (swiglu || !p.a_f16) rb[u] = ld_u32x4(swiglu ? src + (size_t)p.K * 2 : src + 16);
        if (PRO && p.pro == CUTHIP_PRO_RMSNORM) {
          const uint8_t *w = reinterpret_cast<const uint8_t *>(p.norm_w + k);
          wa[u] = ld_u32x4(w);
          wb[u] = ld_u32x4(w + 16);
        }
      }
    }
  }
  __device__ void store(const GemvParams &p, uint32_t base, int tid, uint32_t gpr, half_t *xs, float *sxs, int xrow,
                        int sxrow) {
#pragma unroll
    for (int u = 0; u < MT * XR; ++u) {
      const uint32_t m = u / XR, gi = base + (u % XR) * THREADS + tid, k = gi * 8;
      const bool active = m < p.M && gi < gpr, ok = active && k < p.K;
      half_t h[8];
      if (PRO && p.pro == CUTHIP_PRO_SWIGLU) {
        half8_t g = __builtin_bit_cast(half8_t, ra[u]), up = __builtin_bit_cast(half8_t, rb[u]);
#pragma unroll
        for (int i = 0; i < 8; ++i) {
          float gf = (float)g[i];
          h[i] = (half_t)(gf / (1.0f + __expf(-gf)) * (float)up[i]);
        }
      } else {
        float x[8];
        if (p.a_f16) {
          half8_t v = __builtin_bit_cast(half8_t, ra[u]);
#pragma unroll
          for (int i = 0; i < 8; ++i) x[i] = (float)v[i];
        } else {
          f32x4 lo = __builtin_bit_cast(f32x4, ra[u]), hi = __builtin_bit_cast(f32x4, rb[u]);
          x[0] = lo.x; x[1] = lo.y; x[2] = lo.z; x[3] = lo.w; x[4] = hi.x; x[5] = hi.y; x[6] = hi.z; x[7] = hi.w;
        }
        if (PRO && p.pro == CUTHIP_PRO_RMSNORM) {
          f32x4 w0 = __builtin_bit_cast(f32x4, wa[u]), w1 = __builtin_bit_cast(f32x4, wb[u]);
          const float w[8] = {w0.x, w0.y, w0.z, w0.w, w1.x, w1.y, w1.z, w1.w};
          float q = 0.0f;
#pragma unroll
          for (int i = 0; i < 8; ++i) {
            q = fmaf(x[i], x[i], q);
            x[i] *= w[i];
          }
          if (ok) ssq[m] += q;
        }
#pragma unroll
        for (int i = 0; i < 8; ++i) h[i] = (half_t)x[i];
      }
      stage_put<SUBK>(h, ok, active, m, gi, xs, sxs, xrow, sxrow);
    }
  }
};

// fp16 activations without a prologue (every decode matmul).  Same groups of 8 per thread as the general path (a wave's
// load is 1 KB contiguous; whole 32-element sub-blocks per thread were tried and cost 6 % at batch 1: a load instruction
// then touches 64 lines instead of 8), but no conversion: the sum of a group is four v_dot2 against (1, 1), the sums of
// the 2 or 4 groups of a sub-block meet through DPP quad permutes instead of LDS shuffles, the reordering is four byte
// permutes.  A wave issues one instruction per four cycles whatever its kind, so a shorter start-up is time won before
// the first product.
template <int SUBK, int THREADS, int MT, int XR> struct XStageF16 {
  u32x4 r[MT * XR];
  __device__ void load(const GemvParams &p, uint32_t base, int tid) {
#pragma unroll
    for (int u = 0; u < MT * XR; ++u) {
      const uint32_t m = u / XR, gi = base + (u % XR) * THREADS + tid, k = gi * 8;
      if (m < p.M && k < p.K) r[u] = ld_u32x4(reinterpret_cast<const uint8_t *>(p.A) + ((size_t)m * p.strideA + k) * 2u);
    }
  }
  static __device__ __forceinline__ float quad_xor_add(float s, bool two) {
    // every lane of the quad executes this (callers keep it outside divergent code)
    s += __builtin_bit_cast(float, __builtin_amdgcn_update_dpp(0, __builtin_bit_cast(int, s), 0xB1, 0xF, 0xF, true));   // lanes (1 0 3 2)
    if (two) s += __builtin_bit_cast(float, __builtin_amdgcn_update_dpp(0, __builtin_bit_cast(int, s), 0x4E, 0xF, 0xF, true));   // lanes (2 3 0 1)
    return s;
  }
  __device__ void store(const GemvParams &p, uint32_t base, int tid, uint32_t gpr, half_t *xs, float *sxs, int xrow, int sxrow) {
    const half2_t one{(half_t)1.0f, (half_t)1.0f};
#pragma unroll
    for (int u = 0; u < MT * XR; ++u) {
      const uint32_t m = u / XR, gi = base + (u % XR) * THREADS + tid, k = gi * 8;
      const bool active = m < p.M && gi < gpr, ok = active && k < p.K;   // groups between K and the padded length hold zeros
      const uint32_t e0 = ok ? r[u].x : 0u, e1 = ok ? r[u].y : 0u, e2 = ok ? r[u].z : 0u, e3 = ok ? r[u].w : 0u;
      float s = __builtin_amdgcn_fdot2(__builtin_bit_cast(half2_t, e0), one, 0.0f, false);
      s = __builtin_amdgcn_fdot2(__builtin_bit_cast(half2_t, e1), one, s, false);
      s = __builtin_amdgcn_fdot2(__builtin_bit_cast(half2_t, e2), one, s, false);
      s = __builtin_amdgcn_fdot2(__builtin_bit_cast(half2_t, e3), one, s, false);
      s = quad_xor_add(s, SUBK == 32);
      if (active) {
        // halves (0 1)(2 3)(4 5)(6 7) -> (0 2)(1 3)(4 6)(5 7)
        *reinterpret_cast<u32x4 *>(xs + m * xrow + (gi >> 3) * kXGroup + (gi & 7) * 8) =
            u32x4{__builtin_amdgcn_perm(e1, e0, 0x05040100u), __builtin_amdgcn_perm(e1, e0, 0x07060302u),
                  __builtin_amdgcn_perm(e3, e2, 0x05040100u), __builtin_amdgcn_perm(e3, e2, 0x07060302u)};
        constexpr uint32_t per = SUBK / 8;
        if ((gi & (per - 1)) == 0) sxs[m * sxrow + gi / per] = s;
      }
    }
  }
};

// Activations = the output of a split-context decode attention that has not been merged yet (CUTHIP_PRO_ATTN_MERGE):
// A holds, per query head, mrg_nsplit records [max, sum, o[mrg_head_dim]] (fp32, o un-normalised), K = heads x
// mrg_head_dim.  A thread folds the records of its group of 8 dimensions: weights exp(max_s - max), the sum of the
// weighted sums as the divisor.  All loads of a group are requested together (one memory round trip); every workgroup
// reads all records, which pays while the records are few (at most kMergeMax per head).
constexpr int kMergeMax = 8;
typedef uint32_t u32x4_a8 __attribute__((ext_vector_type(4), aligned(8)));
typedef float f32x2_a8 __attribute__((ext_vector_type(2), aligned(8)));
template <int SUBK, int THREADS> struct XStageMerge {
  u32x4 oa[kMergeMax], ob[kMergeMax];
  f32x2_a8 ml[kMergeMax];
  __device__ void load(const GemvParams &p, uint32_t gi) {
    const uint32_t k = gi * 8;
    if (k >= p.K) return;
    const uint32_t hd = p.mrg_head_dim, head = k / hd, d0 = k - head * hd, rec = 2 + hd;
    const float *base = reinterpret_cast<const float *>(p.A) + (size_t)head * p.mrg_nsplit * rec;
#pragma unroll
    for (int s = 0; s < kMergeMax; ++s) {
      if ((uint32_t)s < p.mrg_nsplit) {
        const float *r = base + (size_t)s * rec;
        ml[s] = *reinterpret_cast<const f32x2_a8 *>(r);
        oa[s] = *reinterpret_cast<const u32x4_a8 *>(r + 2 + d0);
        ob[s] = *reinterpret_cast<const u32x4_a8 *>(r + 2 + d0 + 4);
      }
    }
  }
  __device__ void store(const GemvParams &p, uint32_t gi, uint32_t gpr, half_t *xs, float *sxs, int xrow, int sxrow) {
    const bool active = gi < gpr, ok = active && gi * 8 < p.K;
    float x[8] = {0.0f, 0.0f, 0.0f, 0.0f, 0.0f, 0.0f, 0.0f, 0.0f};
    if (ok) {
      float M = -INFINITY;
#pragma unroll
      for (int s = 0; s < kMergeMax; ++s)
        if ((uint32_t)s < p.mrg_nsplit) M = fmaxf(M, ml[s].x);
      float L = 0.0f;
#pragma unroll
      for (int s = 0; s < kMergeMax; ++s) {
        if ((uint32_t)s < p.mrg_nsplit) {
          const float w = ml[s].x == -INFINITY ? 0.0f : __expf(ml[s].x - M);   // an empty split weighs nothing
          L = fmaf(ml[s].y, w, L);
          const f32x4 a = __builtin_bit_cast(f32x4, oa[s]), b = __builtin_bit_cast(f32x4, ob[s]);
          x[0] = fmaf(a.x, w, x[0]); x[1] = fmaf(a.y, w, x[1]); x[2] = fmaf(a.z, w, x[2]); x[3] = fmaf(a.w, w, x[3]);
          x[4] = fmaf(b.x, w, x[4]); x[5] = fmaf(b.y, w, x[5]); x[6] = fmaf(b.z, w, x[6]); x[7] = fmaf(b.w, w, x[7]);
        }
      }
      const float inv = L > 0.0f ? 1.0f / L : 0.0f;   // an empty sequence gives zeros
#pragma unroll
      for (int i = 0; i < 8; ++i) x[i] *= inv;
    }
    half_t h[8];
#pragma unroll
    for (int i = 0; i < 8; ++i) h[i] = (half_t)x[i];
    stage_put<SUBK>(h, ok, active, 0u, gi, xs, sxs, xrow, sxrow);
  }
};

// bits of GemvParams::hot, the flag word among the leading kernel arguments of the 8-row kernels (see gemv_rows8_kernel)
constexpr uint32_t kHotAF16 = 1u, kHotCF16 = 2u, kHotEpiShift = 2, kHotRopeShift = 5, kHotNextNorm = 1u << 7, kHotSumsq = 1u << 8;

// ---- the kernel -----------------------------------------------------------------
// MT: batch rows held (1, 2 or 4); RWG x KW waves per workgroup; D ring depth.
// MT == 1 takes the lane-local dot-product path (v_dot2_f32_f16 on the same
// subnormal operands: a quarter of the issue cycles of the matrix-core path,
// whose 32 A-rows would be 7/8 padding); MT > 1 goes through the matrix core.
// PRE: the launch has epilogue operands to request at its start (the D of a binary epilogue, the weight of a carried
// norm, the tables of the RoPE epilogue).  Without them (PRE = false: plain products, the consumer side of a carried
// norm, the row-pair and arg-max epilogues) nothing of the argument block beyond the leading kernel arguments is read
// before the weight ring is requested.
// PRO: 0 = activations as they are; 1 = the RMSNorm / SiLU(gate) * up prologues; 2 = the attention-merge prologue
template <int FMT, int MT, int RWG, int KW, int D, int XWANT, int PRO, bool PRE = true>
__device__ __forceinline__ void rows8_body(const GemvParams &p, const uint32_t bid) {
  using S = Rows8<FMT>;
  constexpr bool DOT = MT <= rows8_dot_max<FMT>();
  constexpr int WAVES = RWG * KW, THREADS = 64 * WAVES;
  // accumulators: dot path one per batch row; matrix-core path rows 4m + g of C, RQ quads of four pieces
  constexpr int R = DOT ? MT : 2 * MT, RQ = DOT ? MT : R / 4;
  extern __shared__ __attribute__((aligned(16))) uint8_t lds[];

  const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
  const int rg = wave / KW, kw = wave - rg * KW;
  LaneCtx c;
  c.kg = lane >> 5;
  const int j = lane & 31;
  c.g = j & 3;
  const int r8 = j >> 2;
  if (DOT) S::init_dot(c);
  else S::init(c);

  const uint32_t kpad = p.nsteps * 256u;
  const int xrow = (int)(p.nsteps * kXStep), sxrow = (int)(p.nsteps * S::NSUB);
  half_t *xs = reinterpret_cast<half_t *>(lds);
  float *sxs = reinterpret_cast<float *>(lds + (size_t)MT * xrow * 2);
  float *nrm = sxs + MT * sxrow;   // [MT][WAVES] per-wave shares of sum(x^2) (RMSNorm prologue)

  const uint32_t n0 = (bid * RWG + rg) * 8u;
  const uint32_t n = min(n0 + (uint32_t)r8, p.N - 1);
  const uint8_t *row = p.W + (size_t)n * p.row_bytes;
  const uint32_t sb = (uint32_t)(((uint64_t)p.nsteps * kw) / KW);
  const uint32_t se = (uint32_t)(((uint64_t)p.nsteps * (kw + 1)) / KW);
  const uint32_t cnt = se - sb, last = min(se > sb ? se - 1 : sb, p.nsteps - 1);

  // activation loads first (they must not queue behind the weight loads), then the weight ring, then the
  // conversion of the activations; batches beyond the first (large M * K only) are staged behind the ring
  // groups of 8 activations per thread and batch row in the first batch: sized so that typical shapes need no
  // second batch (every further batch is one more memory round trip before the first step can start)
  constexpr int XCAP = 8 / MT, XR = XWANT < XCAP ? XWANT : XCAP;
  const uint32_t gpr = kpad / 8;   // 8-element groups per padded row
  // fp16 activations and no prologue: the short staging; otherwise the general one
  const bool fastx = !PRO && p.a_f16;
  XStage<S::SUBK, THREADS, MT, XR, PRO == 1> xst;
  XStageF16<S::SUBK, THREADS, MT, XR> xsf;
  XStageMerge<S::SUBK, THREADS> xsm;
  xst.init();
  if constexpr (PRO == 2) xsm.load(p, (uint32_t)tid);
  else if (fastx) xsf.load(p, 0, tid);
  else xst.load(p, 0, tid, gpr);
  // Batch 1: the epilogue's operands for this thread's output row (D of a binary epilogue, the weight of a carried
  // norm) are requested now, right behind the activations, so that the end of the workgroup does not wait for them
  // (behind the weight ring they cost the launch 0.2 us more).
  // Valid because each output element is read (as D) and written (as C) by the same thread only.
  // (D as raw bits: a conversion right behind the load is a use, and the wait for it would take the ring with it)
  uint32_t pre_d_bits = 0u;
  float pre_g = 0.0f, pre_cs = 0.0f, pre_sn = 0.0f;
  uint32_t rope_pos = 0u;
  const uint32_t prow = KW == 1 ? n0 + (uint32_t)r8 : (bid * RWG + (uint32_t)tid / 8) * 8u + ((uint32_t)tid & 7u);
  if constexpr (PRE) {
    const bool pre_ok = MT == 1 && (KW == 1 || tid < RWG * 8) && prow < p.N;
    if (pre_ok) {
      if (p.epi.kind == CUTHIP_EPI_BINARY)
        pre_d_bits = p.c_f16 ? (uint32_t)reinterpret_cast<const uint16_t *>(p.epi.D)[prow] : reinterpret_cast<const uint32_t *>(p.epi.D)[prow];
      if (p.hot & kHotNextNorm) pre_g = p.next_norm_w[prow];
    }
    rope_pos = p.rope.mode ? (p.rope.pos_read ? p.rope.pos : p.rope.params[0]) : 0u;
    if (pre_ok && p.rope.mode == 1 && rope_pos < p.rope.max_pos) {
      const size_t ti = (size_t)rope_pos * (p.rope.head_dim / 2) + ((prow % p.rope.head_dim) >> 1);
      pre_cs = p.rope.cosT[ti];
      pre_sn = p.rope.sinT[ti];
    }
  }
  // carried RMSNorm, consumer side: the K / 8 partial sums of squares travel like the activations: requested ahead of
  // the weight ring, one share per thread, folded per wave and across the waves through LDS at the staging barrier
  // (the order of the additions depends on the launch shape only)
  constexpr int CP = 4;
  const uint32_t nparts = (MT == 1 && (p.hot & kHotSumsq)) ? (p.K + 7) / 8 : 0u;   // batch 1 only: the LDS of larger batches has no room for it
  float cpart[CP];
#pragma unroll
  for (int jj = 0; jj < CP; ++jj) {
    const uint32_t i = (uint32_t)tid + (uint32_t)jj * THREADS;
    cpart[jj] = i < nparts ? p.sumsq_parts[i] : 0.0f;
  }
  typename S::Raw buf[D];
#pragma unroll
  for (int i = 0; i < D; ++i) {
    S::load(buf[i], row, min(sb + i, last), c, p.K);
    __builtin_amdgcn_sched_barrier(0);   // keep issue order = ring order, so that step i waits for its own loads only
  }
  if constexpr (PRO == 2) {
    xsm.store(p, (uint32_t)tid, gpr, xs, sxs, xrow, sxrow);
    for (uint32_t base = THREADS; base < gpr; base += THREADS) {
      xsm.load(p, base + (uint32_t)tid);
      xsm.store(p, base + (uint32_t)tid, gpr, xs, sxs, xrow, sxrow);
    }
  } else if (fastx) {
    xsf.store(p, 0, tid, gpr, xs, sxs, xrow, sxrow);
    for (uint32_t base = THREADS * XR; base < gpr; base += THREADS * XR) {
      xsf.load(p, base, tid);
      xsf.store(p, base, tid, gpr, xs, sxs, xrow, sxrow);
    }
  } else {
    xst.store(p, 0, tid, gpr, xs, sxs, xrow, sxrow);
    for (uint32_t base = THREADS * XR; base < gpr; base += THREADS * XR) {
      xst.load(p, base, tid, gpr);
      xst.store(p, base, tid, gpr, xs, sxs, xrow, sxrow);
    }
  }
  if (!PRO && nparts) {
    float t = (cpart[0] + cpart[1]) + (cpart[2] + cpart[3]);
    for (uint32_t i = (uint32_t)tid + CP * THREADS; i < nparts; i += THREADS) t += p.sumsq_parts[i];
    t = wave_sum_all(t);
    if (lane == 0) nrm[wave] = t;
  }
  if (PRO == 1 && p.pro == CUTHIP_PRO_RMSNORM) {
#pragma unroll
    for (int m = 0; m < MT; ++m) {
      const float t = wave_sum_all(xst.ssq[m]);
      if (lane == 0) nrm[m * WAVES + wave] = t;
    }
  }
  __syncthreads();
  // RMSNorm prologue: the scalar rsqrt(mean(x^2) + eps) multiplies the finished dot products
  float xscale[MT];
#pragma unroll
  for (int m = 0; m < MT; ++m) {
    xscale[m] = 1.0f;
    if (PRO == 1 && p.pro == CUTHIP_PRO_RMSNORM) {
      float t = 0.0f;
      for (int w = 0; w < WAVES; ++w) t += nrm[m * WAVES + w];
      xscale[m] = 1.0f / sqrtf(t / (float)p.K + p.eps);
    }
  }
  // RMSNorm carried over from the producer of the activations: one scalar for the whole (batch-1) product
  float carry_scale = 1.0f;
  if (!PRO && nparts) {
    float t = 0.0f;
    for (int w = 0; w < WAVES; ++w) t += nrm[w];
    carry_scale = 1.0f / sqrtf(t / (float)p.K + p.eps);
  }

  // Matrix-core path: A-row j of this lane is batch row j>>2 (clamped), piece j&3, and accumulator quad q
  // holds batch row 2q + kg.  Dot path: the lane's own slice of every batch row, accumulator q = batch row q.
  const half_t *xbase = DOT ? xs + S::x_offset_dot(c) : xs + min(j >> 2, (int)p.M - 1) * xrow + S::x_offset(c);
  const float *sxq[RQ];
#pragma unroll
  for (int q = 0; q < RQ; ++q) sxq[q] = sxs + (DOT ? 0 : min(2 * q + c.kg, (int)p.M - 1) * sxrow);

  float acc[R], cacc[RQ];
#pragma unroll
  for (int r = 0; r < R; ++r) acc[r] = 0.0f;
#pragma unroll
  for (int q = 0; q < RQ; ++q) cacc[q] = 0.0f;

  auto do_step = [&](const typename S::Raw &raw, uint32_t step) {
    if constexpr (DOT) {
      S::template dot<MT>(raw, xbase + step * kXStep, xrow, sxq[0] + step * S::NSUB, sxrow, c, acc, cacc);
    } else {
      const float *sx[RQ];
#pragma unroll
      for (int q = 0; q < RQ; ++q) sx[q] = sxq[q] + step * S::NSUB;
      S::template compute<R>(raw, xbase + step * kXStep, sx, c, acc, cacc);
    }
    // keep the scale FMAs of this step here: without the pin they are sunk behind the last step and spill
#pragma unroll
    for (int r = 0; r < R; ++r) asm volatile("" : "+v"(acc[r]));
#pragma unroll
    for (int q = 0; q < RQ; ++q) asm volatile("" : "+v"(cacc[q]));
  };

  uint32_t i0 = 0;
  for (; i0 + 2 * D <= cnt; i0 += D) {   // steady state: every refill is in range, no branches around loads
#pragma unroll
    for (int u = 0; u < D; ++u) {
      do_step(buf[u], sb + i0 + u);
      S::load(buf[u], row, sb + i0 + u + D, c, p.K);
      __builtin_amdgcn_sched_barrier(0);
    }
  }
#pragma unroll
  for (int u = 0; u < 2 * D; ++u) {      // tail: at most 2D - 1 steps
    uint32_t i = i0 + u;
    if (i < cnt) {
      do_step(buf[u % D], sb + i);
      if (i + D < cnt) S::load(buf[u % D], row, sb + i + D, c, p.K);
    }
  }

  // One value per (weight row, batch row): dot path = sum over the 8 lanes of the row; matrix-core path =
  // the valid accumulator (row 4m + g of C) summed over the four pieces.  Then fold the K ranges.
  const float pre_d = p.c_f16 ? (float)__builtin_bit_cast(half_t, (uint16_t)pre_d_bits) : __builtin_bit_cast(float, pre_d_bits);
  float out[RQ];
  bool writer;
  if constexpr (DOT) {
#pragma unroll
    for (int q = 0; q < RQ; ++q) {
      float v = S::finish_dot(acc[q], cacc[q]);
      v = add_xor32(add_xor2(add_xor1(v)));
      out[q] = (PRO == 1 ? v * xscale[q] : v) * carry_scale;   // linear in the partial sums: applied before the K ranges are folded
    }
    writer = c.g == 0 && c.kg == 0;
  } else {
#pragma unroll
    for (int q = 0; q < RQ; ++q) {
      float v = c.g == 0 ? acc[4 * q] : c.g == 1 ? acc[4 * q + 1] : c.g == 2 ? acc[4 * q + 2] : acc[4 * q + 3];
      v = S::finish(v, cacc[q]);
      v = add_xor2(add_xor1(v));
      out[q] = v * carry_scale;   // batch row 2q + kg
    }
    writer = c.g == 0;
  }
  float carry_sq = 0.0f;
  float am_v = -INFINITY;          // this lane's candidate for the arg-max of the wave's 8 rows (writer lanes only)
  uint32_t am_i = 0xFFFFFFFFu;
  // SwiGLU over row pairs: weight rows 2i / 2i+1 are gate_i / up_i, C[m, i] = silu(gate) * up.  The partner row
  // sits four lanes up (same piece, same K half); in the folded path it is the next thread.
  const bool swiglu = p.epi.kind == CUTHIP_EPI_SWIGLU_PAIRS;
  if (KW == 1) {
    if (MT == 1 && p.rope.mode) {
      float partner = __shfl_xor(out[0], 4);   // row r8 ^ 1 of this wave
      if (writer && n0 + r8 < p.N) rope_store(p.rope, n0 + r8, out[0], partner, pre_cs, pre_sn, rope_pos);
    } else if (swiglu) {
#pragma unroll
      for (int q = 0; q < RQ; ++q) {
        float up = __shfl_down(out[q], 4);
        int m = DOT ? q : 2 * q + c.kg;
        if (writer && (r8 & 1) == 0 && n0 + r8 + 1 < p.N && m < (int)p.M)
          store_plain(p.C, p.c_f16, (size_t)m * p.strideC + (n0 + r8) / 2, apply_unary(CUTHIP_UNARY_SILU, out[q]) * up);
      }
    } else if (writer && n0 + r8 < p.N) {
#pragma unroll
      for (int q = 0; q < RQ; ++q) {
        int m = DOT ? q : 2 * q + c.kg;
        if (m < (int)p.M) {
          if (MT == 1 && p.epi.kind == CUTHIP_EPI_BINARY) {
            float v = apply_binary(p.epi.op, out[q], pre_d);
            store_plain(p.C, p.c_f16, n0 + r8, v);
            if (p.next_sumsq_parts) {
              p.next_x16[n0 + r8] = (half_t)(v * pre_g);
              carry_sq = v * v;
            }
          } else {
            float v = store_out_value(p.C, p.epi, p.c_f16, (size_t)m * p.strideC + n0 + r8, out[q]);
            if (p.next_sumsq_parts && m == 0) {
              p.next_x16[n0 + r8] = (half_t)(v * p.next_norm_w[n0 + r8]);
              carry_sq = v * v;
            }
            if (MT == 1) {
              am_v = p.c_f16 ? (float)(half_t)v : v;   // the value as C holds it
              am_i = n0 + r8;
            }
          }
        }
      }
    }
    if (MT == 1 && p.argmax_parts) {   // (uniform) largest of the wave's rows, the first one on a tie
#pragma unroll
      for (int o = 32; o > 0; o >>= 1) {
        const float ov = __shfl_xor(am_v, o);
        const uint32_t oi = __shfl_xor(am_i, o);
        if (ov > am_v || (ov == am_v && oi < am_i)) {
          am_v = ov;
          am_i = oi;
        }
      }
      if (lane == 0 && n0 < p.N) p.argmax_parts[n0 / 8] = ArgmaxPart{am_v, am_i};
    }
  } else {
    __syncthreads();   // all waves are done with the staged activations
    float *red = reinterpret_cast<float *>(lds);   // [RWG][KW][MT][8]
    if (writer) {
#pragma unroll
      for (int q = 0; q < RQ; ++q) {
        int m = DOT ? q : 2 * q + c.kg;
        if (m < MT) red[((rg * KW + kw) * MT + m) * 8 + r8] = out[q];
      }
    }
    __syncthreads();
    if (tid < RWG * MT * 8) {
      int rgi = tid / (MT * 8), m = (tid / 8) % MT, rr = tid & 7;
      uint32_t nn = (bid * RWG + rgi) * 8u + rr;
      float v = 0.0f;
#pragma unroll
      for (int k = 0; k < KW; ++k) v += red[((rgi * KW + k) * MT + m) * 8 + rr];
      if (MT == 1 && p.rope.mode) {
        float partner = __shfl_xor(v, 1);
        if (nn < p.N) rope_store(p.rope, nn, v, partner, pre_cs, pre_sn, rope_pos);
      } else if (swiglu) {
        float up = __shfl_down(v, 1);
        if (m < (int)p.M && (rr & 1) == 0 && nn + 1 < p.N)
          store_plain(p.C, p.c_f16, (size_t)m * p.strideC + nn / 2, apply_unary(CUTHIP_UNARY_SILU, v) * up);
      } else if (m < (int)p.M && nn < p.N) {
        if (MT == 1 && p.epi.kind == CUTHIP_EPI_BINARY) {   // nn == prow here
          v = apply_binary(p.epi.op, v, pre_d);
          store_plain(p.C, p.c_f16, nn, v);
          if (p.next_sumsq_parts) {
            p.next_x16[nn] = (half_t)(v * pre_g);
            carry_sq = v * v;
          }
        } else {
          v = store_out_value(p.C, p.epi, p.c_f16, (size_t)m * p.strideC + nn, v);
          if (p.next_sumsq_parts && m == 0) {
            p.next_x16[nn] = (half_t)(v * p.next_norm_w[nn]);
            carry_sq = v * v;
          }
        }
      }
    }
  }
  // producer side of the carried RMSNorm: sum(C^2) of each group of 8 rows to its own slot
  if (p.next_sumsq_parts) {
    if (KW == 1) {   // one row group per wave, its writers are 8 of the lanes
      carry_sq = wave_sum_all(carry_sq);
      if (lane == 0 && n0 < p.N) p.next_sumsq_parts[n0 / 8] = carry_sq;
    } else {         // folded epilogue: thread 8 g + r of the workgroup holds row r of its g-th row group
      carry_sq = add_xor4(add_xor2(add_xor1(carry_sq)));
      const uint32_t grp = bid * RWG + (uint32_t)tid / 8;
      if (tid < RWG * 8 && (tid & 7) == 0 && grp * 8 < p.N) p.next_sumsq_parts[grp] = carry_sq;
    }
  }
}

// What a wave needs for its first loads travels as leading scalar kernel arguments: with kernel-argument preloading
// (-mllvm -amdgpu-kernarg-preload-count, gfx940 and later) they arrive in SGPRs with the wave, and the activation loads
// go out without a scalar-memory round trip in front of them (a cold read of the argument block costs about 0.3 us).
// The flag word says which of the optional pointers of GemvParams are set, so that a launch without them never reads them.
inline uint32_t rows8_hot_flags(const GemvParams &p) {
  return (p.a_f16 ? kHotAF16 : 0u) | (p.c_f16 ? kHotCF16 : 0u) | ((uint32_t)p.epi.kind << kHotEpiShift) |
         ((uint32_t)p.rope.mode << kHotRopeShift) | (p.next_norm_w ? kHotNextNorm : 0u) | (p.sumsq_parts ? kHotSumsq : 0u);
}
// Copies the preloaded arguments over the fields of the by-value block, so that the body reads registers for them.
__device__ __forceinline__ void rows8_take_hot(GemvParams &p, const void *A, uint32_t K, uint32_t strideA, uint32_t nsteps,
                                               uint32_t flags) {
  p.A = A; p.K = K; p.strideA = strideA; p.nsteps = nsteps;
  p.a_f16 = (int)(flags & kHotAF16); p.c_f16 = (int)((flags & kHotCF16) != 0);
  p.epi.kind = (int)((flags >> kHotEpiShift) & 7u);
  p.rope.mode = (int)((flags >> kHotRopeShift) & 3u);
  p.hot = flags;   // which of the optional pointers are set: tested in place of the pointers, which are then only read where set
}
template <int FMT, int MT, int RWG, int KW, int D, int XWANT, int PRO, bool PRE>
__global__ void __launch_bounds__(64 * RWG * KW, 2)
gemv_rows8_kernel(const uint8_t *W, const void *A, const float *sumsq_parts, uint32_t M, uint32_t K, uint32_t N, uint32_t strideA,
                  uint32_t nsteps, uint32_t row_bytes, uint32_t flags, GemvParams p) {
  p.W = W; p.M = M; p.N = N; p.row_bytes = row_bytes; p.sumsq_parts = sumsq_parts;
  p.rope.pos_read = 0;
  rows8_take_hot(p, A, K, strideA, nsteps, flags);
  rows8_body<FMT, MT, RWG, KW, D, XWANT, PRO, PRE>(p, blockIdx.x);
}

// K split across workgroups for long rows and few of them (the down projection at batch 2-8): workgroup
// (part, block) multiplies the K range `part` of 8 row groups and writes fp32 partial products
// partial[part][m][n]; a second kernel sums the parts and applies the epilogue.  Eight row groups per workgroup
// keep the staging of the activations (all of a K range per workgroup) an eighth of what one row group per
// workgroup would read, and the K ranges supply the workgroups that N / 64 alone would not.
template <int FMT, int MT, int D>
__global__ void __launch_bounds__(64 * 8, 2) gemv_rows8_ksplit_kernel(GemvParams p, uint32_t nblocks, uint32_t part_steps,
                                                                       float *partial) {
  const uint32_t part = blockIdx.x / nblocks, bid = blockIdx.x - part * nblocks;
  const uint32_t k_lo = part * part_steps * 256u, k_hi = min(p.K, k_lo + part_steps * 256u);
  if (k_lo >= p.K) return;   // the host launches no empty part (k_hi - k_lo would wrap around)
  p.A = reinterpret_cast<const uint8_t *>(p.A) + (size_t)k_lo * (p.a_f16 ? 2 : 4);
  p.W += (size_t)(k_lo / Fmt<FMT>::elems) * Fmt<FMT>::bytes;
  p.K = k_hi - k_lo;
  p.nsteps = (p.K + 255) / 256;
  p.C = partial + (size_t)part * p.M * p.N;
  p.strideC = p.N;
  p.c_f16 = 0;
  p.epi = Epilogue{CUTHIP_EPI_NONE, 0, nullptr};
  rows8_body<FMT, MT, 8, 1, D, 1, false>(p, bid);
}

// Two weight tensors (formats FA, FB) against the same batch-1 activations in one launch: workgroups
// [0, blocks_a) take the rows of the first, the rest the rows of the second.  Saves a launch and a kernel
// start where a small projection (w_v) sits next to a larger one (w_q | w_k) of another format.
template <int FA, int FB, int RWG, int KW, int D, int XWANT>
__global__ void __launch_bounds__(64 * RWG * KW, 2)
gemv_rows8_pair_kernel(const void *A, const uint32_t *rope_params, uint32_t K, uint32_t strideA, uint32_t nsteps, uint32_t flags_a,
                       uint32_t flags_b, uint32_t blocks_a, GemvParams pa, GemvParams pb) {
  // The position of the RoPE epilogue is requested first of all (its pointer is among the preloaded arguments): the
  // table loads of the prologue depend on it, and the weight ring is requested behind them.  Without RoPE the host
  // passes the (aligned) start of the activations instead, so that the load needs no branch.
  const uint32_t pos = rope_params[0];
  pa.M = pb.M = 1u;   // the pair launch is a batch-1 launch
  pa.rope.pos = pb.rope.pos = pos;
  pa.rope.pos_read = pb.rope.pos_read = 1;
  if (blockIdx.x < blocks_a) {
    rows8_take_hot(pa, A, K, strideA, nsteps, flags_a);
    rows8_body<FA, 1, RWG, KW, D, XWANT, false>(pa, blockIdx.x);
  } else {
    rows8_take_hot(pb, A, K, strideA, nsteps, flags_b);
    rows8_body<FB, 1, RWG, KW, D, XWANT, false>(pb, blockIdx.x - blocks_a);
  }
}

inline size_t rows8_lds_bytes_rt(int fmt, uint32_t nsteps, int mt);
template <int FMT> static size_t rows8_lds_bytes(const GemvParams &p, int mt) {
  static_assert(Rows8<FMT>::NSUB == (FMT == CUTHIP_Q6_K ? 16 : 8), "rows8_lds_bytes_rt assumes these sub-block counts");
  return rows8_lds_bytes_rt(FMT, p.nsteps, mt);
}

template <int FMT, int MT, int RWG, int KW, int D, int XWANT, int PRO = 0, bool PRE = false>
static int launch_rows8(const GemvParams &p, hipStream_t stream) {
  if constexpr (MT == 1 && PRO == 0) {
    if (p.pro == CUTHIP_PRO_ATTN_MERGE) return launch_rows8<FMT, MT, RWG, KW, D, XWANT, 2, true>(p, stream);
    if (p.pro) return launch_rows8<FMT, MT, RWG, KW, D, XWANT, 1, true>(p, stream);
    if constexpr (!PRE) {   // epilogue operands to request at the start: the instance that does
      if (p.epi.kind == CUTHIP_EPI_BINARY || p.next_norm_w || p.rope.mode) return launch_rows8<FMT, MT, RWG, KW, D, XWANT, 0, true>(p, stream);
    }
  }
  size_t lds = rows8_lds_bytes<FMT>(p, MT);
  size_t red = (size_t)RWG * KW * MT * 8 * 4;
  if (red > lds) lds = red;
  auto kern = gemv_rows8_kernel<FMT, MT, RWG, KW, D, XWANT, PRO, PRE>;
  if (lds > 64 * 1024) {
    if (int rc = check_hip(hipFuncSetAttribute(reinterpret_cast<const void *>(kern),
                                               hipFuncAttributeMaxDynamicSharedMemorySize, (int)lds),
                           "hipFuncSetAttribute"))
      return rc;
  }
  uint32_t groups = (p.N + 7) / 8;
  dim3 grid((groups + RWG - 1) / RWG), block(64 * RWG * KW);
  hipLaunchKernelGGL(kern, grid, block, lds, stream, p.W, p.A, p.sumsq_parts, p.M, p.K, p.N, p.strideA, p.nsteps, p.row_bytes, rows8_hot_flags(p), p);
  return check_hip(hipGetLastError(), "gemv launch");
}

// Workgroup shapes: (RWG row groups, KW step ranges).  K is split while the
// grid would otherwise have fewer than ~6 waves per CU and every wave keeps at
// least 4 steps.
template <int FMT, int MT> static int launch_rows8_shape(const GemvParams &p, int rwg, int kw, hipStream_t stream) {
  constexpr int D = 4;   // 4 steps in flight per wave cover the memory latency; deeper rings slow the stream down
  // last argument: groups of 8 activations a thread stages per batch row in the first batch (K / 8 / threads,
  // rounded up to what the shape class usually needs)
  if (kw == 1) {
    if (rwg >= 8 || MT == 8) return launch_rows8<FMT, MT, 8, 1, D, 1>(p, stream);
    return launch_rows8<FMT, MT, 4, 1, D, 2>(p, stream);
  }
  if (kw == 2) return launch_rows8<FMT, MT, 2, 2, D, 4>(p, stream);
  if (kw == 4) {
    if constexpr (MT == 1) {
      // two row groups share one staging of a long x; a ring of two steps here: with 14 steps per wave and eight
      // waves per workgroup the deeper ring only delays the first step (4096 x 14336: 8.3 us against 8.7 us)
      if (rwg == 2) return launch_rows8<FMT, MT, 2, 4, 2, 4>(p, stream);
    }
    if (p.nsteps <= 16) return launch_rows8<FMT, MT, 1, 4, D, 2>(p, stream);
    return launch_rows8<FMT, MT, 1, 4, D, 8>(p, stream);
  }
  return launch_rows8<FMT, MT, 1, 8, D, 4>(p, stream);
}

template <int FA, int FB, int RWG, int KW, int D, int XWANT>
static int launch_rows8_pair(const GemvParams &pa, const GemvParams &pb, hipStream_t stream) {
  size_t la = rows8_lds_bytes<FA>(pa, 1), lb = rows8_lds_bytes<FB>(pb, 1), red = (size_t)RWG * KW * 8 * 4;
  size_t lds = la > lb ? la : lb;
  if (red > lds) lds = red;
  auto kern = gemv_rows8_pair_kernel<FA, FB, RWG, KW, D, XWANT>;
  if (lds > 64 * 1024) {
    if (int rc = check_hip(hipFuncSetAttribute(reinterpret_cast<const void *>(kern),
                                               hipFuncAttributeMaxDynamicSharedMemorySize, (int)lds),
                           "hipFuncSetAttribute"))
      return rc;
  }
  uint32_t blocks_a = ((pa.N + 7) / 8 + RWG - 1) / RWG, blocks_b = ((pb.N + 7) / 8 + RWG - 1) / RWG;
  // (both tensors share the activations: A, K, strideA and nsteps are those of the first)
  const uint32_t *pos_ptr = (pa.rope.mode || pb.rope.mode) ? pa.rope.params : reinterpret_cast<const uint32_t *>((uintptr_t)pa.A & ~(uintptr_t)3);
  hipLaunchKernelGGL(kern, dim3(blocks_a + blocks_b), dim3(64 * RWG * KW), lds, stream, pa.A, pos_ptr, pa.K, pa.strideA,
                     pa.nsteps, rows8_hot_flags(pa), rows8_hot_flags(pb), blocks_a, pa, pb);
  return check_hip(hipGetLastError(), "gemv pair launch");
}

// LDS of one workgroup of the 8-row GEMV: mt batch rows of staged activations and their per-sub-block sums (Q6_K has 16
// sub-blocks per 256 elements, the other formats 8); at batch 1 eight more floats, the per-wave shares of sum(x^2) of
// the RMSNorm prologue and of the carried norm, which exist at batch 1 only.  Without them 8 rows of K = 4096 and 4 rows
// of K = 8192 of Q6_K take exactly 80 KB, so that two workgroups share a CU.
inline size_t rows8_lds_bytes_rt(int fmt, uint32_t nsteps, int mt) {
  const size_t nsub = fmt == CUTHIP_Q6_K ? 16 : 8;
  return (size_t)mt * ((size_t)nsteps * kXStep * 2 + (size_t)nsteps * nsub * 4) + (mt == 1 ? 8 * 4 : 0);
}

// LDS a workgroup may ask for.  More would fit (160 KB per CU), but every workgroup stages all of its activations:
// at 129 KB (4 batch rows, K = 14336) the staging traffic makes this kernel slower than the 32-row fallback
// (30 us against 23.5 us for 4096 x 14336), so such shapes stay with the fallback.
constexpr size_t kRows8LdsBudget = 96 * 1024;

inline int rows8_batch_class(uint32_t M) { return M <= 1 ? 1 : (M <= 2 ? 2 : (M <= 4 ? 4 : 8)); }

// parts of K for the split across workgroups: enough parts for one workgroup of eight waves per CU, at least 4 steps per
// part (4096 x 14336 at batch 8: four parts of 14 steps 14.8 us per launch of an FFN step, eight parts of 7 steps 16.5),
// and as many more as it takes for the activations of one part to fit the LDS budget (8 rows of K = 28672: 8 parts)
inline uint32_t rows8_ksplit_parts(int fmt, uint32_t M, uint32_t N, uint32_t nsteps) {
  const uint32_t blocks = ((N + 7) / 8 + 7) / 8;
  uint32_t s = 1;
  while (s < 16 && blocks * s < 256 && nsteps / (2 * s) >= 4) s *= 2;
  const int mt = rows8_batch_class(M < 2 ? 2 : M);
  while (s < nsteps && rows8_lds_bytes_rt(fmt, (nsteps + s - 1) / s, mt) > kRows8LdsBudget) s *= 2;
  return s;
}

// steps per part and the number of non-empty parts (rounding the steps up can leave the last of the wanted parts empty)
inline void rows8_ksplit_layout(int fmt, uint32_t M, uint32_t N, uint32_t nsteps, uint32_t *part_steps, uint32_t *parts) {
  const uint32_t want = rows8_ksplit_parts(fmt, M, N, nsteps);
  *part_steps = (nsteps + want - 1) / want;
  *parts = (nsteps + *part_steps - 1) / *part_steps;
}

template <int FMT, int MT> static int launch_rows8_ksplit_mt(const GemvParams &p, float *partial, hipStream_t stream) {
  constexpr int D = 4;
  uint32_t parts, part_steps;
  rows8_ksplit_layout(FMT, p.M, p.N, p.nsteps, &part_steps, &parts);
  GemvParams q = p;
  q.K = min(p.K, part_steps * 256u);
  q.nsteps = part_steps;
  size_t lds = rows8_lds_bytes<FMT>(q, MT);
  auto kern = gemv_rows8_ksplit_kernel<FMT, MT, D>;
  if (lds > 64 * 1024) {
    if (int rc = check_hip(hipFuncSetAttribute(reinterpret_cast<const void *>(kern),
                                               hipFuncAttributeMaxDynamicSharedMemorySize, (int)lds),
                           "hipFuncSetAttribute"))
      return rc;
  }
  const uint32_t nblocks = ((p.N + 7) / 8 + 7) / 8;
  hipLaunchKernelGGL(kern, dim3(nblocks * parts), dim3(512), lds, stream, p, nblocks, part_steps, partial);
  return check_hip(hipGetLastError(), "gemv split-K launch");
}

// M = 2..8; returns the number of parts through *parts_out (the caller sums them)
template <int FMT> int launch_rows8_ksplit(const GemvParams &p, float *partial, uint32_t *parts_out, hipStream_t stream) {
  uint32_t part_steps;
  rows8_ksplit_layout(FMT, p.M, p.N, p.nsteps, &part_steps, parts_out);
  if (p.M <= 2) return launch_rows8_ksplit_mt<FMT, 2>(p, partial, stream);
  if (p.M <= 4) return launch_rows8_ksplit_mt<FMT, 4>(p, partial, stream);
  return launch_rows8_ksplit_mt<FMT, 8>(p, partial, stream);
}

struct Rows8Shape { int rwg, kw; };
Rows8Shape pick_rows8_shape(int fmt, uint32_t M, uint32_t N, uint32_t nsteps);

// true if the rows8 kernel can take the problem (activations must fit in LDS)
template <int FMT> bool rows8_fits(const GemvParams &p) {
  if (p.M > 8) return false;
  return rows8_lds_bytes<FMT>(p, rows8_batch_class(p.M)) <= kRows8LdsBudget;
}

template <int FMT> int launch_rows8_fmt(const GemvParams &p, hipStream_t stream) {
  Rows8Shape s = pick_rows8_shape(FMT, p.M, p.N, p.nsteps);
  if (FMT == CUTHIP_Q6_K && s.rwg > 4) s.rwg = 4;   // measured on the 128256 x 4096 head: 103 us against 110-114 with 8 row groups
  if (p.M <= 1) return launch_rows8_shape<FMT, 1>(p, s.rwg, s.kw, stream);
  if (p.M <= 2) return launch_rows8_shape<FMT, 2>(p, s.rwg, s.kw, stream);
  if (p.M <= 4) return launch_rows8_shape<FMT, 4>(p, s.rwg, s.kw, stream);
  return launch_rows8_shape<FMT, 8>(p, s.rwg, s.kw, stream);
}

// Pair launch for the K-quant formats at the shapes a decode step uses; returns false (nothing launched) for
// anything else, and the caller issues two launches.
template <int FA, int FB> bool launch_rows8_pair_fmt(const GemvParams &pa, const GemvParams &pb, hipStream_t stream, int *rc) {
  if (pa.M != 1 || pb.M != 1 || pa.K != pb.K || pa.pro || pb.pro) return false;
  if (rows8_lds_bytes<FA>(pa, 1) > kRows8LdsBudget || rows8_lds_bytes<FB>(pb, 1) > kRows8LdsBudget) return false;
  Rows8Shape s = pick_rows8_shape(FA, 1, pa.N + pb.N, pa.nsteps);
  constexpr int D = 4;
  if (s.kw == 1 && s.rwg < 8) *rc = launch_rows8_pair<FA, FB, 4, 1, D, 2>(pa, pb, stream);
  else if (s.kw == 2) *rc = launch_rows8_pair<FA, FB, 2, 2, D, 4>(pa, pb, stream);
  // four steps per wave: a ring of two (1.730 against 1.750 ms per token of an 8B decode step with a ring of four)
  else if (s.kw == 4 && pa.nsteps <= 16) *rc = launch_rows8_pair<FA, FB, 1, 4, 2, 2>(pa, pb, stream);
  else return false;
  return true;
}

}  // namespace cuthip
