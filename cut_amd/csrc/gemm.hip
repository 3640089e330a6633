// Prefill GEMM on native GGUF blocks for gfx950:
//   C[m,n] = sum_k A[m,k] * dequant(W)[n,k],  M > 32.
//
// Supersedes MatMulQ{4,8}CoopMatTiled.cu (operators/impl/matmul): 32x32x16
// tiles with one 16x16x16 MMA per warp between two barriers.  Here a workgroup
// of four waves owns a BM x 128 tile of C (BM = 256, 128 or - up to 64 rows of A - 64), each wave a
// (BM/2) x 64 sub-tile held in fp32 accumulators, and walks K in slices of 64.
// Per slice the workgroup
//   * copies the A slice to LDS as fp16 (fp32 activations are rounded once),
//   * decodes the W slice straight from the GGUF blocks: every thread takes one
//     32-element quantization sub-block of one weight row, evaluates the
//     reference's fp32 expression (d*sc)*q - dmin*m for it and stores the 32
//     values to LDS as fp16 (round to nearest even), so each weight is decoded
//     once per BM rows of activations,
//   * feeds both tiles to v_mfma_f32_32x32x16_f16 (fp32 accumulate).
// Both LDS tiles are K-contiguous with a 16-byte row pad, which is the operand
// layout of the MFMA (lane l: row l & 31, k = 8*(l >> 5) .. +7) and keeps the
// 16-byte fragment reads off each other's banks.
//
// The global loads of slice t+1 are issued before the MFMAs of slice t and
// land in registers; two workgroups fit on a CU, so one computes while the
// other waits at its barrier.  Workgroup ids are remapped so that all M-tiles
// of one 128-column weight panel run on the same XCD and share its L2.
//
// Error budget against the fp32 CPU path: weights rounded to fp16 (2^-11
// relative), fp16 activations exact, fp32 accumulation: ~3e-4 normwise.
#include <type_traits>

#include "common.hpp"
#include "gemm_store.hpp"

namespace cuthip {

struct GemmParams {
  const uint8_t *W;
  const void *A;
  void *C;
  Epilogue epi;
  uint32_t M, K, N, strideA, strideC;
  uint32_t row_bytes;
  uint32_t mtiles, ntiles;
  int a_f16, c_f16;
  int vec_store;   // C (and a binary epilogue's operand) allow 16-byte accesses
  // K split over ksplit workgroups per tile (ranges of kper elements, a multiple of the slice): each writes fp32
  // partial products [split][M][N] and a reduce kernel applies the epilogue; 1 = the tile's workgroup writes C itself
  uint32_t ksplit, kper;
  float *partial;
};

constexpr int kBN = 128, kBK = 64, kLdsRow = kBK + 8;  // halfs per LDS row

// defined with the two-pass GEMM: C = epilogue(sum of the fp32 partial products)
int launch_splitk_reduce(const float *partial, uint32_t ksplit, uint32_t M, uint32_t N, void *C, uint32_t strideC, Epilogue epi,
                         int c_f16, hipStream_t stream);

// ---- decode of one 32-element sub-block -------------------------------------
// sub: index of the 32-element sub-block inside its row (k = 32*sub .. +31).
// Raw holds what one thread loads for it; decode() writes 32 fp16 values.
template <int FMT> struct Sub;

template <> struct Sub<CUTHIP_Q4_K> {
  struct Raw { u32x4 hdr; u32x4 q[2]; };
  __device__ static void load(Raw &r, const uint8_t *row, uint32_t sub) {
    const uint8_t *blk = row + (size_t)(sub >> 3) * 144;
    r.hdr = ld_u32x4(blk);
    const uint8_t *qs = blk + 16 + 32 * ((sub & 7) >> 1);
    r.q[0] = ld_u32x4(qs);
    r.q[1] = ld_u32x4(qs + 16);
  }
  __device__ static void decode(const Raw &r, uint32_t sub, half_t (&w)[32]) {
    uint32_t j = sub & 7;
    float d = f16bits_to_f32(r.hdr.x & 0xFFFF), dmin = f16bits_to_f32(r.hdr.x >> 16);
    uint32_t sc_lo, sc_hi, m_lo, m_hi;
    q4k_scales(r.hdr.y, r.hdr.z, r.hdr.w, sc_lo, sc_hi, m_lo, m_hi);
    uint32_t bsh = 8 * (j & 3);
    float d1 = d * (float)(((j < 4 ? sc_lo : sc_hi) >> bsh) & 0xFF);
    float dm1 = dmin * (float)(((j < 4 ? m_lo : m_hi) >> bsh) & 0xFF);
    uint32_t sh = (j & 1) * 4;
#pragma unroll
    for (int i = 0; i < 8; ++i) {
      uint32_t word = i < 4 ? r.q[0][i] : r.q[1][i - 4];
      word = (word >> sh) & 0x0F0F0F0Fu;
      asm volatile("" : "+v"(word));   // one shift + mask per four quants, then v_cvt_f32_ubyte0..3
      w[4 * i + 0] = (half_t)(d1 * cvt_ubyte0(word) - dm1);
      w[4 * i + 1] = (half_t)(d1 * cvt_ubyte1(word) - dm1);
      w[4 * i + 2] = (half_t)(d1 * cvt_ubyte2(word) - dm1);
      w[4 * i + 3] = (half_t)(d1 * cvt_ubyte3(word) - dm1);
    }
  }
};

template <> struct Sub<CUTHIP_Q6_K> {
  // qh1: half of the 32 high-bit bytes of the block's half H.  The two threads of a pair (tid, tid ^ 1: the two
  // sub-blocks of one weight row in a slice) need the same 32 bytes; the even one loads the first 16, the odd one the
  // second 16, and decode() exchanges them inside the quad.  The blocks are 2-byte aligned, and what such loads return
  // through the vector memory path is what the decode of this format is short of.
  // sd: the even thread loads the pair's two scale bytes (they are adjacent), the odd one the last scale bytes and d;
  // one small load per thread and slice instead of two.
  struct Raw { u32x4 ql[2]; u32x4 qh1; uint32_t sd; };
  __device__ static void load(Raw &r, const uint8_t *row, uint32_t sub) {
    const uint8_t *blk = row + (size_t)(sub >> 3) * 210;
    uint32_t H = (sub >> 2) & 1, s = sub & 3;
    const uint8_t *ql = blk + 64 * H + 32 * (s & 1), *qh = blk + 128 + 32 * H;
    r.ql[0] = ld_u32x4(ql); r.ql[1] = ld_u32x4(ql + 16);
    r.qh1 = ld_u32x4(qh + 16 * (threadIdx.x & 1));
    r.sd = ld_u32((threadIdx.x & 1) ? blk + 206 : blk + 192 + 8 * H + 2 * (s & 2));
  }
  __device__ static void decode(const Raw &r, uint32_t sub, half_t (&w)[32]) {
    uint32_t s = sub & 3;
    const uint32_t sc2 = (uint32_t)__builtin_amdgcn_mov_dpp((int)r.sd, 0xA0, 0xF, 0xF, true);   // the pair's scales
    const uint32_t dd = (uint32_t)__builtin_amdgcn_mov_dpp((int)r.sd, 0xF5, 0xF, 0xF, true);    // d in the high half
    const uint32_t sc = (threadIdx.x & 1) ? sc2 >> 16 : sc2 & 0xFFFF;
    float d = f16bits_to_f32(dd >> 16);
    float dsc0 = d * (float)(int)(int8_t)(sc & 0xFF), dsc1 = d * (float)(int)(int8_t)(sc >> 8);
    const float off0 = -32.0f * dsc0, off1 = -32.0f * dsc1;
    uint32_t lsh = (s >> 1) * 4, hsh = 2 * s;
    uint32_t qh[8];   // quad_perm [0,0,2,2]: the even thread's 16 bytes; [1,1,3,3]: the odd thread's
#pragma unroll
    for (int i = 0; i < 4; ++i) {
      qh[i] = (uint32_t)__builtin_amdgcn_mov_dpp((int)r.qh1[i], 0xA0, 0xF, 0xF, true);
      qh[4 + i] = (uint32_t)__builtin_amdgcn_mov_dpp((int)r.qh1[i], 0xF5, 0xF, 0xF, true);
    }
#pragma unroll
    for (int i = 0; i < 8; ++i) {
      uint32_t wl = i < 4 ? r.ql[0][i] : r.ql[1][i - 4], wh = qh[i];
      uint32_t q6 = ((wl >> lsh) & 0x0F0F0F0Fu) | (((wh >> hsh) & 0x03030303u) << 4);
      asm volatile("" : "+v"(q6));
      // dsc * (q - 32) as one fused multiply-add with the exact constant -32 dsc: the same real number rounded once,
      // hence the same bits, and one instruction per weight less
      const float dsc = i < 4 ? dsc0 : dsc1, off = i < 4 ? off0 : off1;  // elements 0-15 / 16-31 of the 32
      w[4 * i + 0] = (half_t)__builtin_fmaf(dsc, cvt_ubyte0(q6), off);
      w[4 * i + 1] = (half_t)__builtin_fmaf(dsc, cvt_ubyte1(q6), off);
      w[4 * i + 2] = (half_t)__builtin_fmaf(dsc, cvt_ubyte2(q6), off);
      w[4 * i + 3] = (half_t)__builtin_fmaf(dsc, cvt_ubyte3(q6), off);
    }
  }
};

template <> struct Sub<CUTHIP_Q8_0> {
  struct Raw { u32x4 q[2]; uint32_t d; };
  __device__ static void load(Raw &r, const uint8_t *row, uint32_t sub) {
    const uint8_t *blk = row + (size_t)sub * 34;
    r.d = ld_u16(blk);
    r.q[0] = ld_u32x4(blk + 2);
    r.q[1] = ld_u32x4(blk + 18);
  }
  __device__ static void decode(const Raw &r, uint32_t, half_t (&w)[32]) {
    const float d = f16bits_to_f32(r.d), off = -128.0f * d;   // d * (q + 128 - 128) as one exact fused multiply-add
#pragma unroll
    for (int i = 0; i < 8; ++i) {
      uint32_t word = (i < 4 ? r.q[0][i] : r.q[1][i - 4]) ^ 0x80808080u;  // q + 128 as unsigned bytes
      w[4 * i + 0] = (half_t)__builtin_fmaf(d, cvt_ubyte0(word), off);
      w[4 * i + 1] = (half_t)__builtin_fmaf(d, cvt_ubyte1(word), off);
      w[4 * i + 2] = (half_t)__builtin_fmaf(d, cvt_ubyte2(word), off);
      w[4 * i + 3] = (half_t)__builtin_fmaf(d, cvt_ubyte3(word), off);
    }
  }
};

template <> struct Sub<CUTHIP_Q4_0> {
  struct Raw { u32x4 q; uint32_t d; };
  __device__ static void load(Raw &r, const uint8_t *row, uint32_t sub) {
    const uint8_t *blk = row + (size_t)sub * 18;
    r.d = ld_u16(blk);
    r.q = ld_u32x4(blk + 2);
  }
  __device__ static void decode(const Raw &r, uint32_t, half_t (&w)[32]) {
    const float d = f16bits_to_f32(r.d), off = -8.0f * d;   // d * (q - 8) as one exact fused multiply-add
#pragma unroll
    for (int i = 0; i < 4; ++i) {
      uint32_t lo = r.q[i] & 0x0F0F0F0Fu, hi = (r.q[i] >> 4) & 0x0F0F0F0Fu;
      w[4 * i + 0] = (half_t)__builtin_fmaf(d, cvt_ubyte0(lo), off);
      w[4 * i + 1] = (half_t)__builtin_fmaf(d, cvt_ubyte1(lo), off);
      w[4 * i + 2] = (half_t)__builtin_fmaf(d, cvt_ubyte2(lo), off);
      w[4 * i + 3] = (half_t)__builtin_fmaf(d, cvt_ubyte3(lo), off);
      w[16 + 4 * i + 0] = (half_t)__builtin_fmaf(d, cvt_ubyte0(hi), off);
      w[16 + 4 * i + 1] = (half_t)__builtin_fmaf(d, cvt_ubyte1(hi), off);
      w[16 + 4 * i + 2] = (half_t)__builtin_fmaf(d, cvt_ubyte2(hi), off);
      w[16 + 4 * i + 3] = (half_t)__builtin_fmaf(d, cvt_ubyte3(hi), off);
    }
  }
};

typedef _Float16 half8v __attribute__((ext_vector_type(8)));
typedef __attribute__((address_space(3))) uint8_t lds_u8g;

// ---- the kernel -----------------------------------------------------------------
template <int FMT, int BM, bool AF16>
__global__ void __launch_bounds__(256, 2) gemm_kernel(GemmParams p) {
  using S = Sub<FMT>;
  constexpr int MI = BM / 64;          // 32-row MFMA tiles per wave along M
  constexpr int AV = BM * kBK / 8 / 256;  // 16-byte A vectors per thread per slice
  extern __shared__ __attribute__((aligned(16))) uint8_t lds[];
  half_t *As = reinterpret_cast<half_t *>(lds);             // [BM][kLdsRow]
  half_t *Bs = As + BM * kLdsRow;                           // [kBN][kLdsRow]

  // XCD-aware tile order: ids id, id+8, id+16, ... share an XCD; give them the
  // M-tiles of the same weight panel.
  const uint32_t tiles = p.mtiles * p.ntiles, split = blockIdx.x / tiles;
  uint32_t id = blockIdx.x - split * tiles, mt, nt;
  if (p.ntiles % 8 == 0) {
    uint32_t xcd = id & 7, slot = id >> 3;
    nt = (slot / p.mtiles) * 8 + xcd;
    mt = slot % p.mtiles;
  } else {
    nt = id / p.mtiles;
    mt = id % p.mtiles;
  }
  const uint32_t m0 = mt * BM, n0 = nt * kBN;
  const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
  const int wm = wave >> 1, wn = wave & 1;

  // weight decode assignment: thread -> (row n0 + tid/2, sub-block tid&1 of the slice)
  const uint32_t brow = min(n0 + (uint32_t)(tid >> 1), p.N - 1);
  const uint8_t *wrow = p.W + (size_t)brow * p.row_bytes;
  const uint32_t bsub = tid & 1;
  const uint32_t nsub = p.K / 32;  // sub-blocks per row

  f32x16 acc[MI][2];
#pragma unroll
  for (int i = 0; i < MI; ++i)
#pragma unroll
    for (int j = 0; j < 2; ++j) acc[i][j] = f32x16{0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0};

  typename S::Raw braw;
  u32x4 araw[AV], araw2[AF16 ? 1 : AV];  // araw2: second half of an fp32 group of 8

  auto load_slice = [&](uint32_t k0) {
    uint32_t sub = min(k0 / 32 + bsub, nsub - 1);
    S::load(braw, wrow, sub);
#pragma unroll
    for (int v = 0; v < AV; ++v) {
      int idx = v * 256 + tid;              // vector index in the [BM][8] grid of the slice
      uint32_t r = min(m0 + (uint32_t)(idx >> 3), p.M - 1), kc = k0 + (idx & 7) * 8;
      kc = min(kc, p.K - 8);
      size_t off = (size_t)r * p.strideA + kc;
      if constexpr (AF16) {
        araw[v] = ld_u32x4(reinterpret_cast<const uint8_t *>(p.A) + off * 2);
      } else {
        araw[v] = ld_u32x4(reinterpret_cast<const uint8_t *>(p.A) + off * 4);
        araw2[v] = ld_u32x4(reinterpret_cast<const uint8_t *>(p.A) + off * 4 + 16);
      }
    }
  };
  // TAIL: the last slice of a K that is not a multiple of 64 (Q8_0 / Q4_0 only); columns past K are zeroed
  auto store_slice = [&](uint32_t k0, auto tail) {
    constexpr bool TAIL = decltype(tail)::value;
    half_t w[32];
    S::decode(braw, k0 / 32 + bsub, w);
    const bool live = !TAIL || k0 + 32 * bsub < p.K;
    half_t *dst = Bs + (tid >> 1) * kLdsRow + 32 * bsub;
#pragma unroll
    for (int c = 0; c < 4; ++c) {
      half8v o;
#pragma unroll
      for (int e = 0; e < 8; ++e) o[e] = w[8 * c + e];
      if (TAIL && !live) o = half8v{0, 0, 0, 0, 0, 0, 0, 0};
      *reinterpret_cast<half8v *>(dst + 8 * c) = o;
    }
#pragma unroll
    for (int v = 0; v < AV; ++v) {
      int idx = v * 256 + tid;
      half8v o;
      if constexpr (AF16) {
        o = __builtin_bit_cast(half8v, araw[v]);
      } else {
        f32x4 lo = __builtin_bit_cast(f32x4, araw[v]), hi = __builtin_bit_cast(f32x4, araw2[v]);
        o = half8v{(half_t)lo.x, (half_t)lo.y, (half_t)lo.z, (half_t)lo.w,
                   (half_t)hi.x, (half_t)hi.y, (half_t)hi.z, (half_t)hi.w};
      }
      if (TAIL && !(k0 + (idx & 7) * 8 < p.K)) o = half8v{0, 0, 0, 0, 0, 0, 0, 0};
      *reinterpret_cast<half8v *>(As + (idx >> 3) * kLdsRow + (idx & 7) * 8) = o;
    }
  };
  auto mma_slice = [&]() {
    const half_t *a_base = As + (wm * (BM / 2) + (lane & 31)) * kLdsRow + 8 * (lane >> 5);
    const half_t *b_base = Bs + (wn * 64 + (lane & 31)) * kLdsRow + 8 * (lane >> 5);
#pragma unroll
    for (int s = 0; s < kBK / 16; ++s) {
      half8v bf[2], af[MI];
#pragma unroll
      for (int j = 0; j < 2; ++j) bf[j] = *reinterpret_cast<const half8v *>(b_base + 32 * j * kLdsRow + 16 * s);
#pragma unroll
      for (int i = 0; i < MI; ++i) af[i] = *reinterpret_cast<const half8v *>(a_base + 32 * i * kLdsRow + 16 * s);
#pragma unroll
      for (int i = 0; i < MI; ++i)
#pragma unroll
        for (int j = 0; j < 2; ++j)
          acc[i][j] = __builtin_amdgcn_mfma_f32_32x32x16_f16(af[i], bf[j], acc[i][j], 0, 0, 0);
    }
  };

  // this workgroup's K range [kb, ke): all of K without a split; only the last range can end in a partial slice
  const uint32_t kb = split * p.kper, ke = min(p.K, kb + p.kper);
  const uint32_t nfull = (ke - kb) / kBK, nslices = (ke - kb + kBK - 1) / kBK;
  load_slice(kb);
  for (uint32_t t = 0; t < nfull; ++t) {
    __syncthreads();           // everyone is done reading the previous slice
    store_slice(kb + t * kBK, std::false_type{});
    __syncthreads();
    if (t + 1 < nslices) load_slice(kb + (t + 1) * kBK);
    mma_slice();
  }
  if (nfull < nslices) {
    __syncthreads();
    store_slice(kb + nfull * kBK, std::true_type{});
    __syncthreads();
    mma_slice();
  }

  // C tile through LDS, a 32-row stripe of the wave's sub-tile at a time (gemm_store.hpp); the operand tiles are free
  // once every wave has multiplied the last slice
  // the output staging reuses the operand tiles (the launch asks for the larger of the two)
  __syncthreads();
  lds_f32 *stage = (lds_f32 *)(lds_u8g *)(lds) + wave * stripe_floats<2>();
  Epilogue epi = p.epi;
  const uint32_t Mrows = p.M, Ncols = p.N;
  uint32_t ldc = p.strideC;
  void *cbase = p.C;
  int c_f16 = p.c_f16;
  bool vec = p.vec_store != 0;
  if (p.ksplit > 1) {   // fp32 partial products of this K range; the reduce kernel owns the epilogue
    cbase = p.partial + (size_t)split * p.M * p.N;
    ldc = p.N;
    c_f16 = 0;
    epi.kind = CUTHIP_EPI_NONE;
    vec = p.N % 4 == 0;
  }
  // the common cases get the short store loops: no operator, or the residual add; fp32 partial products
  const int fast = !vec ? 0 : !c_f16 ? (p.ksplit > 1 ? 3 : 0) : epi.kind == CUTHIP_EPI_NONE ? 1
                   : (epi.kind == CUTHIP_EPI_BINARY && epi.op == CUTHIP_BINARY_ADD) ? 2 : 0;
  static_for<MI>([&](auto ii) __attribute__((always_inline)) {
    constexpr int i = decltype(ii)::value;
    stage_tile32<2>(stage, 0, acc[i][0], lane);
    stage_tile32<2>(stage, 1, acc[i][1], lane);
    if (fast == 1) store_staged32<2, 1>(stage, m0 + wm * (BM / 2) + 32 * i, n0 + wn * 64, Mrows, Ncols, cbase, ldc, c_f16, epi, vec, lane);
    else if (fast == 2) store_staged32<2, 2>(stage, m0 + wm * (BM / 2) + 32 * i, n0 + wn * 64, Mrows, Ncols, cbase, ldc, c_f16, epi, vec, lane);
    else if (fast == 3) store_staged32<2, 3>(stage, m0 + wm * (BM / 2) + 32 * i, n0 + wn * 64, Mrows, Ncols, cbase, ldc, c_f16, epi, vec, lane);
    else store_staged32<2, 0>(stage, m0 + wm * (BM / 2) + 32 * i, n0 + wn * 64, Mrows, Ncols, cbase, ldc, c_f16, epi, vec, lane);
  });
}

// K ranges per 128-row tile for a problem of 128 x 128 tiles with scratch_bytes of room for the partial products
uint32_t tiled_gemm_ksplit(uint32_t M, uint32_t K, uint32_t N, size_t scratch_bytes) {
  const uint64_t tiles = (uint64_t)((M + 127) / 128) * ((N + kBN - 1) / kBN);
  const uint32_t nslices = (K + kBK - 1) / kBK;
  uint32_t ks = 1;
  while (ks < 16 && tiles * ks < 384 && nslices / (2 * ks) >= 8 && (uint64_t)2 * ks * M * N * 4 <= scratch_bytes) ks *= 2;
  return ks;
}

template <int FMT, int BM, bool AF16> static int launch_gemm_bm(GemmParams p, hipStream_t stream) {
  p.mtiles = (p.M + BM - 1) / BM;
  p.ntiles = (p.N + kBN - 1) / kBN;
  size_t lds = (size_t)(BM + kBN) * kLdsRow * 2;
  if (lds < 4 * stripe_floats<2>() * 4) lds = 4 * stripe_floats<2>() * 4;
  auto kern = gemm_kernel<FMT, BM, AF16>;
  if (lds > 64 * 1024) {
    if (int rc = check_hip(hipFuncSetAttribute(reinterpret_cast<const void *>(kern),
                                               hipFuncAttributeMaxDynamicSharedMemorySize, (int)lds),
                           "hipFuncSetAttribute"))
      return rc;
  }
  // K split: with a scratch area at hand and too few tiles for the chip, up to sixteen K ranges of at least eight
  // slices each (a workgroup walks its slices one memory round trip at a time, so short of two workgroups per CU
  // the launch is bound by that latency: 14336 x 4096 at 64 rows 66 us unsplit)
  const uint64_t tiles = (uint64_t)p.mtiles * p.ntiles;
  const uint32_t nslices = (p.K + kBK - 1) / kBK;
  uint32_t ks = 1;
  if (p.partial && BM <= 128) {
    ks = tiled_gemm_ksplit(p.M, p.K, p.N, p.kper);
    const uint32_t want = (uint32_t)g_tuning.gemm_ksplit;   // forced by a test or a sweep
    if (want >= 1 && want <= 16 && (uint64_t)want * p.M * p.N * 4 <= p.kper) ks = want;
  }
  const uint32_t per = (nslices + ks - 1) / ks;
  p.kper = per * kBK;                      // (on entry: bytes of scratch behind partial)
  p.ksplit = (nslices + per - 1) / per;    // no empty range
  if (p.ksplit == 1) p.kper = p.K + kBK;
  uint64_t grid = tiles * p.ksplit;
  if (grid > 0x7FFFFFFFull) {
    set_error("cuthip_matmul_gguf: problem too large for one launch");
    return CUTHIP_ERR_INVALID;
  }
  hipLaunchKernelGGL(kern, dim3((uint32_t)grid), dim3(256), lds, stream, p);
  if (int rc = check_hip(hipGetLastError(), "gemm launch")) return rc;
  if (p.ksplit == 1) return CUTHIP_OK;
  return launch_splitk_reduce(p.partial, p.ksplit, p.M, p.N, p.C, p.strideC, p.epi, p.c_f16, stream);
}

template <int FMT> static int launch_gemm_fmt(const GemmParams &p, hipStream_t stream) {
  // 256-row tiles once they fill the chip (>= 2 workgroups per CU), else 128-row tiles.
  // fp32 activations and Q6_K need more staging registers and always take 128 rows.
  if (!p.a_f16) return p.M <= 64 ? launch_gemm_bm<FMT, 64, false>(p, stream) : launch_gemm_bm<FMT, 128, false>(p, stream);
  uint64_t tiles256 = (uint64_t)((p.M + 255) / 256) * ((p.N + kBN - 1) / kBN);
  if constexpr (FMT != CUTHIP_Q6_K) {
    if (tiles256 >= 512) return launch_gemm_bm<FMT, 256, true>(p, stream);
  }
  // up to 64 rows: 64-row tiles, half the matrix-core work per slice (14336 x 4096 at 33-64 rows 28-29 us against 33-34)
  if (p.M <= 64) return launch_gemm_bm<FMT, 64, true>(p, stream);
  return launch_gemm_bm<FMT, 128, true>(p, stream);
}

// scratch: 16-byte aligned room for fp32 partial products of a K split (nullptr / 0: none, one workgroup per tile)
int launch_gemm(int fmt, const void *W, const void *A, int a_f16, void *C, int c_f16, uint32_t M, uint32_t K, uint32_t N,
                uint32_t strideA, uint32_t strideC, Epilogue epi, hipStream_t stream, void *scratch, size_t scratch_bytes) {
  GemmParams p;
  p.W = reinterpret_cast<const uint8_t *>(W);
  p.A = A;
  p.C = C;
  p.epi = epi;
  p.M = M; p.K = K; p.N = N; p.strideA = strideA; p.strideC = strideC;
  p.row_bytes = (uint32_t)((uint64_t)(K / fmt_elems(fmt)) * fmt_bytes(fmt));
  p.mtiles = p.ntiles = 0;
  p.a_f16 = a_f16; p.c_f16 = c_f16;
  p.vec_store = store8_aligned(C, strideC, c_f16, epi) ? 1 : 0;
  p.ksplit = 1;
  p.partial = scratch && (uintptr_t)scratch % 16 == 0 ? reinterpret_cast<float *>(scratch) : nullptr;
  p.kper = (uint32_t)(scratch_bytes < 0xFFFFFFFFull ? scratch_bytes : 0xFFFFFFFFull);   // launch_gemm_bm turns it into the range
  switch (fmt) {
  case CUTHIP_Q8_0: return launch_gemm_fmt<CUTHIP_Q8_0>(p, stream);
  case CUTHIP_Q4_0: return launch_gemm_fmt<CUTHIP_Q4_0>(p, stream);
  case CUTHIP_Q4_K: return launch_gemm_fmt<CUTHIP_Q4_K>(p, stream);
  default: return launch_gemm_fmt<CUTHIP_Q6_K>(p, stream);
  }
}

}  // namespace cuthip
