// Streaming quantized GEMV / skinny GEMM on native GGUF blocks for gfx950:
//   C[m,n] = sum_k A[m,k] * dequant(W)[n,k],  M <= 32 per pass.
//
// Supersedes MatMulQ{4,8}GemvKPar8.cu (operators/impl/matmul), whose lanes
// gather 4 bytes at a stride of N across k; here the weights stay in the GGUF
// file layout (row n = K/blk consecutive blocks) and are streamed once with
// 8- and 16-byte loads.
//
// Work decomposition.  The unit of work is one wave instruction tile of
// v_mfma_f32_32x32x16_f16: 32 B-columns x 16 k.  A workgroup owns RT = 32/KP
// consecutive weight rows and the whole K range.  K is cut in steps of 256
// elements; the WAVES waves of the workgroup take contiguous step ranges, and
// inside a wave the 32 MFMA columns are (row, part) pairs: column j serves
// weight row n0 + j/KP and the part j%KP of the wave's step range.  KP > 1
// keeps all 256 CUs busy when N/32 is smaller than the CU count (the 4096-row
// projections of an 8B model) without atomics: the MFMA A-row j likewise
// carries the activations of batch row j/KP for the same part j%KP, so
// C[j][j'] is a valid partial sum exactly when both belong to the same part.
// Partial sums of all (wave, part) pairs are folded through LDS at the end.
// Lane l serves column/row l & 31 and the half kg = l >> 5 of each 16-wide
// k-slice (A and B operands both hold k = 8*kg .. 8*kg+7).
//
// Arithmetic.  The packed quants are turned into fp16 *subnormals* with one
// AND per pair of weights: a nibble left in bits 0-3 of a 16-bit lane is the
// fp16 number q * 2^-24 (bits 4-7: q * 2^-20), exact, and the matrix core
// multiplies subnormals exactly.  One MFMA chain therefore yields the exact
// integer dot product sum(q * x) of one quantization sub-block for 32 columns,
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
//
// Memory.  Every lane keeps the loads of up to D steps in flight (a register
// ring), so a wave has up to D * 4.6 KB outstanding; nothing is re-read.  When
// the step count per part is a compile-time constant (CNT > 0) the whole wave
// body is straight-line code: loads are unconditional and in program order
// (activations first), so each consumer waits only for its own data
// (s_waitcnt vmcnt(n) with the exact n) and computes while later steps are
// still in flight.  The generic path (CNT == 0) handles any K with loops.
#pragma once
#include "gemv_formats.hpp"

namespace cuthip {

// ---- staging of the activations, generic path ---------------------------------
// Fills the wave's LDS tile: staged row a = m*KP + part holds elements
// [(part_base(part) + t0)*256, +steps*256) of batch row m as fp16 in the
// (0,2,1,3,4,6,5,7) order, and sxs the sums of every SUBK consecutive (rounded)
// elements.  Elements past K are zero.
template <int SUBK, int KP, int XROW, int SXROW>
__device__ inline void stage_x(const GemvParams &p, uint32_t sb, uint32_t cnt, uint32_t t0, int steps, half_t *xs,
                               float *sxs, int lane) {
  const int groups_per_row = steps * 32;  // 8-element groups
  const int total = (int)p.M * KP * groups_per_row;
  for (int i0 = 0; i0 < total; i0 += kWave) {
    int t = i0 + lane;
    bool active = t < total;
    int a = active ? t / groups_per_row : 0;  // staged row = m*KP + part
    int gi = active ? t - a * groups_per_row : 0;
    int m = a / KP, part = a - m * KP;
    uint32_t k = (sb + (uint32_t)part * cnt + t0) * 256u + (uint32_t)gi * 8;
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
      *reinterpret_cast<half8_t *>(xs + a * XROW + gi * 8) = o;
      constexpr int per = SUBK / 8;
      if ((gi & (per - 1)) == 0) sxs[a * SXROW + gi / per] = s;
    }
  }
}

// ---- staging of the activations, straight-line path -----------------------------
// Same result as stage_x, split in two branch-free halves: x_load issues the
// global loads of the whole tile into registers (before any weight load),
// x_store converts, permutes and writes them to LDS.
template <int XI> struct XTile { u32x4 a[XI]; u32x4 b[XI]; };  // b: second half of an fp32 group

template <int KP, int CNT, int XI>
__device__ inline void x_load(const GemvParams &p, uint32_t sb, int lane, XTile<XI> &xt) {
  constexpr int groups_per_row = CNT * 32;
  const int total = (int)p.M * KP * groups_per_row;
  const uint32_t esz = p.a_f16 ? 2u : 4u;
  const uint32_t b_off = p.a_f16 ? 0u : 16u;  // fp16: the second load re-reads the same line and is unused
#pragma unroll
  for (int it = 0; it < XI; ++it) {
    int t = it * kWave + lane;
    int a = t / groups_per_row, gi = t - a * groups_per_row;
    int m = a / KP, part = a - m * KP;
    uint32_t k = (sb + (uint32_t)part * CNT) * 256u + (uint32_t)gi * 8;
    bool ok = t < total && k < p.K;
    size_t off = ok ? ((size_t)m * p.strideA + k) * esz : 0;
    const uint8_t *src = reinterpret_cast<const uint8_t *>(p.A) + off;
    xt.a[it] = ld_u32x4(src);
    xt.b[it] = ld_u32x4(src + b_off);
  }
}

template <int SUBK, int KP, int CNT, int XROW, int SXROW, int XI>
__device__ inline void x_store(const GemvParams &p, uint32_t sb, half_t *xs, float *sxs, int lane,
                               const XTile<XI> &xt) {
  constexpr int groups_per_row = CNT * 32;
  const int total = (int)p.M * KP * groups_per_row;
#pragma unroll
  for (int it = 0; it < XI; ++it) {
    int t = it * kWave + lane;
    int a = t / groups_per_row, gi = t - a * groups_per_row;
    int m = a / KP, part = a - m * KP;
    uint32_t k = (sb + (uint32_t)part * CNT) * 256u + (uint32_t)gi * 8;
    bool active = t < total;
    bool ok = active && k < p.K;
    half8_t v16 = __builtin_bit_cast(half8_t, xt.a[it]);
    f32x4 lo = __builtin_bit_cast(f32x4, xt.a[it]), hi = __builtin_bit_cast(f32x4, xt.b[it]);
    half_t h32[8] = {(half_t)lo.x, (half_t)lo.y, (half_t)lo.z, (half_t)lo.w,
                     (half_t)hi.x, (half_t)hi.y, (half_t)hi.z, (half_t)hi.w};
    half_t h[8];
#pragma unroll
    for (int i = 0; i < 8; ++i) {
      half_t e = p.a_f16 ? v16[i] : h32[i];
      h[i] = ok ? e : (half_t)0.0f;
    }
    float s = 0.0f;
#pragma unroll
    for (int i = 0; i < 8; ++i) s += (float)h[i];
    s += __shfl_xor(s, 1);
    if (SUBK == 32) s += __shfl_xor(s, 2);
    if (active) {
      half8_t o{h[0], h[2], h[1], h[3], h[4], h[6], h[5], h[7]};
      *reinterpret_cast<half8_t *>(xs + a * XROW + gi * 8) = o;
      constexpr int per = SUBK / 8;
      if ((gi & (per - 1)) == 0) sxs[a * SXROW + gi / per] = s;
    }
  }
}

// ---- the kernel -----------------------------------------------------------------
// CNT > 0: every wave owns exactly CNT*KP steps (nsteps == WAVES*KP*CNT up to
// the last part's tail, which is masked), CNT <= TB, and TileCfg::PIPE holds.
template <int FMT, int MT, int WAVES, int KP, int CNT>
__global__ void __launch_bounds__(64 * WAVES, 2) gemv_kernel(GemvParams p) {
  using S = Step<FMT>;
  using T = TileCfg<MT, KP>;
  constexpr int R = T::R, TB = T::TB, D = T::D, XROW = T::XROW, SXROW = TB * S::NSUB;
  constexpr int RT = 32 / KP;                                   // weight rows per workgroup
  constexpr int WAVE_LDS = T::ROWS * (XROW * 2 + SXROW * 4);    // bytes per wave
  static_assert(TB % D == 0, "ring depth must divide the tile");
  static_assert(CNT == 0 || (T::PIPE && CNT <= TB), "straight-line path needs a single register-staged tile");
  extern __shared__ __attribute__((aligned(16))) uint8_t lds[];

  const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
  const int kg = lane >> 5, j = lane & 31;
  const int part = j % KP, jr = j / KP;                         // as B column: row n0+jr; as A row: batch row jr
  const uint32_t n0 = blockIdx.x * (uint32_t)RT;
  const uint32_t n = min(n0 + (uint32_t)jr, p.N - 1);
  const uint8_t *row = p.W + (size_t)n * p.row_bytes;

  half_t *xs = reinterpret_cast<half_t *>(lds + wave * WAVE_LDS);
  float *sxs = reinterpret_cast<float *>(lds + wave * WAVE_LDS + T::ROWS * XROW * 2);
  const int nrows = (int)p.M * KP;
  const half_t *xrow = xs + (min(jr, (int)p.M - 1) * KP + part) * XROW;

  // this wave's steps [sb, se), cut in KP parts of cnt steps
  const uint32_t sb = (uint32_t)(((uint64_t)p.nsteps * wave) / WAVES);
  const uint32_t se = (uint32_t)(((uint64_t)p.nsteps * (wave + 1)) / WAVES);
  const uint32_t cnt = CNT > 0 ? (uint32_t)CNT : (se - sb + KP - 1) / KP;
  const uint32_t ps = sb + (uint32_t)part * cnt;                // first step of this lane's part
  const uint32_t last = p.nsteps - 1;

  float acc[R];
#pragma unroll
  for (int r = 0; r < R; ++r) acc[r] = 0.0f;

  if constexpr (CNT > 0) {
    constexpr int XI = (T::ROWS * CNT * 32 + kWave - 1) / kWave;
    constexpr int DD = CNT < 4 ? CNT : 4;   // ring depth: measured flat between 1 and 4
    XTile<XI> xt;
    x_load<KP, CNT, XI>(p, sb, lane, xt);
    typename S::Raw buf[DD];
#pragma unroll
    for (int i = 0; i < DD; ++i) S::load(buf[i], row, min(ps + i, last), kg, p.K);
    __builtin_amdgcn_sched_barrier(0);
    x_store<S::SUBK, KP, CNT, XROW, SXROW, XI>(p, sb, xs, sxs, lane, xt);
    __builtin_amdgcn_sched_barrier(0);
    __builtin_amdgcn_wave_barrier();
    asm volatile("" ::: "memory");
#pragma unroll
    for (int i = 0; i < CNT; ++i) {
      bool valid = ps + i < se;
      S::template compute<R, SXROW>(buf[i % DD], xrow + i * 256, sxs + i * S::NSUB, kg, nrows, valid, acc);
      if (i + DD < CNT) S::load(buf[i % DD], row, min(ps + i + DD, last), kg, p.K);
      // Pin the accumulators here: otherwise the optimizer sinks every scale
      // FMA into the guarded store after the final barrier and has to keep
      // (spill) all MFMA results until then.
#pragma unroll
      for (int r = 0; r < R; ++r) asm volatile("" : "+v"(acc[r]));
      __builtin_amdgcn_sched_barrier(0);  // one step at a time: bounds the live registers
    }
  } else {
    typename S::Raw buf[D];
#pragma unroll
    for (int i = 0; i < D; ++i)
      if ((uint32_t)i < cnt) S::load(buf[i], row, min(ps + i, last), kg, p.K);
    for (uint32_t t0 = 0; t0 < cnt; t0 += TB) {
      int tb = (int)min((uint32_t)TB, cnt - t0);
      __builtin_amdgcn_wave_barrier();
      asm volatile("" ::: "memory");
      stage_x<S::SUBK, KP, XROW, SXROW>(p, sb, cnt, t0, tb, xs, sxs, lane);
      __builtin_amdgcn_wave_barrier();
      asm volatile("" ::: "memory");
#pragma unroll
      for (int b = 0; b < TB; ++b) {
        uint32_t i = t0 + b;
        if (i < cnt) {
          bool valid = ps + i < se;
          S::template compute<R, SXROW>(buf[b % D], xrow + b * 256, sxs + b * S::NSUB, kg, nrows, valid, acc);
          if (i + D < cnt) S::load(buf[b % D], row, min(ps + i + D, last), kg, p.K);
        }
      }
    }
  }

  // Fold the partial sums of all (wave, part) pairs and write C with the fused epilogue.
  __syncthreads();
  float *red = reinterpret_cast<float *>(lds);  // [WAVES*KP][MT][RT], reuses the staging area
#pragma unroll
  for (int r = 0; r < R; ++r) {
    int a = acc_row(r, kg);
    int m = a / KP, pa = a - m * KP;
    if (pa == part && m < (int)p.M) red[((wave * KP + pa) * MT + m) * RT + jr] = acc[r];
  }
  __syncthreads();
  for (int t = threadIdx.x; t < (int)p.M * RT; t += 64 * WAVES) {
    int m = t / RT, c = t - m * RT;
    uint32_t nn = n0 + c;
    if (nn >= p.N) continue;
    float v = 0.0f;
#pragma unroll
    for (int w = 0; w < WAVES * KP; ++w) v += red[(w * MT + m) * RT + c];
    store_out(p.C, p.epi, p.c_f16, (size_t)m * p.strideC + nn, v);
  }
}

template <int FMT, int MT, int WAVES, int KP> static size_t gemv_lds_bytes() {
  using S = Step<FMT>;
  using T = TileCfg<MT, KP>;
  size_t per_wave = (size_t)T::ROWS * (T::XROW * 2 + T::TB * S::NSUB * 4);
  size_t red = (size_t)WAVES * MT * 32 * 4;
  size_t a = per_wave * WAVES;
  return a > red ? a : red;
}

template <int FMT, int MT, int WAVES, int KP, int CNT>
static int launch_one(const GemvParams &p, hipStream_t stream) {
  size_t lds = gemv_lds_bytes<FMT, MT, WAVES, KP>();
  auto kern = gemv_kernel<FMT, MT, WAVES, KP, CNT>;
  if (lds > 64 * 1024) {
    if (int rc = check_hip(hipFuncSetAttribute(reinterpret_cast<const void *>(kern),
                                               hipFuncAttributeMaxDynamicSharedMemorySize, (int)lds),
                           "hipFuncSetAttribute"))
      return rc;
  }
  constexpr int RT = 32 / KP;
  dim3 grid((p.N + RT - 1) / RT), block(64 * WAVES);
  hipLaunchKernelGGL(kern, grid, block, lds, stream, p);
  return check_hip(hipGetLastError(), "gemv launch");
}

// Straight-line instances exist for the (WAVES, KP, CNT) shapes the heuristic
// produces at the projection sizes of 7-8B models; everything else runs the
// generic loop.
template <int FMT, int MT, int WAVES, int KP>
static int launch_cnt(const GemvParams &p, hipStream_t stream) {
  if constexpr (TileCfg<MT, KP>::PIPE) {
    if (p.nsteps % WAVES == 0) {
      uint32_t per_wave = p.nsteps / WAVES, cnt = (per_wave + KP - 1) / KP;
      constexpr int TB = TileCfg<MT, KP>::TB;
      if (cnt == 2 && TB >= 2) return launch_one<FMT, MT, WAVES, KP, 2>(p, stream);
      if (cnt == 4 && TB >= 4) return launch_one<FMT, MT, WAVES, KP, 4>(p, stream);
      if constexpr (WAVES >= 4 && KP == 1 && MT == 1) {
        if (cnt == 7) return launch_one<FMT, MT, WAVES, KP, 7>(p, stream);
      }
    }
  }
  return launch_one<FMT, MT, WAVES, KP, 0>(p, stream);
}

template <int FMT, int MT, int KP> static int launch_waves(const GemvParams &p, int waves, hipStream_t stream) {
  switch (waves) {
  case 1: return launch_cnt<FMT, MT, 1, KP>(p, stream);
  case 2: return launch_cnt<FMT, MT, 2, KP>(p, stream);
  case 4: return launch_cnt<FMT, MT, 4, KP>(p, stream);
  default:
    // the wide tiles keep many accumulators per lane: at most 4 waves (256 VGPRs each)
    if constexpr (MT * KP > 16) return launch_cnt<FMT, MT, 4, KP>(p, stream);
    else return launch_cnt<FMT, MT, 8, KP>(p, stream);
  }
}

template <int FMT, int MT> static int launch_kp(const GemvParams &p, int kp, int waves, hipStream_t stream) {
  if constexpr (MT <= 8) {
    if (kp >= 2) return launch_waves<FMT, MT, 2>(p, waves, stream);
  }
  return launch_waves<FMT, MT, 1>(p, waves, stream);
}

struct GemvShape { int kp, waves; };
GemvShape pick_gemv_shape(uint32_t N, uint32_t nsteps, int mt);

template <int FMT> int launch_fmt(GemvParams p, hipStream_t stream) {
  // M <= 8 in one pass; larger M in passes of up to 32 activation rows.
  if (p.M <= 8) {
    int mt = p.M <= 1 ? 1 : p.M <= 2 ? 2 : p.M <= 4 ? 4 : 8;
    GemvShape s = pick_gemv_shape(p.N, p.nsteps, mt);
    switch (mt) {
    case 1: return launch_kp<FMT, 1>(p, s.kp, s.waves, stream);
    case 2: return launch_kp<FMT, 2>(p, s.kp, s.waves, stream);
    case 4: return launch_kp<FMT, 4>(p, s.kp, s.waves, stream);
    default: return launch_kp<FMT, 8>(p, s.kp, s.waves, stream);
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
    GemvShape s = pick_gemv_shape(p.N, p.nsteps, 32);
    if (int rc = launch_kp<FMT, 32>(q, 1, s.waves, stream)) return rc;
  }
  return CUTHIP_OK;
}

}  // namespace cuthip
