// Streaming matmul on Q4_K blocks for a handful of activation rows (5 <= M <= 32):
//   C[m,n] = sum_k A[m,k] * dequant(W)[n,k]
// between the 8-row GEMV (whose matrix-core path spends three quarters of every product on mismatched pieces)
// and the tiled GEMM (which decodes every weight to fp16 through LDS, three vector instructions per weight).
// Supersedes MatMulQ4GemvKPar8.cu / MatMulQ4TiledReg.cu (operators/impl/matmul) at these batch sizes.
//
// Two waves share 16 weight rows and each walks half of the workgroup's K range in steps of one 256-element
// super-block; per 32-element sub-block one v_mfma_f32_16x16x32_f16 multiplies the 16 (or 32) activation rows with
// the 16 weight rows: lane l holds the 8 weights k = 8 (l >> 4) .. + 7 of row l & 15, which are 8 consecutive bytes of
// the block (low nibbles: sub-block 2g, high nibbles: sub-block 2g + 1).  The nibbles are turned into fp16 without a conversion: an integer below 1024 in the low bits
// of a half IS the subnormal integer * 2^-24.  The 6-bit sub-block scale is multiplied in as an integer
// (v_pk_mul_lo_u16: 15 * 63 < 1024, still exact), so all eight sub-blocks of a super-block accumulate in one MFMA
// chain and the fp32 super-block scale d * 2^24 is applied once per step.  The "- dmin * m" term is a second chain on
// the same activation fragments against fragments that hold the 6-bit min of the sub-block in every element:
// sum_k x[k] * m[sub(k)], exact for the same reason.  Products and sums are therefore those of the fp32 reference
// expression (d * sc) * q - dmin * m up to the order of the fp32 additions.
//
// Activations are staged once per workgroup as fp16 rows in LDS (fp32 inputs rounded to nearest even), row pitch
// = range + 16 bytes so that the 16 rows of a fragment read hit different banks; the K range of a workgroup is
// bounded by LDS (132 KB), longer rows are split over workgroups (fp32 partial products, summed by the reduce kernel
// of the two-pass GEMM, which applies the epilogue).  After the staging barrier the loop has no barrier: each lane
// keeps kStreamDepth steps of weight loads in flight in a register ring and waits only for the step it multiplies.
//
// Measured (MI355X, HIP-graph replay, Q4_K 14336 x 4096): 15.0 us at 9-16 rows (two passes of the 8-row GEMV: 25),
// 21 us at 17-32 rows (tiled GEMM with K split: 30); at 8 rows and fewer the 8-row GEMV is the faster one (13 us):
// both spend about 0.05 vector instructions per weight on the unpack, which bounds them well before HBM does.
#include <type_traits>

#include "common.hpp"

namespace cuthip {

int launch_splitk_reduce(const float *partial, uint32_t ksplit, uint32_t M, uint32_t N, void *C, uint32_t strideC, Epilogue epi,
                         int c_f16, hipStream_t stream);

struct StreamParams {
  const uint8_t *W;
  const void *A;
  void *C;
  Epilogue epi;
  uint32_t M, K, N, strideA, strideC, row_bytes;
  int a_f16, c_f16;
  uint32_t nblocks;       // workgroups along N (16 RG weight rows each)
  uint32_t range_steps;   // 256-element steps per K range
  uint32_t ksplit;
  float *partial;         // [ksplit][M][N] when ksplit > 1
};

typedef uint16_t u16x2 __attribute__((ext_vector_type(2)));
typedef __attribute__((address_space(3))) uint8_t lds_u8s;

constexpr int kStreamDepth = 2;   // steps of weight loads in flight per lane (waves have 4 to 8 steps: 15.0 us against 16.5 with four)
constexpr uint32_t kStripBytes = 192 * 16;          // LDS per wave for the blocks of a step
constexpr uint32_t kStreamLdsMax = 132 * 1024;     // staged activations: 16 rows of 4096 (the strips of eight waves take 24 KB more)

// two 4-bit fields at bits 0 and 16 times a 6-bit scale: no carry between the fields, one full-rate 24-bit multiply
__device__ __forceinline__ uint32_t pk_mul_u16(uint32_t a, uint32_t b) { return __umul24(a, b); }
__device__ __forceinline__ half8_t as_frag(uint32_t a, uint32_t b, uint32_t c, uint32_t d) {
  return __builtin_bit_cast(half8_t, u32x4{a, b, c, d});
}

// MT: activation tiles of 16 rows (1 or 2); RG: groups of 16 weight rows per workgroup; KW: waves that share a group,
// each on its own part of the steps.  RG x KW = 8 waves wherever the range is long enough (two waves per SIMD: one
// wave alone cannot hide its own LDS and matrix-core latencies).
template <int MT, int KW, int RG>
__global__ void __launch_bounds__(64 * RG * KW) gemm_stream_q4k_kernel(StreamParams p) {
  extern __shared__ __attribute__((aligned(16))) uint8_t lds[];
  constexpr int D = kStreamDepth, THREADS = 64 * RG * KW;
  const uint32_t split = blockIdx.x / p.nblocks, bid = blockIdx.x - split * p.nblocks;
  const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6, rg = wave % RG, kw = wave / RG;
  const uint32_t s_lo = split * p.range_steps, nsteps = p.K / 256;
  const uint32_t rcnt = min(p.range_steps, nsteps - s_lo);   // steps of this workgroup; the host launches no empty range
  const uint32_t range_k = rcnt * 256, pitch = range_k * 2 + 16;   // bytes per staged activation row
  const uint32_t strip0 = 16 * MT * (p.range_steps * 512 + 16);     // the weight strips lie behind the activations
  const uint32_t sb = rcnt * kw / KW, cnt = rcnt * (kw + 1) / KW - sb;   // this wave's steps: [sb, sb + cnt) of the range

  const uint32_t n = (bid * RG + rg) * 16 + (lane & 15), kq = lane >> 4;

  // The 16 blocks of a step (16 rows x 144 bytes) are fetched as 144 pieces of 16 bytes, piece c = row c / 9, part
  // c % 9, by lanes c, c - 64, c - 128: neighbouring lanes read neighbouring bytes, every cache line is requested
  // once.  (Fetched in the operand layout - 8 bytes per lane, the four lanes of a row 16 lanes apart - every line
  // was requested four times: 17.6 us against 15.7 for 14336 x 4096 at 16 rows.)  The pieces go through a wave-private
  // strip of LDS, from which each lane picks its row's header and its 8 bytes of every 32-byte group.
  const uint8_t *piece[3];
#pragma unroll
  for (int j = 0; j < 3; ++j) {
    const uint32_t c = min((uint32_t)lane + 64u * j, 143u), r = c / 9, part = c - 9 * r;
    piece[j] = p.W + (size_t)min((bid * RG + rg) * 16 + r, p.N - 1) * p.row_bytes + (size_t)(s_lo + sb) * 144 + 16 * part;
  }
  struct Raw { u32x4 c[3]; };
  auto load = [&](Raw &r, uint32_t step) __attribute__((always_inline)) {
#pragma unroll
    for (int j = 0; j < 3; ++j) r.c[j] = ld_u32x4(piece[j] + (size_t)step * 144);
  };

  // activations first (they must not queue behind the weight loads), in batches of kSB 16-byte pieces per thread;
  // the weight ring is requested behind the first batch
  constexpr int kSB = 16;
  const uint32_t cpr = range_k / 8, chunks = p.M * cpr;   // 8-element pieces per row, in all
  const uint32_t k_lo = s_lo * 256;
  u32x4 xa[kSB], xb[kSB];
  auto stage_load = [&](uint32_t base) __attribute__((always_inline)) {
#pragma unroll
    for (int i = 0; i < kSB; ++i) {
      const uint32_t c = min(base + (uint32_t)i * THREADS + (uint32_t)tid, chunks - 1), r = c / cpr, col = c - r * cpr;
      const size_t off = (size_t)r * p.strideA + k_lo + col * 8;
      if (p.a_f16) {
        xa[i] = ld_u32x4(reinterpret_cast<const uint8_t *>(p.A) + off * 2);
      } else {
        xa[i] = ld_u32x4(reinterpret_cast<const uint8_t *>(p.A) + off * 4);
        xb[i] = ld_u32x4(reinterpret_cast<const uint8_t *>(p.A) + off * 4 + 16);
      }
    }
  };
  auto stage_store = [&](uint32_t base) __attribute__((always_inline)) {
#pragma unroll
    for (int i = 0; i < kSB; ++i) {
      const uint32_t c = base + (uint32_t)i * THREADS + (uint32_t)tid;
      if (c < chunks) {
        const uint32_t r = c / cpr, col = c - r * cpr;
        u32x4 o = xa[i];
        if (!p.a_f16) {
          const f32x4 lo = __builtin_bit_cast(f32x4, xa[i]), hi = __builtin_bit_cast(f32x4, xb[i]);
          const half8_t h{(half_t)lo.x, (half_t)lo.y, (half_t)lo.z, (half_t)lo.w, (half_t)hi.x, (half_t)hi.y, (half_t)hi.z, (half_t)hi.w};
          o = __builtin_bit_cast(u32x4, h);
        }
        *reinterpret_cast<u32x4 *>(lds + (size_t)r * pitch + col * 16) = o;
      }
    }
  };
  stage_load(0);
  Raw buf[D];
#pragma unroll
  for (int i = 0; i < D; ++i) {
    load(buf[i], min((uint32_t)i, cnt ? cnt - 1 : 0u));
    __builtin_amdgcn_sched_barrier(0);   // issue order = ring order: step i waits for its own loads only
  }
  stage_store(0);
  for (uint32_t base = kSB * THREADS; base < chunks; base += kSB * THREADS) {
    stage_load(base);
    stage_store(base);
  }
  __syncthreads();

  f32x4 acc[MT];
#pragma unroll
  for (int t = 0; t < MT; ++t) acc[t] = f32x4{0, 0, 0, 0};
  // fragment of activation tile t, sub-block s of a step: row 16 t + (lane & 15), k = 32 s + 8 kq .. + 7; rows at
  // and beyond M hold whatever the LDS held: their products land in accumulator rows that are never stored
  const lds_u8s *xbase = (const lds_u8s *)(lds) + (size_t)(lane & 15) * pitch + kq * 16;

  // wave-private strip: 144 pieces + the 48 duplicates that the lanes past piece 143 hold (written to the end, never read)
  lds_u8s *strip = (lds_u8s *)(lds) + strip0 + (size_t)wave * kStripBytes;
  struct Blk { u32x4 hdr; u32x2 q[4]; };   // what a lane multiplies in a step: its row's header, 8 bytes of each group
  // pieces of a step -> strip -> the lane's operands (same wave, LDS in order: the strip's earlier reads are done);
  // issuing this a step ahead of the products measured no different
  auto deliver = [&](const Raw &raw, Blk &r) __attribute__((always_inline)) {
    __builtin_amdgcn_wave_barrier();
#pragma unroll
    for (int j = 0; j < 3; ++j)
      *reinterpret_cast<__attribute__((address_space(3))) u32x4 *>(strip + ((size_t)lane + 64 * j) * 16) = raw.c[j];
    __builtin_amdgcn_wave_barrier();
    const lds_u8s *blk = strip + (size_t)(lane & 15) * 144;
    r.hdr = *reinterpret_cast<const __attribute__((address_space(3))) u32x4 *>(blk);
#pragma unroll
    for (int g = 0; g < 4; ++g) r.q[g] = *reinterpret_cast<const __attribute__((address_space(3))) u32x2 *>(blk + 16 + 32 * g + 8 * kq);
    __builtin_amdgcn_wave_barrier();
  };
  auto do_step = [&](const Blk &r, uint32_t step) __attribute__((always_inline)) {
    const float d = f16bits_to_f32(r.hdr.x & 0xFFFF) * 16777216.0f, dmin = f16bits_to_f32(r.hdr.x >> 16) * 16777216.0f;
    uint32_t sc4[2], m4[2];
    q4k_scales(r.hdr.y, r.hdr.z, r.hdr.w, sc4[0], sc4[1], m4[0], m4[1]);
    f32x4 t_main[MT], t_min[MT];
#pragma unroll
    for (int t = 0; t < MT; ++t) t_main[t] = t_min[t] = f32x4{0, 0, 0, 0};
    const lds_u8s *xs = xbase + (size_t)(sb + step) * 512;
#pragma unroll
    for (int g = 0; g < 4; ++g) {
      // (scale | scale << 16) and (min | min << 16) of sub-blocks 2g and 2g + 1: byte (2g) & 3 / (2g + 1) & 3 of dword g >> 1
      const uint32_t scw = sc4[g >> 1], mw = m4[g >> 1];
      const uint32_t sel0 = (g & 1) ? 0x0c060c06u : 0x0c040c04u, sel1 = (g & 1) ? 0x0c070c07u : 0x0c050c05u;
      const uint32_t sc0 = (scw >> (16 * (g & 1))) & 0xFFu, sc1 = (scw >> (16 * (g & 1) + 8)) & 0xFFu;
      const uint32_t mn0 = __builtin_amdgcn_perm(mw, 0, sel0), mn1 = __builtin_amdgcn_perm(mw, 0, sel1);
      // bytes b0..b3 of a dword -> halves (b0, b1) and (b2, b3), so that the 8 weights stay in the order of k
      const uint32_t w0 = r.q[g].x, w1 = r.q[g].y;
      const uint32_t p0 = __builtin_amdgcn_perm(w0, 0, 0x0c050c04u), p1 = __builtin_amdgcn_perm(w0, 0, 0x0c070c06u);
      const uint32_t p2 = __builtin_amdgcn_perm(w1, 0, 0x0c050c04u), p3 = __builtin_amdgcn_perm(w1, 0, 0x0c070c06u);
      constexpr uint32_t kNib = 0x000F000Fu;
      const half8_t lo = as_frag(pk_mul_u16(p0 & kNib, sc0), pk_mul_u16(p1 & kNib, sc0), pk_mul_u16(p2 & kNib, sc0),
                                 pk_mul_u16(p3 & kNib, sc0));
      const half8_t hi = as_frag(pk_mul_u16((p0 >> 4) & kNib, sc1), pk_mul_u16((p1 >> 4) & kNib, sc1),
                                 pk_mul_u16((p2 >> 4) & kNib, sc1), pk_mul_u16((p3 >> 4) & kNib, sc1));
      const half8_t mlo = as_frag(mn0, mn0, mn0, mn0), mhi = as_frag(mn1, mn1, mn1, mn1);
#pragma unroll
      for (int t = 0; t < MT; ++t) {
        const lds_u8s *xt = xs + (size_t)t * 16 * pitch + g * 128;
        const half8_t x0 = *reinterpret_cast<const __attribute__((address_space(3))) half8_t *>(xt);
        const half8_t x1 = *reinterpret_cast<const __attribute__((address_space(3))) half8_t *>(xt + 64);
        t_main[t] = __builtin_amdgcn_mfma_f32_16x16x32_f16(x0, lo, t_main[t], 0, 0, 0);
        t_min[t] = __builtin_amdgcn_mfma_f32_16x16x32_f16(x0, mlo, t_min[t], 0, 0, 0);
        t_main[t] = __builtin_amdgcn_mfma_f32_16x16x32_f16(x1, hi, t_main[t], 0, 0, 0);
        t_min[t] = __builtin_amdgcn_mfma_f32_16x16x32_f16(x1, mhi, t_min[t], 0, 0, 0);
      }
    }
#pragma unroll
    for (int t = 0; t < MT; ++t)
#pragma unroll
      for (int e = 0; e < 4; ++e) {
        acc[t][e] = fmaf(d, t_main[t][e], acc[t][e]);
        acc[t][e] = fmaf(-dmin, t_min[t][e], acc[t][e]);
      }
  };

  // Ring slot i % D holds the pieces of step i.  Every refill is issued, past the end of the range at the range's
  // last step again (a few redundant loads of valid memory): with no load under a condition the compiler counts the
  // loads in flight exactly and every step waits for its own pieces only, also in ranges shorter than 2 D steps.
  const uint32_t last = cnt ? cnt - 1 : 0u;
  for (uint32_t i0 = 0; i0 < cnt; i0 += D) {
#pragma unroll
    for (int u = 0; u < D; ++u) {
      const uint32_t i = i0 + u;
      if (i < cnt) {           // uniform; no global load inside
        Blk blk;
        deliver(buf[u], blk);
        do_step(blk, i);
      }
      load(buf[u], min(i + D, last));
      __builtin_amdgcn_sched_barrier(0);
    }
  }
  // the K parts of a row group meet in LDS (the staged activations are no longer needed)
  if constexpr (KW > 1) {
    __syncthreads();
    // [KW - 1][RG row groups][MT * 4 registers][64 lanes]
    float *red = reinterpret_cast<float *>(lds) + ((size_t)(kw > 0 ? kw - 1 : 0) * RG + rg) * 64 * MT * 4 + lane;
    if (kw > 0) {
#pragma unroll
      for (int t = 0; t < MT; ++t)
#pragma unroll
        for (int e = 0; e < 4; ++e) red[(t * 4 + e) * 64] = acc[t][e];
    }
    __syncthreads();
    if (kw > 0) return;
#pragma unroll
    for (int w = 1; w < KW; ++w)
#pragma unroll
      for (int t = 0; t < MT; ++t)
#pragma unroll
        for (int e = 0; e < 4; ++e) acc[t][e] += red[((size_t)(w - 1) * RG * 64 * MT * 4) + (t * 4 + e) * 64];
  }
  // accumulator register e of lane l, tile t: row 16 t + 4 (l >> 4) + e, column (weight row) n
  if (n < p.N) {
#pragma unroll
    for (int t = 0; t < MT; ++t)
#pragma unroll
      for (int e = 0; e < 4; ++e) {
        const uint32_t m = 16 * t + 4 * kq + e;
        if (m < p.M) {
          if (p.ksplit > 1) p.partial[((size_t)split * p.M + m) * p.N + n] = acc[t][e];
          else store_out(p.C, p.epi, p.c_f16, (size_t)m * p.strideC + n, acc[t][e]);
        }
      }
  }
}

// K ranges of the streaming kernel: as few as LDS allows (one range of up to kStreamLdsMax bytes of staged
// activations), more while the grid has fewer workgroups than CUs and a range keeps at least 8 steps
// (and the scratch memory holds the partial products of twice as many)
// Weight rows per workgroup: 64 (four row groups, two waves each), or with two activation tiles 128 (eight row groups
// of one wave: half as many workgroups stage the activations; 14336 x 4096 at 32 rows 21 us against 26) wherever that
// still leaves a workgroup for every second CU (4096 x 4096: 18 us against 14 otherwise)
static uint32_t stream_block_rows(uint32_t M, uint32_t K, uint32_t N) {
  if (M <= 16) return 64;
  const uint32_t ks_lds = (K / 256 + 7) / 8;   // ranges of at most eight steps with 32 staged rows
  return (N + 127) / 128 * ks_lds >= 128 ? 128 : 64;
}
static void stream_layout(uint32_t M, uint32_t K, uint32_t N, size_t scratch_bytes, uint32_t *range_steps, uint32_t *ksplit) {
  const uint32_t mt = (M + 15) / 16, nsteps = K / 256, nblocks = (N + stream_block_rows(M, K, N) - 1) / stream_block_rows(M, K, N);
  const uint32_t max_steps = (kStreamLdsMax / (16 * mt) - 16) / 512;
  uint32_t ks = (nsteps + max_steps - 1) / max_steps;
  while (ks < 16 && nblocks * ks < 192 && nsteps / (2 * ks) >= 8 && scratch_bytes >= (size_t)2 * ks * M * N * sizeof(float)) ks *= 2;
  *range_steps = (nsteps + ks - 1) / ks;
  *ksplit = (nsteps + *range_steps - 1) / *range_steps;
}

bool stream_gemm_fits(int fmt, uint32_t M, uint32_t K, uint32_t N, uint32_t strideA, int a_f16, const void *A) {
  const size_t asz = a_f16 ? 2 : 4;
  return fmt == CUTHIP_Q4_K && M >= 1 && M <= 32 && K % 256 == 0 && K >= 256 && (uintptr_t)A % 16 == 0 && (strideA * asz) % 16 == 0 &&
         (uint64_t)M * N < 0x7FFFFFFFull;
}
// bytes of scratch the launch cannot do without (0: the K range of a workgroup may cover all of K)
size_t stream_gemm_scratch(uint32_t M, uint32_t K, uint32_t N) {
  uint32_t rs, ks;
  stream_layout(M, K, N, 0, &rs, &ks);
  return ks > 1 ? (size_t)ks * M * N * sizeof(float) : 0;
}

int launch_stream_gemm(const void *W, const void *A, int a_f16, void *C, int c_f16, uint32_t M, uint32_t K, uint32_t N,
                       uint32_t strideA, uint32_t strideC, Epilogue epi, void *scratch, size_t scratch_bytes, hipStream_t stream) {
  StreamParams p;
  p.W = reinterpret_cast<const uint8_t *>(W);
  p.A = A;
  p.C = C;
  p.epi = epi;
  p.M = M; p.K = K; p.N = N; p.strideA = strideA; p.strideC = strideC;
  p.row_bytes = K / 256 * 144;
  p.a_f16 = a_f16; p.c_f16 = c_f16;
  const uint32_t block_rows = stream_block_rows(M, K, N);
  p.nblocks = (N + block_rows - 1) / block_rows;
  if (!scratch || (uintptr_t)scratch % 16 != 0) scratch_bytes = 0;
  stream_layout(M, K, N, scratch_bytes, &p.range_steps, &p.ksplit);
  p.partial = reinterpret_cast<float *>(scratch);
  if (p.ksplit > 1 && scratch_bytes < (size_t)p.ksplit * M * N * sizeof(float)) {
    set_error("streaming matmul: K = %u at %u rows needs %zu bytes of scratch for its %u K ranges", K, M,
              (size_t)p.ksplit * M * N * sizeof(float), p.ksplit);
    return CUTHIP_ERR_INVALID;
  }
  const uint32_t mt = (M + 15) / 16;
  const size_t lds = (size_t)16 * mt * ((size_t)p.range_steps * 512 + 16) + 8 * kStripBytes;
  // four row groups: two waves each once a wave keeps at least two steps
  const bool two = block_rows == 64 && p.range_steps >= 4;
  auto kern = block_rows == 128 ? gemm_stream_q4k_kernel<2, 1, 8>
              : mt == 1 ? (two ? gemm_stream_q4k_kernel<1, 2, 4> : gemm_stream_q4k_kernel<1, 1, 4>)
                        : (two ? gemm_stream_q4k_kernel<2, 2, 4> : gemm_stream_q4k_kernel<2, 1, 4>);
  const uint32_t threads = block_rows == 128 || two ? 512 : 256;
  if (lds > 64 * 1024) {
    if (int rc = check_hip(hipFuncSetAttribute(reinterpret_cast<const void *>(kern), hipFuncAttributeMaxDynamicSharedMemorySize,
                                               (int)lds),
                           "hipFuncSetAttribute"))
      return rc;
  }
  hipLaunchKernelGGL(kern, dim3(p.nblocks * p.ksplit), dim3(threads), lds, stream, p);
  if (int rc = check_hip(hipGetLastError(), "streaming matmul launch")) return rc;
  if (p.ksplit == 1) return CUTHIP_OK;
  return launch_splitk_reduce(p.partial, p.ksplit, M, N, C, strideC, epi, c_f16, stream);
}

}  // namespace cuthip
