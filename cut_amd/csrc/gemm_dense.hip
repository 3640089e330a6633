// Two-pass prefill matmul for gfx950 (variant MatMulGgufDequantGemm):
//   pass 1  dequantizes the GGUF weight tensor once into an fp16 [N, K] workspace
//           (the dequant kernel of this library, HBM-bound: ~25 us for 14336 x 4096),
//   pass 2  C[m,n] = sum_k A[m,k] * W16[n,k] as a dense fp16 MFMA GEMM.
// The single-launch GEMM (gemm.hip) decodes every weight once per 256 rows of
// activations, i.e. M/256 times; for M in the thousands the decode ALU work, not
// the MFMA, bounds it.  Here each weight is decoded exactly once and the GEMM's
// inner loop contains nothing but MFMAs, LDS fragment reads and copy instructions.
// Supersedes MatMulQ{4,8}CoopMatTiled.cu (operators/impl/matmul) for large M.
//
// The GEMM (two kernels on the same tiles, loads and LDS image: gemm_dense16_kernel on 16 x 16 x 32 MFMAs, the one that
// runs, and gemm_dense_kernel on 32 x 32 x 16 MFMAs, kept behind CUT_HIP_DENSE_MFMA16=0 for comparison; what follows
// describes the latter, the former says where it differs): a workgroup of four waves owns a BM x BN tile of C,
// each wave a sub-tile in fp32 accumulators (AGPRs), K walked in slices
// of 64.  Both operands go global -> LDS with global_load_lds_dwordx4 (no VGPR
// round trip): one instruction fills 8 tile rows x 128 bytes = 1 KB of LDS, lane i
// at byte 16 i; the lane fetches the chunk of its row that belongs at that position
// of an XOR-swizzled image (chunk c of row r sits at c ^ ((r >> 1) & 7)), so that the
// MFMA fragment reads (lane l: row l & 31, chunk 2 s + (l >> 5) of k-step s) spread
// over all 64 banks.  Two LDS stages; the
// loads of slice t+1 are in flight while slice t is multiplied.
//
// Issue order is explicit.  A wave has the SIMD to itself (one wave per SIMD), so a
// burst of memory instructions stalls its MFMA stream: 16 loads in a row cost ~1000
// cycles per slice, 8 LDS reads in a row ~90.  Every MFMA is therefore followed by
// at most one LDS read and one global load, the loads spread over the slice at the
// rate the texture path sustains (64 B/clk per CU), and the fragment reads of k-step
// s+1 are issued under the MFMAs of k-step s.  The LDS reads are inline asm with
// hand-placed s_waitcnt, because the compiler's own counter tracking waits for all
// outstanding LDS-direct loads before any LDS read.  The last k-step of a slice is
// multiplied after the barrier, under the first fragment reads of the next slice.
//
// Numerics: weights rounded to fp16 once (2^-11 relative), fp32 activations rounded
// to fp16 once, fp32 accumulation: the same error budget as the single-launch GEMM.
#include <stdio.h>
#include <stdlib.h>

#include "common.hpp"
#include "gemm_store.hpp"

namespace cuthip {

int launch_dequant_any(int fmt, const void *blocks, void *out, int out_dtype, uint32_t rows, uint32_t cols,
                       uint32_t out_stride, hipStream_t stream);

typedef _Float16 half8v __attribute__((ext_vector_type(8)));
typedef __attribute__((address_space(3))) uint8_t lds_u8;

struct DenseParams {
  const uint8_t *A, *W;  // fp16 [M, strideA], fp16 [N, K]
  void *C;
  Epilogue epi;
  uint32_t M, N, K, strideA, strideC, mtiles, ntiles;
  int c_f16;
  uint32_t ksplit, kper;  // K is cut into ksplit ranges of kper (a multiple of 128); a workgroup multiplies one range
  float *partial;         // ksplit > 1: fp32 [ksplit][M][N] partial products instead of C
  // L2 warm-up: in every slice a workgroup touches, pf_dist slices ahead, every pf_wsplit-th row of its weight panel
  // and every pf_asplit-th row of its activation tile; the workgroups that run beside it on the same XCD and share the
  // panel (the tile) touch the other rows.
  uint32_t pf_dist, pf_wsplit, pf_asplit;
  int vec_store;          // C (and a binary epilogue's operand) allow 16-byte accesses
};

[[maybe_unused]] constexpr int kDBK = 64;   // K elements per LDS stage

// WM: waves along M (4 / WM along N); a wave owns a (BM / WM) x (BN / WN) sub-tile
template <int BM, int BN, int WM = 2>
__global__ void __launch_bounds__(256, 1) gemm_dense_kernel(DenseParams p) {
#if defined(__HIP_DEVICE_COMPILE__)  // LDS address-space casts and AMDGPU inline asm: the host pass only needs the stub
  constexpr int WN = 4 / WM;
  constexpr int MI = BM / (32 * WM), NJ = BN / (32 * WN);  // 32 x 32 MFMA tiles per wave: MI x NJ
  constexpr int NM = MI * NJ;                  // MFMAs per k-step of 16
  constexpr int NLA = BM / 32, NL = (BM + BN) / 32;  // LDS-direct loads per wave per slice (A, total)
  constexpr int NPF = 2;                     // L2 warm-up loads per wave per slice: 4 waves x 64 lanes x NPF lines
  // one load every LSTEP-th MFMA slot of the slice, the warm-up loads in its last NPF slots
#ifndef CUTHIP_LSTEP_CAP
#define CUTHIP_LSTEP_CAP 3
#endif
  constexpr int LSTEP = (4 * NM - NPF - 1) / (NL - 1) < CUTHIP_LSTEP_CAP ? (4 * NM - NPF - 1) / (NL - 1) : CUTHIP_LSTEP_CAP;
  static_assert((NJ == 4 && (MI == 4 || MI == 2)) || (NJ == 7 && MI == 2), "tile shape");
  static_assert((BM + BN) * 128 * 2 <= 160 * 1024, "two LDS stages");
  static_assert(LSTEP >= 1 && (NL - 1) * LSTEP < 4 * NM - NPF, "the loads of a slice precede its warm-up loads");
  static_assert(4 * stripe_floats<NJ>() * 4 <= (BM + BN) * 128 * 2, "the output staging reuses the operand stages");
  __shared__ __attribute__((aligned(1024))) uint8_t lds[(BM + BN) * 128 * 2];
  uint8_t *const sA0 = lds, *const sA1 = lds + BM * 128, *const sB0 = lds + BM * 256, *const sB1 = lds + BM * 256 + BN * 128;
  __shared__ uint32_t pf_sink[4 * 64];       // where they land; never read

  // XCD-aware tile order: ids id, id+8, id+16, ... share an XCD and its L2; give
  // them the M-tiles of the same weight panels.
  // (the quotients come out of the vector ALU: readfirstlane moves what depends on them back to SGPRs, where the
  // scalar-base loads below need their addresses)
  const uint32_t tiles = p.mtiles * p.ntiles, split = __builtin_amdgcn_readfirstlane(blockIdx.x / tiles);
  uint32_t id = blockIdx.x - split * tiles, mt, nt, aphase = 0;
  if (p.ntiles % 8 == 0) {
    uint32_t xcd = id & 7, slot = id >> 3;
    nt = (slot / p.mtiles) * 8 + xcd;
    mt = slot % p.mtiles;
    aphase = (slot / p.mtiles) % p.pf_asplit;
  } else {
    nt = id / p.mtiles;
    mt = id % p.mtiles;
  }
  mt = __builtin_amdgcn_readfirstlane(mt);
  nt = __builtin_amdgcn_readfirstlane(nt);
  aphase = __builtin_amdgcn_readfirstlane(aphase);
  const uint32_t m0 = mt * BM, n0 = nt * BN;
  const int tid = threadIdx.x, lane = tid & 63, wave = __builtin_amdgcn_readfirstlane(tid >> 6);   // wave: in an SGPR
  const int wm = wave / WN, wn = wave % WN;

  // copy assignment: load v of wave w fills the 8-row group 4 v + w of its tile
  uint32_t aoff[NLA], boff[BN / 32];
  // tile row r keeps its 16-byte chunk c at position c ^ ((r >> 1) & 7): the 16 lanes the LDS serves per cycle
  // (16 consecutive rows, one chunk index) then cover all 64 banks.  For the row 8 g + (lane >> 3) of 8-row group
  // g = 4 v + wave that key is (4 (wave & 1) + (lane >> 4)) & 7, the same for every v.
  const uint32_t chunk = ((lane & 7) ^ ((4 * (wave & 1) + (lane >> 4)) & 7)) * 16;
#pragma unroll
  for (int v = 0; v < NLA; ++v) {
    uint32_t r = min(m0 + 8 * (4 * v + wave) + (lane >> 3), p.M - 1);
    aoff[v] = r * p.strideA * 2 + chunk;
  }
#pragma unroll
  for (int v = 0; v < BN / 32; ++v) {
    uint32_t r = min(n0 + 8 * (4 * v + wave) + (lane >> 3), p.N - 1);
    boff[v] = r * p.K * 2 + chunk;
  }
  // the lambdas below capture plain locals, never a field of p: a captured parameter block is copied to scratch memory
  const uint8_t *const gA = p.A, *const gW = p.W;
  const uint32_t pf_dist = p.pf_dist, Mrows = p.M, Ncols = p.N;
  auto load_one = [&](int l, uint8_t *na, uint8_t *nb, uint32_t k0) {
    // As text, in the form scalar base + 32-bit lane offset with the LDS address moved to M0 from an SGPR: through
    // the builtin every load costs a 64-bit vector add and a v_readfirstlane between the MFMAs.  M0 is not on the
    // clobber list (the compiler reserves it and says so); every instruction of this kernel that reads M0 sits in a
    // statement like this one, behind its own s_mov.
    const uint8_t *g = (l < NLA ? gA : gW) + (size_t)k0 * 2;
    const uint32_t voff = l < NLA ? aoff[l] : boff[l - NLA];
    const uint32_t dst = (uint32_t)(uintptr_t)(lds_u8 *)(l < NLA ? na : nb) + (4 * (l < NLA ? l : l - NLA) + wave) * 1024;
    asm volatile("s_mov_b32 m0, %2\n\ts_nop 0\n\tglobal_load_lds_dwordx4 %0, %1" ::"v"(voff), "s"(g), "s"(dst) : "memory");
  };

  // Line q = 256 i + tid of the warm-up: the first ceil(BN / wsplit) are rows of the weight panel, the next
  // ceil(BM / asplit) rows of the activation tile; what is left over repeats the first line of the panel.
  const uint8_t *pfp[NPF];
  {
    const uint32_t nw = (BN + p.pf_wsplit - 1) / p.pf_wsplit, na = (BM + p.pf_asplit - 1) / p.pf_asplit;
#pragma unroll
    for (int i = 0; i < NPF; ++i) {
      const uint32_t q = 256 * i + tid;
      uint32_t wr = mt % p.pf_wsplit + (q < nw ? q : 0) * p.pf_wsplit, ar = aphase + (q - nw) * p.pf_asplit;
      const bool is_a = q >= nw && q - nw < na && ar < BM;
      wr = min(n0 + min(wr, (uint32_t)BN - 1), p.N - 1);
      ar = min(m0 + ar, p.M - 1);
      pfp[i] = is_a ? p.A + (size_t)ar * p.strideA * 2 : p.W + (size_t)wr * p.K * 2;
    }
  }
  auto warm_one = [&](int i, uint32_t k0) {
    const uint8_t *g = pfp[i] + (size_t)k0 * 2;
    const uint32_t dst = (uint32_t)(uintptr_t)(lds_u8 *)(reinterpret_cast<uint8_t *>(pf_sink)) + wave * 256;
    asm volatile("s_mov_b32 m0, %1\n\ts_nop 0\n\tglobal_load_lds_dword %0, off" ::"v"(g), "s"(dst) : "memory");
  };

  f32x16 acc[MI][NJ];
#pragma unroll
  for (int i = 0; i < MI; ++i)
#pragma unroll
    for (int j = 0; j < NJ; ++j) acc[i][j] = f32x16{0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0};

  const uint32_t arow = (wm * (BM / WM) + (lane & 31)) * 128, brow = (wn * (BN / WN) + (lane & 31)) * 128;
  uint32_t xs[4];
#pragma unroll
  for (int s = 0; s < 4; ++s) xs[s] = ((2 * s + (lane >> 5)) ^ ((lane >> 1) & 7)) * 16;

  half8v fa[2][MI], fb[2][NJ];
  // Waits until at most n of this wave's LDS reads are outstanding.  The fragment registers then pass through an
  // empty statement, so that no MFMA that uses them can be scheduled above the wait, and so that any register copy the
  // allocator makes for them is placed behind the wait too: the fragment reads are text the compiler cannot see into,
  // and a copy in front of the wait would read registers the LDS has not written yet.
#define CUTHIP_WAIT_FRAGS(f, n)                                                                                  \
  asm volatile("s_waitcnt lgkmcnt(" #n ")" ::: "memory");                                                          \
  __builtin_amdgcn_sched_barrier(0);                                                                               \
  asm volatile(""                                                                                                  \
               : "+v"(fa[f][0]), "+v"(fa[f][1]), "+v"(fa[f][MI - 2]), "+v"(fa[f][MI - 1]), "+v"(fb[f][0]),         \
                 "+v"(fb[f][1]), "+v"(fb[f][2]), "+v"(fb[f][3]), "+v"(fb[f][NJ - 3]), "+v"(fb[f][NJ - 2]),           \
                 "+v"(fb[f][NJ - 1]))

  // The NM MFMAs of one k-step on fragment set f.  After MFMA idx: the idx-th fragment read of k-step s of
  // (sa, sb) into the other set, and, in every LSTEP-th slot of the slice (g = position of the group in the
  // slice), one load of the next slice (k0) into (na, nb).
  auto group = [&](int g, int f, const uint8_t *sa, const uint8_t *sb, int s, uint8_t *na, uint8_t *nb, uint32_t k0,
                   uint32_t kpf) {
    const uint32_t pa = (uint32_t)(uintptr_t)(lds_u8 *)(sa) + arow + xs[s];
    const uint32_t pb = (uint32_t)(uintptr_t)(lds_u8 *)(sb) + brow + xs[s];
#pragma unroll
    for (int idx = 0; idx < NM; ++idx) {
      const int i = idx / NJ, j = idx % NJ;
      acc[i][j] = __builtin_amdgcn_mfma_f32_32x32x16_f16(fa[f][i], fb[f][j], acc[i][j], 0, 0, 0);
      if (idx < MI)
        asm volatile("ds_read_b128 %0, %1 offset:%2" : "=v"(fa[f ^ 1][idx]) : "v"(pa), "n"(idx * 4096) : "memory");
      else if (idx < MI + NJ)
        asm volatile("ds_read_b128 %0, %1 offset:%2" : "=v"(fb[f ^ 1][idx - MI]) : "v"(pb), "n"((idx - MI) * 4096) : "memory");
      const int q = g * NM + idx;
      if (q % LSTEP == 0 && q / LSTEP < NL) load_one(q / LSTEP, na, nb, k0);
      if (g == 3 && idx >= NM - NPF) warm_one(idx - (NM - NPF), kpf);   // younger than every load of the slice
      __builtin_amdgcn_sched_barrier(0);
    }
  };

  const uint32_t kbeg = __builtin_amdgcn_readfirstlane(split * p.kper), nsl = p.kper / kDBK, klast = kbeg + p.kper - kDBK;
  // One slice, entered right after a barrier with nothing in flight.  Set 1 holds the fragments of the previous
  // slice's last k-step; its MFMAs run under the first fragment reads of this slice.  The loads of the slice
  // after the last one re-read the last slice (never used) instead of branching around the MFMAs.
  auto slice = [&](uint8_t *sa, uint8_t *sb, uint8_t *na, uint8_t *nb, uint32_t t) {
    const uint32_t k0 = min(kbeg + (t + 1) * kDBK, klast), kpf = min(kbeg + (t + pf_dist) * kDBK, klast);
    group(0, 1, sa, sb, 0, na, nb, k0, kpf);
    CUTHIP_WAIT_FRAGS(0, 0);
    group(1, 0, sa, sb, 1, na, nb, k0, kpf);
    CUTHIP_WAIT_FRAGS(1, 0);
    group(2, 1, sa, sb, 2, na, nb, k0, kpf);
    CUTHIP_WAIT_FRAGS(0, 0);
    group(3, 0, sa, sb, 3, na, nb, k0, kpf);
    // The next slice has landed in (na, nb).  The warm-up loads of this slice stay in flight (memory returns in order
    // and they are the youngest); those of the slice before had this whole slice to come back.
    asm volatile("s_waitcnt vmcnt(%0)" ::"n"(NPF) : "memory");
    CUTHIP_WAIT_FRAGS(1, 0);                           // and this wave is done reading (sa, sb)
    __builtin_amdgcn_sched_barrier(0);
    asm volatile("s_barrier" ::: "memory");   // as text: before __syncthreads() or the builtin the compiler waits for every load in flight
    __builtin_amdgcn_sched_barrier(0);
  };

  for (uint32_t d = 1; d < p.pf_dist; ++d)
#pragma unroll
    for (int i = 0; i < NPF; ++i) warm_one(i, min(kbeg + d * kDBK, klast));
#pragma unroll
  for (int l = 0; l < NL; ++l) load_one(l, sA0, sB0, kbeg);
#pragma unroll
  for (int i = 0; i < MI; ++i) fa[1][i] = half8v{0, 0, 0, 0, 0, 0, 0, 0};
#pragma unroll
  for (int j = 0; j < NJ; ++j) fb[1][j] = half8v{0, 0, 0, 0, 0, 0, 0, 0};
  asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
  __syncthreads();
  for (uint32_t t = 0; t < nsl; t += 2) {  // nsl is even (host check)
    slice(sA0, sB0, sA1, sB1, t);
    slice(sA1, sB1, sA0, sB0, t + 1);
  }
#pragma unroll
  for (int i = 0; i < MI; ++i)
#pragma unroll
    for (int j = 0; j < NJ; ++j)
      acc[i][j] = __builtin_amdgcn_mfma_f32_32x32x16_f16(fa[1][i], fb[1][j], acc[i][j], 0, 0, 0);
  asm volatile("s_waitcnt vmcnt(0)" ::: "memory");   // the last warm-up loads: nothing may land after the exit
#undef CUTHIP_WAIT_FRAGS

  // C tile through LDS, a 32-row stripe of the wave's sub-tile at a time.  The operand stages are free once every
  // wave has its last loads back and has read its last fragments.
  __syncthreads();
  lds_f32 *stage = (lds_f32 *)(lds_u8 *)(lds) + wave * stripe_floats<NJ>();
  void *cbase = p.C;
  uint32_t ldc = p.strideC;
  int c_f16 = p.c_f16;
  Epilogue epi = p.epi;
  if (p.ksplit > 1) {   // fp32 partial products [ksplit][M][N]; the reduce kernel applies the epilogue
    cbase = p.partial + (size_t)split * p.M * p.N;
    ldc = p.N;
    c_f16 = 0;
    epi.kind = CUTHIP_EPI_NONE;
  }
  const bool vec = p.ksplit > 1 ? p.N % 4 == 0 : p.vec_store != 0;
  // the common cases get the short store loops: no operator, or the residual add
  const int fast = !vec ? 0 : (!c_f16 ? (epi.kind == CUTHIP_EPI_NONE ? 3 : 0)
                               : epi.kind == CUTHIP_EPI_NONE ? 1
                               : (epi.kind == CUTHIP_EPI_BINARY && epi.op == CUTHIP_BINARY_ADD) ? 2 : 0);
  static_for<MI>([&](auto ii) __attribute__((always_inline)) {
    constexpr int i = decltype(ii)::value;
    static_for<NJ>([&](auto jj) __attribute__((always_inline)) {
      constexpr int j = decltype(jj)::value;
      stage_tile32<NJ>(stage, j, acc[i][j], lane);
    });
    const uint32_t r0 = m0 + wm * (BM / WM) + 32 * i, c0 = n0 + wn * (BN / WN);
    if (fast == 1) store_staged32<NJ, 1>(stage, r0, c0, Mrows, Ncols, cbase, ldc, c_f16, epi, vec, lane);
    else if (fast == 2) store_staged32<NJ, 2>(stage, r0, c0, Mrows, Ncols, cbase, ldc, c_f16, epi, vec, lane);
    else if (fast == 3) store_staged32<NJ, 3>(stage, r0, c0, Mrows, Ncols, cbase, ldc, c_f16, epi, vec, lane);
    else store_staged32<NJ, 0>(stage, r0, c0, Mrows, Ncols, cbase, ldc, c_f16, epi, vec, lane);
  });
#endif
}

// ---- the same GEMM on v_mfma_f32_16x16x32_f16 ------------------------------------------------------------------------
// Same tiles, loads, LDS image and stages as gemm_dense_kernel; the products are 16 x 16 x 32 MFMAs (4 passes) instead
// of 32 x 32 x 16 (8 passes).  The part throttles its clock under matrix-core load, less so under this instruction (a
// loop of nothing but MFMAs on random fp16 data: 1.55-1.71 PFLOP/s against 1.47-1.60), and the vendor's kernel, which
// uses it, runs at 1.83 GHz where gemm_dense_kernel runs at 1.5-1.6.
// A wave's sub-tile is MI x NJ tiles of 16 x 16.  Per 32-wide k-step it walks the B fragments j = 0 .. NJ-1 and
// multiplies each with the MI A fragments of the step; B fragments are read kAhead fragments ahead into a ring of
// eight, A fragments a step ahead into the other half of a double buffer.  The fragment reads are ordinary LDS loads
// (the compiler places the exact s_waitcnt lgkmcnt before each first use; it knows nothing of the LDS-direct loads,
// which are text, so it adds no wait for them).  All reads of a slice have been issued kTail + 2 groups before its end;
// the wave then waits for them, for its loads of the next slice and for the barrier, and multiplies the last kTail
// groups from registers behind the barrier, under the first reads of the next slice.
typedef __attribute__((address_space(3))) half8v lds_half8v;

template <int BM, int BN, int WM = 2>
__global__ void __launch_bounds__(256, 1) gemm_dense16_kernel(DenseParams p) {
#if defined(__HIP_DEVICE_COMPILE__)
  constexpr int WN = 4 / WM;
  constexpr int MI = BM / (16 * WM), NJ = BN / (16 * WN);   // 16 x 16 MFMA tiles per wave
  constexpr int NB = 2 * NJ;                                 // B fragments per slice (two k-steps of 32)
  // B fragments read ahead; groups multiplied behind the barrier (2..6 ahead and tails of 2..4 measured within noise)
  constexpr int kAhead = 6, kTail = 3;
  constexpr int NLA = BM / 32, NL = (BM + BN) / 32;          // LDS-direct loads per wave per slice (A, total)
  constexpr int NPF = 2;
  constexpr int LFIRST = 0, LLAST = (NB - kTail - 1) * MI;   // MFMA slots of a slice that carry a load
  // one load every fourth MFMA at most: the last one then has half a slice to land (every second measured 4 % slower,
  // every sixth 1 % slower)
  constexpr int LSTEP = (LLAST - LFIRST) / NL < 4 ? (LLAST - LFIRST) / NL : 4;
  static_assert(NB % 8 == 0 || (2 * NB) % 8 == 0, "the B ring of eight must close over the two slices of a loop trip");
  constexpr int kARd = (MI + NJ - 4) / (NJ - 3);             // A-fragment reads per group: the last one a group before k-step 1
  static_assert(NJ >= kAhead + 2 && LSTEP >= 1 && MI >= 2, "tile shape");
  static_assert(kARd < MI && 2 + (MI + kARd - 1) / kARd <= NJ - 1, "the A fragments of k-step 1 are read during k-step 0");
  static_assert((BM + BN) * 128 * 2 <= 160 * 1024, "two LDS stages");
  static_assert(4 * stripe_floats<NJ / 2>() * 4 <= (BM + BN) * 128 * 2, "the output staging reuses the operand stages");
  __shared__ __attribute__((aligned(1024))) uint8_t lds[(BM + BN) * 128 * 2];
  uint8_t *const sA0 = lds, *const sA1 = lds + BM * 128, *const sB0 = lds + BM * 256, *const sB1 = lds + BM * 256 + BN * 128;
  __shared__ uint32_t pf_sink[4 * 64];

  const uint32_t tiles = p.mtiles * p.ntiles, split = __builtin_amdgcn_readfirstlane(blockIdx.x / tiles);
  uint32_t id = blockIdx.x - split * tiles, mt, nt, aphase = 0;
  if (p.ntiles % 8 == 0) {
    uint32_t xcd = id & 7, slot = id >> 3;
    nt = (slot / p.mtiles) * 8 + xcd;
    mt = slot % p.mtiles;
    aphase = (slot / p.mtiles) % p.pf_asplit;
  } else {
    nt = id / p.mtiles;
    mt = id % p.mtiles;
  }
  mt = __builtin_amdgcn_readfirstlane(mt);
  nt = __builtin_amdgcn_readfirstlane(nt);
  aphase = __builtin_amdgcn_readfirstlane(aphase);
  const uint32_t m0 = mt * BM, n0 = nt * BN;
  const int tid = threadIdx.x, lane = tid & 63, wave = __builtin_amdgcn_readfirstlane(tid >> 6);
  const int wm = wave / WN, wn = wave % WN;

  uint32_t aoff[NLA], boff[BN / 32];
  const uint32_t chunk = ((lane & 7) ^ ((4 * (wave & 1) + (lane >> 4)) & 7)) * 16;
#pragma unroll
  for (int v = 0; v < NLA; ++v) {
    uint32_t r = min(m0 + 8 * (4 * v + wave) + (lane >> 3), p.M - 1);
    aoff[v] = r * p.strideA * 2 + chunk;
  }
#pragma unroll
  for (int v = 0; v < BN / 32; ++v) {
    uint32_t r = min(n0 + 8 * (4 * v + wave) + (lane >> 3), p.N - 1);
    boff[v] = r * p.K * 2 + chunk;
  }
  const uint8_t *const gA = p.A, *const gW = p.W;
  const uint32_t pf_dist = p.pf_dist, Mrows = p.M, Ncols = p.N;
  auto load_one = [&](int l, uint8_t *na, uint8_t *nb, uint32_t k0) {
    const uint8_t *g = (l < NLA ? gA : gW) + (size_t)k0 * 2;
    const uint32_t voff = l < NLA ? aoff[l] : boff[l - NLA];
    const uint32_t dst = (uint32_t)(uintptr_t)(lds_u8 *)(l < NLA ? na : nb) + (4 * (l < NLA ? l : l - NLA) + wave) * 1024;
    asm volatile("s_mov_b32 m0, %2\n\ts_nop 0\n\tglobal_load_lds_dwordx4 %0, %1" ::"v"(voff), "s"(g), "s"(dst) : "memory");
  };
  const uint8_t *pfp[NPF];
  {
    const uint32_t nw = (BN + p.pf_wsplit - 1) / p.pf_wsplit, na = (BM + p.pf_asplit - 1) / p.pf_asplit;
#pragma unroll
    for (int i = 0; i < NPF; ++i) {
      const uint32_t q = 256 * i + tid;
      uint32_t wr = mt % p.pf_wsplit + (q < nw ? q : 0) * p.pf_wsplit, ar = aphase + (q - nw) * p.pf_asplit;
      const bool is_a = q >= nw && q - nw < na && ar < BM;
      wr = min(n0 + min(wr, (uint32_t)BN - 1), p.N - 1);
      ar = min(m0 + ar, p.M - 1);
      pfp[i] = is_a ? p.A + (size_t)ar * p.strideA * 2 : p.W + (size_t)wr * p.K * 2;
    }
  }
  auto warm_one = [&](int i, uint32_t k0) {
    const uint8_t *g = pfp[i] + (size_t)k0 * 2;
    const uint32_t dst = (uint32_t)(uintptr_t)(lds_u8 *)(reinterpret_cast<uint8_t *>(pf_sink)) + wave * 256;
    asm volatile("s_mov_b32 m0, %1\n\ts_nop 0\n\tglobal_load_lds_dword %0, off" ::"v"(g), "s"(dst) : "memory");
  };

  f32x4 acc[MI][NJ];
#pragma unroll
  for (int i = 0; i < MI; ++i)
#pragma unroll
    for (int j = 0; j < NJ; ++j) acc[i][j] = f32x4{0, 0, 0, 0};

  // fragment of 16 rows x 32 k: lane l holds row l & 15, the 8 halfs of chunk 4 s + (l >> 4) of k-step s; rows of a
  // fragment start at a multiple of 16, so the swizzle key (row >> 1) & 7 is ((l & 15) >> 1)
  const uint32_t arow = (wm * (BM / WM) + (lane & 15)) * 128, brow = (wn * (BN / WN) + (lane & 15)) * 128;
  uint32_t xs[2];
#pragma unroll
  for (int s2 = 0; s2 < 2; ++s2) xs[s2] = ((4 * s2 + (lane >> 4)) ^ ((lane & 15) >> 1)) * 16;
  auto read_a = [&](const uint8_t *sa, int s2, int i) -> half8v {
    return *reinterpret_cast<const lds_half8v *>((const lds_u8 *)(sa) + arow + xs[s2] + i * 2048);
  };
  auto read_b = [&](const uint8_t *sb, int t) -> half8v {   // t: fragment of the slice, k-step t / NJ, tile t % NJ
    return *reinterpret_cast<const lds_half8v *>((const lds_u8 *)(sb) + brow + xs[t / NJ] + (t % NJ) * 2048);
  };

  half8v fa[2][MI], fb[8];
  const uint32_t kbeg = __builtin_amdgcn_readfirstlane(split * p.kper), nsl = p.kper / kDBK, klast = kbeg + p.kper - kDBK;

  // MFMA group g of a slice: B fragment g (ring slot (ring0 + g) & 7) against the MI A fragments of its k-step.
  // With each MFMA at most one LDS read and one load: the reads of this slice's own fragments while they are still
  // ahead (rd_b, rd_a), or - in the tail, behind the barrier - the first reads of the next slice (next_*).
  // cur_*: the stage this group's fragments came from and later reads of this slice go to; nxt_*: the other stage.
  auto group = [&](auto gg, auto ring0c, const uint8_t *ca, const uint8_t *cb, uint8_t *na, uint8_t *nb, uint32_t k0, uint32_t kpf,
                   auto tailc) {
    constexpr int g = decltype(gg)::value, ring0 = decltype(ring0c)::value;
    constexpr bool tail = decltype(tailc)::value;   // this group belongs to the slice before (ca, cb): registers only
    constexpr int s2 = g / NJ, j = g % NJ;
    static_for<MI>([&](auto ii) __attribute__((always_inline)) {
      constexpr int i = decltype(ii)::value;
      // as text with the accumulator tied to itself in an AGPR: through the builtin the allocator rotated accumulators
      // through spare registers and copied them back behind the MFMAs (36 dependent copies per slice)
      asm volatile("v_mfma_f32_16x16x32_f16 %0, %1, %2, %0" : "+a"(acc[i][j]) : "v"(fa[s2][i]), "v"(fb[(ring0 + g) & 7]));
      if constexpr (!tail) {
        // B fragment kAhead groups ahead, with the first MFMA of the group
        if constexpr (i == 0 && g + kAhead < NB) fb[(ring0 + g + kAhead) & 7] = read_b(cb, g + kAhead);
        // A fragments of the second k-step, kARd per group from group 2 on, all on their way before that step begins
        if constexpr (i >= 1 && i <= kARd && g >= 2 && (g - 2) * kARd + (i - 1) < MI)
          fa[1][(g - 2) * kARd + (i - 1)] = read_a(ca, 1, (g - 2) * kARd + (i - 1));
        constexpr int q = g * MI + i;
        if constexpr (q >= LFIRST && (q - LFIRST) % LSTEP == 0 && (q - LFIRST) / LSTEP < NL)
          load_one((q - LFIRST) / LSTEP, na, nb, k0);
        if constexpr (g == NB - kTail - 1 && i < NPF) warm_one(i, kpf);   // younger than every load of the slice
      } else {
        // tail of the slice before: (ca, cb) is the stage just released by the barrier; its first fragments
        constexpr int q = (g - (NB - kTail)) * MI + i;   // slot within the tail
        if constexpr (q < MI) fa[0][q] = read_a(ca, 0, q);
        else if constexpr (q - MI < kAhead) fb[(ring0 + NB + (q - MI)) & 7] = read_b(cb, q - MI);
      }
      __builtin_amdgcn_sched_barrier(0);
    });
  };
  static_assert(kTail * MI >= MI + kAhead, "the tail has a slot for each first read of the next slice");

  // One slice on stage (ca, cb), whose first fragments are already on their way: groups 0 .. NB - kTail - 1, the
  // waits and the barrier, then the last kTail groups from registers with the first reads of the next stage (na, nb).
  auto slice = [&](auto ring0c, const uint8_t *ca, const uint8_t *cb, uint8_t *na, uint8_t *nb, uint32_t t) {
    const uint32_t k0 = min(kbeg + (t + 1) * kDBK, klast), kpf = min(kbeg + (t + pf_dist) * kDBK, klast);
    static_for<NB - kTail>([&](auto gg) __attribute__((always_inline)) {
      group(gg, ring0c, ca, cb, na, nb, k0, kpf, std::false_type{});
    });
    // every read of this stage has been issued at least two groups ago; the next slice has landed in (na, nb)
    asm volatile("s_waitcnt vmcnt(%0) lgkmcnt(0)" ::"n"(NPF) : "memory");
    __builtin_amdgcn_sched_barrier(0);
    asm volatile("s_barrier" ::: "memory");
    __builtin_amdgcn_sched_barrier(0);
    static_for<kTail>([&](auto tt) __attribute__((always_inline)) {
      group(std::integral_constant<int, NB - kTail + decltype(tt)::value>{}, ring0c, na, nb, nullptr, nullptr, 0, 0, std::true_type{});
    });
  };

  for (uint32_t d = 1; d < p.pf_dist; ++d)
#pragma unroll
    for (int i = 0; i < NPF; ++i) warm_one(i, min(kbeg + d * kDBK, klast));
#pragma unroll
  for (int l = 0; l < NL; ++l) load_one(l, sA0, sB0, kbeg);
  asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
  __syncthreads();
  // first fragments of the first slice (what a tail would have read)
#pragma unroll
  for (int i = 0; i < MI; ++i) fa[0][i] = read_a(sA0, 0, i);
#pragma unroll
  for (int t = 0; t < kAhead; ++t) fb[t] = read_b(sB0, t);
  for (uint32_t t = 0; t < nsl; t += 2) {  // nsl is even (host check)
    slice(std::integral_constant<int, 0>{}, sA0, sB0, sA1, sB1, t);
    slice(std::integral_constant<int, NB & 7>{}, sA1, sB1, sA0, sB0, t + 1);
  }
  asm volatile("s_waitcnt vmcnt(0)" ::: "memory");   // the last warm-up loads: nothing may land after the exit

  // C through LDS, a 32-row stripe (two rows of 16 x 16 tiles) at a time.  Register r of lane l of a tile: row
  // 4 (l >> 4) + r, column l & 15.
  __syncthreads();
  constexpr int NJ32 = NJ / 2;
  lds_f32 *stage = (lds_f32 *)(lds_u8 *)(lds) + wave * stripe_floats<NJ32>();
  void *cbase = p.C;
  uint32_t ldc = p.strideC;
  int c_f16 = p.c_f16;
  Epilogue epi = p.epi;
  if (p.ksplit > 1) {
    cbase = p.partial + (size_t)split * p.M * p.N;
    ldc = p.N;
    c_f16 = 0;
    epi.kind = CUTHIP_EPI_NONE;
  }
  const bool vec = p.ksplit > 1 ? p.N % 4 == 0 : p.vec_store != 0;
  const int fast = !vec ? 0 : (!c_f16 ? (epi.kind == CUTHIP_EPI_NONE ? 3 : 0)
                               : epi.kind == CUTHIP_EPI_NONE ? 1
                               : (epi.kind == CUTHIP_EPI_BINARY && epi.op == CUTHIP_BINARY_ADD) ? 2 : 0);
  static_for<MI / 2>([&](auto ii) __attribute__((always_inline)) {
    constexpr int i2 = decltype(ii)::value;
    static_for<2 * NJ>([&](auto tt) __attribute__((always_inline)) {
      constexpr int h = decltype(tt)::value / NJ, j = decltype(tt)::value % NJ;   // h: upper / lower 16 rows of the stripe
      lds_f32 *wr = stage + (16 * h + 4 * (lane >> 4)) * stripe_ld<NJ32>() + 16 * j + (lane & 15);
      const f32x4 a = acc[2 * i2 + h][j];
      static_for<4>([&](auto rr) __attribute__((always_inline)) { wr[decltype(rr)::value * stripe_ld<NJ32>()] = a[decltype(rr)::value]; });
    });
    const uint32_t r0 = m0 + wm * (BM / WM) + 32 * i2, c0 = n0 + wn * (BN / WN);
    if (fast == 1) store_staged32<NJ32, 1>(stage, r0, c0, Mrows, Ncols, cbase, ldc, c_f16, epi, vec, lane);
    else if (fast == 2) store_staged32<NJ32, 2>(stage, r0, c0, Mrows, Ncols, cbase, ldc, c_f16, epi, vec, lane);
    else if (fast == 3) store_staged32<NJ32, 3>(stage, r0, c0, Mrows, Ncols, cbase, ldc, c_f16, epi, vec, lane);
    else store_staged32<NJ32, 0>(stage, r0, c0, Mrows, Ncols, cbase, ldc, c_f16, epi, vec, lane);
  });
#endif
}

// fp32 [M, strideA] -> fp16 [M, K] (round to nearest even), 8 elements per thread
__global__ void __launch_bounds__(256) cvt_rows_kernel(const float *src, half_t *dst, uint32_t K, uint32_t strideA,
                                                       uint32_t chunks) {
  uint32_t row = blockIdx.x / chunks, c = (blockIdx.x % chunks) * 256 + threadIdx.x;
  if (c * 8 >= K) return;
  const float *s = src + (size_t)row * strideA + c * 8;
  f32x4 lo = *reinterpret_cast<const f32x4 *>(s), hi = *reinterpret_cast<const f32x4 *>(s + 4);
  half8v o{(half_t)lo.x, (half_t)lo.y, (half_t)lo.z, (half_t)lo.w, (half_t)hi.x, (half_t)hi.y, (half_t)hi.z, (half_t)hi.w};
  *reinterpret_cast<half8v *>(dst + (size_t)row * K + c * 8) = o;
}

// C = epilogue(sum over the K ranges of the fp32 partial products), one output per thread
__global__ void __launch_bounds__(256) splitk_reduce_kernel(const float *partial, uint32_t ksplit, uint32_t M, uint32_t N,
                                                            void *C, uint32_t strideC, Epilogue epi, int c_f16) {
  const size_t i = (size_t)blockIdx.x * 256 + threadIdx.x, mn = (size_t)M * N;
  if (i >= mn) return;
  float v = 0.0f;
  for (uint32_t s = 0; s < ksplit; ++s) v += partial[s * mn + i];
  const uint32_t row = (uint32_t)(i / N), col = (uint32_t)(i - (size_t)row * N);
  store_out(C, epi, c_f16, (size_t)row * strideC + col, v);
}

// The same for eight consecutive outputs per thread when there is no operator and rows allow 16-byte accesses: every
// load of every K range is requested before the first add, the sum leaves in one store (two for fp32 C).
template <bool F16OUT>
__global__ void __launch_bounds__(256) splitk_reduce8_kernel(const float *partial, uint32_t ksplit, uint32_t M, uint32_t N, void *C,
                                                             uint32_t strideC) {
  const size_t mn = (size_t)M * N, i = ((size_t)blockIdx.x * 256 + threadIdx.x) * 8;
  if (i >= mn) return;
  f32x4 lo = {0.0f, 0.0f, 0.0f, 0.0f}, hi = lo;
  uint32_t s = 0;
  for (; s + 4 <= ksplit; s += 4) {   // four K ranges in flight at a time
    f32x4 a[4], b[4];
#pragma unroll
    for (int u = 0; u < 4; ++u) {
      const f32x4 *src = reinterpret_cast<const f32x4 *>(partial + (s + u) * mn + i);
      a[u] = src[0];
      b[u] = src[1];
    }
#pragma unroll
    for (int u = 0; u < 4; ++u) {
      lo += a[u];
      hi += b[u];
    }
  }
  for (; s < ksplit; ++s) {
    const f32x4 *src = reinterpret_cast<const f32x4 *>(partial + s * mn + i);
    lo += src[0];
    hi += src[1];
  }
  const uint32_t row = (uint32_t)(i / N), col = (uint32_t)(i - (size_t)row * N);
  const size_t idx = (size_t)row * strideC + col;
  if constexpr (F16OUT) {
    const half8_t o{(half_t)lo[0], (half_t)lo[1], (half_t)lo[2], (half_t)lo[3], (half_t)hi[0], (half_t)hi[1], (half_t)hi[2], (half_t)hi[3]};
    *reinterpret_cast<half8_t *>(reinterpret_cast<half_t *>(C) + idx) = o;
  } else {
    f32x4 *cp = reinterpret_cast<f32x4 *>(reinterpret_cast<float *>(C) + idx);
    cp[0] = lo;
    cp[1] = hi;
  }
}

// sums the fp32 partial products [ksplit][M][N] of a K split into C through the epilogue (same order of additions in
// both kernels: K range 0 first)
int launch_splitk_reduce(const float *partial, uint32_t ksplit, uint32_t M, uint32_t N, void *C, uint32_t strideC, Epilogue epi,
                         int c_f16, hipStream_t stream) {
  const uint64_t mn = (uint64_t)M * N;
  if (epi.kind == CUTHIP_EPI_NONE && N % 8 == 0 && (uintptr_t)partial % 16 == 0 && store8_aligned(C, strideC, c_f16, epi)) {
    const dim3 grid((uint32_t)((mn / 8 + 255) / 256));
    if (c_f16) hipLaunchKernelGGL(splitk_reduce8_kernel<true>, grid, dim3(256), 0, stream, partial, ksplit, M, N, C, strideC);
    else hipLaunchKernelGGL(splitk_reduce8_kernel<false>, grid, dim3(256), 0, stream, partial, ksplit, M, N, C, strideC);
  } else {
    hipLaunchKernelGGL(splitk_reduce_kernel, dim3((uint32_t)((mn + 255) / 256)), dim3(256), 0, stream, partial, ksplit, M, N, C,
                       strideC, epi, c_f16);
  }
  return check_hip(hipGetLastError(), "split-K reduce launch");
}

template <int BM, int BN, int WM = 2> static int launch_dense_bm(DenseParams p, hipStream_t stream) {
  p.mtiles = (p.M + BM - 1) / BM;
  p.ntiles = (p.N + BN - 1) / BN;
  // Who runs beside whom: with the XCD-aware order an XCD's 32 CUs hold 32 consecutive slots = the M-tiles of
  // 32 / mtiles weight panels.  Otherwise every workgroup warms all its own lines.
  p.pf_dist = 3;
  p.pf_wsplit = p.pf_asplit = 1;
  if (p.ntiles % 8 == 0) {
    p.pf_wsplit = p.mtiles < 32 ? p.mtiles : 32;
    const uint32_t panels = 32 / p.pf_wsplit, per_xcd = p.ntiles / 8;
    p.pf_asplit = panels < per_xcd ? panels : per_xcd;
    if (p.pf_asplit == 0) p.pf_asplit = 1;
  }
  if (g_tuning.dense_pf >= 0) p.pf_dist = (uint32_t)g_tuning.dense_pf;
  uint64_t grid = (uint64_t)p.mtiles * p.ntiles * p.ksplit;
  if (grid > 0x7FFFFFFFull) {
    set_error("cuthip_matmul_gguf_ws: problem too large for one launch");
    return CUTHIP_ERR_INVALID;
  }
  // the 16 x 16 x 32 kernel unless the tuning key dense_mfma16 = 0 asks for the 32 x 32 x 16 one (kept for comparison)
  const bool mfma16 = g_tuning.dense_mfma16 != 0;
  if (mfma16) hipLaunchKernelGGL((gemm_dense16_kernel<BM, BN, WM>), dim3((uint32_t)grid), dim3(256), 0, stream, p);
  else hipLaunchKernelGGL((gemm_dense_kernel<BM, BN, WM>), dim3((uint32_t)grid), dim3(256), 0, stream, p);
  return check_hip(hipGetLastError(), "dense gemm launch");
}

// Shapes the two-pass path takes: K a multiple of 128 (two LDS stages per loop trip), 16-byte aligned rows of A,
// and operands small enough for 32-bit byte offsets.
bool dense_gemm_fits(uint32_t M, uint32_t K, uint32_t N, uint32_t strideA, int a_f16, const void *A) {
  if (K % 128 != 0 || M == 0 || N == 0) return false;
  if ((uint64_t)N * K * 2 >= (1ull << 32)) return false;
  if (a_f16) {
    if ((uintptr_t)A % 16 != 0 || strideA % 8 != 0 || (uint64_t)M * strideA * 2 >= (1ull << 32)) return false;
  } else {
    if ((uintptr_t)A % 16 != 0 || strideA % 4 != 0 || (uint64_t)M * K * 2 >= (1ull << 32)) return false;
  }
  return true;
}

// Tile shape and number of K ranges.  Candidates in the order of their measured cost per multiply-add on whole rounds
// (2048 x 14336 x 4096, every shape forced in turn on one box): 256 x 224 (four waves along M) 0.96, 128 x 448 1.00,
// 256 x 256 1.03, 128 x 256 1.24.  A shape costs rounds over the 256 CUs x tile area x that factor; tiles that hang
// over the edge of C count in full.  When the best shape leaves most of the chip idle, K is split over 128 x 256
// tiles instead (partials in the workspace, summed by a second kernel).
struct DenseShape { int bm, bn; uint32_t ksplit; };
static DenseShape pick_dense_shape(uint32_t M, uint32_t K, uint32_t N) {
  if (g_tuning.dense_bn && K % ((uint32_t)g_tuning.dense_ks * 128) == 0)   // forced by a test or a sweep
    return DenseShape{g_tuning.dense_bm, g_tuning.dense_bn, (uint32_t)g_tuning.dense_ks};
  static const struct { int bm, bn; double cost; } cands[] = {{256, 224, 0.96}, {128, 448, 1.00}, {256, 256, 1.03}, {128, 256, 1.24}};
  int best = 0;
  double best_t = 0.0;
  uint64_t best_tiles = 0;
  for (int c = 0; c < 4; ++c) {
    const uint64_t tiles = (uint64_t)((M + cands[c].bm - 1) / cands[c].bm) * ((N + cands[c].bn - 1) / cands[c].bn);
    const double t = (double)((tiles + 255) / 256) * cands[c].bm * cands[c].bn * cands[c].cost;
    if (c == 0 || t < best_t) {
      best = c;
      best_t = t;
      best_tiles = tiles;
    }
  }
  if (best_tiles >= 192) return DenseShape{cands[best].bm, cands[best].bn, 1};
  const uint64_t tiles128 = (uint64_t)((M + 127) / 128) * ((N + 255) / 256);
  uint32_t s = 1;
  while (s < 8 && tiles128 * s < 192 && K % (2 * s * 128) == 0) s *= 2;
  if (s == 1) return DenseShape{cands[best].bm, cands[best].bn, 1};
  return DenseShape{128, 256, s};
}

static size_t align256(size_t n) { return (n + 255) & ~(size_t)255; }

// scratch the vendor GEMM may use (variant 5) behind the dequantized weights and the converted activations
constexpr size_t kBlasLtScratch = (size_t)32 << 20;

bool blaslt_available();
int launch_blaslt_gemm(const void *Wd, const void *A16, void *C, int c_f16, uint32_t M, uint32_t K, uint32_t N, uint32_t strideA,
                       uint32_t strideC, void *workspace, size_t workspace_bytes, hipStream_t stream);

size_t dense_gemm_workspace(uint32_t M, uint32_t K, uint32_t N, int a_f16) {
  DenseShape sh = pick_dense_shape(M, K, N);
  const size_t partial = sh.ksplit > 1 ? (size_t)sh.ksplit * M * N * 4 : 0;
  return align256((size_t)N * K * 2) + align256(a_f16 ? 0 : (size_t)M * K * 2) + (partial > kBlasLtScratch ? partial : kBlasLtScratch);
}

// workspace of the GEMM on resident fp16 weights: converted activations (fp32 input only) + split-K partials / scratch
size_t dense_f16_workspace(uint32_t M, uint32_t K, uint32_t N, int a_f16) {
  return dense_gemm_workspace(M, K, N, a_f16) - align256((size_t)N * K * 2);
}

// Cost models in microseconds for the automatic choice between the two-pass path and the single-launch GEMM, fitted to
// a sweep over the weight shapes of an 8B model (all formats, M = 16 .. 2048, HIP-graph replay, MI355X):
//   two-pass      3 + N K (bytes per weight + 2) / 6.0 MB   the dequantization (reads the blocks, writes fp16)
//                 + 17 + max(2 ceil128(M) N K / 1.25 PFLOP/s,  the dense GEMM (tiles are at least 128 rows high; up to 256 rows
//                            2 N K / 3.5 MB)                  it is bound by reading the fp16 weights: 128 and 256 x 28672 x 4096
//                                                             both take 147-148 us on Q6_K, 14336 x 4096 76 and 79)
//   single launch K x c_fmt x max(1, tiles / 256)            c = 14.7 ns (Q4_K, Q4_0), 17 ns (Q8_0: 256 x 28672 x 4096 122 us,
//                 512 rows 220, 256 x 14336 x 4096 73-76), 19.5 ns (Q6_K: 256 x 28672 x 4096 133-139 us,
//                 512 x 14336 x 4096 139):
//                 a workgroup decodes its K-long strip of weights once per 128 rows of A, and nothing overlaps that
//                 walk until every CU holds more than one 128 x 128 tile.
// Measured against them (Q4_K, M x N x K): 64 x 4096 x 4096 38 / 62 us, 512 x 14336 x 4096 99 / 105, 512 x 28672 x 4096
// 173 / 203, 256 x 28672 x 4096 147 / 107; Q6_K 64 x 14336 x 4096 79 / 104.
//                 + 5 where the GEMM splits K (a third launch sums the partial products): 1024 x 1024 x 4096 36 us
double dense_cost_us(int fmt, uint32_t M, uint32_t K, uint32_t N) {
  const double nk = (double)N * K, bpw = (double)fmt_bytes(fmt) / fmt_elems(fmt);
  const double split = pick_dense_shape(M, K, N).ksplit > 1 ? 5.0 : 0.0;
  const double mfma = 2.0 * (double)((M + 127) / 128 * 128) * nk / 1.25e9, stream = 2.0 * nk / 3.5e6;
  return 3.0 + nk * (bpw + 2.0) / 6.0e6 + 17.0 + (mfma > stream ? mfma : stream) + split;
}
double single_launch_rows_cost_us(int fmt, uint32_t M, uint32_t K, uint32_t N) {
  const double c = fmt == CUTHIP_Q6_K ? 19.5e-3 : fmt == CUTHIP_Q8_0 ? 17.0e-3 : 14.7e-3;
  const double tiles = (double)((M + 127) / 128) * ((N + 127) / 128);
  return K * c * (tiles > 256.0 ? tiles / 256.0 : 1.0);
}

// use_blaslt: the dense GEMM goes to hipBLASLt (no epilogue there: the caller checks)
int launch_dense_gemm(int fmt, const void *W, const void *A, int a_f16, void *C, int c_f16, uint32_t M, uint32_t K,
                      uint32_t N, uint32_t strideA, uint32_t strideC, Epilogue epi, void *workspace, hipStream_t stream,
                      int use_blaslt) {
  // fmt < 0: W already holds the dequantized fp16 weights [N][K] (cuthip_matmul_dense_f16); the workspace then starts
  // with the converted activations.  Otherwise the weights are dequantized to the head of the workspace first.
  const bool resident = fmt < 0;
  uint8_t *ws = reinterpret_cast<uint8_t *>(workspace);
  const uint8_t *w16 = resident ? reinterpret_cast<const uint8_t *>(W) : ws;
  uint8_t *after_w = resident ? ws : ws + align256((size_t)N * K * 2);
  if (!resident) {
    if (int rc = launch_dequant_any(fmt, W, ws, CUTHIP_F16, N, K, K, stream)) return rc;
  }
  DenseParams p;
  p.W = w16;
  p.A = reinterpret_cast<const uint8_t *>(A);
  p.strideA = strideA;
  if (!a_f16) {
    half_t *a16 = reinterpret_cast<half_t *>(after_w);
    uint32_t chunks = (K / 8 + 255) / 256;
    hipLaunchKernelGGL(cvt_rows_kernel, dim3(M * chunks), dim3(256), 0, stream, reinterpret_cast<const float *>(A), a16, K,
                       strideA, chunks);
    if (int rc = check_hip(hipGetLastError(), "activation convert launch")) return rc;
    p.A = reinterpret_cast<const uint8_t *>(a16);
    p.strideA = K;
  }
  if (use_blaslt) {
    uint8_t *scratch = after_w + align256(a_f16 ? 0 : (size_t)M * K * 2);
    const int rc = launch_blaslt_gemm(w16, p.A, C, c_f16, M, K, N, p.strideA, strideC, scratch, kBlasLtScratch, stream);
    // 1 = asked for by variant index: its errors are the caller's; 2 = automatic choice: a shape the library has no
    // kernel for goes on to the GEMM below (nothing has been enqueued for it yet)
    if (rc == CUTHIP_OK || use_blaslt == 1 || rc != CUTHIP_ERR_INVALID) return rc;
  }
  p.C = C;
  p.epi = epi;
  p.M = M; p.N = N; p.K = K; p.strideC = strideC;
  p.mtiles = p.ntiles = 0;
  p.c_f16 = c_f16;
  p.vec_store = store8_aligned(C, strideC, c_f16, epi) ? 1 : 0;
  const DenseShape sh = pick_dense_shape(M, K, N);
  p.ksplit = sh.ksplit;
  p.kper = K / sh.ksplit;
  p.partial = reinterpret_cast<float *>(after_w + align256(a_f16 ? 0 : (size_t)M * K * 2));
  int rc;
  if (sh.bn == 448) rc = launch_dense_bm<128, 448>(p, stream);
  else if (sh.bn == 224) rc = launch_dense_bm<256, 224, 4>(p, stream);
  else if (sh.bm == 256) rc = launch_dense_bm<256, 256>(p, stream);
  else rc = launch_dense_bm<128, 256>(p, stream);
  if (rc) return rc;
  if (sh.ksplit > 1) {
    return launch_splitk_reduce(p.partial, sh.ksplit, M, N, C, strideC, epi, c_f16, stream);
  }
  return CUTHIP_OK;
}

}  // namespace cuthip
