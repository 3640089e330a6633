// The small operators between the quantized matmuls of one decode step, for
// gfx950: RMSNorm, RoPE + KV-cache write, GQA decode attention over an fp16
// KV cache, SiLU(gate) * up, arg-max.  Semantics follow the reference
// kernels (operators/impl/rmsnorm/RMSNorm.cu, attention/FusedRoPEKVWrite.cu,
// attention/Attention.cu): fp32 arithmetic, half-split RoPE with cos / sin
// tables [pos][headDim/2], cache rows [pos][alignedKvDim], position and
// sequence length read from a device buffer so that a captured graph can be
// replayed for the next token.
//
// The attention differs from the reference in structure, not in result: the
// reference runs one workgroup per query head over the whole context (every
// K/V row is read nRep times, scores staged in 8 KB of shared memory).  Here
// a workgroup owns one KV head and a chunk of 64 positions; its four waves
// are the (up to four at a time) query heads sharing that KV head, so K and V
// are read from HBM once, staged in LDS, and the softmax is carried as
// (max, sum, weighted V) partials (the usual split-context decode attention).
// A second, small kernel merges the partials.  Merging inside the first kernel
// (the workgroup that draws the last ticket of a KV head's counter reads the
// records back; all workgroups of a head placed on one XCD so that records
// and tickets stay in that XCD's L2; no fences) was built and measured: the
// three dependent hops (stores acknowledged, ticket, records read back) cost
// 5.5 us against the 4.5 us of the merge launch (12.8 us against 11.4 us per
// layer), because every dependent memory access costs about a microsecond
// here, in the XCD's own L2 as well.
#include <cmath>
#include <cstdint>
#include <cstdlib>
#include <mutex>

#include "gemv_formats.hpp"

namespace cuthip {

__device__ inline float ld_act(const void *p, int f16, size_t i) {
  return f16 ? (float)reinterpret_cast<const half_t *>(p)[i] : reinterpret_cast<const float *>(p)[i];
}
__device__ inline void st_act(void *p, int f16, size_t i, float v) {
  if (f16)
    reinterpret_cast<half_t *>(p)[i] = (half_t)v;
  else
    reinterpret_cast<float *>(p)[i] = v;
}
__device__ inline float wave_sum(float v) {
#pragma unroll
  for (int o = 32; o > 0; o >>= 1) v += __shfl_xor(v, o);
  return v;
}
__device__ inline float wave_max(float v) {
#pragma unroll
  for (int o = 32; o > 0; o >>= 1) v = fmaxf(v, __shfl_xor(v, o));
  return v;
}

// ---- RMSNorm: out = x * rsqrt(mean(x^2) + eps) * weight; one workgroup per row ----
// A thread owns groups of 8 consecutive elements; up to kNormGroups of them stay in registers between the two
// passes and all their loads are issued before the first use (a decode row is a few KB: one memory round trip).
constexpr int kNormGroups = 4;   // 256 threads x 8 elements x 4 = rows of up to 8192 elements without a re-read

// vec_ok: the row allows 16-byte loads; otherwise (or in the last, short group) the up to 8 elements are loaded singly
template <bool F16> __device__ inline void ld8(const void *p, size_t i, uint32_t n_left, bool vec_ok, float (&v)[8]) {
  if (vec_ok && n_left >= 8) {
    if (F16) {
      half8_t h = *reinterpret_cast<const half8_t *>(reinterpret_cast<const half_t *>(p) + i);
#pragma unroll
      for (int e = 0; e < 8; ++e) v[e] = (float)h[e];
    } else {
      f32x4 a = *reinterpret_cast<const f32x4 *>(reinterpret_cast<const float *>(p) + i);
      f32x4 b = *reinterpret_cast<const f32x4 *>(reinterpret_cast<const float *>(p) + i + 4);
      v[0] = a.x; v[1] = a.y; v[2] = a.z; v[3] = a.w; v[4] = b.x; v[5] = b.y; v[6] = b.z; v[7] = b.w;
    }
  } else {
#pragma unroll
    for (int e = 0; e < 8; ++e) v[e] = (uint32_t)e < n_left ? ld_act(p, F16, i + e) : 0.0f;
  }
}

template <bool XF16, bool OF16>
__global__ void __launch_bounds__(256) rmsnorm_kernel(const void *x, const float *weight, void *out, uint32_t dim,
                                                      uint32_t stride, float eps, int aligned) {
  __shared__ float red[4];
  const uint32_t row = blockIdx.x, tid = threadIdx.x;
  const size_t off = (size_t)row * stride;
  float v[kNormGroups][8];
  float s = 0.0f;
#pragma unroll
  for (int g = 0; g < kNormGroups; ++g) {
    uint32_t i = (g * 256 + tid) * 8;
    if (i < dim) ld8<XF16>(x, off + i, dim - i, aligned != 0, v[g]);   // unaligned rows: element loads
  }
#pragma unroll
  for (int g = 0; g < kNormGroups; ++g) {
    uint32_t i = (g * 256 + tid) * 8;
    if (i < dim)
#pragma unroll
      for (int e = 0; e < 8; ++e) s = fmaf(v[g][e], v[g][e], s);
  }
  for (uint32_t i = kNormGroups * 2048 + tid; i < dim; i += 256) {   // rows longer than the register window
    float t = ld_act(x, XF16, off + i);
    s = fmaf(t, t, s);
  }
  s = wave_sum(s);
  if ((tid & 63) == 0) red[tid >> 6] = s;
  __syncthreads();
  float total = red[0] + red[1] + red[2] + red[3];
  float scale = 1.0f / sqrtf(total / (float)dim + eps);
  const bool wide = aligned && reinterpret_cast<uintptr_t>(out) % 16 == 0 && reinterpret_cast<uintptr_t>(weight) % 16 == 0;
#pragma unroll
  for (int g = 0; g < kNormGroups; ++g) {
    uint32_t i = (g * 256 + tid) * 8;
    if (i < dim) {
      uint32_t n = min(dim - i, 8u);
      if (wide && n == 8) {   // 16-byte weight loads and output stores
        f32x4 w0 = *reinterpret_cast<const f32x4 *>(weight + i), w1 = *reinterpret_cast<const f32x4 *>(weight + i + 4);
        float r[8] = {v[g][0] * scale * w0.x, v[g][1] * scale * w0.y, v[g][2] * scale * w0.z, v[g][3] * scale * w0.w,
                      v[g][4] * scale * w1.x, v[g][5] * scale * w1.y, v[g][6] * scale * w1.z, v[g][7] * scale * w1.w};
        if (OF16) {
          half8_t h;
#pragma unroll
          for (int e = 0; e < 8; ++e) h[e] = (half_t)r[e];
          *reinterpret_cast<half8_t *>(reinterpret_cast<half_t *>(out) + off + i) = h;
        } else {
          float *o = reinterpret_cast<float *>(out) + off + i;
          *reinterpret_cast<f32x4 *>(o) = f32x4{r[0], r[1], r[2], r[3]};
          *reinterpret_cast<f32x4 *>(o + 4) = f32x4{r[4], r[5], r[6], r[7]};
        }
      } else {
        for (uint32_t e = 0; e < n; ++e) st_act(out, OF16, off + i + e, v[g][e] * scale * weight[i + e]);
      }
    }
  }
  for (uint32_t i = kNormGroups * 2048 + tid; i < dim; i += 256)
    st_act(out, OF16, off + i, ld_act(x, XF16, off + i) * scale * weight[i]);
}

// ---- RoPE on q and k, k and v appended to the cache at position params[0] ----
__global__ void __launch_bounds__(256) rope_kv_kernel(const void *q, const void *k, const void *v, int in_f16,
                                                      const uint32_t *params, const float *cosT, const float *sinT,
                                                      half_t *kCache, half_t *vCache, void *qOut, int qout_f16, uint32_t qDim,
                                                      uint32_t kvDim, uint32_t headDim, uint32_t alignedKvDim,
                                                      uint32_t maxPositions) {
  const uint32_t gid = blockIdx.x * 256 + threadIdx.x, halfDim = headDim / 2;
  if (gid >= qDim + 2 * kvDim) return;
  const uint32_t pos = params[0];
  if (pos >= maxPositions) return;   // past the caches and the tables: nothing is read or written
  const float *c = cosT + (size_t)pos * halfDim, *s = sinT + (size_t)pos * halfDim;
  auto rot = [&](const void *src, uint32_t i) {
    uint32_t d = i % headDim;
    if (d < halfDim) return ld_act(src, in_f16, i) * c[d] - ld_act(src, in_f16, i + halfDim) * s[d];
    return ld_act(src, in_f16, i - halfDim) * s[d - halfDim] + ld_act(src, in_f16, i) * c[d - halfDim];
  };
  if (gid < qDim) {
    st_act(qOut, qout_f16, gid, rot(q, gid));
  } else if (gid < qDim + kvDim) {
    uint32_t i = gid - qDim;
    kCache[(size_t)pos * alignedKvDim + i] = (half_t)rot(k, i);
  } else {
    uint32_t i = gid - qDim - kvDim;
    vCache[(size_t)pos * alignedKvDim + i] = (half_t)ld_act(v, in_f16, i);
  }
}

// ---- decode attention, split over the context ----
constexpr int kAttnChunk = 64;    // positions per workgroup (one per lane)
constexpr int kAttnMaxHd = 128;   // head dimension limit (as the reference's sharedQ[128])
constexpr int kAttnRow = kAttnMaxHd + 8;   // LDS row in halfs: +16 bytes keeps the 64 rows off each other's banks

// partial layout per (query head h, split s): [m, l, o[headDim]] floats at ((h * nsplit + s) * (2 + headDim))
// HD: the head dimension when it is the common 128 (loops over it unroll and their LDS reads overlap), 0 = any
// The arguments that the first loads need (up to and including headDimArg: 14 dwords) lead the list: with
// kernel-argument preloading they arrive in SGPRs with the wave, and the loads of q, K and V wait for no scalar load.
template <int HD>
__global__ void __launch_bounds__(256) attn_partial_kernel(const void *q, const half_t *kCache, const half_t *vCache,
                                                           const uint32_t *params, uint32_t alignedKvDim, uint32_t maxSeqLen,
                                                           uint32_t nHeads, uint32_t nKvHeads, int q_f16, uint32_t headDimArg,
                                                           float *partial, float scale, uint32_t nsplit) {
  const uint32_t headDim = HD ? (uint32_t)HD : headDimArg;
  __shared__ __attribute__((aligned(16))) half_t Ks[kAttnChunk * kAttnRow];
  __shared__ __attribute__((aligned(16))) half_t Vs[kAttnChunk * kAttnRow];
  __shared__ __attribute__((aligned(16))) float Qs[4 * kAttnMaxHd];
  __shared__ __attribute__((aligned(16))) float Ps[4 * kAttnChunk];
  const uint32_t kvH = blockIdx.x, split = blockIdx.y, nRep = nHeads / nKvHeads;
  const uint32_t tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
  const uint32_t seqLen = min(params[1], maxSeqLen);   // a length beyond the cache capacity attends the capacity only
  const uint32_t t0 = split * kAttnChunk;
  const uint32_t nvalid = t0 < seqLen ? min((uint32_t)kAttnChunk, seqLen - t0) : 0u;

  // Every load of the start-up is requested before the first of them is used, so that the kernel begins with one
  // memory round trip: the query of the first pass (raw bits, converted later: a conversion right behind the load is a
  // use, and the compiler then waits for it on the spot), then the chunk of K and V.  Written as a loop with the
  // store right behind each load, the staging waited for four round trips in turn, and the query for two more.
  uint32_t q_raw[2] = {0u, 0u};
  {
    const uint32_t h0 = kvH * nRep + (wave < nRep ? wave : 0);
    const size_t qi = (size_t)h0 * headDim + min(lane, headDim - 1);   // lanes beyond the head dimension read a valid element
    const size_t qj = (size_t)h0 * headDim + min(lane + 64, headDim - 1);
    if (q_f16) {
      q_raw[0] = reinterpret_cast<const uint16_t *>(q)[qi];
      q_raw[1] = reinterpret_cast<const uint16_t *>(q)[qj];
    } else {
      q_raw[0] = reinterpret_cast<const uint32_t *>(q)[qi];
      q_raw[1] = reinterpret_cast<const uint32_t *>(q)[qj];
    }
  }
  // stage the chunk of K and V (16-byte pieces; rows past the sequence are zero).  The loads do not wait for the
  // sequence length (every row below the cache capacity is readable); rows past the sequence are zeroed afterwards.
  const uint32_t pieces = headDim / 8;
  if constexpr (HD != 0) {
    constexpr int IT = kAttnChunk * (HD / 8) / 256;
    static_assert(IT * 256 == kAttnChunk * (HD / 8), "one 16-byte piece per thread and round");
    u32x4 kraw[IT], vraw[IT];
#pragma unroll
    for (int it = 0; it < IT; ++it) {
      const uint32_t i = tid + 256u * it, r = i / (HD / 8), c8 = i % (HD / 8);
      const size_t off = (size_t)min(t0 + r, maxSeqLen - 1) * alignedKvDim + kvH * headDim + c8 * 8;
      kraw[it] = ld_u32x4(reinterpret_cast<const uint8_t *>(kCache + off));
      vraw[it] = ld_u32x4(reinterpret_cast<const uint8_t *>(vCache + off));
    }
    __builtin_amdgcn_sched_barrier(0);
#pragma unroll
    for (int it = 0; it < IT; ++it) {
      const uint32_t i = tid + 256u * it, r = i / (HD / 8), c8 = i % (HD / 8);
      const bool past = r >= nvalid;
      *reinterpret_cast<u32x4 *>(Ks + r * kAttnRow + c8 * 8) = past ? u32x4{0, 0, 0, 0} : kraw[it];
      *reinterpret_cast<u32x4 *>(Vs + r * kAttnRow + c8 * 8) = past ? u32x4{0, 0, 0, 0} : vraw[it];
    }
  } else {
    for (uint32_t i = tid; i < kAttnChunk * pieces; i += 256) {
      uint32_t r = i / pieces, c8 = i % pieces;
      size_t off = (size_t)min(t0 + r, maxSeqLen - 1) * alignedKvDim + kvH * headDim + c8 * 8;
      u32x4 kv = ld_u32x4(reinterpret_cast<const uint8_t *>(kCache + off));
      u32x4 vv = ld_u32x4(reinterpret_cast<const uint8_t *>(vCache + off));
      if (r >= nvalid) {
        kv = u32x4{0, 0, 0, 0};
        vv = u32x4{0, 0, 0, 0};
      }
      *reinterpret_cast<u32x4 *>(Ks + r * kAttnRow + c8 * 8) = kv;
      *reinterpret_cast<u32x4 *>(Vs + r * kAttnRow + c8 * 8) = vv;
    }
  }
  float q_pre[2];
#pragma unroll
  for (int e = 0; e < 2; ++e)
    q_pre[e] = q_f16 ? (float)__builtin_bit_cast(half_t, (uint16_t)q_raw[e]) : __builtin_bit_cast(float, q_raw[e]);
  // query heads of this KV head are handled four at a time, one per wave
  for (uint32_t rep0 = 0; rep0 < nRep; rep0 += 4) {
    const uint32_t rep = rep0 + wave;
    const bool live = rep < nRep;
    const uint32_t h = kvH * nRep + (live ? rep : 0);
    if (rep0 == 0) {
      // the first pass' query goes to LDS ahead of the staging barrier (each wave reads only its own), so that the
      // pass costs one workgroup barrier, not two
#pragma unroll
      for (int e = 0; e < 2; ++e)
        if (lane + 64 * e < headDim) Qs[wave * kAttnMaxHd + lane + 64 * e] = q_pre[e];
      __syncthreads();   // K, V staged
    } else {
      __syncthreads();   // Qs, Ps free again
      for (uint32_t d = lane; d < headDim; d += 64) Qs[wave * kAttnMaxHd + d] = ld_act(q, q_f16, (size_t)h * headDim + d);
      __syncthreads();
    }
    // score of position t0 + lane: q is read as broadcast 16-byte pieces
    float sc = 0.0f;
    const half_t *krow = Ks + lane * kAttnRow;
    const f32x4 *qv = reinterpret_cast<const f32x4 *>(Qs + wave * kAttnMaxHd);
#pragma unroll
    for (uint32_t d = 0; d < headDim; d += 8) {
      half8_t k8 = *reinterpret_cast<const half8_t *>(krow + d);
      f32x4 qa = qv[d / 4], qb = qv[d / 4 + 1];
      sc = fmaf(qa.x, (float)k8[0], sc); sc = fmaf(qa.y, (float)k8[1], sc);
      sc = fmaf(qa.z, (float)k8[2], sc); sc = fmaf(qa.w, (float)k8[3], sc);
      sc = fmaf(qb.x, (float)k8[4], sc); sc = fmaf(qb.y, (float)k8[5], sc);
      sc = fmaf(qb.z, (float)k8[6], sc); sc = fmaf(qb.w, (float)k8[7], sc);
    }
    sc = lane < nvalid ? sc * scale : -INFINITY;
    float m = wave_max(sc);
    float p = lane < nvalid ? expf(sc - m) : 0.0f;
    float l = wave_sum(p);
    Ps[wave * kAttnChunk + lane] = p;   // zero for positions past the sequence
    __builtin_amdgcn_wave_barrier();
    asm volatile("s_waitcnt lgkmcnt(0)" ::: "memory");
    // weighted V: lane owns the adjacent dims 2 * lane and 2 * lane + 1 (one 4-byte LDS read per position),
    // four weights per 16-byte read; rows past the sequence are zero and carry zero weight
    float o0 = 0.0f, o1 = 0.0f;
    typedef _Float16 half2v __attribute__((ext_vector_type(2)));
    const f32x4 *pv = reinterpret_cast<const f32x4 *>(Ps + wave * kAttnChunk);
    const uint32_t dcol = min(2 * lane, (uint32_t)kAttnMaxHd - 2);
#pragma unroll
    for (uint32_t t = 0; t < (uint32_t)kAttnChunk; t += 4) {
      f32x4 p4 = pv[t / 4];
      half2v v0 = *reinterpret_cast<const half2v *>(Vs + (t + 0) * kAttnRow + dcol);
      half2v v1 = *reinterpret_cast<const half2v *>(Vs + (t + 1) * kAttnRow + dcol);
      half2v v2 = *reinterpret_cast<const half2v *>(Vs + (t + 2) * kAttnRow + dcol);
      half2v v3 = *reinterpret_cast<const half2v *>(Vs + (t + 3) * kAttnRow + dcol);
      o0 = fmaf(p4.x, (float)v0.x, o0); o1 = fmaf(p4.x, (float)v0.y, o1);
      o0 = fmaf(p4.y, (float)v1.x, o0); o1 = fmaf(p4.y, (float)v1.y, o1);
      o0 = fmaf(p4.z, (float)v2.x, o0); o1 = fmaf(p4.z, (float)v2.y, o1);
      o0 = fmaf(p4.w, (float)v3.x, o0); o1 = fmaf(p4.w, (float)v3.y, o1);
    }
    if (live) {
      float *dst = partial + ((size_t)h * nsplit + split) * (2 + headDim);
      if (lane == 0) {
        dst[0] = nvalid ? m : -INFINITY;
        dst[1] = l;
      }
      if (2 * lane + 1 < headDim) {
        dst[2 + 2 * lane] = o0;
        dst[2 + 2 * lane + 1] = o1;
      }
    }
  }
}

// ---- decode attention with few, wide context splits (head dimension 128) ----
// One workgroup per (query head, split), at most kAttnWideSplits splits per head, so that a consumer can fold the
// records of a head while it stages its activations (the output projection, gemv_rows8.hpp) and the merge launch
// disappears.  Split s takes the 64-position chunks s, s + nsplit, s + 2 * nsplit, ...: one chunk per wave and pass,
// so a short sequence in a large cache still spreads over the splits.  Every wave works alone until the end (its own
// K chunk in LDS, V straight from memory into registers: a lane's 16-byte piece of V covers 8 dimensions of one
// position, and the lane multiplies it by that position's weight), then the four waves' (max, sum, o) are folded
// into the one record [max, sum, o[128]] of the split.  The query heads that share a KV head read the same chunk:
// the block index puts them on the same XCD (equal index modulo 8 when nKvHeads * nsplit is a multiple of 8), so
// the chunk crosses the fabric once.
constexpr int kAttnWideSplits = 8;
constexpr size_t kAttnWideLds = 4 * (size_t)kAttnChunk * kAttnRow * 2 + 4 * kAttnChunk * 4 + kAttnMaxHd * 4;

__global__ void __launch_bounds__(256) attn_partial_wide_kernel(const void *q, const half_t *kCache, const half_t *vCache,
                                                                const uint32_t *params, uint32_t alignedKvDim,
                                                                uint32_t maxSeqLen, uint32_t nHeads, uint32_t nKvHeads,
                                                                int q_f16, uint32_t nsplit, float *partial, float scale) {
  constexpr uint32_t HD = 128;
  extern __shared__ __attribute__((aligned(16))) uint8_t wide_lds[];
  const uint32_t tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
  half_t *Ks = reinterpret_cast<half_t *>(wide_lds) + (size_t)wave * kAttnChunk * kAttnRow;   // this wave's chunk of K
  float *Pp = reinterpret_cast<float *>(wide_lds + 4 * (size_t)kAttnChunk * kAttnRow * 2) + wave * kAttnChunk;
  float *Qs = reinterpret_cast<float *>(wide_lds + 4 * (size_t)kAttnChunk * kAttnRow * 2 + 4 * kAttnChunk * 4);
  const uint32_t nRep = nHeads / nKvHeads, per_rep = nKvHeads * nsplit;
  const uint32_t rep = blockIdx.x / per_rep, rem = blockIdx.x - rep * per_rep;
  const uint32_t kvH = rem / nsplit, split = rem - kvH * nsplit, h = kvH * nRep + rep;
  const uint32_t grp = lane >> 4, c8 = lane & 15;   // V / K piece of a pass: position 4 * it + grp, dimensions 8 * c8 ..

  // the query (raw bits) and the first pass's chunk of K and V are requested before anything is used; none of these
  // loads waits for the sequence length (every row below the cache capacity is readable, rows past the sequence are
  // masked afterwards)
  uint32_t q_raw = 0u;
  if (tid < HD) q_raw = q_f16 ? (uint32_t)reinterpret_cast<const uint16_t *>(q)[(size_t)h * HD + tid]
                              : reinterpret_cast<const uint32_t *>(q)[(size_t)h * HD + tid];
  float m_run = -INFINITY, l_run = 0.0f, o_run[8];
#pragma unroll
  for (int e = 0; e < 8; ++e) o_run[e] = 0.0f;
  uint32_t seqLen = 0u;
  for (uint32_t pass = 0;; ++pass) {
    const uint32_t t0 = (split + nsplit * (wave + 4u * pass)) * (uint32_t)kAttnChunk;
    // pass 0 runs for every wave (its barrier publishes the query); later passes end at the sequence length
    if (pass > 0 && t0 >= seqLen) break;
    u32x4 kr[16], vr[16];
#pragma unroll
    for (int it = 0; it < 16; ++it) {
      const size_t off = (size_t)min(t0 + 4u * it + grp, maxSeqLen - 1) * alignedKvDim + kvH * HD + c8 * 8;
      kr[it] = ld_u32x4(reinterpret_cast<const uint8_t *>(kCache + off));
    }
#pragma unroll
    for (int it = 0; it < 16; ++it) {
      const size_t off = (size_t)min(t0 + 4u * it + grp, maxSeqLen - 1) * alignedKvDim + kvH * HD + c8 * 8;
      vr[it] = ld_u32x4(reinterpret_cast<const uint8_t *>(vCache + off));
    }
    __builtin_amdgcn_sched_barrier(0);
    if (pass == 0) {
      seqLen = min(params[1], maxSeqLen);   // a length beyond the cache capacity attends the capacity only
      if (tid < HD) Qs[tid] = q_f16 ? (float)__builtin_bit_cast(half_t, (uint16_t)q_raw) : __builtin_bit_cast(float, q_raw);
    }
    const uint32_t nvalid = t0 < seqLen ? min((uint32_t)kAttnChunk, seqLen - t0) : 0u;
#pragma unroll
    for (int it = 0; it < 16; ++it) *reinterpret_cast<u32x4 *>(Ks + (4 * it + grp) * kAttnRow + c8 * 8) = kr[it];
    if (pass == 0) __syncthreads();   // the query, and this wave's K
    else {
      __builtin_amdgcn_wave_barrier();
      asm volatile("s_waitcnt lgkmcnt(0)" ::: "memory");
    }
    // score of position t0 + lane
    float sc = 0.0f;
    const half_t *krow = Ks + lane * kAttnRow;
    const f32x4 *qv = reinterpret_cast<const f32x4 *>(Qs);
#pragma unroll
    for (uint32_t d = 0; d < HD; d += 8) {
      half8_t k8 = *reinterpret_cast<const half8_t *>(krow + d);
      f32x4 qa = qv[d / 4], qb = qv[d / 4 + 1];
      sc = fmaf(qa.x, (float)k8[0], sc); sc = fmaf(qa.y, (float)k8[1], sc);
      sc = fmaf(qa.z, (float)k8[2], sc); sc = fmaf(qa.w, (float)k8[3], sc);
      sc = fmaf(qb.x, (float)k8[4], sc); sc = fmaf(qb.y, (float)k8[5], sc);
      sc = fmaf(qb.z, (float)k8[6], sc); sc = fmaf(qb.w, (float)k8[7], sc);
    }
    sc = lane < nvalid ? sc * scale : -INFINITY;
    const float m_c = wave_max(sc);
    const float pw = lane < nvalid ? expf(sc - m_c) : 0.0f;
    const float l_c = wave_sum(pw);
    // weights to LDS in the order the V pieces want them: group g holds positions g, g + 4, g + 8, ...
    Pp[(lane & 3) * 16 + (lane >> 2)] = pw;
    __builtin_amdgcn_wave_barrier();
    asm volatile("s_waitcnt lgkmcnt(0)" ::: "memory");
    float o_c[8];
#pragma unroll
    for (int e = 0; e < 8; ++e) o_c[e] = 0.0f;
    const f32x4 *pv = reinterpret_cast<const f32x4 *>(Pp + grp * 16);
    // rows past the sequence carry weight zero, but what the cache holds there is anything: masked to zero (only a
    // chunk that the sequence ends in pays for the masks)
    if (nvalid < (uint32_t)kAttnChunk) {
#pragma unroll
      for (int it = 0; it < 16; ++it)
        if (4u * it + grp >= nvalid) vr[it] = u32x4{0, 0, 0, 0};
    }
#pragma unroll
    for (int i4 = 0; i4 < 4; ++i4) {
      const f32x4 p4 = pv[i4];
      const float pj[4] = {p4.x, p4.y, p4.z, p4.w};
#pragma unroll
      for (int u = 0; u < 4; ++u) {
        const half8_t v8 = __builtin_bit_cast(half8_t, vr[4 * i4 + u]);
#pragma unroll
        for (int e = 0; e < 8; ++e) o_c[e] = fmaf(pj[u], (float)v8[e], o_c[e]);
      }
    }
    // fold the chunk into the wave's running (max, sum, o)
    const float m_new = fmaxf(m_run, m_c);
    const float a = m_run == -INFINITY ? 0.0f : expf(m_run - m_new), b = m_c == -INFINITY ? 0.0f : expf(m_c - m_new);
    l_run = a * l_run + b * l_c;
#pragma unroll
    for (int e = 0; e < 8; ++e) o_run[e] = a * o_run[e] + b * o_c[e];
    m_run = m_new;
    __builtin_amdgcn_wave_barrier();   // the next pass overwrites Ks and Pp
  }
  // the four position groups of the wave hold shares of the same dimensions
#pragma unroll
  for (int e = 0; e < 8; ++e) {
    o_run[e] += __shfl_xor(o_run[e], 16);
    o_run[e] += __shfl_xor(o_run[e], 32);
  }
  // fold the waves: their (max, sum, o) go through LDS (each wave's own K region is free now)
  float *mine = reinterpret_cast<float *>(Ks);
  if (lane < 16) {
#pragma unroll
    for (int e = 0; e < 8; ++e) mine[2 + 8 * lane + e] = o_run[e];
  }
  if (lane == 0) {
    mine[0] = m_run;
    mine[1] = l_run;
  }
  __syncthreads();
  if (tid < HD) {
    const float *w0 = reinterpret_cast<const float *>(wide_lds);
    constexpr size_t kStride = (size_t)kAttnChunk * kAttnRow * 2 / 4;   // floats between the waves' regions
    float M = -INFINITY;
#pragma unroll
    for (int w = 0; w < 4; ++w) M = fmaxf(M, w0[w * kStride]);
    float L = 0.0f, o = 0.0f;
#pragma unroll
    for (int w = 0; w < 4; ++w) {
      const float mw = w0[w * kStride];
      const float f = mw == -INFINITY ? 0.0f : expf(mw - M);
      L = fmaf(w0[w * kStride + 1], f, L);
      o = fmaf(w0[w * kStride + 2 + tid], f, o);
    }
    float *dst = partial + ((size_t)h * nsplit + split) * (2 + HD);
    if (tid == 0) {
      dst[0] = M;
      dst[1] = L;
    }
    dst[2 + tid] = o;
  }
}

// One workgroup of 128 threads per query head: the (max, sum) pairs of the splits are taken one per lane, so the
// merge weights need two wave reductions instead of a serial walk over the splits; thread d then sums dimension d.
constexpr int kAttnMaxSplit = 1024;   // splits per head the merge kernel holds weights for (context of 65,536)

__global__ void __launch_bounds__(128) attn_merge_kernel(const float *partial, const uint32_t *params, void *out, int out_f16,
                                                         uint32_t headDim, uint32_t nsplit) {
  __shared__ float Ws[kAttnMaxSplit];
  __shared__ float red[4];
  const uint32_t h = blockIdx.x, tid = threadIdx.x;
  // every split has a record (empty ones carry max = -inf, sum = 0), so the merge does not need the sequence length
  // and its loads do not wait for it
  (void)params;
  const uint32_t used = nsplit;
  const uint32_t rec = 2 + headDim;
  const float *base = partial + (size_t)h * nsplit * rec;
  // up to 32 splits (a context of 2048): this thread's dimension of every split is requested now, together with the
  // (max, sum) pairs, so that the whole merge costs one memory round trip instead of three
  constexpr uint32_t kPre = 32;
  const bool pre = used <= kPre;
  float ov[kPre];
#pragma unroll
  for (uint32_t s = 0; s < kPre; ++s) ov[s] = (pre && s < used && tid < headDim) ? base[(size_t)s * rec + 2 + tid] : 0.0f;
  if (pre) {
    // up to 32 splits: every wave holds all (max, sum) pairs, one per lane, and folds them by itself: no LDS, no
    // workgroup barrier; the weight of split s comes out of lane s
    const uint32_t ls = tid & 63;
    const bool have = ls < used;
    const float ms = have ? base[(size_t)ls * rec] : -INFINITY, lsum = have ? base[(size_t)ls * rec + 1] : 0.0f;
    const float M = wave_max(ms);
    const float w = ms == -INFINITY ? 0.0f : expf(ms - M);   // an empty split (and an empty sequence: M = -inf) weighs nothing
    const float L = wave_sum(lsum * w);
    float o = 0.0f;   // every lane takes part in the shuffles; threads beyond the head dimension hold zeros
#pragma unroll
    for (uint32_t s = 0; s < kPre; ++s) o = fmaf(ov[s], __shfl(w, (int)s), o);
    if (tid < headDim) st_act(out, out_f16, (size_t)h * headDim + tid, L > 0.0f ? o / L : 0.0f);
    return;
  }
  float m = -INFINITY;
  for (uint32_t s = tid; s < used; s += 128) m = fmaxf(m, base[(size_t)s * rec]);
  m = wave_max(m);
  if ((tid & 63) == 0) red[tid >> 6] = m;
  __syncthreads();
  const float M = fmaxf(red[0], red[1]);
  float l = 0.0f;
  for (uint32_t s = tid; s < used; s += 128) {
    float ms = base[(size_t)s * rec];
    float w = ms == -INFINITY ? 0.0f : expf(ms - M);   // an empty split (and an empty sequence: M = -inf) weighs nothing
    Ws[s] = w;
    l = fmaf(base[(size_t)s * rec + 1], w, l);
  }
  l = wave_sum(l);
  if ((tid & 63) == 0) red[2 + (tid >> 6)] = l;
  __syncthreads();
  const float L = red[2] + red[3];
  if (tid < headDim) {
    float o = 0.0f;
#pragma unroll 8
    for (uint32_t s = 0; s < used; ++s) o = fmaf(base[(size_t)s * rec + 2 + tid], Ws[s], o);
    st_act(out, out_f16, (size_t)h * headDim + tid, L > 0.0f ? o / L : 0.0f);
  }
}

// ---- SiLU(gate) * up on the output of a fused gate+up matmul: in = [gate(n) | up(n)] ----
__global__ void __launch_bounds__(256) silu_mul_kernel(const void *in, int in_f16, void *out, int out_f16, uint32_t n) {
  uint32_t i = blockIdx.x * 256 + threadIdx.x;
  if (i >= n) return;
  float g = ld_act(in, in_f16, i), u = ld_act(in, in_f16, (size_t)n + i);
  st_act(out, out_f16, i, g / (1.0f + __expf(-g)) * u);
}

// ---- arg-max (first index of the maximum), one workgroup ----
__global__ void __launch_bounds__(1024) argmax_kernel(const void *x, int x_f16, uint32_t n, uint32_t *out) {
  __shared__ float bv[16];
  __shared__ uint32_t bi[16];
  const uint32_t tid = threadIdx.x;
  float best = -INFINITY;
  uint32_t idx = 0xFFFFFFFFu;
  auto consider = [&](float v, uint32_t i) {
    if (v > best || (v == best && i < idx)) {
      best = v;
      idx = i;
    }
  };
  // 16-byte loads, four per thread in flight: with one scalar load per trip every trip pays a memory latency
  uint32_t done = 0;
  if ((uintptr_t)x % 16 == 0) {
    const uint32_t per = x_f16 ? 8 : 4, nvec = n / per;
    const u32x4 *xv = reinterpret_cast<const u32x4 *>(x);
    for (uint32_t b = tid; b < nvec; b += 4 * 1024) {
      u32x4 v[4];
#pragma unroll
      for (int u = 0; u < 4; ++u) v[u] = xv[min(b + u * 1024, nvec - 1)];
#pragma unroll
      for (int u = 0; u < 4; ++u) {
        const uint32_t vi = b + u * 1024;
        if (vi >= nvec) break;
        if (x_f16) {
          half8_t h = __builtin_bit_cast(half8_t, v[u]);
#pragma unroll
          for (int e = 0; e < 8; ++e) consider((float)h[e], vi * 8 + e);
        } else {
          f32x4 f = __builtin_bit_cast(f32x4, v[u]);
#pragma unroll
          for (int e = 0; e < 4; ++e) consider(f[e], vi * 4 + e);
        }
      }
    }
    done = nvec * per;
  }
  for (uint32_t i = done + tid; i < n; i += 1024) consider(ld_act(x, x_f16, i), i);
#pragma unroll
  for (int o = 32; o > 0; o >>= 1) {
    float ov = __shfl_xor(best, o);
    uint32_t oi = __shfl_xor(idx, o);
    if (ov > best || (ov == best && oi < idx)) {
      best = ov;
      idx = oi;
    }
  }
  if ((tid & 63) == 0) {
    bv[tid >> 6] = best;
    bi[tid >> 6] = idx;
  }
  __syncthreads();
  if (tid == 0) {
    for (int w = 1; w < 16; ++w)
      if (bv[w] > best || (bv[w] == best && bi[w] < idx)) {
        best = bv[w];
        idx = bi[w];
      }
    out[0] = idx;
  }
}

// ---- greedy sampling after the matmul that produced the logits ----
// One workgroup.  The matmul left, per group of 8 vocabulary rows, the largest logit and its row (ArgmaxPart); this
// kernel applies the repetition penalty to the listed tokens (RepetitionPenalty.cu:19-41: logit > 0 ? logit / f :
// logit * f, written back to the logits), re-derives the groups whose winner was one of them, and reduces.  Without
// parts (parts == nullptr) it scans the logits themselves.  List semantics are those of the dense factor vector the
// runner fills (llama.cpp:2566-2592): a token listed several times is penalised once, with the factor of its last entry.
constexpr uint32_t kMaxPenalized = 1024;

__device__ inline void better(float v, uint32_t i, float &best, uint32_t &idx) {
  if (v > best || (v == best && i < idx)) {
    best = v;
    idx = i;
  }
}

__global__ void __launch_bounds__(1024) argmax_finish_kernel(const ArgmaxPart *parts, void *logits, int x_f16, uint32_t n,
                                                             const int32_t *pen_tokens, const float *pen_factors,
                                                             uint32_t n_pen, uint32_t *out) {
  __shared__ int32_t ptok[kMaxPenalized];
  __shared__ float pval[kMaxPenalized];   // the penalised logit of an effective entry
  __shared__ float bv[16];
  __shared__ uint32_t bi[16];
  const uint32_t tid = threadIdx.x;
  float best = -INFINITY;
  uint32_t idx = 0xFFFFFFFFu;
  if (tid < n_pen) ptok[tid] = pen_tokens[tid];
  __syncthreads();
  // every barrier below is reached by all threads: the per-entry work is predicated, never the barrier
  const bool mine = tid < n_pen;
  const int32_t t = mine ? ptok[tid] : -1;
  bool effective = mine && t >= 0 && (uint32_t)t < n;
  for (uint32_t k = tid + 1; effective && k < n_pen; ++k) effective = ptok[k] != t;   // a later entry of the same token wins
  float v = 0.0f;
  if (effective) {
    const float l = ld_act(logits, x_f16, (size_t)t), f = pen_factors[tid];
    v = l > 0.0f ? l / f : l * f;
    st_act(logits, x_f16, (size_t)t, v);
    if (x_f16) v = (float)(half_t)v;   // as stored
  }
  __syncthreads();            // every entry has read its token before any is marked
  if (mine) {
    if (!effective) ptok[tid] = -1;
    pval[tid] = v;
  }
  __syncthreads();
  // value of row r as the penalised logits hold it: listed rows from the table above (their stores may not be
  // visible to the other waves yet), all others from memory
  auto row_value = [&](uint32_t r) {
    for (uint32_t k = 0; k < n_pen; ++k)
      if (ptok[k] == (int32_t)r) return pval[k];
    return ld_act(logits, x_f16, (size_t)r);
  };
  if (parts) {
    const uint32_t ngroups = (n + 7) / 8;
    constexpr int kInFlight = 8;   // pairs requested together: one memory round trip per 8192 groups instead of one per 1024
    for (uint32_t g0 = tid; g0 < ngroups; g0 += 1024 * kInFlight) {
      ArgmaxPart p[kInFlight];
#pragma unroll
      for (int u = 0; u < kInFlight; ++u) p[u] = parts[min(g0 + u * 1024, ngroups - 1)];
#pragma unroll
      for (int u = 0; u < kInFlight; ++u) {
        const uint32_t g = g0 + u * 1024;
        if (g >= ngroups) break;
        bool listed = false;
        for (uint32_t k = 0; k < n_pen; ++k) listed |= ptok[k] >= 0 && ((uint32_t)ptok[k] >> 3) == g;
        if (!listed) {
          better(p[u].value, p[u].index, best, idx);
        } else {
          for (uint32_t r = g * 8; r < min(n, g * 8 + 8); ++r) better(row_value(r), r, best, idx);
        }
      }
    }
  } else {
    for (uint32_t r = tid; r < n; r += 1024) better(n_pen ? row_value(r) : ld_act(logits, x_f16, (size_t)r), r, best, idx);
  }
#pragma unroll
  for (int o = 32; o > 0; o >>= 1) {
    float ov = __shfl_xor(best, o);
    uint32_t oi = __shfl_xor(idx, o);
    better(ov, oi, best, idx);
  }
  if ((tid & 63) == 0) {
    bv[tid >> 6] = best;
    bi[tid >> 6] = idx;
  }
  __syncthreads();
  if (tid == 0) {
    for (int w = 1; w < 16; ++w) better(bv[w], bi[w], best, idx);
    out[0] = idx;
  }
}

// ---- RepetitionPenaltyOpNode on a dense factor vector (RepetitionPenalty.cu:19-41) ----
__global__ void __launch_bounds__(256) repetition_penalty_kernel(const float *logits, const float *factors, float *out, uint32_t n) {
  const uint32_t i = blockIdx.x * 256 + threadIdx.x;
  if (i >= n) return;
  const float l = logits[i], f = factors[i];
  out[i] = l > 0.0f ? l / f : l * f;
}

// ---- EmbeddingCol (operators/impl/memory/EmbeddingCol.cu:16-44): gather from a table kept column-wise ----
// format 0: fp16 table; 1: int8 table with fp16 scales per 32 dims (the loader's separated Q8_0 tensors)
__global__ void __launch_bounds__(256) embedding_col_kernel(const uint32_t *indices, const void *matrix, const uint16_t *scales,
                                                            float *out, uint32_t numIndices, uint32_t embDim,
                                                            uint32_t vocabStride, uint32_t scaleStride, uint32_t outStride,
                                                            uint32_t vocab, int format) {
  const uint32_t gid = blockIdx.x * 256 + threadIdx.x;
  if (gid >= numIndices * embDim) return;
  const uint32_t i = gid / embDim, d = gid % embDim, t = indices[i];
  float v = 0.0f;
  if (t < vocab) {   // an index past the table reads nothing and yields zero
    const size_t idx = (size_t)d * vocabStride + t;
    if (format == 0) {
      v = f16bits_to_f32(reinterpret_cast<const uint16_t *>(matrix)[idx]);
    } else {
      const int b = reinterpret_cast<const int8_t *>(matrix)[idx];
      v = (float)b * f16bits_to_f32(scales[(size_t)(d >> 5) * scaleStride + t]);
    }
  }
  out[(size_t)i * outStride + d] = v;
}

static bool bad_dtype(int d) { return d != CUTHIP_F32 && d != CUTHIP_F16; }

}  // namespace cuthip

using namespace cuthip;

extern "C" {

int cuthip_rmsnorm(const void *x, int x_dtype, const float *weight, void *out, int out_dtype, uint32_t rows, uint32_t dim,
                   uint32_t stride, float eps, void *stream) {
  if (!x || !weight || !out || rows == 0 || dim == 0 || stride < dim || bad_dtype(x_dtype) || bad_dtype(out_dtype)) {
    set_error("cuthip_rmsnorm: bad argument (rows %u, dim %u, stride %u)", rows, dim, stride);
    return CUTHIP_ERR_INVALID;
  }
  const bool xf = x_dtype == CUTHIP_F16, of = out_dtype == CUTHIP_F16;
  // 16-byte loads need rows that start on a 16-byte boundary
  const int aligned = (reinterpret_cast<uintptr_t>(x) % 16 == 0) && (stride % 8 == 0);
  auto kern = xf ? (of ? rmsnorm_kernel<true, true> : rmsnorm_kernel<true, false>)
                 : (of ? rmsnorm_kernel<false, true> : rmsnorm_kernel<false, false>);
  hipLaunchKernelGGL(kern, dim3(rows), dim3(256), 0, (hipStream_t)stream, x, weight, out, dim, stride, eps, aligned);
  return check_hip(hipGetLastError(), "rmsnorm launch");
}

int cuthip_rope_kv_write(const void *q, const void *k, const void *v, int in_dtype, const uint32_t *runtime_params,
                         const float *cos_table, const float *sin_table, void *k_cache, void *v_cache, void *q_out,
                         int q_out_dtype, uint32_t q_dim, uint32_t kv_dim, uint32_t head_dim, uint32_t aligned_kv_dim,
                         uint32_t max_positions, void *stream) {
  if (!q || !k || !v || !runtime_params || !cos_table || !sin_table || !k_cache || !v_cache || !q_out || head_dim == 0 ||
      head_dim % 2 || q_dim % head_dim || kv_dim % head_dim || aligned_kv_dim < kv_dim || bad_dtype(in_dtype) ||
      bad_dtype(q_out_dtype)) {
    set_error("cuthip_rope_kv_write: bad argument (q_dim %u, kv_dim %u, head_dim %u)", q_dim, kv_dim, head_dim);
    return CUTHIP_ERR_INVALID;
  }
  uint32_t total = q_dim + 2 * kv_dim;
  hipLaunchKernelGGL(rope_kv_kernel, dim3((total + 255) / 256), dim3(256), 0, (hipStream_t)stream, q, k, v,
                     in_dtype == CUTHIP_F16, runtime_params, cos_table, sin_table, (half_t *)k_cache, (half_t *)v_cache, q_out,
                     q_out_dtype == CUTHIP_F16, q_dim, kv_dim, head_dim, aligned_kv_dim, max_positions);
  return check_hip(hipGetLastError(), "rope launch");
}

size_t cuthip_attn_decode_workspace_bytes(uint32_t n_heads, uint32_t head_dim, uint32_t max_seq_len) {
  size_t nsplit = (max_seq_len + kAttnChunk - 1) / kAttnChunk;
  return (size_t)n_heads * nsplit * (2 + head_dim) * sizeof(float);
}

// Argument checks shared by the two attention entry points (the workspace is checked by each).
static int attn_check_args(const char *who, const void *q, int q_dtype, const void *k_cache, const void *v_cache,
                           const uint32_t *runtime_params, const void *out, int out_dtype, uint32_t n_heads,
                           uint32_t n_kv_heads, uint32_t head_dim, uint32_t aligned_kv_dim, uint32_t max_seq_len) {
  if (!q || !k_cache || !v_cache || !runtime_params || !out || n_heads == 0 || n_kv_heads == 0 || n_heads % n_kv_heads ||
      head_dim == 0 || head_dim > kAttnMaxHd || head_dim % 8 || max_seq_len == 0 || aligned_kv_dim < n_kv_heads * head_dim ||
      aligned_kv_dim % 8 || bad_dtype(q_dtype) || bad_dtype(out_dtype)) {
    set_error("%s: bad argument (heads %u/%u, head_dim %u (<= %d, multiple of 8), aligned_kv_dim %u)", who, n_heads, n_kv_heads,
              head_dim, kAttnMaxHd, aligned_kv_dim);
    return CUTHIP_ERR_INVALID;
  }
  if ((max_seq_len + kAttnChunk - 1) / kAttnChunk > (uint32_t)kAttnMaxSplit) {
    set_error("%s: max_seq_len %u exceeds %d", who, max_seq_len, kAttnMaxSplit * kAttnChunk);
    return CUTHIP_ERR_INVALID;
  }
  return CUTHIP_OK;
}

// The two launches of the split-context attention; `partial` holds cuthip_attn_decode_workspace_bytes() bytes.
static int attn_launch(const void *q, int q_dtype, const void *k_cache, const void *v_cache, const uint32_t *runtime_params,
                       void *out, int out_dtype, uint32_t n_heads, uint32_t n_kv_heads, uint32_t head_dim,
                       uint32_t aligned_kv_dim, float scale, uint32_t max_seq_len, void *partial, hipStream_t s) {
  uint32_t nsplit = (max_seq_len + kAttnChunk - 1) / kAttnChunk;
  auto partial_kernel = head_dim == 128 ? attn_partial_kernel<128> : attn_partial_kernel<0>;
  hipLaunchKernelGGL(partial_kernel, dim3(n_kv_heads, nsplit), dim3(256), 0, s, q, (const half_t *)k_cache,
                     (const half_t *)v_cache, runtime_params, aligned_kv_dim, max_seq_len, n_heads, n_kv_heads,
                     (int)(q_dtype == CUTHIP_F16), head_dim, (float *)partial, scale, nsplit);
  if (int rc = check_hip(hipGetLastError(), "attention launch")) return rc;
  hipLaunchKernelGGL(attn_merge_kernel, dim3(n_heads), dim3(128), 0, s, (const float *)partial, runtime_params, out,
                     out_dtype == CUTHIP_F16, head_dim, nsplit);
  return check_hip(hipGetLastError(), "attention merge launch");
}

int cuthip_attn_decode(const void *q, int q_dtype, const void *k_cache, const void *v_cache, const uint32_t *runtime_params,
                       void *out, int out_dtype, uint32_t n_heads, uint32_t n_kv_heads, uint32_t head_dim,
                       uint32_t aligned_kv_dim, float scale, uint32_t max_seq_len, void *workspace, size_t workspace_bytes,
                       void *stream) {
  if (int rc = attn_check_args("cuthip_attn_decode", q, q_dtype, k_cache, v_cache, runtime_params, out, out_dtype, n_heads,
                               n_kv_heads, head_dim, aligned_kv_dim, max_seq_len))
    return rc;
  if (!workspace || (uintptr_t)workspace % 4 != 0 ||
      workspace_bytes < cuthip_attn_decode_workspace_bytes(n_heads, head_dim, max_seq_len)) {
    set_error("cuthip_attn_decode: workspace of %zu bytes, need %zu", workspace ? workspace_bytes : (size_t)0,
              cuthip_attn_decode_workspace_bytes(n_heads, head_dim, max_seq_len));
    return CUTHIP_ERR_INVALID;
  }
  return attn_launch(q, q_dtype, k_cache, v_cache, runtime_params, out, out_dtype, n_heads, n_kv_heads, head_dim,
                     aligned_kv_dim, scale, max_seq_len, workspace, (hipStream_t)stream);
}

uint32_t cuthip_attn_partial_splits(uint32_t max_seq_len) {
  const uint32_t chunks = (max_seq_len + kAttnChunk - 1) / kAttnChunk;
  return chunks < (uint32_t)kAttnWideSplits ? chunks : (uint32_t)kAttnWideSplits;
}

size_t cuthip_attn_partial_bytes(uint32_t n_heads, uint32_t head_dim, uint32_t max_seq_len) {
  return (size_t)n_heads * cuthip_attn_partial_splits(max_seq_len) * (2 + head_dim) * sizeof(float);
}

int cuthip_attn_decode_partial(const void *q, int q_dtype, const void *k_cache, const void *v_cache,
                               const uint32_t *runtime_params, uint32_t n_heads, uint32_t n_kv_heads, uint32_t head_dim,
                               uint32_t aligned_kv_dim, float scale, uint32_t max_seq_len, void *records, size_t records_bytes,
                               void *stream) {
  // (the records stand in for the output in the shared checks)
  if (int rc = attn_check_args("cuthip_attn_decode_partial", q, q_dtype, k_cache, v_cache, runtime_params, records, CUTHIP_F32,
                               n_heads, n_kv_heads, head_dim, aligned_kv_dim, max_seq_len))
    return rc;
  if (head_dim != 128) {
    set_error("cuthip_attn_decode_partial: head_dim %u (the wide-split kernel is built for 128; use cuthip_attn_decode)", head_dim);
    return CUTHIP_ERR_INVALID;
  }
  if ((uintptr_t)records % 8 != 0 || records_bytes < cuthip_attn_partial_bytes(n_heads, head_dim, max_seq_len)) {
    set_error("cuthip_attn_decode_partial: records of %zu bytes, need %zu, 8-byte aligned", records_bytes,
              cuthip_attn_partial_bytes(n_heads, head_dim, max_seq_len));
    return CUTHIP_ERR_INVALID;
  }
  const uint32_t nsplit = cuthip_attn_partial_splits(max_seq_len);
  static std::once_flag lds_once;
  static int lds_rc = CUTHIP_OK;
  std::call_once(lds_once, [] {
    lds_rc = check_hip(hipFuncSetAttribute(reinterpret_cast<const void *>(attn_partial_wide_kernel),
                                           hipFuncAttributeMaxDynamicSharedMemorySize, (int)kAttnWideLds),
                       "hipFuncSetAttribute(attention LDS)");
  });
  if (lds_rc) return lds_rc;
  hipLaunchKernelGGL(attn_partial_wide_kernel, dim3(n_heads * nsplit), dim3(256), kAttnWideLds, (hipStream_t)stream, q,
                     (const half_t *)k_cache, (const half_t *)v_cache, runtime_params, aligned_kv_dim, max_seq_len, n_heads,
                     n_kv_heads, (int)(q_dtype == CUTHIP_F16), nsplit, (float *)records, scale);
  return check_hip(hipGetLastError(), "attention launch");
}

int cuthip_attn_merge(const void *records, uint32_t nsplit, uint32_t n_heads, uint32_t head_dim, void *out, int out_dtype,
                      void *stream) {
  if (!records || !out || nsplit == 0 || nsplit > (uint32_t)kAttnMaxSplit || n_heads == 0 || head_dim == 0 ||
      head_dim > (uint32_t)kAttnMaxHd || (uintptr_t)records % 4 != 0 || bad_dtype(out_dtype)) {
    set_error("cuthip_attn_merge: bad argument (splits %u (<= %d), heads %u, head_dim %u (<= %d))", nsplit, kAttnMaxSplit,
              n_heads, head_dim, kAttnMaxHd);
    return CUTHIP_ERR_INVALID;
  }
  hipLaunchKernelGGL(attn_merge_kernel, dim3(n_heads), dim3(128), 0, (hipStream_t)stream, (const float *)records,
                     (const uint32_t *)nullptr, out, out_dtype == CUTHIP_F16, head_dim, nsplit);
  return check_hip(hipGetLastError(), "attention merge launch");
}

}  // extern "C"

// ---- the attention without a caller workspace: partial results in a device array of this library ----
// One copy of the array exists on every GPU the library runs on, at its own address, until the process ends.  The
// array's name is a host-side stand-in; the device address is taken once per device with hipGetSymbolAddress.
namespace cuthip {
constexpr size_t kAttnStaticBytes = 4u << 20;   // 4 MiB: 32 heads of dimension 128 up to a cache capacity of 16,128
constexpr int kMaxDevices = 64;
static __device__ __align__(256) unsigned char scratch[kAttnStaticBytes];
static void *g_scratch_ptr[kMaxDevices];   // per device; written under g_scratch_mu
static std::mutex g_scratch_mu;

// Device address of `scratch` on the device that owns `stream` (the current device for the null stream), looked up
// on first use there with that device current; nullptr after set_error.
static void *attn_static_ptr(hipStream_t stream) {
  int cur = -1, dev = -1;
  if (check_hip(hipGetDevice(&cur), "hipGetDevice")) return nullptr;
  dev = cur;
  if (stream) {
    hipDevice_t sd = 0;
    if (check_hip(hipStreamGetDevice(stream, &sd), "hipStreamGetDevice")) return nullptr;
    dev = (int)sd;
  }
  if (dev < 0 || dev >= kMaxDevices) {
    set_error("attention scratch: device index %d beyond %d", dev, kMaxDevices);
    return nullptr;
  }
  std::lock_guard<std::mutex> lock(g_scratch_mu);
  if (!g_scratch_ptr[dev]) {
    void *ptr = nullptr;
    if (dev != cur && check_hip(hipSetDevice(dev), "hipSetDevice")) return nullptr;
    const int rc = check_hip(hipGetSymbolAddress(&ptr, HIP_SYMBOL(scratch)), "hipGetSymbolAddress(scratch)");
    if (dev != cur) (void)hipSetDevice(cur);
    if (rc) return nullptr;
    g_scratch_ptr[dev] = ptr;
  }
  return g_scratch_ptr[dev];
}

// called by cuthip_init with the chosen device current
int attn_static_setup() { return attn_static_ptr(nullptr) ? CUTHIP_OK : CUTHIP_ERR_HIP; }
}  // namespace cuthip

extern "C" {

size_t cuthip_attn_decode_static_max_bytes(void) { return kAttnStaticBytes; }


int cuthip_attn_decode_static(const void *q, int q_dtype, const void *k_cache, const void *v_cache,
                              const uint32_t *runtime_params, void *out, int out_dtype, uint32_t n_heads, uint32_t n_kv_heads,
                              uint32_t head_dim, uint32_t aligned_kv_dim, float scale, uint32_t max_seq_len, void *stream) {
  if (int rc = attn_check_args("cuthip_attn_decode_static", q, q_dtype, k_cache, v_cache, runtime_params, out, out_dtype,
                               n_heads, n_kv_heads, head_dim, aligned_kv_dim, max_seq_len))
    return rc;
  const size_t need = cuthip_attn_decode_workspace_bytes(n_heads, head_dim, max_seq_len);
  if (need > kAttnStaticBytes) {
    set_error("cuthip_attn_decode_static: %u heads of dimension %u over a cache of %u positions need %zu bytes of partial "
              "results, the built-in scratch holds %zu; use cuthip_attn_decode with a workspace", n_heads, head_dim,
              max_seq_len, need, kAttnStaticBytes);
    return CUTHIP_ERR_INVALID;
  }
  void *ptr = attn_static_ptr((hipStream_t)stream);
  if (!ptr) return CUTHIP_ERR_HIP;
  // every split record of this call's launch shape is written before the merge reads it, so nothing of an earlier
  // call's contents is read and nothing needs clearing
  return attn_launch(q, q_dtype, k_cache, v_cache, runtime_params, out, out_dtype, n_heads, n_kv_heads, head_dim,
                     aligned_kv_dim, scale, max_seq_len, ptr, (hipStream_t)stream);
}

int cuthip_silu_mul(const void *gate_up, int in_dtype, void *out, int out_dtype, uint32_t n, void *stream) {
  if (!gate_up || !out || n == 0 || bad_dtype(in_dtype) || bad_dtype(out_dtype)) {
    set_error("cuthip_silu_mul: bad argument");
    return CUTHIP_ERR_INVALID;
  }
  hipLaunchKernelGGL(silu_mul_kernel, dim3((n + 255) / 256), dim3(256), 0, (hipStream_t)stream, gate_up,
                     in_dtype == CUTHIP_F16, out, out_dtype == CUTHIP_F16, n);
  return check_hip(hipGetLastError(), "silu_mul launch");
}

int cuthip_argmax(const void *x, int x_dtype, uint32_t n, uint32_t *out_index, void *stream) {
  if (!x || !out_index || n == 0 || bad_dtype(x_dtype)) {
    set_error("cuthip_argmax: bad argument");
    return CUTHIP_ERR_INVALID;
  }
  hipLaunchKernelGGL(argmax_kernel, dim3(1), dim3(1024), 0, (hipStream_t)stream, x, x_dtype == CUTHIP_F16, n, out_index);
  return check_hip(hipGetLastError(), "argmax launch");
}

}  // extern "C"

extern "C" {

int cuthip_argmax_penalized(void *logits, int x_dtype, uint32_t n, const int32_t *pen_tokens, const float *pen_factors,
                            uint32_t n_pen, uint32_t *out_index, void *stream) {
  if (!logits || !out_index || n == 0 || bad_dtype(x_dtype) || n_pen > kMaxPenalized || (n_pen && (!pen_tokens || !pen_factors))) {
    set_error("cuthip_argmax_penalized: bad argument (n %u, %u penalised tokens, at most %u)", n, n_pen, kMaxPenalized);
    return CUTHIP_ERR_INVALID;
  }
  hipLaunchKernelGGL(argmax_finish_kernel, dim3(1), dim3(1024), 0, (hipStream_t)stream, (const ArgmaxPart *)nullptr, logits,
                     x_dtype == CUTHIP_F16, n, pen_tokens, pen_factors, n_pen, out_index);
  return check_hip(hipGetLastError(), "argmax launch");
}

int cuthip_repetition_penalty(const float *logits, const float *factors, float *out, uint32_t n, void *stream) {
  if (!logits || !factors || !out) {
    set_error("cuthip_repetition_penalty: null argument");
    return CUTHIP_ERR_INVALID;
  }
  if (n == 0) return CUTHIP_OK;
  hipLaunchKernelGGL(repetition_penalty_kernel, dim3((n + 255) / 256), dim3(256), 0, (hipStream_t)stream, logits, factors, out, n);
  return check_hip(hipGetLastError(), "repetition penalty launch");
}

int cuthip_embedding_col(const uint32_t *indices, const void *matrix, const uint16_t *scales, float *out, uint32_t num_indices,
                         uint32_t emb_dim, uint32_t vocab_stride, uint32_t scale_stride, uint32_t out_stride, uint32_t vocab,
                         int format, void *stream) {
  if (!indices || !matrix || !out || (format != 0 && format != 1) || (format == 1 && !scales) || out_stride < emb_dim ||
      vocab > vocab_stride || (format == 1 && vocab > scale_stride) || (uint64_t)num_indices * emb_dim > 0xFFFFFFFFull) {
    set_error("cuthip_embedding_col: bad argument (format %d, emb_dim %u, vocab %u, strides %u %u %u)", format, emb_dim, vocab,
              vocab_stride, scale_stride, out_stride);
    return CUTHIP_ERR_INVALID;
  }
  const uint32_t total = num_indices * emb_dim;
  if (total == 0) return CUTHIP_OK;
  hipLaunchKernelGGL(embedding_col_kernel, dim3((total + 255) / 256), dim3(256), 0, (hipStream_t)stream, indices, matrix, scales,
                     out, num_indices, emb_dim, vocab_stride, scale_stride, out_stride, vocab, format);
  return check_hip(hipGetLastError(), "embedding launch");
}

}  // extern "C"

namespace cuthip {
// second launch of cuthip_matmul_gguf_argmax (gemv.hip): arguments validated there
int launch_argmax_finish(const ArgmaxPart *parts, void *logits, int x_f16, uint32_t n, const int32_t *pen_tokens,
                         const float *pen_factors, uint32_t n_pen, uint32_t *out_index, hipStream_t stream) {
  hipLaunchKernelGGL(argmax_finish_kernel, dim3(1), dim3(1024), 0, stream, parts, logits, x_f16, n, pen_tokens, pen_factors,
                     n_pen, out_index);
  return check_hip(hipGetLastError(), "argmax launch");
}
uint32_t max_penalized() { return kMaxPenalized; }
}  // namespace cuthip
