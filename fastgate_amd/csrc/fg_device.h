// Device-side building blocks shared by the gfx950 kernels: vector types, 16-byte global
// loads, packed-fp16 dot products with fp32 accumulation, wave64 DPP reductions.
#pragma once
#include <hip/hip_runtime.h>
#include <stdint.h>

#include "fg_flags.h"

namespace fg {

typedef _Float16 half_t;
typedef _Float16 half2_t __attribute__((ext_vector_type(2)));
typedef _Float16 half8_t __attribute__((ext_vector_type(8)));
typedef float float4_t __attribute__((ext_vector_type(4)));
typedef uint32_t u32x4 __attribute__((ext_vector_type(4)));
typedef uint32_t u32x2 __attribute__((ext_vector_type(2)));

constexpr int kWave = 64;

// 16-byte global load.  STREAM marks data that is read exactly once (the weights) with the
// non-temporal hint so it does not displace the activation panel from the caches.
template <bool STREAM>
__device__ __forceinline__ u32x4 load16(const void* p) {
  if constexpr (STREAM) {
    return __builtin_nontemporal_load(reinterpret_cast<const u32x4*>(p));
  } else {
    return *reinterpret_cast<const u32x4*>(p);
  }
}

__device__ __forceinline__ half2_t as_half2(uint32_t v) { return __builtin_bit_cast(half2_t, v); }
__device__ __forceinline__ half8_t as_half8(u32x4 v) { return __builtin_bit_cast(half8_t, v); }

// acc + Σ_{i<8} w_i·x_i: four v_dot2_f32_f16, products and sum kept in fp32.
__device__ __forceinline__ float dot8(u32x4 w, u32x4 x, float acc) {
  acc = __builtin_amdgcn_fdot2(as_half2(w.x), as_half2(x.x), acc, false);
  acc = __builtin_amdgcn_fdot2(as_half2(w.y), as_half2(x.y), acc, false);
  acc = __builtin_amdgcn_fdot2(as_half2(w.z), as_half2(x.z), acc, false);
  acc = __builtin_amdgcn_fdot2(as_half2(w.w), as_half2(x.w), acc, false);
  return acc;
}

template <int CTRL>
__device__ __forceinline__ float dpp_f32(float v) {
  return __builtin_bit_cast(
      float, __builtin_amdgcn_update_dpp(0, __builtin_bit_cast(int, v), CTRL, 0xf, 0xf, true));
}
template <int CTRL>
__device__ __forceinline__ int dpp_i32(int v) {
  return __builtin_amdgcn_update_dpp(0, v, CTRL, 0xf, 0xf, true);
}

// Sum over each DPP row (16 consecutive lanes); every lane of the row ends with the row sum.
// quad_perm[1,0,3,2], quad_perm[2,3,0,1], row_half_mirror, row_mirror.
__device__ __forceinline__ float row16_allreduce(float v) {
  v += dpp_f32<0xB1>(v);
  v += dpp_f32<0x4E>(v);
  v += dpp_f32<0x141>(v);
  v += dpp_f32<0x140>(v);
  return v;
}
__device__ __forceinline__ int row16_allreduce(int v) {
  v += dpp_i32<0xB1>(v);
  v += dpp_i32<0x4E>(v);
  v += dpp_i32<0x141>(v);
  v += dpp_i32<0x140>(v);
  return v;
}

__device__ __forceinline__ uint16_t f32_to_f16_bits(float v) {
  return __builtin_bit_cast(uint16_t, static_cast<half_t>(v));
}
__device__ __forceinline__ float f16_bits_to_f32(uint16_t b) {
  return static_cast<float>(__builtin_bit_cast(half_t, b));
}

// First K step of a workgroup whose waves walk K in `nsteps` steps (wrapping around).
// Weight rows are K*2 bytes apart -- a power of two for the usual K -- so workgroups that
// walk K in lockstep sit on the same HBM and L2 channels at the same time.  Workgroups are
// dealt to the 8 XCDs round-robin by linear id; numbering them within their XCD (id / 8)
// spreads the start positions evenly over each XCD's L2 channels as well as over the chip
// (starting at id % nsteps instead leaves each XCD on 1/8 of the positions: 2.2x slower at
// K = 8192 with 16 steps).
// Flag bit 1 selects id % nsteps: with exactly 8 steps every XCD then owns one K band at a time,
// which measured 9% faster at K = N = 8192 and must not be used with other step counts.
__device__ __forceinline__ int stagger_start(int nsteps, int flags) {
  const unsigned lid = blockIdx.x + gridDim.x * (blockIdx.y + gridDim.y * blockIdx.z);
  return (int)(((flags & 2) ? lid : (lid >> 3)) % (unsigned)nsteps);
}

// Σ_{p < np} base[p * stride], p ascending, with all MAXP reads issued before the first add.  A loop
// to a run-time bound compiles to read, wait, add per term: up to 32 dependent LDS round trips at
// the end of every workgroup.  Terms past np re-read term 0 and add +0.
template <int MAXP>
__device__ __forceinline__ float lds_sum(const float* base, int stride, int np) {
  float v[MAXP];
#pragma unroll
  for (int p = 0; p < MAXP; ++p) v[p] = base[(p < np ? p : 0) * stride];
  float s = 0.f;
#pragma unroll
  for (int p = 0; p < MAXP; ++p) s += p < np ? v[p] : 0.f;
  return s;
}
__device__ __forceinline__ int lds_sum_i32(const int* base, int stride, int np) {
  int v[16];
#pragma unroll
  for (int p = 0; p < 16; ++p) v[p] = base[(p < np ? p : 0) * stride];
  int s = 0;
#pragma unroll
  for (int p = 0; p < 16; ++p) s += p < np ? v[p] : 0;
  return s;
}

// Orders LDS traffic among the lanes of one wavefront (data handed from lane to lane through
// a wave-private LDS region).  The LDS unit serves a wave's requests in order; this only keeps
// the compiler from moving the accesses across the hand-over point.  No s_barrier is issued.
__device__ __forceinline__ void wave_lds_sync() {
  __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront");
  __builtin_amdgcn_wave_barrier();
  __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "wavefront");
}

// ---------------------------------------------------------------------------------------
// Split-K completion inside one launch.  Every workgroup of a tile stores its fp32 partial
// to part[z][m][n], then arrives at the tile's counter; the workgroup that arrives last sums
// the S partials in ascending z (so the result does not depend on arrival order), writes C
// and puts the counter back to zero for the next call.  The only atomic RMW is on the counter.
//
// The workgroups of a tile run on different XCDs, whose L2s are not coherent with each other.
// Agent-scope fences would fix that by writing back / invalidating a whole L2 (measured: 2-8x
// slower kernels), so the partials never live in L2 instead: they are written and read with
// relaxed agent-scope atomic accesses (write-through stores, L2-bypassing loads), and every wave
// waits for the acknowledgement of its stores (an explicit s_waitcnt vmcnt(0)) before the barrier
// that precedes the counter update.
// ---------------------------------------------------------------------------------------
__device__ __forceinline__ void store_partial(float* p, float v, bool coherent) {
  if (coherent) __hip_atomic_store(p, v, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
  else *p = v;
}
__device__ __forceinline__ float load_partial(const float* p) {
  return __hip_atomic_load(p, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
}

// 16-byte forms of the same two accesses (HIP has no 16-byte atomics): raw buffer accesses on
// the partials buffer with the agent-scope cache policy bit (sc1) -- the encoding the 4-byte
// agent-scope atomics above compile to, four columns per instruction instead of one.  `idx` is
// the element index into `base`, a multiple of 4; the buffer is at most 2 GiB.
constexpr int kCachePolicyAgent = 16;  // sc1
__device__ __forceinline__ __amdgpu_buffer_rsrc_t partials_rsrc(const float* base) {
  return __builtin_amdgcn_make_buffer_rsrc(const_cast<float*>(base), 0, 0x7fffffff, 0x00020000);
}
__device__ __forceinline__ void store_partial4(float* base, size_t idx, float4_t v, bool coherent) {
  if (coherent) {
    __builtin_amdgcn_raw_buffer_store_b128(__builtin_bit_cast(u32x4, v), partials_rsrc(base),
                                           (int)(idx * 4), 0, kCachePolicyAgent);
  } else {
    *reinterpret_cast<float4_t*>(base + idx) = v;
  }
}
__device__ __forceinline__ float4_t load_partial4(const float* base, size_t idx) {
  return __builtin_bit_cast(float4_t, __builtin_amdgcn_raw_buffer_load_b128(
                                          partials_rsrc(base), (int)(idx * 4), 0, kCachePolicyAgent));
}

// ---------------------------------------------------------------------------------------
// Value written to C.  The flag word of a launch: bit 0 C += (accumulate), bit 1 start stagger
// of the [N,K] kernels, bit 4 add bias[n] (fp16, one per output column), bits 5-7 activation
// (FG_ACT_*).  Bias and activation are applied in fp32 to the finished sum, before the single
// rounding to fp16.
// ---------------------------------------------------------------------------------------
__device__ __forceinline__ float activate(float v, int act) {
  switch (act) {
    case FG_ACT_RELU: return v > 0.f ? v : 0.f;
    case FG_ACT_GELU: return 0.5f * v * (1.f + erff(v * 0.70710678118654752f));
    case FG_ACT_GELU_TANH: {
      const float u = 0.79788456080286536f * (v + 0.044715f * v * v * v);
      return 0.5f * v * (1.f + tanhf(u));
    }
    case FG_ACT_SILU: return v / (1.f + __expf(-v));
    default: return v;
  }
}
__device__ __forceinline__ float apply_tail(float v, int n, const void* bias, int flags) {
  if (flags & kFlagTailMask) {
    if (flags & kFlagBias) v += static_cast<float>(static_cast<const half_t*>(bias)[n]);
    v = activate(v, (flags >> kFlagActShift) & 7);
  }
  return v;
}
__device__ __forceinline__ half_t finish_value(float sum, const half_t* c, int n, const void* bias,
                                               int flags) {
  if (flags & kFlagAccumulate) sum += static_cast<float>(*c);
  return static_cast<half_t>(apply_tail(sum, n, bias, flags));
}

__device__ __forceinline__ bool splitk_last_arriver(int* counter, int S) {
  __shared__ int s_last;
  // Every wave waits until its own partial stores are acknowledged (write-through: they are in
  // memory then) before the barrier that precedes the arrival.  The workgroup-scope release
  // alone does not do that: the waves of a workgroup share a CU, so the compiler emits no wait
  // for it, and an arrival could overtake a partial on its way through another L2 channel.
  __builtin_amdgcn_fence(__ATOMIC_RELEASE, "workgroup");
  // s_waitcnt immediate of gfx9 (gfx950 included): vmcnt in bits 3:0 and 15:14, expcnt in 6:4,
  // lgkmcnt in 11:8.  vmcnt = 0 waits for every outstanding vector-memory access of the wave; the
  // other two counters are left at their largest value, which waits for nothing.
  constexpr int kVmcnt = 0, kExpcntNoWait = 7, kLgkmcntNoWait = 15;
  constexpr int kWaitStores = (kVmcnt & 15) | (kExpcntNoWait << 4) | (kLgkmcntNoWait << 8) | ((kVmcnt >> 4) << 14);
  static_assert(kWaitStores == 0x0F70, "s_waitcnt vmcnt(0) in the gfx9 encoding");
  __builtin_amdgcn_s_waitcnt(kWaitStores);
  __syncthreads();
  if (threadIdx.x == 0) {
    const int old = __hip_atomic_fetch_add(counter, 1, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
    const int last = old == S - 1;
    if (last) __hip_atomic_store(counter, 0, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
    s_last = last;
  }
  __syncthreads();
  __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "workgroup");
  return s_last != 0;
}

// ---------------------------------------------------------------------------------------
// Split-K completion in one memory round trip.  Every output element owns one 64-bit word
// (zero between calls).  A workgroup adds its fp32 partial, converted to fixed point, together
// with an arrival count in the low bits, using one relaxed agent-scope atomic add that returns
// the previous word.  The thread whose add returns S - 1 previous arrivals holds, in
// (previous + own), the complete sum of that element: it writes C and puts the word back to
// zero.  Integer addition is associative, so the sum does not depend on arrival order; all
// communication goes through the one atomic word, so no ordering between different locations is
// needed (no fence, no write-through wait, no counter, no barrier), and different elements of a
// tile may be completed by different workgroups.
//   word = value (54 bits, two's complement, units of 2^-28) | poisoned arrivals (5) | arrivals (5)
// A partial that fixed point cannot hold (NaN, infinite, or |p| >= 2^20, sixteen times the fp16
// range) arrives "poisoned": value 0, the fp32 partial itself stored in its slot [z][m][n] of the
// partial area behind the header, and bit z set in a second word of the element, both before the
// arrival, with release / acquire fences around the pair (that path alone pays for agent-scope
// fences and for memory beyond the header).  The thread that completes a poisoned element adds the
// flagged partials in ascending z, in fp32, to the fixed-point sum of the others: two huge
// partials of opposite sign cancel as they do in every other completion, and NaN and the
// infinities follow from fp32 arithmetic.
// ---------------------------------------------------------------------------------------
constexpr float kFixLimit = 1048576.f;  // 2^20

// Fixed-point image of p (|p| < 2^20) in units of 2^-28, rounded to nearest: exact for every fp32
// value of magnitude 2^-4 or more, off by at most 2^-29 below (the smallest fp16 step is 2^-24).
__device__ __forceinline__ int64_t fix_from_float(float p) {
  const float scaled = p * 16.f;                         // exact
  const float hi = __builtin_floorf(scaled);             // |hi| <= 2^24, an integer
  const float lo = __builtin_rintf((scaled - hi) * 16777216.f);  // [0, 2^24], exact difference
  return ((int64_t)(int)hi << 24) + (int64_t)(int)lo;
}
// Correctly rounded fp32 value of v * 2^-28 (|v| < 2^53).
__device__ __forceinline__ float fix_to_float(int64_t v) {
  const double d = (double)(int)(v >> 24) * 16777216.0 + (double)(int)(v & 0xFFFFFF);
  return (float)d * 3.7252902984619140625e-09f;          // 2^-28
}
// True for a partial that must arrive poisoned (the comparison is false for NaN).
__device__ __forceinline__ bool fix_poisoned(float p) { return !(__builtin_fabsf(p) < kFixLimit); }
// Word a partial arrives with.
__device__ __forceinline__ uint64_t fix_word(float p, bool poisoned) {
  if (poisoned) return (1ull << 5) | 1ull;
  return ((uint64_t)fix_from_float(p) << 10) | 1ull;
}

// NB elements of one thread: partial p[i] of output element idx[i] (= m * N + n) from K range z
// arrives; the atomics of the batch are issued back to back before the first result is looked
// at.  `part` is the partial area ([S][MN] floats), touched for poisoned partials only; `maskw`
// holds one word per element (bit z: slot z of the element holds a poisoned partial).
template <int NB>
__device__ __forceinline__ void fix_arrive(uint64_t* acc, uint32_t* maskw, float* part, int z, size_t MN,
                                           const size_t (&idx)[NB], const float (&p)[NB],
                                           const bool (&valid)[NB], int S, half_t* C, int N,
                                           const void* bias, int flags) {
  uint64_t own[NB], old[NB];
#pragma unroll
  for (int i = 0; i < NB; ++i) {
    const bool poisoned = fix_poisoned(p[i]);
    own[i] = fix_word(p[i], poisoned);
    if (valid[i] && poisoned) {
      __hip_atomic_store(part + (size_t)z * MN + idx[i], p[i], __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
      __hip_atomic_fetch_or(maskw + idx[i], 1u << z, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
      __builtin_amdgcn_fence(__ATOMIC_RELEASE, "agent");
    }
  }
#pragma unroll
  for (int i = 0; i < NB; ++i)
    old[i] = valid[i] ? __hip_atomic_fetch_add(acc + idx[i], own[i], __ATOMIC_RELAXED,
                                               __HIP_MEMORY_SCOPE_AGENT)
                      : 0ull;
#pragma unroll
  for (int i = 0; i < NB; ++i) {
    if (!valid[i] || (int)(old[i] & 31u) != S - 1) continue;
    const uint64_t word = old[i] + own[i];
    float total = fix_to_float((int64_t)word >> 10);
    if ((word >> 5) & 31u) {
      __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "agent");
      uint32_t mask = __hip_atomic_load(maskw + idx[i], __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
      __hip_atomic_store(maskw + idx[i], 0u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
      float huge = 0.f;
      while (mask) {
        const int zz = __builtin_ctz(mask);
        mask &= mask - 1u;
        huge += __hip_atomic_load(part + (size_t)zz * MN + idx[i], __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
      }
      total += huge;
    }
    __hip_atomic_store(acc + idx[i], 0ull, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
    half_t* c = C + idx[i];
    *c = finish_value(total, c, (int)(idx[i] % (size_t)N), bias, flags);
  }
}

// Arrival of a workgroup at its tile's counter; the ordering is splitk_last_arriver's.  Returns 1 to
// the workgroup that arrives last (which has put the counter back to zero), 0 to the others.
__device__ __forceinline__ int splitk_arrive(int* counter, int S, int* s_word) {
  __builtin_amdgcn_fence(__ATOMIC_RELEASE, "workgroup");
  __builtin_amdgcn_s_waitcnt(0x0F70);  // vmcnt(0): this wave's partial stores are acknowledged
  __syncthreads();
  if (threadIdx.x == 0) {
    const int old = __hip_atomic_fetch_add(counter, 1, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
    const bool last = old == S - 1;
    if (last) __hip_atomic_store(counter, 0, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
    *s_word = last ? 1 : 0;
  }
  __syncthreads();
  __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "workgroup");
  return *s_word;
}

// 16 bytes of a partial that a workgroup of the same XCD stored with an ordinary store, served by
// the XCD's L2, where that store landed.  A workgroup-scope load (sc0) may be answered by this CU's
// L1 when the line is there, so the caller must be the first on its CU to touch the line since the
// kernel began (a kernel starts with the L1 invalidated): read a partial once, after its flag, and
// never poll with this load -- the second poll would see the first one's line for ever.
__device__ __forceinline__ float4_t load_partial4_l2(const float* base, size_t idx) {
  constexpr int kCachePolicyWorkgroup = 1;  // sc0
  return __builtin_bit_cast(float4_t, __builtin_amdgcn_raw_buffer_load_b128(
                                          partials_rsrc(base), (int)(idx * 4), 0, kCachePolicyWorkgroup));
}
// NQ groups of a thread at once: sum[q] = Σ_z part[z][off[q]..+3], z ascending; the loads of all groups
// of a batch of partials are in flight together.  Slots past S re-read the last partial and add +0.
// Offsets are bytes: the lane's own in the vector offset, z * (bytes of one partial) in the scalar
// offset of the buffer load, so a load costs one instruction (the buffer is below 2 GiB).
template <int NQ, int BATCH, bool MEM>
__device__ __forceinline__ void sum_partials_z_batched(const float* part, int S, int z_bytes, const int (&off)[NQ],
                                                       float4_t (&sum)[NQ]) {
  constexpr int kPolicy = MEM ? kCachePolicyAgent : 1;  // sc1: past the L2s; sc0: this XCD's L2 (see load_partial4_l2)
  const __amdgpu_buffer_rsrc_t rsrc = partials_rsrc(part);
#pragma unroll
  for (int q = 0; q < NQ; ++q) sum[q] = float4_t{0.f, 0.f, 0.f, 0.f};
  for (int z0 = 0; z0 < S; z0 += BATCH) {
    float4_t v[NQ][BATCH];
#pragma unroll
    for (int u = 0; u < BATCH; ++u) {
      const int z = z0 + u < S ? z0 + u : S - 1;
#pragma unroll
      for (int q = 0; q < NQ; ++q)
        v[q][u] = __builtin_bit_cast(float4_t, __builtin_amdgcn_raw_buffer_load_b128(rsrc, off[q], z * z_bytes, kPolicy));
    }
#pragma unroll
    for (int u = 0; u < BATCH; ++u) {
      const float4_t zero = {0.f, 0.f, 0.f, 0.f};
#pragma unroll
      for (int q = 0; q < NQ; ++q) sum[q] += z0 + u < S ? v[q][u] : zero;
    }
  }
}
template <int NQ, bool MEM>
__device__ __forceinline__ void sum_partials_z(const float* part, int S, int z_bytes, const int (&off)[NQ],
                                               float4_t (&sum)[NQ]) {
  if (S <= 4) sum_partials_z_batched<NQ, 4, MEM>(part, S, z_bytes, off, sum);
  else sum_partials_z_batched<NQ, 8, MEM>(part, S, z_bytes, off, sum);
}

// Σ_z part[z][off..off+3] in ascending z.  The loads of a batch are all issued before the first
// add: one memory round trip per batch instead of one per partial (a plain `for z` loop compiles
// to load, wait, add).  Slots past S re-read the last partial and contribute +0, which leaves
// every sum unchanged (a sum that started from +0 is never -0).
template <int BATCH>
__device__ __forceinline__ float4_t sum_partials_batched(const float* part, int S, size_t MN,
                                                         size_t off) {
  float4_t sum = {0.f, 0.f, 0.f, 0.f};
  for (int z0 = 0; z0 < S; z0 += BATCH) {
    float4_t v[BATCH];
#pragma unroll
    for (int u = 0; u < BATCH; ++u) {
      const int z = z0 + u < S ? z0 + u : S - 1;
      v[u] = load_partial4(part, (size_t)z * MN + off);
    }
#pragma unroll
    for (int u = 0; u < BATCH; ++u) {
      const float4_t zero = {0.f, 0.f, 0.f, 0.f};
      sum += z0 + u < S ? v[u] : zero;
    }
  }
  return sum;
}
// DEEP: splits beyond four are common for the caller ([K,N] kernels), worth eight or sixteen loads
// in flight and the registers they take.
template <bool DEEP>
__device__ __forceinline__ float4_t sum_partials(const float* part, int S, size_t MN, size_t off) {
  if constexpr (DEEP) {
    if (S > 8) return sum_partials_batched<16>(part, S, MN, off);
    if (S > 4) return sum_partials_batched<8>(part, S, MN, off);
  }
  return sum_partials_batched<4>(part, S, MN, off);
}

// C[m0..m0+mcnt)[n0..n0+ncnt) = fp16( Σ_z part[z] (+ C) ); ncnt and n0 are multiples of 4.
template <bool DEEP>
__device__ __forceinline__ void splitk_reduce_tile(const float* part, half_t* C, int S, int M, int N,
                                                   int m0, int mcnt, int n0, int ncnt,
                                                   int flags, const void* bias) {
  typedef half_t half4v __attribute__((ext_vector_type(4)));
  const int nq = ncnt >> 2;
  const size_t MN = (size_t)M * N;
  for (int e = threadIdx.x; e < mcnt * nq; e += blockDim.x) {
    const int m = m0 + e / nq, n = n0 + (e % nq) * 4;
    if (m >= M) continue;
    const size_t off = (size_t)m * N + n;
    const float4_t sum0 = sum_partials<DEEP>(part, S, MN, off);
    float4_t sum = sum0;
    half4v* c = reinterpret_cast<half4v*>(C + off);
    if (flags & kFlagAccumulate) {
      const half4v old = *c;
#pragma unroll
      for (int k = 0; k < 4; ++k) sum[k] += static_cast<float>(old[k]);
    }
    half4v out;
#pragma unroll
    for (int k = 0; k < 4; ++k) out[k] = static_cast<half_t>(apply_tail(sum[k], n + k, bias, flags));
    *c = out;
  }
}

// One element's partial of a split launch: to its slot of the workspace (second kernel or counter
// protocol), or straight into the element's accumulator word (atomic protocol).
__device__ __forceinline__ void publish_partial(float* ws, int* counters, half_t* C, int M, int N,
                                                int mg, int n, float sum, int flags, const void* bias) {
  if (flags & kFlagFixSplit) {
    uint64_t* facc = reinterpret_cast<uint64_t*>(reinterpret_cast<unsigned char*>(counters) + kWsCounterBytes);
    uint32_t* fcls = reinterpret_cast<uint32_t*>(facc + kWsAccElems);
    const size_t idx[1] = {(size_t)mg * N + n};
    const float part[1] = {sum};
    const bool valid[1] = {true};
    fix_arrive<1>(facc, fcls, ws, (int)blockIdx.z, (size_t)M * N, idx, part, valid, gridDim.z, C, N, bias, flags);
  } else {
    store_partial(ws + ((size_t)blockIdx.z * M + mg) * N + n, sum, counters != nullptr);
  }
}

// Shared tail of every GEMM kernel: the workgroup has stored its fp32 partial of the tile
// (m0.., n0..) when gridDim.z > 1; with counters it also completes the split-K sum in place,
// without counters a second kernel does.
template <int MROWS, int NCOLS, bool DEEP = false>
__device__ __forceinline__ void finish_splitk(float* ws, int* counters, half_t* C, int M, int N,
                                              int m0, int n0, int flags, const void* bias,
                                              int tile_x = -1) {
  if (tile_x < 0) tile_x = blockIdx.x;
  if (gridDim.z > 1 && counters != nullptr && !(flags & kFlagFixSplit)) {
    if (splitk_last_arriver(counters + blockIdx.y * gridDim.x + tile_x, gridDim.z))
      splitk_reduce_tile<DEEP>(ws, C, gridDim.z, M, N, m0, MROWS, n0, NCOLS, flags, bias);
  }
}

}  // namespace fg
