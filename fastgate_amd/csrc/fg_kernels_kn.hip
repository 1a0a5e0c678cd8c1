// fp16 kernels for weights stored [K,N] (row k holds the weights of every output column).
//
// A 16-byte load of a [K,N] matrix yields 8 neighbouring columns at one k, while both
// v_dot2_f32_f16 and the MFMA B operand want neighbouring k for one column.  Each lane
// therefore owns an 8(k) x 8(n) block per step: 8 loads from 8 consecutive rows, then 32
// v_perm_b32 transpose it in registers into 8 columns x 4 registers of k-pairs.  No LDS is
// used for the weights.  Lane l = (j = l%16, g = l/16): columns n0+8j..+7 (16 lanes cover
// 256 contiguous bytes of a row), rows 32*unit+8g..+7.  Workgroup tile = 128 columns;
// waves (and gridDim.z workgroups) interleave over K and meet in LDS / the workspace.
//
// Replaces the device side of eed_hgemm_m8n128k64x4_v7 / _v8 (backend/cuda/hk/edgemm.cuh:
// 1669-1868, 1873-2049), eed_hgemm_m8n256k32x8 (:2241-2414) and the flat_gemm kernels
// (backend/cuda/hk/flatgemm.cuh:18-915) of the reference.
#include "fg_device.h"
#include "fg_internal.h"
#include <atomic>

namespace fg {

constexpr uint32_t kSelLo = 0x05040100u;  // (lo16 of S1, lo16 of S0)
constexpr uint32_t kSelHi = 0x07060302u;  // (hi16 of S1, hi16 of S0)

// rows[i] = 8 columns of row k0+i  ->  bt[c] = 8 consecutive k of column c (4 k-pairs).
__device__ __forceinline__ void transpose8x8(const u32x4 (&rows)[8], u32x4 (&bt)[8]) {
#pragma unroll
  for (int p = 0; p < 4; ++p) {
#pragma unroll
    for (int c = 0; c < 4; ++c) {
      const uint32_t even = rows[2 * p][c], odd = rows[2 * p + 1][c];
      bt[2 * c][p] = __builtin_amdgcn_perm(odd, even, kSelLo);
      bt[2 * c + 1][p] = __builtin_amdgcn_perm(odd, even, kSelHi);
    }
  }
}

// Column tile of workgroup (x, z).  All bytes a workgroup has in flight sit in one 256-byte column
// band, i.e. at one offset within 1 KB whenever the rows are a multiple of 1 KB apart, and the
// memory system serves such a CU measurably slower (N = 8192: 9 % against rows 8192 + 128 apart).
// Workgroups that share a CU therefore take neighbouring bands: the grid fills the CUs plane by
// plane (x fastest), so every z plane is shifted by the number of full rounds of 256 workgroups
// dispatched before it.  Each plane still covers every tile once, so a tile keeps one workgroup
// per z.  K = N = 8192, M = 1 (512 workgroups): 24.2 -> 23.1 us; one workgroup a CU: unchanged.
__device__ __forceinline__ int kn_tile(int x, int z, int gx, int cus) {
  const int round = (int)((z * gx * gridDim.y) / cus);
  return (x + round) % gx;
}

// ---------------------------------------------------------------------------------------
// MFMA variant.  The weights are the MFMA's first operand (rows of the 16 x 16 result = columns
// of W) and the activations its second, so the result comes out transposed: MFMA i of a step owns
// the columns n0 + 8*jj + i (jj = row of the result) and lane (j, g) ends up with
//   acc[i][r] = C[m = j][n = n0 + 32g + 8r + i],
// 32 consecutive columns of one row of C.  That makes every later step row-shaped: 16-byte LDS
// writes and reads, 16-byte partial stores that fill whole 512-byte rows, 8-byte stores to C.
//
// Work items (column tile, K split z, row block y) come from a one-dimensional grid:
//  * plain order: x fastest, every z plane shifted by the rounds of CUs dispatched before it
//    (kn_tile's rule);
//  * XCD-local order (kFlagXcdLocal): the hardware deals the workgroups of a launch to the XCDs
//    round-robin in the order of their linear ids, starting at an XCD that depends on what was
//    launched before (measured: XCC id == (id + c) % xccs for every workgroup of a launch, c
//    constant within it and changing between launches, also between the nodes of a graph).  Ids
//    that are equal modulo xccs therefore share an XCD whatever c is.  Every residue class is
//    handed a contiguous run of column tiles and all S workgroups of a tile get ids of that
//    class, z ascending with the id: the partners of a tile share one L2 and one dispatch queue.
//
// Split-K completion in XCD-local order ("mailbox").  The partners exchange their partials with
// ordinary stores and loads that stay in the XCD's L2 (acknowledged by the L2, not by memory) and
// signal them with flags, without any atomic, counter or workgroup barrier on the way:
//   partner z < S - 1   every wave stores its share of the partial, waits for the L2's
//                       acknowledgement (vmcnt) and stores the launch's tag to its flag word;
//   owner   z = S - 1   the partner that is dispatched last.  After its own K walk wave 0 polls the
//                       (S - 1) x waves flags of the tile (L1-bypassing loads served by the L2),
//                       then every thread adds the partials in ascending z, its own last, and
//                       writes C.
// The tag names the launch and the XCD: a number the host counts up with every enqueue, the XCC id
// of the wave that writes or expects the flag, the queue the dispatch packet sits in and the
// packet's index in that queue (which also tells apart the replays of a captured graph, whose
// kernel arguments never change).  Flags left behind by earlier launches never match, so nothing
// has to be cleared and nothing is read or counted when a workgroup starts.
// Nothing depends on where the hardware really puts a workgroup.  A flag counts only when it
// carries the owner's own XCC id: a partner that ran on another XCD (its stores are in an L2 the
// owner cannot see) is never taken for delivered, and a flag of this launch from another XCD ends
// the wait at once.  The owner polls a bounded number of times -- partners are dispatched before it
// from the same queue, so their flags come within microseconds -- and recomputes from A and W
// every partial it has no flag for, in the same order of operations: the result is bit for bit
// the same, only later.  kFlagPretendForeign makes a fifth of the workgroups behave as if they
// were misplaced (tests): such a partner stores nothing, such an owner does not poll.
// ---------------------------------------------------------------------------------------
constexpr int kRedStride = 132;  // floats per row of the cross-wave buffer: 128 + 4 keeps 16-byte
                                 // alignment and puts consecutive rows on different LDS banks

// XCC (= XCD) the wave runs on: bits 3:0 of hardware register 20 on gfx942 / gfx950.
__device__ __forceinline__ int xcc_id() {
  return (int)__builtin_amdgcn_s_getreg((3 << 11) | (0 << 6) | 20) & 15;
}

// AQL dispatch packet index of this launch in its queue (64-bit, counts up with every packet).
extern "C" __device__ unsigned long long fg_dispatch_id(void) __asm("llvm.amdgcn.dispatch.id");

// 64-bit name of this launch on this XCD, never zero: host enqueue count (20 bits, 1..2^20-1) | XCC id
// (4 bits) | queue (8 bits of the queue descriptor's address) | low 32 bits of the packet index.
constexpr unsigned long long kTagXccMask = 0xFull << 40;
__device__ __forceinline__ unsigned long long launch_tag(unsigned int nonce) {
  const unsigned long long q = reinterpret_cast<unsigned long long>(__builtin_amdgcn_queue_ptr());
  return ((unsigned long long)nonce << 44) | ((unsigned long long)xcc_id() << 40) | (((q >> 12) & 0xFFull) << 32) |
         (fg_dispatch_id() & 0xFFFFFFFFull);
}
// A flag word of this launch written on another XCD.
__device__ __forceinline__ bool tag_is_foreign(unsigned long long flag, unsigned long long tag) {
  return flag != tag && ((flag ^ tag) & ~kTagXccMask) == 0;
}

struct KnItem {
  int tile, z, y;
  bool home;  // false: behaves as if it ran on another XCD than its partners (tests only)
};
// x / d and x % d for a divisor whose log2 the host passes when it is a power of two (-1 otherwise):
// the usual tile, XCD and CU counts are, and a division by a run-time value costs some 40
// instructions before the workgroup's first load can go out.
__device__ __forceinline__ int div_by(int x, int d, int log2d) { return log2d >= 0 ? x >> log2d : x / d; }
__device__ __forceinline__ int mod_by(int x, int d, int log2d) { return log2d >= 0 ? x & (d - 1) : x % d; }

__device__ __forceinline__ KnItem kn_item(int M, int flags, const KnGeo& geo) {
  KnItem it;
  const int L = (int)blockIdx.x;
  int l = L;
  it.y = 0;
  if (M > 16) {  // more than one block of rows: the grid repeats per block
    const int per_y = (int)gridDim.x / ((M + 15) >> 4);
    it.y = L / per_y;
    l = L - it.y * per_y;
  }
  it.home = true;
  if (flags & kFlagXcdLocal) {
    const int xcd = mod_by(l, geo.xccs, geo.log2_xccs), n = div_by(l, geo.xccs, geo.log2_xccs);
    const int a = mod_by(n, geo.tq, geo.log2_tq);
    it.z = div_by(n, geo.tq, geo.log2_tq);
    const int round = div_by(L - xcd - a * geo.xccs, geo.cus, geo.log2_cus);  // full rounds of CUs before this plane
    it.tile = xcd * geo.tq + mod_by(a + round, geo.tq, geo.log2_tq);           // >= tiles: nothing to do
    if (flags & kFlagPretendForeign) it.home = L % 5 != 3;
  } else {
    const int x = mod_by(l, geo.tiles, geo.log2_tiles);
    it.z = div_by(l, geo.tiles, geo.log2_tiles);
    const int round = div_by(L - x, geo.cus, geo.log2_cus);
    it.tile = mod_by(x + round, geo.tiles, geo.log2_tiles);
  }
  return it;
}

// (8 waves with one K unit in flight: two workgroups must fit a CU, i.e. four waves a SIMD, at most 128 registers)
template <int U, int NW>
__global__ __launch_bounds__(64 * NW, (NW == 8 && U == 1) ? 4 : 1) void kn_mfma_kernel(const half_t* __restrict__ A,
                                                      const half_t* __restrict__ W,
                                                      half_t* __restrict__ C,
                                                      float* __restrict__ ws, int* counters, int M, int N,
                                                      int K, int flags, const void* bias, int ldw, KnGeo geo) {
  typedef half_t half4v __attribute__((ext_vector_type(4)));
  constexpr int NT = 64 * NW;     // threads
  constexpr int NQ = 512 / NT;    // 16-byte groups of the 16 x 128 tile per thread
  __shared__ __attribute__((aligned(16))) float red[NW][16][kRedStride];
  __shared__ int s_arrival;
  __shared__ int s_state;  // the mailbox owner's waves agree here (see there)
  const int lane = threadIdx.x & 63;
  const int wave = threadIdx.x >> 6;
  const int j = lane & 15, g = lane >> 4;
  const KnItem it = kn_item(M, flags, geo);
  const int S = geo.splitk;
  if (threadIdx.x == 0) s_state = 0;  // published by the barrier of the cross-wave sum
  const bool mailbox = (flags & kFlagXcdLocal) != 0 && S > 1;
  if (it.tile >= geo.tiles) return;
  if (mailbox && !it.home && it.z != S - 1) return;  // the owner will recompute this share
  const int n0 = it.tile * 128;
  const int m0 = it.y * 16;
  const int rows = M - m0 < 16 ? M - m0 : 16;
  const int nunits = K >> 5;
  const bool arow = j < rows;
  const half_t* Ap = A + (size_t)(m0 + (arow ? j : 0)) * K + g * 8;
  const half_t* Wp = W + (size_t)(g * 8) * ldw + n0 + j * 8;

  // Partial sum of K split zz over this workgroup's waves: part[q] = four columns of row
  // (q * NT + tid) / 32.  Called with zz = it.z, and by the recomputing fallback with every zz.
  float4_t part[NQ];
  auto compute_partial = [&](int zz) {
    float4_t acc[8];
#pragma unroll
    for (int i = 0; i < 8; ++i) acc[i] = float4_t{0.f, 0.f, 0.f, 0.f};
    const u32x4 zero = {0u, 0u, 0u, 0u};
    const int slots = NW * S;
    for (int u0 = (zz * NW + wave) * U; u0 < nunits; u0 += slots * U) {
      u32x4 rws[U][8];
      u32x4 a[U];
#pragma unroll
      for (int u = 0; u < U; ++u) {
        const int unit = u0 + u;
        const bool ok = unit < nunits;
#pragma unroll
        for (int i = 0; i < 8; ++i)
          rws[u][i] = ok ? load16<true>(Wp + (size_t)(unit * 32 + i) * ldw) : zero;
        a[u] = (ok && arow) ? load16<false>(Ap + (size_t)unit * 32) : zero;
      }
#pragma unroll
      for (int u = 0; u < U; ++u) {
        u32x4 bt[8];
        transpose8x8(rws[u], bt);
#pragma unroll
        for (int i = 0; i < 8; ++i)
          acc[i] = __builtin_amdgcn_mfma_f32_16x16x32_f16(as_half8(bt[i]), as_half8(a[u]), acc[i], 0,
                                                          0, 0);
      }
    }
    float* mine = &red[wave][j][32 * g];
#pragma unroll
    for (int r = 0; r < 4; ++r) {
      *reinterpret_cast<float4_t*>(mine + 8 * r) = float4_t{acc[0][r], acc[1][r], acc[2][r], acc[3][r]};
      *reinterpret_cast<float4_t*>(mine + 8 * r + 4) = float4_t{acc[4][r], acc[5][r], acc[6][r], acc[7][r]};
    }
    __syncthreads();
#pragma unroll
    for (int q = 0; q < NQ; ++q) {
      const int e = q * NT + (int)threadIdx.x;
      float4_t v[NW];
#pragma unroll
      for (int w = 0; w < NW; ++w) v[w] = *reinterpret_cast<const float4_t*>(&red[w][e >> 5][(e & 31) * 4]);
      float4_t sum = {0.f, 0.f, 0.f, 0.f};
#pragma unroll
      for (int w = 0; w < NW; ++w) sum += v[w];
      part[q] = sum;
    }
  };

  // Finished sums of this thread's groups to C (the only place that looks at the flag word's
  // accumulate / bias / activation bits: a plain product pays one uniform branch).
  auto write_out = [&](const float4_t (&tot)[NQ]) {
#pragma unroll
    for (int q = 0; q < NQ; ++q) {
      const int e = q * NT + (int)threadIdx.x;
      const int m = e >> 5, c0 = (e & 31) * 4;
      if (m >= rows) continue;
      half4v* c = reinterpret_cast<half4v*>(C + (size_t)(m0 + m) * N + n0 + c0);
      float4_t v = tot[q];
      if (flags & (kFlagAccumulate | kFlagTailMask)) {
        if (flags & kFlagAccumulate) {
          const half4v old = *c;
#pragma unroll
          for (int k = 0; k < 4; ++k) v[k] += static_cast<float>(old[k]);
        }
#pragma unroll
        for (int k = 0; k < 4; ++k) v[k] = apply_tail(v[k], n0 + c0 + k, bias, flags);
      }
      half4v out;
#pragma unroll
      for (int k = 0; k < 4; ++k) out[k] = static_cast<half_t>(v[k]);
      *c = out;
    }
  };

  compute_partial(it.z);
  if (S == 1) {
    write_out(part);
    return;
  }
  if (flags & kFlagFixSplit) {
    // one atomic per output element, consecutive lanes on consecutive columns
    uint64_t* facc = reinterpret_cast<uint64_t*>(reinterpret_cast<unsigned char*>(counters) + kWsCounterBytes);
    uint32_t* fcls = reinterpret_cast<uint32_t*>(facc + kWsAccElems);
    constexpr int NB = NW >= 8 ? 4 : 8;  // elements a thread: 16 x 128 over the workgroup
    size_t idx[NB];
    float p[NB];
    bool valid[NB];
#pragma unroll
    for (int i = 0; i < NB; ++i) {
      const int e = i * NT + (int)threadIdx.x;
      const int m = e >> 7, c = e & 127;
      valid[i] = m < rows;
      float v[NW];
#pragma unroll
      for (int w = 0; w < NW; ++w) v[w] = red[w][m][c];
      float sum = 0.f;
#pragma unroll
      for (int w = 0; w < NW; ++w) sum += v[w];
      p[i] = sum;
      idx[i] = (size_t)(m0 + (valid[i] ? m : 0)) * N + n0 + c;
    }
    fix_arrive<NB>(facc, fcls, ws, it.z, (size_t)M * N, idx, p, valid, S, C, N, bias, flags);
    return;
  }
  // partials [z][m][n]: through memory (write-through) for the counter protocol across XCDs,
  // ordinary stores when the kernel boundary or the shared L2 makes them visible
  const bool coherent = counters != nullptr && !mailbox;
  const bool owner = mailbox && it.z == S - 1;
  if (!owner) {
#pragma unroll
    for (int q = 0; q < NQ; ++q) {
      const int e = q * NT + (int)threadIdx.x;
      const int m = e >> 5, c0 = (e & 31) * 4;
      if (m < rows) store_partial4(ws, ((size_t)it.z * M + m0 + m) * N + n0 + c0, part[q], coherent);
    }
  }
  if (counters == nullptr) return;  // a second kernel sums the partials

  float4_t tot[NQ];
  int off[NQ];                      // byte offset of the thread's groups within one partial
  const int z_bytes = M * N * 4;    // the in-launch completions keep all partials below 2 GiB
#pragma unroll
  for (int q = 0; q < NQ; ++q) {
    const int e = q * NT + (int)threadIdx.x;
    const int m = e >> 5;
    off[q] = ((m0 + (m < rows ? m : 0)) * N + n0 + (e & 31) * 4) * 4;
  }
  if (!mailbox) {
    const int arrived = splitk_arrive(counters + it.y * geo.tiles + it.tile, S, &s_arrival);
    if (arrived == 0) return;
    sum_partials_z<NQ, true>(ws, S, z_bytes, off, tot);
    write_out(tot);
    return;
  }

  // ---- mailbox ----
  unsigned long long* mb_flags = reinterpret_cast<unsigned long long*>(reinterpret_cast<unsigned char*>(counters) + kWsMailboxFlagsOffset) +
                                 (size_t)((it.y * geo.tiles + it.tile) * S) * NW;
  const unsigned long long tag = launch_tag(geo.nonce);
  if (!owner) {
    __builtin_amdgcn_s_waitcnt(0x0F70);  // vmcnt(0): this wave's share of the partial is in the L2
    if (lane == 0) __hip_atomic_store(mb_flags + it.z * NW + wave, tag, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_WORKGROUP);
    return;
  }
  // Owner, eight partners at a time (one flag per lane, one pass): every wave polls for itself and
  // loads a partner's partial the moment that partner's flags are up.  Partials of partners that
  // finished microseconds ago have left the L2 by now; loading them while waiting for the last
  // partner takes that memory latency off the end of the kernel.  The values wait in registers and
  // are added in ascending z afterwards.  The waves do not meet at a barrier, so they agree through
  // one LDS word on whether anybody gives up: 0 undecided, 1 some wave has seen every flag (then
  // every wave will), 2 wave 0 has polled `spin_limit` times in vain or some wave has found a flag of
  // this launch from another XCD (everybody recomputes).
  constexpr int PF = 8;
  const unsigned int all = (1u << (S - 1)) - 1u;  // S <= 32
  if (it.home) {
    // (more than eight partners: eight at a time, in ascending z; the sum runs on in that order)
    const __amdgpu_buffer_rsrc_t rsrc = partials_rsrc(ws);
    float4_t run[NQ];
#pragma unroll
    for (int q = 0; q < NQ; ++q) run[q] = float4_t{0.f, 0.f, 0.f, 0.f};
    bool give_up = false;
    int spins = 0;
    for (int c0 = 0; c0 < S - 1 && !give_up; c0 += PF) {
      const int np = S - 1 - c0 < PF ? S - 1 - c0 : PF;
      const int nflags = np * NW;  // <= 64: one flag per lane
      const unsigned int all_c = (1u << np) - 1u;
      float4_t v[PF][NQ];
      unsigned int loaded = 0;
      for (;; ++spins) {
        const unsigned long long f =
            lane < nflags ? __hip_atomic_load(mb_flags + c0 * NW + lane, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT) : tag;
        const unsigned long long b = __builtin_amdgcn_ballot_w64(f == tag);
        const bool misplaced = __builtin_amdgcn_ballot_w64(tag_is_foreign(f, tag)) != 0;  // a partner on another XCD
#pragma unroll
        for (int z = 0; z < PF; ++z) {
          const unsigned long long lanes = ((1ull << NW) - 1) << (z * NW);
          if (z < np && !((loaded >> z) & 1u) && (b & lanes) == lanes) {
#pragma unroll
            for (int q = 0; q < NQ; ++q)
              v[z][q] = __builtin_bit_cast(float4_t, __builtin_amdgcn_raw_buffer_load_b128(rsrc, off[q], (c0 + z) * z_bytes, 1));
            loaded |= 1u << z;
          }
        }
        if (loaded == all_c) break;
        if (__hip_atomic_load(&s_state, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_WORKGROUP) == 2) {
          give_up = true;
          break;
        }
        if (misplaced || (wave == 0 && spins >= geo.spin_limit)) {
          int seen = 0;
          if (lane == 0) {
            __hip_atomic_compare_exchange_strong(&s_state, &seen, 2, __ATOMIC_RELAXED, __ATOMIC_RELAXED,
                                                 __HIP_MEMORY_SCOPE_WORKGROUP);
          }
          seen = __builtin_amdgcn_readfirstlane(seen);
          if (seen != 1) {  // nobody has everything: give up (a wave that has, keeps the others going)
            give_up = true;
            break;
          }
        }
        __builtin_amdgcn_s_sleep(1);
      }
      if (give_up) break;
#pragma unroll
      for (int z = 0; z < PF; ++z)
        if (z < np) {
#pragma unroll
          for (int q = 0; q < NQ; ++q) run[q] += v[z][q];
        }
    }
    if (!give_up) {
      int seen = 0;
      if (lane == 0) {
        __hip_atomic_compare_exchange_strong(&s_state, &seen, 1, __ATOMIC_RELAXED, __ATOMIC_RELAXED,
                                             __HIP_MEMORY_SCOPE_WORKGROUP);
      }
      give_up = __builtin_amdgcn_readfirstlane(seen) == 2;
    }
    if (!give_up) {
#pragma unroll
      for (int q = 0; q < NQ; ++q) tot[q] = run[q] + part[q];
      write_out(tot);
      return;
    }
    // every wave arrives here: recompute all partials (what was loaded is not used)
    if (threadIdx.x == 0) s_arrival = 0;
  } else {
    // owner: which partners have delivered?  Wave 0 polls, one flag per lane and pass.
    const int nflags = (S - 1) * NW;
    if (wave == 0) {
      unsigned int ready = 0;  // bit z: all waves of partner z have flagged
      if (it.home) {
        bool done = false, misplaced = false;
        for (int spins = 0; !done && !misplaced && spins < geo.spin_limit; ++spins) {
          done = true;
          for (int base = 0; base < nflags; base += 64) {
            const int idx = base + lane;
            const unsigned long long f =
                idx < nflags ? __hip_atomic_load(mb_flags + idx, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT) : tag;
            done = done && __builtin_amdgcn_ballot_w64(f == tag) == ~0ull;
            misplaced = misplaced || __builtin_amdgcn_ballot_w64(tag_is_foreign(f, tag)) != 0;
          }
          if (!done && !misplaced) __builtin_amdgcn_s_sleep(1);
        }
        if (done) {
          ready = all;
        } else {
          // not everything came: one more look, partner by partner (NW consecutive lanes each)
          for (int base = 0; base < nflags; base += 64) {
            const int idx = base + lane;
            const bool ok = idx < nflags &&
                            __hip_atomic_load(mb_flags + idx, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT) == tag;
            const unsigned long long b = __builtin_amdgcn_ballot_w64(ok);
            for (int k = 0; k < 64 / NW && base / NW + k < S - 1; ++k)
              if (((b >> (k * NW)) & ((1ull << NW) - 1)) == ((1ull << NW) - 1)) ready |= 1u << (base / NW + k);
          }
        }
      }
      if (lane == 0) s_arrival = (int)ready;
    }
  }
  __syncthreads();
  const unsigned int ready = (unsigned int)s_arrival;
  if (ready == all) {
    sum_partials_z<NQ, false>(ws, S - 1, z_bytes, off, tot);
#pragma unroll
    for (int q = 0; q < NQ; ++q) tot[q] += part[q];
  } else {
    // some partial is missing (its workgroup runs on another XCD, or the flag did not come in
    // time): take what has been delivered, recompute the rest, same order of additions
    float4_t own[NQ];
#pragma unroll
    for (int q = 0; q < NQ; ++q) {
      own[q] = part[q];
      tot[q] = float4_t{0.f, 0.f, 0.f, 0.f};
    }
    for (int zz = 0; zz < S - 1; ++zz) {
      if ((ready >> zz) & 1u) {
#pragma unroll
        for (int q = 0; q < NQ; ++q) tot[q] += load_partial4_l2(ws, (size_t)zz * M * N + (size_t)(off[q] >> 2));
      } else {
        __syncthreads();  // the cross-wave buffer is read by every wave until here
        compute_partial(zz);
#pragma unroll
        for (int q = 0; q < NQ; ++q) tot[q] += part[q];
      }
    }
#pragma unroll
    for (int q = 0; q < NQ; ++q) tot[q] += own[q];
  }
  write_out(tot);
}

// ---------------------------------------------------------------------------------------
// v_dot2 variant for few rows of A: acc[i][m] per lane, the activations of the lane's 8 k
// positions are one 16-byte load per row m (identical for the 16 lanes of a DPP row).
// The four k-groups g of a wave are summed in LDS together with the waves.
// ---------------------------------------------------------------------------------------
template <int MB, int U, bool STREAM, int NW>
__global__ __launch_bounds__(64 * NW) void kn_dot2_kernel(const half_t* __restrict__ A,
                                                      const half_t* __restrict__ W,
                                                      half_t* __restrict__ C,
                                                      float* __restrict__ ws, int* counters, int M, int N,
                                                      int K, int flags, const void* bias, int ldw, int cus) {
  __shared__ float red[4 * NW][MB][128];  // NW = most waves per workgroup
  const int lane = threadIdx.x & 63;
  const int wave = threadIdx.x >> 6;
  const int nw = blockDim.x >> 6;
  const int j = lane & 15, g = lane >> 4;
  const int tile_x = kn_tile(blockIdx.x, blockIdx.z, gridDim.x, cus);
  const int n0 = tile_x * 128;
  const int m0 = blockIdx.y * MB;
  const int slots = nw * gridDim.z;
  const int slot = blockIdx.z * nw + wave;
  const int nunits = K >> 5;

  float acc[8][MB];
#pragma unroll
  for (int i = 0; i < 8; ++i)
#pragma unroll
    for (int m = 0; m < MB; ++m) acc[i][m] = 0.f;

  const half_t* Ap = A + (size_t)m0 * K + g * 8;
  const half_t* Wp = W + (size_t)(g * 8) * ldw + n0 + j * 8;
  const u32x4 zero = {0u, 0u, 0u, 0u};

  for (int u0 = slot * U; u0 < nunits; u0 += slots * U) {
    u32x4 rows[U][8];
    u32x4 xr[U][MB];
#pragma unroll
    for (int u = 0; u < U; ++u) {
      const int unit = u0 + u;
      const bool ok = unit < nunits;
#pragma unroll
      for (int i = 0; i < 8; ++i)
        rows[u][i] = ok ? load16<STREAM>(Wp + (size_t)(unit * 32 + i) * ldw) : zero;
#pragma unroll
      for (int m = 0; m < MB; ++m)
        xr[u][m] =
            (ok && (m0 + m) < M) ? load16<false>(Ap + (size_t)m * K + (size_t)unit * 32) : zero;
    }
#pragma unroll
    for (int u = 0; u < U; ++u) {
      u32x4 bt[8];
      transpose8x8(rows[u], bt);
#pragma unroll
      for (int i = 0; i < 8; ++i)
#pragma unroll
        for (int m = 0; m < MB; ++m) acc[i][m] = dot8(bt[i], xr[u][m], acc[i][m]);
    }
  }

#pragma unroll
  for (int m = 0; m < MB; ++m)
#pragma unroll
    for (int i = 0; i < 8; ++i) red[wave * 4 + g][m][8 * j + i] = acc[i][m];
  __syncthreads();
  if (gridDim.z > 1 && (flags & kFlagFixSplit)) {
    uint64_t* facc = reinterpret_cast<uint64_t*>(reinterpret_cast<unsigned char*>(counters) + kWsCounterBytes);
    uint32_t* fcls = reinterpret_cast<uint32_t*>(facc + kWsAccElems);
    const int rows = M - m0 < MB ? M - m0 : MB;
    constexpr int NB = MB >= 4 ? 2 : 1;
    for (int base = 0; base < rows * 128; base += NB * blockDim.x) {
      size_t idx[NB];
      float part[NB];
      bool valid[NB];
#pragma unroll
      for (int i = 0; i < NB; ++i) {
        const int e = base + i * (int)blockDim.x + (int)threadIdx.x;
        valid[i] = e < rows * 128;
        const int m = valid[i] ? e >> 7 : 0, nn = e & 127;
        part[i] = lds_sum<4 * NW>(&red[0][m][nn], MB * 128, nw * 4);
        idx[i] = (size_t)(m0 + m) * N + n0 + nn;
      }
      fix_arrive<NB>(facc, fcls, ws, (int)blockIdx.z, (size_t)M * N, idx, part, valid, gridDim.z, C, N, bias, flags);
    }
    return;
  }
  for (int e = threadIdx.x; e < MB * 128; e += blockDim.x) {
    const int m = e >> 7, nn = e & 127;
    const float sum = lds_sum<4 * NW>(&red[0][m][nn], MB * 128, nw * 4);
    const int mg = m0 + m, n = n0 + nn;
    if (mg < M) {
      if (gridDim.z == 1) {
        half_t* c = C + (size_t)mg * N + n;
        *c = finish_value(sum, c, n, bias, flags);
      } else {
        store_partial(ws + ((size_t)blockIdx.z * M + mg) * N + n, sum, counters != nullptr);
      }
    }
  }
  finish_splitk<MB, 128, true>(ws, counters, C, M, N, m0, n0, flags, bias, tile_x);
}

// ---------------------------------------------------------------------------------------
// Host launchers
// ---------------------------------------------------------------------------------------
template <int MB, int U>
static void kn_dot2_go(const fg_plan_t& p, const GemmArgs& a, hipStream_t s) {
  const dim3 grid(p.grid_x, p.grid_y, p.grid_z), block(p.block);
  auto* A = static_cast<const half_t*>(a.A);
  auto* W = static_cast<const half_t*>(a.W);
  auto* C = static_cast<half_t*>(a.C);
  if constexpr (MB <= 2) {
    if (p.waves == 8) {
      hipLaunchKernelGGL((kn_dot2_kernel<MB, U, true, 8>), grid, block, 0, s, A, W, C, a.ws, a.counters, a.M,
                         a.N, a.K, a.accumulate, a.bias, a.ldw, a.cus);
      return;
    }
  }
  if (p.stream_w)
    hipLaunchKernelGGL((kn_dot2_kernel<MB, U, true, 4>), grid, block, 0, s, A, W, C, a.ws, a.counters, a.M, a.N,
                       a.K, a.accumulate, a.bias, a.ldw, a.cus);
  else
    hipLaunchKernelGGL((kn_dot2_kernel<MB, U, false, 4>), grid, block, 0, s, A, W, C, a.ws, a.counters, a.M, a.N,
                       a.K, a.accumulate, a.bias, a.ldw, a.cus);
}

template <int MB>
static bool kn_dot2_u(const fg_plan_t& p, const GemmArgs& a, hipStream_t s) {
  switch (p.unroll) {
    case 1: kn_dot2_go<MB, 1>(p, a, s); return true;
    case 2: kn_dot2_go<MB, 2>(p, a, s); return true;
    case 4:
      if constexpr (MB < 8) { kn_dot2_go<MB, 4>(p, a, s); return true; }
      return false;
    default: return false;
  }
}

bool launch_kn_dot2(const fg_plan_t& p, const GemmArgs& a, hipStream_t s) {
  if (p.waves > 4 && p.m_block > 2) return false;  // 8 waves are built for one or two rows only
  switch (p.m_block) {
    case 1: return kn_dot2_u<1>(p, a, s);
    case 2: return kn_dot2_u<2>(p, a, s);
    case 4: return kn_dot2_u<4>(p, a, s);
    case 8: return kn_dot2_u<8>(p, a, s);
    default: return false;
  }
}

template <int U>
static void kn_mfma_go(const fg_plan_t& p, const GemmArgs& a, hipStream_t s) {
  auto* A = static_cast<const half_t*>(a.A);
  auto* W = static_cast<const half_t*>(a.W);
  auto* C = static_cast<half_t*>(a.C);
  KnGeo geo;
  geo.tiles = p.grid_x;
  geo.splitk = p.splitk;
  geo.cus = a.cus;
  geo.xccs = a.xccs;
  geo.tq = (p.grid_x + a.xccs - 1) / a.xccs;
  auto log2_of = [](int v) {
    int l = -1;
    if (v > 0 && (v & (v - 1)) == 0)
      for (l = 0; (1 << l) < v; ++l) {}
    return l;
  };
  geo.log2_tiles = log2_of(geo.tiles), geo.log2_tq = log2_of(geo.tq), geo.log2_xccs = log2_of(geo.xccs), geo.log2_cus = log2_of(geo.cus);
  geo.spin_limit = (a.accumulate & kFlagPretendForeign) ? 64 : (1 << 14);  // some 10 ms of polling
  // a new number for every enqueue of a launch that uses the flags (1 .. 2^24 - 1, wrapping)
  static std::atomic<unsigned int> enqueues{0};
  geo.nonce = (a.accumulate & kFlagXcdLocal) ? enqueues.fetch_add(1, std::memory_order_relaxed) % 0xFFFFFu + 1u : 0u;
  // one-dimensional grid: row blocks x splits x column tiles; in XCD-local order every XCD gets the
  // same number of column tiles (the last ones may be empty)
  const int tiles_padded = (a.accumulate & kFlagXcdLocal) ? (p.grid_x + a.xccs - 1) / a.xccs * a.xccs : p.grid_x;
  const dim3 grid((unsigned)tiles_padded * p.splitk * p.grid_y), block(p.block);
  if (p.waves == 8) {
    hipLaunchKernelGGL((kn_mfma_kernel<U, 8>), grid, block, 0, s, A, W, C, a.ws, a.counters, a.M, a.N, a.K,
                       a.accumulate, a.bias, a.ldw, geo);
  } else {
    hipLaunchKernelGGL((kn_mfma_kernel<U, 4>), grid, block, 0, s, A, W, C, a.ws, a.counters, a.M, a.N, a.K,
                       a.accumulate, a.bias, a.ldw, geo);
  }
}

bool launch_kn_mfma(const fg_plan_t& p, const GemmArgs& a, hipStream_t s) {
  if (p.waves != 4 && p.waves != 8) return false;
  if ((long long)p.grid_x * p.splitk * p.grid_y + 8LL * p.splitk * p.grid_y > 0x7fffffffLL) return false;
  switch (p.unroll) {
    case 1: kn_mfma_go<1>(p, a, s); return true;
    case 2: kn_mfma_go<2>(p, a, s); return true;
    case 4: kn_mfma_go<4>(p, a, s); return true;
    default: return false;
  }
}

}  // namespace fg
