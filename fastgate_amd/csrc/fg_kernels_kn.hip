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
// MFMA variant: 8 MFMAs per step, MFMA i owns the columns n0 + 8*jj + i (jj = B-operand
// column index), so acc[i][r] = D[m = 4g + r][n = n0 + 8j + i]: a lane ends up with 8
// consecutive columns per row, which makes the epilogue 16-byte stores.
// ---------------------------------------------------------------------------------------
template <int U, bool STREAM, int NW>
__global__ __launch_bounds__(64 * NW) void kn_mfma_kernel(const half_t* __restrict__ A,
                                                      const half_t* __restrict__ W,
                                                      half_t* __restrict__ C,
                                                      float* __restrict__ ws, int* counters, int M, int N,
                                                      int K, int flags, const void* bias, int ldw, int cus) {
  __shared__ float red[NW][16][128];  // NW = most waves per workgroup
  const int lane = threadIdx.x & 63;
  const int wave = threadIdx.x >> 6;
  const int nw = blockDim.x >> 6;
  const int j = lane & 15, g = lane >> 4;
  const int tile_x = kn_tile(blockIdx.x, blockIdx.z, gridDim.x, cus);
  const int n0 = tile_x * 128;
  const int m0 = blockIdx.y * 16;
  const int slots = nw * gridDim.z;
  const int slot = blockIdx.z * nw + wave;
  const int nunits = K >> 5;

  float4_t acc[8];
#pragma unroll
  for (int i = 0; i < 8; ++i) acc[i] = float4_t{0.f, 0.f, 0.f, 0.f};

  const bool arow = (m0 + j) < M;
  const half_t* Ap = A + (size_t)(m0 + (arow ? j : 0)) * K + g * 8;
  const half_t* Wp = W + (size_t)(g * 8) * ldw + n0 + j * 8;
  const u32x4 zero = {0u, 0u, 0u, 0u};

  for (int u0 = slot * U; u0 < nunits; u0 += slots * U) {
    u32x4 rows[U][8];
    u32x4 a[U];
#pragma unroll
    for (int u = 0; u < U; ++u) {
      const int unit = u0 + u;
      const bool ok = unit < nunits;
#pragma unroll
      for (int i = 0; i < 8; ++i)
        rows[u][i] = ok ? load16<STREAM>(Wp + (size_t)(unit * 32 + i) * ldw) : zero;
      a[u] = (ok && arow) ? load16<false>(Ap + (size_t)unit * 32) : zero;
    }
#pragma unroll
    for (int u = 0; u < U; ++u) {
      u32x4 bt[8];
      transpose8x8(rows[u], bt);
#pragma unroll
      for (int i = 0; i < 8; ++i)
        acc[i] = __builtin_amdgcn_mfma_f32_16x16x32_f16(as_half8(a[u]), as_half8(bt[i]), acc[i], 0,
                                                        0, 0);
    }
  }

#pragma unroll
  for (int r = 0; r < 4; ++r)
#pragma unroll
    for (int i = 0; i < 8; ++i) red[wave][4 * g + r][8 * j + i] = acc[i][r];
  __syncthreads();
  if (gridDim.z > 1 && (flags & kFlagFixSplit)) {
    // one atomic per output element, consecutive lanes on consecutive columns
    uint64_t* facc = reinterpret_cast<uint64_t*>(reinterpret_cast<unsigned char*>(counters) + kWsCounterBytes);
    uint32_t* fcls = reinterpret_cast<uint32_t*>(facc + kWsAccElems);
    const int rows = M - m0 < 16 ? M - m0 : 16;
    // up to eight elements a thread (16 rows on four waves), their atomics in flight together
    constexpr int NB = NW >= 8 ? 4 : 8;
    for (int base = 0; base < rows * 128; base += NB * blockDim.x) {
      size_t idx[NB];
      float part[NB];
      bool valid[NB];
#pragma unroll
      for (int i = 0; i < NB; ++i) {
        const int e = base + i * (int)blockDim.x + (int)threadIdx.x;
        valid[i] = e < rows * 128;
        const int m = valid[i] ? e >> 7 : 0, c = e & 127;
        part[i] = lds_sum<NW>(&red[0][m][c], 16 * 128, nw);
        idx[i] = (size_t)(m0 + m) * N + n0 + c;
      }
      fix_arrive<NB>(facc, fcls, idx, part, valid, gridDim.z, C, N, bias, flags);
    }
    return;
  }
  // 16 x 128 outputs in groups of four columns: the 32 lanes of a half wave cover one 512-byte row
  // with consecutive 16-byte pieces, so every store instruction writes whole rows (partials that go
  // out as 16 bytes at a 32-byte stride, two instructions to fill a row, take the write-through
  // path twice as long).
  for (int e = threadIdx.x; e < 512; e += blockDim.x) {
    const int m = e >> 5, c0 = (e & 31) * 4;
    const int mg = m0 + m;
    if (mg < M) {
      // the reads of all waves in flight before the first add
      float4_t v[NW];
#pragma unroll
      for (int w = 0; w < NW; ++w) v[w] = *reinterpret_cast<const float4_t*>(&red[w < nw ? w : 0][m][c0]);
      float4_t sum = {0.f, 0.f, 0.f, 0.f};
      const float4_t zero4 = {0.f, 0.f, 0.f, 0.f};
#pragma unroll
      for (int w = 0; w < NW; ++w) sum += w < nw ? v[w] : zero4;
      if (gridDim.z == 1) {
        typedef half_t half4v __attribute__((ext_vector_type(4)));
        half4v* c = reinterpret_cast<half4v*>(C + (size_t)mg * N + n0 + c0);
        if (flags & kFlagAccumulate) {
          const half4v old = *c;
#pragma unroll
          for (int i = 0; i < 4; ++i) sum[i] += static_cast<float>(old[i]);
        }
        half4v out;
#pragma unroll
        for (int i = 0; i < 4; ++i) out[i] = static_cast<half_t>(apply_tail(sum[i], n0 + c0 + i, bias, flags));
        *c = out;
      } else {
        store_partial4(ws, ((size_t)blockIdx.z * M + mg) * N + n0 + c0, sum, counters != nullptr);
      }
    }
  }
  finish_splitk<16, 128, true>(ws, counters, C, M, N, m0, n0, flags, bias, tile_x);
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
      fix_arrive<NB>(facc, fcls, idx, part, valid, gridDim.z, C, N, bias, flags);
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
  const dim3 grid(p.grid_x, p.grid_y, p.grid_z), block(p.block);
  auto* A = static_cast<const half_t*>(a.A);
  auto* W = static_cast<const half_t*>(a.W);
  auto* C = static_cast<half_t*>(a.C);
  if (p.waves == 8) {
    hipLaunchKernelGGL((kn_mfma_kernel<U, true, 8>), grid, block, 0, s, A, W, C, a.ws, a.counters, a.M, a.N, a.K,
                       a.accumulate, a.bias, a.ldw, a.cus);
  } else if (p.stream_w) {
    hipLaunchKernelGGL((kn_mfma_kernel<U, true, 4>), grid, block, 0, s, A, W, C, a.ws, a.counters, a.M, a.N, a.K,
                       a.accumulate, a.bias, a.ldw, a.cus);
  } else {
    hipLaunchKernelGGL((kn_mfma_kernel<U, false, 4>), grid, block, 0, s, A, W, C, a.ws, a.counters, a.M, a.N, a.K,
                       a.accumulate, a.bias, a.ldw, a.cus);
  }
}

bool launch_kn_mfma(const fg_plan_t& p, const GemmArgs& a, hipStream_t s) {
  switch (p.unroll) {
    case 1: kn_mfma_go<1>(p, a, s); return true;
    case 2: kn_mfma_go<2>(p, a, s); return true;
    case 4: kn_mfma_go<4>(p, a, s); return true;
    default: return false;
  }
}

}  // namespace fg
