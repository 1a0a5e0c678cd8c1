// int8-weight GEMV kernels, weights [N,K] row-major (16 weights per 16-byte load).
//
//  * w8a16: fp16 activations.  Four int8 of a register become two half2 without leaving the
//    integer pipe's cheap ops: flip the sign bit (w+128 as unsigned), splice each byte under
//    the exponent 0x64 (fp16 value 1024 + byte), subtract 1152 with v_pk_add_f16 -> the exact
//    integer as fp16, then v_dot2_f32_f16 against the activations (fp32 accumulation).  The
//    per-output-channel scale and the zero point are applied once per output.
//  * i8i8: int8 activations, v_dot4_i32_i8, exact int32 result.
//
// Replaces the device side of gemv_quantized_int8 (backend/cuda/hk/fastgemv.cuh:316-389,
// 8-byte loads, int8 -> fp32 convert, scalar FMAs) of the reference.
#include "fg_device.h"
#include "fg_internal.h"

namespace fg {

__device__ __forceinline__ void i8x4_to_half2x2(uint32_t w, half2_t& lo, half2_t& hi) {
  const uint32_t t = w ^ 0x80808080u;
  const half2_t bias = {static_cast<half_t>(1152.f), static_cast<half_t>(1152.f)};
  lo = as_half2(__builtin_amdgcn_perm(0x64646464u, t, 0x04010400u)) - bias;
  hi = as_half2(__builtin_amdgcn_perm(0x64646464u, t, 0x04030402u)) - bias;
}

template <int MB, int RN, int U>
__global__ __launch_bounds__(512) void w8a16_kernel(const int8_t* __restrict__ Wq,
                                                    const half_t* __restrict__ X,
                                                    const half_t* __restrict__ scale,
                                                    float scalar_scale, float zero_point,
                                                    half_t* __restrict__ Y, int M, int N, int K) {
  __shared__ float red[32][RN * MB];
  __shared__ float redx[32][MB];
  const int lane = threadIdx.x & 63;
  const int wave = threadIdx.x >> 6;
  const int nw = blockDim.x >> 6;
  const int n0 = blockIdx.x * RN;
  const int nq = K >> 4;  // 16-weight chunks per row
  const bool use_zp = zero_point != 0.f;

  float acc[RN][MB];
  float xsum[MB];
#pragma unroll
  for (int m = 0; m < MB; ++m) {
    xsum[m] = 0.f;
#pragma unroll
    for (int r = 0; r < RN; ++r) acc[r][m] = 0.f;
  }
  const int8_t* Wt = Wq + (size_t)n0 * K;
  const u32x4 zero = {0u, 0u, 0u, 0u};
  const half2_t ones = {static_cast<half_t>(1.f), static_cast<half_t>(1.f)};

  const int nsteps = (nq + nw * (64 * U) - 1) / (nw * (64 * U));
  int step = stagger_start(nsteps, 0);
  for (int it = 0; it < nsteps; ++it) {
    const int q0 = (step * nw + wave) * (64 * U);
    step = step + 1 == nsteps ? 0 : step + 1;
    u32x4 wr[U][RN];
    u32x4 xr[U][MB][2];
#pragma unroll
    for (int u = 0; u < U; ++u) {
      const int q = q0 + u * 64 + lane;
      const bool ok = q < nq;
#pragma unroll
      for (int r = 0; r < RN; ++r)
        wr[u][r] = ok ? load16<true>(Wt + (size_t)r * K + (size_t)q * 16) : zero;
#pragma unroll
      for (int m = 0; m < MB; ++m) {
        const bool okm = ok && m < M;
        const half_t* xp = X + (size_t)m * K + (size_t)q * 16;
        xr[u][m][0] = okm ? load16<false>(xp) : zero;
        xr[u][m][1] = okm ? load16<false>(xp + 8) : zero;
      }
    }
#pragma unroll
    for (int u = 0; u < U; ++u) {
#pragma unroll
      for (int r = 0; r < RN; ++r) {
#pragma unroll
        for (int c = 0; c < 4; ++c) {
          half2_t lo, hi;
          i8x4_to_half2x2(wr[u][r][c], lo, hi);
#pragma unroll
          for (int m = 0; m < MB; ++m) {
            const u32x4 xv = xr[u][m][c >> 1];
            const uint32_t x0 = (c & 1) ? xv.z : xv.x, x1 = (c & 1) ? xv.w : xv.y;
            acc[r][m] = __builtin_amdgcn_fdot2(lo, as_half2(x0), acc[r][m], false);
            acc[r][m] = __builtin_amdgcn_fdot2(hi, as_half2(x1), acc[r][m], false);
          }
        }
      }
      if (use_zp) {
#pragma unroll
        for (int m = 0; m < MB; ++m)
#pragma unroll
          for (int h = 0; h < 2; ++h)
#pragma unroll
            for (int c = 0; c < 4; ++c)
              xsum[m] = __builtin_amdgcn_fdot2(as_half2(xr[u][m][h][c]), ones, xsum[m], false);
      }
    }
  }

#pragma unroll
  for (int m = 0; m < MB; ++m) {
#pragma unroll
    for (int r = 0; r < RN; ++r) {
      const float v = row16_allreduce(acc[r][m]);
      if ((lane & 15) == 0) red[wave * 4 + (lane >> 4)][r * MB + m] = v;
    }
    const float xs = row16_allreduce(xsum[m]);
    if ((lane & 15) == 0) redx[wave * 4 + (lane >> 4)][m] = xs;
  }
  __syncthreads();
  for (int t = threadIdx.x; t < RN * MB; t += blockDim.x) {
    const int m = t / RN, r = t % RN;
    float sum = 0.f, xs = 0.f;
    for (int p = 0; p < nw * 4; ++p) {
      sum += red[p][r * MB + m];
      xs += redx[p][m];
    }
    const int n = n0 + r;
    if (m < M) {
      float s = scalar_scale;
      if (scale != nullptr) s *= static_cast<float>(scale[n]);
      Y[(size_t)m * N + n] = static_cast<half_t>((sum - zero_point * xs) * s);
    }
  }
}

template <int MB, int RN, int U>
__global__ __launch_bounds__(256) void i8i8_kernel(const int8_t* __restrict__ Wq,
                                                   const int8_t* __restrict__ Xq,
                                                   int32_t* __restrict__ out, int M, int N, int K) {
  __shared__ int red[16][RN * MB];
  const int lane = threadIdx.x & 63;
  const int wave = threadIdx.x >> 6;
  const int nw = blockDim.x >> 6;
  const int n0 = blockIdx.x * RN;
  const int nq = K >> 4;

  int acc[RN][MB];
#pragma unroll
  for (int r = 0; r < RN; ++r)
#pragma unroll
    for (int m = 0; m < MB; ++m) acc[r][m] = 0;
  const int8_t* Wt = Wq + (size_t)n0 * K;
  const u32x4 zero = {0u, 0u, 0u, 0u};

  const int nsteps = (nq + nw * (64 * U) - 1) / (nw * (64 * U));
  int step = stagger_start(nsteps, 0);
  for (int it = 0; it < nsteps; ++it) {
    const int q0 = (step * nw + wave) * (64 * U);
    step = step + 1 == nsteps ? 0 : step + 1;
    u32x4 wr[U][RN];
    u32x4 xr[U][MB];
#pragma unroll
    for (int u = 0; u < U; ++u) {
      const int q = q0 + u * 64 + lane;
      const bool ok = q < nq;
#pragma unroll
      for (int r = 0; r < RN; ++r)
        wr[u][r] = ok ? load16<true>(Wt + (size_t)r * K + (size_t)q * 16) : zero;
#pragma unroll
      for (int m = 0; m < MB; ++m)
        xr[u][m] = (ok && m < M) ? load16<false>(Xq + (size_t)m * K + (size_t)q * 16) : zero;
    }
#pragma unroll
    for (int u = 0; u < U; ++u)
#pragma unroll
      for (int r = 0; r < RN; ++r)
#pragma unroll
        for (int m = 0; m < MB; ++m)
#pragma unroll
          for (int c = 0; c < 4; ++c)
            acc[r][m] = __builtin_amdgcn_sdot4((int)wr[u][r][c], (int)xr[u][m][c], acc[r][m], false);
  }

#pragma unroll
  for (int r = 0; r < RN; ++r)
#pragma unroll
    for (int m = 0; m < MB; ++m) {
      const int v = row16_allreduce(acc[r][m]);
      if ((lane & 15) == 0) red[wave * 4 + (lane >> 4)][r * MB + m] = v;
    }
  __syncthreads();
  for (int t = threadIdx.x; t < RN * MB; t += blockDim.x) {
    const int m = t / RN, r = t % RN;
    int sum = 0;
    for (int p = 0; p < nw * 4; ++p) sum += red[p][r * MB + m];
    if (m < M) out[(size_t)m * N + n0 + r] = sum;
  }
}

__global__ __launch_bounds__(256) void dequant_i32_f16_kernel(const int32_t* __restrict__ acc,
                                                              const half_t* __restrict__ scale,
                                                              float x_scale, half_t* __restrict__ y,
                                                              int M, int N) {
  const size_t total = (size_t)M * N;
  for (size_t i = (size_t)blockIdx.x * blockDim.x + threadIdx.x; i < total;
       i += (size_t)gridDim.x * blockDim.x) {
    float s = x_scale;
    if (scale != nullptr) s *= static_cast<float>(scale[i % N]);
    y[i] = static_cast<half_t>(static_cast<float>(acc[i]) * s);
  }
}

// ---------------------------------------------------------------------------------------
// Host launchers.  Rows per workgroup: 8 when that still yields >= 512 workgroups, else 4.
// Waves per workgroup: as many (<= 4) as the row has 1 KB pieces.
// ---------------------------------------------------------------------------------------
static int i8_waves(int K) {
  const int pieces = (K / 16 + 63) / 64;
  return pieces >= 4 ? 4 : (pieces >= 2 ? 2 : 1);
}

template <int MB>
static void w8a16_go(const W8A16Args& a, hipStream_t s) {
  auto* Wq = static_cast<const int8_t*>(a.Wq);
  auto* X = static_cast<const half_t*>(a.x);
  auto* sc = static_cast<const half_t*>(a.scale);
  auto* Y = static_cast<half_t*>(a.y);
  const dim3 block(64 * i8_waves(a.K));
  if (MB == 1) {  // measured best at K = N = 8192 (12.6 us): 4 rows, one load group in flight
    hipLaunchKernelGGL((w8a16_kernel<1, 4, 1>), dim3(a.N / 4), block, 0, s, Wq, X, sc,
                       a.scalar_scale, a.zero_point, Y, a.M, a.N, a.K);
    return;
  }
  if (a.N / 8 >= 512 && MB <= 4) {
    hipLaunchKernelGGL((w8a16_kernel<MB, 8, 2>), dim3(a.N / 8), block, 0, s, Wq, X, sc,
                       a.scalar_scale, a.zero_point, Y, a.M, a.N, a.K);
  } else {
    hipLaunchKernelGGL((w8a16_kernel<MB, 4, 2>), dim3(a.N / 4), block, 0, s, Wq, X, sc,
                       a.scalar_scale, a.zero_point, Y, a.M, a.N, a.K);
  }
}

bool launch_w8a16(const W8A16Args& a, hipStream_t s) {
  if (a.M == 1) w8a16_go<1>(a, s);
  else if (a.M == 2) w8a16_go<2>(a, s);
  else if (a.M <= 4) w8a16_go<4>(a, s);
  else if (a.M <= 8) w8a16_go<8>(a, s);
  else return false;
  return true;
}

template <int MB>
static void i8i8_go(const void* Wq, const void* xq, int32_t* acc, int M, int N, int K,
                    hipStream_t s) {
  auto* W = static_cast<const int8_t*>(Wq);
  auto* X = static_cast<const int8_t*>(xq);
  const dim3 block(64 * i8_waves(K));
  if (MB == 1) {
    hipLaunchKernelGGL((i8i8_kernel<1, 4, 1>), dim3(N / 4), block, 0, s, W, X, acc, M, N, K);
    return;
  }
  if (N / 8 >= 512 && MB <= 4) {
    hipLaunchKernelGGL((i8i8_kernel<MB, 8, 2>), dim3(N / 8), block, 0, s, W, X, acc, M, N, K);
  } else {
    hipLaunchKernelGGL((i8i8_kernel<MB, 4, 2>), dim3(N / 4), block, 0, s, W, X, acc, M, N, K);
  }
}

bool launch_i8i8_i32(const void* Wq, const void* xq, int32_t* acc, int M, int N, int K,
                     hipStream_t s) {
  if (M == 1) i8i8_go<1>(Wq, xq, acc, M, N, K, s);
  else if (M == 2) i8i8_go<2>(Wq, xq, acc, M, N, K, s);
  else if (M <= 4) i8i8_go<4>(Wq, xq, acc, M, N, K, s);
  else if (M <= 8) i8i8_go<8>(Wq, xq, acc, M, N, K, s);
  else return false;
  return true;
}

void launch_dequant_i32_f16(const int32_t* acc, const void* scale, float x_scale, void* y, int M,
                            int N, hipStream_t s) {
  const size_t total = (size_t)M * N;
  const int blocks = (int)((total + 255) / 256 < 1024 ? (total + 255) / 256 : 1024);
  hipLaunchKernelGGL(dequant_i32_f16_kernel, dim3(blocks), dim3(256), 0, s, acc,
                     static_cast<const half_t*>(scale), x_scale, static_cast<half_t*>(y), M, N);
}

}  // namespace fg
