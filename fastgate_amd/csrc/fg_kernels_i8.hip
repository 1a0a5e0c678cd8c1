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

// Per-channel scale of the output a thread writes at the end, fetched ahead of the weight stream
// as raw bits.  Converting it at the point of the load would make the wave wait for this cold
// load before it issues anything else (measured: 0.3 us on the whole call at K = N = 8192);
// scale_value() keeps the conversion, and with it the wait, at the point of use.
__device__ __forceinline__ uint32_t scale_fetch(const half_t* scale, int n, bool mine) {
  uint32_t raw = 0x3c00u;  // 1.0
  if (scale != nullptr && mine) raw = reinterpret_cast<const uint16_t*>(scale)[n];
  return raw;
}
__device__ __forceinline__ float scale_value(uint32_t raw) {
  asm volatile("" : "+v"(raw));
  return f16_bits_to_f32((uint16_t)raw);
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
  // scale of the output this thread writes at the end, fetched ahead of the weight stream (a load
  // issued after the last barrier would add its whole latency to the workgroup's life)
  static_assert(RN * MB <= 64, "one output per thread of the first wave");
  const uint32_t scale_raw = scale_fetch(scale, n0 + (int)threadIdx.x % RN, threadIdx.x < RN * MB);

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
    const float sum = lds_sum<32>(&red[0][r * MB + m], RN * MB, nw * 4);
    const float xs = lds_sum<32>(&redx[0][m], MB, nw * 4);
    const int n = n0 + r;
    if (m < M)
      Y[(size_t)m * N + n] =
          static_cast<half_t>((sum - zero_point * xs) * (scalar_scale * scale_value(scale_raw)));
  }
}

// ---------------------------------------------------------------------------------------
// One activation row: the dot products go to the matrix pipe.  v_mfma_f32_4x4x4_16B_f16
// multiplies, in each block of four lanes, the A rows of the four lanes with the B columns of the
// four lanes.  With A = the lane's activations and B = the lane's weights, both at the lane's own
// k positions, the diagonal D[j][j] of a block is lane j's own dot product; the other twelve
// products are never read.  The memory side is that of w8a16_kernel (lanes along K, 16 weights of
// RN rows per lane and step); the VALU is left with the int8 -> fp16 conversion alone, 80
// operations per step instead of 112.  K = N = 8192: 12.4 -> 12.0 us.
// ---------------------------------------------------------------------------------------
typedef _Float16 half4_t __attribute__((ext_vector_type(4)));

template <int RN, int U, bool FULL>
__global__ __launch_bounds__(256) void w8a16_m1_kernel(const int8_t* __restrict__ Wq,
                                                       const half_t* __restrict__ X,
                                                       const half_t* __restrict__ scale,
                                                       float scalar_scale, float zero_point,
                                                       half_t* __restrict__ Y, int N, int K) {
  __shared__ float red[16][RN];
  __shared__ float redx[16];
  const int lane = threadIdx.x & 63;
  const int wave = threadIdx.x >> 6;
  const int nw = blockDim.x >> 6;
  const int n0 = blockIdx.x * RN;
  const int nq = K >> 4;  // 16-weight chunks per row
  const bool use_zp = zero_point != 0.f;
  static_assert(RN <= 64, "one output per thread of the first wave");
  const uint32_t scale_raw = scale_fetch(scale, n0 + (int)threadIdx.x, threadIdx.x < RN);

  float4_t acc[RN];
  float4_t xsum = {0.f, 0.f, 0.f, 0.f};
#pragma unroll
  for (int r = 0; r < RN; ++r) acc[r] = float4_t{0.f, 0.f, 0.f, 0.f};
  const int8_t* Wt = Wq + (size_t)n0 * K;
  const u32x4 zero = {0u, 0u, 0u, 0u};
  const half4_t ones = {static_cast<half_t>(1.f), static_cast<half_t>(1.f), static_cast<half_t>(1.f),
                        static_cast<half_t>(1.f)};

  const int nsteps = (nq + nw * (64 * U) - 1) / (nw * (64 * U));
  int step = stagger_start(nsteps, 0);
  for (int it = 0; it < nsteps; ++it) {
    const int q0 = (step * nw + wave) * (64 * U);
    step = step + 1 == nsteps ? 0 : step + 1;
    u32x4 wr[U][RN];
    u32x4 xr[U][2];
#pragma unroll
    for (int u = 0; u < U; ++u) {
      const int q = q0 + u * 64 + lane;
      const bool ok = FULL || q < nq;  // FULL: every step of every wave is inside the row
      const half_t* xp = X + (size_t)q * 16;
      xr[u][0] = ok ? load16<false>(xp) : zero;
      xr[u][1] = ok ? load16<false>(xp + 8) : zero;
#pragma unroll
      for (int r = 0; r < RN; ++r)
        wr[u][r] = ok ? load16<true>(Wt + (size_t)r * K + (size_t)q * 16) : zero;
    }
#pragma unroll
    for (int u = 0; u < U; ++u) {
      half4_t ax[4];  // activations under weight register c: x[4c .. 4c+3]
#pragma unroll
      for (int c = 0; c < 4; ++c) {
        const u32x4 xv = xr[u][c >> 1];
        ax[c] = __builtin_bit_cast(half4_t, (c & 1) ? u32x2{xv.z, xv.w} : u32x2{xv.x, xv.y});
      }
      if (use_zp) {
#pragma unroll
        for (int c = 0; c < 4; ++c) xsum = __builtin_amdgcn_mfma_f32_4x4x4f16(ax[c], ones, xsum, 0, 0, 0);
      }
#pragma unroll
      for (int c = 0; c < 4; ++c) {
#pragma unroll
        for (int r = 0; r < RN; ++r) {
          half2_t lo, hi;
          i8x4_to_half2x2(wr[u][r][c], lo, hi);
          const half4_t bw = {lo[0], lo[1], hi[0], hi[1]};
          acc[r] = __builtin_amdgcn_mfma_f32_4x4x4f16(ax[c], bw, acc[r], 0, 0, 0);
        }
      }
    }
  }

  // D[i][j] sits in element i of lane j: the diagonal element of this lane's block
  const bool odd = (lane & 1) != 0, upper = (lane & 2) != 0;
  auto diag = [&](const float4_t& v) {
    const float lo = odd ? v[1] : v[0], hi = odd ? v[3] : v[2];
    return upper ? hi : lo;
  };
#pragma unroll
  for (int r = 0; r < RN; ++r) {
    const float v = row16_allreduce(diag(acc[r]));
    if ((lane & 15) == 0) red[wave * 4 + (lane >> 4)][r] = v;
  }
  {
    const float xs = row16_allreduce(diag(xsum));
    if ((lane & 15) == 0) redx[wave * 4 + (lane >> 4)] = xs;
  }
  __syncthreads();
  if (threadIdx.x < RN) {
    const int r = threadIdx.x;
    const float sum = lds_sum<16>(&red[0][r], RN, nw * 4);
    const float xs = lds_sum<16>(&redx[0], 1, nw * 4);
    Y[n0 + r] = static_cast<half_t>((sum - zero_point * xs) * (scalar_scale * scale_value(scale_raw)));
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
    const int sum = lds_sum_i32(&red[0][r * MB + m], RN * MB, nw * 4);
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
// w4a16: unsigned 4-bit weights, two per byte, the low nibble first (element 2i in bits 0-3 of
// byte i, element 2i+1 in bits 4-7: uint4_2 of backend/cuda/hk/utility.cuh:13-36), fp16
// activations.  A register w of 8 nibbles n0..n7 becomes four half2 with four v_and_or and one
// shift, by letting the exponent absorb the nibble's position:
//   (w      & 0x000F000F) | 0x64006400 = (1024 + n0, 1024 + n4)     (w >> 8 likewise: n2, n6)
//   (w      & 0x00F000F0) | 0x54005400 = (  64 + n1,   64 + n5)     (w >> 8 likewise: n3, n7)
// The 1024 is subtracted in fp16 (exact); the 64 stays in and is removed once per output as
// 64·Σ x over the odd positions, which costs two v_dot2 per 8 activations shared by all rows
// (products of at most 79·|x| instead of 15·|x| in the fp32 sum: two bits of headroom, not ten).
// The activations are paired the same way, (x_j, x_{j+4}), once per chunk.
// Replaces gemv_quantized_int4 (backend/cuda/hk/fastgemv.cuh:394-495), which the reference
// defines but never launches.  Lanes along K: one 16-byte load = 32 weights of one row.
// Launched for one activation row; two to four rows take w4a16_r_kernel below.
// ---------------------------------------------------------------------------------------
template <int MB, int RN>
__global__ __launch_bounds__(256) void w4a16_kernel(const uint8_t* __restrict__ Wq,
                                                    const half_t* __restrict__ X,
                                                    const half_t* __restrict__ scale,
                                                    float scalar_scale, float zero_point,
                                                    half_t* __restrict__ Y, int M, int N, int K) {
  __shared__ float red[16][RN * MB];
  __shared__ float redx[16][MB];
  __shared__ float redo[16][MB];
  const int lane = threadIdx.x & 63;
  const int wave = threadIdx.x >> 6;
  const int nw = blockDim.x >> 6;
  const int n0 = blockIdx.x * RN;
  const int nq = K >> 5;        // 32-weight chunks per row
  const size_t rowb = (size_t)K >> 1;  // bytes per weight row
  const bool use_zp = zero_point != 0.f;
  // scale of the output this thread writes at the end, fetched ahead of the weight stream
  static_assert(RN * MB <= 64, "one output per thread of the first wave");
  const uint32_t scale_raw = scale_fetch(scale, n0 + (int)threadIdx.x % RN, threadIdx.x < RN * MB);

  float acc[RN][MB];
  float xsum[MB], xodd[MB];
#pragma unroll
  for (int m = 0; m < MB; ++m) {
    xsum[m] = 0.f;
    xodd[m] = 0.f;
#pragma unroll
    for (int r = 0; r < RN; ++r) acc[r][m] = 0.f;
  }
  const uint8_t* Wt = Wq + (size_t)n0 * rowb;
  const u32x4 zero = {0u, 0u, 0u, 0u};
  const half2_t ones = {static_cast<half_t>(1.f), static_cast<half_t>(1.f)};
  const half2_t bias = {static_cast<half_t>(1024.f), static_cast<half_t>(1024.f)};

  const int nsteps = (nq + nw * 64 - 1) / (nw * 64);
  int step = stagger_start(nsteps, 0);
  for (int it = 0; it < nsteps; ++it) {
    const int q = (step * nw + wave) * 64 + lane;
    step = step + 1 == nsteps ? 0 : step + 1;
    const bool ok = q < nq;
    u32x4 wr[RN];
#pragma unroll
    for (int r = 0; r < RN; ++r) wr[r] = ok ? load16<true>(Wt + (size_t)r * rowb + (size_t)q * 16) : zero;
    // xp[m][d][j] = (x[8d + j], x[8d + j + 4]) for the 8 activations under weight register d
    uint32_t xp[MB][4][4];
#pragma unroll
    for (int m = 0; m < MB; ++m) {
      const bool okm = ok && m < M;
      const half_t* xptr = X + (size_t)m * K + (size_t)q * 32;
#pragma unroll
      for (int d = 0; d < 4; ++d) {
        const u32x4 xv = okm ? load16<false>(xptr + 8 * d) : zero;  // x[8d .. 8d+7]
        xp[m][d][0] = __builtin_amdgcn_perm(xv.z, xv.x, 0x05040100u);  // (x0, x4)
        xp[m][d][1] = __builtin_amdgcn_perm(xv.z, xv.x, 0x07060302u);  // (x1, x5)
        xp[m][d][2] = __builtin_amdgcn_perm(xv.w, xv.y, 0x05040100u);  // (x2, x6)
        xp[m][d][3] = __builtin_amdgcn_perm(xv.w, xv.y, 0x07060302u);  // (x3, x7)
        xodd[m] = __builtin_amdgcn_fdot2(as_half2(xp[m][d][1]), ones, xodd[m], false);
        xodd[m] = __builtin_amdgcn_fdot2(as_half2(xp[m][d][3]), ones, xodd[m], false);
        if (use_zp) {
          xsum[m] = __builtin_amdgcn_fdot2(as_half2(xp[m][d][0]), ones, xsum[m], false);
          xsum[m] = __builtin_amdgcn_fdot2(as_half2(xp[m][d][2]), ones, xsum[m], false);
        }
      }
    }
#pragma unroll
    for (int r = 0; r < RN; ++r)
#pragma unroll
      for (int d = 0; d < 4; ++d) {
        const uint32_t w = wr[r][d], w8 = w >> 8;
        const half2_t wv[4] = {as_half2((w & 0x000F000Fu) | 0x64006400u) - bias,
                               as_half2((w & 0x00F000F0u) | 0x54005400u),
                               as_half2((w8 & 0x000F000Fu) | 0x64006400u) - bias,
                               as_half2((w8 & 0x00F000F0u) | 0x54005400u)};
#pragma unroll
        for (int j = 0; j < 4; ++j)
#pragma unroll
          for (int m = 0; m < MB; ++m)
            acc[r][m] = __builtin_amdgcn_fdot2(wv[j], as_half2(xp[m][d][j]), acc[r][m], false);
      }
  }

  // xsum holds Σ x over the even positions (only when a zero point needs it), xodd over the odd
#pragma unroll
  for (int m = 0; m < MB; ++m) {
#pragma unroll
    for (int r = 0; r < RN; ++r) {
      const float v = row16_allreduce(acc[r][m]);
      if ((lane & 15) == 0) red[wave * 4 + (lane >> 4)][r * MB + m] = v;
    }
    const float xe = row16_allreduce(xsum[m]);
    const float xo = row16_allreduce(xodd[m]);
    if ((lane & 15) == 0) {
      redx[wave * 4 + (lane >> 4)][m] = xe;
      redo[wave * 4 + (lane >> 4)][m] = xo;
    }
  }
  __syncthreads();
  for (int t = threadIdx.x; t < RN * MB; t += blockDim.x) {
    const int m = t / RN, r = t % RN;
    const float sum = lds_sum<16>(&red[0][r * MB + m], RN * MB, nw * 4);
    const float xe = lds_sum<16>(&redx[0][m], MB, nw * 4);
    const float xo = lds_sum<16>(&redo[0][m], MB, nw * 4);
    const int n = n0 + r;
    if (m < M)
      Y[(size_t)m * N + n] = static_cast<half_t>((sum - 64.f * xo - zero_point * (xe + xo)) *
                                                 (scalar_scale * scale_value(scale_raw)));
  }
}

// ---------------------------------------------------------------------------------------
// w8a16 with both operands staged through wave-private LDS (the int8 sibling of the fp16
// row-load kernel).  Per step a wave loads a 256-byte band (256 k) of the tile's 16 weight rows
// -- 4 rows x 256 B per instruction -- and the matching 512-byte band of the activation rows,
// parks them in LDS strips and reads them back in v_mfma_f32_16x16x32_f16 operand order: 8 bytes
// of one weight row per lane, converted to 8 fp16 there, against 16 bytes of one activation row.
// The activations are fetched once per 16 weight rows instead of once per 4, the dot products run
// on the matrix pipe, and the VALU only converts.  16-column tiles, 8 waves interleaving over K.
// XROWS = activation rows staged: 4, 8 or 16.
// ---------------------------------------------------------------------------------------
template <int XROWS, int NW, int BW, int CB>
__global__ __launch_bounds__(64 * NW) void w8a16_r_kernel(const int8_t* __restrict__ Wq,
                                                          const half_t* __restrict__ X,
                                                          const half_t* __restrict__ scale,
                                                          float scalar_scale, float zero_point,
                                                          half_t* __restrict__ Y, int M, int N, int K) {
  // BW: weight bytes (= k) per row and band, 256 or 128.  CB: 16-column blocks per tile sharing the
  // staged activations (tile = 16 * CB columns).  BW = 128 with CB = 2 reads half the activation
  // bytes per weight byte of BW = 256 with CB = 1.
  constexpr int BX = 2 * BW;           // activation bytes per row and band
  constexpr int LPW = BW / 16;         // lanes per weight row piece
  constexpr int RPW = 64 / LPW;        // weight rows per load instruction
  constexpr int WI = 16 * CB / RPW;    // weight load instructions per step
  constexpr int LPX = BX / 16;         // lanes per activation row piece
  constexpr int RPX = 64 / LPX;        // activation rows per load instruction
  constexpr int XI = XROWS / RPX;      // activation load instructions per step
  constexpr int UNITS = BW / 32;       // 32-wide MFMA K units per band
  constexpr int RSW = BW + 16;         // LDS bytes per staged weight row
  constexpr int RSX = BX + 16;         // ... per staged activation row
  constexpr int WSTRIP = 16 * CB * RSW;
  constexpr int XSTRIP = XROWS * RSX;
  constexpr int WAVE_LDS = WSTRIP + XSTRIP;
  static_assert(XROWS % RPX == 0, "whole load instructions");
  static_assert(WAVE_LDS >= 2 * CB * 256 * (int)sizeof(float), "reduction scratch fits");
  __shared__ __attribute__((aligned(16))) unsigned char smem[NW * WAVE_LDS];
  const int lane = threadIdx.x & 63;
  const int wave = threadIdx.x >> 6;
  const int nw = blockDim.x >> 6;
  const int j = lane & 15, g = lane >> 4;          // operand order
  const int hw = lane / LPW, cw = lane % LPW;      // weight load order: row RPW*i + hw, piece cw
  const int hx = lane / LPX, cx = lane % LPX;      // activation load order: row RPX*i + hx, piece cx
  const int n0 = blockIdx.x * (16 * CB);
  const int nbands = (K + BW - 1) / BW;            // K % 128 == 0: the last band may be partial
  const bool use_zp = zero_point != 0.f;
  // scale of the output this thread writes at the end, fetched ahead of the weight stream
  static_assert(16 * 16 * CB <= 64 * NW, "one output per thread");
  const uint32_t scale_raw =
      scale_fetch(scale, n0 + (int)threadIdx.x % (16 * CB), threadIdx.x < 16 * 16 * CB);
  unsigned char* wstrip = smem + wave * WAVE_LDS;
  unsigned char* xstrip = wstrip + WSTRIP;
  const u32x4 zero = {0u, 0u, 0u, 0u};

  const int8_t* Wp = Wq + (size_t)(n0 + hw) * K + cw * 16;
  const half_t* Xp = X + (size_t)hx * K + cx * 8;
  bool xrow[XI];
#pragma unroll
  for (int i = 0; i < XI; ++i) xrow[i] = (RPX * i + hx) < M;
  const int stw_off = hw * RSW + cw * 16;
  const int stx_off = hx * RSX + cx * 16;
  const int ldw_off = j * RSW + g * 8;
  const int ldx_off = (j % XROWS) * RSX + g * 16;  // MFMA rows beyond XROWS re-read staged rows; unused

  auto load_band = [&](int band, u32x4(&w)[WI], u32x4(&x)[XI]) {
    const bool okw = band < nbands && (band * BW + cw * 16) < K;
    const bool okx = band < nbands && (band * BW + cx * 8) < K;
#pragma unroll
    for (int i = 0; i < WI; ++i)
      w[i] = okw ? load16<true>(Wp + (size_t)(RPW * i) * K + (size_t)band * BW) : zero;
#pragma unroll
    for (int i = 0; i < XI; ++i)
      x[i] = (okx && xrow[i]) ? load16<false>(Xp + (size_t)(RPX * i) * K + (size_t)band * BW) : zero;
  };
  float4_t acc[CB], xacc = {0.f, 0.f, 0.f, 0.f};
#pragma unroll
  for (int b = 0; b < CB; ++b) acc[b] = float4_t{0.f, 0.f, 0.f, 0.f};
  const half8_t ones8 = {static_cast<half_t>(1.f), static_cast<half_t>(1.f), static_cast<half_t>(1.f),
                         static_cast<half_t>(1.f), static_cast<half_t>(1.f), static_cast<half_t>(1.f),
                         static_cast<half_t>(1.f), static_cast<half_t>(1.f)};
  auto multiply = [&](const u32x4(&w)[WI], const u32x4(&x)[XI]) {
#pragma unroll
    for (int i = 0; i < WI; ++i) *reinterpret_cast<u32x4*>(wstrip + stw_off + RPW * i * RSW) = w[i];
#pragma unroll
    for (int i = 0; i < XI; ++i) *reinterpret_cast<u32x4*>(xstrip + stx_off + RPX * i * RSX) = x[i];
    wave_lds_sync();
#pragma unroll
    for (int u = 0; u < UNITS; ++u) {
      const u32x4 xv = *reinterpret_cast<const u32x4*>(xstrip + ldx_off + u * 64);
#pragma unroll
      for (int b = 0; b < CB; ++b) {
        const u32x2 wv = *reinterpret_cast<const u32x2*>(wstrip + b * 16 * RSW + ldw_off + u * 32);
        half2_t h0, h1, h2, h3;
        i8x4_to_half2x2(wv.x, h0, h1);
        i8x4_to_half2x2(wv.y, h2, h3);
        const half8_t wb = {h0[0], h0[1], h1[0], h1[1], h2[0], h2[1], h3[0], h3[1]};
        acc[b] = __builtin_amdgcn_mfma_f32_16x16x32_f16(as_half8(xv), wb, acc[b], 0, 0, 0);
      }
      if (use_zp) xacc = __builtin_amdgcn_mfma_f32_16x16x32_f16(as_half8(xv), ones8, xacc, 0, 0, 0);
    }
    wave_lds_sync();
  };

  u32x4 w0[WI], w1[WI], x0[XI], x1[XI];
  const int nsteps = (nbands + nw - 1) / nw;
  int step = stagger_start(nsteps, 0);
  auto next_band = [&]() {
    const int band = step * nw + wave;
    step = step + 1 == nsteps ? 0 : step + 1;
    return band;
  };
  load_band(next_band(), w0, x0);
  for (int it = 0; it < nsteps; it += 2) {
    if (it + 1 < nsteps) load_band(next_band(), w1, x1);
    multiply(w0, x0);
    if (it + 1 >= nsteps) break;
    if (it + 2 < nsteps) load_band(next_band(), w0, x0);
    multiply(w1, x1);
  }

  // acc[b][r] = D[m = 4g + r][column 16b + j] (xacc: sum of x of row m in every column); the waves
  // meet in LDS: red[wave][0] = products [16][16*CB], red[wave][1] = activation sums [16][16]
  constexpr int TN = 16 * CB;
  __syncthreads();
  float(*red)[2][16 * TN] = reinterpret_cast<float(*)[2][16 * TN]>(smem);
#pragma unroll
  for (int r = 0; r < 4; ++r) {
#pragma unroll
    for (int b = 0; b < CB; ++b) red[wave][0][(4 * g + r) * TN + 16 * b + j] = acc[b][r];
    red[wave][1][(4 * g + r) * 16 + j] = xacc[r];
  }
  __syncthreads();
  for (int e = threadIdx.x; e < 16 * TN; e += blockDim.x) {
    const int m = e / TN, n = n0 + e % TN;
    if (m < M) {
      const float sum = lds_sum<NW>(&red[0][0][e], 2 * 16 * TN, nw);
      const float xs = lds_sum<NW>(&red[0][1][m * 16 + (e & 15)], 2 * 16 * TN, nw);
      Y[(size_t)m * N + n] =
          static_cast<half_t>((sum - zero_point * xs) * (scalar_scale * scale_value(scale_raw)));
    }
  }
}

// ---------------------------------------------------------------------------------------
// w4a16 with both operands staged through wave-private LDS (4-bit sibling of w8a16_r_kernel).
// A band is 512 k: 256 bytes of each of the tile's 16 weight rows (4 rows x 256 B per load
// instruction) and 1 KB of each activation row (one row per instruction).  The activations are
// parked already paired the way the nibble conversion produces its halves -- (x0,x4),(x1,x5),
// (x2,x6),(x3,x7) per 8 k -- so the 4 bytes a lane reads per MFMA unit turn into the B operand with
// one shift, four v_and_or and four exact fp16 subtractions, and the dot products run on the
// matrix pipe.  XROWS = activation rows staged (2 or 4).
// ---------------------------------------------------------------------------------------
template <int XROWS>
__global__ __launch_bounds__(512) void w4a16_r_kernel(const uint8_t* __restrict__ Wq,
                                                      const half_t* __restrict__ X,
                                                      const half_t* __restrict__ scale,
                                                      float scalar_scale, float zero_point,
                                                      half_t* __restrict__ Y, int M, int N, int K) {
  constexpr int NW = 8;
  constexpr int RSW = 256 + 16;      // LDS bytes per staged weight row (512 k)
  constexpr int RSX = 1024 + 16;     // ... per staged activation row
  constexpr int WSTRIP = 16 * RSW;
  constexpr int XSTRIP = XROWS * RSX;
  constexpr int WAVE_LDS = WSTRIP + XSTRIP;
  static_assert(WAVE_LDS >= 2 * 256 * (int)sizeof(float), "reduction scratch fits");
  __shared__ __attribute__((aligned(16))) unsigned char smem[NW * WAVE_LDS];
  const int lane = threadIdx.x & 63;
  const int wave = threadIdx.x >> 6;
  const int nw = blockDim.x >> 6;
  const int j = lane & 15, g = lane >> 4;        // operand order
  const int hw = lane >> 4, cw = lane & 15;      // weight load order: row 4i + hw, piece cw (32 k)
  const int n0 = blockIdx.x * 16;
  const int nbands = (K + 511) >> 9;             // K % 128 == 0: the last band may be partial
  const size_t rowb = (size_t)K >> 1;            // bytes per weight row
  const bool use_zp = zero_point != 0.f;
  // scale of the output this thread writes at the end, fetched ahead of the weight stream
  const uint32_t scale_raw = scale_fetch(scale, n0 + (int)(threadIdx.x & 15), threadIdx.x < 256);
  unsigned char* wstrip = smem + wave * WAVE_LDS;
  unsigned char* xstrip = wstrip + WSTRIP;
  const u32x4 zero = {0u, 0u, 0u, 0u};

  const uint8_t* Wp = Wq + (size_t)(n0 + hw) * rowb + cw * 16;
  const half_t* Xp = X + lane * 8;
  const int stw_off = hw * RSW + cw * 16;
  const int stx_off = lane * 16;
  const int ldw_off = j * RSW + g * 4;
  const int ldx_off = (j % XROWS) * RSX + g * 16;  // MFMA rows beyond XROWS re-read staged rows; unused

  auto load_band = [&](int band, u32x4(&w)[4], u32x4(&x)[XROWS]) {
    const bool okw = band < nbands && (band * 512 + cw * 32) < K;
    const bool okx = band < nbands && (band * 512 + lane * 8) < K;
#pragma unroll
    for (int i = 0; i < 4; ++i) w[i] = okw ? load16<true>(Wp + (size_t)(4 * i) * rowb + (size_t)band * 256) : zero;
#pragma unroll
    for (int i = 0; i < XROWS; ++i)
      x[i] = (okx && i < M) ? load16<false>(Xp + (size_t)i * K + (size_t)band * 512) : zero;
  };
  float4_t acc = {0.f, 0.f, 0.f, 0.f}, xacc = {0.f, 0.f, 0.f, 0.f};
  const half8_t ones8 = {static_cast<half_t>(1.f), static_cast<half_t>(1.f), static_cast<half_t>(1.f),
                         static_cast<half_t>(1.f), static_cast<half_t>(1.f), static_cast<half_t>(1.f),
                         static_cast<half_t>(1.f), static_cast<half_t>(1.f)};
  const half2_t b1024 = {static_cast<half_t>(1024.f), static_cast<half_t>(1024.f)};
  const half2_t b64 = {static_cast<half_t>(64.f), static_cast<half_t>(64.f)};
  auto multiply = [&](const u32x4(&w)[4], const u32x4(&x)[XROWS]) {
#pragma unroll
    for (int i = 0; i < 4; ++i) *reinterpret_cast<u32x4*>(wstrip + stw_off + 4 * i * RSW) = w[i];
#pragma unroll
    for (int i = 0; i < XROWS; ++i) {
      const u32x4 xv = x[i];  // x0..x7 -> (x0,x4) (x1,x5) (x2,x6) (x3,x7)
      const u32x4 xp = {__builtin_amdgcn_perm(xv.z, xv.x, 0x05040100u), __builtin_amdgcn_perm(xv.z, xv.x, 0x07060302u),
                        __builtin_amdgcn_perm(xv.w, xv.y, 0x05040100u), __builtin_amdgcn_perm(xv.w, xv.y, 0x07060302u)};
      *reinterpret_cast<u32x4*>(xstrip + stx_off + i * RSX) = xp;
    }
    wave_lds_sync();
#pragma unroll
    for (int u = 0; u < 16; ++u) {
      const u32x4 xa = *reinterpret_cast<const u32x4*>(xstrip + ldx_off + u * 64);
      const uint32_t wd = *reinterpret_cast<const uint32_t*>(wstrip + ldw_off + u * 16), w8 = wd >> 8;
      const half2_t p0 = as_half2((wd & 0x000F000Fu) | 0x64006400u) - b1024;   // (n0, n4)
      const half2_t p1 = as_half2((wd & 0x00F000F0u) | 0x54005400u) - b64;     // (n1, n5)
      const half2_t p2 = as_half2((w8 & 0x000F000Fu) | 0x64006400u) - b1024;   // (n2, n6)
      const half2_t p3 = as_half2((w8 & 0x00F000F0u) | 0x54005400u) - b64;     // (n3, n7)
      const half8_t wb = {p0[0], p0[1], p1[0], p1[1], p2[0], p2[1], p3[0], p3[1]};
      acc = __builtin_amdgcn_mfma_f32_16x16x32_f16(as_half8(xa), wb, acc, 0, 0, 0);
      if (use_zp) xacc = __builtin_amdgcn_mfma_f32_16x16x32_f16(as_half8(xa), ones8, xacc, 0, 0, 0);
    }
    wave_lds_sync();
  };

  u32x4 w0[4], w1[4], x0[XROWS], x1[XROWS];
  const int nsteps = (nbands + nw - 1) / nw;
  int step = stagger_start(nsteps, 0);
  auto next_band = [&]() {
    const int band = step * nw + wave;
    step = step + 1 == nsteps ? 0 : step + 1;
    return band;
  };
  load_band(next_band(), w0, x0);
  for (int it = 0; it < nsteps; it += 2) {
    if (it + 1 < nsteps) load_band(next_band(), w1, x1);
    multiply(w0, x0);
    if (it + 1 >= nsteps) break;
    if (it + 2 < nsteps) load_band(next_band(), w0, x0);
    multiply(w1, x1);
  }

  // acc[r] = D[m = 4g + r][column j] (xacc: sum of x of row m in every column); waves meet in LDS
  __syncthreads();
  float(*red)[2][256] = reinterpret_cast<float(*)[2][256]>(smem);
#pragma unroll
  for (int r = 0; r < 4; ++r) {
    red[wave][0][(4 * g + r) * 16 + j] = acc[r];
    red[wave][1][(4 * g + r) * 16 + j] = xacc[r];
  }
  __syncthreads();
  for (int e = threadIdx.x; e < 256; e += blockDim.x) {
    const int m = e >> 4, n = n0 + (e & 15);
    if (m < M) {
      const float sum = lds_sum<NW>(&red[0][0][e], 512, nw);
      const float xs = lds_sum<NW>(&red[0][1][e], 512, nw);
      Y[(size_t)m * N + n] =
          static_cast<half_t>((sum - zero_point * xs) * (scalar_scale * scale_value(scale_raw)));
    }
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

// Measured (us per call; lanes-along-K kernel / row-load kernel on 256-byte bands):
//   K = N = 8192   M=1 12.6 / 14.3   M=2 15.1 / 14.2   M=4 21.1 / 14.9   M=8 32.9 / 17.2
//   K = N = 16384  M=1 41.2 / 44.8   M=8  -   / 49.7
// The row-load kernel exists with 8 waves only.
bool launch_w8a16(const W8A16Args& a, hipStream_t s) {
  auto* Wq = static_cast<const int8_t*>(a.Wq);
  auto* X = static_cast<const half_t*>(a.x);
  auto* sc = static_cast<const half_t*>(a.scale);
  auto* Y = static_cast<half_t*>(a.y);
  const int t32 = a.N / 32;
  // 32-column tiles on 128-byte bands read half the activation bytes per weight byte.  Measured
  // against 16-column tiles (us):
  //  * two workgroups (16 waves) on every CU, 448..512 tiles or a multiple of 512: K = N = 16384 M=8
  //    44.8 / 49.3, K=4096 N=16384 14.9 / 17.3, K=4096 N=14336 M=8 13.7 / 14.5 -- but not with rows
  //    8 KB apart: K=8192 N=16384 M=8 27.6 / 25.2;
  //  * one workgroup on every CU (N = 8192): long rows or 15..16 activation rows only, K=16384 M=8
  //    25.4 / 27.3, K=28672 M=14 47.8 / 55.4, K=4096 M=16 10.5 / 11.1, against K=8192 M=8 16.9 /
  //    14.9, K=28672 M=4 40.0 / 38.7, K=2048 M=16 7.7 / 7.1;
  //  * 13..16 rows from 160 tiles on: N=5120 K=11008 M=16 19.5 / 23.0, N=14336 K=14336 44.5 / 55.1.
  const bool aligned = a.N % 32 == 0;
  const bool two_per_cu = aligned && ((t32 >= 448 && t32 <= 512) || (t32 >= 512 && t32 % 512 == 0)) &&
                          (a.K != 8192 || a.M > 8);
  const bool one_per_cu = aligned && t32 == 256 &&
                          ((a.M >= 15 && a.K >= 4096) || (a.K >= 16384 && (a.M >= 5 || a.K < 24576)));
  const bool many_rows = aligned && a.M >= 13 && t32 >= 160 && t32 != 256;
  const bool wide = two_per_cu || one_per_cu || many_rows;
  // 16-column tiles take 128-byte bands (smaller strips, more steps in flight): M=8, 128- / 256-byte
  // bands: K = N = 8192 14.5 / 15.7, K = N = 4096 7.0 / 7.3, K=4096 N=14336 14.6 / 16.1, K=11008
  // N=5120 17.7 / 19.3 -- except long rows of narrow outputs, K=14336 N=4096 M=4 14.8 / 13.9.
  const bool bw256 = a.N <= 4096 && a.K >= 14336;
#define FG_W8A16_R(XR, BW, CB)                                                                    \
  hipLaunchKernelGGL((w8a16_r_kernel<XR, 8, BW, CB>), dim3(a.N / (16 * CB)), dim3(512), 0, s, Wq, \
                     X, sc, a.scalar_scale, a.zero_point, Y, a.M, a.N, a.K)
  if (a.M == 1) {  // 4 rows per workgroup, one load group in flight
    const int nw = i8_waves(a.K);
    if ((a.K / 16) % (64 * nw) == 0)
      hipLaunchKernelGGL((w8a16_m1_kernel<4, 1, true>), dim3(a.N / 4), dim3(64 * nw), 0, s, Wq, X, sc,
                         a.scalar_scale, a.zero_point, Y, a.N, a.K);
    else
      hipLaunchKernelGGL((w8a16_m1_kernel<4, 1, false>), dim3(a.N / 4), dim3(64 * nw), 0, s, Wq, X, sc,
                         a.scalar_scale, a.zero_point, Y, a.N, a.K);
  } else if (a.M <= 4 && (a.N <= 2048 || (a.M == 2 && a.N <= 6144))) {
    // narrow outputs leave the 16-column tiles of the row-load kernel on half the CUs or fewer: lanes
    // along K, four weight rows a workgroup (N=2048 K=8192: M=2 8.8 -> 6.0 us, M=4 9.0 -> 7.3;
    // N=1024 K=4096 M=4 5.8 -> 4.4; N=4096 K=8192 M=4 9.6 -> 11.6 the other way; two rows up to
    // N = 6144: N=4096 K=8192 9.5 -> 9.1, N=8192 K=4096 8.6 -> 9.0)
    if (a.M <= 2)
      hipLaunchKernelGGL((w8a16_kernel<2, 4, 1>), dim3(a.N / 4), dim3(64 * i8_waves(a.K)), 0, s, Wq, X,
                         sc, a.scalar_scale, a.zero_point, Y, a.M, a.N, a.K);
    else
      hipLaunchKernelGGL((w8a16_kernel<4, 4, 1>), dim3(a.N / 4), dim3(64 * i8_waves(a.K)), 0, s, Wq, X,
                         sc, a.scalar_scale, a.zero_point, Y, a.M, a.N, a.K);
  } else if (a.M <= 4) {  // 2 rows take the 4-row strip too: K=14336 N=4096 M=2 13.1 us
    if (wide) FG_W8A16_R(4, 128, 2);
    else if (bw256) FG_W8A16_R(4, 256, 1);
    else FG_W8A16_R(4, 128, 1);
  } else if (a.M <= 8) {
    if (wide) FG_W8A16_R(8, 128, 2);
    else if (bw256) FG_W8A16_R(8, 256, 1);
    else FG_W8A16_R(8, 128, 1);
  } else if (a.M <= 16) {
    // 16-row activation strip on 128-byte bands only (the 256-byte form would need 100 KB of LDS)
    if (wide) FG_W8A16_R(16, 128, 2);
    else FG_W8A16_R(16, 128, 1);
  } else {
    return false;
  }
#undef FG_W8A16_R
  return true;
}

bool launch_w4a16(const W8A16Args& a, hipStream_t s) {
  auto* Wq = static_cast<const uint8_t*>(a.Wq);
  auto* X = static_cast<const half_t*>(a.x);
  auto* sc = static_cast<const half_t*>(a.scale);
  auto* Y = static_cast<half_t*>(a.y);
  if (a.M < 1 || a.M > 4) return false;
  if (a.M == 1) {
    // one activation row: the dot2 kernel's straight 1 KB row pieces are the shorter path
    const int pieces = (a.K / 32 + 63) / 64;  // 1 KB pieces per weight row
    const dim3 block(64 * (pieces >= 4 ? 4 : (pieces >= 2 ? 2 : 1)));
    // rows longer than 4 KB: eight rows a workgroup share each activation piece (K = N = 16384
    // 29.9 -> 26.6 us, N=4096 K=14336 10.5 -> 9.5; K = N = 8192 10.15 -> 10.24 the other way)
    if (a.K > 8192 && a.N % 8 == 0)
      hipLaunchKernelGGL((w4a16_kernel<1, 8>), dim3(a.N / 8), block, 0, s, Wq, X, sc, a.scalar_scale,
                         a.zero_point, Y, a.M, a.N, a.K);
    else
      hipLaunchKernelGGL((w4a16_kernel<1, 4>), dim3(a.N / 4), block, 0, s, Wq, X, sc, a.scalar_scale,
                         a.zero_point, Y, a.M, a.N, a.K);
  } else if (a.M == 2) {
    hipLaunchKernelGGL((w4a16_r_kernel<2>), dim3(a.N / 16), dim3(512), 0, s, Wq, X, sc, a.scalar_scale,
                       a.zero_point, Y, a.M, a.N, a.K);
  } else {
    hipLaunchKernelGGL((w4a16_r_kernel<4>), dim3(a.N / 16), dim3(512), 0, s, Wq, X, sc, a.scalar_scale,
                       a.zero_point, Y, a.M, a.N, a.K);
  }
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
