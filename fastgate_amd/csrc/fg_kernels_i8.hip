// int8- and int4-weight GEMV kernels, weights [N,K] row-major.
//
//  * w8a16 / w4a16: fp16 activations.  The integers reach v_dot2_f32_f16 or the MFMA as fp16
//    subnormals (a byte or nibble in the low mantissa bits under a zero exponent is that number
//    times 2^-24, exactly; see wq_m1_kernel), products and sums are fp32, and the per-output-channel
//    scale and the zero point are applied once per output.
//  * i8i8: int8 activations, v_dot4_i32_i8, exact int32 result.
//
// Replaces the device side of gemv_quantized_int8 (backend/cuda/hk/fastgemv.cuh:316-389,
// 8-byte loads, int8 -> fp32 convert, scalar FMAs) of the reference.
#include "fg_device.h"
#include "fg_internal.h"

namespace fg {

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

// The zero point (and the 128 that the subnormal form of int8 carries) leaves a dot product as one
// term, constant x Σx.  An activation row that holds an infinity or a NaN makes Σx non-finite, and
// that term would then turn every output of the row into NaN, where element-by-element arithmetic
// -- sum += x (float(w) - zp), backend/cuda/hk/fastgemv.cuh:344-363 -- gives ±inf when infinities
// of one sign meet weights on one side of the zero point.  Σx is non-finite for such rows only
// (finite halves cannot overflow an fp32 sum), so the thread that writes an output looks at it
// and, for such a row, computes its one output again the reference's way: K steps in one thread,
// paid only by input that is already broken.  BITS = 4: two nibbles a byte, the even k low.
__device__ __forceinline__ bool not_finite(float v) { return !(__builtin_fabsf(v) <= 3.4028234664e38f); }
template <int BITS>
__device__ float elementwise_dot(const uint8_t* __restrict__ wrow, const half_t* __restrict__ xrow, int K,
                                 float zero_point) {
  float s = 0.f;
  for (int k = 0; k < K; ++k) {
    int w;
    if (BITS == 8) {
      w = static_cast<int8_t>(wrow[k]);
    } else {
      const uint32_t b = wrow[k >> 1];
      w = (k & 1) ? b >> 4 : b & 15u;
    }
    s += static_cast<float>(xrow[k]) * (static_cast<float>(w) - zero_point);
  }
  return s;
}

// ---------------------------------------------------------------------------------------
// MR activation rows: one (the GEMV proper), and up to four where the launchers say so; int8 and int4
// weights.
//  * Lanes own 8 activations each, not 16 weight bytes: a chunk is UD 16-byte units of x a lane
//    (unit 64 d + lane, d < UD), so every x load is one contiguous KB per wave, and the weights
//    under a unit are 8 bytes (int8) or 4 bytes (int4) per row: UD 8- or 4-byte loads a row,
//    each contiguous over the wave.  With 16 weight bytes a lane, the lane's x is 32 or 64
//    bytes at that stride from its neighbour's: two or four loads that each touch every cache
//    line of the wave's span, which cost more than the weight loads themselves.
//  * The integers reach v_dot2_f32_f16 as fp16 subnormals: a byte or nibble in the low mantissa
//    bits of a half with a zero exponent field IS that number times 2^-24 (a nibble in bits 4-7:
//    times 2^-20), exactly.  Kernels keep fp16 subnormals (the compiler's default float mode
//    for gfx9), products and sums are fp32, and the power of two is put back once per output.
//    int8: 3 integer operations per 4 weights (sign flip to w + 128, two byte shuffles), the 128
//    taken out once per output as 128 Σx; int4: 5 per 8 weights (a shift, four masks) and no
//    constant at all -- against 5 and 7 with a bias to subtract in fp16.
//  * Waves of a workgroup interleave over the chunks of K; 16-lane sums by DPP, the rest through
//    LDS in a fixed order.
// K = N = 8192, one GPU, us per call: int4 9.5 -> 7.6 (a plain read of the 32 MiB: 6.1).  The x
// loads still cost 0.8 us of that (timed with x replaced by constants), for int8 too: 4 KB of x
// from L2 per 4 KB of weights from memory, whatever cache policy the weight loads carry; staging x
// in LDS once per 16-wave workgroup moves the cost into the wait before the first decode.
// Replaces the device side of gemv_quantized_int8 (backend/cuda/hk/fastgemv.cuh:316-389) and of
// gemv_quantized_int4 (:394-495, defined there but never launched) for one row.
// ---------------------------------------------------------------------------------------
template <int BITS, int RN, int NWV, int UD, int MR>
__global__ __launch_bounds__(64 * NWV) void wq_m1_kernel(const uint8_t* __restrict__ Wq,
                                                         const half_t* __restrict__ X,
                                                         const half_t* __restrict__ scale,
                                                         float scalar_scale, float zero_point,
                                                         half_t* __restrict__ Y, int N, int K) {
  constexpr int WB = BITS == 4 ? 4 : 8;  // weight bytes under one 16-byte unit of x
  typedef uint32_t wreg_t __attribute__((ext_vector_type(WB / 4)));
  constexpr int RC = RN + 1;             // columns of the reduction table per activation row: RN sums and Σx
  __shared__ float red[NWV * 4][MR * RC];
  const int lane = threadIdx.x & 63;
  const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);  // uniform: addresses stay scalar
  const int n0 = blockIdx.x * RN;
  const size_t rowb = BITS == 4 ? (size_t)K >> 1 : (size_t)K;
  static_assert(MR * RN <= 64, "one output per thread of the first wave");
  const uint32_t scale_raw = scale_fetch(scale, n0 + (int)threadIdx.x % RN, threadIdx.x < MR * RN);
  // the constant that comes out with Σx: the zero point, and int8's + 128
  const float zp = BITS == 4 ? zero_point : zero_point + 128.f;
  const bool use_xsum = zp != 0.f;
  const uint8_t* Wt = Wq + (size_t)n0 * rowb;  // uniform; the lane's part is a 32-bit offset
  const uint32_t lane_w = lane * WB, lane_x = lane * 16;
  const half2_t ones = {static_cast<half_t>(1.f), static_cast<half_t>(1.f)};
  float acc0[MR][RN], acc1[MR][RN];
  float xsum[MR];
#pragma unroll
  for (int m = 0; m < MR; ++m) {
    xsum[m] = 0.f;
#pragma unroll
    for (int r = 0; r < RN; ++r) acc0[m][r] = acc1[m][r] = 0.f;
  }

  constexpr int kNonTemporal = 2;  // the nt bit of a buffer load's cache policy
  const __amdgpu_buffer_rsrc_t wrs =
      __builtin_amdgcn_make_buffer_rsrc(const_cast<uint8_t*>(Wt), 0, (int)(RN * rowb), 0x00020000);
  __amdgpu_buffer_rsrc_t xrs[MR];
#pragma unroll
  for (int m = 0; m < MR; ++m)
    xrs[m] = __builtin_amdgcn_make_buffer_rsrc(const_cast<half_t*>(X + (size_t)m * K), 0, K * 2, 0x00020000);
  const int nunits = K >> 3;
  const int nchunks = (nunits + 64 * UD - 1) / (64 * UD);
  for (int ch = wave; ch < nchunks; ch += NWV) {
    wreg_t wr[RN][UD];
    u32x4 xv[MR][UD];
    // Buffer loads: a lane past the end of K gets zeros for x (the descriptor ends with the row), so
    // whatever its weight load returns -- the start of the next row, or zeros past the workgroup's
    // last row -- multiplies to zero: no predicate, no branch around any of the loads.
#pragma unroll
    for (int r = 0; r < RN; ++r)
#pragma unroll
      for (int d = 0; d < UD; ++d) {
        const int off = r * (int)rowb + (ch * (64 * UD) + 64 * d) * WB + (int)lane_w;
        if constexpr (WB == 4) wr[r][d][0] = __builtin_amdgcn_raw_buffer_load_b32(wrs, off, 0, kNonTemporal);
        else wr[r][d] = __builtin_bit_cast(wreg_t, __builtin_amdgcn_raw_buffer_load_b64(wrs, off, 0, kNonTemporal));
      }
#pragma unroll
    for (int m = 0; m < MR; ++m)
#pragma unroll
      for (int d = 0; d < UD; ++d)
        xv[m][d] = __builtin_bit_cast(u32x4, __builtin_amdgcn_raw_buffer_load_b128(
                                                 xrs[m], (ch * (64 * UD) + 64 * d) * 16 + (int)lane_x, 0, 0));
    if (use_xsum) {
#pragma unroll
      for (int m = 0; m < MR; ++m)
#pragma unroll
        for (int d = 0; d < UD; ++d)
#pragma unroll
          for (int i = 0; i < 4; ++i) xsum[m] = __builtin_amdgcn_fdot2(as_half2(xv[m][d][i]), ones, xsum[m], false);
    }
    if (BITS == 4) {  // (x_j, x_{j+4}): the halves that meet nibbles j and j + 4 of a register
#pragma unroll
      for (int m = 0; m < MR; ++m)
#pragma unroll
        for (int d = 0; d < UD; ++d) {
          const u32x4 t = xv[m][d];
          xv[m][d].x = __builtin_amdgcn_perm(t.z, t.x, 0x05040100u);
          xv[m][d].y = __builtin_amdgcn_perm(t.z, t.x, 0x07060302u);
          xv[m][d].z = __builtin_amdgcn_perm(t.w, t.y, 0x05040100u);
          xv[m][d].w = __builtin_amdgcn_perm(t.w, t.y, 0x07060302u);
        }
    }
#pragma unroll
    for (int r = 0; r < RN; ++r)
#pragma unroll
      for (int d = 0; d < UD; ++d) {
        if constexpr (BITS == 4) {
          const uint32_t w = wr[r][d][0], w8 = w >> 8;  // nibbles 0,4 | 1,5 | 2,6 | 3,7
          const uint32_t n04 = w & 0x000F000Fu, n15 = w & 0x00F000F0u, n26 = w8 & 0x000F000Fu, n37 = w8 & 0x00F000F0u;
#pragma unroll
          for (int m = 0; m < MR; ++m) {
            acc0[m][r] = __builtin_amdgcn_fdot2(as_half2(n04), as_half2(xv[m][d].x), acc0[m][r], false);
            acc1[m][r] = __builtin_amdgcn_fdot2(as_half2(n15), as_half2(xv[m][d].y), acc1[m][r], false);
            acc0[m][r] = __builtin_amdgcn_fdot2(as_half2(n26), as_half2(xv[m][d].z), acc0[m][r], false);
            acc1[m][r] = __builtin_amdgcn_fdot2(as_half2(n37), as_half2(xv[m][d].w), acc1[m][r], false);
          }
        } else {
#pragma unroll
          for (int h = 0; h < 2; ++h) {
            const uint32_t t = wr[r][d][h] ^ 0x80808080u;  // w + 128 as unsigned bytes
            const uint32_t b01 = __builtin_amdgcn_perm(0u, t, 0x04010400u);  // halves (b0, b1)
            const uint32_t b23 = __builtin_amdgcn_perm(0u, t, 0x04030402u);  // halves (b2, b3)
#pragma unroll
            for (int m = 0; m < MR; ++m) {
              acc0[m][r] = __builtin_amdgcn_fdot2(as_half2(b01), as_half2(xv[m][d][2 * h]), acc0[m][r], false);
              acc1[m][r] = __builtin_amdgcn_fdot2(as_half2(b23), as_half2(xv[m][d][2 * h + 1]), acc1[m][r], false);
            }
          }
        }
      }
  }

#pragma unroll
  for (int m = 0; m < MR; ++m) {
#pragma unroll
    for (int r = 0; r < RN; ++r) {
      // int4: acc1 holds the nibbles that sat 4 bits up
      const float a = BITS == 4 ? acc0[m][r] * 16777216.f + acc1[m][r] * 1048576.f
                                : (acc0[m][r] + acc1[m][r]) * 16777216.f;
      const float v = row16_allreduce(a);
      if ((lane & 15) == 0) red[wave * 4 + (lane >> 4)][m * RC + r] = v;
    }
    const float xs = row16_allreduce(xsum[m]);
    if ((lane & 15) == 0) red[wave * 4 + (lane >> 4)][m * RC + RN] = xs;
  }
  __syncthreads();
  if (threadIdx.x < MR * RN) {
    const int m = threadIdx.x / RN, r = threadIdx.x % RN;
    const float sum = lds_sum<NWV * 4>(&red[0][m * RC + r], MR * RC, NWV * 4);
    const float xs = lds_sum<NWV * 4>(&red[0][m * RC + RN], MR * RC, NWV * 4);
    float v = sum - zp * xs;
    if (not_finite(xs)) v = elementwise_dot<BITS>(Wt + (size_t)r * rowb, X + (size_t)m * K, K, zero_point);
    Y[(size_t)m * N + n0 + r] = static_cast<half_t>(v * (scalar_scale * scale_value(scale_raw)));
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
// w8a16 with both operands staged through wave-private LDS (the int8 sibling of the fp16
// row-load kernel).  Per step a wave loads a 256-byte band (256 k) of the tile's 16 weight rows
// -- 4 rows x 256 B per instruction -- and the matching 512-byte band of the activation rows,
// parks them in LDS strips and reads them back in v_mfma_f32_16x16x32_f16 operand order: 8 bytes
// of one weight row per lane, converted to 8 fp16 there, against 16 bytes of one activation row.
// The activations are fetched once per 16 weight rows instead of once per 4, the dot products run
// on the matrix pipe, and the VALU only converts.  16-column tiles, 8 waves interleaving over K.
// XROWS = activation rows staged: 4, 8 or 16.
// ---------------------------------------------------------------------------------------
template <int XROWS, int NW, int BW, int CB, int DEPTH = 2>
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
        // bytes as fp16 subnormals: (w + 128) 2^-24, two integer operations fewer per register than
        // building normal numbers and subtracting their bias; the 128 leaves with the zero point
        const uint32_t t0 = wv.x ^ 0x80808080u, t1 = wv.y ^ 0x80808080u;
        const u32x4 wb = {__builtin_amdgcn_perm(0u, t0, 0x04010400u), __builtin_amdgcn_perm(0u, t0, 0x04030402u),
                          __builtin_amdgcn_perm(0u, t1, 0x04010400u), __builtin_amdgcn_perm(0u, t1, 0x04030402u)};
        acc[b] = __builtin_amdgcn_mfma_f32_16x16x32_f16(as_half8(xv), as_half8(wb), acc[b], 0, 0, 0);
      }
      xacc = __builtin_amdgcn_mfma_f32_16x16x32_f16(as_half8(xv), ones8, xacc, 0, 0, 0);
    }
    wave_lds_sync();
  };

  // DEPTH bands of a wave in flight or in use: the loads of band t + DEPTH - 1 go out before band t is
  // multiplied
  u32x4 wbuf[DEPTH][WI], xbuf[DEPTH][XI];
  const int nsteps = (nbands + nw - 1) / nw;
  int step = stagger_start(nsteps, 0);
  auto next_band = [&]() {
    const int band = step * nw + wave;
    step = step + 1 == nsteps ? 0 : step + 1;
    return band;
  };
#pragma unroll
  for (int d = 0; d < DEPTH - 1; ++d)
    if (d < nsteps) load_band(next_band(), wbuf[d], xbuf[d]);
  for (int it = 0; it < nsteps; it += DEPTH) {
#pragma unroll
    for (int d = 0; d < DEPTH; ++d) {
      if (it + d >= nsteps) break;
      if (it + d + DEPTH - 1 < nsteps)
        load_band(next_band(), wbuf[(d + DEPTH - 1) % DEPTH], xbuf[(d + DEPTH - 1) % DEPTH]);
      multiply(wbuf[d], xbuf[d]);
    }
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
      float v = sum * 16777216.f - (zero_point + 128.f) * xs;
      if (not_finite(xs))
        v = elementwise_dot<8>(reinterpret_cast<const uint8_t*>(Wq) + (size_t)n * K, X + (size_t)m * K, K, zero_point);
      Y[(size_t)m * N + n] = static_cast<half_t>(v * (scalar_scale * scale_value(scale_raw)));
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
      float v = sum - zero_point * xs;
      if (not_finite(xs)) v = elementwise_dot<4>(Wq + (size_t)n * rowb, X + (size_t)m * K, K, zero_point);
      Y[(size_t)m * N + n] = static_cast<half_t>(v * (scalar_scale * scale_value(scale_raw)));
    }
  }
}

// ---------------------------------------------------------------------------------------
// Host launchers.  The integer-dot kernel: rows per workgroup 8 when that still yields >= 512
// workgroups, else 4; waves per workgroup as many (<= 4) as the row has 1 KB pieces.
// ---------------------------------------------------------------------------------------
static int i8_waves(int K) {
  const int pieces = (K / 16 + 63) / 64;
  return pieces >= 4 ? 4 : (pieces >= 2 ? 2 : 1);
}

// One activation row.  A wave's chunk is 1 KB of each weight row (2048 k of int4 in four units a
// lane, 1024 k of int8 in two); a workgroup has as many waves as K has chunks, up to 8, rounded up
// to a power of two, and takes four weight rows -- two when the whole matrix is 8 MiB or less,
// where four rows leave too few workgroups.  Measured, us per call, previous kernels -> these
// (N x K): int4 8192 x 8192 10.6 -> 8.7, 4096 x 4096 5.7 -> 4.1, 28672 x 4096 16.2 -> 11.6,
// 4096 x 14336 10.1 -> 8.1, 16384 x 16384 27.9 -> 24.5; int8 8192 x 8192 13.3 -> 12.1,
// 4096 x 4096 5.7 -> 5.25, 28672 x 4096 20.8 -> 18.8, 4096 x 14336 12.6 -> 11.4, 16384 x 16384
// 41.9 -> 40.6.  int8 with four units a lane (2 KB of a row per wave): 8192 x 8192 13.0.
// Loads through buffer descriptors that end with the row (no predicate, so no branch around each of
// the 10 .. 20 small loads of a chunk), six alternating runs each: int4 8192 x 8192 8.57 -> 8.15, 4096
// x 4096 4.08 -> 3.98; int8 12.25 -> 12.17, 5.30 -> 5.21.
// Two activation rows of int4 (MR = 2) against the row-load MFMA kernel: 8192 x 8192 11.4 -> 10.6,
// 4096 x 4096 5.7 -> 5.0, 4096 x 14336 11.6 -> 10.7, 28672 x 4096 level; the second row costs 2 us at
// 8192 x 8192 because its x traffic (64 MiB from L2) is twice the weights'; eight weight rows a
// workgroup to halve it lose more in occupancy (11.9).  int8 keeps its row-load kernel for two rows.
template <int BITS, int MR>
static void launch_wq_m1(const W8A16Args& a, hipStream_t s) {
  auto* Wq = static_cast<const uint8_t*>(a.Wq);
  auto* X = static_cast<const half_t*>(a.x);
  auto* sc = static_cast<const half_t*>(a.scale);
  auto* Y = static_cast<half_t*>(a.y);
  constexpr int UD = BITS == 4 ? 4 : 2;
  const int chunks = (a.K + 512 * UD - 1) / (512 * UD);
  const bool small = (size_t)a.N * a.K * BITS / 8 <= (8u << 20);
#define FG_WQ_M1(RN, NWV)                                                                         \
  hipLaunchKernelGGL((wq_m1_kernel<BITS, RN, NWV, UD, MR>), dim3(a.N / RN), dim3(64 * NWV), 0, s, Wq, \
                     X, sc, a.scalar_scale, a.zero_point, Y, a.N, a.K)
#define FG_WQ_M1_ROWS(NWV) \
  if (small) FG_WQ_M1(2, NWV); else FG_WQ_M1(4, NWV)
  if (chunks > 4) { FG_WQ_M1_ROWS(8); }
  else if (chunks > 2) { FG_WQ_M1_ROWS(4); }
  else if (chunks > 1) { FG_WQ_M1_ROWS(2); }
  else { FG_WQ_M1_ROWS(1); }
#undef FG_WQ_M1_ROWS
#undef FG_WQ_M1
}

// An earlier kernel with lanes along K (16 weight bytes a lane) against the row-load kernel on 256-byte
// bands, us per call: K = N = 8192 M=1 12.6 / 14.3, M=2 15.1 / 14.2, M=4 21.1 / 14.9, M=8 32.9 / 17.2.
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
  //  * one workgroup on every CU (N = 8192): long rows or 12..16 activation rows only (15..16 before three bands were in flight), K=16384 M=8
  //    25.4 / 27.3, K=28672 M=14 47.8 / 55.4, K=4096 M=16 10.5 / 11.1, against K=8192 M=8 16.9 /
  //    14.9, K=28672 M=4 40.0 / 38.7, K=2048 M=16 7.7 / 7.1;
  //  * 13..16 rows from 160 tiles on: N=5120 K=11008 M=16 19.5 / 23.0, N=14336 K=14336 44.5 / 55.1.
  const bool aligned = a.N % 32 == 0;
  const bool two_per_cu = aligned && ((t32 >= 448 && t32 <= 512) || (t32 >= 512 && t32 % 512 == 0)) &&
                          (a.K != 8192 || a.M > 8);
  const bool one_per_cu = aligned && t32 == 256 &&
                          ((a.M >= 12 && a.K >= 4096) || (a.K >= 16384 && (a.M >= 5 || a.K < 24576)));
  const bool many_rows = aligned && a.M >= 13 && t32 >= 160 && t32 != 256;
  const bool wide = two_per_cu || one_per_cu || many_rows;
  // 16-column tiles take 128-byte bands (smaller strips, more steps in flight): M=8, 128- / 256-byte
  // bands: K = N = 8192 14.5 / 15.7, K = N = 4096 7.0 / 7.3, K=4096 N=14336 14.6 / 16.1, K=11008
  // N=5120 17.7 / 19.3 -- except long rows of narrow outputs, K=14336 N=4096 M=4 14.8 / 13.9.
  const bool bw256 = a.N <= 4096 && a.K >= 14336;
#define FG_W8A16_R(XR, BW, CB)                                                                    \
  hipLaunchKernelGGL((w8a16_r_kernel<XR, 8, BW, CB>), dim3(a.N / (16 * CB)), dim3(512), 0, s, Wq, \
                     X, sc, a.scalar_scale, a.zero_point, Y, a.M, a.N, a.K)
  // Two rows run the lanes-over-x kernel on two rows -- except where the 16-column tiles of the row-load
  // kernel fill the CUs evenly (us, two-row kernel / row-load kernel: N=4096 K=4096 6.0 / 7.1, K=14336
  // 13.2 / 14.7; N=11008 K=4096 10.8 / 12.5; N=12288 K=3072 9.2 / 10.9, K=8192 20.0 / 20.8; N=28672 K=4096
  // 22.0 / 24.0; N=2048 K=8192 6.1 / 6.8; N=1024 K=4096 3.7 / 4.5; but N=8192 K=8192 14.6 / 13.5, K=11008
  // 18.4 / 17.0, K=4096 8.6 / 8.4, but K=2048 5.6 / 6.2; N=16384 K=8192 25.5 / 23.5; level at N=13824
  // K=5120 and N=14336 K=4096).  Three and four rows only against narrow outputs, which leave the row-load kernel on
  // half the CUs or fewer (M=4: N=1024 K=4096 4.5 / 5.3, N=2048 K=2048 4.3 / 5.6, K=8192 7.8 / 8.1;
  // N=4096 K=4096 7.6 / 6.6 and N=8192 K=8192 23.2 / 13.7 the other way).
  const bool even_tiles = a.N % 8192 == 0 && a.K >= 4096;
  if (a.M == 1) {
    launch_wq_m1<8, 1>(a, s);
  } else if (a.M == 2 && !even_tiles) {
    launch_wq_m1<8, 2>(a, s);
  } else if (a.M == 3 && a.N <= 2048) {
    launch_wq_m1<8, 3>(a, s);
  } else if (a.M == 4 && a.N <= 2048) {
    launch_wq_m1<8, 4>(a, s);
  } else if (a.M <= 4) {  // 2 rows take the 4-row strip too: K=14336 N=4096 M=2 13.1 us
    if (wide) FG_W8A16_R(4, 128, 2);
    else if (bw256) FG_W8A16_R(4, 256, 1);
    else FG_W8A16_R(4, 128, 1);
  } else if (a.M <= 8) {
    if (wide) FG_W8A16_R(8, 128, 2);
    else if (bw256) FG_W8A16_R(8, 256, 1);
    else FG_W8A16_R(8, 128, 1);
  } else if (a.M <= 16) {
    // 16-row activation strip on 128-byte bands only (the 256-byte form would need 100 KB of LDS).
    // 32-column tiles with three bands of a wave in flight instead of two (us): N = K = 8192 M=16 17.3 /
    // 18.2, K=16384 25.9 / 27.5; N=16384 K=8192 31.3 / 32.7; N=14336 K=4096 17.2 / 18.1 -- with eight rows
    // level or behind (N = K = 8192 15.3 / 14.7 against 16-column tiles, N=14336 K=4096 15.2 / 13.6), and
    // 16-column tiles lose with any deeper pipeline (M=16 19.9 with three, 21.4 with four).  With three in
    // flight the one-a-CU form at N = 8192 pays from 12 rows on (K=4096 M=12 9.8 / 10.6, K=8192 M=13 17.0 /
    // 17.5; M=9 level).
    if (wide)
      hipLaunchKernelGGL((w8a16_r_kernel<16, 8, 128, 2, 3>), dim3(a.N / 32), dim3(512), 0, s, Wq, X, sc,
                         a.scalar_scale, a.zero_point, Y, a.M, a.N, a.K);
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
    launch_wq_m1<4, 1>(a, s);
  } else if (a.M == 2) {
    launch_wq_m1<4, 2>(a, s);
  } else if (a.N <= 2048) {
    // narrow outputs leave the 16-column tiles of the row-load kernel on half the CUs or fewer (M=4, us,
    // lanes-over-x / row-load: N=1024 K=4096 4.6 / 5.3, K=8192 5.3 / 7.4; N=2048 K=2048 4.3 / 5.0, K=8192
    // 7.5 / 7.7; N=3072 K=3072 5.7 / 5.3 and N=4096 K=4096 6.6 / 5.7 the other way)
    if (a.M == 3) launch_wq_m1<4, 3>(a, s);
    else launch_wq_m1<4, 4>(a, s);
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
