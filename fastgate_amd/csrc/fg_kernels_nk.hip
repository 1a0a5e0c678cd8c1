// fp16 kernels for weights stored [N,K] (each output column's weights contiguous along K).
//
// All kernels stream W exactly once with 16-byte loads.  Rows of W are K*2 bytes apart -- a
// power of two for the usual K -- so every kernel here is built to keep the set of rows it
// has in flight small and to start different workgroups at different K positions; otherwise
// all workgroups sit on the same few HBM channels at the same time.
//
// Replaces the device side of gemv_fp16 / gemm_fp16 (backend/cuda/hk/fastgemv.cuh:503-561,
// 244-311), eed_hgemm_m8n128k64x4_v7_bt (hk/edgemm.cuh:1467-1667) and
// gemm_m8n128k64x4_v8_tr (hk/edgemm_tr.cuh:371-549) of the reference.
#include "fg_device.h"
#include "fg_internal.h"

namespace fg {

// ---------------------------------------------------------------------------------------
// v_dot2 kernel.  Workgroup = blockDim.x/64 waves, tile = RN columns of C x MB rows of A.
// Lane l of wave slot s owns the 16-byte chunks q = (step*slots + s)*64*U + u*64 + l of
// every row of its tile: 1 KB contiguous per row and load instruction.  The matching slice
// of A is re-read per step (an L2 hit, 1/RN of the weight traffic) straight into registers,
// so the main loop has no LDS traffic and no barrier.
// ---------------------------------------------------------------------------------------
template <int MB, int RN, int U, bool STREAM>
__global__ __launch_bounds__(256) void nk_dot2_kernel(const half_t* __restrict__ A,
                                                      const half_t* __restrict__ W,
                                                      half_t* __restrict__ C,
                                                      float* __restrict__ ws, int* counters, int M,
                                                      int N, int K, int flags, const void* bias) {
  __shared__ float red[16][RN * MB];
  const int lane = threadIdx.x & 63;
  const int wave = threadIdx.x >> 6;
  const int nw = blockDim.x >> 6;
  const int n0 = blockIdx.x * RN;
  const int m0 = blockIdx.y * MB;
  const int slots = nw * gridDim.z;
  const int slot = blockIdx.z * nw + wave;
  const int nq = K >> 3;

  float acc[RN][MB];
#pragma unroll
  for (int r = 0; r < RN; ++r)
#pragma unroll
    for (int m = 0; m < MB; ++m) acc[r][m] = 0.f;

  const half_t* Wt = W + (size_t)n0 * K;
  const half_t* At = A + (size_t)m0 * K;
  const u32x4 zero = {0u, 0u, 0u, 0u};

  const int nsteps = (nq + slots * (64 * U) - 1) / (slots * (64 * U));
  int step = stagger_start(nsteps, flags);
  for (int it = 0; it < nsteps; ++it) {
    const int q0 = (step * slots + slot) * (64 * U);
    step = step + 1 == nsteps ? 0 : step + 1;
    u32x4 wr[U][RN];
    u32x4 xr[U][MB];
#pragma unroll
    for (int u = 0; u < U; ++u) {
      const int q = q0 + u * 64 + lane;
      const bool ok = q < nq;
#pragma unroll
      for (int r = 0; r < RN; ++r)
        wr[u][r] = ok ? load16<STREAM>(Wt + (size_t)r * K + (size_t)q * 8) : zero;
#pragma unroll
      for (int m = 0; m < MB; ++m)
        xr[u][m] = (ok && (m0 + m) < M) ? load16<false>(At + (size_t)m * K + (size_t)q * 8) : zero;
    }
#pragma unroll
    for (int u = 0; u < U; ++u)
#pragma unroll
      for (int r = 0; r < RN; ++r)
#pragma unroll
        for (int m = 0; m < MB; ++m) acc[r][m] = dot8(wr[u][r], xr[u][m], acc[r][m]);
  }

  // 64 lanes -> 4 row sums per wave (DPP), then waves x 4 partials through LDS.
#pragma unroll
  for (int r = 0; r < RN; ++r)
#pragma unroll
    for (int m = 0; m < MB; ++m) {
      const float v = row16_allreduce(acc[r][m]);
      if ((lane & 15) == 0) red[wave * 4 + (lane >> 4)][r * MB + m] = v;
    }
  __syncthreads();
  for (int t = threadIdx.x; t < RN * MB; t += blockDim.x) {
    const int m = t / RN, r = t % RN;
    const float sum = lds_sum<16>(&red[0][r * MB + m], RN * MB, nw * 4);
    const int mg = m0 + m, n = n0 + r;
    if (mg < M) {
      if (gridDim.z == 1) {
        half_t* c = C + (size_t)mg * N + n;
        *c = finish_value(sum, c, n, bias, flags);
      } else {
        publish_partial(ws, counters, C, M, N, mg, n, sum, flags, bias);
      }
    }
  }
  finish_splitk<MB, RN>(ws, counters, C, M, N, m0, n0, flags, bias);
}

// ---------------------------------------------------------------------------------------
// MFMA 4x4x4 kernel.  v_mfma_f32_4x4x4_16B_f16 multiplies 16 independent 4x4x4 blocks; here
// block b = lane/4 owns the 8 k positions 128*chunk + 8b..8b+7 (two MFMAs of 4 k each) and its
// four lanes j = lane%4 own four neighbouring weight rows.  One 16-byte load instruction of a
// wave therefore reads 4 weight rows x 256 contiguous bytes -- the same row-friendly pattern as
// the v_dot2 kernel with a 4-row tile, instead of the 16 rows x 64 bytes the 16x16x32 operand
// layout forces -- and one instruction per 4 rows of A replaces 4*4 v_dot2.
// acc[g][i] at lane (b,j) is the partial C[m0+4g+i][n+j] over the k positions of block b; the
// 16 blocks are summed once per output.
// ---------------------------------------------------------------------------------------
typedef _Float16 half4_t __attribute__((ext_vector_type(4)));

__device__ __forceinline__ half4_t lo4(u32x4 v) { return __builtin_bit_cast(half4_t, u32x2{v.x, v.y}); }
__device__ __forceinline__ half4_t hi4(u32x4 v) { return __builtin_bit_cast(half4_t, u32x2{v.z, v.w}); }

// The waves of a workgroup interleave over K, every wave covers all 4*R4 columns of the tile
// and re-reads its slice of A from L2 (4 rows x 256 B per instruction, which is what makes it
// lose to the row-load kernel below once M exceeds 4).
template <int MG, int R4, int U, bool STREAM>
__global__ __launch_bounds__(256) void nk_mfma4_kernel(const half_t* __restrict__ A,
                                                       const half_t* __restrict__ W,
                                                       half_t* __restrict__ C,
                                                       float* __restrict__ ws, int* counters, int M,
                                                       int N, int K, int flags, const void* bias) {
  __shared__ float red[16][R4 * MG * 16];
  const int lane = threadIdx.x & 63;
  const int wave = threadIdx.x >> 6;
  const int nw = blockDim.x >> 6;
  const int j = lane & 3, b = lane >> 2;
  const int n0 = blockIdx.x * (4 * R4);
  const int m0 = blockIdx.y * (4 * MG);
  const int slots = nw * gridDim.z;
  const int slot = blockIdx.z * nw + wave;
  const int nchunks = K >> 7;

  float4_t acc[R4][MG];
#pragma unroll
  for (int r = 0; r < R4; ++r)
#pragma unroll
    for (int g = 0; g < MG; ++g) acc[r][g] = float4_t{0.f, 0.f, 0.f, 0.f};

  const half_t* Wp = W + (size_t)(n0 + j) * K + b * 8;
  const half_t* Ap = A + (size_t)(m0 + j) * K + b * 8;
  const u32x4 zero = {0u, 0u, 0u, 0u};

  const int nsteps = (nchunks + slots * U - 1) / (slots * U);
  int step = stagger_start(nsteps, flags);
  for (int it = 0; it < nsteps; ++it) {
    const int c0 = (step * slots + slot) * U;
    step = step + 1 == nsteps ? 0 : step + 1;
    u32x4 w[U][R4];
    u32x4 a[U][MG];
#pragma unroll
    for (int u = 0; u < U; ++u) {
      const int c = c0 + u;
      const bool ok = c < nchunks;
#pragma unroll
      for (int r = 0; r < R4; ++r)
        w[u][r] = ok ? load16<STREAM>(Wp + (size_t)(4 * r) * K + (size_t)c * 128) : zero;
#pragma unroll
      for (int g = 0; g < MG; ++g)
        a[u][g] = (ok && (m0 + 4 * g + j) < M)
                      ? load16<false>(Ap + (size_t)(4 * g) * K + (size_t)c * 128)
                      : zero;
    }
#pragma unroll
    for (int u = 0; u < U; ++u)
#pragma unroll
      for (int r = 0; r < R4; ++r)
#pragma unroll
        for (int g = 0; g < MG; ++g) {
          acc[r][g] = __builtin_amdgcn_mfma_f32_4x4x4f16(lo4(a[u][g]), lo4(w[u][r]), acc[r][g], 0, 0, 0);
          acc[r][g] = __builtin_amdgcn_mfma_f32_4x4x4f16(hi4(a[u][g]), hi4(w[u][r]), acc[r][g], 0, 0, 0);
        }
  }

  // Sum the 16 blocks: 4 per DPP row with row_ror:4 / row_ror:8, the 4 rows and the waves in LDS.
#pragma unroll
  for (int r = 0; r < R4; ++r)
#pragma unroll
    for (int g = 0; g < MG; ++g)
#pragma unroll
      for (int i = 0; i < 4; ++i) {
        float v = acc[r][g][i];
        v += dpp_f32<0x124>(v);
        v += dpp_f32<0x128>(v);
        if ((lane & 12) == 0) red[wave * 4 + (lane >> 4)][((r * MG + g) * 4 + i) * 4 + j] = v;
      }
  __syncthreads();
  for (int e = threadIdx.x; e < R4 * MG * 16; e += blockDim.x) {
    // e = ((g*4 + i) * R4 + r) * 4 + jj : consecutive threads write consecutive columns
    const int jj = e & 3, r = (e >> 2) % R4, gi = (e >> 2) / R4, g = gi >> 2, i = gi & 3;
    const float sum = lds_sum<16>(&red[0][((r * MG + g) * 4 + i) * 4 + jj], R4 * MG * 16, nw * 4);
    const int mg = m0 + 4 * g + i, n = n0 + 4 * r + jj;
    if (mg < M) {
      if (gridDim.z == 1) {
        half_t* c = C + (size_t)mg * N + n;
        *c = finish_value(sum, c, n, bias, flags);
      } else {
        publish_partial(ws, counters, C, M, N, mg, n, sum, flags, bias);
      }
    }
  }
  finish_splitk<4 * MG, 4 * R4>(ws, counters, C, M, N, m0, n0, flags, bias);
}

// ---------------------------------------------------------------------------------------
// MFMA 16x16x32 kernel with row-friendly loads for BOTH operands, no split-K needed.
// What makes re-reading A expensive is the shape of the loads, not their volume: read as
// 16 rows x 64 B (operand order) or 4 rows x 256 B, a 16-row A costs as much as the weights;
// read as whole contiguous row pieces it costs under 10 % (a load-only probe with 16 weight rows
// and 16 activation rows per step: 24.5 us against 22.7 us without the activation rows, at
// K = N = 8192).  So here a wave loads, per step, a BAND-byte band (BAND/2 k) of the tile's weight
// rows and of the A rows -- 64 lanes x 16 B cover 1024/BAND rows per instruction -- parks both in
// wave-private LDS strips (rows padded by 16 B, which spreads both the row-order stores and the
// operand-order loads over all banks; SQ_LDS_BANK_CONFLICT still counts about 400 cycles per wave
// at K = N = 8192, M = 16 -- 819 200 per dispatch, under 1 % of a wave's run time -- so the padding
// is not exact, and not worth more LDS) and reads them
// back in operand order for BAND/64 MFMAs per 16-column block.  The tile is only 16 (or, with
// CB = 2, 32) columns wide, so N/16 workgroups fill the chip without split-K and there is no second
// pass; the waves of a workgroup interleave over the bands of K and meet in LDS once at the end.
// Occupancy decides the rest: 256-byte bands need 35 KB of LDS and about 100 VGPRs per four
// waves, so two 8-wave workgroups fit a CU (16 waves per CU; M = 16 at K = N = 8192: 24.6 us
// against 26.0 us with four waves on 512-byte bands).
// ---------------------------------------------------------------------------------------
template <int AROWS, int BAND, bool FULL, int NW, int CB, bool RAGGED = false>
__global__ __launch_bounds__(64 * NW) void nk_mfma_r_kernel(const half_t* __restrict__ A,
                                                        const half_t* __restrict__ W,
                                                        half_t* __restrict__ C,
                                                        float* __restrict__ ws, int* counters, int M,
                                                        int N, int K, int flags, const void* bias) {
  // AROWS: rows of A staged per step (8 covers M <= 8, 16 covers M <= 16, 32 two MFMA row blocks per
  // workgroup so that 17..32 rows still read the weights once).  BAND: bytes of K per
  // row and step (512, 256 or 128).  FULL: K is a multiple of the band and the bands divide evenly
  // over the waves -- no masks needed.  RAGGED: the tile is N / gridDim.x columns wide, fewer than
  // the 16 * CB the column blocks hold; the spare rows are never loaded and never stored.
  constexpr int LPR = BAND / 16;       // lanes per row piece
  constexpr int RPI = 64 / LPR;        // rows per load instruction
  constexpr int WI = 16 * CB / RPI;    // load instructions per step for the weights (CB blocks of 16 rows)
  constexpr int AI = AROWS / RPI;      // ... for the activations
  constexpr int UNITS = BAND / 64;     // 32-wide MFMA K units per band
  constexpr int BK = BAND / 2;         // K positions per band
  constexpr int RS = BAND + 16;        // LDS bytes per staged row
  constexpr int WSTRIP = 16 * CB * RS;  // weights of one wave
  constexpr int ASTRIP = AROWS * RS;   // activations of one wave (rows beyond AROWS re-read row j%8)
  constexpr int MBLK = AROWS == 32 ? 2 : 1;  // 16-row MFMA blocks per workgroup
  constexpr int WAVE_LDS = WSTRIP + ASTRIP;
  static_assert(WAVE_LDS >= CB * MBLK * 256 * (int)sizeof(float), "reduction scratch fits");
  __shared__ __attribute__((aligned(16))) unsigned char smem[NW * WAVE_LDS];  // NW = most waves
  const int lane = threadIdx.x & 63;
  const int wave = threadIdx.x >> 6;
  const int nw = blockDim.x >> 6;
  const int j = lane & 15, g = lane >> 4;       // operand order: row j, 8 k at 8g within a unit
  const int h = lane / LPR, c = lane % LPR;     // load order: row RPI*i + h, 16-byte piece c
  const int tw = RAGGED ? N / (int)gridDim.x : 16 * CB;  // columns of this tile
  const int n0 = blockIdx.x * tw;
  const int m0 = blockIdx.y * (16 * MBLK);
  const int slots = nw * gridDim.z;
  const int slot = blockIdx.z * nw + wave;
  const int nbands = (K + BK - 1) / BK;  // K % 128 == 0: the last band may be partial
  unsigned char* wstrip = smem + wave * WAVE_LDS;
  unsigned char* astrip = wstrip + WSTRIP;
  const u32x4 zero = {0u, 0u, 0u, 0u};

  const half_t* Wp = W + (size_t)(n0 + h) * K + c * 8;
  const half_t* Ap = A + (size_t)(m0 + h) * K + c * 8;
  bool arow[AI];
#pragma unroll
  for (int i = 0; i < AI; ++i) arow[i] = (m0 + RPI * i + h) < M;
  // LDS byte offsets: where this lane parks its pieces, and where it reads its operands.  With
  // an 8-row A strip the MFMA rows 8..15 re-read rows 0..7; their results are never stored.
  const int st_off = h * RS + c * 16;
  const int ldw_off = j * RS + g * 16;
  const int lda_off = (AROWS >= 16 ? j : (j & 7)) * RS + g * 16;

  auto load_band = [&](int band, u32x4(&w)[WI], u32x4(&a)[AI]) {
    const bool ok = FULL || (band < nbands && (band * BK + c * 8) < K);
#pragma unroll
    for (int i = 0; i < WI; ++i)
      w[i] = (ok && (!RAGGED || RPI * i + h < tw))
                 ? load16<true>(Wp + (size_t)(RPI * i) * K + (size_t)band * BK)
                 : zero;
#pragma unroll
    for (int i = 0; i < AI; ++i)
      a[i] = (ok && arow[i]) ? load16<false>(Ap + (size_t)(RPI * i) * K + (size_t)band * BK) : zero;
  };
  float4_t acc[CB][MBLK];
#pragma unroll
  for (int b = 0; b < CB; ++b)
#pragma unroll
    for (int mb = 0; mb < MBLK; ++mb) acc[b][mb] = float4_t{0.f, 0.f, 0.f, 0.f};
  auto multiply = [&](const u32x4(&w)[WI], const u32x4(&a)[AI]) {
#pragma unroll
    for (int i = 0; i < WI; ++i) *reinterpret_cast<u32x4*>(wstrip + st_off + RPI * i * RS) = w[i];
#pragma unroll
    for (int i = 0; i < AI; ++i) *reinterpret_cast<u32x4*>(astrip + st_off + RPI * i * RS) = a[i];
    wave_lds_sync();
#pragma unroll
    for (int u = 0; u < UNITS; ++u) {
      u32x4 av[MBLK];
#pragma unroll
      for (int mb = 0; mb < MBLK; ++mb)
        av[mb] = *reinterpret_cast<const u32x4*>(astrip + mb * 16 * RS + lda_off + u * 64);
#pragma unroll
      for (int b = 0; b < CB; ++b) {
        const u32x4 bv = *reinterpret_cast<const u32x4*>(wstrip + b * 16 * RS + ldw_off + u * 64);
#pragma unroll
        for (int mb = 0; mb < MBLK; ++mb)
          acc[b][mb] = __builtin_amdgcn_mfma_f32_16x16x32_f16(as_half8(av[mb]), as_half8(bv), acc[b][mb], 0, 0, 0);
      }
    }
    wave_lds_sync();
  };

  // Two register sets, alternating: the next band is in flight while this one is multiplied.
  u32x4 w0[WI], w1[WI], a0[AI], a1[AI];
  const int nsteps = (nbands + slots - 1) / slots;
  int step = stagger_start(nsteps, flags);
  auto next_band = [&]() {
    const int band = step * slots + slot;
    step = step + 1 == nsteps ? 0 : step + 1;
    return band;
  };
  load_band(next_band(), w0, a0);
  for (int it = 0; it < nsteps; it += 2) {
    if (it + 1 < nsteps) load_band(next_band(), w1, a1);
    multiply(w0, a0);
    if (it + 1 >= nsteps) break;
    if (it + 2 < nsteps) load_band(next_band(), w0, a0);
    multiply(w1, a1);
  }

  // acc[b][mb][r] = D[m = 16 mb + 4g + r][column 16b + j]; the waves' partials meet in LDS
  constexpr int TN = 16 * CB;
  constexpr int TM = 16 * MBLK;
  __syncthreads();
  float(*red)[TM * TN] = reinterpret_cast<float(*)[TM * TN]>(smem);
#pragma unroll
  for (int b = 0; b < CB; ++b)
#pragma unroll
    for (int mb = 0; mb < MBLK; ++mb)
#pragma unroll
      for (int r = 0; r < 4; ++r) red[wave][(16 * mb + 4 * g + r) * TN + 16 * b + j] = acc[b][mb][r];
  __syncthreads();
  for (int e = threadIdx.x; e < TM * TN; e += blockDim.x) {
    const float sum = lds_sum<NW>(&red[0][e], TM * TN, nw);
    const int mg = m0 + e / TN, n = n0 + e % TN;
    if (e / TN < AROWS && mg < M && (!RAGGED || e % TN < tw)) {
      if (gridDim.z == 1) {
        half_t* cp = C + (size_t)mg * N + n;
        *cp = finish_value(sum, cp, n, bias, flags);
      } else {
        publish_partial(ws, counters, C, M, N, mg, n, sum, flags, bias);
      }
    }
  }
  finish_splitk<TM, TN>(ws, counters, C, M, N, m0, n0, flags, bias);
}

// ---------------------------------------------------------------------------------------
// Host launchers
// ---------------------------------------------------------------------------------------
#define FG_LAUNCH(KERNEL, p, a, s)                                                           \
  hipLaunchKernelGGL(KERNEL, dim3((p).grid_x, (p).grid_y, (p).grid_z), dim3((p).block), 0, s, \
                     static_cast<const half_t*>((a).A), static_cast<const half_t*>((a).W),    \
                     static_cast<half_t*>((a).C), (a).ws, (a).counters, (a).M, (a).N, (a).K,  \
                     (a).accumulate, (a).bias)

template <int MB, int RN, int U>
static void nk_dot2_go(const fg_plan_t& p, const GemmArgs& a, hipStream_t s) {
  if (p.stream_w) FG_LAUNCH((nk_dot2_kernel<MB, RN, U, true>), p, a, s);
  else FG_LAUNCH((nk_dot2_kernel<MB, RN, U, false>), p, a, s);
}

template <int MB, int RN>
static bool nk_dot2_u(const fg_plan_t& p, const GemmArgs& a, hipStream_t s) {
  if constexpr (MB * RN <= 64) {
    switch (p.unroll) {
      case 1: nk_dot2_go<MB, RN, 1>(p, a, s); return true;
      case 2:
        if constexpr (RN * 2 <= 32) { nk_dot2_go<MB, RN, 2>(p, a, s); return true; }
        return false;
      case 4:
        if constexpr (RN * 4 <= 32) { nk_dot2_go<MB, RN, 4>(p, a, s); return true; }
        return false;
      default: return false;
    }
  } else {
    return false;
  }
}

template <int MB>
static bool nk_dot2_rn(const fg_plan_t& p, const GemmArgs& a, hipStream_t s) {
  switch (p.tile_n) {
    case 4: return nk_dot2_u<MB, 4>(p, a, s);
    case 8: return nk_dot2_u<MB, 8>(p, a, s);
    case 16: return nk_dot2_u<MB, 16>(p, a, s);
    default: return false;
  }
}

bool launch_nk_dot2(const fg_plan_t& p, const GemmArgs& a, hipStream_t s) {
  switch (p.m_block) {
    case 1: return nk_dot2_rn<1>(p, a, s);
    case 2: return nk_dot2_rn<2>(p, a, s);
    case 4: return nk_dot2_rn<4>(p, a, s);
    case 8: return nk_dot2_rn<8>(p, a, s);
    default: return false;
  }
}

template <int MG, int R4, int U>
static void nk_mfma4_go(const fg_plan_t& p, const GemmArgs& a, hipStream_t s) {
  if (p.stream_w) FG_LAUNCH((nk_mfma4_kernel<MG, R4, U, true>), p, a, s);
  else FG_LAUNCH((nk_mfma4_kernel<MG, R4, U, false>), p, a, s);
}

template <int MG, int R4>
static bool nk_mfma4_u(const fg_plan_t& p, const GemmArgs& a, hipStream_t s) {
  if constexpr (MG * R4 <= 16) {
    switch (p.unroll) {
      case 1: nk_mfma4_go<MG, R4, 1>(p, a, s); return true;
      case 2:
        if constexpr ((MG + R4) * 2 <= 24) { nk_mfma4_go<MG, R4, 2>(p, a, s); return true; }
        return false;
      case 4:
        if constexpr ((MG + R4) * 4 <= 24) { nk_mfma4_go<MG, R4, 4>(p, a, s); return true; }
        return false;
      default: return false;
    }
  } else {
    return false;
  }
}

template <int MG>
static bool nk_mfma4_r(const fg_plan_t& p, const GemmArgs& a, hipStream_t s) {
  switch (p.tile_n) {
    case 4: return nk_mfma4_u<MG, 1>(p, a, s);
    case 8: return nk_mfma4_u<MG, 2>(p, a, s);
    case 16: return nk_mfma4_u<MG, 4>(p, a, s);
    case 32: return nk_mfma4_u<MG, 8>(p, a, s);
    default: return false;
  }
}

bool launch_nk_mfma4(const fg_plan_t& p, const GemmArgs& a, hipStream_t s) {
  switch (p.m_block) {
    case 4: return nk_mfma4_r<1>(p, a, s);
    case 8: return nk_mfma4_r<2>(p, a, s);
    case 12: return nk_mfma4_r<3>(p, a, s);
    case 16: return nk_mfma4_r<4>(p, a, s);
    default: return false;
  }
}

// Transposing variant: unroll = rows per tile (8 or 16), tile_n = rows * T with T in {2,4,8}.
template <int AROWS, int BAND, int CB>
static void nk_mfma_r_go(const fg_plan_t& p, const GemmArgs& a, hipStream_t s) {
  const int slots = p.waves * p.grid_z;
  const int bk = BAND / 2;
  const bool full = a.K % bk == 0 && (a.K / bk) % slots == 0;
  if constexpr (BAND <= 256) {
    if (p.waves == 8) {
      if (full) FG_LAUNCH((nk_mfma_r_kernel<AROWS, BAND, true, 8, CB>), p, a, s);
      else FG_LAUNCH((nk_mfma_r_kernel<AROWS, BAND, false, 8, CB>), p, a, s);
      return;
    }
  }
  if (full) FG_LAUNCH((nk_mfma_r_kernel<AROWS, BAND, true, 4, CB>), p, a, s);
  else FG_LAUNCH((nk_mfma_r_kernel<AROWS, BAND, false, 4, CB>), p, a, s);
}

template <int CB>
static bool nk_mfma_r_cb(const fg_plan_t& p, const GemmArgs& a, hipStream_t s) {
  if (p.m_block == 32) {  // two 16-row blocks per workgroup, 128-byte bands
    if (p.band != 128) return false;
    nk_mfma_r_go<32, 128, CB>(p, a, s);
    return true;
  }
  const bool half_m = a.M <= 8;  // one block row whose A strip needs only 8 rows
  switch (p.band) {
    case 128:
      if (half_m) nk_mfma_r_go<8, 128, CB>(p, a, s);
      else nk_mfma_r_go<16, 128, CB>(p, a, s);
      return true;
    case 256:
      if (half_m) nk_mfma_r_go<8, 256, CB>(p, a, s);
      else nk_mfma_r_go<16, 256, CB>(p, a, s);
      return true;
    case 512:
      if (half_m) nk_mfma_r_go<8, 512, CB>(p, a, s);
      else nk_mfma_r_go<16, 512, CB>(p, a, s);
      return true;
    default:
      return false;
  }
}

// band = bytes of K per row and step: 512 (two rows per load instruction, four waves at most),
// 256 or 128 (four or eight rows per instruction, up to eight waves).  tile_n = 16, 32, 48 or 64
// (one to four 16-column blocks sharing the staged activations; 48 and 64 on 128-byte bands only).
bool launch_nk_mfma_r(const fg_plan_t& p, const GemmArgs& a, hipStream_t s) {
  if (p.m_block != 16 && p.m_block != 32) return false;
  if (p.m_block == 32 && (p.tile_n % 16 != 0 || p.tile_n > 48)) return false;
  if (p.waves > 4 && !(p.waves == 8 && p.band <= 256)) return false;
  if (p.tile_n == 16) return nk_mfma_r_cb<1>(p, a, s);
  if (p.tile_n == 32) return nk_mfma_r_cb<2>(p, a, s);
  if (p.tile_n % 16 != 0) {
    // tile = N / grid.x columns in two or three column blocks, the last one partly filled: lets
    // N / 256 columns go to each of 256 workgroups when that is not a multiple of 16
    if (p.band != 128 || p.waves != 8 || p.grid_z != 1 || p.tile_n < 17 || p.tile_n > 47) return false;
    const bool half_m = a.M <= 8;
    if (p.tile_n < 32) {
      if (half_m) FG_LAUNCH((nk_mfma_r_kernel<8, 128, false, 8, 2, true>), p, a, s);
      else FG_LAUNCH((nk_mfma_r_kernel<16, 128, false, 8, 2, true>), p, a, s);
    } else {
      if (half_m) FG_LAUNCH((nk_mfma_r_kernel<8, 128, false, 8, 3, true>), p, a, s);
      else FG_LAUNCH((nk_mfma_r_kernel<16, 128, false, 8, 3, true>), p, a, s);
    }
    return true;
  }
  if (p.tile_n == 48 || p.tile_n == 64) {  // three or four column blocks: 128-byte bands only
    if (p.band != 128) return false;
    const bool half_m = a.M <= 8;
    if (p.m_block == 32) {
      nk_mfma_r_go<32, 128, 3>(p, a, s);
      return true;
    }
    if (p.tile_n == 48) {
      if (half_m) nk_mfma_r_go<8, 128, 3>(p, a, s);
      else nk_mfma_r_go<16, 128, 3>(p, a, s);
    } else {
      if (half_m) nk_mfma_r_go<8, 128, 4>(p, a, s);
      else nk_mfma_r_go<16, 128, 4>(p, a, s);
    }
    return true;
  }
  return false;
}

}  // namespace fg
