// Host-side contract between the C ABI (fg_capi.hip) and the kernel translation units.
// Each kernel file exports one launcher that maps a validated plan onto a template
// instantiation; the launchers return false when the plan names a combination that was not
// instantiated.
#pragma once
#include <hip/hip_runtime.h>
#include <stddef.h>
#include <stdint.h>

#include "fg_flags.h"
#include "fg_plan.h"

namespace fg {

struct GemmArgs {
  const void* A;  // fp16 [M,K]
  const void* W;  // fp16 [N,K] or [K,N]
  void* C;        // fp16 [M,N]
  float* ws;      // fp32 [S,M,N] partials when plan.splitk > 1
  int* counters;  // per-tile arrival counters (fused split-K) or null (second-pass kernel)
  int M, N, K;
  int accumulate;  // flag word: bit 0 C += A*W; bit 1 plan.stagger (start step = workgroup id %
                   // steps); bit 4 add bias; bits 5-7 activation (FG_ACT_*)
  const void* bias;  // fp16 [N] when bit 4 is set
  int ldw;           // elements between consecutive rows of W; [K,N] kernels only (else N or K)
  int cus;           // compute units of the device ([K,N] kernels spread column bands over them)
  int xccs = 8;      // XCDs (L2 domains) the device dispatches workgroups to round-robin
};

// Geometry of the [K,N] MFMA kernel's one-dimensional grid.
struct KnGeo {
  int tiles;   // 128-column tiles of the output
  int splitk;  // workgroups per tile
  int cus;     // compute units of the device
  int xccs;    // XCDs of the device
  int tq;      // column tiles per XCD in XCD-local order: ceil(tiles / xccs)
  int log2_tiles, log2_tq, log2_xccs, log2_cus;  // log2 of those that are powers of two, else -1
  int spin_limit;  // polls of the mailbox owner before it recomputes what has not been delivered
  unsigned int nonce;  // host-side enqueue number of the launch (mailbox tags), 0 when unused
};

// Tile sets that exist as instantiations (the planner and the validators share these).

bool launch_nk_dot2(const fg_plan_t& p, const GemmArgs& a, hipStream_t s);
bool launch_nk_mfma4(const fg_plan_t& p, const GemmArgs& a, hipStream_t s);
bool launch_nk_mfma_r(const fg_plan_t& p, const GemmArgs& a, hipStream_t s);
bool launch_kn_dot2(const fg_plan_t& p, const GemmArgs& a, hipStream_t s);
bool launch_kn_mfma(const fg_plan_t& p, const GemmArgs& a, hipStream_t s);

// Second pass of split-K: C[m,n] = fp16( tail( Σ_s ws[s,m,n] (+ C[m,n]) ) ), fixed summation
// order; `flags` and `bias` as in GemmArgs.
void launch_splitk_reduce(const float* ws, void* C, int S, int M, int N, int flags,
                          const void* bias, hipStream_t s);

struct W8A16Args {
  const void* Wq;     // int8 [N,K]
  const void* x;      // fp16 [M,K]
  const void* scale;  // fp16 [N] or null
  float scalar_scale, zero_point;
  void* y;  // fp16 [M,N]
  int M, N, K;
};
bool launch_w8a16(const W8A16Args& a, hipStream_t s);
bool launch_w4a16(const W8A16Args& a, hipStream_t s);  // Wq: two unsigned nibbles per byte, [N,K/2]
bool launch_i8i8_i32(const void* Wq, const void* xq, int32_t* acc, int M, int N, int K,
                     hipStream_t s);
void launch_dequant_i32_f16(const int32_t* acc, const void* scale, float x_scale, void* y, int M,
                            int N, hipStream_t s);

// Split-K workspace: a header of arrival counters (zero between calls), then the partials.
void launch_fill_zero(void* p, size_t bytes, hipStream_t s);

constexpr int kStreamReadBlocks = 2048;
void launch_stream_read(const void* src, size_t bytes, void* sink, hipStream_t s);

}  // namespace fg
