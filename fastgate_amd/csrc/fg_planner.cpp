// Launch planner of libfastgate: which kernel, tile, wave count and split-K a (M, N, K, layout)
// call runs with.  Plain C++ with no HIP dependency, so that it also builds for the host alone
// (the unit tests compile it with -fsanitize=address,undefined and sweep it).
// Replaces the reference's hard-coded split rule (backend/cuda/hk/edgemm.cu:287-305).
#include "fg_plan.h"

#include <algorithm>
#include <cmath>
#include <cstring>

namespace fg {

// Tile sets that exist as kernel instantiations.
bool nk_dot2_supported(int mb, int rn, int u) {
  const bool mb_ok = mb == 1 || mb == 2 || mb == 4 || mb == 8;
  const bool rn_ok = rn == 4 || rn == 8 || rn == 16;
  const bool u_ok = u == 1 || u == 2 || u == 4;
  return mb_ok && rn_ok && u_ok && mb * rn <= 64 && rn * u <= 32;
}

bool nk_mfma4_supported(int m_block, int tile_n, int u) {
  const int mg = m_block / 4, r4 = tile_n / 4;
  if (m_block % 4 || tile_n % 4) return false;
  const bool mg_ok = mg >= 1 && mg <= 4;
  const bool r4_ok = r4 == 1 || r4 == 2 || r4 == 4 || r4 == 8;
  const bool u_ok = u == 1 || u == 2 || u == 4;
  return mg_ok && r4_ok && u_ok && mg * r4 <= 16 && (mg + r4) * u <= 24;
}

bool kn_dot2_supported(int mb, int u) {
  return (mb == 1 || mb == 2 || mb == 4 || mb == 8) && (u == 1 || u == 2 || u == 4) &&
         !(mb == 8 && u == 4);
}
bool kn_mfma_supported(int u) { return u == 1 || u == 2 || u == 4; }

namespace {

// Compute units the rules aim at.  The rules were fitted on 256 (MI355X); the C ABI sets the
// current device's count once.
int kCUs = 256;
int kXccs = 8;


int ceil_div(int a, int b) { return (a + b - 1) / b; }

int pick_waves(int items) { return items >= 4 ? 4 : (items >= 2 ? 2 : 1); }

// Work items = groups of `unroll` K units handed round-robin to waves*S slots.  Returns the
// fraction of slot-steps that carry real work (1.0 = perfectly even).
double balance(int items, int slots) {
  const int per = ceil_div(items, slots);
  return (double)items / ((double)per * slots);
}

// Cross-workgroup split-K factor for the K-interleaved kernels.  A split costs S*M*N*8 bytes
// of fp32 partial traffic and the arrival protocol, so it is only taken when the un-split
// grid leaves CUs idle.
int pick_splitk(int tiles, int waves, int items, int M, int N, int K, int target_wgs) {
  static const int cand[] = {1, 2, 3, 4, 6, 8, 12, 16};
  int best = 1;
  double best_score = -1.0;
  for (int S : cand) {
    if (S > 1 && items / (waves * S) < 2) continue;  // keep >= 2 steps per wave
    const double fill = std::min(1.0, (double)tiles * S / target_wgs);
    const double extra = S > 1 ? (8.0 * S * M * N) / (2.0 * K * N) : 0.0;  // partials vs weights
    double score = balance(items, waves * S) * fill / (1.0 + extra);
    if (S > 1) score *= 0.95;
    if (score > best_score + 1e-9) {
      best_score = score;
      best = S;
    }
  }
  return best;
}

int validate_shape(int M, int N, int K, int w_layout) {
  if (M <= 0 || N <= 0 || K <= 0) return FG_ERR_INVALID_ARG;
  if (w_layout != FG_W_KN && w_layout != FG_W_NK) return FG_ERR_INVALID_ARG;
  if (N % 128 != 0 || K % 128 != 0) return FG_ERR_ALIGN128;
  return FG_OK;
}

// Fills grid/block/workspace from the tile fields; rejects tiles that were not built.
int finish_plan(int M, int N, int K, fg_plan_t* p) {
  const int max_waves =
      ((p->kernel == FG_KERNEL_NK_MFMA_R && (p->band ? p->band : 256 * p->unroll) <= 256) ||
       p->kernel == FG_KERNEL_KN_MFMA ||
       (p->kernel == FG_KERNEL_KN_DOT2 && p->m_block <= 2))
          ? 8
          : 4;
  if (p->splitk < 1 || p->waves < 1 || p->waves > max_waves || (p->waves & (p->waves - 1))) {
    return FG_ERR_INVALID_ARG;
  }
  switch (p->kernel) {
    case FG_KERNEL_NK_DOT2:
      if (!nk_dot2_supported(p->m_block, p->tile_n, p->unroll)) return FG_ERR_UNSUPPORTED;
      break;
    case FG_KERNEL_NK_MFMA4:
      if (!nk_mfma4_supported(p->m_block, p->tile_n, p->unroll)) return FG_ERR_UNSUPPORTED;
      break;
    case FG_KERNEL_NK_MFMA_R:
      // 16, 32, 48, 64, or any width from 17 to 47 that divides N (one partly filled column
      // block; 128-byte bands, 8 waves, no split-K)
      if (p->tile_n != 32 && p->tile_n != 48 && p->tile_n != 64 &&
          !(p->tile_n > 16 && p->tile_n < 48 && N % p->tile_n == 0)) {
        p->tile_n = 16;
      }
      if (p->tile_n % 16 != 0 && (p->splitk != 1 || p->waves != 8)) return FG_ERR_UNSUPPORTED;
      p->m_block = p->m_block == 32 ? 32 : 16;  // 32: two row blocks per workgroup (128-byte bands)
      if (p->band == 0) {
        if (p->unroll != 1 && p->unroll != 2) return FG_ERR_UNSUPPORTED;
        p->band = 256 * p->unroll;
      }
      if (p->band != 128 && p->band != 256 && p->band != 512) return FG_ERR_UNSUPPORTED;
      if ((p->tile_n > 32 || p->tile_n % 16 != 0 || p->m_block == 32) && p->band != 128) return FG_ERR_UNSUPPORTED;
      if (p->m_block == 32 && (p->tile_n % 16 != 0 || p->tile_n > 48)) return FG_ERR_UNSUPPORTED;
      p->unroll = p->band == 512 ? 2 : 1;
      break;
    case FG_KERNEL_KN_DOT2:
      p->tile_n = 128;
      if (!kn_dot2_supported(p->m_block, p->unroll)) return FG_ERR_UNSUPPORTED;
      break;
    case FG_KERNEL_KN_MFMA:
      p->tile_n = 128;
      p->m_block = 16;
      if (!kn_mfma_supported(p->unroll)) return FG_ERR_UNSUPPORTED;
      if (p->waves != 4 && p->waves != 8) return FG_ERR_UNSUPPORTED;  // the wave count is a template argument
      break;
    default:
      return FG_ERR_UNSUPPORTED;
  }
  if (N % p->tile_n != 0) return FG_ERR_UNSUPPORTED;
  if (p->splitk > 65535) return FG_ERR_INVALID_ARG;
  p->grid_x = N / p->tile_n;
  p->grid_y = ceil_div(M, p->m_block);
  if (p->grid_y > 65535) return FG_ERR_INVALID_ARG;  // HIP's limit on grid.y
  p->grid_z = p->splitk;
  p->block = 64 * p->waves;
  if (p->fused < 0 || p->fused > 4) return FG_ERR_INVALID_ARG;
  if (p->splitk > 1 && p->fused >= 3 && (p->kernel != FG_KERNEL_KN_MFMA || p->splitk > kMailboxMaxSplit)) return FG_ERR_UNSUPPORTED;
  if (p->splitk > 1) {
    if ((long long)p->grid_x * p->grid_y > kWsMaxTiles) p->fused = 0;
    // the in-launch completion addresses the partials with 32-bit byte offsets
    if ((unsigned long long)p->splitk * M * N * sizeof(float) > 0x7fffffffull) p->fused = 0;
    p->workspace_bytes = kWsHeaderBytes + (size_t)p->splitk * M * N * sizeof(float);
  } else {
    p->workspace_bytes = 0;
  }
  return FG_OK;
}

// Wider tiles of the row-load kernel on 128-byte bands.  Two, three or a ragged number of column
// blocks share a staged band of activations and a band carries half the activation bytes, so the
// L2 traffic for A drops to a quarter or less of the 16-column / 256-byte form -- but the grid
// shrinks with the tile, so it has to land on whole CUs: 192..256 workgroups of 8 waves (one a
// CU) or 448..512 (two a CU).  Candidates, measured against the 16-column form (us):
//   32 columns            K = N = 8192 M=16 22.8 / 24.7, M=8 22.9 / 23.3; K = N = 6144 M=16 16.6 / 18.9;
//                         K=2048 N=8192 M=16 7.9 / 9.0; K=4096 N=16384 M=16 22.4 / 24.3 (4 waves)
//   32 columns, split-K   N=3072 K=12288 M=16 S=2 18.2 / 19.4 (M <= 8: 16.3 / 16.1, so M >= 9 only);
//                         N=2560 K=10240 M=16 S=3 13.3 / 16.7; N=5120 K=13824 S=3 (two a CU) 24.8 / 27.0
//   48 columns            N = 12288: K=3072 M=16 14.4 / 15.9, K=12288 47.0 / 52.6; N=3072 K=12288 split 4 ways
//   64 columns            N = 28672, K = 8192
//   N/256 or N/512 columns with a partly filled last block (masked loads cost a little):
//                         N=11008 K=4096 M=16 17.4 / 19.0 (M=8: 17.4 / 17.0); N=10240 K=8192 M=16
//                         28.4 / 33.0; N = K = 5120 M=8 12.1 / 14.1; N=6144 K=4096 M=16 11.2 / 12.9
//                         (24 columns, against 32); N=13824 K=5120 M=16 26.1 / 30.3 (27 columns, two a CU)
// 384 workgroups (N = 12288 at 32 columns) leave half the CUs with one: 46+ us against 45.
struct WideTile {
  int tile_n = 0, waves = 0, splitk = 1;
};
WideTile pick_wide_tile(int M, int N, int K, int splitk) {
  WideTile best;
  double best_fill = 0.0;
  // a later candidate replaces an earlier one only when it fills the CUs better by `margin`
  auto offer = [&](int tile, int waves, int S, int wgs, bool allowed, double margin = 0.04) {
    if (!allowed) return;
    const double fill = (double)wgs / (double)(ceil_div(wgs, kCUs) * kCUs);
    if (fill > best_fill + margin) {
      best_fill = fill;
      best = WideTile{tile, waves, S};
    }
  };
  const bool auto_split = splitk == 0;
  // Rows that do not start on a 2 KB boundary (K not a multiple of 1024) cost the 128-byte-band
  // tiles their lead: N=12288 K=11008 M=8 48 columns 49.6 us against 42.4 for 16 columns on 256-byte
  // bands, K=10752 46.4 / 41.9, while K=10240 and K=11264 are 40.2 and 42.6 with 48 columns;
  // N=8192 K=11008 M=8 32 columns 31.1 / 29.8, N=16384 59.0 / 55.6.  With 9..16 rows the 32-column
  // forms stay level.
  const bool odd_pitch = K % 1024 != 0 && K > 4096;
  if (N % 32 == 0) {
    const int t32 = N / 32;
    // not at K = 4096, where rows 8 KB apart make this form 8-15 % slower than 16-column tiles
    // (N=8192 M=8 14.6 us against 12.5; K = 3840 and 4352 are unaffected)
    offer(32, 8, 1, t32, t32 <= kCUs && 4 * t32 >= 3 * kCUs && (M >= 4 || t32 < kCUs) && K != 4096 &&
                             (!odd_pitch || M >= 9 || 8 * t32 < 7 * kCUs));
    // short rows of very wide outputs: two 8-wave workgroups of 32 columns on every CU
    // (K=2048: N=14336 M=8 12.1 -> 11.3 us, N=16384 M=16 13.7 -> 12.7)
    offer(32, 8, 1, t32, K > 1024 && K <= 2048 && M >= 4 && t32 <= 2 * kCUs && 8 * t32 >= 13 * kCUs);
    // 64 columns on 13/16 of the CUs or more beat two 4-wave workgroups of 32 on each
    // (N=14336 K=4096: M=8 21.0 -> 20.0 us, M=16 21.9 -> 20.8; N=13824 K=5120 M=8 25.8 -> 24.7)
    if (N % 64 == 0) {
      const int t64 = N / 64;
      offer(64, 8, 1, t64, M >= 5 && K >= 2048 && t64 < kCUs && 16 * t64 >= 13 * kCUs);
      // ... already on 25/32 of them from K = 4096 on (N=12800 M=8: K=4096 20.1 -> 18.3 us, K=8192
      // 38.1 -> 33.7; N=13056 M=16: K=4096 22.8 -> 19.9, K=12288 64.4 -> 53.6)
      offer(64, 8, 1, t64, M >= 5 && K >= 4096 && t64 < kCUs && 32 * t64 >= 25 * kCUs);
      // ... and one 64-column workgroup on every CU for 12 rows and more (N=16384 M=16: K=5120
      // 30.1 -> 28.0 us, K=14336 73.4 -> 70.5)
      offer(64, 8, 1, t64, M >= 12 && K >= 5120 && t64 == kCUs);
    }
    offer(32, 4, 1, t32, 8 * t32 >= 7 * 2 * kCUs && t32 <= 2 * kCUs && (t32 == 2 * kCUs ? M >= 5 : M >= 9) &&
                             (!odd_pitch || M >= 9));
  }
  if (N % 48 == 0) {
    const int t48 = N / 48;
    // (one a CU from four rows on: N=9216 M=4 K=4096 14.9 -> 14.2 us, K=8192 27.7 -> 25.5)
    offer(48, 8, 1, t48, !odd_pitch && ((M >= (t48 < kCUs ? 3 : 8) && t48 <= kCUs && 4 * t48 >= 3 * kCUs) ||
                                        (t48 == 2 * kCUs && M >= 9)));
  }
  if (N % 64 == 0) {
    // very wide outputs (N=28672 K=8192 M=16: 64 columns 72.1 us, 32 columns 74.0, 16 columns 81+)
    const int t64 = N / 64;
    offer(64, 8, 1, t64, M >= 9 && K >= 8192 && t64 <= 2 * kCUs && 8 * t64 >= 7 * 2 * kCUs);
  }
  if (N % 32 == 0 && auto_split && N / 32 < 3 * kCUs / 4) {
    // split-K keeps at least 3072 k per split (six 128-byte bands for each of eight waves)
    const int t32 = N / 32;
    for (int S = 2; S <= 4; ++S) {
      const int wgs = t32 * S;
      // (64 tiles or fewer split four ways from 2048 k a split: N=2048 M=16 K=8192 10.2 -> 9.7 us,
      // K=11008 12.8 -> 11.9; two ways only beyond K = 8192: N=4096 K=8192 M=16 15.0 against 14.3
      // for 16 columns unsplit)
      const bool long_k = t32 <= 64 ? K / S >= 2048 : K / S >= 3072 && (S > 2 || K > 8192);
      offer(32, 8, S, wgs, long_k && M >= 9 && wgs <= kCUs && 4 * wgs >= 3 * kCUs);
    }
    // (80 tiles split three ways already from 1365 k a split: N=2560 M=16 K=4096 8.0 -> 7.4 us, K=8192
    // 12.7 -> 10.6; eight rows from K = 6144 on, 9.4 -> 8.3 and 10.8 -> 9.9)
    offer(32, 8, 3, 3 * t32, t32 == 80 && ((M >= 9 && K >= 4096) || (M == 8 && K >= 6144)));
    if (N % 48 == 0) {
      // (N=3072 K=12288 M=16: 48 columns split 4 ways 16.4 us, 32 columns split 2 ways 17.9)
      const int t48 = N / 48;
      for (int S = 2; S <= 4; ++S) {
        const int wgs = t48 * S;
        // (64 tiles: from 1536 k a split, N=3072 K=6144 M=16 11.3 -> 10.6 us; 8 rows only with long
        // K, K=14336 18.1 -> 17.3 but K=6144 9.4 -> 10.1)
        const bool ok48 = (t48 <= 64 && S == 4) ? K / S >= 1536 && (M >= 9 || (M == 8 && K >= 12288))
                                               : K / S >= 3072 && M >= 9;
        offer(48, 8, S, wgs, ok48 && wgs <= kCUs && 4 * wgs >= 3 * kCUs);
      }
    }
    // two workgroups a CU, only where no split lands on one a CU
    bool one_a_cu = false;
    for (int S = 1; S <= 4; ++S) one_a_cu |= t32 * S <= kCUs && 4 * t32 * S >= 3 * kCUs;
    for (int S = 2; S <= 4 && !one_a_cu; ++S) {
      const int wgs = t32 * S;
      offer(32, 8, S, wgs, K / S >= 3072 && M >= 4 && wgs <= 2 * kCUs && 8 * wgs >= 7 * 2 * kCUs);
    }
  }
  // Ragged tiles pay for their masked loads and empty operand slots: they need a clearly better
  // fill (N = 7168, M = 9: 28 columns 19.4 us, 32 columns 18.2), three column blocks (33..47 columns) against 48 columns too (N = 9216:
  // 36 columns 17.3 us, 48 columns 15.5), and two ragged workgroups a CU lose to 448 workgroups of
  // 32 columns (N=14336 K=4096 M=16: 23.9 / 22.0).
  if (K >= 1024 && N % kCUs == 0) {
    const int tw = N / kCUs;
    const bool thin16 = N / 16 < 3 * kCUs / 2;  // 16-column tiles would leave CUs with one workgroup
    // (K = 4096 again, two nearly full column blocks: N=7168 M=9 28 columns 14.4 us against 13.0 for
    // 16; N=6144 24 columns 10.9 / 11.6 and N=11008 43 columns 17.0 / 18.4 are unaffected)
    offer(tw, 8, 1, kCUs,
          tw >= 20 && tw < 48 && tw % 16 != 0 && (M >= 9 || (thin16 && M >= 3)) && !(K == 4096 && tw > 24 && tw < 32),
          tw > 32 ? 0.3 : 0.15);
  }
  if (K >= 1024 && N % (2 * kCUs) == 0) {
    const int tw = N / (2 * kCUs);
    // (not over 64-column tiles on 25/32 of the CUs or more: N=12800 M=16 K=8192 25 columns 35.5 us,
    // 64 columns 34.3; N=13824 K=4096 27 columns 21.3 / 20.4, K=8192 37.4 / 36.3; at K = 5120 the two
    // are within 4 % either way: N=12800 M=9 23.4 / 24.4, N=13824 M=16 26.2 / 25.8.  Rows off 2 KB
    // boundaries were not measured and keep the ragged form.)
    offer(tw, 8, 1, 2 * kCUs, tw >= 20 && tw < 48 && tw % 16 != 0 && M >= 9 && (best.tile_n != 64 || odd_pitch), 0.15);
  }
  return best;
}

int make_plan(int M, int N, int K, int w_layout, int splitk, fg_plan_t* p) {
  std::memset(p, 0, sizeof(*p));
  p->stream_w = 1;
  // Split-K can finish inside the launch (the last workgroup of a tile sums the partials) or
  // in a second kernel.  Measured at K = N = 8192, S = 4 (us per call, second kernel / in-launch):
  // [K,N] M=1 26.4 / 25.0, M=8 26.2 / 25.2, M=16 26.5 / 25.9.  Beyond one block of 16 rows the
  // second kernel takes over.
  p->fused = M <= 16;
  int items = 1;
  bool row_tiles = false;   // the 16-column row-load kernel picks its own split
  bool wide_tiles = false;  // ... in its 32-column form
  int wide_band_waves = 0, wide_band_split = 0;  // ... on 128-byte bands: waves and split are fixed
  if (w_layout == FG_W_NK) {
    // Measured on MI355X at K = N = 8192 (us per call): M=1 dot2 tile 4: 21.6-22.4; M=4 dot2
    // 24.3 / mfma4 22.3; M=8 dot2 27.8 / mfma4 25.6 / row-load 23.3; M=16 mfma4 36 / direct
    // 16x16x32 31.7 / transposing 27.3 / row-load 24.6.  Every rule below is the measured winner of
    // a sweep over K = N in 1024..16384 and the LLaMA / DiT projection shapes for its range.
    const bool huge = K >= 16384 && N >= 16384;  // the 4x4x4 MFMA kernel's zone, also for M <= 2
    if ((M <= 2 && !huge) || (M <= 4 && N <= 2048 && K >= 8192)) {
      // (few, long rows at M = 3..4: v_dot2 8.8-9.3 us against 9.4-9.5 for N = 2048, K = 8192)
      p->kernel = FG_KERNEL_NK_DOT2;
      p->m_block = M <= 2 ? M : 4;
      p->tile_n = 4;
      // two load groups in flight beyond K = 8192 (K=11008 N=4096 M=1 16.7 -> 15.8 us, K=14336
      // 20.0 -> 19.0); start steps by workgroup id below K = 8192 and between 8192 and 16384, by
      // workgroup id / 8 at 8192 (22.0 -> 21.8) and from 16384 on (N=4096 23.2 -> 21.6, N=8192
      // 42.5 -> 40.2, N=14336 71.5 -> 68.8)
      p->unroll = (K > 8192 || M > 2) ? 2 : 1;
      // K = 5120 is two and a half steps of four waves: four load groups in flight make it one (inside a
      // replayed graph, M=1: N=4096 8.96 -> 8.37 us, N=5120 10.25 -> 9.81, N=8192 14.61 -> 14.22)
      if (K == 5120 && M <= 2) p->unroll = 4;
      items = ceil_div(K / 8, 64 * p->unroll);
      p->stagger = M <= 2 ? (K < 8192 || (K > 8192 && K < 16384)) : items <= 16;
    } else if (M <= 8 && huge) {
      // (K = N = 16384: M = 1 79.8 us against 82.1 for v_dot2, M = 2 79.1 / 81.5, M = 4 78.7 against
      // 79.9 for the row-load kernel, M = 8 77.5 / 78.9; at
      // N = 8192, K = 28672 the row-load kernel is ahead, M = 8 69.8 / 78.3)
      p->kernel = FG_KERNEL_NK_MFMA4;
      p->m_block = M <= 4 ? 4 : 8;
      if (K >= 16384) {
        p->tile_n = 32, p->unroll = 1;
      } else if (K == 8192 || N <= 4096) {
        // two chunks per wave and step: 8 steps at K = 8192, one K band per XCD
        p->tile_n = N <= 4096 ? 8 : 16, p->unroll = K >= 256 ? 2 : 1, p->stagger = K <= 8192;
      } else {
        p->tile_n = 16, p->unroll = 1;
      }
      items = ceil_div(K / 128, p->unroll);
    } else {
      // M >= 3: 16-column tiles, weights and activations as contiguous row pieces through LDS,
      // 8 waves on 256-byte bands.  Measured against the best of the other [N,K] kernels (us):
      // K = N = 8192 M=8 23.2 / 25.6, M=16 24.6 / 27.3; K=3072 N=12288 M=16 15.6 / 21.0;
      // K=12288 N=3072 M=16 19.1 / 20.3; K = N = 4096 M=8 7.8 / 9.5; K=4096 N=11008 M=8 16.5 / 20.1.
      // At K = 16384 four waves on 512-byte bands are level or slightly ahead (M=16 84.3 / 85.8).
      // M = 3..4 against the 4x4x4 kernel: K = N = 4096 8.7-8.9 / 9.2-9.5, K = N = 8192 22.9 / 22.3-24.0,
      // K=12288 N=3072 14.6 / 15.2-16.0, K=4096 N=11008 15.8 / 16.6-16.9.
      p->kernel = FG_KERNEL_NK_MFMA_R;
      p->m_block = 16;
      p->tile_n = 16;
      p->unroll = (K >= 16384 && N >= 8192) ? 2 : 1;
      items = ceil_div(K, 128 * p->unroll);
      row_tiles = true;
      if (M > 16) {
        // 32 rows of A per workgroup (two MFMA row blocks on 128-byte bands): 17..32 rows read the
        // weights once instead of twice
        p->m_block = 32;
        p->unroll = 1;
        p->band = 128;
        items = ceil_div(K, 64);
      }
      if (!wide_tiles && M <= 32 && splitk <= 1) {
        WideTile wt = pick_wide_tile(M < 16 ? M : 16, N, K, splitk);
        if (M > 16 && (wt.tile_n % 16 != 0 || wt.tile_n > 48)) wt = WideTile{};  // no ragged or 64-column form
        if (wt.tile_n) {
          p->tile_n = wt.tile_n;
          p->unroll = 1;
          p->band = 128;
          wide_tiles = true;
          wide_band_waves = wt.waves;
          wide_band_split = wt.splitk;
        }
      }
    }
  } else {
    const size_t weights = (size_t)N * K;
    if (M <= 2 && (weights < ((size_t)1 << 27) || (weights < ((size_t)1 << 28) && (M == 1 || N <= 12288 || (K <= 8192 && (N == 18432 || N == 22016)))))) {
      // One or two rows take the v_dot2 kernel up to 2^28 weights: its deep splits cost little now
      // that they complete through one atomic per element (M = 1, v_dot2 / MFMA kernel, us:
      // K=16384 N=8192 42.5 / 45.4, K=11008 N=12288 42.8 / 45.6, K=16384 N=12288 62.0 / 66.2,
      // K=8192 N=16384 42.2 / 44.0; at K = N = 16384 the two are level and the MFMA kernel stays;
      // two rows from 2^27 weights on only up to N = 12288: K=16384 N=12288 63.2 / 66.1, but
      // K=16384 N=14336 76.0 / 74.0; two widths measured later with K = 8192 again: N=18432 49.3 / 52.0,
      // N=22016 60.9 / 70.7).
      p->kernel = FG_KERNEL_KN_DOT2;
      p->m_block = M;
    } else {
      p->kernel = FG_KERNEL_KN_MFMA;  // 26.3 us against 29.8 for v_dot2 at M = 4, K = N = 8192
      p->m_block = 16;
    }
    p->tile_n = 128;
    // one 32-row unit in flight per wave and step: with the split-K tail no longer waiting on
    // each partial in turn, deeper splits of shorter steps win (v_dot2, M = 1, two units / one:
    // K = N = 4096 10.5 / 9.7 us, K=3072 N=12288 16.7 / 15.5, K=4096 N=11008 18.5 / 17.3)
    p->unroll = 1;
    items = ceil_div(K / 32, p->unroll);
  }
  {
    p->waves = (row_tiles && !wide_tiles && p->unroll == 1 && items >= 16) ? 8 : pick_waves(items);
    if (p->kernel == FG_KERNEL_NK_DOT2 && K == 5120 && M <= 2) p->waves = 4;  // (measured with four)
    if (wide_band_waves) {
      p->waves = wide_band_waves;
      while (p->waves > 1 && p->waves > K / 64) p->waves >>= 1;  // one 128-byte band per wave at least
    }
    const int tiles = (N / p->tile_n) * ceil_div(M, p->m_block);
    if (splitk > 0) {
      p->splitk = splitk;
    } else if (w_layout == FG_W_KN) {
      // [K,N] tiles are 128 columns wide, so the grid needs split-K to cover the chip: the
      // factor that brings tiles*S closest to one workgroup per CU.
      int best = 1;
      bool half_filled = false;  // fewer workgroups than CUs on purpose
      if ((size_t)N * K < ((size_t)1 << 26) && items >= 16 && M <= 16) {
        // Below 8192 x 8192 the call is latency-bound: 8 waves per workgroup and half the split
        // (about 192 workgroups) shorten every wave's chain of dependent loads.  Measured (us,
        // 4 waves / 8 waves, M = 4): K=N=4096 12.3 / 11.2, K=4096 N=11008 20.1 / 18.1,
        // K=3072 N=12288 17.2 / 15.9, K=12288 N=3072 20.5 / 17.8, K=N=2048 12.3 / 8.8.
        // Here the in-launch reduction also wins for 9..16 rows (M = 16: K=3072 N=12288 17.2 us
        // against 17.9 with the second kernel, K=12288 N=3072 18.9 / 20.0, K=4096 N=11008 19.3 /
        // 20.3); at 8192 x 8192 the second kernel stays 0.6 us ahead for them.
        // Sixteen tiles or fewer with K <= 8192 leave each wave one or two units at 192 workgroups:
        // aim at 128 there (N=2048: K=4096 M=1 9.7 -> 8.1 us, M=16 10.8 -> 9.0; K=8192 12.0 -> 10.6).
        // Eight tiles with long K take a 24-way split (N=1024 K=28672: M=1 15.3 -> 13.8, M=16 17.9
        // -> 16.2) as long as every wave keeps two units.
        // Sixteen column tiles or fewer: with the atomic completion a deep split is cheap, so the
        // grid aims at every CU (one or two rows: one and a half workgroups of four waves a CU)
        // instead of half of them (N=2048 K=8192, 8 ways -> deeper: M=1 9.9 -> 8.1 us, M=8 11.3 ->
        // 9.8, M=16 12.2 -> 11.4; N=2048 K=16384 M=1 14.0 -> 12.7; N=1024 K=11008 M=4 8.7 -> 7.7).
        // For nine rows and more splits of 3, 6 and 12 are offered too (K = N = 4096 M=16: 6 ways
        // 10.9 us, 8 ways 11.7).
        // Eight tiles keep eight waves and three quarters of the CUs (N=1024 K=16384 M=1: 24 ways
        // of eight waves 8.6 us, 31 ways of four 9.3); nine rows and more go from 192 to 256
        // workgroups beyond K = 8192 (N=2048 M=16: K=8192 12 ways 11.3 us / 16 ways 12+, K=16384
        // 17.6 / 16.7).
        const bool narrow = tiles <= 16;
        p->waves = (narrow && tiles > 8 && M <= 2) ? 4 : 8;
        p->fused = 1;
        half_filled = narrow;  // (keeps the search over every integer split below out of this range)
        double target = 192.0;
        if (narrow && tiles > 8) target = M <= 2 ? 384.0 : ((M <= 8 || K > 8192) ? 256.0 : 192.0);
        double best_dist = 1e30;
        static const int kSplits[] = {1, 2, 3, 4, 6, 8, 12, 16, 24, 31};
        for (int S : kSplits) {
          if ((S == 3 || S == 6 || S == 12) && M <= 8) continue;
          if (items / (p->waves * S) < 1) break;
          if (S > 16 && !narrow) break;
          // 9..16 rows: the partials of a split that leaves a wave one unit cost more than the
          // idle CUs once there are more than 192 workgroups (N=4096 K=2048 M=12: 8 ways 10.3 us,
          // 4 ways 8.3; N=2048 K=2048 M=16: 8 ways 7.4, 4 ways 7.9)
          if (M > 8 && S > 1 && items / (p->waves * S) < 2 && tiles * S > 192) break;
          const double dist = std::fabs(std::log2((double)tiles * S / target));
          if (dist < best_dist - 1e-9) {
            best_dist = dist;
            best = S;
          }
        }
      } else if ((size_t)N * K >= ((size_t)1 << 18)) {  // 1024 x 1024: 7.7 us with S = 8 against 9.0 without
        // up to eight rows the partials are small enough for two workgroups per CU to pay, the more
        // so as the two take neighbouring column bands (K = N = 8192, S = 8 / S = 4: M=1 23.1 / 24.3
        // us, M=4 23.9 / 25.4, M=8 24.7 / 24.9; K=4096 N=16384 M=1 S = 4 / 2: 23.3 / 24.5)
        const bool two_a_cu = (size_t)N * K <= ((size_t)1 << 26) && ((M <= 8 && tiles <= 64) || (M <= 2 && tiles <= 128));
        const int target = two_a_cu ? 2 * kCUs : kCUs;
        double best_ratio = 1e30;
        for (int S = 1; S <= 16; S *= 2) {
          if (items / (p->waves * S) < 1) break;
          const double r = (double)tiles * S / target;
          const double ratio = r > 1.0 ? r : 1.0 / (r * r);  // idle CUs cost more than a deeper split
          if (ratio < best_ratio - 1e-9) {
            best_ratio = ratio;
            best = S;
          }
        }
      }
      // v_dot2 on 2^27 weights and more: four waves, each left with about eight 32-row units, up to
      // four workgroups a CU (K=16384 N=8192 M=1: 16 ways 42.5 us, 4 ways 45+)
      bool deep_dot2 = false;
      if (p->kernel == FG_KERNEL_KN_DOT2 && (size_t)N * K >= ((size_t)1 << 27)) {
        static const int kDeep[] = {16, 10, 8, 5, 4, 2};
        for (int S : kDeep) {
          if (tiles * S <= 4 * kCUs && items / (4 * S) >= 8) {
            best = S;
            p->waves = 4;
            deep_dot2 = true;
            break;
          }
        }
      }
      p->splitk = best;
      // the v_dot2 kernel wants eight waves on every CU: K=4096 N=16384, M = 1, S = 2:
      // 26.9 us with four waves a workgroup, 24.3 with eight
      if (p->kernel == FG_KERNEL_KN_DOT2 && p->waves == 4 && tiles * best < 2 * kCUs &&
          items / (8 * best) >= 2 && !deep_dot2 && !half_filled) {
        p->waves = 8;
      }
      // 9..16 rows at 8192 x 8192: 26.0 us with eight waves against 26.5 with four (at 16384 x 16384
      // four stay ahead, 82.3 against 89)
      if (p->kernel == FG_KERNEL_KN_MFMA && M > 8 && p->waves == 4 &&
          (size_t)N * K <= ((size_t)1 << 26) && items / (8 * best) >= 2) {
        p->waves = 8;
      }
      // The rules above only try powers of two.  When their choice leaves the CUs unevenly loaded
      // (tiles * S just over a multiple of 256: 80 tiles x 4 = 320 workgroups take 36 us where
      // 80 x 3 = 240 take 29), search every S with either one 8-wave workgroup per CU or two
      // 4-wave ones, scored by how evenly the CUs are filled, how evenly K divides over the wave
      // slots, the partial traffic and the length of each wave's chain of loads.  Fitted to
      // sweeps over N in {5120, 6144, 9216, 10240, 11008, 12288, 13824, 14336} x K in {3072..13824}.
      {
        auto score = [&](int S, int w) {
          const int n = tiles * S;
          const int per_cu = ceil_div(n, kCUs);
          const double fill = (double)n / ((double)per_cu * kCUs);
          const double per_wave = (double)items / (w * S);
          const double chain = per_wave >= 8.0 ? 1.0 : std::sqrt(per_wave / 8.0);
          const double partials = 1.0 / (1.0 + 4.0 * S * M / K);
          // 9..16 rows: two 4-wave workgroups a CU write twice the partials of one 8-wave workgroup
          // for the same K range and lose to it at equal fill (N=5120 K=8192 M=16: 11 splits of 4
          // waves 20.4 us, 5 of 8 waves 19.2; N=9216 K=4096 18.2 / 17.6)
          // (four rows and more, too, since the split completes through atomics: N=5120 K=4096 M=8
          // 11 splits of 4 waves 11.8 us, 6 of 8 waves 10.9)
          const double two_a_cu = w == 4 ? (M > 8 ? 0.88 : (M >= 4 ? 0.94 : 1.0)) : 1.0;
          return fill * balance(items, w * S) * partials * chain * two_a_cu;
        };
        const int n0 = tiles * p->splitk;
        const double fill0 = (double)n0 / ((double)ceil_div(n0, kCUs) * kCUs);
        if (fill0 < 0.85 && !half_filled && M <= 16 && (size_t)N * K >= ((size_t)1 << 22)) {
          double best_score = score(p->splitk, p->waves) * 1.05;  // switch for a clear win only
          int best_s = 0, best_w = 0;
          for (int S = 1; S <= 16; ++S) {
            const int per_cu = ceil_div(tiles * S, kCUs);
            if (per_cu > 2) break;
            const int w = per_cu == 1 ? 8 : 4;
            if (items / (w * S) < 2) break;
            const double sc = score(S, w);
            if (sc > best_score + 1e-9) {
              best_score = sc;
              best_s = S;
              best_w = w;
            }
          }
          if (best_s) {
            p->splitk = best_s;
            p->waves = best_w;
          }
        }
      }
      // 9..16 rows, four splits of 64 tiles (one workgroup on every CU) and at least eight units a
      // wave: eight waves with two units in flight (K = N = 8192 M=16 26.2 -> 25.7 us, K=14336
      // 42.0 -> 41.2; not with rows off 2 KB boundaries, and not with other splits: K=4096 N=12288
      // 21.1 -> 21.6)
      if (p->kernel == FG_KERNEL_KN_MFMA && M > 8 && M <= 16 && tiles == 64 && p->splitk == 4 &&
          K % 1024 == 0 && items / (8 * 4) >= 8 && (size_t)N * K <= ((size_t)1 << 27)) {
        p->waves = 8;
        p->unroll = 2;
      }
      // One or two rows: two 4-wave workgroups a CU on neighbouring column bands instead of one
      // 8-wave workgroup, where that lands on 448..512 workgroups and leaves every wave four units
      // (M=1, twice the split with 4 waves / 8 waves: K=14336 N=8192 37.3 / 40.6 us, K=11008 N=8192
      // 30.4 / 32.4, K=5120 N=16384 28.2 / 29.8; M=2: K=11008 N=4096 17.6 / 18.5, K=4096 N=8192
      // 14.1 / 14.7); two units a wave are enough (five alternating runs each, minimum: K = N = 4096
      // M=1 8.03 / 8.29, M=2 8.31 / 8.62; K=5120 N=4096 9.11 / 9.89; K=6144 N=4096 10.35 / 10.82;
      // K=3072 N=8192 10.53 / 11.09; K=5120 N=3072 7.98 / 8.18; one and a half are not: K=3072
      // N=4096 7.96 / 7.88)
      {
        const int twice = 2 * tiles * p->splitk;
        if (splitk == 0 && M <= 2 && p->kernel == FG_KERNEL_KN_DOT2 && p->waves == 8 &&
            p->splitk <= 12 && twice >= 448 && twice <= 2 * kCUs && items / (4 * 2 * p->splitk) >= 2) {
          p->splitk *= 2;
          p->waves = 4;
        }
      }
    } else if (wide_band_split) {
      p->splitk = wide_band_split;
      p->fused = 1;
    } else if (row_tiles) {
      // 192 tiles still run best unsplit (K=12288 N=3072 M=8: 16.0 us against 17.4 with S = 4);
      // 128 tiles or fewer want two workgroups per CU once K is long (N=2048: K=8192 M=16
      // 10.5 us with S = 2 against 12.4, K=16384 15.7 against 21.7).  The partials of a 16-column
      // tile are small, so the split always completes inside the launch.
      // (from K = 5120 on for 8 rows and more: N=1024 K=6144 M=16 10.2 -> 7.9 us, N=2048 K=6144
      // M=8 9.0 -> 8.0)
      int S = (tiles > kCUs / 2 || K < (M >= 8 ? 5120 : 8192)) ? 1 : ceil_div(kCUs, tiles);
      while (S > 1 && items / (p->waves * S) < 2) --S;  // keep two bands per wave
      p->splitk = S;
      p->fused = 1;
      // with only two 256-byte bands left per wave, four of 128 bytes pipeline better
      // (N=1024 K=8192 S=4: M=8 7.8 us against 8.9, M=16 8.0 / 9.4)
      if (S > 1 && p->unroll == 1 && items / (p->waves * S) <= 2) p->band = 128;
      // the same for short rows of wide outputs (K=2048 M=8: N=10240 10.6 -> 9.4 us, N=12288 M=4
      // 11.1 -> 10.0; K=1024 N=13824 M=8 8.0 -> 7.7; K=4096 N=12288 M=6 18.5 -> 16.8)
      if (S == 1 && p->unroll == 1 && K >= 1024 && (K <= 2048 ? N >= 8192 : (K <= 4096 && N >= 12288))) {
        p->band = 128;
        p->waves = 8;
      }
    } else {
      p->splitk = pick_splitk(tiles, p->waves, items, M, N, K, kCUs);
    }
  }
  const int st = finish_plan(M, N, K, p);
  if (st != FG_OK) return st;
  // In-launch completion through one fixed-point atomic per output element (fused = 2) instead of
  // partials + arrival counter (fused = 1): one memory round trip after the K loop instead of
  // three, but S * M * N atomics.  Measured over 11 N x 7 K x 6 M on both layouts (us gained over
  // the counter protocol): every v_dot2 split 0.5 .. 2.5, every [N,K] split 0.3 .. 1.9.  For the
  // [K,N] MFMA kernel, whose counter protocol writes its partials as whole 512-byte rows, 385
  // splits (M = 3 .. 16) put the break-even at: eight waves, 16 splits or more 0.3 .. 2.4 gained
  // up to 2^20 atomics; 8 .. 15 splits 0.2 .. 1.4 gained up to 6 * 2^16 atomics, level to 0.9 lost
  // above; fewer splits 0.2 gained on average below 3 * 2^16, 0.1 .. 1.9 lost above.  Four waves:
  // gained only from 16 splits on, or from 8 below 3 * 2^16; 0.2 .. 2.0 lost otherwise.
  if (p->splitk > 1 && p->fused == 1 && p->splitk <= kFixMaxSplit && (size_t)M * N <= kWsAccElems) {
    const size_t atomics = (size_t)p->splitk * M * N;
    bool atomic = true;
    if (p->kernel == FG_KERNEL_KN_MFMA) {
      const size_t unit = (size_t)1 << 16;
      if (p->splitk >= 16) atomic = atomics < 16 * unit;
      else if (p->splitk >= 8) atomic = atomics <= (p->waves >= 8 ? 6 : 3) * unit;
      else atomic = p->waves >= 8 && atomics < 3 * unit;
    }
    if (atomic) p->fused = 2;
  }
  // [K,N] MFMA kernel, up to 16 rows: completion through flags in one XCD's L2 (fused = 3).  Its
  // partials never leave the L2 and nobody waits for an atomic, so it pays where the partials are
  // large (nine rows and more) and it favours deeper splits of 4-wave workgroups, two or three a CU.
  // Fitted to a sweep of 10 N x 8 K x M in {4, 8, 16} with about 100 plans a cell (us, this rule /
  // the counter or atomic plan it replaces): N = K = 8192 M=8 24.1 / 24.7, M=16 24.5 / 25.3;
  // N=8192 K=16384 M=16 43.8 / 46.3; N=12288 K=8192 M=8 34.4 / 36.3, K=12288 M=16 50.0 / 52.7;
  // N=16384 K=3072 M=8 18.6 / 19.8; N=11008 K=4096 M=16 18.6 / 19.3; N=4096 K=4096 M=16 10.1 / 10.6;
  // N=3072 K=4096 M=16 8.8 / 9.9; N=2048 K=12288 M=16 13.0 / 14.1.  Not taken where it measured level
  // or behind: 14 336 columns, N = 16384 with few rows and long K, short K.  A later pass over
  // N in {4096, 8192} x 10 K x M in {4, 8, 16} widened the 64-tile rows (N = 8192: M=4 K=5504 17.9 /
  // 19.0, K=11008 31.2 / 32.5; M=8 K=4096 14.4 / 14.8, K=6144 19.2 / 20.1; M=16 K=5504 18.7 / 19.4,
  // K=6144 19.3 / 20.4 with two units a step) and added long K at 32 tiles (N=4096 K=11008 M=8 18.3 /
  // 18.8, K=14336 21.9 / 22.4; level for M=4 and for K = 12288).  A third pass put widths between
  // the fitted ones beside them (N in {5120, 6144, 10240, 12288} x 9 K x M in {4, 8, 16}, the library's
  // plan beside every flag plan that fills 224..1024 wave slots): 48 tiles x 9 splits (N=6144 K=4096
  // M=8 12.1 / 12.4, K=8192 M=16 20.4 / 21.1, K=11008 24.6 / 25.3; K=3072 behind), 80 tiles x 6
  // (N=10240 K=4096 M=16 17.2 / 18.3, K=11008 37.9 / 39.6, K=16384 53.5 / 55.9), 40 tiles x 6 from
  // K = 8192 on for seven rows and more (N=5120 K=8192 M=16 18.0 / 18.5, level at K = 12288), and 96
  // tiles from K = 2048 on for eight rows and fewer (N=12288 K=3072 M=8 15.7 / 16.4).  The same for
  // N in {2560, 3584, 9216, 18432, 20480, 24576}: 72 tiles x 7 (N=9216 K=4096 M=8 15.7 / 17.3, K=8192
  // 26.3 / 28.4, K=16384 48.0 / 51.4), 144 x 5 (N=18432 K=4096 M=16 27.1 / 30.9, K=16384 95.8 / 105.1),
  // 160 x 6 with two units a step up to eight rows (N=20480 K=8192 M=4 53.4 / 55.5), 192 x 4 (N=24576
  // K=8192 M=16 65.9 / 69.3), and nine rows and more on 20 and 28 tiles with short K (N=2560 K=4096
  // 8.8 / 9.5, N=3584 K=3072 8.8 / 9.3); 100 tiles x 7 (N=12800 K=6144 M=16 28.9 / 31.7, K=16384 M=8
  // 67.6 / 72.0; x 4 below K = 4096) and 172 x 4 (N=22016 K=4096 M=8 32.0 / 34.1, K=8192 M=16 60.8 /
  // 67.6, K=16384 119 / 133; x 3 = 516 workgroups is 3..9 % behind the unsplit plan).  12, 36, 56, 108,
  // 112, 120, 216, 224 and 256 tiles measured level or behind.
  if (splitk == 0 && p->kernel == FG_KERNEL_KN_MFMA && M >= 3 && M <= 16 && p->grid_y == 1 && kXccs > 1) {
    const int tiles = N / 128, units = K / 32;
    int S = 0, w = 4, U = 1;
    // (only the column counts the sweep covered: a split that fills the CUs unevenly costs far more
    // than the completion saves -- 48 tiles x 6 = 288 workgroups: 25 % slower than 5 x 8 waves)
    if (M > 8) {
      if (tiles == 16) S = 16;
      else if (tiles == 24 && K <= 8192 && M > 12) S = 8;
      else if (tiles == 32) S = 8;
      else if (tiles == 64 && K >= 4096) S = 8, U = K >= 6144 ? 2 : 1;
      else if (tiles == 20 && K >= 4096 && K <= 6144) S = 8, w = 8;
      else if (tiles == 28 && K <= 4096) S = 8, w = K == 4096 ? 8 : 4;
      else if (tiles == 40 && K >= 8192) S = 6;
      else if (tiles == 48 && K >= 4096) S = 9;
      else if (tiles == 72) S = 7;
      else if (tiles == 80 && K >= 3072) S = 6;
      else if (tiles == 100) S = K >= 4096 ? 7 : 4;
      else if (tiles == 144) S = 5;
      else if (tiles == 172) S = 4;
      else if (tiles == 192 && K >= 4096) S = 4;
      else if (tiles == 86) S = 5;
      else if (tiles == 96) S = 8;
      else if (tiles == 128 && K <= 4096) S = 4, w = 8;
      else if (tiles == 128) S = p->splitk, w = p->waves, U = p->unroll;
    } else {
      if (tiles == 64 && K >= 3072) S = 8;
      else if (tiles == 32 && K >= 11008 && M >= 7) S = 8;
      else if (tiles == 86 && K >= 3072 && K <= 4096 && M == 8) S = 5;
      else if (tiles == 40 && K >= 8192 && M >= 7) S = 6;
      else if (tiles == 48 && K >= 4096) S = 9;
      else if (tiles == 72) S = 7;
      else if (tiles == 80 && K >= 3072) S = 6;
      else if (tiles == 100) S = K >= 4096 ? 7 : 4;
      else if (tiles == 144) S = 5;
      else if (tiles == 160 && K >= 4096) S = 6, U = 2;
      else if (tiles == 172) S = 4;
      else if (tiles == 192 && K >= 5120) S = 4;
      else if (tiles == 96 && K >= 2048) S = 8;
      else if (tiles == 128 && K < 4096) S = 4, w = 8;
      else if (tiles == 128 && K == 4096) S = p->splitk, w = p->waves, U = p->unroll;
    }
    // every wave keeps two K units at least; the flag words and the owner's mask have their limits
    if (S > 1 && S <= kMailboxMaxSplit && units / (w * S * U) >= 2 &&
        (size_t)tiles * S * w <= kWsMailboxFlags) {
      fg_plan_t q = *p;
      q.splitk = S, q.waves = w, q.unroll = U, q.fused = 3;
      if (finish_plan(M, N, K, &q) == FG_OK && q.fused == 3) *p = q;
    }
  }
  // One or two rows, [K,N] v_dot2 kernel, widths between the fitted ones with K = 4096 .. 8192: three or
  // four 4-wave workgroups a CU, completed by atomics.  From a pass over 14 widths x K in {4096, 8192},
  // the plan above beside every v_dot2 plan that fills 200..1100 wave slots (us, M = 1, this rule / the
  // plan it replaces): N=6144 K=4096 10.8 / 11.4, K=8192 18.5 / 19.1; N=9216 K=8192 25.5 / 26.3; N=10240
  // K=8192 28.1 / 28.8; N=11008 K=4096 16.8 / 17.4; N=12288 K=4096 18.4 / 19.1, K=8192 33.2 / 34.0;
  // N=12800 K=4096 19.4 / 20.0, K=8192 35.0 / 36.3; N=18432 K=4096 25.7 / 27.3, K=8192 48.0 / 49.8;
  // N=22016 K=4096 31.5 / 37.4, K=8192 59.3 / 61.0.  20, 28, 40, 56, 108 and 112 tiles measured within
  // 2 % of their plans.
  if (splitk == 0 && p->kernel == FG_KERNEL_KN_DOT2 && M <= 2 && K >= 4096 && K <= 8192) {
    const int tiles = N / 128;
    int S = 0, U = 1;
    if (tiles == 48) S = 16, U = K <= 4096 ? 2 : 1;
    else if (tiles == 72 && K >= 8192) S = 14;
    else if (tiles == 80 && K >= 8192) S = 12, U = 2;
    else if (tiles == 86 && K <= 4096) S = 5;
    else if (tiles == 96) S = 10;
    else if (tiles == 100) S = 10, U = K >= 8192 ? 2 : 1;
    else if (tiles == 144) S = 7;
    else if (tiles == 172) S = 4, U = 2;
    if (S && (K / 32) / (4 * S * U) >= 1) {
      fg_plan_t q = *p;
      q.splitk = S, q.waves = 4, q.unroll = U, q.fused = 2;
      if (finish_plan(M, N, K, &q) == FG_OK && q.fused == 2) *p = q;
    }
  }
  // Small problems (4 Mi weights or fewer, up to 16 rows).  Their kernels last 3 .. 7 us, a handful
  // of dependent memory round trips, and what shortens them is more, shorter waves, each with one
  // or two loads to wait for.  Fitted to per-launch times inside a replayed graph of 64 launches
  // (no host launch rate in the figure) over N x K in {512 .. 4096}^2, about 150 plans a cell
  // (us, this rule / the plan it replaces):
  //  * [K,N]: the v_dot2 kernel on two rows a workgroup, four waves, one 32-row unit a wave (K / 128
  //    splits, 16 at most), completed by atomics: 1024 x 1024 M=1 3.8 / 4.5, M=8 4.2 / 5.6, M=16
  //    4.8 / 6.1; N=1024 K=2048 M=8 4.9 / 5.8; N=2048 K=1024 M=8 4.9 / 5.8; N=2048 K=512 M=16 4.8 /
  //    6.1.  Beyond 2 Mi weights only up to four rows (2048 x 2048 M=4 5.2 / 5.8, N=4096 K=1024 M=2
  //    4.8 / 5.4), beyond 1 Mi up to eight; nine rows and more (eight from 4096 columns) then take
  //    the MFMA kernel with the flag completion, one unit a wave (2048 x 2048 M=16 6.2 / 7.3,
  //    N=4096 K=1024 M=16 5.8 / 6.4, N=1024 K=4096 M=16 6.9 / 7.5, N=2048 K=1024 M=16 5.2 / 6.3).
  //  * [N,K] row-load kernel: eight waves; 64 tiles or fewer split K four ways, on 128-byte bands up
  //    to K = 2048 (1024 x 1024 M=8 3.5 / 4.0, M=16 3.9 / 4.3; N=1024 K=2048 M=16 4.2 / 5.0; N=1024
  //    K=4096 M=4 4.6 / 5.8, M=16 5.2 / 7.3; N=512 K=2048 M=8 3.6 / 4.5); wider outputs with K up to
  //    1024 stay unsplit on 128-byte bands (N=2048 K=1024 M=8 3.8 / 4.2, N=4096 K=1024 M=16 4.4 / 4.8).
  if (splitk == 0 && M <= 16 && (size_t)N * K <= ((size_t)1 << 22)) {
    fg_plan_t q = *p;
    bool change = false;
    if (w_layout == FG_W_KN) {
      if ((size_t)N * K <= ((size_t)1 << 20) || ((size_t)N * K <= ((size_t)1 << 21) && M <= 8) || M <= 4) {
        q.kernel = FG_KERNEL_KN_DOT2;
        q.m_block = M == 1 ? 1 : 2;
        q.waves = 4, q.unroll = 1;
        q.splitk = K / 128 < 1 ? 1 : (K / 128 > 16 ? 16 : K / 128);
        q.fused = q.splitk > 1 ? 2 : 0;
        change = true;
      } else if ((M > 8 || (M == 8 && N >= 4096)) && kXccs > 1) {
        q.kernel = FG_KERNEL_KN_MFMA;
        q.m_block = 16, q.unroll = 1;
        q.splitk = K <= 2048 ? 8 : 16;
        q.waves = K / 32 / q.splitk >= 8 ? 8 : 4;
        q.fused = 3;
        change = K / 32 >= q.splitk * q.waves;
      }
    } else if (p->kernel == FG_KERNEL_NK_MFMA_R && p->tile_n == 16 && p->m_block == 16 && K >= 512) {
      q.waves = 8, q.unroll = 1;
      if (N <= 1024 && K >= 1024) {
        q.splitk = 4, q.fused = 2, q.band = K <= 2048 ? 128 : 0;
        change = true;
      } else if (K <= 1024) {
        q.splitk = 1, q.fused = 0, q.band = 128;
        change = true;
      }
    }
    if (change && finish_plan(M, N, K, &q) == FG_OK) *p = q;
  }
  return FG_OK;
}

}  // namespace

void set_compute_units(int cus) {
  if (cus >= 16 && cus <= 4096) kCUs = cus;
}
int compute_units() { return kCUs; }
void set_xccs(int x) {
  if (x >= 1 && x <= 64) kXccs = x;
}
int xccs() { return kXccs; }

int plan_validate_shape(int M, int N, int K, int w_layout) { return validate_shape(M, N, K, w_layout); }
int plan_make(int M, int N, int K, int w_layout, int splitk, fg_plan_t* p) {
  return make_plan(M, N, K, w_layout, splitk, p);
}
int plan_finish(int M, int N, int K, fg_plan_t* p) { return finish_plan(M, N, K, p); }

}  // namespace fg
