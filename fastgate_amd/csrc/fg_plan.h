// Host-only interface of the launch planner (fg_planner.cpp): no HIP types.
#pragma once
#include <stddef.h>
#include <stdint.h>

#include "fg_flags.h"

namespace fg {

// Tile sets that exist as instantiations (the planner and the launchers share these).
bool nk_dot2_supported(int m_block, int tile_n, int unroll);
bool nk_mfma4_supported(int m_block, int tile_n, int unroll);
bool kn_dot2_supported(int m_block, int unroll);
bool kn_mfma_supported(int unroll);

// FG_OK, FG_ERR_INVALID_ARG or FG_ERR_ALIGN128.
int plan_validate_shape(int M, int N, int K, int w_layout);
// The library's plan (splitk 0) or its plan around a forced split.  Shape already validated.
int plan_make(int M, int N, int K, int w_layout, int splitk, fg_plan_t* p);
// Checks a caller-edited plan and fills grid, block and workspace size.
int plan_finish(int M, int N, int K, fg_plan_t* p);

// Compute units of the device the plans are for (default 256).
void set_compute_units(int cus);
int compute_units();
// XCDs (L2 domains) of that device (default 8).
void set_xccs(int xccs);
int xccs();

constexpr int kWsMaxTiles = (int)(kWsCounterBytes / sizeof(int));

}  // namespace fg
