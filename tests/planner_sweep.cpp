// Sweep of the launch planner on the host, meant to be built with
//   g++ -std=c++17 -O1 -g -fsanitize=address,undefined -fno-sanitize-recover=all
// together with fastgate_amd/csrc/fg_planner.cpp (tests/test_planner_sanitized.py does).
// Every plan the planner returns must be launchable: grid and block inside HIP's limits, the tile
// dividing N, the kernel/tile combination instantiated (the plan passes plan_finish again
// unchanged), the workspace size exact in 64-bit arithmetic and the completion protocol inside
// its limits.  Prints the number of plans checked; any violation aborts with a message.
#include <cstdio>
#include <cstdlib>
#include <cstring>
#include <vector>

#include "fg_plan.h"

static long long checked = 0;

static void fail(const char* what, int M, int N, int K, int layout, int splitk, const fg_plan_t& p) {
  std::fprintf(stderr,
               "planner sweep: %s at M=%d N=%d K=%d layout=%d splitk=%d -> kernel=%d S=%d fused=%d tile_n=%d "
               "m_block=%d waves=%d unroll=%d band=%d grid=(%d,%d,%d) block=%d ws=%zu\n",
               what, M, N, K, layout, splitk, p.kernel, p.splitk, p.fused, p.tile_n, p.m_block, p.waves,
               p.unroll, p.band, p.grid_x, p.grid_y, p.grid_z, p.block, p.workspace_bytes);
  std::exit(1);
}

static void check(int M, int N, int K, int layout, int splitk) {
  fg_plan_t p;
  std::memset(&p, 0xA5, sizeof(p));
  const int v = fg::plan_validate_shape(M, N, K, layout);
  if (v != FG_OK) fail("shape refused", M, N, K, layout, splitk, p);
  const int st = fg::plan_make(M, N, K, layout, splitk, &p);
  ++checked;
  if (st != FG_OK) {
    // only a forced split may be refused, and only for sizes HIP cannot launch
    if (splitk == 0) fail("library plan refused", M, N, K, layout, splitk, p);
    return;
  }
#define REQUIRE(cond) \
  if (!(cond)) fail(#cond, M, N, K, layout, splitk, p)
  const bool kn = p.kernel == FG_KERNEL_KN_DOT2 || p.kernel == FG_KERNEL_KN_MFMA;
  const bool nk = p.kernel == FG_KERNEL_NK_DOT2 || p.kernel == FG_KERNEL_NK_MFMA4 || p.kernel == FG_KERNEL_NK_MFMA_R;
  REQUIRE(layout == FG_W_KN ? kn : nk);
  REQUIRE(p.splitk >= 1 && (splitk == 0 || p.splitk == splitk));
  REQUIRE(p.tile_n >= 1 && N % p.tile_n == 0 && p.grid_x == N / p.tile_n);
  REQUIRE(p.m_block >= 1 && p.grid_y == (M + p.m_block - 1) / p.m_block);
  REQUIRE(p.grid_x >= 1 && p.grid_y >= 1 && p.grid_y <= 65535 && p.grid_z == p.splitk && p.grid_z <= 65535);
  REQUIRE(p.waves == 1 || p.waves == 2 || p.waves == 4 || p.waves == 8);
  REQUIRE(p.block == 64 * p.waves);
  REQUIRE(p.fused == 0 || p.fused == 1 || p.fused == 2 || p.fused == 3);
  const unsigned long long partials = 4ull * (unsigned long long)p.splitk * (unsigned long long)M * (unsigned long long)N;
  REQUIRE(p.workspace_bytes == (p.splitk > 1 ? (size_t)(fg::kWsHeaderBytes + partials) : (size_t)0));
  if (p.splitk > 1 && p.fused == 1) {
    REQUIRE((long long)p.grid_x * p.grid_y <= fg::kWsMaxTiles);
    REQUIRE(partials <= 0x7fffffffull);
  }
  if (p.splitk > 1 && p.fused == 2) {
    REQUIRE(p.splitk <= fg::kFixMaxSplit);
    REQUIRE((unsigned long long)M * N <= fg::kWsAccElems);
  }
  if (p.splitk > 1 && p.fused == 3) {
    // flags in one XCD's L2: the [K,N] MFMA kernel only, one block of rows, within the flag words and the owner's mask
    REQUIRE(p.kernel == FG_KERNEL_KN_MFMA && p.grid_y == 1 && splitk == 0);
    REQUIRE(p.splitk <= fg::kMailboxMaxSplit);
    REQUIRE((unsigned long long)p.grid_x * p.splitk * p.waves <= fg::kWsMailboxFlags);
    // every wave has a K unit; two, unless the whole problem is small (4 Mi weights or fewer)
    REQUIRE((K / 32) / (p.waves * p.splitk * p.unroll) >= ((unsigned long long)N * K <= (1ull << 22) ? 1 : 2));
  }
  if (p.kernel == FG_KERNEL_KN_MFMA) REQUIRE(p.waves == 4 || p.waves == 8);
  if (splitk == 0 && M <= 16) REQUIRE(p.splitk == 1 || p.fused != 0);  // up to 16 rows complete in the launch
  // the combination is instantiated: the launchers' own validator accepts it and changes nothing
  fg_plan_t q = p;
  REQUIRE(fg::plan_finish(M, N, K, &q) == FG_OK);
  REQUIRE(std::memcmp(&q, &p, sizeof(p)) == 0);
  switch (p.kernel) {
    case FG_KERNEL_NK_DOT2: REQUIRE(fg::nk_dot2_supported(p.m_block, p.tile_n, p.unroll)); break;
    case FG_KERNEL_NK_MFMA4: REQUIRE(fg::nk_mfma4_supported(p.m_block, p.tile_n, p.unroll)); break;
    case FG_KERNEL_KN_DOT2: REQUIRE(fg::kn_dot2_supported(p.m_block, p.unroll) && p.tile_n == 128); break;
    case FG_KERNEL_KN_MFMA: REQUIRE(fg::kn_mfma_supported(p.unroll) && p.tile_n == 128 && p.m_block == 16); break;
    case FG_KERNEL_NK_MFMA_R:
      REQUIRE(p.band == 128 || p.band == 256 || p.band == 512);
      REQUIRE(p.m_block == 16 || p.m_block == 32);
      break;
    default: REQUIRE(false);
  }
#undef REQUIRE
}

int main(int argc, char** argv) {
  const bool full = !(argc > 1 && std::strcmp(argv[1], "quick") == 0);
  std::vector<int> dims;
  for (int v = 128; v <= 8192; v += 128) dims.push_back(v);
  for (int v = 8704; v <= 32768; v += 512) dims.push_back(v);
  for (int v : {4224, 4992, 5504, 6912, 10752, 11008, 13824, 14336 + 128, 28672 + 128, 32768 - 128}) dims.push_back(v);
  std::vector<int> ms;
  for (int m = 1; m <= 17; ++m) ms.push_back(m);
  for (int m : {24, 31, 32, 33, 48, 64}) ms.push_back(m);
  const int splits_all[] = {0, 1, 2, 3, 5, 8, 16, 31, 32, 64};
  for (int cus : {256, 304, 64}) {  // the fitted part, a larger and a much smaller one
    fg::set_compute_units(cus);
    for (int layout = 0; layout <= 1; ++layout)
      for (int M : ms)
        for (size_t ni = 0; ni < dims.size(); ++ni)
          for (size_t ki = 0; ki < dims.size(); ++ki) {
            const int N = dims[ni], K = dims[ki];
            check(M, N, K, layout, 0);
            // forced splits on a thinner grid (every third size, all of them with `full`)
            if (full || (ni % 3 == 0 && ki % 3 == 0 && cus == 256))
              for (int s : splits_all)
                if (s) check(M, N, K, layout, s);
          }
    if (!full && cus != 256) continue;
  }
  // sizes at HIP's limits
  fg::set_compute_units(256);
  for (int layout = 0; layout <= 1; ++layout) {
    check(16 * 65535, 128, 128, layout, 0);
    check(1, 128 * 16384, 128, layout, 0);
    check(1, 128, 128 * 16384, layout, 0);
    check(16, 1 << 20, 1 << 10, layout, 64);
  }
  std::printf("%lld plans checked\n", checked);
  return 0;
}
