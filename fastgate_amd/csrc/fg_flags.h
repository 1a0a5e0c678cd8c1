// Flag word handed to every GEMM kernel (host and device code share these).
#pragma once
#include "../../include/fastgate.h"

namespace fg {
constexpr int kFlagAccumulate = 1;    // C += A*W
constexpr int kFlagStagger = 2;       // start step = workgroup id % steps ([N,K] kernels)
constexpr int kFlagBias = 16;         // add bias[n] to the finished sum
constexpr int kFlagActShift = 5;      // bits 5-7: FG_ACT_*
constexpr int kFlagTailMask = 0xF0;   // any bias or activation work at all
}  // namespace fg
