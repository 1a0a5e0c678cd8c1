// Flag word handed to every GEMM kernel (host and device code share these).
#pragma once
#include "../../include/fastgate.h"

namespace fg {
constexpr int kFlagAccumulate = 1;    // C += A*W
constexpr int kFlagStagger = 2;       // start step = workgroup id % steps ([N,K] kernels)
constexpr int kFlagFixSplit = 8;      // split-K completes through one fixed-point atomic per element
constexpr int kFlagBias = 16;         // add bias[n] to the finished sum
constexpr int kFlagActShift = 5;      // bits 5-7: FG_ACT_*
constexpr int kFlagTailMask = 0xF0;   // any bias or activation work at all
// Split-K workspace header (zero between calls): arrival counters of the counter protocol, then
// one 64-bit accumulator word and one 32-bit class word per output element of the atomic protocol.
constexpr unsigned long kWsCounterBytes = 65536;
constexpr unsigned long kWsAccElems = 262144;  // M * N the atomic protocol can take
constexpr int kFixMaxSplit = 31;              // arrivals an accumulator word can count
constexpr unsigned long kWsHeaderBytes = kWsCounterBytes + kWsAccElems * 12;
}  // namespace fg
