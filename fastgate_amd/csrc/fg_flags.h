// Flag word handed to every GEMM kernel (host and device code share these).
#pragma once
#include "../../include/fastgate.h"

namespace fg {
constexpr int kFlagAccumulate = 1;    // C += A*W
constexpr int kFlagStagger = 2;       // start step = workgroup id % steps ([N,K] kernels)
constexpr int kFlagFixSplit = 8;      // split-K completes through one fixed-point atomic per element
constexpr int kFlagXcdLocal = 256;    // [K,N] MFMA kernel: the workgroups of a tile share one XCD and
                                      // exchange their partials through its L2, signalled by flags
constexpr int kFlagPretendForeign = 512;  // test hook of that order: some workgroups report that they
                                          // run on another XCD than their tile's, which sends the
                                          // completing workgroup down the recomputing path
constexpr int kFlagBias = 16;         // add bias[n] to the finished sum
constexpr int kFlagActShift = 5;      // bits 5-7: FG_ACT_*
constexpr int kFlagTailMask = 0xF0;   // any bias or activation work at all
// Split-K workspace header (zero between calls): arrival counters of the counter protocol, then
// one 64-bit accumulator word and one 32-bit class word per output element of the atomic protocol.
constexpr unsigned long kWsCounterBytes = 65536;
constexpr unsigned long kWsAccElems = 262144;  // M * N the atomic protocol can take
constexpr int kFixMaxSplit = 31;              // arrivals an accumulator word can count
// ... then the flag words of the mailbox completion: one 64-bit word per wave of every partner
// workgroup.  They hold launch tags that no later launch repeats, so they are never cleared.
constexpr unsigned long kWsMailboxFlags = 65536;
constexpr unsigned long kWsMailboxFlagsOffset = kWsCounterBytes + kWsAccElems * 12;
constexpr int kMailboxMaxSplit = 32;          // partners the owner's ready mask can hold, plus itself
constexpr unsigned long kWsHeaderBytes = kWsMailboxFlagsOffset + kWsMailboxFlags * 8;
}  // namespace fg
