// Measurement-only instances of the direct-to-LDS matmul kernel (csrc/kernels/matmul_dma_kernel.h):
// the same K loop with parts of its operand feed left out or redirected, so that what remains can
// be timed on its own.  None of them computes anything meaningful; the kernel library never
// instantiates them.
#pragma once

#include "../kernels/matmul_dma_kernel.h"

namespace afir {
namespace dma {

// no global -> LDS loads in the K loop after the ring fill: MFMAs, LDS operand reads, waits, barriers
struct NoLoads : FullFeed {
  static constexpr bool kLoads = false;
};
// ... and no LDS operand reads either: MFMAs, waits and barriers only
struct NoLoadsNoReads : FullFeed {
  static constexpr bool kLoads = false;
  static constexpr bool kOperandReads = false;
};
// every load reads the same 1 KiB: the cost of issuing the loads and writing LDS, without the
// memory system behind them
struct LoadsOfOneKiB : FullFeed {
  __device__ static void source(const char *&base, uint32_t &lane_offset, const void *a, int lane) {
    base = static_cast<const char *>(a);
    lane_offset = (uint32_t)lane * 16u;
  }
};
// real addresses, but the walk over K wraps after 8 stages (256 k): the operand panels of the
// 32 tiles an XCD works on together are then 1.5 MiB and stay in its 4 MiB L2, so that every
// load but the first few is an L2 hit.  What separates this from the full kernel is the cost
// of the L2 misses; what separates it from LoadsOfOneKiB is the cost of the L2 hits.
struct L2Resident : FullFeed {
  static constexpr int kWrapStages = 8;
};

}  // namespace dma
}  // namespace afir
