// What the kernels of the per-tile lists share: the record the counting sort by tile leaves for every instance
// and the last step of every per-tile sort.
#pragma once

#include "gs_common.h"

namespace gs {

// One (Gaussian, tile) instance as the scatter writes it into its tile's segment, with one 16-byte store:
// x = Gaussian, y = emission index (its place in the order duplicateWithKeys emits instances,
// cuda_rasterizer/rasterizer_impl.cu:74-117), z = bits of the view-space depth, w = 0.
typedef uint4 TileRecord;

// The per-tile sorts order a tile's instances by (depth bits, place in the unsorted segment), or by the leading
// bits of the depth only: (depth bits - lo) >> shift.  The reference's order is (depth bits, emission index) (a
// stable sort of instances emitted in that order, rasterizer_impl.cu:675-684), which differs only inside runs of
// entries with the same sorted-on depth field.  This writes entry i of a sorted list of n entries to its final
// place: sorted[q] = (depth bits << 32 | emission index) for every q < n; an entry that has a neighbour with its
// depth field looks its run up and takes the place that (depth bits, emission index) has in it (emission indices
// are distinct).  Runs are rare and short in real views; a run of L entries costs L reads per entry.
template <typename SortedArray>
__device__ __forceinline__ void emit_list_entry(uint32_t tile, uint32_t start, uint32_t n, uint32_t i,
                                                uint32_t gaussian, const SortedArray& sorted,
                                                uint64_t* __restrict__ keys, uint32_t* __restrict__ emission,
                                                uint32_t* __restrict__ point_list, uint32_t lo = 0u,
                                                uint32_t shift = 0u) {
  const uint64_t me = sorted(i);
  const uint32_t depth_bits = (uint32_t)(me >> 32), e = (uint32_t)me;
  const auto field = [&](uint64_t x) { return ((uint32_t)(x >> 32) - lo) >> shift; };
  const uint32_t mine = field(me);
  uint32_t pos = i;
  const bool tie = (i > 0u && field(sorted(i - 1u)) == mine) || (i + 1u < n && field(sorted(i + 1u)) == mine);
  if (tie) {
    uint32_t s = i;
    while (s > 0u && field(sorted(s - 1u)) == mine) s--;
    uint32_t below = 0;
    for (uint32_t q = s; q < n; q++) {
      const uint64_t other = sorted(q);
      if (field(other) != mine) break;
      below += other < me ? 1u : 0u;
    }
    pos = s + below;
  }
  keys[start + pos] = ((uint64_t)tile << 32) | (uint64_t)depth_bits;
  emission[start + pos] = e;
  point_list[start + pos] = gaussian;
}

}  // namespace gs
