// Merge-path partitioning of a CSR row-pointer array.
//
// A segmented reduction over CSR has two kinds of work items: the E edges and
// the N row ends. Walking both lists in merged order (a row end is taken as
// soon as all of its edges are consumed) and cutting that walk into equal
// pieces gives every workgroup, and every lane group inside it, the same
// number of items whatever the degree distribution: a 46 000-edge row is
// spread over many tiles, a run of empty rows costs one item each.
//
// The cut on diagonal d is the pair (i, j), i + j = d, where
//   i = #{ r in [0, N) : indptr[r + 1] + r + 1 <= d }
// is the number of row ends taken and j the number of edges taken.
#pragma once

#include "device_utils.h"

namespace ts {

// 64-ary search of one diagonal by a whole wavefront: every step probes 64
// evenly spaced rows at once, so 2.4 M rows need 4 dependent global loads
// instead of the 22 of a binary search. `ptr` is the batch's indptr (N + 1
// entries). All lanes must call; the result is wave-uniform.
__device__ __forceinline__ int64_t merge_search_wave(const int64_t *__restrict__ ptr,
                                                     int64_t N, int64_t E, int64_t d) {
  const int lane = threadIdx.x & (kWave - 1);
  int64_t lo = d > E ? d - E : 0;
  int64_t hi = d < N ? d : N;
  while (hi > lo) {
    const int64_t span = hi - lo;
    const int64_t step = (span + kWave - 1) / kWave;
    const int64_t p = lo + (int64_t)(lane + 1) * step - 1;
    bool taken = false;
    if (p < hi) taken = (ptr[p + 1] + p + 1 <= d);
    const int c = __popcll(__ballot(taken));
    const int64_t nvalid = span / step;  // probes that fell inside [lo, hi)
    if (c >= nvalid) {
      lo = lo + nvalid * step;
    } else {
      hi = lo + (int64_t)(c + 1) * step - 1;
      lo = lo + (int64_t)c * step;
    }
  }
  return lo;
}

// Binary search of a diagonal inside a tile whose row pointers sit in LDS as
// offsets relative to the tile's first edge. nr rows end inside the tile, ne
// edges lie inside it.
__device__ __forceinline__ int merge_search_lds(const int32_t *s_ptr, int nr, int ne, int d) {
  int lo = d > ne ? d - ne : 0;
  int hi = d < nr ? d : nr;
  while (lo < hi) {
    const int mid = (lo + hi) >> 1;
    if (s_ptr[mid + 1] + mid + 1 <= d)
      lo = mid + 1;
    else
      hi = mid;
  }
  return lo;
}

}  // namespace ts
