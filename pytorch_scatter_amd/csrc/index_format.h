// Index formats either side of the reductions: sorted index <-> row pointers, and the one-time
// stable sort of an unsorted index (row numbers perm + row pointers) after which a scatter runs
// as a segmented reduction over permuted rows.
#pragma once

#include "device_utils.h"

namespace ts {

// sort key of an entry: its index, or N for an index outside [0, N) (sorted behind the last row)
static __global__ __launch_bounds__(kBlock) void index_keys_kernel(const int64_t *__restrict__ index,
                                                                 uint32_t *__restrict__ keys, int64_t E, int64_t N) {
  for (int64_t e = (int64_t)blockIdx.x * kBlock + threadIdx.x; e < E; e += (int64_t)gridDim.x * kBlock) {
    const int64_t v = index[e];
    keys[e] = (v >= 0 && v < N) ? (uint32_t)v : (uint32_t)N;
  }
}

// ptr[r] = first position e with keys[e] >= r, for r in [0, N]; thread e owns the rows
// (keys[e-1], keys[e]], thread E the rows after the last key
static __global__ __launch_bounds__(kBlock) void keys_to_indptr_kernel(const uint32_t *__restrict__ keys,
                                                                     int64_t *__restrict__ ptr, int64_t N, int64_t E) {
  __shared__ GapList s_gaps;
  if (threadIdx.x == 0) s_gaps.n = 0;
  __syncthreads();
  const int64_t e = (int64_t)blockIdx.x * kBlock + threadIdx.x;
  int64_t lo = e == 0 || e > E ? 0 : (int64_t)keys[e - 1] + 1;
  int64_t hi = e >= E ? N : (int64_t)keys[e];
  if (hi > N) hi = N;
  if (e > E) hi = lo - 1;
  gap_rows(ptr, lo, hi, e, s_gaps);  // (no lane leaves early: the wavefront writes long ranges together)
  __syncthreads();
  gap_rows_finish(ptr, s_gaps);
}

static __global__ __launch_bounds__(kBlock) void row_numbers_kernel(int64_t *__restrict__ p, int64_t total, int64_t N) {
  for (int64_t i = (int64_t)blockIdx.x * kBlock + threadIdx.x; i < total; i += (int64_t)gridDim.x * kBlock) p[i] = i % N;
}

inline unsigned index_grid(int64_t n) {
  int64_t g = (n + kBlock - 1) / kBlock;
  if (g > 65535 * 16) g = 65535 * 16;
  return (unsigned)(g < 1 ? 1 : g);
}

// Stable radix sort of 32-bit keys (bits [0, end_bit)) that returns the sorted keys and, as perm, the
// original position of every sorted entry. Defined in index_sort.hip on top of rocPRIM's device-wide
// radix sort (the one library primitive of this library: a one-time set-up step, not a reduction).
size_t sort_keys_temp_bytes(int64_t n, int end_bit);
int sort_keys_to_perm(void *temp, size_t temp_bytes, const uint32_t *keys_in, uint32_t *keys_out, int32_t *perm,
                      int64_t n, int end_bit, hipStream_t s);

}  // namespace ts
