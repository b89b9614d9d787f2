// Segmented reduction over CSR row pointers for narrow rows (K <= 16 elements,
// at most 64 bytes per entry): attention scores, degrees, per-head scalars.
//
// With so few bytes per entry the wide kernel's lane groups would each chase
// their own cache line. Here a workgroup stages the entries of its merge-path
// tile in LDS with full 16-byte coalesced loads and then reduces from LDS:
// one lane per (row, column) for ordinary rows, one wavefront per row for rows
// with more than 64 entries inside the tile (64 lanes stride over the entries,
// then a shuffle tree). Tiles, the workspace for rows that cross tiles and the
// second kernel that combines them are those of the wide kernel. Results do not
// depend on scheduling: no atomics.
//
// Semantics as in csr_reduce.h (csrc/cpu/segment_csr_cpu.cpp:54-88): strict
// compare so the first index wins ties, mean = T(sum) / T(count), empty row -> 0
// with arg = E.
#pragma once

#include "csr_reduce.h"

namespace ts {

constexpr int kSmallLongRow = 64;  // more entries than this inside a tile: one wavefront per row

// LDS layout of a tile, in 16-byte units
__host__ __device__ inline int csr_small_ptr_vecs(int BI) { return (BI + 2 + 3) / 4; }
inline size_t csr_small_lds_bytes(int BI, int64_t K, int elem_bytes) {
  return (size_t)csr_small_ptr_vecs(BI) * 16 + (((size_t)BI * K * elem_bytes + 15) / 16 + 1) * 16;
}

template <typename T, int REDUCE>
__global__ __launch_bounds__(kBlock) void csr_reduce_small_kernel(CsrReduceArgs a) {
  typedef typename Acc<T>::type A;
  typedef uint32_t u4 __attribute__((ext_vector_type(4)));
  constexpr bool kArg = (REDUCE == TS_MIN || REDUCE == TS_MAX);

  // dynamic LDS, sized by the tile: [row pointers: BI + 2, padded to 16 bytes][entries: BI * K elements + 16 bytes]
  extern __shared__ u4 s_dyn[];
  int32_t *s_ptr = reinterpret_cast<int32_t *>(s_dyn);
  u4 *s_raw = s_dyn + csr_small_ptr_vecs(a.BI);
  __shared__ int32_t s_long[kMaxBlockItems / kSmallLongRow + 2];
  __shared__ int32_t s_nlong;
  __shared__ int64_t s_cut[2];

  const int tid = threadIdx.x;
  const int K = (int)a.K;
  const int64_t b = blockIdx.z;
  const int64_t *ptr = a.indptr + b * a.indptr_batch_stride;
  const T *src_b = static_cast<const T *>(a.src) + b * a.E * a.K;
  T *out_b = static_cast<T *>(a.out) + b * a.N * a.K;
  int64_t *arg_b = kArg ? a.arg_out + b * a.N * a.K : nullptr;
  T *count_b = a.count_out ? static_cast<T *>(a.count_out) + b * a.N : nullptr;

  // ---- tile cut: two wavefronts search the two diagonals concurrently
  const int64_t total = a.N + a.E;
  const int64_t d0 = (int64_t)blockIdx.x * a.BI;
  const int64_t d1 = d0 + a.BI < total ? d0 + a.BI : total;
  const int wave = tid / kWave;
  const int lane = tid & (kWave - 1);
  if (wave < 2) {
    const int64_t i = merge_search_wave(ptr, a.N, a.E, wave == 0 ? d0 : d1);
    if (lane == 0) s_cut[wave] = i;
  }
  if (tid == 0) s_nlong = 0;
  if (a.status_reset && a.status != nullptr && tid == 0 && (blockIdx.x | blockIdx.z) == 0)
    __hip_atomic_exchange(a.status, (unsigned long long)a.status_nonce, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);  // this kernel never waits
  __syncthreads();
  const int64_t i0 = s_cut[0], i1 = s_cut[1];
  const int64_t j0 = d0 - i0;
  const int nr = (int)(i1 - i0);         // row ends inside the tile
  const int ne = (int)((d1 - i1) - j0);  // entries inside the tile

  // ---- row pointers, relative to the tile's first entry, and the entries themselves
  const int64_t last = i1 + 1 < a.N ? i1 + 1 : a.N;
  const int nload = (int)(last - i0) + 1;  // ptr[i0 .. last]
  for (int t = tid; t < nload; t += kBlock) s_ptr[t] = (int32_t)(ptr[i0 + t] - j0);
  // whole 16-byte granules around the tile's entries: a granule never crosses a page,
  // so the bytes before the first and after the last entry are safe to read
  const T *p_first = src_b + j0 * K;
  const int shift = ne > 0 ? (int)((reinterpret_cast<uintptr_t>(p_first) & 15) / sizeof(T)) : 0;
  const int nvec = ne > 0 ? (int)(((size_t)(shift + ne * K) * sizeof(T) + 15) / 16) : 0;
  const u4 *p0 = reinterpret_cast<const u4 *>(p_first - shift);
  for (int t = tid; t < nvec; t += kBlock) s_raw[t] = __builtin_nontemporal_load(p0 + t);
  __syncthreads();
  const T *s_src = reinterpret_cast<const T *>(s_raw) + shift;

  // ---- which rows the tile sees
  const bool has_open_row = i1 < a.N;                 // the row after the last row end
  const bool head_exists = i0 < a.N && s_ptr[0] < 0;  // row i0 began in an earlier tile
  const int nrows = nr + (has_open_row ? 1 : 0);
  enum { kComplete = 0, kHead = 1, kTail = 2, kNone = 3 };
  auto classify = [&](int r, int &lo, int &hi) -> int {
    const bool open = r == nr;
    lo = s_ptr[r] > 0 ? s_ptr[r] : 0;
    hi = open ? ne : s_ptr[r + 1];
    if (r == 0 && head_exists) return kHead;
    if (open) return hi > lo ? kTail : kNone;
    return kComplete;
  };

  A *ws_val_blk = static_cast<A *>(a.ws_vals) + ((b * a.nblk + blockIdx.x) * 2) * a.K;
  int32_t *ws_arg_blk = kArg ? a.ws_args + ((b * a.nblk + blockIdx.x) * 2) * a.K : nullptr;
  auto deliver = [&](int r, int k, int kind, A acc, int32_t arg) {
    if (kind == kComplete) {
      finalize_row<T, 1, REDUCE>(a, out_b, arg_b, count_b, i0 + r, k, k, &acc, &arg,
                                 (int64_t)s_ptr[r + 1] - (int64_t)s_ptr[r], true);
    } else if (kind == kHead) {
      ws_val_blk[k] = acc;
      if (kArg) ws_arg_blk[k] = arg;
    } else if (kind == kTail) {
      ws_val_blk[a.K + k] = acc;
      if (kArg) ws_arg_blk[a.K + k] = arg;
    }
  };

  // ---- one lane per (row, column); long rows are left to whole wavefronts
  const int n_units = nrows * K;
  for (int u = tid; u < n_units; u += kBlock) {
    const int r = u / K;
    const int k = u - r * K;
    int lo, hi;
    const int kind = classify(r, lo, hi);
    if (kind == kNone) continue;
    if (hi - lo > kSmallLongRow) {
      if (k == 0) s_long[atomicAdd(&s_nlong, 1)] = r;
      continue;
    }
    A acc = acc_init<A, REDUCE>();
    int32_t arg = 0;
    const T *q = s_src + lo * K + k;
    for (int e = lo; e < hi; ++e, q += K) reduce_step<A, REDUCE>(acc, arg, to_acc<T>(*q), (int32_t)(j0 + e));
    deliver(r, k, kind, acc, arg);
  }
  __syncthreads();

  // ---- long rows: the lanes of a wavefront stride over the entries, then a shuffle tree
  const int nlong = s_nlong;
  for (int qi = wave; qi < nlong; qi += kBlock / kWave) {
    const int r = s_long[qi];
    int lo, hi;
    const int kind = classify(r, lo, hi);
    for (int k = 0; k < K; ++k) {
      A acc = acc_init<A, REDUCE>();
      int32_t arg = 0;
      for (int e = lo + lane; e < hi; e += kWave)
        reduce_step<A, REDUCE>(acc, arg, to_acc<T>(s_src[e * K + k]), (int32_t)(j0 + e));
      auto tree_step = [&](A oacc, int32_t oarg) {
        if (REDUCE == TS_SUM || REDUCE == TS_MEAN) {
          acc = acc + oacc;
        } else {
          // equal values: the smaller position wins, as in a walk in entry order
          const bool better = (REDUCE == TS_MIN ? oacc < acc : oacc > acc) || (oacc == acc && oarg < arg);
          if (better) { acc = oacc; arg = oarg; }
        }
      };
      // lane i takes lane i + 32, 16, ... 1 (row shifts and row / half swaps in the vector ALU): lane 0 ends with
      // the row's result
      tree_step(lane_down_any<32>(acc), lane_down<32>(arg));
      tree_step(lane_down_any<16>(acc), lane_down<16>(arg));
      tree_step(lane_down_any<8>(acc), lane_down<8>(arg));
      tree_step(lane_down_any<4>(acc), lane_down<4>(arg));
      tree_step(lane_down_any<2>(acc), lane_down<2>(arg));
      tree_step(lane_down_any<1>(acc), lane_down<1>(arg));
      if (lane == 0) deliver(r, k, kind, acc, arg);
    }
  }

  // ---- what the second kernel needs to know about this tile
  if (tid == 0 && blockIdx.y == 0) {
    int64_t *meta = a.ws_meta + (b * a.nblk + blockIdx.x) * 4;
    int lo, hi;
    const bool tail = has_open_row && classify(nr, lo, hi) == kTail;
    meta[2] = tail ? i0 + nr : -1;
    if (tail) {
      meta[3] = (int64_t)s_ptr[nr + 1] - (int64_t)s_ptr[nr];  // full length of the open row
      // the tile in which it ends: its row-end item sits at merge position row + indptr[row + 1]
      meta[0] = ((i0 + nr) + ((int64_t)s_ptr[nr + 1] + j0)) / a.BI;
    }
  }
}

// Second kernel of the narrow-row reduction: rows that cross tiles. A group of G lanes (one lane per
// column, 64 / G groups per wavefront) serves one tile that opened such a row; nearly always the row
// ends in the next tile and everything that needs is requested at once. A hub row, however, passes
// through hundreds of these small tiles. Its chain is not walked by one group: the tile in which the
// row ends is known (the first kernel derives it from the row pointer), so the wavefront's groups take
// every (64 / G)-th tile of the chain, several loads in flight each, and a shuffle tree combines them.
// The order of the combination is fixed by the tiling (for min / max ties go to the smaller
// position), so the result does not depend on timing.
template <typename T, int REDUCE>
__global__ __launch_bounds__(kBlock) void csr_reduce_fixup_wave_kernel(CsrReduceArgs a) {
  typedef typename Acc<T>::type A;
  constexpr bool kArg = (REDUCE == TS_MIN || REDUCE == TS_MAX);
  constexpr int PF = 8;
  const int G = a.G;  // power of two, at most 16
  const int S = kWave / G;
  const int lane = threadIdx.x & (kWave - 1);
  const int j = lane / G;
  const int lg = lane - j * G;
  const bool col_ok = lg < a.K;
  const int64_t c = col_ok ? lg : 0;
  const int64_t b = blockIdx.z;
  const int64_t wave = (int64_t)blockIdx.x * (kBlock / kWave) + threadIdx.x / kWave;
  const int64_t t = wave * S + j;
  const bool valid = t < a.nblk;
  const int64_t tc = valid ? t : a.nblk - 1;
  const int64_t *meta = a.ws_meta + (b * a.nblk) * 4;
  const A *vals = static_cast<const A *>(a.ws_vals) + (b * a.nblk) * 2 * a.K;
  const int32_t *args = kArg ? a.ws_args + (b * a.nblk) * 2 * a.K : nullptr;

  // a chain of more than kLongChain tiles (one row that holds most of a large input: 4 M entries of 16 floats in
  // one row pass through 15 k tiles, 220 us for one wavefront) is shared by the wavefronts of the workgroup; the
  // tiles of a workgroup number fewer than that, so at most one such chain begins in them
  constexpr int kLongChain = 512;
  constexpr int WV = kBlock / kWave;
  __shared__ long long s_chain[3];  // t, last, first thread of the group that owns the row
  __shared__ int s_nchain;
  __shared__ A s_pv[WV][16];
  __shared__ int32_t s_pa[WV][16];
  if (threadIdx.x == 0) s_nchain = 0;
  __syncthreads();

  auto absorb = [&](A &x, int32_t &xa, A y, int32_t ya) {
    if (kArg) {
      const bool better = (REDUCE == TS_MIN ? y < x : y > x) || (y == x && ya < xa);
      if (better) { x = y; xa = ya; }
    } else {
      x = x + y;
    }
  };

  // everything the usual case needs is requested at once
  const int64_t row = meta[tc * 4 + 2];
  const int64_t count = meta[tc * 4 + 3];
  int64_t last = meta[tc * 4 + 0];  // the tile in which the row ends, left by the tile that opened it
  const int64_t tn = tc + 1 < a.nblk ? tc + 1 : tc;
  A acc = vals[(tc * 2 + 1) * a.K + c];
  int32_t arg = kArg ? args[(tc * 2 + 1) * a.K + c] : 0;
  const A next_val = vals[(tn * 2) * a.K + c];
  const int32_t next_arg = kArg ? args[(tn * 2) * a.K + c] : 0;
  const bool has = valid && row >= 0;
  if (!has || last >= a.nblk) last = has ? a.nblk - 1 : tc;
  if (has && last > t) absorb(acc, arg, next_val, next_arg);

  bool shared_chain = false;
  if (has && last - t - 1 > kLongChain && lg == 0 && atomicAdd(&s_nchain, 1) == 0) {
    s_chain[0] = t;
    s_chain[1] = last;
    s_chain[2] = threadIdx.x;
    shared_chain = true;
  }
  // chains that go on beyond the next tile: the whole wavefront works on one at a time
  uint64_t pending = __ballot(has && last > t + 1 && lg == 0 && !shared_chain);
  while (pending != 0) {
    const int leader = __ffsll((unsigned long long)pending) - 1;
    pending &= pending - 1;
    const int64_t t_s = __shfl(t, leader);
    const int64_t last_s = __shfl(last, leader);
    A part = acc_init<A, REDUCE>();
    int32_t part_arg = 0x7FFFFFFF;
    for (int64_t t0 = t_s + 2 + j; t0 <= last_s; t0 += (int64_t)S * PF) {
      A hv[PF];
      int32_t ha[PF];
#pragma unroll
      for (int q = 0; q < PF; ++q) {
        const int64_t tt = t0 + (int64_t)q * S <= last_s ? t0 + (int64_t)q * S : last_s;
        hv[q] = vals[(tt * 2) * a.K + c];
        ha[q] = kArg ? args[(tt * 2) * a.K + c] : 0;
      }
#pragma unroll
      for (int q = 0; q < PF; ++q) {
        if (t0 + (int64_t)q * S <= last_s) absorb(part, part_arg, hv[q], ha[q]);
      }
    }
    for (int off = S / 2; off >= 1; off >>= 1) {
      const A o = __shfl_down(part, off * G);
      const int32_t oa = __shfl_down(part_arg, off * G);
      absorb(part, part_arg, o, oa);
    }
    // group 0 holds the chain's total: hand it to the group that owns the row
    const A total = __shfl(part, lg);
    const int32_t total_arg = __shfl(part_arg, lg);
    if (j == leader / G) absorb(acc, arg, total, total_arg);
  }
  __syncthreads();
  if (s_nchain > 0) {  // uniform: the long chain, every wavefront a share of its tiles
    const int64_t t_s = s_chain[0], last_s = s_chain[1];
    const int owner = (int)s_chain[2];
    const int wv = threadIdx.x / kWave;
    A part = acc_init<A, REDUCE>();
    int32_t part_arg = 0x7FFFFFFF;
    const int64_t stride = (int64_t)WV * S;
    for (int64_t t0 = t_s + 2 + wv * S + j; t0 <= last_s; t0 += stride * PF) {
      A hv[PF];
      int32_t ha[PF];
#pragma unroll
      for (int q = 0; q < PF; ++q) {
        const int64_t tt = t0 + (int64_t)q * stride <= last_s ? t0 + (int64_t)q * stride : last_s;
        hv[q] = vals[(tt * 2) * a.K + c];
        ha[q] = kArg ? args[(tt * 2) * a.K + c] : 0;
      }
#pragma unroll
      for (int q = 0; q < PF; ++q) {
        if (t0 + (int64_t)q * stride <= last_s) absorb(part, part_arg, hv[q], ha[q]);
      }
    }
    for (int off = S / 2; off >= 1; off >>= 1) {
      const A o = __shfl_down(part, off * G);
      const int32_t oa = __shfl_down(part_arg, off * G);
      absorb(part, part_arg, o, oa);
    }
    if (j == 0) {
      s_pv[wv][lg] = part;
      s_pa[wv][lg] = part_arg;
    }
    __syncthreads();
    if ((int)threadIdx.x >= owner && (int)threadIdx.x < owner + G) {
      for (int w2 = 0; w2 < WV; ++w2) absorb(acc, arg, s_pv[w2][lg], s_pa[w2][lg]);
    }
  }
  if (has) {
    T *out_b = static_cast<T *>(a.out) + b * a.N * a.K;
    int64_t *arg_b = kArg ? a.arg_out + b * a.N * a.K : nullptr;
    T *count_b = a.count_out ? static_cast<T *>(a.count_out) + b * a.N : nullptr;
    finalize_row<T, 1, REDUCE>(a, out_b, arg_b, count_b, row, lg, lg, &acc, &arg, count, col_ok);
  }
}

template <typename T, int REDUCE>
int launch_csr_reduce_small_t(const CsrReduceArgs &a, const CsrPlan &p, int64_t B, hipStream_t stream) {
  dim3 grid((unsigned)p.nblk, 1, (unsigned)B);
  hipLaunchKernelGGL((csr_reduce_small_kernel<T, REDUCE>), grid, dim3(kBlock),
                     csr_small_lds_bytes(p.BI, a.K, (int)sizeof(T)), stream, a);
  if (p.nblk > 1) {  // a single tile has no rows that cross tiles
    const int W = (kBlock / kWave) * (kWave / p.G);  // tiles per workgroup
    dim3 grid2((unsigned)((p.nblk + W - 1) / W), 1, (unsigned)B);
    hipLaunchKernelGGL((csr_reduce_fixup_wave_kernel<T, REDUCE>), grid2, dim3(kBlock), 0, stream, a);
  }
  return hipGetLastError() == hipSuccess ? TS_OK : TS_ERR_LAUNCH;
}

template <typename T>
int launch_csr_reduce_small(const CsrReduceArgs &a, const CsrPlan &p, int64_t B, int reduce, hipStream_t stream) {
  switch (reduce) {
  case TS_SUM: return launch_csr_reduce_small_t<T, TS_SUM>(a, p, B, stream);
  case TS_MEAN: return launch_csr_reduce_small_t<T, TS_MEAN>(a, p, B, stream);
  case TS_MIN: return launch_csr_reduce_small_t<T, TS_MIN>(a, p, B, stream);
  case TS_MAX: return launch_csr_reduce_small_t<T, TS_MAX>(a, p, B, stream);
  default: return TS_ERR_UNSUPPORTED;
  }
}

}  // namespace ts
