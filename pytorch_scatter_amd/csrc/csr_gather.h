// Expansion of per-row vectors to their edges (gather_csr) and the fused
// backward of segment_csr(mean), plus the index -> row-pointer conversion that
// lets segment_coo share the CSR reduction.
//
// Same merge-path tiling as the reduction: every worker gets the same number
// of (row loads + edge stores), so a hub row of 46 000 edges is written by
// many workers and a run of short rows keeps U independent row loads in
// flight. Stores are streaming 16-byte writes; `out` is never read.
#pragma once

#include "device_utils.h"
#include "merge_path.h"
#include "csr_reduce.h"

namespace ts {

struct CsrGatherArgs {
  const void *src;     // [B, N, K]
  const int64_t *indptr;
  void *out;           // [B, E, K]
  int64_t N, E, K;
  int64_t indptr_batch_stride;
  int G, BI, ipw;
  int64_t nblk;
};

// DIV: divide each row by T(max(row length, 1)) before expanding it
// (SegmentMeanCSR::backward, csrc/segment_csr.cpp:94-111).
template <typename T, int VEC, bool DIV>
__global__ __launch_bounds__(kBlock) void csr_gather_kernel(CsrGatherArgs a) {
  constexpr int U = 4;
  __shared__ int32_t s_ptr[kMaxBlockItems + 2];
  __shared__ int64_t s_cut[2];

  const int tid = threadIdx.x;
  const int G = a.G;
  const int w = tid / G;
  const int lg = tid - w * G;
  const int64_t col = (int64_t)blockIdx.y * (G * VEC) + (int64_t)lg * VEC;
  const bool col_ok = col < a.K;
  const int64_t b = blockIdx.z;

  const int64_t *ptr = a.indptr + b * a.indptr_batch_stride;
  const T *src_b = static_cast<const T *>(a.src) + b * a.N * a.K;
  T *out_b = static_cast<T *>(a.out) + b * a.E * a.K;

  const int64_t total = a.N + a.E;
  const int64_t d0 = (int64_t)blockIdx.x * a.BI;
  const int64_t d1 = d0 + a.BI < total ? d0 + a.BI : total;
  const int wave = tid / kWave;
  if (wave < 2) {
    const int64_t i = merge_search_wave(ptr, a.N, a.E, wave == 0 ? d0 : d1);
    if ((tid & (kWave - 1)) == 0) s_cut[wave] = i;
  }
  __syncthreads();
  const int64_t i0 = s_cut[0], i1 = s_cut[1];
  const int64_t j0 = d0 - i0;
  const int nr = (int)(i1 - i0);
  const int ne = (int)((d1 - i1) - j0);
  const int64_t last = i1 + 1 < a.N ? i1 + 1 : a.N;
  const int nload = (int)(last - i0) + 1;
  for (int t = tid; t < nload; t += kBlock) s_ptr[t] = (int32_t)(ptr[i0 + t] - j0);
  __syncthreads();

  const int ipw = a.ipw;
  const int tile_items = nr + ne;
  int dw0 = w * ipw;
  int dw1 = dw0 + ipw;
  dw0 = dw0 < tile_items ? dw0 : tile_items;
  dw1 = dw1 < tile_items ? dw1 : tile_items;
  const int ri0 = merge_search_lds(s_ptr, nr, ne, dw0);
  const int ri1 = merge_search_lds(s_ptr, nr, ne, dw1);
  const int je0 = dw0 - ri0;
  const int je1 = dw1 - ri1;
  if (je1 <= je0 || !col_ok) return;

  // rows ri0 .. ri1 can own edges of [je0, je1); rows past the last real row cannot
  int rlast = ri1;
  if (i0 + rlast >= a.N) rlast = (int)(a.N - 1 - i0);
  for (int rb = ri0; rb <= rlast; rb += U) {
    Vec<T, VEC> x[U];
#pragma unroll
    for (int u = 0; u < U; ++u) {
      const int r = rb + u <= rlast ? rb + u : rlast;
      x[u] = load_vec<T, VEC>(src_b + (i0 + r) * a.K + col);
    }
#pragma unroll
    for (int u = 0; u < U; ++u) {
      const int r = rb + u;
      if (r <= rlast) {
        const int32_t rs = s_ptr[r];
        const int32_t re = s_ptr[r + 1];
        const int s = rs > je0 ? rs : je0;
        const int t = re < je1 ? re : je1;
        if (t > s) {
          Vec<T, VEC> y = x[u];
          if (DIV) {
            const T c = count_as<T>((int64_t)re - (int64_t)rs);
#pragma unroll
            for (int v = 0; v < VEC; ++v) y.v[v] = div_elem<T>(y.v[v], c);
          }
          T *op = out_b + (j0 + s) * a.K + col;
          for (int e = s; e < t; ++e, op += a.K) store_vec<T, VEC>(op, y);  // plain stores: measured 4-8 % above streaming stores for pure write streams
        }
      }
    }
  }
}

// Narrow rows (at most 64 bytes per entry): one lane per 16 bytes of `out`. The
// workgroup first writes the row of every entry of its tile into LDS (a mark at
// each row start and a running maximum), so a lane looks its row up with one LDS
// read and the stores of a wavefront are one contiguous kilobyte whatever K is;
// the few source rows of a tile are re-read through the vector L1. Needs `out` 16-byte aligned for the vector stores
// (vec_ok), else every element is stored on its own.
// VROW: rows are whole 16-byte granules (K * sizeof(T) a multiple of 16, src and out aligned):
// a granule then lies in one row and is moved with one 16-byte load and store.
template <typename T, bool DIV, bool VROW>
__global__ __launch_bounds__(kBlock) void csr_gather_small_kernel(CsrGatherArgs a, int vec_ok) {
  constexpr int VE = kVecBytes / (int)sizeof(T);
  __shared__ int32_t s_ptr[kMaxBlockItems + 2];
  __shared__ int32_t s_row[VROW ? kMaxBlockItems : 1];  // local row of every entry of the tile (VROW)
  __shared__ int32_t s_wtot[kBlock / kWave];
  __shared__ int64_t s_cut[2];

  const int tid = threadIdx.x;
  const int K = (int)a.K;
  const int64_t b = blockIdx.z;
  const int64_t *ptr = a.indptr + b * a.indptr_batch_stride;
  const T *src_b = static_cast<const T *>(a.src) + b * a.N * a.K;
  T *out_b = static_cast<T *>(a.out) + b * a.E * a.K;

  const int64_t total = a.N + a.E;
  const int64_t d0 = (int64_t)blockIdx.x * a.BI;
  const int64_t d1 = d0 + a.BI < total ? d0 + a.BI : total;
  const int wave = tid / kWave;
  if (wave < 2) {
    const int64_t i = merge_search_wave(ptr, a.N, a.E, wave == 0 ? d0 : d1);
    if ((tid & (kWave - 1)) == 0) s_cut[wave] = i;
  }
  __syncthreads();
  const int64_t i0 = s_cut[0], i1 = s_cut[1];
  const int64_t j0 = d0 - i0;
  const int ne = (int)((d1 - i1) - j0);
  if (ne <= 0) return;
  const int64_t last = i1 + 1 < a.N ? i1 + 1 : a.N;
  const int nload = (int)(last - i0) + 1;  // ptr[i0 .. last]
  for (int t = tid; t < nload; t += kBlock) s_ptr[t] = (int32_t)(ptr[i0 + t] - j0);
  __syncthreads();
  const int rmax = nload - 2;  // last local row whose end is known; i0 + rmax <= N - 1
  if (rmax < 0) return;
  // entries in front of indptr[0] or behind indptr[N] belong to no row and are left as they are
  const int64_t w0 = ptr[0] - j0, w1 = ptr[a.N] - j0;
  const int e_lo = w0 < 0 ? 0 : (w0 > ne ? ne : (int)w0);
  const int e_hi = w1 < 0 ? 0 : (w1 > ne ? ne : (int)w1);
  if (e_hi <= e_lo) return;
  const int64_t fbase = j0 * K;  // element offset of the tile's first entry: entry numbers below are relative to it

  if (!VROW) {
    // Rows of 1-3 elements: a 16-byte granule of out covers several entries. Its first entry's row comes
    // from a binary search of the tile's row pointers (about ten LDS reads), the following entries
    // advance from there; no per-entry row table, no barriers.
    const int64_t f0 = (j0 + e_lo) * K, f1 = (j0 + e_hi) * K;
    const int64_t g0 = f0 / VE, g1 = (f1 + VE - 1) / VE;
    for (int64_t g = g0 + tid; g < g1; g += kBlock) {
      const int64_t fb = g * VE > f0 ? g * VE : f0;
      const int64_t fe = (g + 1) * VE < f1 ? (g + 1) * VE : f1;
      const unsigned rel = (unsigned)(fb - fbase);  // 32-bit arithmetic relative to the tile
      int e = (int)(rel / (unsigned)K);          // entry, relative to the tile
      int k = (int)(rel - (unsigned)e * (unsigned)K);
      int lo = 0, hi = rmax;  // the last row that starts at or before e (rows without entries share a start)
      while (lo < hi) {
        const int mid = (lo + hi + 1) >> 1;
        if (s_ptr[mid] <= e) lo = mid; else hi = mid - 1;
      }
      int row = lo;
      Vec<T, VE> y;
#pragma unroll
      for (int i = 0; i < VE; ++i) {
        if (fb + i < fe) {
          T v = src_b[(i0 + row) * a.K + k];
          if (DIV) v = div_elem<T>(v, count_as<T>((int64_t)s_ptr[row + 1] - (int64_t)s_ptr[row]));
          y.v[i] = v;
          if (++k == K) {
            k = 0;
            ++e;
            if (row < rmax && s_ptr[row + 1] <= e) {
              // the next row that has entries may lie thousands of rows on (the sparse end of a sorted index:
              // walking there a row at a time took 80 us for 20 k entries over 50 k rows): gallop, then bisect
              int lo = row + 1, hi = rmax + 1, step = 1;  // s_ptr[lo] <= e; hi: first row known to start behind e
              while (lo + step <= rmax) {
                if (s_ptr[lo + step] <= e) {
                  lo += step;
                  step <<= 1;
                } else {
                  hi = lo + step;
                  break;
                }
              }
              while (hi - lo > 1) {
                const int mid = (lo + hi) >> 1;
                if (s_ptr[mid] <= e) lo = mid; else hi = mid;
              }
              row = lo;
            }
          }
        }
      }
      if (vec_ok && fe - fb == VE) {
        store_vec<T, VE>(out_b + fb, y);
      } else {
#pragma unroll
        for (int i = 0; i < VE; ++i)
          if (fb + i < fe) out_b[fb + i] = y.v[i];
      }
    }
    return;
  }

  // ---- row of every entry of the tile: mark the first entry of each non-empty row, then a
  // running maximum over the entries (entries before the first mark belong to row 0)
  const int lane = tid & (kWave - 1);
  for (int e = tid; e < ne; e += kBlock) s_row[e] = 0;
  __syncthreads();
  for (int r = tid; r <= rmax; r += kBlock) {
    const int st = s_ptr[r];
    if (st >= 0 && st < ne && s_ptr[r + 1] > st) s_row[st] = r;
  }
  __syncthreads();
  {
    const int chunk = (ne + kBlock - 1) / kBlock;
    const int base = tid * chunk;
    int run = 0;
    for (int i = 0; i < chunk; ++i)
      if (base + i < ne) run = run > s_row[base + i] ? run : s_row[base + i];
    int incl = run;
#pragma unroll
    for (int d = 1; d < kWave; d <<= 1) {
      const int o = __shfl_up(incl, d);
      if (lane >= d) incl = incl > o ? incl : o;
    }
    if (lane == kWave - 1) s_wtot[wave] = incl;
    __syncthreads();
    int m = 0;
    for (int w2 = 0; w2 < wave; ++w2) m = m > s_wtot[w2] ? m : s_wtot[w2];
    const int up = lane_up1(incl);
    if (lane > 0) m = m > up ? m : up;
    for (int i = 0; i < chunk; ++i) {
      if (base + i < ne) {
        m = m > s_row[base + i] ? m : s_row[base + i];
        s_row[base + i] = m;
      }
    }
  }
  __syncthreads();

  // elements of out_b this tile owns, cut into 16-byte granules of the whole buffer
  const int64_t f0 = (j0 + e_lo) * K, f1 = (j0 + e_hi) * K;
  const int64_t g0 = f0 / VE, g1 = (f1 + VE - 1) / VE;
  const int64_t gbase = fbase / VE;  // rows are whole granules here
  if (VROW) {
    const int kv = K / VE;  // granules per row
    constexpr int U = 4;  // independent row loads in flight per lane
    for (int64_t gb = g0 + tid; gb < g1; gb += (int64_t)U * kBlock) {
      int row[U];
      Vec<T, VE> y[U];
#pragma unroll
      for (int u = 0; u < U; ++u) {
        const int64_t g = gb + (int64_t)u * kBlock < g1 ? gb + (int64_t)u * kBlock : gb;
        const unsigned gl = (unsigned)(g - gbase);  // 32-bit arithmetic relative to the tile
        const int e = (int)(gl / (unsigned)kv);
        const int c = (int)(gl - (unsigned)e * (unsigned)kv);
        row[u] = s_row[e];
        y[u] = load_vec<T, VE>(src_b + (i0 + row[u]) * a.K + c * VE);
      }
#pragma unroll
      for (int u = 0; u < U; ++u) {
        const int64_t g = gb + (int64_t)u * kBlock;
        if (g < g1) {
          if (DIV) {
            const T cnt = count_as<T>((int64_t)s_ptr[row[u] + 1] - (int64_t)s_ptr[row[u]]);
#pragma unroll
            for (int i = 0; i < VE; ++i) y[u].v[i] = div_elem<T>(y[u].v[i], cnt);
          }
          store_vec<T, VE>(out_b + g * VE, y[u]);
        }
      }
    }
    return;
  }
}

template <typename T>
int launch_csr_gather_small(const CsrGatherArgs &a, const CsrPlan &p, int64_t B, bool divide, hipStream_t stream) {
  dim3 grid((unsigned)p.nblk, 1, (unsigned)B);
  // every batch's slice of out starts on a 16-byte boundary
  const int vec_ok = (reinterpret_cast<uintptr_t>(a.out) & 15) == 0 &&
                     (B == 1 || (a.E * a.K * (int64_t)sizeof(T)) % 16 == 0);
  const bool vrow = p.vec > 1;  // the plan found whole 16-byte granules per row and aligned buffers
  if (divide) {
    if (vrow)
      hipLaunchKernelGGL((csr_gather_small_kernel<T, true, true>), grid, dim3(kBlock), 0, stream, a, vec_ok);
    else
      hipLaunchKernelGGL((csr_gather_small_kernel<T, true, false>), grid, dim3(kBlock), 0, stream, a, vec_ok);
  } else {
    if (vrow)
      hipLaunchKernelGGL((csr_gather_small_kernel<T, false, true>), grid, dim3(kBlock), 0, stream, a, vec_ok);
    else
      hipLaunchKernelGGL((csr_gather_small_kernel<T, false, false>), grid, dim3(kBlock), 0, stream, a, vec_ok);
  }
  return hipGetLastError() == hipSuccess ? TS_OK : TS_ERR_LAUNCH;
}

template <typename T, int VEC>
int launch_csr_gather_v(const CsrGatherArgs &a, const CsrPlan &p, int64_t B, bool divide,
                        hipStream_t stream) {
  dim3 grid((unsigned)p.nblk, (unsigned)p.ychunks, (unsigned)B);
  if (divide)
    hipLaunchKernelGGL((csr_gather_kernel<T, VEC, true>), grid, dim3(kBlock), 0, stream, a);
  else
    hipLaunchKernelGGL((csr_gather_kernel<T, VEC, false>), grid, dim3(kBlock), 0, stream, a);
  return hipGetLastError() == hipSuccess ? TS_OK : TS_ERR_LAUNCH;
}

template <typename T> int launch_csr_gather(const CsrGatherArgs &a, const CsrPlan &p, int64_t B,
                                            bool divide, hipStream_t stream);

#define TS_INSTANTIATE_CSR_GATHER(T, FULLVEC)                                               \
  template <> int launch_csr_gather<T>(const CsrGatherArgs &a, const CsrPlan &p, int64_t B, \
                                       bool divide, hipStream_t stream) {                   \
    if (p.small) return launch_csr_gather_small<T>(a, p, B, divide, stream);                \
    if (p.vec == FULLVEC) return launch_csr_gather_v<T, FULLVEC>(a, p, B, divide, stream);  \
    return launch_csr_gather_v<T, 1>(a, p, B, divide, stream);                              \
  }

// ---- sorted index -> row pointers -----------------------------------------
// ptr[r] = first position e with index[e] >= r, for r in [0, N]. Thread e owns
// the rows (index[e-1], index[e]]; thread E owns the rows after the last index.
// Values outside [0, N) are clamped so that a malformed index cannot make the
// reduction read or write out of bounds.
// entries per thread: 4 for a large index (a quarter of the wavefronts to launch), 1 below 2^20 entries, where the
// launch is cheap either way and the rows of a sparse stretch of the index then spread over four times as many
// wavefronts (20 k entries of a sorted Zipf index over 50 k rows: the last thousand entries own 45 k rows)
constexpr int kCooPtrPerThread = 4;
template <int PER>
static __global__ __launch_bounds__(kBlock) void coo_to_indptr_kernel(const int64_t *__restrict__ index,
                                                               int64_t *__restrict__ ptr, int64_t N,
                                                               int64_t E, int64_t index_batch_stride,
                                                               const int *gate = nullptr, int gate_want = 0) {
  // gate (optional): run only if (*gate != 0) == (gate_want != 0) -- a scatter that found its index sorted
  if (gate != nullptr && (*gate != 0) != (gate_want != 0)) return;
  __shared__ GapList s_gaps;
  if (threadIdx.x == 0) s_gaps.n = 0;
  __syncthreads();
  const int64_t b = blockIdx.y;
  const int64_t e0 = ((int64_t)blockIdx.x * kBlock + threadIdx.x) * PER;
  const int64_t *idx = index + b * index_batch_stride;
  int64_t *p = ptr + b * (N + 1);
  int64_t v[PER + 1];
  v[0] = e0 == 0 || e0 > E ? -1 : idx[e0 - 1];
#pragma unroll
  for (int i = 0; i < PER; ++i) v[i + 1] = e0 + i < E ? idx[e0 + i] : N;
#pragma unroll
  for (int i = 0; i < PER; ++i) {  // (no lane leaves early: the wavefront writes long ranges together)
    const int64_t e = e0 + i;
    int64_t lo = v[i] + 1;
    int64_t hi = e == E ? N : v[i + 1];
    if (lo < 0) lo = 0;
    if (hi > N) hi = N;
    if (e > E) hi = lo - 1;
    gap_rows(p, lo, hi, e, s_gaps);
  }
  __syncthreads();
  gap_rows_finish(p, s_gaps);
}

}  // namespace ts
