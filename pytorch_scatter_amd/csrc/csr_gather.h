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
    if (p.vec == FULLVEC) return launch_csr_gather_v<T, FULLVEC>(a, p, B, divide, stream);  \
    return launch_csr_gather_v<T, 1>(a, p, B, divide, stream);                              \
  }

// ---- sorted index -> row pointers -----------------------------------------
// ptr[r] = first position e with index[e] >= r, for r in [0, N]. Thread e owns
// the rows (index[e-1], index[e]]; thread E owns the rows after the last index.
// Values outside [0, N) are clamped so that a malformed index cannot make the
// reduction read or write out of bounds.
static __global__ __launch_bounds__(kBlock) void coo_to_indptr_kernel(const int64_t *__restrict__ index,
                                                               int64_t *__restrict__ ptr, int64_t N,
                                                               int64_t E, int64_t index_batch_stride) {
  const int64_t b = blockIdx.y;
  const int64_t e = (int64_t)blockIdx.x * kBlock + threadIdx.x;
  if (e > E) return;
  const int64_t *idx = index + b * index_batch_stride;
  int64_t *p = ptr + b * (N + 1);
  int64_t lo = e == 0 ? 0 : idx[e - 1] + 1;
  int64_t hi = e == E ? N : idx[e];
  if (lo < 0) lo = 0;
  if (hi > N) hi = N;
  for (int64_t r = lo; r <= hi; ++r) p[r] = e;
}

}  // namespace ts
