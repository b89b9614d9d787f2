// out[b, e, :] = src[b, index[b, e], :]   (gather_coo) and the fused backward
// of segment_coo(mean), which divides the gathered row by count[index].
//
// Edges are independent, so the split is a plain even one: a workgroup takes
// W * epw consecutive edges, its workers (G lanes holding one 16-byte-per-lane
// slice of a row) interleave over them and keep U index loads, then U row
// loads, in flight. A sorted index makes neighbouring edges hit the same source
// row, which then comes from the vector L1 / L2 rather than from HBM.
#pragma once

#include <stdlib.h>

#include "device_utils.h"

namespace ts {

struct CooGatherArgs {
  const void *src;      // [B, N, K]
  const int64_t *index; // [B, E] (batch stride may be 0)
  const void *count;    // [B, N] element-typed, DIV only
  void *out;            // [B, E, K]
  int64_t N, E, K;
  int64_t index_batch_stride;
  int G;
  int epw;              // edges per worker
};

template <typename T, int VEC, bool DIV>
__global__ __launch_bounds__(kBlock) void coo_gather_kernel(CooGatherArgs a) {
  constexpr int U = 4;
  const int G = a.G;
  const int W = kBlock / G;
  const int w = threadIdx.x / G;
  const int lg = threadIdx.x - w * G;
  const int64_t col = (int64_t)blockIdx.y * (G * VEC) + (int64_t)lg * VEC;
  if (col >= a.K) return;
  const int64_t b = blockIdx.z;
  const int64_t *idx = a.index + b * a.index_batch_stride;
  const T *src_b = static_cast<const T *>(a.src) + b * a.N * a.K;
  const T *cnt_b = DIV ? static_cast<const T *>(a.count) + b * a.N : nullptr;
  T *out_b = static_cast<T *>(a.out) + b * a.E * a.K;

  // Workers of a workgroup interleave: worker w takes edges base + w, base + w + W, ... so that one
  // wavefront instruction covers 64 / G consecutive edges (contiguous in out, and in src for a sorted index).
  const int64_t base = (int64_t)blockIdx.x * W * a.epw;
  int64_t blk_end = base + (int64_t)W * a.epw;
  if (blk_end > a.E) blk_end = a.E;
  const int64_t e0 = base + w;
  if (e0 >= blk_end) return;
  const int64_t e_last = e0 + ((blk_end - 1 - e0) / W) * W;  // last edge of this worker
  // software pipeline on the index: the indices of batch i+1 are in flight while
  // the rows of batch i are fetched and stored
  auto load_idx = [&](int64_t *n, int64_t e) {
#pragma unroll
    for (int u = 0; u < U; ++u) {
      const int64_t ee = e + (int64_t)u * W <= e_last ? e + (int64_t)u * W : e_last;
      n[u] = idx[ee];
    }
  };
  int64_t n[U];
  load_idx(n, e0);
  for (int64_t e = e0; e <= e_last; e += (int64_t)U * W) {
    int64_t nn[U];
    load_idx(nn, e + (int64_t)U * W <= e_last ? e + (int64_t)U * W : e);
    Vec<T, VEC> x[U];
    T c[U];
#pragma unroll
    for (int u = 0; u < U; ++u) {
      // an index outside [0, N) must not read out of bounds
      const int64_t r = n[u] < 0 ? 0 : (n[u] >= a.N ? a.N - 1 : n[u]);
      x[u] = load_vec<T, VEC>(src_b + r * a.K + col);
      if (DIV) c[u] = cnt_b[r];
    }
#pragma unroll
    for (int u = 0; u < U; ++u) {
      const int64_t eu = e + (int64_t)u * W;
      if (eu <= e_last) {
        if (DIV) {
#pragma unroll
          for (int v = 0; v < VEC; ++v) x[u].v[v] = div_elem<T>(x[u].v[v], c[u]);
        }
        // streaming stores keep the source rows (re-read by neighbouring edges) in cache
        store_vec_stream<T, VEC>(out_b + eu * a.K + col, x[u]);
      }
    }
#pragma unroll
    for (int u = 0; u < U; ++u) n[u] = nn[u];
  }
}

// Rows that cannot be moved in 16-byte pieces (K not a multiple of the vector width, or src off the
// 16-byte grid): the lanes walk the FLAT output, so no lane idles whatever K is (a worker of 64 lanes for
// K = 33 leaves 31 of them without work) and every store instruction covers consecutive addresses. A lane
// owns VE consecutive elements of out (one 16-byte store when out is on the 16-byte grid, VE = 1
// otherwise); they belong to one or several neighbouring edges, whose rows it reads element by element.
// A workgroup owns a contiguous range of edges that starts on a 16-byte boundary of out; a lane's (edge,
// column) advances by a fixed step, without a division in the loop. The indices of the next step are in
// flight while the rows of this one are fetched.
template <typename T, bool DIV, int VE>
__global__ __launch_bounds__(kBlock) void coo_gather_flat_kernel(CooGatherArgs a, int epb) {
  const int K = (int)a.K;
  const int64_t b = blockIdx.z;
  const int64_t *idx = a.index + b * a.index_batch_stride;
  const T *src_b = static_cast<const T *>(a.src) + b * a.N * a.K;
  const T *cnt_b = DIV ? static_cast<const T *>(a.count) + b * a.N : nullptr;
  T *out_b = static_cast<T *>(a.out) + b * a.E * a.K;
  const int64_t e_lo = (int64_t)blockIdx.x * epb;
  const int64_t e_hi = e_lo + epb < a.E ? e_lo + epb : a.E;
  if (e_lo >= e_hi) return;
  const int n_edges = (int)(e_hi - e_lo);
  const int total = n_edges * K;  // elements of this workgroup, < 2^31
  constexpr int kStep = kBlock * VE;
  const int de = kStep / K, dk = kStep - de * K;  // one step of the workgroup in (edge, column)
  int f = threadIdx.x * VE;
  int e = f / K;
  int k = f - e * K;
  T *out_blk = out_b + e_lo * a.K;
  const int64_t *idx_blk = idx + e_lo;
  // edge and column of this lane's VE elements, and the rows they come from
  auto locate = [&](int *ee, int *kk, int64_t *r) {
    int e1 = e, k1 = k;
#pragma unroll
    for (int i = 0; i < VE; ++i) {
      ee[i] = e1 < n_edges ? e1 : n_edges - 1;
      kk[i] = k1;
      r[i] = idx_blk[ee[i]];
      if (++k1 == K) { k1 = 0; ++e1; }
    }
    e += de;
    k += dk;
    if (k >= K) { k -= K; ++e; }
  };
  int ee[VE], kk[VE];
  int64_t r[VE];
  locate(ee, kk, r);
  while (f < total) {
    int een[VE], kkn[VE];
    int64_t rn[VE];
    locate(een, kkn, rn);
    Vec<T, VE> y;
#pragma unroll
    for (int i = 0; i < VE; ++i) {
      const uint64_t ur = (uint64_t)r[i];
      const int64_t row = ur < (uint64_t)a.N ? (int64_t)ur : (r[i] < 0 ? 0 : a.N - 1);  // never read out of bounds
      T v = src_b[row * a.K + kk[i]];
      if (DIV) v = div_elem<T>(v, cnt_b[row]);
      y.v[i] = v;
    }
    if (VE > 1 && f + VE <= total) {
      store_vec_stream<T, VE>(out_blk + f, y);
    } else {
#pragma unroll
      for (int i = 0; i < VE; ++i)
        if (f + i < total) out_blk[f + i] = y.v[i];
    }
#pragma unroll
    for (int i = 0; i < VE; ++i) { kk[i] = kkn[i]; r[i] = rn[i]; }
    f += kStep;
  }
}

struct CooGatherPlan {
  int vec, G, ychunks, epw;
  int64_t nblk;
};

inline CooGatherPlan coo_gather_plan(int64_t E, int64_t K, int elem_bytes, bool aligned16) {
  CooGatherPlan p;
  const int full = kVecBytes / elem_bytes;
  p.vec = (aligned16 && full > 1 && K % full == 0) ? full : 1;
  const int64_t lanes = (K + p.vec - 1) / p.vec;
  int G = 1;
  while (G < lanes && G < kWave) G <<= 1;
  p.G = G;
  p.ychunks = (int)((K + (int64_t)G * p.vec - 1) / ((int64_t)G * p.vec));
  const int W = kBlock / G;
  p.epw = 8;  // measured best from 0.5 M to 62 M edges: short ranges keep more workgroups in flight
  if (const char *env = getenv("TS_COO_EPW")) p.epw = atoi(env) > 0 ? atoi(env) : p.epw;  // tuning aid
  const int64_t per_block = (int64_t)W * p.epw;
  p.nblk = (E + per_block - 1) / per_block;
  if (p.nblk < 1) p.nblk = 1;
  return p;
}

template <typename T, int VEC>
int launch_coo_gather_v(const CooGatherArgs &a, const CooGatherPlan &p, int64_t B, bool divide,
                        hipStream_t stream) {
  if (VEC == 1 && a.K < (1 << 20) && !getenv("TS_COO_NO_FLAT")) {  // env: tuning aid
    constexpr int VE = kVecBytes / (int)sizeof(T);
    // ~8 K elements per workgroup, a whole number of 16-byte pieces of out
    int64_t epb = (8192 / a.K + VE - 1) / VE * VE;
    if (epb < VE) epb = VE;
    const int64_t nblk = (a.E + epb - 1) / epb;
    // every batch's slice of out has to start on the 16-byte grid for the vector stores
    const bool vec_out = (reinterpret_cast<uintptr_t>(a.out) & 15) == 0 &&
                         (B == 1 || (a.E * a.K * (int64_t)sizeof(T)) % 16 == 0);
    if (nblk < 0x7FFFFFFFll) {
      dim3 grid((unsigned)nblk, 1, (unsigned)B);
      if (vec_out) {
        if (divide)
          hipLaunchKernelGGL((coo_gather_flat_kernel<T, true, VE>), grid, dim3(kBlock), 0, stream, a, (int)epb);
        else
          hipLaunchKernelGGL((coo_gather_flat_kernel<T, false, VE>), grid, dim3(kBlock), 0, stream, a, (int)epb);
      } else {
        if (divide)
          hipLaunchKernelGGL((coo_gather_flat_kernel<T, true, 1>), grid, dim3(kBlock), 0, stream, a, (int)epb);
        else
          hipLaunchKernelGGL((coo_gather_flat_kernel<T, false, 1>), grid, dim3(kBlock), 0, stream, a, (int)epb);
      }
      return hipGetLastError() == hipSuccess ? TS_OK : TS_ERR_LAUNCH;
    }
  }
  dim3 grid((unsigned)p.nblk, (unsigned)p.ychunks, (unsigned)B);
  if (divide)
    hipLaunchKernelGGL((coo_gather_kernel<T, VEC, true>), grid, dim3(kBlock), 0, stream, a);
  else
    hipLaunchKernelGGL((coo_gather_kernel<T, VEC, false>), grid, dim3(kBlock), 0, stream, a);
  return hipGetLastError() == hipSuccess ? TS_OK : TS_ERR_LAUNCH;
}

template <typename T> int launch_coo_gather(const CooGatherArgs &a, const CooGatherPlan &p,
                                            int64_t B, bool divide, hipStream_t stream);

#define TS_INSTANTIATE_COO_GATHER(T, FULLVEC)                                                \
  template <> int launch_coo_gather<T>(const CooGatherArgs &a, const CooGatherPlan &p,       \
                                       int64_t B, bool divide, hipStream_t stream) {         \
    if (p.vec == FULLVEC) return launch_coo_gather_v<T, FULLVEC>(a, p, B, divide, stream);   \
    return launch_coo_gather_v<T, 1>(a, p, B, divide, stream);                               \
  }

}  // namespace ts
