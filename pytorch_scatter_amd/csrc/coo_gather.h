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
