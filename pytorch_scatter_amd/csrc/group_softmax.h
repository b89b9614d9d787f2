// Softmax and log-softmax over the entries that share an index, forward and
// backward, for one index per row (the index addresses dim, every column of a
// row belongs to the same group):
//
//   m[n,k]   = max over the group            (entries have to beat lowest(), NaN never wins;
//                                             a group without a winner uses 0: what scatter_max
//                                             hands to torch_scatter/composite/softmax.py:16-18)
//   e[i,k]   = exp(src[i,k] - m[index[i],k])
//   s[n,k]   = sum of e over the group
//   softmax      out = e / s[index[i]]                          (composite/softmax.py:20-29)
//   log_softmax  out = (src - m) - log(s + eps)[index[i]]       (composite/softmax.py:45-59)
//
// The reference runs this as two scatters, two gathers and four elementwise
// passes. An index that is in order takes the one-pass tiles of group_fused.h;
// any other index (and whatever those tiles decline) takes the kernels of this
// file, three passes over src: group maxima as order-preserving
// integer keys (atomic max), group sums in the accumulate type (atomic add),
// and the elementwise finish that recomputes e from src. The first two reuse
// the wavefront pre-reduction of runs of equal neighbouring indices, so a
// sorted index costs one atomic per group and wavefront. Every intermediate
// that the reference holds in a tensor of the element type is rounded to the
// element type here as well; the group sums accumulate in fp32 for 16-bit
// floats (the reference adds in the element type).
//
// Backward (what autograd derives from the same formulas):
//   softmax      grad_src = y * (g - S[index]),       S = group sum of y * g
//   log_softmax  grad_src = g - exp(y) * G[index],    G = group sum of g
#pragma once

#include <math.h>

#include "scatter.h"

namespace ts {

// order-preserving unsigned keys of the accumulate type; -0.0 folds onto +0.0
template <typename F> struct OrdKey;
template <> struct OrdKey<float> {
  typedef uint32_t bits;
  __device__ static bits enc(float v) { return Key<float>::enc(v); }
  __device__ static float dec(bits k) { return Key<float>::dec(k); }
};
template <> struct OrdKey<double> {
  typedef uint64_t bits;
  __device__ static bits enc(double v) {
    uint64_t u = (uint64_t)__double_as_longlong(v);
    if (u == 0x8000000000000000ull) u = 0;
    return (u >> 63) ? ~u : (u | 0x8000000000000000ull);
  }
  __device__ static double dec(bits k) {
    return __longlong_as_double((long long)((k >> 63) ? (k & 0x7FFFFFFFFFFFFFFFull) : ~k));
  }
};

__device__ __forceinline__ float exp_acc(float v) { return expf(v); }
__device__ __forceinline__ double exp_acc(double v) { return exp(v); }
__device__ __forceinline__ float log_acc(float v) { return logf(v); }
__device__ __forceinline__ double log_acc(double v) { return log(v); }
__device__ __forceinline__ float sqrt_acc(float v) { return sqrtf(v); }
__device__ __forceinline__ float max_acc(float a, float b) { return fmaxf(a, b); }
__device__ __forceinline__ double max_acc(double a, double b) { return fmax(a, b); }
__device__ __forceinline__ double sqrt_acc(double v) { return sqrt(v); }

// a value of the accumulate type as the element type would hold it
template <typename T> __device__ __forceinline__ typename Acc<T>::type round_elem(typename Acc<T>::type v) {
  return to_acc<T>(from_acc<T>(v));
}
// key of "no entry has won": entries have to beat lowest() of the element type
template <typename T> __device__ __forceinline__ typename OrdKey<typename Acc<T>::type>::bits group_empty_key() {
  return OrdKey<typename Acc<T>::type>::enc(to_acc<T>(ElemLim<T>::lowest()));
}

enum {
  GS_SOFTMAX = 0, GS_LOG_SOFTMAX = 1, GS_SOFTMAX_BWD = 2, GS_LOG_SOFTMAX_BWD = 3, GS_LSE = 4, GS_LSE_BWD = 5,
  GS_STD = 6, GS_STD_BWD = 7,
  GS_STD_BINS = 8, GS_LSE_BINS = 9  // std / logsumexp forward through buckets of groups (group_binned.h)
};

struct BinArgs;
struct FusedReduceArgs;

struct GroupArgs {
  const void *src;       // [B, E, K]: forward input; backward: the forward result y
  const void *grad;      // [B, E, K]: backward only, gradient of the result
  const int64_t *index;  // index[b * sb + e * se]
  void *out;             // [B, E, K]
  void *gmax;            // [B, N, 2, K]: the keys of a group's maxima (forward) in [.., 0, :],
  void *gsum;            // its sums in the accumulate type in [.., 1, :] (gsum = gmax + K words)
  int64_t gs;            // words from one group to the next: 2K like that, or K when only the sums are used (then gsum = gmax)
  int64_t B, E, K, N;
  int64_t sb, se;
  double eps;
  const void *node_out;   // [B, N, K]: logsumexp backward, the forward result
  const void *node_grad;  // [B, N, K]: logsumexp backward, its gradient
  int from_neg_inf;       // the group maximum starts from -inf (logsumexp) instead of lowest() (softmax)
  const void *total;      // [B, N, K]: std, the group sums of src in the element type
  const int32_t *count;   // [B, N]: std, entries per group (exact)
  int unbiased;           // std: divide by count - 1
  const int *gate = nullptr;  // the three passes of softmax run only if *gate != 0 (null: always)
  int *flag = nullptr;        // softmax: a word behind the workspace of the three passes, for the one-pass kernels
  size_t ws_bytes = 0;        //          bytes of that workspace (gmax is its start)
  void *fused_ws = nullptr;     // softmax: scratch for the one-pass tiles beyond the workspace of the three passes (whose
  size_t fused_ws_bytes = 0;    //          front holds their records only while it is large enough: few, large groups)
  const void *coef = nullptr;   // std / logsumexp backward: [B, N, 2, K] in the accumulate type, what an entry needs of its
                                // group side by side (group_coef_kernel); null: gathered from the group arrays
  void *total_w = nullptr;      // std through buckets: the group sums [B, N, K] in the element type are written here,
  int32_t *count_w = nullptr;   // and the entries per group [B, N] here
  const BinArgs *bins = nullptr;  // (host) plan of the buckets
  const FusedReduceArgs *tiles = nullptr;  // (host) std / logsumexp: plan of the one-pass tiles in front of the buckets
  int tiles_force = 0;                     //        ... which run whatever a sample of the index looks like
};

// std: the group mean as the reference forms it (composite/std.py:27-31: sum / clamp(count, 1), in the
// element type) and the divisor of the squared deviations (:36-38: count or clamp(count - 1, 1), plus 1e-6)
template <typename T> __device__ __forceinline__ typename Acc<T>::type group_mean(T total, int32_t count) {
  typedef typename Acc<T>::type F;
  const F c = round_elem<T>((F)(count < 1 ? 1 : count));
  return round_elem<T>(to_acc<T>(total) / c);
}
template <typename T> __device__ __forceinline__ typename Acc<T>::type group_divisor(int32_t count, int unbiased) {
  typedef typename Acc<T>::type F;
  F c = round_elem<T>((F)(count < 1 ? 1 : count));
  if (unbiased) {
    c = round_elem<T>(c - (F)1);
    if (c < (F)1) c = (F)1;
  }
  return round_elem<T>(c + (F)1e-6);
}

inline size_t group_align(size_t v) { return (v + 255) / 256 * 256; }
// bytes of workspace: keys and sums, each [B, N, K] in 8 bytes at most, and behind them the word that tells
// the one-pass kernels (group_fused.h) and the three passes apart
inline size_t group_three_pass_bytes(int64_t B, int64_t N, int64_t K, int elem_bytes) {
  const size_t acc = elem_bytes == 8 ? 8 : 4;
  return 2 * group_align((size_t)(B * N * K) * acc);
}
inline size_t group_workspace_bytes(int64_t B, int64_t N, int64_t K, int elem_bytes) {
  return group_three_pass_bytes(B, N, K, elem_bytes) + 256;
}

template <typename T>
__global__ __launch_bounds__(kBlock) void group_init_kernel(GroupArgs g, int with_max) {
  typedef typename Acc<T>::type F;
  typedef typename OrdKey<F>::bits KB;
  if (g.gate != nullptr && *g.gate == 0) return;
  // a group's K keys and K sums lie side by side (one 64-byte line for eight floats): slot (node, k) of the keys
  // is word node * 2K + k from gmax on, of the sums the same from gsum = gmax + K on
  const int64_t n = g.B * g.N * g.gs;
  KB *keys = static_cast<KB *>(g.gmax);
  F *sums = reinterpret_cast<F *>(g.gmax);
  const KB empty = g.from_neg_inf ? OrdKey<F>::enc(-INFINITY) : group_empty_key<T>();
  for (int64_t i = (int64_t)blockIdx.x * kBlock + threadIdx.x; i < n; i += (int64_t)gridDim.x * kBlock) {
    if (g.gs == g.K || ((i / g.K) & 1) != 0)
      sums[i] = (F)0;
    else if (with_max)
      keys[i] = empty;
  }
}

// ---- pass 1: group maxima as keys
template <typename T, int C_> struct GroupMaxRun {
  typedef T Elem;
  typedef typename Acc<T>::type F;
  typedef typename OrdKey<F>::bits A;
  static constexpr int C = C_;
  static constexpr int EW = 1;
  static constexpr int U = 4;
  const T *src;
  A *gmax;
  int64_t K, gs;
  __device__ A identity() const { return (A)0; }
  __device__ void load(int64_t e, int64_t, int64_t col, int, A *x) const {
    const Vec<T, C> r = load_vec_stream<T, C>(src + e * K + col);
#pragma unroll
    for (int c = 0; c < C; ++c) {
      const F v = to_acc<T>(r.v[c]);
      x[c] = v != v ? (A)0 : OrdKey<F>::enc(v);  // NaN never wins
    }
  }
  __device__ void combine(A &x, const A &y) const { x = x > y ? x : y; }
  // a running maximum is improved rarely, so read first (a stale read only costs a spare atomic);
  // not in rows of the wavefront that look sorted, where each slot gets one atomic anyway
  bool check = true;
  __device__ void begin_row(int heads, int entries) { check = heads * 2 > entries; }
  __device__ void emit(int node, int64_t col, const A *x) const {
    A *p = gmax + (int64_t)node * gs + col;
    if (!check || x[0] > *p) __hip_atomic_fetch_max(p, x[0], __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
  }
};

template <typename T, int C, bool SERIAL>
__global__ __launch_bounds__(kBlock) void group_max_run_kernel(ScatterArgs a, GroupArgs g, int lshift,
                                                               int rows_per_wave) {
  typedef typename GroupMaxRun<T, C>::A A;
  __shared__ A s_stage[kBlock / kWave][kWave * C];
  if (g.gate != nullptr && *g.gate == 0) return;
  GroupMaxRun<T, C> p;
  p.src = static_cast<const T *>(g.src);
  p.gmax = static_cast<A *>(g.gmax);
  p.K = g.K;
  p.gs = g.gs;
  run_wave<SERIAL>(a, lshift, rows_per_wave, p, s_stage[threadIdx.x / kWave]);
}

// the group maximum a row is shifted by. Softmax: a group in which nothing beat lowest() shifts by 0
// (scatter_max's result for an untouched slot); logsumexp starts from -inf and keeps it.
template <typename T, int C, bool LSE = false>
__device__ __forceinline__ void group_shift(const void *gmax, int64_t slot, typename Acc<T>::type *m) {
  typedef typename Acc<T>::type F;
  typedef typename OrdKey<F>::bits KB;
  const Vec<KB, C> k = load_vec<KB, C>(static_cast<const KB *>(gmax) + slot);
  const KB empty = group_empty_key<T>();
#pragma unroll
  for (int c = 0; c < C; ++c) m[c] = (!LSE && k.v[c] == empty) ? (F)0 : OrdKey<F>::dec(k.v[c]);
}

// ---- pass 2: group sums of a per-entry term
//   GS_SOFTMAX / GS_LOG_SOFTMAX   exp(src - m[node])
//   GS_SOFTMAX_BWD                y * g
//   GS_LOG_SOFTMAX_BWD            g
template <typename T, int C_, int MODE> struct GroupSumRun : HotState<typename Acc<T>::type> {
  typedef T Elem;
  typedef typename Acc<T>::type A;
  static constexpr int C = C_;
  static constexpr int EW = 1;
  static constexpr int U = 4;
  const T *src;
  const T *grad;
  const void *gmax;
  A *gsum;
  const T *total;
  const int32_t *count;
  int64_t K, gs;
  __device__ A identity() const { return (A)0; }
  __device__ void load(int64_t e, int64_t, int64_t col, int node, A *x) const {
    if constexpr (MODE == GS_SOFTMAX || MODE == GS_LOG_SOFTMAX || MODE == GS_LSE) {
      const Vec<T, C> r = load_vec_stream<T, C>(src + e * K + col);
      if (node < 0) {
#pragma unroll
        for (int c = 0; c < C; ++c) x[c] = (A)0;
        return;
      }
      A m[C];
      group_shift<T, C, MODE == GS_LSE>(gmax, (int64_t)node * gs + col, m);
#pragma unroll
      for (int c = 0; c < C; ++c) {
        A z = round_elem<T>(to_acc<T>(r.v[c]) - m[c]);
        if (MODE == GS_LSE && z != z) z = -INFINITY;  // NaN entries and -inf - -inf drop out (logsumexp.py:41)
        x[c] = round_elem<T>(exp_acc(z));
      }
    } else if constexpr (MODE == GS_STD) {
      const Vec<T, C> r = load_vec_stream<T, C>(src + e * K + col);
      if (node < 0) {
#pragma unroll
        for (int c = 0; c < C; ++c) x[c] = (A)0;
        return;
      }
      const Vec<T, C> tot = load_vec<T, C>(total + (int64_t)node * K + col);
      const int32_t cnt = count[node];
#pragma unroll
      for (int c = 0; c < C; ++c) {
        const A d = round_elem<T>(to_acc<T>(r.v[c]) - group_mean<T>(tot.v[c], cnt));
        x[c] = round_elem<T>(d * d);
      }
    } else if constexpr (MODE == GS_SOFTMAX_BWD) {
      const Vec<T, C> y = load_vec_stream<T, C>(src + e * K + col);
      const Vec<T, C> gr = load_vec_stream<T, C>(grad + e * K + col);
#pragma unroll
      for (int c = 0; c < C; ++c) x[c] = to_acc<T>(y.v[c]) * to_acc<T>(gr.v[c]);
    } else {
      const Vec<T, C> gr = load_vec_stream<T, C>(grad + e * K + col);
#pragma unroll
      for (int c = 0; c < C; ++c) x[c] = to_acc<T>(gr.v[c]);
    }
  }
  __device__ void combine(A &x, const A &y) const { x = x + y; }
  __device__ void emit(int node, int64_t col, const A *x) {
    if (this->template to_table<1>(node, col, x)) return;  // a hub group: summed in LDS first
    to_memory(node, col, x);
  }
  __device__ void to_memory(int node, int64_t col, const A *x) const {
    atomic_add_elem<A>(gsum + (int64_t)node * gs + col, x[0]);
  }
};

template <typename T, int C, int MODE, bool SERIAL>
__global__ __launch_bounds__(kBlock) void group_sum_run_kernel(ScatterArgs a, GroupArgs g, int lshift,
                                                               int rows_per_wave, int hot_rlog) {
  typedef typename Acc<T>::type A;
  __shared__ A s_stage[kBlock / kWave][kWave * C];
  __shared__ typename HotSlot<A>::type s_hot[kHotAcc];
  __shared__ uint32_t s_tags[kHotRowsMax];
  if (g.gate != nullptr && *g.gate == 0) return;
  GroupSumRun<T, C, MODE> p;
  p.src = static_cast<const T *>(g.src);
  p.grad = static_cast<const T *>(g.grad);
  p.gmax = g.gmax;
  p.gsum = static_cast<A *>(g.gsum);
  p.total = static_cast<const T *>(g.total);
  p.count = g.count;
  p.K = g.K;
  p.gs = g.gs;
  p.hot_init(s_hot, s_tags, hot_rlog, lshift + LogC<C>::value);
  run_wave<SERIAL>(a, lshift, rows_per_wave, p, s_stage[threadIdx.x / kWave]);
  p.hot.template flush<1>([&](int node, int j, const A *x) {
    if (p.colbase + j < p.K) p.to_memory(node, p.colbase + j, x);
  });
}

// The same pass through a workgroup's accumulator table (the design of scatter_add_lds_kernel in scatter.h): the
// terms of a group meet in LDS and reach gsum once per group and workgroup. The run kernel above sends every term
// of an unsorted index to memory, and the terms of a hub group to one address, 7 ns apiece: 1 M single values, 30 %
// of them in one group: 2.0 ms for this pass (100 k x 8: 0.34 ms); its hot rows do not catch such a group.
template <typename T, int MODE>
__global__ __launch_bounds__(kLdsAddBlock) void group_sum_lds_kernel(ScatterArgs a, GroupArgs g, int tn_mask, int64_t epb) {
  typedef typename Acc<T>::type A;
  typedef double LdsAcc;
  constexpr int U = 4;
  __shared__ LdsAcc s_acc[kLdsAcc];
  __shared__ int32_t s_tags[kLdsAccRows];
  if (g.gate != nullptr && *g.gate == 0) return;
  GroupSumRun<T, 1, MODE> p;
  p.src = static_cast<const T *>(g.src);
  p.grad = static_cast<const T *>(g.grad);
  p.gmax = g.gmax;
  p.gsum = static_cast<A *>(g.gsum);
  p.total = static_cast<const T *>(g.total);
  p.count = g.count;
  p.K = g.K;
  p.gs = g.gs;
  const int K = (int)g.K;
  const int tn = tn_mask + 1;
  for (int i = threadIdx.x; i < tn * K; i += kLdsAddBlock) s_acc[i] = 0.0;
  for (int i = threadIdx.x; i < tn; i += kLdsAddBlock) s_tags[i] = -1;
  __syncthreads();
  const EdgeLanes m = edge_lanes(K, kLdsAddBlock);
  const int64_t be_lo = (int64_t)blockIdx.x * epb;
  int64_t be_hi = be_lo + epb;
  if (be_hi > a.B * a.E) be_hi = a.B * a.E;
  if (m.active) {
    for (int64_t be0 = be_lo + m.el; be0 < be_hi; be0 += (int64_t)m.epp * U) {
      for (int k = m.cl; k < K; k += m.L) {
        A x[U];
        int node[U];
        int64_t bec[U], pos[U];
#pragma unroll
        for (int u = 0; u < U; ++u) {
          const int64_t be = be0 + (int64_t)u * m.epp;
          bec[u] = be < be_hi ? be : be0;
          int64_t b;
          split_edge(bec[u], a.B, a.E, b, pos[u]);
          const int64_t idx = a.index[b * a.sb + pos[u] * a.se];
          node[u] = (be < be_hi && idx >= 0 && idx < a.N) ? (int)(b * a.N + idx) : -1;
        }
#pragma unroll
        for (int u = 0; u < U; ++u) p.load(bec[u], pos[u], k, node[u], &x[u]);
#pragma unroll
        for (int u = 0; u < U; ++u) {
          if (node[u] < 0) continue;
          const int row = node[u] & tn_mask;
          int tag = s_tags[row];
          if (tag == -1) {
            const int old = atomicCAS(&s_tags[row], -1, node[u]);
            tag = old == -1 ? node[u] : old;
          }
          if (tag == node[u])
            __hip_atomic_fetch_add(&s_acc[row * K + k], (LdsAcc)x[u], __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_WORKGROUP);
          else
            p.to_memory(node[u], k, &x[u]);
        }
      }
    }
  }
  __syncthreads();
  for (int i = threadIdx.x; i < tn * K; i += kLdsAddBlock) {
    const LdsAcc v = s_acc[i];
    if (v == 0.0) continue;
    const int row = i / K;
    const A out = (A)v;
    p.to_memory(s_tags[row], i - row * K, &out);
  }
}
// Pass 1 the same way: the keys of a group meet in LDS (an atomic max there) and each workgroup sends one key per
// group it met to gmax. Under a hub the run kernel reads and raises one address from every wavefront: 1 M single
// values, 30 % of them in one group: 100-320 us for this pass.
template <typename T>
__global__ __launch_bounds__(kLdsAddBlock) void group_max_lds_kernel(ScatterArgs a, GroupArgs g, int tn_mask, int64_t epb) {
  typedef typename GroupMaxRun<T, 1>::A KB;
  constexpr int U = 4;
  __shared__ KB s_keys[kLdsAcc];
  __shared__ int32_t s_tags[kLdsAccRows];
  if (g.gate != nullptr && *g.gate == 0) return;
  GroupMaxRun<T, 1> p;
  p.src = static_cast<const T *>(g.src);
  p.gmax = static_cast<KB *>(g.gmax);
  p.K = g.K;
  p.gs = g.gs;
  const int K = (int)g.K;
  const int tn = tn_mask + 1;
  for (int i = threadIdx.x; i < tn * K; i += kLdsAddBlock) s_keys[i] = (KB)0;
  for (int i = threadIdx.x; i < tn; i += kLdsAddBlock) s_tags[i] = -1;
  __syncthreads();
  const EdgeLanes m = edge_lanes(K, kLdsAddBlock);
  const int64_t be_lo = (int64_t)blockIdx.x * epb;
  int64_t be_hi = be_lo + epb;
  if (be_hi > a.B * a.E) be_hi = a.B * a.E;
  if (m.active) {
    for (int64_t be0 = be_lo + m.el; be0 < be_hi; be0 += (int64_t)m.epp * U) {
      for (int k = m.cl; k < K; k += m.L) {
        KB x[U];
        int node[U];
#pragma unroll
        for (int u = 0; u < U; ++u) {
          const int64_t be = be0 + (int64_t)u * m.epp;
          const int64_t bec = be < be_hi ? be : be0;
          int64_t b, pos;
          split_edge(bec, a.B, a.E, b, pos);
          const int64_t idx = a.index[b * a.sb + pos * a.se];
          node[u] = (be < be_hi && idx >= 0 && idx < a.N) ? (int)(b * a.N + idx) : -1;
          p.load(bec, pos, k, node[u], &x[u]);
        }
#pragma unroll
        for (int u = 0; u < U; ++u) {
          if (node[u] < 0 || x[u] == (KB)0) continue;  // 0: a NaN, which never wins
          const int row = node[u] & tn_mask;
          int tag = s_tags[row];
          if (tag == -1) {
            const int old = atomicCAS(&s_tags[row], -1, node[u]);
            tag = old == -1 ? node[u] : old;
          }
          if (tag == node[u])
            __hip_atomic_fetch_max(&s_keys[row * K + k], x[u], __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_WORKGROUP);
          else
            p.emit(node[u], k, &x[u]);
        }
      }
    }
  }
  __syncthreads();
  for (int i = threadIdx.x; i < tn * K; i += kLdsAddBlock) {
    const KB v = s_keys[i];
    if (v == (KB)0) continue;
    const int row = i / K;
    p.emit(s_tags[row], i - row * K, &v);
  }
}
template <typename T>
void launch_group_max_lds(const ScatterArgs &a, const GroupArgs &g, int tn, hipStream_t stream) {
  const int64_t n_edges = g.B * g.E;
  const int64_t epb = per_cu_chunk_edges(0, n_edges, sum_table_min_chunk(g.K, 4),
                                         131072 / g.K > 2048 ? 131072 / g.K : 2048);
  hipLaunchKernelGGL(group_max_lds_kernel<T>, dim3((unsigned)((n_edges + epb - 1) / epb)), dim3(kLdsAddBlock), 0, stream,
                     a, g, tn - 1, epb);
}

// sizes from which the pass goes through the table: 2^16 terms, rows of up to 128 columns (64 table rows), group
// numbers that fit 31 bits; entries per workgroup as for the sums of scatter (sum_table_min_chunk)
inline bool group_sum_table_ok(const GroupArgs &g, int *tn_out) {
  int tn = 1;
  while ((int64_t)tn * 2 * g.K <= kLdsAcc && tn * 2 <= kLdsAccRows) tn *= 2;
  *tn_out = tn;
  if (const char *env = getenv("TS_GROUP_TABLE")) {  // tuning aid: 0 keeps the run kernel
    if (atoi(env) == 0) return false;
  }
  // Up to 2^23 terms. Beyond, the run kernels are ahead on the index of a graph (9 M entries of 8 floats of a real
  // graph in random order: softmax 1182 us, 1339 us with both passes through the table; scatter_std of the same
  // entries in order 436 -> 703 us), and their hot rows do hold a hub at that size (10 M x 8 with a 20 % hub: no
  // extra cost).
  const int64_t n_src = g.B * g.E * g.K;
  return tn >= 64 && g.B * g.N < 0x7FFFFFFFll && n_src >= ((int64_t)1 << 16) && n_src < ((int64_t)1 << 23);
}
template <typename T, int MODE>
void launch_group_sum_lds(const ScatterArgs &a, const GroupArgs &g, int tn, hipStream_t stream) {
  const int64_t n_edges = g.B * g.E;
  const int64_t epb = per_cu_chunk_edges(0, n_edges, sum_table_min_chunk(g.K, 4),
                                         131072 / g.K > 2048 ? 131072 / g.K : 2048);
  hipLaunchKernelGGL((group_sum_lds_kernel<T, MODE>), dim3((unsigned)((n_edges + epb - 1) / epb)), dim3(kLdsAddBlock), 0,
                     stream, a, g, tn - 1, epb);
}

// What the backward pass of std / logsumexp needs of a group, side by side in the accumulate type ([B, N, 2, K]):
//   std        mean = total / max(count, 1),  w = grad / (std * divisor)   ->  grad_in = w * (src - mean)
//   logsumexp  the forward result,            grad                         ->  grad_in = grad * exp(src - result)
// With an index that is not in order every entry fetches its group's values from a line of its own per array (std: total,
// count, std, grad; 9 M x 8 floats: 689 us); here it is one line.
template <typename T, int MODE>
__global__ __launch_bounds__(kBlock) void group_coef_kernel(GroupArgs g, void *coef) {
  typedef typename Acc<T>::type F;
  const int64_t n = g.B * g.N * g.K;
  F *rec = static_cast<F *>(coef);
  const T *o = static_cast<const T *>(g.node_out), *go = static_cast<const T *>(g.node_grad);
  for (int64_t i = (int64_t)blockIdx.x * kBlock + threadIdx.x; i < n; i += (int64_t)gridDim.x * kBlock) {
    const int64_t node = i / g.K, k = i - node * g.K;
    F c0, c1;
    if (MODE == GS_STD_BWD) {
      const int32_t cnt = g.count[node];
      c0 = group_mean<T>(static_cast<const T *>(g.total)[i], cnt);
      c1 = to_acc<T>(go[i]) / (to_acc<T>(o[i]) * group_divisor<T>(cnt, g.unbiased));
    } else {
      c0 = to_acc<T>(o[i]);
      c1 = to_acc<T>(go[i]);
    }
    rec[node * 2 * g.K + k] = c0;
    rec[node * 2 * g.K + g.K + k] = c1;
  }
}

// ---- pass 3: the elementwise finish
template <typename T, int VEC, int MODE>
__global__ __launch_bounds__(kBlock) void group_finish_kernel(GroupArgs g) {
  typedef typename Acc<T>::type F;
  constexpr int U = 4;
  if (g.gate != nullptr && *g.gate == 0) return;
  const T *src = static_cast<const T *>(g.src);
  const T *grad = static_cast<const T *>(g.grad);
  const F *gsum = static_cast<const F *>(g.gsum);
  T *out = static_cast<T *>(g.out);
  const int64_t kv = g.K / VEC;
  const EdgeLanes m = edge_lanes(kv, kBlock);
  if (!m.active) return;
  const int64_t n_edges = g.B * g.E;
  const int64_t stride = (int64_t)gridDim.x * m.epp;
  const F eps = (F)g.eps;
  for (int64_t be0 = (int64_t)blockIdx.x * m.epp + m.el; be0 < n_edges; be0 += stride * U) {
    for (int64_t cv = m.cl; cv < kv; cv += m.L) {
      const int64_t k0 = cv * VEC;
      Vec<T, VEC> x[U], y[U];
      int64_t idx[U], bb[U];
#pragma unroll
      for (int u = 0; u < U; ++u) {
        const int64_t be = be0 + u * stride < n_edges ? be0 + u * stride : be0;
        int64_t ee;
        split_edge(be, g.B, g.E, bb[u], ee);
        x[u] = load_vec_stream<T, VEC>(src + be * g.K + k0);
        if (MODE == GS_SOFTMAX_BWD || MODE == GS_LOG_SOFTMAX_BWD) y[u] = load_vec_stream<T, VEC>(grad + be * g.K + k0);
        idx[u] = g.index[bb[u] * g.sb + ee * g.se];
      }
#pragma unroll
      for (int u = 0; u < U; ++u) {
        const int64_t be = be0 + u * stride;
        if (be >= n_edges) continue;
        Vec<T, VEC> r;
        if (idx[u] < 0 || idx[u] >= g.N) {  // an entry that belongs to no group
#pragma unroll
          for (int v = 0; v < VEC; ++v) r.v[v] = from_acc<T>((F)0);
          store_vec_stream<T, VEC>(out + be * g.K + k0, r);
          continue;
        }
        const int64_t slot = (bb[u] * g.N + idx[u]) * g.K + k0;
        if constexpr (MODE == GS_STD_BWD || MODE == GS_LSE_BWD) {
          if (g.coef != nullptr) {
            // one line per entry instead of three or four: std (mean, grad / (std * divisor)), logsumexp (result, grad)
            const F *rec = static_cast<const F *>(g.coef) + (bb[u] * g.N + idx[u]) * 2 * g.K + k0;
            const Vec<F, VEC> c0 = load_vec<F, VEC>(rec), c1 = load_vec<F, VEC>(rec + g.K);
#pragma unroll
            for (int v = 0; v < VEC; ++v) {
              const F xv = to_acc<T>(x[u].v[v]);
              if (MODE == GS_STD_BWD) {
                r.v[v] = from_acc<T>(c1.v[v] * (xv - c0.v[v]));
              } else {
                const F w = exp_acc(xv - c0.v[v]);
                r.v[v] = from_acc<T>(xv != xv || w != w ? (F)0 : c1.v[v] * w);
              }
            }
            store_vec_stream<T, VEC>(out + be * g.K + k0, r);
            continue;
          }
        }
        if constexpr (MODE == GS_STD_BWD) {
          // d std / d src = (src - mean) / (std * divisor); a group whose std is 0 gets 0 / 0 = NaN,
          // as autograd gives for the reference's sqrt at 0
          const Vec<T, VEC> o = load_vec<T, VEC>(static_cast<const T *>(g.node_out) + slot);
          const Vec<T, VEC> go = load_vec<T, VEC>(static_cast<const T *>(g.node_grad) + slot);
          const Vec<T, VEC> tot = load_vec<T, VEC>(static_cast<const T *>(g.total) + slot);
          const int32_t cnt = g.count[bb[u] * g.N + idx[u]];
          const F div = group_divisor<T>(cnt, g.unbiased);
#pragma unroll
          for (int v = 0; v < VEC; ++v) {
            const F d = to_acc<T>(x[u].v[v]) - group_mean<T>(tot.v[v], cnt);
            r.v[v] = from_acc<T>(to_acc<T>(go.v[v]) * d / (to_acc<T>(o.v[v]) * div));
          }
          store_vec_stream<T, VEC>(out + be * g.K + k0, r);
          continue;
        }
        if constexpr (MODE == GS_LSE_BWD) {
          // d logsumexp / d src = exp(src - result) (= exp(z) / (sum + eps)); NaN entries dropped out forward
          const Vec<T, VEC> o = load_vec<T, VEC>(static_cast<const T *>(g.node_out) + slot);
          const Vec<T, VEC> go = load_vec<T, VEC>(static_cast<const T *>(g.node_grad) + slot);
#pragma unroll
          for (int v = 0; v < VEC; ++v) {
            const F xv = to_acc<T>(x[u].v[v]);
            const F w = exp_acc(xv - to_acc<T>(o.v[v]));
            r.v[v] = from_acc<T>(xv != xv || w != w ? (F)0 : to_acc<T>(go.v[v]) * w);
          }
          store_vec_stream<T, VEC>(out + be * g.K + k0, r);
          continue;
        }
        const int64_t wslot = (bb[u] * g.N + idx[u]) * g.gs + k0;  // keys and sums of a group side by side
        const Vec<F, VEC> s = load_vec<F, VEC>(gsum + wslot);
        F mx[VEC];
        if (MODE == GS_SOFTMAX || MODE == GS_LOG_SOFTMAX) group_shift<T, VEC>(g.gmax, wslot, mx);
#pragma unroll
        for (int v = 0; v < VEC; ++v) {
          const F xv = to_acc<T>(x[u].v[v]);
          F res;
          if (MODE == GS_SOFTMAX) {
            const F e = round_elem<T>(exp_acc(round_elem<T>(xv - mx[v])));
            res = e / round_elem<T>(s.v[v]);
          } else if (MODE == GS_LOG_SOFTMAX) {
            const F z = round_elem<T>(xv - mx[v]);
            F l = round_elem<T>(log_acc(round_elem<T>(round_elem<T>(s.v[v]) + eps)));
            // keeps the compiler from folding the subtraction's negation into the float -> half
            // conversion as a two-element vector negation, which this backend cannot select
            asm volatile("" : "+v"(l));
            res = z - l;
          } else if (MODE == GS_SOFTMAX_BWD) {
            res = xv * (to_acc<T>(y[u].v[v]) - s.v[v]);
          } else {
            res = to_acc<T>(y[u].v[v]) - exp_acc(xv) * s.v[v];
          }
          r.v[v] = from_acc<T>(res);
        }
        store_vec_stream<T, VEC>(out + be * g.K + k0, r);
      }
    }
  }
}

// logsumexp: result per group, log(sum + eps) + max with the reference's clean-up
// (composite/logsumexp.py:51-54: NaN and -inf -> 0, +inf -> largest finite value)
template <typename T>
__global__ __launch_bounds__(kBlock) void group_lse_finish_kernel(GroupArgs g) {
  typedef typename Acc<T>::type F;
  typedef typename OrdKey<F>::bits KB;
  const int64_t n = g.B * g.N * g.K;
  const KB *gmax = static_cast<const KB *>(g.gmax);
  const F *gsum = static_cast<const F *>(g.gsum);
  T *out = static_cast<T *>(g.out);
  const F eps = (F)g.eps;
  for (int64_t i = (int64_t)blockIdx.x * kBlock + threadIdx.x; i < n; i += (int64_t)gridDim.x * kBlock) {
    const int64_t node = i / g.K, w = node * g.gs + (i - node * g.K);
    const F m = OrdKey<F>::dec(gmax[w]);
    const F l = round_elem<T>(log_acc(round_elem<T>(round_elem<T>(gsum[w]) + eps)));
    F o = round_elem<T>(l + m);
    if (o != o || o == -INFINITY) o = (F)0;
    if (o == INFINITY) o = to_acc<T>(ElemLim<T>::max());
    out[i] = from_acc<T>(o);
  }
}

// std: result per group, sqrt(sum of squared deviations / divisor) (composite/std.py:33-39)
template <typename T>
__global__ __launch_bounds__(kBlock) void group_std_finish_kernel(GroupArgs g) {
  typedef typename Acc<T>::type F;
  const int64_t n = g.B * g.N * g.K;
  const F *gsum = static_cast<const F *>(g.gsum);
  T *out = static_cast<T *>(g.out);
  for (int64_t i = (int64_t)blockIdx.x * kBlock + threadIdx.x; i < n; i += (int64_t)gridDim.x * kBlock) {
    const F div = group_divisor<T>(g.count[i / g.K], g.unbiased);
    const int64_t node = i / g.K;
    out[i] = from_acc<T>(sqrt_acc(round_elem<T>(round_elem<T>(gsum[node * g.gs + (i - node * g.K)]) / div)));
  }
}

}  // namespace ts
#include "group_fused.h"
namespace ts {

// ---- host side
inline ScatterArgs group_index_args(const GroupArgs &g) {
  ScatterArgs a = {};
  a.index = g.index;
  a.B = g.B;
  a.E = g.E;
  a.K = g.K;
  a.N = g.N;
  a.sb = g.sb;
  a.se = g.se;
  a.sk = 0;
  return a;
}

}  // namespace ts
#include "group_binned.h"
#include "group_fused_reduce.h"
namespace ts {

// std / logsumexp forward: the one-pass tiles for an index in order where they apply, then (gated on their verdict)
// the passes through buckets of groups
template <typename T, int VEC, int MODE>
int launch_group_reduce(const GroupArgs &g, hipStream_t stream) {
  if (g.tiles == nullptr) return launch_group_bins<T, VEC, MODE>(g, stream);
  const int rc = launch_group_reduce_fused<T, VEC, MODE>(g, *g.tiles, g.tiles_force != 0, stream);
  if (rc != TS_OK) return rc;
  return launch_group_bins<T, VEC, MODE>(g, stream, g.tiles->flag);
}

template <typename T, int VEC, int MODE>
int launch_group_softmax_m(const GroupArgs &g_in, hipStream_t stream) {
  constexpr bool kForward = MODE == GS_SOFTMAX || MODE == GS_LOG_SOFTMAX;
  GroupArgs g = g_in;
  const int64_t n_edges = g.B * g.E;
  if (g.B * g.N >= 0x7FFFFFFFll) return TS_ERR_UNSUPPORTED;
  const RunGrid rg = run_grid(n_edges, g.K / VEC, VEC, VEC * (int)sizeof(T));
  if (!rg.ok) return TS_ERR_UNSUPPORTED;
  // An index that looks sorted goes through the one-pass kernels first; the three passes below then run only
  // if those found a descent. TS_GROUP_FUSED: 0 never, 2 at any size and whatever the index looks like.
  int fused_mode = 1;
  if (const char *env = getenv("TS_GROUP_FUSED")) fused_mode = atoi(env);
  FusedArgs f;
  if (fused_mode != 0 && g.flag != nullptr &&
      group_fused_plan(g, MODE, (int)sizeof(T), g.gmax, g.ws_bytes, fused_mode == 2, f)) {
    const int rc = launch_group_fused<T, VEC, MODE>(g, f, fused_mode == 2, stream);
    if (rc != TS_OK) return rc;
    g.gate = f.flag;
  }
  if constexpr (kForward) {
    if (g.bins != nullptr) {
      // any other index, with the larger workspace: key and sum of every group from one gather of src through
      // buckets of groups (group_binned.h), then the elementwise finish
      const int rc = launch_group_bins<T, VEC, GS_SOFTMAX>(g, stream, const_cast<int *>(g.gate));
      if (rc != TS_OK) return rc;
      hipLaunchKernelGGL((group_finish_kernel<T, VEC, MODE>), dim3(scatter_grid(n_edges, g.K / VEC, kBlock, 4)),
                         dim3(kBlock), 0, stream, g);
      return hipGetLastError() == hipSuccess ? TS_OK : TS_ERR_LAUNCH;
    }
  }
  const ScatterArgs a = group_index_args(g);
  const dim3 gd(rg.blocks, rg.ychunks);
  hipLaunchKernelGGL(group_init_kernel<T>, dim3(grid_for(g.B * g.N * g.K)), dim3(kBlock), 0, stream, g,
                     kForward ? 1 : 0);
  int tn = 1;
  const bool table = group_sum_table_ok(g, &tn);
  if (kForward && table)
    launch_group_max_lds<T>(a, g, tn, stream);
  else if (kForward)
    TS_LAUNCH_RUN(rg.serial, (group_max_run_kernel<T, VEC, true>), (group_max_run_kernel<T, VEC, false>), gd, stream, a, g,
                  rg.lshift, rg.rpw);
  if (table)
    launch_group_sum_lds<T, MODE>(a, g, tn, stream);
  else
    TS_LAUNCH_RUN(rg.serial, (group_sum_run_kernel<T, VEC, MODE, true>), (group_sum_run_kernel<T, VEC, MODE, false>), gd,
                  stream, a, g, rg.lshift, rg.rpw, rg.hot_rlog);
  hipLaunchKernelGGL((group_finish_kernel<T, VEC, MODE>), dim3(scatter_grid(n_edges, g.K / VEC, kBlock, 4)),
                     dim3(kBlock), 0, stream, g);
  return hipGetLastError() == hipSuccess ? TS_OK : TS_ERR_LAUNCH;
}

template <typename T, int VEC>
int launch_group_lse_v(const GroupArgs &g, bool backward, hipStream_t stream) {
  const int64_t n_edges = g.B * g.E;
  if (g.B * g.N >= 0x7FFFFFFFll) return TS_ERR_UNSUPPORTED;
  if (backward) {
    if (g.coef != nullptr)
      hipLaunchKernelGGL((group_coef_kernel<T, GS_LSE_BWD>), dim3(grid_for(g.B * g.N * g.K)), dim3(kBlock), 0, stream, g,
                         const_cast<void *>(g.coef));
    hipLaunchKernelGGL((group_finish_kernel<T, VEC, GS_LSE_BWD>), dim3(scatter_grid(n_edges, g.K / VEC, kBlock, 4)),
                       dim3(kBlock), 0, stream, g);
    return hipGetLastError() == hipSuccess ? TS_OK : TS_ERR_LAUNCH;
  }
  const RunGrid rg = run_grid(n_edges, g.K / VEC, VEC, VEC * (int)sizeof(T));
  if (!rg.ok) return TS_ERR_UNSUPPORTED;
  const ScatterArgs a = group_index_args(g);
  const dim3 gd(rg.blocks, rg.ychunks);
  const unsigned g_out = grid_for(g.B * g.N * g.K);
  hipLaunchKernelGGL(group_init_kernel<T>, dim3(g_out), dim3(kBlock), 0, stream, g, 1);
  int tn = 1;
  const bool table = group_sum_table_ok(g, &tn);
  if (table)
    launch_group_max_lds<T>(a, g, tn, stream);
  else
    TS_LAUNCH_RUN(rg.serial, (group_max_run_kernel<T, VEC, true>), (group_max_run_kernel<T, VEC, false>), gd, stream, a, g,
                  rg.lshift, rg.rpw);
  if (table)
    launch_group_sum_lds<T, GS_LSE>(a, g, tn, stream);
  else
    TS_LAUNCH_RUN(rg.serial, (group_sum_run_kernel<T, VEC, GS_LSE, true>), (group_sum_run_kernel<T, VEC, GS_LSE, false>), gd,
                  stream, a, g, rg.lshift, rg.rpw, rg.hot_rlog);
  hipLaunchKernelGGL(group_lse_finish_kernel<T>, dim3(g_out), dim3(kBlock), 0, stream, g);
  return hipGetLastError() == hipSuccess ? TS_OK : TS_ERR_LAUNCH;
}

template <typename T, int VEC>
int launch_group_std_v(const GroupArgs &g, bool backward, hipStream_t stream) {
  const int64_t n_edges = g.B * g.E;
  if (g.B * g.N >= 0x7FFFFFFFll) return TS_ERR_UNSUPPORTED;
  if (backward) {
    if (g.coef != nullptr)
      hipLaunchKernelGGL((group_coef_kernel<T, GS_STD_BWD>), dim3(grid_for(g.B * g.N * g.K)), dim3(kBlock), 0, stream, g,
                         const_cast<void *>(g.coef));
    hipLaunchKernelGGL((group_finish_kernel<T, VEC, GS_STD_BWD>), dim3(scatter_grid(n_edges, g.K / VEC, kBlock, 4)),
                       dim3(kBlock), 0, stream, g);
    return hipGetLastError() == hipSuccess ? TS_OK : TS_ERR_LAUNCH;
  }
  const RunGrid rg = run_grid(n_edges, g.K / VEC, VEC, VEC * (int)sizeof(T));
  if (!rg.ok) return TS_ERR_UNSUPPORTED;
  const ScatterArgs a = group_index_args(g);
  const dim3 gd(rg.blocks, rg.ychunks);
  const unsigned g_out = grid_for(g.B * g.N * g.K);
  hipLaunchKernelGGL(group_init_kernel<T>, dim3(g_out), dim3(kBlock), 0, stream, g, 0);
  int tn = 1;
  if (n_edges > 0 && group_sum_table_ok(g, &tn))
    launch_group_sum_lds<T, GS_STD>(a, g, tn, stream);
  else if (n_edges > 0)
    TS_LAUNCH_RUN(rg.serial, (group_sum_run_kernel<T, VEC, GS_STD, true>), (group_sum_run_kernel<T, VEC, GS_STD, false>), gd,
                  stream, a, g, rg.lshift, rg.rpw, rg.hot_rlog);
  hipLaunchKernelGGL(group_std_finish_kernel<T>, dim3(g_out), dim3(kBlock), 0, stream, g);
  return hipGetLastError() == hipSuccess ? TS_OK : TS_ERR_LAUNCH;
}

template <typename T, int VEC>
int launch_group_softmax_v(const GroupArgs &g, int mode, hipStream_t stream) {
  switch (mode) {
  case GS_STD: return launch_group_std_v<T, VEC>(g, false, stream);
  case GS_STD_BWD: return launch_group_std_v<T, VEC>(g, true, stream);
  case GS_STD_BINS: return launch_group_reduce<T, VEC, GS_STD>(g, stream);
  case GS_LSE_BINS: return launch_group_reduce<T, VEC, GS_LSE>(g, stream);
  case GS_LSE: return launch_group_lse_v<T, VEC>(g, false, stream);
  case GS_LSE_BWD: return launch_group_lse_v<T, VEC>(g, true, stream);
  case GS_SOFTMAX: return launch_group_softmax_m<T, VEC, GS_SOFTMAX>(g, stream);
  case GS_LOG_SOFTMAX: return launch_group_softmax_m<T, VEC, GS_LOG_SOFTMAX>(g, stream);
  case GS_SOFTMAX_BWD: return launch_group_softmax_m<T, VEC, GS_SOFTMAX_BWD>(g, stream);
  case GS_LOG_SOFTMAX_BWD: return launch_group_softmax_m<T, VEC, GS_LOG_SOFTMAX_BWD>(g, stream);
  default: return TS_ERR_BAD_ARG;
  }
}

template <typename T> int launch_group_softmax(const GroupArgs &g, int mode, int vec, hipStream_t stream);

#define TS_INSTANTIATE_GROUP_SOFTMAX(T, FULLVEC)                                                      \
  template <> int launch_group_softmax<T>(const GroupArgs &g, int mode, int vec, hipStream_t stream) { \
    if (vec == FULLVEC) return launch_group_softmax_v<T, FULLVEC>(g, mode, stream);                  \
    return launch_group_softmax_v<T, 1>(g, mode, stream);                                            \
  }

}  // namespace ts
