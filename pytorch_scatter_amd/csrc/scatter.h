// Scatter with an unsorted index: out[b, index[b,e,k], k] (op)= src[b,e,k].
//
// sum / mul update `out` in place with device-scope atomics in the element
// type (the reference accumulates in scalar_t as well, csrc/cpu/scatter_cpu.cpp
// :74-76): native add for f32 / f64 / i32 / i64, packed pair add for bf16 / f16
// when the pair is 4-byte aligned, compare-and-swap on the containing word
// otherwise.
//
// min / max of element types up to 32 bits run in ONE pass over src: value
// and position are packed into a 64-bit key
//     key = order(value) << 32 | (0xFFFFFFFE - e)
// and reduced with a 64-bit unsigned atomic max into the int64 arg_out buffer
// itself, so no extra memory is needed. A larger value wins; among equal
// values the smaller e wins, which is the CPU rule (first index wins,
// csrc/cpu/reducer.h:63-67) and makes the result independent of scheduling.
// The low word 0xFFFFFFFF marks "initial / previous content": an entry has to
// beat it strictly. A cheap read of the current key skips the atomic for the
// vast majority of entries (a running maximum is improved only O(log n)
// times). A last pass over [B, N, K] unpacks value and arg.
// 64-bit element types use the reference's two-pass scheme with a
// deterministic arg (atomic min over matching positions).
//
// With one index per row (the message-passing call) the kernels do not issue
// one atomic per element: a wavefront combines runs of equal neighbouring
// indices first (run_reduce_wave for narrow rows, run_serial_wave from 128
// bytes per entry), sums keep the rows of hub nodes in a small LDS table per
// workgroup (HotRows), and heavily contended inputs reduce into LDS tables of
// accumulators or keys before they touch memory. Given scratch memory, large
// inputs with rows of 64 bytes and more are first binned by bucket of output
// rows, so that a workgroup's table holds every row it can meet
// (scatter_binned.h).
#pragma once

#include <limits>
#include <type_traits>
#include <stdlib.h>

#include "device_utils.h"

// Which kernels the last ts_scatter* call of this thread launched (TS_ROUTE_* of include/ts_hip.h; defined in
// capi.hip): a host-side note for tests and tools, read back through ts_scatter_last_route().
extern "C" void ts_note_scatter_route(int route);

namespace ts {

// ---------------------------------------------------------------- atomics
template <typename T, typename F>
__device__ __forceinline__ void atomic_rmw_word(T *addr, F fn) {
  // read-modify-write of a 1/2/4-byte element through its 32-bit container
  static_assert(sizeof(T) <= 4, "");
  uintptr_t a = reinterpret_cast<uintptr_t>(addr);
  uint32_t *word = reinterpret_cast<uint32_t *>(a & ~(uintptr_t)3);
  const int shift = (int)(a & 3) * 8;
  const uint32_t mask = (sizeof(T) == 4) ? 0xFFFFFFFFu : (((1u << (sizeof(T) * 8)) - 1u) << shift);
  uint32_t old = __hip_atomic_load(word, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
  while (true) {
    uint32_t bits = (old & mask) >> shift;
    T cur;
    __builtin_memcpy(&cur, &bits, sizeof(T));
    T nv = fn(cur);
    uint32_t nbits = 0;
    __builtin_memcpy(&nbits, &nv, sizeof(T));
    uint32_t desired = (old & ~mask) | ((nbits << shift) & mask);
    if (desired == old) return;
    if (__hip_atomic_compare_exchange_strong(word, &old, desired, __ATOMIC_RELAXED, __ATOMIC_RELAXED,
                                             __HIP_MEMORY_SCOPE_AGENT))
      return;
  }
}
template <typename T, typename F>
__device__ __forceinline__ void atomic_rmw_dword(T *addr, F fn) {
  static_assert(sizeof(T) == 8, "");
  uint64_t *word = reinterpret_cast<uint64_t *>(addr);
  uint64_t old = __hip_atomic_load(word, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
  while (true) {
    T cur;
    __builtin_memcpy(&cur, &old, 8);
    T nv = fn(cur);
    uint64_t desired;
    __builtin_memcpy(&desired, &nv, 8);
    if (desired == old) return;
    if (__hip_atomic_compare_exchange_strong(word, &old, desired, __ATOMIC_RELAXED, __ATOMIC_RELAXED,
                                             __HIP_MEMORY_SCOPE_AGENT))
      return;
  }
}
template <typename T, typename F> __device__ __forceinline__ void atomic_rmw(T *addr, F fn) {
  if constexpr (sizeof(T) == 8)
    atomic_rmw_dword<T>(addr, fn);
  else
    atomic_rmw_word<T>(addr, fn);
}

// element arithmetic in the element type (16-bit floats: via float, one rounding)
template <typename T> __device__ __forceinline__ T add_elem(T a, T b) { return (T)(a + b); }
template <> __device__ __forceinline__ bf16_t add_elem<bf16_t>(bf16_t a, bf16_t b) {
  return float_to_bf16(bf16_to_float(a) + bf16_to_float(b));
}
template <> __device__ __forceinline__ f16_t add_elem<f16_t>(f16_t a, f16_t b) {
  return (f16_t)((float)a + (float)b);
}
template <typename T> __device__ __forceinline__ T mul_elem(T a, T b) { return (T)(a * b); }
template <> __device__ __forceinline__ bf16_t mul_elem<bf16_t>(bf16_t a, bf16_t b) {
  return float_to_bf16(bf16_to_float(a) * bf16_to_float(b));
}
template <> __device__ __forceinline__ f16_t mul_elem<f16_t>(f16_t a, f16_t b) {
  return (f16_t)((float)a * (float)b);
}

template <typename T> __device__ __forceinline__ void atomic_add_elem(T *p, T v) {
  atomic_rmw<T>(p, [v](T cur) { return add_elem<T>(cur, v); });
}
template <> __device__ __forceinline__ void atomic_add_elem<float>(float *p, float v) {
  unsafeAtomicAdd(p, v);  // global_atomic_add_f32, no return value
}
template <> __device__ __forceinline__ void atomic_add_elem<double>(double *p, double v) {
  unsafeAtomicAdd(p, v);  // global_atomic_add_f64
}
template <> __device__ __forceinline__ void atomic_add_elem<int32_t>(int32_t *p, int32_t v) {
  __hip_atomic_fetch_add(p, v, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
}
template <> __device__ __forceinline__ void atomic_add_elem<int64_t>(int64_t *p, int64_t v) {
  __hip_atomic_fetch_add(p, v, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
}

// One 16-bit float without a compare-and-swap loop (which collapses when many lanes add to the same
// element): a packed-pair add on the 32-bit word that holds the element, with +0.0 for the
// neighbour. x + 0.0 leaves every value alone (a -0.0 neighbour turns into +0.0, which compares
// equal), so this is only used when the neighbour is an element of the same buffer [lo, hi).
template <typename T> __device__ __forceinline__ void atomic_add_half(T *p, T v, const T *lo, const T *hi) {
  static_assert(sizeof(T) == 2, "");
  const uintptr_t a = reinterpret_cast<uintptr_t>(p);
  T *w = reinterpret_cast<T *>(a & ~(uintptr_t)3);
  if (w < lo || w + 2 > hi) {
    atomic_add_elem<T>(p, v);
    return;
  }
  const bool upper = (a & 2) != 0;
  if constexpr (__is_same(T, bf16_t)) {
    typedef short v2s __attribute__((ext_vector_type(2)));
    v2s pk;
    pk.x = upper ? (short)0 : (short)v.x;
    pk.y = upper ? (short)v.x : (short)0;
    __builtin_amdgcn_global_atomic_fadd_v2bf16(reinterpret_cast<v2s *>(w), pk);
  } else {
    typedef _Float16 v2h __attribute__((ext_vector_type(2)));
    v2h pk;
    pk.x = upper ? (_Float16)0 : (_Float16)v;
    pk.y = upper ? (_Float16)v : (_Float16)0;
    __builtin_amdgcn_global_atomic_fadd_v2f16(reinterpret_cast<v2h *>(w), pk);
  }
}

// both 16-bit floats of a 4-byte aligned word in one packed add
template <typename T> __device__ __forceinline__ void atomic_add_pair(T *w, T v0, T v1) {
  static_assert(sizeof(T) == 2, "");
  if constexpr (__is_same(T, bf16_t)) {
    typedef short v2s __attribute__((ext_vector_type(2)));
    v2s pk;
    pk.x = (short)v0.x;
    pk.y = (short)v1.x;
    __builtin_amdgcn_global_atomic_fadd_v2bf16(reinterpret_cast<v2s *>(w), pk);
  } else {
    typedef _Float16 v2h __attribute__((ext_vector_type(2)));
    v2h pk;
    pk.x = (_Float16)v0;
    pk.y = (_Float16)v1;
    __builtin_amdgcn_global_atomic_fadd_v2f16(reinterpret_cast<v2h *>(w), pk);
  }
}

// ------------------------------------------------ order-preserving 32-bit keys
// order(v) is monotone in v; -0.0 is folded onto +0.0 so that the two compare
// equal as they do under the reference's `<` / `>`.
template <typename T> struct Key;
template <> struct Key<float> {
  __device__ static uint32_t enc(float v) {
    uint32_t u = __float_as_uint(v);
    if (u == 0x80000000u) u = 0;
    return (u & 0x80000000u) ? ~u : (u | 0x80000000u);
  }
  __device__ static float dec(uint32_t k) {
    return __uint_as_float((k & 0x80000000u) ? (k & 0x7FFFFFFFu) : ~k);
  }
  __device__ static bool is_nan(float v) { return v != v; }
  static constexpr bool kFloat = true;
};
template <> struct Key<bf16_t> {
  __device__ static uint32_t enc(bf16_t v) { return Key<float>::enc(bf16_to_float(v)); }
  __device__ static bf16_t dec(uint32_t k) { bf16_t r; r.x = (uint16_t)(__float_as_uint(Key<float>::dec(k)) >> 16); return r; }
  __device__ static bool is_nan(bf16_t v) { return (v.x & 0x7FFF) > 0x7F80; }
  static constexpr bool kFloat = true;
};
template <> struct Key<f16_t> {
  __device__ static uint32_t enc(f16_t v) { return Key<float>::enc((float)v); }
  __device__ static f16_t dec(uint32_t k) { return (f16_t)Key<float>::dec(k); }
  __device__ static bool is_nan(f16_t v) { return v != v; }
  static constexpr bool kFloat = true;
};
template <typename I> struct IntKey {
  __device__ static uint32_t enc(I v) { return (uint32_t)(int32_t)v ^ 0x80000000u; }
  __device__ static I dec(uint32_t k) { return (I)(int32_t)(k ^ 0x80000000u); }
  __device__ static bool is_nan(I) { return false; }
  static constexpr bool kFloat = false;
};
template <> struct Key<int32_t> : IntKey<int32_t> {};
template <> struct Key<int16_t> : IntKey<int16_t> {};
template <> struct Key<int8_t> : IntKey<int8_t> {};
template <> struct Key<uint8_t> : IntKey<uint8_t> {};

constexpr uint32_t kKeepLow = 0xFFFFFFFFu;  // low word of "initial / previous content"

template <typename T, bool IS_MAX> __device__ __forceinline__ uint64_t pack_key(T v, uint32_t low) {
  uint32_t k = Key<T>::enc(v);
  if (!IS_MAX) k = ~k;
  return ((uint64_t)k << 32) | low;
}

// ------------------------------------------------------------------ kernels
struct ScatterArgs {
  const void *src;
  const int64_t *index;
  void *out;
  int64_t *arg_out;
  int64_t B, E, K, N;
  int64_t sb, se, sk;  // index strides
  int out_given;
  int precheck;        // read before the atomic: 0 none, 1 cached, 2 device-coherent, 3 streaming
  int lds_cache;       // reduce hot slots in LDS first: 0 never, 1 for large inputs, 2 always
  int64_t lds_epb;     // entries per workgroup chunk of that variant, 0 = default
  int run_reduce = 1;  // sum: pre-reduce runs of equal neighbouring indices in the wavefront
  int lds_k1 = 1;      // min/max with K == 1: the 1024-lane table kernel
  void *bin_ws = nullptr;  // optional workspace: min/max of wide rows through buckets of output rows
  size_t bin_ws_bytes = 0;
  int bin_any_size = 0;    // tuning aid / tests: also for inputs below the size from which it pays
  const int *skip_flag = nullptr;  // sum kernels: leave at once if *skip_flag != 0 (the binned pass did the work)
  int skip_inverse = 0;            // ... if *skip_flag == 0 instead
  int skip_want = -1;              // >= 0 (table kernel only): run only if *skip_flag == skip_want
  int32_t *count_out = nullptr;    // sum through the buckets: also count the entries of every output row into this
                                   // zeroed [B * N] array ...
  const int **count_flag = nullptr;  // ... and leave the buckets' flag here (still null afterwards: the call took another
                                   // route and nothing was counted)
  int *count_done = nullptr;       // (host) a small sum counts into count_out (not zeroed by the caller) in the launch that
                                   // adds (scatter_add_count_run_kernel) and sets this to 1: the counts are complete;
                                   // 2: the table kernel behind the value buckets counts for the verdict "skewed"
  int *order_ws = nullptr;         // sum of narrow rows: a word of scratch for the sample of the index that picks the kernel
  int skew_probe = 1;              // min/max: sample the index for skew (needs 256 bytes of workspace): 0 never, 2 at any size
  const int *skew_flag = nullptr;  // min/max kernels behind the probe: run only if (*skew_flag != 0) == (skew_want != 0)
  int skew_want = 0;
  // A caller that can finish the scatter with the segmented reduction when the index turns out to be sorted
  // (it launches that reduction afterwards, gated on the flag) sets sorted_route. The launcher then lets the
  // count pass of the buckets check the whole index (in order, inside [0, N)), reports through *route_flag the
  // device flag that reads 0 for such an index once the count pass has run, and launches nothing else that
  // would handle the sorted case; *route_flag stays null when the buckets were not taken.
  int sorted_route = 0;
  const int **route_flag = nullptr;
  int64_t *route_ptr = nullptr;  // [B][N + 1]: the row pointers of a sorted index, written by the place pass
};

// Inputs for which the min/max launcher samples the index (see index_skew_kernel): rows of 2-256 columns of
// 4-byte elements (16 bf16 columns lose through the table: 762 -> 1025 us), at least 32 M elements (the sample
// and the launch that returns at once cost 10-20 us), fewer than 32 entries per output row on average.
inline bool skew_probe_shape(int64_t B, int64_t E, int64_t K, int64_t N, int elem_bytes, bool any_size) {
  return elem_bytes == 4 && K > 1 && K <= 256 && B * E >= 8192 &&
         (any_size || (B * E * K >= ((int64_t)1 << 23) && E < 32 * N));
}

// ---- thread -> (edge, column) mapping shared by the scatter kernels ------------
// A workgroup covers `epp` edges per pass with `L` lanes per edge, each lane
// holding VEC consecutive columns; the column of a lane never changes, so the
// hot loops are free of integer division. Rows wider than the workgroup are
// covered by a loop over column chunks.
struct EdgeLanes {
  int L;    // lanes per edge
  int epp;  // edges per pass of the workgroup
  int el;   // this thread's edge slot, < epp (threads beyond are idle)
  int cl;   // this thread's column lane, < L
  bool active;
};
__device__ __forceinline__ EdgeLanes edge_lanes(int64_t kv, int block) {
  EdgeLanes m;
  m.L = kv < block ? (int)kv : block;
  m.epp = block / m.L;
  m.el = (int)threadIdx.x / m.L;
  m.cl = (int)threadIdx.x - m.el * m.L;
  m.active = m.el < m.epp;
  return m;
}
// flat edge number -> (batch, position); the division only happens for batched inputs
__device__ __forceinline__ void split_edge(const int64_t be, const int64_t B, const int64_t E, int64_t &b,
                                           int64_t &e) {
  if (B == 1) {
    b = 0;
    e = be;
  } else {
    b = be / E;
    e = be - b * E;
  }
}

// sum / mul: one atomic per element, consecutive lanes on consecutive columns
template <typename T, int VEC, int REDUCE>
__global__ __launch_bounds__(kBlock) void scatter_atomic_kernel(ScatterArgs a) {
  constexpr int U = 4;
  if (a.skip_flag != nullptr && *a.skip_flag != 0) return;
  const T *src = static_cast<const T *>(a.src);
  T *out = static_cast<T *>(a.out);
  const int64_t kv = a.K / VEC;
  const EdgeLanes m = edge_lanes(kv, kBlock);
  if (!m.active) return;
  const int64_t n_edges = a.B * a.E;
  const int64_t stride = (int64_t)gridDim.x * m.epp;
  for (int64_t be0 = (int64_t)blockIdx.x * m.epp + m.el; be0 < n_edges; be0 += stride * U) {
    for (int64_t cv = m.cl; cv < kv; cv += m.L) {
      const int64_t k0 = cv * VEC;
      Vec<T, VEC> x[U];
      int64_t idx[U], bb[U], ee[U];
#pragma unroll
      for (int u = 0; u < U; ++u) {
        const int64_t be = be0 + u * stride;
        split_edge(be < n_edges ? be : be0, a.B, a.E, bb[u], ee[u]);
        x[u] = load_vec_stream<T, VEC>(src + (bb[u] * a.E + ee[u]) * a.K + k0);
        idx[u] = a.index[bb[u] * a.sb + ee[u] * a.se + k0 * a.sk];
      }
#pragma unroll
      for (int u = 0; u < U; ++u) {
        const bool live = be0 + u * stride < n_edges;
        int64_t id = idx[u];
#pragma unroll
        for (int v = 0; v < VEC; ++v) {
          if (v > 0 && a.sk != 0 && live) id = a.index[bb[u] * a.sb + ee[u] * a.se + (k0 + v) * a.sk];
          const bool valid = live && id >= 0 && id < a.N;
          T *p = out + (bb[u] * a.N + (valid ? id : 0)) * a.K + k0 + v;
          const T val = x[u].v[v];
          if (REDUCE == TS_SUM) {
            if (!valid) continue;
            if constexpr (__is_same(T, bf16_t) || __is_same(T, f16_t))
              atomic_add_half<T>(p, val, out, out + a.B * a.N * a.K);
            else
              atomic_add_elem<T>(p, val);
          } else {
            // There is no atomic product: a compare-and-swap loop, whose time grows with the square of the lanes
            // that meet in one element (100 k entries, 30 % of them on one row: 418 ms). The lanes of a wavefront
            // that multiply into the same element therefore combine first and send one of them.
            uint64_t todo = __ballot(valid);
            const int lane = threadIdx.x & (kWave - 1);
            while (todo != 0) {
              const int leader = __ffsll((unsigned long long)todo) - 1;
              const uint64_t mine = reinterpret_cast<uint64_t>(p);
              const uint64_t target = ((uint64_t)(uint32_t)__shfl((int)(mine >> 32), leader) << 32) |
                                      (uint32_t)__shfl((int)(uint32_t)mine, leader);
              const uint64_t same = __ballot(valid && mine == target) & todo;
              T prod = val;  // the leader's own factor; the others follow in lane order
              uint64_t bits = 0;
              __builtin_memcpy(&bits, &val, sizeof(T));
              for (uint64_t rest = same & (same - 1); rest != 0; rest &= rest - 1) {
                const int j = __ffsll((unsigned long long)rest) - 1;
                const uint64_t other = ((uint64_t)(uint32_t)__shfl((int)(bits >> 32), j) << 32) |
                                       (uint32_t)__shfl((int)(uint32_t)bits, j);
                T factor;
                __builtin_memcpy(&factor, &other, sizeof(T));
                prod = mul_elem<T>(prod, factor);
              }
              if (lane == leader) atomic_rmw<T>(p, [prod](T cur) { return mul_elem<T>(cur, prod); });
              todo &= ~same;
            }
          }
        }
      }
    }
  }
}

// packed-pair add for 16-bit floats: two neighbouring columns in one atomic
// (requires K even, one index per row, 4-byte aligned src/out)
template <typename T>
__global__ __launch_bounds__(kBlock) void scatter_add_pk16_kernel(ScatterArgs a) {
  if (a.skip_flag != nullptr && *a.skip_flag != 0) return;
  const T *src = static_cast<const T *>(a.src);
  T *out = static_cast<T *>(a.out);
  const int64_t kv = a.K / 2;
  const EdgeLanes m = edge_lanes(kv, kBlock);
  if (!m.active) return;
  const int64_t n_edges = a.B * a.E;
  for (int64_t be = (int64_t)blockIdx.x * m.epp + m.el; be < n_edges; be += (int64_t)gridDim.x * m.epp) {
    int64_t b, e;
    split_edge(be, a.B, a.E, b, e);
    const int64_t idx = a.index[b * a.sb + e * a.se];
    if (idx < 0 || idx >= a.N) continue;
    for (int64_t cv = m.cl; cv < kv; cv += m.L) {
      const int64_t k0 = cv * 2;
      T *p = out + (b * a.N + idx) * a.K + k0;
      const T *q = src + be * a.K + k0;
      if constexpr (__is_same(T, bf16_t)) {
        typedef short v2s __attribute__((ext_vector_type(2)));
        __builtin_amdgcn_global_atomic_fadd_v2bf16(reinterpret_cast<v2s *>(p), *reinterpret_cast<const v2s *>(q));
      } else {
        typedef _Float16 v2h __attribute__((ext_vector_type(2)));
        __builtin_amdgcn_global_atomic_fadd_v2f16(reinterpret_cast<v2h *>(p), *reinterpret_cast<const v2h *>(q));
      }
    }
  }
}

// ---- wavefront pre-reduction of equal neighbouring indices -------------------------
// Message-passing indices are sorted or nearly so: neighbouring entries address the
// same output row, and one atomic per element would serialise them on one cache
// line. Here a wavefront owns a contiguous range of entries and reads it row by
// row (64 / L entries of L lanes each, C columns = up to 16 bytes per lane, fully
// coalesced). Runs of equal node ids inside a row are combined across lanes with
// shuffles; the run that reaches the end of a row is carried in registers into the
// next row instead of being written, so a run of any length costs one atomic per
// element and wavefront. An index without repeats degenerates to one atomic per
// element. Finished runs go through a per-wavefront LDS buffer so that the atomics
// of one instruction fall on consecutive addresses (whole cache lines) although a
// lane holds C neighbouring columns. One index per row (sk == 0) and B * N < 2^31
// are required.
//
// The policy P supplies the value type and its operations:
//   P::A, P::C, P::EW          accumulator type, columns per lane, columns per atomic
//   load(e, pos, col, node, x) x[0..C) = columns col.. of entry e (position pos inside its batch,
//                              output row node or -1)
//   combine(x, y)              x = x (op) y, one column
//   identity()
//   emit(node, col, x)         combine EW columns x[0..EW) into the output slot with one atomic
//   begin_row(heads, entries)  called once per wavefront row of more than one entry, before the
//                              emissions of its finished runs: number of runs and of entries in it
// (bx, by: the workgroup's place in the grid of this reduction, blockIdx for a kernel that holds nothing else)
template <typename P>
__device__ __forceinline__ void run_reduce_wave(const ScatterArgs &a, const int lshift, const int rows_per_wave,
                                                P &p, typename P::A *stage, const unsigned bx, const unsigned by) {
  typedef typename P::A A;
  constexpr int U = P::U;
  constexpr int C = P::C;
  constexpr int EW = P::EW;
  constexpr int cshift = C == 1 ? 0 : (C == 2 ? 1 : (C == 4 ? 2 : (C == 8 ? 3 : 4)));
  static_assert((1 << cshift) == C && C % EW == 0, "");
  const int lane = threadIdx.x & (kWave - 1);
  const int L = 1 << lshift;       // lanes per entry
  const int epr = kWave >> lshift; // entries per wavefront row
  const int el = lane >> lshift;
  const int cl = lane & (L - 1);
  const int64_t colbase = (int64_t)by * (L * C);
  const int64_t col = colbase + cl * C;
  const bool col_ok = col < a.K;
  const int64_t n_edges = a.B * a.E;
  const int64_t wave = (int64_t)bx * (kBlock / kWave) + (threadIdx.x / kWave);
  const int64_t lo = wave * rows_per_wave * epr;
  int64_t hi = lo + (int64_t)rows_per_wave * epr;
  if (hi > n_edges) hi = n_edges;
  if (lo >= hi) return;
  // bit 0 of every entry slot of the wavefront
  const uint64_t slot_bits = L == kWave ? 1ull : ~0ull / ((1ull << L) - 1ull);

  // Write the slots named in `mask` (bit slot * L) to the output: node id per lane in n,
  // values in v. Lanes re-read the values from LDS so that consecutive lanes hold
  // consecutive columns of one slot.
  auto write_slots = [&](const uint64_t mask, const int n, const A *v) {
    if constexpr (C == EW) {  // one atomic per lane: consecutive lanes already hold consecutive columns
      if (((mask >> (el << lshift)) & 1ull) && col_ok) p.emit(n, col, v);
      return;
    }
    __builtin_amdgcn_fence(__ATOMIC_ACQ_REL, "wavefront");  // earlier reads of the buffer are done
#pragma unroll
    for (int c = 0; c < C; ++c) stage[lane * C + c] = v[c];
    __builtin_amdgcn_fence(__ATOMIC_ACQ_REL, "wavefront");
    __builtin_amdgcn_wave_barrier();
#pragma unroll
    for (int it = 0; it < C / EW; ++it) {
      const int f = (lane + kWave * it) * EW;          // element of the wavefront row
      const int slot = f >> (lshift + cshift);
      const int j = f & ((L << cshift) - 1);           // column inside the slot
      const int node = __shfl(n, slot << lshift);
      if (((mask >> (slot << lshift)) & 1ull) && colbase + j < a.K) p.emit(node, colbase + j, stage + f);
    }
  };

  A carry[C];
#pragma unroll
  for (int c = 0; c < C; ++c) carry[c] = p.identity();
  int carry_node = -1;

  for (int64_t r0 = lo; r0 < hi; r0 += (int64_t)U * epr) {
    int node[U];
    A x[U][C];
#pragma unroll
    for (int u = 0; u < U; ++u) {
      const int64_t e = r0 + (int64_t)u * epr + el;
      const bool ok = e < hi;
      const int64_t ec = ok ? e : hi - 1;
      int64_t b, pos;
      split_edge(ec, a.B, a.E, b, pos);
      const int64_t idx = a.index[b * a.sb + pos * a.se];
      node[u] = (ok && idx >= 0 && idx < a.N) ? (int)(b * a.N + idx) : -1;
      p.load(ec, pos, col_ok ? col : 0, node[u], x[u]);
    }
#pragma unroll
    for (int u = 0; u < U; ++u) {
      if (r0 + (int64_t)u * epr >= hi) break;  // uniform
      const int n = node[u];
      A v[C];
#pragma unroll
      for (int c = 0; c < C; ++c) v[c] = x[u][c];
      // the run carried over from the previous row continues in slot 0, or is written now
      const int n0 = __builtin_amdgcn_readfirstlane(n);
      if (carry_node == n0) {
        if (el == 0) {
#pragma unroll
          for (int c = 0; c < C; ++c) p.combine(v[c], carry[c]);
        }
      } else if (carry_node >= 0) {
        write_slots(1ull, carry_node, carry);
      }
      int h_slot = 0;
      if (epr > 1) {
        const int prev = __shfl_up(n, L);
        const bool head = (el == 0) || (n != prev);
        const uint64_t hm = __ballot(head) & slot_bits;
        p.begin_row(__popcll(hm), epr);
        // slots from this one to the end of its run
        const uint64_t after = (el + 1 < epr) ? (hm >> ((el + 1) << lshift)) : 0ull;
        const int rem = after ? ((__ffsll((unsigned long long)after) - 1) >> lshift) + 1 : epr - el;
        if (hm != slot_bits) {  // a row without equal neighbours has nothing to combine
          for (int d = 1; d < epr; d <<= 1) {
#pragma unroll
            for (int c = 0; c < C; ++c) {
              const A t = __shfl_down(v[c], d << lshift);
              if (d < rem) p.combine(v[c], t);
            }
          }
        }
        h_slot = (63 - __clzll((long long)hm)) >> lshift;  // head of the last run of the row
        // heads of finished runs with a valid node
        const uint64_t em = __ballot(head && el != h_slot && n >= 0) & slot_bits;
        if (em != 0) write_slots(em, n, v);
      }
      carry_node = __shfl(n, h_slot << lshift);
#pragma unroll
      for (int c = 0; c < C; ++c) carry[c] = __shfl(v[c], (h_slot << lshift) + cl);
    }
  }
  if (carry_node >= 0) write_slots(1ull, carry_node, carry);
}

// The same reduction for rows of 8 and more lanes (128 bytes and up per entry): with so few entries per
// wavefront row the shuffles of the scheme above cost more than the loads. Here every entry slot of the
// wavefront walks its OWN contiguous part of the wavefront's range, one entry per step, and keeps the
// running value of its current run in registers: equal neighbours cost one add per column and no
// cross-lane traffic at all; a run is written when the node id changes (through the same LDS transposition,
// for all slots that changed in that step at once). Each slot reads 128 bytes or more of one entry per
// load, so the memory system still sees whole lines. Runs cut at the border between two slots' parts cost
// one extra atomic.
template <typename P>
__device__ __forceinline__ void run_serial_wave(const ScatterArgs &a, const int lshift, const int rows_per_wave,
                                                P &p, typename P::A *stage, const unsigned bx, const unsigned by) {
  typedef typename P::A A;
  constexpr int U = P::U;
  constexpr int C = P::C;
  constexpr int EW = P::EW;
  constexpr int cshift = C == 1 ? 0 : (C == 2 ? 1 : (C == 4 ? 2 : (C == 8 ? 3 : 4)));
  const int lane = threadIdx.x & (kWave - 1);
  const int L = 1 << lshift;
  const int epr = kWave >> lshift;  // entry slots of the wavefront
  const int el = lane >> lshift;
  const int cl = lane & (L - 1);
  const int64_t colbase = (int64_t)by * (L * C);
  const int64_t col = colbase + cl * C;
  const bool col_ok = col < a.K;
  const int64_t n_edges = a.B * a.E;
  const int64_t wave = (int64_t)bx * (kBlock / kWave) + (threadIdx.x / kWave);
  const int64_t lo = wave * rows_per_wave * epr;
  int64_t hi = lo + (int64_t)rows_per_wave * epr;
  if (hi > n_edges) hi = n_edges;
  if (lo >= hi) return;
  const int64_t s_lo = lo + (int64_t)el * rows_per_wave;  // this slot's part
  const int64_t s_hi = s_lo + rows_per_wave < hi ? s_lo + rows_per_wave : hi;
  const uint64_t slot_bits = L == kWave ? 1ull : ~0ull / ((1ull << L) - 1ull);

  auto write_slots = [&](const uint64_t mask, const int n, const A *v) {
    if constexpr (C == EW) {
      if (((mask >> (el << lshift)) & 1ull) && col_ok) p.emit(n, col, v);
      return;
    }
    __builtin_amdgcn_fence(__ATOMIC_ACQ_REL, "wavefront");
#pragma unroll
    for (int c = 0; c < C; ++c) stage[lane * C + c] = v[c];
    __builtin_amdgcn_fence(__ATOMIC_ACQ_REL, "wavefront");
    __builtin_amdgcn_wave_barrier();
#pragma unroll
    for (int it = 0; it < C / EW; ++it) {
      const int f = (lane + kWave * it) * EW;
      const int slot = f >> (lshift + cshift);
      const int j = f & ((L << cshift) - 1);
      const int node = __shfl(n, slot << lshift);
      if (((mask >> (slot << lshift)) & 1ull) && colbase + j < a.K) p.emit(node, colbase + j, stage + f);
    }
  };

  A acc[C];
#pragma unroll
  for (int c = 0; c < C; ++c) acc[c] = p.identity();
  int cur = -1;
  for (int r0 = 0; r0 < rows_per_wave; r0 += U) {
    int node[U];
    A x[U][C];
#pragma unroll
    for (int u = 0; u < U; ++u) {
      const int64_t e = s_lo + r0 + u;
      const bool ok = e < s_hi;
      const int64_t ec = ok ? e : hi - 1;
      int64_t b, pos;
      split_edge(ec, a.B, a.E, b, pos);
      const int64_t idx = a.index[b * a.sb + pos * a.se];
      node[u] = (ok && idx >= 0 && idx < a.N) ? (int)(b * a.N + idx) : -1;
      p.load(ec, pos, col_ok ? col : 0, node[u], x[u]);
    }
#pragma unroll
    for (int u = 0; u < U; ++u) {
      if (r0 + u >= rows_per_wave) break;  // uniform
      const int n = node[u];
      const bool change = n != cur;
      p.begin_row(__popcll(__ballot(change) & slot_bits), epr);
      const uint64_t em = __ballot(change && cur >= 0) & slot_bits;
      if (em != 0) write_slots(em, cur, acc);
      if (change) {
        cur = n;
#pragma unroll
        for (int c = 0; c < C; ++c) acc[c] = x[u][c];
      } else {
#pragma unroll
        for (int c = 0; c < C; ++c) p.combine(acc[c], x[u][c]);
      }
    }
  }
  // what is left in the slots are runs cut by the end of a part; for a hub they all belong to one node,
  // so they go out like the entries of an unsorted index (table of hot rows, read before the atomic)
  p.begin_row(epr, epr);
  const uint64_t em = __ballot(cur >= 0) & slot_bits;
  if (em != 0) write_slots(em, cur, acc);
}

// the scheme by row width: shuffles for narrow rows, one slot per part of the range from 128 bytes per
// entry (lane_bytes = bytes of src a lane loads per entry)
__host__ __device__ inline bool run_is_serial(int lshift, int lane_bytes) { return (lane_bytes << lshift) >= 128; }
// (a kernel holds one of the two: with both behind a run-time branch the small latency-bound launches
// were 3 us slower, whichever branch they took)
template <bool SERIAL, typename P>
__device__ __forceinline__ void run_wave(const ScatterArgs &a, const int lshift, const int rows_per_wave, P &p,
                                         typename P::A *stage, const unsigned bx, const unsigned by) {
  if constexpr (SERIAL)
    run_serial_wave(a, lshift, rows_per_wave, p, stage, bx, by);
  else
    run_reduce_wave(a, lshift, rows_per_wave, p, stage, bx, by);
}
template <bool SERIAL, typename P>
__device__ __forceinline__ void run_wave(const ScatterArgs &a, const int lshift, const int rows_per_wave, P &p,
                                         typename P::A *stage) {
  run_wave<SERIAL>(a, lshift, rows_per_wave, p, stage, blockIdx.x, blockIdx.y);
}

// ---- hot rows of a workgroup ------------------------------------------------------
// An unsorted index with a hub (a node that owns 1 % or more of the entries, as in
// power-law graphs) puts every entry of the hub on one address: about 10 ns per
// atomic, one after the other (measured: 10 M entries with a 20 % hub take 20 ms
// instead of 0.5 ms). The sum kernels therefore keep a small LDS table of
// accumulator rows per workgroup. A row is handed to a node only when the node
// shows up twice in a row among the emissions that hash to it: a hub passes that
// test almost at once, the one-off nodes of a sorted or uniform index practically
// never do, so they cost one LDS read and keep going to memory directly. Confirmed
// rows never change owner; they are added to the output once, when the workgroup
// is done. Every value is added exactly once, either to its node's confirmed row
// or to memory.
constexpr int kHotAcc = 2048;                    // accumulators per workgroup
constexpr int kHotRowsMax = 512;
constexpr uint32_t kHotConfirmed = 0x80000000u;  // tag bit: the row belongs to the node for good
constexpr uint32_t kHotNone = 0x7FFFFFFFu;       // no candidate yet (node ids stay below 2^31 - 1)
template <typename A> struct HotOk { static constexpr bool value = sizeof(A) >= 4; };  // LDS atomics: 32 / 64 bits

// Slot type of the table: fp32 sums are kept in double slots. ds_add_f32 loses its rate when many lanes meet on one
// address, which is what a hub row is; ds_add_f64 and the integer adds keep theirs.
template <typename A> struct HotSlot { typedef A type; };
template <> struct HotSlot<float> { typedef double type; };

template <typename A> struct HotRows {
  typedef typename HotSlot<A>::type S;
  S *acc;          // [rows][1 << wshift]
  uint32_t *tags;  // [rows]
  int rlog;        // log2(rows), < 0: no table
  int wshift;      // log2 of the columns per row (the column chunk of the workgroup)
  __device__ int row_of(int node) const { return (int)(((uint32_t)node * 0x9E3779B1u) >> (32 - rlog)); }
  // true: x[0..EW) went into the workgroup's row of `node` at columns j..; false: the caller adds them to memory
  template <int EW> __device__ bool add(int node, int j, const A *x) const {
    if (rlog < 0) return false;
    const int row = row_of(node);
    const uint32_t mine = (uint32_t)node | kHotConfirmed;
    const uint32_t t = __hip_atomic_load(&tags[row], __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_WORKGROUP);
    if (t != mine) {
      // only the lane of column 0 moves the tag, so the other columns of one entry cannot confirm it
      if ((t & kHotConfirmed) || j != 0) return false;
      if (t != (uint32_t)node) {  // remember as the candidate
        atomicCAS(&tags[row], t, (uint32_t)node);
        return false;
      }
      const uint32_t old = atomicCAS(&tags[row], t, mine);  // second time in a row: confirm
      if (old != t && old != mine) return false;
    }
#pragma unroll
    for (int w = 0; w < EW; ++w)
      __hip_atomic_fetch_add(&acc[(row << wshift) + j + w], (S)x[w], __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_WORKGROUP);
    return true;
  }
  __device__ void clear() const {
    if (rlog < 0) return;
    for (int i = threadIdx.x; i < (1 << (rlog + wshift)); i += blockDim.x) acc[i] = (S)0;
    for (int i = threadIdx.x; i < (1 << rlog); i += blockDim.x) tags[i] = kHotNone;
    __syncthreads();
  }
  // add the confirmed rows to the output: emit(node, column inside the chunk, EW accumulators)
  template <int EW, typename F> __device__ void flush(F emit) const {
    if (rlog < 0) return;
    __syncthreads();
    for (int i = threadIdx.x * EW; i < (1 << (rlog + wshift)); i += blockDim.x * EW) {
      const uint32_t t = tags[i >> wshift];
      if (!(t & kHotConfirmed)) continue;
      bool any = false;
      A x[EW];
#pragma unroll
      for (int w = 0; w < EW; ++w) {
        x[w] = (A)acc[i + w];
        any = any || acc[i + w] != (S)0;
      }
      if (any) emit((int)(t & ~kHotConfirmed), i & ((1 << wshift) - 1), x);
    }
  }
};
// log2 of the rows of the table for column chunks of 1 << wshift columns; -1: chunk too wide for a table
inline int hot_rows_log(int wshift) {
  int rlog = 0;
  while ((2 << rlog) <= kHotRowsMax && ((2 << rlog) << wshift) <= kHotAcc) ++rlog;
  return rlog >= 3 ? rlog : -1;
}

// What a sum policy keeps to use the table. Rows of the wavefront in which at least half of the
// entries continue a run look sorted: their few emissions go to memory directly and the table costs
// them nothing. (Hub entries sprinkled over an otherwise sorted index are not caught that way.)
template <typename A> struct HotState {
  HotRows<A> hot;
  int64_t colbase;  // first column of the workgroup's chunk
  bool active;
  __device__ void hot_init(typename HotSlot<A>::type *acc, uint32_t *tags, int rlog, int wshift) {
    hot.acc = acc;
    hot.tags = tags;
    hot.rlog = HotOk<A>::value ? rlog : -1;
    hot.wshift = wshift;
    colbase = (int64_t)blockIdx.y << wshift;
    active = true;
    hot.clear();
  }
  __device__ void begin_row(int heads, int entries) { active = heads * 2 > entries; }
  template <int EW> __device__ bool to_table(int node, int64_t col, const A *x) {
    if constexpr (HotOk<A>::value) return active && hot.template add<EW>(node, (int)(col - colbase), x);
    return false;
  }
};

// sum: up to 16 bytes per lane; 16-bit floats accumulate in fp32 and are written
// with the packed-pair atomic. src == nullptr adds 1 per entry (the count of scatter mean).
// EW_ = columns per atomic: a whole 32-bit word for element types below 32 bits, or 1 (rows whose
// length or alignment rules that out; the element then goes through a compare-and-swap on its word)
template <typename T, int C_, int EW_ = (sizeof(T) < 4 ? 4 / (int)sizeof(T) : 1), bool HOT = true>
struct AddRun : HotState<typename Acc<T>::type> {
  typedef typename Acc<T>::type A;
  typedef T Elem;
  static constexpr int C = C_;
  static constexpr int EW = EW_;
  static constexpr int U = 4;
  const T *src;
  T *out;
  const T *out_end;
  int64_t K;
  __device__ A identity() const { return (A)0; }
  __device__ void load(int64_t e, int64_t, int64_t col, int, A *x) const {
    if (src == nullptr) {
#pragma unroll
      for (int c = 0; c < C; ++c) x[c] = (A)1;
      return;
    }
    const Vec<T, C> r = load_vec_stream<T, C>(src + e * K + col);
#pragma unroll
    for (int c = 0; c < C; ++c) x[c] = to_acc<T>(r.v[c]);
  }
  __device__ void combine(A &x, const A &y) const { x = x + y; }
  __device__ void begin_row(int heads, int entries) {
    if constexpr (HOT) HotState<A>::begin_row(heads, entries);
  }
  __device__ void emit(int node, int64_t col, const A *x) {
    if constexpr (HOT) {
      if (this->template to_table<EW>(node, col, x)) return;
    }
    to_memory(node, col, x);
  }
  __device__ void to_memory(int node, int64_t col, const A *x) const {
    T *p = out + (int64_t)node * K + col;
    if constexpr (EW > 1 && std::is_integral<T>::value && sizeof(T) < 4) {
      // 8- and 16-bit integers: one compare-and-swap on the 32-bit word that holds EW neighbouring columns
      // (a CAS per element would make the lanes of one word fight each other)
      typedef typename std::make_unsigned<T>::type UT;
      constexpr int bits = 8 * (int)sizeof(T);
      uint32_t *word = reinterpret_cast<uint32_t *>(p);
      uint32_t old = __hip_atomic_load(word, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
      while (true) {
        uint32_t nw = 0;
#pragma unroll
        for (int j = 0; j < EW; ++j) {
          const T cur = (T)(UT)(old >> (bits * j));
          const T nv = (T)(cur + x[j]);
          nw |= (uint32_t)(UT)nv << (bits * j);
        }
        if (nw == old) return;
        if (__hip_atomic_compare_exchange_strong(word, &old, nw, __ATOMIC_RELAXED, __ATOMIC_RELAXED,
                                                 __HIP_MEMORY_SCOPE_AGENT))
          return;
      }
    } else if constexpr (EW == 2) {
      if constexpr (__is_same(T, bf16_t)) {
        typedef short v2s __attribute__((ext_vector_type(2)));
        v2s pk;
        pk.x = (short)float_to_bf16(x[0]).x;
        pk.y = (short)float_to_bf16(x[1]).x;
        __builtin_amdgcn_global_atomic_fadd_v2bf16(reinterpret_cast<v2s *>(p), pk);
      } else {
        typedef _Float16 v2h __attribute__((ext_vector_type(2)));
        v2h pk;
        pk.x = (_Float16)x[0];
        pk.y = (_Float16)x[1];
        __builtin_amdgcn_global_atomic_fadd_v2f16(reinterpret_cast<v2h *>(p), pk);
      }
    } else if constexpr (__is_same(T, bf16_t) || __is_same(T, f16_t)) {
      atomic_add_half<T>(p, from_acc<T>(x[0]), out, out_end);
    } else {
      atomic_add_elem<T>(p, from_acc<T>(x[0]));
    }
  }
};

template <int C> struct LogC { static constexpr int value = C == 1 ? 0 : (C == 2 ? 1 : (C == 4 ? 2 : (C == 8 ? 3 : 4))); };

// HOT = false: the variant for inputs too small for the table to pay (its code and LDS cost a
// latency-bound launch about a microsecond even when it is switched off at run time)
template <typename T, int C, int EW, bool SERIAL, bool HOT>
__global__ __launch_bounds__(kBlock) void scatter_add_run_kernel(ScatterArgs a, int lshift, int rows_per_wave,
                                                                 int hot_rlog) {
  typedef typename Acc<T>::type A;
  constexpr bool kTable = HOT && HotOk<A>::value;
  if (a.skip_flag != nullptr && *a.skip_flag != 0) return;
  __shared__ A s_stage[kBlock / kWave][kWave * C];
  __shared__ typename HotSlot<A>::type s_hot[kTable ? kHotAcc : 1];
  __shared__ uint32_t s_tags[kTable ? kHotRowsMax : 1];
  AddRun<T, C, EW, kTable> p;
  p.src = static_cast<const T *>(a.src);
  p.out = static_cast<T *>(a.out);
  p.out_end = p.out + a.B * a.N * a.K;
  p.K = a.K;
  if constexpr (kTable) p.hot_init(s_hot, s_tags, hot_rlog, lshift + LogC<C>::value);
  run_wave<SERIAL>(a, lshift, rows_per_wave, p, s_stage[threadIdx.x / kWave]);
  if constexpr (kTable) {
    p.hot.template flush<EW>([&](int node, int j, const A *x) {
      if (p.colbase + j < p.K) p.to_memory(node, p.colbase + j, x);
    });
  }
}


// scatter mean of a small input, where the launches are the cost (five of 3 us each: out cleared, sum, counts
// cleared, count, divide): one launch clears out and the counts, one launch adds and counts -- the first sum_blocks
// workgroups along x are the grid of scatter_add_run_kernel, the workgroups behind them (first column chunk only) that
// of the count, a sum of ones into int32 through the same run reduction.
template <typename T>
__global__ __launch_bounds__(kBlock) void fill_out_count_kernel(T *out, int64_t n_out, int32_t *count, int64_t n_count) {
  for (int64_t i = (int64_t)blockIdx.x * kBlock + threadIdx.x; i < n_out + n_count; i += (int64_t)gridDim.x * kBlock) {
    if (i < n_out)
      out[i] = small_const<T>(0);
    else
      count[i - n_out] = 0;
  }
}
template <typename T, int C, int EW, bool SERIAL>
__global__ __launch_bounds__(kBlock) void scatter_add_count_run_kernel(ScatterArgs a, int lshift, int rows_per_wave,
                                                                       ScatterArgs cnt, int count_rows_per_wave,
                                                                       unsigned sum_blocks) {
  typedef typename Acc<T>::type A;
  __shared__ A s_stage[kBlock / kWave][kWave * C];
  if (blockIdx.x < sum_blocks) {
    AddRun<T, C, EW, false> p;
    p.src = static_cast<const T *>(a.src);
    p.out = static_cast<T *>(a.out);
    p.out_end = p.out + a.B * a.N * a.K;
    p.K = a.K;
    run_wave<SERIAL>(a, lshift, rows_per_wave, p, s_stage[threadIdx.x / kWave], blockIdx.x, blockIdx.y);
  } else if (blockIdx.y == 0) {
    AddRun<int32_t, 1, 1, false> q;
    q.src = nullptr;  // adds 1 per entry
    q.out = static_cast<int32_t *>(cnt.out);
    q.out_end = q.out + cnt.B * cnt.N;
    q.K = 1;
    // (one column per lane and atomic: the staging buffer is not used)
    run_reduce_wave(cnt, 0, count_rows_per_wave, q, static_cast<typename AddRun<int32_t, 1, 1, false>::A *>(nullptr),
                    blockIdx.x - sum_blocks, 0u);
  }
}

// rows of a wavefront in the kernel above: long enough to carry runs across rows, short enough to
// leave ~8 K wavefronts
inline int run_rows_per_wave(int64_t n_edges, int epr, int cap = 32) {
  const int64_t rows = (n_edges + epr - 1) / epr;
  int64_t rpw = rows / 8192;
  if (rpw > cap) rpw = cap;
  if (rpw < 1) rpw = 1;
  if (const char *env = getenv("TS_RUN_RPW")) rpw = atoi(env) > 0 ? atoi(env) : rpw;  // tuning aid
  return (int)(rpw <= 4 ? rpw : (rpw + 3) / 4 * 4);
}
// launch shape of the run kernels for rows of `kc` lanes
struct RunGrid {
  int lshift, rpw;
  unsigned blocks, ychunks;
  bool ok;
  int hot_rlog;  // log2 of the rows of the hot-row table, -1: none
  bool serial;   // run_serial_wave instead of run_reduce_wave
};
// launches the SERIAL = true or false instantiation of a run kernel named by the macro arguments
#define TS_LAUNCH_RUN(SERIAL_FLAG, KERNEL_T, KERNEL_F, GRID, STREAM, ...)                      \
  do {                                                                                         \
    if (SERIAL_FLAG)                                                                           \
      hipLaunchKernelGGL(KERNEL_T, GRID, dim3(kBlock), 0, STREAM, __VA_ARGS__);                \
    else                                                                                       \
      hipLaunchKernelGGL(KERNEL_F, GRID, dim3(kBlock), 0, STREAM, __VA_ARGS__);                \
  } while (0)
// c > 0: a sum kernel with c columns per lane that may keep a hot-row table. The table pays once a
// workgroup sees enough entries for a hub to repeat: large inputs, with longer ranges per wavefront.
// launches the instantiation of scatter_add_run_kernel for (serial, hot)
template <typename T, int C, int EW>
void launch_add_run(const ScatterArgs &a, const RunGrid &g, hipStream_t stream) {
  const dim3 gd(g.blocks, g.ychunks);
  if (g.hot_rlog >= 0)
    TS_LAUNCH_RUN(g.serial, (scatter_add_run_kernel<T, C, EW, true, true>), (scatter_add_run_kernel<T, C, EW, false, true>),
                  gd, stream, a, g.lshift, g.rpw, g.hot_rlog);
  else
    TS_LAUNCH_RUN(g.serial, (scatter_add_run_kernel<T, C, EW, true, false>),
                  (scatter_add_run_kernel<T, C, EW, false, false>), gd, stream, a, g.lshift, g.rpw, g.hot_rlog);
}
inline RunGrid run_grid(int64_t n_edges, int64_t kc, int c, int lane_bytes) {
  RunGrid g;
  g.lshift = 0;
  while ((1 << g.lshift) < kc && g.lshift < 6) ++g.lshift;
  const int L = 1 << g.lshift, epr = kWave >> g.lshift;
  g.hot_rlog = -1;
  // The table from 2^18 entries on; for rows of 128 bytes and more from 2^15. Below, a hub serialises the atomics of
  // its row (Zipf(1.2) index, 32 k - 262 k entries of 32 / 64 floats: 120 - 1040 us without the table, 42 - 270 us
  // with it), while a uniform index pays the tag look-ups (+10-18 %, 3-7 us at these sizes). Narrower rows keep 2^18:
  // 200 k entries of 16 floats under a uniform index 16.4 us without, 22.7 us with the table (536 against 159 us
  // under the Zipf index). These sizes now matter for the element types and strided indices that
  // scatter_add_lds_kernel does not take (see sum_table_by_size).
  int64_t hot_min = run_is_serial(g.lshift, lane_bytes) ? (int64_t)1 << 15 : (int64_t)1 << 18;
  if (const char *env = getenv("TS_SCATTER_HOT_MIN")) hot_min = atoll(env);  // tuning aid
  if (c > 0 && n_edges >= hot_min && !getenv("TS_SCATTER_NO_HOT")) {  // env: tuning aid
    int cshift = 0;
    while ((1 << cshift) < c) ++cshift;
    g.hot_rlog = hot_rows_log(g.lshift + cshift);
  }
  // longer ranges where a workgroup should see a hub repeat, and where every slot walks its own part
  const bool serial = run_is_serial(g.lshift, lane_bytes);
  g.serial = serial;
  g.rpw = run_rows_per_wave(n_edges, epr, serial || g.hot_rlog >= 0 ? 64 : 32);
  // a slot only combines what lies inside its own part: keep the parts at 16 entries or more -- but not for small
  // inputs, where a part is a chain of dependent reads and atomics and 16 of them are the whole call (min / max
  // of 8192 entries of 32 floats: 42 us with parts of 16, 15 us with parts of 4; sums 11 us either way)
  // Sums keep 16 from 2^17 entries on (a sorted index combines more per part: 262 k entries of 32 floats 24 us with
  // parts of 16, 35 us with parts of 4); min / max have nothing to combine before the keys and want 16 k wavefronts
  // first (131 k / 262 k entries of 32 floats onto 100 k rows: 71 / 85 us with parts of 16, 48 / 72 us with 4 / 8).
  const int64_t ychunks = (kc + L - 1) / L;
  if (serial && !getenv("TS_RUN_RPW")) {
    int floor_rpw = n_edges < ((int64_t)1 << 17) ? 4 : 16;
    if (c == 0) {
      const int64_t wave_rows = (n_edges + epr - 1) / epr * ychunks;
      floor_rpw = wave_rows >= 16 * 16384 ? 16 : wave_rows >= 8 * 16384 ? 8 : 4;
    }
    if (g.rpw < floor_rpw) g.rpw = floor_rpw;
  }
  const int64_t waves = (n_edges + (int64_t)g.rpw * epr - 1) / ((int64_t)g.rpw * epr);
  const int64_t blocks = (waves + kBlock / kWave - 1) / (kBlock / kWave);
  g.ok = blocks < 0x7FFFFFFFll && ychunks <= 65535;
  g.blocks = (unsigned)blocks;
  g.ychunks = (unsigned)ychunks;
  return g;
}

// ---- packed-key min/max -----------------------------------------------------
template <typename T, bool IS_MAX>
__global__ __launch_bounds__(kBlock) void scatter_key_init_kernel(ScatterArgs a) {
  const int64_t n = a.B * a.N * a.K;
  const T *out = static_cast<const T *>(a.out);
  uint64_t *keys = reinterpret_cast<uint64_t *>(a.arg_out);
  for (int64_t i = (int64_t)blockIdx.x * kBlock + threadIdx.x; i < n; i += (int64_t)gridDim.x * kBlock) {
    uint64_t k;
    if (a.out_given) {
      const T prev = out[i];
      // a NaN already in out can never be beaten (comparisons with it are false)
      k = Key<T>::is_nan(prev) ? ~(uint64_t)0 : pack_key<T, IS_MAX>(prev, kKeepLow);
    } else {
      k = pack_key<T, IS_MAX>(IS_MAX ? ElemLim<T>::lowest() : ElemLim<T>::max(), kKeepLow);
    }
    keys[i] = k;
  }
}

// keys of one lane's VEC columns against the global table: read the current
// keys first (one vector load), then issue atomics only for the improvements
template <int VEC>
__device__ __forceinline__ void keys_to_global(uint64_t *p, const uint64_t *key, int precheck) {
  uint64_t cur[VEC];
  if (precheck != 0) {
#pragma unroll
    for (int v = 0; v < VEC; ++v) {
      if (precheck == 2)
        cur[v] = __hip_atomic_load(p + v, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
      else if (precheck == 3)
        cur[v] = __builtin_nontemporal_load(p + v);
      else
        cur[v] = p[v];  // cached read: a stale value only costs a spare atomic
    }
  }
#pragma unroll
  for (int v = 0; v < VEC; ++v) {
    if (key[v] == 0) continue;  // nothing to contribute (NaN or index out of range)
    if (precheck != 0 && key[v] <= cur[v]) continue;
    __hip_atomic_fetch_max(p + v, key[v], __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
  }
}

// keys of the VEC columns a lane holds for one edge; 0 = nothing to contribute
template <typename T, int VEC, bool IS_MAX>
__device__ __forceinline__ void make_keys(const Vec<T, VEC> &x, int64_t e, uint64_t *key) {
  const uint32_t low = 0xFFFFFFFEu - (uint32_t)e;
#pragma unroll
  for (int v = 0; v < VEC; ++v)
    key[v] = Key<T>::is_nan(x.v[v]) ? 0 : pack_key<T, IS_MAX>(x.v[v], low);  // NaN never wins
}

// straight to the global table (per-element index, small inputs, very wide rows)
template <typename T, int VEC, bool IS_MAX>
__global__ __launch_bounds__(kBlock) void scatter_key_kernel(ScatterArgs a) {
  constexpr int U = 4;
  const T *src = static_cast<const T *>(a.src);
  uint64_t *keys = reinterpret_cast<uint64_t *>(a.arg_out);
  const int64_t kv = a.K / VEC;
  const EdgeLanes m = edge_lanes(kv, kBlock);
  if (!m.active) return;
  const int64_t n_edges = a.B * a.E;
  const int64_t stride = (int64_t)gridDim.x * m.epp;
  for (int64_t be0 = (int64_t)blockIdx.x * m.epp + m.el; be0 < n_edges; be0 += stride * U) {
    for (int64_t cv = m.cl; cv < kv; cv += m.L) {
      const int64_t k0 = cv * VEC;
      Vec<T, VEC> x[U];
      int64_t idx[U], bb[U], ee[U];
#pragma unroll
      for (int u = 0; u < U; ++u) {
        const int64_t be = be0 + u * stride;
        split_edge(be < n_edges ? be : be0, a.B, a.E, bb[u], ee[u]);  // re-doing an edge is harmless under max
        x[u] = load_vec_stream<T, VEC>(src + (bb[u] * a.E + ee[u]) * a.K + k0);
        idx[u] = a.index[bb[u] * a.sb + ee[u] * a.se + k0 * a.sk];
      }
#pragma unroll
      for (int u = 0; u < U; ++u) {
        uint64_t key[VEC];
        make_keys<T, VEC, IS_MAX>(x[u], ee[u], key);
        if (a.sk == 0) {
          if (idx[u] < 0 || idx[u] >= a.N) continue;
          keys_to_global<VEC>(keys + (bb[u] * a.N + idx[u]) * a.K + k0, key, a.precheck);
        } else {
#pragma unroll
          for (int v = 0; v < VEC; ++v) {
            const int64_t id = v == 0 ? idx[u] : a.index[bb[u] * a.sb + ee[u] * a.se + (k0 + v) * a.sk];
            if (id < 0 || id >= a.N) continue;
            keys_to_global<1>(keys + (bb[u] * a.N + id) * a.K + k0 + v, key + v, a.precheck);
          }
        }
      }
    }
  }
}

// packed keys with the wavefront pre-reduction of run_reduce_wave: the largest key of a run of equal
// neighbouring indices goes to the table with one read and at most one atomic
template <typename T, int C_, bool IS_MAX>
struct KeyRun {
  typedef uint64_t A;
  typedef T Elem;
  static constexpr int C = C_;
  static constexpr int EW = 1;
  static constexpr int U = 4;
  const T *src;
  uint64_t *keys;
  int64_t K;
  int precheck;
  __device__ A identity() const { return 0; }
  __device__ void load(int64_t e, int64_t pos, int64_t col, int, A *x) const {
    const Vec<T, C> r = load_vec_stream<T, C>(src + e * K + col);
    make_keys<T, C, IS_MAX>(r, pos, x);
  }
  __device__ void combine(A &x, const A &y) const { x = x > y ? x : y; }
  // The read before the atomic pays where a slot collects many entries that do not sit next to each
  // other (a hub in an unsorted index). In a row of the wavefront in which at least half of the
  // entries continue a run the index looks sorted: one atomic per slot anyway, and the read would
  // only make the wavefront wait for memory.
  bool check = true;
  __device__ void begin_row(int heads, int entries) { check = heads * 2 > entries; }
  __device__ void emit(int node, int64_t col, const A *x) const {
    keys_to_global<1>(keys + (int64_t)node * K + col, x, check ? precheck : 0);
  }
};

template <typename T, int C, bool IS_MAX, bool SERIAL>
__global__ __launch_bounds__(kBlock) void scatter_key_run_kernel(ScatterArgs a, int lshift, int rows_per_wave) {
  __shared__ uint64_t s_stage[kBlock / kWave][kWave * C];
  if (a.skew_flag != nullptr && (*a.skew_flag != 0) != (a.skew_want != 0)) return;
  KeyRun<T, C, IS_MAX> p;
  p.src = static_cast<const T *>(a.src);
  p.keys = reinterpret_cast<uint64_t *>(a.arg_out);
  p.K = a.K;
  p.precheck = a.precheck;
  run_wave<SERIAL>(a, lshift, rows_per_wave, p, s_stage[threadIdx.x / kWave]);
}

// ---- packed-key min/max with a workgroup-private cache of hot slots ---------
// Skewed indices (a hub node owning 20 % of the entries) would serialise on a
// handful of global addresses. Each workgroup therefore reduces its chunk of
// entries into an LDS table first -- direct-mapped on the node id, one row of K
// keys per cached node, claimed with a compare-and-swap on the tag -- and only
// writes the per-node winners to global memory once per chunk. Entries whose
// table row is taken by another node go to global memory directly, after the
// same read-before-atomic test. One index per row is required (sk == 0).
constexpr int kLdsKeys = 4096;        // 32 KB of 64-bit keys
constexpr int kLdsBlock = 256;  // 3 workgroups per CU (LDS-limited) at <= 168 VGPRs

template <typename T, int VEC, bool IS_MAX, int TAGS>
__global__ __launch_bounds__(kLdsBlock, (TAGS <= 256 ? 4 : 1)) void scatter_key_lds_kernel(ScatterArgs a, int tn_mask, int64_t epb) {
  constexpr int U = VEC == 1 ? 8 : 4;
  __shared__ uint64_t s_keys[kLdsKeys];
  __shared__ int32_t s_tags[TAGS];  // TAGS >= table rows: kLdsKeys for narrow rows, 256 for K >= 16
  if (a.skew_flag != nullptr && (*a.skew_flag != 0) != (a.skew_want != 0)) return;
  const int K = (int)a.K;
  const int tn = tn_mask + 1;
  for (int i = threadIdx.x; i < tn * K; i += kLdsBlock) s_keys[i] = 0;
  for (int i = threadIdx.x; i < tn; i += kLdsBlock) s_tags[i] = -1;
  __syncthreads();

  const T *src = static_cast<const T *>(a.src);
  uint64_t *gkeys = reinterpret_cast<uint64_t *>(a.arg_out);
  const int kv = K / VEC;
  const EdgeLanes m = edge_lanes(kv, kLdsBlock);
  const int64_t be_lo = (int64_t)blockIdx.x * epb;
  int64_t be_hi = be_lo + epb;
  if (be_hi > a.B * a.E) be_hi = a.B * a.E;

  if (m.active) {
    for (int64_t be0 = be_lo + m.el; be0 < be_hi; be0 += (int64_t)m.epp * U) {
      for (int cv = m.cl; cv < kv; cv += m.L) {
        const int k0 = cv * VEC;
        Vec<T, VEC> x[U];
        int64_t idx[U], bb[U], ee[U];
#pragma unroll
        for (int u = 0; u < U; ++u) {
          const int64_t be = be0 + (int64_t)u * m.epp;
          split_edge(be < be_hi ? be : be0, a.B, a.E, bb[u], ee[u]);
          x[u] = load_vec_stream<T, VEC>(src + (bb[u] * a.E + ee[u]) * a.K + k0);
          idx[u] = a.index[bb[u] * a.sb + ee[u] * a.se];
        }
        uint64_t key[U][VEC];
        int64_t miss_node[U];
#pragma unroll
        for (int u = 0; u < U; ++u) {
          miss_node[u] = -1;
          if (idx[u] < 0 || idx[u] >= a.N) continue;
          make_keys<T, VEC, IS_MAX>(x[u], ee[u], key[u]);
          const int node = (int)(bb[u] * a.N + idx[u]);
          const int row = node & tn_mask;
          int tag = s_tags[row];
          if (tag == -1) {
            const int old = atomicCAS(&s_tags[row], -1, node);
            tag = old == -1 ? node : old;
          }
          if (tag == node) {
            uint64_t *p = &s_keys[row * K + k0];
            // cheap filter on the value half only (one 32-bit LDS read per element): an entry whose
            // value key is below the cached one cannot win; ties and improvements take the 64-bit atomic
            const uint32_t *hi = reinterpret_cast<const uint32_t *>(p) + 1;
#pragma unroll
            for (int v = 0; v < VEC; ++v)
              if ((uint32_t)(key[u][v] >> 32) >= lds_peek(hi + 2 * v) && key[u][v] != 0)
                __hip_atomic_fetch_max(p + v, key[u][v], __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_WORKGROUP);
          } else {
            miss_node[u] = node;
          }
        }
        // entries whose table row belongs to another node: all reads first, then the atomics
        uint64_t cur[U][VEC];
#pragma unroll
        for (int u = 0; u < U; ++u) {
          if (miss_node[u] < 0) continue;
          const uint64_t *p = gkeys + miss_node[u] * a.K + k0;
#pragma unroll
          for (int v = 0; v < VEC; ++v) cur[u][v] = p[v];  // cached read: a stale value only costs a spare atomic
        }
#pragma unroll
        for (int u = 0; u < U; ++u) {
          if (miss_node[u] < 0) continue;
          uint64_t *p = gkeys + miss_node[u] * a.K + k0;
#pragma unroll
          for (int v = 0; v < VEC; ++v)
            if (key[u][v] > cur[u][v])
              __hip_atomic_fetch_max(p + v, key[u][v], __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
        }
      }
    }
  }
  __syncthreads();
  // per-node winners of this chunk -> global table
  for (int i0 = threadIdx.x; i0 < tn * K; i0 += kLdsBlock * 4) {
    uint64_t key[4], cur[4];
    uint64_t *p[4];
#pragma unroll
    for (int j = 0; j < 4; ++j) {
      const int i = i0 + j * kLdsBlock;
      key[j] = i < tn * K ? s_keys[i] : 0;
      p[j] = nullptr;
      if (key[j] != 0) {
        const int row = i / K;
        p[j] = gkeys + (int64_t)s_tags[row] * a.K + (i - row * K);
        cur[j] = *p[j];
      }
    }
#pragma unroll
    for (int j = 0; j < 4; ++j)
      if (key[j] != 0 && key[j] > cur[j])
        __hip_atomic_fetch_max(p[j], key[j], __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
  }
}

// Is the index skewed? The table kernel above gains 2x on an unsorted index in which a few output rows own
// much of the input (10 M entries of 8 / 32 floats onto 1 M rows, Zipf(1.2): 486 -> 244 / 1166 -> 681 us) and
// loses as much on a uniform or sorted one, and the average number of entries per row does not tell them
// apart. One workgroup looks at 1024 entries spread evenly over the index: *flag = 1 if at least a quarter
// of them repeat an output row seen before (a hash set in LDS) and the sampled neighbours are not in
// ascending order (a sorted index stays with the run kernel), else 0. The two kernels launched behind it
// read the flag and one of them returns at once.
constexpr int kSkewSamples = 1024;  // one per lane: widely spaced loads, most of them miss the TLB
constexpr int kSkewSlots = 2048;
constexpr int kSkewBlock = 1024;

static __global__ __launch_bounds__(kSkewBlock) void index_skew_kernel(ScatterArgs a, int *flag) {
  __shared__ int s_set[kSkewSlots];
  __shared__ int s_dup, s_desc;
  for (int i = threadIdx.x; i < kSkewSlots; i += kSkewBlock) s_set[i] = -1;
  if (threadIdx.x == 0) { s_dup = 0; s_desc = 0; }
  __syncthreads();
  const int64_t n = a.B * a.E;
  const int64_t step = n / kSkewSamples;  // the host only launches this with n >= 2 * kSkewSamples
  int dup = 0, desc = 0;
  constexpr int PER = kSkewSamples / kSkewBlock;
  int64_t idx[PER], nxt[PER], bb[PER];
#pragma unroll
  for (int j = 0; j < PER; ++j) {  // all loads first: one memory latency for the whole sample
    const int64_t be = (int64_t)(threadIdx.x + j * kSkewBlock) * step;
    int64_t e, b1, e1;
    split_edge(be, a.B, a.E, bb[j], e);
    split_edge(be + 1, a.B, a.E, b1, e1);
    idx[j] = a.index[bb[j] * a.sb + e * a.se];
    nxt[j] = a.index[b1 * a.sb + e1 * a.se];
    if (b1 != bb[j]) nxt[j] = idx[j];
  }
#pragma unroll
  for (int j = 0; j < PER; ++j) {
    if (nxt[j] < idx[j]) ++desc;
    if (idx[j] < 0 || idx[j] >= a.N) continue;
    const int node = (int)(bb[j] * a.N + idx[j]);
    unsigned h = ((unsigned)node * 2654435761u) >> 21;  // 11 bits
    for (int probe = 0; probe < 16; ++probe) {
      const int old = atomicCAS(&s_set[h], -1, node);
      if (old == -1) break;
      if (old == node) { ++dup; break; }
      h = (h + 1) & (kSkewSlots - 1);
    }
  }
  if (dup) atomicAdd(&s_dup, dup);
  if (desc) atomicAdd(&s_desc, desc);
  __syncthreads();
  if (threadIdx.x == 0) *flag = (s_dup * 4 >= kSkewSamples && s_desc * 64 >= kSkewSamples) ? 1 : 0;
}

// One value per entry (K == 1): the same table, written for occupancy. The general kernel above keeps
// eight entries with their 64-bit bookkeeping per lane (143 VGPRs, three wavefronts per SIMD) and the
// counters show it bound by latency, not by L2 or HBM; this one holds 32-bit state only (58 VGPRs), runs
// 1024 lanes on one 48 KB table and keeps the next batch of loads in flight while the current one goes
// through the table.

constexpr int kLdsBlockK1 = 1024;

template <typename T, bool IS_MAX>
__global__ __launch_bounds__(kLdsBlockK1) void scatter_key_lds_k1_kernel(ScatterArgs a, int64_t epb) {
  constexpr int U = 4;
  constexpr int mask = kLdsKeys - 1;
  __shared__ uint64_t s_keys[kLdsKeys];
  __shared__ int32_t s_tags[kLdsKeys];
  for (int i = threadIdx.x; i < kLdsKeys; i += kLdsBlockK1) {
    s_keys[i] = 0;
    s_tags[i] = -1;
  }
  __syncthreads();

  const T *src = static_cast<const T *>(a.src);
  uint64_t *gkeys = reinterpret_cast<uint64_t *>(a.arg_out);
  const int64_t lo = (int64_t)blockIdx.x * epb;
  int64_t hi = lo + epb;
  if (hi > a.B * a.E) hi = a.B * a.E;
  const int n_batches = (int)((hi - lo + (int64_t)kLdsBlockK1 * U - 1) / ((int64_t)kLdsBlockK1 * U));

  // loads of one batch: value, node id and position of U entries (entries past the end repeat the last one)
  auto load = [&](int batch, T *x, int *node, uint32_t *pos) {
#pragma unroll
    for (int u = 0; u < U; ++u) {
      int64_t e = lo + ((int64_t)batch * U + u) * kLdsBlockK1 + threadIdx.x;
      const bool ok = e < hi;
      if (!ok) e = hi - 1;
      int64_t b, p;
      split_edge(e, a.B, a.E, b, p);
      x[u] = src[e];
      const int64_t idx = a.index[b * a.sb + p * a.se];
      node[u] = (ok && idx >= 0 && idx < a.N) ? (int)(b * a.N + idx) : -1;
      pos[u] = (uint32_t)p;
    }
  };

  T x[U], xn[U];
  int node[U], noden[U];
  uint32_t pos[U], posn[U];
  if (n_batches > 0) load(0, x, node, pos);
  for (int batch = 0; batch < n_batches; ++batch) {
    load(batch + 1 < n_batches ? batch + 1 : batch, xn, noden, posn);  // unconditional: exact wait counts
    uint64_t key[U];
    bool miss[U];
#pragma unroll
    for (int u = 0; u < U; ++u) {
      miss[u] = false;
      key[u] = 0;
      if (node[u] < 0 || Key<T>::is_nan(x[u])) continue;  // NaN never wins
      key[u] = pack_key<T, IS_MAX>(x[u], 0xFFFFFFFEu - pos[u]);
      const int row = node[u] & mask;
      int tag = s_tags[row];
      if (tag == -1) {
        const int old = atomicCAS(&s_tags[row], -1, node[u]);
        tag = old == -1 ? node[u] : old;
      }
      if (tag == node[u]) {
        // value half first (one 32-bit LDS read): an entry below the cached value cannot win
        const uint32_t cur_hi = lds_peek(reinterpret_cast<const uint32_t *>(&s_keys[row]) + 1);
        if ((uint32_t)(key[u] >> 32) >= cur_hi)
          __hip_atomic_fetch_max(&s_keys[row], key[u], __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_WORKGROUP);
      } else {
        miss[u] = true;
      }
    }
    // entries whose table row belongs to another node: all reads first, then the atomics
    uint64_t cur[U];
#pragma unroll
    for (int u = 0; u < U; ++u)
      if (miss[u]) cur[u] = gkeys[node[u]];  // cached read: a stale value only costs a spare atomic
#pragma unroll
    for (int u = 0; u < U; ++u)
      if (miss[u] && key[u] > cur[u])
        __hip_atomic_fetch_max(gkeys + node[u], key[u], __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
#pragma unroll
    for (int u = 0; u < U; ++u) {
      x[u] = xn[u];
      node[u] = noden[u];
      pos[u] = posn[u];
    }
  }
  __syncthreads();
  // per-node winners of this chunk -> global table
  constexpr int F = 4;
  for (int i0 = threadIdx.x; i0 < kLdsKeys; i0 += kLdsBlockK1 * F) {
    uint64_t key[F], cur[F];
    int tag[F];
#pragma unroll
    for (int j = 0; j < F; ++j) {
      const int i = i0 + j * kLdsBlockK1;
      key[j] = i < kLdsKeys ? s_keys[i] : 0;
      tag[j] = i < kLdsKeys ? s_tags[i] : 0;
      if (key[j] != 0) cur[j] = gkeys[tag[j]];
    }
#pragma unroll
    for (int j = 0; j < F; ++j)
      if (key[j] != 0 && key[j] > cur[j])
        __hip_atomic_fetch_max(gkeys + tag[j], key[j], __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
  }
}

// ---- sum with a workgroup-private accumulator table ------------------------------
// Same idea as the packed-key table above, for additions: a hub node that owns
// 20 % of the entries would otherwise put two million atomics on one address
// (measured: 29 ms for 10 M entries). Rows of fp32 accumulators are claimed per
// node in LDS (ds_add_f32), written back with one global atomic per touched
// element and chunk. 16-bit inputs gain accuracy on the way (fp32 partial sums,
// one rounding per chunk instead of one per entry). src == nullptr adds 1.0 per
// entry (the count of scatter mean).
constexpr int kLdsAcc = 8192;         // accumulators of the table (64 KB of double slots)
constexpr int kLdsAccRows = 4096;     // 16 KB of tags
constexpr int kLdsAddBlock = 1024;    // one table per 16 wavefronts: every workgroup adds its table to out once

// slot of the accumulator table: double for the floating types, the element's own width for int32 / int64
template <typename T> struct TableSlot { typedef double type; };
template <> struct TableSlot<int32_t> { typedef int32_t type; };
template <> struct TableSlot<int64_t> { typedef long long type; };

// What leaves the table for `out` (rows that missed it, and the table itself at the end). The rows of a hub are
// in every workgroup's table, so thousands of workgroups add to the same elements: 16-bit floats go through the
// packed-pair add of the hardware, not through a compare-and-swap loop (4 M entries of 8 bf16 under a Zipf(1.2)
// index: 14 ms with the loop).
template <typename T> __device__ __forceinline__ void table_add_out(T *p, T v, const T *lo, const T *hi) {
  if constexpr (__is_same(T, bf16_t) || __is_same(T, f16_t))
    atomic_add_half<T>(p, v, lo, hi);
  else
    atomic_add_elem<T>(p, v);
}

// the table's slot *= v: LDS has no atomic product, so a compare-and-swap loop on the slot's bits (an LDS round trip
// per try, and only the lanes of one workgroup meet there)
template <typename L> __device__ __forceinline__ void lds_slot_mul(L *slot, L v) {
  typedef typename std::conditional<sizeof(L) == 8, uint64_t, uint32_t>::type U;
  static_assert(sizeof(L) == sizeof(U), "");
  U *word = reinterpret_cast<U *>(slot);
  U old = __hip_atomic_load(word, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_WORKGROUP);
  while (true) {
    L cur;
    __builtin_memcpy(&cur, &old, sizeof(L));
    const L nv = cur * v;
    U desired;
    __builtin_memcpy(&desired, &nv, sizeof(L));
    if (desired == old) return;
    if (__hip_atomic_compare_exchange_strong(word, &old, desired, __ATOMIC_RELAXED, __ATOMIC_RELAXED,
                                             __HIP_MEMORY_SCOPE_WORKGROUP))
      return;
  }
}

// MUL = true: the same table for products (slots start at 1 and are multiplied into out). A product has no
// hardware atomic at all, so every entry that reaches memory is a compare-and-swap loop whose time grows with
// the square of the entries that meet in one element (1 M entries of 8 floats, 30 % of them on one row: 89 ms
// through scatter_atomic_kernel); here a row's entries meet in LDS and memory sees one factor per row and workgroup.
// COUNT = true (sums): the entries of every output row are counted as well, into the zeroed int32 array a.count_out
// (scatter mean), in a table of their own beside the sums; the lane that holds an entry's first column counts it.
template <typename T, bool MUL = false, bool COUNT = false>
__global__ __launch_bounds__(kLdsAddBlock) void scatter_add_lds_kernel(ScatterArgs a, int tn_mask, int64_t epb) {
  constexpr int U = 4;
  if (a.skip_flag != nullptr && a.skip_want >= 0) {
    if (*a.skip_flag != a.skip_want) return;
  } else if (a.skip_flag != nullptr && (*a.skip_flag != 0) != (a.skip_inverse != 0)) {
    return;
  }
  // double slots for the floating types: ds_add_f32 loses its rate when many lanes meet on one address (a hub, or a
  // sorted index whose neighbouring entries share a row), ds_add_f64 does not (Zipf(1.2) index, K = 8: 391 -> 263 us;
  // sorted: 476 -> 177 us). Integers keep their own width (their sums wrap, which a double cannot follow).
  typedef typename TableSlot<T>::type LdsAcc;
  __shared__ LdsAcc s_acc[kLdsAcc];
  __shared__ int32_t s_tags[kLdsAccRows];
  __shared__ int32_t s_cnt[COUNT ? kLdsAccRows : 1];
  const int K = (int)a.K;
  const int tn = tn_mask + 1;
  for (int i = threadIdx.x; i < tn * K; i += kLdsAddBlock) s_acc[i] = (LdsAcc)(MUL ? 1 : 0);
  for (int i = threadIdx.x; i < tn; i += kLdsAddBlock) s_tags[i] = -1;
  if constexpr (COUNT) {
    for (int i = threadIdx.x; i < tn; i += kLdsAddBlock) s_cnt[i] = 0;
  }
  __syncthreads();

  const T *src = static_cast<const T *>(a.src);
  T *out = static_cast<T *>(a.out);
  const EdgeLanes m = edge_lanes(K, kLdsAddBlock);
  const T *out_end = out + a.B * a.N * a.K;
  const int64_t be_lo = (int64_t)blockIdx.x * epb;
  int64_t be_hi = be_lo + epb;
  if (be_hi > a.B * a.E) be_hi = a.B * a.E;

  if (m.active) {
    for (int64_t be0 = be_lo + m.el; be0 < be_hi; be0 += (int64_t)m.epp * U) {
      for (int k = m.cl; k < K; k += m.L) {
        typename Acc<T>::type x[U];  // widened for the table only where it is added (doubles here cost 30 % of the kernel)
        int64_t idx[U], bb[U], ee[U];
#pragma unroll
        for (int u = 0; u < U; ++u) {
          const int64_t be = be0 + (int64_t)u * m.epp;
          split_edge(be < be_hi ? be : be0, a.B, a.E, bb[u], ee[u]);
          x[u] = src ? to_acc<T>(src[(bb[u] * a.E + ee[u]) * a.K + k]) : (typename Acc<T>::type)1;
          idx[u] = a.index[bb[u] * a.sb + ee[u] * a.se];
        }
#pragma unroll
        for (int u = 0; u < U; ++u) {
          if (be0 + (int64_t)u * m.epp >= be_hi) continue;
          if (idx[u] < 0 || idx[u] >= a.N) continue;
          const int node = (int)(bb[u] * a.N + idx[u]);
          const int row = node & tn_mask;
          int tag = s_tags[row];
          if (tag == -1) {
            const int old = atomicCAS(&s_tags[row], -1, node);
            tag = old == -1 ? node : old;
          }
          if constexpr (COUNT) {
            if (k == 0) atomicAdd(tag == node ? &s_cnt[row] : a.count_out + node, 1);
          }
          if (MUL) {
            if (tag == node) {
              lds_slot_mul<LdsAcc>(&s_acc[row * K + k], (LdsAcc)x[u]);
            } else {
              const T f = from_acc<T>(x[u]);
              atomic_rmw<T>(out + (int64_t)node * a.K + k, [f](T cur) { return mul_elem<T>(cur, f); });
            }
          } else if (tag == node) {
            __hip_atomic_fetch_add(&s_acc[row * K + k], (LdsAcc)x[u], __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_WORKGROUP);
          } else {
            table_add_out<T>(out + (int64_t)node * a.K + k, from_acc<T>(x[u]), out, out_end);
          }
        }
      }
    }
  }
  __syncthreads();
  if constexpr (COUNT) {
    for (int i = threadIdx.x; i < tn; i += kLdsAddBlock) {
      const int32_t c = s_cnt[i];
      if (c != 0) atomicAdd(a.count_out + s_tags[i], c);
    }
  }
  if constexpr (MUL) {
    for (int i = threadIdx.x; i < tn * K; i += kLdsAddBlock) {
      const LdsAcc v = s_acc[i];
      if (v == (LdsAcc)1) continue;
      const int row = i / K;
      const T f = from_acc<T>((typename Acc<T>::type)v);
      atomic_rmw<T>(out + (int64_t)s_tags[row] * a.K + (i - row * K), [f](T cur) { return mul_elem<T>(cur, f); });
    }
    return;
  }
  if constexpr (__is_same(T, bf16_t) || __is_same(T, f16_t)) {
    // two neighbouring columns per packed add when the rows allow it
    if ((K & 1) == 0 && (reinterpret_cast<uintptr_t>(out) & 3) == 0) {
      for (int i = 2 * threadIdx.x; i < tn * K; i += 2 * kLdsAddBlock) {
        const float v0 = (float)s_acc[i], v1 = (float)s_acc[i + 1];
        if (v0 == 0.0f && v1 == 0.0f) continue;
        const int row = i / K;
        atomic_add_pair<T>(out + (int64_t)s_tags[row] * a.K + (i - row * K), from_acc<T>(v0), from_acc<T>(v1));
      }
      return;
    }
  }
  for (int i = threadIdx.x; i < tn * K; i += kLdsAddBlock) {
    const LdsAcc v = s_acc[i];
    if (v == (LdsAcc)0) continue;
    const int row = i / K;
    table_add_out<T>(out + (int64_t)s_tags[row] * a.K + (i - row * K), from_acc<T>((typename Acc<T>::type)v), out, out_end);
  }
}

template <typename T, bool IS_MAX>
__global__ __launch_bounds__(kBlock) void scatter_key_final_kernel(ScatterArgs a) {
  const int64_t n = a.B * a.N * a.K;
  const T *src = static_cast<const T *>(a.src);
  T *out = static_cast<T *>(a.out);
  uint64_t *keys = reinterpret_cast<uint64_t *>(a.arg_out);
  for (int64_t i = (int64_t)blockIdx.x * kBlock + threadIdx.x; i < n; i += (int64_t)gridDim.x * kBlock) {
    const uint64_t key = keys[i];
    const uint32_t low = (uint32_t)key;
    if (low == kKeepLow) {  // nothing beat the initial / previous content
      if (!a.out_given) out[i] = zero_elem<T>();
      a.arg_out[i] = a.E;
    } else {
      const int64_t e = (int64_t)(0xFFFFFFFEu - low);
      uint32_t k = (uint32_t)(key >> 32);
      if (!IS_MAX) k = ~k;
      T val = Key<T>::dec(k);
      if (Key<T>::kFloat && k == 0x80000000u) {
        // a zero: fetch it from src to keep the sign bit of the winning entry
        const int64_t bn = i / a.K;
        const int64_t kk = i - bn * a.K;
        const int64_t b = bn / a.N;
        val = src[(b * a.E + e) * a.K + kk];
      }
      out[i] = val;
      a.arg_out[i] = e;
    }
  }
}

// ---- two-pass min/max for 64-bit element types --------------------------------
// First pass: the value, by compare-and-swap. A slot that an entry strictly improves gets kArgOpen into its arg_out
// (filled with E before): the second pass looks for positions only there, so a slot in which no entry beat the
// initial or previous content keeps E even if an entry equals that content.
constexpr int64_t kArgOpen = INT64_MAX;
template <typename T, bool IS_MAX> __device__ __forceinline__ bool wide_improve(T *slot, T val) {
  static_assert(sizeof(T) == 8, "");
  uint64_t *word = reinterpret_cast<uint64_t *>(slot);
  uint64_t old = __hip_atomic_load(word, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
  uint64_t desired;
  __builtin_memcpy(&desired, &val, 8);
  while (true) {
    T cur;
    __builtin_memcpy(&cur, &old, 8);
    if (!(IS_MAX ? val > cur : val < cur)) return false;
    if (__hip_atomic_compare_exchange_strong(word, &old, desired, __ATOMIC_RELAXED, __ATOMIC_RELAXED,
                                             __HIP_MEMORY_SCOPE_AGENT))
      return true;
  }
}
template <typename T, bool IS_MAX>
__global__ __launch_bounds__(kBlock) void scatter_minmax_wide_kernel(ScatterArgs a) {
  const T *src = static_cast<const T *>(a.src);
  T *out = static_cast<T *>(a.out);
  const int64_t n = a.B * a.E * a.K;
  for (int64_t i = (int64_t)blockIdx.x * kBlock + threadIdx.x; i < n; i += (int64_t)gridDim.x * kBlock) {
    const int64_t be = i / a.K;
    const int64_t k = i - be * a.K;
    const int64_t b = be / a.E;
    const int64_t e = be - b * a.E;
    const int64_t idx = a.index[b * a.sb + e * a.se + k * a.sk];
    if (idx < 0 || idx >= a.N) continue;
    const T val = src[i];
    const int64_t o = (b * a.N + idx) * a.K + k;
    if (wide_improve<T, IS_MAX>(out + o, val)) a.arg_out[o] = kArgOpen;
  }
}
// order-preserving 64-bit keys of the 64-bit element types; 0 stands for "no entry" in the table below
template <typename T> struct WideKey;
template <> struct WideKey<int64_t> {
  __device__ static uint64_t enc(int64_t v) { return (uint64_t)v ^ 0x8000000000000000ull; }
  __device__ static int64_t dec(uint64_t k) { return (int64_t)(k ^ 0x8000000000000000ull); }
  __device__ static bool is_nan(int64_t) { return false; }
};
template <> struct WideKey<double> {
  __device__ static uint64_t enc(double v) {
    uint64_t u = (uint64_t)__double_as_longlong(v);
    if (u == 0x8000000000000000ull) u = 0;  // -0.0 and +0.0 compare equal
    return (u >> 63) ? ~u : (u | 0x8000000000000000ull);
  }
  __device__ static double dec(uint64_t k) {
    return __longlong_as_double((long long)((k >> 63) ? (k & 0x7FFFFFFFFFFFFFFFull) : ~k));
  }
  __device__ static bool is_nan(double v) { return v != v; }
};

// First pass of min / max for 64-bit elements when many entries meet in an output slot: the compare-and-swap
// loop of scatter_minmax_wide_kernel starts with a read that is coherent across the XCDs, and those reads queue
// up at the memory side when they fall on few lines (16.7 M entries onto 64 k slots: 4.4 ms, 3.8 G entries/s).
// Here a workgroup keeps a table of keys in LDS for the rows it meets (tags as in scatter_add_lds_kernel) and
// sends every touched slot to memory once, at the end; rows that miss the table go the old way.
template <typename T, bool IS_MAX>
__global__ __launch_bounds__(kLdsAddBlock) void scatter_minmax_wide_lds_kernel(ScatterArgs a, int tn_mask, int64_t epb) {
  constexpr int U = 4;
  __shared__ unsigned long long s_key[kLdsAcc];
  __shared__ int32_t s_tags[kLdsAccRows];
  const int K = (int)a.K;
  const int tn = tn_mask + 1;
  for (int i = threadIdx.x; i < tn * K; i += kLdsAddBlock) s_key[i] = 0;
  for (int i = threadIdx.x; i < tn; i += kLdsAddBlock) s_tags[i] = -1;
  __syncthreads();
  const T *src = static_cast<const T *>(a.src);
  T *out = static_cast<T *>(a.out);
  const EdgeLanes m = edge_lanes(K, kLdsAddBlock);
  const int64_t be_lo = (int64_t)blockIdx.x * epb;
  int64_t be_hi = be_lo + epb;
  if (be_hi > a.B * a.E) be_hi = a.B * a.E;
  auto to_memory = [&](int64_t o, T val) {
    if (wide_improve<T, IS_MAX>(out + o, val)) a.arg_out[o] = kArgOpen;
  };
  if (m.active) {
    for (int64_t be0 = be_lo + m.el; be0 < be_hi; be0 += (int64_t)m.epp * U) {
      for (int k = m.cl; k < K; k += m.L) {
        T x[U];
        int64_t idx[U], bb[U], ee[U];
#pragma unroll
        for (int u = 0; u < U; ++u) {
          const int64_t be = be0 + (int64_t)u * m.epp;
          split_edge(be < be_hi ? be : be0, a.B, a.E, bb[u], ee[u]);
          x[u] = src[(bb[u] * a.E + ee[u]) * a.K + k];
          idx[u] = a.index[bb[u] * a.sb + ee[u] * a.se];
        }
#pragma unroll
        for (int u = 0; u < U; ++u) {
          if (be0 + (int64_t)u * m.epp >= be_hi) continue;
          if (idx[u] < 0 || idx[u] >= a.N || WideKey<T>::is_nan(x[u])) continue;  // a NaN never wins
          const int node = (int)(bb[u] * a.N + idx[u]);
          const int row = node & tn_mask;
          int tag = s_tags[row];
          if (tag == -1) {
            const int old = atomicCAS(&s_tags[row], -1, node);
            tag = old == -1 ? node : old;
          }
          const uint64_t enc = WideKey<T>::enc(x[u]);
          const unsigned long long key = IS_MAX ? enc : ~enc;
          if (tag == node && key != 0)
            __hip_atomic_fetch_max(&s_key[row * K + k], key, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_WORKGROUP);
          else
            to_memory((int64_t)node * a.K + k, x[u]);
        }
      }
    }
  }
  __syncthreads();
  for (int i = threadIdx.x; i < tn * K; i += kLdsAddBlock) {
    const unsigned long long key = s_key[i];
    if (key == 0) continue;
    const int row = i / K;
    to_memory((int64_t)s_tags[row] * a.K + (i - row * K), WideKey<T>::dec(IS_MAX ? key : ~key));
  }
}

template <typename T>
__global__ __launch_bounds__(kBlock) void scatter_arg_wide_kernel(ScatterArgs a) {
  const T *src = static_cast<const T *>(a.src);
  const T *out = static_cast<const T *>(a.out);
  const int64_t n = a.B * a.E * a.K;
  for (int64_t i = (int64_t)blockIdx.x * kBlock + threadIdx.x; i < n; i += (int64_t)gridDim.x * kBlock) {
    const int64_t be = i / a.K;
    const int64_t k = i - be * a.K;
    const int64_t b = be / a.E;
    const int64_t e = be - b * a.E;
    const int64_t idx = a.index[b * a.sb + e * a.se + k * a.sk];
    if (idx < 0 || idx >= a.N) continue;
    const int64_t o = (b * a.N + idx) * a.K + k;
    if (src[i] != out[o]) continue;
    // only slots that the first pass improved (no longer E); the position only ever goes down, so read it first
    // (among many equal values nearly every entry is too late)
    const int64_t seen = __hip_atomic_load(a.arg_out + o, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
    if (seen != a.E && e < seen) __hip_atomic_fetch_min(a.arg_out + o, e, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
  }
}

inline unsigned grid_for(int64_t n, int per_thread = 1) {
  int64_t blocks = (n + (int64_t)kBlock * per_thread - 1) / ((int64_t)kBlock * per_thread);
  if (blocks < 1) blocks = 1;
  const int64_t cap = 256 * 32;  // 256 CUs x 32 workgroups: enough to fill the chip, grid-stride beyond
  return (unsigned)(blocks < cap ? blocks : cap);
}

}  // namespace ts
#include "scatter_binned.h"
#include "scatter_k1.h"
#include "scatter_k1_sum.h"
namespace ts {

// ---- elementwise helpers --------------------------------------------------------
template <typename T>
__global__ __launch_bounds__(kBlock) void fill_kernel(T *p, int64_t n, T value) {
  for (int64_t i = (int64_t)blockIdx.x * kBlock + threadIdx.x; i < n; i += (int64_t)gridDim.x * kBlock)
    p[i] = value;
}
// The fill of a sum whose kernel is picked by a sample of the index: the first workgroup also takes the sample
// of bin_sample_kernel (the same entries and the same verdict in *flag), which saves that kernel's launch and
// hides its loads behind the fill (5-7 us of a 25 us call).
template <typename T>
__global__ __launch_bounds__(kBlock) void fill_sample_kernel(T *p, int64_t n, T value, ScatterArgs a, int *flag) {
  __shared__ int s_desc;
  constexpr int PER = kBinBlock / kBlock;
  int desc = 0;
  if (blockIdx.x == 0) {
    if (threadIdx.x == 0) s_desc = 0;
    const int64_t ne = a.B * a.E;  // the host asks for a sample only with ne >= 2 * kBinBlock
    int64_t idx[PER], nxt[PER];
    bool same[PER];
#pragma unroll
    for (int j = 0; j < PER; ++j) {
      const int64_t be = (int64_t)(threadIdx.x * PER + j) * (ne / kBinBlock);
      const int64_t b = be / a.E, e = be - b * a.E;
      const int64_t b1 = (be + 1) / a.E, e1 = be + 1 - b1 * a.E;
      idx[j] = a.index[b * a.sb + e * a.se];
      nxt[j] = a.index[b1 * a.sb + e1 * a.se];
      same[j] = b1 == b;
    }
#pragma unroll
    for (int j = 0; j < PER; ++j) desc += same[j] && nxt[j] < idx[j] ? 1 : 0;
  }
  for (int64_t i = (int64_t)blockIdx.x * kBlock + threadIdx.x; i < n; i += (int64_t)gridDim.x * kBlock)
    p[i] = value;
  if (blockIdx.x == 0) {
    __syncthreads();
    if (desc) atomicAdd(&s_desc, desc);
    __syncthreads();
    if (threadIdx.x == 0) *flag = s_desc * 64 >= kBinBlock ? 1 : 0;
  }
}
// out[out == init] = 0 (csrc/cuda/scatter_cuda.cu:126-127)
template <typename T>
__global__ __launch_bounds__(kBlock) void mask_init_kernel(T *p, int64_t n, T init) {
  for (int64_t i = (int64_t)blockIdx.x * kBlock + threadIdx.x; i < n; i += (int64_t)gridDim.x * kBlock)
    if (p[i] == init) p[i] = (T)0;
}

// ---- host side --------------------------------------------------------------------
template <typename T> struct IsWide { static constexpr bool value = sizeof(T) == 8; };

// Entries per workgroup chunk of the LDS-table kernels: ~64 K elements per chunk amortise writing the
// table back (measured optimum: 16384 entries for K = 1, 2048 for K = 32), capped so that narrow rows
// do not leave fewer than ~512 workgroups.
inline int64_t lds_chunk_edges(int64_t forced, int64_t K, int64_t n_edges) {
  if (forced > 0) return forced;
  int64_t epb = ((int64_t)1 << 16) / K;
  if (epb > 16384) epb = 16384;
  while (epb > 256 && n_edges / epb < 512) epb /= 2;
  return epb < 64 ? 64 : epb;
}

// Entries per workgroup when one large workgroup per CU (or a small multiple of the CU count) shares a
// table: the table is written back once per workgroup, so fewer and larger chunks win as long as all CUs
// are busy (measured for min/max with K = 1: 256 chunks of 39 k entries 83 us, 610 chunks of 16 k 98 us).
inline int64_t per_cu_chunk_edges(int64_t forced, int64_t n_edges, int64_t min_epb, int64_t max_epb) {
  if (forced > 0) return forced;
  int dev = 0, cus = 256;
  if (hipGetDevice(&dev) == hipSuccess &&
      hipDeviceGetAttribute(&cus, hipDeviceAttributeMultiprocessorCount, dev) != hipSuccess)
    cus = 0;
  if (cus < 1) cus = 256;
  const int64_t rounds = (n_edges + (int64_t)cus * max_epb - 1) / ((int64_t)cus * max_epb);
  const int64_t epb = (n_edges + cus * rounds - 1) / (cus * rounds);
  return epb < min_epb ? min_epb : epb;
}

// workgroups needed so that every edge is visited once: `block` threads cover
// block / min(kv, block) edges per pass and U passes per loop trip
inline unsigned scatter_grid(int64_t n_edges, int64_t kv, int block, int U) {
  const int64_t L = kv < block ? kv : block;
  const int64_t per_block = (block / L) * U;
  int64_t blocks = (n_edges + per_block - 1) / per_block;
  if (blocks < 1) blocks = 1;
  const int64_t cap = 256 * 64;
  return (unsigned)(blocks < cap ? blocks : cap);
}

// Sizes from which a sum goes through the LDS table kernel (scatter_add_lds_kernel). The table is the kernel
// that a skewed index cannot hurt: a hub's entries meet in LDS, where the run kernel sends each of them to one
// address in memory, 10 ns apiece (Zipf(1.2) index, us run kernel / table: 16 k entries of 32 floats 56 / 11,
// 65 k entries 143 / 14, 200 k entries of 16 floats 479 / 27, 131 k single values 268 / 11). With chunks sized
// for one workgroup per CU it costs a uniform or sorted index nothing where the call is bound by its two launches
// (up to 2^19 elements: 10.4-11.5 us either way), 1-4 us at 2^21 elements (200 k x 16 floats onto 10 k rows:
// 16.2 / 19.9 us), and from 2^23 elements it is level or ahead. Its write-back is a phase of its own after the
// entries, which shows where the atomics miss the L2 (+1 us on the smallest calls, +4 us for rows of 64 floats onto
// 100 k rows), so the smallest inputs stay with the run kernel for as long as a hub costs less than that: 4-byte
// elements go through the table from 2^16 elements, rows of 33-64 columns from 2^18, wider ones (a table of 64
// rows: 4096 entries of 128 floats onto 100 k rows, uniform 13.6 / 18.9 us, Zipf 37 / 19 us) from 2^19.
// Other element types keep the sizes measured for them: a
// contended index (32 and more entries per output row) from 2^17 elements, narrow rows from 2^18 entries or 2^22
// elements; 2-byte elements are flushed with packed adds and lose through the table under an uncontended index
// (16 MB of 32 bf16 per entry: 17 -> 50 us). Rows of 32 and more columns stay under 300 MB of input (9-10 M entries:
// a sorted index takes 450 us through the run kernel with its hot rows and 940 us through the table; an unsorted
// one has the workspace path).
inline bool sum_table_by_size(int64_t B, int64_t E, int64_t K, int64_t N, int elem_bytes) {
  const int64_t n_edges = B * E, n_src = n_edges * K;
  if (n_src < ((int64_t)1 << 16)) return false;
  if (K >= 32 && n_src * elem_bytes >= (int64_t)300000000) return false;
  if (elem_bytes == 4 && n_src >= ((int64_t)1 << (K <= 32 ? 16 : K <= 64 ? 18 : 19))) return true;
  if (n_src < ((int64_t)1 << 17)) return false;
  if (n_edges >= 32 * B * N) return true;
  if (elem_bytes == 4) return false;
  return K < 32 && (n_src >= ((int64_t)1 << 22) || n_edges >= ((int64_t)1 << 18));
}
// entries per workgroup of that kernel at least: 2048 elements, 64 entries (8192 entries of 32 floats: 17.4 us in
// chunks of 512, 10.6 us in chunks of 64; the chunk of a larger input is its share of one workgroup per CU)
// 2-byte elements keep chunks of 16384 elements: every partial sum that leaves the table is rounded to the element
// type, and with one entry per row and chunk nothing has been combined in fp32 before that (300 k single bf16 values
// onto 5000 rows: RMS error 0.105 in chunks of 2048, 0.074 for the reference's entry-by-entry adds, less in large chunks).
inline int64_t sum_table_min_chunk(int64_t K, int elem_bytes) {
  if (elem_bytes == 2) return 16384 / K > 256 ? 16384 / K : 256;
  return 2048 / K > 64 ? 2048 / K : 64;
}

template <typename T, int VEC>
int launch_scatter_v(const ScatterArgs &args, int reduce, hipStream_t stream) {
  ScatterArgs a = args;
  T *out = static_cast<T *>(a.out);
  const int64_t n_out = a.B * a.N * a.K;
  const int64_t n_src = a.B * a.E * a.K;
  const int64_t n_edges = a.B * a.E;
  const unsigned g_out = grid_for(n_out);
  if (reduce == TS_SUM || reduce == TS_MUL) {
    // A small sum whose caller wants the entries per output row as well (scatter mean): cleared, added and counted
    // in two launches (scatter_add_count_run_kernel). Below 2^16 elements, where the run kernel takes every sum.
    if constexpr (!(std::is_integral<T>::value && sizeof(T) < 4)) {
      if (reduce == TS_SUM && a.count_out != nullptr && a.count_done != nullptr && n_src > 0 &&
          n_src < ((int64_t)1 << 16) && a.run_reduce && a.lds_cache != 2 && !a.bin_any_size && a.sk == 0 &&
          a.B * a.N < 0x7FFFFFFFll) {
        constexpr int CN = sizeof(T) < 4 ? 4 / (int)sizeof(T) : 1;
        const bool word_ok = CN == 1 || (a.K % CN == 0 && (reinterpret_cast<uintptr_t>(a.out) & 3) == 0 &&
                                         (reinterpret_cast<uintptr_t>(a.src) & 3) == 0);
        const int c = word_ok ? CN : 1;
        const RunGrid g = run_grid(n_edges, a.K / c, c, c * (int)sizeof(T));
        const RunGrid gc = run_grid(n_edges, 1, 1, 4);
        if (g.ok && gc.ok && g.hot_rlog < 0 && (uint64_t)g.blocks + gc.blocks < 0x7FFFFFFFull) {
          ScatterArgs cnt = a;
          cnt.src = nullptr;
          cnt.out = a.count_out;
          cnt.K = 1;
          cnt.out_given = 1;
          const int64_t n_clear = (a.out_given ? 0 : n_out) + a.B * a.N;
          hipLaunchKernelGGL(fill_out_count_kernel<T>, dim3(grid_for(n_clear)), dim3(kBlock), 0, stream, out,
                             a.out_given ? (int64_t)0 : n_out, a.count_out, a.B * a.N);
          const dim3 gd(g.blocks + gc.blocks, g.ychunks);
          ts_note_scatter_route(TS_ROUTE_SUM_COUNT_RUNS);
          if (word_ok)
            TS_LAUNCH_RUN(g.serial, (scatter_add_count_run_kernel<T, CN, CN, true>),
                          (scatter_add_count_run_kernel<T, CN, CN, false>), gd, stream, a, g.lshift, g.rpw, cnt, gc.rpw,
                          g.blocks);
          else
            TS_LAUNCH_RUN(g.serial, (scatter_add_count_run_kernel<T, 1, 1, true>),
                          (scatter_add_count_run_kernel<T, 1, 1, false>), gd, stream, a, g.lshift, g.rpw, cnt, gc.rpw,
                          g.blocks);
          *a.count_done = 1;
          return hipGetLastError() == hipSuccess ? TS_OK : TS_ERR_LAUNCH;
        }
      }
    }
    // Large inputs with rows of 64 bytes and more, given a workspace: unless the index is sorted (found out by
    // the first pass), the entries are binned by bucket of output rows and summed in LDS (scatter_binned.h);
    // the kernels launched below then return at once. A sorted index stays with them: they combine its runs
    // (or, for a caller with sorted_route, is left to that caller's segmented reduction: then out is cleared
    // only if the buckets are going to add into it).
    BinPlan bp;
    bp.ok = false;
    int lshift = -1;
    if constexpr (BinSlotOk<T>::value) {
      if (reduce == TS_SUM && n_src > 0 && a.bin_ws != nullptr && a.sk == 0 && a.K % VEC == 0) {
        bp = bin_plan(a.B, a.E, a.K, a.N, (int)sizeof(T), a.bin_ws, a.bin_ws_bytes, a.bin_any_size != 0,
                      (int)sizeof(typename BinSlot<T>::type), false, true);
        lshift = bp.ok ? bin_lane_shift(bp.p, VEC) : -1;
        if constexpr (sizeof(T) == 4) {
          // up to eight 4-byte values per entry: the values travel in the binned words (bin_plan_payload)
          if (!bp.ok && a.K <= kBinPayloadCols && a.lds_cache) {
            bp = bin_plan_payload(a.B, a.E, a.K, a.N, (int)sizeof(T), a.bin_ws, a.bin_ws_bytes, a.bin_any_size != 0);
            lshift = bp.ok ? 0 : -1;
          }
        }
      }
    }
    // Single 4-byte values between the sizes of the table kernel and of the value buckets, given a workspace: tables
    // handed over in slabs (scatter_k1_sum.h), with the counts of scatter mean if the caller wants them.
    // TS_SCATTER_SLABS (tuning aid): 0 never, 2 at any size.
    if constexpr (__is_same(T, float) || __is_same(T, int32_t)) {
      const char *env = getenv("TS_SCATTER_SLABS");
      const int slab_mode = env ? atoi(env) : 1;
      if (reduce == TS_SUM && lshift < 0 && n_src > 0 && slab_mode != 0 && a.bin_ws != nullptr && a.sk == 0 && a.se == 1 &&
          a.lds_cache == 1 && a.src != nullptr && (reinterpret_cast<uintptr_t>(a.src) & 15) == 0 &&
          (reinterpret_cast<uintptr_t>(a.index) & 15) == 0) {
        const bool with_count = a.count_out != nullptr && a.count_done != nullptr;
        const S1Plan sp = s1_plan(a.B, a.E, a.K, a.N, (int)sizeof(T), a.bin_ws, a.bin_ws_bytes, with_count, slab_mode == 2);
        if (sp.ok) {
          ScatterArgs s = a;
          if (!with_count) s.count_out = nullptr;
          if (with_count) {
            hipLaunchKernelGGL(fill_out_count_kernel<T>, dim3(grid_for((a.out_given ? 0 : n_out) + a.N)), dim3(kBlock), 0,
                               stream, out, a.out_given ? (int64_t)0 : n_out, a.count_out, a.N);
          } else if (!a.out_given) {
            hipLaunchKernelGGL(fill_kernel<T>, dim3(g_out), dim3(kBlock), 0, stream, out, n_out, small_const<T>(0));
          }
          ts_note_scatter_route(TS_ROUTE_SUM_SLABS);
          launch_scatter_s1<T>(s, sp, stream);
          if (with_count) *a.count_done = 1;
          return hipGetLastError() == hipSuccess ? TS_OK : TS_ERR_LAUNCH;
        }
      }
    }
    const bool routed = lshift >= 0 && a.sorted_route && a.route_flag != nullptr && !a.out_given;
    // sums that go through the LDS table (scatter_add_lds_kernel; the sizes and crossovers are with its launch
    // below), and whether a sample of the index picks between it and the run kernel
    bool use_lds = false, sampled = false, three_way = false;
    const bool payload = lshift >= 0 && bp.p.payload != 0;
    int tn = 1;
    if constexpr (__is_same(T, float) || __is_same(T, bf16_t) || __is_same(T, f16_t) || __is_same(T, double) ||
                  __is_same(T, int32_t) || __is_same(T, int64_t)) {
      if (reduce == TS_SUM && n_src > 0) {
        while ((int64_t)tn * 2 * a.K <= kLdsAcc && tn * 2 <= kLdsAccRows) tn *= 2;
        // (behind the buckets only an index in order arrives here: that one has the table only if contended)
        const bool by_size = sum_table_by_size(a.B, a.E, a.K, a.N, (int)sizeof(T)) &&
                             (lshift < 0 || payload || n_edges >= 32 * a.B * a.N);
        use_lds = a.lds_cache && a.sk == 0 && tn >= 64 && a.B * a.N < 0x7FFFFFFFll && (a.lds_cache == 2 || by_size);
        // single values through the buckets: the sample of the index gives one of three answers (sorted: the run
        // kernel; skewed: the table kernel; even: the buckets), which needs the table kernel and the sample
        three_way = payload && use_lds && n_edges >= 2 * kBinBlock && !getenv("TS_BIN_NO_SAMPLE");
        if (payload && !three_way) use_lds = false;
        // (a sample of the index: from 2^23 elements, where a sorted index does better through the run kernel;
        // below, the table is level with it and the launch that returns at once would cost 2-4 us)
        sampled = use_lds && a.lds_cache != 2 && a.order_ws != nullptr && a.skip_flag == nullptr && lshift < 0 &&
                  a.run_reduce && n_edges >= 2 * kBinBlock && n_src >= ((int64_t)1 << 23);
      }
    }
    // a caller that wants the entries per output row as well (scatter mean), where the table kernel takes the sum by
    // itself: it counts too, and the counts are cleared with out
    bool count_here = false;
    if constexpr (!(std::is_integral<T>::value && sizeof(T) < 4)) {
      count_here = a.count_out != nullptr && a.count_done != nullptr && use_lds && !sampled && !three_way && lshift < 0 &&
                   a.lds_cache != 2 && !a.bin_any_size;
    }
    if (count_here) {
      const int64_t n_clear = (a.out_given ? 0 : n_out) + a.B * a.N;
      hipLaunchKernelGGL(fill_out_count_kernel<T>, dim3(grid_for(n_clear)), dim3(kBlock), 0, stream, out,
                         a.out_given ? (int64_t)0 : n_out, a.count_out, a.B * a.N);
    } else if (!a.out_given && !routed) {
      if (sampled)
        hipLaunchKernelGGL(fill_sample_kernel<T>, dim3(g_out), dim3(kBlock), 0, stream, out, n_out, small_const<T>(0),
                           a, a.order_ws);
      else
        hipLaunchKernelGGL(fill_kernel<T>, dim3(g_out), dim3(kBlock), 0, stream, out, n_out,
                           small_const<T>(reduce == TS_MUL ? 1 : 0));
    } else if (sampled) {
      hipLaunchKernelGGL(bin_sample_kernel, dim3(1), dim3(kBinBlock), 0, stream, a, a.order_ws);
    }
    if constexpr (BinSlotOk<T>::value) {
      if (lshift >= 0) {
        ts_note_scatter_route(payload ? TS_ROUTE_SUM_VALUE_BUCKETS : routed ? TS_ROUTE_SUM_BUCKETS_OR_SEGMENTED
                                                                              : TS_ROUTE_SUM_BUCKETS_OR_RUNS);
        if (a.count_out != nullptr && a.count_flag != nullptr && (payload || bp.p.rshift <= kBinCountShift)) {
          bp.p.count_out = a.count_out;
          *a.count_flag = bp.p.unsorted;
        }
        launch_binned_add<T, VEC>(a, bp.p, lshift, stream, routed ? n_out : 0, three_way);
        a.skip_flag = bp.p.unsorted;
        if (routed) {
          *a.route_flag = bp.p.unsorted;
          return hipGetLastError() == hipSuccess ? TS_OK : TS_ERR_LAUNCH;
        }
      }
    }
    if (n_src > 0) {
      // one element per lane: the 64 atomics of a wavefront then cover whole cache lines
      // (4 lines per instruction for fp32 instead of 16 with 4 elements per lane)
      const unsigned g = scatter_grid(n_edges, a.K, kBlock, 4);
      if (reduce == TS_SUM) {
        if constexpr (__is_same(T, float) || __is_same(T, bf16_t) || __is_same(T, f16_t) || __is_same(T, double) ||
                      __is_same(T, int32_t) || __is_same(T, int64_t)) {
          // many entries per output slot: reduce in LDS first (see scatter_add_lds_kernel)
          // (sizes: sum_table_by_size)
          if (use_lds) {
            // The table is for an index in no particular order. One that is sorted does better through the run
            // kernel below (9 M entries of the graph of C3, sorted: K = 8 343 against 156 us, K = 4 152 / 96,
            // K = 1 60 / 44; shuffled: 448 / 463), so with a word of scratch a sample of the index decides on the
            // device: the table returns at once if the index looks sorted, the run kernel if not.
            // (the sample was taken with the fill of out above)
            ScatterArgs t = a;
            if (sampled) {
              t.skip_flag = a.order_ws;
              t.skip_inverse = 1;
              a.skip_flag = a.order_ws;
            }
            if (three_way) t.skip_want = 2;  // (skip_flag is the buckets' flag: 2 = unsorted and skewed)
            const int64_t epb = per_cu_chunk_edges(a.lds_epb, n_edges, sum_table_min_chunk(a.K, (int)sizeof(T)),
                                                   131072 / a.K > 2048 ? 131072 / a.K : 2048);
            if (lshift < 0) ts_note_scatter_route(sampled ? TS_ROUTE_SUM_TABLE_OR_RUNS : TS_ROUTE_SUM_TABLE);
            if (count_here) {
              hipLaunchKernelGGL((scatter_add_lds_kernel<T, false, true>), dim3((unsigned)((n_edges + epb - 1) / epb)),
                                 dim3(kLdsAddBlock), 0, stream, t, tn - 1, epb);
              *a.count_done = 1;
              return hipGetLastError() == hipSuccess ? TS_OK : TS_ERR_LAUNCH;
            }
            // behind value buckets that count as well: the table kernel, which takes a skewed index from them, counts too
            // (*count_done = 2 tells the caller, which then has no table of counts to launch for that verdict)
            if (three_way && lshift >= 0 && bp.p.count_out != nullptr && a.count_done != nullptr) {
              hipLaunchKernelGGL((scatter_add_lds_kernel<T, false, true>), dim3((unsigned)((n_edges + epb - 1) / epb)),
                                 dim3(kLdsAddBlock), 0, stream, t, tn - 1, epb);
              *a.count_done = 2;
            } else {
              hipLaunchKernelGGL(scatter_add_lds_kernel<T>, dim3((unsigned)((n_edges + epb - 1) / epb)),
                                 dim3(kLdsAddBlock), 0, stream, t, tn - 1, epb);
            }
            if (!sampled && !three_way) return hipGetLastError() == hipSuccess ? TS_OK : TS_ERR_LAUNCH;
          }
        }
        {
          // one index per row: sum runs of equal neighbouring indices in the wavefront first.
          // Element types below 32 bits are written one 32-bit word (2 or 4 columns) at a time.
          constexpr int CN = sizeof(T) < 4 ? 4 / (int)sizeof(T) : 1;  // columns per lane without 16-byte loads
          const bool word_ok = CN == 1 || (a.K % CN == 0 && (reinterpret_cast<uintptr_t>(a.out) & 3) == 0 &&
                                           (reinterpret_cast<uintptr_t>(a.src) & 3) == 0);
          if (a.run_reduce && a.sk == 0 && a.B * a.N < 0x7FFFFFFFll && !word_ok) {
            // rows that cannot be written word by word: one column per lane and atomic
            const RunGrid g = run_grid(n_edges, a.K, 1, (int)sizeof(T));
            if (g.ok) {
              if (lshift < 0 && !use_lds) ts_note_scatter_route(TS_ROUTE_SUM_RUNS);
              launch_add_run<T, 1, 1>(a, g, stream);
              return hipGetLastError() == hipSuccess ? TS_OK : TS_ERR_LAUNCH;
            }
          }
          if (a.run_reduce && a.sk == 0 && a.B * a.N < 0x7FFFFFFFll && word_ok) {
            constexpr int C = VEC > 1 ? VEC : CN;
            // 16-byte loads pay once the instruction rate limits the stream; small inputs are bound by
            // latency and do better with one atomic per lane straight from registers
            const bool wide = C > CN && n_src * (int64_t)sizeof(T) > ((int64_t)32 << 20);
            const RunGrid g = run_grid(n_edges, a.K / (wide ? C : CN), wide ? C : CN, (wide ? C : CN) * (int)sizeof(T));
            if (g.ok) {
              constexpr int EWD = sizeof(T) < 4 ? 4 / (int)sizeof(T) : 1;  // a whole 32-bit word per atomic
              if (lshift < 0 && !use_lds) ts_note_scatter_route(TS_ROUTE_SUM_RUNS);
              if (wide)
                launch_add_run<T, C, EWD>(a, g, stream);
              else
                launch_add_run<T, CN, EWD>(a, g, stream);
              return hipGetLastError() == hipSuccess ? TS_OK : TS_ERR_LAUNCH;
            }
          }
        }
        if constexpr (__is_same(T, bf16_t) || __is_same(T, f16_t)) {
          if (a.K % 2 == 0 && a.sk == 0 && (reinterpret_cast<uintptr_t>(a.out) & 3) == 0 &&
              (reinterpret_cast<uintptr_t>(a.src) & 3) == 0) {
            ts_note_scatter_route(TS_ROUTE_SUM_ATOMIC);
            hipLaunchKernelGGL(scatter_add_pk16_kernel<T>, dim3(scatter_grid(n_edges, a.K / 2, kBlock, 1)),
                               dim3(kBlock), 0, stream, a);
            return hipGetLastError() == hipSuccess ? TS_OK : TS_ERR_LAUNCH;
          }
        }
        ts_note_scatter_route(TS_ROUTE_SUM_ATOMIC);
        hipLaunchKernelGGL((scatter_atomic_kernel<T, 1, TS_SUM>), dim3(g), dim3(kBlock), 0, stream, a);
      } else {
        // products of the types that the accumulator table takes, one index per row: through the table from 2^16
        // elements on (below, the call is its launches)
        if constexpr (__is_same(T, float) || __is_same(T, bf16_t) || __is_same(T, f16_t) || __is_same(T, double) ||
                      __is_same(T, int32_t) || __is_same(T, int64_t)) {
          int tm = 1;
          while ((int64_t)tm * 2 * a.K <= kLdsAcc && tm * 2 <= kLdsAccRows) tm *= 2;
          if (a.lds_cache && a.sk == 0 && tm >= 64 && a.B * a.N < 0x7FFFFFFFll && n_src >= ((int64_t)1 << 16)) {
            const int64_t epb = per_cu_chunk_edges(a.lds_epb, n_edges, sum_table_min_chunk(a.K, 4),
                                                   131072 / a.K > 2048 ? 131072 / a.K : 2048);
            ts_note_scatter_route(TS_ROUTE_MUL_TABLE);
            hipLaunchKernelGGL((scatter_add_lds_kernel<T, true>), dim3((unsigned)((n_edges + epb - 1) / epb)),
                               dim3(kLdsAddBlock), 0, stream, a, tm - 1, epb);
            return hipGetLastError() == hipSuccess ? TS_OK : TS_ERR_LAUNCH;
          }
        }
        ts_note_scatter_route(TS_ROUTE_MUL_ATOMIC);
        hipLaunchKernelGGL((scatter_atomic_kernel<T, 1, TS_MUL>), dim3(g), dim3(kBlock), 0, stream, a);
      }
    }
  } else if (reduce == TS_MIN || reduce == TS_MAX) {
    const bool is_max = reduce == TS_MAX;
    if constexpr (IsWide<T>::value) {
      const unsigned g_src = grid_for(n_src);
      const T init = is_max ? std::numeric_limits<T>::lowest() : std::numeric_limits<T>::max();
      if (!a.out_given)
        hipLaunchKernelGGL(fill_kernel<T>, dim3(g_out), dim3(kBlock), 0, stream, out, n_out, init);
      hipLaunchKernelGGL(fill_kernel<int64_t>, dim3(g_out), dim3(kBlock), 0, stream, a.arg_out, n_out, a.E);
      if (n_src > 0) {
        // several entries per output slot: keys meet in LDS first (scatter_minmax_wide_lds_kernel)
        int tn = 1;
        while ((int64_t)tn * 2 * a.K <= kLdsAcc && tn * 2 <= kLdsAccRows) tn *= 2;
        ts_note_scatter_route(TS_ROUTE_MINMAX_64BIT);
        const bool table = a.lds_cache && a.sk == 0 && tn >= 16 && a.B * a.N < 0x7FFFFFFFll &&
                           (a.lds_cache == 2 || (n_edges >= ((int64_t)1 << 17) && n_edges >= 4 * a.B * a.N));
        if (table) {
          const int64_t epb = per_cu_chunk_edges(a.lds_epb, n_edges, 16384 / a.K > 256 ? 16384 / a.K : 256,
                                                 131072 / a.K > 2048 ? 131072 / a.K : 2048);
          const dim3 gt((unsigned)((n_edges + epb - 1) / epb));
          if (is_max)
            hipLaunchKernelGGL((scatter_minmax_wide_lds_kernel<T, true>), gt, dim3(kLdsAddBlock), 0, stream, a, tn - 1, epb);
          else
            hipLaunchKernelGGL((scatter_minmax_wide_lds_kernel<T, false>), gt, dim3(kLdsAddBlock), 0, stream, a, tn - 1, epb);
        } else if (is_max) {
          hipLaunchKernelGGL((scatter_minmax_wide_kernel<T, true>), dim3(g_src), dim3(kBlock), 0, stream, a);
        } else {
          hipLaunchKernelGGL((scatter_minmax_wide_kernel<T, false>), dim3(g_src), dim3(kBlock), 0, stream, a);
        }
      }
      if (!a.out_given)
        hipLaunchKernelGGL(mask_init_kernel<T>, dim3(g_out), dim3(kBlock), 0, stream, out, n_out, init);
      if (n_src > 0)
        hipLaunchKernelGGL(scatter_arg_wide_kernel<T>, dim3(g_src), dim3(kBlock), 0, stream, a);
    } else {
      if (a.E >= 0xFFFFFFFEll) return TS_ERR_UNSUPPORTED;
      // LDS-cached variant: one index per row, at least 16 table rows (rows of up to 256 columns: 4 M entries of
      // 128 floats under a Zipf index take 0.74 ms with a table of 32 rows and 3.9 ms through the run kernel),
      // node ids that fit 31 bits,
      // and enough entries per output slot for repeats inside a chunk to be likely (a uniform
      // index with few entries per slot is served better by the direct kernel)
      int tn = 1;
      while ((int64_t)tn * 2 * a.K <= kLdsKeys) tn *= 2;
      // one value per entry: the table kernel whatever the number of entries per output row (10 M entries onto
      // 1 M rows, Zipf(1.2) index: 235 -> 77 us; uniform index: 266 -> 251 us); wider rows only when contended
      // (a uniform index with ten entries per row loses: K = 8 554 -> 737 us)
      const bool contended = a.lds_cache && a.sk == 0 && a.B * a.N < 0x7FFFFFFFll &&
                             (a.lds_cache == 2 ||
                              (n_src >= ((int64_t)1 << 20) &&
                               ((a.K == 1 && n_src >= ((int64_t)1 << 23)) || n_edges >= 32 * a.B * a.N)));
      const bool use_lds = contended && tn >= 16;
      // entries per workgroup chunk: large enough to amortise writing the table back,
      // small enough to leave a few thousand workgroups
      const int64_t epb = lds_chunk_edges(a.lds_epb, a.K, n_edges);
      const unsigned g_lds = (unsigned)((n_edges + epb - 1) / epb);
      const unsigned g_key = scatter_grid(n_edges, a.K / VEC, kBlock, 4);
      if constexpr (sizeof(T) == 4) {
        // one value per entry, a workspace whose key table reads as zero: per-workgroup tables handed over in slabs
        // instead of atomics, misses filtered by a pipelined read (scatter_k1.h)
        if (a.lds_cache && a.lds_k1 && !a.out_given && a.K == 1 && a.B == 1 && a.se == 1 && a.bin_ws != nullptr &&
            ((reinterpret_cast<uintptr_t>(a.src) | reinterpret_cast<uintptr_t>(a.index)) & 15) == 0) {
          const K1Plan kp = k1_plan(a.B, a.E, a.K, a.N, (int)sizeof(T), a.bin_ws, a.bin_ws_bytes, a.lds_cache == 2);
          if (kp.ok) {
            ts_note_scatter_route(TS_ROUTE_MINMAX_K1_SLABS);
            if (is_max)
              launch_scatter_k1<T, true>(a, kp, stream);
            else
              launch_scatter_k1<T, false>(a, kp, stream);
            return hipGetLastError() == hipSuccess ? TS_OK : TS_ERR_LAUNCH;
          }
        }
      }
      if ((a.lds_cache || a.bin_any_size) && a.sk == 0 && a.B * a.N < 0x7FFFFFFFll && a.bin_ws != nullptr &&
          a.K % VEC == 0 && n_src > 0) {
        // large inputs of wide rows with a workspace: entries binned by bucket of output rows, no table misses.
        // Also for an index with few entries per output row (10 M entries onto 1 M rows, uniform / Zipf(1.2) /
        // sorted index: K = 16 894 / 784 / 537 -> 565 / 452 / 357 us, K = 32 1618 / 1169 / 662 -> 757 / 645 / 614 us)
        const BinPlan bp = bin_plan(a.B, a.E, a.K, a.N, (int)sizeof(T), a.bin_ws, a.bin_ws_bytes, a.bin_any_size != 0, 8,
                                    true);
        if (bp.ok && (bp.p.slices == 1 || bin_lane_shift(bp.p, VEC) >= 0)) {
          ts_note_scatter_route(a.sorted_route && a.route_flag != nullptr ? TS_ROUTE_MINMAX_BUCKETS_OR_SEGMENTED
                                                                          : TS_ROUTE_MINMAX_BUCKETS);
          if (is_max)
            launch_binned_keys<T, VEC, true>(a, bp.p, stream);
          else
            launch_binned_keys<T, VEC, false>(a, bp.p, stream);
          if (a.sorted_route && a.route_flag != nullptr) *a.route_flag = bp.p.unsorted;
          return hipGetLastError() == hipSuccess ? TS_OK : TS_ERR_LAUNCH;
        }
      }
      // one index per row, few entries per slot: combine runs of equal neighbouring indices in the
      // wavefront before going to the table (a sorted index then costs one atomic per slot)
      if (!use_lds && a.run_reduce && a.sk == 0 && a.B * a.N < 0x7FFFFFFFll && n_src > 0) {
        constexpr int KC = VEC > 4 ? 4 : VEC;  // columns per lane: 64-bit keys, so at most four
        const RunGrid g = run_grid(n_edges, a.K / KC, 0, KC * (int)sizeof(T));
        if (g.ok) {
          const dim3 gd(g.blocks, g.ychunks);
          // few entries per output row on average, 256 bytes of workspace: the sample of the index decides
          // between this kernel and the table kernel (index_skew_kernel); both are launched, one returns at once
          const bool probe = a.skew_probe && a.lds_cache == 1 && a.K % VEC == 0 && a.bin_ws != nullptr &&
                             a.bin_ws_bytes >= 256 && ((uintptr_t)a.bin_ws & 3) == 0 &&
                             skew_probe_shape(a.B, a.E, a.K, a.N, (int)sizeof(T), a.skew_probe == 2);
          ts_note_scatter_route(probe ? TS_ROUTE_MINMAX_RUNS_OR_TABLE : TS_ROUTE_MINMAX_RUNS);
          ScatterArgs ar = a, al = a;
          if (probe) {
            ar.skew_flag = al.skew_flag = static_cast<const int *>(a.bin_ws);
            ar.skew_want = 0;
            al.skew_want = 1;
            hipLaunchKernelGGL(index_skew_kernel, dim3(1), dim3(kSkewBlock), 0, stream, a, static_cast<int *>(a.bin_ws));
          }
          if (is_max) {
            hipLaunchKernelGGL((scatter_key_init_kernel<T, true>), dim3(g_out), dim3(kBlock), 0, stream, a);
            TS_LAUNCH_RUN(g.serial, (scatter_key_run_kernel<T, KC, true, true>), (scatter_key_run_kernel<T, KC, true, false>),
                          gd, stream, ar, g.lshift, g.rpw);
            if (probe && tn <= 256)
              hipLaunchKernelGGL((scatter_key_lds_kernel<T, VEC, true, 256>), dim3(g_lds), dim3(kLdsBlock), 0, stream,
                                 al, tn - 1, epb);
            else if (probe)
              hipLaunchKernelGGL((scatter_key_lds_kernel<T, VEC, true, kLdsKeys>), dim3(g_lds), dim3(kLdsBlock), 0,
                                 stream, al, tn - 1, epb);
            hipLaunchKernelGGL((scatter_key_final_kernel<T, true>), dim3(g_out), dim3(kBlock), 0, stream, a);
          } else {
            hipLaunchKernelGGL((scatter_key_init_kernel<T, false>), dim3(g_out), dim3(kBlock), 0, stream, a);
            TS_LAUNCH_RUN(g.serial, (scatter_key_run_kernel<T, KC, false, true>),
                          (scatter_key_run_kernel<T, KC, false, false>), gd, stream, ar, g.lshift, g.rpw);
            if (probe && tn <= 256)
              hipLaunchKernelGGL((scatter_key_lds_kernel<T, VEC, false, 256>), dim3(g_lds), dim3(kLdsBlock), 0, stream,
                                 al, tn - 1, epb);
            else if (probe)
              hipLaunchKernelGGL((scatter_key_lds_kernel<T, VEC, false, kLdsKeys>), dim3(g_lds), dim3(kLdsBlock), 0,
                                 stream, al, tn - 1, epb);
            hipLaunchKernelGGL((scatter_key_final_kernel<T, false>), dim3(g_out), dim3(kBlock), 0, stream, a);
          }
          return hipGetLastError() == hipSuccess ? TS_OK : TS_ERR_LAUNCH;
        }
      }
      if (use_lds && a.K == 1 && n_src > 0 && a.lds_k1) {
        ts_note_scatter_route(TS_ROUTE_MINMAX_TABLE_K1);
          const int64_t epb1 = per_cu_chunk_edges(a.lds_epb, n_edges, 16384, 131072);
        const unsigned g1 = (unsigned)((n_edges + epb1 - 1) / epb1);
        if (is_max) {
          hipLaunchKernelGGL((scatter_key_init_kernel<T, true>), dim3(g_out), dim3(kBlock), 0, stream, a);
          hipLaunchKernelGGL((scatter_key_lds_k1_kernel<T, true>), dim3(g1), dim3(kLdsBlockK1), 0, stream, a, epb1);
          hipLaunchKernelGGL((scatter_key_final_kernel<T, true>), dim3(g_out), dim3(kBlock), 0, stream, a);
        } else {
          hipLaunchKernelGGL((scatter_key_init_kernel<T, false>), dim3(g_out), dim3(kBlock), 0, stream, a);
          hipLaunchKernelGGL((scatter_key_lds_k1_kernel<T, false>), dim3(g1), dim3(kLdsBlockK1), 0, stream, a, epb1);
          hipLaunchKernelGGL((scatter_key_final_kernel<T, false>), dim3(g_out), dim3(kBlock), 0, stream, a);
        }
        return hipGetLastError() == hipSuccess ? TS_OK : TS_ERR_LAUNCH;
      }
      ts_note_scatter_route(use_lds ? TS_ROUTE_MINMAX_TABLE : TS_ROUTE_MINMAX_ATOMIC);
      if (is_max) {
        hipLaunchKernelGGL((scatter_key_init_kernel<T, true>), dim3(g_out), dim3(kBlock), 0, stream, a);
        if (n_src > 0) {
          if (use_lds && tn <= 256)
            hipLaunchKernelGGL((scatter_key_lds_kernel<T, VEC, true, 256>), dim3(g_lds), dim3(kLdsBlock), 0, stream,
                               a, tn - 1, epb);
          else if (use_lds)
            hipLaunchKernelGGL((scatter_key_lds_kernel<T, VEC, true, kLdsKeys>), dim3(g_lds), dim3(kLdsBlock), 0,
                               stream, a, tn - 1, epb);
          else
            hipLaunchKernelGGL((scatter_key_kernel<T, VEC, true>), dim3(g_key), dim3(kBlock), 0, stream, a);
        }
        hipLaunchKernelGGL((scatter_key_final_kernel<T, true>), dim3(g_out), dim3(kBlock), 0, stream, a);
      } else {
        hipLaunchKernelGGL((scatter_key_init_kernel<T, false>), dim3(g_out), dim3(kBlock), 0, stream, a);
        if (n_src > 0) {
          if (use_lds && tn <= 256)
            hipLaunchKernelGGL((scatter_key_lds_kernel<T, VEC, false, 256>), dim3(g_lds), dim3(kLdsBlock), 0, stream,
                               a, tn - 1, epb);
          else if (use_lds)
            hipLaunchKernelGGL((scatter_key_lds_kernel<T, VEC, false, kLdsKeys>), dim3(g_lds), dim3(kLdsBlock), 0,
                               stream, a, tn - 1, epb);
          else
            hipLaunchKernelGGL((scatter_key_kernel<T, VEC, false>), dim3(g_key), dim3(kBlock), 0, stream, a);
        }
        hipLaunchKernelGGL((scatter_key_final_kernel<T, false>), dim3(g_out), dim3(kBlock), 0, stream, a);
      }
    }
  } else {
    return TS_ERR_UNSUPPORTED;
  }
  return hipGetLastError() == hipSuccess ? TS_OK : TS_ERR_LAUNCH;
}

// vec: elements per lane the caller found safe (alignment, K divisible)
template <typename T> int launch_scatter(const ScatterArgs &a, int reduce, int vec, hipStream_t stream);

#define TS_INSTANTIATE_SCATTER(T, FULLVEC)                                                       \
  template <> int launch_scatter<T>(const ScatterArgs &a, int reduce, int vec, hipStream_t stream) { \
    if (vec == FULLVEC) return launch_scatter_v<T, FULLVEC>(a, reduce, stream);                  \
    return launch_scatter_v<T, 1>(a, reduce, stream);                                            \
  }

}  // namespace ts
