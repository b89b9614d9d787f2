// Segmented reduction over CSR row pointers (segment_csr, and segment_coo once
// its sorted index has been turned into row pointers).
//
// One pass over src. The merged list of edges and row ends is cut into tiles of
// `BI` items per workgroup and `BI / W` items per lane group ("worker": G lanes
// that together hold one 16-byte-per-lane slice of a feature row). A worker
// walks its edges in order with U loads in flight, keeps the running reduction
// in registers and writes every row that starts and ends inside its range
// straight to `out`. A row that crosses a worker boundary leaves partials in
// LDS which the workgroup combines in edge order; a row that crosses a
// workgroup boundary leaves partials (carries) in the global workspace. The tile in
// which such a row ends collects the carries of the tiles before it in tile order
// (look-back, carry_* below: memory-side atomics, nonce-tagged flags, a bounded wait);
// 8- and 16-bit accumulators, more than four column chunks and the narrow-row kernel
// leave the combination to a small second kernel instead. Either way the order of the
// combination is fixed by the tiling, so the result is independent of scheduling.
// If the bounded wait runs out (row pointers that are not monotone, or a producer tile
// that did not run for seconds) the row is written as empty (0, arg = E) and the call's
// nonce is left in the second status word of the workspace (see CsrReduceArgs::status).
//
// Semantics follow the reference CPU loop (csrc/cpu/segment_csr_cpu.cpp:54-88):
// accumulate in float for 16-bit floats, strict compare so the first index
// wins ties, mean = T(sum) / T(count), empty row -> 0 with arg = E.
#pragma once

#include <stdlib.h>

#include "device_utils.h"
#include "merge_path.h"

namespace ts {

constexpr int kMaxBlockItems = 2048;  // rows + edges per workgroup tile
#ifndef TS_CSR_U
#define TS_CSR_U 4
#endif
#ifndef TS_CSR_BLOCK
#define TS_CSR_BLOCK 256
#endif
constexpr int kCsrBlock = TS_CSR_BLOCK;  // lanes per workgroup of csr_reduce_kernel
constexpr int kCsrMaxItems = kMaxBlockItems * kCsrBlock / 256;  // rows + edges per tile of csr_reduce_kernel
constexpr int kSharedWalkMin = 32;  // tiles a row must have passed through before the workgroup shares the walk
constexpr int kLoadsInFlight = TS_CSR_U;  // U: 16-byte loads per lane per batch (two batches in flight)

struct CsrReduceArgs {
  const void *src;
  const int64_t *indptr;
  void *out;
  int64_t *arg_out;   // min/max
  void *count_out;    // optional, mean: T(max(count, 1)) per row
  int64_t N, E, K;
  int64_t indptr_batch_stride;
  int accumulate;     // combine with the previous content of out (segment_coo with out=)
  int G;              // lanes per worker
  int BI;             // items per workgroup tile (= workers * ipw)
  int ipw;            // items per worker
  int64_t nblk;       // tiles per batch
  // workspace
  void *ws_vals;      // Acc [B][nblk][2][K]
  int32_t *ws_args;   // int32 [B][nblk][2][K]  (min/max)
  int64_t *ws_meta;   // int64 [B][nblk][4]: head_row, head_closes, tail_row, length of the tail row
                      // (look-back mode: one carry flag per column chunk instead)
  int lookback;       // rows that cross tiles are finished inside the kernel (see carry_* below)
  uint64_t nonce;     // tag of this call's carry flags, never 0
  // optional: entry e of the row-pointer order lives in row perm[e] of src (a scatter whose index was
  // sorted once: perm = stable argsort of the index). Positions handed to arg_out stay in row-pointer order.
  const int32_t *perm;
  int64_t perm_batch_stride;
  int perm_args;      // min / max with perm: the kernel itself writes positions in src's order and applies
                      // scatter's rule for slots that never beat the initial value (no pass over arg_out after it)
  // status words of the call (device memory, two 64-bit words, may be null): word 0 receives status_nonce from
  // the first tile when status_reset is set ("the latest call"), word 1 receives status_nonce from a tile whose
  // look-back ran out of polls ("the latest call that gave a row up"). The call gave a row up iff the two are
  // equal afterwards: no write has to be ordered against another one, and a word left by an earlier call
  // never matches.
  // optional gate (a scatter whose index turned out to be sorted takes this reduction instead of the buckets):
  // the kernel returns at once unless (*gate != 0) == (gate_want != 0). scatter_rule: min / max write a slot whose
  // entries never beat the initial value of the element type as 0 with position E, as scatter does
  // (csrc/cpu/scatter_cpu.cpp:81-82). Both need the look-back mode and a call without perm / accumulate.
  const int *gate = nullptr;
  int gate_want = 0;
  int scatter_rule = 0;
  unsigned long long *status;
  int status_reset;
  uint64_t status_nonce;  // never 0; the same for every slice of one call
  int carry_spin;     // polls per batch of carry flags before the look-back gives up; < 0: give up without polling
};

// ---- rows that cross tiles, finished without a second kernel ---------------------------------
// The tile in which such a row ends walks back over the tiles before it. A tile whose last row is
// still open at its end publishes that row's partial result as its carry: kCarryTail when the row
// began inside the tile, kCarryPass when it only passes through (then the walk continues with the
// tile before). Carries and flags move through device-scope read-modify-write atomics, which execute
// at the memory side and so are coherent between the XCDs' L2 caches without a cache write-back (a
// release fence per workgroup was measured and made the kernel 4x slower). The flag is written
// after the wavefront has received the returns of its carry writes, i.e. after they were performed.
// Tiles only ever wait for tiles with a smaller index, which the dispatcher started earlier, and
// publishing never waits, so the walk cannot deadlock; it is bounded all the same: when the polls run out
// (an indptr that is not monotone never publishes what the walk waits for) the row is written as empty and
// the call's status word is set. A flag holds the call's nonce, so stale workspace content never
// matches, and its reader clears it, so a replay of a captured launch (same nonce, same workspace)
// starts clean.
constexpr uint64_t kCarryTail = 1, kCarryPass = 2;
constexpr int kCarrySpin = 1 << 20;  // default of CsrReduceArgs::carry_spin

template <typename A> struct CarryBits { typedef uint32_t type; };
template <> struct CarryBits<double> { typedef uint64_t type; };
template <> struct CarryBits<int64_t> { typedef uint64_t type; };

template <typename A> __device__ __forceinline__ uint64_t carry_put(A *p, A v) {
  typedef typename CarryBits<A>::type U;
  static_assert(sizeof(U) == sizeof(A), "");
  U bits;
  __builtin_memcpy(&bits, &v, sizeof(A));
  return (uint64_t)__hip_atomic_exchange(reinterpret_cast<U *>(p), bits, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
}
template <typename A> __device__ __forceinline__ A carry_get(A *p) {
  typedef typename CarryBits<A>::type U;
  const U bits = __hip_atomic_fetch_or(reinterpret_cast<U *>(p), (U)0, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
  A v;
  __builtin_memcpy(&v, &bits, sizeof(A));
  return v;
}

template <typename A, int REDUCE>
__device__ __forceinline__ void reduce_step(A &acc, int32_t &arg, A v, int32_t e) {
  if (REDUCE == TS_SUM || REDUCE == TS_MEAN) {
    acc = acc + v;
  } else if (REDUCE == TS_MIN) {
    if (v < acc) { acc = v; arg = e; }
  } else {
    if (v > acc) { acc = v; arg = e; }
  }
}

// Write one finished row slice. `count` is the full length of the row.
// ACCUM: 0 = `out` is overwritten (known at compile time: the row-end code sits in divergent control flow,
// where every instruction counts), -1 = decided by a.accumulate at run time.
// PERM: 0 rows in place, 1 rows through a.perm, 2 rows in place under a.gate with scatter's rule for min / max
template <typename T, int VEC, int REDUCE, int ACCUM = -1, int PERM = 0>
__device__ __forceinline__ void finalize_row_at(const CsrReduceArgs &a, T *op, int64_t *ap, T *count_slot,
                                                const typename Acc<T>::type *acc, const int32_t *arg,
                                                int64_t count, const int32_t *perm_b = nullptr) {
  // op / ap: the row's slice in out / arg_out; count_slot: where the row's count goes (mean with a count output)
  typedef typename Acc<T>::type A;
  const bool accumulate = ACCUM < 0 ? a.accumulate != 0 : ACCUM != 0;
  if (accumulate && count == 0) return;  // rows without entries keep their content
  Vec<T, VEC> o;
  int64_t oa[VEC];
  Vec<T, VEC> prev;
  if (accumulate) prev = load_vec<T, VEC>(op);
#pragma unroll
  for (int v = 0; v < VEC; ++v) {
    A x = acc[v];
    if (REDUCE == TS_SUM || REDUCE == TS_MEAN) {
      if (accumulate) x = to_acc<T>(prev.v[v]) + x;
      T t = from_acc<T>(x);
      if (REDUCE == TS_MEAN && count > 1) t = div_elem<T>(t, count_as<T>(count));  // x / 1 == x
      o.v[v] = t;
    } else {
      if (accumulate) {
        const A p = to_acc<T>(prev.v[v]);
        const bool beats = (REDUCE == TS_MIN) ? (x < p) : (x > p);
        o.v[v] = beats ? from_acc<T>(x) : prev.v[v];
        oa[v] = beats ? (int64_t)arg[v] : a.E;
      } else {
        o.v[v] = count > 0 ? from_acc<T>(x) : zero_elem<T>();
        oa[v] = count > 0 ? (int64_t)arg[v] : a.E;
        if constexpr (PERM != 0) {
          if ((PERM == 2 || perm_b != nullptr) && count > 0) {
            // scatter's view of the slot: the position in src's order, or 0 and E if nothing beat the initial
            // value of the element type (csrc/cpu/scatter_cpu.cpp:81-82)
            const A lim = to_acc<T>(REDUCE == TS_MAX ? ElemLim<T>::lowest() : ElemLim<T>::max());
            const A xv = to_acc<T>(o.v[v]);
            if ((REDUCE == TS_MAX) ? (xv > lim) : (xv < lim)) {
              if (PERM == 1) oa[v] = perm_b[arg[v]];
            } else {
              o.v[v] = zero_elem<T>();
              oa[v] = a.E;
            }
          }
        }
      }
    }
  }
  store_vec<T, VEC>(op, o);
  if (REDUCE == TS_MIN || REDUCE == TS_MAX) {
#pragma unroll
    for (int v = 0; v < VEC; ++v) ap[v] = oa[v];
  }
  if (REDUCE == TS_MEAN && count_slot != nullptr) *count_slot = count_as<T>(count > 0 ? count : 1);
}

template <typename T, int VEC, int REDUCE, int ACCUM = -1, int PERM = 0>
__device__ __forceinline__ void finalize_row(const CsrReduceArgs &a, T *out_b, int64_t *arg_b,
                                             T *count_b, int64_t row, int64_t col, int lg,
                                             const typename Acc<T>::type *acc, const int32_t *arg,
                                             int64_t count, bool col_ok, const int32_t *perm_b = nullptr) {
  if (!col_ok) return;
  constexpr bool kArg = REDUCE == TS_MIN || REDUCE == TS_MAX;
  finalize_row_at<T, VEC, REDUCE, ACCUM, PERM>(a, out_b + row * a.K + col, kArg ? arg_b + row * a.K + col : nullptr,
                                               (count_b != nullptr && col == 0 && lg == 0) ? count_b + row : nullptr,
                                               acc, arg, count, perm_b);
}

// Workgroups per CU the register allocation aims at: six for sum / mean of 4- and 8-byte types (80 VGPRs;
// mean would take 82 and drop to five, measured 7 % slower on 146 MB inputs). The other instantiations keep
// the compiler's choice (forcing five on the 16-bit mean cost 3 % on 16 GB inputs).
template <typename T, int VEC, int REDUCE, int PERM = 0> constexpr int csr_reduce_min_blocks() {
  return PERM == 1 ? 1 : ((REDUCE == TS_SUM || REDUCE == TS_MEAN) && sizeof(T) >= 4 ? 6 : 1);  // PERM: 8 KB more LDS
}
template <typename T, int VEC, int REDUCE, int ACCUM, int PERM = 0>
__global__ __launch_bounds__(kCsrBlock, (csr_reduce_min_blocks<T, VEC, REDUCE, PERM>())) void csr_reduce_kernel(CsrReduceArgs a) {
  typedef typename Acc<T>::type A;
  constexpr bool kArg = (REDUCE == TS_MIN || REDUCE == TS_MAX);
  constexpr int U = kLoadsInFlight;

  __shared__ int32_t s_ptr[kCsrMaxItems + 4];  // row pointers of the tile + one sentinel
  __shared__ int32_t s_perm[PERM == 1 ? kCsrMaxItems : 1];  // source rows of the tile's entries
  __shared__ A s_val[2 * kCsrBlock * VEC];
  __shared__ int32_t s_arg[kArg ? 2 * kCsrBlock * VEC : 1];
  __shared__ int32_t s_head_row[kCsrBlock];    // local row of the head partial, -1: none
  __shared__ int32_t s_head_closes[kCsrBlock];
  __shared__ int32_t s_tail_row[kCsrBlock];    // local row of the tail partial, -1: none
  __shared__ int64_t s_cut[2];
  if constexpr (PERM == 2) {
    if (a.gate != nullptr && (*a.gate != 0) != (a.gate_want != 0)) return;  // the same for every wavefront of the grid
  }

  const int tid = threadIdx.x;
  const int G = a.G;
  const int W = kCsrBlock / G;
  const int w = tid / G;
  const int lg = tid - w * G;
  const int CW = G * VEC;
  const int64_t col = (int64_t)blockIdx.y * CW + (int64_t)lg * VEC;
  const bool col_ok = col < a.K;
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
  if constexpr (kCsrBlock >= 2 * kWave) {
    if (wave < 2) {
      const int64_t i = merge_search_wave(ptr, a.N, a.E, wave == 0 ? d0 : d1);
      if ((tid & (kWave - 1)) == 0) s_cut[wave] = i;
    }
  } else {
    const int64_t ia = merge_search_wave(ptr, a.N, a.E, d0), ib = merge_search_wave(ptr, a.N, a.E, d1);
    if (tid == 0) { s_cut[0] = ia; s_cut[1] = ib; }
  }
  if (a.status_reset && a.status != nullptr && tid == 0 && (blockIdx.x | blockIdx.y | blockIdx.z) == 0)
    __hip_atomic_exchange(a.status, (unsigned long long)a.status_nonce, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
  __syncthreads();
  const int64_t i0 = s_cut[0], i1 = s_cut[1];
  const int64_t j0 = d0 - i0;
  const int nr = (int)(i1 - i0);         // row ends inside the tile
  const int ne = (int)((d1 - i1) - j0);  // edges inside the tile

  // ---- row pointers of the tile into LDS, relative to the tile's first edge
  const int64_t last = i1 + 1 < a.N ? i1 + 1 : a.N;
  const int nload = (int)(last - i0) + 1;  // ptr[i0 .. last]
  for (int t = tid; t < nload; t += kCsrBlock) s_ptr[t] = (int32_t)(ptr[i0 + t] - j0);
  if (tid == 0) { s_ptr[nload] = INT32_MAX; s_ptr[nload + 1] = INT32_MAX; }  // rows past the last one never end
  const int32_t *arg_perm = nullptr;  // set: positions leave the kernel in src's order
  if constexpr (PERM == 1) {
    const int32_t *perm_b = a.perm + b * a.perm_batch_stride;
    const int32_t last_row = a.E > 0 ? (int32_t)(a.E - 1) : 0;
    for (int t = tid; t < ne; t += kCsrBlock) {
      const int32_t r = perm_b[j0 + t];
      s_perm[t] = r < 0 ? 0 : (r > last_row ? last_row : r);  // a malformed perm must not read outside src
    }
    if (kArg && a.perm_args) arg_perm = perm_b;
  }
  s_head_row[tid] = -1;
  s_tail_row[tid] = -1;
  __syncthreads();

  // ---- worker cut
  const int ipw = a.ipw;
  const int tile_items = nr + ne;
  int dw0 = w * ipw;
  int dw1 = dw0 + ipw;
  dw0 = dw0 < tile_items ? dw0 : tile_items;
  dw1 = dw1 < tile_items ? dw1 : tile_items;
  const int ri0 = merge_search_lds(s_ptr, nr, ne, dw0);
  const int ri1 = merge_search_lds(s_ptr, nr, ne, dw1);
  int je0 = dw0 - ri0;
  const int je1 = dw1 - ri1;
  // Entries in front of the first row pointer (indptr[0] > 0) belong to no row. Only row 0 can begin
  // behind a worker's first entry: every other row begins where the row before it ended.
  if (i0 + ri0 == 0 && s_ptr[0] > je0) je0 = s_ptr[0] < je1 ? s_ptr[0] : je1;

  auto row_end = [&](int r) -> int32_t { return s_ptr[r + 1]; };  // r + 1 <= nload + 1: a sentinel at the latest

  A acc[VEC];
  int32_t arg[VEC];
#pragma unroll
  for (int v = 0; v < VEC; ++v) { acc[v] = acc_init<A, REDUCE>(); arg[v] = 0; }

  const bool has_work = (ri1 > ri0) || (je1 > je0);
  // the worker's first row began before the worker's first edge
  const bool head_open = has_work && (i0 + ri0 < a.N) && (s_ptr[ri0] < je0);

  A *my_head_val = s_val + (size_t)w * CW + lg * VEC;
  A *my_tail_val = s_val + (size_t)kCsrBlock * VEC + (size_t)w * CW + lg * VEC;
  int32_t *my_head_arg = s_arg + (kArg ? (size_t)w * CW + lg * VEC : 0);
  int32_t *my_tail_arg = s_arg + (kArg ? (size_t)kCsrBlock * VEC + (size_t)w * CW + lg * VEC : 0);

  int r = ri0;
  T *op_row = out_b + (i0 + r) * a.K + (col_ok ? col : 0);
  int64_t *ap_row = kArg ? arg_b + (i0 + r) * a.K + (col_ok ? col : 0) : nullptr;
  T *cp_row = (count_b != nullptr && col == 0 && lg == 0) ? count_b + (i0 + r) : nullptr;
  int32_t rbeg = s_ptr[r];       // first edge of row r
  int32_t rend = row_end(r);
  int32_t rnext = row_end(r + 1);  // read one row ahead: a row end then never waits for LDS

  auto flush = [&]() {
    if (r == ri0 && head_open) {
#pragma unroll
      for (int v = 0; v < VEC; ++v) {
        my_head_val[v] = acc[v];
        if (kArg) my_head_arg[v] = arg[v];
      }
      if (lg == 0) { s_head_row[w] = r; s_head_closes[w] = 1; }
    } else if (col_ok) {
      finalize_row_at<T, VEC, REDUCE, ACCUM, PERM>(a, op_row, ap_row, cp_row, acc, arg,
                                                   (int64_t)(int32_t)(rend - rbeg), arg_perm);  // the length fits 32 bits
    }
#pragma unroll
    for (int v = 0; v < VEC; ++v) acc[v] = acc_init<A, REDUCE>();
    ++r;
    op_row += a.K;  // the slices of row r in out / arg_out / count: no 64-bit multiply per row end
    if (kArg) ap_row += a.K;
    if (cp_row != nullptr) ++cp_row;
    rbeg = rend;
    rend = rnext;
    rnext = row_end(r + 1);
  };

  const int64_t col_ld = col_ok ? col : 0;  // idle lanes re-read column 0
  const T *src_col = src_b + col_ld;
  // Software pipeline: the loads of batch i+1 are issued before batch i is
  // reduced, so a wavefront always has U to 2U 16-byte loads outstanding.
  auto load_batch = [&](Vec<T, VEC> *x, int e) {
#pragma unroll
    for (int u = 0; u < U; ++u) {
      int ee = e + u < je1 ? e + u : je1 - 1;
      const int64_t srow = PERM == 1 ? (int64_t)s_perm[ee] : j0 + ee;
      x[u] = load_vec_stream<T, VEC>(src_col + srow * a.K);
    }
  };
  Vec<T, VEC> x[U];
  if (je0 < je1) load_batch(x, je0);
  for (int e = je0; e < je1; e += U) {
    Vec<T, VEC> y[U];
    load_batch(y, e + U);  // unconditional (addresses are clamped): keeps the wait counts exact
#pragma unroll
    for (int u = 0; u < U; ++u) {
      const int ce = e + u;
      if (ce < je1) {
        while (ce >= rend) flush();
        const int32_t ge = (int32_t)(j0 + ce);
#pragma unroll
        for (int v = 0; v < VEC; ++v) reduce_step<A, REDUCE>(acc[v], arg[v], to_acc<T>(x[u].v[v]), ge);
      }
    }
#pragma unroll
    for (int u = 0; u < U; ++u) x[u] = y[u];
  }
  while (r < ri1) flush();

  // edges of a row whose end lies beyond this worker
  if (has_work && (i0 + r < a.N)) {
    const int32_t rs = s_ptr[r];
    const int first = rs > je0 ? rs : je0;
    if (je1 > first) {
      if (r == ri0 && head_open) {
#pragma unroll
        for (int v = 0; v < VEC; ++v) {
          my_head_val[v] = acc[v];
          if (kArg) my_head_arg[v] = arg[v];
        }
        if (lg == 0) { s_head_row[w] = r; s_head_closes[w] = 0; }
      } else {
#pragma unroll
        for (int v = 0; v < VEC; ++v) {
          my_tail_val[v] = acc[v];
          if (kArg) my_tail_arg[v] = arg[v];
        }
        if (lg == 0) s_tail_row[w] = r;
      }
    }
  }
  constexpr bool kCarryOk = sizeof(A) >= 4;  // carries move through 32- and 64-bit atomics
  const bool lookback = kCarryOk && a.lookback != 0;
  // default: the tile leaves no open row; the worker that does overwrites this after the barrier
  if (!lookback && tid == 0 && blockIdx.y == 0) a.ws_meta[(b * a.nblk + blockIdx.x) * 4 + 2] = -1;
  __syncthreads();
  // The row that entered the tile from the one before began more than kSharedWalkMin tiles back (a hub row):
  // if it ends here, the walk over those tiles is shared by the whole workgroup. Every lane derives the same
  // answer from LDS, so tiles without such a row, nearly all, pay two LDS reads and no barrier.
  bool shared_walk = false;
  if (lookback && s_head_row[0] >= 0) {
    const int row0 = s_head_row[0];
    shared_walk = (i0 + row0) + ((int64_t)s_ptr[row0] + j0) < ((int64_t)blockIdx.x - kSharedWalkMin) * a.BI;
  }

  // ---- combine partials of rows that cross worker boundaries, in edge order
  A *ws_val_blk = static_cast<A *>(a.ws_vals) + ((b * a.nblk + blockIdx.x) * 2) * a.K;
  int32_t *ws_arg_blk = kArg ? a.ws_args + ((b * a.nblk + blockIdx.x) * 2) * a.K : nullptr;
  int64_t *meta = a.ws_meta + (b * a.nblk + blockIdx.x) * 4;

  // look-back mode: this tile's carry slot is the second of its two partial slots
  uint64_t *carry_flags = reinterpret_cast<uint64_t *>(a.ws_meta) + (b * a.nblk) * 4 + blockIdx.y;
  // Where element v of this lane's slice sits inside a carry row. The lanes of a worker hold VEC neighbouring
  // columns each, so instruction v of a carry written column by column would touch G addresses VEC elements apart
  // -- every 64-byte sector of the row VEC times over, and each of those atomics is a read-modify-write of a
  // sector at the memory side (C5: 254 MB written next to 614 MB of output). With whole column chunks the
  // carry row is stored transposed instead: instruction v covers G neighbouring elements. Reader and writer
  // use the same rule; the layout is private to the look-back.
  const bool carry_transposed = a.K % CW == 0;
  auto carry_pos = [&](int v) -> int64_t {
    return carry_transposed ? (int64_t)blockIdx.y * CW + (int64_t)v * G + lg : col + v;
  };
  auto publish_carry = [&](uint64_t kind) {
    if constexpr (kCarryOk) {
    uint64_t sink = 0;
    if (col_ok) {
#pragma unroll
      for (int v = 0; v < VEC; ++v) {
        sink |= carry_put<A>(ws_val_blk + a.K + carry_pos(v), acc[v]);
        if (kArg) sink |= carry_put<int32_t>(ws_arg_blk + a.K + carry_pos(v), arg[v]);
      }
    }
    asm volatile("" ::"v"(sink) : "memory");  // the returns are in: the carry is in memory
    if (lg == 0)
      __hip_atomic_exchange(carry_flags + (int64_t)blockIdx.x * 4, (a.nonce << 2) | kind, __ATOMIC_RELAXED,
                            __HIP_MEMORY_SCOPE_AGENT);
    }
  };
  // acc / arg hold the last part of a row that began in an earlier tile: put the carries of the tiles before
  // in front. first_tile is the tile in which the row began (from its row pointer), so the tiles to visit
  // are known in advance and are polled and read several at a time: a hub row that passes through hundreds
  // of tiles costs a few memory round trips per batch, not per tile.
  // (start, stride): the tiles start, start - stride, ... down to first_tile; one worker walking alone takes
  // (blockIdx.x - 1, 1), the workers of a workgroup that share a long walk take every W-th tile each.
  // false: the wait for a carry ran out; the status word is set and the caller writes the row as empty
  auto walk_back = [&](int64_t first_tile, int64_t start, int64_t stride) -> bool {
    if constexpr (kCarryOk) {
    constexpr int PF = VEC <= 4 ? 4 : 2;
    A *vals_b = static_cast<A *>(a.ws_vals) + (b * a.nblk) * 2 * a.K;
    int32_t *args_b = kArg ? a.ws_args + (b * a.nblk) * 2 * a.K : nullptr;
    const int64_t c = col_ok ? col : 0;
    if (first_tile < 0) first_tile = 0;
    for (int64_t hi = start; hi >= first_tile; hi -= PF * stride) {
      const int64_t left = (hi - first_tile) / stride + 1;
      const int n = left < PF ? (int)left : PF;  // tiles hi, hi - stride, ...
      bool ready[PF];
#pragma unroll
      for (int q = 0; q < PF; ++q) ready[q] = q >= n;
      int spin = a.carry_spin;
      while (spin >= 0) {
        uint64_t f[PF];
#pragma unroll
        for (int q = 0; q < PF; ++q)
          f[q] = ready[q] ? 0 : __hip_atomic_fetch_or(carry_flags + (hi - q * stride) * 4, 0ull, __ATOMIC_RELAXED,
                                                       __HIP_MEMORY_SCOPE_AGENT);
        bool all = true;
#pragma unroll
        for (int q = 0; q < PF; ++q) {
          ready[q] = ready[q] || (f[q] >> 2) == a.nonce;
          all = all && ready[q];
        }
        if (all || --spin <= 0) break;
        __builtin_amdgcn_s_sleep(4);
      }
      if (spin <= 0) {  // e.g. indptr not monotone: these carries will never be published
        if (lg == 0 && a.status != nullptr)
          __hip_atomic_exchange(a.status + 1, (unsigned long long)a.status_nonce, __ATOMIC_RELAXED,
                                __HIP_MEMORY_SCOPE_AGENT);
        return false;
      }
      asm volatile("" ::: "memory");
      A early[PF][VEC];
      int32_t early_arg[PF][VEC];
#pragma unroll
      for (int q = 0; q < PF; ++q) {
        if (q < n) {
#pragma unroll
          for (int v = 0; v < VEC; ++v) {
            const int64_t cp = col_ok ? carry_pos(v) : (int64_t)v;
            early[q][v] = carry_get<A>(vals_b + ((hi - q * stride) * 2 + 1) * a.K + cp);
            if (kArg) early_arg[q][v] = carry_get<int32_t>(args_b + ((hi - q * stride) * 2 + 1) * a.K + cp);
          }
        }
      }
#pragma unroll
      for (int q = 0; q < PF; ++q) {
        if (q < n) {
#pragma unroll
          for (int v = 0; v < VEC; ++v) {
            if (kArg) {
              reduce_step<A, REDUCE>(early[q][v], early_arg[q][v], acc[v], arg[v]);  // earlier entries win ties
              arg[v] = early_arg[q][v];
              acc[v] = early[q][v];
            } else {
              acc[v] = early[q][v] + acc[v];
            }
          }
        }
      }
      asm volatile("" ::: "memory");
      if (lg == 0) {
#pragma unroll
        for (int q = 0; q < PF; ++q)
          if (q < n)
            __hip_atomic_exchange(carry_flags + (hi - q * stride) * 4, 0ull, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
      }
    }
    }
    return true;
  };

  auto absorb_head = [&](int ww) {
    const A *hv = s_val + (size_t)ww * CW + lg * VEC;
    const int32_t *ha = s_arg + (kArg ? (size_t)ww * CW + lg * VEC : 0);
#pragma unroll
    for (int v = 0; v < VEC; ++v) {
      if (kArg)
        reduce_step<A, REDUCE>(acc[v], arg[v], hv[v], ha[v]);
      else
        acc[v] = acc[v] + hv[v];
    }
  };

  if (s_tail_row[w] >= 0) {
    // this worker opened a row: gather the heads of the workers after it
    const int row = s_tail_row[w];
#pragma unroll
    for (int v = 0; v < VEC; ++v) { acc[v] = my_tail_val[v]; if (kArg) arg[v] = my_tail_arg[v]; }
    bool closed = false;
    for (int ww = w + 1; ww < W && !closed; ++ww) {
      if (s_head_row[ww] < 0) continue;  // worker without items (tile end)
      absorb_head(ww);
      closed = s_head_closes[ww] != 0;
    }
    if (closed) {
      finalize_row<T, VEC, REDUCE, ACCUM, PERM>(a, out_b, arg_b, count_b, i0 + row, col, lg, acc, arg,
                                                (int64_t)s_ptr[row + 1] - (int64_t)s_ptr[row], col_ok, arg_perm);
    } else if (lookback) {
      publish_carry(kCarryTail);
    } else {
      if (col_ok) {
#pragma unroll
        for (int v = 0; v < VEC; ++v) {
          ws_val_blk[a.K + col + v] = acc[v];
          if (kArg) ws_arg_blk[a.K + col + v] = arg[v];
        }
      }
      if (lg == 0 && blockIdx.y == 0) {
        meta[2] = i0 + row;
        meta[3] = (int64_t)s_ptr[row + 1] - (int64_t)s_ptr[row];  // full length of the row
      }
    }
  }
  if (w == 0) {
    // the row that entered the tile from the previous one
    if (s_head_row[0] >= 0) {
#pragma unroll
      for (int v = 0; v < VEC; ++v) { acc[v] = my_head_val[v]; if (kArg) arg[v] = my_head_arg[v]; }
      bool closed = s_head_closes[0] != 0;
      for (int ww = 1; ww < W && !closed; ++ww) {
        if (s_head_row[ww] < 0) continue;
        absorb_head(ww);
        closed = s_head_closes[ww] != 0;
      }
      if (lookback) {
        if (closed) {
          const int row = s_head_row[0];
          // the row's first entry sits at merge position (row index + row pointer)
          int64_t first_tile = ((i0 + row) + ((int64_t)s_ptr[row] + j0)) / a.BI;
          if (first_tile < 0) first_tile = 0;
          if (shared_walk) {
#pragma unroll
            for (int v = 0; v < VEC; ++v) { my_tail_val[v] = acc[v]; if (kArg) my_tail_arg[v] = arg[v]; }
            if (lg == 0) s_cut[0] = first_tile;
          } else {
            const bool ok = walk_back(first_tile, (int64_t)blockIdx.x - 1, 1);
            if (!ok) {
#pragma unroll
              for (int v = 0; v < VEC; ++v) acc[v] = acc_init<A, REDUCE>();  // the row is written as empty
            }
            finalize_row<T, VEC, REDUCE, ACCUM, PERM>(a, out_b, arg_b, count_b, i0 + row, col, lg, acc, arg,
                                                      ok ? (int64_t)s_ptr[row + 1] - (int64_t)s_ptr[row] : 0, col_ok,
                                                      arg_perm);
          }
        } else {
          publish_carry(kCarryPass);
          if (shared_walk && lg == 0) s_cut[0] = -1;  // the row goes on: nothing to walk here
        }
      } else {
        if (col_ok) {
#pragma unroll
          for (int v = 0; v < VEC; ++v) {
            ws_val_blk[col + v] = acc[v];
            if (kArg) ws_arg_blk[col + v] = arg[v];
          }
        }
        if (lg == 0 && blockIdx.y == 0) { meta[0] = i0 + s_head_row[0]; meta[1] = closed ? 1 : 0; }
      }
    } else if (!lookback && lg == 0 && blockIdx.y == 0) {
      meta[0] = -1;
      meta[1] = 0;
    }
  }

  // ---- a long walk shared by the workgroup: worker w collects the carries of the tiles
  // blockIdx.x - 1 - w, - W, ... into a partial of its own; worker 0 then folds the partials in worker order.
  // The grouping is fixed by the tiling, so the result is the same on every call.
  if constexpr (kCarryOk) {
    if (!shared_walk) return;
    __syncthreads();
    const int64_t first_tile = s_cut[0];
    if (first_tile < 0) return;
#pragma unroll
    for (int v = 0; v < VEC; ++v) { acc[v] = acc_init<A, REDUCE>(); arg[v] = INT32_MAX; }
    const bool ok = walk_back(first_tile, (int64_t)blockIdx.x - 1 - w, W);
    A *part_val = s_val + (size_t)w * CW + lg * VEC;  // the head slots: read for the last time before the barrier
    int32_t *part_arg = s_arg + (kArg ? (size_t)w * CW + lg * VEC : 0);
#pragma unroll
    for (int v = 0; v < VEC; ++v) { part_val[v] = acc[v]; if (kArg) part_arg[v] = arg[v]; }
    if (!ok && lg == 0) s_head_closes[0] = -1;  // read before the first barrier for the last time; now: a walk failed
    __syncthreads();
    if (w != 0) return;
    const bool all_ok = s_head_closes[0] != -1;
#pragma unroll
    for (int v = 0; v < VEC; ++v) { acc[v] = my_tail_val[v]; if (kArg) arg[v] = my_tail_arg[v]; }
    for (int ww = 0; ww < W; ++ww) {
      const A *pv = s_val + (size_t)ww * CW + lg * VEC;
      const int32_t *pa = s_arg + (kArg ? (size_t)ww * CW + lg * VEC : 0);
#pragma unroll
      for (int v = 0; v < VEC; ++v) {
        if (kArg) {
          // any order: the better value, on ties the smaller position
          const bool better = (REDUCE == TS_MIN) ? (pv[v] < acc[v]) : (pv[v] > acc[v]);
          if (better || (pv[v] == acc[v] && pa[v] < arg[v])) { acc[v] = pv[v]; arg[v] = pa[v]; }
        } else {
          acc[v] = pv[v] + acc[v];
        }
      }
    }
    const int row = s_head_row[0];
    if (!all_ok) {
#pragma unroll
      for (int v = 0; v < VEC; ++v) acc[v] = acc_init<A, REDUCE>();  // the row is written as empty
    }
    finalize_row<T, VEC, REDUCE, ACCUM, PERM>(a, out_b, arg_b, count_b, i0 + row, col, lg, acc, arg,
                                              all_ok ? (int64_t)s_ptr[row + 1] - (int64_t)s_ptr[row] : 0, col_ok,
                                              arg_perm);
  }
}

// Second kernel: rows that cross workgroup tiles. One worker per tile that
// opened such a row walks the following tiles' head partials in order.
template <typename T, int VEC, int REDUCE>
__global__ __launch_bounds__(kBlock) void csr_reduce_fixup_kernel(CsrReduceArgs a) {
  typedef typename Acc<T>::type A;
  constexpr bool kArg = (REDUCE == TS_MIN || REDUCE == TS_MAX);
  const int G = a.G;
  const int W = kBlock / G;
  const int w = threadIdx.x / G;
  const int lg = threadIdx.x - w * G;
  const int64_t col = (int64_t)blockIdx.y * (G * VEC) + (int64_t)lg * VEC;
  const bool col_ok = col < a.K;
  const int64_t b = blockIdx.z;
  const int64_t t = (int64_t)blockIdx.x * W + w;
  if (t >= a.nblk) return;
  const int64_t *meta = a.ws_meta + (b * a.nblk) * 4;
  const A *vals = static_cast<const A *>(a.ws_vals) + (b * a.nblk) * 2 * a.K;
  const int32_t *args = kArg ? a.ws_args + (b * a.nblk) * 2 * a.K : nullptr;
  const int64_t c = col_ok ? col : 0;

  // Nearly every open row ends in the next tile: everything that case needs is loaded at
  // once (one memory latency instead of a chain of five), whether or not it turns out to be used.
  const int64_t tn = t + 1 < a.nblk ? t + 1 : t;
  const int64_t row = meta[t * 4 + 2];
  const int64_t count = meta[t * 4 + 3];  // length of that row, left by the tile that opened it
  int64_t next_row = meta[tn * 4 + 0];
  int64_t next_closes = meta[tn * 4 + 1];
  A acc[VEC], hv[VEC];
  int32_t arg[VEC], ha[VEC];
#pragma unroll
  for (int v = 0; v < VEC; ++v) {
    acc[v] = vals[(t * 2 + 1) * a.K + c + v];
    arg[v] = kArg ? args[(t * 2 + 1) * a.K + c + v] : 0;
    hv[v] = vals[(tn * 2) * a.K + c + v];
    ha[v] = kArg ? args[(tn * 2) * a.K + c + v] : 0;
  }
  if (row < 0) return;
  bool done = next_row != row;  // cannot happen for a well-formed indptr
  if (!done) {
#pragma unroll
    for (int v = 0; v < VEC; ++v) {
      if (kArg)
        reduce_step<A, REDUCE>(acc[v], arg[v], hv[v], ha[v]);
      else
        acc[v] = acc[v] + hv[v];
    }
    done = next_closes != 0;
  }
  // A hub row passes through many tiles. Their partials are fetched several tiles at a time (the
  // loads do not depend on each other) and combined in tile order, so the walk costs one memory
  // latency per batch instead of one per tile.
  constexpr int PF = VEC == 1 ? 16 : (VEC <= 4 ? 8 : (VEC <= 8 ? 4 : 2));
  for (int64_t t0 = t + 2; !done && t0 < a.nblk; t0 += PF) {
    int64_t nrow[PF], ncl[PF];
    A bv[PF][VEC];
    int32_t ba[PF][VEC];
#pragma unroll
    for (int q = 0; q < PF; ++q) {
      const int64_t tt = t0 + q < a.nblk ? t0 + q : a.nblk - 1;
      nrow[q] = meta[tt * 4 + 0];
      ncl[q] = meta[tt * 4 + 1];
#pragma unroll
      for (int v = 0; v < VEC; ++v) {
        bv[q][v] = vals[(tt * 2) * a.K + c + v];
        ba[q][v] = kArg ? args[(tt * 2) * a.K + c + v] : 0;
      }
    }
#pragma unroll
    for (int q = 0; q < PF; ++q) {
      if (!done) {
        if (t0 + q >= a.nblk || nrow[q] != row) {
          done = true;
        } else {
#pragma unroll
          for (int v = 0; v < VEC; ++v) {
            if (kArg)
              reduce_step<A, REDUCE>(acc[v], arg[v], bv[q][v], ba[q][v]);
            else
              acc[v] = acc[v] + bv[q][v];
          }
          done = ncl[q] != 0;
        }
      }
    }
  }
  T *out_b = static_cast<T *>(a.out) + b * a.N * a.K;
  int64_t *arg_b = kArg ? a.arg_out + b * a.N * a.K : nullptr;
  T *count_b = a.count_out ? static_cast<T *>(a.count_out) + b * a.N : nullptr;
  finalize_row<T, VEC, REDUCE>(a, out_b, arg_b, count_b, row, col, lg, acc, arg, count, col_ok);
}

// ---- host side -----------------------------------------------------------

// narrow rows (csr_small.h, csr_gather_small_kernel): at most 16 elements and 64 bytes per entry
constexpr int kSmallMaxK = 16;
constexpr int kSmallMaxRowBytes = 64;
constexpr int kSmallStageBytes = 16 * 1024;  // entries of one tile
inline bool csr_small_ok(int64_t K, int elem_bytes) {
  if (const char *env = getenv("TS_CSR_SMALL")) {  // tuning aid: 0 sends narrow rows to the wide kernel
    if (atoi(env) == 0) return false;
  }
  return K >= 1 && K <= kSmallMaxK && K * elem_bytes <= kSmallMaxRowBytes;
}
// items (rows + entries) per tile so that the entries fit the LDS stage
inline int csr_small_tile_items(int64_t K, int elem_bytes) {
  int bi = kSmallStageBytes / (int)(K * elem_bytes);
  if (bi > kMaxBlockItems) bi = kMaxBlockItems;
  return bi & ~63;
}

struct CsrPlan {
  int vec;       // elements per lane (16 bytes worth, or 1)
  int G;         // lanes per worker
  int BI;        // items per tile
  int ipw;       // items per worker
  int64_t nblk;  // tiles per batch
  int ychunks;   // column chunks
  bool small;    // narrow rows: the LDS-staged kernel
};

// with_arg: the reduction is min / max (positions carried along); for the expansion: the variant that divides
inline CsrPlan csr_plan(int64_t N, int64_t E, int64_t K, int elem_bytes, bool aligned16, bool expand = false,
                        bool with_arg = false, bool allow_small = true) {
  CsrPlan p;
  p.small = false;
  // narrow rows: always for the reduction; for the expansion when a row is at most 8 bytes or
  // consists of whole, aligned 16-byte granules (other widths do better with the wide kernel)
  const bool granules = aligned16 && (K * elem_bytes) % kVecBytes == 0;
  if (allow_small && csr_small_ok(K, elem_bytes) && (!expand || K * elem_bytes <= 8 || granules)) {
    p.small = true;
    p.vec = (expand && granules) ? kVecBytes / elem_bytes : 1;
    p.G = 1;
    while (p.G < K) p.G <<= 1;
    p.ychunks = 1;
    // the reduction stages the tile's entries in LDS; the expansion only its row pointers
    p.BI = expand ? kMaxBlockItems : csr_small_tile_items(K, elem_bytes);
    p.ipw = p.BI / (kBlock / p.G);
    p.nblk = (N + E + p.BI - 1) / p.BI;
    if (p.nblk < 1) p.nblk = 1;
    return p;
  }
  const int full = kVecBytes / elem_bytes;
  p.vec = (aligned16 && full > 1 && K % full == 0) ? full : 1;
  const int64_t lanes = (K + p.vec - 1) / p.vec;
  int G = 1;
  while (G < lanes && G < kWave) G <<= 1;
  p.G = G;
  p.ychunks = (int)((K + (int64_t)G * p.vec - 1) / ((int64_t)G * p.vec));
  const int64_t items = N + E;
  const int W = (expand ? kBlock : kCsrBlock) / G;
  const int cap = (expand ? kMaxBlockItems : kCsrMaxItems) / W;  // LDS holds the row pointers of one tile
  // Items per worker, from sweeps on 146 MB / 366 MB / 6 GB / 16 GB inputs (the curve is flat within 1-2 %
  // except for a few sharp optima): reductions 24 below 1 M items (more, shorter workgroups: the kernel is
  // latency bound there), 72 up to 32 M, 64 above; the write-bound expansion likes short ranges at every size
  // (a workgroup then writes ~100 KB and retires).
  int want = items >= ((int64_t)32 << 20) ? 64 : (items >= ((int64_t)1 << 20) ? 72 : 24);
  // min / max carry the positions too (101 VGPRs, four workgroups per CU): fewer, longer ranges
  if (with_arg && want < 40) want = 40;
  // expansion of very large inputs: 6 items per worker for the plain copy, 8 for the variant that divides
  // (with_arg doubles as that flag here); both then reach 70.5 % of peak on 62 M entries of 256 bytes, the
  // neighbouring values 63-67 %
  if (expand) want = items >= ((int64_t)32 << 20) ? (with_arg ? 8 : 6) : 24;
  if (const char *env = getenv("TS_CSR_IPW")) want = atoi(env);  // tuning aid
  if (want > cap) want = cap;
  int ipw = want;
  if (ipw > cap) ipw = cap;
  if (ipw < 1) ipw = 1;
  p.ipw = ipw;
  p.BI = W * ipw;
  p.nblk = (items + p.BI - 1) / p.BI;
  if (p.nblk < 1) p.nblk = 1;
  return p;
}

inline size_t csr_ws_bytes(const CsrPlan &p, int64_t B, int64_t K, int acc_bytes, bool with_arg,
                           size_t *off_args, size_t *off_meta) {
  auto up = [](size_t x) { return (x + 255) & ~(size_t)255; };
  size_t vals = up((size_t)B * p.nblk * 2 * K * acc_bytes);
  size_t args = with_arg ? up((size_t)B * p.nblk * 2 * K * 4) : 0;
  size_t meta = up((size_t)B * p.nblk * 4 * 8);
  if (off_args) *off_args = vals;
  if (off_meta) *off_meta = vals + args;
  return vals + args + meta;
}

template <typename T, int VEC, int REDUCE>
int launch_csr_reduce_t(const CsrReduceArgs &a, const CsrPlan &p, int64_t B, hipStream_t stream) {
  dim3 grid((unsigned)p.nblk, (unsigned)p.ychunks, (unsigned)B);
  if (a.perm != nullptr) {
    if (a.accumulate) return TS_ERR_UNSUPPORTED;
    hipLaunchKernelGGL((csr_reduce_kernel<T, VEC, REDUCE, 0, 1>), grid, dim3(kCsrBlock), 0, stream, a);
  } else if (a.gate != nullptr || a.scatter_rule) {
    if (a.accumulate || !(a.lookback || p.nblk <= 1)) return TS_ERR_UNSUPPORTED;
    hipLaunchKernelGGL((csr_reduce_kernel<T, VEC, REDUCE, 0, 2>), grid, dim3(kCsrBlock), 0, stream, a);
  } else if (a.accumulate)
    hipLaunchKernelGGL((csr_reduce_kernel<T, VEC, REDUCE, -1>), grid, dim3(kCsrBlock), 0, stream, a);
  else
    hipLaunchKernelGGL((csr_reduce_kernel<T, VEC, REDUCE, 0>), grid, dim3(kCsrBlock), 0, stream, a);
  if (p.nblk > 1 && !a.lookback) {  // a single tile has no rows that cross tiles
    const int W = kBlock / p.G;
    dim3 grid2((unsigned)((p.nblk + W - 1) / W), (unsigned)p.ychunks, (unsigned)B);
    hipLaunchKernelGGL((csr_reduce_fixup_kernel<T, VEC, REDUCE>), grid2, dim3(kBlock), 0, stream, a);
  }
  return hipGetLastError() == hipSuccess ? TS_OK : TS_ERR_LAUNCH;
}

template <typename T, int VEC>
int launch_csr_reduce_v(const CsrReduceArgs &a, const CsrPlan &p, int64_t B, int reduce,
                        hipStream_t stream) {
  switch (reduce) {
  case TS_SUM: return launch_csr_reduce_t<T, VEC, TS_SUM>(a, p, B, stream);
  case TS_MEAN: return launch_csr_reduce_t<T, VEC, TS_MEAN>(a, p, B, stream);
  case TS_MIN: return launch_csr_reduce_t<T, VEC, TS_MIN>(a, p, B, stream);
  case TS_MAX: return launch_csr_reduce_t<T, VEC, TS_MAX>(a, p, B, stream);
  default: return TS_ERR_UNSUPPORTED;
  }
}

// One entry per element type, each defined in its own translation unit.
template <typename T> int launch_csr_reduce(const CsrReduceArgs &a, const CsrPlan &p, int64_t B,
                                            int reduce, hipStream_t stream);

template <typename T>
int launch_csr_reduce_small(const CsrReduceArgs &a, const CsrPlan &p, int64_t B, int reduce, hipStream_t stream);

#define TS_INSTANTIATE_CSR_REDUCE(T, FULLVEC)                                               \
  template <> int launch_csr_reduce<T>(const CsrReduceArgs &a, const CsrPlan &p, int64_t B, \
                                       int reduce, hipStream_t stream) {                    \
    if (p.small) return launch_csr_reduce_small<T>(a, p, B, reduce, stream);                \
    if (p.vec == FULLVEC) return launch_csr_reduce_v<T, FULLVEC>(a, p, B, reduce, stream);  \
    return launch_csr_reduce_v<T, 1>(a, p, B, reduce, stream);                              \
  }

}  // namespace ts
