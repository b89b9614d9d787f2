// Group statistics with one result per group -- scatter_std (composite/std.py:8-41) and scatter_logsumexp
// (composite/logsumexp.py:8-57) -- through buckets of groups, for an index in any order (included by
// group_softmax.h).
//
// The three passes of group_softmax.h read src two or three times and meet in memory through atomics. Here
// the entries are first binned by bucket of R neighbouring groups with the passes of scatter_binned.h (count, scan,
// place: 8-byte words (group inside its bucket, entry number)); then one workgroup per chunk of a bucket gathers
// the rows of its entries ONCE, sorts them by group in LDS (an integer atomic per entry gives its rank inside its
// group) and makes both sweeps of the statistic over each group's rows there, in registers:
//   std        sweep 1: sum per group (the count is known)   sweep 2: squared deviations from the group mean
//   logsumexp  sweep 1: maximum per group                    sweep 2: sum of exp(src - maximum)
// A bucket that fits one chunk (the usual case: R is chosen so that an average bucket fills about half a chunk)
// writes its groups' results directly, with the roundings of the reference's sequence. The chunks of a larger
// bucket (the groups of hub nodes) leave their partials as slabs -- deviations relative to the chunk's own mean,
// sums relative to the chunk's own maximum -- and group_bin_combine_kernel merges the slabs of a bucket
// (pairwise update of (n, sum, M2); sums rescaled by exp(m_chunk - m)) and writes the results; it also writes the
// groups of buckets that received no entry. No float atomics anywhere: a result depends on the order of the index
// only through the order in which a group's entries are added.
#pragma once

namespace ts {

constexpr int kGroupBinU = 8;         // units (one entry's VEC columns) per lane: a chunk is held in registers
constexpr int kGroupBinRows = 2048;   // groups per bucket at most
constexpr int kGroupBinSlots = 8192;  // groups x columns of a bucket at most (the slab of a chunk: 16 bytes per slot)
constexpr int kGroupBinLong = 64;     // entries of a group inside a chunk from which on a wavefront takes the group
constexpr int kGroupBinCoop = 2;      // up to this many long groups in a chunk, the whole workgroup takes them one by one
constexpr int kGroupBinCoopLanes = 8;  // and held by at least this many lanes (few entries per step of one wavefront),
constexpr int kGroupBinCoopEntries = 2048;  // or a group of at least this many entries
constexpr int kGroupBinCoopCols = 64;  // ... for rows of up to this many columns
constexpr int kGroupBinMaxLong = 128;  // such groups per chunk at most (a chunk holds at most 8192 entries)
constexpr int kGroupBinMaxLanes = 32;  // lanes per entry at most (a chunk then holds 256 entries)

// 8-byte words of a chunk's slab: two tables and the counts
__host__ __device__ inline size_t group_bin_slab_words(int table, int rows) { return 2 * (size_t)table + ((size_t)rows + 1) / 2; }

struct GroupBinPlan {
  bool ok;
  BinArgs p;
  size_t bytes;
};

// vec: columns per lane (the caller's choice: 16 bytes when K allows it, else 1)
inline GroupBinPlan group_bin_plan(int64_t B, int64_t E, int64_t K, int64_t N, int elem_bytes, int vec, void *ws,
                                   size_t ws_bytes, bool any_size) {
  GroupBinPlan r;
  r.ok = false;
  r.bytes = 0;
  const int64_t n_edges = B * E, rows = B * N;
  if (n_edges < 1 || rows < 1 || K < 1 || n_edges >= 0xFFFFFFFEll || rows >= 0x7FFFFFFFll) return r;
  if (vec < 1 || K % vec != 0) return r;
  const int64_t lanes = K / vec;
  if (lanes > kGroupBinMaxLanes || K > kGroupBinSlots) return r;
  // six launches: below a few MB the three passes are ahead; so they are with single values in few, large groups
  // (their LDS tables hold every group: 4 M values in 4 k groups, random order: logsumexp 70 against 125 us)
  if (!any_size && n_edges * K * elem_bytes < ((int64_t)4 << 20)) return r;
  if (!any_size && K == 1 && n_edges > 256 * rows) return r;
  const int64_t epw = kWave / lanes;  // entries per row of a wavefront
  const int64_t chunk = (int64_t)(kBinBlock / kWave) * kGroupBinU * epw;
  // groups per bucket: a power of two whose table fits, and so that an average bucket fills at most 0.6 chunks
  int rshift = 0;
  auto fits = [&](int rs) { return ((int64_t)1 << rs) * K <= kGroupBinSlots && ((int64_t)1 << rs) <= kGroupBinRows; };
  while (fits(rshift + 1) && ((int64_t)2 << rshift) * n_edges * 5 <= chunk * 3 * rows) ++rshift;
  while (((rows + ((int64_t)1 << rshift) - 1) >> rshift) > kBinMaxBuckets && fits(rshift + 1)) ++rshift;
  const int64_t nb = (rows + ((int64_t)1 << rshift) - 1) >> rshift;
  if (nb > kBinMaxBuckets) return r;
  BinArgs &p = r.p;
  p = BinArgs();
  p.rshift = rshift;
  p.kc = (int)K;
  p.slices = 1;
  p.nb = (int)nb;
  {
    const int64_t rounds = (n_edges + (int64_t)512 * kBinPlaceChunk - 1) / ((int64_t)512 * kBinPlaceChunk);
    int64_t tile = (((n_edges + 512 * rounds - 1) / (512 * rounds)) + kBinPlaceBlock - 1) & ~(int64_t)(kBinPlaceBlock - 1);
    if (tile < kBinPlaceBlock) tile = kBinPlaceBlock;
    if (tile > kBinPlaceChunk) tile = kBinPlaceChunk;
    p.place_tile = (int)tile;
    p.n_place = (n_edges + tile - 1) / tile;
  }
  p.chunk = (int)chunk;
  p.max_wgs = n_edges / chunk + nb + 1;
  const int table = (int)(K << rshift);
  const int64_t n_slabs = 2 * (n_edges / chunk) + 2;  // a bucket of m >= 2 chunks holds more than (m - 1) chunks of entries
  const size_t slab_bytes = group_bin_slab_words(table, 1 << rshift) * 8;
  if ((size_t)n_slabs * slab_bytes > ((size_t)1 << 30)) return r;  // (an upper bound: every chunk of every bucket among several)
  auto up = [](size_t x) { return (x + 255) & ~(size_t)255; };
  size_t off = 0;
  auto take = [&](size_t bytes) { const size_t o = off; off += up(bytes); return o; };
  const size_t o_tot = take((size_t)nb * 8), o_cur = take((size_t)nb * 8), o_st = take((size_t)(nb + 1) * 8);
  const size_t o_cs = take((size_t)(nb + 1) * 4), o_wb = take((size_t)p.max_wgs * 4);
  const size_t o_bin = take((size_t)n_edges * 8);
  const size_t o_ss = take((size_t)(nb + 1) * 4), o_cl = take((size_t)(nb + 2) * 4);
  const size_t o_sl = take((size_t)n_slabs * slab_bytes);
  r.bytes = off;
  if (ws == nullptr || ws_bytes < off || (reinterpret_cast<uintptr_t>(ws) & 15) != 0) return r;
  char *base = static_cast<char *>(ws);
  p.totals = reinterpret_cast<unsigned long long *>(base + o_tot);
  p.cursor = reinterpret_cast<unsigned long long *>(base + o_cur);
  p.starts = reinterpret_cast<int64_t *>(base + o_st);
  p.chunk_start = reinterpret_cast<int32_t *>(base + o_cs);
  p.wg_bucket = reinterpret_cast<int32_t *>(base + o_wb);
  p.binned = reinterpret_cast<uint64_t *>(base + o_bin);
  p.unsorted = nullptr;  // an index in any order takes these passes
  p.slab_start = reinterpret_cast<int32_t *>(base + o_ss);
  p.comb_list = reinterpret_cast<int32_t *>(base + o_cl);
  p.comb_count = p.comb_list + nb;
  p.slabs = reinterpret_cast<uint64_t *>(base + o_sl);
  r.ok = true;
  return r;
}

// ---- the partial of one (group, column): std (n, sum, M2), logsumexp (key of the maximum, sum relative to it)
template <typename T, int MODE> struct GroupBinPart {
  typedef typename Acc<T>::type F;
  typedef typename OrdKey<F>::bits KB;
  uint64_t a;  // std: bits of the sum (double); logsumexp: the key
  double b;    // std: M2; logsumexp: the sum
  int32_t n;   // std: entries
  __device__ static GroupBinPart identity() {
    GroupBinPart s;
    s.a = MODE == GS_STD ? 0ull : MODE == GS_LSE ? (uint64_t)OrdKey<F>::enc(-INFINITY) : (uint64_t)group_empty_key<T>();
    s.b = 0.0;
    s.n = 0;
    return s;
  }
  // the partial of a later chunk joins this one
  __device__ void absorb(const GroupBinPart &o) {
    if constexpr (MODE == GS_STD) {
      if (o.n == 0) return;
      if (n == 0) {
        *this = o;
        return;
      }
      const double sa = __longlong_as_double((long long)a), sb = __longlong_as_double((long long)o.a);
      const double na = (double)n, nb = (double)o.n;
      const double d = sa / na - sb / nb;
      b = b + o.b + d * d * (na * nb / (na + nb));
      a = (uint64_t)__double_as_longlong(sa + sb);
      n += o.n;
    } else {
      const KB ka = (KB)a, kb = (KB)o.a;
      // no maximum yet: logsumexp starts from -inf; softmax from lowest(), and a partial in which nothing beat it
      // was summed relative to 0 and holds 0 or NaN, taken as is
      const KB none = MODE == GS_LSE ? OrdKey<F>::enc(-INFINITY) : group_empty_key<T>();
      if (MODE != GS_LSE && (ka == none || kb == none)) {
        if (kb > ka) a = o.a;
        b = b + o.b;
        return;
      }
      if (kb > ka) {
        const double fac = ka == none ? 0.0 : (double)exp_acc(OrdKey<F>::dec(ka) - OrdKey<F>::dec(kb));
        b = b * fac + o.b;
        a = o.a;
      } else {
        const double fac = kb == ka ? 1.0 : (kb <= none ? 0.0 : (double)exp_acc(OrdKey<F>::dec(kb) - OrdKey<F>::dec(ka)));
        b = b + o.b * fac;
      }
    }
  }
};

// One finished (group, column) -> the outputs, with the roundings of the reference's sequence: element i of [B * N, K].
// std: a = sum, b = sum of squared deviations, n = entries (composite/std.py:27-39); also the group sum in the
// element type and the count, which the backward pass reads. logsumexp: log(sum + eps) + max with the clean-up
// of composite/logsumexp.py:51-54.
template <typename T, int MODE>
__device__ __forceinline__ void group_bin_emit(const GroupArgs &g, int64_t i, int64_t row, int k,
                                               const GroupBinPart<T, MODE> &s) {
  typedef typename Acc<T>::type F;
  typedef typename OrdKey<F>::bits KB;
  T *out = static_cast<T *>(g.out);
  if constexpr (MODE == GS_STD) {
    const F div = group_divisor<T>(s.n, g.unbiased);
    out[i] = from_acc<T>(sqrt_acc(round_elem<T>(round_elem<T>((F)s.b) / div)));
    static_cast<T *>(g.total_w)[i] = from_acc<T>((F)__longlong_as_double((long long)s.a));
    if (k == 0) g.count_w[row] = s.n;
  } else if constexpr (MODE == GS_SOFTMAX) {
    // the group's key and sum, side by side, for the elementwise finish of group_softmax.h
    const int64_t slot = row * g.gs + k;
    static_cast<KB *>(g.gmax)[slot] = (KB)s.a;
    static_cast<F *>(g.gsum)[slot] = (F)s.b;
  } else {
    const F m = OrdKey<F>::dec((KB)s.a);
    const F l = round_elem<T>(log_acc(round_elem<T>(round_elem<T>((F)s.b) + (F)g.eps)));
    F o = round_elem<T>(l + m);
    if (o != o || o == -INFINITY) o = (F)0;
    if (o == INFINITY) o = to_acc<T>(ElemLim<T>::max());
    out[i] = from_acc<T>(o);
  }
}

// One workgroup per chunk of a bucket. lanes: lanes per entry (K / VEC), epw: entries per row of a wavefront (64 / lanes).
// LDS float atomics are slow on this part (ds_add_f64 about 2 lanes per clock, ds_add_f32 fewer: 150 us per sweep over
// 9 M entries of 8 floats), so the chunk is sorted by group instead, with one integer atomic per ENTRY: its rank
// inside its group. The rows of src then lie group by group in LDS and the statistic is a loop per (group, columns)
// in registers: one lane for a group of up to kGroupBinLong entries, a wavefront for a longer one.
template <typename T, int VEC, int MODE>
__global__ __launch_bounds__(kBinBlock) void group_bin_kernel(GroupArgs g, BinArgs p, int lanes, int epw) {
  typedef typename Acc<T>::type F;
  typedef typename OrdKey<F>::bits KB;
  typedef GroupBinPart<T, MODE> Part;
  typedef uint32_t u4 __attribute__((ext_vector_type(4)));
  constexpr int U = kGroupBinU, W = kBinBlock / kWave;
  extern __shared__ u4 s_dyn[];               // the chunk's rows of src, group by group: [entries][K] of T
  __shared__ int32_t s_n[kGroupBinRows];      // entries per group
  __shared__ int32_t s_off[kGroupBinRows + 1];  // first staged entry of a group
  __shared__ int32_t s_wsum[W];
  __shared__ int32_t s_long[kGroupBinMaxLong];  // groups for a wavefront
  __shared__ int s_nlong;
  __shared__ double s_part[W][kGroupBinCoopCols];  // where the wavefronts that share a long group meet
  if (p.unsorted != nullptr && *p.unsorted != 1) return;  // the caller's one-pass kernels took the call
  const int wg = (int)blockIdx.x;
  const int bucket = p.wg_bucket[wg];
  if (bucket < 0) return;
  const int K = (int)g.K, R = 1 << p.rshift, table = K << p.rshift;
  const int tid = threadIdx.x, lane = tid & (kWave - 1), wave = tid / kWave;
  for (int i = tid; i < R; i += kBinBlock) s_n[i] = 0;
  if (tid == 0) s_nlong = 0;
  const int chunks = p.chunk_start[bucket + 1] - p.chunk_start[bucket];
  const int64_t lo = p.starts[bucket] + ((int64_t)wg - p.chunk_start[bucket]) * p.chunk;
  int64_t hi = lo + p.chunk;
  if (hi > p.starts[bucket + 1]) hi = p.starts[bucket + 1];
  const int n = (int)(hi - lo);

  // ---- the chunk: every unit's entry word, then its VEC columns of src, all in flight. A wavefront takes epw
  // neighbouring entries at a time, `lanes` lanes each.
  const T *src = static_cast<const T *>(g.src);
  const int sub = lane / lanes;
  const int col = (lane - sub * lanes) * VEC;
  uint64_t word[U];
#pragma unroll
  for (int u = 0; u < U; ++u) {
    const int j = (wave + u * W) * epw + sub;
    word[u] = (sub < epw && j < n) ? p.binned[lo + j] : ~0ull;
  }
  Vec<T, VEC> x[U];
#pragma unroll
  for (int u = 0; u < U; ++u) {
    const int64_t e = word[u] == ~0ull ? 0 : (int64_t)(uint32_t)word[u];
    x[u] = load_vec_stream<T, VEC>(src + e * K + col);
  }
  __syncthreads();

  // ---- rank of every entry inside its group (the entry's first lane asks, the others copy)
  int32_t rank[U];
#pragma unroll
  for (int u = 0; u < U; ++u) {
    int32_t r = 0;
    if (word[u] != ~0ull && col == 0) r = atomicAdd(&s_n[(int)(word[u] >> 32)], 1);
    rank[u] = lanes > 1 ? __shfl(r, sub * lanes) : r;
  }
  __syncthreads();
  // ---- first staged entry of every group: exclusive scan of the counts, one or two groups per lane
  {
    const int per = (R + kBinBlock - 1) / kBinBlock;
    const int r0 = tid * per;
    const int32_t c0 = r0 < R ? s_n[r0] : 0, c1 = (per == 2 && r0 + 1 < R) ? s_n[r0 + 1] : 0;
    const int32_t mine = c0 + c1;
    const int32_t incl = wave_inclusive_sum(mine);
    if (lane == kWave - 1) s_wsum[wave] = incl;
    __syncthreads();
    int32_t base = incl - mine;
    for (int w2 = 0; w2 < wave; ++w2) base += s_wsum[w2];
    const bool wide_ok = (lanes & (lanes - 1)) == 0;  // a wavefront shares a group through butterflies
    if (r0 < R) {
      s_off[r0] = base;
      if (wide_ok && c0 > kGroupBinLong) s_long[atomicAdd(&s_nlong, 1)] = r0;
    }
    if (per == 2 && r0 + 1 < R) {
      s_off[r0 + 1] = base + c0;
      if (wide_ok && c1 > kGroupBinLong) s_long[atomicAdd(&s_nlong, 1)] = r0 + 1;
    }
    if (tid == 0) s_off[R] = n;
  }
  __syncthreads();
  T *s_val = reinterpret_cast<T *>(s_dyn);
#pragma unroll
  for (int u = 0; u < U; ++u) {
    if (word[u] == ~0ull) continue;
    store_vec<T, VEC>(s_val + (int64_t)(s_off[(int)(word[u] >> 32)] + rank[u]) * K + col, x[u]);
  }
  __syncthreads();

  // ---- the statistic of group r, columns c .. c + VEC - 1, by the lanes (first, first + step, ...) of its entries;
  // wide: those lanes are the lanes of one wavefront that hold the same columns, and meet in a butterfly.
  // A bucket in one chunk: the reference's roundings. A chunk among several: relative to the chunk's own mean / maximum.
  const bool single = chunks == 1;
  const int64_t first_elem = ((int64_t)bucket << p.rshift) * K;  // first element of the bucket in [B * N, K]
  const int64_t total = g.B * g.N * g.K;
  uint64_t *slab = single ? nullptr
                          : p.slabs + ((int64_t)p.slab_start[bucket] + (wg - p.chunk_start[bucket])) *
                                          (int64_t)group_bin_slab_words(table, R);
  // the lanes that share a group meet in a butterfly: a wavefront's lanes with the same columns (offsets 32 ... lanes),
  // or `share` neighbouring lanes (offsets share / 2 ... 1)
  // coop: all wavefronts of the workgroup share the group (a chunk with one or two long groups: the groups of hub nodes, or
  // few groups of many entries each); their totals meet in LDS, added in wavefront order.
  auto stat = [&](int r, int c, int first, int step, int off_hi, int off_lo, bool coop) {
    auto meet = [&](auto (&v)[VEC], auto op) {  // the VEC columns of this lane at once: two barriers per meeting
#pragma unroll
      for (int j = 0; j < VEC; ++j)
        for (int off = off_hi; off >= off_lo; off >>= 1) v[j] = op(v[j], __shfl_xor(v[j], off));
      if (coop) {
        if (sub == 0) {
#pragma unroll
          for (int j = 0; j < VEC; ++j) s_part[wave][c + j] = (double)v[j];
        }
        __syncthreads();
#pragma unroll
        for (int j = 0; j < VEC; ++j) {
          auto t = (decltype(v[j] + v[j]))s_part[0][c + j];
          for (int w2 = 1; w2 < W; ++w2) t = op(t, (decltype(v[j] + v[j]))s_part[w2][c + j]);
          v[j] = t;
        }
        __syncthreads();
      }
    };
    const bool wide = off_hi >= off_lo;
    const int e0 = s_off[r], cnt = s_n[r];
    Part part[VEC];
    // the lane's entries first, first + step, ..., four LDS reads in flight
    auto for_entries = [&](auto &&fn) {
      for (int e = first; e < cnt; e += 4 * step) {
        Vec<T, VEC> y[4];
#pragma unroll
        for (int q = 0; q < 4; ++q) {
          const int eq = e + q * step;
          y[q] = load_vec<T, VEC>(s_val + (e0 + (eq < cnt ? eq : e)) * K + c);
        }
#pragma unroll
        for (int q = 0; q < 4; ++q)
          if (e + q * step < cnt) fn(y[q]);
      }
    };
    if constexpr (MODE == GS_STD) {
      // a lane adds its few entries in the accumulate type; the lanes of a group meet in double precision
      F acc[VEC];
      double sum[VEC], m2[VEC];
#pragma unroll
      for (int v = 0; v < VEC; ++v) acc[v] = (F)0;
      for_entries([&](const Vec<T, VEC> &y) {
#pragma unroll
        for (int v = 0; v < VEC; ++v) acc[v] += to_acc<T>(y.v[v]);
      });
#pragma unroll
      for (int v = 0; v < VEC; ++v) sum[v] = (double)acc[v], acc[v] = (F)0;
      if (wide) meet(sum, [](double a, double b) { return a + b; });
      if (single) {
        F mean[VEC];
#pragma unroll
        for (int v = 0; v < VEC; ++v) mean[v] = group_mean<T>(from_acc<T>((F)sum[v]), cnt);
        for_entries([&](const Vec<T, VEC> &y) {
#pragma unroll
          for (int v = 0; v < VEC; ++v) {
            const F d = round_elem<T>(to_acc<T>(y.v[v]) - mean[v]);
            acc[v] += round_elem<T>(d * d);
          }
        });
      } else {
        F mean[VEC];  // the chunk's own mean (its rounding changes the squared deviations in second order only)
#pragma unroll
        for (int v = 0; v < VEC; ++v) mean[v] = (F)(sum[v] / (double)(cnt < 1 ? 1 : cnt));
        for_entries([&](const Vec<T, VEC> &y) {
#pragma unroll
          for (int v = 0; v < VEC; ++v) {
            const F d = to_acc<T>(y.v[v]) - mean[v];
            acc[v] += d * d;
          }
        });
      }
#pragma unroll
      for (int v = 0; v < VEC; ++v) m2[v] = (double)acc[v];
      if (wide) meet(m2, [](double a, double b) { return a + b; });
#pragma unroll
      for (int v = 0; v < VEC; ++v) {
        part[v].a = (uint64_t)__double_as_longlong(sum[v]);
        part[v].b = m2[v];
        part[v].n = cnt;
      }
    } else {
      F top[VEC], acc[VEC];
      double sum[VEC];
#pragma unroll
      for (int v = 0; v < VEC; ++v) top[v] = -INFINITY, acc[v] = (F)0;
      for_entries([&](const Vec<T, VEC> &y) {
#pragma unroll
        for (int v = 0; v < VEC; ++v) top[v] = max_acc(top[v], to_acc<T>(y.v[v]));  // a NaN never wins
      });
      bool won[VEC];
      if (wide) meet(top, [](F a, F b) { return max_acc(a, b); });
#pragma unroll
      for (int v = 0; v < VEC; ++v) {
        top[v] = OrdKey<F>::dec(OrdKey<F>::enc(top[v]));  // -0.0 folds onto +0.0
        // softmax: an entry has to beat lowest(); a group without a winner is shifted by 0 (composite/softmax.py:16-18)
        won[v] = MODE == GS_LSE || top[v] > to_acc<T>(ElemLim<T>::lowest());
        if (!won[v]) top[v] = (F)0;
      }
      for_entries([&](const Vec<T, VEC> &y) {
#pragma unroll
        for (int v = 0; v < VEC; ++v) {
          F z = round_elem<T>(to_acc<T>(y.v[v]) - top[v]);
          if (MODE == GS_LSE && z != z) z = -INFINITY;  // NaN entries and -inf - -inf drop out (logsumexp.py:41)
          acc[v] += round_elem<T>(exp_acc(z));
        }
      });
#pragma unroll
      for (int v = 0; v < VEC; ++v) sum[v] = (double)acc[v];
      if (wide) meet(sum, [](double a, double b) { return a + b; });
#pragma unroll
      for (int v = 0; v < VEC; ++v) {
        part[v].a = won[v] ? (uint64_t)OrdKey<F>::enc(top[v]) : (uint64_t)group_empty_key<T>();
        part[v].b = sum[v];
        part[v].n = 0;
      }
    }
    if (first != 0) return;
#pragma unroll
    for (int v = 0; v < VEC; ++v) {
      const int i = r * K + c + v;
      if (single) {
        if (first_elem + i < total) group_bin_emit<T, MODE>(g, first_elem + i, ((int64_t)bucket << p.rshift) + r, c + v, part[v]);
      } else {
        slab[i] = part[v].a;
        reinterpret_cast<double *>(slab)[table + i] = part[v].b;
        if (MODE == GS_STD && c + v == 0) reinterpret_cast<int32_t *>(slab + 2 * (size_t)table)[r] = part[v].n;
      }
    }
  };
  const int nlong = s_nlong;
  // `share` neighbouring lanes per (group, columns): as many as keep all lanes busy, eight at most
  int share = 1;
  while (share < 8 && R * lanes * share * 2 <= kBinBlock) share *= 2;
  const int slane = tid & (share - 1);
  for (int i0 = 0; i0 < R * lanes * share; i0 += kBinBlock) {  // whole lane groups stay together (butterflies)
    const int i = (i0 + tid) / share;
    const bool live = i0 + tid < R * lanes * share;
    const int r = live ? i / lanes : 0;
    const bool mine = live && !(nlong > 0 && s_n[r] > kGroupBinLong);
    // (a lane group that has no item still takes part in the butterflies of its wavefront)
    stat(r, (i - r * lanes) * VEC, mine ? slane : 0x7FFFFFF0, share, share / 2, 1, false);
  }
  // (rows held by few lanes: only for a group of kGroupBinCoopEntries entries and more, where one wavefront would need
  // tens of rounds; below that the barriers of the meeting cost more)
  bool coop = nlong > 0 && nlong <= kGroupBinCoop && K <= kGroupBinCoopCols;
  if (coop && lanes < kGroupBinCoopLanes) {
    int most = 0;
    for (int q = 0; q < nlong; ++q) most = s_n[s_long[q]] > most ? s_n[s_long[q]] : most;
    coop = most >= kGroupBinCoopEntries;
  }
  if (coop) {
    for (int q = 0; q < nlong; ++q) stat(s_long[q], col, wave * epw + sub, W * epw, kWave / 2, lanes, true);
  } else {
    for (int q = wave; q < nlong; q += W) stat(s_long[q], col, sub, epw, kWave / 2, lanes, false);
  }
}

// Buckets that were not reduced in exactly one chunk: their slabs merged, slab by slab in chunk order, element by
// element (none: a bucket without entries, whose groups get the result of an empty group). A bucket of few chunks:
// 1024 neighbouring elements per workgroup and step, every lane walks the slabs. A bucket of many chunks (the hubs of
// a skewed index): 64 elements at a time, the wavefronts share the slabs and meet in LDS in wavefront order.
template <typename T, int MODE>
__global__ __launch_bounds__(kBinBlock) void group_bin_combine_kernel(GroupArgs g, BinArgs p) {
  typedef GroupBinPart<T, MODE> Part;
  constexpr int W = kBinBlock / kWave;
  __shared__ uint64_t s_pa[W][kCombPos];
  __shared__ double s_pb[W][kCombPos];
  __shared__ int32_t s_pn[W][kCombPos];
  if (p.unsorted != nullptr && *p.unsorted != 1) return;
  const int lane = threadIdx.x & (kWave - 1), wave = threadIdx.x / kWave;
  const int K = (int)g.K, R = 1 << p.rshift, table = K << p.rshift;
  const int64_t words = (int64_t)group_bin_slab_words(table, R);
  const int n_few = p.comb_count[0], n_many = p.comb_count[1];
  const int64_t total = g.B * g.N * g.K;
  auto load = [&](const uint64_t *slab, int pos) {
    Part s;
    s.a = slab[pos];
    s.b = reinterpret_cast<const double *>(slab)[table + pos];
    s.n = MODE == GS_STD ? reinterpret_cast<const int32_t *>(slab + 2 * (size_t)table)[pos / K] : 0;
    return s;
  };
  const int parts = (table + kCombPos - 1) / kCombPos;
  for (int64_t item = blockIdx.x; item < (int64_t)n_many * parts; item += gridDim.x) {
    const int bucket = p.comb_list[p.nb - 1 - (int)(item / parts)];
    const int m = p.chunk_start[bucket + 1] - p.chunk_start[bucket];
    const int pos = (int)(item % parts) * kCombPos + lane;
    const int64_t first = ((int64_t)bucket << p.rshift) * K;
    const uint64_t *slab0 = p.slabs + (int64_t)p.slab_start[bucket] * words;
    const int pp = pos < table ? pos : 0;
    // wavefront w takes the slabs [w * per, (w + 1) * per): chunk order is kept
    const int per = (m + W - 1) / W;
    const int s_lo = wave * per, s_hi = s_lo + per < m ? s_lo + per : m;
    Part acc = Part::identity();
    constexpr int U = 4;
    for (int s0 = s_lo; s0 < s_hi; s0 += U) {
      Part t[U];
#pragma unroll
      for (int u = 0; u < U; ++u) t[u] = load(slab0 + (int64_t)(s0 + u < s_hi ? s0 + u : s0) * words, pp);
#pragma unroll
      for (int u = 0; u < U; ++u)
        if (s0 + u < s_hi) acc.absorb(t[u]);
    }
    s_pa[wave][lane] = acc.a;
    s_pb[wave][lane] = acc.b;
    s_pn[wave][lane] = acc.n;
    __syncthreads();
    if (wave == 0) {
      for (int w2 = 1; w2 < W; ++w2) {
        Part t;
        t.a = s_pa[w2][lane];
        t.b = s_pb[w2][lane];
        t.n = s_pn[w2][lane];
        acc.absorb(t);
      }
      if (pos < table && first + pos < total)
        group_bin_emit<T, MODE>(g, first + pos, ((int64_t)bucket << p.rshift) + pos / K, pos % K, acc);
    }
    __syncthreads();
  }
  const int blocks = (table + kBinBlock - 1) / kBinBlock;
  for (int64_t item = blockIdx.x; item < (int64_t)n_few * blocks; item += gridDim.x) {
    const int bucket = p.comb_list[item / blocks];
    const int m = p.chunk_start[bucket + 1] - p.chunk_start[bucket];
    const int pos = (int)(item % blocks) * kBinBlock + (int)threadIdx.x;
    const int64_t first = ((int64_t)bucket << p.rshift) * K;
    if (pos >= table || first + pos >= total) continue;
    const uint64_t *slab0 = p.slabs + (int64_t)p.slab_start[bucket] * words;
    Part acc = Part::identity();
    constexpr int U = 4;
    for (int s0 = 0; s0 < m; s0 += U) {
      Part t[U];
#pragma unroll
      for (int u = 0; u < U; ++u) t[u] = load(slab0 + (int64_t)(s0 + u < m ? s0 + u : s0) * words, pos);
#pragma unroll
      for (int u = 0; u < U; ++u)
        if (s0 + u < m) acc.absorb(t[u]);
    }
    group_bin_emit<T, MODE>(g, first + pos, ((int64_t)bucket << p.rshift) + pos / K, pos % K, acc);
  }
}

// count, scan, place (scatter_binned.h), then the chunks and the buckets of several chunks
// gate (softmax): a word that the caller's one-pass kernels leave at 1 when the index was not in order; every pass
// here then runs only if it reads 1
template <typename T, int VEC, int MODE>
int launch_group_bins(const GroupArgs &g, hipStream_t stream, int *gate = nullptr) {
  if (g.bins == nullptr) return TS_ERR_BAD_ARG;
  BinArgs p = *g.bins;
  if (gate != nullptr) {
    p.unsorted = gate;
    p.sampled = 1;  // the count pass does not judge the index, it reads the verdict
  }
  const ScatterArgs a = group_index_args(g);
  if (gate == nullptr)  // (with a gate: its owner's sample kernel has cleared the totals)
    hipLaunchKernelGGL(bin_clear_kernel, dim3((p.nb + kBlock - 1) / kBlock), dim3(kBlock), 0, stream, p.totals, p.nb,
                       (int *)nullptr);
  launch_bin_count(a, p, stream);
  hipLaunchKernelGGL(bin_scan_kernel, dim3(1), dim3(kBinBlock), 0, stream, p);
  if (bin_place_sorted_ok(p))
    hipLaunchKernelGGL(bin_place_sorted_kernel, dim3((unsigned)((a.B * a.E + kBinSortTile - 1) / kBinSortTile)),
                       dim3(kBinPlaceBlock), 0, stream, a, p);
  else if (p.nb <= kBinSmallCap)
    hipLaunchKernelGGL(bin_place_kernel<kBinSmallCap>, dim3((unsigned)p.n_place), dim3(kBinPlaceBlock), 0, stream, a, p);
  else
    hipLaunchKernelGGL(bin_place_kernel<kBinMaxBuckets>, dim3((unsigned)p.n_place), dim3(kBinPlaceBlock), 0, stream, a, p);
  const int lanes = (int)(g.K / VEC), epw = kWave / lanes;
  // the chunk's rows of src in LDS: up to 128 KB, one workgroup per CU
  const size_t lds = ((size_t)p.chunk * g.K * sizeof(T) + 15) & ~(size_t)15;
  if (hipFuncSetAttribute(reinterpret_cast<const void *>(&group_bin_kernel<T, VEC, MODE>),
                          hipFuncAttributeMaxDynamicSharedMemorySize, (int)lds) != hipSuccess)
    return TS_ERR_LAUNCH;
  hipLaunchKernelGGL((group_bin_kernel<T, VEC, MODE>), dim3((unsigned)p.max_wgs), dim3(kBinBlock), lds, stream, g, p, lanes,
                     epw);
  hipLaunchKernelGGL((group_bin_combine_kernel<T, MODE>), dim3(1024), dim3(kBinBlock), 0, stream, g, p);
  return hipGetLastError() == hipSuccess ? TS_OK : TS_ERR_LAUNCH;
}

}  // namespace ts
