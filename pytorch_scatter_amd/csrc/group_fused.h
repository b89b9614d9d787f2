// Softmax / log-softmax over groups in one pass, forward and backward, for an index that is in order
// (included by group_softmax.h).
//
// With a sorted index a group is a run of neighbouring entries. A workgroup stages a tile of entries in LDS
// (16-byte coalesced loads), finds the runs from the index, and finishes every run that lies inside the tile
// there: maximum, sum of exponentials and result all come from LDS, so src is read once and out written once
// (composite/softmax.py:8-59 makes two scatters, two gathers and four elementwise passes of it). A run that
// crosses a tile border leaves a partial per tile (maximum as a key, sum relative to that maximum); a second
// kernel puts the partials of a run together (sums rescaled by exp(m_tile - m_run)) and finishes those entries
// from src. Every tile checks the order of its part of the index; one descent anywhere sets a flag, and the
// caller's three-pass kernels, gated on that flag, then overwrite the result. No atomics on data: the result
// does not depend on scheduling.
//
//   forward   m = run maximum (entries beat lowest(), NaN never wins, no winner: 0), e = exp(src - m),
//             s = sum e;  softmax e / s,  log-softmax (src - m) - log(s + eps)
//   backward  softmax: y * (g - sum y * g);  log-softmax: g - exp(y) * sum g
#pragma once

namespace ts {

constexpr int kFusedMaxTile = 2048;   // entries per tile at most (run starts are 16-bit words with a flag bit)
constexpr int kFusedShortRun = 12;    // runs of up to this many entries inside a tile: one lane per (run, columns)
constexpr int kFusedGroup = 8;        // longer ones: eight lanes, and a wavefront from kFusedGroup * kFusedShortRun entries on
constexpr int kFusedRowBytes = 128;   // widest row the tiles are built for
constexpr int kFusedPer = kFusedMaxTile / kBlock;
constexpr int kFusedVecs = 8;          // 16-byte units of a tile (forward) or of its two tiles (backward) per lane: 32 KB
constexpr int kFusedFragBlock = 128;  // second kernel: one wavefront for the run that enters a tile, one for the run that leaves

struct FusedArgs {
  int te;            // entries per tile: kBlock * epl
  int epl;           // neighbouring entries per lane when the runs are found
  int G;             // second kernel: lanes per partial (power of two >= min(K, 64))
  int tile_vecs;     // 16-byte units of LDS per staged tile
  int short_run;     // runs of more entries than this inside a tile take eight lanes,
  int long_run;      // of more than this a wavefront
  int64_t nt;        // tiles per batch
  int32_t *meta;     // [B * nt][4]: entries of the entering run, first entry of the leaving run, entries, tile is one run that enters and leaves
  void *ckey;        // [B * nt][2][K] forward: keys of the partial maxima (entering, leaving)
  void *csum;        // [B * nt][2][K] partial sums
  int *flag;         // != 0: the index is not in order, nothing here runs (or counts)
};

inline bool group_fused_mode(int mode) {
  return mode == GS_SOFTMAX || mode == GS_LOG_SOFTMAX || mode == GS_SOFTMAX_BWD || mode == GS_LOG_SOFTMAX_BWD;
}

// bytes of the tiles' records for a call of this shape (0: the tiles do not apply), the larger of forward and backward
inline size_t group_fused_scratch_bytes(int64_t B, int64_t E, int64_t K, int elem_bytes) {
  const int64_t row = K * elem_bytes;
  if (row > kFusedRowBytes || E < 2) return 0;
  size_t most = 0;
  for (int backward = 0; backward < 2; ++backward) {
    int64_t te = (backward ? 16384 : 32768) / row;
    int epl = 1;
    while (epl * 2 * kBlock <= te && epl * 2 <= kFusedPer) epl *= 2;
    te = (int64_t)epl * kBlock;
    const size_t tiles = (size_t)(B * ((E + te - 1) / te));
    const size_t acc = elem_bytes == 8 ? 8 : 4;
    auto up = [](size_t x) { return (x + 255) & ~(size_t)255; };
    const size_t end = up(tiles * 16) + 2 * up(tiles * 2 * K * acc);
    if (end > most) most = end;
  }
  return most;
}

// Scratch of the tiles, carved from the front of the group workspace (the three-pass kernels rewrite that
// space if they run at all); the flag sits behind the workspace of the three passes.
inline bool group_fused_plan(const GroupArgs &g, int mode, int elem_bytes, void *ws, size_t ws_three_pass,
                             bool force, FusedArgs &f) {
  if (!group_fused_mode(mode)) return false;
  const bool backward = mode == GS_SOFTMAX_BWD || mode == GS_LOG_SOFTMAX_BWD;
  const int64_t row = g.K * elem_bytes;
  if (row > kFusedRowBytes || g.E < 2) return false;
  auto al16 = [](const void *p) { return (reinterpret_cast<uintptr_t>(p) & 15) == 0; };
  if (!al16(g.src) || !al16(g.out) || (backward && !al16(g.grad))) return false;
  if (g.B > 1 && (g.E * row) % 16 != 0) return false;  // every batch starts on a 16-byte border
  // the launches that return at once cost more than the passes saved below these sizes (sorted index, 9 entries
  // per group, 32-byte rows: forward 31 against 34 us at 8 MB, 45 against 79 us at 32 MB; backward 63 against
  // 51 us and 52 against 58 us)
  if (!force && g.B * g.E * row < ((int64_t)(backward ? 32 : 16) << 20)) return false;
  int64_t te = (backward ? 16384 : 32768) / row;  // 32 KB of LDS per tile
  if (const char *env = getenv("TS_GROUP_TILE")) te = atoi(env);  // tuning aid
  int epl = 1;
  while (epl * 2 * kBlock <= te && epl * 2 <= kFusedPer) epl *= 2;
  te = (int64_t)epl * kBlock;
  if (te * row * (backward ? 2 : 1) > (int64_t)kFusedVecs * kBlock * 16) return false;
  f.te = (int)te;
  f.short_run = kFusedShortRun;
  f.long_run = kFusedGroup * kFusedShortRun;
  if (const char *env = getenv("TS_GROUP_SHORT_RUN")) f.short_run = atoi(env) < 4 ? 4 : atoi(env);  // tuning aids
  if (const char *env = getenv("TS_GROUP_LONG_RUN")) f.long_run = atoi(env);
  if (f.long_run < f.short_run) f.long_run = f.short_run;
  f.epl = epl;
  f.nt = (g.E + te - 1) / te;
  if (g.B * f.nt >= 0x7FFFFFFFll) return false;
  int G = 1;
  while (G < g.K && G < kWave) G *= 2;
  f.G = G;
  f.tile_vecs = (int)((te * row + 15) / 16);
  const size_t acc = elem_bytes == 8 ? 8 : 4;
  auto up = [](size_t x) { return (x + 255) & ~(size_t)255; };
  const size_t tiles = (size_t)(g.B * f.nt);
  const size_t o_key = up(tiles * 16), o_sum = o_key + up(tiles * 2 * g.K * acc);
  const size_t end = o_sum + up(tiles * 2 * g.K * acc);
  // the records of the tiles: in the caller's extra scratch when it has room, else in the front of the three passes'
  // workspace (which they rewrite if they run at all)
  // (rows of up to 64 bytes: with few, large groups every run crosses tiles, and for wider rows the three passes are then
  // ahead -- 4 M entries in 4 k groups, sorted: 8 floats 184 -> 148 us with the tiles, 64 bf16 892 -> 1058 us)
  const bool extra = g.fused_ws != nullptr && end <= g.fused_ws_bytes && row <= 64 &&
                     (reinterpret_cast<uintptr_t>(g.fused_ws) & 15) == 0;
  if (!extra && end > ws_three_pass) return false;
  char *base = extra ? static_cast<char *>(g.fused_ws) : static_cast<char *>(ws);
  f.meta = reinterpret_cast<int32_t *>(base);
  f.ckey = base + o_key;
  f.csum = base + o_sum;
  f.flag = reinterpret_cast<int *>(static_cast<char *>(ws) + ws_three_pass);  // (always behind the three passes' part)
  return true;
}

// A look at up to 1024 pairs of neighbours spread over the index: *flag = 1 (not in order, the tiles do not
// run) if at least 1/64 of them descend, else 0 (the tiles run and check every pair).
// Also clears `clear_n` 8-byte words at `clear` (the bucket totals of the passes that follow an index found out of order).
static __global__ __launch_bounds__(1024) void group_order_sample_kernel(GroupArgs g, int *flag, int force,
                                                                          unsigned long long *clear, int clear_n) {
  __shared__ int s_desc, s_pairs;
  for (int i = threadIdx.x; i < clear_n; i += 1024) clear[i] = 0;
  if (threadIdx.x == 0) { s_desc = 0; s_pairs = 0; }
  __syncthreads();
  const int64_t total = g.B * g.E;
  const int64_t step = (total - 1) / 1024 + 1;
  const int64_t be = (int64_t)threadIdx.x * step;
  if (be + 1 < total) {
    const int64_t b = be / g.E, e = be - b * g.E;
    if (e + 1 < g.E) {
      const int64_t *idx = g.index + b * g.sb;
      atomicAdd(&s_pairs, 1);
      if (idx[(e + 1) * g.se] < idx[e * g.se]) atomicAdd(&s_desc, 1);
    }
  }
  __syncthreads();
  if (threadIdx.x == 0) *flag = (!force && s_desc * 64 >= s_pairs && s_desc > 0) ? 1 : 0;
}

// combination of two partials of a run, a before b: maximum as a key, sum relative to that maximum.
// A partial in which nothing beat lowest() (key == empty) was summed relative to 0 and holds 0 or NaN: taken as is.
template <typename T>
__device__ __forceinline__ void fused_absorb(typename OrdKey<typename Acc<T>::type>::bits &ka, typename Acc<T>::type &sa,
                                             typename OrdKey<typename Acc<T>::type>::bits kb, typename Acc<T>::type sb) {
  typedef typename Acc<T>::type F;
  typedef typename OrdKey<F>::bits KB;
  const KB empty = group_empty_key<T>();
  if (kb > ka) {
    const F fac = ka == empty ? (F)1 : exp_acc(OrdKey<F>::dec(ka) - OrdKey<F>::dec(kb));
    sa = sa * fac + sb;
    ka = kb;
  } else {
    const F fac = (kb == empty || kb == ka) ? (F)1 : exp_acc(OrdKey<F>::dec(kb) - OrdKey<F>::dec(ka));
    sa = sa + sb * fac;
  }
}

__device__ __forceinline__ float fast_rcp(float v) { return __builtin_amdgcn_rcpf(v); }
__device__ __forceinline__ double fast_rcp(double v) { return 1.0 / v; }

// Which entries of the tile begin a run, and whether that run's index lies outside [0, N). The index is loaded
// coalesced (lane tid takes entries tid, tid + 256, ...: with one value per entry the index is two thirds of the
// bytes); an entry's predecessor comes from the neighbouring lane, for the first lane of a wavefront from memory.
// The flags go through LDS (a byte per entry) so that afterwards every lane holds those of its EPL neighbouring
// entries e0 .. e0 + EPL - 1 as bit masks. All index loads are issued before `between` runs (the caller's stores
// of the staged tile, which wait for the tile's loads). Ends with the workgroup in step (barrier).
template <int EPL, typename Between>
__device__ __forceinline__ void fused_find_runs(const int64_t *idx, int64_t se, int64_t j0, int tid, int ne, int64_t E,
                                                int64_t N, uint8_t *s_flag, Between &&between, uint32_t &headmask,
                                                uint32_t &badmask, bool &descent, bool &enters, bool &leaves) {
  const int lane = tid & (kWave - 1);
  int64_t id[EPL], edge[EPL];
#pragma unroll
  for (int q = 0; q < EPL; ++q) {
    const int e = tid + q * kBlock;
    id[q] = e < ne ? idx[(j0 + e) * se] : 0;
  }
#pragma unroll
  for (int q = 0; q < EPL; ++q) {
    const int e = tid + q * kBlock;
    edge[q] = (lane == 0 && e < ne && j0 + e > 0) ? idx[(j0 + e - 1) * se] : 0;
  }
  const int e_last = ne - 1;
  const bool owns_last = (e_last & (kBlock - 1)) == tid;
  int64_t next = 0;
  const bool have_next = owns_last && j0 + ne < E;
  if (have_next) next = idx[(j0 + ne) * se];
  between();
#pragma unroll
  for (int q = 0; q < EPL; ++q) {
    const int e = tid + q * kBlock;
    const int64_t up = lane_up1_64(id[q]);  // by every lane, lane 0 included: its value is what lane 1 reads
    const int64_t prev = lane == 0 ? edge[q] : up;
    if (e < ne) {
      const bool have_prev = j0 + e > 0;
      const bool head = e == 0 || id[q] != prev;
      const bool bad = head && (id[q] < 0 || id[q] >= N);
      if (have_prev && id[q] < prev) descent = true;
      if (e == 0 && have_prev && id[q] == prev) enters = true;
      if (e == e_last && have_next && next == id[q]) leaves = true;
      s_flag[e] = (uint8_t)((head ? 1 : 0) | (bad ? 2 : 0));
    }
  }
  __syncthreads();
  const int e0 = tid * EPL;
#pragma unroll
  for (int i = 0; i < EPL; ++i) {
    if (e0 + i < ne) {
      const uint32_t fl = s_flag[e0 + i];
      headmask |= (fl & 1u) << i;
      badmask |= (fl >> 1 & 1u) << i;
    }
  }
}

template <typename T, int CV, int MODE>
__global__ __launch_bounds__(kBlock, 4) void group_fused_kernel(GroupArgs g, FusedArgs f) {
  typedef typename Acc<T>::type F;
  typedef typename OrdKey<F>::bits KB;
  typedef uint32_t u4 __attribute__((ext_vector_type(4)));
  constexpr bool kBackward = MODE == GS_SOFTMAX_BWD || MODE == GS_LOG_SOFTMAX_BWD;
  constexpr int W = kBlock / kWave;
  // [tile of src][backward: tile of grad][run starts: te + 2 16-bit words, bit 15: index outside [0, N)]
  extern __shared__ u4 s_dyn[];
  __shared__ int s_wsum[W];
  __shared__ int s_info[6];  // run enters from the tile before, run leaves into the next tile, runs for a wavefront, descent seen,
                             // runs for eight lanes, some run belongs to no group
  __shared__ uint32_t s_bad[kFusedMaxTile / 32];  // forward: entries of runs that belong to no group
  __shared__ int32_t s_long[kFusedMaxTile / 4 + 2];  // runs for eight lanes from the front, for a wavefront from the back
  if (*f.flag != 0) return;
  const int tid = threadIdx.x, lane = tid & (kWave - 1), wave = tid / kWave;
  if (tid < 6) s_info[tid] = 0;
  if (tid < kFusedMaxTile / 32) s_bad[tid] = 0;
  __syncthreads();
  const int K = (int)g.K;
  const int64_t b = blockIdx.x / f.nt, t = blockIdx.x - b * f.nt;
  const int64_t j0 = t * f.te;
  const int ne = (int)(g.E - j0 < f.te ? g.E - j0 : f.te);
  T *s_src = reinterpret_cast<T *>(s_dyn);
  T *s_grad = reinterpret_cast<T *>(s_dyn + f.tile_vecs);
  uint16_t *s_start = reinterpret_cast<uint16_t *>(s_dyn + (kBackward ? 2 : 1) * f.tile_vecs);

  // ---- the tile of src (and grad): whole 16-byte units (the unit behind the last entry stays inside its page),
  // every load of the tile and of the index in flight before the first one is waited for
  const int nvec = (int)(((size_t)ne * K * sizeof(T) + 15) / 16);
  const int nstage = kBackward ? 2 * f.tile_vecs : f.tile_vecs;  // unit v of the staged space: tile v / tile_vecs
  u4 stage[kFusedVecs];
  {
    const u4 *p0 = reinterpret_cast<const u4 *>(static_cast<const T *>(g.src) + (b * g.E + j0) * K);
    const u4 *p1 = kBackward ? reinterpret_cast<const u4 *>(static_cast<const T *>(g.grad) + (b * g.E + j0) * K) : p0;
#pragma unroll
    for (int q = 0; q < kFusedVecs; ++q) {
      const int v = tid + q * kBlock;
      const bool second = kBackward && v >= f.tile_vecs;
      const int vv = second ? v - f.tile_vecs : v;
      if (v < nstage && vv < nvec) stage[q] = __builtin_nontemporal_load((second ? p1 : p0) + vv);
    }
  }

  // ---- runs: a lane looks at epl neighbouring entries
  const int64_t *idx = g.index + b * g.sb;
  const int e0 = tid * f.epl;
  uint8_t *s_flag = reinterpret_cast<uint8_t *>(s_start);  // read by all lanes before the run starts are written
  uint32_t headmask = 0, badmask = 0;
  bool descent = false, lane_enters = false, lane_leaves = false;
  auto stage_to_lds = [&]() {
#pragma unroll
    for (int q = 0; q < kFusedVecs; ++q) {
      const int v = tid + q * kBlock;
      const int vv = (kBackward && v >= f.tile_vecs) ? v - f.tile_vecs : v;
      if (v < nstage && vv < nvec) s_dyn[v] = stage[q];
    }
  };
  switch (f.epl) {
  case 1: fused_find_runs<1>(idx, g.se, j0, tid, ne, g.E, g.N, s_flag, stage_to_lds, headmask, badmask, descent, lane_enters, lane_leaves); break;
  case 2: fused_find_runs<2>(idx, g.se, j0, tid, ne, g.E, g.N, s_flag, stage_to_lds, headmask, badmask, descent, lane_enters, lane_leaves); break;
  case 4: fused_find_runs<4>(idx, g.se, j0, tid, ne, g.E, g.N, s_flag, stage_to_lds, headmask, badmask, descent, lane_enters, lane_leaves); break;
  default: fused_find_runs<8>(idx, g.se, j0, tid, ne, g.E, g.N, s_flag, stage_to_lds, headmask, badmask, descent, lane_enters, lane_leaves); break;
  }
  if (lane_enters) s_info[0] = 1;
  if (lane_leaves) s_info[1] = 1;
  if (badmask != 0) s_info[5] = 1;
  const int heads = __popc(headmask);
  const int incl = wave_inclusive_sum(heads);
  if (lane == kWave - 1) s_wsum[wave] = incl;
  if (__ballot(descent) != 0 && lane == 0) s_info[3] = 1;
  __syncthreads();
  int base = incl - heads, nruns = 0;
#pragma unroll
  for (int w = 0; w < W; ++w) {
    if (w < wave) base += s_wsum[w];
    nruns += s_wsum[w];
  }
#pragma unroll
  for (int i = 0; i < kFusedPer; ++i) {
    if (headmask & (1u << i)) s_start[base++] = (uint16_t)((e0 + i) | ((badmask >> i & 1u) << 15));
  }
  if (tid == 0) s_start[nruns] = (uint16_t)ne;
  __syncthreads();
  if (s_info[3] != 0) {
    // not in order: whatever this launch writes is overwritten by the gated passes that follow
    if (tid == 0 && __hip_atomic_load(f.flag, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT) == 0) atomicOr(f.flag, 1);
    return;
  }
  const bool enters = s_info[0] != 0, leaves = s_info[1] != 0;

  const int64_t tile = b * f.nt + t;
  KB *ckey = static_cast<KB *>(f.ckey) + tile * 2 * K;
  F *csum = static_cast<F *>(f.csum) + tile * 2 * K;
  const F eps = (F)g.eps;

  // The runs of the tile, CV columns at a time: one lane per (run, columns) for short runs, eight lanes or a
  // wavefront for longer ones. fn(run, first column, first entry of this lane, step): the lanes that share a run
  // meet in butterflies, so every one of them holds the run's result. `classify` sorts the longer runs into
  // the two lists first (a later pass over the same tile reuses them).
  const int kc = K / CV;
  const int kc_shift = (kc & (kc - 1)) == 0 ? __ffs(kc) - 1 : -1;  // a division per unit otherwise
  auto for_runs = [&](auto &&fn, bool classify) {
    for (int u = tid; u < nruns * kc; u += kBlock) {
      const int r = kc_shift >= 0 ? u >> kc_shift : u / kc, c = u - r * kc;
      const int len = (s_start[r + 1] & 0x7FFF) - (s_start[r] & 0x7FFF);
      if (len > f.short_run) {
        if (classify && c == 0) {
          if (len > f.long_run)
            s_long[kFusedMaxTile / 4 + 1 - atomicAdd(&s_info[2], 1)] = r;
          else
            s_long[atomicAdd(&s_info[4], 1)] = r;
        }
        continue;
      }
      fn(r, c * CV, 0, 1);
    }
    if (classify) __syncthreads();
    const int nmed = s_info[4], nlong = s_info[2];
    for (int u = tid / kFusedGroup; u < nmed * kc; u += kBlock / kFusedGroup) {
      const int q = kc_shift >= 0 ? u >> kc_shift : u / kc;
      fn(s_long[q], (u - q * kc) * CV, tid & (kFusedGroup - 1), kFusedGroup);
    }
    for (int q = wave; q < nlong; q += W) {
      const int r = s_long[kFusedMaxTile / 4 + 1 - q];
      for (int c = 0; c < kc; ++c) fn(r, c * CV, lane, kWave);
    }
  };
  // the entries of a run that this launch finishes: all of them unless the run enters or leaves the tile
  const int w_lo = enters ? (s_start[1] & 0x7FFF) : 0;  // nruns == 1: s_start[1] == ne
  const int w_hi = leaves ? (s_start[nruns - 1] & 0x7FFF) : ne;
  T *out_t = static_cast<T *>(g.out) + (b * g.E + j0) * K;
  constexpr int kPer = 16 / (int)sizeof(T);
  const int el_lo = w_lo * K, el_hi = w_hi * K;

  if constexpr (!kBackward) {
    // Forward. The tile's values stay in the registers they were loaded into; LDS holds, element by element,
    // first the values, then the run's maximum, then exp(value - maximum), then the run's divisor (or logarithm):
    // the passes over the runs only reduce and spread (cheap, one lane per run), exp and the division run one
    // lane per element.
    const KB empty = group_empty_key<T>();
    constexpr bool kSameType = sizeof(T) == sizeof(F);
    // maximum over the entries that are no NaN (maxnum returns the other operand); a winner has to beat lowest()
    const F lowest = to_acc<T>(ElemLim<T>::lowest());
    auto run_max = [&](int r, int c0, int first, int step) {
      const int lo = s_start[r] & 0x7FFF, hi = s_start[r + 1] & 0x7FFF;
      F top[CV];
#pragma unroll
      for (int v = 0; v < CV; ++v) top[v] = -INFINITY;
      for (int e = lo + first; e < hi; e += step) {
        const Vec<T, CV> x = load_vec<T, CV>(s_src + e * K + c0);
#pragma unroll
        for (int v = 0; v < CV; ++v) top[v] = max_acc(top[v], to_acc<T>(x.v[v]));
      }
#pragma unroll
      for (int v = 0; v < CV; ++v) top[v] = group_butterfly(top[v], step, [](F p, F q) { return max_acc(p, q); });
      const bool frag_in = r == 0 && enters, frag_out = r == nruns - 1 && leaves;
      if ((frag_in || frag_out) && first == 0) {
#pragma unroll
        for (int v = 0; v < CV; ++v) ckey[(frag_in ? 0 : 1) * K + c0 + v] = top[v] > lowest ? OrdKey<F>::enc(top[v]) : empty;
      }
      Vec<T, CV> m;
#pragma unroll
      for (int v = 0; v < CV; ++v) m.v[v] = from_acc<T>(top[v] > lowest ? top[v] : (F)0);
      for (int e = lo + first; e < hi; e += step) store_vec<T, CV>(s_src + e * K + c0, m);
    };
    auto run_sum = [&](int r, int c0, int first, int step) {
      const int lo = s_start[r] & 0x7FFF, hi = s_start[r + 1] & 0x7FFF;
      F s[CV];
#pragma unroll
      for (int v = 0; v < CV; ++v) s[v] = (F)0;
      for (int e = lo + first; e < hi; e += step) {
        const Vec<T, CV> x = load_vec<T, CV>(s_src + e * K + c0);
#pragma unroll
        for (int v = 0; v < CV; ++v) s[v] += to_acc<T>(x.v[v]);
      }
#pragma unroll
      for (int v = 0; v < CV; ++v) s[v] = group_butterfly(s[v], step, [](F p, F q) { return p + q; });
      const bool frag_in = r == 0 && enters, frag_out = r == nruns - 1 && leaves;
      if (frag_in || frag_out) {
        if (first == 0) {
#pragma unroll
          for (int v = 0; v < CV; ++v) csum[(frag_in ? 0 : 1) * K + c0 + v] = s[v];
        }
        return;
      }
      Vec<T, CV> d;
#pragma unroll
      for (int v = 0; v < CV; ++v) {
        if (MODE == GS_SOFTMAX)  // fp32 / fp64: the reciprocal, one division per run instead of one per entry
          d.v[v] = kSameType ? from_acc<T>((F)1 / s[v]) : from_acc<T>(s[v]);
        else
          d.v[v] = from_acc<T>(log_acc(round_elem<T>(round_elem<T>(s[v]) + eps)));
      }
      for (int e = lo + first; e < hi; e += step) store_vec<T, CV>(s_src + e * K + c0, d);
      if ((s_start[r] >> 15) != 0 && c0 == 0) {  // a run that belongs to no group: its entries yield 0
        for (int e = lo + first; e < hi; e += step) atomicOr(&s_bad[e >> 5], 1u << (e & 31));
      }
    };

    for_runs(run_max, true);
    __syncthreads();
#pragma unroll
    for (int q = 0; q < kFusedVecs; ++q) {
      const int v = tid + q * kBlock;
      if (v < nvec) {
        Vec<T, kPer> x, m;
        __builtin_memcpy(&x, &stage[q], 16);
        __builtin_memcpy(&m, &s_dyn[v], 16);
#pragma unroll
        for (int i = 0; i < kPer; ++i) {
          const F z = round_elem<T>(to_acc<T>(x.v[i]) - to_acc<T>(m.v[i]));
          m.v[i] = from_acc<T>(exp_acc(z));
          x.v[i] = MODE == GS_SOFTMAX ? m.v[i] : from_acc<T>(z);
        }
        __builtin_memcpy(&s_dyn[v], &m, 16);
        __builtin_memcpy(&stage[q], &x, 16);
      }
    }
    __syncthreads();
    for_runs(run_sum, false);
    __syncthreads();
    const bool any_bad = s_info[5] != 0;
#pragma unroll
    for (int q = 0; q < kFusedVecs; ++q) {
      const int v = tid + q * kBlock;
      if (v < nvec && (v + 1) * kPer > el_lo && v * kPer < el_hi) {
        Vec<T, kPer> x, d;
        __builtin_memcpy(&x, &stage[q], 16);
        __builtin_memcpy(&d, &s_dyn[v], 16);
#pragma unroll
        for (int i = 0; i < kPer; ++i) {
          F res;
          if (MODE == GS_SOFTMAX) {
            // 16-bit floats: e and the rounded sum are exact in fp32 and the quotient is rounded to 8 or 11 bits,
            // so the hardware reciprocal (1 ulp of fp32) stands in for the division
            res = to_acc<T>(x.v[i]) * (kSameType ? to_acc<T>(d.v[i]) : fast_rcp(to_acc<T>(d.v[i])));
          } else {
            F l = to_acc<T>(d.v[i]);
            asm volatile("" : "+v"(l));  // see group_finish_kernel
            res = to_acc<T>(x.v[i]) - l;
          }
          if (any_bad) {
            const int e = (v * kPer + i) / K;
            if (e < ne && (s_bad[e >> 5] >> (e & 31) & 1u) != 0) res = (F)0;
          }
          x.v[i] = from_acc<T>(res);
        }
        if (v * kPer >= el_lo && (v + 1) * kPer <= el_hi) {
          u4 r;
          __builtin_memcpy(&r, &x, 16);
          __builtin_nontemporal_store(r, reinterpret_cast<u4 *>(out_t) + v);
        } else {
#pragma unroll
          for (int i = 0; i < kPer; ++i) {
            if (v * kPer + i >= el_lo && v * kPer + i < el_hi) out_t[v * kPer + i] = x.v[i];
          }
        }
      }
    }
  } else {
    // Backward: the tiles of y and g in LDS, one pass over the runs that sums and finishes in place.
    auto run_bwd = [&](int r, int c0, int first, int step) {
      const int lo = s_start[r] & 0x7FFF, hi = s_start[r + 1] & 0x7FFF;
      const bool valid = (s_start[r] >> 15) == 0;
      const bool frag_in = r == 0 && enters, frag_out = r == nruns - 1 && leaves;
      F s[CV];
#pragma unroll
      for (int v = 0; v < CV; ++v) s[v] = (F)0;
      for (int e = lo + first; e < hi; e += step) {
        const Vec<T, CV> y = load_vec<T, CV>(s_src + e * K + c0);
        const Vec<T, CV> gr = load_vec<T, CV>(s_grad + e * K + c0);
#pragma unroll
        for (int v = 0; v < CV; ++v)
          s[v] += MODE == GS_SOFTMAX_BWD ? to_acc<T>(y.v[v]) * to_acc<T>(gr.v[v]) : to_acc<T>(gr.v[v]);
      }
#pragma unroll
      for (int v = 0; v < CV; ++v) s[v] = group_butterfly(s[v], step, [](F p, F q) { return p + q; });
      if (frag_in || frag_out) {
        if (first == 0) {
#pragma unroll
          for (int v = 0; v < CV; ++v) csum[(frag_in ? 0 : 1) * K + c0 + v] = s[v];
        }
        return;
      }
      for (int e = lo + first; e < hi; e += step) {
        Vec<T, CV> y = load_vec<T, CV>(s_src + e * K + c0);
        const Vec<T, CV> gr = load_vec<T, CV>(s_grad + e * K + c0);
#pragma unroll
        for (int v = 0; v < CV; ++v) {
          const F yv = to_acc<T>(y.v[v]), gv = to_acc<T>(gr.v[v]);
          const F res = MODE == GS_SOFTMAX_BWD ? yv * (gv - s[v]) : gv - exp_acc(yv) * s[v];
          y.v[v] = from_acc<T>(valid ? res : (F)0);
        }
        store_vec<T, CV>(s_src + e * K + c0, y);
      }
    };
    for_runs(run_bwd, true);
    __syncthreads();
    // the finished runs leave the tile: whole 16-byte units, single elements at the two ends
    if (w_hi > w_lo) {
      const int v_lo = (el_lo + kPer - 1) / kPer, v_hi = el_hi / kPer;
      if (v_lo >= v_hi) {
        for (int i = el_lo + tid; i < el_hi; i += kBlock) out_t[i] = s_src[i];
      } else {
        u4 *q = reinterpret_cast<u4 *>(out_t);
        for (int v = v_lo + tid; v < v_hi; v += kBlock) __builtin_nontemporal_store(s_dyn[v], q + v);
        for (int i = el_lo + tid; i < v_lo * kPer; i += kBlock) out_t[i] = s_src[i];
        for (int i = v_hi * kPer + tid; i < el_hi; i += kBlock) out_t[i] = s_src[i];
      }
    }
  }
  if (tid == 0) {
    const bool one = nruns == 1 && enters && leaves;
    int32_t *meta = f.meta + tile * 4;
    meta[0] = enters ? w_lo : 0;
    meta[1] = one ? ne : (leaves ? w_hi : ne);
    meta[2] = ne;
    meta[3] = one ? 1 : 0;
  }
}

// Second kernel: the run that enters a tile (wavefront 0) and the run that leaves it (wavefront 1). The partials
// of such a run are those of the tile in which it begins (its leaving run), of the tiles it fills, and of the tile
// in which it ends (its entering run). Every tile of the run combines them in the same order, so all of them use
// the same maximum and sum; then the workgroup finishes the tile's entries of the two runs from src.
template <typename T, int MODE>
__global__ __launch_bounds__(kFusedFragBlock) void group_fused_fragment_kernel(GroupArgs g, FusedArgs f) {
  typedef typename Acc<T>::type F;
  typedef typename OrdKey<F>::bits KB;
  constexpr bool kBackward = MODE == GS_SOFTMAX_BWD || MODE == GS_LOG_SOFTMAX_BWD;
  extern __shared__ double s_fin_raw[];  // [2 runs][K]: maximum, sum
  F *s_fin = reinterpret_cast<F *>(s_fin_raw);
  if (*f.flag != 0) return;
  const int tid = threadIdx.x, lane = tid & (kWave - 1), wave = tid / kWave;
  const int K = (int)g.K;
  const int64_t b = blockIdx.x / f.nt, t = blockIdx.x - b * f.nt;
  const int64_t j0 = t * f.te;
  const int32_t *meta_b = f.meta + b * f.nt * 4;
  const int head_len = meta_b[t * 4 + 0], tail_start = meta_b[t * 4 + 1], ne = meta_b[t * 4 + 2];
  const bool whole = meta_b[t * 4 + 3] != 0;
  const bool has = wave == 0 ? head_len > 0 : tail_start < ne;
  if (has) {
    auto filled = [&](int64_t i) { return meta_b[i * 4 + 3] != 0; };
    int64_t first = t, last = t;
    if (wave == 0) {
      // the tile in which the run begins: the nearest one before t that the run does not fill (tile 0 cannot be filled)
      first = t - 1;
      while (true) {
        const int64_t i = first - lane;
        const uint64_t stop = __ballot(i <= 0 || !filled(i));
        if (stop != 0) {
          first -= __ffsll((unsigned long long)stop) - 1;
          break;
        }
        first -= kWave;
      }
      if (first < 0) first = 0;
    }
    if (wave == 1 || whole) {
      last = t + 1;
      while (true) {
        const int64_t i = last + lane;
        const uint64_t stop = __ballot(i >= f.nt - 1 || !filled(i));
        if (stop != 0) {
          last += __ffsll((unsigned long long)stop) - 1;
          break;
        }
        last += kWave;
      }
      if (last > f.nt - 1) last = f.nt - 1;
    }
    const int G = f.G, S = kWave / G;
    const int j = lane / G, lg = lane - j * G;
    const KB *ckey = static_cast<const KB *>(f.ckey) + b * f.nt * 2 * K;
    const F *csum = static_cast<const F *>(f.csum) + b * f.nt * 2 * K;
    for (int k0 = 0; k0 < K; k0 += G) {
      const int k = k0 + lg;
      const bool col_ok = k < K;
      KB key = kBackward ? (KB)0 : group_empty_key<T>();
      F sum = (F)0;
      for (int64_t i = first + j; i <= last; i += S) {
        const int64_t p = (i * 2 + (i == first ? 1 : 0)) * K + (col_ok ? k : 0);
        if constexpr (kBackward) {
          sum += csum[p];
        } else {
          fused_absorb<T>(key, sum, ckey[p], csum[p]);
        }
      }
      for (int off = S / 2; off >= 1; off >>= 1) {
        const KB ok = __shfl_down(key, off * G);
        const F os = __shfl_down(sum, off * G);
        if constexpr (kBackward) {
          sum += os;
        } else {
          fused_absorb<T>(key, sum, ok, os);
        }
      }
      if (j == 0 && col_ok) {
        F m = (F)0;
        if constexpr (!kBackward) m = key == group_empty_key<T>() ? (F)0 : OrdKey<F>::dec(key);
        s_fin[(wave * K + k) * 2] = m;
        s_fin[(wave * K + k) * 2 + 1] = sum;
      }
    }
  }
  __syncthreads();
  const T *src_t = static_cast<const T *>(g.src) + (b * g.E + j0) * K;
  const T *grad_t = kBackward ? static_cast<const T *>(g.grad) + (b * g.E + j0) * K : nullptr;
  T *out_t = static_cast<T *>(g.out) + (b * g.E + j0) * K;
  const int64_t *idx = g.index + b * g.sb;
  const F eps = (F)g.eps;
  for (int w = 0; w < 2; ++w) {
    const int lo = w == 0 ? 0 : tail_start, hi = w == 0 ? head_len : ne;
    if (hi <= lo) continue;
    const int64_t group = idx[(j0 + (w == 0 ? 0 : ne - 1)) * g.se];
    const bool valid = group >= 0 && group < g.N;
    for (int i = lo * K + tid; i < hi * K; i += kFusedFragBlock) {
      const int k = i % K;
      const F m = s_fin[(w * K + k) * 2], s = s_fin[(w * K + k) * 2 + 1];
      const F xv = to_acc<T>(src_t[i]);
      F res;
      if (MODE == GS_SOFTMAX) {
        res = round_elem<T>(exp_acc(round_elem<T>(xv - m))) / round_elem<T>(s);
      } else if (MODE == GS_LOG_SOFTMAX) {
        F l = round_elem<T>(log_acc(round_elem<T>(round_elem<T>(s) + eps)));
        asm volatile("" : "+v"(l));  // see group_finish_kernel
        res = round_elem<T>(xv - m) - l;
      } else if (MODE == GS_SOFTMAX_BWD) {
        res = xv * (to_acc<T>(grad_t[i]) - s);
      } else {
        res = to_acc<T>(grad_t[i]) - exp_acc(xv) * s;
      }
      out_t[i] = from_acc<T>(valid ? res : (F)0);
    }
  }
}

template <typename T, int CV, int MODE>
int launch_group_fused(const GroupArgs &g, const FusedArgs &f, bool force, hipStream_t stream) {
  constexpr bool kBackward = MODE == GS_SOFTMAX_BWD || MODE == GS_LOG_SOFTMAX_BWD;
  typedef typename Acc<T>::type F;
  hipLaunchKernelGGL(group_order_sample_kernel, dim3(1), dim3(1024), 0, stream, g, f.flag, force ? 1 : 0,
                     g.bins != nullptr ? g.bins->totals : nullptr, g.bins != nullptr ? g.bins->nb : 0);
  const size_t lds = (size_t)f.tile_vecs * 16 * (kBackward ? 2 : 1) + ((size_t)f.te + 2) * 2;
  const unsigned tiles = (unsigned)(g.B * f.nt);
  hipLaunchKernelGGL((group_fused_kernel<T, CV, MODE>), dim3(tiles), dim3(kBlock), lds, stream, g, f);
  hipLaunchKernelGGL((group_fused_fragment_kernel<T, MODE>), dim3(tiles), dim3(kFusedFragBlock),
                     (size_t)g.K * 4 * sizeof(F), stream, g, f);
  return hipGetLastError() == hipSuccess ? TS_OK : TS_ERR_LAUNCH;
}

}  // namespace ts
