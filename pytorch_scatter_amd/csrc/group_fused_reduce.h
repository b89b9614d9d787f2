// scatter_std / scatter_logsumexp in one pass for an index that is in order (included by group_softmax.h behind
// group_binned.h, whose partial type and result rules it shares).
//
// As in group_fused.h a workgroup stages a tile of entries in LDS, finds the runs of equal indices and finishes every
// run that lies inside the tile: here the result is one value per GROUP, so a lane (eight lanes, a wavefront for
// longer runs) walks the run's rows twice -- sum, then squared deviations; maximum, then sum of exponentials -- and
// writes the group's result, with the roundings of the reference's sequence (composite/std.py:27-39,
// logsumexp.py:39-54). A run that crosses a tile border leaves a partial per tile, (n, sum, M2 about the tile's own
// mean) or (maximum as a key, sum relative to it); the second kernel merges the partials of such a run in the tile
// where it ends (GroupBinPart::absorb) and writes its group. Groups without entries are zeroed by a fill launched
// first. Every tile checks the order of its part of the index; one descent sets the flag, and the passes through
// buckets of groups, launched behind and gated on that flag, then write every result again.
#pragma once

namespace ts {

constexpr int kReduceRowBytes = 256;  // widest row of these tiles
constexpr int kReduceVecsWide = 16;   // 16-byte units per lane of a tile of such rows

struct FusedReduceArgs {
  int te;            // entries per tile: kBlock * epl
  int epl;           // neighbouring entries per lane when the runs are found
  int tile_vecs;     // 16-byte units of LDS per staged tile
  int short_run;     // runs of more entries than this inside a tile take eight lanes,
  int long_run;      // of more than this a wavefront
  int64_t nt;        // tiles per batch
  int kcols;         // columns of a row that a workgroup takes: K, or a slice of 256 bytes of a wider row (then
  int slices;        // K / kcols workgroups share a tile of entries, each on its own columns)
  int32_t *meta;     // [B * nt][4]: entries of the entering run, first entry of the leaving run, entries, tile is one run that enters and leaves
  uint64_t *pa;      // [B * nt][2][K] partials of the entering / leaving run: GroupBinPart::a
  double *pb;        //                                                        GroupBinPart::b
  int *flag;         // != 0: the index is not in order, nothing here runs (or counts)
};

struct FusedReducePlan {
  bool ok;
  size_t bytes;  // scratch of the tiles: 0 when they do not apply
  FusedReduceArgs f;
};

// rows of up to 256 bytes, or of a whole number of 256-byte column slices; from 16 MB of input (the launches that
// return at once under any other index)
inline FusedReducePlan group_reduce_fused_plan(int64_t B, int64_t E, int64_t K, int64_t N, int elem_bytes, bool aligned,
                                               void *ws, size_t ws_bytes, bool force) {
  FusedReducePlan r;
  r.ok = false;
  r.bytes = 0;
  const int64_t row_all = K * elem_bytes;
  // rows of more than 256 bytes in column slices of 256 bytes (a whole number of them)
  const int64_t slices = row_all > kReduceRowBytes ? row_all / kReduceRowBytes : 1;
  if (slices * kReduceRowBytes != row_all && slices > 1) return r;
  const int64_t row = row_all / slices;
  if (E < 2 || !aligned) return r;
  if (B > 1 && (E * row_all) % 16 != 0) return r;
  if (!force && B * E * row_all < ((int64_t)16 << 20)) return r;
  // rows of more than 128 bytes (256 entries per tile): not for few groups of many entries, whose runs all cross several
  // tiles (4 M entries of 64 floats in 4 k groups: std 1034 us, 628 us through the buckets behind)
  if (!force && row > kFusedRowBytes && E > 64 * N) return r;
  int64_t te = 32768 / row;  // 32 KB of rows per tile; rows of more than 128 bytes: 256 entries, 64 KB
  if (te < kBlock) te = kBlock;
  if (const char *env = getenv("TS_GROUP_TILE")) te = atoi(env);  // tuning aid
  int epl = 1;
  while (epl * 2 * kBlock <= te && epl * 2 <= kFusedPer) epl *= 2;
  te = (int64_t)epl * kBlock;
  if (te * row > (int64_t)kReduceVecsWide * kBlock * 16) return r;
  FusedReduceArgs &f = r.f;
  f.te = (int)te;
  f.epl = epl;
  f.short_run = kFusedShortRun;
  f.long_run = kFusedGroup * kFusedShortRun;
  f.nt = (E + te - 1) / te;
  f.slices = (int)slices;
  f.kcols = (int)(K / slices);
  if (B * f.nt >= 0x7FFFFFFFll || slices > 65535) return r;
  f.tile_vecs = (int)((te * row + 15) / 16);
  auto up = [](size_t x) { return (x + 255) & ~(size_t)255; };
  const size_t tiles = (size_t)(B * f.nt);
  const size_t o_pa = up(tiles * 16), o_pb = o_pa + up(tiles * 2 * K * 8), o_flag = o_pb + up(tiles * 2 * K * 8);
  r.bytes = o_flag + 256;
  if (ws == nullptr || ws_bytes < r.bytes || (reinterpret_cast<uintptr_t>(ws) & 15) != 0) return r;
  char *base = static_cast<char *>(ws);
  f.meta = reinterpret_cast<int32_t *>(base);
  f.pa = reinterpret_cast<uint64_t *>(base + o_pa);
  f.pb = reinterpret_cast<double *>(base + o_pb);
  f.flag = reinterpret_cast<int *>(base + o_flag);
  r.ok = true;
  return r;
}

// results of groups without entries (the tiles write the groups they meet): zeros
template <typename T, int MODE>
__global__ __launch_bounds__(kBlock) void group_reduce_fill_kernel(GroupArgs g, const int *flag) {
  if (*flag != 0) return;
  const int64_t n = g.B * g.N * g.K;
  T *out = static_cast<T *>(g.out), *total = static_cast<T *>(g.total_w);
  for (int64_t i = (int64_t)blockIdx.x * kBlock + threadIdx.x; i < n; i += (int64_t)gridDim.x * kBlock) {
    out[i] = from_acc<T>((typename Acc<T>::type)0);
    if (MODE == GS_STD) {
      total[i] = from_acc<T>((typename Acc<T>::type)0);
      if (i < g.B * g.N) g.count_w[i] = 0;
    }
  }
}

// NV: 16-byte units of the tile per lane (8: 32 KB of rows, four workgroups per CU; 16: rows of up to 256 bytes, 64 KB)
template <typename T, int CV, int MODE, int NV>
__global__ __launch_bounds__(kBlock, NV > 8 ? 2 : 4) void group_reduce_fused_kernel(GroupArgs g, FusedReduceArgs f) {
  typedef typename Acc<T>::type F;
  typedef GroupBinPart<T, MODE> Part;
  typedef uint32_t u4 __attribute__((ext_vector_type(4)));
  constexpr int W = kBlock / kWave;
  extern __shared__ u4 s_dyn[];  // [tile of src][run starts: te + 2 16-bit words, bit 15: index outside [0, N)]
  __shared__ int s_wsum[W];
  __shared__ int s_info[6];  // run enters, run leaves, runs for a wavefront, descent seen, runs for eight lanes, (unused)
  __shared__ int32_t s_long[kFusedMaxTile / 4 + 2];  // runs for eight lanes from the front, for a wavefront from the back
  if (*f.flag != 0) return;
  const int tid = threadIdx.x, lane = tid & (kWave - 1), wave = tid / kWave;
  if (tid < 6) s_info[tid] = 0;
  __syncthreads();
  const int K = f.kcols;                       // columns of this workgroup, row pitch of the staged tile
  const int64_t KR = g.K;                      // columns of a row in memory
  const int k_first = (int)blockIdx.y * K;     // first column of this workgroup's slice
  const int64_t b = blockIdx.x / f.nt, t = blockIdx.x - b * f.nt;
  const int64_t j0 = t * f.te;
  const int ne = (int)(g.E - j0 < f.te ? g.E - j0 : f.te);
  T *s_src = reinterpret_cast<T *>(s_dyn);
  uint16_t *s_start = reinterpret_cast<uint16_t *>(s_dyn + f.tile_vecs);

  // ---- the tile of src: whole 16-byte units, every load of the tile and of the index in flight together
  const int nvec = (int)(((size_t)ne * K * sizeof(T) + 15) / 16);
  u4 stage[NV];
  {
    const T *tile0 = static_cast<const T *>(g.src) + (b * g.E + j0) * KR + k_first;
    const u4 *p0 = reinterpret_cast<const u4 *>(tile0);
    const int vps = K * (int)sizeof(T) / 16;  // (slices: 16-byte units of an entry's slice, a power of two)
#pragma unroll
    for (int q = 0; q < NV; ++q) {
      const int v = tid + q * kBlock;
      if (v < f.tile_vecs && v < nvec) {
        if (f.slices == 1) {
          stage[q] = __builtin_nontemporal_load(p0 + v);  // the tile is one range of memory
        } else {
          const int ev = v / vps;
          stage[q] = __builtin_nontemporal_load(reinterpret_cast<const u4 *>(tile0 + (int64_t)ev * KR) + (v - ev * vps));
        }
      }
    }
  }
  const int64_t *idx = g.index + b * g.sb;
  const int e0 = tid * f.epl;
  uint8_t *s_flag = reinterpret_cast<uint8_t *>(s_start);  // read by all lanes before the run starts are written
  uint32_t headmask = 0, badmask = 0;
  bool descent = false, lane_enters = false, lane_leaves = false;
  auto stage_to_lds = [&]() {
#pragma unroll
    for (int q = 0; q < NV; ++q) {
      const int v = tid + q * kBlock;
      if (v < f.tile_vecs && v < nvec) s_dyn[v] = stage[q];
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

  // ---- the statistic of run r, columns c0 .. c0 + CV - 1, by `step` neighbouring lanes (1, 8 or 64) that take the
  // run's entries in turn and meet in a butterfly
  auto run_stat = [&](int r, int c0, int first, int step) {
    const int lo = s_start[r] & 0x7FFF, hi = s_start[r + 1] & 0x7FFF, cnt = hi - lo;
    const bool frag_in = r == 0 && enters, frag_out = r == nruns - 1 && leaves;
    const bool single = !(frag_in || frag_out);
    Part part[CV];
    if constexpr (MODE == GS_STD) {
      F acc[CV];
      double sum[CV], m2[CV];
#pragma unroll
      for (int v = 0; v < CV; ++v) acc[v] = (F)0;
      for (int e = lo + first; e < hi; e += step) {
        const Vec<T, CV> y = load_vec<T, CV>(s_src + e * K + c0);
#pragma unroll
        for (int v = 0; v < CV; ++v) acc[v] += to_acc<T>(y.v[v]);
      }
      F mean[CV];
#pragma unroll
      for (int v = 0; v < CV; ++v) {
        sum[v] = group_butterfly((double)acc[v], step, [](double p, double q) { return p + q; });
        // inside the tile: the reference's mean; a run that goes on in another tile: this tile's own mean
        mean[v] = single ? group_mean<T>(from_acc<T>((F)sum[v]), cnt) : (F)(sum[v] / (double)cnt);
        acc[v] = (F)0;
      }
      for (int e = lo + first; e < hi; e += step) {
        const Vec<T, CV> y = load_vec<T, CV>(s_src + e * K + c0);
#pragma unroll
        for (int v = 0; v < CV; ++v) {
          if (single) {
            const F d = round_elem<T>(to_acc<T>(y.v[v]) - mean[v]);
            acc[v] += round_elem<T>(d * d);
          } else {
            const F d = to_acc<T>(y.v[v]) - mean[v];
            acc[v] += d * d;
          }
        }
      }
#pragma unroll
      for (int v = 0; v < CV; ++v) {
        m2[v] = group_butterfly((double)acc[v], step, [](double p, double q) { return p + q; });
        part[v].a = (uint64_t)__double_as_longlong(sum[v]);
        part[v].b = m2[v];
        part[v].n = cnt;
      }
    } else {
      F top[CV], acc[CV];
#pragma unroll
      for (int v = 0; v < CV; ++v) top[v] = -INFINITY, acc[v] = (F)0;
      for (int e = lo + first; e < hi; e += step) {
        const Vec<T, CV> y = load_vec<T, CV>(s_src + e * K + c0);
#pragma unroll
        for (int v = 0; v < CV; ++v) top[v] = max_acc(top[v], to_acc<T>(y.v[v]));  // a NaN never wins
      }
#pragma unroll
      for (int v = 0; v < CV; ++v) {
        top[v] = group_butterfly(top[v], step, [](F p, F q) { return max_acc(p, q); });
        top[v] = OrdKey<F>::dec(OrdKey<F>::enc(top[v]));  // -0.0 folds onto +0.0
      }
      for (int e = lo + first; e < hi; e += step) {
        const Vec<T, CV> y = load_vec<T, CV>(s_src + e * K + c0);
#pragma unroll
        for (int v = 0; v < CV; ++v) {
          F z = round_elem<T>(to_acc<T>(y.v[v]) - top[v]);
          if (z != z) z = -INFINITY;  // NaN entries and -inf - -inf drop out (logsumexp.py:41)
          acc[v] += round_elem<T>(exp_acc(z));
        }
      }
#pragma unroll
      for (int v = 0; v < CV; ++v) {
        part[v].a = (uint64_t)OrdKey<F>::enc(top[v]);
        part[v].b = group_butterfly((double)acc[v], step, [](double p, double q) { return p + q; });
        part[v].n = 0;
      }
    }
    if (first != 0) return;
    if (!single) {
      const int64_t slot = (tile * 2 + (frag_in ? 0 : 1)) * KR + k_first + c0;
#pragma unroll
      for (int v = 0; v < CV; ++v) {
        f.pa[slot + v] = part[v].a;
        f.pb[slot + v] = part[v].b;
      }
      return;
    }
    if ((s_start[r] >> 15) != 0) return;  // a run that belongs to no group
    const int64_t row = b * g.N + idx[(j0 + lo) * g.se];
#pragma unroll
    for (int v = 0; v < CV; ++v) group_bin_emit<T, MODE>(g, row * KR + k_first + c0 + v, row, k_first + c0 + v, part[v]);
  };

  // one lane per (run, columns) for short runs, eight lanes or a wavefront for longer ones
  const int kc = K / CV;
  const int kc_shift = (kc & (kc - 1)) == 0 ? __ffs(kc) - 1 : -1;
  for (int u = tid; u < nruns * kc; u += kBlock) {
    const int r = kc_shift >= 0 ? u >> kc_shift : u / kc, c = u - r * kc;
    const int len = (s_start[r + 1] & 0x7FFF) - (s_start[r] & 0x7FFF);
    if (len > f.short_run) {
      if (c == 0) {
        if (len > f.long_run)
          s_long[kFusedMaxTile / 4 + 1 - atomicAdd(&s_info[2], 1)] = r;
        else
          s_long[atomicAdd(&s_info[4], 1)] = r;
      }
      continue;
    }
    run_stat(r, c * CV, 0, 1);
  }
  __syncthreads();
  const int nmed = s_info[4], nlong = s_info[2];
  // (whole groups of eight lanes: a lane without a run still takes part in its neighbours' butterflies)
  for (int u0 = 0; u0 < nmed * kc * kFusedGroup; u0 += kBlock) {
    const int u = (u0 + tid) / kFusedGroup;
    const bool live = u < nmed * kc;
    const int q = live ? (kc_shift >= 0 ? u >> kc_shift : u / kc) : 0;
    run_stat(s_long[q], live ? (u - q * kc) * CV : 0, live ? (tid & (kFusedGroup - 1)) : 0x7FF0, kFusedGroup);
  }
  for (int q = wave; q < nlong; q += W) {
    const int r = s_long[kFusedMaxTile / 4 + 1 - q];
    for (int c = 0; c < kc; ++c) run_stat(r, c * CV, lane, kWave);
  }
  if (tid == 0 && blockIdx.y == 0) {
    const int w_lo = enters ? (s_start[1] & 0x7FFF) : 0;  // nruns == 1: s_start[1] == ne
    const int w_hi = leaves ? (s_start[nruns - 1] & 0x7FFF) : ne;
    const bool one = nruns == 1 && enters && leaves;
    int32_t *meta = f.meta + tile * 4;
    meta[0] = enters ? w_lo : 0;
    meta[1] = one ? ne : (leaves ? w_hi : ne);
    meta[2] = ne;
    meta[3] = one ? 1 : 0;
  }
}

// Second kernel, one wavefront per tile: the run that entered the tile and ends in it. Its partials are those of the
// tile in which it begins (that tile's leaving run), of the tiles it fills, and of this tile (its entering run).
template <typename T, int MODE>
__global__ __launch_bounds__(kWave) void group_reduce_fragment_kernel(GroupArgs g, FusedReduceArgs f, int G) {
  typedef GroupBinPart<T, MODE> Part;
  if (*f.flag != 0) return;
  const int lane = threadIdx.x;
  const int K = (int)g.K;
  const int64_t b = blockIdx.x / f.nt, t = blockIdx.x - b * f.nt;
  const int32_t *meta_b = f.meta + b * f.nt * 4;
  const int head_len = meta_b[t * 4 + 0];
  if (head_len <= 0 || meta_b[t * 4 + 3] != 0) return;  // no run from an earlier tile ends here
  auto filled = [&](int64_t i) { return meta_b[i * 4 + 3] != 0; };
  int64_t first = t - 1;
  while (true) {  // the nearest tile before t that the run does not fill (tile 0 cannot be filled)
    const int64_t i = first - lane;
    const uint64_t stop = __ballot(i <= 0 || !filled(i));
    if (stop != 0) {
      first -= __ffsll((unsigned long long)stop) - 1;
      break;
    }
    first -= kWave;
  }
  if (first < 0) first = 0;
  const int64_t group = g.index[b * g.sb + t * f.te * g.se];  // the run's index: that of the tile's first entry
  const bool valid = group >= 0 && group < g.N;
  const int S = kWave / G;
  const int j = lane / G, lg = lane - j * G;
  const uint64_t *pa = f.pa + b * f.nt * 2 * K;
  const double *pb = f.pb + b * f.nt * 2 * K;
  for (int k0 = 0; k0 < K; k0 += G) {
    const int k = k0 + lg;
    const bool col_ok = k < K;
    Part acc = Part::identity();
    for (int64_t i = first + j; i <= t; i += S) {
      const int64_t p = (i * 2 + (i == first ? 1 : 0)) * K + (col_ok ? k : 0);
      Part o;
      o.a = pa[p];
      o.b = pb[p];
      o.n = i == first ? meta_b[i * 4 + 2] - meta_b[i * 4 + 1] : meta_b[i * 4 + 0];
      acc.absorb(o);
    }
    for (int off = S / 2; off >= 1; off >>= 1) {
      Part o;
      o.a = ((uint64_t)(uint32_t)__shfl_down((int)(acc.a >> 32), off * G) << 32) |
            (uint32_t)__shfl_down((int)(uint32_t)acc.a, off * G);
      o.b = __shfl_down(acc.b, off * G);
      o.n = __shfl_down(acc.n, off * G);
      acc.absorb(o);
    }
    if (j == 0 && col_ok && valid) {
      const int64_t row = b * g.N + group;
      group_bin_emit<T, MODE>(g, row * K + k, row, k, acc);
    }
  }
}

// sample of the index (also clears the bucket totals of the passes behind), fill, tiles, fragments
template <typename T, int CV, int MODE>
int launch_group_reduce_fused(const GroupArgs &g, const FusedReduceArgs &f, bool force, hipStream_t stream) {
  hipLaunchKernelGGL(group_order_sample_kernel, dim3(1), dim3(1024), 0, stream, g, f.flag, force ? 1 : 0,
                     g.bins != nullptr ? g.bins->totals : nullptr, g.bins != nullptr ? g.bins->nb : 0);
  hipLaunchKernelGGL((group_reduce_fill_kernel<T, MODE>), dim3(grid_for(g.B * g.N * g.K)), dim3(kBlock), 0, stream, g,
                     f.flag);
  const size_t lds = (size_t)f.tile_vecs * 16 + ((size_t)f.te + 2) * 2;
  const unsigned tiles = (unsigned)(g.B * f.nt);
  if ((int64_t)f.tile_vecs > (int64_t)kFusedVecs * kBlock) {
    if (hipFuncSetAttribute(reinterpret_cast<const void *>(&group_reduce_fused_kernel<T, CV, MODE, kReduceVecsWide>),
                            hipFuncAttributeMaxDynamicSharedMemorySize, (int)lds) != hipSuccess)
      return TS_ERR_LAUNCH;
    hipLaunchKernelGGL((group_reduce_fused_kernel<T, CV, MODE, kReduceVecsWide>), dim3(tiles, (unsigned)f.slices), dim3(kBlock), lds, stream, g, f);
  } else {
    hipLaunchKernelGGL((group_reduce_fused_kernel<T, CV, MODE, kFusedVecs>), dim3(tiles, (unsigned)f.slices), dim3(kBlock), lds, stream, g, f);
  }
  int G = 1;
  while (G < g.K && G < kWave) G *= 2;
  hipLaunchKernelGGL((group_reduce_fragment_kernel<T, MODE>), dim3(tiles), dim3(kWave), 0, stream, g, f, G);
  return hipGetLastError() == hipSuccess ? TS_OK : TS_ERR_LAUNCH;
}

}  // namespace ts
