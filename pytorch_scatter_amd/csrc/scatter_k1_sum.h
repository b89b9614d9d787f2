// scatter sum (and the count of scatter mean) of one 4-byte value per entry (K == 1) with a workspace, for the sizes
// between the table kernel and the value buckets (included by scatter.h).
//
// Half a million to two million single values under an index in no order onto many rows: the table kernel
// (scatter_add_lds_kernel) has nothing to combine -- a workgroup's share of the entries holds about as many different
// rows as entries -- so it ends in one device atomic per entry after all, a third from the rows that miss its 4096
// table rows and the rest from writing the table back (1 M values onto 100 k rows, uniform index: 58 us, 50 ps per
// atomic; torch's scatter_add_ the same). The value buckets of scatter_binned.h need six launches and pay from 2 M
// entries. Here, as for min / max of single values (scatter_k1.h):
//
//  * main: up to 256 workgroups of 1024 lanes, one table of kS1Rows (node, sum[, count]) rows each, direct mapped by
//    node & (kS1Rows - 1), first come first served; an entry whose row belongs to another node goes to memory with
//    a device atomic. A workgroup has a few thousand entries, so most of them find a row.
//  * the table is not written back with atomics: a workgroup whose table holds kS1Few rows or more stores all of
//    it into its own slab of the workspace with plain coalesced stores and marks the slab as used. A table with
//    fewer rows (a few hubs), or of a share of the index that is in order, is cheaper to write back row by row with
//    atomics, and its slab stays unused, so an index in order pays for one more launch only.
//  * final: a workgroup takes kS1FinalRows table rows, reads them from all used slabs (neighbouring lanes read
//    neighbouring rows), adds up equal tags in LDS and adds the totals to out / count, one lane per output row, after
//    the main kernel's atomics have landed.
// out (and count) are cleared, or hold the caller's previous content, before the main kernel.
#pragma once

namespace ts {

constexpr int kS1Rows = 8192;      // rows of a workgroup's table
constexpr int kS1Block = 1024;
constexpr int kS1Groups = 256;     // workgroups of the main kernel at most: one per CU
constexpr int kS1PerRow = 64;      // output rows that may share a table row: N <= kS1PerRow * kS1Rows
constexpr int kS1Few = 1536;       // a table with fewer rows in use is written back with atomics (Zipf(1.2) index, 1 M entries
                                   // onto 100 k rows, 1000 rows per table: 31 against 34 us; uniform: 3100 rows, 66 against 35 us)
constexpr int kS1FinalRows = 16;   // table rows per workgroup of the final kernel
constexpr int kS1FinalBlock = 256;
constexpr int kS1MinChunk = 2048;  // entries per workgroup at least

struct S1Plan {
  bool ok;
  int G;            // workgroups of the main kernel (slabs)
  int J;            // output rows per table row
  int64_t epb;      // entries per workgroup, a multiple of four
  size_t bytes;     // workspace
  int32_t *used;    // [G]: 1 = the slab holds the workgroup's table
  uint32_t *slab_vals;  // [G][kS1Rows], bits of the element type
  int32_t *slab_tags;   // [G][kS1Rows]
  int32_t *slab_cnts;   // [G][kS1Rows], with counts only
};

// any_size: also outside the sizes where it pays (tests). The first 256 bytes of the workspace stay free for the
// caller's own flag.
inline S1Plan s1_plan(int64_t B, int64_t E, int64_t K, int64_t N, int elem_bytes, void *ws, size_t ws_bytes,
                      bool with_count, bool any_size) {
  S1Plan p = {};
  if (B != 1 || K != 1 || elem_bytes != 4 || E < 1 || N < 1 || E >= 0x7FFFFFFFll || N > (int64_t)kS1PerRow * kS1Rows)
    return p;
  // below, the table kernel's write-back is cheaper than the slabs (262 k entries: 15 us); above, a workgroup's share
  // holds more different rows than its table and the value buckets take over
  if (!any_size && (E < ((int64_t)1 << 19) || E >= ((int64_t)1 << 21))) return p;
  int64_t G = (E + kS1MinChunk - 1) / kS1MinChunk;
  if (G > kS1Groups) G = kS1Groups;
  p.G = (int)G;
  p.J = (int)((N + kS1Rows - 1) / kS1Rows);
  p.epb = ((E + G - 1) / G + 3) & ~(int64_t)3;
  auto up = [](size_t x) { return (x + 255) & ~(size_t)255; };
  const size_t o_used = 256, o_vals = o_used + up((size_t)G * 4);
  const size_t o_tags = o_vals + up((size_t)G * kS1Rows * 4);
  const size_t o_cnts = o_tags + up((size_t)G * kS1Rows * 4);
  p.bytes = o_cnts + (with_count ? up((size_t)G * kS1Rows * 4) : 0);
  if (ws == nullptr || ws_bytes < p.bytes || (reinterpret_cast<uintptr_t>(ws) & 15) != 0) return p;
  char *base = static_cast<char *>(ws);
  p.used = reinterpret_cast<int32_t *>(base + o_used);
  p.slab_vals = reinterpret_cast<uint32_t *>(base + o_vals);
  p.slab_tags = reinterpret_cast<int32_t *>(base + o_tags);
  p.slab_cnts = with_count ? reinterpret_cast<int32_t *>(base + o_cnts) : nullptr;
  p.ok = true;
  return p;
}

// T: float or int32_t. src == nullptr adds 1 per entry. COUNT: the entries of every output row are counted into
// a.count_out as well.
template <typename T, bool COUNT>
__global__ __launch_bounds__(kS1Block) void scatter_s1_main_kernel(ScatterArgs a, S1Plan p) {
  static_assert(sizeof(T) == 4, "four entries per 16-byte load");
  typedef typename TableSlot<T>::type Slot;  // double for float: its LDS add keeps its rate when lanes meet on a row
  typedef int64_t i64x2 __attribute__((ext_vector_type(2)));
  constexpr int mask = kS1Rows - 1;
  __shared__ Slot s_val[kS1Rows];
  __shared__ int32_t s_tags[kS1Rows];
  __shared__ int32_t s_cnt[COUNT ? kS1Rows : 1];
  __shared__ int32_t s_occ, s_mixed;
  for (int i = threadIdx.x; i < kS1Rows; i += kS1Block) {
    s_val[i] = (Slot)0;
    s_tags[i] = -1;
    if constexpr (COUNT) s_cnt[i] = 0;
  }
  if (threadIdx.x == 0) {
    s_occ = 0;
    s_mixed = 0;
  }
  __syncthreads();

  const T *src = static_cast<const T *>(a.src);
  T *out = static_cast<T *>(a.out);
  const int64_t total4 = a.E & ~(int64_t)3;  // entries covered in groups of four
  const int64_t lo = (int64_t)blockIdx.x * p.epb;
  const int64_t hi = lo + p.epb < total4 ? lo + p.epb : total4;
  auto add = [&](int64_t idx, T x) {
    if (idx < 0 || idx >= a.N) return;
    const int node = (int)idx;
    const int row = node & mask;
    int tag = lds_peek(&s_tags[row]);
    if (tag == -1) {
      const int old = atomicCAS(&s_tags[row], -1, node);
      tag = old == -1 ? node : old;
    }
    if (tag == node) {
      __hip_atomic_fetch_add(&s_val[row], (Slot)x, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_WORKGROUP);
      if constexpr (COUNT) atomicAdd(&s_cnt[row], 1);
    } else {
      atomic_add_elem<T>(out + node, x);
      if constexpr (COUNT) atomicAdd(a.count_out + node, 1);
    }
  };
  // (every lane takes part in every round, so that neighbours can compare their entries)
  bool ascending = true;
  for (int64_t base = lo; base < hi; base += (int64_t)kS1Block * 4) {
    const int64_t e0 = base + (int64_t)threadIdx.x * 4;
    const bool live = e0 < hi;
    const int64_t ec = live ? e0 : lo;
    const i64x2 ia = __builtin_nontemporal_load(reinterpret_cast<const i64x2 *>(a.index + ec));
    const i64x2 ib = __builtin_nontemporal_load(reinterpret_cast<const i64x2 *>(a.index + ec) + 1);
    Vec<T, 4> x;
    if (src != nullptr) {
      x = load_vec_stream<T, 4>(src + ec);
    } else {
#pragma unroll
      for (int u = 0; u < 4; ++u) x.v[u] = (T)1;
    }
    // is this share of the index in order? (judged inside each wavefront's strip)
    const int64_t next = __shfl_down(ia.x, 1);
    const bool has_next = (threadIdx.x & (kWave - 1)) != kWave - 1 && e0 + 4 < hi;
    if (live && !(ia.x <= ia.y && ia.y <= ib.x && ib.x <= ib.y && (!has_next || ib.y <= next))) ascending = false;
    if (live) {
      add(ia.x, x.v[0]);
      add(ia.y, x.v[1]);
      add(ib.x, x.v[2]);
      add(ib.y, x.v[3]);
    }
  }
  if (!ascending) s_mixed = 1;
  // the last E % 4 entries
  if (blockIdx.x == gridDim.x - 1 && (int64_t)threadIdx.x < a.E - total4) {
    const int64_t e = total4 + threadIdx.x;
    add(a.index[e], src != nullptr ? src[e] : (T)1);
  }
  __syncthreads();
  {
    int mine = 0;
    for (int i = threadIdx.x; i < kS1Rows; i += kS1Block) mine += s_tags[i] != -1 ? 1 : 0;
    mine = wave_inclusive_sum(mine);
    if ((threadIdx.x & (kWave - 1)) == kWave - 1 && mine != 0) atomicAdd(&s_occ, mine);
  }
  __syncthreads();
  if (s_occ < kS1Few || s_mixed == 0) {
    // few rows (a few hubs), or a share of the index that is in order (its rows are neighbours in memory and no other
    // workgroup's, so the atomics come cheap: 1 M entries onto 500 k rows, 1700 rows per table, 11 against 28 us):
    // written back one by one, the slab stays unused
    for (int i = threadIdx.x; i < kS1Rows; i += kS1Block) {
      const int tag = s_tags[i];
      if (tag == -1) continue;
      atomic_add_elem<T>(out + tag, (T)s_val[i]);
      if constexpr (COUNT) atomicAdd(a.count_out + tag, s_cnt[i]);
    }
    if (threadIdx.x == 0) p.used[blockIdx.x] = 0;
    return;
  }
  uint32_t *sv = p.slab_vals + (int64_t)blockIdx.x * kS1Rows;
  int32_t *st = p.slab_tags + (int64_t)blockIdx.x * kS1Rows;
  for (int i = threadIdx.x; i < kS1Rows; i += kS1Block) {
    const T v = (T)s_val[i];
    uint32_t bits;
    __builtin_memcpy(&bits, &v, 4);
    sv[i] = bits;
    st[i] = s_tags[i];
    if constexpr (COUNT) p.slab_cnts[(int64_t)blockIdx.x * kS1Rows + i] = s_cnt[i];
  }
  if (threadIdx.x == 0) p.used[blockIdx.x] = 1;
}

template <typename T, bool COUNT>
__global__ __launch_bounds__(kS1FinalBlock) void scatter_s1_final_kernel(ScatterArgs a, S1Plan p) {
  typedef typename TableSlot<T>::type Slot;
  constexpr int RB = kS1FinalRows;
  constexpr int WG = kS1FinalBlock / RB;  // groups of slabs
  __shared__ Slot s_slot[RB * kS1PerRow];
  __shared__ int32_t s_cslot[COUNT ? RB * kS1PerRow : 1];
  __shared__ int32_t s_any;
  const int J = p.J;
  // no slab in use (an index in order): nothing to do
  if (__syncthreads_or((int)threadIdx.x < p.G && p.used[threadIdx.x] != 0) == 0) return;
  for (int i = threadIdx.x; i < RB * J; i += kS1FinalBlock) {
    s_slot[i] = (Slot)0;
    if constexpr (COUNT) s_cslot[i] = 0;
  }
  if (threadIdx.x == 0) s_any = 0;
  __syncthreads();
  const int r0 = blockIdx.x * RB;
  const int rl = threadIdx.x % RB;
  const int wg = threadIdx.x / RB;
  {
    // equal tags of slabs that follow each other (a hub is in every table) are added in registers first
    int cur_tag = -1, cur_cnt = 0;
    Slot cur = (Slot)0;
    bool any = false;
    auto flush = [&]() {
      if (cur_tag < 0) return;
      __hip_atomic_fetch_add(&s_slot[rl * J + cur_tag / kS1Rows], cur, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_WORKGROUP);
      if constexpr (COUNT) atomicAdd(&s_cslot[rl * J + cur_tag / kS1Rows], cur_cnt);
      any = true;
    };
    constexpr int U = 8;
    for (int w0 = wg; w0 < p.G; w0 += WG * U) {
      uint32_t v[U];
      int32_t t[U], c[U];
#pragma unroll
      for (int u = 0; u < U; ++u) {
        const int w = w0 + u * WG;
        const bool live = w < p.G && p.used[w] != 0;
        const int64_t at = (int64_t)(live ? w : 0) * kS1Rows + r0 + rl;
        t[u] = live ? p.slab_tags[at] : -1;
        v[u] = live ? p.slab_vals[at] : 0u;
        c[u] = (COUNT && live) ? p.slab_cnts[at] : 0;
      }
#pragma unroll
      for (int u = 0; u < U; ++u) {
        if (t[u] < 0) continue;
        T x;
        __builtin_memcpy(&x, &v[u], 4);
        if (t[u] == cur_tag) {
          cur += (Slot)x;
          cur_cnt += c[u];
        } else {
          flush();
          cur_tag = t[u];
          cur = (Slot)x;
          cur_cnt = c[u];
        }
      }
    }
    flush();
    if (any) s_any = 1;
  }
  __syncthreads();
  if (s_any == 0) return;  // no slab in use, or none of these rows
  T *out = static_cast<T *>(a.out);
  for (int i = threadIdx.x; i < RB * J; i += kS1FinalBlock) {
    const int j = i / RB, r = i - j * RB;  // neighbouring lanes: neighbouring output rows
    const int64_t n = (int64_t)j * kS1Rows + r0 + r;
    if (n >= a.N) continue;
    if constexpr (COUNT) {
      // (a row with entries in a slab has a count there; its sum may still be zero)
      const int32_t c = s_cslot[r * J + j];
      if (c == 0) continue;
      a.count_out[n] += c;
      out[n] = (T)((Slot)out[n] + s_slot[r * J + j]);
    } else {
      const Slot v = s_slot[r * J + j];
      if (v != (Slot)0) out[n] = (T)((Slot)out[n] + v);
    }
  }
}

template <typename T>
void launch_scatter_s1(const ScatterArgs &a, const S1Plan &p, hipStream_t stream) {
  if (a.count_out != nullptr) {
    hipLaunchKernelGGL((scatter_s1_main_kernel<T, true>), dim3((unsigned)p.G), dim3(kS1Block), 0, stream, a, p);
    hipLaunchKernelGGL((scatter_s1_final_kernel<T, true>), dim3(kS1Rows / kS1FinalRows), dim3(kS1FinalBlock), 0, stream,
                       a, p);
  } else {
    hipLaunchKernelGGL((scatter_s1_main_kernel<T, false>), dim3((unsigned)p.G), dim3(kS1Block), 0, stream, a, p);
    hipLaunchKernelGGL((scatter_s1_final_kernel<T, false>), dim3(kS1Rows / kS1FinalRows), dim3(kS1FinalBlock), 0, stream,
                       a, p);
  }
}

}  // namespace ts
