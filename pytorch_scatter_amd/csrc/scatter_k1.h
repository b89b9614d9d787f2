// scatter min / max (+arg) of one 4-byte value per entry (K == 1) with a workspace (included by scatter.h).
//
// What the time of such a call consists of (10 M entries of a Zipf(1.2) index onto 100 k rows, 121 MB, measured
// by switching stages off): the stream itself takes 16 us and the LDS table work a few more, but every update of
// the packed-key table in memory is a device atomic, and those complete at about 26 G/s when their addresses
// are scattered (one transaction per lane), whatever their scope and whether or not a stream runs next to
// them: 0.8 M entries that miss a 4096-row table and 1 M table rows written back by 256 workgroups at the
// same moment (so that a read before the atomic filters nothing) cost 60 us of the 77 us of the kernel without
// workspace (scatter_key_lds_k1_kernel). Its two helper launches (initial fill of the keys, unpacking) add
// 5 us each. Here:
//
//  * main: 256 workgroups of 1024 lanes, one table of kK1Rows (node, packed key) rows each, direct mapped by
//    node & (kK1Rows - 1), first come first served (8192 rows: 3.8 % of the entries miss, 4096 rows: 8 %).
//    Fourteen wavefronts stream: a lane takes four consecutive entries per batch with 16-byte loads and keeps
//    kK1Depth batches in flight. Their loop holds loads and LDS accesses only, all loads unconditional: an
//    atomic or a conditional load inside it makes the compiler wait for every outstanding access at each
//    turn (reads and writes return out of order with respect to each other, and a load that may not have
//    been issued cannot be counted). An entry whose row belongs to another node is pushed into a queue in
//    LDS; the two remaining wavefronts do nothing but take entries from their queue and issue the atomics.
//  * the table is not written back with atomics: every workgroup stores its rows (tag, key) into its own
//    slab of the workspace with plain coalesced stores (24 bytes of traffic per row instead of an atomic);
//  * final: a workgroup takes kK1FinalRows table rows, reads them from all slabs (neighbouring lanes read
//    neighbouring rows), combines equal tags in registers and LDS, adds what the key table in memory holds
//    for each of the output rows that map to these table rows, and writes out / arg_out directly.
// The key table must read as zero when the call starts and is put back to zero by the final kernel, so a
// caller that reuses its workspace pays for no initial fill: two launches in all.
// Both waits in the main kernel are bounded (a producer waiting for room in its queue, a consumer waiting for
// its producers): if one of them ever runs out, entries are lost, and the kernel says so in a word behind the key
// table (K1Plan::fail), which stays set until the caller clears it.
//
// Keys are those of scatter.h: order(value) << 32 | (0xFFFFFFFE - position), larger wins, so equal values
// keep the smallest position (csrc/cpu/reducer.h:63-67). A value that does not beat the initial value of the
// reduction (lowest() for max, max() for min) counts as no entry (csrc/cpu/scatter_cpu.cpp:81-82): the final
// kernel tests for it, since a table that starts at zero cannot.
#pragma once

namespace ts {

constexpr int kK1Rows = 8192;     // rows of a workgroup's table (64 KB of keys, 32 KB of tags)
constexpr int kK1Block = 1024;
constexpr int kK1Queues = 2;      // wavefronts of a workgroup that only issue atomics, one queue each
constexpr int kK1StreamWaves = kK1Block / kWave - kK1Queues;
constexpr int kK1QueueCap = 1024; // entries per queue (12 KB)
constexpr int kK1Depth = 3;       // batches of loads in flight per lane
constexpr int kK1Batch = kK1StreamWaves * kWave * 4;
constexpr int kK1Groups = 256;    // workgroups of the main kernel: one per CU
constexpr int kK1PerRow = 64;     // output rows that may share a table row: N <= kK1PerRow * kK1Rows
constexpr int kK1FinalRows = 16;  // table rows per workgroup of the final kernel
constexpr int kK1FinalBlock = 256;
constexpr int kK1Spin = 1 << 24;  // polls of a producer that waits for room in its queue (about a second)

struct K1Plan {
  bool ok;
  int G;               // workgroups of the main kernel (slabs)
  int J;               // output rows per table row
  int64_t epb;         // entries per workgroup, a multiple of four
  size_t bytes;        // workspace
  size_t zero_bytes;   // its leading part that must be zero before the call and is zero after it
  uint64_t *gkeys;     // [N]
  unsigned long long *fail;  // set (sticky) when a bounded wait of the main kernel ran out: entries were lost
  int spin;            // polls of a producer that waits for room in its queue
  uint64_t *slab_keys; // [G][kK1Rows]
  int32_t *slab_tags;  // [G][kK1Rows]
};

inline K1Plan k1_plan(int64_t B, int64_t E, int64_t K, int64_t N, int elem_bytes, void *ws, size_t ws_bytes,
                      bool any_size) {
  K1Plan p = {};
  if (B != 1 || K != 1 || elem_bytes != 4 || E < 1 || N < 1 || E >= 0xFFFFFFFEll ||
      N > (int64_t)kK1PerRow * kK1Rows || (!any_size && E < ((int64_t)1 << 14)))
    return p;
  int64_t G = (E + kK1Batch - 1) / kK1Batch;
  if (G > kK1Groups) G = kK1Groups;
  p.G = (int)G;
  p.J = (int)((N + kK1Rows - 1) / kK1Rows);
  p.epb = ((E + G - 1) / G + 3) & ~(int64_t)3;
  auto up = [](size_t x) { return (x + 255) & ~(size_t)255; };
  // The key table takes the room of the largest N this plan serves, whatever N is: a workspace kept from call
  // to call then has the same zero-on-entry part for every call, and the slabs of one call never land in what a
  // later call with more output rows reads as its (zero) key table.
  const size_t o_fail = up((size_t)kK1PerRow * kK1Rows * 8), o_keys = o_fail + 256;
  const size_t o_tags = o_keys + up((size_t)G * kK1Rows * 8);
  p.zero_bytes = o_keys;  // the key table and the word behind it
  p.spin = kK1Spin;
  if (const char *env = getenv("TS_K1_SPIN")) p.spin = atoi(env);  // test aid: 0 = a producer never waits
  p.bytes = o_tags + up((size_t)G * kK1Rows * 4);
  if (ws == nullptr || ws_bytes < p.bytes || (reinterpret_cast<uintptr_t>(ws) & 15) != 0) return p;
  p.gkeys = static_cast<uint64_t *>(ws);
  p.fail = reinterpret_cast<unsigned long long *>(static_cast<char *>(ws) + o_fail);
  p.slab_keys = reinterpret_cast<uint64_t *>(static_cast<char *>(ws) + o_keys);
  p.slab_tags = reinterpret_cast<int32_t *>(static_cast<char *>(ws) + o_tags);
  p.ok = true;
  return p;
}

template <typename T, bool IS_MAX>
__global__ __launch_bounds__(kK1Block) void scatter_k1_main_kernel(ScatterArgs a, K1Plan p) {
  static_assert(sizeof(T) == 4, "four entries per 16-byte load");
  typedef int64_t i64x2 __attribute__((ext_vector_type(2)));
  constexpr int D = kK1Depth;
  constexpr int mask = kK1Rows - 1;
  __shared__ uint64_t s_keys[kK1Rows];
  __shared__ int32_t s_tags[kK1Rows];
  __shared__ uint64_t s_qkey[kK1Queues][kK1QueueCap];
  __shared__ int32_t s_qnode[kK1Queues][kK1QueueCap];
  __shared__ int32_t s_tail[kK1Queues], s_head[kK1Queues];
  __shared__ int32_t s_done, s_fail;
  for (int i = threadIdx.x; i < kK1Rows; i += kK1Block) {
    s_keys[i] = 0;
    s_tags[i] = -1;
  }
  for (int i = threadIdx.x; i < kK1Queues * kK1QueueCap; i += kK1Block) (&s_qnode[0][0])[i] = -1;
  if (threadIdx.x < kK1Queues) { s_tail[threadIdx.x] = 0; s_head[threadIdx.x] = 0; }
  if (threadIdx.x == 0) { s_done = 0; s_fail = 0; }
  __syncthreads();

  const T *src = static_cast<const T *>(a.src);
  uint64_t *gkeys = p.gkeys;
  const int wave = threadIdx.x / kWave, lane = threadIdx.x & (kWave - 1);
  const int64_t total4 = a.E & ~(int64_t)3;  // entries covered in groups of four
  const int64_t lo = (int64_t)blockIdx.x * p.epb;
  const int64_t hi = lo + p.epb < total4 ? lo + p.epb : total4;
  const int n_batches = hi > lo ? (int)((hi - lo + kK1Batch - 1) / kK1Batch) : 0;

  if (wave < kK1StreamWaves) {
    // ---- streaming wavefronts: loads and LDS only, so that the loads of kK1Depth batches stay in flight
    i64x2 ia[D], ib[D];
    Vec<T, 4> xv[D];
    auto load = [&](int batch, int d) {
      int64_t e0 = lo + (int64_t)batch * kK1Batch + (int64_t)threadIdx.x * 4;
      if (e0 >= hi) e0 = lo;  // a lane without entries re-reads the chunk's first group (the result is not used)
      ia[d] = __builtin_nontemporal_load(reinterpret_cast<const i64x2 *>(a.index + e0));
      ib[d] = __builtin_nontemporal_load(reinterpret_cast<const i64x2 *>(a.index + e0) + 1);
      xv[d] = load_vec_stream<T, 4>(src + e0);
    };
    // an entry whose table row belongs to another node: handed to the wavefronts that issue the atomics
    const int q = wave % kK1Queues;
    auto push = [&](int node, uint64_t key) {
      const int slot = atomicAdd(&s_tail[q], 1);
      // the slot is free once the consumer has passed slot - cap; the consumer never waits for a producer
      int spin = 0;
      for (; slot - lds_peek(&s_head[q]) >= kK1QueueCap && spin < p.spin; ++spin) __builtin_amdgcn_s_sleep(2);
      // ran out: the store below overwrites an entry the consumer has not taken yet
      if (slot - lds_peek(&s_head[q]) >= kK1QueueCap) s_fail = 1;
      s_qkey[q][slot & (kK1QueueCap - 1)] = key;
      __hip_atomic_store(&s_qnode[q][slot & (kK1QueueCap - 1)], node, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_WORKGROUP);
    };
    auto process = [&](int batch, int d) {
      const int64_t e0 = lo + (int64_t)batch * kK1Batch + (int64_t)threadIdx.x * 4;
      const bool live = e0 < hi;
      const int64_t idx[4] = {ia[d].x, ia[d].y, ib[d].x, ib[d].y};
      int node[4], tag[4];
      uint32_t kv[4], cur_hi[4];
#pragma unroll
      for (int u = 0; u < 4; ++u) {
        const bool ok = live && idx[u] >= 0 && idx[u] < a.N && !Key<T>::is_nan(xv[d].v[u]);  // NaN never wins
        node[u] = ok ? (int)idx[u] : -1;
        kv[u] = Key<T>::enc(xv[d].v[u]);
        if (!IS_MAX) kv[u] = ~kv[u];
      }
#pragma unroll
      for (int u = 0; u < 4; ++u) {
        const int row = node[u] & mask;
        tag[u] = lds_peek(&s_tags[row]);
        cur_hi[u] = lds_peek(reinterpret_cast<const uint32_t *>(&s_keys[row]) + 1);
      }
#pragma unroll
      for (int u = 0; u < 4; ++u) {
        if (node[u] < 0) continue;
        const int row = node[u] & mask;
        if (tag[u] == -1) {
          const int old = atomicCAS(&s_tags[row], -1, node[u]);
          tag[u] = old == -1 ? node[u] : old;
        }
        if (tag[u] == node[u] && kv[u] < cur_hi[u]) continue;  // below the cached value: cannot win
        const uint64_t key = ((uint64_t)kv[u] << 32) | (0xFFFFFFFEu - (uint32_t)(e0 + u));
        if (tag[u] == node[u])
          __hip_atomic_fetch_max(&s_keys[row], key, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_WORKGROUP);
        else
          push(node[u], key);
      }
    };
    // every load is issued unconditionally (batches past the end repeat the last one): only then does the
    // compiler know how many loads are in flight at each use and wait for just the oldest
    if (n_batches > 0) {
#pragma unroll
      for (int d = 0; d < D; ++d) load(d < n_batches ? d : n_batches - 1, d);
      for (int batch = 0; batch < n_batches; batch += D) {
#pragma unroll
        for (int d = 0; d < D; ++d) {
          if (batch + d < n_batches) process(batch + d, d);  // uniform over the workgroup
          load(batch + d + D < n_batches ? batch + d + D : n_batches - 1, d);
        }
      }
    }
    // the last E % 4 entries
    if (blockIdx.x == gridDim.x - 1 && (int64_t)threadIdx.x < a.E - total4) {
      const int64_t e = total4 + threadIdx.x;
      const int64_t idx = a.index[e];
      const T x = src[e];
      if (idx >= 0 && idx < a.N && !Key<T>::is_nan(x)) push((int)idx, pack_key<T, IS_MAX>(x, 0xFFFFFFFEu - (uint32_t)e));
    }
    if (lane == 0) atomicAdd(&s_done, 1);  // after this wavefront's last push
  } else {
    // ---- the wavefronts that issue the atomics: one queue each, entries taken in order
    const int q = wave - kK1StreamWaves;
    int head = 0, idle = 0;
    for (; idle < (1 << 26);) {
      const int at = (head + lane) & (kK1QueueCap - 1);
      const int node = lds_peek(&s_qnode[q][at]);
      const uint64_t ready = __ballot(node != -1);
      const int cnt = ready == ~(uint64_t)0 ? kWave : __ffsll((unsigned long long)~ready) - 1;  // leading run
      if (cnt == 0) {
        if (lds_peek(&s_done) == kK1StreamWaves && head == lds_peek(&s_tail[q])) break;
        __builtin_amdgcn_s_sleep(4);
        ++idle;
        continue;
      }
      if (lane < cnt) {
        const uint64_t key = s_qkey[q][at];
        __hip_atomic_fetch_max(gkeys + node, key, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
        __hip_atomic_store(&s_qnode[q][at], -1, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_WORKGROUP);
      }
      head += cnt;
      if (lane == 0) __hip_atomic_store(&s_head[q], head, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_WORKGROUP);
    }
    if (idle >= (1 << 26)) s_fail = 1;  // left with entries still queued
  }
  __syncthreads();
  if (threadIdx.x == 0 && s_fail != 0)
    __hip_atomic_fetch_or(p.fail, 1ull, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
  uint64_t *sk = p.slab_keys + (int64_t)blockIdx.x * kK1Rows;
  int32_t *st = p.slab_tags + (int64_t)blockIdx.x * kK1Rows;
  for (int i = threadIdx.x; i < kK1Rows; i += kK1Block) {
    sk[i] = s_keys[i];
    st[i] = s_tags[i];
  }
}

template <typename T, bool IS_MAX>
__global__ __launch_bounds__(kK1FinalBlock) void scatter_k1_final_kernel(ScatterArgs a, K1Plan p) {
  constexpr int RB = kK1FinalRows;
  constexpr int WG = kK1FinalBlock / RB;  // groups of slabs
  __shared__ uint64_t s_slot[RB * kK1PerRow];
  const int J = p.J;
  for (int i = threadIdx.x; i < RB * J; i += kK1FinalBlock) s_slot[i] = 0;
  __syncthreads();
  const int r0 = blockIdx.x * RB;
  const int rl = threadIdx.x % RB;
  const int wg = threadIdx.x / RB;
  {
    int cur_tag = -1;
    uint64_t cur_key = 0;
    auto flush = [&]() {
      if (cur_tag >= 0)
        __hip_atomic_fetch_max(&s_slot[rl * J + cur_tag / kK1Rows], cur_key, __ATOMIC_RELAXED,
                               __HIP_MEMORY_SCOPE_WORKGROUP);
    };
    constexpr int U = 8;
    for (int w0 = wg; w0 < p.G; w0 += WG * U) {
      uint64_t k[U];
      int32_t t[U];
#pragma unroll
      for (int u = 0; u < U; ++u) {
        const int w = w0 + u * WG;
        const int64_t at = (int64_t)(w < p.G ? w : w0) * kK1Rows + r0 + rl;
        k[u] = p.slab_keys[at];
        t[u] = p.slab_tags[at];
      }
#pragma unroll
      for (int u = 0; u < U; ++u) {
        if (w0 + u * WG >= p.G || k[u] == 0) continue;
        if (t[u] == cur_tag) {
          cur_key = k[u] > cur_key ? k[u] : cur_key;
        } else {
          flush();
          cur_tag = t[u];
          cur_key = k[u];
        }
      }
    }
    flush();
  }
  __syncthreads();
  const T *src = static_cast<const T *>(a.src);
  T *out = static_cast<T *>(a.out);
  // a value part at or below this one did not beat the initial value of the reduction
  uint32_t lim = Key<T>::enc(IS_MAX ? ElemLim<T>::lowest() : ElemLim<T>::max());
  if (!IS_MAX) lim = ~lim;
  for (int i = threadIdx.x; i < RB * J; i += kK1FinalBlock) {
    const int j = i / RB, r = i - j * RB;  // neighbouring lanes: neighbouring output rows
    const int64_t n = (int64_t)j * kK1Rows + r0 + r;
    if (n >= a.N) continue;
    uint64_t key = s_slot[r * J + j];
    const uint64_t mem = p.gkeys[n];
    if (mem != 0) p.gkeys[n] = 0;  // the table is handed back as it was found
    key = mem > key ? mem : key;
    const uint32_t kv = (uint32_t)(key >> 32);
    if (key == 0 || kv <= lim) {
      out[n] = zero_elem<T>();
      a.arg_out[n] = a.E;
    } else {
      const int64_t e = (int64_t)(0xFFFFFFFEu - (uint32_t)key);
      const uint32_t k = IS_MAX ? kv : ~kv;
      T val = Key<T>::dec(k);
      if (Key<T>::kFloat && k == 0x80000000u) val = src[e];  // a zero: keep the sign bit of the winning entry
      out[n] = val;
      a.arg_out[n] = e;
    }
  }
}

template <typename T, bool IS_MAX>
void launch_scatter_k1(const ScatterArgs &a, const K1Plan &p, hipStream_t stream) {
  hipLaunchKernelGGL((scatter_k1_main_kernel<T, IS_MAX>), dim3((unsigned)p.G), dim3(kK1Block), 0, stream, a, p);
  hipLaunchKernelGGL((scatter_k1_final_kernel<T, IS_MAX>), dim3(kK1Rows / kK1FinalRows), dim3(kK1FinalBlock), 0, stream,
                     a, p);
}

}  // namespace ts
