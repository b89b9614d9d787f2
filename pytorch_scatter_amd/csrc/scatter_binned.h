// scatter min / max / sum for wide rows through buckets of output rows (included by scatter.h).
//
// The packed-key table of one workgroup (scatter_key_lds_kernel) holds 128 rows of 32 keys; with a heavy-tailed
// index a quarter of the entries miss it and go to the table in memory one 256-byte row at a time. Here the
// entries are first binned by bucket of R consecutive output rows, R * K keys = 64 KB of LDS, so that a
// workgroup which reduces (a chunk of) one bucket holds every row it can meet: no misses, no tags, and the
// only traffic besides the stream is the table written back once per chunk.
//   count  : at most 512 workgroups with equal shares of the index, each a histogram over the buckets in LDS that
//            it adds to the bucket totals (also: is the index in order?)
//   scan   : bucket starts, chunks per bucket, the (bucket, chunk) of every reducing workgroup
//   place  : a workgroup per tile of the index: its own histogram again, one atomic per bucket reserves the tile's
//            run of slots, every entry -> (row inside its bucket, entry number) in its run (8 bytes)
//   reduce : a workgroup per chunk of a bucket: rows of src by entry number, packed keys into the LDS table,
//            table -> global table with a read before each atomic
// The order inside a bucket is whatever the placement gives; the packed keys carry the positions, so the result
// (value, first position among equal values) does not depend on it. Sums use the same passes with a table of
// accumulators (bin_add_wave_kernel) unless the count pass finds the index sorted.
#pragma once

namespace ts {

constexpr int kBinKeys = 8192;        // keys of the LDS table: 64 KB, two workgroups per CU
constexpr int kBinBlock = 1024;
constexpr int kBinMaxBuckets = 16384;  // LDS histogram of count / place (their LDS is sized for 8192 or 16384 buckets)
constexpr int kBinSmallCap = 8192;
constexpr int kBinChunk = 8192;       // entries per chunk of a bucket in reduce (fewer for inputs under 4 M entries)
constexpr int kBinPlaceChunk = 10240;  // most entries per workgroup in place: one batch of 10 per lane
constexpr int kCombPos = 64;          // combining kernel: keys per step of a bucket of many chunks,
constexpr int kCombFew = 32;          // many: more than this
constexpr int kBinCountShift = 10;   // rows per bucket (log2) up to which bin_add_wave_kernel can count entries per row as well
constexpr int kBinPlaceBlock = 1024;   // (measured slower: 256 lanes x 4 batches, 64 K entries per workgroup, 8 K)

// 4-byte values per entry that travel with their bucket (bin_plan_payload): one value in an 8-byte word, several in a
// record of K + 1 32-bit words (the values, then the row in the bucket)
constexpr int kBinPayloadCols = 4;

struct BinArgs {
  int rshift;              // log2 of the rows per bucket
  int kc;                  // columns of a row that one reducing workgroup holds in LDS (K when slices == 1)
  int slices;              // K / kc: reducing workgroups per chunk, each on its own columns of the same entries
  int chunk;               // entries per reducing workgroup
  int nb;                  // buckets
  int place_tile;          // entries per workgroup of place: a multiple of 1024, one batch at most
  int64_t n_place;         // workgroups of place
  int64_t max_wgs;         // workgroups of reduce (upper bound of the chunks)
  unsigned long long *totals;  // [nb] entries per bucket
  unsigned long long *cursor;  // [nb] next free slot
  int64_t *starts;         // [nb + 1]
  int32_t *chunk_start;    // [nb + 1]
  int32_t *wg_bucket;      // [max_wgs] bucket of a reducing workgroup, -1: none
  uint64_t *binned;        // [B * E] (row in bucket << 32) | entry number
  int32_t *slab_start;     // min / max: [nb + 1] first slab of a bucket that is reduced in more than one chunk
  uint64_t *slabs;         // min / max: [slab][K << rshift] the tables of those chunks
  int32_t *comb_list;      // min / max: buckets that the combining kernel finishes (not exactly one chunk): those of
                           //            up to kCombFew chunks from the front, those of more from slot nb - 1 down
  int32_t *comb_count;     //            how many of either

  int *unsorted;           // sum only (else null): 1 = the buckets take the call (set by the count pass or by a sample when
                           // the index is not sorted); 0 = sorted, 2 = (single values only) unsorted but skewed: both
                           // leave the call to other kernels, and every pass of the buckets returns at once;
                           // a sorted index is left to the kernels that combine runs, and the passes after
                           // the count return at once
  int strict = 0;          // the count pass also reports an index outside [0, N) as unsorted (a caller that hands a
                           // sorted index to the segmented reduction needs both)
  int sampled = 0;         // sum only: *unsorted was set before the count pass from a sample of the index
                           // (bin_sample_kernel); then the count pass returns at once as well
  int payload = 0;         // sum of one 4-byte value per entry: the low half of a binned word holds the value's bits
                           // instead of the entry number, so the reducing pass never goes back to src
  int planes = 1;          // ... of `planes` 4-byte values per entry (rows of up to 16 bytes); more than one: binned holds
                           // records of planes + 1 32-bit words, the values and then the row in the bucket
  int sort_tile = 6144;    // entries per workgroup of the place pass that sorts its tile in LDS (records: fewer)
  int32_t *count_out = nullptr;  // sums: the adding pass also counts the entries of every output row into this
                           // [B * N] array (the divisor of a mean, from the same words); row buckets: rshift <= kBinCountShift
};

struct BinPlan {
  bool ok;
  BinArgs p;
  size_t bytes;
};

// slot_bytes: size of a table slot (8: packed keys of min / max, 4 or 8: accumulators of a sum)
// slabs: min / max (workspace for the tables of chunks); whole_pow2: see below
inline BinPlan bin_plan(int64_t B, int64_t E, int64_t K, int64_t N, int elem_bytes, void *ws, size_t ws_bytes,
                        bool any_size = false, int slot_bytes = 8, bool slabs = false, bool whole_pow2 = false) {
  BinPlan r;
  r.ok = false;
  r.bytes = 0;
  const int64_t n_edges = B * E, rows = B * N;
  // Rows of 64 bytes and more. Sums from 64 MB of input (below, the five extra launches cost more than the misses:
  // Zipf(1.2) / uniform index onto 100 k rows of 32 floats, 64 MB: 72 / 91 us with the buckets, and the table of
  // scatter_add_lds_kernel takes the sizes below), and with two entries per output row: every bucket is flushed
  // whatever it received (96 MB / 256 MB of 32 ... 128 floats per entry onto 1 M rows, uniform index: 155 / 224,
  // 237 / 332, 379 / 513 us with the buckets, 104 / 248, 126 / 274, 175 / 314 us without) -- up to 300 MB, where the
  // table of scatter_add_lds_kernel stops taking wide rows and the buckets are the path that a hub cannot hurt
  // (1 GB of 128 floats per entry, one entry per row, Zipf(1.2): 607 us with the buckets, 1226 us without).
  // min / max: the other path fills a table of 8-byte keys as large as out and walks it once more at the end, so
  // the crossover moves with that table (uniform index, us without / with the buckets):
  //   keys of 2.5 MB (10 k rows of 32 floats):  16 MB 30 / 57, 48 MB 90 / 92, 64 MB 98 / 96
  //   keys of 10 - 25 MB:                        16 MB 39 / 54 and 48 / 49, 24 MB 56 / 55 and 65 / 52, 48 MB 93 / 60
  //   keys of 256 MB and 1 GB (1 M rows):        4 MB 159 / 122 and 777 / 562, 64 MB 256 / 184 and 842 / 514
  // (a Zipf(1.2) index gains earlier: keys of 25 MB, 8 MB of input: 64 / 49 us)
  const int64_t key_bytes = rows * K * 8;
  const int64_t minmax_bytes = key_bytes >= ((int64_t)256 << 20) ? ((int64_t)1 << 20)
                               : key_bytes >= ((int64_t)8 << 20) ? ((int64_t)24 << 20) : ((int64_t)64 << 20);
  const int64_t min_bytes = slabs ? minmax_bytes : ((int64_t)64 << 20);
  if (K * elem_bytes < 64 || (!any_size && n_edges * K * elem_bytes < min_bytes) ||
      (!any_size && !slabs && n_edges < 2 * rows && n_edges * K * elem_bytes < (int64_t)300000000) ||
      n_edges >= 0xFFFFFFFEll || rows >= 0x7FFFFFFFll || rows < 1)
    return r;
  const int64_t slots = (int64_t)kBinKeys * 8 / slot_bytes;
  // The LDS table holds R rows of kc columns, R * kc = slots. Rows that are too wide for a bucket count within
  // the histograms of count / place (K = 128 floats onto 1.5 M rows: 64 rows per bucket, 23 k buckets) are cut
  // into slices of kc columns: a bucket keeps more rows, and K / kc workgroups reduce each of its chunks, every
  // one on its own columns of the same entries. Slices are 1024 ... 64 bytes wide, the widest that fits.
  auto shift_for = [&](int64_t kc) {
    int rs = 0;
    while (((int64_t)2 << rs) * kc <= slots) ++rs;
    return rs;
  };
  auto fits = [&](int64_t kc) {
    const int rs = shift_for(kc);
    return kc <= kBinKeys / 16 && ((int64_t)1 << rs) <= slots / 16 &&  // the padding holds one slot per row
           ((rows + ((int64_t)1 << rs) - 1) >> rs) <= kBinMaxBuckets;
  };
  // whole_pow2 (sums, which have the wavefront kernel only): a row is kept whole only if 1 ... 64 lanes with 16 bytes
  // each hold it, a power of two of them
  const int64_t lanes = K * elem_bytes / 16;
  const bool whole_ok = !whole_pow2 || (K * elem_bytes % 16 == 0 && lanes <= 64 && (lanes & (lanes - 1)) == 0);
  int64_t kc = K;
  if (!whole_ok || !fits(K)) {
    kc = 0;
    for (int64_t bytes = 1024; bytes >= 64 && kc == 0; bytes >>= 1) {
      const int64_t c = bytes / elem_bytes;
      if (c < K && K % c == 0 && fits(c)) kc = c;
    }
    if (kc == 0) return r;
  }
  const int rshift = shift_for(kc);
  const int64_t nb = (rows + ((int64_t)1 << rshift) - 1) >> rshift;
  BinArgs &p = r.p;
  p.rshift = rshift;
  p.kc = (int)kc;
  p.slices = (int)(K / kc);
  p.nb = (int)nb;
  // Place: a workgroup holds its tile in registers (up to 16 entries per lane). Two workgroups fit a CU, so the
  // tiles are sized for a whole number of rounds of 512 workgroups (10 M entries in tiles of 16384: 611 workgroups,
  // a round of 512 and a round of 99 that takes as long).
  {
    const int64_t rounds = (n_edges + (int64_t)512 * kBinPlaceChunk - 1) / ((int64_t)512 * kBinPlaceChunk);
    int64_t tile = (((n_edges + 512 * rounds - 1) / (512 * rounds)) + kBinPlaceBlock - 1) & ~(int64_t)(kBinPlaceBlock - 1);
    if (const char *env = getenv("TS_BIN_PLACE_TILE")) tile = atoi(env);  // tuning aid
    if (tile < kBinPlaceBlock) tile = kBinPlaceBlock;
    if (tile > kBinPlaceChunk) tile = kBinPlaceChunk;
    tile &= ~(int64_t)(kBinPlaceBlock - 1);
    p.place_tile = (int)tile;
    p.n_place = (n_edges + tile - 1) / tile;
  }
  // A reducing workgroup walks its chunk in steps of a few rows per lane group, each step a memory latency:
  // 8 K entries take it about 200 us whatever the input, which is fine once there are a few workgroups per CU
  // (4 M entries and more) and far too long for a smaller input. Those get shorter chunks: about 512 workgroups.
  int64_t chunk = kBinChunk;
  if (const char *env = getenv("TS_BIN_CHUNK")) chunk = atoi(env);  // tuning aid
  if (n_edges < (int64_t)512 * kBinChunk) {
    chunk = (n_edges / 512 + 63) & ~(int64_t)63;
    if (chunk < 1024) chunk = 1024;
    // a bucket of average size in one chunk: a bucket cut into several chunks hands a whole table per chunk to the
    // combining kernel, whatever the chunk's size (524 k entries over 391 buckets in chunks of 1024: 324 us, 50 MB of slabs)
    const int64_t twice_avg = (2 * n_edges / nb + 63) & ~(int64_t)63;
    if (slabs && chunk < twice_avg) chunk = twice_avg < kBinChunk ? twice_avg : kBinChunk;
  }
  p.chunk = (int)chunk;
  p.max_wgs = n_edges / chunk + nb + 1;
  auto up = [](size_t x) { return (x + 255) & ~(size_t)255; };
  size_t off = 0;
  auto take = [&](size_t bytes) { const size_t o = off; off += up(bytes); return o; };
  const size_t o_tot = take((size_t)nb * 8), o_cur = take((size_t)nb * 8), o_st = take((size_t)(nb + 1) * 8);
  const size_t o_cs = take((size_t)(nb + 1) * 4), o_wb = take((size_t)p.max_wgs * 4);
  const size_t o_bin = take((size_t)n_edges * 8), o_flag = take(256);
  // A bucket with m >= 2 chunks holds more than (m - 1) * chunk entries: at most 2 * n_edges / chunk slabs in all.
  const int64_t n_slabs = slabs ? 2 * (n_edges / chunk) + 2 : 0;
  const size_t o_ss = take(slabs ? (size_t)(nb + 1) * 4 : 0), o_cl = take(slabs ? (size_t)(nb + 2) * 4 : 0);
  const size_t o_sl = take((size_t)n_slabs * ((size_t)K << rshift) * 8);
  r.bytes = off;
  if (ws == nullptr || ws_bytes < off || (reinterpret_cast<uintptr_t>(ws) & 15) != 0) return r;
  char *base = static_cast<char *>(ws);
  p.totals = reinterpret_cast<unsigned long long *>(base + o_tot);
  p.cursor = reinterpret_cast<unsigned long long *>(base + o_cur);
  p.starts = reinterpret_cast<int64_t *>(base + o_st);
  p.chunk_start = reinterpret_cast<int32_t *>(base + o_cs);
  p.wg_bucket = reinterpret_cast<int32_t *>(base + o_wb);
  p.binned = reinterpret_cast<uint64_t *>(base + o_bin);
  p.unsorted = reinterpret_cast<int *>(base + o_flag);  // callers that do not want the check set it to null
  p.slab_start = slabs ? reinterpret_cast<int32_t *>(base + o_ss) : nullptr;
  p.comb_list = slabs ? reinterpret_cast<int32_t *>(base + o_cl) : nullptr;
  p.comb_count = slabs ? p.comb_list + nb : nullptr;
  p.slabs = slabs ? reinterpret_cast<uint64_t *>(base + o_sl) : nullptr;
  r.ok = true;
  return r;
}

// Sums of ONE 4-byte value per entry (K == 1: degrees, edge weights, attention scores) under an unsorted index.
// The kernels without workspace pay one device atomic per entry that misses their LDS table (about 21 G entries/s
// whatever is done: 46 M entries onto 1 M rows 2.2 ms). Here the value travels with its bucket: the place pass writes
// (row in bucket, value) words, and the reducing pass streams the words of a bucket's chunk, adds them in an LDS
// table of the bucket's rows and adds every touched row to out once per chunk. Traffic per entry: 8 bytes of index
// twice, 4 of src, 8 written and 8 read again, against one scattered atomic. Buckets are small (64 ... 4096 rows,
// at most a sixteenth of a chunk) so that the write-back stays below a sixteenth of the entries.
inline BinPlan bin_plan_payload(int64_t B, int64_t E, int64_t K, int64_t N, int elem_bytes, void *ws, size_t ws_bytes,
                                bool any_size = false) {
  BinPlan r;
  r.ok = false;
  r.bytes = 0;
  const int64_t n_edges = B * E, rows = B * N;
  if (K < 1 || K > kBinPayloadCols || elem_bytes != 4 || n_edges >= 0xFFFFFFFEll || rows >= 0x7FFFFFFFll || rows < 1) return r;
  if (K > 1 && n_edges * (K + 1) >= 0xFFFFFFFEll) return r;
  // from 2 M entries: an even index gains from there on (74 against 106 us; 2.3 M entries of a graph in random order
  // 85 against 125 us); a skewed one, which the sample hands to the table kernel, pays about 15 us for the launches
  // that return at once (2.3 M entries: 51 against 36 us)
  // (several values per entry: the place pass grows with them, the atomics they replace do not -- three values from
  // 3 M entries, four from 4 M: 2.2 M / 3 M entries of four floats 121 / 149 us against 115 / 155 us)
  if (!any_size && n_edges < (K <= 2 ? (int64_t)1 << 21 : K == 3 ? (int64_t)3 << 20 : (int64_t)1 << 22)) return r;
  // chunk: entries per reducing workgroup, about 1024 workgroups, 2048 ... 65536 entries
  int64_t chunk = (n_edges / 1024 + 1023) & ~(int64_t)1023;
  if (chunk < 2048) chunk = 2048;
  if (chunk > 65536) chunk = 65536;
  if (const char *env = getenv("TS_BIN_CHUNK")) chunk = atoi(env) > 0 ? atoi(env) : chunk;  // tuning aid
  // rows per bucket: as many as the table holds (4096). Fewer, larger buckets make the place pass cheaper (21 M entries:
  // 256 rows 580 us, 1024 rows 494, 4096 rows 393 for the whole call), which outweighs the longer write-back per chunk.
  // (K values per entry: the table's 4096 slots hold 4096 / K rows, rounded down to a power of two)
  int top = 12;
  while (((int64_t)K << top) > 4096) --top;
  int rshift = top;
  if (const char *env = getenv("TS_BIN_PAYLOAD_RSHIFT")) rshift = atoi(env);  // tuning aid
  while (rshift < top && ((rows + ((int64_t)1 << rshift) - 1) >> rshift) > kBinMaxBuckets) ++rshift;
  if (rshift > top) rshift = top;
  if (rshift < 0) rshift = 0;
  const int64_t nb = (rows + ((int64_t)1 << rshift) - 1) >> rshift;
  if (nb > kBinMaxBuckets) return r;                       // more output rows than 16384 buckets of 4096 hold
  if (K > 1 && nb > 2048) return r;                        // records are placed by the pass that sorts its tile only
  if (!any_size && n_edges < 2 * nb * 64) return r;        // nearly empty buckets: every one still costs its share
  BinArgs &p = r.p;
  p.rshift = rshift;
  p.kc = 1;
  p.slices = 1;
  p.nb = (int)nb;
  p.payload = 1;
  p.planes = (int)K;
  // records: as many entries per tile as the 48 KB stage holds, in whole rounds of the workgroup
  if (K > 1) p.sort_tile = (int)(12288 / (K + 1) / kBinPlaceBlock) * kBinPlaceBlock;
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
  auto up = [](size_t x) { return (x + 255) & ~(size_t)255; };
  size_t off = 0;
  auto take = [&](size_t bytes) { const size_t o = off; off += up(bytes); return o; };
  const size_t o_tot = take((size_t)nb * 8), o_cur = take((size_t)nb * 8), o_st = take((size_t)(nb + 1) * 8);
  const size_t o_cs = take((size_t)(nb + 1) * 4), o_wb = take((size_t)p.max_wgs * 4);
  const size_t o_bin = take(K > 1 ? (size_t)n_edges * 4 * (size_t)(K + 1) : (size_t)n_edges * 8), o_flag = take(256);
  r.bytes = off;
  if (ws == nullptr || ws_bytes < off || (reinterpret_cast<uintptr_t>(ws) & 15) != 0) return r;
  char *base = static_cast<char *>(ws);
  p.totals = reinterpret_cast<unsigned long long *>(base + o_tot);
  p.cursor = reinterpret_cast<unsigned long long *>(base + o_cur);
  p.starts = reinterpret_cast<int64_t *>(base + o_st);
  p.chunk_start = reinterpret_cast<int32_t *>(base + o_cs);
  p.wg_bucket = reinterpret_cast<int32_t *>(base + o_wb);
  p.binned = reinterpret_cast<uint64_t *>(base + o_bin);
  p.unsorted = reinterpret_cast<int *>(base + o_flag);
  p.slab_start = nullptr;
  p.comb_list = nullptr;
  p.comb_count = nullptr;
  p.slabs = nullptr;
  r.ok = true;
  return r;
}

// node (b * N + index) of entry be, -1 for an index outside [0, N)
__device__ __forceinline__ int64_t bin_node(const ScatterArgs &a, int64_t be) {
  int64_t b = 0, e = be;
  if (a.B > 1) { b = be / a.E; e = be - b * a.E; }
  const int64_t idx = a.index[b * a.sb + e * a.se];
  return (idx >= 0 && idx < a.N) ? b * a.N + idx : -1;
}

constexpr int kBinPer = 10;  // entries per lane in place (all index loads in flight; three words per entry stay in
                             // registers: with 16 the kernel needs 91 VGPRs, which is one workgroup per CU instead of two)
constexpr int kBinBatch = kBinPer * kBinPlaceBlock;

// total of the per-wavefront sums of a workgroup scan (valid entries of a tile)
__device__ __forceinline__ int run_total(const int32_t *wsum) {
  int t = 0;
#pragma unroll
  for (int w = 0; w < kBinPlaceBlock / kWave; ++w) t += wsum[w];
  return t;
}

// buckets of the kBinPer entries of a lane, all index loads in flight at once; -1: no bucket
// check: descent is set when an entry's node lies below that of the entry before it. The entry before is the
// neighbouring lane's (a shuffle); only the first lane of a wavefront loads it.
__device__ __forceinline__ void bin_buckets(const ScatterArgs &a, const BinArgs &p, int64_t lo, int64_t hi,
                                            int32_t *bucket, int32_t *local, bool check, bool &descent,
                                            bool strict = false) {
  int64_t node[kBinPer];
#pragma unroll
  for (int j = 0; j < kBinPer; ++j) {
    const int64_t be = lo + threadIdx.x + (int64_t)j * kBinPlaceBlock;
    node[j] = be < hi ? bin_node(a, be) : -1;
  }
  if (check) {
    // The entry before a lane's entry is the neighbouring lane's (a shuffle); the first lane of a wavefront needs the
    // entry before the wavefront's first one. One load instruction fetches those of all kBinPer rows: lane j
    // loads the entry in front of row j.
    const int lane = threadIdx.x & (kWave - 1);
    int64_t edge = -1;
    if (lane < kBinPer) {
      const int64_t be = lo + (int64_t)(threadIdx.x - lane) + (int64_t)lane * kBinPlaceBlock;
      if (be > 0 && be < hi) edge = bin_node(a, be - 1);
    }
#pragma unroll
    for (int j = 0; j < kBinPer; ++j) {
      const int elo = __builtin_amdgcn_readlane((int)(uint32_t)edge, j), ehi = __builtin_amdgcn_readlane((int)(edge >> 32), j);
      const int64_t up = lane_up1_64(node[j]);  // by every lane: lane 0's value is what lane 1 reads
      const int64_t prev = lane == 0 ? (int64_t)(((uint64_t)(uint32_t)ehi << 32) | (uint32_t)elo) : up;
      descent = descent || (node[j] >= 0 && prev >= 0 && node[j] < prev);
      if (strict && node[j] < 0 && lo + threadIdx.x + (int64_t)j * kBinPlaceBlock < hi) descent = true;
    }
  }
#pragma unroll
  for (int j = 0; j < kBinPer; ++j) {
    bucket[j] = node[j] >= 0 ? (int32_t)(node[j] >> p.rshift) : -1;
    if (local != nullptr) local[j] = (int32_t)(node[j] & (((int64_t)1 << p.rshift) - 1));
  }
}

// Adds 1 to counter[bucket] for every lane with bucket >= 0 and returns the value before the lane's own
// addition. Twice over, the lanes that share the bucket of the first lane still waiting go through one atomic
// of their leader (with a heavy-tailed index nearly all lanes: the bucket of the hubs, which would otherwise
// queue up on one LDS address); whoever is left adds on its own.
__device__ __forceinline__ int32_t bin_take(int32_t *counter, int32_t bucket) {
  int32_t before = 0;
  bool waiting = bucket >= 0;
#pragma unroll
  for (int round = 0; round < 2; ++round) {
    const uint64_t todo = __ballot(waiting);
    if (todo == 0) break;
    // head and first are the same for the whole wavefront: scalar registers, v_readlane instead of a shuffle
    const int head = __builtin_ctzll((unsigned long long)todo);
    const int32_t first = __builtin_amdgcn_readlane(bucket, head);
    const bool with_head = waiting && bucket == first;
    const uint64_t same = __ballot(with_head);
    // lanes of `same` below this one (v_mbcnt): the head's is 0
    const int32_t below = (int32_t)__builtin_amdgcn_mbcnt_hi((uint32_t)(same >> 32),
                                                             __builtin_amdgcn_mbcnt_lo((uint32_t)same, 0u));
    int32_t base = 0;
    if (with_head && below == 0) base = atomicAdd(&counter[first], __popcll(same));
    base = __builtin_amdgcn_readlane(base, head);
    if (with_head) {
      before = base + below;
      waiting = false;
    }
  }
  if (waiting) before = atomicAdd(&counter[bucket], 1);
  return before;
}

// Does the index look sorted? Sums of a sorted (or nearly sorted) index are left to the kernels that combine
// runs, and finding that out with the full count pass costs 60-150 us for 10 M entries. It is a question of speed
// only (both paths are correct for any index), so a sample answers it: 1024 evenly spaced entries and their right
// neighbours, *flag = 1 (not sorted) if at least 1/64 of the pairs descend.
// (totals: the buckets' counts [nb], cleared here on the way, which saves their own launch; null: none)
static __global__ __launch_bounds__(kBinBlock) void bin_sample_kernel(ScatterArgs a, int *flag,
                                                                      unsigned long long *totals = nullptr, int nb = 0) {
  __shared__ int s_desc;
  for (int i = threadIdx.x; i < nb; i += kBinBlock) totals[i] = 0;
  if (threadIdx.x == 0) s_desc = 0;
  __syncthreads();
  const int64_t n = a.B * a.E;  // the host launches this only with n >= 2 * kBinBlock
  const int64_t be = (int64_t)threadIdx.x * (n / kBinBlock);
  const int64_t b = be / a.E, e = be - b * a.E;
  const int64_t b1 = (be + 1) / a.E, e1 = be + 1 - b1 * a.E;
  const int64_t idx = a.index[b * a.sb + e * a.se];
  const int64_t nxt = a.index[b1 * a.sb + e1 * a.se];
  if (b1 == b && nxt < idx) atomicAdd(&s_desc, 1);
  __syncthreads();
  if (threadIdx.x == 0) *flag = s_desc * 64 >= kBinBlock ? 1 : 0;
}

// The same sample for sums of single values, with a third answer. The buckets pay for an index that spreads evenly
// over the output rows (8 M entries onto 1 M rows, uniform: 126 us against 409 us through the table kernel); under a
// skewed index the table kernel's hot rows absorb most entries and it wins (Zipf(1.5): 56 against 165 us). So the
// sample also counts how many of its 1024 entries name a row that an earlier one named (a hash set in LDS):
// *flag = 0 sorted-looking, 2 not sorted and at least three quarters repeat (the table kernel), 1 else (buckets).
// (Around two thirds -- a Zipf(1.2) index -- the two are level from 8 M entries: 8-10 M onto 1 M rows 152-160 us
// through the buckets and 106-195 us through the table, by where the hot rows lie; at 86 %, Zipf(1.5), the table takes
// 56 us. Below 8 M entries the table is sometimes ahead at two thirds -- Zipf(1.2), 64 % repeats, 2.2 / 4.3 M entries
// onto 270 k rows: 51 / 89 us against 77 / 101 us through the buckets -- and sometimes far behind: the same onto 1 M
// rows 141 / 79 us against 80 / 106 us. A bar of one half below 8 M entries was measured and lost more than it won, the
// launches that return included; the buckets' time does not depend on where the hot rows lie.)
// (quarters: the bar in quarters of the sample. Several values per entry: one half, since the buckets' time grows with
// the values per entry and the table's does not.)
static __global__ __launch_bounds__(kBinBlock) void bin_sample_skew_kernel(ScatterArgs a, int *flag, int quarters,
                                                                           unsigned long long *totals, int nb) {
  constexpr int kSlots = 2048;
  __shared__ int s_set[kSlots];
  __shared__ int s_desc, s_dup;
  for (int i = threadIdx.x; i < nb; i += kBinBlock) totals[i] = 0;  // (the buckets' counts, cleared on the way)
  for (int i = threadIdx.x; i < kSlots; i += kBinBlock) s_set[i] = -1;
  if (threadIdx.x == 0) { s_desc = 0; s_dup = 0; }
  __syncthreads();
  const int64_t n = a.B * a.E;  // the host launches this only with n >= 2 * kBinBlock
  const int64_t be = (int64_t)threadIdx.x * (n / kBinBlock);
  const int64_t b = be / a.E, e = be - b * a.E;
  const int64_t b1 = (be + 1) / a.E, e1 = be + 1 - b1 * a.E;
  const int64_t idx = a.index[b * a.sb + e * a.se];
  const int64_t nxt = a.index[b1 * a.sb + e1 * a.se];
  if (b1 == b && nxt < idx) atomicAdd(&s_desc, 1);
  if (idx >= 0 && idx < a.N) {
    const int node = (int)(b * a.N + idx);
    unsigned h = ((unsigned)node * 2654435761u) >> 21;  // 11 bits
    for (int probe = 0; probe < 16; ++probe) {
      const int old = atomicCAS(&s_set[h], -1, node);
      if (old == -1) break;
      if (old == node) { atomicAdd(&s_dup, 1); break; }
      h = (h + 1) & (kSlots - 1);
    }
  }
  __syncthreads();
  if (threadIdx.x == 0) *flag = s_desc * 64 < kBinBlock ? 0 : (s_dup * 4 >= quarters * kBinBlock ? 2 : 1);
}

// Count pass: entries per bucket (and, for callers that ask, whether the index is in order and inside [0, N)).
// At most two workgroups per CU, each with an equal share of the entries, which it walks in batches of four
// entries per lane with the loads of the next batch in flight while this one is counted (a workgroup per 16384
// entries ran in rounds: 611 workgroups = 512 + 99, every one loading, then counting, then writing: 44 us).
// 72 scalar registers at most: with 92 (the two argument structs) a SIMD holds seven of these wavefronts instead of
// eight, which is one 1024-lane workgroup per CU instead of two (SPI_RA_SGPR_SIMD_FULL was the stall counter).
constexpr int kBinCountPer = 4;
constexpr int kBinCountBatch = kBinCountPer * kBinPlaceBlock;
constexpr int kBinCountGroups = 512;
template <int CAP>
static __global__ __launch_bounds__(kBinPlaceBlock) __attribute__((amdgpu_num_sgpr(72))) void bin_count_kernel(ScatterArgs a, BinArgs p) {
  __shared__ int32_t s_hist[CAP];
  __shared__ int s_hist_flag;
  if (p.sampled && *p.unsorted != 1) return;
  for (int i = threadIdx.x; i < p.nb; i += kBinPlaceBlock) s_hist[i] = 0;
  if (threadIdx.x == 0) s_hist_flag = 0;
  __syncthreads();
  const int64_t n = a.B * a.E;
  const int64_t per = (n + gridDim.x - 1) / gridDim.x;
  const int64_t lo = (int64_t)blockIdx.x * per;
  const int64_t hi = lo + per < n ? lo + per : n;
  const bool check = p.unsorted != nullptr && !p.sampled;
  const bool strict = p.strict != 0;
  const int lane = threadIdx.x & (kWave - 1);
  int64_t node[kBinCountPer], next[kBinCountPer];
  auto load = [&](int64_t b0, int64_t *x) {
#pragma unroll
    for (int j = 0; j < kBinCountPer; ++j) {
      const int64_t be = b0 + threadIdx.x + (int64_t)j * kBinPlaceBlock;
      x[j] = be < hi ? bin_node(a, be) : -1;
    }
  };
  bool descent = false;
  if (lo < hi) load(lo, node);
  for (int64_t b0 = lo; b0 < hi; b0 += kBinCountBatch) {
    load(b0 + kBinCountBatch, next);  // unconditional: past the end every lane gets -1 without a load
    if (check) {
      // The entry before a lane's entry is the neighbouring lane's (a shuffle); the first lane of a wavefront needs
      // the entry before the wavefront's first one: lane j loads it for row j (one load instruction for all rows).
      int64_t edge = -1;
      if (lane < kBinCountPer) {
        const int64_t be = b0 + (int64_t)(threadIdx.x - lane) + (int64_t)lane * kBinPlaceBlock;
        if (be > 0 && be < hi) edge = bin_node(a, be - 1);
      }
#pragma unroll
      for (int j = 0; j < kBinCountPer; ++j) {
        const int elo = __builtin_amdgcn_readlane((int)(uint32_t)edge, j), ehi = __builtin_amdgcn_readlane((int)(edge >> 32), j);
        const int64_t up = lane_up1_64(node[j]);  // by every lane: lane 0's value is what lane 1 reads
      const int64_t prev = lane == 0 ? (int64_t)(((uint64_t)(uint32_t)ehi << 32) | (uint32_t)elo) : up;
        descent = descent || (node[j] >= 0 && prev >= 0 && node[j] < prev);
        if (strict && node[j] < 0 && b0 + threadIdx.x + (int64_t)j * kBinPlaceBlock < hi) descent = true;
      }
    }
#pragma unroll
    for (int j = 0; j < kBinCountPer; ++j) {
      bin_take(s_hist, node[j] >= 0 ? (int32_t)(node[j] >> p.rshift) : -1);
      node[j] = next[j];
    }
  }
  // one flag for the whole launch: a workgroup that saw a descent sets it unless it reads as set already (ten
  // thousand wavefronts doing so one by one on the same address cost 100 us)
  if (__ballot(descent) != 0) s_hist_flag = 1;
  __syncthreads();
  if (check && threadIdx.x == 0 && s_hist_flag != 0 &&
      __hip_atomic_load(p.unsorted, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT) == 0)
    atomicOr(p.unsorted, 1);
  for (int i = threadIdx.x; i < p.nb; i += kBinPlaceBlock) {
    const int32_t h = s_hist[i];
    if (h != 0) atomicAdd(&p.totals[i], (unsigned long long)h);
  }
}

// one workgroup: prefix sums over the buckets and the list of reducing workgroups
static __global__ __launch_bounds__(kBinBlock) void bin_scan_kernel(BinArgs p) {
  constexpr int PER = kBinMaxBuckets / kBinBlock;
  __shared__ int64_t s_t[kBinBlock];
  __shared__ int64_t s_c[kBinBlock];
  __shared__ int32_t s_m[kBinBlock];  // slabs: chunks of buckets with more than one
  __shared__ int32_t s_l[kBinBlock];  // buckets for the combining kernel: those without exactly one chunk,
  __shared__ int32_t s_g[kBinBlock];  // of which more than kCombFew chunks
  __shared__ int32_t s_cs[kBinMaxBuckets + 1];  // chunk_start, for the search at the end
  if (p.unsorted != nullptr && *p.unsorted != 1) return;  // sorted: none of the later passes runs
  // a bucket holds fewer than 2^32 entries (the plan refuses larger inputs): 32-bit counts and divisions
  // every lane owns `per` neighbouring buckets, no more than the bucket count asks for: the integer divisions below
  // are the kernel's time (sixteen per lane on one CU took 10 us whatever the number of buckets)
  const int per = (p.nb + kBinBlock - 1) / kBinBlock;
  uint32_t t[PER], c[PER];
  int64_t sum_t = 0, sum_c = 0;
  int32_t sum_m = 0, sum_l = 0, sum_g = 0;
#pragma unroll
  for (int j = 0; j < PER; ++j) {
    if (j >= per) break;  // the same for every lane
    const int i = threadIdx.x * per + j;
    t[j] = i < p.nb ? (uint32_t)p.totals[i] : 0u;
    const uint32_t q = t[j] / (uint32_t)p.chunk;
    c[j] = q + (t[j] - q * (uint32_t)p.chunk != 0 ? 1u : 0u);
    sum_t += t[j];
    sum_c += c[j];
    sum_m += c[j] > 1 ? (int32_t)c[j] : 0;
    sum_l += (i < p.nb && c[j] != 1 && c[j] <= (uint32_t)kCombFew) ? 1 : 0;
    sum_g += c[j] > (uint32_t)kCombFew ? 1 : 0;
  }
  s_g[threadIdx.x] = sum_g;
  s_t[threadIdx.x] = sum_t;
  s_c[threadIdx.x] = sum_c;
  s_m[threadIdx.x] = sum_m;
  s_l[threadIdx.x] = sum_l;
  __syncthreads();
  for (int d = 1; d < kBinBlock; d <<= 1) {  // inclusive scan over the threads
    int64_t vt = 0, vc = 0;
    int32_t vm = 0, vl = 0, vg = 0;
    if ((int)threadIdx.x >= d) {
      vt = s_t[threadIdx.x - d]; vc = s_c[threadIdx.x - d]; vm = s_m[threadIdx.x - d]; vl = s_l[threadIdx.x - d];
      vg = s_g[threadIdx.x - d];
    }
    __syncthreads();
    s_t[threadIdx.x] += vt;
    s_c[threadIdx.x] += vc;
    s_m[threadIdx.x] += vm;
    s_l[threadIdx.x] += vl;
    s_g[threadIdx.x] += vg;
    __syncthreads();
  }
  int64_t run_t = s_t[threadIdx.x] - sum_t, run_c = s_c[threadIdx.x] - sum_c;
  int32_t run_m = s_m[threadIdx.x] - sum_m, run_l = s_l[threadIdx.x] - sum_l, run_g = s_g[threadIdx.x] - sum_g;
  const int64_t all_c = s_c[kBinBlock - 1];
  if (p.comb_count != nullptr && threadIdx.x == 0) {
    p.comb_count[0] = s_l[kBinBlock - 1];
    p.comb_count[1] = s_g[kBinBlock - 1];
  }
#pragma unroll
  for (int j = 0; j < PER; ++j) {
    if (j >= per) break;
    const int i = threadIdx.x * per + j;
    if (i < p.nb) {
      p.starts[i] = run_t;
      p.cursor[i] = (unsigned long long)run_t;
      p.chunk_start[i] = (int32_t)run_c;
      s_cs[i] = (int32_t)run_c;
      if (p.slab_start != nullptr) {
        p.slab_start[i] = run_m;
        if (c[j] > (uint32_t)kCombFew)
          p.comb_list[p.nb - 1 - run_g] = i;
        else if (c[j] != 1)
          p.comb_list[run_l] = i;
      }
    }
    if (i == p.nb) { p.starts[i] = run_t; p.chunk_start[i] = (int32_t)run_c; }
    run_t += t[j];
    run_c += c[j];
    run_m += c[j] > 1 ? (int32_t)c[j] : 0;
    run_l += (i < p.nb && c[j] != 1 && c[j] <= (uint32_t)kCombFew) ? 1 : 0;
    run_g += c[j] > (uint32_t)kCombFew ? 1 : 0;
  }
  if (threadIdx.x == kBinBlock - 1 && p.nb == per * kBinBlock) {  // nobody owns index nb then
    p.starts[p.nb] = run_t;
    p.chunk_start[p.nb] = (int32_t)run_c;
  }
  __syncthreads();  // the chunk starts are complete
  for (int64_t k = threadIdx.x; k < p.max_wgs; k += kBinBlock) {
    int32_t b = -1;
    if (k < all_c) {  // the bucket whose chunks include k: last i with chunk_start[i] <= k
      int lo = 0, hi = p.nb - 1;
      while (lo < hi) {
        const int mid = (lo + hi + 1) >> 1;
        if (s_cs[mid] <= k) lo = mid; else hi = mid - 1;
      }
      b = lo;
    }
    p.wg_bucket[k] = b;
  }
}

// ptr[b][r] = first e with index[b][e] >= r, from the `tile` entries at lo of the flattened index (which is in order
// and inside [0, N)), in rounds of one entry per lane: what a place pass leaves for the segmented reduction that
// finishes a sorted index
__device__ __forceinline__ void bin_row_pointers(const ScatterArgs &a, int64_t lo, int tile, GapList &s_gaps) {
  // Long ranges of rows without entries are written by the wavefront or, through the list, by the workgroup
  // (gap_rows): one list for the whole tile, emptied once at the end -- a range that finds the list full stays with
  // its wavefront. (One barrier pair per round of 1024 entries, and a 64-bit division per entry for the batch row,
  // made this pass 53 us for 9 M entries, 37 us without.)
  if (threadIdx.x == 0) s_gaps.n = 0;
  __syncthreads();
  const int64_t n_all = a.B * a.E;
  for (int j = 0; j < kBinPer; ++j) {
    if (j * kBinPlaceBlock >= tile) break;  // uniform
    const int64_t be = lo + threadIdx.x + (int64_t)j * kBinPlaceBlock;
    const bool live = be < n_all;
    int64_t b = 0, e = live ? be : 0;
    if (a.B > 1 && live) {
      b = be / a.E;
      e = be - b * a.E;
    }
    const int64_t *idx = a.index + b * a.sb;
    int64_t top = live ? idx[e] : -1;
    int64_t bot = e == 0 ? 0 : idx[e - 1] + 1;
    if (bot < 0) bot = 0;
    if (top > a.N) top = a.N;
    if (!live) top = bot - 1;
    // the ranges are written through pointers relative to batch 0: lanes of one wavefront may
    // belong to two batches
    const int64_t off = b * (a.N + 1);
    gap_rows(a.route_ptr, off + bot, off + top, e, s_gaps);
    const bool last = live && e == a.E - 1;
    const int64_t tl = top < 0 ? 0 : top + 1;
    gap_rows(a.route_ptr, off + tl, last ? off + a.N : off + tl - 1, a.E, s_gaps);
  }
  __syncthreads();
  gap_rows_finish(a.route_ptr, s_gaps);
}

// (eight wavefronts per SIMD, i.e. at most 64 vector registers: two workgroups per CU at CAP = 8192; left to itself
// the compiler takes 66-71, which is one: Zipf(1.2), 391 buckets, 10 M entries 65 against 55 us)
template <int CAP>
static __global__ __launch_bounds__(kBinPlaceBlock) __attribute__((amdgpu_waves_per_eu(8, 8)))
void bin_place_kernel(ScatterArgs a, BinArgs p) {
  __shared__ uint32_t s_base[CAP];
  __shared__ int32_t s_cnt[CAP];
  if (p.unsorted != nullptr && *p.unsorted != 1) {
    // A sorted index (or, for single values, a skewed one that the table kernel takes): nothing to place. A caller that finishes it with the segmented reduction gets the row
    // pointers from this launch instead: ptr[b][r] = first e with index[b][e] >= r (the count pass has checked
    // that the index is in order and inside [0, N)).
    if (a.route_ptr != nullptr) {
      __shared__ GapList s_gaps;
      bin_row_pointers(a, (int64_t)blockIdx.x * p.place_tile, p.place_tile, s_gaps);
    }
    return;
  }
  for (int i = threadIdx.x; i < p.nb; i += kBinPlaceBlock) s_cnt[i] = 0;
  __syncthreads();
  // the workgroup's tile (one batch at most, held in registers): rank inside the workgroup per bucket, then one
  // atomic per bucket that occurs reserves the workgroup's run, then the words go out
  const int64_t lo = (int64_t)blockIdx.x * p.place_tile;
  const int64_t hi = lo + p.place_tile < a.B * a.E ? lo + p.place_tile : a.B * a.E;
  int32_t bucket[kBinPer], local[kBinPer], rank[kBinPer];
  bool unused = false;
  bin_buckets(a, p, lo, hi, bucket, local, false, unused);
#pragma unroll
  for (int j = 0; j < kBinPer; ++j) rank[j] = bin_take(s_cnt, bucket[j]);
  __syncthreads();
  for (int i = threadIdx.x; i < p.nb; i += kBinPlaceBlock) {
    const int32_t h = s_cnt[i];
    if (h != 0) s_base[i] = (uint32_t)atomicAdd(&p.cursor[i], (unsigned long long)h);
  }
  __syncthreads();
#pragma unroll
  for (int j = 0; j < kBinPer; ++j) {
    if (bucket[j] < 0) continue;
    const int64_t be = lo + threadIdx.x + (int64_t)j * kBinPlaceBlock;
    // (payload: one 4-byte value per entry, K == 1, so entry be of the flattened [B, E] is element be of src)
    const uint32_t low = (p.payload && a.src != nullptr) ? static_cast<const uint32_t *>(a.src)[be]
                                                         : (p.payload ? 1u : (uint32_t)be);  // no src: a count of ones
    p.binned[s_base[bucket[j]] + (uint32_t)rank[j]] = ((uint64_t)(uint32_t)local[j] << 32) | low;
  }
}
static_assert(kBinPlaceChunk == kBinBatch, "the place pass holds a workgroup's entries in registers: one batch");

// The place pass for (row in bucket, value) words under an index in no particular order. With every lane of a
// wavefront bound for another bucket the 8-byte stores of bin_place_kernel each open a memory line of their own
// (21 M entries of a uniform index over 358 buckets: 290 us, and 111 us with the same words stored in entry order).
// Here the tile is sorted by bucket in LDS first -- the ranks give every entry its place behind the tile's
// exclusive prefix over the buckets -- and written out in that order: neighbouring lanes, neighbouring words of one
// bucket's run. A staged word carries its bucket in bits 44 and up (the row in the bucket needs 12 bits at most), so
// the lane that writes it finds the run's base. Tiles of kBinSortTile entries, at most kBinSortBuckets buckets: 64 KB
// of LDS, two workgroups per CU.
constexpr int kBinSortTile = 6144;
constexpr int kBinSortBuckets = 2048;
// (eight wavefronts per SIMD = two workgroups per CU: the branch that writes row pointers would otherwise cost
// the placing branch its registers, 70 instead of 60)
static __global__ __launch_bounds__(kBinPlaceBlock) __attribute__((amdgpu_waves_per_eu(8, 8)))
void bin_place_sorted_kernel(ScatterArgs a, BinArgs p) {
  __shared__ uint64_t s_stage[kBinSortTile];
  __shared__ int32_t s_cnt[kBinSortBuckets];   // counts, then the tile's exclusive prefix
  __shared__ uint32_t s_base[kBinSortBuckets];  // first word of the tile's run in every bucket
  __shared__ int32_t s_wsum[kBinPlaceBlock / kWave];
  const int64_t lo = (int64_t)blockIdx.x * kBinSortTile;
  const int64_t hi = lo + kBinSortTile < a.B * a.E ? lo + kBinSortTile : a.B * a.E;
  if (p.unsorted != nullptr && *p.unsorted != 1) {
    // nothing to place; a caller that finishes a sorted index with the segmented reduction gets its row pointers
    if (a.route_ptr != nullptr) {
      __shared__ GapList s_gaps;
      bin_row_pointers(a, lo, kBinSortTile, s_gaps);
    }
    return;
  }
  for (int i = threadIdx.x; i < p.nb; i += kBinPlaceBlock) s_cnt[i] = 0;
  __syncthreads();
  int32_t bucket[kBinPer], local[kBinPer], rank[kBinPer];
  bool unused = false;
  bin_buckets(a, p, lo, hi, bucket, local, false, unused);
#pragma unroll
  for (int j = 0; j < kBinPer; ++j) rank[j] = bin_take(s_cnt, bucket[j]);
  __syncthreads();
  // reserve the tile's runs, then turn the counts into the tile's exclusive prefix: every lane owns `per`
  // neighbouring buckets
  const int per = (p.nb + kBinPlaceBlock - 1) / kBinPlaceBlock;
  const int b0 = threadIdx.x * per;
  int32_t mine = 0;
  for (int j = 0; j < per; ++j) {
    const int i = b0 + j;
    if (i >= p.nb) break;
    const int32_t h = s_cnt[i];
    if (h != 0) s_base[i] = (uint32_t)atomicAdd(&p.cursor[i], (unsigned long long)h);
    mine += h;
  }
  const int lane = threadIdx.x & (kWave - 1), wave = threadIdx.x / kWave;
  const int32_t incl = wave_inclusive_sum(mine);
  if (lane == kWave - 1) s_wsum[wave] = incl;
  __syncthreads();
  int32_t run = incl - mine;
  for (int w2 = 0; w2 < wave; ++w2) run += s_wsum[w2];
  for (int j = 0; j < per; ++j) {
    const int i = b0 + j;
    if (i >= p.nb) break;
    const int32_t h = s_cnt[i];
    s_cnt[i] = run;
    run += h;
  }
  __syncthreads();
#pragma unroll
  for (int j = 0; j < kBinPer; ++j) {
    if (bucket[j] < 0) continue;
    const int64_t be = lo + threadIdx.x + (int64_t)j * kBinPlaceBlock;
    const uint32_t low = (p.payload && a.src != nullptr) ? static_cast<const uint32_t *>(a.src)[be]
                                                         : (p.payload ? 1u : (uint32_t)be);
    s_stage[s_cnt[bucket[j]] + rank[j]] =
        ((uint64_t)(uint32_t)bucket[j] << 44) | ((uint64_t)(uint32_t)local[j] << 32) | low;
  }
  __syncthreads();
  const int total = run_total(s_wsum);  // the tile's entries with an index inside [0, N)
  for (int pos = threadIdx.x; pos < total; pos += kBinPlaceBlock) {
    const uint64_t w = s_stage[pos];
    const uint32_t b = (uint32_t)(w >> 44);
    p.binned[s_base[b] + (uint32_t)(pos - s_cnt[b])] = w & (((uint64_t)1 << 44) - 1);
  }
}

// The same place pass for records of several values (BinArgs::planes > 1): a staged record is planes + 1 32-bit words,
// the entry's values and then (bucket << 12 | row in the bucket); the tile holds as many entries as fit the stage
// (BinArgs::sort_tile). The records leave in the order of the stage, 32-bit word by word: neighbouring lanes,
// neighbouring words of one bucket's run.
static __global__ __launch_bounds__(kBinPlaceBlock) __attribute__((amdgpu_waves_per_eu(8, 8)))
void bin_place_records_kernel(ScatterArgs a, BinArgs p) {
  __shared__ uint32_t s_stage[2 * kBinSortTile];
  __shared__ int32_t s_cnt[kBinSortBuckets];   // counts, then the tile's exclusive prefix
  __shared__ uint32_t s_base[kBinSortBuckets];  // first record of the tile's run in every bucket
  __shared__ int32_t s_wsum[kBinPlaceBlock / kWave];
  if (p.unsorted != nullptr && *p.unsorted != 1) return;
  const int64_t lo = (int64_t)blockIdx.x * p.sort_tile;
  const int64_t hi = lo + p.sort_tile < a.B * a.E ? lo + p.sort_tile : a.B * a.E;
  for (int i = threadIdx.x; i < p.nb; i += kBinPlaceBlock) s_cnt[i] = 0;
  __syncthreads();
  int32_t bucket[kBinPer], local[kBinPer], rank[kBinPer];
  bool unused = false;
  bin_buckets(a, p, lo, hi, bucket, local, false, unused);
#pragma unroll
  for (int j = 0; j < kBinPer; ++j) rank[j] = bin_take(s_cnt, bucket[j]);
  __syncthreads();
  const int per = (p.nb + kBinPlaceBlock - 1) / kBinPlaceBlock;
  const int b0 = threadIdx.x * per;
  int32_t mine = 0;
  for (int j = 0; j < per; ++j) {
    const int i = b0 + j;
    if (i >= p.nb) break;
    const int32_t h = s_cnt[i];
    if (h != 0) s_base[i] = (uint32_t)atomicAdd(&p.cursor[i], (unsigned long long)h);
    mine += h;
  }
  const int lane = threadIdx.x & (kWave - 1), wave = threadIdx.x / kWave;
  const int32_t incl = wave_inclusive_sum(mine);
  if (lane == kWave - 1) s_wsum[wave] = incl;
  __syncthreads();
  int32_t run = incl - mine;
  for (int w2 = 0; w2 < wave; ++w2) run += s_wsum[w2];
  for (int j = 0; j < per; ++j) {
    const int i = b0 + j;
    if (i >= p.nb) break;
    const int32_t h = s_cnt[i];
    s_cnt[i] = run;
    run += h;
  }
  __syncthreads();
  const int K = p.planes, R = K + 1;
  const uint32_t *src = static_cast<const uint32_t *>(a.src);
#pragma unroll
  for (int j = 0; j < kBinPer; ++j) {
    if (bucket[j] < 0) continue;
    const int64_t be = lo + threadIdx.x + (int64_t)j * kBinPlaceBlock;
    uint32_t *rec = s_stage + (s_cnt[bucket[j]] + rank[j]) * R;
    for (int k = 0; k < K; ++k) rec[k] = src[be * K + k];
    rec[K] = ((uint32_t)bucket[j] << 12) | (uint32_t)local[j];
  }
  __syncthreads();
  const int total = run_total(s_wsum);  // the tile's entries with an index inside [0, N)
  uint32_t *words = reinterpret_cast<uint32_t *>(p.binned);
  for (int d = threadIdx.x; d < total * R; d += kBinPlaceBlock) {
    const int pos = d / R, j = d - pos * R;
    const uint32_t tail = s_stage[pos * R + K];
    const uint32_t b = tail >> 12;
    const int64_t dest = (int64_t)s_base[b] + (pos - s_cnt[b]);
    words[dest * R + j] = j == K ? (tail & 0xFFFu) : s_stage[d];
  }
}

// One finished packed key -> out / arg_out (element i of [B, N, K]): what scatter_key_init_kernel and
// scatter_key_final_kernel do for the kernels that keep their keys in arg_out. key == 0: no entry.
template <typename T, bool IS_MAX>
__device__ __forceinline__ void bin_emit(const ScatterArgs &a, int64_t i, uint64_t key) {
  T *out = static_cast<T *>(a.out);
  const uint32_t kv = (uint32_t)(key >> 32);
  bool has = key != 0;
  if (a.out_given) {
    // an entry has to beat the previous content strictly; a NaN in out is never beaten
    const T prev = out[i];
    uint32_t pk = Key<T>::enc(prev);
    if (!IS_MAX) pk = ~pk;
    has = has && !Key<T>::is_nan(prev) && kv > pk;
    if (!has) {
      a.arg_out[i] = a.E;
      return;
    }
  } else {
    // a value that does not beat the initial value of the reduction counts as no entry
    uint32_t lim = Key<T>::enc(IS_MAX ? ElemLim<T>::lowest() : ElemLim<T>::max());
    if (!IS_MAX) lim = ~lim;
    has = has && kv > lim;
    if (!has) {
      out[i] = zero_elem<T>();
      a.arg_out[i] = a.E;
      return;
    }
  }
  const int64_t e = (int64_t)(0xFFFFFFFEu - (uint32_t)key);
  const uint32_t k = IS_MAX ? kv : ~kv;
  T val = Key<T>::dec(k);
  if (Key<T>::kFloat && k == 0x80000000u) {
    // a zero: fetch it from src to keep the sign bit of the winning entry
    const int64_t bn = i / a.K;
    val = static_cast<const T *>(a.src)[((bn / a.N) * a.E + e) * a.K + (i - bn * a.K)];
  }
  out[i] = val;
  a.arg_out[i] = e;
}

// The table of one chunk (rows K + 1 keys apart) leaves the workgroup without atomics: a bucket that is
// reduced in one chunk goes straight to out / arg_out; the chunks of a larger bucket store their tables in
// slabs of the workspace, which bin_combine_kernel puts together. (Writing the tables into one table of keys
// in memory with a read and an atomic per key took 56 of 300 us for 10 M entries of 32 floats: 13 M atomics,
// most of them on the 8192 keys of the bucket that holds the hubs.)
template <typename T, bool IS_MAX>
__device__ __forceinline__ void bin_flush_keys(const ScatterArgs &a, const BinArgs &p, int bucket, int wg, int slice,
                                               const uint64_t *s_keys) {
  const int K = (int)a.K, kc = p.kc;
  const int c0 = slice * kc;                                    // first column of this workgroup's slice
  const int64_t first = ((int64_t)bucket << p.rshift) * a.K;   // first element of the bucket in [B * N, K]
  const int64_t rows_left = a.B * a.N - ((int64_t)bucket << p.rshift);  // rows that exist
  const int table = kc << p.rshift;
  const int chunks = p.chunk_start[bucket + 1] - p.chunk_start[bucket];
  if (chunks == 1) {
    for (int i = threadIdx.x; i < table; i += kBinBlock) {
      const int row = i / kc;
      if (row < rows_left) bin_emit<T, IS_MAX>(a, first + (int64_t)row * K + c0 + (i - row * kc), s_keys[i + row]);
    }
  } else {
    uint64_t *slab = p.slabs + ((int64_t)p.slab_start[bucket] + (wg - p.chunk_start[bucket])) * ((int64_t)K << p.rshift);
    for (int i = threadIdx.x; i < table; i += kBinBlock) {
      const int row = i / kc;
      slab[row * K + c0 + (i - row * kc)] = s_keys[i + row];  // row `row` of the table starts `row` keys later
    }
  }
}

// Buckets that were not reduced in exactly one chunk: the maximum over the slabs of their chunks (none: a bucket
// without entries), element by element, to out / arg_out. A workgroup takes 1024 neighbouring keys of one bucket.
// A bucket of few chunks (an index with many entries per output row everywhere: 2-4 chunks in every bucket) gives
// every lane one key and walks the slabs in order; a bucket of many chunks (the one that holds the hubs of a skewed
// index: a thousand slabs) is taken 64 keys at a time, the wavefronts share the slabs, sixteen loads in flight
// each, and meet in LDS.
template <typename T, bool IS_MAX>
__global__ __launch_bounds__(kBinBlock) void bin_combine_kernel(ScatterArgs a, BinArgs p) {
  constexpr int W = kBinBlock / kWave;
  __shared__ uint64_t s_part[W][kCombPos];
  if (p.unsorted != nullptr && *p.unsorted != 1) return;  // sorted index: left to the caller's segmented reduction
  const int lane = threadIdx.x & (kWave - 1), wave = threadIdx.x / kWave;
  const int table = (int)a.K << p.rshift;
  const int n_few = p.comb_count[0], n_many = p.comb_count[1];
  const int64_t total = a.B * a.N * a.K;
  // buckets of many chunks first (the long items), 64 keys per workgroup and step
  const int parts = (table + kCombPos - 1) / kCombPos;
  for (int64_t item = blockIdx.x; item < (int64_t)n_many * parts; item += gridDim.x) {
    const int bucket = p.comb_list[p.nb - 1 - (int)(item / parts)];
    const int m = p.chunk_start[bucket + 1] - p.chunk_start[bucket];
    const int pos = (int)(item % parts) * kCombPos + lane;
    const int64_t first = ((int64_t)bucket << p.rshift) * a.K;
    const uint64_t *slab = p.slabs + (int64_t)p.slab_start[bucket] * table + (pos < table ? pos : 0);
    uint64_t best = 0;
    constexpr int U = 16;  // loads in flight per lane: the slabs of a bucket with a thousand chunks in four round trips
    for (int s0 = wave; s0 < m; s0 += W * U) {
      uint64_t k[U];
#pragma unroll
      for (int u = 0; u < U; ++u) k[u] = slab[(int64_t)(s0 + u * W < m ? s0 + u * W : s0) * table];
#pragma unroll
      for (int u = 0; u < U; ++u) best = k[u] > best ? k[u] : best;
    }
    s_part[wave][lane] = best;
    __syncthreads();
    if (wave == 0) {
#pragma unroll
      for (int w2 = 1; w2 < W; ++w2) best = s_part[w2][lane] > best ? s_part[w2][lane] : best;
      if (pos < table && first + pos < total) bin_emit<T, IS_MAX>(a, first + pos, best);
    }
    __syncthreads();
  }
  // buckets of few chunks, 1024 keys per workgroup and step
  const int blocks = (table + kBinBlock - 1) / kBinBlock;
  for (int64_t item = blockIdx.x; item < (int64_t)n_few * blocks; item += gridDim.x) {
    const int bucket = p.comb_list[item / blocks];
    const int m = p.chunk_start[bucket + 1] - p.chunk_start[bucket];
    const int pos = (int)(item % blocks) * kBinBlock + (int)threadIdx.x;
    const int64_t first = ((int64_t)bucket << p.rshift) * a.K;
    if (pos >= table || first + pos >= total) continue;
    const uint64_t *slab = p.slabs + (int64_t)p.slab_start[bucket] * table + pos;
    constexpr int U = 8;
    uint64_t best = 0;
    for (int s0 = 0; s0 < m; s0 += U) {
      uint64_t k[U];
#pragma unroll
      for (int u = 0; u < U; ++u) k[u] = slab[(int64_t)(s0 + u < m ? s0 + u : s0) * table];
#pragma unroll
      for (int u = 0; u < U; ++u) best = k[u] > best ? k[u] : best;
    }
    bin_emit<T, IS_MAX>(a, first + pos, best);
  }
}

template <typename T, int VEC, bool IS_MAX>
__global__ __launch_bounds__(kBinBlock) void bin_reduce_kernel(ScatterArgs a, BinArgs p) {
  constexpr int U = 4;  // 63 VGPRs: two workgroups per CU (eight rows in flight per lane: 74 VGPRs, one workgroup)
  // rows are K + 1 keys apart: with K a multiple of 32 the rows would all start in the same LDS bank and the
  // lanes of a wavefront, which hold the same columns of different rows, would queue up behind each other
  __shared__ uint64_t s_keys[kBinKeys + kBinKeys / 16];
  if (p.unsorted != nullptr && *p.unsorted != 1) return;
  const int bucket = p.wg_bucket[blockIdx.x];
  if (bucket < 0) return;
  const int K = (int)a.K;
  const int KP = K + 1;
  const int rows = 1 << p.rshift;
  for (int i = threadIdx.x; i < rows * KP; i += kBinBlock) s_keys[i] = 0;
  __syncthreads();

  const T *src = static_cast<const T *>(a.src);
  const int64_t lo = p.starts[bucket] + ((int64_t)blockIdx.x - p.chunk_start[bucket]) * p.chunk;
  int64_t hi = lo + p.chunk;
  if (hi > p.starts[bucket + 1]) hi = p.starts[bucket + 1];
  const EdgeLanes m = edge_lanes(K / VEC, kBinBlock);  // K / VEC <= 512: one column slice per lane
  if (m.active) {
    const int k0 = m.cl * VEC;
    for (int64_t s0 = lo + m.el; s0 < hi; s0 += (int64_t)m.epp * U) {
      uint64_t ent[U];
#pragma unroll
      for (int u = 0; u < U; ++u) {
        const int64_t s = s0 + (int64_t)u * m.epp;
        ent[u] = p.binned[s < hi ? s : s0];
      }
      Vec<T, VEC> x[U];
#pragma unroll
      for (int u = 0; u < U; ++u) x[u] = load_vec_stream<T, VEC>(src + (int64_t)(uint32_t)ent[u] * a.K + k0);
#pragma unroll
      for (int u = 0; u < U; ++u) {
        if (s0 + (int64_t)u * m.epp >= hi) continue;
        int64_t e = (int64_t)(uint32_t)ent[u];
        if (a.B > 1) e -= (e / a.E) * a.E;  // position inside the batch
        uint64_t key[VEC];
        make_keys<T, VEC, IS_MAX>(x[u], e, key);
        uint64_t *row = &s_keys[(int)(ent[u] >> 32) * KP + k0];
        // filter on the value half (one 32-bit LDS read per element): below the cached key cannot win
        const uint32_t *hi32 = reinterpret_cast<const uint32_t *>(row) + 1;
#pragma unroll
        for (int v = 0; v < VEC; ++v)
          if (key[v] != 0 && (uint32_t)(key[v] >> 32) >= lds_peek(hi32 + 2 * v))
            __hip_atomic_fetch_max(row + v, key[v], __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_WORKGROUP);
      }
    }
  }
  __syncthreads();
  bin_flush_keys<T, IS_MAX>(a, p, bucket, (int)blockIdx.x, 0, s_keys);
}

// The same reduction for rows held by a power-of-two number of lanes (<= 64): a wavefront reads 64 entry words
// with one coalesced load (the next 64 are in flight while these are worked on) and hands them to its lane
// groups by shuffle, so the rows of an entry are requested without first waiting for its entry word.
template <typename T, int VEC, bool IS_MAX>
__global__ __launch_bounds__(kBinBlock) void bin_reduce_wave_kernel(ScatterArgs a, BinArgs p, int lshift) {
  constexpr int U = 4;  // eight rows in flight per lane: 90 VGPRs, one workgroup per CU, no gain
  __shared__ uint64_t s_keys[kBinKeys + kBinKeys / 16];  // rows K + 1 keys apart (LDS banks, see above)
  if (p.unsorted != nullptr && *p.unsorted != 1) return;
  const int wg = (int)(blockIdx.x / (unsigned)p.slices), slice = (int)(blockIdx.x - (unsigned)wg * p.slices);
  const int bucket = p.wg_bucket[wg];
  if (bucket < 0) return;
  const int KP = p.kc + 1;
  const int rows = 1 << p.rshift;
  for (int i = threadIdx.x; i < rows * KP; i += kBinBlock) s_keys[i] = 0;
  __syncthreads();

  const T *src = static_cast<const T *>(a.src);
  const int64_t lo = p.starts[bucket] + ((int64_t)wg - p.chunk_start[bucket]) * p.chunk;
  int64_t hi = lo + p.chunk;
  if (hi > p.starts[bucket + 1]) hi = p.starts[bucket + 1];
  const int lane = threadIdx.x & (kWave - 1), wave = threadIdx.x / kWave;
  const int g = lane >> lshift;                 // lane group: one entry at a time
  const int gpw = kWave >> lshift;              // lane groups per wavefront
  const int k0 = (lane & ((1 << lshift) - 1)) * VEC;         // column inside the slice
  const int ksrc = slice * p.kc + k0;                        // column of the row
  constexpr int64_t kStride = (int64_t)(kBinBlock / kWave) * kWave;  // entries per pass of the workgroup
  if (lo < hi) {
    int64_t base = lo + (int64_t)wave * kWave;
    uint64_t ent_next = p.binned[base + lane < hi ? base + lane : hi - 1];
    for (; base < hi; base += kStride) {
      const uint64_t ent = ent_next;
      const int64_t nb = base + kStride;
      ent_next = p.binned[nb + lane < hi ? nb + lane : hi - 1];  // unconditional: exact wait counts
      const int n = hi - base < kWave ? (int)(hi - base) : kWave;
      const uint32_t ent_lo = (uint32_t)ent, ent_hi = (uint32_t)(ent >> 32);
      for (int i0 = 0; i0 < n; i0 += gpw * U) {
        uint32_t e_row[U], e_ent[U];
        Vec<T, VEC> x[U];
#pragma unroll
        for (int u = 0; u < U; ++u) {
          const int i = i0 + u * gpw + g;
          const int from = i < n ? i : n - 1;
          e_ent[u] = (uint32_t)__shfl((int)ent_lo, from);
          e_row[u] = (uint32_t)__shfl((int)ent_hi, from);
          x[u] = load_vec_stream<T, VEC>(src + (int64_t)e_ent[u] * a.K + ksrc);
        }
#pragma unroll
        for (int u = 0; u < U; ++u) {
          if (i0 + u * gpw + g >= n) continue;
          int64_t e = (int64_t)e_ent[u];
          if (a.B > 1) e -= (e / a.E) * a.E;  // position inside the batch
          uint64_t key[VEC];
          make_keys<T, VEC, IS_MAX>(x[u], e, key);
          uint64_t *row = &s_keys[(int)e_row[u] * KP + k0];
          const uint32_t *hi32 = reinterpret_cast<const uint32_t *>(row) + 1;
#pragma unroll
          for (int v = 0; v < VEC; ++v)
            if (key[v] != 0 && (uint32_t)(key[v] >> 32) >= lds_peek(hi32 + 2 * v))
              __hip_atomic_fetch_max(row + v, key[v], __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_WORKGROUP);
        }
      }
    }
  }
  __syncthreads();
  bin_flush_keys<T, IS_MAX>(a, p, bucket, wg, slice, s_keys);
}

static __global__ __launch_bounds__(kBlock) void bin_clear_kernel(unsigned long long *totals, int n, int *flag) {
  const int i = blockIdx.x * kBlock + threadIdx.x;
  if (i < n) totals[i] = 0;
  if (i == 0 && flag != nullptr) *flag = 0;
}

// ---- sum: the same buckets with a table of accumulators (fp32 for 16-bit floats). Every entry is one LDS
// atomic add; the table goes to `out` with one atomic per touched element and chunk.
// Slot type of the table: floating types accumulate in double. ds_add_f64 and the integer adds keep their rate
// when many lanes meet on one address (a hub row); ds_add_f32 does not (measured: 10 M entries of a Zipf(1.2)
// index, K = 32: 2.2 ms with fp32 slots, 0.44 ms with int32 or double slots).
template <typename T> struct BinSlot { typedef double type; };
template <> struct BinSlot<int32_t> { typedef int32_t type; };
template <> struct BinSlot<int64_t> { typedef int64_t type; };
template <typename T> struct BinSlotOk { static constexpr bool value = sizeof(typename Acc<T>::type) >= 4; };

template <typename T, int VEC>
__global__ __launch_bounds__(kBinBlock) void bin_add_wave_kernel(ScatterArgs a, BinArgs p, int lshift) {
  typedef typename BinSlot<T>::type A;
  typedef typename Acc<T>::type F;
  constexpr int U = 4;
  constexpr int kSlots = (kBinKeys + kBinKeys / 16) * 8 / (int)sizeof(A);
  __shared__ A s_acc[kSlots];  // rows K + 1 slots apart (LDS banks)
  __shared__ int32_t s_num[1 << kBinCountShift];  // entries per row, for a caller that wants them (BinArgs::count_out)
  if (p.unsorted != nullptr && *p.unsorted != 1) return;
  const int wg = (int)(blockIdx.x / (unsigned)p.slices), slice = (int)(blockIdx.x - (unsigned)wg * p.slices);
  const int bucket = p.wg_bucket[wg];
  if (bucket < 0) return;
  const int K = (int)a.K, kc = p.kc;
  const int KP = kc + 1;
  const int rows = 1 << p.rshift;
  const bool counting = p.count_out != nullptr && slice == 0;  // the workgroups of one column slice count
  for (int i = threadIdx.x; i < rows * KP; i += kBinBlock) s_acc[i] = (A)0;
  if (counting)
    for (int i = threadIdx.x; i < rows; i += kBinBlock) s_num[i] = 0;
  __syncthreads();

  const T *src = static_cast<const T *>(a.src);
  const int64_t lo = p.starts[bucket] + ((int64_t)wg - p.chunk_start[bucket]) * p.chunk;
  int64_t hi = lo + p.chunk;
  if (hi > p.starts[bucket + 1]) hi = p.starts[bucket + 1];
  const int lane = threadIdx.x & (kWave - 1), wave = threadIdx.x / kWave;
  const int g = lane >> lshift;
  const int gpw = kWave >> lshift;
  const int k0 = (lane & ((1 << lshift) - 1)) * VEC;  // column inside the slice
  const int c0 = slice * kc;                          // first column of the slice
  constexpr int64_t kStride = (int64_t)(kBinBlock / kWave) * kWave;
  if (lo < hi) {
    int64_t base = lo + (int64_t)wave * kWave;
    uint64_t ent_next = p.binned[base + lane < hi ? base + lane : hi - 1];
    for (; base < hi; base += kStride) {
      const uint64_t ent = ent_next;
      const int64_t nb = base + kStride;
      ent_next = p.binned[nb + lane < hi ? nb + lane : hi - 1];
      const int n = hi - base < kWave ? (int)(hi - base) : kWave;
      const uint32_t ent_lo = (uint32_t)ent, ent_hi = (uint32_t)(ent >> 32);
      for (int i0 = 0; i0 < n; i0 += gpw * U) {
        uint32_t e_row[U];
        Vec<T, VEC> x[U];
#pragma unroll
        for (int u = 0; u < U; ++u) {
          const int i = i0 + u * gpw + g;
          const int from = i < n ? i : n - 1;
          const uint32_t e_ent = (uint32_t)__shfl((int)ent_lo, from);
          e_row[u] = (uint32_t)__shfl((int)ent_hi, from);
          x[u] = load_vec_stream<T, VEC>(src + (int64_t)e_ent * a.K + c0 + k0);
        }
#pragma unroll
        for (int u = 0; u < U; ++u) {
          if (i0 + u * gpw + g >= n) continue;
          A *row = &s_acc[(int)e_row[u] * KP + k0];
#pragma unroll
          for (int v = 0; v < VEC; ++v)
            __hip_atomic_fetch_add(row + v, (A)to_acc<T>(x[u].v[v]), __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_WORKGROUP);
          if (counting && k0 == 0)  // the lane with the row's first columns
            __hip_atomic_fetch_add(&s_num[e_row[u]], 1, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_WORKGROUP);
        }
      }
    }
  }
  __syncthreads();
  T *out = static_cast<T *>(a.out) + ((int64_t)bucket << p.rshift) * a.K + c0;
  const int64_t rows_left = a.B * a.N - ((int64_t)bucket << p.rshift);  // rows that exist
  const int table = kc << p.rshift;
  if (counting) {
    for (int i = threadIdx.x; i < rows && i < rows_left; i += kBinBlock) {
      const int32_t c = s_num[i];
      if (c != 0) atomicAdd(p.count_out + ((int64_t)bucket << p.rshift) + i, c);
    }
  }
  if constexpr (sizeof(T) == 2) {
    // two neighbouring columns per packed atomic (kc is even here: whole 16-byte vectors per lane)
    if ((reinterpret_cast<uintptr_t>(a.out) & 3) == 0) {
      for (int i = 2 * threadIdx.x; i < table; i += 2 * kBinBlock) {
        const int row = i / kc;
        if (row >= rows_left) break;
        const A v0 = s_acc[i + row], v1 = s_acc[i + 1 + row];
        if (v0 == (A)0 && v1 == (A)0) continue;
        T *dst = out + (int64_t)row * K + (i - row * kc);
        if constexpr (__is_same(T, bf16_t)) {
          typedef short v2s __attribute__((ext_vector_type(2)));
          v2s pk;
          pk.x = (short)float_to_bf16((float)v0).x;
          pk.y = (short)float_to_bf16((float)v1).x;
          __builtin_amdgcn_global_atomic_fadd_v2bf16(reinterpret_cast<v2s *>(dst), pk);
        } else {
          typedef _Float16 v2h __attribute__((ext_vector_type(2)));
          v2h pk;
          pk.x = (_Float16)(float)v0;
          pk.y = (_Float16)(float)v1;
          __builtin_amdgcn_global_atomic_fadd_v2f16(reinterpret_cast<v2h *>(dst), pk);
        }
      }
      return;
    }
  }
  for (int i = threadIdx.x; i < table; i += kBinBlock) {
    const int row = i / kc;
    if (row >= rows_left) break;
    const A v = s_acc[i + row];
    if (v == (A)0) continue;
    T *dst = out + (int64_t)row * K + (i - row * kc);
    if constexpr (sizeof(T) == 2)  // no compare-and-swap loop: hundreds of chunks of a hub bucket meet here
      atomic_add_half<T>(dst, from_acc<T>((F)v), static_cast<T *>(a.out), static_cast<T *>(a.out) + a.B * a.N * a.K);
    else
      atomic_add_elem<T>(dst, from_acc<T>((F)v));
  }
}

// Sum of one 4-byte value per entry from (row in bucket, value) words: see bin_plan_payload. A workgroup streams
// its chunk of a bucket with 16-byte loads (two words per lane, four loads in flight), adds into the bucket's table
// in LDS (double slots for floats: ds_add_f64 keeps its rate when many lanes meet on one address, a hub row) and
// adds every row it touched to out once.
// COUNT: the entries of every row are counted as well (BinArgs::count_out), in a second table.
template <typename T, bool COUNT = false>
__global__ __launch_bounds__(kBinBlock) void bin_add_payload_kernel(ScatterArgs a, BinArgs p) {
  static_assert(sizeof(T) == 4, "one 4-byte value per word");
  typedef typename BinSlot<T>::type A;
  typedef unsigned long long u64x2 __attribute__((ext_vector_type(2)));
  constexpr int U = 4;
  __shared__ A s_acc[4096];
  __shared__ int32_t s_num[COUNT ? 4096 : 1];
  if (p.unsorted != nullptr && *p.unsorted != 1) return;
  const int wg = (int)blockIdx.x;
  const int bucket = p.wg_bucket[wg];
  if (bucket < 0) return;
  const int rows = 1 << p.rshift;
  for (int i = threadIdx.x; i < rows; i += kBinBlock) {
    s_acc[i] = (A)0;
    if (COUNT) s_num[i] = 0;
  }
  __syncthreads();
  const int64_t lo = p.starts[bucket] + ((int64_t)wg - p.chunk_start[bucket]) * p.chunk;
  int64_t hi = lo + p.chunk;
  if (hi > p.starts[bucket + 1]) hi = p.starts[bucket + 1];
  auto add = [&](unsigned long long w) {
    T v;
    const uint32_t bits = (uint32_t)w;
    __builtin_memcpy(&v, &bits, 4);
    const uint32_t row = (uint32_t)(w >> 32) & (uint32_t)(rows - 1);
    __hip_atomic_fetch_add(&s_acc[row], (A)v, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_WORKGROUP);
    if (COUNT) __hip_atomic_fetch_add(&s_num[row], 1, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_WORKGROUP);
  };
  if (lo < hi) {
    // words lo .. hi - 1; the 16-byte loads start at an even word
    const int64_t first = lo & ~(int64_t)1;
    const u64x2 *pairs = reinterpret_cast<const u64x2 *>(p.binned + first);
    const int64_t n_pairs = (hi - first + 1) >> 1;  // the last pair may reach one word past hi: inside the array or its padding
    for (int64_t base = 0; base < n_pairs; base += (int64_t)U * kBinBlock) {
      u64x2 w[U];
#pragma unroll
      for (int u = 0; u < U; ++u) {
        const int64_t i = base + (int64_t)u * kBinBlock + threadIdx.x;
        w[u] = __builtin_nontemporal_load(pairs + (i < n_pairs ? i : n_pairs - 1));
      }
#pragma unroll
      for (int u = 0; u < U; ++u) {
        const int64_t i = base + (int64_t)u * kBinBlock + threadIdx.x;
        if (i >= n_pairs) continue;
        const int64_t e0 = first + 2 * i;
        if (e0 >= lo) add(w[u].x);
        if (e0 + 1 < hi) add(w[u].y);
      }
    }
  }
  __syncthreads();
  T *out = static_cast<T *>(a.out) + ((int64_t)bucket << p.rshift);
  const int64_t rows_left = a.B * a.N - ((int64_t)bucket << p.rshift);  // rows that exist
  for (int i = threadIdx.x; i < rows && i < rows_left; i += kBinBlock) {
    const A v = s_acc[i];
    if (v != (A)0) atomic_add_elem<T>(out + i, (T)v);
    if (COUNT) {
      const int32_t c = s_num[i];
      if (c != 0) atomicAdd(p.count_out + ((int64_t)bucket << p.rshift) + i, c);
    }
  }
}

// The same sum from records of several values per entry (BinArgs::planes > 1, bin_place_records_kernel): slot
// row * planes + k of the table is element k of the row.
template <typename T, bool COUNT = false>
__global__ __launch_bounds__(kBinBlock) void bin_add_records_kernel(ScatterArgs a, BinArgs p) {
  static_assert(sizeof(T) == 4, "4-byte values");
  typedef typename BinSlot<T>::type A;
  constexpr int U = 4;
  __shared__ A s_acc[4096];
  __shared__ int32_t s_num[COUNT ? 4096 : 1];
  if (p.unsorted != nullptr && *p.unsorted != 1) return;
  const int wg = (int)blockIdx.x;
  const int bucket = p.wg_bucket[wg];
  if (bucket < 0) return;
  const int rows = 1 << p.rshift;
  const int K = p.planes, R = K + 1;
  for (int i = threadIdx.x; i < rows * K; i += kBinBlock) s_acc[i] = (A)0;
  if (COUNT) {
    for (int i = threadIdx.x; i < rows; i += kBinBlock) s_num[i] = 0;
  }
  __syncthreads();
  const int64_t lo = p.starts[bucket] + ((int64_t)wg - p.chunk_start[bucket]) * p.chunk;
  int64_t hi = lo + p.chunk;
  if (hi > p.starts[bucket + 1]) hi = p.starts[bucket + 1];
  const uint32_t *words = reinterpret_cast<const uint32_t *>(p.binned);
  for (int64_t base = lo; base < hi; base += (int64_t)U * kBinBlock) {
    uint32_t w[U][kBinPayloadCols + 1];
#pragma unroll
    for (int u = 0; u < U; ++u) {
      const int64_t e = base + (int64_t)u * kBinBlock + threadIdx.x;
      const uint32_t *rec = words + (e < hi ? e : lo) * R;
#pragma unroll
      for (int k = 0; k <= kBinPayloadCols; ++k) w[u][k] = k < R ? __builtin_nontemporal_load(rec + k) : 0u;
    }
#pragma unroll
    for (int u = 0; u < U; ++u) {
      if (base + (int64_t)u * kBinBlock + threadIdx.x >= hi) continue;
      uint32_t tail = 0;
#pragma unroll
      for (int k = 0; k <= kBinPayloadCols; ++k) tail = k == K ? w[u][k] : tail;
      const uint32_t row = tail & (uint32_t)(rows - 1);
#pragma unroll
      for (int k = 0; k < kBinPayloadCols; ++k) {
        if (k >= K) break;
        T v;
        __builtin_memcpy(&v, &w[u][k], 4);
        __hip_atomic_fetch_add(&s_acc[row * K + k], (A)v, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_WORKGROUP);
      }
      if (COUNT) __hip_atomic_fetch_add(&s_num[row], 1, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_WORKGROUP);
    }
  }
  __syncthreads();
  T *out = static_cast<T *>(a.out) + ((int64_t)bucket << p.rshift) * K;
  const int64_t rows_left = a.B * a.N - ((int64_t)bucket << p.rshift);  // rows that exist
  for (int i = threadIdx.x; i < rows * K && i < rows_left * K; i += kBinBlock) {
    const A v = s_acc[i];
    if (v != (A)0) atomic_add_elem<T>(out + i, (T)v);
  }
  if (COUNT) {
    for (int i = threadIdx.x; i < rows && i < rows_left; i += kBinBlock) {
      const int32_t c = s_num[i];
      if (c != 0) atomicAdd(p.count_out + ((int64_t)bucket << p.rshift) + i, c);
    }
  }
}

// Which plans the place pass that sorts its tile in LDS first (bin_place_sorted_kernel) takes, of those it has room
// for (2048 buckets of up to 4096 rows): value words always, entry words from 512 buckets on. Under an even index
// every 8-byte store of the plain pass is a line of its own and the sorted pass wins at any number of buckets (10 M
// entries over 391 / 977 buckets: 65 / 76 against 86 / 116 us; 46 M over 1860: 433 against 628 us); under a skewed
// index, whose runs are long as they are, the plain pass does (Zipf(1.2), 391 buckets: 55 against 64 us). The host
// does not know which it has; the heavy-tailed indices measured here come with few buckets. (Choosing per tile, from
// the tile's largest bucket, was measured: both branches in one kernel spill and lose 10 us each.)
inline bool bin_place_sorted_ok(const BinArgs &p) {
  return p.nb <= kBinSortBuckets && p.rshift <= 12 && (p.payload || p.nb >= 512) &&
         !getenv("TS_BIN_NO_SORTED_PLACE");  // env: tuning aid
}

// the count pass: equal shares of the entries for at most kBinCountGroups workgroups
inline void launch_bin_count(const ScatterArgs &a, const BinArgs &p, hipStream_t stream) {
  int64_t groups = (a.B * a.E + kBinCountBatch - 1) / kBinCountBatch;
  if (groups > kBinCountGroups) groups = kBinCountGroups;
  if (groups < 1) groups = 1;
  if (p.nb <= kBinSmallCap)
    hipLaunchKernelGGL(bin_count_kernel<kBinSmallCap>, dim3((unsigned)groups), dim3(kBinPlaceBlock), 0, stream, a, p);
  else
    hipLaunchKernelGGL(bin_count_kernel<kBinMaxBuckets>, dim3((unsigned)groups), dim3(kBinPlaceBlock), 0, stream, a, p);
}

// log2 of the lanes that hold the kc columns of a slice, VEC columns each: the wavefront kernels want a power of
// two up to 64. -1: no such number (then only bin_reduce_kernel can take the plan, and only without slices).
inline int bin_lane_shift(const BinArgs &p, int vec) {
  if (p.kc % vec != 0) return -1;
  const int kv = p.kc / vec;
  int lshift = 0;
  while ((1 << lshift) < kv) ++lshift;
  return ((1 << lshift) == kv && kv <= kWave) ? lshift : -1;
}

// min / max through the buckets: every element of out / arg_out is written by the reducing or the combining kernel
template <typename T, int VEC, bool IS_MAX>
void launch_binned_keys(const ScatterArgs &a, const BinArgs &plan, hipStream_t stream) {
  BinArgs p = plan;
  if (a.sorted_route && a.route_flag != nullptr)
    p.strict = 1;          // the count pass checks the index; the caller finishes a sorted one
  else
    p.unsorted = nullptr;  // min / max take this path for sorted indices too
  hipLaunchKernelGGL(bin_clear_kernel, dim3((p.nb + kBlock - 1) / kBlock), dim3(kBlock), 0, stream, p.totals, p.nb,
                     p.unsorted);
  launch_bin_count(a, p, stream);
  hipLaunchKernelGGL(bin_scan_kernel, dim3(1), dim3(kBinBlock), 0, stream, p);
  if (bin_place_sorted_ok(p))
    hipLaunchKernelGGL(bin_place_sorted_kernel, dim3((unsigned)((a.B * a.E + kBinSortTile - 1) / kBinSortTile)),
                       dim3(kBinPlaceBlock), 0, stream, a, p);
  else if (p.nb <= kBinSmallCap)  // 64 KB of cursors, two workgroups per CU; above: 128 KB, one
    hipLaunchKernelGGL(bin_place_kernel<kBinSmallCap>, dim3((unsigned)p.n_place), dim3(kBinPlaceBlock), 0, stream, a, p);
  else
    hipLaunchKernelGGL(bin_place_kernel<kBinMaxBuckets>, dim3((unsigned)p.n_place), dim3(kBinPlaceBlock), 0, stream, a, p);
  const int lshift = bin_lane_shift(p, VEC);
  if (lshift >= 0 && (p.slices > 1 || !getenv("TS_BIN_NO_WAVE")))  // env: tuning aid
    hipLaunchKernelGGL((bin_reduce_wave_kernel<T, VEC, IS_MAX>), dim3((unsigned)(p.max_wgs * p.slices)), dim3(kBinBlock), 0,
                       stream, a, p, lshift);
  else
    hipLaunchKernelGGL((bin_reduce_kernel<T, VEC, IS_MAX>), dim3((unsigned)p.max_wgs), dim3(kBinBlock), 0, stream, a, p);
  hipLaunchKernelGGL((bin_combine_kernel<T, IS_MAX>), dim3(2048), dim3(kBinBlock), 0, stream, a, p);
}

// sum: count (with the test for a sorted index), scan, place, add. The caller launches its usual sum kernels
// afterwards with skip_flag = p.unsorted: they run only if the index turned out to be sorted.
// out[i] = 0 unless the index is sorted (then nobody adds into out: the caller's segmented reduction writes it)
template <typename T>
__global__ __launch_bounds__(kBlock) void bin_zero_out_kernel(T *out, int64_t n, const int *unsorted) {
  if (*unsorted != 1) return;
  for (int64_t i = (int64_t)blockIdx.x * kBlock + threadIdx.x; i < n; i += (int64_t)gridDim.x * kBlock)
    out[i] = zero_elem<T>();
}

// zero_out: elements of out to clear once the count pass has found the index unsorted (0: the caller has cleared it)
// three_way: the caller has the table kernel behind this launch for a skewed index (flag value 2, see
// bin_sample_skew_kernel); needs the sample (no sorted_route, enough entries), else the answer stays 0 / 1
template <typename T, int VEC>
void launch_binned_add(const ScatterArgs &a, const BinArgs &plan, int lshift, hipStream_t stream, int64_t zero_out = 0,
                       bool three_way = false) {
  BinArgs p = plan;
  p.sampled = a.B * a.E >= 2 * kBinBlock && !getenv("TS_BIN_NO_SAMPLE");  // env: tuning aid (sorted = no descent at all)
  if (a.sorted_route && a.route_flag != nullptr) {  // the caller's segmented reduction needs the whole index checked
    p.sampled = 0;
    p.strict = 1;
  }
  if (p.sampled && three_way)
    hipLaunchKernelGGL(bin_sample_skew_kernel, dim3(1), dim3(kBinBlock), 0, stream, a, p.unsorted, p.planes > 1 ? 2 : 3,
                       p.totals, p.nb);
  else if (p.sampled)
    hipLaunchKernelGGL(bin_sample_kernel, dim3(1), dim3(kBinBlock), 0, stream, a, p.unsorted, p.totals, p.nb);
  else  // (the sample kernels clear the buckets' counts on the way)
    hipLaunchKernelGGL(bin_clear_kernel, dim3((p.nb + kBlock - 1) / kBlock), dim3(kBlock), 0, stream, p.totals, p.nb,
                       p.unsorted);
  launch_bin_count(a, p, stream);
  if (zero_out > 0)
    hipLaunchKernelGGL(bin_zero_out_kernel<T>, dim3(grid_for(zero_out)), dim3(kBlock), 0, stream, static_cast<T *>(a.out),
                       zero_out, p.unsorted);
  hipLaunchKernelGGL(bin_scan_kernel, dim3(1), dim3(kBinBlock), 0, stream, p);
  if (p.payload && p.planes > 1)
    hipLaunchKernelGGL(bin_place_records_kernel, dim3((unsigned)((a.B * a.E + p.sort_tile - 1) / p.sort_tile)),
                       dim3(kBinPlaceBlock), 0, stream, a, p);
  else if (bin_place_sorted_ok(p))
    hipLaunchKernelGGL(bin_place_sorted_kernel, dim3((unsigned)((a.B * a.E + kBinSortTile - 1) / kBinSortTile)),
                       dim3(kBinPlaceBlock), 0, stream, a, p);
  else if (p.nb <= kBinSmallCap)  // 64 KB of cursors, two workgroups per CU; above: 128 KB, one
    hipLaunchKernelGGL(bin_place_kernel<kBinSmallCap>, dim3((unsigned)p.n_place), dim3(kBinPlaceBlock), 0, stream, a, p);
  else
    hipLaunchKernelGGL(bin_place_kernel<kBinMaxBuckets>, dim3((unsigned)p.n_place), dim3(kBinPlaceBlock), 0, stream, a, p);
  if constexpr (sizeof(T) == 4) {
    if (p.payload && p.planes > 1) {
      if (p.count_out != nullptr)
        hipLaunchKernelGGL((bin_add_records_kernel<T, true>), dim3((unsigned)p.max_wgs), dim3(kBinBlock), 0, stream, a, p);
      else
        hipLaunchKernelGGL((bin_add_records_kernel<T, false>), dim3((unsigned)p.max_wgs), dim3(kBinBlock), 0, stream, a, p);
      return;
    }
    if (p.payload) {
      if (p.count_out != nullptr)
        hipLaunchKernelGGL((bin_add_payload_kernel<T, true>), dim3((unsigned)p.max_wgs), dim3(kBinBlock), 0, stream, a, p);
      else
        hipLaunchKernelGGL((bin_add_payload_kernel<T, false>), dim3((unsigned)p.max_wgs), dim3(kBinBlock), 0, stream, a, p);
      return;
    }
  }
  hipLaunchKernelGGL((bin_add_wave_kernel<T, VEC>), dim3((unsigned)(p.max_wgs * p.slices)), dim3(kBinBlock), 0, stream, a, p,
                     lshift);
}

}  // namespace ts
