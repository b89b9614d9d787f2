// Plain streaming kernels that measure what the memory system of the device sustains: the ceilings the
// reduction / expansion kernels are held against (python3 -m benchmark.hw_probes --ceilings / --ceiling-matrix /
// --atomics). Not part of the operator library: built by benchmark/probe/Makefile as libts_probe.so and loaded
// by the benchmark scripts only.
#include <hip/hip_runtime.h>
#include <stdint.h>

namespace {
typedef uint32_t u4 __attribute__((ext_vector_type(4)));
constexpr int kThreads = 256;
constexpr int kU = 8;  // 16-byte accesses in flight per lane

// one chunk of kU * kThreads vectors per workgroup and trip, grid-stride over the chunks
__global__ __launch_bounds__(kThreads) void read_kernel(const u4 *__restrict__ p, size_t n, u4 *sink) {
  u4 acc = {0, 0, 0, 0};
  const size_t chunk = (size_t)kU * kThreads;
  for (size_t base = (size_t)blockIdx.x * chunk; base < n; base += (size_t)gridDim.x * chunk) {
    u4 x[kU];
#pragma unroll
    for (int u = 0; u < kU; ++u) {
      const size_t i = base + (size_t)u * kThreads + threadIdx.x;
      x[u] = i < n ? __builtin_nontemporal_load(p + i) : acc;
    }
#pragma unroll
    for (int u = 0; u < kU; ++u) acc ^= x[u];
  }
  if (acc.x == 0x12345678u && acc.y == 0x9abcdef0u) sink[0] = acc;  // keeps the loads alive, never true
}

__global__ __launch_bounds__(kThreads) void write_kernel(u4 *__restrict__ q, size_t n) {
  const u4 v = {1, 2, 3, (uint32_t)threadIdx.x};
  const size_t chunk = (size_t)kU * kThreads;
  for (size_t base = (size_t)blockIdx.x * chunk; base < n; base += (size_t)gridDim.x * chunk) {
#pragma unroll
    for (int u = 0; u < kU; ++u) {
      const size_t i = base + (size_t)u * kThreads + threadIdx.x;
      if (i < n) q[i] = v;
    }
  }
}

// reads `ratio` vectors for every vector it writes: ratio 1 = copy, 3 = the mix of a max + arg reduction over
// rows of a few entries, 26 = a mean over 26 entries per row
__global__ __launch_bounds__(kThreads) void mix_kernel(const u4 *__restrict__ p, u4 *__restrict__ q, size_t n_write,
                                                       int ratio) {
  const size_t chunk = (size_t)kU * kThreads;
  for (size_t base = (size_t)blockIdx.x * chunk; base < n_write; base += (size_t)gridDim.x * chunk) {
    u4 acc[kU];
#pragma unroll
    for (int u = 0; u < kU; ++u) acc[u] = u4{0, 0, 0, 0};
    for (int r = 0; r < ratio; ++r) {
      u4 x[kU];
#pragma unroll
      for (int u = 0; u < kU; ++u) {
        const size_t i = base + (size_t)u * kThreads + threadIdx.x;
        x[u] = i < n_write ? __builtin_nontemporal_load(p + (size_t)r * n_write + i) : acc[u];
      }
#pragma unroll
      for (int u = 0; u < kU; ++u) acc[u] ^= x[u];
    }
#pragma unroll
    for (int u = 0; u < kU; ++u) {
      const size_t i = base + (size_t)u * kThreads + threadIdx.x;
      if (i < n_write) q[i] = acc[u];
    }
  }
}

// ---- the matrix of mixed streams ------------------------------------------------------------------------------
// A "unit" is `burst` contiguous bytes on the light side of the mix and ratio * burst contiguous bytes on the
// heavy side. heavy_read: a unit reads ratio * burst bytes of p and writes burst bytes of q (a reduction over
// `ratio` entries per row); else it reads burst bytes of p and writes ratio * burst bytes of q (an expansion).
// Workgroups walk the units grid-stride. U 16-byte loads are in flight per lane; NT_LOAD / NT_STORE pick
// non-temporal accesses. SPLIT: workgroups specialise instead -- workgroup b of every group of (ratio + 1) does
// nothing but the light side, the others nothing but the heavy side (same bytes in all), so that read-only and
// write-only workgroups are co-resident on the CUs.
template <bool NT>
__device__ __forceinline__ u4 ld(const u4 *p) { return NT ? __builtin_nontemporal_load(p) : *p; }
template <bool NT>
__device__ __forceinline__ void st(u4 *q, u4 v) { if (NT) __builtin_nontemporal_store(v, q); else *q = v; }

template <int U, bool NT_LOAD>
__device__ __forceinline__ u4 read_span(const u4 *__restrict__ p, size_t vecs, u4 acc, int lane, int lanes) {
  for (size_t base = 0; base < vecs; base += (size_t)U * lanes) {
    u4 x[U];
#pragma unroll
    for (int u = 0; u < U; ++u) {
      const size_t i = base + (size_t)u * lanes + lane;
      x[u] = i < vecs ? ld<NT_LOAD>(p + i) : acc;
    }
#pragma unroll
    for (int u = 0; u < U; ++u) acc ^= x[u];
  }
  return acc;
}
template <bool NT_STORE>
__device__ __forceinline__ void write_span(u4 *__restrict__ q, size_t vecs, u4 v, int lane, int lanes) {
  for (size_t i = lane; i < vecs; i += lanes) st<NT_STORE>(q + i, v);
}

// A workgroup is cut into workers of `lanes` lanes (a power of two, 16 ... 256: min(256, burst / 16)), one unit
// at a time per worker -- the shape of the reduction kernels, where 16 lanes hold one 256-byte row.
template <int U, bool NT_LOAD, bool NT_STORE, bool SPLIT>
__global__ __launch_bounds__(kThreads) void matrix_kernel(const u4 *__restrict__ p, u4 *__restrict__ q, size_t units,
                                                          size_t burst_vecs, int ratio, int heavy_read, int lanes, int stagger) {
  const size_t rd = heavy_read ? burst_vecs * ratio : burst_vecs, wr = heavy_read ? burst_vecs : burst_vecs * ratio;
  const int lane = threadIdx.x % lanes, per_wg = kThreads / lanes;
  const size_t worker = (size_t)blockIdx.x * per_wg + threadIdx.x / lanes, workers_all = (size_t)gridDim.x * per_wg;
  u4 acc = {1, 2, 3, (uint32_t)threadIdx.x};
  if (!SPLIT) {
    if (stagger && worker < units) {
      // the workers of a workgroup fall out of step: worker w first reads w / per_wg of a unit's heavy-or-light
      // read span (once), so that from then on the workers' writes come at different moments instead of together
      const size_t part = rd * (size_t)(threadIdx.x / lanes) / per_wg;
      acc = read_span<U, NT_LOAD>(p + worker * rd, part, acc, lane, lanes);
    }
    for (size_t unit = worker; unit < units; unit += workers_all) {
      acc = read_span<U, NT_LOAD>(p + unit * rd, rd, acc, lane, lanes);
      write_span<NT_STORE>(q + unit * wr, wr, acc, lane, lanes);
    }
  } else {
    // whole workgroups specialise; every workgroup moves the same number of bytes, walked as spans of burst_vecs
    const int role = blockIdx.x % (ratio + 1);          // 0: light side only
    const bool reads = (role == 0) != (heavy_read != 0);
    const bool heavy_side = role != 0;
    const size_t spans = units * (reads ? rd : wr) / burst_vecs;   // spans of this side in all
    const size_t light_wgs = (gridDim.x + ratio) / (ratio + 1);
    const size_t wgs = heavy_side ? gridDim.x - light_wgs : light_wgs;
    const size_t my_wg = heavy_side ? (size_t)(blockIdx.x - blockIdx.x / (ratio + 1) - 1) : (size_t)(blockIdx.x / (ratio + 1));
    for (size_t sp = my_wg * per_wg + threadIdx.x / lanes; sp < spans; sp += wgs * per_wg) {
      if (reads) acc = read_span<U, NT_LOAD>(p + sp * burst_vecs, burst_vecs, acc, lane, lanes);
      else write_span<NT_STORE>(q + sp * burst_vecs, burst_vecs, acc, lane, lanes);
    }
    if (reads && acc.x == 0x12345678u && acc.y == 0x9abcdef0u) q[0] = acc;  // keeps the loads alive, never true
  }
}

__device__ __forceinline__ uint32_t hash32(uint32_t x) {
  x ^= x >> 16; x *= 0x7feb352dU; x ^= x >> 15; x *= 0x846ca68bU; x ^= x >> 16;
  return x;
}
// 64-bit atomic max, device scope, without return. pattern 0: every lane its own pseudo-random slot of `slots`
// (one transaction per lane); pattern 1: lane i of every workgroup -> slots i, i + 1024, ... below `slots`
// (neighbouring lanes neighbouring addresses, every workgroup the same addresses: a table written back)
__global__ __launch_bounds__(1024) void atomic_kernel(unsigned long long *tab, uint32_t slots, int iters, int pattern) {
  const uint32_t t = blockIdx.x * 1024 + threadIdx.x;
  if (pattern == 0) {
    for (int it = 0; it < iters; ++it) {
      const uint32_t h = hash32(t * 7919u + it * 104729u);
      __hip_atomic_fetch_max(tab + h % slots, (unsigned long long)h << 20, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
    }
  } else {
    for (uint32_t i = threadIdx.x; i < slots; i += 1024)
      __hip_atomic_fetch_max(tab + i, (unsigned long long)hash32(blockIdx.x * 7919u + i) << 20, __ATOMIC_RELAXED,
                             __HIP_MEMORY_SCOPE_AGENT);
  }
}
}  // namespace

extern "C" {
// 256 workgroups of 1024 lanes issue atomics on a table of `slots` 8-byte slots (see atomic_kernel); returns the
// number of atomics of the launch, or -1 on a launch error.
long long ts_probe_atomics(void *table, unsigned slots, int iters, int pattern, void *stream) {
  hipLaunchKernelGGL(atomic_kernel, dim3(256), dim3(1024), 0, static_cast<hipStream_t>(stream),
                     static_cast<unsigned long long *>(table), slots, iters, pattern);
  if (hipGetLastError() != hipSuccess) return -1;
  return pattern == 0 ? 256ll * 1024 * iters : 256ll * slots;
}

// One cell of the matrix of mixed streams (matrix_kernel): `units` units of `burst` bytes (a multiple of 256) on the
// light side and ratio * burst on the heavy side; a must hold the bytes read and b the bytes written.
// depth: 16-byte loads in flight per lane (4, 8 or 16); grid: workgroups of 256 lanes; stagger: the workers of a
// workgroup run out of step (their writes come at different moments). Returns 0, 1 (launch error)
// or 2 (bad argument).
int ts_probe_matrix(const void *a, void *b, size_t units, size_t burst, int ratio, int heavy_read, int depth,
                    int nt_load, int nt_store, int split, int grid, int stagger, void *stream) {
  if (burst == 0 || burst % 256 != 0 || ratio < 1 || grid < 1 || (split && grid < ratio + 1)) return 2;
  hipStream_t s = static_cast<hipStream_t>(stream);
  const u4 *p = static_cast<const u4 *>(a);
  u4 *q = static_cast<u4 *>(b);
  const size_t bv = burst / 16;
  int lanes = 16;   // lanes of a worker: min(256, burst / 16) rounded down to a power of two, at least 16
  while (lanes < kThreads && (size_t)lanes * 2 <= bv) lanes *= 2;
#define TS_PROBE_LAUNCH(U, NL, NS, SP)                                                                         \
  hipLaunchKernelGGL((matrix_kernel<U, NL, NS, SP>), dim3(grid), dim3(kThreads), 0, s, p, q, units, bv, ratio, \
                     heavy_read, lanes, stagger)
#define TS_PROBE_FLAGS(U)                                                             \
  do {                                                                                \
    if (split) {                                                                      \
      if (nt_load && nt_store) TS_PROBE_LAUNCH(U, true, true, true);                  \
      else if (nt_load) TS_PROBE_LAUNCH(U, true, false, true);                        \
      else if (nt_store) TS_PROBE_LAUNCH(U, false, true, true);                       \
      else TS_PROBE_LAUNCH(U, false, false, true);                                    \
    } else {                                                                          \
      if (nt_load && nt_store) TS_PROBE_LAUNCH(U, true, true, false);                 \
      else if (nt_load) TS_PROBE_LAUNCH(U, true, false, false);                       \
      else if (nt_store) TS_PROBE_LAUNCH(U, false, true, false);                      \
      else TS_PROBE_LAUNCH(U, false, false, false);                                   \
    }                                                                                 \
  } while (0)
  if (depth == 4) TS_PROBE_FLAGS(4);
  else if (depth == 8) TS_PROBE_FLAGS(8);
  else if (depth == 16) TS_PROBE_FLAGS(16);
  else return 2;
#undef TS_PROBE_FLAGS
#undef TS_PROBE_LAUNCH
  return hipGetLastError() == hipSuccess ? 0 : 1;
}

// mode 0: read `bytes` from a.  1: write `bytes` to b.  2..: read (mode - 1) * bytes from a and write `bytes` to b
// (2 = copy). a must hold max(1, mode - 1) * bytes, b `bytes`; both 16-byte aligned. Returns 0 or 1 (launch error).
int ts_probe_stream(int mode, const void *a, void *b, size_t bytes, void *stream) {
  const size_t n = bytes / 16;
  const int grid = 256 * 8;
  hipStream_t s = static_cast<hipStream_t>(stream);
  if (mode == 0)
    hipLaunchKernelGGL(read_kernel, dim3(grid), dim3(kThreads), 0, s, static_cast<const u4 *>(a), n, static_cast<u4 *>(b));
  else if (mode == 1)
    hipLaunchKernelGGL(write_kernel, dim3(grid), dim3(kThreads), 0, s, static_cast<u4 *>(b), n);
  else
    hipLaunchKernelGGL(mix_kernel, dim3(grid), dim3(kThreads), 0, s, static_cast<const u4 *>(a), static_cast<u4 *>(b), n,
                       mode - 1);
  return hipGetLastError() == hipSuccess ? 0 : 1;
}
}
