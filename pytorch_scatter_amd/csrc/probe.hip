// Plain streaming kernels that measure what the memory system of the device sustains: the ceilings the
// reduction / expansion kernels are held against (bench.py --probe-ceilings). Not part of the operator
// library: built as libts_probe.so and loaded by the benchmark only.
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
