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
}  // namespace

extern "C" {
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
