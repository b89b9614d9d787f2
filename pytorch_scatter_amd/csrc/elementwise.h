// Small passes over [B, N, K] that complete the reductions: the count and the
// division of scatter(mean), and the backward of every min/max flavour.
#pragma once

#include "device_utils.h"
#include "scatter.h"

namespace ts {

// count[b, index[b, e]] += 1 (int32: exact)
static __global__ __launch_bounds__(kBlock) void scatter_count_kernel(const int64_t *__restrict__ index,
                                                               int32_t *__restrict__ count, int64_t B,
                                                               int64_t E, int64_t N, int64_t sb, int64_t se) {
  const int64_t n = B * E;
  for (int64_t i = (int64_t)blockIdx.x * kBlock + threadIdx.x; i < n; i += (int64_t)gridDim.x * kBlock) {
    const int64_t b = i / E;
    const int64_t e = i - b * E;
    const int64_t idx = index[b * sb + e * se];
    if (idx < 0 || idx >= N) continue;
    atomicAdd(count + b * N + idx, 1);
  }
}

template <typename T> struct IsFloatElem { static constexpr bool value = false; };
template <> struct IsFloatElem<float> { static constexpr bool value = true; };
template <> struct IsFloatElem<double> { static constexpr bool value = true; };
template <> struct IsFloatElem<bf16_t> { static constexpr bool value = true; };
template <> struct IsFloatElem<f16_t> { static constexpr bool value = true; };

// out /= (T)max(count, 1): true division for floats, floor division for
// integers (csrc/scatter.cpp:138-141)
template <typename T>
__global__ __launch_bounds__(kBlock) void divide_by_count_kernel(T *__restrict__ out,
                                                                 const int32_t *__restrict__ count,
                                                                 int64_t rows, int64_t K) {
  const int64_t n = rows * K;
  for (int64_t i = (int64_t)blockIdx.x * kBlock + threadIdx.x; i < n; i += (int64_t)gridDim.x * kBlock) {
    const int32_t ci = count[i / K];
    const int64_t c = ci < 1 ? 1 : (int64_t)ci;
    if constexpr (IsFloatElem<T>::value) {
      out[i] = div_elem<T>(out[i], count_as<T>(c));
    } else {
      const T d = (T)c;
      const T x = out[i];
      if (d == 0) {
        out[i] = 0;  // an 8/16-bit count that wrapped to 0: undefined upstream
      } else {
        T q = (T)(x / d);
        if ((x % d != 0) && ((x < 0) != (d < 0))) q = (T)(q - 1);
        out[i] = q;
      }
    }
  }
}

// grad_in = 0, then grad_in[b, arg[b,n,k], k] = grad_out[b,n,k] where arg < E
template <typename T>
__global__ __launch_bounds__(kBlock) void arg_backward_kernel(const T *__restrict__ grad_out,
                                                              const int64_t *__restrict__ arg,
                                                              T *__restrict__ grad_in, int64_t B,
                                                              int64_t N, int64_t E, int64_t K) {
  const int64_t n = B * N * K;
  for (int64_t i = (int64_t)blockIdx.x * kBlock + threadIdx.x; i < n; i += (int64_t)gridDim.x * kBlock) {
    const int64_t e = arg[i];
    if (e < 0 || e >= E) continue;
    const int64_t bn = i / K;
    const int64_t k = i - bn * K;
    const int64_t b = bn / N;
    grad_in[(b * E + e) * K + k] = grad_out[i];
  }
}

// After a min / max over permuted rows (a scatter through a sorted index): positions in row-pointer order
// become positions in the caller's order, and a slot whose entries never beat scatter's initial value
// (lowest() / max() of the element type) reads 0 with position E, as scatter leaves it
// (csrc/cpu/scatter_cpu.cpp:81-82). A slot without entries already holds 0 and E.
template <typename T, bool IS_MAX>
__global__ __launch_bounds__(kBlock) void sorted_args_kernel(T *__restrict__ out, int64_t *__restrict__ arg,
                                                             const int32_t *__restrict__ perm, int64_t total,
                                                             int64_t per_batch, int64_t E, int64_t perm_batch_stride) {
  typedef typename Acc<T>::type A;
  const A lim = to_acc<T>(IS_MAX ? ElemLim<T>::lowest() : ElemLim<T>::max());
  for (int64_t i = (int64_t)blockIdx.x * kBlock + threadIdx.x; i < total; i += (int64_t)gridDim.x * kBlock) {
    const int64_t a = arg[i];
    if (a < 0 || a >= E) continue;
    const A v = to_acc<T>(out[i]);
    const bool beat = IS_MAX ? (v > lim) : (v < lim);
    if (beat) {
      arg[i] = perm[(i / per_batch) * perm_batch_stride + a];
    } else {
      out[i] = zero_elem<T>();
      arg[i] = E;
    }
  }
}

template <typename T> int launch_sorted_args(void *out, int64_t *arg, const int32_t *perm, int64_t B, int64_t per_batch,
                                             int64_t E, int64_t perm_batch_stride, bool is_max, hipStream_t stream);
template <typename T> int launch_divide_by_count(void *out, const int32_t *count, int64_t rows, int64_t K,
                                                 hipStream_t stream);
template <typename T> int launch_arg_backward(const void *grad_out, const int64_t *arg, void *grad_in,
                                              int64_t B, int64_t N, int64_t E, int64_t K,
                                              hipStream_t stream);

#define TS_INSTANTIATE_ELEMENTWISE(T)                                                              \
  template <> int launch_sorted_args<T>(void *out, int64_t *arg, const int32_t *perm, int64_t B,   \
                                        int64_t per_batch, int64_t E, int64_t perm_batch_stride,   \
                                        bool is_max, hipStream_t stream) {                         \
    const int64_t total = B * per_batch;                                                           \
    if (total > 0 && is_max)                                                                       \
      hipLaunchKernelGGL((sorted_args_kernel<T, true>), dim3(grid_for(total)), dim3(kBlock), 0,    \
                         stream, static_cast<T *>(out), arg, perm, total, per_batch, E,            \
                         perm_batch_stride);                                                       \
    else if (total > 0)                                                                            \
      hipLaunchKernelGGL((sorted_args_kernel<T, false>), dim3(grid_for(total)), dim3(kBlock), 0,   \
                         stream, static_cast<T *>(out), arg, perm, total, per_batch, E,            \
                         perm_batch_stride);                                                       \
    return hipGetLastError() == hipSuccess ? TS_OK : TS_ERR_LAUNCH;                                \
  }                                                                                                \
  template <> int launch_divide_by_count<T>(void *out, const int32_t *count, int64_t rows, int64_t K, \
                                            hipStream_t stream) {                                  \
    if (rows * K > 0)                                                                              \
      hipLaunchKernelGGL(divide_by_count_kernel<T>, dim3(grid_for(rows * K)), dim3(kBlock), 0,     \
                         stream, static_cast<T *>(out), count, rows, K);                           \
    return hipGetLastError() == hipSuccess ? TS_OK : TS_ERR_LAUNCH;                                \
  }                                                                                                \
  template <> int launch_arg_backward<T>(const void *grad_out, const int64_t *arg, void *grad_in,  \
                                         int64_t B, int64_t N, int64_t E, int64_t K,               \
                                         hipStream_t stream) {                                     \
    if (B * E * K > 0)                                                                             \
      hipLaunchKernelGGL(fill_kernel<T>, dim3(grid_for(B * E * K, 4)), dim3(kBlock), 0, stream,    \
                         static_cast<T *>(grad_in), B * E * K, small_const<T>(0));                 \
    if (B * N * K > 0)                                                                             \
      hipLaunchKernelGGL(arg_backward_kernel<T>, dim3(grid_for(B * N * K)), dim3(kBlock), 0,       \
                         stream, static_cast<const T *>(grad_out), arg, static_cast<T *>(grad_in), \
                         B, N, E, K);                                                              \
    return hipGetLastError() == hipSuccess ? TS_OK : TS_ERR_LAUNCH;                                \
  }

}  // namespace ts
