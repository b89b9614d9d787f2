// Device-side building blocks shared by the gfx950 kernels: element types,
// 16-byte vector access, accumulate-type conversions and the reducer rules.
#pragma once

#include <hip/hip_runtime.h>
#include <stdint.h>

#include "../../include/ts_hip.h"
#include "dpp.h"

namespace ts {

constexpr int kWave = 64;         // CDNA wavefront width
constexpr int kBlock = 256;       // threads per workgroup: 4 wavefronts
constexpr int kVecBytes = 16;     // one global_load_dwordx4 per lane

struct bf16_t { uint16_t x; };    // bfloat16 carried as its bit pattern

// ---- row pointers of a sorted index: the rows between two neighbouring entries ---------------------
// The thread that owns entry e writes ptr[r] = e for the rows r in (index[e-1], index[e]]. That is one row or
// two for most entries, and now and then all the rows that no entry falls into: the tail of an output with
// more rows than the index reaches, the rows either side of a lone hub. One lane writing such a range alone
// takes 26 ns per row (20 000 entries that all name row 25 000 of 50 000: 0.67 ms; the rows behind an index
// that ends at row 500: 1.3 ms). So only ranges of up to kGapSerial rows are written by their lane; longer ones
// by the wavefront, 64 rows per store instruction, and those above kGapWave rows by the whole workgroup after a
// barrier (a list in LDS; when it is full the wavefront keeps the range). Every row is still written by the
// workgroup of the lane that owns it, whatever the index holds, so an index that is not sorted gives wrong
// row pointers as before and never unwritten ones.
constexpr int kGapSerial = 8;
constexpr int kGapWave = 2048;
constexpr int kGapSlots = 32;
struct GapList {
  long long v[kGapSlots][3];  // lo, hi, e
  int n;
};
// called by every lane of a wavefront together; hi < lo: nothing to write for this lane
__device__ __forceinline__ void gap_rows(int64_t *p, int64_t lo, int64_t hi, int64_t e, GapList &list) {
  int64_t n = hi - lo + 1;
  if (n > 0 && n <= kGapSerial)
    for (int64_t r = lo; r <= hi; ++r) p[r] = e;
  if (n > kGapWave) {
    const int slot = atomicAdd(&list.n, 1);
    if (slot < kGapSlots) {
      list.v[slot][0] = lo;
      list.v[slot][1] = hi;
      list.v[slot][2] = e;
      n = 0;
    }
  }
  unsigned long long todo = __ballot(n > kGapSerial);
  const int lane = threadIdx.x & (kWave - 1);
  while (todo) {
    const int from = __ffsll(todo) - 1;
    todo &= todo - 1;
    const long long lo_s = __shfl((long long)lo, from), hi_s = __shfl((long long)hi, from);
    const long long e_s = __shfl((long long)e, from);
    for (long long r = lo_s + lane; r <= hi_s; r += kWave) p[r] = e_s;
  }
}
// after a __syncthreads() behind the last gap_rows of the workgroup: the ranges that were left to all of it
__device__ __forceinline__ void gap_rows_finish(int64_t *p, const GapList &list) {
  const int cnt = list.n < kGapSlots ? list.n : kGapSlots;
  for (int g = 0; g < cnt; ++g) {
    const long long lo = list.v[g][0], hi = list.v[g][1], e = list.v[g][2];
    for (long long r = lo + threadIdx.x; r <= hi; r += blockDim.x) p[r] = e;
  }
}
typedef _Float16 f16_t;

// ---- accumulate type (the reference's at::opmath_type: float for 16-bit
// floats, the type itself otherwise; csrc/cpu/segment_csr_cpu.cpp:62)
template <typename T> struct Acc { typedef T type; };
template <> struct Acc<bf16_t> { typedef float type; };
template <> struct Acc<f16_t> { typedef float type; };

__device__ __forceinline__ float bf16_to_float(bf16_t h) {
  return __uint_as_float((uint32_t)h.x << 16);
}
// round to nearest even; NaN -> 0x7FC0 (what c10::BFloat16 does)
__device__ __forceinline__ bf16_t float_to_bf16(float f) {
  uint32_t u = __float_as_uint(f);
  bf16_t r;
  if ((u & 0x7FFFFFFFu) > 0x7F800000u) {
    r.x = 0x7FC0;
  } else {
    r.x = (uint16_t)((u + 0x7FFFu + ((u >> 16) & 1u)) >> 16);
  }
  return r;
}

template <typename T> __device__ __forceinline__ typename Acc<T>::type to_acc(T v) { return v; }
template <> __device__ __forceinline__ float to_acc<bf16_t>(bf16_t v) { return bf16_to_float(v); }
template <> __device__ __forceinline__ float to_acc<f16_t>(f16_t v) { return (float)v; }

template <typename T> __device__ __forceinline__ T from_acc(typename Acc<T>::type v) { return (T)v; }
template <> __device__ __forceinline__ bf16_t from_acc<bf16_t>(float v) { return float_to_bf16(v); }
template <> __device__ __forceinline__ f16_t from_acc<f16_t>(float v) { return (f16_t)v; }

// (scalar_t)count of the reference's Reducer::write (csrc/cpu/reducer.h:74-75)
template <typename T> __device__ __forceinline__ T count_as(int64_t c) { return (T)c; }
template <> __device__ __forceinline__ bf16_t count_as<bf16_t>(int64_t c) { return float_to_bf16((float)c); }
template <> __device__ __forceinline__ f16_t count_as<f16_t>(int64_t c) { return (f16_t)(float)c; }

// val / (scalar_t)count evaluated in the element type: 16-bit floats divide in
// float and round once, integers truncate.
template <typename T> __device__ __forceinline__ T div_elem(T a, T b) { return a / b; }
template <> __device__ __forceinline__ bf16_t div_elem<bf16_t>(bf16_t a, bf16_t b) {
  return float_to_bf16(bf16_to_float(a) / bf16_to_float(b));
}
template <> __device__ __forceinline__ f16_t div_elem<f16_t>(f16_t a, f16_t b) {
  return (f16_t)((float)a / (float)b);
}

// 0 or 1 in the element type, usable on the host (fill values)
template <typename T> __host__ __device__ inline T small_const(int v) { return (T)v; }
template <> __host__ __device__ inline bf16_t small_const<bf16_t>(int v) {
  bf16_t r;
  r.x = v ? 0x3F80 : 0;
  return r;
}

template <typename T> __device__ __forceinline__ T zero_elem() { return (T)0; }
template <> __device__ __forceinline__ bf16_t zero_elem<bf16_t>() { bf16_t r; r.x = 0; return r; }

// ---- limits in the accumulate type (Reducer::init, csrc/cuda/reducer.cuh:46-55)
template <typename A> struct Lim;
template <> struct Lim<float> {
  __device__ static float max() { return 3.402823466e+38f; }
  __device__ static float lowest() { return -3.402823466e+38f; }
};
template <> struct Lim<double> {
  __device__ static double max() { return 1.7976931348623157e+308; }
  __device__ static double lowest() { return -1.7976931348623157e+308; }
};
template <> struct Lim<int32_t> {
  __device__ static int32_t max() { return INT32_MAX; }
  __device__ static int32_t lowest() { return INT32_MIN; }
};
template <> struct Lim<int64_t> {
  __device__ static int64_t max() { return INT64_MAX; }
  __device__ static int64_t lowest() { return INT64_MIN; }
};
template <> struct Lim<int16_t> {
  __device__ static int16_t max() { return INT16_MAX; }
  __device__ static int16_t lowest() { return INT16_MIN; }
};
template <> struct Lim<int8_t> {
  __device__ static int8_t max() { return INT8_MAX; }
  __device__ static int8_t lowest() { return INT8_MIN; }
};
template <> struct Lim<uint8_t> {
  __device__ static uint8_t max() { return UINT8_MAX; }
  __device__ static uint8_t lowest() { return 0; }
};

// limits in the element type itself (scatter accumulates in scalar_t)
template <typename T> struct ElemLim {
  __device__ static T max() { return Lim<T>::max(); }
  __device__ static T lowest() { return Lim<T>::lowest(); }
};
template <> struct ElemLim<bf16_t> {
  __device__ static bf16_t max() { bf16_t r; r.x = 0x7F7F; return r; }
  __device__ static bf16_t lowest() { bf16_t r; r.x = 0xFF7F; return r; }
};
template <> struct ElemLim<f16_t> {
  __device__ static f16_t max() { return (f16_t)65504.0f; }
  __device__ static f16_t lowest() { return (f16_t)-65504.0f; }
};

template <typename A, int REDUCE> __device__ __forceinline__ A acc_init() {
  if (REDUCE == TS_MUL || REDUCE == TS_DIV) return (A)1;
  if (REDUCE == TS_MIN) return Lim<A>::max();
  if (REDUCE == TS_MAX) return Lim<A>::lowest();
  return (A)0;
}

// A read of a 32-bit word of LDS that may change under the reader (tags, the value half of a packed key): not
// kept in a register across uses, and not a `volatile` access, which the compiler leaves in the generic address
// space (a flat load) and follows with a wait for every load the wavefront has in flight.
__device__ __forceinline__ uint32_t lds_peek(const uint32_t *p) {
  return __hip_atomic_load(p, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_WORKGROUP);
}
__device__ __forceinline__ int32_t lds_peek(const int32_t *p) {
  return __hip_atomic_load(p, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_WORKGROUP);
}

// ---- 16-byte vectors of VEC elements
template <typename T, int VEC> struct alignas(sizeof(T) * VEC) Vec { T v[VEC]; };

template <typename T, int VEC>
__device__ __forceinline__ Vec<T, VEC> load_vec(const T *p) {
  return *reinterpret_cast<const Vec<T, VEC> *>(p);
}
// streaming load: data that is read exactly once should not displace reusable
// lines (indptr tiles, output rows) from the caches
template <typename T, int VEC>
__device__ __forceinline__ Vec<T, VEC> load_vec_stream(const T *p) {
  typedef Vec<T, VEC> V;
  if constexpr (sizeof(V) == 16) {
    typedef uint32_t u4 __attribute__((ext_vector_type(4)));
    u4 r = __builtin_nontemporal_load(reinterpret_cast<const u4 *>(p));
    V out;
    __builtin_memcpy(&out, &r, 16);
    return out;
  } else if constexpr (sizeof(V) == 8) {
    typedef uint32_t u2 __attribute__((ext_vector_type(2)));
    u2 r = __builtin_nontemporal_load(reinterpret_cast<const u2 *>(p));
    V out;
    __builtin_memcpy(&out, &r, 8);
    return out;
  } else {
    return *reinterpret_cast<const V *>(p);
  }
}
template <typename T, int VEC>
__device__ __forceinline__ void store_vec(T *p, const Vec<T, VEC> &v) {
  *reinterpret_cast<Vec<T, VEC> *>(p) = v;
}
template <typename T, int VEC>
__device__ __forceinline__ void store_vec_stream(T *p, const Vec<T, VEC> &v) {
  typedef Vec<T, VEC> V;
  if constexpr (sizeof(V) == 16) {
    typedef uint32_t u4 __attribute__((ext_vector_type(4)));
    u4 r;
    __builtin_memcpy(&r, &v, 16);
    __builtin_nontemporal_store(r, reinterpret_cast<u4 *>(p));
  } else if constexpr (sizeof(V) == 8) {
    typedef uint32_t u2 __attribute__((ext_vector_type(2)));
    u2 r;
    __builtin_memcpy(&r, &v, 8);
    __builtin_nontemporal_store(r, reinterpret_cast<u2 *>(p));
  } else {
    *reinterpret_cast<V *>(p) = v;
  }
}

}  // namespace ts
