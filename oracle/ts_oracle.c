/*
 * TEST INFRASTRUCTURE ONLY -- CPU oracle for the scatter / segment / gather
 * reduction path. Nothing under oracle/ is part of the shipped library: only
 * the tests, the smoke check and the benchmark's cpu_baseline leg load it, and
 * only as the checker / the timed CPU baseline.
 *
 * It restates, in plain C, the single-threaded loops of the reference's CPU
 * path so that loop order, accumulate types and tie-breaking are the same:
 *   tso_scatter       csrc/cpu/scatter_cpu.cpp:52-83
 *   tso_segment_csr   csrc/cpu/segment_csr_cpu.cpp:54-88
 *   tso_gather_csr    csrc/cpu/segment_csr_cpu.cpp:141-159
 *   tso_segment_coo   csrc/cpu/segment_coo_cpu.cpp:78-137
 *   tso_gather_coo    csrc/cpu/segment_coo_cpu.cpp:186-211
 *   reducer rules     csrc/cpu/reducer.h:43-84
 *   index addressing  csrc/cpu/index_info.h:41-63
 * Shape checks, output allocation and the op-level maths (mean of scatter,
 * backward formulas) live in ts_oracle.py next to this file.
 *
 * Parity pins (see tests/test_oracle_*.py): every known-answer table of the
 * reference's tests, torch library equivalents, brute-force restatements on
 * tiny inputs, and -- where it builds -- the reference's own CPU objects in
 * oracle/_ref. Deliberately unpinned corners (undefined upstream): the arg of
 * a slot whose values never beat the initial value, 8-bit mean counts that
 * wrap to 0.
 */
#include <stdint.h>
#include <stdlib.h>
#include <float.h>
#include <limits.h>

#include "ts_oracle_types.h"

#define TSO_MAX_DIMS 25

typedef struct {
  const int64_t *data;
  int dims;
  int64_t sizes[TSO_MAX_DIMS];
  int64_t strides[TSO_MAX_DIMS];
} tso_index_info;

/* IndexToOffset::get, csrc/cpu/index_info.h:41-50 */
static inline int64_t tso_index_to_offset(int64_t idx, const tso_index_info *info) {
  int64_t offset = 0;
  for (int i = info->dims - 1; i >= 0; --i) {
    offset += (idx % info->sizes[i]) * info->strides[i];
    idx /= info->sizes[i];
  }
  return offset;
}

/* IndexPtrToOffset::get, csrc/cpu/index_info.h:52-63 */
static inline int64_t tso_indptr_to_offset(int64_t idx, const tso_index_info *info) {
  int64_t last = info->sizes[info->dims - 1] - 1;
  int64_t offset = (idx % last) * info->strides[info->dims - 1];
  idx /= last;
  for (int i = info->dims - 2; i >= 0; --i) {
    offset += (idx % info->sizes[i]) * info->strides[i];
    idx /= info->sizes[i];
  }
  return offset;
}

static int tso_fill_info(tso_index_info *info, const int64_t *data, int dims,
                         const int64_t *sizes, const int64_t *strides) {
  if (dims <= 0 || dims >= TSO_MAX_DIMS) return 1;
  info->data = data;
  info->dims = dims;
  for (int i = 0; i < dims; i++) {
    info->sizes[i] = sizes[i];
    info->strides[i] = strides[i];
  }
  return 0;
}

/* ---- Half / BFloat16 arithmetic: compute in float, round once per step ---- */
static inline tso_half h_from_f(float f) { return tso_float_to_half(f); }
static inline float h_to_f(tso_half h) { return tso_half_to_float(h); }
static inline tso_bf16 b_from_f(float f) { return tso_float_to_bf16(f); }
static inline float b_to_f(tso_bf16 h) { return tso_bf16_to_float(h); }
static inline tso_half h_const(uint16_t x) { tso_half h; h.x = x; return h; }
static inline tso_bf16 b_const(uint16_t x) { tso_bf16 h; h.x = x; return h; }

/* ---------------------------------------------------------------- float */
#define SFX f32
#define ST float
#define MT float
#define S2M(x) (x)
#define M2S(x) (x)
#define S_FROM_INT(c) ((float)(c))
#define S_ADD(a, b) ((a) + (b))
#define S_MUL(a, b) ((a) * (b))
#define S_DIV(a, b) ((a) / (b))
#define S_LT(a, b) ((a) < (b))
#define S_GT(a, b) ((a) > (b))
#define S_EQ(a, b) ((a) == (b))
#define M_ADD(a, b) ((a) + (b))
#define M_MUL(a, b) ((a) * (b))
#define M_DIV(a, b) ((a) / (b))
#define M_LT(a, b) ((a) < (b))
#define M_GT(a, b) ((a) > (b))
#define S_ZERO 0.0f
#define S_ONE 1.0f
#define S_MAX FLT_MAX
#define S_LOWEST (-FLT_MAX)
#define M_ZERO 0.0f
#define M_ONE 1.0f
#define M_MAX FLT_MAX
#define M_LOWEST (-FLT_MAX)
#define S_DIVISOR_IS_ZERO(x) 0
#include "ts_oracle_impl.inc"

/* --------------------------------------------------------------- double */
#define SFX f64
#define ST double
#define MT double
#define S2M(x) (x)
#define M2S(x) (x)
#define S_FROM_INT(c) ((double)(c))
#define S_ADD(a, b) ((a) + (b))
#define S_MUL(a, b) ((a) * (b))
#define S_DIV(a, b) ((a) / (b))
#define S_LT(a, b) ((a) < (b))
#define S_GT(a, b) ((a) > (b))
#define S_EQ(a, b) ((a) == (b))
#define M_ADD(a, b) ((a) + (b))
#define M_MUL(a, b) ((a) * (b))
#define M_DIV(a, b) ((a) / (b))
#define M_LT(a, b) ((a) < (b))
#define M_GT(a, b) ((a) > (b))
#define S_ZERO 0.0
#define S_ONE 1.0
#define S_MAX DBL_MAX
#define S_LOWEST (-DBL_MAX)
#define M_ZERO 0.0
#define M_ONE 1.0
#define M_MAX DBL_MAX
#define M_LOWEST (-DBL_MAX)
#define S_DIVISOR_IS_ZERO(x) 0
#include "ts_oracle_impl.inc"

/* ----------------------------------------------------------------- half */
#define SFX f16
#define ST tso_half
#define MT float
#define S2M(x) h_to_f(x)
#define M2S(x) h_from_f(x)
#define S_FROM_INT(c) h_from_f((float)(c))
#define S_ADD(a, b) h_from_f(h_to_f(a) + h_to_f(b))
#define S_MUL(a, b) h_from_f(h_to_f(a) * h_to_f(b))
#define S_DIV(a, b) h_from_f(h_to_f(a) / h_to_f(b))
#define S_LT(a, b) (h_to_f(a) < h_to_f(b))
#define S_GT(a, b) (h_to_f(a) > h_to_f(b))
#define S_EQ(a, b) (h_to_f(a) == h_to_f(b))
#define M_ADD(a, b) ((a) + (b))
#define M_MUL(a, b) ((a) * (b))
#define M_DIV(a, b) ((a) / (b))
#define M_LT(a, b) ((a) < (b))
#define M_GT(a, b) ((a) > (b))
#define S_ZERO h_const(0x0000)
#define S_ONE h_const(0x3C00)
#define S_MAX h_const(0x7BFF)    /* 65504 */
#define S_LOWEST h_const(0xFBFF) /* -65504 */
#define M_ZERO 0.0f
#define M_ONE 1.0f
#define M_MAX FLT_MAX
#define M_LOWEST (-FLT_MAX)
#define S_DIVISOR_IS_ZERO(x) 0
#include "ts_oracle_impl.inc"

/* ------------------------------------------------------------- bfloat16 */
#define SFX bf16
#define ST tso_bf16
#define MT float
#define S2M(x) b_to_f(x)
#define M2S(x) b_from_f(x)
#define S_FROM_INT(c) b_from_f((float)(c))
#define S_ADD(a, b) b_from_f(b_to_f(a) + b_to_f(b))
#define S_MUL(a, b) b_from_f(b_to_f(a) * b_to_f(b))
#define S_DIV(a, b) b_from_f(b_to_f(a) / b_to_f(b))
#define S_LT(a, b) (b_to_f(a) < b_to_f(b))
#define S_GT(a, b) (b_to_f(a) > b_to_f(b))
#define S_EQ(a, b) (b_to_f(a) == b_to_f(b))
#define M_ADD(a, b) ((a) + (b))
#define M_MUL(a, b) ((a) * (b))
#define M_DIV(a, b) ((a) / (b))
#define M_LT(a, b) ((a) < (b))
#define M_GT(a, b) ((a) > (b))
#define S_ZERO b_const(0x0000)
#define S_ONE b_const(0x3F80)
#define S_MAX b_const(0x7F7F)
#define S_LOWEST b_const(0xFF7F)
#define M_ZERO 0.0f
#define M_ONE 1.0f
#define M_MAX FLT_MAX
#define M_LOWEST (-FLT_MAX)
#define S_DIVISOR_IS_ZERO(x) 0
#include "ts_oracle_impl.inc"

/* ------------------------------------------------------ integer families.
 * C++ evaluates `a + b` on narrow integers in int and converts back, which
 * wraps; the casts below do the same. */
#define SFX i32
#define ST int32_t
#define MT int32_t
#define S2M(x) (x)
#define M2S(x) (x)
#define S_FROM_INT(c) ((int32_t)(c))
#define S_ADD(a, b) ((int32_t)((uint32_t)(a) + (uint32_t)(b)))
#define S_MUL(a, b) ((int32_t)((uint32_t)(a) * (uint32_t)(b)))
#define S_DIV(a, b) ((int32_t)((a) / (b)))
#define S_LT(a, b) ((a) < (b))
#define S_GT(a, b) ((a) > (b))
#define S_EQ(a, b) ((a) == (b))
#define M_ADD(a, b) S_ADD(a, b)
#define M_MUL(a, b) S_MUL(a, b)
#define M_DIV(a, b) S_DIV(a, b)
#define M_LT(a, b) ((a) < (b))
#define M_GT(a, b) ((a) > (b))
#define S_ZERO 0
#define S_ONE 1
#define S_MAX INT32_MAX
#define S_LOWEST INT32_MIN
#define M_ZERO 0
#define M_ONE 1
#define M_MAX INT32_MAX
#define M_LOWEST INT32_MIN
#define S_DIVISOR_IS_ZERO(x) ((x) == 0)
#include "ts_oracle_impl.inc"

#define SFX i64
#define ST int64_t
#define MT int64_t
#define S2M(x) (x)
#define M2S(x) (x)
#define S_FROM_INT(c) ((int64_t)(c))
#define S_ADD(a, b) ((int64_t)((uint64_t)(a) + (uint64_t)(b)))
#define S_MUL(a, b) ((int64_t)((uint64_t)(a) * (uint64_t)(b)))
#define S_DIV(a, b) ((int64_t)((a) / (b)))
#define S_LT(a, b) ((a) < (b))
#define S_GT(a, b) ((a) > (b))
#define S_EQ(a, b) ((a) == (b))
#define M_ADD(a, b) S_ADD(a, b)
#define M_MUL(a, b) S_MUL(a, b)
#define M_DIV(a, b) S_DIV(a, b)
#define M_LT(a, b) ((a) < (b))
#define M_GT(a, b) ((a) > (b))
#define S_ZERO 0
#define S_ONE 1
#define S_MAX INT64_MAX
#define S_LOWEST INT64_MIN
#define M_ZERO 0
#define M_ONE 1
#define M_MAX INT64_MAX
#define M_LOWEST INT64_MIN
#define S_DIVISOR_IS_ZERO(x) ((x) == 0)
#include "ts_oracle_impl.inc"

#define SFX i16
#define ST int16_t
#define MT int16_t
#define S2M(x) (x)
#define M2S(x) (x)
#define S_FROM_INT(c) ((int16_t)(c))
#define S_ADD(a, b) ((int16_t)((int)(a) + (int)(b)))
#define S_MUL(a, b) ((int16_t)((int)(a) * (int)(b)))
#define S_DIV(a, b) ((int16_t)((int)(a) / (int)(b)))
#define S_LT(a, b) ((a) < (b))
#define S_GT(a, b) ((a) > (b))
#define S_EQ(a, b) ((a) == (b))
#define M_ADD(a, b) S_ADD(a, b)
#define M_MUL(a, b) S_MUL(a, b)
#define M_DIV(a, b) S_DIV(a, b)
#define M_LT(a, b) ((a) < (b))
#define M_GT(a, b) ((a) > (b))
#define S_ZERO 0
#define S_ONE 1
#define S_MAX INT16_MAX
#define S_LOWEST INT16_MIN
#define M_ZERO 0
#define M_ONE 1
#define M_MAX INT16_MAX
#define M_LOWEST INT16_MIN
#define S_DIVISOR_IS_ZERO(x) ((x) == 0)
#include "ts_oracle_impl.inc"

#define SFX i8
#define ST int8_t
#define MT int8_t
#define S2M(x) (x)
#define M2S(x) (x)
#define S_FROM_INT(c) ((int8_t)(c))
#define S_ADD(a, b) ((int8_t)((int)(a) + (int)(b)))
#define S_MUL(a, b) ((int8_t)((int)(a) * (int)(b)))
#define S_DIV(a, b) ((int8_t)((int)(a) / (int)(b)))
#define S_LT(a, b) ((a) < (b))
#define S_GT(a, b) ((a) > (b))
#define S_EQ(a, b) ((a) == (b))
#define M_ADD(a, b) S_ADD(a, b)
#define M_MUL(a, b) S_MUL(a, b)
#define M_DIV(a, b) S_DIV(a, b)
#define M_LT(a, b) ((a) < (b))
#define M_GT(a, b) ((a) > (b))
#define S_ZERO 0
#define S_ONE 1
#define S_MAX INT8_MAX
#define S_LOWEST INT8_MIN
#define M_ZERO 0
#define M_ONE 1
#define M_MAX INT8_MAX
#define M_LOWEST INT8_MIN
#define S_DIVISOR_IS_ZERO(x) ((x) == 0)
#include "ts_oracle_impl.inc"

#define SFX u8
#define ST uint8_t
#define MT uint8_t
#define S2M(x) (x)
#define M2S(x) (x)
#define S_FROM_INT(c) ((uint8_t)(c))
#define S_ADD(a, b) ((uint8_t)((int)(a) + (int)(b)))
#define S_MUL(a, b) ((uint8_t)((int)(a) * (int)(b)))
#define S_DIV(a, b) ((uint8_t)((int)(a) / (int)(b)))
#define S_LT(a, b) ((a) < (b))
#define S_GT(a, b) ((a) > (b))
#define S_EQ(a, b) ((a) == (b))
#define M_ADD(a, b) S_ADD(a, b)
#define M_MUL(a, b) S_MUL(a, b)
#define M_DIV(a, b) S_DIV(a, b)
#define M_LT(a, b) ((a) < (b))
#define M_GT(a, b) ((a) > (b))
#define S_ZERO 0
#define S_ONE 1
#define S_MAX UINT8_MAX
#define S_LOWEST 0
#define M_ZERO 0
#define M_ONE 1
#define M_MAX UINT8_MAX
#define M_LOWEST 0
#define S_DIVISOR_IS_ZERO(x) ((x) == 0)
#include "ts_oracle_impl.inc"

/* ------------------------------------------------------------ dispatch */
static const int tso_elem_size[9] = {4, 8, 2, 2, 4, 8, 2, 1, 1};
static const int tso_math_size[9] = {4, 8, 4, 4, 4, 8, 2, 1, 1};

#define TSO_DISPATCH(dtype, CALL)                                              \
  switch (dtype) {                                                             \
  case TSO_F32: { CALL(f32, float, float) } break;                             \
  case TSO_F64: { CALL(f64, double, double) } break;                           \
  case TSO_F16: { CALL(f16, tso_half, float) } break;                          \
  case TSO_BF16: { CALL(bf16, tso_bf16, float) } break;                        \
  case TSO_I32: { CALL(i32, int32_t, int32_t) } break;                         \
  case TSO_I64: { CALL(i64, int64_t, int64_t) } break;                         \
  case TSO_I16: { CALL(i16, int16_t, int16_t) } break;                         \
  case TSO_I8: { CALL(i8, int8_t, int8_t) } break;                             \
  case TSO_U8: { CALL(u8, uint8_t, uint8_t) } break;                           \
  default: return 2;                                                           \
  }

int tso_elem_bytes(int dtype) {
  return (dtype >= 0 && dtype < 9) ? tso_elem_size[dtype] : -1;
}

/* Return codes: 0 ok, 1 "Input mismatch", 2 bad dtype/argument. */

int tso_scatter(const void *src, const int64_t *index, int index_dims,
                const int64_t *index_sizes, const int64_t *index_strides,
                void *out, int64_t *arg_out, int64_t B, int64_t E, int64_t K,
                int64_t N, int dtype, int reduce, int out_given) {
  tso_index_info info;
  if (tso_fill_info(&info, index, index_dims, index_sizes, index_strides)) return 2;
#define CALL(sfx, S, M)                                                        \
  scatter_##sfx((const S *)src, &info, (S *)out, arg_out, B, E, K, N, reduce,  \
                out_given);
  TSO_DISPATCH(dtype, CALL)
#undef CALL
  return 0;
}

int tso_segment_csr(const void *src, const int64_t *indptr, int indptr_dims,
                    const int64_t *indptr_sizes, const int64_t *indptr_strides,
                    void *out, int64_t *arg_out, int64_t N, int64_t K,
                    int64_t E, int dtype, int reduce) {
  tso_index_info info;
  if (tso_fill_info(&info, indptr, indptr_dims, indptr_sizes, indptr_strides)) return 2;
  if (dtype < 0 || dtype >= 9) return 2;
  void *vals = malloc((size_t)(K > 0 ? K : 1) * (size_t)tso_math_size[dtype]);
  int64_t *args = (int64_t *)malloc((size_t)(K > 0 ? K : 1) * sizeof(int64_t));
#define CALL(sfx, S, M)                                                        \
  segment_csr_##sfx((const S *)src, &info, (S *)out, arg_out, N, K, E, reduce, \
                    (M *)vals, args);
  TSO_DISPATCH(dtype, CALL)
#undef CALL
  free(vals);
  free(args);
  return 0;
}

int tso_gather_csr(const void *src, const int64_t *indptr, int indptr_dims,
                   const int64_t *indptr_sizes, const int64_t *indptr_strides,
                   void *out, int64_t N, int64_t K, int64_t E, int dtype) {
  tso_index_info info;
  if (tso_fill_info(&info, indptr, indptr_dims, indptr_sizes, indptr_strides)) return 2;
#define CALL(sfx, S, M) gather_csr_##sfx((const S *)src, &info, (S *)out, N, K, E);
  TSO_DISPATCH(dtype, CALL)
#undef CALL
  return 0;
}

int tso_segment_coo(const void *src, const int64_t *index, int index_dims,
                    const int64_t *index_sizes, const int64_t *index_strides,
                    void *out, void *second, int64_t B, int64_t E, int64_t K,
                    int64_t N, int dtype, int reduce, int out_given) {
  tso_index_info info;
  if (tso_fill_info(&info, index, index_dims, index_sizes, index_strides)) return 2;
  if (dtype < 0 || dtype >= 9) return 2;
  void *vals = malloc((size_t)(K > 0 ? K : 1) * (size_t)tso_math_size[dtype]);
  int64_t *args = (int64_t *)malloc((size_t)(K > 0 ? K : 1) * sizeof(int64_t));
#define CALL(sfx, S, M)                                                        \
  segment_coo_##sfx((const S *)src, &info, (S *)out, second, B, E, K, N,       \
                    reduce, out_given, (M *)vals, args);
  TSO_DISPATCH(dtype, CALL)
#undef CALL
  free(vals);
  free(args);
  return 0;
}

int tso_gather_coo(const void *src, const int64_t *index, int index_dims,
                   const int64_t *index_sizes, const int64_t *index_strides,
                   void *out, int64_t B, int64_t E, int64_t K, int64_t N,
                   int dtype) {
  tso_index_info info;
  int rc = 0;
  if (tso_fill_info(&info, index, index_dims, index_sizes, index_strides)) return 2;
#define CALL(sfx, S, M)                                                        \
  rc = gather_coo_##sfx((const S *)src, &info, (S *)out, B, E, K, N);
  TSO_DISPATCH(dtype, CALL)
#undef CALL
  return rc;
}
