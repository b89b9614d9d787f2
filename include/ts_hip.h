/*
 * ts_hip.h -- C ABI of the MI355X (gfx950) scatter / segment / gather kernels.
 *
 * This is the boundary a torch_scatter-style host layer binds against in place
 * of the reference's csrc/cuda launchers (scatter_cuda.h, segment_csr_cuda.h, segment_coo_cuda.h). Plain pointers and sizes only:
 * no torch types, no exceptions, no allocation, no host synchronisation. The
 * caller owns every buffer (device memory), holds the device guard and passes
 * the stream to launch on. Every function returns TS_OK or a TS_ERR_* code;
 * ts_error_string() turns a code into text.
 *
 * Shapes use the reference's flattening (csrc/cuda/scatter_cuda.cu:105-110,
 * segment_csr_cuda.cu:144-146, segment_coo_cuda.cu:208-212):
 *   B  product of the dimensions before the reduced dimension
 *   E  length of the reduced dimension of the edge-side tensor
 *   K  product of the trailing (feature) dimensions
 *   N  length of the reduced dimension of the node-side tensor
 * src/out are contiguous row-major [B, E|N, K]. index / indptr are int64.
 * arg outputs are int64 with E as the "empty slot" sentinel.
 */
#ifndef TS_HIP_H
#define TS_HIP_H

#include <stddef.h>
#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

typedef void *ts_stream_t; /* a hipStream_t; NULL is the default stream */

/* element types of src/out (AT_DISPATCH_ALL_TYPES_AND2(Half, BFloat16),
 * csrc/cuda/scatter_cuda.cu:114) */
enum ts_dtype {
  TS_F32 = 0, TS_F64 = 1, TS_F16 = 2, TS_BF16 = 3, TS_I32 = 4, TS_I64 = 5,
  TS_I16 = 6, TS_I8 = 7, TS_U8 = 8
};

/* reduction codes, same order as the reference enum (csrc/cuda/reducer.cuh:8) */
enum ts_reduce {
  TS_SUM = 0, TS_MEAN = 1, TS_MUL = 2, TS_DIV = 3, TS_MIN = 4, TS_MAX = 5
};

enum ts_status {
  TS_OK = 0,
  TS_ERR_BAD_ARG = 1,     /* null pointer, negative size, unknown code */
  TS_ERR_UNSUPPORTED = 2, /* combination this library has no kernel for */
  TS_ERR_WORKSPACE = 3,   /* workspace missing or too small */
  TS_ERR_LAUNCH = 4       /* the HIP runtime rejected a launch */
};

const char *ts_error_string(int status);

/* HIP_VERSION this library was built against.
 * Replaces scatter::cuda_version(), csrc/version.cpp:28-38. */
int64_t ts_hip_version(void);

/* ------------------------------------------------------------ segment_csr
 * out[b, n, :] = reduce over e in [indptr[b, n], indptr[b, n+1]) of src[b, e, :]
 * Replaces segment_csr_cuda, csrc/cuda/segment_csr_cuda.cu:97-168 (kernels
 * :15-95). Every row of out is written (empty row: 0, arg = E); mean divides
 * by max(count, 1). reduce in {SUM, MEAN, MIN, MAX}; arg_out is required for
 * MIN/MAX and ignored otherwise.
 *
 * indptr holds N+1 entries per batch row, unit inner stride;
 * indptr_batch_stride is the element distance between batch rows (0 when one
 * indptr row is shared by all batches).
 *
 * workspace: ts_segment_csr_workspace_bytes() bytes of device scratch for the
 * partial results of rows that cross a tile boundary.
 *
 * Status words: two uint64 at workspace + ts_segment_csr_workspace_bytes() -
 * TS_STATUS_BYTES (for ts_segment_coo and ts_segment_csr_permuted: the same
 * offset from the end of what their own *_workspace_bytes() report). Every
 * call writes a tag of its own (never 0) into word 0. A row that crosses tiles
 * is finished by the tile in which it ends, which waits (bounded) for the
 * partial results of the tiles before it; if that wait runs out -- row
 * pointers that are not monotone, an index that is not sorted, or a tile that
 * did not run for seconds -- the row is written as empty (0, arg = E; left
 * untouched with out_given) and the call's tag is written into word 1. After
 * the stream has finished, word 1 == word 0 means that the latest call gave at
 * least one row up (ts_status_gave_up below); anything else: every row is
 * complete. Neither write has to happen before the other, and what an earlier
 * call left in word 1 never equals a later call's tag. Nothing in the library
 * reads the words back: a caller that cannot vouch for its row pointers must
 * (16 bytes, device to host). The torch operators do so after every segment
 * call when the environment variable TS_CHECK_STATUS is set to 1, and raise.
 */
#define TS_STATUS_BYTES 256
/* words: a host copy of the two status words; 1 if the latest call gave a row up, else 0. Host arithmetic only:
 * no device call. No counterpart in the reference, whose kernels neither wait nor report. */
int ts_status_gave_up(const unsigned long long *words);
size_t ts_segment_csr_workspace_bytes(int64_t B, int64_t N, int64_t E, int64_t K,
                                      int dtype, int reduce);
int ts_segment_csr(const void *src, const int64_t *indptr, void *out,
                   int64_t *arg_out, int64_t B, int64_t N, int64_t E, int64_t K,
                   int64_t indptr_batch_stride, int dtype, int reduce,
                   void *workspace, size_t workspace_bytes, ts_stream_t stream);

/* ts_segment_csr without a workspace argument and without any allocation, for callers that cannot
 * allocate device memory (code under HIP graph capture, tight serving loops, harnesses that forbid
 * hipMalloc). It has no counterpart in the reference. Same kernels and same results as ts_segment_csr;
 * the partial results of rows that cross a tile boundary go to a device array of
 * TS_STATIC_SCRATCH_BYTES that the library holds on every GPU it runs on until the process ends.
 * Inputs whose ts_segment_csr_workspace_bytes() exceeds that size return TS_ERR_WORKSPACE and launch
 * nothing. All calls on one GPU share the array: calls that overlap in time on one GPU (two streams,
 * two threads) race; calls on one stream, one after the other, are safe. */
#define TS_STATIC_SCRATCH_BYTES (8u << 20)
int ts_segment_csr_static(const void *src, const int64_t *indptr, void *out,
                          int64_t *arg_out, int64_t B, int64_t N, int64_t E, int64_t K,
                          int64_t indptr_batch_stride, int dtype, int reduce,
                          ts_stream_t stream);

/* ------------------------------------------------------------- gather_csr
 * out[b, e, :] = src[b, n, :] for e in [indptr[b, n], indptr[b, n+1])
 * Replaces gather_csr_cuda, csrc/cuda/segment_csr_cuda.cu:219-281 (kernels
 * :170-217). Positions of out not covered by any row are left untouched.
 */
int ts_gather_csr(const void *src, const int64_t *indptr, void *out, int64_t B,
                  int64_t N, int64_t E, int64_t K, int64_t indptr_batch_stride,
                  int dtype, ts_stream_t stream);

/* Fused backward of segment_csr(mean):
 *   grad_in[b, e, :] = grad_out[b, n, :] / (T)max(count_n, 1)
 * One pass instead of the reference's gather + gather-of-count + divide,
 * SegmentMeanCSR::backward, csrc/segment_csr.cpp:94-111. The count is cast to
 * the element type before the division, as there. Floating types only.
 */
int ts_segment_mean_csr_backward(const void *grad_out, const int64_t *indptr,
                                 void *grad_in, int64_t B, int64_t N, int64_t E,
                                 int64_t K, int64_t indptr_batch_stride,
                                 int dtype, ts_stream_t stream);

/* ------------------------------------------------------------ segment_coo
 * Reduction keyed by a non-decreasing index (index[b, e] in [0, N)).
 * Replaces segment_coo_cuda, csrc/cuda/segment_coo_cuda.cu:152-283 (kernels
 * :14-150).
 *   out_given == 0: every row of out is written (row without entries: 0,
 *                   arg = E).
 *   out_given != 0: rows with entries are combined with their previous
 *                   content (sum: prev + sum; mean: (prev + sum) / count;
 *                   min/max: entries must strictly beat prev, else arg = E);
 *                   other rows are left untouched. arg_out must be pre-filled
 *                   with E by the caller in this mode.
 * count_out (MEAN only, may be NULL): [B, N] element-typed, max(count, 1).
 * index: unit inner stride, index_batch_stride elements between batch rows
 * (0 when shared).
 *
 * workspace: ts_segment_coo_workspace_bytes() bytes; holds the row-pointer
 * array derived from the index and the cross-tile partials.
 */
size_t ts_segment_coo_workspace_bytes(int64_t B, int64_t N, int64_t E, int64_t K,
                                      int dtype, int reduce);
int ts_segment_coo(const void *src, const int64_t *index, void *out,
                   void *arg_out, void *count_out, int64_t B, int64_t N,
                   int64_t E, int64_t K, int64_t index_batch_stride, int dtype,
                   int reduce, int out_given, void *workspace,
                   size_t workspace_bytes, ts_stream_t stream);

/* ------------------------------------------------------------- gather_coo
 * out[b, e, :] = src[b, index[b, e], :]
 * Replaces gather_coo_cuda, csrc/cuda/segment_coo_cuda.cu:327-382 (kernels
 * :285-325).
 */
int ts_gather_coo(const void *src, const int64_t *index, void *out, int64_t B,
                  int64_t N, int64_t E, int64_t K, int64_t index_batch_stride,
                  int dtype, ts_stream_t stream);

/* Fused backward of segment_coo(mean):
 *   grad_in[b, e, :] = grad_out[b, index[b,e], :] / count[b, index[b,e]]
 * SegmentMeanCOO::backward, csrc/segment_coo.cpp:99-112. count is the
 * element-typed [B, N] tensor the forward produced.
 */
int ts_segment_mean_coo_backward(const void *grad_out, const int64_t *index,
                                 const void *count, void *grad_in, int64_t B,
                                 int64_t N, int64_t E, int64_t K,
                                 int64_t index_batch_stride, int dtype,
                                 ts_stream_t stream);

/* ---------------------------------------------------------------- scatter
 * out[b, index[b,e,k], k] (op)= src[b, e, k]   for an unsorted index.
 * Replaces scatter_cuda, csrc/cuda/scatter_cuda.cu:58-138 (kernels :13-56),
 * including its helper passes: the initial fill, the init->0 masking and the
 * arg resolution. reduce in {SUM, MUL, MIN, MAX} (mean is sum + ts_scatter_count
 * + ts_divide_by_count, as ScatterMean does, csrc/scatter.cpp:115-161).
 *   out_given == 0: out is initialised by the call; untouched slots end as 0
 *                   (1 for MUL) with arg = E.
 *   out_given != 0: accumulate into out; arg_out (MIN/MAX) is fully written:
 *                   E where no entry strictly beat the previous content.
 * Ties keep the smallest e (the CPU rule, csrc/cpu/reducer.h:63-67).
 * SUM of 8- and 16-bit integers, and MUL of any type, have no hardware atomic: they loop on a compare-and-swap
 * of the word around the element, as the reference does (csrc/cuda/atomics.cuh), and that loop slows down with
 * the square of the entries that meet in one output row. For such sums a caller widens to int32 first (the
 * operator library does: the wrap-around of an int32 sum agrees with the narrow type's modulo 2^8 / 2^16);
 * products of 32- and 64-bit types and of 16-bit floats, one index per row, from 2^16 elements and rows of up
 * to 128 columns, meet in a table in LDS first and reach memory as one factor per row and workgroup (100 k
 * entries of 8 floats, 30 % of them on one row: 112 ms -> 0.3 ms; floating-point products are accumulated
 * in fp64 there, so fewer roundings than the reference's factor-by-factor loop); the others combine inside the
 * wavefront before the loop.
 * The index element of (b, e, k) is index[b*sb + e*se + k*sk]; a 1-D index
 * broadcast along dim is sb = 0, se = 1, sk = 0.
 */
int ts_scatter(const void *src, const int64_t *index, void *out,
               int64_t *arg_out, int64_t B, int64_t E, int64_t K, int64_t N,
               int64_t index_stride_b, int64_t index_stride_e,
               int64_t index_stride_k, int dtype, int reduce, int out_given,
               ts_stream_t stream);

/* ts_scatter with an optional workspace (ts_scatter_workspace_bytes; 0 = no use for one). With it,
 * MIN / MAX of large inputs with rows of 64 bytes and more, and SUM of such rows under an index that
 * is not sorted, first bin the entries by bucket of output rows (8 bytes per entry) and reduce every
 * bucket in LDS: no atomics on the table in memory except one write-back per chunk. MIN / MAX of
 * other large inputs of 4-byte elements with few entries per output row ask for 256 bytes: one flag,
 * written by a sample of the index, that picks the kernel for a skewed or an even index; so do SUMs
 * at the sizes that go through the accumulator table in LDS (from 2^23 elements on the sample keeps a
 * sorted index with the kernel that combines its runs: about twice as fast). SUM of up to four floats
 * or int32 per entry: from 2^21 entries the values travel with their bucket (8 bytes of scratch per entry
 * for one value, 4 * (K + 1) for several). SUM of one float or int32 per entry (K == 1, B == 1, N <= 524288, contiguous index, src and
 * index on 16-byte borders) from 2^19 entries: every workgroup keeps a table in LDS and hands it over in a
 * slab of the workspace instead of writing it back with atomics. MIN / MAX: same
 * results as ts_scatter; SUM: the same sum in another order of additions. No counterpart in the reference
 * (scatter_cuda allocates nothing beyond its outputs, csrc/cuda/scatter_cuda.cu:54-138). */
size_t ts_scatter_workspace_bytes(int64_t B, int64_t E, int64_t K, int64_t N,
                                  int dtype, int reduce);
/* MIN / MAX of one 4-byte value per entry (K == 1, B == 1, E >= 16384, N <= 524288) keep their table of packed
 * keys in the first ts_scatter_workspace_zero_bytes() bytes of the workspace instead of in arg_out. That part has
 * one size (4 MiB) for every such call, whatever N, so a workspace kept across calls with different N stays
 * valid: everything a call writes behind it (its slabs) is never read as zero by a later call. The last
 * TS_STATUS_BYTES of that part are not keys but one uint64 that the call sets to 1, and nobody resets, if one
 * of the two bounded waits inside the kernel ran out (a lane waiting about a second for room in a queue in
 * LDS): then entries were lost and the result is not to be trusted; the caller clears the word with the rest
 * of the part. The torch operators read it after such a call when TS_CHECK_STATUS=1 is set. Those bytes
 * must read as zero when ts_scatter_with_workspace starts, and the call puts them back to zero before it ends:
 * a caller that keeps its workspace from call to call (one per stream) clears it once and never pays for an
 * initial fill again; a caller that takes fresh memory for every call clears that part first
 * (hipMemsetAsync on the same stream). 0: no such part. No counterpart in the reference. */
size_t ts_scatter_workspace_zero_bytes(int64_t B, int64_t E, int64_t K, int64_t N,
                                       int dtype, int reduce);
int ts_scatter_with_workspace(const void *src, const int64_t *index, void *out,
                              int64_t *arg_out, int64_t B, int64_t E, int64_t K,
                              int64_t N, int64_t index_stride_b,
                              int64_t index_stride_e, int64_t index_stride_k,
                              int dtype, int reduce, int out_given, void *workspace,
                              size_t workspace_bytes, ts_stream_t stream);

/* Which kernels the last ts_scatter / ts_scatter_with_workspace call of the calling thread launched: a host-side
 * note for tests and tools (no device call, no synchronisation). Where two kernels are launched and a flag
 * written on the device picks the one that does the work (a sample or a full check of the index), the name says
 * both. No counterpart in the reference, which has one kernel per reduction (csrc/cuda/scatter_cuda.cu:13-56). */
enum ts_scatter_route {
  TS_ROUTE_NONE = 0,
  TS_ROUTE_SUM_ATOMIC = 1,               /* one atomic per element (per packed pair for 16-bit floats) */
  TS_ROUTE_SUM_RUNS = 2,                 /* runs of equal neighbouring indices combined in the wavefront, hot rows in LDS */
  TS_ROUTE_SUM_TABLE = 3,                /* accumulator table in LDS per workgroup */
  TS_ROUTE_SUM_TABLE_OR_RUNS = 4,        /* a sample of the index picks: table (unsorted) or runs (sorted) */
  TS_ROUTE_SUM_BUCKETS_OR_RUNS = 5,      /* workspace: entries binned by bucket of output rows; a sorted-looking index: runs */
  TS_ROUTE_SUM_BUCKETS_OR_SEGMENTED = 6, /* workspace: buckets; an index found sorted: the segmented reduction */
  TS_ROUTE_MUL_ATOMIC = 7,
  TS_ROUTE_MUL_TABLE = 8,
  TS_ROUTE_MINMAX_ATOMIC = 9,            /* packed 64-bit keys, one atomic max per element */
  TS_ROUTE_MINMAX_RUNS = 10,             /* runs combined in the wavefront first */
  TS_ROUTE_MINMAX_RUNS_OR_TABLE = 11,    /* a sample of the index picks: runs (even / sorted) or key table in LDS (skewed) */
  TS_ROUTE_MINMAX_TABLE = 12,            /* key table in LDS per workgroup */
  TS_ROUTE_MINMAX_TABLE_K1 = 13,         /* the same for one value per entry */
  TS_ROUTE_MINMAX_K1_SLABS = 14,         /* workspace, one value per entry: tables handed over in slabs */
  TS_ROUTE_MINMAX_BUCKETS = 15,          /* workspace: entries binned by bucket of output rows */
  TS_ROUTE_MINMAX_BUCKETS_OR_SEGMENTED = 16, /* the same; an index found sorted: the segmented reduction */
  TS_ROUTE_MINMAX_64BIT = 17,            /* 64-bit elements: value pass, then position pass */
  TS_ROUTE_SUM_VALUE_BUCKETS = 18,       /* workspace, one 4-byte value per entry: the values travel in the binned words;
                                            a sample of the index picks buckets (even), table (skewed) or runs (sorted) */
  TS_ROUTE_SUM_COUNT_RUNS = 19,          /* ts_scatter_sum_count_with_workspace below 2^16 elements: runs, the entries per
                                            output row counted by the same launch */
  TS_ROUTE_SUM_SLABS = 20                /* workspace, one 4-byte value per entry, 2^19 to 2^21 entries: a table per workgroup,
                                            handed over in slabs (no atomics for the write-back) */
};
/* Self-test of the fixed-pattern cross-lane helpers the kernels use (DPP row shifts, wave_shr:1,
 * v_permlane16_swap / v_permlane32_swap: csrc/dpp.h): one wavefront applies each helper to x = 3 * lane + 1 and
 * writes TS_LANE_OPS_ROWS rows of 64 int32 to out (device memory). tests/test_gpu_lane_ops.py holds the
 * expected rows. No counterpart in the reference, whose kernels shuffle (csrc/cuda/utils.cuh:38-47). */
#define TS_LANE_OPS_ROWS 17
int ts_selftest_lane_ops(int32_t *out, ts_stream_t stream);
int ts_scatter_last_route(void);
const char *ts_scatter_route_name(int route);

/* count[b, index[b*sb + e*se]] += 1 as int32 (exact for any group size below 2^31), count pre-zeroed by the
 * call. The count half of ScatterMean::forward, csrc/scatter.cpp:131-137, which sums ones in the element
 * type: equal wherever that sum is exact (any size for int32 / int64 / double), and exact beyond 2^24 entries
 * per group in float and 2^8 / 2^11 in bf16 / half, where a running total of ones in the element type stalls. */
int ts_scatter_count(const int64_t *index, int32_t *count, int64_t B, int64_t E,
                     int64_t N, int64_t index_stride_b, int64_t index_stride_e,
                     ts_stream_t stream);

/* The same count with scratch memory (ts_scatter_count_workspace_bytes; 0 = no use for it): from 2 M entries on an
 * unsorted index is binned by bucket of output rows (8 bytes per entry) and counted in LDS, as
 * ts_scatter_with_workspace does for the sum of one value per entry. Same result. */
size_t ts_scatter_count_workspace_bytes(int64_t B, int64_t E, int64_t N);
int ts_scatter_count_with_workspace(const int64_t *index, int32_t *count, int64_t B,
                                    int64_t E, int64_t N, int64_t index_stride_b,
                                    int64_t index_stride_e, void *workspace,
                                    size_t workspace_bytes, ts_stream_t stream);

/* Sum and entries per output row in one call: the two halves of ScatterMean::forward, csrc/scatter.cpp:122-141,
 * before its division, for one index per row (index[b * index_stride_b + e * index_stride_e]). out as
 * ts_scatter_with_workspace(reduce = sum, index_stride_k = 0) leaves it, count as ts_scatter_count leaves it. When
 * the sum goes through buckets of output rows (ts_scatter_sum_count_workspace_bytes() of scratch: wide rows from
 * 64 MB, single 4-byte values from 2 M entries) the index is read and binned once for both: the adding pass keeps
 * a table of counts beside its sums. Where the sum is one launch (runs below 2^16 elements, the table in LDS above,
 * see ts_scatter_route) that launch counts too, and one launch clears out and count. Every other case is the two
 * calls in a row. */
size_t ts_scatter_sum_count_workspace_bytes(int64_t B, int64_t E, int64_t K, int64_t N, int dtype);
int ts_scatter_sum_count_with_workspace(const void *src, const int64_t *index, void *out,
                                        int32_t *count, int64_t B, int64_t E, int64_t K, int64_t N,
                                        int64_t index_stride_b, int64_t index_stride_e,
                                        int dtype, int out_given, void *workspace,
                                        size_t workspace_bytes, ts_stream_t stream);

/* out[b, n, k] = out[b, n, k] / (T)max(count[b, n], 1): true division for
 * floating types, floor division for integers (csrc/scatter.cpp:138-141). */
int ts_divide_by_count(void *out, const int32_t *count, int64_t B, int64_t N,
                       int64_t K, int dtype, ts_stream_t stream);

/* Backward of every min/max flavour (csrc/scatter.cpp:184-196,
 * segment_coo.cpp:132-144, segment_csr.cpp:130-142):
 *   grad_in = 0; grad_in[b, arg[b,n,k], k] = grad_out[b,n,k] where arg < E.
 */
int ts_arg_backward(const void *grad_out, const int64_t *arg, void *grad_in,
                    int64_t B, int64_t N, int64_t E, int64_t K, int dtype,
                    ts_stream_t stream);

/* ---------------------------------------------------------- group softmax
 * Softmax / log-softmax over the entries that share an index, one index per
 * row (index[b*sb + e*se] addresses all K columns of entry e):
 *   m = group max, s = group sum of exp(src - m)
 *   log_space == 0:  out = exp(src - m) / s
 *   log_space != 0:  out = (src - m) - log(s + eps)
 * Replaces the op sequences of torch_scatter/composite/softmax.py:16-29 and
 * :45-59 (scatter_max, gather, sub, exp, scatter_sum, gather, div); the
 * reference has no single launcher for it. Three passes over src for an index
 * in any order. An index that is in order along E, with rows of up to 128
 * bytes and from 16 MB of input on (32 MB backward), takes one pass: tiles of
 * entries are finished in LDS, every tile checks the order of its part of the
 * index, and the three passes run behind them only if a tile found a descent
 * (the word at workspace + ts_group_softmax_workspace_bytes() - 256 is then
 * 1, else 0). That path
 * multiplies by the reciprocal of the group sum (fp32 / fp64: within 1 ulp of
 * the quotient). Floating types only. Entries whose index lies outside [0, N)
 * belong to no group and yield 0. The backward call takes the forward result:
 *   log_space == 0:  grad_in = result * (grad_out - S),  S = group sum of result * grad_out
 *   log_space != 0:  grad_in = grad_out - exp(result) * G,  G = group sum of grad_out
 * workspace: ts_group_softmax_workspace_bytes() bytes of device scratch,
 * 16-byte aligned. TS_ERR_UNSUPPORTED when B * N does not fit 31 bits.
 */
size_t ts_group_softmax_workspace_bytes(int64_t B, int64_t N, int64_t K,
                                        int dtype);
int ts_group_softmax(const void *src, const int64_t *index, void *out,
                     int64_t B, int64_t E, int64_t K, int64_t N,
                     int64_t index_stride_b, int64_t index_stride_e, int dtype,
                     int log_space, double eps, void *workspace,
                     size_t workspace_bytes, ts_stream_t stream);
int ts_group_softmax_backward(const void *result, const void *grad_out,
                              const int64_t *index, void *grad_in, int64_t B,
                              int64_t E, int64_t K, int64_t N,
                              int64_t index_stride_b, int64_t index_stride_e,
                              int dtype, int log_space, void *workspace,
                              size_t workspace_bytes, ts_stream_t stream);

/* logsumexp over the entries that share an index, one index per row:
 *   out[b, n, k] = log(sum_group exp(src - m) + eps) + m,  m = group max starting from -inf;
 *   NaN entries drop out; NaN and -inf results (empty groups) become 0, +inf the largest finite value.
 * Replaces the op sequence of torch_scatter/composite/logsumexp.py:8-57 for the call without `out`
 * (the reference has no single launcher for it). out is [B, N, K] and fully written when E > 0.
 * Backward: grad_in[b, e, k] = grad_out[b, n, k] * exp(src[b, e, k] - out[b, n, k]), n = index of e.
 * Workspace as for ts_group_softmax. Floating types only.
 */
int ts_group_logsumexp(const void *src, const int64_t *index, void *out,
                       int64_t B, int64_t E, int64_t K, int64_t N,
                       int64_t index_stride_b, int64_t index_stride_e,
                       int dtype, double eps, void *workspace,
                       size_t workspace_bytes, ts_stream_t stream);
int ts_group_logsumexp_backward(const void *src, const int64_t *index,
                                const void *out, const void *grad_out,
                                void *grad_in, int64_t B, int64_t E, int64_t K,
                                int64_t N, int64_t index_stride_b,
                                int64_t index_stride_e, int dtype,
                                ts_stream_t stream);
/* The same with ts_group_softmax_workspace_bytes() of scratch (result and grad_out of a group side by side). */
int ts_group_logsumexp_backward_with_workspace(const void *src, const int64_t *index, const void *out,
                                               const void *grad_out, void *grad_in, int64_t B, int64_t E,
                                               int64_t K, int64_t N, int64_t index_stride_b,
                                               int64_t index_stride_e, int dtype, void *workspace,
                                               size_t workspace_bytes, ts_stream_t stream);

/* Standard deviation over the entries that share an index, one index per row, given the group sums
 * `total` ([B, N, K], element type: ts_scatter with SUM) and the entries per group `count` ([B, N]
 * int32: ts_scatter_count):
 *   mean = total / max(count, 1);  out = sqrt(sum_group (src - mean)^2 / (d + 1e-6)),
 *   d = max(count - 1, 1) if unbiased else max(count, 1).
 * Replaces the second half of torch_scatter/composite/std.py:8-41 (gather of the mean, sub, mul,
 * scatter_sum, div, sqrt) for the call without `out`; the reference has no single launcher for it.
 * Backward: grad_in[b, e, k] = grad_out[b, n, k] * (src - mean) / (out[b, n, k] * (d + 1e-6)).
 * Workspace as for ts_group_softmax. Floating types only.
 */
int ts_group_std(const void *src, const int64_t *index, const void *total,
                 const int32_t *count, void *out, int64_t B, int64_t E, int64_t K,
                 int64_t N, int64_t index_stride_b, int64_t index_stride_e,
                 int dtype, int unbiased, void *workspace, size_t workspace_bytes,
                 ts_stream_t stream);
int ts_group_std_backward(const void *src, const int64_t *index,
                          const void *total, const int32_t *count,
                          const void *out, const void *grad_out, void *grad_in,
                          int64_t B, int64_t E, int64_t K, int64_t N,
                          int64_t index_stride_b, int64_t index_stride_e,
                          int dtype, int unbiased, ts_stream_t stream);
/* The same backward pass with ts_group_softmax_workspace_bytes() of scratch: what an entry needs of its group (mean and
 * grad_out / (out * divisor)) is first laid side by side, one memory line per entry instead of four under an index
 * that is not in order. Without workspace (null): as ts_group_std_backward. */
int ts_group_std_backward_with_workspace(const void *src, const int64_t *index, const void *total,
                                         const int32_t *count, const void *out, const void *grad_out,
                                         void *grad_in, int64_t B, int64_t E, int64_t K, int64_t N,
                                         int64_t index_stride_b, int64_t index_stride_e, int dtype,
                                         int unbiased, void *workspace, size_t workspace_bytes,
                                         ts_stream_t stream);

/* scatter_std and scatter_logsumexp through buckets of groups (no counterpart in the reference, whose
 * torch_scatter/composite/std.py:8-41 and logsumexp.py:8-57 compose scatter operators): the entries are binned
 * by bucket of neighbouring groups, then src is gathered once and both sweeps of the statistic run in LDS, whatever
 * the order of the index. ts_group_bins_workspace_bytes() is the scratch this takes, 0 when the route does not apply
 * (small inputs, rows held by more than 32 lanes, more groups than 16384 buckets hold).
 * ts_group_std_forward writes the group sums (total, element type), the entries per group (count, int32) and the
 * standard deviation (out) in one call: what ts_scatter(sum) + ts_scatter_count + ts_group_std leave. It needs that
 * workspace: TS_ERR_UNSUPPORTED when the route does not apply, TS_ERR_WORKSPACE when the workspace is too small.
 * ts_group_logsumexp takes the same route by itself when its workspace has that size. */
size_t ts_group_bins_workspace_bytes(int64_t B, int64_t E, int64_t K, int64_t N, int dtype);
/* The workspace with which every route of ts_group_softmax, ts_group_softmax_backward and ts_group_logsumexp is open
 * to a call of this shape: the three passes' part (ts_group_softmax_workspace_bytes), the buckets of groups where
 * they apply, and behind them the records of the one-pass tiles (which otherwise live in the three passes' part and
 * are declined when that is too small: few groups of many entries). Never smaller than either of the other two. */
size_t ts_group_workspace_bytes(int64_t B, int64_t E, int64_t K, int64_t N, int dtype);
int ts_group_std_forward(const void *src, const int64_t *index, void *total, int32_t *count, void *out,
                         int64_t B, int64_t E, int64_t K, int64_t N, int64_t index_stride_b,
                         int64_t index_stride_e, int dtype, int unbiased, void *workspace,
                         size_t workspace_bytes, ts_stream_t stream);

/* ---- index formats either side of the reductions. The reference has no operator for these steps:
 * its benchmark takes `row` and `rowptr` from the same sparse matrix (benchmark/scatter_segment.py:38-41)
 * and segment_coo's documentation asks the caller for a sorted index (torch_scatter/segment_coo.py:80-83).
 */

/* Sorted index [B, E] -> row pointers [B, N+1]: indptr[b, r] = first e with index[b, e] >= r. */
int ts_index_to_indptr(const int64_t *index, int64_t *indptr, int64_t B, int64_t E,
                       int64_t N, int64_t index_batch_stride, ts_stream_t stream);

/* Row pointers [B, N+1] -> sorted index [B, E] (E = indptr[b, N]): index[b, e] = r for
 * e in [indptr[b, r], indptr[b, r+1]). */
size_t ts_indptr_to_index_workspace_bytes(int64_t B, int64_t N);
int ts_indptr_to_index(const int64_t *indptr, int64_t *index, int64_t B, int64_t N,
                       int64_t E, int64_t indptr_batch_stride, void *workspace,
                       size_t workspace_bytes, ts_stream_t stream);

/* One-time stable sort of an unsorted index [E] with values in [0, N):
 *   perm[E] (int32): index[perm[0]] <= index[perm[1]] <= ..., equal values in order of position;
 *   indptr[N+1]: row pointers of the sorted order.
 * An index outside [0, N) sorts behind the last row: indptr[N] < E then tells the caller.
 * E, N < 2^31 - 1. */
size_t ts_sort_index_workspace_bytes(int64_t E, int64_t N);
int ts_sort_index(const int64_t *index, int32_t *perm, int64_t *indptr, int64_t E,
                  int64_t N, void *workspace, size_t workspace_bytes, ts_stream_t stream);

/* ts_segment_csr over permuted rows: entry e of the row-pointer order is row perm[b, e] of src,
 *   out[b, n, k] = reduce over e in [indptr[b, n], indptr[b, n+1]) of src[b, perm[b, e], k].
 * With perm / indptr from ts_sort_index this is scatter (csrc/cuda/scatter_cuda.cu:54-138) for an
 * index that is used many times: one pass over src, no atomics, the same bits on every call.
 * arg_out (MIN / MAX) holds positions in src's order (perm applied); ties keep the smallest position
 * as perm is stable. A slot without entries, or whose entries never beat scatter's initial value
 * (lowest() / max() of the element type), reads 0 with position E (csrc/cpu/scatter_cpu.cpp:81-82).
 * perm_batch_stride: 0 (one perm for all b) or E. */
size_t ts_segment_csr_permuted_workspace_bytes(int64_t B, int64_t N, int64_t E, int64_t K,
                                               int dtype, int reduce);
int ts_segment_csr_permuted(const void *src, const int32_t *perm, const int64_t *indptr,
                            void *out, int64_t *arg_out, int64_t B, int64_t N, int64_t E,
                            int64_t K, int64_t perm_batch_stride,
                            int64_t indptr_batch_stride, int dtype, int reduce,
                            void *workspace, size_t workspace_bytes, ts_stream_t stream);

#ifdef __cplusplus
}
#endif
#endif /* TS_HIP_H */
