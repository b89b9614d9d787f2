// The C ABI declared in include/ts_hip.h: argument checks, kernel plans and
// dispatch on the element type. Nothing here allocates or synchronises.
#include <hip/hip_runtime.h>
#include <hip/hip_version.h>
#include <stdlib.h>

#include <atomic>
#include <chrono>
#include <type_traits>

#include "csr_reduce.h"
#include "csr_gather.h"
#include "coo_gather.h"
#include "scatter.h"
#include "elementwise.h"
#include "group_softmax.h"
#include "index_format.h"

using namespace ts;

namespace {

const int kElemBytes[9] = {4, 8, 2, 2, 4, 8, 2, 1, 1};
const int kAccBytes[9] = {4, 8, 4, 4, 4, 8, 2, 1, 1};

inline bool valid_dtype(int d) { return d >= 0 && d < 9; }
inline bool aligned16(const void *p) { return (reinterpret_cast<uintptr_t>(p) & 15) == 0; }
inline bool is_float_dtype(int d) { return d == TS_F32 || d == TS_F64 || d == TS_F16 || d == TS_BF16; }

#define TS_DISPATCH(dtype, EXPR)                      \
  switch (dtype) {                                    \
  case TS_F32: { typedef float T; return EXPR; }      \
  case TS_F64: { typedef double T; return EXPR; }     \
  case TS_F16: { typedef f16_t T; return EXPR; }      \
  case TS_BF16: { typedef bf16_t T; return EXPR; }    \
  case TS_I32: { typedef int32_t T; return EXPR; }    \
  case TS_I64: { typedef int64_t T; return EXPR; }    \
  case TS_I16: { typedef int16_t T; return EXPR; }    \
  case TS_I8: { typedef int8_t T; return EXPR; }      \
  case TS_U8: { typedef uint8_t T; return EXPR; }     \
  default: return TS_ERR_BAD_ARG;                     \
  }

int dispatch_csr_reduce(int dtype, const CsrReduceArgs &a, const CsrPlan &p, int64_t B, int reduce,
                        hipStream_t s) {
  TS_DISPATCH(dtype, launch_csr_reduce<T>(a, p, B, reduce, s))
}
int dispatch_csr_gather(int dtype, const CsrGatherArgs &a, const CsrPlan &p, int64_t B, bool divide,
                        hipStream_t s) {
  TS_DISPATCH(dtype, launch_csr_gather<T>(a, p, B, divide, s))
}
int dispatch_coo_gather(int dtype, const CooGatherArgs &a, const CooGatherPlan &p, int64_t B,
                        bool divide, hipStream_t s) {
  TS_DISPATCH(dtype, launch_coo_gather<T>(a, p, B, divide, s))
}
int dispatch_scatter(int dtype, const ScatterArgs &a, int reduce, int vec, hipStream_t s) {
  TS_DISPATCH(dtype, launch_scatter<T>(a, reduce, vec, s))
}
int dispatch_divide(int dtype, void *out, const int32_t *count, int64_t rows, int64_t K, hipStream_t s) {
  TS_DISPATCH(dtype, launch_divide_by_count<T>(out, count, rows, K, s))
}
int dispatch_sorted_args(int dtype, void *out, int64_t *arg, const int32_t *perm, int64_t B, int64_t per_batch,
                         int64_t E, int64_t perm_batch_stride, bool is_max, hipStream_t s) {
  TS_DISPATCH(dtype, launch_sorted_args<T>(out, arg, perm, B, per_batch, E, perm_batch_stride, is_max, s))
}
int dispatch_arg_backward(int dtype, const void *g, const int64_t *arg, void *gi, int64_t B, int64_t N,
                          int64_t E, int64_t K, hipStream_t s) {
  TS_DISPATCH(dtype, launch_arg_backward<T>(g, arg, gi, B, N, E, K, s))
}

int dispatch_group_softmax(int dtype, const GroupArgs &g, int mode, int vec, hipStream_t s) {
  switch (dtype) {
  case TS_F32: return launch_group_softmax<float>(g, mode, vec, s);
  case TS_F64: return launch_group_softmax<double>(g, mode, vec, s);
  case TS_F16: return launch_group_softmax<f16_t>(g, mode, vec, s);
  case TS_BF16: return launch_group_softmax<bf16_t>(g, mode, vec, s);
  default: return TS_ERR_UNSUPPORTED;
  }
}

// The reductions keep edge positions in 32 bits inside a tile. B is only bounded by the 64-bit element
// offsets: kernels that put the batch into a grid dimension are launched in slices (for_batch_slices).
inline bool sizes_ok(int64_t B, int64_t N, int64_t E, int64_t K) {
  return B >= 0 && N >= 0 && E >= 0 && K >= 0 && E < 0x7FFFFFFFll && N < 0x7FFFFFFFll &&
         B < 0x7FFFFFFFll && K < ((int64_t)1 << 40);
}

// grid.y / grid.z hold at most 65535 workgroups: batches beyond that take further launches on the
// same stream. fn(first batch, number of batches) -> status.
constexpr int64_t kMaxGridBatches = 65535;
template <typename F> int for_batch_slices(int64_t B, F fn) {
  for (int64_t b0 = 0; b0 < B; b0 += kMaxGridBatches) {
    const int rc = fn(b0, B - b0 < kMaxGridBatches ? B - b0 : kMaxGridBatches);
    if (rc != TS_OK) return rc;
  }
  return TS_OK;
}
template <typename P> inline P *offset_bytes(P *p, int64_t bytes) {
  typedef typename std::conditional<std::is_const<P>::value, const char, char>::type C;
  return p == nullptr ? nullptr : reinterpret_cast<P *>(reinterpret_cast<C *>(p) + bytes);
}

int env_int(const char *name, int fallback) {
  const char *v = getenv(name);
  return v ? atoi(v) : fallback;
}

// Tag of one call's carry flags: a process-wide counter that starts at the clock, 1 .. 2^61.
uint64_t next_nonce() {
  static std::atomic<uint64_t> counter{(uint64_t)std::chrono::steady_clock::now().time_since_epoch().count()};
  return (counter.fetch_add(1, std::memory_order_relaxed) & ((1ull << 61) - 1)) + 1;
}

struct CsrWs {
  size_t total, off_args, off_meta;
};

CsrWs csr_workspace(const CsrPlan &p, int64_t B, int64_t K, int dtype, int reduce) {
  CsrWs w;
  w.total = csr_ws_bytes(p, B, K, kAccBytes[dtype], reduce == TS_MIN || reduce == TS_MAX, &w.off_args,
                         &w.off_meta);
  return w;
}

// Workspace for either plan: buffers that are not 16-byte aligned take one element per lane,
// which changes the tile size and with it the number of partial results.
// The last kStatusBytes of what the *_workspace_bytes functions report hold the call's status word.
constexpr size_t kStatusBytes = 256;
size_t csr_workspace_max(int64_t B, int64_t N, int64_t E, int64_t K, int dtype, int reduce, bool allow_small = true) {
  const bool wa = reduce == TS_MIN || reduce == TS_MAX;
  const size_t w1 = csr_workspace(csr_plan(N, E, K, kElemBytes[dtype], true, false, wa, allow_small), B, K, dtype, reduce).total;
  const size_t w0 = csr_workspace(csr_plan(N, E, K, kElemBytes[dtype], false, false, wa, allow_small), B, K, dtype, reduce).total;
  return (w1 > w0 ? w1 : w0) + kStatusBytes;
}
inline unsigned long long *status_word(void *ws, size_t reported_bytes) {
  return reinterpret_cast<unsigned long long *>(static_cast<char *>(ws) + reported_bytes - kStatusBytes);
}

int run_csr_reduce_slice(const void *src, const int64_t *indptr, void *out, int64_t *arg_out, void *count_out,
                         int64_t B, int64_t N, int64_t E, int64_t K, int64_t indptr_batch_stride, int dtype,
                         int reduce, int accumulate, void *ws, size_t ws_bytes, hipStream_t stream,
                         const int32_t *perm, int64_t perm_batch_stride, bool want_perm_args, bool *perm_args_done,
                         unsigned long long *status, bool status_reset, uint64_t status_nonce,
                         const int *gate = nullptr, int scatter_rule = 0) {
  const bool al = aligned16(src) && aligned16(out);
  // permuted rows always take the wide kernel (the narrow one stages consecutive entries), and so does a gated call
  const CsrPlan p = csr_plan(N, E, K, kElemBytes[dtype], al, false, reduce == TS_MIN || reduce == TS_MAX,
                             perm == nullptr && gate == nullptr && !scatter_rule);
  const CsrWs w = csr_workspace(p, B, K, dtype, reduce);
  if (ws == nullptr || ws_bytes < w.total) return TS_ERR_WORKSPACE;
  CsrReduceArgs a;
  a.src = src;
  a.indptr = indptr;
  a.out = out;
  a.arg_out = arg_out;
  a.count_out = count_out;
  a.N = N;
  a.E = E;
  a.K = K;
  a.indptr_batch_stride = indptr_batch_stride;
  a.accumulate = accumulate;
  a.G = p.G;
  a.BI = p.BI;
  a.ipw = p.ipw;
  a.nblk = p.nblk;
  a.ws_vals = ws;
  a.ws_args = reinterpret_cast<int32_t *>(static_cast<char *>(ws) + w.off_args);
  a.ws_meta = reinterpret_cast<int64_t *>(static_cast<char *>(ws) + w.off_meta);
  // rows that cross tiles are finished inside the kernel when the carries fit 32- / 64-bit atomics and the
  // four words of workspace per tile give every column chunk its flag; else by the second kernel
  a.lookback = !p.small && kAccBytes[dtype] >= 4 && p.ychunks <= 4 && p.nblk > 1 && env_int("TS_CSR_LOOKBACK", 1);
  a.nonce = next_nonce();
  a.status = status;
  a.status_reset = status_reset ? 1 : 0;
  a.status_nonce = status_nonce;
  a.carry_spin = env_int("TS_CSR_SPIN", kCarrySpin);  // test aid: -1 makes every look-back give up at once
  a.perm = perm;
  a.perm_batch_stride = perm_batch_stride;
  a.gate = gate;
  a.gate_want = 0;
  a.scatter_rule = scatter_rule;
  // every row is finished inside the first kernel unless the second one runs: then the positions can leave it
  // in src's order right away;
  // when the output is large: the lookup at every row end makes the wavefront wait, a pass over [N, K]
  // afterwards moves 20 bytes per element (C4, 3.2 M elements: 13 us as a pass, +17 us fused; 68 M: 334 vs 150 us)
  a.perm_args = perm != nullptr && (a.lookback || p.nblk <= 1) && want_perm_args;
  if (perm_args_done) *perm_args_done = a.perm_args != 0;
  if (p.ychunks > kMaxGridBatches) return TS_ERR_UNSUPPORTED;
  return dispatch_csr_reduce(dtype, a, p, B, reduce, stream);
}

int run_csr_reduce(const void *src, const int64_t *indptr, void *out, int64_t *arg_out, void *count_out,
                   int64_t B, int64_t N, int64_t E, int64_t K, int64_t indptr_batch_stride, int dtype,
                   int reduce, int accumulate, void *ws, size_t ws_bytes, unsigned long long *status,
                   hipStream_t stream, const int32_t *perm = nullptr, int64_t perm_batch_stride = 0,
                   bool *perm_args_done = nullptr, const int *gate = nullptr, int scatter_rule = 0) {
  const int64_t s = kElemBytes[dtype];
  const bool want_perm_args = B * N * K >= ((int64_t)8 << 20);
  const uint64_t status_nonce = next_nonce();  // one for all slices: the status words describe the whole call
  // every slice reuses the workspace: the launches follow each other on one stream
  return for_batch_slices(B, [&](int64_t b0, int64_t nb) {
    return run_csr_reduce_slice(offset_bytes(src, b0 * E * K * s), indptr + b0 * indptr_batch_stride,
                                offset_bytes(out, b0 * N * K * s), arg_out ? arg_out + b0 * N * K : nullptr,
                                offset_bytes(count_out, b0 * N * s), nb, N, E, K, indptr_batch_stride, dtype, reduce,
                                accumulate, ws, ws_bytes, stream, perm ? perm + b0 * perm_batch_stride : nullptr,
                                perm_batch_stride, want_perm_args, perm_args_done, status, b0 == 0, status_nonce, gate,
                                scatter_rule);
  });
}

// A scatter whose index turns out to be sorted (found by the count pass of the buckets) is finished by the
// segmented reduction instead: sorted index -> row pointers -> one pass over src without atomics, both gated on
// the device flag. The reduction must finish every row inside its first kernel (look-back), which needs 4- or
// 8-byte accumulators and at most four column chunks. Extra workspace behind that of the buckets: the row
// pointers, then the reduction's own.
struct SortedRoute {
  bool ok;
  size_t ptr_bytes, csr_bytes;
};
SortedRoute sorted_route_plan(int64_t B, int64_t E, int64_t K, int64_t N, int dtype, int reduce) {
  SortedRoute r = {false, 0, 0};
  if (!env_int("TS_SCATTER_SORTED_ROUTE", 1) || !env_int("TS_CSR_LOOKBACK", 1)) return r;
  if (reduce != TS_SUM && reduce != TS_MIN && reduce != TS_MAX) return r;
  if (kAccBytes[dtype] < 4 || B < 1 || E < 1) return r;
  const bool wa = reduce != TS_SUM;
  for (int al = 0; al < 2; ++al) {
    const CsrPlan p = csr_plan(N, E, K, kElemBytes[dtype], al != 0, false, wa, false);
    if (p.small || p.ychunks > 4) return r;
  }
  r.ptr_bytes = ((size_t)B * (N + 1) * 8 + 255) & ~(size_t)255;
  r.csr_bytes = csr_workspace_max(B, N, E, K, dtype, reduce, false) - kStatusBytes;
  r.ok = true;
  return r;
}

int run_csr_gather(int dtype, const CsrGatherArgs &args, const CsrPlan &p, int64_t B, bool divide, hipStream_t s) {
  if (p.ychunks > kMaxGridBatches) return TS_ERR_UNSUPPORTED;
  const int64_t sz = kElemBytes[dtype];
  return for_batch_slices(B, [&](int64_t b0, int64_t nb) {
    CsrGatherArgs a = args;
    a.src = offset_bytes(args.src, b0 * args.N * args.K * sz);
    a.indptr = args.indptr + b0 * args.indptr_batch_stride;
    a.out = offset_bytes(args.out, b0 * args.E * args.K * sz);
    return dispatch_csr_gather(dtype, a, p, nb, divide, s);
  });
}

int run_coo_gather(int dtype, const CooGatherArgs &args, const CooGatherPlan &p, int64_t B, bool divide,
                   hipStream_t s) {
  if (p.ychunks > kMaxGridBatches) return TS_ERR_UNSUPPORTED;
  const int64_t sz = kElemBytes[dtype];
  return for_batch_slices(B, [&](int64_t b0, int64_t nb) {
    CooGatherArgs a = args;
    a.src = offset_bytes(args.src, b0 * args.N * args.K * sz);
    a.index = args.index + b0 * args.index_batch_stride;
    a.count = offset_bytes(args.count, b0 * args.N * sz);
    a.out = offset_bytes(args.out, b0 * args.E * args.K * sz);
    return dispatch_coo_gather(dtype, a, p, nb, divide, s);
  });
}

// sorted index [B, E] -> row pointers [B, N + 1] (contiguous)
int run_coo_to_indptr(const int64_t *index, int64_t *ptr, int64_t B, int64_t E, int64_t N, int64_t index_batch_stride,
                      hipStream_t s, const int *gate = nullptr, int gate_want = 0) {
  const int per = E < ((int64_t)1 << 20) ? 1 : kCooPtrPerThread;
  const int64_t per_block = (int64_t)kBlock * per;
  return for_batch_slices(B, [&](int64_t b0, int64_t nb) {
    dim3 grid((unsigned)((E + 1 + per_block - 1) / per_block), (unsigned)nb);
    if (per == 1)
      hipLaunchKernelGGL(coo_to_indptr_kernel<1>, grid, dim3(kBlock), 0, s, index + b0 * index_batch_stride,
                         ptr + b0 * (N + 1), N, E, index_batch_stride, gate, gate_want);
    else
      hipLaunchKernelGGL(coo_to_indptr_kernel<kCooPtrPerThread>, grid, dim3(kBlock), 0, s,
                         index + b0 * index_batch_stride, ptr + b0 * (N + 1), N, E, index_batch_stride, gate, gate_want);
    return hipGetLastError() == hipSuccess ? (int)TS_OK : (int)TS_ERR_LAUNCH;
  });
}

}  // namespace

extern "C" {

namespace {
thread_local int g_scatter_route = TS_ROUTE_NONE;
}
void ts_note_scatter_route(int route) { g_scatter_route = route; }
int ts_scatter_last_route(void) { return g_scatter_route; }
const char *ts_scatter_route_name(int route) {
  static const char *const names[] = {
      "none", "sum: atomic", "sum: runs", "sum: table", "sum: table or runs (sample)", "sum: buckets or runs (sample)",
      "sum: buckets or segmented reduction (index checked)", "mul: atomic", "mul: table", "min/max: atomic",
      "min/max: runs", "min/max: runs or table (sample)", "min/max: table", "min/max: table, one value per entry",
      "min/max: slabs, one value per entry", "min/max: buckets", "min/max: buckets or segmented reduction (index checked)",
      "min/max: 64-bit elements, two passes", "sum: single values in buckets, table or runs (sample)",
      "sum: runs, entries per row counted by the same launch", "sum: single values, tables in slabs"};
  return route >= 0 && route < (int)(sizeof(names) / sizeof(names[0])) ? names[route] : "unknown";
}

namespace {
// every fixed-pattern cross-lane helper of dpp.h applied to x = 3 * lane + 1, one row of 64 results each
__global__ __launch_bounds__(kWave) void lane_ops_selftest_kernel(int32_t *out) {
  const int lane = threadIdx.x;
  const int x = 3 * lane + 1;
  int row = 0;
  out[64 * row++ + lane] = lane_up1(x);
  out[64 * row++ + lane] = lane_xor<1>(x);
  out[64 * row++ + lane] = lane_xor<2>(x);
  out[64 * row++ + lane] = lane_xor<4>(x);
  out[64 * row++ + lane] = lane_xor<8>(x);
  out[64 * row++ + lane] = lane_xor<16>(x);
  out[64 * row++ + lane] = lane_xor<32>(x);
  out[64 * row++ + lane] = lane_down<1>(x);
  out[64 * row++ + lane] = lane_down<2>(x);
  out[64 * row++ + lane] = lane_down<4>(x);
  out[64 * row++ + lane] = lane_down<8>(x);
  out[64 * row++ + lane] = lane_down<16>(x);
  out[64 * row++ + lane] = lane_down<32>(x);
  out[64 * row++ + lane] = wave_inclusive_sum(x);
  out[64 * row++ + lane] = (int)lane_up1_64(((int64_t)x << 32) | (uint32_t)(x + 7));
  out[64 * row++ + lane] = (int)(lane_up1_64(((int64_t)x << 32) | (uint32_t)(x + 7)) >> 32);
  float f = (float)x * 0.5f;
  out[64 * row++ + lane] = (int)(lane_xor<16>(f) * 2.0f);
}
}  // namespace

int ts_selftest_lane_ops(int32_t *out, ts_stream_t stream) {
  if (!out) return TS_ERR_BAD_ARG;
  hipLaunchKernelGGL(lane_ops_selftest_kernel, dim3(1), dim3(kWave), 0, static_cast<hipStream_t>(stream), out);
  return hipGetLastError() == hipSuccess ? TS_OK : TS_ERR_LAUNCH;
}

int ts_status_gave_up(const unsigned long long *words) {
  return words != nullptr && words[0] != 0 && words[1] == words[0];
}

const char *ts_error_string(int status) {
  switch (status) {
  case TS_OK: return "ok";
  case TS_ERR_BAD_ARG: return "bad argument (null pointer, negative size or unknown dtype/reduce code)";
  case TS_ERR_UNSUPPORTED: return "unsupported combination of dtype / reduce / size";
  case TS_ERR_WORKSPACE: return "workspace missing or too small";
  case TS_ERR_LAUNCH: return "HIP kernel launch failed";
  default: return "unknown status";
  }
}

int64_t ts_hip_version(void) { return HIP_VERSION; }


size_t ts_segment_csr_workspace_bytes(int64_t B, int64_t N, int64_t E, int64_t K, int dtype, int reduce) {
  if (!valid_dtype(dtype) || !sizes_ok(B, N, E, K)) return 0;
  // the plan may fall back to one element per lane for unaligned buffers; the
  // tile count does not depend on that choice
  return csr_workspace_max(B, N, E, K, dtype, reduce);
}

int ts_segment_csr(const void *src, const int64_t *indptr, void *out, int64_t *arg_out, int64_t B,
                   int64_t N, int64_t E, int64_t K, int64_t indptr_batch_stride, int dtype, int reduce,
                   void *workspace, size_t workspace_bytes, ts_stream_t stream) {
  if (!valid_dtype(dtype) || !sizes_ok(B, N, E, K)) return TS_ERR_BAD_ARG;
  if (reduce != TS_SUM && reduce != TS_MEAN && reduce != TS_MIN && reduce != TS_MAX) return TS_ERR_UNSUPPORTED;
  if (B * N * K == 0) return TS_OK;
  if (!indptr || !out || (E * K > 0 && !src)) return TS_ERR_BAD_ARG;
  if ((reduce == TS_MIN || reduce == TS_MAX) && !arg_out) return TS_ERR_BAD_ARG;
  const size_t need = csr_workspace_max(B, N, E, K, dtype, reduce);
  if (!workspace || workspace_bytes < need) return TS_ERR_WORKSPACE;
  return run_csr_reduce(src, indptr, out, arg_out, nullptr, B, N, E, K, indptr_batch_stride, dtype, reduce, 0,
                        workspace, need - kStatusBytes, status_word(workspace, need), static_cast<hipStream_t>(stream));
}

int ts_gather_csr(const void *src, const int64_t *indptr, void *out, int64_t B, int64_t N, int64_t E,
                  int64_t K, int64_t indptr_batch_stride, int dtype, ts_stream_t stream) {
  if (!valid_dtype(dtype) || !sizes_ok(B, N, E, K)) return TS_ERR_BAD_ARG;
  if (B * E * K == 0 || N == 0) return TS_OK;
  if (!src || !indptr || !out) return TS_ERR_BAD_ARG;
  const CsrPlan p = csr_plan(N, E, K, kElemBytes[dtype], aligned16(src) && aligned16(out), true);
  CsrGatherArgs a;
  a.src = src;
  a.indptr = indptr;
  a.out = out;
  a.N = N;
  a.E = E;
  a.K = K;
  a.indptr_batch_stride = indptr_batch_stride;
  a.G = p.G;
  a.BI = p.BI;
  a.ipw = p.ipw;
  a.nblk = p.nblk;
  return run_csr_gather(dtype, a, p, B, false, static_cast<hipStream_t>(stream));
}

int ts_segment_mean_csr_backward(const void *grad_out, const int64_t *indptr, void *grad_in, int64_t B,
                                 int64_t N, int64_t E, int64_t K, int64_t indptr_batch_stride, int dtype,
                                 ts_stream_t stream) {
  if (!valid_dtype(dtype) || !sizes_ok(B, N, E, K)) return TS_ERR_BAD_ARG;
  if (!is_float_dtype(dtype)) return TS_ERR_UNSUPPORTED;
  if (B * E * K == 0 || N == 0) return TS_OK;
  if (!grad_out || !indptr || !grad_in) return TS_ERR_BAD_ARG;
  const CsrPlan p = csr_plan(N, E, K, kElemBytes[dtype], aligned16(grad_out) && aligned16(grad_in), true, true);
  CsrGatherArgs a;
  a.src = grad_out;
  a.indptr = indptr;
  a.out = grad_in;
  a.N = N;
  a.E = E;
  a.K = K;
  a.indptr_batch_stride = indptr_batch_stride;
  a.G = p.G;
  a.BI = p.BI;
  a.ipw = p.ipw;
  a.nblk = p.nblk;
  return run_csr_gather(dtype, a, p, B, true, static_cast<hipStream_t>(stream));
}

// ---- ts_segment_csr for callers that cannot allocate: the partial results of rows that cross tiles
// live in a file-scope device array instead of a caller's workspace. Every GPU holds its own copy
// of the array at its own address; the address is looked up once per device, with that device current.
constexpr size_t kStaticScratchBytes = (size_t)TS_STATIC_SCRATCH_BYTES;
constexpr int kStaticScratchDevices = 64;
static __device__ __align__(256) unsigned char scratch[kStaticScratchBytes];
static std::atomic<void *> g_scratch_ptr[kStaticScratchDevices];

static int static_scratch_ptr(void **out) {
  int dev = -1;
  if (hipGetDevice(&dev) != hipSuccess || dev < 0 || dev >= kStaticScratchDevices) return TS_ERR_LAUNCH;
  void *p = g_scratch_ptr[dev].load(std::memory_order_acquire);
  if (p == nullptr) {
    if (hipGetSymbolAddress(&p, HIP_SYMBOL(scratch)) != hipSuccess || p == nullptr) return TS_ERR_LAUNCH;
    g_scratch_ptr[dev].store(p, std::memory_order_release);
  }
  *out = p;
  return TS_OK;
}

int ts_segment_csr_static(const void *src, const int64_t *indptr, void *out, int64_t *arg_out, int64_t B,
                          int64_t N, int64_t E, int64_t K, int64_t indptr_batch_stride, int dtype, int reduce,
                          ts_stream_t stream) {
  if (!valid_dtype(dtype) || !sizes_ok(B, N, E, K)) return TS_ERR_BAD_ARG;
  if (reduce != TS_SUM && reduce != TS_MEAN && reduce != TS_MIN && reduce != TS_MAX) return TS_ERR_UNSUPPORTED;
  if (B * N * K == 0) return TS_OK;
  if (!indptr || !out || (E * K > 0 && !src)) return TS_ERR_BAD_ARG;
  if ((reduce == TS_MIN || reduce == TS_MAX) && !arg_out) return TS_ERR_BAD_ARG;
  // the array is fixed in size: larger inputs must bring a workspace (ts_segment_csr)
  const size_t need = csr_workspace_max(B, N, E, K, dtype, reduce);
  if (need > kStaticScratchBytes) return TS_ERR_WORKSPACE;
  void *ws = nullptr;
  const int rc = static_scratch_ptr(&ws);
  if (rc != TS_OK) return rc;
  // Nothing in the array has to start at zero: the carry flags of a call hold that call's nonce, and
  // the second kernel only reads what the first one wrote in the same call.
  return run_csr_reduce(src, indptr, out, arg_out, nullptr, B, N, E, K, indptr_batch_stride, dtype, reduce, 0, ws,
                        need - kStatusBytes, status_word(ws, need), static_cast<hipStream_t>(stream));
}

size_t ts_segment_csr_permuted_workspace_bytes(int64_t B, int64_t N, int64_t E, int64_t K, int dtype, int reduce) {
  if (!valid_dtype(dtype) || !sizes_ok(B, N, E, K)) return 0;
  return csr_workspace_max(B, N, E, K, dtype, reduce, false);
}

int ts_segment_csr_permuted(const void *src, const int32_t *perm, const int64_t *indptr, void *out,
                            int64_t *arg_out, int64_t B, int64_t N, int64_t E, int64_t K,
                            int64_t perm_batch_stride, int64_t indptr_batch_stride, int dtype, int reduce,
                            void *workspace, size_t workspace_bytes, ts_stream_t stream) {
  if (!valid_dtype(dtype) || !sizes_ok(B, N, E, K)) return TS_ERR_BAD_ARG;
  if (reduce != TS_SUM && reduce != TS_MEAN && reduce != TS_MIN && reduce != TS_MAX) return TS_ERR_UNSUPPORTED;
  if (E >= 0x7FFFFFFFll) return TS_ERR_UNSUPPORTED;  // 32-bit row numbers
  if (B * N * K == 0) return TS_OK;
  if (!indptr || !out || (E * K > 0 && (!src || !perm))) return TS_ERR_BAD_ARG;
  if ((reduce == TS_MIN || reduce == TS_MAX) && !arg_out) return TS_ERR_BAD_ARG;
  hipStream_t s = static_cast<hipStream_t>(stream);
  bool args_done = false;
  const size_t need = csr_workspace_max(B, N, E, K, dtype, reduce, false);
  if (!workspace || workspace_bytes < need) return TS_ERR_WORKSPACE;
  const int rc = run_csr_reduce(src, indptr, out, arg_out, nullptr, B, N, E, K, indptr_batch_stride, dtype, reduce,
                                0, workspace, need - kStatusBytes, status_word(workspace, need), s, perm,
                                perm_batch_stride, &args_done);
  if (rc != TS_OK || (reduce != TS_MIN && reduce != TS_MAX) || args_done) return rc;
  return dispatch_sorted_args(dtype, out, arg_out, perm, B, N * K, E, perm_batch_stride, reduce == TS_MAX, s);
}

size_t ts_segment_coo_workspace_bytes(int64_t B, int64_t N, int64_t E, int64_t K, int dtype, int reduce) {
  if (!valid_dtype(dtype) || !sizes_ok(B, N, E, K)) return 0;
  const size_t ptr_bytes = ((size_t)B * (N + 1) * 8 + 255) & ~(size_t)255;
  return ptr_bytes + csr_workspace_max(B, N, E, K, dtype, reduce);
}

int ts_segment_coo(const void *src, const int64_t *index, void *out, void *arg_out, void *count_out,
                   int64_t B, int64_t N, int64_t E, int64_t K, int64_t index_batch_stride, int dtype,
                   int reduce, int out_given, void *workspace, size_t workspace_bytes, ts_stream_t stream) {
  if (!valid_dtype(dtype) || !sizes_ok(B, N, E, K)) return TS_ERR_BAD_ARG;
  if (reduce != TS_SUM && reduce != TS_MEAN && reduce != TS_MIN && reduce != TS_MAX) return TS_ERR_UNSUPPORTED;
  if (B * N * K == 0) return TS_OK;
  if (!out || (E > 0 && (!index || (K > 0 && !src)))) return TS_ERR_BAD_ARG;
  if ((reduce == TS_MIN || reduce == TS_MAX) && !arg_out) return TS_ERR_BAD_ARG;
  const size_t ptr_bytes = ((size_t)B * (N + 1) * 8 + 255) & ~(size_t)255;
  const size_t need = ptr_bytes + csr_workspace_max(B, N, E, K, dtype, reduce);
  if (!workspace || workspace_bytes < need) return TS_ERR_WORKSPACE;
  hipStream_t s = static_cast<hipStream_t>(stream);
  int64_t *ptr = static_cast<int64_t *>(workspace);
  const int rc = run_coo_to_indptr(index, ptr, B, E, N, index_batch_stride, s);
  if (rc != TS_OK) return rc;
  return run_csr_reduce(src, ptr, out, static_cast<int64_t *>(arg_out), count_out, B, N, E, K, N + 1, dtype,
                        reduce, out_given ? 1 : 0, static_cast<char *>(workspace) + ptr_bytes,
                        need - ptr_bytes - kStatusBytes, status_word(workspace, need), s);
}

int ts_gather_coo(const void *src, const int64_t *index, void *out, int64_t B, int64_t N, int64_t E,
                  int64_t K, int64_t index_batch_stride, int dtype, ts_stream_t stream) {
  if (!valid_dtype(dtype) || !sizes_ok(B, N, E, K)) return TS_ERR_BAD_ARG;
  if (B * E * K == 0 || N == 0) return TS_OK;
  if (!src || !index || !out) return TS_ERR_BAD_ARG;
  const CooGatherPlan p = coo_gather_plan(E, K, kElemBytes[dtype], aligned16(src) && aligned16(out));
  CooGatherArgs a;
  a.src = src;
  a.index = index;
  a.count = nullptr;
  a.out = out;
  a.N = N;
  a.E = E;
  a.K = K;
  a.index_batch_stride = index_batch_stride;
  a.G = p.G;
  a.epw = p.epw;
  return run_coo_gather(dtype, a, p, B, false, static_cast<hipStream_t>(stream));
}

int ts_segment_mean_coo_backward(const void *grad_out, const int64_t *index, const void *count,
                                 void *grad_in, int64_t B, int64_t N, int64_t E, int64_t K,
                                 int64_t index_batch_stride, int dtype, ts_stream_t stream) {
  if (!valid_dtype(dtype) || !sizes_ok(B, N, E, K)) return TS_ERR_BAD_ARG;
  if (!is_float_dtype(dtype)) return TS_ERR_UNSUPPORTED;
  if (B * E * K == 0 || N == 0) return TS_OK;
  if (!grad_out || !index || !count || !grad_in) return TS_ERR_BAD_ARG;
  const CooGatherPlan p = coo_gather_plan(E, K, kElemBytes[dtype], aligned16(grad_out) && aligned16(grad_in));
  CooGatherArgs a;
  a.src = grad_out;
  a.index = index;
  a.count = count;
  a.out = grad_in;
  a.N = N;
  a.E = E;
  a.K = K;
  a.index_batch_stride = index_batch_stride;
  a.G = p.G;
  a.epw = p.epw;
  return run_coo_gather(dtype, a, p, B, true, static_cast<hipStream_t>(stream));
}

size_t ts_scatter_workspace_bytes(int64_t B, int64_t E, int64_t K, int64_t N, int dtype, int reduce) {
  if (!valid_dtype(dtype) || !sizes_ok(B, N, E, K)) return 0;
  const bool any_size = env_int("TS_SCATTER_BINNED", 1) == 2;
  if (reduce == TS_MIN || reduce == TS_MAX) {
    if (kElemBytes[dtype] > 4) return 0;  // 64-bit elements do not use packed keys
    if (env_int("TS_SCATTER_LDS_K1", 1) && env_int("TS_SCATTER_LDS", 1)) {
      const size_t k1 = k1_plan(B, E, K, N, kElemBytes[dtype], nullptr, 0, env_int("TS_SCATTER_LDS", 1) == 2).bytes;
      if (k1 != 0) return k1;
    }
    const size_t binned = bin_plan(B, E, K, N, kElemBytes[dtype], nullptr, 0, any_size, 8, true).bytes;
    if (binned != 0) {
      const SortedRoute sr = sorted_route_plan(B, E, K, N, dtype, reduce);
      return binned + (sr.ok ? sr.ptr_bytes + sr.csr_bytes : 0);
    }
    // one flag for the sample of the index that picks the kernel when few entries meet in an output row
    const int probe = env_int("TS_SCATTER_SKEW", 1);
    return probe && skew_probe_shape(B, E, K, N, kElemBytes[dtype], probe == 2) ? 256 : 0;
  }
  if (reduce == TS_SUM && kAccBytes[dtype] >= 4) {  // table slots: int32 for int32, 8 bytes for the other types
    const size_t binned = bin_plan(B, E, K, N, kElemBytes[dtype], nullptr, 0, any_size, dtype == TS_I32 ? 4 : 8, false, true).bytes;
    if (binned == 0 && env_int("TS_SCATTER_LDS", 1)) {
      // one 4-byte value per entry: (row in bucket, value) words, 8 bytes of scratch per entry
      const size_t payload = bin_plan_payload(B, E, K, N, kElemBytes[dtype], nullptr, 0, any_size).bytes;
      if (payload != 0) return payload;
      // single 4-byte values from 2^19 entries: a table per workgroup, handed over in slabs (with room for the counts
      // of scatter mean)
      if ((dtype == TS_F32 || dtype == TS_I32) && env_int("TS_SCATTER_LDS", 1) == 1 && env_int("TS_SCATTER_SLABS", 1)) {
        const size_t slabs =
            s1_plan(B, E, K, N, kElemBytes[dtype], nullptr, 0, true, env_int("TS_SCATTER_SLABS", 1) == 2).bytes;
        if (slabs != 0) return slabs;
      }
    }
    if (binned == 0) {
      // one word for the sample of the index that keeps a sorted one away from the table kernel
      const bool table = (is_float_dtype(dtype) || dtype == TS_I32 || dtype == TS_I64) &&
                         env_int("TS_SCATTER_LDS", 1) == 1 && sum_table_by_size(B, E, K, N, kElemBytes[dtype]);
      return table ? 256 : 0;
    }
    const SortedRoute sr = sorted_route_plan(B, E, K, N, dtype, reduce);
    return binned + (sr.ok ? sr.ptr_bytes + sr.csr_bytes : 0);
  }
  return 0;
}

size_t ts_scatter_workspace_zero_bytes(int64_t B, int64_t E, int64_t K, int64_t N, int dtype, int reduce) {
  if (!valid_dtype(dtype) || !sizes_ok(B, N, E, K)) return 0;
  if ((reduce != TS_MIN && reduce != TS_MAX) || kElemBytes[dtype] > 4) return 0;
  if (!env_int("TS_SCATTER_LDS_K1", 1) || !env_int("TS_SCATTER_LDS", 1)) return 0;
  return k1_plan(B, E, K, N, kElemBytes[dtype], nullptr, 0, env_int("TS_SCATTER_LDS", 1) == 2).zero_bytes;
}

int ts_scatter(const void *src, const int64_t *index, void *out, int64_t *arg_out, int64_t B, int64_t E,
               int64_t K, int64_t N, int64_t index_stride_b, int64_t index_stride_e, int64_t index_stride_k,
               int dtype, int reduce, int out_given, ts_stream_t stream) {
  return ts_scatter_with_workspace(src, index, out, arg_out, B, E, K, N, index_stride_b, index_stride_e,
                                   index_stride_k, dtype, reduce, out_given, nullptr, 0, stream);
}

}  // extern "C"
namespace {
// ts_scatter_with_workspace; count_out / count_flag: see ScatterArgs (a sum through the buckets that counts as well)
int scatter_ws_impl(const void *src, const int64_t *index, void *out, int64_t *arg_out, int64_t B,
                    int64_t E, int64_t K, int64_t N, int64_t index_stride_b, int64_t index_stride_e,
                    int64_t index_stride_k, int dtype, int reduce, int out_given, void *workspace,
                    size_t workspace_bytes, ts_stream_t stream, int32_t *count_out, const int **count_flag,
                    int *count_done = nullptr) {
  if (!valid_dtype(dtype) || !sizes_ok(B, N, E, K)) return TS_ERR_BAD_ARG;
  if (reduce != TS_SUM && reduce != TS_MUL && reduce != TS_MIN && reduce != TS_MAX) return TS_ERR_UNSUPPORTED;
  if (B * N * K == 0) return TS_OK;
  if (!out || (B * E * K > 0 && (!src || !index))) return TS_ERR_BAD_ARG;
  if ((reduce == TS_MIN || reduce == TS_MAX) && !arg_out) return TS_ERR_BAD_ARG;
  ScatterArgs a;
  a.src = src;
  a.index = index;
  a.out = out;
  a.arg_out = arg_out;
  a.B = B;
  a.E = E;
  a.K = K;
  a.N = N;
  a.sb = index_stride_b;
  a.se = index_stride_e;
  a.sk = index_stride_k;
  a.out_given = out_given ? 1 : 0;
  a.count_out = count_out;
  a.count_flag = count_flag;
  a.count_done = count_done;
  a.precheck = env_int("TS_SCATTER_PRECHECK", 1);   // tuning aids
  a.lds_cache = env_int("TS_SCATTER_LDS", 1);
  a.lds_epb = env_int("TS_SCATTER_EPB", 0);
  a.run_reduce = env_int("TS_SCATTER_RUNS", 1);
  a.lds_k1 = env_int("TS_SCATTER_LDS_K1", 1);
  a.skew_probe = env_int("TS_SCATTER_SKEW", 1);  // tuning aid: 0 never, 2 at any size
  if (const int binned = env_int("TS_SCATTER_BINNED", 1)) {  // tuning aid: 0 never, 2 at any size
    a.bin_ws = workspace;
    a.bin_ws_bytes = workspace_bytes;
    a.bin_any_size = binned == 2;
  }
  const int full = kVecBytes / kElemBytes[dtype];
  const int vec = (full > 1 && K % full == 0 && aligned16(src)) ? full : 1;
  // sorted index: finished by the segmented reduction (see sorted_route_plan); its workspace lies behind the buckets'
  const int *route_flag = nullptr;
  size_t bin_bytes = 0;
  SortedRoute sr = {false, 0, 0};
  if (a.bin_ws != nullptr && !out_given && index_stride_k == 0 && index_stride_e == 1 && B * E * K > 0) {
    const bool any_size = a.bin_any_size != 0;
    if (reduce == TS_MIN || reduce == TS_MAX)
      bin_bytes = kElemBytes[dtype] > 4 ? 0 : bin_plan(B, E, K, N, kElemBytes[dtype], nullptr, 0, any_size, 8, true).bytes;
    else if (reduce == TS_SUM && kAccBytes[dtype] >= 4)
    {
      bin_bytes = bin_plan(B, E, K, N, kElemBytes[dtype], nullptr, 0, any_size, dtype == TS_I32 ? 4 : 8, false, true).bytes;
      if (bin_bytes == 0 && env_int("TS_SCATTER_LDS", 1))
        bin_bytes = bin_plan_payload(B, E, K, N, kElemBytes[dtype], nullptr, 0, any_size).bytes;
    }
    if (bin_bytes != 0) sr = sorted_route_plan(B, E, K, N, dtype, reduce);
    if (sr.ok && workspace_bytes >= bin_bytes + sr.ptr_bytes + sr.csr_bytes) {
      a.sorted_route = 1;
      a.route_flag = &route_flag;
      a.route_ptr = reinterpret_cast<int64_t *>(static_cast<char *>(workspace) + bin_bytes);
    }
  }
  if (reduce == TS_SUM && bin_bytes == 0 && workspace != nullptr && workspace_bytes >= 256 && aligned16(workspace))
    a.order_ws = static_cast<int *>(workspace);
  const int rc = dispatch_scatter(dtype, a, reduce, vec, static_cast<hipStream_t>(stream));
  if (rc != TS_OK || route_flag == nullptr) return rc;
  // the row pointers of a sorted index come from the place pass of the buckets (bin_place_kernel)
  hipStream_t s = static_cast<hipStream_t>(stream);
  return run_csr_reduce(src, a.route_ptr, out, arg_out, nullptr, B, N, E, K, N + 1, dtype, reduce, 0,
                        static_cast<char *>(workspace) + bin_bytes + sr.ptr_bytes, sr.csr_bytes, nullptr, s, nullptr, 0,
                        nullptr, route_flag, 1);
}
}  // namespace
extern "C" {

int ts_scatter_with_workspace(const void *src, const int64_t *index, void *out, int64_t *arg_out, int64_t B,
                              int64_t E, int64_t K, int64_t N, int64_t index_stride_b, int64_t index_stride_e,
                              int64_t index_stride_k, int dtype, int reduce, int out_given, void *workspace,
                              size_t workspace_bytes, ts_stream_t stream) {
  return scatter_ws_impl(src, index, out, arg_out, B, E, K, N, index_stride_b, index_stride_e, index_stride_k, dtype, reduce,
                         out_given, workspace, workspace_bytes, stream, nullptr, nullptr);
}

size_t ts_scatter_count_workspace_bytes(int64_t B, int64_t E, int64_t N) {
  if (B < 0 || E < 0 || N < 0 || !env_int("TS_SCATTER_LDS", 1) || !env_int("TS_SCATTER_BINNED", 1)) return 0;
  return bin_plan_payload(B, E, 1, N, 4, nullptr, 0, env_int("TS_SCATTER_BINNED", 1) == 2).bytes;
}

int ts_scatter_count(const int64_t *index, int32_t *count, int64_t B, int64_t E, int64_t N,
                     int64_t index_stride_b, int64_t index_stride_e, ts_stream_t stream) {
  return ts_scatter_count_with_workspace(index, count, B, E, N, index_stride_b, index_stride_e, nullptr, 0, stream);
}

int ts_scatter_count_with_workspace(const int64_t *index, int32_t *count, int64_t B, int64_t E, int64_t N,
                                    int64_t index_stride_b, int64_t index_stride_e, void *workspace,
                                    size_t workspace_bytes, ts_stream_t stream) {
  if (B < 0 || E < 0 || N < 0) return TS_ERR_BAD_ARG;
  if (B * N == 0) return TS_OK;
  if (!count || (B * E > 0 && !index)) return TS_ERR_BAD_ARG;
  hipStream_t s = static_cast<hipStream_t>(stream);
  hipLaunchKernelGGL(fill_kernel<int32_t>, dim3(grid_for(B * N)), dim3(kBlock), 0, s, count, B * N, (int32_t)0);
  if (B * E > 0) {
    // a sum of ones with K = 1: same kernels as scatter sum (src == nullptr adds 1.0 per entry)
    ScatterArgs a;
    a.src = nullptr;
    a.index = index;
    a.out = count;
    a.arg_out = nullptr;
    a.B = B;
    a.E = E;
    a.K = 1;
    a.N = N;
    a.sb = index_stride_b;
    a.se = index_stride_e;
    a.sk = 0;
    a.out_given = 1;
    a.precheck = 1;
    a.lds_cache = env_int("TS_SCATTER_LDS", 1);
    a.lds_epb = env_int("TS_SCATTER_EPB", 0);
    bool binned = false, three_way = false;
    // A large count under an unsorted index, given scratch: the entries are binned by bucket of output rows like a sum
    // of one value per entry (bin_plan_payload; the "value" of an entry is 1) instead of one device atomic per entry
    // that misses the table. A sample of the index decides; the kernels below then run only for an index that looks sorted.
    if (workspace != nullptr && a.lds_cache && env_int("TS_SCATTER_BINNED", 1) && env_int("TS_SCATTER_RUNS", 1) &&
        B * N < 0x7FFFFFFFll) {  // (the kernels behind it that can be told to stand back)
      const BinPlan bp = bin_plan_payload(B, E, 1, N, 4, workspace, workspace_bytes, env_int("TS_SCATTER_BINNED", 1) == 2);
      if (bp.ok) {
        // the sample of the index gives one of three answers: sorted (the run kernel below), skewed (the table
        // kernel below), even (the buckets); without the table kernel or the sample only the first and the last
        three_way = a.lds_cache == 1 && sum_table_by_size(B, E, 1, N, 4) && B * E >= 2 * kBinBlock &&
                    !getenv("TS_BIN_NO_SAMPLE");
        launch_binned_add<int32_t, 1>(a, bp.p, 0, s, 0, three_way);
        a.skip_flag = bp.p.unsorted;
        binned = true;
      }
    }
    // the sizes from which the sum of one float per entry goes through the accumulator table (a hub otherwise
    // costs an atomic on one address per entry: 4 M entries under a Zipf(1.2) index 1.3 ms against 0.08 ms)
    const bool contended = a.lds_cache == 2 || (a.lds_cache == 1 && sum_table_by_size(B, E, 1, N, 4));
    if (binned) {
      // behind the buckets: the table kernel for a skewed index (flag 2), the run kernel for a sorted one (flag 0)
      if (three_way) {
        ScatterArgs t = a;
        t.skip_want = 2;
        const int64_t epb = per_cu_chunk_edges(a.lds_epb, B * E, sum_table_min_chunk(1, 4), 131072);
        hipLaunchKernelGGL(scatter_add_lds_kernel<int32_t>, dim3((unsigned)((B * E + epb - 1) / epb)), dim3(kLdsAddBlock),
                           0, s, t, kLdsAccRows - 1, epb);
      }
      const RunGrid g = run_grid(B * E, 1, 1, 4);
      launch_add_run<int32_t, 1, 1>(a, g, s);
    } else if (contended && B * N < 0x7FFFFFFFll) {
      const int64_t epb = per_cu_chunk_edges(a.lds_epb, B * E, sum_table_min_chunk(1, 4), 131072);
      hipLaunchKernelGGL(scatter_add_lds_kernel<int32_t>, dim3((unsigned)((B * E + epb - 1) / epb)), dim3(kLdsAddBlock), 0,
                         s, a, kLdsAccRows - 1, epb);
    } else if (env_int("TS_SCATTER_RUNS", 1) && B * N < 0x7FFFFFFFll) {
      // runs of equal neighbouring indices (sorted input) are counted in the wavefront first
      const RunGrid g = run_grid(B * E, 1, 1, 4);
      launch_add_run<int32_t, 1, 1>(a, g, s);
    } else {
      hipLaunchKernelGGL(scatter_count_kernel, dim3(grid_for(B * E)), dim3(kBlock), 0, s, index, count, B, E, N,
                         index_stride_b, index_stride_e);
    }
  }
  return hipGetLastError() == hipSuccess ? TS_OK : TS_ERR_LAUNCH;
}

size_t ts_scatter_sum_count_workspace_bytes(int64_t B, int64_t E, int64_t K, int64_t N, int dtype) {
  const size_t sum = ts_scatter_workspace_bytes(B, E, K, N, dtype, TS_SUM);
  const size_t cnt = ts_scatter_count_workspace_bytes(B, E, N);
  return sum > cnt ? sum : cnt;
}

int ts_scatter_sum_count_with_workspace(const void *src, const int64_t *index, void *out, int32_t *count, int64_t B,
                                        int64_t E, int64_t K, int64_t N, int64_t index_stride_b,
                                        int64_t index_stride_e, int dtype, int out_given, void *workspace,
                                        size_t workspace_bytes, ts_stream_t stream) {
  if (!valid_dtype(dtype) || !sizes_ok(B, N, E, K)) return TS_ERR_BAD_ARG;
  if (B * N == 0) return TS_OK;
  if (!count) return TS_ERR_BAD_ARG;
  hipStream_t s = static_cast<hipStream_t>(stream);
  // The sum. If it goes through the buckets, their adding pass counts as well (one pass over the index for both) and
  // leaves the buckets' flag here: 1 = the buckets took the call.
  const int *flag = nullptr;
  bool may_fuse = B * E * K > 0 && workspace != nullptr && B * N < 0x7FFFFFFFll && env_int("TS_SCATTER_RUNS", 1) &&
                  env_int("TS_SCATTER_LDS", 1) && env_int("TS_SCATTER_BINNED", 1);
  if (may_fuse) {  // only where the sum has a plan for the buckets (else count is cleared by its own call below)
    const bool any_size = env_int("TS_SCATTER_BINNED", 1) == 2;
    bool planned = kAccBytes[dtype] >= 4 && bin_plan(B, E, K, N, kElemBytes[dtype], workspace, workspace_bytes, any_size,
                                                     dtype == TS_I32 ? 4 : 8, false, true).ok;
    if (!planned && K <= kBinPayloadCols && (dtype == TS_F32 || dtype == TS_I32))
      planned = bin_plan_payload(B, E, K, N, 4, workspace, workspace_bytes, any_size).ok;
    may_fuse = planned;
  }
  if (may_fuse)
    hipLaunchKernelGGL(fill_kernel<int32_t>, dim3(grid_for(B * N)), dim3(kBlock), 0, s, count, B * N, (int32_t)0);
  // (a small sum clears and counts by itself, in the launches that clear out and add: then `counted` reads 1)
  int counted = 0;
  const int rc = scatter_ws_impl(src, index, out, nullptr, B, E, K, N, index_stride_b, index_stride_e, 0, dtype, TS_SUM,
                                 out_given, workspace, workspace_bytes, stream, count, may_fuse ? &flag : nullptr, &counted);
  if (rc != TS_OK || counted == 1) return rc;
  if (flag == nullptr)  // another route: the count on its own (with its own fill)
    return ts_scatter_count_with_workspace(index, count, B, E, N, index_stride_b, index_stride_e, workspace, workspace_bytes,
                                           stream);
  // the kernels behind the buckets, for the counts: the table for a skewed index (flag 2, single values only), runs for
  // a sorted one (flag 0)
  ScatterArgs c;
  c.src = nullptr;
  c.index = index;
  c.out = count;
  c.arg_out = nullptr;
  c.B = B;
  c.E = E;
  c.K = 1;
  c.N = N;
  c.sb = index_stride_b;
  c.se = index_stride_e;
  c.sk = 0;
  c.out_given = 1;
  c.precheck = 1;
  c.lds_cache = env_int("TS_SCATTER_LDS", 1);
  c.lds_epb = env_int("TS_SCATTER_EPB", 0);
  c.skip_flag = flag;
  if (K <= kBinPayloadCols && counted != 2) {  // (the plans whose sample can answer "skewed"; 2: the sum's table counted)
    ScatterArgs t = c;
    t.skip_want = 2;
    const int64_t epb = per_cu_chunk_edges(c.lds_epb, B * E, sum_table_min_chunk(1, 4), 131072);
    hipLaunchKernelGGL(scatter_add_lds_kernel<int32_t>, dim3((unsigned)((B * E + epb - 1) / epb)), dim3(kLdsAddBlock), 0, s,
                       t, kLdsAccRows - 1, epb);
  }
  const RunGrid g = run_grid(B * E, 1, 1, 4);
  launch_add_run<int32_t, 1, 1>(c, g, s);
  return hipGetLastError() == hipSuccess ? TS_OK : TS_ERR_LAUNCH;
}

int ts_divide_by_count(void *out, const int32_t *count, int64_t B, int64_t N, int64_t K, int dtype,
                       ts_stream_t stream) {
  if (!valid_dtype(dtype) || B < 0 || N < 0 || K < 0) return TS_ERR_BAD_ARG;
  if (B * N * K == 0) return TS_OK;
  if (!out || !count) return TS_ERR_BAD_ARG;
  return dispatch_divide(dtype, out, count, B * N, K, static_cast<hipStream_t>(stream));
}

int ts_arg_backward(const void *grad_out, const int64_t *arg, void *grad_in, int64_t B, int64_t N, int64_t E,
                    int64_t K, int dtype, ts_stream_t stream) {
  if (!valid_dtype(dtype) || B < 0 || N < 0 || E < 0 || K < 0) return TS_ERR_BAD_ARG;
  if (B * E * K == 0) return TS_OK;
  if (!grad_in || (B * N * K > 0 && (!grad_out || !arg))) return TS_ERR_BAD_ARG;
  return dispatch_arg_backward(dtype, grad_out, arg, grad_in, B, N, E, K, static_cast<hipStream_t>(stream));
}

namespace {
// std / logsumexp backward with a workspace of ts_group_softmax_workspace_bytes(): the values an entry needs of its group
// are laid side by side first (one more launch over [B, N, K]) when there are at least as many entries as groups
bool group_coef_ok(int64_t B, int64_t E, int64_t N, int64_t K, int dtype, const void *ws, size_t ws_bytes) {
  if (ws == nullptr || (reinterpret_cast<uintptr_t>(ws) & 31) != 0 || !env_int("TS_GROUP_COEF", 1)) return false;
  if (E < N) return false;
  return ws_bytes >= (size_t)(B * N * K) * 2 * (kElemBytes[dtype] == 8 ? 8 : 4);
}
// columns per lane of the bucket kernels: 16 bytes when the row allows it
int group_bins_vec(int64_t K, int dtype, bool aligned) {
  const int full = kVecBytes / kElemBytes[dtype];
  return (full > 1 && K % full == 0 && aligned) ? full : 1;
}
// TS_GROUP_BINS (tuning aid): 0 the buckets of groups never take a call, 2 they take it at any size
GroupBinPlan group_bins_plan(int64_t B, int64_t E, int64_t K, int64_t N, int dtype, bool aligned, void *ws, size_t ws_bytes) {
  const int mode = env_int("TS_GROUP_BINS", 1);
  if (mode == 0) {
    GroupBinPlan r;
    r.ok = false;
    r.bytes = 0;
    return r;
  }
  // the buckets' scratch lies behind the workspace of the three passes (softmax keeps its keys, sums and flag there)
  const size_t front = group_workspace_bytes(B, N, K, kElemBytes[dtype]);
  GroupBinPlan r = group_bin_plan(B, E, K, N, kElemBytes[dtype], group_bins_vec(K, dtype, aligned),
                                  ws != nullptr && ws_bytes > front ? static_cast<char *>(ws) + front : nullptr,
                                  ws_bytes > front ? ws_bytes - front : 0, mode == 2);
  if (r.bytes > 0) r.bytes += front;
  return r;
}
// std / logsumexp: the one-pass tiles for an index in order, their scratch behind that of the buckets (at ws + skip).
// TS_GROUP_FUSED (tuning aid): 0 never, 2 at any size and whatever the index looks like.
FusedReducePlan group_tiles_plan(int64_t B, int64_t E, int64_t K, int64_t N, int dtype, bool aligned, void *ws,
                                 size_t ws_bytes, size_t skip) {
  const int mode = env_int("TS_GROUP_FUSED", 1);
  if (mode == 0 || skip == 0) {
    FusedReducePlan r;
    r.ok = false;
    r.bytes = 0;
    return r;
  }
  return group_reduce_fused_plan(B, E, K, N, kElemBytes[dtype], aligned,
                                 ws != nullptr && ws_bytes > skip ? static_cast<char *>(ws) + skip : nullptr,
                                 ws_bytes > skip ? ws_bytes - skip : 0, mode == 2);
}
}  // namespace

namespace {
int run_group_softmax(const void *src, const void *grad, const int64_t *index, void *out, int64_t B, int64_t E,
                      int64_t K, int64_t N, int64_t sb, int64_t se, int dtype, int mode, double eps, void *workspace,
                      size_t workspace_bytes, hipStream_t stream) {
  if (!valid_dtype(dtype) || !sizes_ok(B, N, E, K)) return TS_ERR_BAD_ARG;
  if (!is_float_dtype(dtype)) return TS_ERR_UNSUPPORTED;
  if (B * E * K == 0) return TS_OK;
  if (!src || !index || !out) return TS_ERR_BAD_ARG;
  if ((mode == GS_SOFTMAX_BWD || mode == GS_LOG_SOFTMAX_BWD) && !grad) return TS_ERR_BAD_ARG;
  if (N == 0 || B * N >= 0x7FFFFFFFll) return TS_ERR_UNSUPPORTED;
  const size_t need = group_workspace_bytes(B, N, K, kElemBytes[dtype]);
  if (!workspace || workspace_bytes < need || !aligned16(workspace)) return TS_ERR_WORKSPACE;
  GroupArgs g;
  g.src = src;
  g.grad = grad;
  g.index = index;
  g.out = out;
  g.gmax = workspace;
  // forward: a group's keys and sums side by side (the finish reads both with one line); backward: sums only
  const bool with_keys = mode == GS_SOFTMAX || mode == GS_LOG_SOFTMAX;
  g.gs = with_keys ? 2 * K : K;
  g.gsum = static_cast<char *>(workspace) + (with_keys ? (size_t)K * (kElemBytes[dtype] == 8 ? 8 : 4) : 0);
  g.B = B;
  g.E = E;
  g.K = K;
  g.N = N;
  g.sb = sb;
  g.se = se;
  g.eps = eps;
  g.node_out = nullptr;
  g.node_grad = nullptr;
  g.from_neg_inf = 0;
  g.total = nullptr;
  g.count = nullptr;
  g.unbiased = 0;
  g.ws_bytes = group_three_pass_bytes(B, N, K, kElemBytes[dtype]);
  g.flag = reinterpret_cast<int *>(static_cast<char *>(workspace) + g.ws_bytes);
  const int full = kVecBytes / kElemBytes[dtype];
  const bool al = aligned16(src) && aligned16(out) && (!grad || aligned16(grad));
  const int vec = (full > 1 && K % full == 0 && al) ? full : 1;
  // forward with a workspace of ts_group_bins_workspace_bytes(): an index that is not in order goes through buckets of groups
  GroupBinPlan plan;
  plan.ok = false;
  if (with_keys) {
    plan = group_bins_plan(B, E, K, N, dtype, al, workspace, workspace_bytes);
    // (rows of up to 128 bytes, where the one-pass tiles take an index in order: for wider rows the three passes are
    // ahead under a sorted index, 1 M x 128 floats 570 against 741 us, and behind under a random one, 663 against 449)
    // (nor for few groups of many entries in rows of more than 64 bytes, which the tiles decline as well: 4 M x 64 bf16
    // in 4 k groups, sorted, 890 against 1116 us)
    const int64_t row_bytes = K * kElemBytes[dtype];
    const bool tiles_cover = row_bytes <= 64 || (row_bytes <= kFusedRowBytes && E <= 64 * N);
    if (plan.ok && group_bins_vec(K, dtype, al) == vec && (tiles_cover || env_int("TS_GROUP_BINS", 1) == 2))
      g.bins = &plan.p;
  }
  // a workspace of ts_group_workspace_bytes(): what lies behind the three passes' (and the buckets') part is scratch
  // for the one-pass tiles
  const size_t used = plan.ok ? plan.bytes : need;
  if (workspace_bytes > used) {
    g.fused_ws = static_cast<char *>(workspace) + used;
    g.fused_ws_bytes = workspace_bytes - used;
  }
  return dispatch_group_softmax(dtype, g, mode, vec, stream);
}
}  // namespace

size_t ts_group_softmax_workspace_bytes(int64_t B, int64_t N, int64_t K, int dtype) {
  if (!valid_dtype(dtype) || B < 0 || N < 0 || K < 0) return 0;
  return group_workspace_bytes(B, N, K, kElemBytes[dtype]);
}

int ts_group_softmax(const void *src, const int64_t *index, void *out, int64_t B, int64_t E, int64_t K, int64_t N,
                     int64_t index_stride_b, int64_t index_stride_e, int dtype, int log_space, double eps,
                     void *workspace, size_t workspace_bytes, ts_stream_t stream) {
  return run_group_softmax(src, nullptr, index, out, B, E, K, N, index_stride_b, index_stride_e, dtype,
                           log_space ? GS_LOG_SOFTMAX : GS_SOFTMAX, eps, workspace, workspace_bytes,
                           static_cast<hipStream_t>(stream));
}

int ts_group_softmax_backward(const void *result, const void *grad_out, const int64_t *index, void *grad_in,
                              int64_t B, int64_t E, int64_t K, int64_t N, int64_t index_stride_b,
                              int64_t index_stride_e, int dtype, int log_space, void *workspace,
                              size_t workspace_bytes, ts_stream_t stream) {
  return run_group_softmax(result, grad_out, index, grad_in, B, E, K, N, index_stride_b, index_stride_e, dtype,
                           log_space ? GS_LOG_SOFTMAX_BWD : GS_SOFTMAX_BWD, 0.0, workspace, workspace_bytes,
                           static_cast<hipStream_t>(stream));
}

int ts_group_logsumexp(const void *src, const int64_t *index, void *out, int64_t B, int64_t E, int64_t K, int64_t N,
                       int64_t index_stride_b, int64_t index_stride_e, int dtype, double eps, void *workspace,
                       size_t workspace_bytes, ts_stream_t stream) {
  if (!valid_dtype(dtype) || !sizes_ok(B, N, E, K)) return TS_ERR_BAD_ARG;
  if (!is_float_dtype(dtype)) return TS_ERR_UNSUPPORTED;
  if (B * N * K == 0) return TS_OK;
  if (!out || (B * E * K > 0 && (!src || !index))) return TS_ERR_BAD_ARG;
  if (B * N >= 0x7FFFFFFFll) return TS_ERR_UNSUPPORTED;
  const size_t need = group_workspace_bytes(B, N, K, kElemBytes[dtype]);
  if (!workspace || workspace_bytes < need || !aligned16(workspace)) return TS_ERR_WORKSPACE;
  GroupArgs g = {};
  g.src = src;
  g.index = index;
  g.out = out;
  if (B * E * K > 0) {
    // a workspace of ts_group_bins_workspace_bytes(): one gather of src through buckets of groups
    const GroupBinPlan plan = group_bins_plan(B, E, K, N, dtype, aligned16(src), workspace, workspace_bytes);
    if (plan.ok) {
      g.B = B;
      g.E = E;
      g.K = K;
      g.N = N;
      g.sb = index_stride_b;
      g.se = index_stride_e;
      g.eps = eps;
      g.bins = &plan.p;
      const FusedReducePlan tiles = group_tiles_plan(B, E, K, N, dtype, aligned16(src), workspace, workspace_bytes, plan.bytes);
      if (tiles.ok) {
        g.tiles = &tiles.f;
        g.tiles_force = env_int("TS_GROUP_FUSED", 1) == 2;
      }
      return dispatch_group_softmax(dtype, g, GS_LSE_BINS, group_bins_vec(K, dtype, aligned16(src)),
                                    static_cast<hipStream_t>(stream));
    }
  }
  g.gmax = workspace;
  g.gs = 2 * K;  // a group's keys and sums side by side
  g.gsum = static_cast<char *>(workspace) + (size_t)K * (kElemBytes[dtype] == 8 ? 8 : 4);
  g.B = B;
  g.E = E;
  g.K = K;
  g.N = N;
  g.sb = index_stride_b;
  g.se = index_stride_e;
  g.eps = eps;
  g.from_neg_inf = 1;
  const int full = kVecBytes / kElemBytes[dtype];
  const int vec = (full > 1 && K % full == 0 && aligned16(src)) ? full : 1;
  return dispatch_group_softmax(dtype, g, GS_LSE, vec, static_cast<hipStream_t>(stream));
}

size_t ts_group_workspace_bytes(int64_t B, int64_t E, int64_t K, int64_t N, int dtype) {
  if (!valid_dtype(dtype) || !is_float_dtype(dtype) || !sizes_ok(B, N, E, K)) return 0;
  const size_t front = group_workspace_bytes(B, N, K, kElemBytes[dtype]);
  const size_t bins = group_bins_plan(B, E, K, N, dtype, true, nullptr, 0).bytes;
  const size_t base = bins > 0 ? bins : front;
  size_t tail = bins > 0 ? group_tiles_plan(B, E, K, N, dtype, true, nullptr, 0, bins).bytes : 0;
  const size_t soft = env_int("TS_GROUP_FUSED", 1) != 0 ? group_fused_scratch_bytes(B, E, K, kElemBytes[dtype]) : 0;
  if (soft > tail) tail = soft;
  return base + tail;
}

size_t ts_group_bins_workspace_bytes(int64_t B, int64_t E, int64_t K, int64_t N, int dtype) {
  if (!valid_dtype(dtype) || !is_float_dtype(dtype) || !sizes_ok(B, N, E, K)) return 0;
  const size_t bins = group_bins_plan(B, E, K, N, dtype, true, nullptr, 0).bytes;
  return bins + group_tiles_plan(B, E, K, N, dtype, true, nullptr, 0, bins).bytes;
}

int ts_group_std_forward(const void *src, const int64_t *index, void *total, int32_t *count, void *out, int64_t B,
                         int64_t E, int64_t K, int64_t N, int64_t index_stride_b, int64_t index_stride_e, int dtype,
                         int unbiased, void *workspace, size_t workspace_bytes, ts_stream_t stream) {
  if (!valid_dtype(dtype) || !sizes_ok(B, N, E, K)) return TS_ERR_BAD_ARG;
  if (!is_float_dtype(dtype)) return TS_ERR_UNSUPPORTED;
  if (B * N * K == 0) return TS_OK;
  if (!out || !total || !count || !src || !index) return TS_ERR_BAD_ARG;
  const bool al = aligned16(src);
  const GroupBinPlan plan = group_bins_plan(B, E, K, N, dtype, al, workspace, workspace_bytes);
  if (plan.bytes == 0) return TS_ERR_UNSUPPORTED;
  if (!plan.ok) return TS_ERR_WORKSPACE;
  GroupArgs g = {};
  g.src = src;
  g.index = index;
  g.out = out;
  g.total_w = total;
  g.count_w = count;
  g.unbiased = unbiased ? 1 : 0;
  g.B = B;
  g.E = E;
  g.K = K;
  g.N = N;
  g.sb = index_stride_b;
  g.se = index_stride_e;
  g.bins = &plan.p;
  const FusedReducePlan tiles = group_tiles_plan(B, E, K, N, dtype, al, workspace, workspace_bytes, plan.bytes);
  if (tiles.ok) {
    g.tiles = &tiles.f;
    g.tiles_force = env_int("TS_GROUP_FUSED", 1) == 2;
  }
  return dispatch_group_softmax(dtype, g, GS_STD_BINS, group_bins_vec(K, dtype, al), static_cast<hipStream_t>(stream));
}

int ts_group_logsumexp_backward(const void *src, const int64_t *index, const void *out, const void *grad_out,
                                void *grad_in, int64_t B, int64_t E, int64_t K, int64_t N, int64_t index_stride_b,
                                int64_t index_stride_e, int dtype, ts_stream_t stream) {
  return ts_group_logsumexp_backward_with_workspace(src, index, out, grad_out, grad_in, B, E, K, N, index_stride_b,
                                                    index_stride_e, dtype, nullptr, 0, stream);
}

int ts_group_logsumexp_backward_with_workspace(const void *src, const int64_t *index, const void *out,
                                               const void *grad_out, void *grad_in, int64_t B, int64_t E, int64_t K,
                                               int64_t N, int64_t index_stride_b, int64_t index_stride_e, int dtype,
                                               void *workspace, size_t workspace_bytes, ts_stream_t stream) {
  if (!valid_dtype(dtype) || !sizes_ok(B, N, E, K)) return TS_ERR_BAD_ARG;
  if (!is_float_dtype(dtype)) return TS_ERR_UNSUPPORTED;
  if (B * E * K == 0) return TS_OK;
  if (!src || !index || !out || !grad_out || !grad_in) return TS_ERR_BAD_ARG;
  if (N == 0 || B * N >= 0x7FFFFFFFll) return TS_ERR_UNSUPPORTED;
  GroupArgs g = {};
  g.src = src;
  g.index = index;
  g.out = grad_in;
  g.node_out = out;
  g.node_grad = grad_out;
  g.B = B;
  g.E = E;
  g.K = K;
  g.N = N;
  g.sb = index_stride_b;
  g.se = index_stride_e;
  const int full = kVecBytes / kElemBytes[dtype];
  const bool al = aligned16(src) && aligned16(grad_in) && aligned16(out) && aligned16(grad_out);
  const int vec = (full > 1 && K % full == 0 && al) ? full : 1;
  if (group_coef_ok(B, E, N, K, dtype, workspace, workspace_bytes)) g.coef = workspace;
  return dispatch_group_softmax(dtype, g, GS_LSE_BWD, vec, static_cast<hipStream_t>(stream));
}

int ts_group_std(const void *src, const int64_t *index, const void *total, const int32_t *count, void *out, int64_t B,
                 int64_t E, int64_t K, int64_t N, int64_t index_stride_b, int64_t index_stride_e, int dtype,
                 int unbiased, void *workspace, size_t workspace_bytes, ts_stream_t stream) {
  if (!valid_dtype(dtype) || !sizes_ok(B, N, E, K)) return TS_ERR_BAD_ARG;
  if (!is_float_dtype(dtype)) return TS_ERR_UNSUPPORTED;
  if (B * N * K == 0) return TS_OK;
  if (!out || !total || !count || (B * E * K > 0 && (!src || !index))) return TS_ERR_BAD_ARG;
  if (B * N >= 0x7FFFFFFFll) return TS_ERR_UNSUPPORTED;
  const size_t need = group_workspace_bytes(B, N, K, kElemBytes[dtype]);
  if (!workspace || workspace_bytes < need || !aligned16(workspace)) return TS_ERR_WORKSPACE;
  GroupArgs g = {};
  g.src = src;
  g.index = index;
  g.out = out;
  g.gmax = workspace;
  g.gs = K;  // sums only
  g.gsum = workspace;
  g.total = total;
  g.count = count;
  g.unbiased = unbiased ? 1 : 0;
  g.B = B;
  g.E = E;
  g.K = K;
  g.N = N;
  g.sb = index_stride_b;
  g.se = index_stride_e;
  const int full = kVecBytes / kElemBytes[dtype];
  const int vec = (full > 1 && K % full == 0 && aligned16(src) && aligned16(total)) ? full : 1;
  return dispatch_group_softmax(dtype, g, GS_STD, vec, static_cast<hipStream_t>(stream));
}

int ts_group_std_backward(const void *src, const int64_t *index, const void *total, const int32_t *count,
                          const void *out, const void *grad_out, void *grad_in, int64_t B, int64_t E, int64_t K,
                          int64_t N, int64_t index_stride_b, int64_t index_stride_e, int dtype, int unbiased,
                          ts_stream_t stream) {
  return ts_group_std_backward_with_workspace(src, index, total, count, out, grad_out, grad_in, B, E, K, N, index_stride_b,
                                              index_stride_e, dtype, unbiased, nullptr, 0, stream);
}

int ts_group_std_backward_with_workspace(const void *src, const int64_t *index, const void *total, const int32_t *count,
                                         const void *out, const void *grad_out, void *grad_in, int64_t B, int64_t E,
                                         int64_t K, int64_t N, int64_t index_stride_b, int64_t index_stride_e, int dtype,
                                         int unbiased, void *workspace, size_t workspace_bytes, ts_stream_t stream) {
  if (!valid_dtype(dtype) || !sizes_ok(B, N, E, K)) return TS_ERR_BAD_ARG;
  if (!is_float_dtype(dtype)) return TS_ERR_UNSUPPORTED;
  if (B * E * K == 0) return TS_OK;
  if (!src || !index || !total || !count || !out || !grad_out || !grad_in) return TS_ERR_BAD_ARG;
  if (N == 0 || B * N >= 0x7FFFFFFFll) return TS_ERR_UNSUPPORTED;
  GroupArgs g = {};
  g.src = src;
  g.index = index;
  g.out = grad_in;
  g.node_out = out;
  g.node_grad = grad_out;
  g.total = total;
  g.count = count;
  g.unbiased = unbiased ? 1 : 0;
  g.B = B;
  g.E = E;
  g.K = K;
  g.N = N;
  g.sb = index_stride_b;
  g.se = index_stride_e;
  const int full = kVecBytes / kElemBytes[dtype];
  const bool al = aligned16(src) && aligned16(grad_in) && aligned16(out) && aligned16(grad_out) && aligned16(total);
  const int vec = (full > 1 && K % full == 0 && al) ? full : 1;
  if (group_coef_ok(B, E, N, K, dtype, workspace, workspace_bytes)) g.coef = workspace;
  return dispatch_group_softmax(dtype, g, GS_STD_BWD, vec, static_cast<hipStream_t>(stream));
}

// ---- index formats
int ts_index_to_indptr(const int64_t *index, int64_t *indptr, int64_t B, int64_t E, int64_t N,
                       int64_t index_batch_stride, ts_stream_t stream) {
  if (B < 0 || E < 0 || N < 0) return TS_ERR_BAD_ARG;
  if (B == 0) return TS_OK;
  if (!indptr || (E > 0 && !index)) return TS_ERR_BAD_ARG;
  return run_coo_to_indptr(index, indptr, B, E, N, index_batch_stride, static_cast<hipStream_t>(stream));
}

size_t ts_indptr_to_index_workspace_bytes(int64_t B, int64_t N) {
  return B < 0 || N < 0 ? 0 : ((size_t)B * N * 8 + 255) & ~(size_t)255;
}

int ts_indptr_to_index(const int64_t *indptr, int64_t *index, int64_t B, int64_t N, int64_t E,
                       int64_t indptr_batch_stride, void *workspace, size_t workspace_bytes, ts_stream_t stream) {
  if (!sizes_ok(B, N, E, 1)) return TS_ERR_BAD_ARG;
  if (B * E == 0 || N == 0) return TS_OK;
  if (!indptr || !index) return TS_ERR_BAD_ARG;
  if (!workspace || workspace_bytes < ts_indptr_to_index_workspace_bytes(B, N) || !aligned16(workspace))
    return TS_ERR_WORKSPACE;
  hipStream_t s = static_cast<hipStream_t>(stream);
  // the row numbers 0 .. N-1 of every batch, expanded along the row pointers like any other source
  int64_t *rows = static_cast<int64_t *>(workspace);
  hipLaunchKernelGGL(row_numbers_kernel, dim3(index_grid(B * N)), dim3(kBlock), 0, s, rows, B * N, N);
  if (hipGetLastError() != hipSuccess) return TS_ERR_LAUNCH;
  return ts_gather_csr(rows, indptr, index, B, N, E, 1, indptr_batch_stride, TS_I64, stream);
}

static int sort_key_bits(int64_t N) {  // keys are 0 .. N (N: an index outside [0, N))
  int bits = 1;
  while (bits < 32 && ((int64_t)1 << bits) <= N) ++bits;
  return bits;
}
static size_t sort_keys_bytes(int64_t E) { return ((size_t)E * 4 + 255) & ~(size_t)255; }

size_t ts_sort_index_workspace_bytes(int64_t E, int64_t N) {
  if (E < 0 || N < 0 || E >= 0x7FFFFFFFll || N >= 0x7FFFFFFFll) return 0;
  return 2 * sort_keys_bytes(E) + ((sort_keys_temp_bytes(E, sort_key_bits(N)) + 255) & ~(size_t)255);
}

int ts_sort_index(const int64_t *index, int32_t *perm, int64_t *indptr, int64_t E, int64_t N, void *workspace,
                  size_t workspace_bytes, ts_stream_t stream) {
  if (E < 0 || N < 0) return TS_ERR_BAD_ARG;
  if (E >= 0x7FFFFFFFll || N >= 0x7FFFFFFFll) return TS_ERR_UNSUPPORTED;
  if (!indptr || (E > 0 && (!index || !perm))) return TS_ERR_BAD_ARG;
  hipStream_t s = static_cast<hipStream_t>(stream);
  const size_t kb = sort_keys_bytes(E);
  uint32_t *keys_in = static_cast<uint32_t *>(workspace);
  uint32_t *keys_out = reinterpret_cast<uint32_t *>(static_cast<char *>(workspace) + kb);
  if (E > 0) {
    const int bits = sort_key_bits(N);
    const size_t temp = sort_keys_temp_bytes(E, bits);
    if (!workspace || !aligned16(workspace) || workspace_bytes < 2 * kb + temp) return TS_ERR_WORKSPACE;
    hipLaunchKernelGGL(index_keys_kernel, dim3(index_grid(E)), dim3(kBlock), 0, s, index, keys_in, E, N);
    if (hipGetLastError() != hipSuccess) return TS_ERR_LAUNCH;
    const int rc = sort_keys_to_perm(static_cast<char *>(workspace) + 2 * kb, temp, keys_in, keys_out, perm, E, bits, s);
    if (rc != TS_OK) return rc;
  }
  hipLaunchKernelGGL(keys_to_indptr_kernel, dim3((unsigned)((E + 1 + kBlock - 1) / kBlock)), dim3(kBlock), 0, s,
                     keys_out, indptr, N, E);
  return hipGetLastError() == hipSuccess ? TS_OK : TS_ERR_LAUNCH;
}

}  // extern "C"
