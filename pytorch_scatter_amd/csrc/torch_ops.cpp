// PyTorch host layer: registers the reference's operator names
// (torch.ops.torch_scatter.*: csrc/scatter.cpp:272-277, segment_coo.cpp:240-246,
// segment_csr.cpp:233-239, version.cpp:41-42) with the same inferred schemas
// and the same forward/backward wiring, on top of the C ABI in ts_hip.h.
//
// PyTorch is used for what it owns: tensors, the caching allocator, the
// current stream and the autograd graph. All arithmetic runs in libts_hip.so.
// There is no CPU path: a CPU tensor is an error, not a fallback.
#include <torch/script.h>

#include <c10/core/DeviceGuard.h>
#include <c10/hip/HIPStream.h>
#include <hip/hip_runtime_api.h>

#include <map>
#include <mutex>

#include "../../include/torchscatter/scatter.h"
#include "../../include/ts_hip.h"

namespace {

using torch::Tensor;
using OptTensor = std::optional<Tensor>;
using OptInt = std::optional<int64_t>;
using torch::autograd::AutogradContext;
using torch::autograd::Variable;
using torch::autograd::variable_list;

// ------------------------------------------------------------------ helpers
void check_input(bool cond) {
  // the reference's CHECK_INPUT (csrc/cuda/utils.cuh:7)
  TORCH_CHECK(cond, "Input mismatch");
}

void check_device(const Tensor &t, const char *name) {
  // the reference's CHECK_CUDA (csrc/cuda/utils.cuh:5-6); HIP tensors carry the CUDA device type
  TORCH_CHECK(t.device().is_cuda(), name,
              " must be CUDA tensor (this build has HIP kernels only, no CPU path)");
}

int dtype_code(const Tensor &t) {
  switch (t.scalar_type()) {
  case at::kFloat: return TS_F32;
  case at::kDouble: return TS_F64;
  case at::kHalf: return TS_F16;
  case at::kBFloat16: return TS_BF16;
  case at::kInt: return TS_I32;
  case at::kLong: return TS_I64;
  case at::kShort: return TS_I16;
  case at::kChar: return TS_I8;
  case at::kByte: return TS_U8;
  default: TORCH_CHECK(false, "torch_scatter: unsupported dtype ", t.scalar_type());
  }
}

int reduce_code(const std::string &reduce) {
  // same strings as the reference's reduce2REDUCE (csrc/cuda/reducer.cuh:10-13);
  // an unknown string throws std::out_of_range there as well
  static const std::map<std::string, int> table = {
      {"sum", TS_SUM}, {"mean", TS_MEAN}, {"mul", TS_MUL}, {"div", TS_DIV}, {"min", TS_MIN}, {"max", TS_MAX}};
  return table.at(reduce);
}

ts_stream_t stream_of(const Tensor &t) {
  return static_cast<ts_stream_t>(c10::hip::getCurrentHIPStream(t.device().index()).stream());
}

void check_status(int status, const char *what) {
  TORCH_CHECK(status == TS_OK, "torch_scatter (", what, "): ", ts_error_string(status));
}

int64_t prod(c10::IntArrayRef sizes, int64_t lo, int64_t hi) {
  int64_t p = 1;
  for (int64_t i = lo; i < hi; ++i) p *= sizes[i];
  return p;
}

// Element stride that addresses dims [lo, hi) of `t` by their row-major linear
// index, if one exists (contiguous within the group, or broadcast).
std::optional<int64_t> collapsed_stride(const Tensor &t, int64_t lo, int64_t hi) {
  int64_t expect = -1;  // stride the next more-significant non-unit dim must have
  int64_t inner = 0;
  bool have = false;
  for (int64_t i = hi - 1; i >= lo; --i) {
    if (t.size(i) == 1) continue;
    if (!have) {
      inner = t.stride(i);
      have = true;
    } else if (t.stride(i) != expect) {
      return std::nullopt;
    }
    expect = t.stride(i) * t.size(i);
  }
  return have ? inner : 0;
}

// Opt-in check of a segment reduction's status words (TS_CHECK_STATUS=1 in the environment, read once): copies
// the 16 bytes back, which waits for the stream, and raises if the call gave a row up (row pointers that are
// not monotone, an index that is not sorted). Off by default: the operators never synchronise on their own.
// (never while the current stream is being captured into a graph: a copy to the host is not allowed there)
bool status_checks_on() {
  static const bool on = [] {
    const char *e = getenv("TS_CHECK_STATUS");
    return e != nullptr && atoi(e) != 0;
  }();
  if (!on) return false;
  hipStreamCaptureStatus capture = hipStreamCaptureStatusNone;
  if (hipStreamIsCapturing(c10::hip::getCurrentHIPStream().stream(), &capture) != hipSuccess) return false;
  return capture == hipStreamCaptureStatusNone;
}
void maybe_check_status_words(const Tensor &ws, size_t ws_bytes, const char *what) {
  if (!status_checks_on() || ws_bytes < TS_STATUS_BYTES || (size_t)ws.numel() < ws_bytes) return;
  const Tensor words = ws.narrow(0, (int64_t)(ws_bytes - TS_STATUS_BYTES), 16).cpu();
  unsigned long long w[2];
  memcpy(w, words.data_ptr(), sizeof(w));
  TORCH_CHECK(!ts_status_gave_up(w), "torch_scatter (", what,
              "): a row that crosses tiles was given up and written as empty -- row pointers that are not "
              "monotone or an index that is not sorted");
}

Tensor workspace(size_t bytes, const Tensor &like) {
  return at::empty({static_cast<int64_t>(bytes > 0 ? bytes : 1)}, like.options().dtype(at::kByte));
}

// A workspace whose first `zero_bytes` bytes must read as zero when a call starts and are left zero by it
// (ts_scatter_workspace_zero_bytes): kept from call to call, one per device and stream, cleared when allocated.
struct KeptWorkspaces {
  std::mutex mu;
  std::map<std::pair<int, void *>, Tensor> kept;
};
KeptWorkspaces &kept_workspaces() {
  static KeptWorkspaces *k = new KeptWorkspaces();  // never destroyed: no frees after the runtime has shut down
  return *k;
}
Tensor kept_workspace(size_t bytes, size_t zero_bytes, const Tensor &like, void *stream) {
  KeptWorkspaces &k = kept_workspaces();
  std::lock_guard<std::mutex> lock(k.mu);
  const auto key = std::make_pair((int)like.get_device(), stream);
  auto it = k.kept.find(key);
  if (it == k.kept.end() || it->second.numel() < (int64_t)bytes) {
    Tensor t = workspace(bytes, like);
    t.narrow(0, 0, (int64_t)zero_bytes).zero_();
    k.kept[key] = t;
    return t;
  }
  return it->second;
}
void drop_kept_workspace(const Tensor &like, void *stream) {  // after a failed call its content is unknown
  KeptWorkspaces &k = kept_workspaces();
  std::lock_guard<std::mutex> lock(k.mu);
  k.kept.erase(std::make_pair((int)like.get_device(), stream));
}

// csrc/scatter.cpp:25-33
Tensor broadcast(Tensor src, const Tensor &other, int64_t dim) {
  if (src.dim() == 1)
    for (int64_t i = 0; i < dim; i++) src = src.unsqueeze(0);
  for (int64_t i = src.dim(); i < other.dim(); i++) src = src.unsqueeze(-1);
  return src.expand(other.sizes().vec());
}

// [B, I] view of an index / indptr tensor whose leading dims were expanded to
// src's: unit inner stride and one batch stride (0 when shared), copying only
// when the layout cannot be described that way.
struct BatchedIndex {
  Tensor t;
  int64_t batch_stride;
};
BatchedIndex batched_index(const Tensor &idx) {
  const int64_t d = idx.dim() - 1;
  auto bs = collapsed_stride(idx, 0, d);
  const bool inner_ok = idx.size(d) <= 1 || idx.stride(d) == 1;
  if (bs.has_value() && inner_ok) return {idx, bs.value()};
  Tensor c = idx.contiguous();
  return {c, c.size(d)};
}

// ------------------------------------------------------------------ scatter
// host half of scatter_cuda (csrc/cuda/scatter_cuda.cu:58-138)
// mean_count (sum only): if the call is a sum under one index per row, the entries of every output row are counted
// in the same call (ts_scatter_sum_count_with_workspace) and the int32 counts [B * N]
// are left here; else it stays undefined
std::tuple<Tensor, OptTensor> scatter_hip(Tensor src, Tensor index, int64_t dim, OptTensor optional_out,
                                          OptInt dim_size, int reduce, Tensor *mean_count = nullptr) {
  check_device(src, "src");
  check_device(index, "index");
  if (optional_out.has_value()) check_device(optional_out.value(), "out");
  c10::DeviceGuard guard(src.device());

  check_input(src.dim() == index.dim());
  for (int64_t i = 0; i < index.dim() - 1; i++) check_input(src.size(i) >= index.size(i));
  TORCH_CHECK(index.scalar_type() == at::kLong, "index must be int64");

  // 8- and 16-bit integers have no atomic add: ts_scatter adds them with a compare-and-swap loop on the 32-bit
  // word around the element, and the cost of that loop grows with the square of the entries that meet in one row
  // (100 k entries, 30 % of them on one row: 0.3 - 0.7 s; int32: 0.3 ms). Their sums run in int32 instead, whose
  // wrap-around agrees with that of the narrow type modulo 2^8 / 2^16, and are cast back (also faster without
  // any contention: 2.25 M entries in random order, one int8 each: 458 against 97 us).
  const auto st = src.scalar_type();
  if (reduce == TS_SUM && (st == at::kChar || st == at::kByte || st == at::kShort) && src.numel() > 0) {
    OptTensor wide_out;
    if (optional_out.has_value()) wide_out = optional_out.value().to(at::kInt);
    Tensor narrow = std::get<0>(scatter_hip(src.to(at::kInt), index, dim, wide_out, dim_size, reduce)).to(st);
    if (!optional_out.has_value()) return std::make_tuple(narrow, OptTensor());
    optional_out.value().copy_(narrow);
    return std::make_tuple(optional_out.value(), OptTensor());
  }

  src = src.contiguous();
  Tensor out;
  if (optional_out.has_value()) {
    out = optional_out.value().contiguous();
    for (int64_t i = 0; i < out.dim(); i++)
      if (i != dim) check_input(src.size(i) == out.size(i));
  } else {
    auto sizes = src.sizes().vec();
    if (dim_size.has_value())
      sizes[dim] = dim_size.value();
    else if (index.numel() == 0)
      sizes[dim] = 0;
    else
      sizes[dim] = 1 + index.max().item<int64_t>();  // host sync, as upstream
    out = at::empty(sizes, src.options());
  }
  const bool minmax = reduce == TS_MIN || reduce == TS_MAX;
  OptTensor arg_out;
  if (minmax) arg_out = at::empty(out.sizes(), index.options());

  if (src.numel() == 0) {
    if (!optional_out.has_value()) out.fill_(0);
    if (minmax) arg_out.value().fill_(src.size(dim));
    return std::make_tuple(out, arg_out);
  }
  // the op layer always hands over an index broadcast to src's shape
  check_input(index.sizes() == src.sizes());

  const int64_t B = prod(src.sizes(), 0, dim);
  const int64_t E = src.size(dim);
  const int64_t K = prod(src.sizes(), dim + 1, src.dim());
  const int64_t N = out.size(dim);

  auto sb = collapsed_stride(index, 0, dim);
  auto sk = collapsed_stride(index, dim + 1, index.dim());
  int64_t se = index.stride(dim);
  if (!sb.has_value() || !sk.has_value()) {
    index = index.contiguous();
    sb = E * K;
    se = K;
    sk = 1;
  }
  if (mean_count != nullptr && reduce == TS_SUM && sk.value() == 0 && B * N < 0x7FFFFFFFll) {
    const size_t cs_bytes = ts_scatter_sum_count_workspace_bytes(B, E, K, N, dtype_code(src));
    Tensor cws = workspace(cs_bytes, src);
    Tensor count = at::empty({B * N}, src.options().dtype(at::kInt));
    check_status(ts_scatter_sum_count_with_workspace(src.data_ptr(), index.data_ptr<int64_t>(), out.data_ptr(),
                                                     count.data_ptr<int32_t>(), B, E, K, N, sb.value(), se, dtype_code(src),
                                                     optional_out.has_value() ? 1 : 0,
                                                     cs_bytes > 0 ? cws.data_ptr() : nullptr, cs_bytes, stream_of(src)),
                 "scatter (sum and count)");
    *mean_count = count;
    return std::make_tuple(out, OptTensor());
  }
  // min / max of large inputs with wide rows can use scratch memory (entries binned by bucket of output rows)
  const size_t ws_bytes = sk.value() == 0 ? ts_scatter_workspace_bytes(B, E, K, N, dtype_code(src), reduce) : 0;
  const size_t ws_zero = ws_bytes > 0 ? ts_scatter_workspace_zero_bytes(B, E, K, N, dtype_code(src), reduce) : 0;
  Tensor ws;
  if (ws_zero > 0)
    ws = kept_workspace(ws_bytes, ws_zero, src, stream_of(src));
  else if (ws_bytes > 0)
    ws = workspace(ws_bytes, src);
  const int rc = ts_scatter_with_workspace(src.data_ptr(), index.data_ptr<int64_t>(), out.data_ptr(),
                                           minmax ? arg_out.value().data_ptr<int64_t>() : nullptr, B, E, K, N,
                                           sb.value(), se, sk.value(), dtype_code(src), reduce,
                                           optional_out.has_value() ? 1 : 0, ws_bytes > 0 ? ws.data_ptr() : nullptr,
                                           ws_bytes, stream_of(src));
  if (rc != TS_OK && ws_zero > 0) drop_kept_workspace(src, stream_of(src));
  check_status(rc, "scatter");
  if (ws_zero >= TS_STATUS_BYTES && status_checks_on()) {
    // min / max of single values: the word behind the key table says whether a bounded wait in the kernel ran out
    const bool lost = ws.narrow(0, (int64_t)(ws_zero - TS_STATUS_BYTES), 8).cpu().view(at::kLong).item<int64_t>() != 0;
    if (lost) drop_kept_workspace(src, stream_of(src));
    TORCH_CHECK(!lost, "torch_scatter (scatter): a bounded wait inside the kernel ran out and entries were lost");
  }
  return std::make_tuple(out, arg_out);
}

// ---------------------------------------------------------------- segment_csr
struct CsrShape {
  Tensor indptr;
  int64_t batch_stride, dim, B;
};
CsrShape expand_indptr(const Tensor &src, Tensor indptr) {
  check_input(src.dim() >= indptr.dim());
  TORCH_CHECK(indptr.scalar_type() == at::kLong, "indptr must be int64");
  auto sizes = indptr.sizes().vec();
  for (int64_t i = 0; i < indptr.dim() - 1; i++) sizes[i] = src.size(i);
  indptr = indptr.expand(sizes);
  CsrShape s;
  s.dim = indptr.dim() - 1;
  s.B = prod(indptr.sizes(), 0, s.dim);
  auto bi = batched_index(indptr);
  s.indptr = bi.t;
  s.batch_stride = bi.batch_stride;
  return s;
}

// host half of segment_csr_cuda (csrc/cuda/segment_csr_cuda.cu:97-168)
std::tuple<Tensor, OptTensor> segment_csr_hip(Tensor src, Tensor indptr, OptTensor optional_out, int reduce) {
  check_device(src, "src");
  check_device(indptr, "indptr");
  if (optional_out.has_value()) check_device(optional_out.value(), "out");
  c10::DeviceGuard guard(src.device());

  CsrShape cs = expand_indptr(src, indptr);
  const int64_t dim = cs.dim;
  src = src.contiguous();

  Tensor out;
  if (optional_out.has_value()) {
    out = optional_out.value().contiguous();
    for (int64_t i = 0; i < out.dim(); i++)
      if (i != dim) check_input(src.size(i) == out.size(i));
    check_input(src.numel() == 0 || out.size(dim) == cs.indptr.size(dim) - 1);
  } else {
    auto sizes = src.sizes().vec();
    sizes[dim] = std::max<int64_t>(cs.indptr.size(dim) - 1, 0);
    out = at::empty(sizes, src.options());
  }
  const bool minmax = reduce == TS_MIN || reduce == TS_MAX;
  OptTensor arg_out;
  if (minmax) arg_out = at::empty(out.sizes(), cs.indptr.options());

  if (src.numel() == 0) {
    if (!optional_out.has_value()) out.fill_(0);
    if (minmax) arg_out.value().fill_(src.size(dim));
    return std::make_tuple(out, arg_out);
  }
  const int64_t N = out.size(dim);
  const int64_t E = src.size(dim);
  const int64_t K = (cs.B * N) > 0 ? out.numel() / (cs.B * N) : 0;
  const size_t ws_bytes = ts_segment_csr_workspace_bytes(cs.B, N, E, K, dtype_code(src), reduce);
  Tensor ws = workspace(ws_bytes, src);
  check_status(ts_segment_csr(src.data_ptr(), cs.indptr.data_ptr<int64_t>(), out.data_ptr(),
                              minmax ? arg_out.value().data_ptr<int64_t>() : nullptr, cs.B, N, E, K,
                              cs.batch_stride, dtype_code(src), reduce, ws.data_ptr(), ws_bytes, stream_of(src)),
               "segment_csr");
  maybe_check_status_words(ws, ws_bytes, "segment_csr");
  return std::make_tuple(out, arg_out);
}

// host half of gather_csr_cuda (csrc/cuda/segment_csr_cuda.cu:219-281);
// `mean_backward` selects the fused gather-and-divide
Tensor gather_csr_hip(Tensor src, Tensor indptr, OptTensor optional_out, bool mean_backward = false) {
  check_device(src, "src");
  check_device(indptr, "indptr");
  if (optional_out.has_value()) check_device(optional_out.value(), "out");
  c10::DeviceGuard guard(src.device());

  CsrShape cs = expand_indptr(src, indptr);
  const int64_t dim = cs.dim;
  check_input(src.size(dim) == 0 || src.size(dim) == cs.indptr.size(dim) - 1);
  src = src.contiguous();

  Tensor out;
  if (optional_out.has_value()) {
    out = optional_out.value().contiguous();
    for (int64_t i = 0; i < out.dim(); i++)
      if (i != dim) check_input(src.size(i) == out.size(i));
  } else {
    auto sizes = src.sizes().vec();
    sizes[dim] = src.numel() > 0 ? cs.indptr.flatten()[-1].item<int64_t>() : 0;  // host sync, as upstream
    out = at::empty(sizes, src.options());
  }
  if (src.numel() == 0) {
    if (!optional_out.has_value()) out.fill_(0);
    return out;
  }
  const int64_t N = src.size(dim);
  const int64_t E = out.size(dim);
  const int64_t K = src.numel() / (cs.B * N);
  if (mean_backward)
    check_status(ts_segment_mean_csr_backward(src.data_ptr(), cs.indptr.data_ptr<int64_t>(), out.data_ptr(), cs.B, N,
                                              E, K, cs.batch_stride, dtype_code(src), stream_of(src)),
                 "segment_mean_csr backward");
  else
    check_status(ts_gather_csr(src.data_ptr(), cs.indptr.data_ptr<int64_t>(), out.data_ptr(), cs.B, N, E, K,
                               cs.batch_stride, dtype_code(src), stream_of(src)),
                 "gather_csr");
  return out;
}

// ---------------------------------------------------------------- segment_coo
struct CooShape {
  Tensor index;
  int64_t batch_stride, dim, B;
};
CooShape expand_index(const Tensor &src, Tensor index, bool expand) {
  check_input(src.dim() >= index.dim());
  TORCH_CHECK(index.scalar_type() == at::kLong, "index must be int64");
  if (expand) {
    auto sizes = index.sizes().vec();
    for (int64_t i = 0; i < index.dim(); i++) sizes[i] = src.size(i);
    index = index.expand(sizes);
  }
  CooShape s;
  s.dim = index.dim() - 1;
  s.B = prod(index.sizes(), 0, s.dim);
  auto bi = batched_index(index);
  s.index = bi.t;
  s.batch_stride = bi.batch_stride;
  return s;
}

// host half of segment_coo_cuda (csrc/cuda/segment_coo_cuda.cu:152-283).
// Second result: arg_out (min/max), count (mean), nothing (sum).
std::tuple<Tensor, OptTensor> segment_coo_hip(Tensor src, Tensor index, OptTensor optional_out, OptInt dim_size,
                                              int reduce) {
  check_device(src, "src");
  check_device(index, "index");
  if (optional_out.has_value()) check_device(optional_out.value(), "out");
  c10::DeviceGuard guard(src.device());

  CooShape cs = expand_index(src, index, true);
  const int64_t dim = cs.dim;
  src = src.contiguous();

  Tensor out;
  if (optional_out.has_value()) {
    out = optional_out.value().contiguous();
    for (int64_t i = 0; i < out.dim(); i++)
      if (i != dim) check_input(src.size(i) == out.size(i));
  } else {
    auto sizes = src.sizes().vec();
    if (dim_size.has_value())
      sizes[dim] = dim_size.value();
    else if (cs.index.numel() == 0)
      sizes[dim] = 0;
    else {
      auto tmp = cs.index.select(dim, cs.index.size(dim) - 1);
      tmp = tmp.numel() > 1 ? tmp.max() : tmp;
      sizes[dim] = 1 + tmp.item<int64_t>();  // host sync, as upstream
    }
    out = at::empty(sizes, src.options());
  }
  const bool minmax = reduce == TS_MIN || reduce == TS_MAX;
  OptTensor second;
  if (minmax) {
    // with `out` given the kernel only touches rows that have entries
    second = optional_out.has_value() ? at::full(out.sizes(), src.size(dim), cs.index.options())
                                      : at::empty(out.sizes(), cs.index.options());
  } else if (reduce == TS_MEAN) {
    auto sizes = cs.index.sizes().vec();
    sizes[dim] = out.size(dim);
    second = optional_out.has_value() ? at::ones(sizes, out.options()) : at::empty(sizes, out.options());
  }
  if (src.numel() == 0 || cs.index.numel() == 0) {
    if (!optional_out.has_value()) out.fill_(0);
    if (minmax) second.value().fill_(src.size(dim));
    if (reduce == TS_MEAN) second.value().fill_(1);
    return std::make_tuple(out, second);
  }
  const int64_t E = src.size(dim);
  const int64_t N = out.size(dim);
  const int64_t K = src.numel() / (cs.B * E);
  const size_t ws_bytes = ts_segment_coo_workspace_bytes(cs.B, N, E, K, dtype_code(src), reduce);
  Tensor ws = workspace(ws_bytes, src);
  check_status(ts_segment_coo(src.data_ptr(), cs.index.data_ptr<int64_t>(), out.data_ptr(),
                              minmax ? second.value().data_ptr() : nullptr,
                              reduce == TS_MEAN ? second.value().data_ptr() : nullptr, cs.B, N, E, K,
                              cs.batch_stride, dtype_code(src), reduce, optional_out.has_value() ? 1 : 0,
                              ws.data_ptr(), ws_bytes, stream_of(src)),
               "segment_coo");
  maybe_check_status_words(ws, ws_bytes, "segment_coo");
  return std::make_tuple(out, second);
}

// host half of gather_coo_cuda (csrc/cuda/segment_coo_cuda.cu:327-382);
// with `count` given: the fused backward of segment_coo(mean)
Tensor gather_coo_hip(Tensor src, Tensor index, OptTensor optional_out, OptTensor count = std::nullopt) {
  check_device(src, "src");
  check_device(index, "index");
  if (optional_out.has_value()) check_device(optional_out.value(), "out");
  c10::DeviceGuard guard(src.device());

  check_input(src.dim() >= index.dim());
  auto sizes = index.sizes().vec();
  for (int64_t i = 0; i < index.dim() - 1; i++) sizes[i] = src.size(i);
  index = index.expand(sizes);
  CooShape cs = expand_index(src, index, false);
  const int64_t dim = cs.dim;
  src = src.contiguous();

  Tensor out;
  if (optional_out.has_value()) {
    out = optional_out.value().contiguous();
    for (int64_t i = 0; i < src.dim(); i++)
      if (i != dim) check_input(src.size(i) == out.size(i));
    check_input(cs.index.size(dim) == out.size(dim));
  } else {
    auto osizes = src.sizes().vec();
    osizes[dim] = cs.index.size(dim);
    out = at::empty(osizes, src.options());
  }
  if (src.numel() == 0 || out.numel() == 0) {
    if (!optional_out.has_value()) out.fill_(0);
    return out;
  }
  const int64_t E = cs.index.size(dim);
  const int64_t N = src.size(dim);
  const int64_t K = out.numel() / (cs.B * E);
  if (count.has_value()) {
    Tensor c = count.value().contiguous();
    check_status(ts_segment_mean_coo_backward(src.data_ptr(), cs.index.data_ptr<int64_t>(), c.data_ptr(),
                                              out.data_ptr(), cs.B, N, E, K, cs.batch_stride, dtype_code(src),
                                              stream_of(src)),
                 "segment_mean_coo backward");
  } else {
    check_status(ts_gather_coo(src.data_ptr(), cs.index.data_ptr<int64_t>(), out.data_ptr(), cs.B, N, E, K,
                               cs.batch_stride, dtype_code(src), stream_of(src)),
                 "gather_coo");
  }
  return out;
}

// Backward of every min/max flavour: the gradient of each output slot goes to
// the position that won it (csrc/scatter.cpp:184-196, segment_coo.cpp:132-144,
// segment_csr.cpp:130-142 do this with a scatter_ into a buffer that has one
// extra slot for the sentinel).
Tensor arg_backward_hip(Tensor grad_out, const Tensor &arg_out, const std::vector<int64_t> &src_shape, int64_t dim) {
  c10::DeviceGuard guard(grad_out.device());
  grad_out = grad_out.contiguous();
  Tensor arg = arg_out.contiguous();
  Tensor grad_in = at::empty(src_shape, grad_out.options());
  const int64_t B = prod(src_shape, 0, dim);
  const int64_t E = src_shape[dim];
  const int64_t K = prod(src_shape, dim + 1, static_cast<int64_t>(src_shape.size()));
  const int64_t N = grad_out.size(dim);
  check_status(ts_arg_backward(grad_out.data_ptr(), arg.data_ptr<int64_t>(), grad_in.data_ptr(), B, N, E, K,
                               dtype_code(grad_out), stream_of(grad_out)),
               "min/max backward");
  return grad_in;
}

std::vector<int64_t> saved_shape(AutogradContext *ctx) {
  return ctx->saved_data["src_shape"].toIntVector();
}

// Backward of scatter sum / mean: grad_in = grad_out gathered along dim by the index (divided by the gathered
// count for mean; csrc/scatter.cpp:70-81, 143-161). With one index per row, which is what the broadcast of a 1-D
// or row-shaped index gives, whole rows are copied by the gather_coo kernel (torch's elementwise gather took
// 1.9 ms where this takes 0.06-0.7 ms: 9 M rows of 8 and 64 floats); an index that differs between the
// columns of a row keeps at::gather.
Tensor gather_grad_rows(const Tensor &grad_out, const Tensor &index, int64_t dim, const OptTensor &count) {
  auto sk = collapsed_stride(index, dim + 1, index.dim());
  const int64_t K = prod(index.sizes(), dim + 1, index.dim());
  const bool per_row = index.dim() == grad_out.dim() && grad_out.numel() > 0 && index.numel() > 0 &&
                       (K == 1 || (sk.has_value() && sk.value() == 0));
  if (!per_row) {
    Tensor grad_in = at::gather(grad_out, dim, index, false);
    if (count.has_value()) grad_in.true_divide_(at::gather(count.value(), dim, index, false));
    return grad_in;
  }
  Tensor rows = index;
  while (rows.dim() > dim + 1) rows = rows.select(rows.dim() - 1, 0);
  OptTensor count_rows;
  if (count.has_value()) {
    Tensor c = count.value();
    while (c.dim() > dim + 1) c = c.select(c.dim() - 1, 0);
    count_rows = c;
  }
  return gather_coo_hip(grad_out.contiguous(), rows, std::nullopt, count_rows);
}

// ------------------------------------------------------- autograd: scatter
// one Function per reduction, wired as ScatterSum/Mul/Mean/Min/Max in csrc/scatter.cpp:54-233
template <int REDUCE> struct ScatterFn : public torch::autograd::Function<ScatterFn<REDUCE>> {
  static variable_list forward(AutogradContext *ctx, Variable src, Variable index, int64_t dim,
                               std::optional<Variable> optional_out, OptInt dim_size) {
    dim = dim < 0 ? src.dim() + dim : dim;
    ctx->saved_data["dim"] = dim;
    ctx->saved_data["src_shape"] = src.sizes();
    Variable old_index = index;
    index = broadcast(index, src, dim);
    Tensor fused_count;  // mean of single values: counted together with the sum
    auto result = scatter_hip(src, index, dim, optional_out, dim_size, REDUCE == TS_MEAN ? TS_SUM : REDUCE,
                              REDUCE == TS_MEAN ? &fused_count : nullptr);
    Variable out = std::get<0>(result);
    if (optional_out.has_value()) ctx->mark_dirty({optional_out.value()});
    if (REDUCE == TS_SUM) {
      ctx->save_for_backward({index});
      return {out};
    }
    if (REDUCE == TS_MUL) {
      ctx->save_for_backward({src, index, out});
      return {out};
    }
    if (REDUCE == TS_MEAN) {
      // count over the index as given (csrc/scatter.cpp:131-141). One index per row (a 1-D index along
      // dim 0, or an index shaped like src's leading dims): the entries are counted straight from the
      // index (no tensor of ones; exact int32 counts) and one kernel clamps, casts and divides.
      bool per_row = old_index.dim() == dim + 1 && src.numel() > 0 && out.numel() > 0 && old_index.size(dim) == src.size(dim);
      for (int64_t i = 0; per_row && i < dim; i++) per_row = old_index.size(i) == src.size(i);
      if (per_row) {
        const int64_t B = prod(src.sizes(), 0, dim), E = src.size(dim), N = out.size(dim);
        const int64_t K = prod(src.sizes(), dim + 1, src.dim());
        const BatchedIndex bi = batched_index(old_index);
        // one index row shared by every batch row (an expanded view): counted once and repeated
        const int64_t Bc = (bi.batch_stride == 0 && B > 1) ? 1 : B;
        Tensor count_f;
        if (fused_count.defined() && fused_count.numel() == B * N) {
          count_f = fused_count;
        } else {
          count_f = at::empty({Bc * N}, src.options().dtype(at::kInt));
          const size_t cws_bytes = ts_scatter_count_workspace_bytes(Bc, E, N);
          Tensor cws = workspace(cws_bytes, src);
          check_status(ts_scatter_count_with_workspace(bi.t.data_ptr<int64_t>(), count_f.data_ptr<int32_t>(), Bc, E, N,
                                                       bi.batch_stride, 1, cws_bytes > 0 ? cws.data_ptr() : nullptr,
                                                       cws_bytes, stream_of(src)),
                       "scatter_mean count");
          if (Bc != B) count_f = count_f.view({1, N}).expand({B, N}).contiguous().view({B * N});
        }
        Tensor out_c = out.contiguous();
        check_status(ts_divide_by_count(out_c.data_ptr(), count_f.data_ptr<int32_t>(), B, N, K, dtype_code(out_c),
                                        stream_of(src)),
                     "scatter_mean divide");
        if (!out_c.is_same(out)) out.copy_(out_c);
        if (src.requires_grad()) {  // the count in the element type, as the backward pass divides by it
          auto count_sizes = out.sizes().vec();
          count_sizes.resize(dim + 1);
          Variable count = broadcast(count_f.clamp_min_(1).to(src.scalar_type()).view(count_sizes), out, dim);
          ctx->save_for_backward({index, count});
        }
        return {out};
      }
      auto ones = at::ones(old_index.sizes(), src.options());
      const int64_t cdim = old_index.dim() <= dim ? old_index.dim() - 1 : dim;
      Variable count = std::get<0>(scatter_hip(ones, old_index, cdim, std::nullopt, out.size(dim), TS_SUM));
      count.masked_fill_(count < 1, 1);
      count = broadcast(count, out, dim);
      if (out.is_floating_point())
        out.true_divide_(count);
      else
        out.div_(count, "floor");
      ctx->save_for_backward({index, count});
      return {out};
    }
    Variable arg_out = std::get<1>(result).value();
    ctx->save_for_backward({index, arg_out});
    ctx->mark_non_differentiable({arg_out});
    return {out, arg_out};
  }

  static variable_list backward(AutogradContext *ctx, variable_list grad_outs) {
    auto grad_out = grad_outs[0];
    auto saved = ctx->get_saved_variables();
    const int64_t dim = ctx->saved_data["dim"].toInt();
    Variable grad_in;
    if (REDUCE == TS_SUM) {
      grad_in = gather_grad_rows(grad_out, saved[0], dim, std::nullopt);
    } else if (REDUCE == TS_MUL) {
      grad_in = at::gather(grad_out * saved[2], dim, saved[1], false).div_(saved[0]);
      grad_in.masked_fill_(grad_in.isnan(), 0);
    } else if (REDUCE == TS_MEAN) {
      grad_in = gather_grad_rows(grad_out, saved[0], dim, saved[1]);
    } else {
      grad_in = arg_backward_hip(grad_out, saved[1], saved_shape(ctx), dim);
    }
    return {grad_in, Variable(), Variable(), Variable(), Variable()};
  }
};

// --------------------------------------------------- autograd: segment_csr
// SegmentSum/Mean/Min/MaxCSR, csrc/segment_csr.cpp:57-174
template <int REDUCE> struct SegmentCsrFn : public torch::autograd::Function<SegmentCsrFn<REDUCE>> {
  static variable_list forward(AutogradContext *ctx, Variable src, Variable indptr,
                               std::optional<Variable> optional_out) {
    ctx->saved_data["src_shape"] = src.sizes();
    auto result = segment_csr_hip(src, indptr, optional_out, REDUCE);
    Variable out = std::get<0>(result);
    if (optional_out.has_value()) ctx->mark_dirty({optional_out.value()});
    if (REDUCE == TS_MIN || REDUCE == TS_MAX) {
      Variable arg_out = std::get<1>(result).value();
      ctx->save_for_backward({indptr, arg_out});
      ctx->mark_non_differentiable({arg_out});
      return {out, arg_out};
    }
    ctx->save_for_backward({indptr});
    return {out};
  }

  static variable_list backward(AutogradContext *ctx, variable_list grad_outs) {
    auto grad_out = grad_outs[0];
    auto saved = ctx->get_saved_variables();
    auto indptr = saved[0];
    auto src_shape = saved_shape(ctx);
    Variable grad_in;
    if (REDUCE == TS_MIN || REDUCE == TS_MAX) {
      grad_in = arg_backward_hip(grad_out, saved[1], src_shape, indptr.dim() - 1);
    } else {
      grad_in = at::empty(src_shape, grad_out.options());
      // mean: one fused gather-and-divide instead of upstream's two gathers
      // and a division (csrc/segment_csr.cpp:100-109)
      if (grad_in.numel() > 0) gather_csr_hip(grad_out, indptr, grad_in, REDUCE == TS_MEAN);
    }
    return {grad_in, Variable(), Variable()};
  }
};

// GatherCSR, csrc/segment_csr.cpp:176-199
struct GatherCsrFn : public torch::autograd::Function<GatherCsrFn> {
  static variable_list forward(AutogradContext *ctx, Variable src, Variable indptr,
                               std::optional<Variable> optional_out) {
    ctx->saved_data["src_shape"] = src.sizes();
    Variable out = gather_csr_hip(src, indptr, optional_out);
    ctx->save_for_backward({indptr});
    if (optional_out.has_value()) ctx->mark_dirty({optional_out.value()});
    return {out};
  }
  static variable_list backward(AutogradContext *ctx, variable_list grad_outs) {
    auto grad_out = grad_outs[0];
    auto indptr = ctx->get_saved_variables()[0];
    Variable grad_in = at::empty(saved_shape(ctx), grad_out.options());
    segment_csr_hip(grad_out, indptr, grad_in, TS_SUM);
    return {grad_in, Variable(), Variable()};
  }
};

// --------------------------------------------------- autograd: segment_coo
// SegmentSum/Mean/Min/MaxCOO, csrc/segment_coo.cpp:57-177
template <int REDUCE> struct SegmentCooFn : public torch::autograd::Function<SegmentCooFn<REDUCE>> {
  static variable_list forward(AutogradContext *ctx, Variable src, Variable index,
                               std::optional<Variable> optional_out, OptInt dim_size) {
    ctx->saved_data["src_shape"] = src.sizes();
    auto result = segment_coo_hip(src, index, optional_out, dim_size, REDUCE);
    Variable out = std::get<0>(result);
    if (optional_out.has_value()) ctx->mark_dirty({optional_out.value()});
    if (REDUCE == TS_SUM) {
      ctx->save_for_backward({index});
      return {out};
    }
    Variable second = std::get<1>(result).value();
    ctx->save_for_backward({index, second});
    if (REDUCE == TS_MEAN) return {out};
    ctx->mark_non_differentiable({second});
    return {out, second};
  }

  static variable_list backward(AutogradContext *ctx, variable_list grad_outs) {
    auto grad_out = grad_outs[0];
    auto saved = ctx->get_saved_variables();
    auto index = saved[0];
    auto src_shape = saved_shape(ctx);
    Variable grad_in;
    if (REDUCE == TS_MIN || REDUCE == TS_MAX) {
      grad_in = arg_backward_hip(grad_out, saved[1], src_shape, index.dim() - 1);
    } else {
      grad_in = at::empty(src_shape, grad_out.options());
      if (grad_in.numel() > 0) {
        if (REDUCE == TS_MEAN)
          gather_coo_hip(grad_out, index, grad_in, saved[1]);  // fused gather / count
        else
          gather_coo_hip(grad_out, index, grad_in);
      }
    }
    return {grad_in, Variable(), Variable(), Variable()};
  }
};

// GatherCOO, csrc/segment_coo.cpp:179-202
struct GatherCooFn : public torch::autograd::Function<GatherCooFn> {
  static variable_list forward(AutogradContext *ctx, Variable src, Variable index,
                               std::optional<Variable> optional_out) {
    ctx->saved_data["src_shape"] = src.sizes();
    Variable out = gather_coo_hip(src, index, optional_out);
    ctx->save_for_backward({index});
    if (optional_out.has_value()) ctx->mark_dirty({optional_out.value()});
    return {out};
  }
  static variable_list backward(AutogradContext *ctx, variable_list grad_outs) {
    auto grad_out = grad_outs[0];
    auto index = ctx->get_saved_variables()[0];
    auto src_shape = saved_shape(ctx);
    Variable grad_in = at::zeros(src_shape, grad_out.options());
    if (grad_out.numel() > 0) segment_coo_hip(grad_out, index, grad_in, std::nullopt, TS_SUM);
    return {grad_in, Variable(), Variable()};
  }
};

// ------------------------------------------------- autograd: group softmax
// scatter_softmax / scatter_log_softmax of torch_scatter/composite/softmax.py:8-59 as one
// operator (upstream composes them in Python from scatter_max, scatter_sum, gather and
// elementwise ops). One index per row runs the fused kernels; an index that differs
// between the columns of a row is composed from the registered operators as upstream does.
struct GroupLayout {
  bool fused;
  int64_t B, E, K, sb, se;
};
GroupLayout group_layout(const Tensor &src, const Tensor &index, int64_t dim) {
  GroupLayout l;
  l.B = prod(src.sizes(), 0, dim);
  l.E = src.size(dim);
  l.K = prod(src.sizes(), dim + 1, src.dim());
  auto sb = collapsed_stride(index, 0, dim);
  auto sk = collapsed_stride(index, dim + 1, index.dim());
  l.fused = sb.has_value() && sk.has_value() && (l.K == 1 || sk.value() == 0);
  l.sb = sb.value_or(0);
  l.se = index.stride(dim);
  return l;
}

struct GroupSoftmaxFn : public torch::autograd::Function<GroupSoftmaxFn> {
  static variable_list forward(AutogradContext *ctx, Variable src, Variable index, int64_t dim, int64_t N,
                               bool log_space, double eps) {
    check_device(src, "src");
    check_device(index, "index");
    c10::DeviceGuard guard(src.device());
    src = src.contiguous();
    const GroupLayout l = group_layout(src, index, dim);
    Tensor out = at::empty_like(src);
    // the workspace that opens every route: three passes, buckets of groups, one-pass tiles
    Tensor ws = workspace(ts_group_workspace_bytes(l.B, l.E, l.K, N, dtype_code(src)), src);
    check_status(ts_group_softmax(src.data_ptr(), index.data_ptr<int64_t>(), out.data_ptr(), l.B, l.E, l.K, N, l.sb,
                                  l.se, dtype_code(src), log_space ? 1 : 0, eps, ws.data_ptr(),
                                  static_cast<size_t>(ws.numel()), stream_of(src)),
                 "scatter_softmax");
    ctx->saved_data["dim"] = dim;
    ctx->saved_data["N"] = N;
    ctx->saved_data["log"] = log_space;
    ctx->save_for_backward({out, index});
    return {out};
  }

  static variable_list backward(AutogradContext *ctx, variable_list grad_outs) {
    auto saved = ctx->get_saved_variables();
    Tensor out = saved[0], index = saved[1];
    Tensor grad_out = grad_outs[0].contiguous();
    c10::DeviceGuard guard(out.device());
    const int64_t dim = ctx->saved_data["dim"].toInt();
    const int64_t N = ctx->saved_data["N"].toInt();
    const bool log_space = ctx->saved_data["log"].toBool();
    const GroupLayout l = group_layout(out, index, dim);
    Tensor grad_in = at::empty_like(out);
    Tensor ws = workspace(ts_group_workspace_bytes(l.B, l.E, l.K, N, dtype_code(out)), out);
    check_status(ts_group_softmax_backward(out.data_ptr(), grad_out.data_ptr(), index.data_ptr<int64_t>(),
                                           grad_in.data_ptr(), l.B, l.E, l.K, N, l.sb, l.se, dtype_code(out),
                                           log_space ? 1 : 0, ws.data_ptr(), static_cast<size_t>(ws.numel()),
                                           stream_of(out)),
                 "scatter_softmax backward");
    return {grad_in, Variable(), Variable(), Variable(), Variable(), Variable()};
  }
};

// scatter_logsumexp of torch_scatter/composite/logsumexp.py:8-57 for the call without `out`
struct GroupLogSumExpFn : public torch::autograd::Function<GroupLogSumExpFn> {
  static variable_list forward(AutogradContext *ctx, Variable src, Variable index, int64_t dim, int64_t N,
                               double eps) {
    check_device(src, "src");
    check_device(index, "index");
    c10::DeviceGuard guard(src.device());
    src = src.contiguous();
    const GroupLayout l = group_layout(src, index, dim);
    auto sizes = src.sizes().vec();
    sizes[dim] = N;
    Tensor out = at::empty(sizes, src.options());
    // the larger workspace of the route through buckets of groups, where that route applies
    const size_t ws_bytes = ts_group_workspace_bytes(l.B, l.E, l.K, N, dtype_code(src));
    Tensor ws = workspace(ws_bytes, src);
    check_status(ts_group_logsumexp(src.data_ptr(), index.data_ptr<int64_t>(), out.data_ptr(), l.B, l.E, l.K, N, l.sb,
                                    l.se, dtype_code(src), eps, ws.data_ptr(), static_cast<size_t>(ws.numel()),
                                    stream_of(src)),
                 "scatter_logsumexp");
    ctx->saved_data["dim"] = dim;
    ctx->save_for_backward({src, index, out});
    return {out};
  }

  static variable_list backward(AutogradContext *ctx, variable_list grad_outs) {
    auto saved = ctx->get_saved_variables();
    Tensor src = saved[0], index = saved[1], out = saved[2];
    Tensor grad_out = grad_outs[0].contiguous();
    c10::DeviceGuard guard(src.device());
    const int64_t dim = ctx->saved_data["dim"].toInt();
    const GroupLayout l = group_layout(src, index, dim);
    Tensor grad_in = at::empty_like(src);
    Tensor ws = workspace(ts_group_softmax_workspace_bytes(l.B, out.size(dim), l.K, dtype_code(src)), src);
    check_status(ts_group_logsumexp_backward_with_workspace(src.data_ptr(), index.data_ptr<int64_t>(), out.data_ptr(),
                                                            grad_out.data_ptr(), grad_in.data_ptr(), l.B, l.E, l.K,
                                                            out.size(dim), l.sb, l.se, dtype_code(src), ws.data_ptr(),
                                                            static_cast<size_t>(ws.numel()), stream_of(src)),
                 "scatter_logsumexp backward");
    return {grad_in, Variable(), Variable(), Variable(), Variable()};
  }
};

// scatter_std of torch_scatter/composite/std.py:8-41 for the call without `out`: group sums and
// counts from the scatter kernels, then one pass for the squared deviations and one per group
struct GroupStdFn : public torch::autograd::Function<GroupStdFn> {
  static variable_list forward(AutogradContext *ctx, Variable src, Variable index, int64_t dim, int64_t N,
                               bool unbiased) {
    check_device(src, "src");
    check_device(index, "index");
    c10::DeviceGuard guard(src.device());
    src = src.contiguous();
    const GroupLayout l = group_layout(src, index, dim);
    Tensor total, count, out;
    const size_t bins_bytes = ts_group_bins_workspace_bytes(l.B, l.E, l.K, N, dtype_code(src));
    if (bins_bytes > 0 && l.B * N * l.K > 0 && (reinterpret_cast<uintptr_t>(src.data_ptr()) & 15) == 0) {
      // group sums, counts and result from one gather of src through buckets of groups
      auto sizes = src.sizes().vec();
      sizes[dim] = N;
      total = at::empty(sizes, src.options());
      count = at::empty({l.B * N}, src.options().dtype(at::kInt));
      out = at::empty_like(total);
      Tensor ws = workspace(bins_bytes, src);
      check_status(ts_group_std_forward(src.data_ptr(), index.data_ptr<int64_t>(), total.data_ptr(),
                                        count.data_ptr<int32_t>(), out.data_ptr(), l.B, l.E, l.K, N, l.sb, l.se,
                                        dtype_code(src), unbiased ? 1 : 0, ws.data_ptr(), bins_bytes, stream_of(src)),
                   "scatter_std");
    } else {
      total = std::get<0>(scatter_hip(src, index, dim, std::nullopt, N, TS_SUM)).contiguous();
      count = at::empty({l.B * N}, src.options().dtype(at::kInt));
      check_status(ts_scatter_count(index.data_ptr<int64_t>(), count.data_ptr<int32_t>(), l.B, l.E, N, l.sb, l.se,
                                    stream_of(src)),
                   "scatter_std count");
      out = at::empty_like(total);
      Tensor ws = workspace(ts_group_softmax_workspace_bytes(l.B, N, l.K, dtype_code(src)), src);
      check_status(ts_group_std(src.data_ptr(), index.data_ptr<int64_t>(), total.data_ptr(), count.data_ptr<int32_t>(),
                                out.data_ptr(), l.B, l.E, l.K, N, l.sb, l.se, dtype_code(src), unbiased ? 1 : 0,
                                ws.data_ptr(), static_cast<size_t>(ws.numel()), stream_of(src)),
                   "scatter_std");
    }
    ctx->saved_data["dim"] = dim;
    ctx->saved_data["unbiased"] = unbiased;
    ctx->save_for_backward({src, index, total, count, out});
    return {out};
  }

  static variable_list backward(AutogradContext *ctx, variable_list grad_outs) {
    auto saved = ctx->get_saved_variables();
    Tensor src = saved[0], index = saved[1], total = saved[2], count = saved[3], out = saved[4];
    Tensor grad_out = grad_outs[0].contiguous();
    c10::DeviceGuard guard(src.device());
    const int64_t dim = ctx->saved_data["dim"].toInt();
    const bool unbiased = ctx->saved_data["unbiased"].toBool();
    const GroupLayout l = group_layout(src, index, dim);
    Tensor grad_in = at::empty_like(src);
    Tensor ws = workspace(ts_group_softmax_workspace_bytes(l.B, out.size(dim), l.K, dtype_code(src)), src);
    check_status(ts_group_std_backward_with_workspace(src.data_ptr(), index.data_ptr<int64_t>(), total.data_ptr(),
                                                      count.data_ptr<int32_t>(), out.data_ptr(), grad_out.data_ptr(),
                                                      grad_in.data_ptr(), l.B, l.E, l.K, out.size(dim), l.sb, l.se,
                                                      dtype_code(src), unbiased ? 1 : 0, ws.data_ptr(),
                                                      static_cast<size_t>(ws.numel()), stream_of(src)),
                 "scatter_std backward");
    return {grad_in, Variable(), Variable(), Variable(), Variable()};
  }
};

// ------------------------------------------------- index formats and the sorted scatter
// Not in the reference: its callers bring `row` and `rowptr` from the same sparse matrix
// (benchmark/scatter_segment.py:38-41). index_to_indptr / indptr_to_index convert between the two,
// sort_index turns an unsorted index into (perm, indptr) once, and scatter_sorted then runs scatter's
// reductions as a segmented reduction over permuted rows: no atomics, the same bits on every call.
void check_long_device(const Tensor &t, const char *name) {
  check_device(t, name);
  TORCH_CHECK(t.scalar_type() == at::kLong, name, " must be int64");
}

Tensor index_to_indptr(Tensor index, int64_t dim_size) {
  check_long_device(index, "index");
  TORCH_CHECK(index.dim() >= 1 && dim_size >= 0, "Input mismatch");
  c10::DeviceGuard guard(index.device());
  index = index.contiguous();
  const int64_t E = index.size(-1), B = E > 0 ? index.numel() / E : prod(index.sizes(), 0, index.dim() - 1);
  auto sizes = index.sizes().vec();
  sizes.back() = dim_size + 1;
  Tensor indptr = at::empty(sizes, index.options());
  check_status(ts_index_to_indptr(index.data_ptr<int64_t>(), indptr.data_ptr<int64_t>(), B, E, dim_size, E,
                                  stream_of(index)),
               "index_to_indptr");
  return indptr;
}

Tensor indptr_to_index(Tensor indptr, OptInt num_entries) {
  check_long_device(indptr, "indptr");
  TORCH_CHECK(indptr.dim() >= 1 && indptr.size(-1) >= 1, "Input mismatch");
  c10::DeviceGuard guard(indptr.device());
  indptr = indptr.contiguous();
  const int64_t N = indptr.size(-1) - 1, B = indptr.numel() / (N + 1);
  // every batch row must hold the same number of entries; without num_entries it is read back
  const int64_t E = num_entries.has_value() ? num_entries.value()
                                            : (indptr.numel() > 0 ? indptr.select(-1, N).max().item<int64_t>() : 0);
  auto sizes = indptr.sizes().vec();
  sizes.back() = E;
  Tensor index = at::empty(sizes, indptr.options());
  if (index.numel() == 0) return index;
  Tensor ws = workspace(ts_indptr_to_index_workspace_bytes(B, N), indptr);
  check_status(ts_indptr_to_index(indptr.data_ptr<int64_t>(), index.data_ptr<int64_t>(), B, N, E, N + 1, ws.data_ptr(),
                                  static_cast<size_t>(ws.numel()), stream_of(indptr)),
               "indptr_to_index");
  return index;
}

std::tuple<Tensor, Tensor> sort_index(Tensor index, int64_t dim_size) {
  check_long_device(index, "index");
  TORCH_CHECK(index.dim() == 1, "sort_index expects a one-dimensional index");
  TORCH_CHECK(dim_size >= 0, "Input mismatch");
  c10::DeviceGuard guard(index.device());
  index = index.contiguous();
  const int64_t E = index.numel();
  Tensor perm = at::empty({E}, index.options().dtype(at::kInt));
  Tensor indptr = at::empty({dim_size + 1}, index.options());
  Tensor ws = workspace(ts_sort_index_workspace_bytes(E, dim_size), index);
  check_status(ts_sort_index(index.data_ptr<int64_t>(), perm.data_ptr<int32_t>(), indptr.data_ptr<int64_t>(), E,
                             dim_size, ws.data_ptr(), static_cast<size_t>(ws.numel()), stream_of(index)),
               "sort_index");
  // one read-back at set-up: entries outside [0, dim_size) sort behind the last row
  TORCH_CHECK(indptr[dim_size].item<int64_t>() == E, "sort_index: index out of range [0, ", dim_size, ")");
  return std::make_tuple(perm, indptr);
}

template <int REDUCE> struct SortedScatterFn : public torch::autograd::Function<SortedScatterFn<REDUCE>> {
  static variable_list forward(AutogradContext *ctx, Variable src, Variable index, Variable perm, Variable indptr,
                               int64_t dim) {
    check_device(src, "src");
    check_long_device(index, "index");
    check_long_device(indptr, "indptr");
    check_device(perm, "perm");
    TORCH_CHECK(perm.scalar_type() == at::kInt, "perm must be int32");
    TORCH_CHECK(src.dim() >= 1, "Input mismatch");
    dim = dim < 0 ? src.dim() + dim : dim;
    TORCH_CHECK(dim >= 0 && dim < src.dim(), "Input mismatch");
    TORCH_CHECK(index.dim() == 1 && perm.dim() == 1 && indptr.dim() == 1 && indptr.numel() >= 1, "Input mismatch");
    const int64_t E = src.size(dim), N = indptr.numel() - 1;
    TORCH_CHECK(index.numel() == E && perm.numel() == E, "Input mismatch");
    c10::DeviceGuard guard(src.device());
    src = src.contiguous();
    perm = perm.contiguous();
    indptr = indptr.contiguous();
    const int64_t B = prod(src.sizes(), 0, dim), K = prod(src.sizes(), dim + 1, src.dim());
    auto sizes = src.sizes().vec();
    sizes[dim] = N;
    constexpr bool kArg = REDUCE == TS_MIN || REDUCE == TS_MAX;
    // integer mean: scatter divides with floor (csrc/scatter.cpp:138-141), the segmented kernel truncates
    const bool int_mean = REDUCE == TS_MEAN && !src.is_floating_point();
    const int reduce = int_mean ? TS_SUM : REDUCE;
    Tensor out = at::empty(sizes, src.options());
    Tensor arg_out = kArg ? at::empty(sizes, index.options()) : Tensor();
    if (out.numel() > 0) {
      const size_t ws_bytes = ts_segment_csr_permuted_workspace_bytes(B, N, E, K, dtype_code(src), reduce);
      Tensor ws = workspace(ws_bytes, src);
      check_status(ts_segment_csr_permuted(src.data_ptr(), perm.data_ptr<int32_t>(), indptr.data_ptr<int64_t>(),
                                           out.data_ptr(), kArg ? arg_out.data_ptr<int64_t>() : nullptr, B, N, E, K, 0,
                                           0, dtype_code(src), reduce, ws.data_ptr(),
                                           static_cast<size_t>(ws.numel()), stream_of(src)),
                   "scatter_sorted");
      maybe_check_status_words(ws, ws_bytes, "scatter_sorted");
    }
    ctx->saved_data["dim"] = dim;
    ctx->saved_data["src_shape"] = src.sizes();
    Variable index_b = broadcast(index, src, dim);
    if (REDUCE == TS_MEAN) {
      Tensor count = (indptr.slice(0, 1, N + 1) - indptr.slice(0, 0, N)).clamp_min_(1);
      if (int_mean) out.div_(broadcast(count.to(src.scalar_type()), out, dim), "floor");
      if (src.requires_grad()) ctx->save_for_backward({index_b, broadcast(count.to(src.scalar_type()), out, dim)});
      return {out};
    }
    if (kArg) {
      ctx->save_for_backward({index_b, arg_out});
      ctx->mark_non_differentiable({arg_out});
      return {out, arg_out};
    }
    ctx->save_for_backward({index_b});
    return {out};
  }

  // as ScatterFn: csrc/scatter.cpp:70-81, 143-161, 184-196
  static variable_list backward(AutogradContext *ctx, variable_list grad_outs) {
    auto grad_out = grad_outs[0];
    auto saved = ctx->get_saved_variables();
    const int64_t dim = ctx->saved_data["dim"].toInt();
    Variable grad_in;
    if (REDUCE == TS_SUM) {
      grad_in = gather_grad_rows(grad_out, saved[0], dim, std::nullopt);
    } else if (REDUCE == TS_MEAN) {
      grad_in = gather_grad_rows(grad_out, saved[0], dim, saved[1]);
    } else {
      grad_in = arg_backward_hip(grad_out, saved[1], saved_shape(ctx), dim);
    }
    return {grad_in, Variable(), Variable(), Variable(), Variable()};
  }
};

}  // namespace

// ------------------------------------------------------- registered functions
// Exported with the names and signatures of the C++ API header (include/torchscatter/scatter.h).
using torch::Tensor;
using OptTensor = std::optional<Tensor>;
using OptInt = std::optional<int64_t>;
Tensor scatter_sum(Tensor src, Tensor index, int64_t dim, OptTensor out, OptInt dim_size) {
  return ScatterFn<TS_SUM>::apply(src, index, dim, out, dim_size)[0];
}
Tensor scatter_mul(Tensor src, Tensor index, int64_t dim, OptTensor out, OptInt dim_size) {
  return ScatterFn<TS_MUL>::apply(src, index, dim, out, dim_size)[0];
}
Tensor scatter_mean(Tensor src, Tensor index, int64_t dim, OptTensor out, OptInt dim_size) {
  return ScatterFn<TS_MEAN>::apply(src, index, dim, out, dim_size)[0];
}
std::tuple<Tensor, Tensor> scatter_min(Tensor src, Tensor index, int64_t dim, OptTensor out, OptInt dim_size) {
  auto r = ScatterFn<TS_MIN>::apply(src, index, dim, out, dim_size);
  return std::make_tuple(r[0], r[1]);
}
std::tuple<Tensor, Tensor> scatter_max(Tensor src, Tensor index, int64_t dim, OptTensor out, OptInt dim_size) {
  auto r = ScatterFn<TS_MAX>::apply(src, index, dim, out, dim_size);
  return std::make_tuple(r[0], r[1]);
}

Tensor segment_sum_csr(Tensor src, Tensor indptr, OptTensor out) {
  return SegmentCsrFn<TS_SUM>::apply(src, indptr, out)[0];
}
Tensor segment_mean_csr(Tensor src, Tensor indptr, OptTensor out) {
  return SegmentCsrFn<TS_MEAN>::apply(src, indptr, out)[0];
}
std::tuple<Tensor, Tensor> segment_min_csr(Tensor src, Tensor indptr, OptTensor out) {
  auto r = SegmentCsrFn<TS_MIN>::apply(src, indptr, out);
  return std::make_tuple(r[0], r[1]);
}
std::tuple<Tensor, Tensor> segment_max_csr(Tensor src, Tensor indptr, OptTensor out) {
  auto r = SegmentCsrFn<TS_MAX>::apply(src, indptr, out);
  return std::make_tuple(r[0], r[1]);
}
Tensor gather_csr(Tensor src, Tensor indptr, OptTensor out) { return GatherCsrFn::apply(src, indptr, out)[0]; }

Tensor segment_sum_coo(Tensor src, Tensor index, OptTensor out, OptInt dim_size) {
  return SegmentCooFn<TS_SUM>::apply(src, index, out, dim_size)[0];
}
Tensor segment_mean_coo(Tensor src, Tensor index, OptTensor out, OptInt dim_size) {
  return SegmentCooFn<TS_MEAN>::apply(src, index, out, dim_size)[0];
}
std::tuple<Tensor, Tensor> segment_min_coo(Tensor src, Tensor index, OptTensor out, OptInt dim_size) {
  auto r = SegmentCooFn<TS_MIN>::apply(src, index, out, dim_size);
  return std::make_tuple(r[0], r[1]);
}
std::tuple<Tensor, Tensor> segment_max_coo(Tensor src, Tensor index, OptTensor out, OptInt dim_size) {
  auto r = SegmentCooFn<TS_MAX>::apply(src, index, out, dim_size);
  return std::make_tuple(r[0], r[1]);
}
Tensor gather_coo(Tensor src, Tensor index, OptTensor out) { return GatherCooFn::apply(src, index, out)[0]; }

int64_t scatter::cuda_version() noexcept { return ts_hip_version(); }

namespace {

Tensor scatter_softmax(Tensor src, Tensor index, int64_t dim, OptInt dim_size, bool log_space, double eps) {
  TORCH_CHECK(src.is_floating_point(), log_space ? "`scatter_log_softmax`" : "`scatter_softmax`",
              " can only be computed over tensors with floating point data types.");
  dim = dim < 0 ? src.dim() + dim : dim;
  index = broadcast(index, src, dim);
  TORCH_CHECK(index.scalar_type() == at::kLong, "index must be int64");
  if (src.numel() == 0) return at::empty_like(src);
  const GroupLayout l = group_layout(src, index, dim);
  const int64_t N = dim_size.has_value() ? dim_size.value() : 1 + index.max().item<int64_t>();
  if (l.fused && N > 0 && l.B * N < 0x7FFFFFFFll)
    return GroupSoftmaxFn::apply(src, index, dim, N, log_space, eps)[0];
  // composite/softmax.py:16-29, :45-59
  Tensor shift = std::get<0>(scatter_max(src, index, dim, std::nullopt, dim_size)).gather(dim, index);
  Tensor z = src - shift;
  if (!log_space) {
    Tensor e = z.exp();
    return e.div(scatter_sum(e, index, dim, std::nullopt, dim_size).gather(dim, index));
  }
  Tensor norm = scatter_sum(z.exp(), index, dim, std::nullopt, dim_size).add(eps).log().gather(dim, index);
  return z.sub(norm);
}

Tensor scatter_logsumexp(Tensor src, Tensor index, int64_t dim, OptTensor out, OptInt dim_size, double eps) {
  TORCH_CHECK(src.is_floating_point(),
              "`scatter_logsumexp` can only be computed over tensors with floating point data types.");
  dim = dim < 0 ? src.dim() + dim : dim;
  index = broadcast(index, src, dim);
  TORCH_CHECK(index.scalar_type() == at::kLong, "index must be int64");
  int64_t N;
  if (out.has_value())
    N = out.value().size(dim);
  else if (dim_size.has_value())
    N = dim_size.value();
  else
    N = index.numel() == 0 ? 0 : 1 + index.max().item<int64_t>();
  auto sizes = src.sizes().vec();
  sizes[dim] = N;
  if (!out.has_value() && src.numel() > 0 && N > 0) {
    const GroupLayout l = group_layout(src, index, dim);
    if (l.fused && l.B * N < 0x7FFFFFFFll) return GroupLogSumExpFn::apply(src, index, dim, N, eps)[0];
  }
  // composite/logsumexp.py:29-57
  const double neg_inf = -std::numeric_limits<double>::infinity();
  Tensor group_max = at::full(sizes, neg_inf, src.options());
  if (src.numel() > 0) scatter_max(src, index, dim, group_max, N);
  Tensor z = src - group_max.gather(dim, index);
  z.masked_fill_(z.isnan(), neg_inf);
  OptTensor previous;
  if (out.has_value()) {
    previous = out.value().clone();
    out = out.value().sub_(group_max).exp_();
  }
  Tensor total = scatter_sum(z.exp_(), index, dim, out, N);
  Tensor result = total.add_(eps).log_().add_(group_max);
  if (!previous.has_value()) return result.nan_to_num_(0.0, std::nullopt, 0.0);
  Tensor bad = result.isfinite().logical_not();
  result.index_put_({bad}, previous.value().index({bad}));
  return result;
}

Tensor scatter_std(Tensor src, Tensor index, int64_t dim, OptTensor out, OptInt dim_size, bool unbiased) {
  dim = dim < 0 ? src.dim() + dim : dim;
  if (out.has_value()) dim_size = out.value().size(dim);
  const Tensor index_given = index;
  index = broadcast(index, src, dim);
  TORCH_CHECK(index.scalar_type() == at::kLong, "index must be int64");
  if (!out.has_value() && src.is_floating_point() && src.numel() > 0) {
    const int64_t N = dim_size.has_value() ? dim_size.value() : 1 + index.max().item<int64_t>();
    const GroupLayout l = group_layout(src, index, dim);
    if (l.fused && N > 0 && l.B * N < 0x7FFFFFFFll) return GroupStdFn::apply(src, index, dim, N, unbiased)[0];
  }
  // composite/std.py:19-41
  const int64_t count_dim = index_given.dim() <= dim ? index_given.dim() - 1 : dim;
  Tensor count = scatter_sum(at::ones(index_given.sizes(), src.options()), index_given, count_dim, std::nullopt, dim_size);
  Tensor total = scatter_sum(src, index, dim, std::nullopt, dim_size);
  count = broadcast(count, total, dim).clamp(1);
  Tensor centred = src - total.div(count).gather(dim, index);
  Tensor sq = scatter_sum(centred * centred, index, dim, out, dim_size);
  if (unbiased) count = count.sub(1).clamp_(1);
  return sq.div(count + 1e-6).sqrt();
}

// (values, positions); positions is an empty tensor unless reduce is min or max
std::tuple<Tensor, Tensor> scatter_sorted(Tensor src, Tensor index, Tensor perm, Tensor indptr, int64_t dim,
                                          std::string reduce) {
  const int code = reduce_code(reduce);
  if ((code == TS_MIN || code == TS_MAX) && src.dim() >= 1 && indptr.dim() == 1 && indptr.numel() >= 1) {
    // rows under 64 bytes: min / max through the atomic kernels are as exact and faster
    const int64_t d = dim < 0 ? src.dim() + dim : dim;
    if (d >= 0 && d < src.dim() && prod(src.sizes(), d + 1, src.dim()) * (int64_t)src.element_size() < 64 &&
        index.numel() == src.size(d)) {
      const int64_t N = indptr.numel() - 1;
      return code == TS_MIN ? scatter_min(src, index, d, std::nullopt, N) : scatter_max(src, index, d, std::nullopt, N);
    }
  }
  switch (code) {
  case TS_SUM:
    return std::make_tuple(SortedScatterFn<TS_SUM>::apply(src, index, perm, indptr, dim)[0],
                           at::empty({0}, index.options()));
  case TS_MEAN:
    return std::make_tuple(SortedScatterFn<TS_MEAN>::apply(src, index, perm, indptr, dim)[0],
                           at::empty({0}, index.options()));
  case TS_MIN: {
    auto r = SortedScatterFn<TS_MIN>::apply(src, index, perm, indptr, dim);
    return std::make_tuple(r[0], r[1]);
  }
  case TS_MAX: {
    auto r = SortedScatterFn<TS_MAX>::apply(src, index, perm, indptr, dim);
    return std::make_tuple(r[0], r[1]);
  }
  default: TORCH_CHECK(false, "scatter_sorted: reduce must be sum, mean, min or max");
  }
}

int64_t cuda_version() { return ts_hip_version(); }  // csrc/version.cpp:28-38 returns HIP_VERSION on ROCm

}  // namespace

static auto registry = torch::RegisterOperators()
                           .op("torch_scatter::cuda_version", &cuda_version)
                           .op("torch_scatter::scatter_sum", &scatter_sum)
                           .op("torch_scatter::scatter_mul", &scatter_mul)
                           .op("torch_scatter::scatter_mean", &scatter_mean)
                           .op("torch_scatter::scatter_min", &scatter_min)
                           .op("torch_scatter::scatter_max", &scatter_max)
                           .op("torch_scatter::segment_sum_csr", &segment_sum_csr)
                           .op("torch_scatter::segment_mean_csr", &segment_mean_csr)
                           .op("torch_scatter::segment_min_csr", &segment_min_csr)
                           .op("torch_scatter::segment_max_csr", &segment_max_csr)
                           .op("torch_scatter::gather_csr", &gather_csr)
                           .op("torch_scatter::segment_sum_coo", &segment_sum_coo)
                           .op("torch_scatter::segment_mean_coo", &segment_mean_coo)
                           .op("torch_scatter::segment_min_coo", &segment_min_coo)
                           .op("torch_scatter::segment_max_coo", &segment_max_coo)
                           .op("torch_scatter::gather_coo", &gather_coo)
                           .op("torch_scatter::scatter_softmax", &scatter_softmax)
                           .op("torch_scatter::scatter_logsumexp", &scatter_logsumexp)
                           .op("torch_scatter::scatter_std", &scatter_std)
                           .op("torch_scatter::index_to_indptr", &index_to_indptr)
                           .op("torch_scatter::indptr_to_index", &indptr_to_index)
                           .op("torch_scatter::sort_index", &sort_index)
                           .op("torch_scatter::scatter_sorted", &scatter_sorted);
