// TEST INFRASTRUCTURE ONLY. Binding of the reference's CPU kernels (compiled
// from /root/reference/csrc/cpu/*.cpp where they lie) under a namespace of
// their own, `ts_ref`, so that they can sit in one process next to the
// product's `torch_scatter::*` operators and serve as a second checker.
//
// The declarations come from the reference's own headers
// (csrc/cpu/scatter_cpu.h:5-8, segment_coo_cpu.h:5-11, segment_csr_cpu.h:5-11);
// nothing of the reference is copied here.
#include <torch/script.h>

#include "cpu/scatter_cpu.h"
#include "cpu/segment_coo_cpu.h"
#include "cpu/segment_csr_cpu.h"

namespace {

using torch::Tensor;
using OptTensor = std::optional<Tensor>;

// An undefined second output is returned as an empty int64 tensor.
Tensor or_empty(const OptTensor &t) {
  return t.has_value() ? t.value() : torch::empty({0}, torch::kLong);
}

std::tuple<Tensor, Tensor> ref_scatter(Tensor src, Tensor index, int64_t dim,
                                       OptTensor out, std::optional<int64_t> dim_size,
                                       std::string reduce) {
  auto r = scatter_cpu(src, index, dim, out, dim_size, reduce);
  return std::make_tuple(std::get<0>(r), or_empty(std::get<1>(r)));
}

std::tuple<Tensor, Tensor> ref_segment_coo(Tensor src, Tensor index, OptTensor out,
                                           std::optional<int64_t> dim_size,
                                           std::string reduce) {
  auto r = segment_coo_cpu(src, index, out, dim_size, reduce);
  return std::make_tuple(std::get<0>(r), or_empty(std::get<1>(r)));
}

std::tuple<Tensor, Tensor> ref_segment_csr(Tensor src, Tensor indptr, OptTensor out,
                                           std::string reduce) {
  auto r = segment_csr_cpu(src, indptr, out, reduce);
  return std::make_tuple(std::get<0>(r), or_empty(std::get<1>(r)));
}

Tensor ref_gather_coo(Tensor src, Tensor index, OptTensor out) {
  return gather_coo_cpu(src, index, out);
}

Tensor ref_gather_csr(Tensor src, Tensor indptr, OptTensor out) {
  return gather_csr_cpu(src, indptr, out);
}

} // namespace

static auto registry = torch::RegisterOperators()
                           .op("ts_ref::scatter", &ref_scatter)
                           .op("ts_ref::segment_coo", &ref_segment_coo)
                           .op("ts_ref::segment_csr", &ref_segment_csr)
                           .op("ts_ref::gather_coo", &ref_gather_coo)
                           .op("ts_ref::gather_csr", &ref_gather_csr);
