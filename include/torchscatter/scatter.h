// C++ API of the gfx950 torch_scatter operator library (libtorchscatter.so /
// _torch_scatter_hip.so). The functions are the ones the reference installs
// for C++ users (csrc/scatter.h:13-80): same names, argument order and return
// types, so code written against that header compiles against this one and
// links against this library instead. Each call goes through the same autograd
// functions as the registered torch.ops.torch_scatter.* operators.
//
// Tensors must live on a HIP device ("cuda" device type under PyTorch-ROCm);
// there is no CPU path and a CPU tensor raises c10::Error.
//
//   #include <torchscatter/scatter.h>
//   auto out = scatter_sum(src, index, /*dim=*/0, std::nullopt, /*dim_size=*/n);
#pragma once

#include <torch/types.h>

#include <cstdint>
#include <optional>
#include <tuple>

#define TORCHSCATTER_API __attribute__((visibility("default")))

namespace scatter {
// HIP_VERSION the kernels were built with (the reference returns the same
// number from a ROCm build, csrc/version.cpp:28-38).
TORCHSCATTER_API int64_t cuda_version() noexcept;
}  // namespace scatter

namespace torchscatter {
using Tensor = torch::Tensor;
using MaybeTensor = std::optional<torch::Tensor>;
using MaybeSize = std::optional<int64_t>;
using WithArg = std::tuple<torch::Tensor, torch::Tensor>;  // (values, arg)
}  // namespace torchscatter

// ---- scatter: out[..., index[i], ...] (op)= src[..., i, ...] along `dim`, index in any order.
// `index` is broadcast to src as the reference does (csrc/scatter.cpp:13-27). Without `out`
// the result has `dim_size` entries along `dim`, or max(index)+1 (which reads the index back).
TORCHSCATTER_API torchscatter::Tensor scatter_sum(torchscatter::Tensor src, torchscatter::Tensor index, int64_t dim,
                                                  torchscatter::MaybeTensor optional_out,
                                                  torchscatter::MaybeSize dim_size);
TORCHSCATTER_API torchscatter::Tensor scatter_mul(torchscatter::Tensor src, torchscatter::Tensor index, int64_t dim,
                                                  torchscatter::MaybeTensor optional_out,
                                                  torchscatter::MaybeSize dim_size);
TORCHSCATTER_API torchscatter::Tensor scatter_mean(torchscatter::Tensor src, torchscatter::Tensor index, int64_t dim,
                                                   torchscatter::MaybeTensor optional_out,
                                                   torchscatter::MaybeSize dim_size);
// min / max also return the position along `dim` of the winning entry (src.size(dim) for an empty row).
TORCHSCATTER_API torchscatter::WithArg scatter_min(torchscatter::Tensor src, torchscatter::Tensor index, int64_t dim,
                                                   torchscatter::MaybeTensor optional_out,
                                                   torchscatter::MaybeSize dim_size);
TORCHSCATTER_API torchscatter::WithArg scatter_max(torchscatter::Tensor src, torchscatter::Tensor index, int64_t dim,
                                                   torchscatter::MaybeTensor optional_out,
                                                   torchscatter::MaybeSize dim_size);

// ---- segment_*_coo: as scatter along the last dimension of `index`, which must be sorted there.
TORCHSCATTER_API torchscatter::Tensor segment_sum_coo(torchscatter::Tensor src, torchscatter::Tensor index,
                                                      torchscatter::MaybeTensor optional_out,
                                                      torchscatter::MaybeSize dim_size);
TORCHSCATTER_API torchscatter::Tensor segment_mean_coo(torchscatter::Tensor src, torchscatter::Tensor index,
                                                       torchscatter::MaybeTensor optional_out,
                                                       torchscatter::MaybeSize dim_size);
TORCHSCATTER_API torchscatter::WithArg segment_min_coo(torchscatter::Tensor src, torchscatter::Tensor index,
                                                       torchscatter::MaybeTensor optional_out,
                                                       torchscatter::MaybeSize dim_size);
TORCHSCATTER_API torchscatter::WithArg segment_max_coo(torchscatter::Tensor src, torchscatter::Tensor index,
                                                       torchscatter::MaybeTensor optional_out,
                                                       torchscatter::MaybeSize dim_size);
// out[..., e, ...] = src[..., index[e], ...]
TORCHSCATTER_API torchscatter::Tensor gather_coo(torchscatter::Tensor src, torchscatter::Tensor index,
                                                 torchscatter::MaybeTensor optional_out);

// ---- segment_*_csr: row r reduces src[indptr[r] : indptr[r+1]] along the last dimension of `indptr`.
TORCHSCATTER_API torchscatter::Tensor segment_sum_csr(torchscatter::Tensor src, torchscatter::Tensor indptr,
                                                      torchscatter::MaybeTensor optional_out);
TORCHSCATTER_API torchscatter::Tensor segment_mean_csr(torchscatter::Tensor src, torchscatter::Tensor indptr,
                                                       torchscatter::MaybeTensor optional_out);
TORCHSCATTER_API torchscatter::WithArg segment_min_csr(torchscatter::Tensor src, torchscatter::Tensor indptr,
                                                       torchscatter::MaybeTensor optional_out);
TORCHSCATTER_API torchscatter::WithArg segment_max_csr(torchscatter::Tensor src, torchscatter::Tensor indptr,
                                                       torchscatter::MaybeTensor optional_out);
// out[..., e, ...] = src[..., r, ...] for indptr[r] <= e < indptr[r+1]
TORCHSCATTER_API torchscatter::Tensor gather_csr(torchscatter::Tensor src, torchscatter::Tensor indptr,
                                                 torchscatter::MaybeTensor optional_out);
