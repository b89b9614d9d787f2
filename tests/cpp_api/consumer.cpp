// A C++ consumer of the installed API, written the way a user of the reference's
// C++ API would write it (README.md:156-168, csrc/scatter.h:13-80): include the
// header, call the free functions on torch tensors.
//
//   consumer --version   prints scatter::cuda_version(); needs no GPU
//   consumer             runs scatter_sum / scatter_max / segment_*_csr / gather_csr on cuda:0,
//                        checks them against host loops and prints "ok"
#include <torchscatter/scatter.h>

#include <torch/torch.h>

#include <cstdio>
#include <cstring>
#include <vector>

static int fail(const char *what) {
  std::printf("FAILED: %s\n", what);
  return 1;
}

int main(int argc, char **argv) {
  if (argc > 1 && std::strcmp(argv[1], "--version") == 0) {
    std::printf("%lld\n", (long long)scatter::cuda_version());
    return 0;
  }
  torch::manual_seed(0);
  const int64_t E = 5000, N = 300, K = 7;
  auto dev = torch::Device(torch::kCUDA, 0);
  auto src_h = torch::randn({E, K});
  auto idx_h = torch::randint(N, {E}, torch::kLong);
  auto src = src_h.to(dev), idx = idx_h.to(dev);

  // scatter_sum / scatter_max against host loops
  auto sum = scatter_sum(src, idx, 0, std::nullopt, N).cpu();
  auto [mx, arg] = scatter_max(src, idx, 0, std::nullopt, N);
  mx = mx.cpu();
  arg = arg.cpu();
  auto want_sum = torch::zeros({N, K}, torch::kDouble);
  auto want_max = torch::full({N, K}, -INFINITY);
  auto want_arg = torch::full({N, K}, E, torch::kLong);
  {
    auto s = src_h.accessor<float, 2>();
    auto i = idx_h.accessor<int64_t, 1>();
    auto ws = want_sum.accessor<double, 2>();
    auto wm = want_max.accessor<float, 2>();
    auto wa = want_arg.accessor<int64_t, 2>();
    for (int64_t e = 0; e < E; e++)
      for (int64_t k = 0; k < K; k++) {
        ws[i[e]][k] += s[e][k];
        if (s[e][k] > wm[i[e]][k]) wm[i[e]][k] = s[e][k], wa[i[e]][k] = e;
      }
  }
  if (!torch::allclose(sum.to(torch::kDouble), want_sum, 1e-5, 1e-5)) return fail("scatter_sum");
  auto hit = want_arg.lt(E);
  if (!torch::equal(mx.masked_select(hit), want_max.masked_select(hit))) return fail("scatter_max values");
  if (!torch::equal(arg, want_arg)) return fail("scatter_max arg");

  // sorted index -> row pointers; the three families must agree
  auto sorted = std::get<0>(idx_h.sort());
  auto counts = torch::bincount(sorted, {}, N);
  auto indptr_h = torch::cat({torch::zeros({1}, torch::kLong), counts.cumsum(0)});
  auto sidx = sorted.to(dev), indptr = indptr_h.to(dev);
  auto a = segment_sum_csr(src, indptr, std::nullopt);
  auto b = segment_sum_coo(src, sidx, std::nullopt, N);
  auto c = scatter_sum(src, sidx, 0, std::nullopt, N);
  if (!torch::allclose(a, b, 1e-5, 1e-5) || !torch::allclose(a, c, 1e-5, 1e-5)) return fail("segment sums");
  auto [m1, a1] = segment_max_csr(src, indptr, std::nullopt);
  auto [m2, a2] = segment_max_coo(src, sidx, std::nullopt, N);
  auto nonempty = counts.gt(0).to(dev).unsqueeze(1).expand({N, K});
  if (!torch::equal(m1.masked_select(nonempty), m2.masked_select(nonempty))) return fail("segment max values");
  if (!torch::equal(a1, a2)) return fail("segment max arg");
  if (!torch::equal(gather_csr(a, indptr, std::nullopt), gather_coo(a, sidx, std::nullopt))) return fail("gathers");

  // autograd through the C++ API: d(sum of means)/d(src) = 1/count of the row
  auto x = src.clone().set_requires_grad(true);
  segment_mean_csr(x, indptr, std::nullopt).sum().backward();
  auto want_grad = (1.0 / counts.to(torch::kFloat)).index_select(0, sorted).unsqueeze(1).expand({E, K}).to(dev);
  if (!torch::allclose(x.grad(), want_grad, 1e-6, 1e-6)) return fail("segment_mean_csr backward");

  std::printf("ok\n");
  return 0;
}
