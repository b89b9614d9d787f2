// Kernel instantiations for element type int64_t.
#include "csr_reduce.h"
#include "csr_small.h"
#include "csr_gather.h"
#include "coo_gather.h"
#include "scatter.h"
#include "elementwise.h"

namespace ts {
TS_INSTANTIATE_CSR_REDUCE(int64_t, 2)
TS_INSTANTIATE_CSR_GATHER(int64_t, 2)
TS_INSTANTIATE_COO_GATHER(int64_t, 2)
TS_INSTANTIATE_SCATTER(int64_t, 2)
TS_INSTANTIATE_ELEMENTWISE(int64_t)
}  // namespace ts
