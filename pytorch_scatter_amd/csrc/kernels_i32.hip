// Kernel instantiations for element type int32_t.
#include "csr_reduce.h"
#include "csr_small.h"
#include "csr_gather.h"
#include "coo_gather.h"
#include "scatter.h"
#include "elementwise.h"

namespace ts {
TS_INSTANTIATE_CSR_REDUCE(int32_t, 4)
TS_INSTANTIATE_CSR_GATHER(int32_t, 4)
TS_INSTANTIATE_COO_GATHER(int32_t, 4)
TS_INSTANTIATE_SCATTER(int32_t, 4)
TS_INSTANTIATE_ELEMENTWISE(int32_t)
}  // namespace ts
