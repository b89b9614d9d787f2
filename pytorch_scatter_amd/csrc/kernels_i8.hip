// Kernel instantiations for element type int8_t.
#include "csr_reduce.h"
#include "csr_small.h"
#include "csr_gather.h"
#include "coo_gather.h"
#include "scatter.h"
#include "elementwise.h"

namespace ts {
TS_INSTANTIATE_CSR_REDUCE(int8_t, 16)
TS_INSTANTIATE_CSR_GATHER(int8_t, 16)
TS_INSTANTIATE_COO_GATHER(int8_t, 16)
TS_INSTANTIATE_SCATTER(int8_t, 16)
TS_INSTANTIATE_ELEMENTWISE(int8_t)
}  // namespace ts
