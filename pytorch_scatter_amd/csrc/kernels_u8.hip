// Kernel instantiations for element type uint8_t.
#include "csr_reduce.h"
#include "csr_small.h"
#include "csr_gather.h"
#include "coo_gather.h"
#include "scatter.h"
#include "elementwise.h"

namespace ts {
TS_INSTANTIATE_CSR_REDUCE(uint8_t, 16)
TS_INSTANTIATE_CSR_GATHER(uint8_t, 16)
TS_INSTANTIATE_COO_GATHER(uint8_t, 16)
TS_INSTANTIATE_SCATTER(uint8_t, 16)
TS_INSTANTIATE_ELEMENTWISE(uint8_t)
}  // namespace ts
