// Kernel instantiations for element type int16_t.
#include "csr_reduce.h"
#include "csr_small.h"
#include "csr_gather.h"
#include "coo_gather.h"
#include "scatter.h"
#include "elementwise.h"

namespace ts {
TS_INSTANTIATE_CSR_REDUCE(int16_t, 8)
TS_INSTANTIATE_CSR_GATHER(int16_t, 8)
TS_INSTANTIATE_COO_GATHER(int16_t, 8)
TS_INSTANTIATE_SCATTER(int16_t, 8)
TS_INSTANTIATE_ELEMENTWISE(int16_t)
}  // namespace ts
