// Kernel instantiations for element type f16_t.
#include "csr_reduce.h"
#include "csr_small.h"
#include "csr_gather.h"
#include "coo_gather.h"
#include "scatter.h"
#include "elementwise.h"
#include "group_softmax.h"

namespace ts {
TS_INSTANTIATE_CSR_REDUCE(f16_t, 8)
TS_INSTANTIATE_CSR_GATHER(f16_t, 8)
TS_INSTANTIATE_COO_GATHER(f16_t, 8)
TS_INSTANTIATE_SCATTER(f16_t, 8)
TS_INSTANTIATE_ELEMENTWISE(f16_t)
TS_INSTANTIATE_GROUP_SOFTMAX(f16_t, 8)
}  // namespace ts
