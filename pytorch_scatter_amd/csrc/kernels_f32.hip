// Kernel instantiations for element type float.
#include "csr_reduce.h"
#include "csr_small.h"
#include "csr_gather.h"
#include "coo_gather.h"
#include "scatter.h"
#include "elementwise.h"
#include "group_softmax.h"

namespace ts {
TS_INSTANTIATE_CSR_REDUCE(float, 4)
TS_INSTANTIATE_CSR_GATHER(float, 4)
TS_INSTANTIATE_COO_GATHER(float, 4)
TS_INSTANTIATE_SCATTER(float, 4)
TS_INSTANTIATE_ELEMENTWISE(float)
TS_INSTANTIATE_GROUP_SOFTMAX(float, 4)
}  // namespace ts
