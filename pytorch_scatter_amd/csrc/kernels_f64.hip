// Kernel instantiations for element type double.
#include "csr_reduce.h"
#include "csr_small.h"
#include "csr_gather.h"
#include "coo_gather.h"
#include "scatter.h"
#include "elementwise.h"
#include "group_softmax.h"

namespace ts {
TS_INSTANTIATE_CSR_REDUCE(double, 2)
TS_INSTANTIATE_CSR_GATHER(double, 2)
TS_INSTANTIATE_COO_GATHER(double, 2)
TS_INSTANTIATE_SCATTER(double, 2)
TS_INSTANTIATE_ELEMENTWISE(double)
TS_INSTANTIATE_GROUP_SOFTMAX(double, 2)
}  // namespace ts
