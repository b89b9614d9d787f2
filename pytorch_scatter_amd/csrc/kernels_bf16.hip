// Kernel instantiations for element type bf16_t.
#include "csr_reduce.h"
#include "csr_small.h"
#include "csr_gather.h"
#include "coo_gather.h"
#include "scatter.h"
#include "elementwise.h"
#include "group_softmax.h"

namespace ts {
TS_INSTANTIATE_CSR_REDUCE(bf16_t, 8)
TS_INSTANTIATE_CSR_GATHER(bf16_t, 8)
TS_INSTANTIATE_COO_GATHER(bf16_t, 8)
TS_INSTANTIATE_SCATTER(bf16_t, 8)
TS_INSTANTIATE_ELEMENTWISE(bf16_t)
TS_INSTANTIATE_GROUP_SOFTMAX(bf16_t, 8)
}  // namespace ts
