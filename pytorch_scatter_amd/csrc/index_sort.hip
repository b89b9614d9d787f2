// The stable sort behind ts_sort_index: rocPRIM's device-wide radix sort of (key, position) pairs.
#include <cstring>
#include <hip/hip_runtime.h>
#include <rocprim/rocprim.hpp>

#include "index_format.h"

namespace ts {

size_t sort_keys_temp_bytes(int64_t n, int end_bit) {
  size_t bytes = 0;
  rocprim::counting_iterator<int32_t> positions(0);
  const hipError_t e = rocprim::radix_sort_pairs(nullptr, bytes, static_cast<const uint32_t *>(nullptr),
                                                 static_cast<uint32_t *>(nullptr), positions,
                                                 static_cast<int32_t *>(nullptr), (size_t)n, 0u, (unsigned)end_bit,
                                                 (hipStream_t)0, false);
  return e == hipSuccess ? bytes : 0;
}

int sort_keys_to_perm(void *temp, size_t temp_bytes, const uint32_t *keys_in, uint32_t *keys_out, int32_t *perm,
                      int64_t n, int end_bit, hipStream_t s) {
  rocprim::counting_iterator<int32_t> positions(0);
  const hipError_t e = rocprim::radix_sort_pairs(temp, temp_bytes, keys_in, keys_out, positions, perm, (size_t)n, 0u,
                                                 (unsigned)end_bit, s, false);
  return e == hipSuccess ? TS_OK : TS_ERR_LAUNCH;
}

}  // namespace ts
