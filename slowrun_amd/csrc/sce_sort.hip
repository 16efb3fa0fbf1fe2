// Stable radix sort of (target, row) pairs: groups the rows by target for the one-hot part
// of dW.  Kept in its own translation unit because it is the only user of rocPRIM.
#include <cstring>
#include <hip/hip_runtime.h>
#include <rocprim/device/device_radix_sort.hpp>
#include <stdint.h>

namespace sce {

// tmp == nullptr: only *tmp_bytes is set.  Returns 0 on success.
int sort_pairs(void* tmp, size_t* tmp_bytes, const int32_t* kin, int32_t* kout, const int32_t* vin, int32_t* vout,
               size_t n, int end_bit, hipStream_t stream) {
  hipError_t e = rocprim::radix_sort_pairs(tmp, *tmp_bytes, kin, kout, vin, vout, n, 0u, (unsigned)end_bit, stream);
  return e == hipSuccess ? 0 : 1;
}

}  // namespace sce
