// Stable radix sort of (uint32 key, uint64 value) pairs by key: rocPRIM's device-wide
// radix sort (a plain library routine), kept in its own translation unit.
#include <cstring>

#include <rocprim/rocprim.hpp>

#include "tn_common.h"

namespace tn {

// Bytes of temporary device storage a sort of n pairs needs.
int sort_pairs_temp_bytes(size_t n, int key_bits, size_t* bytes) {
    *bytes = 0;
    hipError_t e = rocprim::radix_sort_pairs(nullptr, *bytes, (const uint32_t*)nullptr, (uint32_t*)nullptr,
                                             (const uint64_t*)nullptr, (uint64_t*)nullptr, n, 0u, (unsigned)key_bits,
                                             (hipStream_t)0, false);
    if (e != hipSuccess) return fail(TN_ERR_HIP, std::string("rocprim::radix_sort_pairs (size query): ") + hipGetErrorString(e));
    return TN_OK;
}

// Sorts n pairs by the low key_bits bits of the key; equal keys keep their order.
int sort_pairs_u32_u64(void* temp, size_t temp_bytes, const uint32_t* keys_in, uint32_t* keys_out,
                       const uint64_t* vals_in, uint64_t* vals_out, size_t n, int key_bits, hipStream_t st) {
    hipError_t e = rocprim::radix_sort_pairs(temp, temp_bytes, keys_in, keys_out, vals_in, vals_out, n, 0u,
                                             (unsigned)key_bits, st, false);
    if (e != hipSuccess) return fail(TN_ERR_HIP, std::string("rocprim::radix_sort_pairs: ") + hipGetErrorString(e));
    return TN_OK;
}

}  // namespace tn
