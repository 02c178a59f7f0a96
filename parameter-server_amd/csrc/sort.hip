// Sort of (slot, batch index) pairs by slot: the grouping step of duplicate-key aggregation.
// The passes are rocPRIM's LSD radix sort restricted to the bits a slot index can have.
#include "table.h"

#include <cstring>

#include <rocprim/device/device_radix_sort.hpp>

namespace pshbm {

// rocPRIM's default switches to a merge sort (about twenty launches) below 2^20 items; batches
// here are that size, and the Onesweep radix path is several times faster for them.
using SortConfig = rocprim::radix_sort_config<rocprim::default_config, rocprim::default_config,
                                              rocprim::default_config, 8192>;

size_t sort_pairs_temp_bytes(size_t n) {
    size_t bytes = 0;
    uint32_t* k = nullptr;
    (void)rocprim::radix_sort_pairs<SortConfig>(nullptr, bytes, k, k, k, k, n, 0, 32, hipStreamDefault);
    return bytes;
}

hipError_t sort_pairs(void* temp, size_t temp_bytes, const uint32_t* keys_in, uint32_t* keys_out,
                      const uint32_t* vals_in, uint32_t* vals_out, size_t n, unsigned end_bit,
                      hipStream_t s) {
    if (n == 0) return hipSuccess;
    return rocprim::radix_sort_pairs<SortConfig>(temp, temp_bytes, keys_in, keys_out, vals_in, vals_out, n, 0,
                                     end_bit, s);
}

}  // namespace pshbm
