// Stable sort of (key, value) pairs of 32-bit unsigned integers by key, on a given stream.
// The index lists of indexAdd are sorted with it so that every target row finds the source
// rows that add into it as one run, in their original order. rocPRIM's least-significant-digit
// radix sort is stable, which is the property the order of the floating-point adds rests on.
// This file exists on its own so that only it pays for compiling the sort's templates.
#include <cstring>

#include <rocprim/device/device_radix_sort.hpp>

#include "kth_internal.h"

namespace kth {

hipError_t sort_pairs_u32(void* temp, size_t* temp_bytes, const uint32_t* keys_in, uint32_t* keys_out,
                          const uint32_t* vals_in, uint32_t* vals_out, uint32_t n, int end_bit, hipStream_t stream) {
    return rocprim::radix_sort_pairs(temp, *temp_bytes, keys_in, keys_out, vals_in, vals_out, static_cast<size_t>(n), 0u,
                                     static_cast<unsigned int>(end_bit), stream);
}

}  // namespace kth
