// Stable sort of (key, value) pairs of 32-bit unsigned integers by key, on a given stream.
// (and the compaction of flagged positions). The index lists of indexAdd are sorted with it so that every target row finds the source
// rows that add into it as one run, in their original order. rocPRIM's least-significant-digit
// radix sort is stable, which is the property the order of the floating-point adds rests on.
// This file exists on its own so that only it pays for compiling the sort's templates.
#include <cstring>

#include <rocprim/device/device_radix_sort.hpp>
#include <rocprim/device/device_select.hpp>
#include <rocprim/iterator/counting_iterator.hpp>

#include "kth_internal.h"

namespace kth {

hipError_t sort_pairs_u32(void* temp, size_t* temp_bytes, const uint32_t* keys_in, uint32_t* keys_out,
                          const uint32_t* vals_in, uint32_t* vals_out, uint32_t n, int end_bit, hipStream_t stream) {
    return rocprim::radix_sort_pairs(temp, *temp_bytes, keys_in, keys_out, vals_in, vals_out, static_cast<size_t>(n), 0u,
                                     static_cast<unsigned int>(end_bit), stream);
}

// The positions i in [0, n) with flags[i] != 0, in ascending order, and how many there are
// (rocPRIM's select over a counting iterator). With temp == nullptr only *temp_bytes is set.
hipError_t select_flagged_positions(void* temp, size_t* temp_bytes, const uint8_t* flags, uint32_t* positions, uint32_t* count,
                                    uint32_t n, hipStream_t stream) {
    return rocprim::select(temp, *temp_bytes, rocprim::counting_iterator<uint32_t>(0u), flags, positions, count,
                           static_cast<size_t>(n), stream);
}

}  // namespace kth
