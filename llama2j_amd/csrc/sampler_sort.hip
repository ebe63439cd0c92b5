// The sort of J/Sampler.java:97 on the device: Arrays.sort on the ProbIndex objects is a stable sort by
// descending probability (compareTo, J/Sampler.java:64-73); rocPRIM's radix sort of (key, value) pairs is stable
// too, and for the non-negative, NaN-free probabilities that reach it the bit order of float keys is their
// numeric order.  A translation unit of its own keeps the rocPRIM headers out of the kernel sources.
#include <hip/hip_runtime.h>
#include <cstring>
#include <rocprim/device/device_radix_sort.hpp>

namespace l2j {

hipError_t sort_prob_index_desc(void *temp, size_t *temp_bytes, const float *kin, float *kout, const int *vin, int *vout, unsigned n,
                                hipStream_t s)
{
    return rocprim::radix_sort_pairs_desc(temp, *temp_bytes, kin, kout, vin, vout, n, 0u, 32u, s, false);
}

}  // namespace l2j
