// The sort of J/Sampler.java:97 on the device: Arrays.sort on the ProbIndex objects is a stable sort by
// descending probability (compareTo, J/Sampler.java:64-73); rocPRIM's radix sort of (key, value) pairs is stable
// too, and for the non-negative, NaN-free probabilities that reach it the bit order of float keys is their
// numeric order.  A translation unit of its own keeps the rocPRIM headers out of the kernel sources.
#include <hip/hip_runtime.h>
#include <cstring>
#include <rocprim/device/device_radix_sort.hpp>

namespace l2j {

// The pairs are in (k0, v0) on entry; either pair of arrays may be overwritten, and *in_second says where the sorted
// pairs are (with the two buffers handed over as such, rocPRIM need not copy the result into place).
hipError_t sort_prob_index_desc(void *temp, size_t *temp_bytes, float *k0, float *k1, int *v0, int *v1, unsigned n, hipStream_t s,
                                int *in_second)
{
    rocprim::double_buffer<float> keys(k0, k1);
    rocprim::double_buffer<int> values(v0, v1);
    const hipError_t e = rocprim::radix_sort_pairs_desc(temp, *temp_bytes, keys, values, n, 0u, 32u, s, false);
    if (in_second) *in_second = keys.current() == k1 ? 1 : 0;
    return e;
}

}  // namespace l2j
