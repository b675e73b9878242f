// The depth order of the Gaussians: a stable radix sort of (depth bits, index) from rocPRIM.  It runs
// when a depth has changed, not per step.  Kept in a translation unit of its own: these templates
// dominate compile time.
#include <rocprim/device/device_radix_sort.hpp>

#include "common.cuh"
#include "splat_launch.cuh"

namespace xad_splat {

std::size_t depth_sort_temp_bytes(int G) {
    std::size_t bytes = 0;
    (void)rocprim::radix_sort_pairs(nullptr, bytes, static_cast<const std::uint32_t*>(nullptr),
                                    static_cast<std::uint32_t*>(nullptr), static_cast<const std::uint32_t*>(nullptr),
                                    static_cast<std::uint32_t*>(nullptr), static_cast<std::size_t>(G), 0u, 32u,
                                    hipStream_t(nullptr));
    return bytes;
}

int sort_by_depth(hipStream_t s, void* temp, std::size_t temp_bytes, const std::uint32_t* keys_in,
                  std::uint32_t* keys_out, const std::uint32_t* values_in, std::uint32_t* values_out, int G) {
    XAD_HIP_TRY(rocprim::radix_sort_pairs(temp, temp_bytes, keys_in, keys_out, values_in, values_out,
                                          static_cast<std::size_t>(G), 0u, 32u, s));
    return XAD_OK;
}

}  // namespace xad_splat
