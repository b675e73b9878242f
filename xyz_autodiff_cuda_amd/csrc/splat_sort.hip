// Device-wide scan and sort for the splatting step, from rocPRIM.  Kept in a
// translation unit of its own: these templates dominate compile time.
#include <cstring>

#include <rocprim/device/device_radix_sort.hpp>
#include <rocprim/device/device_scan.hpp>

#include "common.cuh"
#include "splat_launch.cuh"

namespace xad_splat {

std::size_t scan_temp_bytes(int G) {
    std::size_t bytes = 0;
    (void)rocprim::exclusive_scan(nullptr, bytes, static_cast<const std::uint32_t*>(nullptr),
                                  static_cast<std::uint32_t*>(nullptr), std::uint32_t(0), static_cast<std::size_t>(G) + 1,
                                  rocprim::plus<std::uint32_t>(), hipStream_t(nullptr));
    return bytes;
}

int exclusive_scan_counts(hipStream_t s, void* temp, std::size_t temp_bytes, const std::uint32_t* counts,
                          std::uint32_t* offsets, int G) {
    // counts has G + 1 entries (the last one is zero), so offsets[G] is the total
    XAD_HIP_TRY(rocprim::exclusive_scan(temp, temp_bytes, counts, offsets, std::uint32_t(0),
                                        static_cast<std::size_t>(G) + 1, rocprim::plus<std::uint32_t>(), s));
    return XAD_OK;
}

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

namespace {

template <typename Key>
std::size_t pair_sort_temp_bytes(std::uint32_t capacity) {
    std::size_t bytes = 0;
    (void)rocprim::radix_sort_pairs(nullptr, bytes, static_cast<const Key*>(nullptr), static_cast<Key*>(nullptr),
                                    static_cast<const std::uint32_t*>(nullptr), static_cast<std::uint32_t*>(nullptr),
                                    static_cast<std::size_t>(capacity), 0u, static_cast<unsigned>(8 * sizeof(Key)),
                                    hipStream_t(nullptr));
    return bytes;
}

template <typename Key>
int pair_sort(hipStream_t s, void* temp, std::size_t temp_bytes, const void* keys_in, void* keys_out,
              const std::uint32_t* values_in, std::uint32_t* values_out, std::uint32_t K, int key_bits) {
    XAD_HIP_TRY(rocprim::radix_sort_pairs(temp, temp_bytes, static_cast<const Key*>(keys_in), static_cast<Key*>(keys_out),
                                          values_in, values_out, static_cast<std::size_t>(K), 0u,
                                          static_cast<unsigned>(key_bits), s));
    return XAD_OK;
}

}  // namespace

std::size_t sort_temp_bytes(std::uint32_t capacity, bool wide_keys) {
    return wide_keys ? pair_sort_temp_bytes<std::uint32_t>(capacity) : pair_sort_temp_bytes<std::uint16_t>(capacity);
}

int sort_pairs(hipStream_t s, void* temp, std::size_t temp_bytes, bool wide_keys, const void* keys_in, void* keys_out,
               const std::uint32_t* values_in, std::uint32_t* values_out, std::uint32_t K, int key_bits) {
    if (K == 0) return XAD_OK;
    return wide_keys ? pair_sort<std::uint32_t>(s, temp, temp_bytes, keys_in, keys_out, values_in, values_out, K, key_bits)
                     : pair_sort<std::uint16_t>(s, temp, temp_bytes, keys_in, keys_out, values_in, values_out, K, key_bits);
}

}  // namespace xad_splat
