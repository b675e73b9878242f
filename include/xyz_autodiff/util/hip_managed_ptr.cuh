#pragma once
// std::unique_ptr over hipMallocManaged memory (reachable from host and device).
//   hip_managed_ptr<T>, makeHipManagedUnique<T>(count = 1), makeHipManagedArray<T>(count)
// On failure the makers print a diagnostic and return nullptr.
// HIP counterpart of xyz-autodiff-cuda include/xyz_autodiff/util/cuda_managed_ptr.cuh:8-62.

#include <hip/hip_runtime_api.h>

#include <cstddef>
#include <iostream>
#include <memory>

template <typename T>
struct HipManagedDeleter {
    void operator()(T* p) const noexcept {
        if (p) (void)hipFree(p);
    }
};

template <typename T>
struct HipManagedDeleter<T[]> {
    void operator()(T* p) const noexcept {
        if (p) (void)hipFree(p);
    }
};

template <typename T>
using hip_managed_ptr = std::unique_ptr<T, HipManagedDeleter<T>>;

namespace xyz_autodiff_util_detail {
template <typename T>
T* managed_allocate(std::size_t count, const char* who) {
    T* p = nullptr;
    const std::size_t bytes = sizeof(T) * count;
    const hipError_t status = hipMallocManaged(reinterpret_cast<void**>(&p), bytes);
    if (status != hipSuccess) {
        std::cerr << "[HIP ERROR] " << who << " failed to allocate " << bytes << " bytes: " << hipGetErrorString(status) << "\n";
        return nullptr;
    }
    return p;
}
}  // namespace xyz_autodiff_util_detail

template <typename T>
hip_managed_ptr<T> makeHipManagedUnique(std::size_t count = 1) {
    return hip_managed_ptr<T>(xyz_autodiff_util_detail::managed_allocate<T>(count, "makeHipManagedUnique"));
}

template <typename T>
hip_managed_ptr<T[]> makeHipManagedArray(std::size_t count) {
    return hip_managed_ptr<T[]>(xyz_autodiff_util_detail::managed_allocate<T>(count, "makeHipManagedArray"));
}
