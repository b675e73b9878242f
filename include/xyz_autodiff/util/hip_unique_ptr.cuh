#pragma once
// std::unique_ptr over hipMalloc'ed device memory.
//   hip_unique_ptr<T>, makeHipUnique<T>(count = 1), makeHipUniqueArray<T>(count)
// Allocation failures throw (see error_checker.cuh); a failing hipFree in the
// deleter is ignored rather than thrown from a destructor.
// HIP counterpart of xyz-autodiff-cuda include/xyz_autodiff/util/cuda_unique_ptr.cuh:10-53.

#include <hip/hip_runtime_api.h>

#include <cstddef>
#include <memory>

#include <xyz_autodiff/util/error_checker.cuh>

template <typename T>
struct HipDeleter {
    void operator()(T* p) const noexcept {
        if (p) (void)hipFree(p);
    }
};

template <typename T>
struct HipDeleter<T[]> {
    void operator()(T* p) const noexcept {
        if (p) (void)hipFree(p);
    }
};

template <typename T>
using hip_unique_ptr = std::unique_ptr<T, HipDeleter<T>>;

template <typename T>
hip_unique_ptr<T> makeHipUnique(std::size_t count = 1) {
    T* p = nullptr;
    CHECK_HIP_ERROR(hipMalloc(reinterpret_cast<void**>(&p), sizeof(T) * count));
    return hip_unique_ptr<T>(p);
}

template <typename T>
hip_unique_ptr<T[]> makeHipUniqueArray(std::size_t count) {
    T* p = nullptr;
    CHECK_HIP_ERROR(hipMalloc(reinterpret_cast<void**>(&p), sizeof(T) * count));
    return hip_unique_ptr<T[]>(p);
}
