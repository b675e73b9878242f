#pragma once
// Host-side check of HIP runtime results: a failed call throws
// std::runtime_error carrying the error name, code, file, line and message.
// HIP counterpart of xyz-autodiff-cuda include/xyz_autodiff/util/error_checker.cuh:7-20
// (same behaviour, HIP-native names; lives in the global namespace like there).

#include <hip/hip_runtime_api.h>

#include <sstream>
#include <stdexcept>

namespace hip {

template <typename File, typename Line>
void check_error(const ::hipError_t status, File&& file, Line&& line) {
    if (status != ::hipSuccess) {
        std::stringstream text;
        text << ::hipGetErrorName(status) << " (" << static_cast<int>(status) << ")@" << file << "#L" << line << ": "
             << ::hipGetErrorString(status);
        throw std::runtime_error{text.str()};
    }
}

}  // namespace hip

#define CHECK_HIP_ERROR(expr) (::hip::check_error((expr), __FILE__, __LINE__))
