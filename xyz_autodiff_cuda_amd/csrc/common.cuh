#pragma once
// Host-side plumbing shared by the C-ABI translation units: error recording,
// HIP call checking, launch geometry.

#include <hip/hip_runtime.h>

#include <cstdarg>
#include <cstddef>
#include <cstdint>
#include <cstdio>

#include "../../include/xad_capi.h"

namespace xad {

// Thread-local text behind xad_last_error().
char* last_error_buffer();
constexpr std::size_t kLastErrorCapacity = 512;

inline int fail(int code, const char* fmt, ...) {
    va_list args;
    va_start(args, fmt);
    std::vsnprintf(last_error_buffer(), kLastErrorCapacity, fmt, args);
    va_end(args);
    return code;
}

inline hipStream_t as_stream(void* s) { return static_cast<hipStream_t>(s); }

inline bool aligned16(const void* p) { return (reinterpret_cast<std::uintptr_t>(p) & 15u) == 0; }

inline unsigned blocks_for(std::size_t items, unsigned block) {
    return static_cast<unsigned>((items + block - 1) / block);
}

}  // namespace xad

// Evaluates a HIP runtime call; on failure records "<call>: <hip message>" with
// file and line and returns XAD_ERR_HIP from the enclosing function.
#define XAD_HIP_TRY(call)                                                                  \
    do {                                                                                   \
        hipError_t xad_status_ = (call);                                                   \
        if (xad_status_ != hipSuccess)                                                     \
            return ::xad::fail(XAD_ERR_HIP, "%s:%d: %s: %s", __FILE__, __LINE__, #call,    \
                               hipGetErrorString(xad_status_));                            \
    } while (0)

#define XAD_REQUIRE(cond, ...)                                                  \
    do {                                                                        \
        if (!(cond)) return ::xad::fail(XAD_ERR_INVALID_ARGUMENT, __VA_ARGS__); \
    } while (0)
