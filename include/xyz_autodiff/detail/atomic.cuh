#pragma once
// One primitive: add a floating-point value to memory that other threads may
// be adding to at the same time.
//
// gfx950 pass: a relaxed, agent-scope hardware floating-point add.  The
// address space is resolved by the compiler where it is known (ds_add_f32 /
// ds_add_f64 for LDS, global_atomic_add_f32 / _f64 for HBM) and by the flat
// instruction otherwise; no compare-and-swap loop is involved, the returned
// value is never requested, so the instruction is issued without a return path.
//
// Host pass: std::atomic_ref, so that the host-core build of the same
// templates may be threaded.

#include <xyz_autodiff/detail/config.cuh>

#if !XAD_DEVICE_PASS
#include <atomic>
#endif

namespace xyz_autodiff {
namespace detail {

template <typename T>
XAD_INLINE void atomic_add(T* address, T value) noexcept {
#if XAD_DEVICE_PASS
    unsafeAtomicAdd(address, value);
#else
    std::atomic_ref<T>(*address).fetch_add(value, std::memory_order_relaxed);
#endif
}

}  // namespace detail
}  // namespace xyz_autodiff
