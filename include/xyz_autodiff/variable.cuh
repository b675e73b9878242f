#pragma once
// Leaves of a per-thread graph.
//
//   Variable<N, T>     owns N values and N gradients.  In a kernel the object is
//                      a local of one lane; after inlining and scalar
//                      replacement each element is one VGPR, and add_grad is a
//                      plain v_add.
//   VariableRef<N, T>  views N values and N gradients that live elsewhere (HBM
//                      or LDS) and may be shared by many lanes; add_grad is a
//                      hardware floating-point atomic.
//
// Same names, template parameter order <N, T> and members as xyz-autodiff-cuda
// (include/xyz_autodiff/variable.cuh:12-59 VariableRef, :62-190 Variable).
// Every member here is callable from host code as well, which the original's
// accessors were not.

#include <cstddef>

#include <xyz_autodiff/concept/variable.cuh>
#include <xyz_autodiff/detail/atomic.cuh>
#include <xyz_autodiff/detail/config.cuh>

namespace xyz_autodiff {

template <std::size_t N, typename T>
    requires FloatingPointConcept<T>
class VariableRef {
public:
    using value_type = T;
    static constexpr std::size_t size = N;

    // `data` and `grad` point at N consecutive elements each.  Neither is
    // owned.  `grad` may be null for a leaf that is only ever read.
    XAD_HD constexpr VariableRef(T* data, T* grad) noexcept : values_(data), grads_(grad) {}

    XAD_INLINE T* data() const noexcept { return values_; }
    XAD_INLINE T* grad() const noexcept { return grads_; }

    // Element access is mutable through a const view: the view is const, the
    // memory it looks at is not.
    XAD_INLINE constexpr T& operator[](std::size_t i) const noexcept { return values_[i]; }
    XAD_INLINE const T& grad(std::size_t i) const noexcept { return grads_[i]; }

    // The one cross-thread operation of the library: any number of lanes, in
    // any block, may add into the same element concurrently.
    XAD_INLINE void add_grad(std::size_t i, T g) const noexcept { detail::atomic_add(grads_ + i, g); }

    // Plain stores: only for memory no other thread is adding to right now.
    XAD_INLINE void zero_grad() const noexcept {
        XAD_UNROLL
        for (std::size_t i = 0; i < N; ++i) grads_[i] = T(0);
    }

private:
    T* const values_;
    T* const grads_;
};

template <std::size_t N, typename T>
    requires FloatingPointConcept<T>
class Variable {
public:
    using value_type = T;
    static constexpr std::size_t size = N;

    XAD_HD constexpr Variable() noexcept : data_{}, grad_{} {}

    // Every element set to `fill`, gradients zero.
    XAD_HD constexpr Variable(const T& fill) noexcept : data_{}, grad_{} {
        XAD_UNROLL
        for (std::size_t i = 0; i < N; ++i) data_[i] = fill;
    }

    // Copy of N elements starting at `src`, gradients zero.
    XAD_HD constexpr Variable(const T* src) noexcept : data_{}, grad_{} {
        XAD_UNROLL
        for (std::size_t i = 0; i < N; ++i) data_[i] = src[i];
    }

    // Values and gradients are both copied; the type stays trivially copyable
    // so the optimiser is free to keep it in registers.
    constexpr Variable(const Variable&) noexcept = default;
    constexpr Variable(Variable&&) noexcept = default;
    constexpr Variable& operator=(const Variable&) noexcept = default;
    constexpr Variable& operator=(Variable&&) noexcept = default;

    XAD_INLINE T* data() noexcept { return data_; }
    XAD_INLINE const T* data() const noexcept { return data_; }
    XAD_INLINE T* grad() noexcept { return grad_; }
    XAD_INLINE const T* grad() const noexcept { return grad_; }

    XAD_INLINE constexpr T& operator[](std::size_t i) noexcept { return data_[i]; }
    XAD_INLINE constexpr const T& operator[](std::size_t i) const noexcept { return data_[i]; }
    XAD_INLINE constexpr const T& grad(std::size_t i) const noexcept { return grad_[i]; }

    XAD_INLINE constexpr void add_grad(std::size_t i, T g) noexcept { grad_[i] += g; }

    XAD_INLINE constexpr void zero_grad() noexcept {
        XAD_UNROLL
        for (std::size_t i = 0; i < N; ++i) grad_[i] = T(0);
    }

    // A view of this object's own storage.  add_grad through the view is
    // atomic, through the object it is not: do not mix them on one element
    // from different threads.
    XAD_INLINE VariableRef<N, T> ref() noexcept { return VariableRef<N, T>(data_, grad_); }
    XAD_INLINE VariableRef<N, T> ref() const noexcept {
        return VariableRef<N, T>(const_cast<T*>(data_), const_cast<T*>(grad_));
    }

private:
    T data_[N];
    T grad_[N];
};

}  // namespace xyz_autodiff
