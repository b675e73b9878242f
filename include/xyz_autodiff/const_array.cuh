#pragma once
// ConstArray<T, N>: a plain fixed-size value array that takes no part in
// differentiation (pixel colours, constants of a graph).  Aggregate-like, any
// element type.  Element-wise + - * / and their compound forms work between two
// ConstArrays, and between a ConstArray and anything that looks like an array of
// the same length and element type (Variable, VariableRef, an operation node):
// that is how a kernel accumulates node outputs into a pixel,
// `pixel += weighted_colour`.
// Same interface as xyz-autodiff-cuda include/xyz_autodiff/const_array.cuh:7-223;
// unlike there, the mixed forms are callable from host code as well.

#include <cstddef>

#include <xyz_autodiff/concept/const_array.cuh>
#include <xyz_autodiff/detail/config.cuh>

namespace xyz_autodiff {

template <typename T, int N>
struct ConstArray {
    using value_type = T;
    static constexpr std::size_t size = N;

    T data[N];

    XAD_HD constexpr ConstArray() = default;

    XAD_HD constexpr ConstArray(const T (&init)[N]) : data{} {
        for (int i = 0; i < N; ++i) data[i] = init[i];
    }

    XAD_INLINE constexpr T& operator[](std::size_t i) noexcept { return data[i]; }
    XAD_INLINE constexpr const T& operator[](std::size_t i) const noexcept { return data[i]; }

    // compound assignment with anything array-like of the same length and element type
    // (ConstArray itself included)
#define XAD_CONST_ARRAY_COMPOUND(op)                                           \
    template <ConstArrayLike Other>                                            \
        requires ConstArrayCompatible<ConstArray, Other> && (Other::size == N) \
    XAD_INLINE constexpr ConstArray& operator op(const Other& rhs) {           \
        for (int i = 0; i < N; ++i) data[i] op rhs[i];                         \
        return *this;                                                          \
    }
    XAD_CONST_ARRAY_COMPOUND(+=)
    XAD_CONST_ARRAY_COMPOUND(-=)
    XAD_CONST_ARRAY_COMPOUND(*=)
    XAD_CONST_ARRAY_COMPOUND(/=)
#undef XAD_CONST_ARRAY_COMPOUND
};

namespace detail {
template <typename A, typename T, int N>
concept MatchesConstArray = ConstArrayLike<A> && ConstArrayCompatible<ConstArray<T, N>, A> && (A::size == N);

template <typename A>
struct is_const_array : std::false_type {};
template <typename T, int N>
struct is_const_array<ConstArray<T, N>> : std::true_type {};
}  // namespace detail

// a op b with a ConstArray on the left and any matching array on the right, or
// the other way round (the right operand then is a ConstArray and the left is not).
#define XAD_CONST_ARRAY_BINARY(op)                                                                   \
    template <typename T, int N, typename Other>                                                     \
        requires detail::MatchesConstArray<Other, T, N>                                              \
    XAD_INLINE constexpr ConstArray<T, N> operator op(const ConstArray<T, N>& lhs, const Other& rhs) { \
        ConstArray<T, N> out;                                                                        \
        for (int i = 0; i < N; ++i) out[i] = lhs[i] op rhs[i];                                       \
        return out;                                                                                  \
    }                                                                                                \
    template <typename T, int N, typename Other>                                                     \
        requires detail::MatchesConstArray<Other, T, N> && (!detail::is_const_array<Other>::value)   \
    XAD_INLINE constexpr ConstArray<T, N> operator op(const Other& lhs, const ConstArray<T, N>& rhs) { \
        ConstArray<T, N> out;                                                                        \
        for (int i = 0; i < N; ++i) out[i] = lhs[i] op rhs[i];                                       \
        return out;                                                                                  \
    }
XAD_CONST_ARRAY_BINARY(+)
XAD_CONST_ARRAY_BINARY(-)
XAD_CONST_ARRAY_BINARY(*)
XAD_CONST_ARRAY_BINARY(/)
#undef XAD_CONST_ARRAY_BINARY

}  // namespace xyz_autodiff
