#pragma once
// Contracts of plain value arrays that take no part in differentiation
// (xyz-autodiff-cuda: include/xyz_autodiff/concept/const_array.cuh:9-27).

#include <concepts>
#include <cstddef>
#include <type_traits>

namespace xyz_autodiff {

// value_type, a static `size` and operator[]: ConstArray, Variable,
// VariableRef and operation nodes all qualify.
template <typename A>
concept ConstArrayLike =
    requires { typename A::value_type; } &&
    requires(A a, std::size_t i) {
        { a[i] } -> std::convertible_to<typename A::value_type>;
        { A::size } -> std::convertible_to<std::size_t>;
    };

template <typename A, typename B>
concept ConstArrayCompatible =
    ConstArrayLike<A> && ConstArrayLike<B> &&
    std::same_as<typename A::value_type, typename B::value_type>;

template <typename A, typename B>
concept ConstArraySameSize = ConstArrayLike<A> && ConstArrayLike<B> && (A::size == B::size);

}  // namespace xyz_autodiff
