#pragma once
// Contracts of the value types a graph is made of.
// Mirrors the public concept names of xyz-autodiff-cuda
// (include/xyz_autodiff/concept/variable.cuh:9-36).

#include <concepts>
#include <cstddef>
#include <type_traits>

namespace xyz_autodiff {

// Scalar types the library differentiates: fp32 (timed paths) and fp64 (checks).
template <typename T>
concept FloatingPointConcept = std::is_same_v<T, float> || std::is_same_v<T, double>;

// A fixed-size vector of values: value_type, a compile-time `size`,
// element access through operator[] and a zero_grad() member.
template <typename V>
concept VariableConcept =
    requires { typename V::value_type; } &&
    FloatingPointConcept<typename V::value_type> &&
    requires(V v, std::size_t i) {
        { V::size } -> std::convertible_to<std::size_t>;
        { v[i] } -> std::convertible_to<typename V::value_type&>;
        { v[i] } -> std::convertible_to<const typename V::value_type&>;
        { v.zero_grad() } -> std::same_as<void>;
    };

// A VariableConcept type that also carries a gradient per element:
// grad(i) reads it, add_grad(i, g) accumulates into it.
template <typename V>
concept DifferentiableVariableConcept =
    VariableConcept<V> &&
    requires(V v, std::size_t i, typename V::value_type g) {
        { v.grad(i) } -> std::convertible_to<const typename V::value_type&>;
        { v.add_grad(i, g) } -> std::same_as<void>;
    };

}  // namespace xyz_autodiff
