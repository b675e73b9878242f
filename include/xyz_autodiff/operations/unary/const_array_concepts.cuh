#pragma once
// What the constant-array operations accept as the constant operand
// (xyz-autodiff-cuda: include/xyz_autodiff/operations/unary/const_array_concepts.cuh:9-12).

#include <concepts>
#include <cstddef>
#include <type_traits>

namespace xyz_autodiff {
namespace op {

// Anything with a value_type whose operator[] yields that type.
template <typename A>
concept ArrayLikeConcept = requires(A a, std::size_t i) {
    { a[i] } -> std::convertible_to<typename std::remove_reference_t<A>::value_type>;
};

}  // namespace op
}  // namespace xyz_autodiff
