#pragma once
// Contract of a fixed-size matrix or matrix view
// (xyz-autodiff-cuda: include/xyz_autodiff/concept/matrix.cuh:10-28).

#include <concepts>
#include <cstddef>
#include <utility>

namespace xyz_autodiff {

// Compile-time rows/cols, (row, col) element access on const and non-const
// objects, a pointer to the underlying storage and a transpose().
template <typename M>
concept MatrixViewConcept =
    requires { typename M::value_type; } &&
    requires(M m, std::size_t r, std::size_t c) {
        { M::rows } -> std::convertible_to<std::size_t>;
        { M::cols } -> std::convertible_to<std::size_t>;
        { m(r, c) } -> std::convertible_to<typename M::value_type>;
        { std::as_const(m)(r, c) } -> std::convertible_to<typename M::value_type>;
        { m.data() } -> std::convertible_to<const typename M::value_type*>;
        { m.transpose() };
    };

}  // namespace xyz_autodiff
