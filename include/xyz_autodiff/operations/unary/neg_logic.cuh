#pragma once
// y = -x, element-wise; dy/dx = -1.
// Counterpart of xyz-autodiff-cuda include/xyz_autodiff/operations/unary/neg_logic.cuh (NegLogic :14-33, factories :36-50).

#include <cstddef>

#include <xyz_autodiff/concept/variable.cuh>
#include <xyz_autodiff/detail/elementwise.cuh>
#include <xyz_autodiff/operations/math.cuh>
#include <xyz_autodiff/operations/operation.cuh>

namespace xyz_autodiff {
namespace op {

namespace rule {
struct Neg {
    template <typename T>
    XAD_INLINE static T value(const T& x) { return -x; }
    template <typename T>
    XAD_INLINE static T slope(const T& x, const T& y) { (void)x; (void)y; return T(-1); }
};
}  // namespace rule

template <std::size_t Dim>
struct NegLogic : detail::MapLogic<Dim, rule::Neg> {};

// Node over the first Dim elements of `input`.
template <std::size_t Dim, DifferentiableVariableConcept Input>
XAD_INLINE auto neg(Input& input) {
    return UnaryOperation<Dim, NegLogic<Dim>, Input>(NegLogic<Dim>{}, input);
}

// Node over every element of `input`.
template <DifferentiableVariableConcept Input>
XAD_INLINE auto neg(Input& input) {
    return neg<Input::size>(input);
}

}  // namespace op
}  // namespace xyz_autodiff
