#pragma once
// y = 1 / (1 + exp(-x)), element-wise; dy/dx = y (1 - y).
// Counterpart of xyz-autodiff-cuda include/xyz_autodiff/operations/unary/sigmoid_logic.cuh (SigmoidLogic :14-36, factories :39-53).

#include <cstddef>

#include <xyz_autodiff/concept/variable.cuh>
#include <xyz_autodiff/detail/elementwise.cuh>
#include <xyz_autodiff/operations/math.cuh>
#include <xyz_autodiff/operations/operation.cuh>

namespace xyz_autodiff {
namespace op {

namespace rule {
struct Sigmoid {
    template <typename T>
    XAD_INLINE static T value(const T& x) { return math::sigmoid(x); }
    template <typename T>
    XAD_INLINE static T slope(const T& x, const T& y) { (void)x; (void)y; return y * (T(1) - y); }
};
}  // namespace rule

template <std::size_t Dim>
struct SigmoidLogic : detail::MapLogic<Dim, rule::Sigmoid> {};

// Node over the first Dim elements of `input`.
template <std::size_t Dim, DifferentiableVariableConcept Input>
XAD_INLINE auto sigmoid(Input& input) {
    return UnaryOperation<Dim, SigmoidLogic<Dim>, Input>(SigmoidLogic<Dim>{}, input);
}

// Node over every element of `input`.
template <DifferentiableVariableConcept Input>
XAD_INLINE auto sigmoid(Input& input) {
    return sigmoid<Input::size>(input);
}

}  // namespace op
}  // namespace xyz_autodiff
