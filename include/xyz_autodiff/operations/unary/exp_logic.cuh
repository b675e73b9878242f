#pragma once
// y = exp(x), element-wise; dy/dx = y.
// Counterpart of xyz-autodiff-cuda include/xyz_autodiff/operations/unary/exp_logic.cuh (ExpLogic :13-35, factories :38-51).

#include <cstddef>

#include <xyz_autodiff/concept/variable.cuh>
#include <xyz_autodiff/detail/elementwise.cuh>
#include <xyz_autodiff/operations/math.cuh>
#include <xyz_autodiff/operations/operation.cuh>

namespace xyz_autodiff {
namespace op {

namespace rule {
struct Exp {
    template <typename T>
    XAD_INLINE static T value(const T& x) { return math::exp(x); }
    template <typename T>
    XAD_INLINE static T slope(const T& x, const T& y) { (void)x; (void)y; return y; }
};
}  // namespace rule

template <std::size_t Dim>
struct ExpLogic : detail::MapLogic<Dim, rule::Exp> {};

// Node over the first Dim elements of `input`.
template <std::size_t Dim, DifferentiableVariableConcept Input>
XAD_INLINE auto exp(Input& input) {
    return UnaryOperation<Dim, ExpLogic<Dim>, Input>(ExpLogic<Dim>{}, input);
}

// Node over every element of `input`.
template <DifferentiableVariableConcept Input>
XAD_INLINE auto exp(Input& input) {
    return exp<Input::size>(input);
}

}  // namespace op
}  // namespace xyz_autodiff
