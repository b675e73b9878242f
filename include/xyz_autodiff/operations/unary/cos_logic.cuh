#pragma once
// y = cos(x), element-wise; dy/dx = -sin(x).
// Counterpart of xyz-autodiff-cuda include/xyz_autodiff/operations/unary/cos_logic.cuh (CosLogic :14-35, factories :38-52).

#include <cstddef>

#include <xyz_autodiff/concept/variable.cuh>
#include <xyz_autodiff/detail/elementwise.cuh>
#include <xyz_autodiff/operations/math.cuh>
#include <xyz_autodiff/operations/operation.cuh>

namespace xyz_autodiff {
namespace op {

namespace rule {
struct Cos {
    template <typename T>
    XAD_INLINE static T value(const T& x) { return math::cos(x); }
    template <typename T>
    XAD_INLINE static T slope(const T& x, const T& y) { (void)x; (void)y; return -math::sin(x); }
};
}  // namespace rule

template <std::size_t Dim>
struct CosLogic : detail::MapLogic<Dim, rule::Cos> {};

// Node over the first Dim elements of `input`.
template <std::size_t Dim, DifferentiableVariableConcept Input>
XAD_INLINE auto cos(Input& input) {
    return UnaryOperation<Dim, CosLogic<Dim>, Input>(CosLogic<Dim>{}, input);
}

// Node over every element of `input`.
template <DifferentiableVariableConcept Input>
XAD_INLINE auto cos(Input& input) {
    return cos<Input::size>(input);
}

}  // namespace op
}  // namespace xyz_autodiff
