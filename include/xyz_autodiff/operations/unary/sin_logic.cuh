#pragma once
// y = sin(x), element-wise; dy/dx = cos(x).
// Counterpart of xyz-autodiff-cuda include/xyz_autodiff/operations/unary/sin_logic.cuh (SinLogic :14-35, factories :38-52).

#include <cstddef>

#include <xyz_autodiff/concept/variable.cuh>
#include <xyz_autodiff/detail/elementwise.cuh>
#include <xyz_autodiff/operations/math.cuh>
#include <xyz_autodiff/operations/operation.cuh>

namespace xyz_autodiff {
namespace op {

namespace rule {
struct Sin {
    template <typename T>
    XAD_INLINE static T value(const T& x) { return math::sin(x); }
    template <typename T>
    XAD_INLINE static T slope(const T& x, const T& y) { (void)x; (void)y; return math::cos(x); }
};
}  // namespace rule

template <std::size_t Dim>
struct SinLogic : detail::MapLogic<Dim, rule::Sin> {};

// Node over the first Dim elements of `input`.
template <std::size_t Dim, DifferentiableVariableConcept Input>
XAD_INLINE auto sin(Input& input) {
    return UnaryOperation<Dim, SinLogic<Dim>, Input>(SinLogic<Dim>{}, input);
}

// Node over every element of `input`.
template <DifferentiableVariableConcept Input>
XAD_INLINE auto sin(Input& input) {
    return sin<Input::size>(input);
}

}  // namespace op
}  // namespace xyz_autodiff
