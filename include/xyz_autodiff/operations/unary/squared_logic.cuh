#pragma once
// y = x^2, element-wise; dy/dx = 2x.
// Counterpart of xyz-autodiff-cuda include/xyz_autodiff/operations/unary/squared_logic.cuh
// (SquaredLogic :11-34, factory :37-45).  The original multiplies by a double
// literal 2.0; doubling is exact in either precision, so results agree.

#include <cstddef>

#include <xyz_autodiff/concept/core_logic.cuh>
#include <xyz_autodiff/detail/elementwise.cuh>
#include <xyz_autodiff/operations/operation.cuh>

namespace xyz_autodiff {
namespace op {

namespace rule {
struct Squared {
    template <typename T>
    XAD_INLINE static T value(const T& x) { return x * x; }
    template <typename T>
    XAD_INLINE static T slope(const T& x, const T&) { return T(2) * x; }
};
}  // namespace rule

template <std::size_t Dim>
struct SquaredLogic : detail::MapLogic<Dim, rule::Squared> {};

template <typename Input>
    requires UnaryLogicParameterConcept<Input>
XAD_INLINE auto squared(Input& input) {
    constexpr std::size_t Dim = Input::size;
    return UnaryOperation<Dim, SquaredLogic<Dim>, Input>(SquaredLogic<Dim>{}, input);
}

}  // namespace op
}  // namespace xyz_autodiff
