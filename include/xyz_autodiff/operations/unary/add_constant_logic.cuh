#pragma once
// y_i = x_i + c for a scalar constant c held by the logic; dy/dx = 1.
// Counterpart of xyz-autodiff-cuda include/xyz_autodiff/operations/unary/add_constant_logic.cuh (AddConstantLogic :13-38, factory :41-48).

#include <cstddef>

#include <xyz_autodiff/concept/core_logic.cuh>
#include <xyz_autodiff/operations/operation.cuh>

namespace xyz_autodiff {
namespace op {

template <typename Input>
    requires UnaryLogicParameterConcept<Input>
struct AddConstantLogic {
    using T = typename Input::value_type;
    static constexpr std::size_t Dim = Input::size;
    using Output = Variable<Dim, T>;
    static constexpr std::size_t outputDim = Dim;

    T constant_c;

    XAD_HD explicit AddConstantLogic(T c) : constant_c(c) {}

    XAD_INLINE void forward(Output& out, const Input& in) const {
        XAD_UNROLL
        for (std::size_t i = 0; i < Dim; ++i) out[i] = in[i] + constant_c;
    }

    XAD_INLINE void backward(const Output& out, Input& in) const {
        XAD_UNROLL
        for (std::size_t i = 0; i < Dim; ++i) in.add_grad(i, out.grad(i));
    }
};

template <typename Input>
    requires UnaryLogicParameterConcept<Input>
XAD_INLINE auto add_constant(Input& input, typename Input::value_type constant) {
    using Logic = AddConstantLogic<Input>;
    return UnaryOperation<Logic::outputDim, Logic, Input>(Logic(constant), input);
}

}  // namespace op
}  // namespace xyz_autodiff
