#pragma once
// y_i = a_i - b_i; the gradient reaches b negated.
// Counterpart of xyz-autodiff-cuda include/xyz_autodiff/operations/binary/sub_logic.cuh (SubLogic :13-42, factory :45-52; unlike there, operands must have equal size).

#include <cstddef>

#include <xyz_autodiff/concept/core_logic.cuh>
#include <xyz_autodiff/operations/operation.cuh>

namespace xyz_autodiff {
namespace op {

template <typename Input1, typename Input2>
    requires BinaryLogicParameterConcept<Input1, Input2> && (Input1::size == Input2::size)
struct SubLogic {
    using T = typename Input1::value_type;
    static constexpr std::size_t Dim = Input1::size;
    using Output = Variable<Dim, T>;
    static constexpr std::size_t outputDim = Dim;

    XAD_INLINE void forward(Output& out, const Input1& lhs, const Input2& rhs) const {
        XAD_UNROLL
        for (std::size_t i = 0; i < Dim; ++i) out[i] = lhs[i] - rhs[i];
    }

    // Both operands may be one and the same object (x op x): each slot is
    // credited separately and the two contributions add up.
    XAD_INLINE void backward(const Output& out, Input1& lhs, Input2& rhs) const {
        XAD_UNROLL
        for (std::size_t i = 0; i < Dim; ++i) {
            const T g = out.grad(i);
            lhs.add_grad(i, g);
            rhs.add_grad(i, -g);
        }
    }
};

template <typename Input1, typename Input2>
    requires BinaryLogicParameterConcept<Input1, Input2>
XAD_INLINE auto sub(Input1& lhs, Input2& rhs) {
    using Logic = SubLogic<Input1, Input2>;
    return BinaryOperation<Logic::outputDim, Logic, Input1, Input2>(Logic{}, lhs, rhs);
}

}  // namespace op
}  // namespace xyz_autodiff
