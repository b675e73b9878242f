#pragma once
// y_i = x_i + k_i for a non-differentiated array k; dy/dx = 1.
// Counterpart of xyz-autodiff-cuda include/xyz_autodiff/operations/unary/const_array_add_logic.cuh (ConstArrayAddLogic :16-38, factory :41-48).
// The logic keeps a reference to the array, which must outlive the node.

#include <cstddef>

#include <xyz_autodiff/concept/variable.cuh>
#include <xyz_autodiff/operations/operation.cuh>
#include <xyz_autodiff/operations/unary/const_array_concepts.cuh>

namespace xyz_autodiff {
namespace op {

template <std::size_t Dim, typename ConstantArray>
    requires ArrayLikeConcept<ConstantArray>
struct ConstArrayAddLogic {
    static constexpr std::size_t outputDim = Dim;

    const ConstantArray& constant_array;

    XAD_HD explicit ConstArrayAddLogic(const ConstantArray& array) : constant_array(array) {}

    template <typename Output, typename Input>
    XAD_INLINE void forward(Output& out, const Input& in) const {
        XAD_UNROLL
        for (std::size_t i = 0; i < Dim; ++i) out[i] = in[i] + constant_array[i];
    }

    template <typename Output, typename Input>
    XAD_INLINE void backward(const Output& out, Input& in) const {
        XAD_UNROLL
        for (std::size_t i = 0; i < Dim; ++i) in.add_grad(i, out.grad(i));
    }
};

template <DifferentiableVariableConcept Input, typename ConstantArray>
    requires ArrayLikeConcept<ConstantArray>
XAD_INLINE auto const_add(Input& input, const ConstantArray& constant_array) {
    constexpr std::size_t Dim = Input::size;
    using Logic = ConstArrayAddLogic<Dim, ConstantArray>;
    return UnaryOperation<Dim, Logic, Input>(Logic(constant_array), input);
}

}  // namespace op
}  // namespace xyz_autodiff
