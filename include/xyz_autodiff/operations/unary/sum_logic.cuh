#pragma once
// y = x_0 + ... + x_{n-1}; every input element receives the output gradient.
// Counterpart of xyz-autodiff-cuda include/xyz_autodiff/operations/unary/sum_logic.cuh (SumLogic :14-36, factories :39-55).

#include <cstddef>

#include <xyz_autodiff/concept/variable.cuh>
#include <xyz_autodiff/operations/math.cuh>
#include <xyz_autodiff/operations/operation.cuh>

namespace xyz_autodiff {
namespace op {

template <std::size_t InputDim>
struct SumLogic {
    static constexpr std::size_t outputDim = 1;

    template <typename Output, typename Input>
    XAD_INLINE void forward(Output& out, const Input& in) const {
        using T = typename Input::value_type;
        T acc = T(0);
        XAD_UNROLL
        for (std::size_t i = 0; i < InputDim; ++i) acc += in[i];
        out[0] = acc;
    }

    template <typename Output, typename Input>
    XAD_INLINE void backward(const Output& out, Input& in) const {
        using T = typename Input::value_type;
        const T g = out.grad(0);
        XAD_UNROLL
        for (std::size_t i = 0; i < InputDim; ++i) in.add_grad(i, g);
    }
};

template <std::size_t Dim, DifferentiableVariableConcept Input>
    requires(Input::size == Dim)
XAD_INLINE auto sum(Input& input) {
    return UnaryOperation<1, SumLogic<Dim>, Input>(SumLogic<Dim>{}, input);
}

template <DifferentiableVariableConcept Input>
XAD_INLINE auto sum(Input& input) {
    return sum<Input::size>(input);
}

}  // namespace op
}  // namespace xyz_autodiff
