#pragma once
// y = sum |x_i|; dy/dx_i = sign(x_i), with sign(0) = 0.
// Counterpart of xyz-autodiff-cuda include/xyz_autodiff/operations/unary/l1_norm_logic.cuh (L1NormLogic :14-37, factories :40-56).

#include <cstddef>

#include <xyz_autodiff/concept/variable.cuh>
#include <xyz_autodiff/operations/math.cuh>
#include <xyz_autodiff/operations/operation.cuh>

namespace xyz_autodiff {
namespace op {

template <std::size_t InputDim>
struct L1NormLogic {
    static constexpr std::size_t outputDim = 1;

    template <typename Output, typename Input>
    XAD_INLINE void forward(Output& out, const Input& in) const {
        using T = typename Input::value_type;
        T acc = T(0);
        XAD_UNROLL
        for (std::size_t i = 0; i < InputDim; ++i) acc += math::abs(in[i]);
        out[0] = acc;
    }

    template <typename Output, typename Input>
    XAD_INLINE void backward(const Output& out, Input& in) const {
        using T = typename Input::value_type;
        const T g = out.grad(0);
        XAD_UNROLL
        for (std::size_t i = 0; i < InputDim; ++i) {
            const T x = in[i];
            const T sign = x > T(0) ? T(1) : (x < T(0) ? T(-1) : T(0));
            in.add_grad(i, g * sign);
        }
    }
};

template <std::size_t Dim, DifferentiableVariableConcept Input>
    requires(Input::size == Dim)
XAD_INLINE auto l1_norm(Input& input) {
    return UnaryOperation<1, L1NormLogic<Dim>, Input>(L1NormLogic<Dim>{}, input);
}

template <DifferentiableVariableConcept Input>
XAD_INLINE auto l1_norm(Input& input) {
    return l1_norm<Input::size>(input);
}

}  // namespace op
}  // namespace xyz_autodiff
