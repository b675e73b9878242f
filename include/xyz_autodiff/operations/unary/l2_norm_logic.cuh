#pragma once
// y = sqrt(sum x_i^2); dy/dx_i = x_i / y.  At (numerically) zero norm, y <= 1e-8, no gradient flows.
// Counterpart of xyz-autodiff-cuda include/xyz_autodiff/operations/unary/l2_norm_logic.cuh (L2NormLogic :14-40, factories :43-59).

#include <cstddef>

#include <xyz_autodiff/concept/variable.cuh>
#include <xyz_autodiff/operations/math.cuh>
#include <xyz_autodiff/operations/operation.cuh>

namespace xyz_autodiff {
namespace op {

template <std::size_t InputDim>
struct L2NormLogic {
    static constexpr std::size_t outputDim = 1;

    template <typename Output, typename Input>
    XAD_INLINE void forward(Output& out, const Input& in) const {
        using T = typename Input::value_type;
        T acc = T(0);
        XAD_UNROLL
        for (std::size_t i = 0; i < InputDim; ++i) acc += in[i] * in[i];
        out[0] = math::sqrt(acc);
    }

    template <typename Output, typename Input>
    XAD_INLINE void backward(const Output& out, Input& in) const {
        using T = typename Input::value_type;
        const T g = out.grad(0);
        const T norm = out[0];
        if (norm > T(1e-8)) {
            XAD_UNROLL
            for (std::size_t i = 0; i < InputDim; ++i) in.add_grad(i, g * in[i] / norm);
        }
    }
};

template <std::size_t Dim, DifferentiableVariableConcept Input>
    requires(Input::size == Dim)
XAD_INLINE auto l2_norm(Input& input) {
    return UnaryOperation<1, L2NormLogic<Dim>, Input>(L2NormLogic<Dim>{}, input);
}

template <DifferentiableVariableConcept Input>
XAD_INLINE auto l2_norm(Input& input) {
    return l2_norm<Input::size>(input);
}

}  // namespace op
}  // namespace xyz_autodiff
