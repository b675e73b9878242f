#pragma once
// xyz_autodiff::broadcast<N>(x): the materialising form of a broadcast, an
// ordinary unary node whose N outputs are copies of x[0] and whose backward
// adds the sum of the N output gradients to x[0].  Lives in namespace
// xyz_autodiff (not op) and is not pulled in by the umbrella header, as in
// xyz-autodiff-cuda (include/xyz_autodiff/operations/unary/broadcast_logic.cuh:11-46).
// Prefer op::broadcast, which needs no registers for the copies.

#include <cstddef>

#include <xyz_autodiff/concept/variable.cuh>
#include <xyz_autodiff/operations/operation.cuh>

namespace xyz_autodiff {

template <std::size_t OutputDim>
struct BroadcastLogic {
    static constexpr std::size_t outputDim = OutputDim;

    template <typename Output, typename Input>
    XAD_INLINE void forward(Output& out, const Input& in) const {
        static_assert(Input::size == 1, "broadcast source must have exactly one element");
        XAD_UNROLL
        for (std::size_t i = 0; i < OutputDim; ++i) out[i] = in[0];
    }

    template <typename Output, typename Input>
    XAD_INLINE void backward(const Output& out, Input& in) const {
        static_assert(Input::size == 1, "broadcast source must have exactly one element");
        typename Input::value_type total(0);
        XAD_UNROLL
        for (std::size_t i = 0; i < OutputDim; ++i) total += out.grad(i);
        in.add_grad(0, total);
    }
};

template <std::size_t OutputDim, DifferentiableVariableConcept Input>
    requires(Input::size == 1)
XAD_INLINE auto broadcast(Input& input) {
    return UnaryOperation<OutputDim, BroadcastLogic<OutputDim>, Input>(BroadcastLogic<OutputDim>{}, input);
}

}  // namespace xyz_autodiff
