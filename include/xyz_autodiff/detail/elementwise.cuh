#pragma once
// Building blocks for element-wise op logic.
//
// A *rule* is a stateless struct with
//     value(x)       -> y            the function
//     slope(x, y)    -> dy/dx        its derivative, free to use x, y or both
// and MapLogic<Dim, Rule> turns it into an op-logic struct (outputDim, forward,
// backward) over Dim elements.  backward() expects `out` to hold the values the
// matching forward() produced: rules whose derivative is a function of the
// result (exp, sigmoid) reuse it instead of evaluating the transcendental a
// second time.

#include <cstddef>

#include <xyz_autodiff/detail/config.cuh>

namespace xyz_autodiff {
namespace detail {

template <std::size_t Dim, typename Rule>
struct MapLogic {
    static constexpr std::size_t outputDim = Dim;

    template <typename Output, typename Input>
    XAD_INLINE void forward(Output& out, const Input& in) const {
        XAD_UNROLL
        for (std::size_t i = 0; i < Dim; ++i) out[i] = Rule::value(in[i]);
    }

    template <typename Output, typename Input>
    XAD_INLINE void backward(const Output& out, Input& in) const {
        XAD_UNROLL
        for (std::size_t i = 0; i < Dim; ++i) in.add_grad(i, out.grad(i) * Rule::slope(in[i], out[i]));
    }
};

}  // namespace detail
}  // namespace xyz_autodiff
