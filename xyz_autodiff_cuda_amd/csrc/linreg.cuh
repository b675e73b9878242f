#pragma once
// Per-sample loss graph of the least-squares example, written against the
// library's public API so that one definition serves the GPU kernels (with
// register, global-memory or accumulator leaves) and the host-core build.
//
//   loss = ((a - x1)^2 + b (c - x2)^2 + d - y)^2
//
// Node for node the graph of compute_gradient_kernel in xyz-autodiff-cuda
// (examples/optimization/tests/test_linear_regression_gradient.cu:47-78).

#include <xyz_autodiff/operations/binary/add_logic.cuh>
#include <xyz_autodiff/operations/binary/mul_logic.cuh>
#include <xyz_autodiff/operations/unary/squared_logic.cuh>
#include <xyz_autodiff/operations/unary/sub_constant_logic.cuh>
#include <xyz_autodiff/variable.cuh>

namespace xad_linreg {

// Forward and backward for one sample; the gradients arrive through the
// leaves' add_grad.  Returns the loss.
template <typename A, typename B, typename C, typename D>
XAD_INLINE typename A::value_type run_loss_graph(A& a, B& b, C& c, D& d, typename A::value_type x1,
                                                 typename A::value_type x2, typename A::value_type y) {
    using namespace xyz_autodiff;
    auto a_minus_x1 = op::sub_constant(a, x1);
    auto x1_term = op::squared(a_minus_x1);
    auto c_minus_x2 = op::sub_constant(c, x2);
    auto x2_squared = op::squared(c_minus_x2);
    auto x2_term = op::mul(b, x2_squared);
    auto both_terms = op::add(x1_term, x2_term);
    auto prediction = op::add(both_terms, d);
    auto residual = op::sub_constant(prediction, y);
    auto loss = op::squared(residual);
    loss.run();
    return loss[0];
}

}  // namespace xad_linreg
