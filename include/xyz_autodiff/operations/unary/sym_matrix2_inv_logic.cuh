#pragma once
// Inverse of a symmetric 2x2 matrix kept as three numbers.
//
//   input  [a, b, c]  stands for  | a b |      output [A, B, C]  for its inverse
//                                 | b c |             | A B |  =  1/det | c -b |
//                                                     | B C |           |-b  a |
//   det = a c - b^2.  A determinant of magnitude below 1e-8 is replaced by
//   +1e-8 in both passes, so the node never divides by zero.
//
// Backward treats b as one parameter (it appears twice in the matrix).  With
// r = 1/det the Jacobian in terms of the *outputs* is
//   dA/da = -A^2      dA/db = -2AB        dA/dc = r - AC
//   dB/da = -AB       dB/db = -r - 2B^2   dB/dc = -BC
//   dC/da = r - AC    dC/db = -2BC        dC/dc = -C^2
// which is the table of xyz-autodiff-cuda
// (include/xyz_autodiff/operations/unary/sym_matrix2_inv_logic.cuh:21-78,
// factory :81-88) with c/det, -b/det, a/det substituted.

#include <cstddef>

#include <xyz_autodiff/concept/variable.cuh>
#include <xyz_autodiff/operations/math.cuh>
#include <xyz_autodiff/operations/operation.cuh>

namespace xyz_autodiff {
namespace op {

template <std::size_t InputDim>
    requires(InputDim == 3)
struct SymMatrix2InvLogic {
    static constexpr std::size_t outputDim = 3;

    // 1 / det with the regularisation described above.
    template <typename T>
    XAD_INLINE static T guarded_inverse_determinant(const T& a, const T& b, const T& c) {
        T det = a * c - b * b;
        if (math::abs(det) < T(1e-8)) det = T(1e-8);
        return T(1) / det;
    }

    template <typename Output, typename Input>
    XAD_INLINE void forward(Output& out, const Input& in) const {
        using T = typename Input::value_type;
        const T a = in[0], b = in[1], c = in[2];
        const T r = guarded_inverse_determinant(a, b, c);
        out[0] = c * r;
        out[1] = -b * r;
        out[2] = a * r;
    }

    template <typename Output, typename Input>
    XAD_INLINE void backward(const Output& out, Input& in) const {
        using T = typename Input::value_type;
        const T a = in[0], b = in[1], c = in[2];
        const T r = guarded_inverse_determinant(a, b, c);
        const T A = c * r, B = -b * r, C = a * r;
        const T gA = out.grad(0), gB = out.grad(1), gC = out.grad(2);

        const T uA = gA * A, uB = gB * B, uC = gC * C;
        const T mixed = r - A * C;
        in.add_grad(0, gC * mixed - A * (uA + uB));
        in.add_grad(1, -(T(2) * B * (uA + uB + uC) + gB * r));
        in.add_grad(2, gA * mixed - C * (uC + uB));
    }
};

template <DifferentiableVariableConcept Input>
    requires(Input::size == 3)
XAD_INLINE auto sym_matrix2_inv(Input& input) {
    return UnaryOperation<3, SymMatrix2InvLogic<3>, Input>(SymMatrix2InvLogic<3>{}, input);
}

}  // namespace op
}  // namespace xyz_autodiff
