#pragma once
// Unit quaternion (x, y, z, w) -> 3x3 rotation matrix, row-major in 9 elements.
//
//       | 1-2(yy+zz)   2(xy-zw)    2(xz+yw)  |
//   R = | 2(xy+zw)     1-2(xx+zz)  2(yz-xw)  |
//       | 2(xz-yw)     2(yz+xw)    1-2(xx+yy)|
//
// The quaternion is taken as given: it is not normalised, and the gradient is
// that of the polynomial above.  Counterpart of xyz-autodiff-cuda
// include/xyz_autodiff/operations/unary/to_rotation_matrix_logic.cuh
// (QuaternionToRotationMatrixLogic :12-114, factory :117-123); the backward
// there is a 4x9 table, here the same sums are grouped by the symmetric and
// antisymmetric parts of the upstream gradient.

#include <cstddef>

#include <xyz_autodiff/concept/variable.cuh>
#include <xyz_autodiff/operations/operation.cuh>

namespace xyz_autodiff {
namespace op {

template <std::size_t InputDim>
    requires(InputDim == 4)
struct QuaternionToRotationMatrixLogic {
    static constexpr std::size_t outputDim = 9;

    template <typename Output, typename Input>
    XAD_INLINE void forward(Output& out, const Input& in) const {
        using T = typename Input::value_type;
        const T x = in[0], y = in[1], z = in[2], w = in[3];
        const T two = T(2), one = T(1);
        out[0] = one - two * (y * y + z * z);
        out[1] = two * (x * y - z * w);
        out[2] = two * (x * z + y * w);
        out[3] = two * (x * y + z * w);
        out[4] = one - two * (x * x + z * z);
        out[5] = two * (y * z - x * w);
        out[6] = two * (x * z - y * w);
        out[7] = two * (y * z + x * w);
        out[8] = one - two * (x * x + y * y);
    }

    template <typename Output, typename Input>
    XAD_INLINE void backward(const Output& out, Input& in) const {
        using T = typename Input::value_type;
        const T x = in[0], y = in[1], z = in[2], w = in[3];
        // s_ij = g_ij + g_ji multiplies the products of two vector components,
        // k_ij = g_ji - g_ij multiplies the products with the scalar part w.
        const T sxy = out.grad(1) + out.grad(3);
        const T sxz = out.grad(2) + out.grad(6);
        const T syz = out.grad(5) + out.grad(7);
        const T kxy = out.grad(3) - out.grad(1);
        const T kzx = out.grad(2) - out.grad(6);
        const T kyz = out.grad(7) - out.grad(5);
        const T g00 = out.grad(0), g11 = out.grad(4), g22 = out.grad(8);
        const T two = T(2), four = T(4);
        in.add_grad(0, two * (y * sxy + z * sxz + w * kyz) - four * x * (g11 + g22));
        in.add_grad(1, two * (x * sxy + z * syz + w * kzx) - four * y * (g00 + g22));
        in.add_grad(2, two * (x * sxz + y * syz + w * kxy) - four * z * (g00 + g11));
        in.add_grad(3, two * (x * kyz + y * kzx + z * kxy));
    }
};

template <DifferentiableVariableConcept Input>
    requires(Input::size == 4)
XAD_INLINE auto quaternion_to_rotation_matrix(Input& quaternion) {
    using Logic = QuaternionToRotationMatrixLogic<4>;
    return UnaryOperation<9, Logic, Input>(Logic{}, quaternion);
}

}  // namespace op
}  // namespace xyz_autodiff
