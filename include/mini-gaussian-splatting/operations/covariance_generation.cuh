#pragma once
// Op logic that turns the scale and rotation of a 2D Gaussian into its
// covariance.
//
//   generate_covariance_matrix(scale, rotation)          M = R(theta) diag(sx, sy)      -> 4 (row-major 2x2)
//   matrix_to_covariance_3param(M)                       Sigma = M M^T                  -> 3 ([S00, S01, S11])
//   scale_rotation_to_covariance_3param(scale, rotation) both steps in one node          -> 3
//
// R(theta) = | cos -sin |   so   M = | sx cos  -sy sin |
//            | sin  cos |            | sx sin   sy cos |
//
// Names, operand sizes and the fused node follow xyz-autodiff-cuda
// (examples/mini-gaussian-splatting/operations/covariance_generation.cuh:
// CovarianceMatrixGenerationLogic :15-76, MatrixToCovariance3ParamLogic :81-136,
// ScaleRotationToCovariance3ParamLogic :142-212, factories :215-238).  The
// backward rules apply the chain rule in the same order as there: first to the
// entries of M, then to (sx, sy, theta).
//
// sin(theta) and cos(theta) are needed by forward and by backward.  The logic
// object remembers the pair together with the angle it belongs to; backward
// reuses it when the angle is bit-for-bit the one forward saw (always, inside a
// graph: the comparison is then resolved at compile time and the second
// evaluation disappears) and evaluates afresh otherwise, e.g. after the
// numerical backward has perturbed the angle.

#include <bit>
#include <cstddef>
#include <cstdint>
#include <type_traits>

#include <xyz_autodiff/concept/core_logic.cuh>
#include <xyz_autodiff/operations/math.cuh>
#include <xyz_autodiff/operations/operation.cuh>

namespace xyz_autodiff {
namespace op {

namespace detail_cov {

template <typename T>
struct AngleMemo {
    using Bits = std::conditional_t<sizeof(T) == 4, std::uint32_t, std::uint64_t>;
    T angle = T(0), sn = T(0), cs = T(1);
    bool filled = false;

    XAD_INLINE void evaluate(T theta) {
        math::sincos(theta, sn, cs);
        angle = theta;
        filled = true;
    }
    XAD_INLINE void lookup(T theta) {
        if (!(filled && std::bit_cast<Bits>(theta) == std::bit_cast<Bits>(angle))) evaluate(theta);
    }
};

// M and the pull-back of a gradient on M to (sx, sy, theta); shared by the
// stand-alone and the fused node.
template <typename T>
struct RotatedScale {
    T sx, sy, cs, sn;
    T m00, m01, m10, m11;

    XAD_INLINE RotatedScale(T sx_, T sy_, const AngleMemo<T>& trig) : sx(sx_), sy(sy_), cs(trig.cs), sn(trig.sn) {
        m00 = sx * cs;
        m01 = -sy * sn;
        m10 = sx * sn;
        m11 = sy * cs;
    }

    template <typename Scale, typename Rotation>
    XAD_INLINE void pull_back(T g00, T g01, T g10, T g11, Scale& scale, Rotation& rotation) const {
        scale.add_grad(0, g00 * cs + g10 * sn);
        scale.add_grad(1, g01 * (-sn) + g11 * cs);
        rotation.add_grad(0, g00 * (-sx * sn) + g01 * (-sy * cs) + g10 * (sx * cs) + g11 * (-sy * sn));
    }
};

}  // namespace detail_cov

template <typename Input1, typename Input2>
    requires BinaryLogicParameterConcept<Input1, Input2> && (Input1::size == 2) && (Input2::size == 1)
struct CovarianceMatrixGenerationLogic {
    using T = typename Input1::value_type;
    static constexpr std::size_t Dim = 4;
    using Output = Variable<Dim, T>;
    static constexpr std::size_t outputDim = Dim;

    mutable detail_cov::AngleMemo<T> trig_;

    XAD_INLINE void forward(Output& out, const Input1& scale, const Input2& rotation) const {
        trig_.evaluate(rotation[0]);
        const detail_cov::RotatedScale<T> m(scale[0], scale[1], trig_);
        out[0] = m.m00;
        out[1] = m.m01;
        out[2] = m.m10;
        out[3] = m.m11;
    }

    XAD_INLINE void backward(const Output& out, Input1& scale, Input2& rotation) const {
        trig_.lookup(rotation[0]);
        const detail_cov::RotatedScale<T> m(scale[0], scale[1], trig_);
        m.pull_back(out.grad(0), out.grad(1), out.grad(2), out.grad(3), scale, rotation);
    }
};

template <typename Input>
    requires UnaryLogicParameterConcept<Input> && (Input::size == 4)
struct MatrixToCovariance3ParamLogic {
    using T = typename Input::value_type;
    static constexpr std::size_t Dim = 3;
    using Output = Variable<Dim, T>;
    static constexpr std::size_t outputDim = Dim;

    XAD_INLINE void forward(Output& out, const Input& M) const {
        const T m00 = M[0], m01 = M[1], m10 = M[2], m11 = M[3];
        out[0] = m00 * m00 + m01 * m01;
        out[1] = m00 * m10 + m01 * m11;
        out[2] = m10 * m10 + m11 * m11;
    }

    XAD_INLINE void backward(const Output& out, Input& M) const {
        const T m00 = M[0], m01 = M[1], m10 = M[2], m11 = M[3];
        const T g00 = out.grad(0), g01 = out.grad(1), g11 = out.grad(2);
        M.add_grad(0, g00 * T(2) * m00 + g01 * m10);
        M.add_grad(1, g00 * T(2) * m01 + g01 * m11);
        M.add_grad(2, g01 * m00 + g11 * T(2) * m10);
        M.add_grad(3, g01 * m01 + g11 * T(2) * m11);
    }
};

template <typename Input1, typename Input2>
    requires BinaryLogicParameterConcept<Input1, Input2> && (Input1::size == 2) && (Input2::size == 1)
struct ScaleRotationToCovariance3ParamLogic {
    using T = typename Input1::value_type;
    static constexpr std::size_t Dim = 3;
    using Output = Variable<Dim, T>;
    static constexpr std::size_t outputDim = Dim;

    mutable detail_cov::AngleMemo<T> trig_;

    XAD_INLINE void forward(Output& out, const Input1& scale, const Input2& rotation) const {
        trig_.evaluate(rotation[0]);
        const detail_cov::RotatedScale<T> m(scale[0], scale[1], trig_);
        out[0] = m.m00 * m.m00 + m.m01 * m.m01;
        out[1] = m.m00 * m.m10 + m.m01 * m.m11;
        out[2] = m.m10 * m.m10 + m.m11 * m.m11;
    }

    XAD_INLINE void backward(const Output& out, Input1& scale, Input2& rotation) const {
        trig_.lookup(rotation[0]);
        const detail_cov::RotatedScale<T> m(scale[0], scale[1], trig_);
        const T g00 = out.grad(0), g01 = out.grad(1), g11 = out.grad(2);
        m.pull_back(g00 * T(2) * m.m00 + g01 * m.m10,
                    g00 * T(2) * m.m01 + g01 * m.m11,
                    g01 * m.m00 + g11 * T(2) * m.m10,
                    g01 * m.m01 + g11 * T(2) * m.m11, scale, rotation);
    }
};

template <typename Input1, typename Input2>
    requires BinaryLogicParameterConcept<Input1, Input2> && (Input1::size == 2) && (Input2::size == 1)
XAD_INLINE auto generate_covariance_matrix(Input1& scale, Input2& rotation) {
    using Logic = CovarianceMatrixGenerationLogic<Input1, Input2>;
    return BinaryOperation<Logic::outputDim, Logic, Input1, Input2>(Logic{}, scale, rotation);
}

template <typename Input>
    requires UnaryLogicParameterConcept<Input> && (Input::size == 4)
XAD_INLINE auto matrix_to_covariance_3param(Input& M) {
    using Logic = MatrixToCovariance3ParamLogic<Input>;
    return UnaryOperation<Logic::outputDim, Logic, Input>(Logic{}, M);
}

template <typename Input1, typename Input2>
    requires BinaryLogicParameterConcept<Input1, Input2> && (Input1::size == 2) && (Input2::size == 1)
XAD_INLINE auto scale_rotation_to_covariance_3param(Input1& scale, Input2& rotation) {
    using Logic = ScaleRotationToCovariance3ParamLogic<Input1, Input2>;
    return BinaryOperation<Logic::outputDim, Logic, Input1, Input2>(Logic{}, scale, rotation);
}

}  // namespace op
}  // namespace xyz_autodiff
