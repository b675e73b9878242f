#pragma once
// Squared Mahalanobis distance of a 2D offset under an inverse covariance kept
// as three numbers [a, b, c] = | a b ; b c |:
//
//     q = a dx^2 + 2 b dx dy + c dy^2
//     dq/d(dx, dy) = (2a dx + 2b dy, 2b dx + 2c dy)     dq/d(a, b, c) = (dx^2, 2 dx dy, dy^2)
//
//   mahalanobis_distance(diff, inv_cov)                       offset is an operand
//   mahalanobis_distance_with_center(px, py, centre, inv_cov) offset = (px, py) - centre, with the
//                                                             point a constant held by the logic;
//                                                             the centre receives the negated gradient
//
// Counterpart of xyz-autodiff-cuda examples/mini-gaussian-splatting/operations/mahalanobis_distance.cuh
// (MahalanobisDistanceLogic :15-64, MahalanobisDistanceWithCenterLogic :72-120, factories :123-146).

#include <cstddef>
#include <type_traits>

#include <xyz_autodiff/concept/core_logic.cuh>
#include <xyz_autodiff/operations/operation.cuh>

namespace xyz_autodiff {
namespace op {

namespace detail_maha {

template <typename T>
XAD_INLINE T quadratic_form(T dx, T dy, T a, T b, T c) {
    return a * dx * dx + T(2) * b * dx * dy + c * dy * dy;
}

template <typename T, typename InvCov>
XAD_INLINE void credit_inverse_covariance(T g, T dx, T dy, InvCov& inv_cov) {
    inv_cov.add_grad(0, g * dx * dx);
    inv_cov.add_grad(1, g * T(2) * dx * dy);
    inv_cov.add_grad(2, g * dy * dy);
}

}  // namespace detail_maha

template <typename Input1, typename Input2>
    requires BinaryLogicParameterConcept<Input1, Input2> && (Input1::size == 2) && (Input2::size == 3)
struct MahalanobisDistanceLogic {
    using T = typename Input1::value_type;
    static constexpr std::size_t Dim = 1;
    using Output = Variable<Dim, T>;
    static constexpr std::size_t outputDim = Dim;

    XAD_INLINE void forward(Output& out, const Input1& diff, const Input2& inv_cov) const {
        out[0] = detail_maha::quadratic_form<T>(diff[0], diff[1], inv_cov[0], inv_cov[1], inv_cov[2]);
    }

    XAD_INLINE void backward(const Output& out, Input1& diff, Input2& inv_cov) const {
        const T g = out.grad(0);
        const T dx = diff[0], dy = diff[1];
        const T a = inv_cov[0], b = inv_cov[1], c = inv_cov[2];
        diff.add_grad(0, g * (T(2) * a * dx + T(2) * b * dy));
        diff.add_grad(1, g * (T(2) * b * dx + T(2) * c * dy));
        detail_maha::credit_inverse_covariance(g, dx, dy, inv_cov);
    }
};

template <typename Input1, typename Input2>
    requires BinaryLogicParameterConcept<Input1, Input2> && (Input1::size == 2) && (Input2::size == 3)
struct MahalanobisDistanceWithCenterLogic {
    using T = typename Input1::value_type;
    static constexpr std::size_t Dim = 1;
    using Output = Variable<Dim, T>;
    static constexpr std::size_t outputDim = Dim;

    T point_x, point_y;

    XAD_HD MahalanobisDistanceWithCenterLogic(T px, T py) : point_x(px), point_y(py) {}

    XAD_INLINE void forward(Output& out, const Input1& center, const Input2& inv_cov) const {
        out[0] = detail_maha::quadratic_form<T>(point_x - center[0], point_y - center[1],
                                                inv_cov[0], inv_cov[1], inv_cov[2]);
    }

    XAD_INLINE void backward(const Output& out, Input1& center, Input2& inv_cov) const {
        const T g = out.grad(0);
        const T dx = point_x - center[0], dy = point_y - center[1];
        const T a = inv_cov[0], b = inv_cov[1], c = inv_cov[2];
        center.add_grad(0, -(g * (T(2) * a * dx + T(2) * b * dy)));
        center.add_grad(1, -(g * (T(2) * b * dx + T(2) * c * dy)));
        detail_maha::credit_inverse_covariance(g, dx, dy, inv_cov);
    }
};

template <typename Input1, typename Input2>
    requires BinaryLogicParameterConcept<Input1, Input2> && (Input1::size == 2) && (Input2::size == 3)
XAD_INLINE auto mahalanobis_distance(Input1& diff, Input2& inv_cov) {
    using Logic = MahalanobisDistanceLogic<Input1, Input2>;
    return BinaryOperation<Logic::outputDim, Logic, Input1, Input2>(Logic{}, diff, inv_cov);
}

template <typename Input1, typename Input2>
    requires BinaryLogicParameterConcept<Input1, Input2> && (Input1::size == 2) && (Input2::size == 3)
XAD_INLINE auto mahalanobis_distance_with_center(typename Input1::value_type point_x,
                                                 typename Input1::value_type point_y,
                                                 Input1& center, Input2& inv_cov) {
    using Logic = MahalanobisDistanceWithCenterLogic<Input1, Input2>;
    return BinaryOperation<Logic::outputDim, Logic, Input1, Input2>(Logic(point_x, point_y), center, inv_cov);
}

}  // namespace op
}  // namespace xyz_autodiff
