#pragma once
// The per-thread benchmark graph, written against the public operator API
// exactly as a user kernel would write it:
//
//   es  = exp(s)                                   s = (log sx, log sy)
//   cov = scale_rotation_to_covariance_3param(es, theta)
//   inv = sym_matrix2_inv(cov)
//   q   = mahalanobis_distance(p, inv)
//   w   = exp(-(q * 0.5)) * sigmoid(o)
//   w.run()   ->   w and d w / d (sx, sy, theta, o, px, py)
//
// It is the per-Gaussian graph of xyz-autodiff-cuda's splatting kernel
// (examples/mini-gaussian-splatting/gaussian_splatting_kernel.cu:86-97) with
// the query point as a differentiable leaf.  Leaves are thread-local
// Variables: every gradient belongs to one problem, so no atomics are needed.
// The function is compiled for gfx950 and for the host cores from this one
// body.

#include <xyz_autodiff/variable.cuh>
#include <xyz_autodiff/operations/unary/exp_logic.cuh>
#include <xyz_autodiff/operations/unary/neg_logic.cuh>
#include <xyz_autodiff/operations/unary/sigmoid_logic.cuh>
#include <xyz_autodiff/operations/unary/sym_matrix2_inv_logic.cuh>
#include <operations/covariance_generation.cuh>
#include <operations/mahalanobis_distance.cuh>
#include <xyz_autodiff/variable_operators.cuh>

namespace xad_chain {

template <typename T>
struct Result {
    T w;
    T d_sx, d_sy, d_theta, d_o, d_px, d_py;
};

template <typename T>
XAD_INLINE Result<T> forward_backward(T sx, T sy, T theta_in, T o, T px, T py) {
    using namespace xyz_autodiff;
    Variable<2, T> s;
    s[0] = sx;
    s[1] = sy;
    Variable<1, T> theta(theta_in);
    Variable<1, T> opacity(o);
    Variable<2, T> p;
    p[0] = px;
    p[1] = py;

    auto es = op::exp(s);
    auto cov = op::scale_rotation_to_covariance_3param(es, theta);
    auto inv = op::sym_matrix2_inv(cov);
    auto q = op::mahalanobis_distance(p, inv);
    auto half_q = q * T(0.5);
    auto neg_half_q = op::neg(half_q);
    auto falloff = op::exp(neg_half_q);
    auto alpha = op::sigmoid(opacity);
    auto w = falloff * alpha;
    w.run();

    return Result<T>{w[0], s.grad(0), s.grad(1), theta.grad(0), opacity.grad(0), p.grad(0), p.grad(1)};
}

}  // namespace xad_chain
