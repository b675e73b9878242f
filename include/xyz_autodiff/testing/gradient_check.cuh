#pragma once
// Analytic-versus-numerical gradient checks for op logic, usable from host code
// and from inside kernels.
//
// The method is that of the testers of xyz-autodiff-cuda
// (include/xyz_autodiff/testing/unary_gradient_tester.cuh:35-93 and :157-247,
// binary_gradient_tester.cuh:190-306): build a node over the logic, run forward,
// seed an upstream gradient, run the analytic backward; do the same with the
// central-difference backward; compare every input gradient with
//     error = min(|a - n|, |a - n| / (|a| + 1e-15)).
// There the testers are gtest fixtures that draw inputs with std::random_device
// and launch <<<1,1>>> kernels themselves; here they are plain functions over
// caller-supplied inputs that return the largest error, so they work in any test
// runner, on either side, and with reproducible inputs.

#include <cstddef>

#include <xyz_autodiff/operations/operation.cuh>
#include <xyz_autodiff/variable.cuh>

namespace xyz_autodiff {
namespace testing {

enum class GradientTag { Analytical, Numerical };

template <typename T>
XAD_INLINE T gradient_error(T analytic, T numeric) {
    const T diff = analytic > numeric ? analytic - numeric : numeric - analytic;
    const T mag = analytic < T(0) ? -analytic : analytic;
    const T rel = diff / (mag + T(1e-15));
    return diff < rel ? diff : rel;
}

// One unary logic, one input vector, one upstream gradient vector.
// `analytic` / `numeric` (optional, In elements each) receive the two gradients.
template <typename Logic, std::size_t In, std::size_t Out, typename T>
XAD_INLINE T check_unary(const Logic& logic, const T* input, const T* upstream, T delta, T* analytic = nullptr,
                         T* numeric = nullptr) {
    T worst = T(0);
    T grads[2][In];
    XAD_UNROLL
    for (int pass = 0; pass < 2; ++pass) {
        Variable<In, T> x(input);
        UnaryOperation<Out, Logic, Variable<In, T>> node(logic, x);
        node.forward();
        XAD_UNROLL
        for (std::size_t j = 0; j < Out; ++j) node.add_grad(j, upstream[j]);
        if (pass == 0)
            node.backward();
        else
            node.backward_numerical(delta);
        XAD_UNROLL
        for (std::size_t i = 0; i < In; ++i) grads[pass][i] = x.grad(i);
    }
    XAD_UNROLL
    for (std::size_t i = 0; i < In; ++i) {
        const T e = gradient_error(grads[0][i], grads[1][i]);
        worst = e > worst ? e : worst;
        if (analytic) analytic[i] = grads[0][i];
        if (numeric) numeric[i] = grads[1][i];
    }
    return worst;
}

// One binary logic; gradients of both inputs are compared.
template <typename Logic, std::size_t In1, std::size_t In2, std::size_t Out, typename T>
XAD_INLINE T check_binary(const Logic& logic, const T* input1, const T* input2, const T* upstream, T delta,
                          T* analytic = nullptr, T* numeric = nullptr) {
    T worst = T(0);
    T grads[2][In1 + In2];
    XAD_UNROLL
    for (int pass = 0; pass < 2; ++pass) {
        Variable<In1, T> a(input1);
        Variable<In2, T> b(input2);
        BinaryOperation<Out, Logic, Variable<In1, T>, Variable<In2, T>> node(logic, a, b);
        node.forward();
        XAD_UNROLL
        for (std::size_t j = 0; j < Out; ++j) node.add_grad(j, upstream[j]);
        if (pass == 0)
            node.backward();
        else
            node.backward_numerical(delta);
        XAD_UNROLL
        for (std::size_t i = 0; i < In1; ++i) grads[pass][i] = a.grad(i);
        XAD_UNROLL
        for (std::size_t i = 0; i < In2; ++i) grads[pass][In1 + i] = b.grad(i);
    }
    XAD_UNROLL
    for (std::size_t i = 0; i < In1 + In2; ++i) {
        const T e = gradient_error(grads[0][i], grads[1][i]);
        worst = e > worst ? e : worst;
        if (analytic) analytic[i] = grads[0][i];
        if (numeric) numeric[i] = grads[1][i];
    }
    return worst;
}

// A whole network.  `Network` is a callable  net.template operator()<Tag>(values, grads, delta)
// that builds its graph on VariableRefs into `values` (read) and `grads`
// (accumulated into) and calls run() or run_numerical(delta) according to Tag:
// the calling convention of the reference's NetworkGradientTester
// (network_gradient_tester.cuh:21-38).  Params is a struct of NumParams values
// of type T and nothing else.  Returns the largest error over all parameters.
template <typename Params, typename Network, std::size_t NumParams, typename T>
XAD_INLINE T check_network(const Network& net, const Params& values, T delta, T* analytic = nullptr, T* numeric = nullptr) {
    static_assert(sizeof(Params) == NumParams * sizeof(T), "Params must be NumParams values of type T");
    Params work = values, ga{}, gn{};
    net.template operator()<GradientTag::Analytical>(&work, &ga, delta);
    work = values;
    net.template operator()<GradientTag::Numerical>(&work, &gn, delta);
    const T* a = reinterpret_cast<const T*>(&ga);
    const T* n = reinterpret_cast<const T*>(&gn);
    T worst = T(0);
    for (std::size_t i = 0; i < NumParams; ++i) {
        const T e = gradient_error(a[i], n[i]);
        worst = e > worst ? e : worst;
        if (analytic) analytic[i] = a[i];
        if (numeric) numeric[i] = n[i];
    }
    return worst;
}

}  // namespace testing
}  // namespace xyz_autodiff
