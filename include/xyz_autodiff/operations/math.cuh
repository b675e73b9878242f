#pragma once
// Scalar math used by the op logic, selected by value type.
//
// Function names and semantics follow the dispatcher of xyz-autodiff-cuda
// (include/xyz_autodiff/operations/math.cuh:14-298).  There the choice between
// the float and double routine was keyed on a CUDA architecture macro; here the
// overload is chosen from T alone and the compiler binds the call to the
// device library in the gfx950 pass and to libm in the host pass, so device
// and host builds of one kernel body run the same formulas.
//
// fp32 routines are the full-accuracy ones (1-2 ulp): gradients of
// ill-conditioned 2x2 inverses amplify input error by the condition number,
// so hardware approximations of sin/cos are not used anywhere.

#include <cmath>
#include <type_traits>

#include <xyz_autodiff/detail/config.cuh>

namespace xyz_autodiff {
namespace math {

#define XAD_MATH_UNARY(name, f32, f64)                         \
    template <typename T>                                      \
    XAD_INLINE T name(const T& x) {                            \
        if constexpr (std::is_same_v<T, float>) {              \
            return f32(x);                                     \
        } else {                                               \
            static_assert(std::is_same_v<T, double>,           \
                          "math::" #name ": float or double"); \
            return f64(x);                                     \
        }                                                      \
    }

XAD_MATH_UNARY(exp, ::expf, ::exp)
XAD_MATH_UNARY(log, ::logf, ::log)
XAD_MATH_UNARY(sin, ::sinf, ::sin)
XAD_MATH_UNARY(cos, ::cosf, ::cos)
XAD_MATH_UNARY(tan, ::tanf, ::tan)
XAD_MATH_UNARY(sinh, ::sinhf, ::sinh)
XAD_MATH_UNARY(cosh, ::coshf, ::cosh)
XAD_MATH_UNARY(tanh, ::tanhf, ::tanh)
XAD_MATH_UNARY(sqrt, ::sqrtf, ::sqrt)
XAD_MATH_UNARY(abs, ::fabsf, ::fabs)

#undef XAD_MATH_UNARY

template <typename T>
XAD_INLINE T pow(const T& base, const T& exponent) {
    if constexpr (std::is_same_v<T, float>) {
        return ::powf(base, exponent);
    } else {
        static_assert(std::is_same_v<T, double>, "math::pow: float or double");
        return ::pow(base, exponent);
    }
}

template <typename T>
XAD_INLINE T max(const T& a, const T& b) {
    if constexpr (std::is_same_v<T, float>) {
        return ::fmaxf(a, b);
    } else {
        static_assert(std::is_same_v<T, double>, "math::max: float or double");
        return ::fmax(a, b);
    }
}

template <typename T>
XAD_INLINE T min(const T& a, const T& b) {
    if constexpr (std::is_same_v<T, float>) {
        return ::fminf(a, b);
    } else {
        static_assert(std::is_same_v<T, double>, "math::min: float or double");
        return ::fmin(a, b);
    }
}

// sin and cos of one angle from a single argument reduction.  Not part of the
// original dispatcher; the rotation-based op logic uses it.
template <typename T>
XAD_INLINE void sincos(const T& x, T& s, T& c) {
    if constexpr (std::is_same_v<T, float>) {
        ::sincosf(x, &s, &c);
    } else {
        static_assert(std::is_same_v<T, double>, "math::sincos: float or double");
        ::sincos(x, &s, &c);
    }
}

// ---- activations ----------------------------------------------------------

template <typename T>
XAD_INLINE T sigmoid(const T& x) {
    return T(1) / (T(1) + exp(-x));
}

template <typename T>
XAD_INLINE T relu(const T& x) {
    return x > T(0) ? x : T(0);
}

template <typename T>
XAD_INLINE T leaky_relu(const T& x, const T& alpha = T(0.01)) {
    return x > T(0) ? x : alpha * x;
}

template <typename T>
XAD_INLINE T elu(const T& x, const T& alpha = T(1)) {
    return x >= T(0) ? x : alpha * (exp(x) - T(1));
}

template <typename T>
XAD_INLINE T softplus(const T& x) {
    return log(T(1) + exp(x));
}

template <typename T>
XAD_INLINE T swish(const T& x) {
    return x * sigmoid(x);
}

// tanh form of GELU: 0.5 x (1 + tanh( sqrt(2/pi) (x + 0.044715 x^3) )).
template <typename T>
XAD_INLINE T gelu(const T& x) {
    const T k = T(0.7978845608028654);
    const T cubic = T(0.044715);
    return T(0.5) * x * (T(1) + tanh(k * (x + cubic * pow(x, T(3)))));
}

}  // namespace math
}  // namespace xyz_autodiff
