#pragma once
// Scalar math used by the op logic, selected by value type.
//
// Function names and semantics follow the dispatcher of xyz-autodiff-cuda
// (include/xyz_autodiff/operations/math.cuh:14-298).  There the choice between
// the float and double routine was keyed on a CUDA architecture macro; here the
// overload is chosen from T alone, so device and host builds of one kernel
// body run the same formulas.
//
// fp32 exp, sin and cos have their own implementations (fp32::exp, fp32::sincos
// below), written once for both passes, accurate to about 1 ulp and a good deal
// shorter than the general library routines:
//   - the per-thread kernels are bound as much by VALU issue as by HBM, and the
//     library expf/sincosf spend most of their instructions on range and
//     denormal handling that a graph of bounded parameters never needs;
//   - device sincosf reduces its argument twice, once for each result.
// Hardware v_sin/v_cos are not used: their absolute error of ~1e-6 turns into a
// rotation error that the 2x2 covariance inverse amplifies.
// Everything else binds to the device library in the gfx950 pass and to libm
// in the host pass.

#include <cmath>
#include <cstdint>
#include <limits>
#include <type_traits>

#include <xyz_autodiff/detail/config.cuh>

namespace xyz_autodiff {
namespace math {

namespace fp32 {

// 2^t for a float exponent: one v_exp_f32 on the device.
XAD_INLINE float exp2_raw(float t) {
#if XAD_DEVICE_PASS
    return __builtin_amdgcn_exp2f(t);
#else
    return ::exp2f(t);
#endif
}

// e^x = 2^(x log2 e).  The product is formed in two pieces, t (rounded) and the
// part e of x*log2(e) that t lost; 2^(t+e) = 2^t (1 + e ln 2) to first order,
// |e| being below 2^-17.  About 1 ulp for |x| up to the overflow threshold;
// results below 2^-126 may be flushed to zero.
XAD_INLINE float exp(float x) {
    constexpr float kLog2eHi = 0x1.715476p+0f;   // log2(e) rounded to float
    constexpr float kLog2eLo = 0x1.4ae0c0p-26f;  // log2(e) - kLog2eHi
    constexpr float kLn2 = 0x1.62e43p-1f;
    const float t = x * kLog2eHi;
    float e = ::fmaf(x, kLog2eHi, -t);
    e = ::fmaf(x, kLog2eLo, e);
    const float r = exp2_raw(t);
    const float refined = ::fmaf(r, e * kLn2, r);
    // At both ends of the range r is already the answer and the refinement is not: r == inf turns it
    // into inf * 0 or inf - inf, and for x = -inf or a product that overflowed to -inf (r == 0) the
    // lost part e is itself inf or NaN.
    return (r == std::numeric_limits<float>::infinity() || r == 0.0f) ? r : refined;
}

// sin and cos of one argument from a single reduction.
//   k = round(|x| * 2/pi);  r = |x| - k*pi/2 in three pieces (Cody-Waite), |r| <= pi/4;
//   sin r and cos r from degree-7 / degree-8 minimax polynomials (Cephes sinf/cosf
//   coefficients); the quadrant k mod 4 picks and signs the results.
// Exact-product reduction holds while k fits the 13 trailing zero bits of the
// leading constant; beyond |x| = 8192 (and for inf/NaN) the library routine runs.
XAD_INLINE void sincos(float x, float& s, float& c) {
    const float ax = ::fabsf(x);
    if (!(ax < 8192.0f)) {
        ::sincosf(x, &s, &c);
        return;
    }
    const float k = ::rintf(ax * 0x1.45f306p-1f);  // 2/pi
    float r = ::fmaf(k, -0x1.921fb4p+0f, ax);       // pi/2, leading 23 bits (one zero at the end)
    r = ::fmaf(k, -0x1.4442d0p-24f, r);             // next piece
    r = ::fmaf(k, -0x1.846988p-48f, r);             // and the next
    const float z = r * r;
    float sp = ::fmaf(z, -1.9515295891e-4f, 8.3321608736e-3f);
    sp = ::fmaf(z, sp, -1.6666654611e-1f);
    sp = ::fmaf(z * r, sp, r);
    float cp = ::fmaf(z, 2.443315711809948e-5f, -1.388731625493765e-3f);
    cp = ::fmaf(z, cp, 4.166664568298827e-2f);
    cp = ::fmaf(z * z, cp, ::fmaf(z, -0.5f, 1.0f));
    const int q = static_cast<int>(k);
    const bool swap = (q & 1) != 0;
    const float s_mag = swap ? cp : sp;
    const float c_mag = swap ? sp : cp;
    const bool s_neg = ((q & 2) != 0) != (x < 0.0f);
    const bool c_neg = ((q + 1) & 2) != 0;
    s = s_neg ? -s_mag : s_mag;
    c = c_neg ? -c_mag : c_mag;
}

}  // namespace fp32

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

XAD_MATH_UNARY(exp, fp32::exp, ::exp)
XAD_MATH_UNARY(log, ::logf, ::log)

template <typename T>
XAD_INLINE T sin(const T& x) {
    if constexpr (std::is_same_v<T, float>) {
        float s, c;
        fp32::sincos(x, s, c);
        return s;
    } else {
        static_assert(std::is_same_v<T, double>, "math::sin: float or double");
        return ::sin(x);
    }
}

template <typename T>
XAD_INLINE T cos(const T& x) {
    if constexpr (std::is_same_v<T, float>) {
        float s, c;
        fp32::sincos(x, s, c);
        return c;
    } else {
        static_assert(std::is_same_v<T, double>, "math::cos: float or double");
        return ::cos(x);
    }
}

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
        fp32::sincos(x, s, c);
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
