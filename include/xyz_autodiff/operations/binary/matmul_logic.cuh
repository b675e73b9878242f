#pragma once
// C = A B for small row-major matrices flattened into variables:
// A is a x b (a*b elements), B is b x c, C is a x c.
//   backward:  dA[i,k] += g[i,j] B[k,j]      dB[k,j] += g[i,j] A[i,k]
// All three extents are template parameters, so every loop unrolls and the
// matrices stay in registers.  This is per-lane arithmetic on 2x2..4x4
// operands, far below the granularity of the matrix cores.
// Counterpart of xyz-autodiff-cuda include/xyz_autodiff/operations/binary/matmul_logic.cuh
// (MatMulLogic :13-69, factories matmul :72-80, matmul_2x2/3x3/4x4 :83-105,
// matvec :108-113, vecmat :116-121).

#include <cstddef>

#include <xyz_autodiff/concept/core_logic.cuh>
#include <xyz_autodiff/operations/operation.cuh>

namespace xyz_autodiff {
namespace op {

template <std::size_t a, std::size_t b, std::size_t c, typename Input1, typename Input2>
    requires BinaryLogicParameterConcept<Input1, Input2> && (Input1::size == a * b) && (Input2::size == b * c)
struct MatMulLogic {
    using T = typename Input1::value_type;
    static constexpr std::size_t rows_A = a;
    static constexpr std::size_t cols_A_rows_B = b;
    static constexpr std::size_t cols_B = c;
    static constexpr std::size_t output_size = a * c;
    using Output = Variable<output_size, T>;
    static constexpr std::size_t outputDim = output_size;

    XAD_INLINE void forward(Output& out, const Input1& A, const Input2& B) const {
        XAD_UNROLL
        for (std::size_t i = 0; i < a; ++i) {
            XAD_UNROLL
            for (std::size_t j = 0; j < c; ++j) {
                T acc = T(0);
                XAD_UNROLL
                for (std::size_t k = 0; k < b; ++k) acc += A[i * b + k] * B[k * c + j];
                out[i * c + j] = acc;
            }
        }
    }

    XAD_INLINE void backward(const Output& out, Input1& A, Input2& B) const {
        XAD_UNROLL
        for (std::size_t i = 0; i < a; ++i) {
            XAD_UNROLL
            for (std::size_t j = 0; j < c; ++j) {
                const T g = out.grad(i * c + j);
                XAD_UNROLL
                for (std::size_t k = 0; k < b; ++k) {
                    const T a_ik = A[i * b + k], b_kj = B[k * c + j];
                    A.add_grad(i * b + k, g * b_kj);
                    B.add_grad(k * c + j, g * a_ik);
                }
            }
        }
    }
};

template <std::size_t a, std::size_t b, std::size_t c, typename Input1, typename Input2>
    requires BinaryLogicParameterConcept<Input1, Input2> && (Input1::size == a * b) && (Input2::size == b * c)
XAD_INLINE auto matmul(Input1& A, Input2& B) {
    using Logic = MatMulLogic<a, b, c, Input1, Input2>;
    return BinaryOperation<Logic::outputDim, Logic, Input1, Input2>(Logic{}, A, B);
}

template <typename Input1, typename Input2>
    requires BinaryLogicParameterConcept<Input1, Input2> && (Input1::size == 4) && (Input2::size == 4)
XAD_INLINE auto matmul_2x2(Input1& A, Input2& B) {
    return matmul<2, 2, 2>(A, B);
}

template <typename Input1, typename Input2>
    requires BinaryLogicParameterConcept<Input1, Input2> && (Input1::size == 9) && (Input2::size == 9)
XAD_INLINE auto matmul_3x3(Input1& A, Input2& B) {
    return matmul<3, 3, 3>(A, B);
}

template <typename Input1, typename Input2>
    requires BinaryLogicParameterConcept<Input1, Input2> && (Input1::size == 16) && (Input2::size == 16)
XAD_INLINE auto matmul_4x4(Input1& A, Input2& B) {
    return matmul<4, 4, 4>(A, B);
}

// y = A x with A m x n.
template <std::size_t m, std::size_t n, typename Input1, typename Input2>
    requires BinaryLogicParameterConcept<Input1, Input2> && (Input1::size == m * n) && (Input2::size == n)
XAD_INLINE auto matvec(Input1& A, Input2& x) {
    return matmul<m, n, 1>(A, x);
}

// y = x A with x of length m and A m x n.
template <std::size_t m, std::size_t n, typename Input1, typename Input2>
    requires BinaryLogicParameterConcept<Input1, Input2> && (Input1::size == m) && (Input2::size == m * n)
XAD_INLINE auto vecmat(Input1& x, Input2& A) {
    return matmul<1, m, n>(x, A);
}

}  // namespace op
}  // namespace xyz_autodiff
