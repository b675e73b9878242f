#pragma once
// DenseMatrix<T, Rows, Cols>: a small row-major matrix that owns its values and
// gradients, usable both as a differentiable variable (flat index) and as a
// matrix ((row, col) index).  operator* multiplies any two matrix views of
// matching inner extent into a DenseMatrix; it is a forward-only convenience
// (no gradient is recorded: use op::matmul inside a graph).
// Same interface as xyz-autodiff-cuda include/xyz_autodiff/dense_matrix.cuh:11-125.
// Extents are template parameters, so the loops below unroll completely and a
// matrix lives in registers; these are 2x2..4x4 per-lane operands.

#include <cstddef>

#include <xyz_autodiff/concept/matrix.cuh>
#include <xyz_autodiff/detail/config.cuh>

namespace xyz_autodiff {

template <typename T, std::size_t Rows, std::size_t Cols>
class DenseMatrix {
public:
    using value_type = T;
    static constexpr std::size_t rows = Rows;
    static constexpr std::size_t cols = Cols;
    static constexpr std::size_t size = Rows * Cols;

    XAD_HD constexpr DenseMatrix() noexcept : data_{}, grad_{} {}

    // ---- as a variable -----------------------------------------------------
    XAD_INLINE T* data() noexcept { return data_; }
    XAD_INLINE const T* data() const noexcept { return data_; }
    XAD_INLINE T* grad() noexcept { return grad_; }
    XAD_INLINE const T* grad() const noexcept { return grad_; }
    XAD_INLINE constexpr T& operator[](std::size_t i) noexcept { return data_[i]; }
    XAD_INLINE constexpr const T& operator[](std::size_t i) const noexcept { return data_[i]; }
    XAD_INLINE constexpr const T& grad(std::size_t i) const noexcept { return grad_[i]; }
    XAD_INLINE constexpr void add_grad(std::size_t i, T g) noexcept { grad_[i] += g; }
    XAD_INLINE constexpr void zero_grad() noexcept {
        XAD_UNROLL
        for (std::size_t i = 0; i < size; ++i) grad_[i] = T(0);
    }

    // ---- as a matrix -------------------------------------------------------
    XAD_INLINE constexpr T& operator()(std::size_t r, std::size_t c) noexcept { return data_[r * Cols + c]; }
    XAD_INLINE constexpr const T& operator()(std::size_t r, std::size_t c) const noexcept { return data_[r * Cols + c]; }

    // A transposed copy of the values (gradients start from zero).
    XAD_INLINE constexpr DenseMatrix<T, Cols, Rows> transpose() const noexcept {
        DenseMatrix<T, Cols, Rows> out;
        XAD_UNROLL
        for (std::size_t r = 0; r < Rows; ++r) {
            XAD_UNROLL
            for (std::size_t c = 0; c < Cols; ++c) out(c, r) = (*this)(r, c);
        }
        return out;
    }

private:
    T data_[Rows * Cols];
    T grad_[Rows * Cols];
};

template <typename A, typename B>
    requires MatrixViewConcept<A> && MatrixViewConcept<B> && (A::cols == B::rows)
XAD_INLINE constexpr DenseMatrix<typename A::value_type, A::rows, B::cols> operator*(const A& a, const B& b) {
    using T = typename A::value_type;
    DenseMatrix<T, A::rows, B::cols> out;
    XAD_UNROLL
    for (std::size_t i = 0; i < A::rows; ++i) {
        XAD_UNROLL
        for (std::size_t j = 0; j < B::cols; ++j) {
            T acc = T(0);
            XAD_UNROLL
            for (std::size_t k = 0; k < A::cols; ++k) acc += a(i, k) * b(k, j);
            out(i, j) = acc;
        }
    }
    return out;
}

}  // namespace xyz_autodiff
