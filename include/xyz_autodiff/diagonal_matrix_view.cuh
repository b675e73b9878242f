#pragma once
// DiagonalMatrixView<T, N, V>: an N-vector variable V seen as the N x N diagonal
// matrix diag(v).  (i, j) yields v[i] on the diagonal and zero elsewhere, flat
// indexing and the gradient interface go straight to the vector, the transpose
// is the view itself.  The view holds a reference: the vector must outlive it.
// Same interface as xyz-autodiff-cuda include/xyz_autodiff/diagonal_matrix_view.cuh:9-101.

#include <cstddef>

#include <xyz_autodiff/detail/config.cuh>
#include <xyz_autodiff/variable.cuh>

namespace xyz_autodiff {

template <typename T, std::size_t N, typename VariableType = VariableRef<N, T>>
class DiagonalMatrixView {
public:
    using value_type = T;
    static constexpr std::size_t rows = N;
    static constexpr std::size_t cols = N;
    static constexpr std::size_t size = N;  // stored elements: the diagonal

    XAD_HD DiagonalMatrixView(VariableType& diagonal) noexcept : diagonal_(diagonal) {}
    XAD_HD DiagonalMatrixView(const DiagonalMatrixView&) noexcept = default;
    DiagonalMatrixView& operator=(const DiagonalMatrixView&) = delete;

    XAD_INLINE T* data() const { return diagonal_.data(); }
    XAD_INLINE T* grad() const { return diagonal_.grad(); }
    XAD_INLINE T& operator[](std::size_t i) const { return diagonal_[i]; }
    XAD_INLINE const T& grad(std::size_t i) const { return diagonal_.grad(i); }
    XAD_INLINE void add_grad(std::size_t i, T g) const { diagonal_.add_grad(i, g); }
    XAD_INLINE void zero_grad() const { diagonal_.zero_grad(); }

    XAD_INLINE constexpr T operator()(std::size_t r, std::size_t c) const { return r == c ? diagonal_[r] : T(0); }

    XAD_INLINE DiagonalMatrixView transpose() const noexcept { return *this; }

    XAD_INLINE VariableType& underlying_variable() { return diagonal_; }
    XAD_INLINE const VariableType& underlying_variable() const { return diagonal_; }

private:
    VariableType& diagonal_;
};

template <std::size_t N, typename T>
XAD_INLINE auto make_diagonal_matrix_view(VariableRef<N, T>& v) {
    return DiagonalMatrixView<T, N, VariableRef<N, T>>(v);
}

template <std::size_t N, typename T>
XAD_INLINE auto make_diagonal_matrix_view(Variable<N, T>& v) {
    return DiagonalMatrixView<T, N, Variable<N, T>>(v);
}

}  // namespace xyz_autodiff
