#pragma once
// SymmetricMatrixView<T, N, V>: an N(N+1)/2-vector variable V seen as a symmetric
// N x N matrix.  Storage is the upper triangle, row by row: row i starts at
// i N - i (i - 1) / 2, so for N = 3 the six stored values are
// (0,0) (0,1) (0,2) (1,1) (1,2) (2,2).  (i, j) and (j, i) refer to the same
// element, flat indexing addresses the storage, the transpose is the view itself.
// Same interface as xyz-autodiff-cuda include/xyz_autodiff/symmetric_matrix_view.cuh:11-107.

#include <cstddef>
#include <type_traits>

#include <xyz_autodiff/concept/matrix.cuh>
#include <xyz_autodiff/concept/variable.cuh>
#include <xyz_autodiff/detail/config.cuh>

namespace xyz_autodiff {

template <typename T, std::size_t N, DifferentiableVariableConcept Variable>
class SymmetricMatrixView {
    static_assert(Variable::size == N * (N + 1) / 2, "a symmetric N x N view needs N (N + 1) / 2 stored values");
    static_assert(std::is_same_v<typename Variable::value_type, T>, "element type of the view and of the storage differ");

public:
    using value_type = T;
    static constexpr std::size_t rows = N;
    static constexpr std::size_t cols = N;
    static constexpr std::size_t size = N * N;
    static constexpr std::size_t storage_size = N * (N + 1) / 2;

    XAD_HD explicit SymmetricMatrixView(Variable& storage) noexcept : storage_(storage) {}
    XAD_HD SymmetricMatrixView(const SymmetricMatrixView&) noexcept = default;

    // Copies the stored values and gradients of `other` into this view's storage.
    XAD_HD SymmetricMatrixView& operator=(const SymmetricMatrixView& other) {
        storage_ = other.storage_;
        return *this;
    }

    // Position of (row, col) in the storage, whichever triangle it lies in.
    XAD_INLINE static constexpr std::size_t storage_index(std::size_t row, std::size_t col) noexcept {
        const std::size_t i = row <= col ? row : col, j = row <= col ? col : row;
        return i * N - i * (i - 1) / 2 + (j - i);
    }

    XAD_INLINE T* data() { return storage_.data(); }
    XAD_INLINE const T* data() const { return storage_.data(); }
    XAD_INLINE T& operator()(std::size_t r, std::size_t c) { return storage_[storage_index(r, c)]; }
    XAD_INLINE const T& operator()(std::size_t r, std::size_t c) const { return storage_[storage_index(r, c)]; }
    XAD_INLINE T& operator[](std::size_t i) { return storage_[i]; }
    XAD_INLINE const T& operator[](std::size_t i) const { return storage_[i]; }

    XAD_INLINE SymmetricMatrixView& transpose() noexcept { return *this; }
    XAD_INLINE const SymmetricMatrixView& transpose() const noexcept { return *this; }

    XAD_INLINE T* grad() { return storage_.grad(); }
    XAD_INLINE const T* grad() const { return storage_.grad(); }
    XAD_INLINE const T& grad(std::size_t i) const { return storage_.grad(i); }
    XAD_INLINE void add_grad(std::size_t i, T g) { storage_.add_grad(i, g); }
    XAD_INLINE void zero_grad() { storage_.zero_grad(); }

    XAD_INLINE auto& underlying_variable() { return storage_; }
    XAD_INLINE const auto& underlying_variable() const { return storage_; }

private:
    Variable& storage_;
};

template <std::size_t N, DifferentiableVariableConcept Variable>
XAD_INLINE auto make_symmetric_matrix_view(Variable& storage) {
    return SymmetricMatrixView<typename Variable::value_type, N, Variable>(storage);
}

}  // namespace xyz_autodiff
