#pragma once
// Arithmetic operators on anything differentiable: leaves, nodes, views.
//
//   v + c, v - c, v * c, v / c     scalar constant c          -> *_constant nodes
//   u + v, u - v, u * v, u / v     same size and scalar type  -> element-wise nodes
//   v + k, v - k                   k any array-like constant  -> const_add / const_sub
//
// Operands are taken by non-const lvalue reference because the resulting node
// keeps a reference to them: `auto t = a * b; auto u = t + c;` works, chaining
// temporaries (`a * b + c`) deliberately does not compile.
// Same overload set as xyz-autodiff-cuda include/xyz_autodiff/variable_operators.cuh:23-79.
// Include after the op headers whose factories it forwards to.
//
// One deliberate difference: `A * B` between two matrix views (DenseMatrix and
// friends) is the matrix product of dense_matrix.cuh, never the element-wise
// node.  With the reference's overload set the element-wise form silently wins
// for two non-const square matrices of equal size once both headers are included.

#include <concepts>

#include <xyz_autodiff/concept/matrix.cuh>
#include <xyz_autodiff/concept/variable.cuh>
#include <xyz_autodiff/operations/binary/add_logic.cuh>
#include <xyz_autodiff/operations/binary/div_logic.cuh>
#include <xyz_autodiff/operations/binary/mul_logic.cuh>
#include <xyz_autodiff/operations/binary/sub_logic.cuh>
#include <xyz_autodiff/operations/unary/add_constant_logic.cuh>
#include <xyz_autodiff/operations/unary/const_array_add_logic.cuh>
#include <xyz_autodiff/operations/unary/const_array_concepts.cuh>
#include <xyz_autodiff/operations/unary/const_array_sub_logic.cuh>
#include <xyz_autodiff/operations/unary/div_constant_logic.cuh>
#include <xyz_autodiff/operations/unary/mul_constant_logic.cuh>
#include <xyz_autodiff/operations/unary/sub_constant_logic.cuh>

namespace xyz_autodiff {

namespace detail {
template <typename U, typename V>
concept SameShape = DifferentiableVariableConcept<U> && DifferentiableVariableConcept<V> &&
                    (U::size == V::size) && std::same_as<typename U::value_type, typename V::value_type>;
}  // namespace detail

#define XAD_SCALAR_OPERATOR(symbol, factory)                                           \
    template <DifferentiableVariableConcept Var>                                        \
    XAD_INLINE auto operator symbol(Var& var, const typename Var::value_type& scalar) { \
        return op::factory(var, scalar);                                                \
    }
XAD_SCALAR_OPERATOR(+, add_constant)
XAD_SCALAR_OPERATOR(-, sub_constant)
XAD_SCALAR_OPERATOR(*, mul_constant)
XAD_SCALAR_OPERATOR(/, div_constant)
#undef XAD_SCALAR_OPERATOR

#define XAD_ELEMENTWISE_OPERATOR(symbol, factory)        \
    template <typename Var1, typename Var2>              \
        requires detail::SameShape<Var1, Var2>           \
    XAD_INLINE auto operator symbol(Var1& lhs, Var2& rhs) { \
        return op::factory(lhs, rhs);                    \
    }
XAD_ELEMENTWISE_OPERATOR(+, add)
XAD_ELEMENTWISE_OPERATOR(-, sub)
XAD_ELEMENTWISE_OPERATOR(/, div)
#undef XAD_ELEMENTWISE_OPERATOR

template <typename Var1, typename Var2>
    requires detail::SameShape<Var1, Var2> && (!(MatrixViewConcept<Var1> && MatrixViewConcept<Var2>))
XAD_INLINE auto operator*(Var1& lhs, Var2& rhs) {
    return op::mul(lhs, rhs);
}

template <DifferentiableVariableConcept Var, typename ConstArray>
    requires op::ArrayLikeConcept<ConstArray>
XAD_INLINE auto operator+(Var& var, const ConstArray& constants) {
    return op::const_add(var, constants);
}

template <DifferentiableVariableConcept Var, typename ConstArray>
    requires op::ArrayLikeConcept<ConstArray>
XAD_INLINE auto operator-(Var& var, const ConstArray& constants) {
    return op::const_sub(var, constants);
}

}  // namespace xyz_autodiff
