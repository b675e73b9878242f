#pragma once
// Compile-time contracts of the public API.  The tests of xyz-autodiff-cuda assert, per operation they cover, that
// the node satisfies VariableConcept, DifferentiableVariableConcept and OperationNode and that a leaf does not
// satisfy OperationNode (tests/operation/base/test_operation_concepts.cu:35-102; the head of every
// tests/operation/{unary,binary}/*_gradient.cu, test_norm_operations.cu:26-47, test_sym_matrix2_inv.cu,
// test_quaternion_to_rotation_matrix.cu:23-37), and for the containers MatrixViewConcept and the ConstArray
// concepts (tests/test_variable.cu:185-188, test_dense_matrix.cu:189-191, test_diagonal_matrix.cu:176-179,
// test_symmetric_matrix.cu:197-200, test_matrix_transpose.cu:180-192, test_const_array.cu:36-70,
// tests/operation/unary/test_const_array_concepts.cu:11-12).  Here the same contracts are asserted for every
// logic of the library, over both kinds of leaf and both value types.  Nothing runs: building is the test.
#include <xyz_autodiff/xyz_autodiff.cuh>
#include <xyz_autodiff/operations/unary/broadcast_logic.cuh>
#include <operations/covariance_generation.cuh>
#include <operations/mahalanobis_distance.cuh>

namespace xad_concepts {

using namespace xyz_autodiff;

template <typename Node>
inline constexpr bool is_node = VariableConcept<Node> && DifferentiableVariableConcept<Node> && OperationNode<Node>;
template <typename Leaf>
inline constexpr bool is_leaf = VariableConcept<Leaf> && DifferentiableVariableConcept<Leaf> && !OperationNode<Leaf> &&
                                ConstArrayLike<Leaf> && op::ArrayLikeConcept<Leaf>;

template <std::size_t Out, typename Logic, typename In>
inline constexpr bool unary_ok = is_node<UnaryOperation<Out, Logic, In>> && UnaryOperation<Out, Logic, In>::size == Out &&
                                 Logic::outputDim == Out;
template <std::size_t Out, typename Logic, typename A, typename B>
inline constexpr bool binary_ok = is_node<BinaryOperation<Out, Logic, A, B>> && BinaryOperation<Out, Logic, A, B>::size == Out &&
                                  Logic::outputDim == Out;

template <std::size_t Out, typename Logic, typename A, typename B, typename C>
inline constexpr bool ternary_ok = is_node<TernaryOperation<Out, Logic, A, B, C>> &&
                                   TernaryOperation<Out, Logic, A, B, C>::size == Out && Logic::outputDim == Out;

// The library ships no three-operand logic; the contract of TernaryLogicConcept / TernaryOperation
// (concept/core_logic.cuh:44-54 and operations/operation.cuh:382-623 of the reference) is asserted with the
// smallest logic a user could write.
template <std::size_t Dim>
struct MulAddLogic {
    static constexpr std::size_t outputDim = Dim;
    template <typename Output, typename A, typename B, typename C>
    XAD_HD void forward(Output& out, const A& a, const B& b, const C& c) const {
        for (std::size_t i = 0; i < Dim; ++i) out[i] = a[i] * b[i] + c[i];
    }
    template <typename Output, typename A, typename B, typename C>
    XAD_HD void backward(const Output& out, A& a, B& b, C& c) const {
        for (std::size_t i = 0; i < Dim; ++i) {
            a.add_grad(i, out.grad(i) * b[i]);
            b.add_grad(i, out.grad(i) * a[i]);
            c.add_grad(i, out.grad(i));
        }
    }
};
struct NotALogic {
    static constexpr std::size_t outputDim = 2;
};

// Every logic over leaves of one kind (Variable or VariableRef) and one value type.
template <template <std::size_t, typename> class Leaf, typename T>
constexpr bool all_logics() {
    using L1 = Leaf<1, T>;
    using L2 = Leaf<2, T>;
    using L3 = Leaf<3, T>;
    using L4 = Leaf<4, T>;
    using L5 = Leaf<5, T>;
    using L6 = Leaf<6, T>;
    using L9 = Leaf<9, T>;
    static_assert(is_leaf<L1> && is_leaf<L2> && is_leaf<L3> && is_leaf<L4> && is_leaf<L5> && is_leaf<L9>);
    // element-wise, one operand
    static_assert(unary_ok<3, op::ExpLogic<3>, L3> && unary_ok<3, op::SinLogic<3>, L3> && unary_ok<3, op::CosLogic<3>, L3>);
    static_assert(unary_ok<2, op::SigmoidLogic<2>, L2> && unary_ok<1, op::NegLogic<1>, L1> && unary_ok<5, op::SquaredLogic<5>, L5>);
    static_assert(unary_ok<3, op::AddConstantLogic<L3>, L3> && unary_ok<3, op::SubConstantLogic<L3>, L3>);
    static_assert(unary_ok<3, op::MulConstantLogic<L3>, L3> && unary_ok<3, op::DivConstantLogic<L3>, L3>);
    // reductions
    static_assert(unary_ok<1, op::SumLogic<4>, L4> && unary_ok<1, op::L1NormLogic<3>, L3> && unary_ok<1, op::L2NormLogic<9>, L9>);
    // small matrices
    static_assert(unary_ok<3, op::SymMatrix2InvLogic<3>, L3> && unary_ok<9, op::QuaternionToRotationMatrixLogic<4>, L4>);
    static_assert(op::QuaternionToRotationMatrixLogic<4>::outputDim == 9);
    static_assert(unary_ok<4, BroadcastLogic<4>, L1>);
    // two operands
    static_assert(binary_ok<3, op::AddLogic<L3, L3>, L3, L3> && binary_ok<3, op::SubLogic<L3, L3>, L3, L3>);
    static_assert(binary_ok<3, op::MulLogic<L3, L3>, L3, L3> && binary_ok<3, op::DivLogic<L3, L3>, L3, L3>);
    static_assert(binary_ok<4, op::MatMulLogic<2, 2, 2, L4, L4>, L4, L4> && binary_ok<9, op::MatMulLogic<3, 3, 3, L9, L9>, L9, L9>);
    static_assert(binary_ok<2, op::MatMulLogic<2, 3, 1, L6, L3>, L6, L3> && binary_ok<2, op::MatMulLogic<1, 3, 2, L3, L6>, L3, L6>);
    // three operands: leaves, and nodes of the other arities as operands
    static_assert(TernaryLogicConcept<MulAddLogic<2>, L2, L2, L2, Variable<2, T>> && ternary_ok<2, MulAddLogic<2>, L2, L2, L2>);
    static_assert(TernaryLogicParameterConcept<L2, L2, L2>);
    static_assert(!TernaryLogicConcept<NotALogic, L2, L2, L2, Variable<2, T>> && !TernaryLogicConcept<op::AddLogic<L2, L2>, L2, L2, L2, Variable<2, T>>);
    static_assert(ternary_ok<2, MulAddLogic<2>, UnaryOperation<2, op::ExpLogic<2>, L2>, L2, BinaryOperation<2, op::MulLogic<L2, L2>, L2, L2>>);
    static_assert(unary_ok<2, op::NegLogic<2>, TernaryOperation<2, MulAddLogic<2>, L2, L2, L2>>);
    // splatting logics
    static_assert(binary_ok<4, op::CovarianceMatrixGenerationLogic<L2, L1>, L2, L1> && unary_ok<3, op::MatrixToCovariance3ParamLogic<L4>, L4>);
    static_assert(binary_ok<3, op::ScaleRotationToCovariance3ParamLogic<L2, L1>, L2, L1>);
    static_assert(binary_ok<1, op::MahalanobisDistanceLogic<L2, L3>, L2, L3>);
    // a node is itself a valid operand: nodes over nodes
    using Inner = UnaryOperation<3, op::ExpLogic<3>, L3>;
    static_assert(unary_ok<3, op::NegLogic<3>, Inner> && binary_ok<3, op::MulLogic<Inner, L3>, Inner, L3>);
    return true;
}

static_assert(all_logics<Variable, float>() && all_logics<Variable, double>());
static_assert(all_logics<VariableRef, float>() && all_logics<VariableRef, double>());

// The factories return nodes of the documented types.
template <typename T>
constexpr bool factories() {
    using L2 = VariableRef<2, T>;
    using L3 = Variable<3, T>;
    static_assert(is_node<decltype(op::exp(std::declval<L3&>()))> && is_node<decltype(op::sigmoid(std::declval<L2&>()))>);
    static_assert(is_node<decltype(op::add(std::declval<L3&>(), std::declval<L3&>()))>);
    static_assert(is_node<decltype(op::sym_matrix2_inv(std::declval<L3&>()))>);
    static_assert(is_node<decltype(std::declval<L3&>() * std::declval<L3&>())> && is_node<decltype(std::declval<L3&>() + T(1))>);
    static_assert(decltype(op::l2_norm(std::declval<L3&>()))::size == 1);
    return true;
}
static_assert(factories<float>() && factories<double>());

// Containers and views.
static_assert(VariableConcept<DenseMatrix<float, 3, 4>> && DifferentiableVariableConcept<DenseMatrix<float, 3, 4>> &&
              MatrixViewConcept<DenseMatrix<float, 3, 4>>);
static_assert(DenseMatrix<float, 2, 3>::rows == 2 && DenseMatrix<float, 2, 3>::cols == 3 && DenseMatrix<float, 3, 2>::rows == 3);
static_assert(VariableConcept<DiagonalMatrixView<float, 4>> && DifferentiableVariableConcept<DiagonalMatrixView<float, 4>> &&
              MatrixViewConcept<DiagonalMatrixView<float, 4>> && MatrixViewConcept<DiagonalMatrixView<double, 3>>);
using DiagView3 = DiagonalMatrixView<float, 3, VariableRef<3, float>>;
static_assert(MatrixViewConcept<DiagView3> && DiagView3::rows == 3 && DiagView3::cols == 3);
using Sym3 = SymmetricMatrixView<float, 3, Variable<6, float>>;
static_assert(VariableConcept<Sym3> && DifferentiableVariableConcept<Sym3> && MatrixViewConcept<Sym3>);
static_assert(MatrixViewConcept<SymmetricMatrixView<double, 4, Variable<10, double>>>);
static_assert(!OperationNode<DenseMatrix<float, 3, 4>> && !OperationNode<DiagView3> && !OperationNode<Sym3>);

// Plain arrays: the library's and a user's.
template <typename T, int N>
struct UserArray {
    using value_type = T;
    static constexpr std::size_t size = N;
    T values[N];
    XAD_HD constexpr T& operator[](std::size_t i) { return values[i]; }
    XAD_HD constexpr const T& operator[](std::size_t i) const { return values[i]; }
};
static_assert(ConstArrayLike<ConstArray<float, 3>> && ConstArrayLike<ConstArray<double, 5>>);
static_assert(ConstArrayLike<UserArray<float, 3>> && ConstArrayLike<UserArray<double, 5>>);
static_assert(ConstArrayLike<Variable<3, float>> && ConstArrayLike<Variable<5, double>> && ConstArrayLike<VariableRef<3, float>> &&
              ConstArrayLike<VariableRef<5, double>>);
static_assert(ConstArrayCompatible<ConstArray<float, 3>, UserArray<float, 3>> && ConstArrayCompatible<ConstArray<float, 3>, Variable<3, float>> &&
              ConstArrayCompatible<ConstArray<float, 3>, VariableRef<3, float>> && ConstArrayCompatible<Variable<3, float>, VariableRef<3, float>>);
static_assert(ConstArraySameSize<ConstArray<float, 3>, UserArray<float, 3>> && ConstArraySameSize<ConstArray<float, 3>, Variable<3, float>> &&
              ConstArraySameSize<ConstArray<float, 3>, VariableRef<3, float>>);
static_assert(!ConstArrayCompatible<ConstArray<float, 3>, ConstArray<double, 3>> && !ConstArraySameSize<ConstArray<float, 3>, ConstArray<float, 5>>);
static_assert(op::ArrayLikeConcept<Variable<3, float>> && op::ArrayLikeConcept<VariableRef<3, float>>);

// What is not a variable must not pass for one.
static_assert(!VariableConcept<int> && !VariableConcept<float*> && !DifferentiableVariableConcept<ConstArray<float, 3>>);

constexpr int kAsserted = 1;

}  // namespace xad_concepts
