#pragma once
// Interior nodes of a per-thread graph: one operation, its operands by
// reference, its output by value.
//
// Class names, template parameter order <OutputSize, Logic, Inputs...>, the
// (const Logic&, Input&...) constructor, member names and typedefs are those of
// xyz-autodiff-cuda (include/xyz_autodiff/operations/operation.cuh:14-174
// UnaryOperation, :177-379 BinaryOperation, :382-623 TernaryOperation), so op
// logic and kernels written against it build unchanged.  The traversal itself
// is different: see detail/node.cuh for how shared sub-graphs are evaluated
// once and differentiated correctly.
//
// Operands are held by reference: they must be named objects that outlive the
// node.  Nodes can be moved but not copied.

#include <cstddef>

#include <xyz_autodiff/concept/core_logic.cuh>
#include <xyz_autodiff/concept/operation_node.cuh>
#include <xyz_autodiff/concept/variable.cuh>
#include <xyz_autodiff/detail/node.cuh>
#include <xyz_autodiff/variable.cuh>

namespace xyz_autodiff {

template <std::size_t OutputSize, typename Logic, typename Input>
    requires UnaryLogicConcept<Logic, Input, Variable<OutputSize, typename Input::value_type>>
class UnaryOperation : public detail::Node<OutputSize, Logic, Input> {
    using Base = detail::Node<OutputSize, Logic, Input>;

public:
    using input_type = Input;
    using Base::Base;
    XAD_HD UnaryOperation(UnaryOperation&&) noexcept = default;
};

template <std::size_t OutputSize, typename Logic, typename Input1, typename Input2>
    requires BinaryLogicConcept<Logic, Input1, Input2, Variable<OutputSize, typename Input1::value_type>>
class BinaryOperation : public detail::Node<OutputSize, Logic, Input1, Input2> {
    using Base = detail::Node<OutputSize, Logic, Input1, Input2>;

public:
    using input1_type = Input1;
    using input2_type = Input2;
    using Base::Base;
    XAD_HD BinaryOperation(BinaryOperation&&) noexcept = default;
};

template <std::size_t OutputSize, typename Logic, typename Input1, typename Input2, typename Input3>
    requires TernaryLogicConcept<Logic, Input1, Input2, Input3,
                                 Variable<OutputSize, typename Input1::value_type>>
class TernaryOperation : public detail::Node<OutputSize, Logic, Input1, Input2, Input3> {
    using Base = detail::Node<OutputSize, Logic, Input1, Input2, Input3>;

public:
    using input1_type = Input1;
    using input2_type = Input2;
    using input3_type = Input3;
    using Base::Base;
    XAD_HD TernaryOperation(TernaryOperation&&) noexcept = default;
};

}  // namespace xyz_autodiff
