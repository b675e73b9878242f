#pragma once
// Contracts of op-logic structs: the stateless (or constant-carrying) objects
// that implement one operation's forward and backward rule
// (xyz-autodiff-cuda: include/xyz_autodiff/concept/core_logic.cuh:10-75).

#include <concepts>
#include <cstddef>
#include <type_traits>

#include "variable.cuh"

namespace xyz_autodiff {

namespace detail {
template <typename L>
concept HasOutputDim = requires {
    { L::outputDim } -> std::convertible_to<std::size_t>;
};
}  // namespace detail

// forward(out, in) fills the output values; backward(out, in) reads out.grad(i)
// and accumulates into the input with in.add_grad(i, g).
template <typename L, typename In, typename Out>
concept UnaryLogicConcept =
    VariableConcept<In> && VariableConcept<Out> && detail::HasOutputDim<L> &&
    requires(L logic, Out& out, const Out& cout, const In& cin, In& in) {
        { logic.forward(out, cin) } -> std::same_as<void>;
        { logic.backward(cout, in) } -> std::same_as<void>;
    };

template <typename L, typename In1, typename In2, typename Out>
concept BinaryLogicConcept =
    VariableConcept<In1> && VariableConcept<In2> && VariableConcept<Out> && detail::HasOutputDim<L> &&
    requires(L logic, Out& out, const Out& cout, const In1& cin1, const In2& cin2, In1& in1, In2& in2) {
        { logic.forward(out, cin1, cin2) } -> std::same_as<void>;
        { logic.backward(cout, in1, in2) } -> std::same_as<void>;
    };

template <typename L, typename In1, typename In2, typename In3, typename Out>
concept TernaryLogicConcept =
    VariableConcept<In1> && VariableConcept<In2> && VariableConcept<In3> && VariableConcept<Out> &&
    detail::HasOutputDim<L> &&
    requires(L logic, Out& out, const Out& cout, const In1& cin1, const In2& cin2, const In3& cin3,
             In1& in1, In2& in2, In3& in3) {
        { logic.forward(out, cin1, cin2, cin3) } -> std::same_as<void>;
        { logic.backward(cout, in1, in2, in3) } -> std::same_as<void>;
    };

// What a factory accepts as operands: differentiable, and of one scalar type.
template <typename In>
concept UnaryLogicParameterConcept = DifferentiableVariableConcept<In>;

template <typename In1, typename In2>
concept BinaryLogicParameterConcept =
    DifferentiableVariableConcept<In1> && DifferentiableVariableConcept<In2> &&
    std::is_same_v<typename In1::value_type, typename In2::value_type>;

template <typename In1, typename In2, typename In3>
concept TernaryLogicParameterConcept =
    BinaryLogicParameterConcept<In1, In2> && DifferentiableVariableConcept<In3> &&
    std::is_same_v<typename In1::value_type, typename In3::value_type>;

}  // namespace xyz_autodiff
