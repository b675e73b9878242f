#pragma once
// Contract of an interior node of a graph
// (xyz-autodiff-cuda: include/xyz_autodiff/concept/operation_node.cuh:10-26).

#include <concepts>
#include <cstddef>

namespace xyz_autodiff {

// Anything that can evaluate itself, reset its own gradient and push its
// gradient on to its inputs, analytically or by central differences.
template <typename N>
concept OperationNode =
    requires { typename N::value_type; } &&
    requires(N n, typename N::value_type delta) {
        { N::size } -> std::convertible_to<std::size_t>;
        { n.forward() } -> std::same_as<void>;
        { n.zero_grad() } -> std::same_as<void>;
        { n.backward() } -> std::same_as<void>;
        { n.backward_numerical(delta) } -> std::same_as<void>;
    };

}  // namespace xyz_autodiff
