#pragma once
// Shared machinery of graph nodes.
//
// A graph is a nest of node objects that live in the registers of one lane.
// Every node holds references to its operands, its own output Variable and a
// one-byte count of consumers that still owe it a gradient.  The traversal
// protocol below is what makes a node that feeds several consumers work:
//
//   forward   A consumer *visits* each operand.  The first visit of a pass
//             evaluates the operand (which in turn visits its own operands);
//             later visits only register one more consumer.  A shared
//             sub-graph is therefore evaluated once, and every edge of the
//             graph is counted exactly once.
//   backward  After a consumer has added its contribution, it releases each
//             operand; the release that brings the count to zero runs the
//             operand's own backward.  Nodes fire in reverse topological
//             order, each exactly once, with their gradient complete.
//
// Several roots may share a sub-graph: forward each root, seed each, backward
// each; the shared nodes fire when the last root has released them, as with the
// counts of xyz-autodiff-cuda (operation.cuh:53-83).  A shared node keeps the
// value of its first evaluation until it has fired, so operands must not change
// between the forward passes of two such roots.
//
// A forward() that no backward() follows leaves visits registered.  Every node
// remembers that it holds a visit on each of its operands, and its next
// evaluation walks them again without registering a second one: the operands
// are evaluated afresh (a forward() always recomputes what lies below it), the
// counts stay what they were, so forward(); forward(); backward() works and
// never disturbs the visits of another root.  There is no separate pass that
// takes visits back: one walk, one call per edge, nothing recursive besides it.
//
// All counts are compile-time constants once the graph is inlined, so none of
// this survives into the ISA: it only decides which calls are emitted.
//
// Nodes written by users against the three-call protocol of xyz-autodiff-cuda
// (forward(); increment_ref_count(); ... decrement_ref_count_and_check(),
// include/xyz_autodiff/operations/operation.cuh:53-83) keep working as
// operands and as consumers of the nodes defined here.

#include <cstddef>
#include <cstdint>
#include <utility>

#include <xyz_autodiff/concept/operation_node.cuh>
#include <xyz_autodiff/concept/variable.cuh>
#include <xyz_autodiff/detail/config.cuh>
#include <xyz_autodiff/variable.cuh>

namespace xyz_autodiff {
namespace detail {

template <typename X>
concept HasVisitProtocol = requires(X x, bool held) { x.xad_visit(held); };

// A consumer reaches one operand during its evaluation.  `held` says that the
// consumer still holds the visit of an earlier evaluation that no backward
// followed: the operand is then evaluated again and not counted again.
template <typename X>
XAD_INLINE void visit_operand(X& x, bool held) {
    if constexpr (HasVisitProtocol<X>) {
        x.xad_visit(held);
    } else if constexpr (OperationNode<X>) {
        x.forward();
        if (!held) x.increment_ref_count();
    }
}

template <typename X>
XAD_INLINE void release_operand(X& x) {
    if constexpr (OperationNode<X>) {
        if (x.decrement_ref_count_and_check()) x.backward();
    }
}

template <typename X, typename T>
XAD_INLINE void release_operand_numerical(X& x, T delta) {
    if constexpr (OperationNode<X>) {
        if (x.decrement_ref_count_and_check()) x.backward_numerical(delta);
    }
}

// References to one, two or three operands.  Written out per arity rather than
// recursively so that the optimiser sees plain reference members.
template <typename... Ins>
struct Operands;

template <typename A>
struct Operands<A> {
    A& a;
    template <typename F>
    XAD_INLINE void each(F&& f) const { f(a); }
    template <typename F>
    XAD_INLINE void all(F&& f) const { f(a); }
};

template <typename A, typename B>
struct Operands<A, B> {
    A& a;
    B& b;
    template <typename F>
    XAD_INLINE void each(F&& f) const { f(a); f(b); }
    template <typename F>
    XAD_INLINE void all(F&& f) const { f(a, b); }
};

template <typename A, typename B, typename C>
struct Operands<A, B, C> {
    A& a;
    B& b;
    C& c;
    template <typename F>
    XAD_INLINE void each(F&& f) const { f(a); f(b); f(c); }
    template <typename F>
    XAD_INLINE void all(F&& f) const { f(a, b, c); }
};

template <typename First, typename...>
struct first_of { using type = First; };

// State and behaviour common to nodes of every arity.
template <std::size_t OutputSize, typename Logic, typename... Ins>
class Node {
public:
    using value_type = typename first_of<Ins...>::type::value_type;
    using output_type = Variable<OutputSize, value_type>;
    static constexpr std::size_t output_size = OutputSize;
    static constexpr std::size_t size = OutputSize;

    Node() = delete;
    Node(const Node&) = delete;
    Node& operator=(const Node&) = delete;
    Node& operator=(Node&&) = delete;

    // A moved node starts with no registered consumers.
    XAD_HD Node(Node&& other) noexcept
        : logic_(other.logic_), in_(other.in_), out_(other.out_), pending_(0), holds_visits_(false) {}

    // Construction records the operands; nothing is evaluated until forward().
    XAD_HD Node(const Logic& logic, Ins&... ins)
        : logic_(logic), in_{ins...}, out_(), pending_(0), holds_visits_(false) {}

    // ---- evaluation -------------------------------------------------------

    // Evaluates the whole sub-graph below this node, each node once.
    XAD_INLINE void forward() { evaluate(); }

    // Propagates this node's gradient to its operands and fires every operand
    // whose last consumer this was.
    XAD_INLINE void backward() {
        const output_type& out = out_;
        in_.all([&](auto&... xs) { logic_.backward(out, xs...); });
        holds_visits_ = false;
        in_.each([](auto& x) { release_operand(x); });
    }

    // Same traversal, with the local Jacobian of every node estimated by
    // central differences of its own forward rule.  The operand elements are
    // perturbed in place and restored, so operands that view shared memory
    // must not be touched by other threads meanwhile; an operand object that
    // is passed twice to one node is perturbed (and credited) once per slot.
    XAD_INLINE void backward_numerical(const value_type delta = value_type(1e-5)) {
        in_.each([&](auto& x) { this->perturb(x, delta); });
        holds_visits_ = false;
        in_.each([&](auto& x) { release_operand_numerical(x, delta); });
    }

    // forward, seed every output gradient with one, backward.
    XAD_INLINE void run() {
        forward();
        seed();
        backward();
    }

    XAD_INLINE void run_numerical(const value_type delta = value_type(1e-5)) {
        forward();
        seed();
        backward_numerical(delta);
    }

    // ---- consumer bookkeeping --------------------------------------------

    XAD_INLINE void increment_ref_count() { ++pending_; }
    // A release without a matching visit is ignored rather than wrapping the count.
    XAD_INLINE bool decrement_ref_count_and_check() { return pending_ != 0 && --pending_ == 0; }

    // The first visit of a pass evaluates the node, later ones only count; a
    // consumer that walks its operands a second time evaluates without counting.
    XAD_INLINE void xad_visit(bool held) {
        const bool fresh = pending_ == 0;
        if (!held) ++pending_;
        if (held || fresh) evaluate();
    }

    // ---- the node as a differentiable variable ---------------------------

    XAD_INLINE output_type& output() { return out_; }
    XAD_INLINE const output_type& output() const { return out_; }

    XAD_INLINE value_type& operator[](std::size_t i) { return out_[i]; }
    XAD_INLINE const value_type& operator[](std::size_t i) const { return out_[i]; }
    XAD_INLINE const value_type& grad(std::size_t i) const { return out_.grad(i); }
    XAD_INLINE void add_grad(std::size_t i, value_type g) { out_.add_grad(i, g); }
    XAD_INLINE void zero_grad() { out_.zero_grad(); }

    XAD_INLINE value_type* data() { return out_.data(); }
    XAD_INLINE const value_type* data() const { return out_.data(); }
    XAD_INLINE value_type* grad() { return out_.grad(); }
    XAD_INLINE const value_type* grad() const { return out_.grad(); }

private:
    // Operands first, then this node.  The node's gradient restarts from zero
    // with every evaluation, so a graph object can be run any number of times.
    XAD_INLINE void evaluate() {
        const bool held = holds_visits_;
        in_.each([held](auto& x) { visit_operand(x, held); });
        holds_visits_ = true;
        out_.zero_grad();
        in_.all([&](const auto&... xs) { logic_.forward(out_, xs...); });
    }

    XAD_INLINE void seed() {
        out_.zero_grad();
        XAD_UNROLL
        for (std::size_t j = 0; j < OutputSize; ++j) out_.add_grad(j, value_type(1));
    }

    template <typename X>
    XAD_INLINE void perturb(X& x, const value_type delta) {
        const value_type step = value_type(2) * delta;
        XAD_UNROLL
        for (std::size_t i = 0; i < X::size; ++i) {
            const value_type centre = x[i];
            output_type hi, lo;
            x[i] = centre + delta;
            in_.all([&](const auto&... xs) { logic_.forward(hi, xs...); });
            x[i] = centre - delta;
            in_.all([&](const auto&... xs) { logic_.forward(lo, xs...); });
            x[i] = centre;
            XAD_UNROLL
            for (std::size_t j = 0; j < OutputSize; ++j) {
                x.add_grad(i, out_.grad(j) * ((hi[j] - lo[j]) / step));
            }
        }
    }

    Logic logic_;
    Operands<Ins...> in_;
    output_type out_;
    std::uint8_t pending_;
    bool holds_visits_;  // one visit registered with every operand and not yet released
};

}  // namespace detail
}  // namespace xyz_autodiff
