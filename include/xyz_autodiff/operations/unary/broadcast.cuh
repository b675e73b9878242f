#pragma once
// op::broadcast<N>(x): a length-1 variable seen as N equal elements, without
// storage of its own.  Reads of any index return x[0]; gradient added at any
// index lands directly on x[0], so the sum over the N positions needs no
// separate backward step.  Class and factory as in xyz-autodiff-cuda
// (include/xyz_autodiff/operations/unary/broadcast.cuh:10-109).
//
// Because there is nothing of its own to reset, zero_grad() clears the
// *source's* gradient, and run() seeds nothing: it is forward() + backward().

#include <cstddef>
#include <cstdint>

#include <xyz_autodiff/concept/operation_node.cuh>
#include <xyz_autodiff/concept/variable.cuh>
#include <xyz_autodiff/detail/node.cuh>

namespace xyz_autodiff::op {

template <typename Input, std::size_t OutputSize>
    requires DifferentiableVariableConcept<Input> && (Input::size == 1) && (OutputSize > 1)
class BroadcastOperator {
public:
    using value_type = typename Input::value_type;
    static constexpr std::size_t size = OutputSize;

    XAD_HD explicit BroadcastOperator(Input& input) : source_(input), pending_(0), holds_visit_(false) {}

    // ---- differentiable-variable face ------------------------------------
    XAD_INLINE const value_type& operator[](std::size_t) const { return source_[0]; }
    XAD_INLINE value_type& operator[](std::size_t) { return const_cast<value_type&>(source_[0]); }
    XAD_INLINE const value_type& grad(std::size_t) const { return source_.grad(0); }
    XAD_INLINE void add_grad(std::size_t, value_type g) { source_.add_grad(0, g); }
    XAD_INLINE void zero_grad() { source_.zero_grad(); }

    // ---- node face: only traversal, no arithmetic --------------------------
    XAD_INLINE void forward() { evaluate(); }
    XAD_INLINE void backward() {
        holds_visit_ = false;
        detail::release_operand(source_);
    }
    XAD_INLINE void backward_numerical(value_type delta = value_type(1e-5)) {
        holds_visit_ = false;
        detail::release_operand_numerical(source_, delta);
    }
    XAD_INLINE void run() {
        forward();
        backward();
    }
    XAD_INLINE void run_numerical(value_type delta = value_type(1e-5)) {
        forward();
        backward_numerical(delta);
    }

    XAD_INLINE void increment_ref_count() const { ++pending_; }
    XAD_INLINE bool decrement_ref_count_and_check() const { return pending_ != 0 && --pending_ == 0; }
    XAD_INLINE void xad_visit(bool held) {
        const bool fresh = pending_ == 0;
        if (!held) ++pending_;
        if (held || fresh) evaluate();
    }

private:
    // a second walk without a backward in between does not count again (see detail/node.cuh)
    XAD_INLINE void evaluate() {
        detail::visit_operand(source_, holds_visit_);
        holds_visit_ = true;
    }

    Input& source_;
    mutable std::uint8_t pending_;
    bool holds_visit_;
};

template <std::size_t OutputSize, typename Input>
    requires DifferentiableVariableConcept<Input> && (Input::size == 1) && (OutputSize > 1)
XAD_INLINE auto broadcast(Input& input) {
    return BroadcastOperator<Input, OutputSize>(input);
}

}  // namespace xyz_autodiff::op
