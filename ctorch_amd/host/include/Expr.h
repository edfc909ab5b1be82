// Fused elementwise expressions (not in the reference, which runs and tapes one kernel per
// operator): an expression over tensors is built with the same operators the Tensor class has and
// evaluated by eval() in ONE pass over memory; the tape records it as ONE operator whose gradients
// for all inputs come from one more pass.
//
//     Expr x(X), r(rv);                                   // X [rows, cols], rv a row vector [cols]
//     Tensor Y = (sigmoid(x / r) - tanh(x) * sin(x) + cos(-x)).eval();
//
// Values and gradients are those of the operator-by-operator form bit for bit: every operator is
// computed by the same per-element code, gradient contributions are formed by the reference's
// formulas (src/AutoDiff.cpp:1216-1416) and added in the order in which the reference's tape would
// add them (reversed depth-first post-order from the result, operands in recorded order).  The
// tape receives ONE gradient per input from the expression: an input that other taped operators use
// as well gets the same contributions, but the expression's share arrives as one sum.
//
// Operands: tensors of one common shape ("full"), and 1-D row vectors of the last dimension's
// length as the right operand of + - * / with a full left operand.  Operators between two row
// vectors, and the unary and float operators on a row vector, are evaluated at once with the
// Tensor operators (they are tiny).  On the host, or when the expression or its gradient program
// does not fit the device program (160 instructions, 32 value slots, 8 tensors, the upstream
// gradient counting as one), eval() evaluates operator by operator.
#ifndef EXPR_H
#define EXPR_H

#include <memory>
#include <vector>

#include "AutoDiff.h"
#include "Tensor.h"

class Expr {
   public:
    struct Node;
    Expr(const Tensor& t);   // NOLINT: a tensor is an expression

    Expr operator+(const Expr& o) const;
    Expr operator-(const Expr& o) const;
    Expr operator*(const Expr& o) const;
    Expr operator/(const Expr& o) const;
    Expr operator+(float s) const;
    Expr operator*(float s) const;
    Expr operator/(float s) const;
    Expr operator-() const;
    Expr relu() const;
    Expr sigmoid() const;
    Expr tanh() const;
    Expr sin() const;
    Expr cos() const;

    // The value as a tensor; taped as one operator when an autograd context is active.
    Tensor eval() const;

    // Size of the device programs compiled last on this thread, for tests and tuning:
    // {forward instructions, forward slots, backward instructions, backward slots}; zeros when the
    // last eval() ran operator by operator.
    struct ProgramStats {
        int forward_insns = 0, forward_slots = 0, backward_insns = 0, backward_slots = 0;
    };
    static ProgramStats last_program_stats();

   private:
    explicit Expr(std::shared_ptr<Node> n) : n_(std::move(n)) {}
    static Expr binary(int code, const Expr& a, const Expr& b);
    static Expr unary(int code, const Expr& a);
    static Expr scalar(int code, const Expr& a, float s);
    std::shared_ptr<Node> n_;
};

inline Expr relu(const Expr& e) { return e.relu(); }
inline Expr sigmoid(const Expr& e) { return e.sigmoid(); }
inline Expr tanh(const Expr& e) { return e.tanh(); }
inline Expr sin(const Expr& e) { return e.sin(); }
inline Expr cos(const Expr& e) { return e.cos(); }

// What the tape keeps for a fused operator, and the call it makes in backward: gradients of the
// inputs in `wanted` (one per input, empty where not wanted or not reached) from the upstream
// gradient g, one launch.  check_div_zero: throw if a divisor has an element below FLT_EPSILON, as
// the tape's Div gradient does.
struct FusedPayload : AutoDiff::OpPayload {
    virtual std::vector<Tensor> backward(const std::vector<const Tensor*>& inputs, const std::vector<bool>& wanted,
                                         const Tensor& g, bool check_div_zero) = 0;
};

#endif
