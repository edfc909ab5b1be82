// Expression builder and its compiler to the launch layer's slot programs (ctamd_expr_run_f32).
#include "Expr.h"

#include <cfloat>
#include <cstring>
#include <cmath>
#include <map>
#include <set>
#include <tuple>
#include <unordered_map>

#include "Ctorch_Error.h"
#include "ctorch_amd.h"
#include "kernels.h"

using ctorch_amd_host::current_stream;

struct Expr::Node {
    int code = -1;                // CTAMD_EX_* of an operator; -1: a tensor operand
    std::shared_ptr<Node> a, b;
    float imm = 0.0f;
    Tensor tensor;                // code == -1: shares the operand's bytes, id and requires_grad
    bool row = false;             // tensor operand used as a row vector
    size_t dims = 0;              // dimensions of the value (a row vector operand: 1)
};

namespace {

constexpr ErrorPlatform kP = ErrorPlatform::kAMD;

bool is_binary(int code) { return code == CTAMD_EX_ADD || code == CTAMD_EX_SUB || code == CTAMD_EX_MUL || code == CTAMD_EX_DIV; }
bool is_scalar(int code) { return code == CTAMD_EX_ADDS || code == CTAMD_EX_MULS || code == CTAMD_EX_DIVS; }

Tensor tensor_binary(int code, const Tensor& a, const Tensor& b) {
    switch (code) {
        case CTAMD_EX_ADD: return a + b;
        case CTAMD_EX_SUB: return a - b;
        case CTAMD_EX_MUL: return a * b;
        default: return a / b;
    }
}
Tensor tensor_unary(int code, const Tensor& a) {
    switch (code) {
        case CTAMD_EX_NEG: return -a;
        case CTAMD_EX_RELU: return a.relu();
        case CTAMD_EX_SIGMOID: return a.sigmoid();
        case CTAMD_EX_TANH: return a.tanh();
        case CTAMD_EX_SIN: return a.sin();
        default: return a.cos();
    }
}
Tensor tensor_scalar(int code, const Tensor& a, float s) {
    switch (code) {
        case CTAMD_EX_ADDS: return a + s;
        case CTAMD_EX_MULS: return a * s;
        default: return a / s;
    }
}

// ---- the expression as a list of values in depth-first post-order (operands before users,
// operands in recorded order, every node once): the order whose reverse the tape walks in backward
struct Value {
    int code;        // CTAMD_EX_LOAD_FULL / LOAD_ROW for a tensor operand (a = port), else the operator
    int a, b;        // operand value indices (b = a for one-operand operators)
    float imm;
};

// ---- straight-line code in single-assignment form, with equal computations shared
struct Code {
    struct I {
        int op, a, b;
        float imm;
        int port;    // loads: input index; stores: output index
    };
    std::vector<I> code;
    std::map<std::tuple<int, int, int, uint32_t, int>, int> seen;
    // cos(-v) = cos(v) and sin(-v) = -sin(v): exact for the single-precision routines of the default
    // math mode, and what lets sin(v) and cos(-v) of one expression share their argument reduction.
    // glibc's sinf / cosf round the quadrant of -v and v differently on the boundary between two
    // quadrants, so programs for the exact mode keep the negation where the expression has it.
    bool fold_signs = false;

    int emit(int op, int a, int b, float imm = 0.0f, int port = 0) {
        if (fold_signs && (op == CTAMD_EX_COS || op == CTAMD_EX_SIN) && code[size_t(a)].op == CTAMD_EX_NEG) {
            const int v = code[size_t(a)].a;
            if (op == CTAMD_EX_COS) return emit(CTAMD_EX_COS, v, v);
            const int s = emit(CTAMD_EX_SIN, v, v);
            return emit(CTAMD_EX_NEG, s, s);
        }
        if (fold_signs && op == CTAMD_EX_NEG && code[size_t(a)].op == CTAMD_EX_NEG) return code[size_t(a)].a;
        uint32_t bits;
        std::memcpy(&bits, &imm, sizeof(bits));
        if (op == CTAMD_EX_ADD || op == CTAMD_EX_MUL) {       // commutative bit for bit: one canonical operand order
            if (a > b) std::swap(a, b);
        }
        auto key = std::make_tuple(op, a, b, bits, port);
        auto it = seen.find(key);
        if (it != seen.end()) return it->second;
        code.push_back({op, a, b, imm, port});
        seen[key] = int(code.size()) - 1;
        return int(code.size()) - 1;
    }
    void effect(int op, int a, int port) { code.push_back({op, a, a, 0.0f, port}); }
};

thread_local Expr::ProgramStats t_stats;

int slots_of(const std::vector<ctamd_expr_insn>& code) {
    int most = 0;
    for (const ctamd_expr_insn& q : code)
        if (q.op != CTAMD_EX_STORE && q.op != CTAMD_EX_STORE_ZP && q.op != CTAMD_EX_DIVCHK && q.dst + 1 > most) most = q.dst + 1;
    return most;
}

bool has_result(int op) { return op != CTAMD_EX_STORE && op != CTAMD_EX_STORE_ZP && op != CTAMD_EX_DIVCHK; }
bool is_load(int op) { return op == CTAMD_EX_LOAD_FULL || op == CTAMD_EX_LOAD_ROW; }

// Slot assignment: a value's slot is free again after its last use; a result may take the slot of
// an operand that dies in the same instruction (operands are read before the result is written).
// False when the program needs more than the launch layer's slots or instructions.
bool lower(const Code& in, std::vector<ctamd_expr_insn>& out) {
    // loads first: the kernel issues the loads at the head of a program together; values nobody
    // reads (a negation that cos(-v) = cos(v) left behind) are dropped
    Code c;
    {
        std::vector<bool> live(in.code.size(), false);
        for (size_t i = in.code.size(); i-- > 0;) {
            const Code::I& q = in.code[i];
            if (!has_result(q.op)) live[i] = true;
            if (live[i] && !is_load(q.op)) live[size_t(q.a)] = live[size_t(q.b)] = true;
        }
        std::vector<int> renumber(in.code.size(), -1);
        for (int pass = 0; pass < 2; ++pass)
            for (size_t i = 0; i < in.code.size(); ++i) {
                Code::I q = in.code[i];
                if (!live[i] || is_load(q.op) != (pass == 0)) continue;
                if (!is_load(q.op)) {
                    q.a = renumber[size_t(q.a)];
                    q.b = renumber[size_t(q.b)];
                }
                renumber[i] = int(c.code.size());
                c.code.push_back(q);
            }
    }
    const int n = int(c.code.size());
    if (n > CTAMD_EXPR_MAX_INSNS) return false;
    std::vector<int> last(size_t(n), -1);
    for (int i = 0; i < n; ++i) {
        const Code::I& q = c.code[size_t(i)];
        if (!is_load(q.op)) {
            last[size_t(q.a)] = i;
            last[size_t(q.b)] = i;
        }
    }
    std::vector<int> slot(size_t(n), -1);
    std::vector<int> free_slots;
    int next_slot = 0;
    out.clear();
    for (int i = 0; i < n; ++i) {
        const Code::I& q = c.code[size_t(i)];
        ctamd_expr_insn o;
        o.op = uint8_t(q.op);
        o.imm = q.imm;
        if (is_load(q.op)) {
            o.a = uint8_t(q.port);
            o.b = 0;
        } else {
            o.a = uint8_t(slot[size_t(q.a)]);
            o.b = uint8_t(slot[size_t(q.b)]);
            if (last[size_t(q.a)] == i) free_slots.push_back(slot[size_t(q.a)]);
            if (q.b != q.a && last[size_t(q.b)] == i) free_slots.push_back(slot[size_t(q.b)]);
        }
        if (has_result(q.op)) {
            int s;
            if (!free_slots.empty()) {
                s = free_slots.back();
                free_slots.pop_back();
            } else {
                s = next_slot++;
            }
            if (s >= CTAMD_EXPR_MAX_SLOTS) return false;
            slot[size_t(i)] = s;
            o.dst = uint8_t(s);
            if (last[size_t(i)] < 0) free_slots.push_back(s);    // never used: free at once
        } else {
            o.dst = uint8_t(q.port);
        }
        out.push_back(o);
    }
    return true;
}

struct Program : FusedPayload {
    std::vector<Value> vals;              // the last one is the result
    std::vector<bool> port_is_row;
    std::vector<size_t> shape;            // of every full value
    size_t rows = 0, cols = 0;
    std::vector<ctamd_expr_insn> forward_code;
    struct Backward {
        bool fits = false;
        bool checks = false;
        std::vector<ctamd_expr_insn> code;
        std::vector<int> out_port;        // output k is the gradient of input out_port[k]
    };
    std::map<std::tuple<unsigned, bool, bool>, Backward> backward_code;   // by (mask of wanted inputs, check_div_zero, default math mode)

    int ports() const { return int(port_is_row.size()); }

    // value v of the expression inside a program under construction (computed once)
    int need(Code& c, std::vector<int>& done, int v) const {
        if (done[size_t(v)] >= 0) return done[size_t(v)];
        const Value& q = vals[size_t(v)];
        int id;
        if (is_load(q.code)) {
            id = c.emit(q.code, 0, 0, 0.0f, q.a);
        } else {
            int a = need(c, done, q.a);
            int b = (q.b == q.a) ? a : need(c, done, q.b);
            id = c.emit(q.code, a, b, q.imm);
        }
        done[size_t(v)] = id;
        return id;
    }

    bool compile_forward() {
        Code c;
        c.fold_signs = ctamd_math_mode() == CTAMD_MATH_FAST;
        std::vector<int> done(vals.size(), -1);
        int root = need(c, done, int(vals.size()) - 1);
        c.effect(CTAMD_EX_STORE, root, 0);
        return lower(c, forward_code);
    }

    // The tape's backward over the expression (src/AutoDiff.cpp:1138-1153 order, :1216-1416
    // formulas, :1870-1907 accumulation) written out as one program: upstream gradient g = input
    // `ports()`, one output per wanted input that the walk reaches.
    void compile_backward(unsigned mask, bool check, bool fast, Backward& out) const {
        const int n = int(vals.size());
        Code c;
        c.fold_signs = fast;
        std::vector<int> done(size_t(n), -1), adj(size_t(n), -1);
        std::vector<bool> wants(size_t(n), false);
        std::set<int> checked;
        for (int v = 0; v < n; ++v) {
            const Value& q = vals[size_t(v)];
            wants[size_t(v)] = is_load(q.code) ? ((mask >> q.a) & 1u) != 0 : (wants[size_t(q.a)] || wants[size_t(q.b)]);
        }
        adj[size_t(n - 1)] = c.emit(CTAMD_EX_LOAD_FULL, 0, 0, 0.0f, ports());
        for (int v = n - 1; v >= 0; --v) {
            const Value& q = vals[size_t(v)];
            if (is_load(q.code) || adj[size_t(v)] < 0 || !wants[size_t(v)]) continue;
            const int g = adj[size_t(v)];
            const int positions = is_binary(q.code) ? 2 : 1;
            for (int pos = 0; pos < positions; ++pos) {
                const int u = pos == 0 ? q.a : q.b;
                if (!wants[size_t(u)]) continue;
                // the reference tells a node's operands apart by tensor id: in x - x and x / x both
                // visits count as the first operand
                const bool first = (pos == 0) || (q.a == q.b);
                int term = g;
                switch (q.code) {
                    case CTAMD_EX_ADD: case CTAMD_EX_ADDS: break;
                    case CTAMD_EX_SUB: term = first ? g : c.emit(CTAMD_EX_NEG, g, g); break;
                    case CTAMD_EX_MUL: term = c.emit(CTAMD_EX_MUL, need(c, done, pos == 0 ? q.b : q.a), g); break;
                    case CTAMD_EX_DIV: {
                        const int b = need(c, done, q.b);
                        if (check && checked.insert(b).second) {
                            c.effect(CTAMD_EX_DIVCHK, b, 0);
                            out.checks = true;
                        }
                        if (first) {
                            term = c.emit(CTAMD_EX_DIV, g, b);
                        } else {
                            int a = need(c, done, q.a);
                            int na = c.emit(CTAMD_EX_NEG, a, a);
                            int num = c.emit(CTAMD_EX_MUL, na, g);
                            int den = c.emit(CTAMD_EX_MUL, b, b);
                            term = c.emit(CTAMD_EX_DIV, num, den);
                        }
                        break;
                    }
                    case CTAMD_EX_NEG: term = c.emit(CTAMD_EX_NEG, g, g); break;
                    case CTAMD_EX_RELU: term = c.emit(CTAMD_EX_RELUMUL, need(c, done, q.a), g); break;
                    case CTAMD_EX_SIGMOID: {
                        int x = need(c, done, q.a);
                        int s = c.emit(CTAMD_EX_SIGMOID, x, x);
                        int om = c.emit(CTAMD_EX_RSUBS, s, s, 1.0f);
                        term = c.emit(CTAMD_EX_MUL, c.emit(CTAMD_EX_MUL, s, om), g);
                        break;
                    }
                    case CTAMD_EX_TANH: {
                        int x = need(c, done, q.a);
                        int t = c.emit(CTAMD_EX_TANH, x, x);
                        int tt = c.emit(CTAMD_EX_MUL, t, t);
                        int om = c.emit(CTAMD_EX_RSUBS, tt, tt, 1.0f);
                        term = c.emit(CTAMD_EX_MUL, om, g);
                        break;
                    }
                    case CTAMD_EX_SIN: {
                        int x = need(c, done, q.a);
                        term = c.emit(CTAMD_EX_MUL, c.emit(CTAMD_EX_COS, x, x), g);
                        break;
                    }
                    case CTAMD_EX_COS: {
                        int x = need(c, done, q.a);
                        int s = c.emit(CTAMD_EX_SIN, x, x);
                        term = c.emit(CTAMD_EX_MUL, c.emit(CTAMD_EX_NEG, s, s), g);
                        break;
                    }
                    case CTAMD_EX_MULS: term = c.emit(CTAMD_EX_MULS, g, g, q.imm); break;
                    case CTAMD_EX_DIVS: term = c.emit(CTAMD_EX_DIVS, g, g, q.imm); break;
                    default: break;
                }
                // the first contribution is the gradient, later ones are added to it in order.  The
                // sum must not be shared with an equal computation elsewhere under another order
                // of operands, but ADD is commutative bit for bit, so sharing is harmless.
                adj[size_t(u)] = adj[size_t(u)] < 0 ? term : c.emit(CTAMD_EX_ADD, adj[size_t(u)], term);
            }
        }
        out.out_port.clear();
        for (int v = 0; v < n; ++v) {
            const Value& q = vals[size_t(v)];
            if (is_load(q.code) && ((mask >> q.a) & 1u) && adj[size_t(v)] >= 0) {
                // "0 +": what the tape's zero-filled buffer does to a first contribution
                c.effect(CTAMD_EX_STORE_ZP, adj[size_t(v)], int(out.out_port.size()));
                out.out_port.push_back(q.a);
            }
        }
        out.fits = int(out.out_port.size()) <= CTAMD_EXPR_MAX_PORTS && ports() + 1 <= CTAMD_EXPR_MAX_PORTS && lower(c, out.code);
    }

    Tensor run_forward(const std::vector<const Tensor*>& inputs) const {
        Tensor r(ShapeTag{}, shape, DType::kFloat, DeviceType::kAMD, false);
        std::vector<const float*> in;
        for (const Tensor* t : inputs) in.push_back(t->fptr());
        float* out[1] = {r.fptr()};
        int rc = ctamd_expr_run_f32(forward_code.data(), int(forward_code.size()), in.data(), int(in.size()), out, 1, nullptr,
                                    rows, cols, current_stream());
        if (rc) Ctorch_Error::throwException(kP, ErrorType::KERNEL_LAUNCH, std::string("Expr::eval: ") + ctamd_last_error());
        return r;
    }

    std::vector<Tensor> backward(const std::vector<const Tensor*>& inputs, const std::vector<bool>& wanted, const Tensor& g,
                                 bool check_div_zero) override {
        unsigned mask = 0;
        for (size_t p = 0; p < wanted.size(); ++p)
            if (wanted[p]) mask |= 1u << p;
        const bool fast = ctamd_math_mode() == CTAMD_MATH_FAST;
        auto key = std::make_tuple(mask, check_div_zero, fast);
        auto it = backward_code.find(key);
        if (it == backward_code.end()) {
            Backward b;
            compile_backward(mask, check_div_zero, fast, b);
            it = backward_code.emplace(key, std::move(b)).first;
        }
        const Backward& b = it->second;
        if (!b.fits)
            Ctorch_Error::throwException(ErrorPlatform::kAutoDiff, ErrorType::UNKNOWN,
                                         "backward: the gradient program of a fused expression does not fit the device");
        if (g.sizes() != shape || !g.is_contiguous())
            Ctorch_Error::throwException(ErrorPlatform::kAutoDiff, ErrorType::DIMENSION,
                                         "backward: upstream gradient of a fused expression has another shape");
        std::vector<Tensor> grads(wanted.size());
        std::vector<const float*> in;
        for (const Tensor* t : inputs) in.push_back(t->fptr());
        in.push_back(g.fptr());
        std::vector<float*> out;
        for (int port : b.out_port) {
            grads[size_t(port)] = Tensor(ShapeTag{}, shape, DType::kFloat, DeviceType::kAMD, false);
            out.push_back(grads[size_t(port)].fptr());
        }
        if (out.empty()) return grads;
        Tensor status;
        int32_t* status_ptr = nullptr;
        const bool checks = b.checks && !ctorch_amd_host::recording();    // a recorded step cannot stop for a host read
        if (b.checks) {
            status = ctorch_amd_host::filled({}, 0.0f, DeviceType::kAMD);  // four zero bytes
            status_ptr = reinterpret_cast<int32_t*>(status.fptr());
        }
        int rc = ctamd_expr_run_f32(b.code.data(), int(b.code.size()), in.data(), int(in.size()), out.data(), int(out.size()),
                                    status_ptr, rows, cols, current_stream());
        if (rc) Ctorch_Error::throwException(kP, ErrorType::KERNEL_LAUNCH, std::string("backward (fused expression): ") + ctamd_last_error());
        if (checks) ctorch_amd_host::defer_status_check(status, "division by zero in the gradient of Div");
        return grads;
    }
};

// ---- from the node graph to a Program
struct Linearizer {
    std::unordered_map<const Expr::Node*, int> index;        // operator nodes
    std::unordered_map<size_t, int> operand_index;           // tensor operands by tensor id and use (full / row)
    std::vector<Tensor> tensors;                             // one per port
    Program* p;

    int visit(const std::shared_ptr<Expr::Node>& n) {
        if (n->code < 0) {
            const size_t key = n->tensor.id() * 2 + (n->row ? 1 : 0);
            auto it = operand_index.find(key);
            if (it != operand_index.end()) return it->second;
            const int port = int(tensors.size());
            tensors.push_back(Tensor::alias(n->tensor));
            p->port_is_row.push_back(n->row);
            p->vals.push_back({n->row ? CTAMD_EX_LOAD_ROW : CTAMD_EX_LOAD_FULL, port, port, 0.0f});
            operand_index[key] = int(p->vals.size()) - 1;
            return int(p->vals.size()) - 1;
        }
        auto it = index.find(n.get());
        if (it != index.end()) return it->second;
        const int a = visit(n->a);
        const int b = n->b ? visit(n->b) : a;
        p->vals.push_back({n->code, a, b, n->imm});
        index[n.get()] = int(p->vals.size()) - 1;
        return int(p->vals.size()) - 1;
    }
};

// operator-by-operator evaluation of the same graph (host tensors, or programs that do not fit)
Tensor eval_plain(const std::shared_ptr<Expr::Node>& n, std::unordered_map<const Expr::Node*, Tensor>& memo) {
    if (n->code < 0) return Tensor::alias(n->tensor);
    auto it = memo.find(n.get());
    if (it != memo.end()) return Tensor::alias(it->second);
    Tensor a = eval_plain(n->a, memo);
    Tensor r = is_binary(n->code) ? tensor_binary(n->code, a, eval_plain(n->b, memo))
             : is_scalar(n->code) ? tensor_scalar(n->code, a, n->imm)
                                  : tensor_unary(n->code, a);
    memo.emplace(n.get(), Tensor::alias(r));
    return r;
}

}  // namespace

Expr::Expr(const Tensor& t) : n_(std::make_shared<Node>()) {
    n_->tensor = Tensor::alias(t);
    n_->dims = t.dim();
}

namespace {
// 1-D tensors up to this size are combined at once by the Tensor operators (they are the row
// vectors of broadcast expressions); longer ones are full operands of a 1-D expression
constexpr size_t kSmallVector = 65536;
bool small_vector(const Expr::Node& n) { return n.code < 0 && n.tensor.dim() <= 1 && n.tensor.numel() <= kSmallVector; }
}  // namespace

// A 1-D tensor operand on the right of a value with more dimensions is a row vector.  Two small
// 1-D tensors, and a one-operand or float operator on one, are combined at once by the Tensor
// operators: their results are what later serves as a row vector.
Expr Expr::binary(int code, const Expr& a, const Expr& b) {
    const Node& x = *a.n_;
    const Node& y = *b.n_;
    if (small_vector(x) && small_vector(y)) return Expr(tensor_binary(code, x.tensor, y.tensor));
    auto n = std::make_shared<Node>();
    n->code = code;
    n->a = a.n_;
    n->b = b.n_;
    n->dims = x.dims;
    if (y.code < 0 && y.tensor.dim() == 1 && x.dims >= 2) {
        // its own node, so that the same tensor can also be a full operand elsewhere
        auto rown = std::make_shared<Node>();
        rown->tensor = Tensor::alias(y.tensor);
        rown->row = true;
        rown->dims = 1;
        n->b = rown;
    }
    return Expr(n);
}
Expr Expr::unary(int code, const Expr& a) {
    if (small_vector(*a.n_)) return Expr(tensor_unary(code, a.n_->tensor));
    auto n = std::make_shared<Node>();
    n->code = code;
    n->a = a.n_;
    n->dims = a.n_->dims;
    return Expr(n);
}
Expr Expr::scalar(int code, const Expr& a, float s) {
    if (code == CTAMD_EX_DIVS && std::fabs(s) < FLT_EPSILON)            // src/Tensor.cpp:919-921
        Ctorch_Error::throwException(ErrorPlatform::kGENERAL, ErrorType::TENSOR_STATE, "division by zero");
    if (small_vector(*a.n_)) return Expr(tensor_scalar(code, a.n_->tensor, s));
    auto n = std::make_shared<Node>();
    n->code = code;
    n->a = a.n_;
    n->dims = a.n_->dims;
    n->imm = s;
    return Expr(n);
}

Expr Expr::operator+(const Expr& o) const { return binary(CTAMD_EX_ADD, *this, o); }
Expr Expr::operator-(const Expr& o) const { return binary(CTAMD_EX_SUB, *this, o); }
Expr Expr::operator*(const Expr& o) const { return binary(CTAMD_EX_MUL, *this, o); }
Expr Expr::operator/(const Expr& o) const { return binary(CTAMD_EX_DIV, *this, o); }
Expr Expr::operator+(float s) const { return scalar(CTAMD_EX_ADDS, *this, s); }
Expr Expr::operator*(float s) const { return scalar(CTAMD_EX_MULS, *this, s); }
Expr Expr::operator/(float s) const { return scalar(CTAMD_EX_DIVS, *this, s); }
Expr Expr::operator-() const { return unary(CTAMD_EX_NEG, *this); }
Expr Expr::relu() const { return unary(CTAMD_EX_RELU, *this); }
Expr Expr::sigmoid() const { return unary(CTAMD_EX_SIGMOID, *this); }
Expr Expr::tanh() const { return unary(CTAMD_EX_TANH, *this); }
Expr Expr::sin() const { return unary(CTAMD_EX_SIN, *this); }
Expr Expr::cos() const { return unary(CTAMD_EX_COS, *this); }

Expr::ProgramStats Expr::last_program_stats() { return t_stats; }

Tensor Expr::eval() const {
    if (n_->code < 0) return Tensor::alias(n_->tensor);                 // a tensor is its own value
    auto program = std::make_shared<Program>();
    Linearizer lin;
    lin.p = program.get();
    lin.visit(n_);

    // shapes: every full operand has the result's shape, every row vector the last dimension's length
    bool fusable = int(lin.tensors.size()) <= CTAMD_EXPR_MAX_PORTS;
    const Tensor* first_full = nullptr;
    for (size_t k = 0; k < lin.tensors.size(); ++k) {
        const Tensor& t = lin.tensors[k];
        if (t.device() != DeviceType::kAMD || t.dtype() != DType::kFloat || !t.is_contiguous()) fusable = false;
        if (!program->port_is_row[k] && !first_full) first_full = &t;
    }
    if (!first_full) fusable = false;
    if (fusable) {
        program->shape = first_full->sizes();
        if (program->shape.empty()) fusable = false;
    }
    if (fusable) {
        program->cols = program->shape.back();
        program->rows = program->cols ? first_full->numel() / program->cols : 0;
        for (size_t k = 0; k < lin.tensors.size(); ++k) {
            const Tensor& t = lin.tensors[k];
            if (program->port_is_row[k] ? (t.numel() != program->cols || program->shape.size() < 2) : (t.sizes() != program->shape))
                Ctorch_Error::throwException(kP, ErrorType::DIMENSION, "Expr::eval: operand shapes do not match");
        }
        // a row vector only as the right operand of a two-operand operator
        for (const Value& q : program->vals)
            if (!is_load(q.code) && program->vals[size_t(q.a)].code == CTAMD_EX_LOAD_ROW) fusable = false;
        if (first_full->numel() == 0) fusable = false;
    }
    if (fusable) fusable = program->compile_forward();
    if (fusable && AutoDiffContext::current()) {
        // the gradient program for the inputs that require gradients must fit as well
        unsigned mask = 0;
        for (size_t k = 0; k < lin.tensors.size(); ++k)
            if (lin.tensors[k].requires_grad()) mask |= 1u << k;
        if (mask) {
            Program::Backward b;
            const bool fast = ctamd_math_mode() == CTAMD_MATH_FAST;
            program->compile_backward(mask, true, fast, b);
            fusable = b.fits;
            program->backward_code.emplace(std::make_tuple(mask, true, fast), std::move(b));
        }
    }
    t_stats = ProgramStats();
    if (!fusable) {
        std::unordered_map<const Node*, Tensor> memo;
        return eval_plain(n_, memo);
    }
    t_stats.forward_insns = int(program->forward_code.size());
    t_stats.forward_slots = slots_of(program->forward_code);
    for (const auto& kv : program->backward_code) {
        t_stats.backward_insns = int(kv.second.code.size());
        t_stats.backward_slots = slots_of(kv.second.code);
    }

    std::vector<const Tensor*> inputs;
    for (const Tensor& t : lin.tensors) inputs.push_back(&t);
    Tensor result = program->run_forward(inputs);
    if (AutoDiff* ctx = AutoDiffContext::current()) {
        std::vector<Tensor*> in;
        bool rg = false;
        for (Tensor& t : lin.tensors) {
            in.push_back(&t);
            rg = rg || t.requires_grad();
        }
        ctx->defer_record(result.id(), op::Fused, in, 0, program);
        result.set_requires_grad(rg);
        if (rg) ctx->commit_record(result);
    }
    return result;
}
