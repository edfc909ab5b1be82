// Tape and backward pass.  The per-operator gradient arithmetic follows the reference's
// AutoDiff::backward (src/AutoDiff.cpp:1216-1862) branch by branch; see AutoDiff.h for the
// deliberate differences.
#include "AutoDiff.h"

#include <cfloat>
#include <cmath>
#include <cstring>

#include <algorithm>

#include "Ctorch_Scheduler.h"
#include "Expr.h"
#include "kernels.h"
#include "ctorch_amd.h"

using namespace ctorch_amd_host;

AutoDiff::Node* AutoDiff::find(size_t id) {
    auto it = id_to_node.find(id);
    return (it == id_to_node.end() || !it->second) ? nullptr : it->second.get();
}

bool AutoDiff::is_relu_layer_output(const Tensor& t) {
    if (t.id() == 0) return false;
    std::lock_guard<std::mutex> lock(records_mutex);
    Node* n = find(t.id());
    return n && !n->is_leaf && n->operation == op::Linear && n->op_param_i != 0;
}

size_t AutoDiff::node_count() {
    std::lock_guard<std::mutex> lock(records_mutex);
    return id_to_node.size();
}

// src/AutoDiff.cpp:246-311
void AutoDiff::make_leaf(Tensor& t, bool requires_grad) {
    if (t.id() == 0) return;
    std::lock_guard<std::mutex> lock(records_mutex);
    Node* n = find(t.id());
    if (n) {
        n->requires_grad = n->requires_grad || requires_grad;
        return;
    }
    auto node = std::make_unique<Node>();
    node->tensor_id = t.id();
    if (leaf_values_ == LeafValues::kReferenceFirstSeen) {
        node->tensor = std::make_unique<Tensor>(t);      // deep copy, kept for the tape's lifetime
        node->tensor->set_id(t.id());
    } else {
        node->tensor = std::make_unique<Tensor>(Tensor::alias(t));
    }
    node->requires_grad = requires_grad;
    node->is_leaf = true;
    id_to_node[t.id()] = std::move(node);
}

// src/AutoDiff.cpp:513-546
void AutoDiff::update_requires_grad(Tensor& t, bool requires_grad) {
    if (t.id() == 0) return;
    std::lock_guard<std::mutex> lock(records_mutex);
    if (Node* n = find(t.id())) n->requires_grad = requires_grad;
}

// src/AutoDiff.cpp:502-510
void AutoDiff::zero_grad(Tensor& t) {
    if (t.id() == 0) return;
    std::lock_guard<std::mutex> lock(records_mutex);
    Node* n = find(t.id());
    // no gradient stored reads as zeros (get_grad) and the next contribution becomes the gradient
    // with its "0 +" pending: the same values as a zero-filled buffer, without the fill
    if (n) {
        n->grad.reset();
        n->grad_plus_zero = false;
        n->grad_assigned = false;
        n->grad_premasked_by = nullptr;
        n->unmasked_grad.reset();
        // A layer below whose gradient this node's backward left at the pre-activation: the gradient of
        // that layer's output could only be formed from the gradient just dropped, so it goes as well
        // (what is left would otherwise be read as the output's gradient by a later pass).
        for (auto it = premasked_.begin(); it != premasked_.end();) {
            Node* below = *it;
            if (below->grad_premasked_by == n) {
                below->grad.reset();
                below->grad_plus_zero = false;
                below->grad_premasked_by = nullptr;
                below->unmasked_grad.reset();
                it = premasked_.erase(it);
            } else {
                ++it;
            }
        }
        premasked_.erase(n);
    }
}

// Not in the reference: the gradient's bytes as the tape holds them (shared, not copied; empty when
// there is none).  Where get_grad has +0 these bytes may hold -0: the "0 +" of the reference's
// zero-filled accumulation buffer is left to the reader.
Tensor AutoDiff::stored_grad(const Tensor& t) {
    if (t.id() == 0) return Tensor();
    std::lock_guard<std::mutex> lock(records_mutex);
    Node* n = find(t.id());
    if (n && n->requires_grad && n->grad && n->grad->sizes() == t.sizes() && !n->grad_premasked_by) return Tensor::alias(*n->grad);
    return Tensor();
}

// src/AutoDiff.cpp:86-243: a copy of the stored gradient, or zeros of the tensor's shape
Tensor AutoDiff::get_grad(const Tensor* t) {
    if (!t || t->id() == 0) return Tensor();
    std::lock_guard<std::mutex> lock(records_mutex);
    Node* n = find(t->id());
    if (n && n->requires_grad && n->grad && n->grad_premasked_by) {
        // the tape holds this layer's gradient at the pre-activation; the gradient of the output is
        // the consumer's product without the mask, formed now
        Node* by = n->grad_premasked_by;
        if (!by->grad) return Tensor(ShapeTag{}, t->shape(), t->dtype(), t->device());
        if (!n->unmasked_grad) {                        // one product, kept for the next reader
            AutoDiffContext::Guard guard(nullptr);      // nothing below is taped
            n->unmasked_grad = std::make_unique<Tensor>(input_gradient(by, n->tensor_id, 0, *by->grad));
            by->shared_term.reset();
        }
        return Tensor::share(*n->unmasked_grad);        // sums of products from +0: no "0 +" pending
    }
    if (n && n->requires_grad && n->grad) {
        // the pending "0 +" (one pass, once); a gradient known to hold no -0 needs none.  The
        // result shares the tape's bytes instead of copying them: the tape never writes through
        // shared bytes (a later contribution goes to a fresh tensor), callers must not either.
        if (!n->grad_plus_zero && !n->grad_assigned) {
            n->grad = std::make_unique<Tensor>(zero_plus(*n->grad, n->grad->sizes()));
            n->grad_plus_zero = true;
        }
        return Tensor::share(*n->grad);
    }
    return Tensor(ShapeTag{}, t->shape(), t->dtype(), t->device());
}

// src/AutoDiff.cpp:314-370: inputs not yet on the tape become leaves; the op is parked until the
// output is known to require a gradient
void AutoDiff::defer_record(size_t output_id, op operation, const std::vector<Tensor*>& inputs, int op_param_i,
                            std::shared_ptr<OpPayload> payload) {
    Pending p{operation, {}, op_param_i, std::move(payload)};
    for (Tensor* in : inputs) {
        if (!in || in->id() == 0) continue;
        make_leaf(*in, in->requires_grad());
        p.input_ids.push_back(in->id());
    }
    std::lock_guard<std::mutex> lock(records_mutex);
    pending_[output_id] = std::move(p);
}

// src/AutoDiff.cpp:373-499
void AutoDiff::commit_record(Tensor& output) {
    std::lock_guard<std::mutex> lock(records_mutex);
    auto it = pending_.find(output.id());
    if (it == pending_.end()) return;
    auto node = std::make_unique<Node>();
    node->tensor_id = output.id();
    node->operation = it->second.operation;
    node->op_param_i = it->second.op_param_i;
    node->payload = std::move(it->second.payload);
    node->input_ids = std::move(it->second.input_ids);
    node->tensor = std::make_unique<Tensor>(Tensor::alias(output));
    node->requires_grad = true;
    node->is_leaf = false;
    pending_.erase(it);
    id_to_node[output.id()] = std::move(node);
}

void AutoDiff::clear_graph() {
    std::lock_guard<std::mutex> lock(records_mutex);
    premasked_.clear();
    id_to_node.clear();
    pending_.clear();
}

// src/AutoDiff.cpp:562-1049, every branch.  In the reference's mode the results are the reference's
// bit for bit (the oracle's co_adjust_grad_shape restates the function and is pinned against it);
// by default the broadcast branch is the mathematics instead: the sum over the dimensions along
// which the operand was broadcast (the reference takes the slice with leading index 0).
Tensor AutoDiff::adjust_grad_shape(const Tensor& grad, const std::vector<size_t>& target) {
    // The equal / 0-D / reshape branches hand the gradient's values on as they are; the broadcast
    // branch adds them to a zero-filled result (`result[i] += g[..]`, :755), which turns -0 into +0.
    // The values returned here are the raw ones; the flag tells a caller that stores them as a
    // root's gradient (which nothing is added to afterwards) that the "0 +" is still due.
    adjust_adds_to_zero_ = false;
    if (grad.sizes() == target) return Tensor::alias(grad);                           // :565-567
    if (grad.sizes().empty()) return filled_from(target, grad);                       // :579-627
    if (grad.dim() < target.size()) {
        // :633-687: the gradient copied into shape [1, .., 1, its dims] (element i from element
        // i % numel, the same count: a reshape), then the function again
        const size_t gr = grad.dim(), tr = target.size();
        std::vector<size_t> padded(tr, 1);
        for (size_t i = 0; i < gr; ++i) padded[tr - gr + i] = grad.sizes()[i];
        return adjust_grad_shape(Tensor::view_shape(grad, padded), target);
    }
    adjust_adds_to_zero_ = true;
    if (grad.dim() == 2 && target.size() == 1 && grad.sizes()[1] == target[0]) {      // :690-757, the bias of a layer
        if (broadcast_grad_ == BroadcastGrad::kColumnSum) {
            term_plus_zero_ = true;                  // a sum that starts from +0 is never -0
            return column_sum(grad);
        }
        return first_row(grad);
    }
    if (target.empty() || (target.size() == 1 && target[0] == 1)) {
        // gradient of a one-element operand that was broadcast over a whole tensor
        Tensor flat = Tensor::alias(grad);
        if (broadcast_grad_ == BroadcastGrad::kColumnSum) {
            Tensor s = sum_all(flat);
            term_plus_zero_ = true;
            return target.empty() ? s : filled_from(target, s);
        }
        Tensor first(ShapeTag{}, target, DType::kFloat, grad.device(), false);
        device_copy_d2d(first.fptr(), grad.fptr(), sizeof(float));
        return first;
    }
    const size_t gr = grad.dim(), tr = target.size();
    bool can_broadcast = true;                                                        // :690-704
    for (size_t i = 1; i <= tr; ++i) {
        const size_t gd = grad.sizes()[gr - i], td = target[tr - i];
        if (gd != td && gd != 1 && td != 1) can_broadcast = false;
    }
    if (!can_broadcast) {
        // :968-1046 (the "can reduce" branch before it, :892-966, cannot be reached: its condition
        // implies the broadcast one): result[i] = g[i] + g[i + n] + ..., in that order from 0
        term_plus_zero_ = false;
        return fold_mod(grad, target);
    }
    size_t tn = 1;
    for (size_t e : target) tn *= e;
    if (broadcast_grad_ == BroadcastGrad::kReferenceRow0) {
        // :706-757: the coordinate loop starts at the LAST dimension with the whole flat index, so
        // result[i] = 0 + g[i] (g[0] when the gradient's last dimension is 1); beyond the gradient's
        // end the reference reads whatever follows its buffer
        if (grad.sizes().back() == 1) return filled_from(target, Tensor::view_element(grad, 0));
        if (tn > grad.numel())
            Ctorch_Error::throwException(ErrorPlatform::kAutoDiff, ErrorType::DIMENSION,
                                         "backward: the reference reads beyond the end of this gradient when it adjusts its shape");
        return leading_elements(grad, target);
    }
    std::vector<size_t> padded(gr, 1);
    for (size_t i = 0; i < tr; ++i) padded[gr - tr + i] = target[i];
    term_plus_zero_ = true;                          // sums (in double, from +0) and their copies
    // leading dimensions summed away and the rest kept whole: a column sum of [rows, cols]
    size_t lead = 0;
    while (lead < gr && padded[lead] == 1) ++lead;
    bool rest_kept = true;
    for (size_t d = lead; d < gr; ++d) rest_kept = rest_kept && padded[d] == grad.sizes()[d];
    if (rest_kept && lead > 0 && grad.is_contiguous()) {
        size_t rows = 1;
        for (size_t d = 0; d < lead; ++d) rows *= grad.sizes()[d];
        if (rows == 1) {
            term_plus_zero_ = false;                 // the values themselves, -0 included
            return Tensor::view_shape(grad, target);
        }
        Tensor sums = column_sum(Tensor::view_shape(grad, {rows, tn}));
        return Tensor::view_shape(sums, target);
    }
    return broadcast_reduce(grad, grad.sizes(), padded, target);
}

namespace {
bool is_row_vector_of(const Tensor& v, const Tensor& m) {
    return v.dim() == 1 && m.dim() == 2 && v.sizes()[0] == m.sizes()[1];
}
}  // namespace

Tensor AutoDiff::input_gradient(Node* node, size_t input_id, size_t input_pos, const Tensor& g) {
    Node* in = find(input_id);
    const Tensor& x = *in->tensor;
    const bool first = (input_id == node->input_ids[0]);   // the reference tells operands apart by id
    // does the term hold no -0?  (then "0 + term" is the term and reading it needs no pass)
    term_plus_zero_ = false;
    const bool upstream_plus_zero = node->grad_plus_zero;
    auto other_node = [&]() -> Node* {
        if (node->input_ids.size() < 2) return nullptr;
        return find(first ? node->input_ids[1] : node->input_ids[0]);
    };
    switch (node->operation) {
        case op::Add:                                                   // :1216-1221
            term_plus_zero_ = upstream_plus_zero;
            return adjust_grad_shape(g, x.sizes());
        case op::Sub: {                                                 // :1222-1233
            term_plus_zero_ = upstream_plus_zero;
            Tensor adj = adjust_grad_shape(g, x.sizes());
            if (first) return adj;
            term_plus_zero_ = false;                                    // -(+0) = -0
            return Neg_AMD_kernel(adj);
        }
        case op::Mul: {                                                 // :1234-1258: other * g
            Node* o = other_node();
            if (!o) return Tensor::alias(g);
            const Tensor& other = *o->tensor;
            if (other.device() == DeviceType::kCPU && other.numel() == 1)       // tensor * float: s * g
                return scalar_op(g, other.item<float>(), op::Mul);
            if (is_row_vector_of(other, g)) return Mul_AMD_kernel(g, other);   // row-broadcast operand
            return Mul_AMD_kernel(other, g);
        }
        case op::Div: {                                                 // :1259-1316
            Node* a_node = find(node->input_ids[0]);
            Node* b_node = find(node->input_ids[1]);
            const Tensor& a = *a_node->tensor;
            const Tensor& b = *b_node->tensor;
            if (b.device() == DeviceType::kCPU && b.numel() == 1) {             // tensor / float
                const float sv = b.item<float>();
                if (check_div_zero_ && std::fabs(sv) < FLT_EPSILON)
                    Ctorch_Error::throwException(ErrorPlatform::kGENERAL, ErrorType::TENSOR_STATE,
                                                 "division by zero in the gradient of Div");
                if (first) return scalar_op(g, sv, op::Div);                    // g / s
                Ctorch_Error::throwException(ErrorPlatform::kAutoDiff, ErrorType::TENSOR_STATE,
                                             "backward: a host scalar operand has no gradient");
            }
            if (check_div_zero_ && any_abs_lt_eps(b))
                Ctorch_Error::throwException(ErrorPlatform::kGENERAL, ErrorType::TENSOR_STATE,
                                             "division by zero in the gradient of Div");
            if (first) return Div_AMD_kernel(g, b);                     // g / b
            if (a.sizes() == b.sizes() && g.sizes() == a.sizes()) return div_backward_b(a, b, g);
            if (is_row_vector_of(b, a) && g.sizes() == a.sizes()) return div_backward_b(a, b, g);   // same order, one pass
            // any other broadcast divisor: ((-a) * g) / (b * b) with the same operation order, op by op
            Tensor na = Neg_AMD_kernel(a);
            Tensor num = Mul_AMD_kernel(na, g);
            Tensor den = Mul_AMD_kernel(b, b);
            return Div_AMD_kernel(num, den);
        }
        case op::Neg: return Neg_AMD_kernel(g);                         // :1317-1319
        case op::ReLU: return relu_backward(x, g);                      // :1320-1371
        case op::Sigmoid: return sigmoid_backward(x, g);                // :1372-1383
        case op::Tanh: return tanh_backward(x, g);                      // :1384-1398
        case op::Sin: return sin_backward(x, g);                        // :1399-1407
        case op::Cos: return cos_backward(x, g);                        // :1408-1416
        case op::Softmax: return softmax_backward(*node->tensor, g, node->op_param_i);   // :1417-1490
        // the loss, MatMul and fused-expression gradients below come out of their kernels with the
        // "0 +" applied or as sums that start from +0
        case op::MSE: {                                                 // :1491-1516
            Node* o = other_node();
            term_plus_zero_ = true;
            return mse_backward(x, *o->tensor, g);
        }
        case op::MAE: {                                                 // :1602-1642
            Node* o = other_node();
            term_plus_zero_ = true;
            return mae_backward(x, *o->tensor, g);
        }
        case op::CE: {                                                  // :1517-1601
            Node* o = other_node();
            term_plus_zero_ = true;
            return cross_entropy_backward(x, *o->tensor, g);
        }
        case op::MatMul: {                                              // :1643-1849
            Node* o = other_node();
            const Tensor& other = *o->tensor;
            if (g.dim() != 2)
                Ctorch_Error::throwException(ErrorPlatform::kAutoDiff, ErrorType::DIMENSION,
                                             "MatMul gradient must be a 2-D tensor");
            term_plus_zero_ = true;                                             // sums of products from +0
            if (first) return MatMul_AMD_kernel(g, Tensor::view_t(other));      // g . B^T
            return MatMul_AMD_kernel(Tensor::view_t(other), g);                 // A^T . g
        }
        case op::Linear: {                                              // the three branches above in one
            const Tensor& gz = linear_pre_activation_grad(node, g);
            if (input_pos == 2) {                                       // bias: Add's branch, shaped by the caller
                if (node->input_grads.size() == 3 && !node->input_grads[2].is_cleared()) {
                    term_plus_zero_ = true;                             // the column sums that came with the weight gradient
                    return Tensor::alias(node->input_grads[2]);
                }
                term_plus_zero_ = node->op_param_i ? false : upstream_plus_zero;   // g * 0 may be -0
                return Tensor::alias(gz);
            }
            term_plus_zero_ = true;
            const Tensor& other = *find(node->input_ids[input_pos == 0 ? 1 : 0])->tensor;
            if (input_pos == 0) return MatMul_AMD_kernel(gz, Tensor::view_t(other));   // gz . W^T
            // When the bias wants its gradient too - the column sums of gz, which the caller would ask
            // for when the bias's turn comes - they are computed with the weight gradient: the same
            // two results bit for bit, and for a small layer one launch instead of two.
            if (bias_grad_with_weight_grad_ && broadcast_grad_ == BroadcastGrad::kColumnSum && node->input_ids.size() == 3 && gz.dim() == 2 &&
                gz.is_contiguous() &&
                gz.device() == DeviceType::kAMD && gz.dtype() == DType::kFloat && node->input_ids[2] != node->input_ids[1] &&
                node->input_ids[2] != node->input_ids[0]) {
                Node* bias = find(node->input_ids[2]);
                if (bias && bias->requires_grad && bias->tensor->dim() == 1 && bias->tensor->sizes()[0] == gz.sizes()[1]) {
                    Tensor sums;
                    Tensor gw = MatMulColSum_AMD_kernel(Tensor::view_t(other), gz, sums);
                    node->input_grads.clear();
                    node->input_grads.resize(3);
                    node->input_grads[2] = std::move(sums);
                    return gw;
                }
            }
            return MatMul_AMD_kernel(Tensor::view_t(other), gz);                        // x^T . gz
        }
        case op::LinearCE: {                                            // Linear's and CE's branches on what the forward pass kept
            auto* kept = dynamic_cast<LinearCEPayload*>(node->payload.get());
            if (!kept)
                Ctorch_Error::throwException(ErrorPlatform::kAutoDiff, ErrorType::TENSOR_STATE, "backward: classifier head without its record");
            // the kept gradients are those for an upstream gradient of 1 (a loss that is the root)
            const bool unit = g.known_value() && *g.known_value() == 1.0f;
            if (!unit && !node->shared_term) node->shared_term = std::make_unique<Tensor>(Mul_AMD_kernel(kept->dz, g));
            const Tensor& gz = unit ? kept->dz : *node->shared_term;
            term_plus_zero_ = true;                                     // sums of products from +0, and "0 +" terms
            if (input_pos == 0) {
                if (unit && !kept->dh.is_cleared() && !kept->dh_masked) return Tensor::alias(kept->dh);
                return MatMul_AMD_kernel(gz, Tensor::view_t(*find(node->input_ids[1])->tensor));   // gz . W^T
            }
            if (input_pos == 1) {
                if (unit) return Tensor::alias(kept->gw);
                return MatMul_AMD_kernel(Tensor::view_t(*find(node->input_ids[0])->tensor), gz);   // h^T . gz
            }
            if (unit && broadcast_grad_ == BroadcastGrad::kColumnSum) return Tensor::alias(kept->gb);
            term_plus_zero_ = false;
            return Tensor::alias(gz);                                   // shaped by the caller (column sums, or row 0)
        }
        case op::Fused: {                                               // every operator branch above, in one launch
            if (node->input_grads.empty()) {
                auto* program = dynamic_cast<FusedPayload*>(node->payload.get());
                if (!program)
                    Ctorch_Error::throwException(ErrorPlatform::kAutoDiff, ErrorType::TENSOR_STATE, "backward: fused operator without its program");
                std::vector<const Tensor*> inputs;
                std::vector<bool> wanted;
                for (size_t id : node->input_ids) {
                    Node* in = find(id);
                    inputs.push_back(in->tensor.get());
                    wanted.push_back(in->requires_grad);
                }
                node->input_grads = program->backward(inputs, wanted, g, check_div_zero_);
            }
            if (input_pos >= node->input_grads.size() || node->input_grads[input_pos].is_cleared())
                return Tensor(ShapeTag{}, x.sizes(), DType::kFloat, x.device());   // not reached: zeros
            term_plus_zero_ = true;                                     // the program stores "0 + term"
            return Tensor::alias(node->input_grads[input_pos]);
        }
        case op::Sum:                                                   // :1850-1855
            term_plus_zero_ = upstream_plus_zero;
            return adjust_grad_shape(g, x.sizes());
        // the methods the reference declares without defining them (include/Tensor.h:824-1072)
        case op::Abs: return unary_declared_backward(op::Abs, x, g);
        case op::Square: return unary_declared_backward(op::Square, x, g);
        case op::Log: return unary_declared_backward(op::Log, x, g);
        case op::Exp: return unary_declared_backward(op::Exp, *node->tensor, g);
        case op::Sqrt: return unary_declared_backward(op::Sqrt, *node->tensor, g);
        case op::Tan: return unary_declared_backward(op::Tan, *node->tensor, g);
        case op::LReLU: {
            float slope = 0.0f;
            std::memcpy(&slope, &node->op_param_i, sizeof(slope));
            return unary_declared_backward(op::LReLU, x, g, slope);
        }
        case op::LogSoftmax: return log_softmax_backward(*node->tensor, g, node->op_param_i);
        case op::Reduce: {
            auto* r = dynamic_cast<ReducePayload*>(node->payload.get());
            if (!r)
                Ctorch_Error::throwException(ErrorPlatform::kAutoDiff, ErrorType::TENSOR_STATE, "backward: reduction without its record");
            return reduce_axis_backward(r->kind, x, *node->tensor, r->index, r->mean, g, r->outer, r->len, r->inner, r->ddof);
        }
        case op::Dot: {                                                 // extension: g * other
            Node* o = other_node();
            Tensor r = Mul_AMD_kernel(Tensor::alias(*o->tensor), g);
            return r;
        }
        default:
            Ctorch_Error::throwException(ErrorPlatform::kAutoDiff, ErrorType::UNKNOWN,
                                         "backward: operator has no gradient");
    }
}

// The gradient at a layer's pre-activation: g * [y > 0], which is the reference's g * [z > 0]
// (:1320-1371) since y = max(0, z); computed once for the three inputs - or g itself when the layer
// has no ReLU, or when the product that formed g applied the mask already.
const Tensor& AutoDiff::linear_pre_activation_grad(Node* node, const Tensor& g) {
    if (!node->op_param_i || node->grad_premasked_by) return g;
    if (!node->shared_term) node->shared_term = std::make_unique<Tensor>(relu_backward(*node->tensor, g));
    return *node->shared_term;
}

// The seed 1.0 on the device is made once per thread and shared (the tape never writes through a
// shared gradient: accumulation goes to a fresh tensor then).
static Tensor& device_seed() {
    thread_local Tensor device_one;
    if (device_one.is_cleared()) device_one = Tensor(1.0f, DeviceType::kAMD);
    return device_one;
}
// Called before a recording starts: a seed made inside one would be a recorded launch into memory
// reserved for that graph, and a backward() outside the graph would read it before any replay.
void prepare_backward_seed() { (void)device_seed(); }

// src/AutoDiff.cpp:548-553
void AutoDiff::backward(Tensor& root) {
    AutoDiffContext::Guard guard(nullptr);
    if (root.device() == DeviceType::kAMD) {
        seed_plus_zero_ = true;
        backward(root, Tensor::alias(device_seed()));
        return;
    }
    Tensor grad_output(1.0f, root.device());
    backward(root, std::move(grad_output));
}

// src/AutoDiff.cpp:1080-1924
void AutoDiff::backward(Tensor& root, Tensor grad_output) {
    AutoDiffContext::Guard guard(nullptr);   // nothing below is taped
    if (root.id() == 0)
        Ctorch_Error::throwException(ErrorPlatform::kAutoDiff, ErrorType::TENSOR_STATE, "backward: invalid root tensor");
    Node* root_node = find(root.id());
    if (!root_node) {
        Ctorch_Error::log(ErrorLevel::ERROR, ErrorPlatform::kAutoDiff, ErrorType::TENSOR_STATE, "backward: root is not on the tape");
        return;
    }
    if (!root_node->requires_grad) return;
    // Gradients are float: the seed is (src/AutoDiff.cpp:548-553), and the reference's backward over
    // a double / int root stops with a DATATYPE exception when that seed meets the typed nodes.
    if (root.dtype() != DType::kFloat || grad_output.dtype() != DType::kFloat)
        Ctorch_Error::throwException(ErrorPlatform::kAutoDiff, ErrorType::DATATYPE, "backward: only float tensors have gradients");
    if (grad_output.device() != root.device()) grad_output = grad_output.to(root.device());
    ctorch_amd_host::drop_deferred_checks();     // of a pass that ended in an exception
    // A gradient that an earlier pass left at a layer's pre-activation is brought back to the
    // gradient of the layer's output before anything is added to it (a pass over a tape that was
    // not cleared adds to what the nodes hold, as the reference's does).
    for (Node* n : premasked_) {
        Node* by = n->grad_premasked_by;
        if (!by) continue;
        n->grad_premasked_by = nullptr;
        if (n->grad && by->grad) {
            n->grad = n->unmasked_grad ? std::move(n->unmasked_grad)
                                       : std::make_unique<Tensor>(input_gradient(by, n->tensor_id, 0, *by->grad));
            n->grad_plus_zero = true;
            by->shared_term.reset();
        } else {
            n->grad.reset();                     // its source is gone: nothing to bring back
            n->grad_plus_zero = false;
        }
        n->unmasked_grad.reset();
    }
    premasked_.clear();
    root_node->grad = std::make_unique<Tensor>(adjust_grad_shape(grad_output, root.sizes()));
    root_node->grad_plus_zero = seed_plus_zero_;
    root_node->grad_assigned = !adjust_adds_to_zero_;     // a seed taken as it is stays as it is (:1126)
    seed_plus_zero_ = false;

    // reversed depth-first post-order, inputs visited in recorded order (:1058-1077, :1138-1153)
    std::vector<Node*> order;
    {
        std::unordered_set<Node*> visited;
        std::vector<std::pair<Node*, size_t>> stack;
        stack.push_back({root_node, 0});
        visited.insert(root_node);
        while (!stack.empty()) {
            Node* n = stack.back().first;
            size_t& next = stack.back().second;
            if (next < n->input_ids.size()) {
                Node* in = find(n->input_ids[next++]);
                if (in && visited.insert(in).second) stack.push_back({in, 0});
            } else {
                order.push_back(n);
                stack.pop_back();
            }
        }
        std::reverse(order.begin(), order.end());
    }

    // how many operator inputs of this pass read each tensor
    std::unordered_map<size_t, int> consumers;
    for (Node* n : order)
        for (size_t id : n->input_ids) ++consumers[id];

    for (Node* node : order) {
        if (!node->requires_grad || !node->grad || node->is_leaf) continue;
        const Tensor& node_grad = *node->grad;
        for (size_t pos = 0; pos < node->input_ids.size(); ++pos) {
            size_t input_id = node->input_ids[pos];
            Node* in = find(input_id);
            if (!in || !in->requires_grad) continue;
            in->grad_assigned = false;               // whatever it holds is added to from here on
            // a second loss of the same predictions: its gradient is added to the one gathered so far
            // in the pass that forms it (the same sum as term-then-accumulate, bit for bit)
            if ((node->operation == op::MSE || node->operation == op::MAE) && pos == 0 && in->grad &&
                node->input_ids.size() == 2 && node->input_ids[1] != input_id && in->grad->is_contiguous() &&
                in->grad->sizes() == in->tensor->sizes() && in->tensor->device() == DeviceType::kAMD) {
                Node* target = find(node->input_ids[1]);
                if (target && target->tensor->sizes() == in->tensor->sizes()) {
                    in->grad = std::make_unique<Tensor>(loss_backward_plus(node->operation == op::MAE, *in->tensor, *target->tensor,
                                                                            node_grad, *in->grad));
                    // the term carries its "0 +"; the sum holds no -0 unless the gathered part did
                    continue;
                }
            }
            // likewise the gradient of a unary operator whose operand other operators use as well
            if ((node->operation == op::ReLU || node->operation == op::Sigmoid || node->operation == op::Tanh ||
                 node->operation == op::Sin || node->operation == op::Cos) && in->grad && in->grad->is_contiguous() &&
                in->grad->sizes() == in->tensor->sizes() && node_grad.sizes() == in->tensor->sizes() &&
                node_grad.is_contiguous() && in->tensor->device() == DeviceType::kAMD) {
                in->grad = std::make_unique<Tensor>(unary_backward_plus(node->operation, *in->tensor, node_grad, *in->grad));
                in->grad_plus_zero = false;          // g * 0 may be -0, and -0 + -0 is -0
                continue;
            }
            // and Neg, the second operand of Sub (gathered + (-g) is gathered - g, bit for bit) and
            // Mul of two full tensors (gathered + other * g)
            const bool joinable = in->grad && in->grad->is_contiguous() && in->grad->sizes() == in->tensor->sizes() &&
                                  node_grad.sizes() == in->tensor->sizes() && node_grad.is_contiguous() &&
                                  in->tensor->device() == DeviceType::kAMD;
            if (joinable && (node->operation == op::Neg ||
                             (node->operation == op::Sub && node->input_ids.size() == 2 && input_id != node->input_ids[0]))) {
                in->grad = std::make_unique<Tensor>(Sub_AMD_kernel(*in->grad, node_grad));
                in->grad_plus_zero = false;
                continue;
            }
            if (joinable && node->operation == op::Mul && node->input_ids.size() == 2 && node->input_ids[0] != node->input_ids[1]) {
                Node* o = find(input_id == node->input_ids[0] ? node->input_ids[1] : node->input_ids[0]);
                if (o && o->tensor->device() == DeviceType::kAMD && o->tensor->sizes() == in->tensor->sizes() &&
                    o->tensor->is_contiguous()) {
                    in->grad = std::make_unique<Tensor>(mul_plus(*o->tensor, node_grad, *in->grad));
                    in->grad_plus_zero = false;
                    continue;
                }
            }
            // and the first operand of Div by a full tensor or a row vector (gathered + g / b), after the
            // zero-divisor check the Div branch makes
            if (joinable && node->operation == op::Div && node->input_ids.size() == 2 && input_id == node->input_ids[0] &&
                node->input_ids[0] != node->input_ids[1]) {
                Node* bn = find(node->input_ids[1]);
                if (bn && bn->tensor->device() == DeviceType::kAMD && bn->tensor->is_contiguous() &&
                    (bn->tensor->sizes() == in->tensor->sizes() || is_row_vector_of(*bn->tensor, *in->tensor))) {
                    if (check_div_zero_ && any_abs_lt_eps(*bn->tensor))
                        Ctorch_Error::throwException(ErrorPlatform::kGENERAL, ErrorType::TENSOR_STATE,
                                                     "division by zero in the gradient of Div");
                    in->grad = std::make_unique<Tensor>(div_plus(node_grad, *bn->tensor, *in->grad));
                    in->grad_plus_zero = false;
                    continue;
                }
            }
            // The output of a ReLU layer read by this product alone: its gradient g . W^T is wanted only
            // times the layer's mask, so the mask rides in the product's launch (one launch instead of
            // two, the same bits: the 0 / 1 factor multiplies the same fp32 product).
            if (fuse_relu_mask_ && pos == 0 && !in->grad && in != root_node && !in->is_leaf &&
                (node->operation == op::Linear || node->operation == op::MatMul) && node->input_ids.size() >= 2 &&
                node->input_ids[1] != input_id && in->operation == op::Linear && in->op_param_i != 0 &&
                consumers[input_id] == 1 && node_grad.dim() == 2 && in->tensor->dim() == 2 &&
                in->tensor->device() == DeviceType::kAMD && in->tensor->is_contiguous() && in->tensor->dtype() == DType::kFloat) {
                Node* wn = find(node->input_ids[1]);
                const Tensor& gz = node->operation == op::Linear ? linear_pre_activation_grad(node, node_grad) : node_grad;
                if (wn && wn->tensor->dim() == 2 && wn->tensor->device() == DeviceType::kAMD && gz.device() == DeviceType::kAMD &&
                    gz.sizes()[0] == in->tensor->sizes()[0] && gz.sizes()[1] == wn->tensor->sizes()[1] &&
                    wn->tensor->sizes()[0] == in->tensor->sizes()[1]) {
                    in->grad = std::make_unique<Tensor>(MatMulReluMask_AMD_kernel(gz, Tensor::view_t(*wn->tensor), *in->tensor));
                    in->grad_plus_zero = false;          // g * 0 may be -0
                    in->grad_premasked_by = node;
                    premasked_.insert(in);
                    continue;
                }
            }
            // The same for a classifier head whose one pass already formed that masked gradient.
            if (fuse_relu_mask_ && pos == 0 && node->operation == op::LinearCE && !in->grad && in != root_node && !in->is_leaf &&
                in->operation == op::Linear && in->op_param_i != 0 && consumers[input_id] == 1 && node_grad.known_value() &&
                *node_grad.known_value() == 1.0f) {
                auto* kept = dynamic_cast<LinearCEPayload*>(node->payload.get());
                if (kept && kept->dh_masked && !kept->dh.is_cleared()) {
                    in->grad = std::make_unique<Tensor>(Tensor::alias(kept->dh));
                    in->grad_plus_zero = false;
                    in->grad_premasked_by = node;
                    premasked_.insert(in);
                    continue;
                }
            }
            Tensor val = input_gradient(node, input_id, pos, node_grad);
            Tensor adj = adjust_grad_shape(val, in->tensor->sizes());
            const bool plus_zero = term_plus_zero_;
            // :1870-1907 is "zero-filled gradient, then grad += val".  Here the first contribution
            // is kept as it is (no pass over memory; it may share its bytes with another node's
            // gradient) and the "0 +" is applied when the gradient is read (get_grad): adding +0
            // only turns -0 into +0, and the sign of a zero in an upstream gradient cannot change
            // any non-zero value downstream.  Later contributions add in place once the bytes are
            // this node's own, else into a fresh tensor.
            if (!in->grad) {
                if (adj.sizes() == in->tensor->sizes()) {
                    in->grad = std::make_unique<Tensor>(Tensor::alias(adj));
                    in->grad_plus_zero = plus_zero;
                } else {
                    in->grad = std::make_unique<Tensor>(zero_plus(adj, in->tensor->sizes()));
                    in->grad_plus_zero = true;
                }
            } else if (in->grad->storage_shared()) {
                in->grad = std::make_unique<Tensor>(sum_of(*in->grad, adj));
                in->grad_plus_zero = in->grad_plus_zero && plus_zero;    // no -0 in, no -0 out
            } else {
                accumulate(*in->grad, adj);
                in->grad_plus_zero = in->grad_plus_zero && plus_zero;
            }
        }
        node->shared_term.reset();
        node->input_grads.clear();
    }
    // checks whose answer a kernel left on the device (a zero divisor seen by a fused gradient
    // program): read now, with every launch of this pass already queued, instead of idling the GPU in
    // the middle of the pass
    ctorch_amd_host::run_deferred_checks();
}
