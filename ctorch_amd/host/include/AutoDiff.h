// Tape autograd over device tensors.  Same public surface as the reference's AutoDiff /
// AutoDiffContext (include/AutoDiff.h:29-67, :144-220): a thread-local current context with an
// RAII Guard, make_leaf / zero_grad / get_grad / backward / clear_graph, and the two-phase
// defer_record / commit_record used by the Tensor methods.
//
// The gradient arithmetic per operator follows src/AutoDiff.cpp:1216-1862 operation by
// operation; on kAMD tensors every piece is a kernel of the launch layer (fused where the
// reference chains several Tensor ops, with the same fp32 operation order inside the kernel), and
// every edge lands with the in-place accumulate of :1870-1907.
// Differences, all deliberate:
//  - nodes hold references (shared storage) to the tensors they describe instead of deep copies
//    (reference: AutoDiff.cpp:286, :465), so taping costs no HBM traffic;
//  - the gradient of a row-broadcast operand ([rows, cols] op [cols]) is the column sum by
//    default; BroadcastGrad::kReferenceRow0 reproduces the reference, which returns row 0 of the
//    upstream gradient (AutoDiff.cpp:690-757, expected by src/tests/test_tensor_grad.cpp:132-138);
//  - CrossEntropy's backward accepts class-index targets (the reference throws, :1569);
//  - backward() does not hold a lock while it runs kernels, so Tensor::backward(grad_output)
//    cannot self-deadlock (reference: Tensor.cpp:549-550 -> AutoDiff.cpp:1157 + :346).
#ifndef CTORCH_AMD_HOST_AUTODIFF_H
#define CTORCH_AMD_HOST_AUTODIFF_H
#include <memory>
#include <mutex>
#include <unordered_map>
#include <unordered_set>
#include <vector>

#include "Tensor.h"

class AutoDiff;

class AutoDiffContext {
   public:
    static AutoDiff*& current() {
        thread_local AutoDiff* ctx = nullptr;
        return ctx;
    }
    class Guard {
        AutoDiff* prev_;

       public:
        explicit Guard(AutoDiff* ctx) : prev_(current()) { current() = ctx; }
        ~Guard() { current() = prev_; }
        Guard(const Guard&) = delete;
        Guard& operator=(const Guard&) = delete;
    };
};

enum class BroadcastGrad { kColumnSum, kReferenceRow0 };
// What the tape reads as a leaf's value in backward: the live tensor (default), or - as the
// reference - the deep copy made when the leaf was first seen and never refreshed
// (src/AutoDiff.cpp:265-278 returns early for a known id), so that after an in-place optimiser
// update the gradients flowing back through a weight matrix still use its first-step values.
enum class LeafValues { kLive, kReferenceFirstSeen };

class AutoDiff {
   public:
    // what an operator needs in backward beyond its inputs (the compiled program of op::Fused)
    struct OpPayload {
        virtual ~OpPayload() = default;
    };
    // a reduction along dimensions (op::Reduce): which one, the [outer, len, inner] reading of the
    // operand, and what the forward pass kept for the gradient
    struct ReducePayload : OpPayload {
        int kind = 0, ddof = 1;
        size_t outer = 1, len = 1, inner = 1;
        Tensor index;    // max / min: position of the extreme element along the axis (int32)
        Tensor mean;     // var / std
    };
    // what Tensor::linear_cross_entropy formed in its one pass (op::LinearCE): the gradient of the logits
    // for an upstream gradient of 1, and from it the gradients of the three inputs
    struct LinearCEPayload : OpPayload {
        Tensor labels, dz, dh, gw, gb;
        bool dh_masked = false;   // dh is already multiplied by [h > 0]: the gradient at the pre-activation of the ReLU layer that produced h
    };
    struct Node {
        size_t tensor_id = 0;
        op operation = op::Add;
        int op_param_i = 0;
        std::vector<size_t> input_ids;
        std::unique_ptr<Tensor> tensor;   // shares storage with the user's tensor
        std::unique_ptr<Tensor> grad;
        bool grad_plus_zero = false;           // grad holds no -0: "0 + grad" (what get_grad returns) is grad itself
        bool grad_assigned = false;            // grad is a root's seed: assigned, not added to zeros (src/AutoDiff.cpp:1126), read as it is
        // Set on a ReLU layer (op::Linear with its ReLU) whose output has one consumer, a product: that
        // consumer's backward formed `grad` already multiplied by [y > 0], i.e. `grad` is the gradient at
        // the pre-activation and the layer's own mask launch is skipped.  get_grad() forms the
        // gradient of the output itself from the consumer when somebody asks for it.
        Node* grad_premasked_by = nullptr;
        std::unique_ptr<Tensor> unmasked_grad;  // with grad_premasked_by: the gradient of the output, once somebody asked for it
        std::unique_ptr<Tensor> shared_term;   // backward only: a factor that several inputs' gradients use
        std::vector<Tensor> input_grads;       // backward only: gradients of all inputs, computed together
        std::shared_ptr<OpPayload> payload;
        bool requires_grad = false;
        bool is_leaf = true;
    };

    AutoDiff() = default;
    ~AutoDiff() = default;

    void make_leaf(Tensor& t, bool requires_grad);
    void update_requires_grad(Tensor& t, bool requires_grad);
    void zero_grad(Tensor& t);
    Tensor get_grad(const Tensor* t);
    Tensor stored_grad(const Tensor& t);   // extension: the stored bytes, shared; see AutoDiff.cpp
    void defer_record(size_t output_id, op operation, const std::vector<Tensor*>& inputs, int op_param_i = 0,
                      std::shared_ptr<OpPayload> payload = nullptr);
    void commit_record(Tensor& output);
    void set_retain_graph(bool retain) { retain_graph_ = retain; }
    void backward(Tensor& root);
    void backward(Tensor& root, Tensor grad_output);
    void clear_graph();
    size_t node_count();
    // whether t is on the tape as the output of a fused layer with its ReLU (Tensor::linear(.., true))
    bool is_relu_layer_output(const Tensor& t);

    void set_broadcast_grad(BroadcastGrad m) { broadcast_grad_ = m; }
    BroadcastGrad broadcast_grad() const { return broadcast_grad_; }
    void set_leaf_values(LeafValues m) { leaf_values_ = m; }
    // Div's backward scans the divisor for |b| < FLT_EPSILON and throws (reference:
    // AutoDiff.cpp:1267-1284).  On the device that is one more pass over b and a host wait; it can
    // be switched off.
    void set_check_div_zero(bool on) { check_div_zero_ = on; }
    // The ReLU mask of a layer in the launch of the product that forms the layer's output gradient
    // (on by default; the gradients are the same bits either way).
    void set_fuse_relu_mask(bool on) { fuse_relu_mask_ = on; }
    bool fuse_relu_mask() const { return fuse_relu_mask_; }
    // The bias gradient of a fused layer (the column sums of the layer's output gradient) computed
    // with the weight gradient, for a small layer in the same launch (on by default; the gradients
    // are the same bits either way).
    void set_bias_grad_with_weight_grad(bool on) { bias_grad_with_weight_grad_ = on; }
    bool bias_grad_with_weight_grad() const { return bias_grad_with_weight_grad_; }

   private:
    struct Pending {
        op operation;
        std::vector<size_t> input_ids;
        int op_param_i;
        std::shared_ptr<OpPayload> payload;
    };
    std::mutex records_mutex;
    std::unordered_map<size_t, std::unique_ptr<Node>> id_to_node;
    std::unordered_map<size_t, Pending> pending_;
    std::unordered_set<Node*> premasked_;    // nodes whose grad_premasked_by is set (what the next backward() has to bring back)
    bool retain_graph_ = false;
    BroadcastGrad broadcast_grad_ = BroadcastGrad::kColumnSum;
    LeafValues leaf_values_ = LeafValues::kLive;
    bool check_div_zero_ = true;
    bool fuse_relu_mask_ = true;
    bool bias_grad_with_weight_grad_ = true;
    bool term_plus_zero_ = false;   // backward: the term just computed holds no -0
    bool seed_plus_zero_ = false;   // backward: the seed gradient holds no -0
    bool adjust_adds_to_zero_ = false;   // the last adjust_grad_shape took a branch in which the reference adds the gradient to zeros

    Node* find(size_t id);
    Tensor adjust_grad_shape(const Tensor& grad, const std::vector<size_t>& target_shape);
    Tensor input_gradient(Node* node, size_t input_id, size_t input_pos, const Tensor& node_grad);
    const Tensor& linear_pre_activation_grad(Node* node, const Tensor& node_grad);
};
// Makes this thread's device seed of backward(root) (a 0-D 1.0) now, if it does not exist yet.
void prepare_backward_seed();

#endif
