// Host-side callers of the storage backend, mirrored from the reference so that one training step issues the same
// sequence of storage calls (and therefore the same kernels and pool traffic) as Ferrox does:
//   Operator<T>          src/ops/mod.rs:16-49  and the operators of src/ops/{basic,matrix,unary,reduction,reshape,
//                        comparison,batched}.rs that the MLP / CNN configs exercise
//   AutoFerroxEngine<T>  src/graph/mod.rs:341-997  (eager tape: apply_operation, backward, accumulate_gradient)
//   Linear, Conv2d, ReLU, Flatten   src/nn/layers/{linear,conv2d,activation,pooling}.rs
//   CCELoss              src/nn/losses/classification.rs:191-257
//   SGD, Adam            src/nn/optim/{sgd,adam}.rs
// With `literal_engine` the engine also performs the reference's per-node deep clone in backward_node
// (src/graph/mod.rs:735-751: get_node_owned clones the node and its tensor just to read its inputs); without it
// that redundant device copy is skipped.  Everything else is issued exactly as the reference issues it.
#pragma once
#include <cmath>
#include <functional>
#include <map>
#include <optional>
#include <set>

#include "hip_storage.hpp"
#include "state_dict.hpp"

namespace ferrox {

template <typename T> using TensorRefs = std::vector<const HipStorage<T>*>;

// ---- Operator: src/ops/mod.rs:16-49 ---------------------------------------------------------------------------
template <typename T> struct Operator {
    virtual ~Operator() = default;
    virtual Tensor<T> compute(const TensorRefs<T>& inputs) const = 0;
    virtual std::vector<Tensor<T>> gradient(Tensor<T> grad_output, const TensorRefs<T>& inputs, const HipStorage<T>* output) const = 0;
    // `needs[i]` tells whether input i takes part in differentiation.  The reference's operators always return
    // every gradient, which is what the default does; fused operators may return a null entry where needs[i] is false.
    virtual std::vector<Tensor<T>> gradient_needs(Tensor<T> grad_output, const TensorRefs<T>& inputs, const HipStorage<T>* output,
                                                  const std::vector<bool>&) const {
        return gradient(std::move(grad_output), inputs, output);
    }
    virtual size_t num_inputs() const = 0;
    virtual bool cache_output() const { return false; }
    virtual const char* name() const = 0;
    // Fused operators only.  output_is_relu(): the output went through a ReLU inside the operator.  The engine sets
    // input0_is_relu_output before it asks for gradients when input 0 is the output of such an operator: the gradient of input 0
    // may then be handed back already multiplied by the ReLU's mask (input 0 > 0), marked with HipStorage::relu_masked_by.
    virtual bool output_is_relu() const { return false; }
    mutable bool input0_is_relu_output = false;
};

// reduce_gradient_for_broadcasting, src/ops/basic.rs:10-53
template <typename T> void reduce_gradient_for_broadcasting(Tensor<T>& grad, const Shape& target) {
    const Shape& gs = grad->shape();
    if (gs == target) return;
    std::vector<size_t> axes;
    size_t ti = target.size();
    for (size_t i = gs.size(); i-- > 0;) {
        if (ti == 0) axes.push_back(i);
        else {
            --ti;
            if (target[ti] == 1 && gs[i] > 1) axes.push_back(i);
        }
    }
    if (!axes.empty()) grad = grad->sum(&axes, false);
    if (grad->shape() != target) grad->reshape(target);
}

// expand_reduction, src/ops/reduction.rs:9-50
template <typename T> Tensor<T> expand_reduction(Tensor<T> g, const std::vector<size_t>* axes, const Shape& input_shape) {
    if (axes) {
        std::vector<size_t> sorted = *axes;
        std::sort(sorted.begin(), sorted.end());
        if (sorted.empty()) return g;
        for (size_t a : sorted) g->unsqueeze(a);
        if (g->shape() != input_shape) g->broadcast_to(input_shape);
        return g;
    }
    const T scalar = g->first();  // device -> host round trip, as in the reference
    return HipStorage<T>::full(input_shape, scalar);
}

template <typename T> struct Add : Operator<T> {  // src/ops/basic.rs:57-130
    Tensor<T> compute(const TensorRefs<T>& in) const override { return in[0]->add(*in[1]); }
    std::vector<Tensor<T>> gradient(Tensor<T> g, const TensorRefs<T>& in, const HipStorage<T>*) const override {
        Tensor<T> g1 = g->clone_storage();
        Tensor<T> g2 = std::move(g);
        reduce_gradient_for_broadcasting(g1, in[0]->shape());
        reduce_gradient_for_broadcasting(g2, in[1]->shape());
        std::vector<Tensor<T>> r;
        r.push_back(std::move(g1));
        r.push_back(std::move(g2));
        return r;
    }
    size_t num_inputs() const override { return 2; }
    const char* name() const override { return "Add"; }
};

template <typename T> struct Mul : Operator<T> {  // src/ops/basic.rs:175-215
    Tensor<T> compute(const TensorRefs<T>& in) const override { return in[0]->mul(*in[1]); }
    std::vector<Tensor<T>> gradient(Tensor<T> g, const TensorRefs<T>& in, const HipStorage<T>*) const override {
        Tensor<T> g1 = g->mul(*in[1]);
        Tensor<T> g2 = g->mul(*in[0]);
        reduce_gradient_for_broadcasting(g1, in[0]->shape());
        reduce_gradient_for_broadcasting(g2, in[1]->shape());
        std::vector<Tensor<T>> r;
        r.push_back(std::move(g1));
        r.push_back(std::move(g2));
        return r;
    }
    size_t num_inputs() const override { return 2; }
    const char* name() const override { return "Mul"; }
};

template <typename T> struct Sub : Operator<T> {  // src/ops/basic.rs:130-169
    Tensor<T> compute(const TensorRefs<T>& in) const override { return in[0]->sub(*in[1]); }
    std::vector<Tensor<T>> gradient(Tensor<T> g, const TensorRefs<T>& in, const HipStorage<T>*) const override {
        Tensor<T> g2 = g->neg();
        Tensor<T> g1 = std::move(g);
        reduce_gradient_for_broadcasting(g1, in[0]->shape());
        reduce_gradient_for_broadcasting(g2, in[1]->shape());
        std::vector<Tensor<T>> r;
        r.push_back(std::move(g1));
        r.push_back(std::move(g2));
        return r;
    }
    size_t num_inputs() const override { return 2; }
    const char* name() const override { return "Sub"; }
};

template <typename T> struct Div : Operator<T> {  // src/ops/basic.rs:221-272 (output cached: the gradient reuses x/y)
    Tensor<T> compute(const TensorRefs<T>& in) const override { return in[0]->div(*in[1]); }
    std::vector<Tensor<T>> gradient(Tensor<T> g, const TensorRefs<T>& in, const HipStorage<T>* out) const override {
        Tensor<T> recomputed;
        if (!out) {
            recomputed = compute(in);
            out = recomputed.get();
        }
        Tensor<T> g1 = g->div(*in[1]);
        reduce_gradient_for_broadcasting(g1, in[0]->shape());
        Tensor<T> q = out->div(*in[1]);
        Tensor<T> nq = q->neg();
        Tensor<T> g2 = g->mul(*nq);
        reduce_gradient_for_broadcasting(g2, in[1]->shape());
        std::vector<Tensor<T>> r;
        r.push_back(std::move(g1));
        r.push_back(std::move(g2));
        return r;
    }
    size_t num_inputs() const override { return 2; }
    bool cache_output() const override { return true; }
    const char* name() const override { return "Div"; }
};

template <typename T> struct AddScalar : Operator<T> {  // src/ops/scalar.rs (AddScalar): the gradient passes through
    T scalar;
    explicit AddScalar(T s) : scalar(s) {}
    Tensor<T> compute(const TensorRefs<T>& in) const override { return in[0]->add_scalar(scalar); }
    std::vector<Tensor<T>> gradient(Tensor<T> g, const TensorRefs<T>&, const HipStorage<T>*) const override {
        std::vector<Tensor<T>> r;
        r.push_back(std::move(g));
        return r;
    }
    size_t num_inputs() const override { return 1; }
    const char* name() const override { return "AddScalar"; }
};

template <typename T> struct Sqrt : Operator<T> {  // src/ops/unary.rs:107-151: g / (2 * sqrt(x)), from the cached output
    Tensor<T> compute(const TensorRefs<T>& in) const override { return in[0]->sqrt(); }
    std::vector<Tensor<T>> gradient(Tensor<T> g, const TensorRefs<T>& in, const HipStorage<T>* out) const override {
        Tensor<T> recomputed;
        if (!out) {
            recomputed = compute(in);
            out = recomputed.get();
        }
        Tensor<T> den = out->mul_scalar(T(2));
        std::vector<Tensor<T>> r;
        r.push_back(g->div(*den));
        return r;
    }
    size_t num_inputs() const override { return 1; }
    bool cache_output() const override { return true; }
    const char* name() const override { return "Sqrt"; }
};

template <typename T> struct MatMul : Operator<T> {  // src/ops/matrix.rs:17-64
    Tensor<T> compute(const TensorRefs<T>& in) const override {
        if (in[0]->ndim() != 2 || in[1]->ndim() != 2) throw Error("MatMul requires 2D tensors (matrices)");
        return in[0]->matmul(*in[1]);
    }
    std::vector<Tensor<T>> gradient(Tensor<T> g, const TensorRefs<T>& in, const HipStorage<T>*) const override {
        Tensor<T> bt = in[1]->clone_storage();
        bt->transpose(nullptr);
        Tensor<T> ga = g->matmul(*bt);
        Tensor<T> at = in[0]->clone_storage();
        at->transpose(nullptr);
        Tensor<T> gb = at->matmul(*g);
        std::vector<Tensor<T>> r;
        r.push_back(std::move(ga));
        r.push_back(std::move(gb));
        return r;
    }
    size_t num_inputs() const override { return 2; }
    const char* name() const override { return "MatMul"; }
};

template <typename T> struct Transpose : Operator<T> {  // src/ops/matrix.rs:66-125 (axes = None)
    Tensor<T> compute(const TensorRefs<T>& in) const override {
        Tensor<T> r = in[0]->clone_storage();
        r->transpose(nullptr);
        return r;
    }
    std::vector<Tensor<T>> gradient(Tensor<T> g, const TensorRefs<T>&, const HipStorage<T>*) const override {
        g->transpose(nullptr);
        std::vector<Tensor<T>> r;
        r.push_back(std::move(g));
        return r;
    }
    size_t num_inputs() const override { return 1; }
    const char* name() const override { return "Transpose"; }
};

template <typename T> struct ReLUOp : Operator<T> {  // src/ops/unary.rs:340-384
    Tensor<T> compute(const TensorRefs<T>& in) const override { return in[0]->relu(); }
    std::vector<Tensor<T>> gradient(Tensor<T> g, const TensorRefs<T>& in, const HipStorage<T>*) const override {
        Tensor<T> mask = in[0]->greater_scalar(T(0));
        std::vector<Tensor<T>> r;
        r.push_back(g->mul(*mask));
        return r;
    }
    size_t num_inputs() const override { return 1; }
    const char* name() const override { return "ReLU"; }
};

template <typename T> struct Log : Operator<T> {  // src/ops/unary.rs:60-95
    Tensor<T> compute(const TensorRefs<T>& in) const override { return in[0]->log(); }
    std::vector<Tensor<T>> gradient(Tensor<T> g, const TensorRefs<T>& in, const HipStorage<T>*) const override {
        std::vector<Tensor<T>> r;
        r.push_back(g->div(*in[0]));
        return r;
    }
    size_t num_inputs() const override { return 1; }
    const char* name() const override { return "Log"; }
};

template <typename T> struct Neg : Operator<T> {  // src/ops/unary.rs:196-236
    Tensor<T> compute(const TensorRefs<T>& in) const override { return in[0]->neg(); }
    std::vector<Tensor<T>> gradient(Tensor<T> g, const TensorRefs<T>&, const HipStorage<T>*) const override {
        std::vector<Tensor<T>> r;
        r.push_back(g->neg());
        return r;
    }
    size_t num_inputs() const override { return 1; }
    const char* name() const override { return "Neg"; }
};

template <typename T> struct Clamp : Operator<T> {  // src/ops/comparison.rs:250-297
    T lo, hi;
    Clamp(T lo_, T hi_) : lo(lo_), hi(hi_) {}
    Tensor<T> compute(const TensorRefs<T>& in) const override { return in[0]->clamp(lo, hi); }
    std::vector<Tensor<T>> gradient(Tensor<T> g, const TensorRefs<T>& in, const HipStorage<T>*) const override {
        Tensor<T> a = in[0]->greater_equal_scalar(lo);
        Tensor<T> b = in[0]->less_equal_scalar(hi);
        Tensor<T> m = a->mul(*b);
        std::vector<Tensor<T>> r;
        r.push_back(g->mul(*m));
        return r;
    }
    size_t num_inputs() const override { return 1; }
    const char* name() const override { return "Clamp"; }
};

template <typename T> struct Softmax : Operator<T> {  // src/ops/batched.rs:4-131 (axis = Some(axis))
    size_t axis;
    explicit Softmax(size_t a) : axis(a) {}
    Tensor<T> compute(const TensorRefs<T>& in) const override { return in[0]->softmax_batched(axis); }
    std::vector<Tensor<T>> gradient(Tensor<T> g, const TensorRefs<T>& in, const HipStorage<T>* out) const override {
        Tensor<T> recomputed;
        if (!out) {
            recomputed = compute(in);
            out = recomputed.get();
        }
        if (out->shape() != g->shape()) throw Error("Softmax gradient: shape mismatch");
        Tensor<T> prod = g->mul(*out);
        std::vector<size_t> ax{axis};
        Tensor<T> sum_prod = prod->sum(&ax, true);
        sum_prod->broadcast_to(out->shape());
        Tensor<T> diff = g->sub(*sum_prod);
        std::vector<Tensor<T>> r;
        r.push_back(out->mul(*diff));
        return r;
    }
    size_t num_inputs() const override { return 1; }
    bool cache_output() const override { return true; }
    const char* name() const override { return "Softmax"; }
};

template <typename T> struct Sum : Operator<T> {  // src/ops/reduction.rs:52-140
    bool has_axes;
    std::vector<size_t> axes;
    bool keep_dims;
    Sum(bool keep) : has_axes(false), keep_dims(keep) {}
    Sum(std::vector<size_t> a, bool keep) : has_axes(true), axes(std::move(a)), keep_dims(keep) {}
    Tensor<T> compute(const TensorRefs<T>& in) const override { return in[0]->sum(has_axes ? &axes : nullptr, keep_dims); }
    std::vector<Tensor<T>> gradient(Tensor<T> g, const TensorRefs<T>& in, const HipStorage<T>*) const override {
        const Shape& is = in[0]->shape();
        Tensor<T> e = (keep_dims && has_axes) ? std::move(g) : expand_reduction<T>(std::move(g), has_axes ? &axes : nullptr, is);
        if (e->shape() != is) e->broadcast_to(is);
        std::vector<Tensor<T>> r;
        r.push_back(std::move(e));
        return r;
    }
    size_t num_inputs() const override { return 1; }
    const char* name() const override { return "Sum"; }
};

template <typename T> struct Mean : Operator<T> {  // src/ops/reduction.rs:141-230 (Mean::new(): all axes, keep_dims false)
    bool has_axes = false;
    std::vector<size_t> axes;
    bool keep_dims = false;
    Mean() = default;
    Mean(std::vector<size_t> a, bool keep) : has_axes(true), axes(std::move(a)), keep_dims(keep) {}  // Mean::along_axes
    Tensor<T> compute(const TensorRefs<T>& in) const override { return in[0]->mean(has_axes ? &axes : nullptr, keep_dims); }
    std::vector<Tensor<T>> gradient(Tensor<T> g, const TensorRefs<T>& in, const HipStorage<T>*) const override {
        const Shape& is = in[0]->shape();
        double n = 1;
        if (has_axes) for (size_t a : axes) n *= (double)is[a];
        else n = (double)numel(is);
        Tensor<T> scaled = g->mul_scalar((T)(1.0 / n));
        Tensor<T> e = (keep_dims && has_axes) ? std::move(scaled) : expand_reduction<T>(std::move(scaled), has_axes ? &axes : nullptr, is);
        if (e->shape() != is) e->broadcast_to(is);
        std::vector<Tensor<T>> r;
        r.push_back(std::move(e));
        return r;
    }
    size_t num_inputs() const override { return 1; }
    const char* name() const override { return "Mean"; }
};

template <typename T> struct Reshape : Operator<T> {  // src/ops/reshape.rs:4-55
    Shape new_shape;
    explicit Reshape(Shape s) : new_shape(std::move(s)) {}
    Tensor<T> compute(const TensorRefs<T>& in) const override {
        Tensor<T> r = in[0]->clone_storage();
        r->reshape(new_shape);
        return r;
    }
    std::vector<Tensor<T>> gradient(Tensor<T> g, const TensorRefs<T>& in, const HipStorage<T>*) const override {
        g->reshape(in[0]->shape());
        std::vector<Tensor<T>> r;
        r.push_back(std::move(g));
        return r;
    }
    size_t num_inputs() const override { return 1; }
    const char* name() const override { return "Reshape"; }
};

template <typename T> struct BroadcastTo : Operator<T> {  // src/ops/reshape.rs:57-115
    Shape target;
    explicit BroadcastTo(Shape s) : target(std::move(s)) {}
    Tensor<T> compute(const TensorRefs<T>& in) const override {
        Tensor<T> r = in[0]->clone_storage();
        r->broadcast_to(target);
        return r;
    }
    std::vector<Tensor<T>> gradient(Tensor<T> g, const TensorRefs<T>& in, const HipStorage<T>*) const override {
        reduce_gradient_for_broadcasting(g, in[0]->shape());
        std::vector<Tensor<T>> r;
        r.push_back(std::move(g));
        return r;
    }
    size_t num_inputs() const override { return 1; }
    const char* name() const override { return "BroadcastTo"; }
};

template <typename T> struct Conv2dOp : Operator<T> {  // src/ops/batched.rs:133-230
    std::pair<size_t, size_t> stride, padding;
    Conv2dOp(std::pair<size_t, size_t> s, std::pair<size_t, size_t> p) : stride(s), padding(p) {}
    Tensor<T> compute(const TensorRefs<T>& in) const override {
        if (in[0]->ndim() != 4) throw Error("Conv2d input must be 4D [batch_size, in_channels, height, width]");
        if (in[1]->ndim() != 4) throw Error("Conv2d filter must be 4D [out_channels, in_channels, kernel_height, kernel_width]");
        if (in[0]->shape()[1] != in[1]->shape()[1]) {
            std::ostringstream m;
            m << "Input channels " << in[0]->shape()[1] << " don't match filter channels " << in[1]->shape()[1];
            throw Error(m.str());
        }
        return in[0]->conv2d(*in[1], stride, padding);
    }
    std::vector<Tensor<T>> gradient(Tensor<T> g, const TensorRefs<T>& in, const HipStorage<T>*) const override {
        Tensor<T> gi = g->deconv2d(*in[1], in[0]->shape(), stride, padding);
        Tensor<T> gf = in[0]->cross_correlation2d(*g, in[1]->shape(), stride, padding);
        std::vector<Tensor<T>> r;
        r.push_back(std::move(gi));
        r.push_back(std::move(gf));
        return r;
    }
    size_t num_inputs() const override { return 2; }
    const char* name() const override { return "Conv2d"; }
};

// MaxPool2D / AvgPool2D: src/ops/pooling.rs:12-230 (square window, one stride, zero padding; the output is cached
// because the max gradient needs to know which positions were selected)
template <typename T> struct Pool2dOp : Operator<T> {
    bool is_max;
    size_t kernel, stride, padding;
    Pool2dOp(bool mx, size_t k, size_t s, size_t p) : is_max(mx), kernel(k), stride(s), padding(p) {}
    Tensor<T> compute(const TensorRefs<T>& in) const override {
        return is_max ? in[0]->maxpool2d(kernel, stride, padding) : in[0]->avgpool2d(kernel, stride, padding);
    }
    std::vector<Tensor<T>> gradient(Tensor<T> g, const TensorRefs<T>& in, const HipStorage<T>* out) const override {
        if (in[0]->ndim() != 4) throw Error(std::string(is_max ? "MaxPool2D" : "AvgPool2D") + " requires 4D input tensor [N, C, H, W]");
        Tensor<T> recomputed;
        if (!out) {
            recomputed = compute(in);
            out = recomputed.get();
        }
        std::vector<Tensor<T>> r;
        r.push_back(is_max ? g->max_unpool2d(*in[0], *out, kernel, stride, padding) : g->avg_unpool2d(*in[0], *out, kernel, stride, padding));
        return r;
    }
    size_t num_inputs() const override { return 1; }
    bool cache_output() const override { return true; }
    const char* name() const override { return is_max ? "MaxPool2D" : "AvgPool2D"; }
};

// ---- AutoFerroxEngine: src/graph/mod.rs:341-997 (eager mode) -------------------------------------------------
using NodeId = size_t;

template <typename T> class AutoFerroxEngine {
    struct Node {
        Tensor<T> tensor;
        std::unique_ptr<Operator<T>> op;  // null for leaves
        std::vector<NodeId> inputs;
        bool requires_grad = false;
        bool is_leaf() const { return !op; }
        bool is_parameter() const { return is_leaf() && requires_grad; }
    };

  public:
    explicit AutoFerroxEngine(bool literal_engine = true) : literal_(literal_engine) {}

    NodeId create_variable(Tensor<T> t, bool requires_grad) {  // :403-408
        const NodeId id = next_id_++;
        Node n;
        n.tensor = std::move(t);
        n.requires_grad = requires_grad;
        nodes_[id] = std::move(n);
        return id;
    }
    NodeId apply_operation(std::unique_ptr<Operator<T>> op, std::vector<NodeId> input_ids) {  // :622-679
        if (input_ids.size() != op->num_inputs()) {
            std::ostringstream m;
            m << "Operation " << op->name() << " expects " << op->num_inputs() << " inputs, got " << input_ids.size();
            throw Error(m.str());
        }
        TensorRefs<T> in = collect(input_ids);
        Tensor<T> result = op->compute(in);
        const NodeId id = next_id_++;
        Node n;
        n.tensor = std::move(result);
        n.op = std::move(op);
        n.inputs = std::move(input_ids);
        n.requires_grad = true;
        nodes_[id] = std::move(n);
        return id;
    }
    const HipStorage<T>* get_tensor(NodeId id) const {
        auto it = nodes_.find(id);
        return it == nodes_.end() ? nullptr : it->second.tensor.get();
    }
    const HipStorage<T>* get_gradient(NodeId id) const {  // :394-396
        auto it = grads_.find(id);
        return it == grads_.end() ? nullptr : it->second.get();
    }
    HipStorage<T>* mutable_tensor(NodeId id) {  // in-place parameter updates of the fused optimizers
        auto it = nodes_.find(id);
        if (it == nodes_.end() || !it->second.is_parameter()) throw Error("Can only update parameter nodes (leaf nodes with requires_grad)");
        return it->second.tensor.get();
    }
    void zero_gradients() { grads_.clear(); }  // :838-840
    void clear_gradient(NodeId id) { grads_.erase(id); }  // :858-860
    void set_gradient(NodeId id, Tensor<T> g) { grads_[id] = std::move(g); }
    void clip_gradient(NodeId id, T coef) {  // :875-881
        auto it = grads_.find(id);
        if (it != grads_.end()) it->second = it->second->mul_scalar(coef);
    }
    void update_parameter(NodeId id, Tensor<T> t) {  // :845-866
        auto it = nodes_.find(id);
        if (it == nodes_.end()) throw Error("Node " + std::to_string(id) + " not found");
        if (!it->second.is_parameter()) throw Error("Can only update parameter nodes (leaf nodes with requires_grad)");
        it->second.tensor = std::move(t);
    }
    // keep_loss: receives the loss tensor itself before the graph is cleaned up (the fused training loop reads it after the
    // step instead of cloning it).  With reuse_unit_seed set, a one-element loss is seeded from a tensor of one 1.0 that is
    // filled once and only ever read, instead of a fresh ones() per step (same value, one kernel fewer).
    bool reuse_unit_seed = false;
    const T* unit_seed_data() const { return unit_seed_ ? unit_seed_->data() : nullptr; }  // null before the first backward()
    void backward(NodeId loss_id, Tensor<T>* keep_loss = nullptr) {  // :700-733
        const HipStorage<T>* loss = get_tensor(loss_id);
        if (!loss) throw Error("Loss node not found");
        if (reuse_unit_seed && loss->size() == 1) {
            if (!unit_seed_) unit_seed_ = HipStorage<T>::ones({1});
            Tensor<T> seed = HipStorage<T>::borrow(*unit_seed_);
            seed->reshape(loss->shape());
            grads_[loss_id] = std::move(seed);
        } else grads_[loss_id] = HipStorage<T>::ones(loss->shape());
        std::set<NodeId> visited;
        std::vector<NodeId> topo;
        topological_sort(loss_id, visited, topo);
        for (auto it = topo.rbegin(); it != topo.rend(); ++it) backward_node(*it);
        if (keep_loss) {
            auto it = nodes_.find(loss_id);
            if (it != nodes_.end()) *keep_loss = std::move(it->second.tensor);
        }
        cleanup();
    }
    size_t num_nodes() const { return nodes_.size(); }

  private:
    TensorRefs<T> collect(const std::vector<NodeId>& ids) const {  // collect_nodes_data, :575-585
        TensorRefs<T> r;
        for (NodeId id : ids) {
            const HipStorage<T>* t = get_tensor(id);
            if (!t) throw Error("[ERROR] Node " + std::to_string(id) + " not found!");
            r.push_back(t);
        }
        return r;
    }
    void topological_sort(NodeId id, std::set<NodeId>& visited, std::vector<NodeId>& order) const {  // :786-808
        if (visited.count(id)) return;
        visited.insert(id);
        auto it = nodes_.find(id);
        if (it != nodes_.end())
            for (NodeId in : it->second.inputs) topological_sort(in, visited, order);
        order.push_back(id);
    }
    void backward_node(NodeId id) {  // :743-783
        auto git = grads_.find(id);
        if (git == grads_.end()) return;
        Tensor<T> grad_output = std::move(git->second);
        grads_.erase(git);
        Node& node = nodes_.at(id);
        Tensor<T> literal_copy;
        if (literal_ && node.tensor) literal_copy = node.tensor->clone_storage();  // get_node_owned's deep clone, :735-751
        if (node.is_leaf()) {
            grads_[id] = std::move(grad_output);
            return;
        }
        TensorRefs<T> in = collect(node.inputs);
        std::vector<bool> needs;
        for (NodeId i : node.inputs) needs.push_back(nodes_.at(i).requires_grad);
        {
            auto pit = node.inputs.empty() ? nodes_.end() : nodes_.find(node.inputs[0]);
            node.op->input0_is_relu_output = pit != nodes_.end() && pit->second.op && pit->second.op->output_is_relu();
        }
        std::vector<Tensor<T>> gs = node.op->gradient_needs(std::move(grad_output), in, node.tensor.get(), needs);
        for (size_t i = 0; i < node.inputs.size(); ++i)
            if (gs[i]) accumulate_gradient(node.inputs[i], std::move(gs[i]));
    }
    void accumulate_gradient(NodeId id, Tensor<T> g) {  // :681-698
        auto it = grads_.find(id);
        if (it != grads_.end()) it->second = it->second->add(*g);
        else grads_[id] = std::move(g);
    }
    void cleanup() {  // :587-620: everything that is not a parameter goes away, with its gradient
        for (auto it = nodes_.begin(); it != nodes_.end();) {
            if (!it->second.is_parameter()) {
                grads_.erase(it->first);
                it = nodes_.erase(it);
            } else ++it;
        }
    }

    bool literal_;
    Tensor<T> unit_seed_;
    NodeId next_id_ = 0;
    std::map<NodeId, Node> nodes_;
    std::map<NodeId, Tensor<T>> grads_;
};

// ---- layers: src/nn/layers ------------------------------------------------------------------------------------
template <typename T> struct Module {
    virtual ~Module() = default;
    virtual NodeId forward(AutoFerroxEngine<T>& g, NodeId input) = 0;
    virtual std::vector<NodeId> parameters() const { return {}; }
    virtual void set_training(bool) {}
    // tensors that are not parameters but persist across steps (BatchNorm's running statistics)
    virtual std::vector<const HipStorage<T>*> state() const { return {}; }
};

// reshape_and_broadcast, src/nn/layers/utils.rs:6-42
template <typename T> NodeId reshape_and_broadcast(NodeId input, NodeId target, AutoFerroxEngine<T>& g) {
    const Shape ts = g.get_tensor(target)->shape();
    const Shape is = g.get_tensor(input)->shape();
    NodeId res = input;
    if (is.size() == 1) {
        Shape ns = ts.size() == 4 ? Shape{1, is[0], 1, 1} : Shape{1, is[0]};
        res = g.apply_operation(std::make_unique<Reshape<T>>(ns), {input});
    }
    if (is != ts) return g.apply_operation(std::make_unique<BroadcastTo<T>>(ts), {res});
    return res;
}

template <typename T> struct Linear : Module<T> {  // src/nn/layers/linear.rs:152-308; weight is [out_features, in_features]
    size_t in_features, out_features;
    NodeId weight = 0, bias = 0;
    bool has_bias = true;
    Linear(AutoFerroxEngine<T>& g, size_t in, size_t out, const T* w, const T* b) : in_features(in), out_features(out) {
        weight = g.create_variable(HipStorage<T>::from_vec(w, {out, in}), true);  // Linear::from_tensors, linear.rs:78-119
        has_bias = b != nullptr;
        if (has_bias) bias = g.create_variable(HipStorage<T>::from_vec(b, {out}), true);
    }
    NodeId forward(AutoFerroxEngine<T>& g, NodeId input) override {
        const Shape& s = g.get_tensor(input)->shape();
        if (s.size() != 1 && s.size() != 2)
            throw Error("Linear layer only supports 1D or 2D inputs, got shape " + fmt_shape(s));
        if (s.back() != in_features) {
            std::ostringstream m;
            m << "Input shape " << fmt_shape(s) << " doesn't match expected last dimension " << in_features;
            throw Error(m.str());
        }
        const NodeId wt = g.apply_operation(std::make_unique<Transpose<T>>(), {weight});
        const NodeId lin = g.apply_operation(std::make_unique<MatMul<T>>(), {input, wt});
        if (!has_bias) return lin;
        const Shape rs = g.get_tensor(lin)->shape();
        if (g.get_tensor(bias)->shape() != rs) {
            const NodeId bb = g.apply_operation(std::make_unique<BroadcastTo<T>>(rs), {bias});
            return g.apply_operation(std::make_unique<Add<T>>(), {lin, bb});
        }
        return g.apply_operation(std::make_unique<Add<T>>(), {lin, bias});
    }
    std::vector<NodeId> parameters() const override { return has_bias ? std::vector<NodeId>{weight, bias} : std::vector<NodeId>{weight}; }
};

template <typename T> struct Conv2d : Module<T> {  // src/nn/layers/conv2d.rs:135-243
    size_t in_channels, out_channels;
    std::pair<size_t, size_t> kernel, stride, padding;
    NodeId weight = 0, bias = 0;
    bool has_bias = true;
    Conv2d(AutoFerroxEngine<T>& g, size_t cin, size_t cout, size_t k, size_t s, size_t p, const T* w, const T* b)
        : in_channels(cin), out_channels(cout), kernel(k, k), stride(s, s), padding(p, p) {
        weight = g.create_variable(HipStorage<T>::from_vec(w, {cout, cin, k, k}), true);
        has_bias = b != nullptr;
        if (has_bias) bias = g.create_variable(HipStorage<T>::from_vec(b, {cout}), true);
    }
    NodeId forward(AutoFerroxEngine<T>& g, NodeId input) override {
        const Shape& s = g.get_tensor(input)->shape();
        if (s.size() != 4) throw Error("Conv2d requires 4D input [batch, channels, height, width], got shape " + fmt_shape(s));
        if (s[1] != in_channels) {
            std::ostringstream m;
            m << "Input channels " << s[1] << " don't match layer channels " << in_channels;
            throw Error(m.str());
        }
        const NodeId conv = g.apply_operation(std::make_unique<Conv2dOp<T>>(stride, padding), {input, weight});
        if (!has_bias) return conv;
        const NodeId bb = reshape_and_broadcast<T>(bias, conv, g);
        return g.apply_operation(std::make_unique<Add<T>>(), {conv, bb});
    }
    std::vector<NodeId> parameters() const override { return has_bias ? std::vector<NodeId>{weight, bias} : std::vector<NodeId>{weight}; }
};

template <typename T> struct ReLU : Module<T> {  // src/nn/layers/activation.rs:47-80
    NodeId forward(AutoFerroxEngine<T>& g, NodeId input) override { return g.apply_operation(std::make_unique<ReLUOp<T>>(), {input}); }
};

template <typename T> struct Pool2d : Module<T> {  // nn::MaxPool2d / AvgPool2d, src/nn/layers/pooling.rs
    bool is_max;
    size_t kernel, stride, padding;
    Pool2d(bool mx, size_t k, size_t s, size_t p) : is_max(mx), kernel(k), stride(s), padding(p) {}
    NodeId forward(AutoFerroxEngine<T>& g, NodeId input) override {
        return g.apply_operation(std::make_unique<Pool2dOp<T>>(is_max, kernel, stride, padding), {input});
    }
};

template <typename T> struct Flatten : Module<T> {  // src/nn/layers/pooling.rs:100-140 (batch-first)
    NodeId forward(AutoFerroxEngine<T>& g, NodeId input) override {
        const Shape& s = g.get_tensor(input)->shape();
        size_t rest = 1;
        for (size_t i = 1; i < s.size(); ++i) rest *= s[i];
        return g.apply_operation(std::make_unique<Reshape<T>>(Shape{s[0], rest}), {input});
    }
};

// BatchNorm composed from graph operators exactly as src/nn/layers/norm.rs:167-336 does (weight = gamma, bias = beta,
// running statistics updated outside the graph with the biased batch variance, norm.rs:127-164).
template <typename T> struct BatchNorm : Module<T> {
    size_t num_features;
    double eps, momentum;
    bool track_running_stats = true, training = true;
    NodeId weight = 0, bias = 0;
    Tensor<T> running_mean, running_var;
    size_t num_batches_tracked = 0;
    BatchNorm(AutoFerroxEngine<T>& g, size_t c, double eps_, double mom, const T* w, const T* b) : num_features(c), eps(eps_), momentum(mom) {
        weight = g.create_variable(HipStorage<T>::from_vec(w, {c}), true);
        bias = g.create_variable(HipStorage<T>::from_vec(b, {c}), true);
        running_mean = HipStorage<T>::zeros({c});  // norm.rs:75-84
        running_var = HipStorage<T>::ones({c});
    }
    void set_training(bool t) override { training = t; }
    std::vector<NodeId> parameters() const override { return {weight, bias}; }
    std::vector<const HipStorage<T>*> state() const override { return {running_mean.get(), running_var.get()}; }
    NodeId forward(AutoFerroxEngine<T>& g, NodeId input) override {
        if (g.get_tensor(input)->ndim() < 2) throw Error("BatchNorm requires at least 2D input [batch_size, features]");
        return (training || !track_running_stats) ? forward_training(g, input) : forward_inference(g, input);
    }

  private:
    void update_running_stats(const HipStorage<T>& batch_mean, const HipStorage<T>& batch_var) {  // norm.rs:127-164
        if (!track_running_stats || !training) return;
        const T mom = (T)momentum, om = (T)(1.0 - momentum);
        ++num_batches_tracked;
        {
            Tensor<T> a = running_mean->mul_scalar(om), b = batch_mean.mul_scalar(mom);
            running_mean = a->add(*b);
        }
        {
            Tensor<T> a = running_var->mul_scalar(om), b = batch_var.mul_scalar(mom);
            running_var = a->add(*b);
        }
    }
    NodeId forward_training(AutoFerroxEngine<T>& g, NodeId input) {  // norm.rs:192-259
        const std::vector<size_t> axes = g.get_tensor(input)->ndim() == 4 ? std::vector<size_t>{0, 2, 3} : std::vector<size_t>{0};
        const NodeId batch_mean = g.apply_operation(std::make_unique<Mean<T>>(axes, false), {input});
        const NodeId mean_b = reshape_and_broadcast<T>(batch_mean, input, g);
        const NodeId centered = g.apply_operation(std::make_unique<Sub<T>>(), {input, mean_b});
        const NodeId sq = g.apply_operation(std::make_unique<Mul<T>>(), {centered, centered});
        const NodeId variance = g.apply_operation(std::make_unique<Mean<T>>(axes, false), {sq});
        const NodeId var_b = reshape_and_broadcast<T>(variance, input, g);
        if (track_running_stats) update_running_stats(*g.get_tensor(batch_mean), *g.get_tensor(variance));
        return finish(g, centered, var_b);
    }
    NodeId forward_inference(AutoFerroxEngine<T>& g, NodeId input) {  // norm.rs:261-290
        const NodeId rm = g.create_variable(running_mean->clone_storage(), false);
        const NodeId rv = g.create_variable(running_var->clone_storage(), false);
        const NodeId mean_b = reshape_and_broadcast<T>(rm, input, g);
        const NodeId centered = g.apply_operation(std::make_unique<Sub<T>>(), {input, mean_b});
        return finish(g, centered, rv);
    }
    NodeId finish(AutoFerroxEngine<T>& g, NodeId centered, NodeId variance) {  // norm.rs:292-336
        const NodeId vpe = g.apply_operation(std::make_unique<AddScalar<T>>((T)eps), {variance});
        const NodeId sd = g.apply_operation(std::make_unique<Sqrt<T>>(), {vpe});
        const NodeId sd_b = reshape_and_broadcast<T>(sd, centered, g);
        const NodeId normalized = g.apply_operation(std::make_unique<Div<T>>(), {centered, sd_b});
        const NodeId w_b = reshape_and_broadcast<T>(weight, normalized, g);
        const NodeId scaled = g.apply_operation(std::make_unique<Mul<T>>(), {normalized, w_b});
        const NodeId b_b = reshape_and_broadcast<T>(bias, normalized, g);
        return g.apply_operation(std::make_unique<Add<T>>(), {scaled, b_b});
    }
};

// GlobalAvgPool2d(flatten = false), src/nn/layers/pooling.rs:604-623: Mean over axes (2, 3) with keep_dims
template <typename T> struct GlobalAvgPool2d : Module<T> {
    NodeId forward(AutoFerroxEngine<T>& g, NodeId input) override {
        if (g.get_tensor(input)->ndim() != 4) throw Error("GlobalAvgPool2d requires 4D input [batch, channels, height, width]");
        return g.apply_operation(std::make_unique<Mean<T>>(std::vector<size_t>{2, 3}, true), {input});
    }
};

// splitmix64 (Steele, Lea & Flood): element i of a dropout mask takes the 53-bit uniform of splitmix64(seed + i),
// the same stream as fx_dropout, so host-built and device-built masks agree.
inline double splitmix64_uniform(uint64_t x) {
    x += 0x9e3779b97f4a7c15ull;
    x = (x ^ (x >> 30)) * 0xbf58476d1ce4e5b9ull;
    x = (x ^ (x >> 27)) * 0x94d049bb133111ebull;
    x ^= x >> 31;
    return (double)(x >> 11) * (1.0 / 9007199254740992.0);
}

// Dropout, src/nn/layers/dropout.rs:56-136: the mask is drawn on the host, one f64 uniform per element, uploaded as
// a constant node and multiplied in.  (The reference's generator is unseeded; call k here uses seed + k * 2^32.)
template <typename T> struct Dropout : Module<T> {
    double p;
    uint64_t seed, calls = 0;
    bool training = true;
    Dropout(double p_, uint64_t seed_) : p(p_), seed(seed_) {
        if (!(p >= 0.0 && p <= 1.0)) throw Error("Dropout probability must be between 0.0 and 1.0");
    }
    void set_training(bool t) override { training = t; }
    NodeId forward(AutoFerroxEngine<T>& g, NodeId input) override {
        if (!training || p == 0.0) return input;
        const Shape shape = g.get_tensor(input)->shape();
        if (p == 1.0) return g.create_variable(HipStorage<T>::zeros(shape), false);
        const size_t n = numel(shape);
        const double keep = 1.0 - p;
        const T scale = (T)(1.0 / keep);
        std::vector<T> mask(n);
        const uint64_t s = seed + (calls++ << 32);
        for (size_t i = 0; i < n; ++i) mask[i] = splitmix64_uniform(s + i) < keep ? scale : T(0);
        const NodeId m = g.create_variable(HipStorage<T>::from_vec(mask.data(), shape), false);
        return g.apply_operation(std::make_unique<Mul<T>>(), {input, m});
    }
};

// ---- CCELoss (softmax cross-entropy, mean reduction): src/nn/losses/classification.rs:191-257 -------------------
template <typename T> NodeId cce_loss(AutoFerroxEngine<T>& g, NodeId predictions, NodeId targets) {
    const NodeId probs_raw = g.apply_operation(std::make_unique<Softmax<T>>(1), {predictions});
    const NodeId probs = g.apply_operation(std::make_unique<Clamp<T>>((T)1e-8, (T)(1.0 - 1e-8)), {probs_raw});
    const NodeId logp = g.apply_operation(std::make_unique<Log<T>>(), {probs});
    const NodeId tl = g.apply_operation(std::make_unique<Mul<T>>(), {targets, logp});
    const NodeId ce = g.apply_operation(std::make_unique<Sum<T>>(std::vector<size_t>{1}, true), {tl});
    const NodeId neg = g.apply_operation(std::make_unique<Neg<T>>(), {ce});
    return g.apply_operation(std::make_unique<Mean<T>>(), {neg});
}

// ---- optimizers: src/nn/optim ---------------------------------------------------------------------------------
// ParameterGroup, src/nn/optim/mod.rs:203-258.  The reference keeps the ids in a HashSet (iteration order arbitrary);
// here they are kept unique in insertion order.
template <typename T> struct ParameterGroup {
    std::vector<NodeId> params;
    std::optional<T> lr, weight_decay, momentum;
    std::string name;
    explicit ParameterGroup(std::string n = "default") : name(std::move(n)) {}
    void add_param(NodeId id) {
        if (std::find(params.begin(), params.end(), id) == params.end()) params.push_back(id);
    }
    SerializableParameterGroup to_serializable() const {  // From<&ParameterGroup>, mod.rs:189-201 (ids sorted: a HashSet has no order)
        SerializableParameterGroup g;
        g.params.assign(params.begin(), params.end());
        std::sort(g.params.begin(), g.params.end());
        if (lr) g.lr = (double)*lr;
        if (weight_decay) g.weight_decay = (double)*weight_decay;
        if (momentum) g.momentum = (double)*momentum;
        g.name = name;
        return g;
    }
    static ParameterGroup from_serializable(const SerializableParameterGroup& s) {  // mod.rs:241-257
        ParameterGroup g(s.name);
        for (size_t id : s.params) g.add_param(id);
        if (s.lr) g.lr = (T)*s.lr;
        if (s.weight_decay) g.weight_decay = (T)*s.weight_decay;
        if (s.momentum) g.momentum = (T)*s.momentum;
        return g;
    }
};

template <typename T> struct Optimizer {  // trait Optimizer, src/nn/optim/mod.rs:328-378
    virtual ~Optimizer() = default;
    virtual void step(AutoFerroxEngine<T>& g) = 0;
    virtual OptimizerStateDict state_dict() const = 0;
    virtual void load_state_dict(const OptimizerStateDict& sd) = 0;
    virtual T get_lr() const = 0;
    virtual void set_lr(T lr) = 0;
    std::vector<ParameterGroup<T>> param_groups;  // new() creates the "default" group

    void add_param(size_t group, NodeId id) { param_groups.at(group).add_param(id); }
    void add_param_group(ParameterGroup<T> group) {
        if (group.params.empty()) throw Error("Invalid parameter group configuration");
        param_groups.push_back(std::move(group));
    }
    // every node id held by some group
    std::set<NodeId> all_params() const {
        std::set<NodeId> r;
        for (const auto& g : param_groups) r.insert(g.params.begin(), g.params.end());
        return r;
    }

  protected:
    void save_groups(OptimizerStateDict& sd) const {  // add_parameter_group, mod.rs:304-311
        for (const auto& g : param_groups) sd.parameter_groups.push_back(g.to_serializable());
    }
    void load_groups(const OptimizerStateDict& sd) {  // param_groups.clear(); push every saved group
        param_groups.clear();
        for (const auto& g : sd.parameter_groups) param_groups.push_back(ParameterGroup<T>::from_serializable(g));
    }
    static T hyper(const OptimizerStateDict& sd, const char* name, T current) {
        auto it = sd.hyperparameters.find(name);
        return it == sd.hyperparameters.end() ? current : (T)it->second;
    }
    // Restores the buffers of one kind.  The reference inserts whatever the file holds; a buffer for a node that no
    // restored group names could never be used again and a buffer of another shape would be read past its end by a
    // fused update, so both are errors here.
    void load_buffers(const OptimizerStateDict& sd, const char* type, std::map<NodeId, Tensor<T>>& into) const {
        const std::set<NodeId> known = all_params();
        for (const auto& kv : sd.parameter_buffers) {
            const TensorBuffer& b = kv.second;
            if (b.buffer_type != type) continue;
            if (!known.count(b.node_id))
                throw Error("optimizer state: buffer '" + std::string(type) + "' names node " + std::to_string(b.node_id) + ", which is in no parameter group");
            into[b.node_id] = b.template to_tensor<T>();
        }
    }
    static void check_buffer(const HipStorage<T>& buf, const HipStorage<T>& w, const char* type, NodeId id) {
        if (buf.shape() != w.shape())
            throw Error("optimizer state: buffer '" + std::string(type) + "' of node " + std::to_string(id) + " has shape " + fmt_shape(buf.shape()) +
                        ", the parameter has " + fmt_shape(w.shape()));
    }
};

// Adam::state_dict / load_state_dict, src/nn/optim/adam.rs:391-556, shared by the composed and the fused optimizer
template <typename T, class Opt> OptimizerStateDict adam_state_dict(const Opt& o) {
    OptimizerStateDict sd;
    sd.optimizer_type = "Adam";
    sd.step_count = (uint64_t)o.step_count;
    sd.hyperparameters["lr"] = (double)o.lr;
    sd.hyperparameters["beta1"] = (double)o.beta1;
    sd.hyperparameters["beta2"] = (double)o.beta2;
    sd.hyperparameters["eps"] = (double)o.eps;
    sd.hyperparameters["weight_decay"] = (double)o.weight_decay;
    sd.hyperparameters["amsgrad"] = o.amsgrad ? 1.0 : 0.0;
    for (const auto& kv : o.m1) sd.template add_buffer<T>(kv.first, *kv.second, "first_moment");
    for (const auto& kv : o.m2) sd.template add_buffer<T>(kv.first, *kv.second, "second_moment");
    if (o.amsgrad)
        for (const auto& kv : o.mmax) sd.template add_buffer<T>(kv.first, *kv.second, "max_second_moment");
    return sd;
}

// bias corrections, adam.rs:110-126
template <typename T> void adam_bias_corrections(T beta1, T beta2, long step_count, T& bc1, T& bc2) {
    const T stepf = (T)step_count;
    const T b1p = std::max((T)std::pow(beta1, stepf), (T)1e-8), b2p = std::max((T)std::pow(beta2, stepf), (T)1e-8);
    bc1 = T(1) - b1p;
    bc2 = T(1) - b2p;
}

template <typename T> struct SGD : Optimizer<T> {  // src/nn/optim/sgd.rs:11-360
    T lr, momentum, weight_decay;
    bool nesterov;
    std::map<NodeId, Tensor<T>> momentum_buffers;
    explicit SGD(T lr_, T momentum_ = T(0), T wd = T(0), bool nesterov_ = false)  // SGD::new, sgd.rs:28-45
        : lr(lr_), momentum(momentum_), weight_decay(wd), nesterov(nesterov_) {
        ParameterGroup<T> g("default");
        g.lr = lr;
        g.weight_decay = weight_decay;
        g.momentum = momentum;
        this->param_groups.push_back(std::move(g));
    }
    T get_lr() const override { return lr; }
    void set_lr(T v) override {  // sgd.rs:271-276
        lr = v;
        for (auto& g : this->param_groups) g.lr = v;
    }
    // clip_grad_norm, sgd.rs:56-101: global L2 norm over every group's gradients (one host read per parameter);
    // when it exceeds max_norm every gradient is scaled by max_norm / norm (engine.clip_gradient).
    T clip_grad_norm(AutoFerroxEngine<T>& g, T max_norm) {
        T total_sq = T(0);
        for (const auto& group : this->param_groups)
            for (NodeId p : group.params)
                if (const HipStorage<T>* grad = g.get_gradient(p)) {
                    Tensor<T> sq = grad->mul(*grad);
                    total_sq += sq->sum(nullptr, false)->first();
                }
        const T total = std::sqrt(total_sq);
        if (total > max_norm) {
            const T coef = max_norm / total;
            for (const auto& group : this->param_groups)
                for (NodeId p : group.params) g.clip_gradient(p, coef);
        }
        return total;
    }
    void step(AutoFerroxEngine<T>& g) override {  // sgd.rs:210-245
        for (const auto& group : this->param_groups) {
            const T glr = group.lr.value_or(lr), gwd = group.weight_decay.value_or(weight_decay), gmom = group.momentum.value_or(momentum);
            for (NodeId p : group.params) {
                const HipStorage<T>* grad = g.get_gradient(p);
                if (!grad) continue;
                const HipStorage<T>* w = g.get_tensor(p);
                if (!w) throw Error("Parameter not found for node " + std::to_string(p));
                Tensor<T> effective;  // apply_weight_decay, sgd.rs:117-134 (rate 0 returns grad.clone())
                if (gwd == T(0)) effective = grad->clone_storage();
                else {
                    Tensor<T> term = w->mul_scalar(gwd);
                    effective = grad->add(*term);
                }
                Tensor<T> nw;
                if (gmom != T(0)) {  // compute_update, sgd.rs:173-206
                    auto it = momentum_buffers.find(p);
                    if (it == momentum_buffers.end()) it = momentum_buffers.emplace(p, HipStorage<T>::zeros(w->shape())).first;
                    else this->check_buffer(*it->second, *w, "momentum", p);
                    {
                        Tensor<T> scaled = it->second->mul_scalar(gmom);
                        it->second = scaled->add(*effective);
                    }
                    if (nesterov) {
                        Tensor<T> look = it->second->mul_scalar(gmom);
                        Tensor<T> update = look->add(*effective);
                        nw = apply_lr(glr, *w, *update);
                    } else nw = apply_lr(glr, *w, *it->second);
                } else nw = apply_lr(glr, *w, *effective);
                g.update_parameter(p, std::move(nw));
            }
        }
    }
    OptimizerStateDict state_dict() const override {  // sgd.rs:278-322
        OptimizerStateDict sd;
        sd.optimizer_type = "SGD";
        sd.step_count = 0;
        sd.hyperparameters["lr"] = (double)lr;
        sd.hyperparameters["momentum"] = (double)momentum;
        sd.hyperparameters["weight_decay"] = (double)weight_decay;
        sd.hyperparameters["nesterov"] = nesterov ? 1.0 : 0.0;
        this->save_groups(sd);
        for (const auto& kv : momentum_buffers) sd.template add_buffer<T>(kv.first, *kv.second, "momentum");
        return sd;
    }
    void load_state_dict(const OptimizerStateDict& sd) override {  // sgd.rs:324-360
        if (sd.optimizer_type != "SGD") throw Error("Type mismatch: Expected SGD state dict, got " + sd.optimizer_type);
        momentum_buffers.clear();
        lr = this->hyper(sd, "lr", lr);
        momentum = this->hyper(sd, "momentum", momentum);
        weight_decay = this->hyper(sd, "weight_decay", weight_decay);
        auto it = sd.hyperparameters.find("nesterov");
        if (it != sd.hyperparameters.end()) nesterov = it->second > 0.5;
        this->load_groups(sd);
        this->load_buffers(sd, "momentum", momentum_buffers);
    }

  protected:
    static Tensor<T> apply_lr(T glr, const HipStorage<T>& w, const HipStorage<T>& update) {  // sgd.rs:136-150
        Tensor<T> scaled = update.mul_scalar(glr);
        return w.sub(*scaled);
    }
};

template <typename T> struct Adam : Optimizer<T> {  // src/nn/optim/adam.rs:11-556
    T lr, beta1, beta2, eps, weight_decay;
    bool amsgrad;
    long step_count = 0;
    std::map<NodeId, Tensor<T>> m1, m2, mmax;
    Adam(T lr_, T b1, T b2, T eps_, T wd, bool amsgrad_ = false)  // Adam::new, adam.rs:40-62
        : lr(lr_), beta1(b1), beta2(b2), eps(eps_), weight_decay(wd), amsgrad(amsgrad_) {
        ParameterGroup<T> g("default");
        g.lr = lr;
        g.weight_decay = weight_decay;
        this->param_groups.push_back(std::move(g));
    }
    T get_lr() const override { return lr; }
    void set_lr(T v) override {
        lr = v;
        for (auto& g : this->param_groups) g.lr = v;
    }
    void step(AutoFerroxEngine<T>& g) override {  // adam.rs:288-358
        step_count += 1;
        T bc1, bc2;
        adam_bias_corrections(beta1, beta2, step_count, bc1, bc2);
        for (const auto& group : this->param_groups) {
            const T glr = group.lr.value_or(lr), gwd = group.weight_decay.value_or(weight_decay);
            for (NodeId p : group.params) {
                const HipStorage<T>* grad = g.get_gradient(p);
                if (!grad) continue;
                if (!g.get_tensor(p)) throw Error("Parameter not found for node " + std::to_string(p));
                Tensor<T> w = g.get_tensor(p)->clone_storage();  // adam.rs:299-302 clones the parameter
                if (!m1.count(p)) m1[p] = HipStorage<T>::zeros(w->shape());
                else this->check_buffer(*m1[p], *w, "first_moment", p);
                {  // first moment: beta1*m + (1-beta1)*g
                    Tensor<T> a = m1[p]->mul_scalar(beta1), b = grad->mul_scalar(T(1) - beta1);
                    m1[p] = a->add(*b);
                }
                if (!m2.count(p)) m2[p] = HipStorage<T>::zeros(w->shape());
                else this->check_buffer(*m2[p], *w, "second_moment", p);
                {  // second moment: beta2*v + (1-beta2)*g*g
                    Tensor<T> gg = grad->mul(*grad);
                    Tensor<T> a = m2[p]->mul_scalar(beta2), b = gg->mul_scalar(T(1) - beta2);
                    m2[p] = a->add(*b);
                }
                Tensor<T> second;
                if (amsgrad) {  // running maximum of the second moment, adam.rs:203-221
                    if (!mmax.count(p)) mmax[p] = HipStorage<T>::zeros(w->shape());
                    else this->check_buffer(*mmax[p], *w, "max_second_moment", p);
                    mmax[p] = mmax[p]->max(*m2[p]);
                    second = mmax[p]->clone_storage();
                } else second = m2[p]->clone_storage();  // take_current_buffer clones
                Tensor<T> t1 = second->div_scalar(bc2);
                Tensor<T> t2 = t1->sqrt();
                Tensor<T> denom = t2->add_scalar(eps);
                Tensor<T> first = m1[p]->clone_storage();
                Tensor<T> u1 = first->div_scalar(bc1);
                Tensor<T> u2 = u1->div(*denom);
                Tensor<T> update = u2->mul_scalar(glr);
                Tensor<T> nw;
                if (gwd != T(0)) {  // decoupled weight decay, adam.rs:259-282
                    Tensor<T> wd = w->mul_scalar(gwd * glr);
                    Tensor<T> s1 = w->sub(*update);
                    nw = s1->sub(*wd);
                } else nw = w->sub(*update);
                g.update_parameter(p, std::move(nw));
            }
        }
    }
    OptimizerStateDict state_dict() const override {
        OptimizerStateDict sd = adam_state_dict<T>(*this);
        this->save_groups(sd);
        return sd;
    }
    void load_state_dict(const OptimizerStateDict& sd) override { adam_load(*this, sd); }

    // Adam::load_state_dict, adam.rs:463-556 (shared with the fused optimizer)
    template <class Opt> static void adam_load(Opt& o, const OptimizerStateDict& sd) {
        if (sd.optimizer_type != "Adam") throw Error("Type mismatch: Expected Adam state dict, got " + sd.optimizer_type);
        o.m1.clear();
        o.m2.clear();
        o.mmax.clear();
        o.step_count = (long)sd.step_count;
        o.lr = Optimizer<T>::hyper(sd, "lr", o.lr);
        o.beta1 = Optimizer<T>::hyper(sd, "beta1", o.beta1);
        o.beta2 = Optimizer<T>::hyper(sd, "beta2", o.beta2);
        o.eps = Optimizer<T>::hyper(sd, "eps", o.eps);
        o.weight_decay = Optimizer<T>::hyper(sd, "weight_decay", o.weight_decay);
        auto it = sd.hyperparameters.find("amsgrad");
        if (it != sd.hyperparameters.end()) o.amsgrad = it->second > 0.5;
        o.load_groups(sd);
        o.load_buffers(sd, "first_moment", o.m1);
        o.load_buffers(sd, "second_moment", o.m2);
        if (o.amsgrad) o.load_buffers(sd, "max_second_moment", o.mmax);
    }
};

}  // namespace ferrox
