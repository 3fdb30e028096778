// Fused variants of the layers, the loss and the optimizers: what Ferrox's nn layer code looks like once it calls
// the fused entry points of include/ferrox_hip.h instead of composing every step from storage ops.  They plug
// into the same AutoFerroxEngine as graph operators; values equal the composed path (same arithmetic per element,
// reductions to tolerance).
//   Linear   : x.W^T through the transposed-operand GEMM (no Transpose node, linear.rs:225-228), bias (+ReLU) in
//              place; backward dX = G.W, dW = G^T.X directly in W's layout (matrix.rs:30-55 materialises two
//              transposes and Transpose::gradient a third), db in one pass (basic.rs:10-53 takes one per axis)
//   Conv2d   : conv, bias (+ReLU) in place (conv2d.rs:203-213 materialises the broadcast bias first); backward
//              skips the data gradient of an input that needs none (the first layer)
//   CCELoss  : one forward and one backward kernel (classification.rs:191-257 builds 7 nodes)
//   BatchNorm: statistics (+ running update), normalise and backward kernels (norm.rs:192-336 builds ~15 nodes);
//              GlobalAvgPool2d as one reduction; Dropout with the mask drawn on the device
//   Adam/SGD : one in-place launch for all parameters (adam.rs:288-358 runs ~14 kernels per parameter and clones the
//              parameter and moments)
#pragma once
#include "autograd.hpp"

namespace ferrox {

template <typename T> struct FusedApi;
#define FERROX_FUSED_API(T, S)                                                                                         \
    template <> struct FusedApi<T> {                                                                                   \
        static int bias_act(fx_ctx* c, T* y, const T* b, int64_t o, int64_t C, int64_t i, int act) { return fx_bias_act_##S(c, y, b, o, C, i, act); } \
        static int bias_grad(fx_ctx* c, const T* g, T* out, int64_t o, int64_t C, int64_t i) { return fx_bias_grad_##S(c, g, out, o, C, i); } \
        static int sce_fwd(fx_ctx* c, const T* x, const T* y, T* p, T* l, int64_t B, int64_t C) { return fx_softmax_ce_fwd_##S(c, x, y, p, l, B, C); } \
        static int sce_bwd(fx_ctx* c, const T* p, const T* y, const T* g, T* d, int64_t B, int64_t C) { return fx_softmax_ce_bwd_##S(c, p, y, g, d, B, C); } \
        static int sce_fwd_unit(fx_ctx* c, const T* x, const T* y, T* p, T* l, T* d, int64_t B, int64_t C) {            \
            return fx_softmax_ce_fwd_unit_grad_##S(c, x, y, p, l, d, B, C);                                            \
        }                                                                                                              \
        static int adam(fx_ctx* c, T* p, const T* g, T* m, T* v, int64_t n, T lr, T b1, T b2, T eps, T wd, T bc1, T bc2) { \
            return fx_adam_step_##S(c, p, g, m, v, n, lr, b1, b2, eps, wd, bc1, bc2);                                  \
        }                                                                                                              \
        static int sgd(fx_ctx* c, T* p, const T* g, int64_t n, T lr) { return fx_sgd_step_##S(c, p, g, n, lr); }       \
        static int adam_multi(fx_ctx* c, int k, T* const* p, const T* const* g, T* const* m, T* const* v, const int64_t* n, T lr, T b1, T b2, \
                              T eps, T wd, T bc1, T bc2) {                                                             \
            return fx_adam_step_multi_##S(c, k, p, g, m, v, n, lr, b1, b2, eps, wd, bc1, bc2);                         \
        }                                                                                                              \
        static int adam_multi_bc(fx_ctx* c, int k, T* const* p, const T* const* g, T* const* m, T* const* v, T* const* x, const int64_t* n, T lr, \
                                 T b1, T b2, T eps, T wd, const T* bc) {                                                \
            return fx_adam_step_multi_bc_##S(c, k, p, g, m, v, x, n, lr, b1, b2, eps, wd, bc);                         \
        }                                                                                                              \
        static int sgd_multi(fx_ctx* c, int k, T* const* p, const T* const* g, const int64_t* n, T lr) { return fx_sgd_step_multi_##S(c, k, p, g, n, lr); } \
        static int sgd_momentum_multi(fx_ctx* c, int k, T* const* p, const T* const* g, T* const* b, const int64_t* n, T lr, T mom, T wd, int nes) { \
            return fx_sgd_momentum_step_multi_##S(c, k, p, g, b, n, lr, mom, wd, nes);                                 \
        }                                                                                                              \
        static int adam_amsgrad_multi(fx_ctx* c, int k, T* const* p, const T* const* g, T* const* m, T* const* v, T* const* x, const int64_t* n, \
                                      T lr, T b1, T b2, T eps, T wd, T bc1, T bc2) {                                   \
            return fx_adam_amsgrad_step_multi_##S(c, k, p, g, m, v, x, n, lr, b1, b2, eps, wd, bc1, bc2);              \
        }                                                                                                              \
        static int relu_bwd(fx_ctx* c, const T* g, const T* x, T* o, int64_t n) { return fx_relu_bwd_##S(c, g, x, o, n); } \
        static int relu_bias_grad(fx_ctx* c, const T* g, const T* y, T* gm, T* db, int64_t o, int64_t C, int64_t i) {  \
            return fx_relu_bwd_bias_grad_##S(c, g, y, gm, db, o, C, i);                                                \
        }                                                                                                              \
        static int linear_bwd(fx_ctx* c, int64_t B, int64_t I, int64_t O, const T* g, const T* W, const T* X, T* dX, T* dW, T* db, int rb) { \
            return fx_linear_bwd_##S(c, B, I, O, g, W, X, dX, dW, db, rb);                                             \
        }                                                                                                              \
        static int gemm_tn_colsum(fx_ctx* c, int64_t M, int64_t N, int64_t K, const T* A, const T* B, T* C, T* s) {      \
            return fx_gemm_tn_colsum_##S(c, M, N, K, A, B, C, s);                                                      \
        }                                                                                                              \
        static int gemm_bias(fx_ctx* c, int ta, int tb, int64_t M, int64_t N, int64_t K, const T* A, const T* B, const T* b, T* C, int act) { \
            return fx_gemm_bias_act_##S(c, ta, tb, M, N, K, A, B, b, C, act);                                          \
        }                                                                                                              \
        static int conv_bias(fx_ctx* c, const T* x, const T* w, const T* b, T* y, const int64_t* d, int act) {         \
            return fx_conv2d_fwd_bias_act_##S(c, x, w, b, y, d[0], d[1], d[2], d[3], d[4], d[5], d[6], d[7], d[8], d[9], d[10], act, nullptr, 0); \
        }                                                                                                              \
        static int conv_bwd_relu_supported(fx_ctx* c, int kind, const int64_t* d) {                                    \
            return fx_conv2d_bwd_relu_supported(c, kind, sizeof(T) == 8 ? FX_F64 : FX_F32, d[0], d[1], d[2], d[3], d[4], d[5], d[6], d[7], d[8], d[9], d[10]); \
        }                                                                                                              \
        static int conv_wgrad_relu_bias(fx_ctx* c, const T* x, const T* g, const T* act, T* dw, T* db, const int64_t* d) { \
            return fx_conv2d_wgrad_relu_bias_##S(c, x, g, act, dw, db, d[0], d[1], d[2], d[3], d[4], d[5], d[6], d[7], d[8], d[9], d[10], nullptr, 0); \
        }                                                                                                              \
        static int conv_dgrad_relu(fx_ctx* c, const T* g, const T* act, const T* w, T* dx, const int64_t* d) {         \
            return fx_conv2d_dgrad_relu_##S(c, g, act, w, dx, d[0], d[1], d[2], d[3], d[4], d[5], d[6], d[7], d[8], d[9], d[10]); \
        }                                                                                                              \
        static int bn_stats(fx_ctx* c, const T* x, T* m, T* v, T* rm, T* rv, double mom, int64_t o, int64_t C, int64_t i) { \
            return fx_batchnorm_stats_##S(c, x, m, v, rm, rv, mom, o, C, i);                                           \
        }                                                                                                              \
        static int bn_fwd(fx_ctx* c, const T* x, const T* m, const T* v, const T* g, const T* b, double eps, T* y, int64_t o, int64_t C, int64_t i, int act) { \
            return fx_batchnorm_fwd_##S(c, x, m, v, g, b, eps, y, o, C, i, act);                                       \
        }                                                                                                              \
        static int bn_bwd(fx_ctx* c, const T* dy, const T* x, const T* ya, const T* m, const T* v, const T* g, double eps, T* dx, T* dg, T* db, \
                          int64_t o, int64_t C, int64_t i, int batch_stats) {                                         \
            return fx_batchnorm_bwd_##S(c, dy, x, ya, m, v, g, eps, dx, dg, db, o, C, i, batch_stats);                 \
        }                                                                                                              \
        static int dropout(fx_ctx* c, const T* x, T* mask, T* y, int64_t n, double p, uint64_t seed) { return fx_dropout_##S(c, x, mask, y, n, p, seed); } \
        static int rmean(fx_ctx* c, const T* i, T* o, int64_t ou, int64_t ax, int64_t in) { return fx_reduce_mean_##S(c, i, o, ou, ax, in); } \
    };
FERROX_FUSED_API(float, f32)
FERROX_FUSED_API(double, f64)
#undef FERROX_FUSED_API

inline fx_ctx* fused_ctx() { return BackendManager::get().ctx(); }

// g * (y > 0): the ReLU mask taken from the activation's OUTPUT (y > 0 exactly when its input was > 0)
template <typename T> Tensor<T> relu_mask_grad(const HipStorage<T>& g, const HipStorage<T>& y) {
    Tensor<T> r = HipStorage<T>::alloc(g.shape());
    fx_ok(FusedApi<T>::relu_bwd(fused_ctx(), g.data(), y.data(), r->data(), (int64_t)g.size()));
    return r;
}

template <typename T> struct LinearFusedOp : Operator<T> {  // inputs: x [B, in], W [out, in], b [out]
    bool relu;
    explicit LinearFusedOp(bool relu_) : relu(relu_) {}
    Tensor<T> compute(const TensorRefs<T>& in) const override {
        const Shape &xs = in[0]->shape(), &ws = in[1]->shape();
        if (xs.size() != 2 || ws.size() != 2 || xs[1] != ws[1]) throw Error("Linear: input " + fmt_shape(xs) + " vs weight " + fmt_shape(ws));
        Tensor<T> y = HipStorage<T>::alloc({xs[0], ws[0]});
        fx_ok(FusedApi<T>::gemm_bias(fused_ctx(), 0, 1, (int64_t)xs[0], (int64_t)ws[0], (int64_t)xs[1], in[0]->data(), in[1]->data(),
                                     in[2]->data(), y->data(), relu ? 1 : 0));
        return y;
    }
    std::vector<Tensor<T>> gradient(Tensor<T> g, const TensorRefs<T>& in, const HipStorage<T>* out) const override {
        return gradient_needs(std::move(g), in, out, {true, true, true});
    }
    std::vector<Tensor<T>> gradient_needs(Tensor<T> g, const TensorRefs<T>& in, const HipStorage<T>* out,
                                          const std::vector<bool>& needs) const override {
        const Shape &xs = in[0]->shape(), &ws = in[1]->shape();
        const int64_t B = (int64_t)xs[0], I = (int64_t)xs[1], O = (int64_t)ws[0];
        std::vector<Tensor<T>> r(3);
        r[2] = HipStorage<T>::alloc({ws[0]});
        // the layer above may have handed g over already multiplied by this layer's ReLU mask (in the store of its data gradient)
        const bool premasked = relu && g->relu_masked_by == static_cast<const void*>(out);
        if (relu && !premasked) {  // mask and bias gradient in one pass over g
            Tensor<T> gm = HipStorage<T>::alloc(g->shape());
            fx_ok(FusedApi<T>::relu_bias_grad(fused_ctx(), g->data(), out->data(), gm->data(), r[2]->data(), B, O, 1));
            g = std::move(gm);
        }
        r[1] = HipStorage<T>::alloc(ws);
        // where no pass over g has produced it, the bias gradient (the column sums of g) comes out of the weight gradient's launch
        T* db = relu && !premasked ? nullptr : r[2]->data();
        if (needs[0]) {  // both products in one call (one launch where both are small)
            const bool below = this->input0_is_relu_output;  // x is the output of a ReLU: dX comes out times that ReLU's mask
            r[0] = HipStorage<T>::alloc(xs);
            fx_ok(FusedApi<T>::linear_bwd(fused_ctx(), B, I, O, g->data(), in[1]->data(), in[0]->data(), r[0]->data(), r[1]->data(), db,
                                          below ? 1 : 0));
            if (below) r[0]->relu_masked_by = static_cast<const void*>(in[0]);
        } else if (db) fx_ok(FusedApi<T>::gemm_tn_colsum(fused_ctx(), O, I, B, g->data(), in[0]->data(), r[1]->data(), db));
        else fx_ok(Api<T>::gemm(fused_ctx(), 1, 0, O, I, B, g->data(), in[0]->data(), r[1]->data()));
        return r;
    }
    size_t num_inputs() const override { return 3; }
    bool output_is_relu() const override { return relu; }
    const char* name() const override { return "LinearFused"; }
};

template <typename T> struct Conv2dFusedOp : Operator<T> {  // inputs: x [B,Cin,H,W], W [Cout,Cin,kh,kw], b [Cout]
    std::pair<size_t, size_t> stride, padding;
    bool relu;
    Conv2dFusedOp(std::pair<size_t, size_t> s, std::pair<size_t, size_t> p, bool relu_) : stride(s), padding(p), relu(relu_) {}
    Tensor<T> compute(const TensorRefs<T>& in) const override {
        const Shape &xs = in[0]->shape(), &ws = in[1]->shape();
        if (xs.size() != 4 || ws.size() != 4 || xs[1] != ws[1]) throw Error("Conv2d: input " + fmt_shape(xs) + " vs filter " + fmt_shape(ws));
        const int64_t d[11] = {(int64_t)xs[0], (int64_t)xs[1], (int64_t)xs[2], (int64_t)xs[3], (int64_t)ws[0], (int64_t)ws[2], (int64_t)ws[3],
                               (int64_t)stride.first, (int64_t)stride.second, (int64_t)padding.first, (int64_t)padding.second};
        Tensor<T> y = HipStorage<T>::alloc({xs[0], ws[0], (xs[2] + 2 * padding.first - ws[2]) / stride.first + 1,
                                            (xs[3] + 2 * padding.second - ws[3]) / stride.second + 1});
        fx_ok(FusedApi<T>::conv_bias(fused_ctx(), in[0]->data(), in[1]->data(), in[2]->data(), y->data(), d, relu ? 1 : 0));
        return y;
    }
    std::vector<Tensor<T>> gradient(Tensor<T> g, const TensorRefs<T>& in, const HipStorage<T>* out) const override {
        return gradient_needs(std::move(g), in, out, {true, true, true});
    }
    std::vector<Tensor<T>> gradient_needs(Tensor<T> g, const TensorRefs<T>& in, const HipStorage<T>* out,
                                          const std::vector<bool>& needs) const override {
        const Shape gs = g->shape();
        std::vector<Tensor<T>> r(3);
        r[2] = HipStorage<T>::alloc({gs[1]});
        if (relu && BackendManager::get().conv_grad_mode == 0) {
            // The consumers of the masked gradient apply the mask themselves while they stage g, and the weight-gradient kernel
            // leaves the bias gradient: no masked copy of g, no separate pass (where both kernels the layer needs exist).
            const Shape &xs = in[0]->shape(), &ws = in[1]->shape();
            const int64_t d[11] = {(int64_t)xs[0], (int64_t)xs[1], (int64_t)xs[2], (int64_t)xs[3], (int64_t)ws[0], (int64_t)ws[2], (int64_t)ws[3],
                                   (int64_t)stride.first, (int64_t)stride.second, (int64_t)padding.first, (int64_t)padding.second};
            if (FusedApi<T>::conv_bwd_relu_supported(fused_ctx(), FX_CONV_WGRAD, d) &&
                (!needs[0] || FusedApi<T>::conv_bwd_relu_supported(fused_ctx(), FX_CONV_DGRAD, d))) {
                r[1] = HipStorage<T>::alloc(ws);
                const int rc = FusedApi<T>::conv_wgrad_relu_bias(fused_ctx(), in[0]->data(), g->data(), out->data(), r[1]->data(), r[2]->data(), d);
                if (rc == FX_OK) {
                    if (needs[0]) {
                        r[0] = HipStorage<T>::alloc(xs);
                        fx_ok(FusedApi<T>::conv_dgrad_relu(fused_ctx(), g->data(), out->data(), in[1]->data(), r[0]->data(), d));
                    }
                    return r;
                }
                if (rc != FX_ERR_UNSUPPORTED) fx_ok(rc);  // a misaligned tensor: the separate passes below
                r[1].reset();
            }
        }
        if (relu) {  // mask and bias gradient in one pass over g
            Tensor<T> gm = HipStorage<T>::alloc(gs);
            fx_ok(FusedApi<T>::relu_bias_grad(fused_ctx(), g->data(), out->data(), gm->data(), r[2]->data(), (int64_t)gs[0], (int64_t)gs[1],
                                              (int64_t)(gs[2] * gs[3])));
            g = std::move(gm);
        } else fx_ok(FusedApi<T>::bias_grad(fused_ctx(), g->data(), r[2]->data(), (int64_t)gs[0], (int64_t)gs[1], (int64_t)(gs[2] * gs[3])));
        if (needs[0]) r[0] = g->deconv2d(*in[1], in[0]->shape(), stride, padding);
        r[1] = in[0]->cross_correlation2d(*g, in[1]->shape(), stride, padding);
        return r;
    }
    size_t num_inputs() const override { return 3; }
    const char* name() const override { return "Conv2dFused"; }
};

template <typename T> struct SoftmaxCEOp : Operator<T> {  // inputs: logits [B,C], targets [B,C]; output: scalar loss
    mutable Tensor<T> probs;        // kept for the backward pass
    mutable Tensor<T> unit_grad;    // d logits for an upstream gradient of 1, written by the forward launch (see below)
    const AutoFerroxEngine<T>* eng;  // or null
    // On an engine that seeds backward() from its one shared tensor of 1.0 (reuse_unit_seed) the loss is normally the root of
    // the tape and its upstream gradient that very tensor: the forward launch then also writes d logits for a gradient of 1,
    // and gradient() hands them out without a launch when the upstream gradient is that tensor (else it runs the kernel).
    explicit SoftmaxCEOp(const AutoFerroxEngine<T>* e = nullptr) : eng(e) {}
    Tensor<T> compute(const TensorRefs<T>& in) const override {
        const Shape& s = in[0]->shape();
        if (s.size() != 2 || in[1]->shape() != s) throw Error("CCELoss: predictions " + fmt_shape(s) + " vs targets " + fmt_shape(in[1]->shape()));
        probs = HipStorage<T>::alloc(s);
        Tensor<T> loss = HipStorage<T>::alloc({});
        if (eng && eng->reuse_unit_seed) {
            unit_grad = HipStorage<T>::alloc(s);
            fx_ok(FusedApi<T>::sce_fwd_unit(fused_ctx(), in[0]->data(), in[1]->data(), probs->data(), loss->data(), unit_grad->data(),
                                            (int64_t)s[0], (int64_t)s[1]));
        } else {
            unit_grad.reset();
            fx_ok(FusedApi<T>::sce_fwd(fused_ctx(), in[0]->data(), in[1]->data(), probs->data(), loss->data(), (int64_t)s[0], (int64_t)s[1]));
        }
        return loss;
    }
    std::vector<Tensor<T>> gradient(Tensor<T> g, const TensorRefs<T>& in, const HipStorage<T>*) const override {
        const Shape& s = in[0]->shape();
        std::vector<Tensor<T>> r(2);
        if (unit_grad && eng && eng->unit_seed_data() && g->data() == eng->unit_seed_data()) {
            r[0] = std::move(unit_grad);
            return r;
        }
        unit_grad.reset();
        r[0] = HipStorage<T>::alloc(s);
        fx_ok(FusedApi<T>::sce_bwd(fused_ctx(), probs->data(), in[1]->data(), g->data(), r[0]->data(), (int64_t)s[0], (int64_t)s[1]));
        return r;  // no gradient for the targets
    }
    size_t num_inputs() const override { return 2; }
    const char* name() const override { return "SoftmaxCE"; }
};

template <typename T> struct LinearFused : Module<T> {
    size_t in_features, out_features;
    NodeId weight = 0, bias = 0;
    bool relu;
    LinearFused(AutoFerroxEngine<T>& g, size_t in, size_t out, const T* w, const T* b, bool relu_) : in_features(in), out_features(out), relu(relu_) {
        weight = g.create_variable(HipStorage<T>::from_vec(w, {out, in}), true);
        bias = g.create_variable(HipStorage<T>::from_vec(b, {out}), true);
    }
    NodeId forward(AutoFerroxEngine<T>& g, NodeId input) override {
        return g.apply_operation(std::make_unique<LinearFusedOp<T>>(relu), {input, weight, bias});
    }
    std::vector<NodeId> parameters() const override { return {weight, bias}; }
};

template <typename T> struct Conv2dFused : Module<T> {
    std::pair<size_t, size_t> stride, padding;
    NodeId weight = 0, bias = 0;
    bool relu;
    Conv2dFused(AutoFerroxEngine<T>& g, size_t cin, size_t cout, size_t k, size_t s, size_t p, const T* w, const T* b, bool relu_)
        : stride(s, s), padding(p, p), relu(relu_) {
        weight = g.create_variable(HipStorage<T>::from_vec(w, {cout, cin, k, k}), true);
        bias = g.create_variable(HipStorage<T>::from_vec(b, {cout}), true);
    }
    NodeId forward(AutoFerroxEngine<T>& g, NodeId input) override {
        return g.apply_operation(std::make_unique<Conv2dFusedOp<T>>(stride, padding, relu), {input, weight, bias});
    }
    std::vector<NodeId> parameters() const override { return {weight, bias}; }
};

// BatchNorm as three kernels (statistics + running update, normalise, backward) instead of ~15 graph nodes.
// inputs: x [N, C, ...], gamma [C], beta [C].  The module's running statistics are updated in place by the
// statistics kernel (training) or read (inference).
template <typename T> struct BatchNormFusedOp : Operator<T> {
    double eps, momentum;
    bool relu;                                 // the ReLU that follows the layer, applied in the same kernels
    bool batch_stats;                          // training (or no running statistics): statistics of this batch
    HipStorage<T>*running_mean, *running_var;  // owned by the module; null when not tracked
    mutable Tensor<T> mean, var;               // batch statistics, kept for the backward pass
    BatchNormFusedOp(double eps_, double mom, bool relu_, bool batch, HipStorage<T>* rm, HipStorage<T>* rv)
        : eps(eps_), momentum(mom), relu(relu_), batch_stats(batch), running_mean(rm), running_var(rv) {}
    static void view(const Shape& s, int64_t& outer, int64_t& C, int64_t& inner) {
        outer = (int64_t)s[0];
        C = (int64_t)s[1];
        inner = 1;
        for (size_t i = 2; i < s.size(); ++i) inner *= (int64_t)s[i];
    }
    Tensor<T> compute(const TensorRefs<T>& in) const override {
        const Shape& xs = in[0]->shape();
        if (xs.size() < 2) throw Error("BatchNorm requires at least 2D input [batch_size, features]");
        int64_t outer, C, inner;
        view(xs, outer, C, inner);
        const T *m, *v;
        if (batch_stats) {
            mean = HipStorage<T>::alloc({(size_t)C});
            var = HipStorage<T>::alloc({(size_t)C});
            fx_ok(FusedApi<T>::bn_stats(fused_ctx(), in[0]->data(), mean->data(), var->data(), running_mean ? running_mean->data() : nullptr,
                                        running_var ? running_var->data() : nullptr, momentum, outer, C, inner));
            m = mean->data();
            v = var->data();
        } else {
            m = running_mean->data();
            v = running_var->data();
        }
        Tensor<T> y = HipStorage<T>::alloc(xs);
        fx_ok(FusedApi<T>::bn_fwd(fused_ctx(), in[0]->data(), m, v, in[1]->data(), in[2]->data(), eps, y->data(), outer, C, inner, relu ? 1 : 0));
        return y;
    }
    std::vector<Tensor<T>> gradient(Tensor<T> g, const TensorRefs<T>& in, const HipStorage<T>* out) const override {
        return gradient_needs(std::move(g), in, out, {true, true, true});
    }
    std::vector<Tensor<T>> gradient_needs(Tensor<T> g, const TensorRefs<T>& in, const HipStorage<T>* out, const std::vector<bool>& needs) const override {
        const Shape& xs = in[0]->shape();
        int64_t outer, C, inner;
        view(xs, outer, C, inner);
        Tensor<T> recomputed;
        if (relu && !out) {
            recomputed = compute(in);
            out = recomputed.get();
        }
        std::vector<Tensor<T>> r(3);
        if (needs[0]) r[0] = HipStorage<T>::alloc(xs);
        r[1] = HipStorage<T>::alloc({(size_t)C});
        r[2] = HipStorage<T>::alloc({(size_t)C});
        const T* m = batch_stats ? mean->data() : running_mean->data();
        const T* v = batch_stats ? var->data() : running_var->data();
        fx_ok(FusedApi<T>::bn_bwd(fused_ctx(), g->data(), in[0]->data(), relu ? out->data() : nullptr, m, v, in[1]->data(), eps, needs[0] ? r[0]->data() : nullptr,
                                  r[1]->data(), r[2]->data(), outer, C, inner, batch_stats ? 1 : 0));
        return r;
    }
    size_t num_inputs() const override { return 3; }
    bool cache_output() const override { return relu; }
    const char* name() const override { return "BatchNormFused"; }
};

template <typename T> struct BatchNormFused : Module<T> {
    double eps, momentum;
    bool track_running_stats = true, training = true, relu = false;
    NodeId weight = 0, bias = 0;
    Tensor<T> running_mean, running_var;
    BatchNormFused(AutoFerroxEngine<T>& g, size_t c, double eps_, double mom, const T* w, const T* b, bool relu_) : eps(eps_), momentum(mom), relu(relu_) {
        weight = g.create_variable(HipStorage<T>::from_vec(w, {c}), true);
        bias = g.create_variable(HipStorage<T>::from_vec(b, {c}), true);
        running_mean = HipStorage<T>::zeros({c});
        running_var = HipStorage<T>::ones({c});
    }
    void set_training(bool t) override { training = t; }
    std::vector<NodeId> parameters() const override { return {weight, bias}; }
    std::vector<const HipStorage<T>*> state() const override { return {running_mean.get(), running_var.get()}; }
    NodeId forward(AutoFerroxEngine<T>& g, NodeId input) override {
        const bool batch = training || !track_running_stats;
        const bool update = training && track_running_stats;
        return g.apply_operation(std::make_unique<BatchNormFusedOp<T>>(eps, momentum, relu, batch, (update || !batch) ? running_mean.get() : nullptr,
                                                                       (update || !batch) ? running_var.get() : nullptr),
                                 {input, weight, bias});
    }
};

// GlobalAvgPool2d as one reduction over the contiguous H*W run of every (n, c) instead of one per axis
template <typename T> struct GlobalAvgPoolFusedOp : Operator<T> {
    Tensor<T> compute(const TensorRefs<T>& in) const override {
        const Shape& s = in[0]->shape();
        if (s.size() != 4) throw Error("GlobalAvgPool2d requires 4D input [batch, channels, height, width]");
        Tensor<T> y = HipStorage<T>::alloc({s[0], s[1], 1, 1});
        fx_ok(FusedApi<T>::rmean(fused_ctx(), in[0]->data(), y->data(), (int64_t)(s[0] * s[1]), (int64_t)(s[2] * s[3]), 1));
        return y;
    }
    std::vector<Tensor<T>> gradient(Tensor<T> g, const TensorRefs<T>& in, const HipStorage<T>*) const override {  // Mean::gradient
        const Shape& s = in[0]->shape();
        Tensor<T> e = g->mul_scalar((T)(1.0 / (double)(s[2] * s[3])));
        e->broadcast_to(s);
        std::vector<Tensor<T>> r;
        r.push_back(std::move(e));
        return r;
    }
    size_t num_inputs() const override { return 1; }
    const char* name() const override { return "GlobalAvgPoolFused"; }
};
template <typename T> struct GlobalAvgPoolFused : Module<T> {
    NodeId forward(AutoFerroxEngine<T>& g, NodeId input) override {
        return g.apply_operation(std::make_unique<GlobalAvgPoolFusedOp<T>>(), {input});
    }
};

// Flatten as a view: the reshaped tensor aliases its input's memory (the graph keeps the input alive until its clean-up)
// instead of the copy that Reshape makes (src/ops/reshape.rs:4-55 clones the tensor first).  Same values, no kernel.
template <typename T> struct ReshapeViewOp : Operator<T> {
    Shape new_shape;
    explicit ReshapeViewOp(Shape s) : new_shape(std::move(s)) {}
    Tensor<T> compute(const TensorRefs<T>& in) const override {
        Tensor<T> r = HipStorage<T>::borrow(*in[0]);
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
    const char* name() const override { return "ReshapeView"; }
};
template <typename T> struct FlattenFused : Module<T> {  // src/nn/layers/pooling.rs:100-140 (batch-first)
    NodeId forward(AutoFerroxEngine<T>& g, NodeId input) override {
        const Shape& s = g.get_tensor(input)->shape();
        size_t rest = 1;
        for (size_t i = 1; i < s.size(); ++i) rest *= s[i];
        return g.apply_operation(std::make_unique<ReshapeViewOp<T>>(Shape{s[0], rest}), {input});
    }
};

// Dropout with the mask drawn on the device (same stream as the host-built mask of Dropout)
template <typename T> struct DropoutFusedOp : Operator<T> {
    double p;
    uint64_t seed;
    mutable Tensor<T> mask;
    DropoutFusedOp(double p_, uint64_t s) : p(p_), seed(s) {}
    Tensor<T> compute(const TensorRefs<T>& in) const override {
        mask = HipStorage<T>::alloc(in[0]->shape());
        Tensor<T> y = HipStorage<T>::alloc(in[0]->shape());
        fx_ok(FusedApi<T>::dropout(fused_ctx(), in[0]->data(), mask->data(), y->data(), (int64_t)in[0]->size(), p, seed));
        return y;
    }
    std::vector<Tensor<T>> gradient(Tensor<T> g, const TensorRefs<T>&, const HipStorage<T>*) const override {
        std::vector<Tensor<T>> r;
        r.push_back(g->mul(*mask));
        return r;
    }
    size_t num_inputs() const override { return 1; }
    const char* name() const override { return "DropoutFused"; }
};
template <typename T> struct DropoutFused : Module<T> {
    double p;
    uint64_t seed, calls = 0;
    bool training = true;
    DropoutFused(double p_, uint64_t seed_) : p(p_), seed(seed_) {
        if (!(p >= 0.0 && p <= 1.0)) throw Error("Dropout probability must be between 0.0 and 1.0");
    }
    void set_training(bool t) override { training = t; }
    NodeId forward(AutoFerroxEngine<T>& g, NodeId input) override {
        if (!training || p == 0.0) return input;
        if (p == 1.0) return g.create_variable(HipStorage<T>::zeros(g.get_tensor(input)->shape()), false);
        return g.apply_operation(std::make_unique<DropoutFusedOp<T>>(p, seed + (calls++ << 32)), {input});
    }
};

template <typename T> NodeId cce_loss_fused(AutoFerroxEngine<T>& g, NodeId predictions, NodeId targets) {
    return g.apply_operation(std::make_unique<SoftmaxCEOp<T>>(&g), {predictions, targets});
}

// SGD with every parameter of a group updated in one launch (fx_sgd_step_multi / fx_sgd_momentum_step_multi); same
// hyper-parameters, groups, buffers, state dictionary and element arithmetic as SGD<T>.
template <typename T> struct SGDFused : SGD<T> {
    explicit SGDFused(T lr_, T momentum_ = T(0), T wd = T(0), bool nesterov_ = false) : SGD<T>(lr_, momentum_, wd, nesterov_) {}
    void step(AutoFerroxEngine<T>& g) override {
        for (const auto& group : this->param_groups) {
            const T glr = group.lr.value_or(this->lr), gwd = group.weight_decay.value_or(this->weight_decay),
                    gmom = group.momentum.value_or(this->momentum);
            std::vector<T*> ps, bufs;
            std::vector<const T*> gs;
            std::vector<int64_t> ns;
            for (NodeId p : group.params) {
                const HipStorage<T>* grad = g.get_gradient(p);
                if (!grad) continue;
                HipStorage<T>* w = g.mutable_tensor(p);
                if (grad->shape() != w->shape()) throw Error("Shape mismatch for GPU subtraction: " + fmt_shape(w->shape()) + " vs " + fmt_shape(grad->shape()));
                if (gmom != T(0)) {
                    auto it = this->momentum_buffers.find(p);
                    if (it == this->momentum_buffers.end()) it = this->momentum_buffers.emplace(p, HipStorage<T>::zeros(w->shape())).first;
                    else this->check_buffer(*it->second, *w, "momentum", p);
                    bufs.push_back(it->second->data());
                }
                ps.push_back(w->data());
                gs.push_back(grad->data());
                ns.push_back((int64_t)w->size());
            }
            if (ps.empty()) continue;
            if (gmom == T(0) && gwd == T(0)) fx_ok(FusedApi<T>::sgd_multi(fused_ctx(), (int)ps.size(), ps.data(), gs.data(), ns.data(), glr));
            else
                fx_ok(FusedApi<T>::sgd_momentum_multi(fused_ctx(), (int)ps.size(), ps.data(), gs.data(), gmom != T(0) ? bufs.data() : nullptr, ns.data(),
                                                      glr, gmom, gwd, this->nesterov ? 1 : 0));
        }
    }
};

// Adam with every parameter of a group updated in one launch (fx_adam_step_multi / fx_adam_amsgrad_step_multi)
template <typename T> struct AdamFused : Adam<T> {
    AdamFused(T lr_, T b1, T b2, T eps_, T wd, bool amsgrad_ = false) : Adam<T>(lr_, b1, b2, eps_, wd, amsgrad_) {}
    ~AdamFused() override {
        if (bc_host) (void)fx_host_free(fused_ctx(), bc_host);
    }
    // Steps that are recorded once and replayed (Model::enable_graph): the bias corrections are the only scalars of the
    // step that change, so the kernel reads them from memory instead of taking them as arguments.  They live in page-locked
    // host memory, which the device reads in place (a recorded launch reads the same address at every replay): the host
    // rewrites the two values before each step, and every step ends with a wait for the loss, so the step before has read
    // them by then.  (A copy to device memory queued per step was a graph node of its own: 4 us of a 210 us step.)
    bool device_bc = false;
    T* bc_host = nullptr;
    void use_device_bias_corrections() {
        if (device_bc) return;
        void* h = nullptr;
        fx_ok(fx_host_alloc(fused_ctx(), (int64_t)(2 * sizeof(T)), &h));
        bc_host = static_cast<T*>(h);
        device_bc = true;
    }
    // the host half of a step whose device half is a graph launch: the caller launches the graph afterwards
    void advance_for_replay() {
        this->step_count += 1;
        adam_bias_corrections(this->beta1, this->beta2, this->step_count, bc_host[0], bc_host[1]);
    }
    void step(AutoFerroxEngine<T>& g) override {
        this->step_count += 1;
        T bc1, bc2;
        adam_bias_corrections(this->beta1, this->beta2, this->step_count, bc1, bc2);
        if (device_bc) {
            bc_host[0] = bc1;
            bc_host[1] = bc2;
        }
        for (const auto& group : this->param_groups) {
            const T glr = group.lr.value_or(this->lr), gwd = group.weight_decay.value_or(this->weight_decay);
            std::vector<T*> ps, ms, vs, xs;
            std::vector<const T*> gs;
            std::vector<int64_t> ns;
            auto buffer = [&](std::map<NodeId, Tensor<T>>& table, NodeId p, const HipStorage<T>& w, const char* type) {
                auto it = table.find(p);
                if (it == table.end()) it = table.emplace(p, HipStorage<T>::zeros(w.shape())).first;
                else this->check_buffer(*it->second, w, type, p);
                return it->second->data();
            };
            for (NodeId p : group.params) {
                const HipStorage<T>* grad = g.get_gradient(p);
                if (!grad) continue;
                HipStorage<T>* w = g.mutable_tensor(p);
                if (grad->shape() != w->shape()) throw Error("Shape mismatch for GPU subtraction: " + fmt_shape(w->shape()) + " vs " + fmt_shape(grad->shape()));
                ms.push_back(buffer(this->m1, p, *w, "first_moment"));
                vs.push_back(buffer(this->m2, p, *w, "second_moment"));
                if (this->amsgrad) xs.push_back(buffer(this->mmax, p, *w, "max_second_moment"));
                ps.push_back(w->data());
                gs.push_back(grad->data());
                ns.push_back((int64_t)w->size());
            }
            if (ps.empty()) continue;
            if (device_bc)
                fx_ok(FusedApi<T>::adam_multi_bc(fused_ctx(), (int)ps.size(), ps.data(), gs.data(), ms.data(), vs.data(), this->amsgrad ? xs.data() : nullptr,
                                                 ns.data(), glr, this->beta1, this->beta2, this->eps, gwd, bc_host));
            else if (this->amsgrad)
                fx_ok(FusedApi<T>::adam_amsgrad_multi(fused_ctx(), (int)ps.size(), ps.data(), gs.data(), ms.data(), vs.data(), xs.data(), ns.data(), glr,
                                                      this->beta1, this->beta2, this->eps, gwd, bc1, bc2));
            else
                fx_ok(FusedApi<T>::adam_multi(fused_ctx(), (int)ps.size(), ps.data(), gs.data(), ms.data(), vs.data(), ns.data(), glr, this->beta1,
                                              this->beta2, this->eps, gwd, bc1, bc2));
        }
    }
};

}  // namespace ferrox
