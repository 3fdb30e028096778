// Replay harness: drives the mirrored Ferrox host stack (autograd.hpp) through a C ABI so that tests and the
// benchmark can run the MLP / CNN training configs end to end against libferrox_hip.so.
// One training step follows examples/common/training.rs:33-81 of the reference:
//   zero_gradients -> create_variable(inputs.clone()), create_variable(targets.clone()) (:125-126) ->
//   model.forward -> loss.forward -> loss.clone().first() (device->host sync) -> backward -> optimizer.step
#include <chrono>
#include <cstdio>
#include <cstdlib>
#include <sstream>

#include "fused.hpp"

using namespace ferrox;

namespace {
thread_local std::string g_err;
// clone_storage() of the op-by-op engines as a second owner of the block (default) or as the device copy the reference makes
bool g_share_clones = true;

struct ModelBase {
    virtual ~ModelBase() = default;
    virtual int num_params() const = 0;
    virtual int64_t param_numel(int i) const = 0;
    virtual void set_batch(const void* x, const Shape& xs, const void* y, const Shape& ys) = 0;
    virtual double train_step(bool optimizer_step = true) = 0;
    virtual void configure(int loss_kind, bool input_requires_grad) = 0;
    virtual void add_param_group(const int* idx, int n, double lr, double wd, double mom) = 0;
    virtual int64_t input_numel() const = 0;
    virtual void get_input_grad(void* host) const = 0;
    virtual void get_param(int i, void* host) const = 0;
    virtual void get_grad(int i, void* host) const = 0;
    virtual void forward_only(void* host_out) = 0;
    virtual int64_t output_numel() = 0;
    virtual void set_training(bool t) = 0;
    virtual int num_state() const = 0;
    virtual int64_t state_numel(int i) const = 0;
    virtual void get_state(int i, void* host) const = 0;
    virtual std::vector<uint8_t> optimizer_state() const = 0;
    virtual void load_optimizer_state(const uint8_t* data, size_t n) = 0;
    virtual void enable_graph(bool on) = 0;
    virtual void graph_info(int64_t* nodes, int64_t* kernels, int64_t* held) const = 0;
};

std::vector<std::string> split(const std::string& s, char sep) {
    std::vector<std::string> out;
    std::stringstream ss(s);
    std::string item;
    while (std::getline(ss, item, sep)) {
        size_t a = item.find_first_not_of(" \t\n"), b = item.find_last_not_of(" \t\n");
        if (a != std::string::npos) out.push_back(item.substr(a, b - a + 1));
    }
    return out;
}

template <typename T> struct Model : ModelBase {
    AutoFerroxEngine<T> graph;
    std::vector<std::unique_ptr<Module<T>>> layers;
    std::vector<NodeId> params;
    std::unique_ptr<Optimizer<T>> opt;
    Tensor<T> x, y;

    bool fused = false;
    // loss: 0 = CCELoss on (prediction, targets); 1 = Sum over every element of the prediction (the reference's
    // plumbing check: relu(conv(x) + b).sum().backward(), Sum::new() of src/ops/reduction.rs:52-140)
    int loss_kind = 0;
    // the batch enters the graph as a leaf that requires a gradient (create_variable(x, true)), kept across steps
    bool input_requires_grad = false;
    bool have_input_node = false;
    NodeId input_node = 0;

    // Recorded steps (enable_graph): after two eager steps on the same batch shape -- the pool then serves every request of
    // a step from its buckets, the scratch region has its size, the conv tiles are timed -- the next step is recorded into a
    // graph once and every later one is a single launch of it.  The recorded step is the eager one call for call, so the
    // results have the same bits.  Only the fused engine is recorded: its optimizers update the parameters in place and
    // its loss is read after the step, whereas the op-by-op engines put every updated parameter into a NEW tensor (a replay
    // would keep reading the old one), read the loss in the middle of a step (training.rs:60-64) and pass Adam's bias
    // corrections as scalar arguments of a dozen elementwise kernels.  Also left eager: models with a Dropout layer (a new
    // mask per step, seeded on the host) and a batch that enters as a leaf with a gradient.
    bool graph_on = false, has_dropout = false;
    fx_graph* step_graph = nullptr;
    bool graph_with_update = true;  // the recorded step includes the optimizer step
    Tensor<T> graph_loss;           // where the recorded step leaves its loss
    int warm_steps = 0;
    ~Model() override { drop_graph(); }
    void drop_graph() {
        if (step_graph) (void)fx_graph_destroy(BackendManager::get().ctx(), step_graph);
        step_graph = nullptr;
        graph_loss.reset();
        warm_steps = 0;
    }
    bool graph_supported() const {
        return fused && !has_dropout && !input_requires_grad;
    }
    void enable_graph(bool on) override {
        if (on && !graph_on)
            if (auto* a = dynamic_cast<AdamFused<T>*>(opt.get())) a->use_device_bias_corrections();
        if (!on) drop_graph();
        graph_on = on;
    }
    void graph_info(int64_t* nodes, int64_t* kernels, int64_t* held) const override {
        *nodes = *kernels = *held = 0;
        if (step_graph) fx_ok(fx_graph_info(step_graph, nodes, kernels, held));
    }

    // engine: 0 = reference op sequence without the per-node deep clones, 1 = reference op sequence as is,
    //         2 = fused layers / loss / optimizers
    Model(const std::string& spec, const std::string& optspec, int engine, const void* const* pv, int np)
        : graph(engine == 1), fused(engine == 2) {
        graph.reuse_unit_seed = fused;
        int pi = 0;
        auto next = [&]() -> const T* {
            if (pi >= np) throw Error("not enough parameter arrays for the layer spec");
            return static_cast<const T*>(pv[pi++]);
        };
        const std::vector<std::string> toks = split(spec, ';');
        for (size_t ti = 0; ti < toks.size(); ++ti) {
            std::stringstream ss(toks[ti]);
            std::string kind;
            ss >> kind;
            // fused mode folds a ReLU that directly follows a linear / conv / batch-norm layer into that layer
            const bool relu_next = fused && ti + 1 < toks.size() && toks[ti + 1] == "relu";
            if (kind == "linear") {
                size_t in, out;
                ss >> in >> out;
                const T* w = next();
                const T* b = next();
                if (fused) {
                    layers.push_back(std::make_unique<LinearFused<T>>(graph, in, out, w, b, relu_next));
                    if (relu_next) ++ti;
                } else layers.push_back(std::make_unique<Linear<T>>(graph, in, out, w, b));
            } else if (kind == "conv") {
                size_t cin, cout, k, s, p;
                ss >> cin >> cout >> k >> s >> p;
                const T* w = next();
                const T* b = next();
                if (fused) {
                    layers.push_back(std::make_unique<Conv2dFused<T>>(graph, cin, cout, k, s, p, w, b, relu_next));
                    if (relu_next) ++ti;
                } else layers.push_back(std::make_unique<Conv2d<T>>(graph, cin, cout, k, s, p, w, b));
            } else if (kind == "maxpool" || kind == "avgpool") {
                size_t k, st, p;
                ss >> k >> st >> p;
                layers.push_back(std::make_unique<Pool2d<T>>(kind == "maxpool", k, st, p));
            } else if (kind == "bn") {  // bn C [eps [momentum]]
                size_t c;
                double eps = 1e-5, mom = 0.1;
                ss >> c;
                if (!(ss >> eps)) eps = 1e-5;
                else if (!(ss >> mom)) mom = 0.1;
                const T* w = next();
                const T* b = next();
                if (fused) {
                    layers.push_back(std::make_unique<BatchNormFused<T>>(graph, c, eps, mom, w, b, relu_next));
                    if (relu_next) ++ti;
                }
                else layers.push_back(std::make_unique<BatchNorm<T>>(graph, c, eps, mom, w, b));
            } else if (kind == "gap") {
                if (fused) layers.push_back(std::make_unique<GlobalAvgPoolFused<T>>());
                else layers.push_back(std::make_unique<GlobalAvgPool2d<T>>());
            } else if (kind == "dropout") {  // dropout p seed
                double p = 0.5;
                uint64_t seed = 0;
                ss >> p >> seed;
                has_dropout = true;
                if (engine == 1) layers.push_back(std::make_unique<Dropout<T>>(p, seed));
                else layers.push_back(std::make_unique<DropoutFused<T>>(p, seed));
            } else if (kind == "relu") layers.push_back(std::make_unique<ReLU<T>>());
            else if (kind == "flatten") {
                if (fused) layers.push_back(std::make_unique<FlattenFused<T>>());
                else layers.push_back(std::make_unique<Flatten<T>>());
            }
            else throw Error("unknown layer '" + kind + "'");
            for (NodeId p : layers.back()->parameters()) params.push_back(p);
        }
        std::stringstream os(optspec);
        std::string kind;
        os >> kind;
        if (kind == "sgd") {  // sgd LR [MOMENTUM [WEIGHT_DECAY [NESTEROV]]]
            double lr = 0.01, mom = 0, wd = 0;
            int nesterov = 0;
            os >> lr;
            if (os >> mom && os >> wd) os >> nesterov;
            if (fused) opt = std::make_unique<SGDFused<T>>((T)lr, (T)mom, (T)wd, nesterov != 0);
            else opt = std::make_unique<SGD<T>>((T)lr, (T)mom, (T)wd, nesterov != 0);
        } else if (kind == "adam") {  // adam LR B1 B2 EPS WEIGHT_DECAY [AMSGRAD]
            double lr = 1e-3, b1 = 0.9, b2 = 0.999, eps = 1e-8, wd = 0;
            int amsgrad = 0;
            os >> lr >> b1 >> b2 >> eps >> wd;
            if (!(os >> amsgrad)) amsgrad = 0;
            if (fused) opt = std::make_unique<AdamFused<T>>((T)lr, (T)b1, (T)b2, (T)eps, (T)wd, amsgrad != 0);
            else opt = std::make_unique<Adam<T>>((T)lr, (T)b1, (T)b2, (T)eps, (T)wd, amsgrad != 0);
        } else throw Error("unknown optimizer '" + kind + "'");
        for (NodeId p : params) opt->add_param(0, p);  // initialize_model, examples/common/training.rs:18-29
    }
    // Moves the listed parameters (indices into the model's parameter list) out of their groups into a new group with
    // its own lr / weight decay / momentum (NaN = not set: the optimizer's value applies), ParameterGroup of optim/mod.rs:203-258.
    void add_param_group(const int* idx, int n, double lr, double wd, double mom) override {
        enter();
        drop_graph();  // lr / weight decay / momentum and the pointer tables are arguments of the recorded kernels
        ParameterGroup<T> group("group" + std::to_string(opt->param_groups.size()));
        for (int k = 0; k < n; ++k) {
            const NodeId id = params.at((size_t)idx[k]);
            for (auto& g : opt->param_groups) g.params.erase(std::remove(g.params.begin(), g.params.end(), id), g.params.end());
            group.add_param(id);
        }
        if (lr == lr) group.lr = (T)lr;
        if (wd == wd) group.weight_decay = (T)wd;
        if (mom == mom) group.momentum = (T)mom;
        opt->add_param_group(std::move(group));
    }
    void set_training(bool t) override {
        drop_graph();  // batch statistics or running statistics: a different kernel sequence
        for (auto& l : layers) l->set_training(t);
    }
    std::vector<const HipStorage<T>*> all_state() const {
        std::vector<const HipStorage<T>*> r;
        for (auto& l : layers)
            for (const HipStorage<T>* s : l->state()) r.push_back(s);
        return r;
    }
    int num_state() const override { return (int)all_state().size(); }
    int64_t state_numel(int i) const override { return (int64_t)all_state().at(i)->size(); }
    void get_state(int i, void* host) const override {
        std::vector<T> v = all_state().at(i)->to_vec();
        std::memcpy(host, v.data(), v.size() * sizeof(T));
    }
    std::vector<uint8_t> optimizer_state() const override { return opt->state_dict().save_to_bytes(); }
    void load_optimizer_state(const uint8_t* data, size_t n) override {
        enter();
        drop_graph();  // the moments move to new tensors: a recording made before would keep updating the old addresses
        opt->load_state_dict(OptimizerStateDict::load_from_bytes(data, n));
    }
    int num_params() const override { return (int)params.size(); }
    int64_t param_numel(int i) const override { return (int64_t)graph.get_tensor(params.at(i))->size(); }
    void set_batch(const void* xv, const Shape& xs, const void* yv, const Shape& ys) override {
        enter();
        if (graph_on && graph_supported() && x && y && x->shape() == xs && y->shape() == ys) {
            // a recorded step reads the batch at the addresses it was recorded with: new data goes there
            fx_ok(fx_h2d(BackendManager::get().ctx(), x->data(), xv, (int64_t)(x->size() * sizeof(T))));
            fx_ok(fx_h2d(BackendManager::get().ctx(), y->data(), yv, (int64_t)(y->size() * sizeof(T))));
            return;
        }
        drop_graph();
        x = HipStorage<T>::from_vec(static_cast<const T*>(xv), xs);
        y = HipStorage<T>::from_vec(static_cast<const T*>(yv), ys);
        if (have_input_node) graph.update_parameter(input_node, x->clone_storage());
    }
    void configure(int kind, bool in_grad) override {
        if (kind != 0 && kind != 1) throw Error("unknown loss kind");
        drop_graph();  // another loss or another kind of input leaf: another step
        loss_kind = kind;
        input_requires_grad = in_grad;
    }
    int64_t input_numel() const override { return x ? (int64_t)x->size() : -1; }
    void get_input_grad(void* host) const override {
        const HipStorage<T>* g = have_input_node ? graph.get_gradient(input_node) : nullptr;
        if (!g) throw Error("no gradient for the input (configure the model with input_requires_grad and run a backward pass)");
        std::vector<T> v = g->to_vec();
        std::memcpy(host, v.data(), v.size() * sizeof(T));
    }
    // The fused engine updates parameters, moments and the batch in place, so its clones must stay copies; the op-by-op engines
    // only ever create new storage, so theirs may share the block (hip_storage.hpp, share_clones).
    void enter() const { BackendManager::get().share_clones = !fused && g_share_clones; }
    NodeId forward(NodeId in) {
        for (auto& l : layers) in = l->forward(graph, in);
        return in;
    }
    // zero_gradients -> forward -> loss -> backward -> update, nothing read back (the loss tensor is handed out): the form a
    // step is recorded in
    Tensor<T> step_body(bool optimizer_step) {
        graph.zero_gradients();
        const NodeId xin = graph.create_variable(fused ? HipStorage<T>::borrow(*x) : x->clone_storage(), false);
        const NodeId pred = forward(xin);
        NodeId loss;
        if (loss_kind == 1) loss = graph.apply_operation(std::make_unique<Sum<T>>(false), {pred});
        else {
            const NodeId yin = graph.create_variable(fused ? HipStorage<T>::borrow(*y) : y->clone_storage(), false);
            loss = fused ? cce_loss_fused<T>(graph, pred, yin) : cce_loss<T>(graph, pred, yin);
        }
        Tensor<T> lval;
        graph.backward(loss, &lval);
        if (optimizer_step) opt->step(graph);
        return lval;
    }
    double train_step(bool optimizer_step) override {
        enter();
        if (!x || !y) throw Error("set_batch was not called");
        if (graph_on && graph_supported()) {
            fx_ctx* c = BackendManager::get().ctx();
            if (step_graph && graph_with_update != optimizer_step) drop_graph();
            if (step_graph) {
                if (optimizer_step)
                    if (auto* a = dynamic_cast<AdamFused<T>*>(opt.get())) a->advance_for_replay();
                fx_ok(fx_graph_launch(c, step_graph));
                return (double)graph_loss->first();
            }
            if (warm_steps >= 2) {
                fx_ok(fx_graph_begin(c));
                Tensor<T> l;
                try {
                    l = step_body(optimizer_step);
                } catch (...) {
                    fx_graph* g = nullptr;
                    if (fx_graph_end(c, &g) == FX_OK && g) (void)fx_graph_destroy(c, g);
                    graph_on = false;  // the step was neither run nor recorded: the caller sees the error, later steps run eagerly
                    throw;
                }
                fx_ok(fx_graph_end(c, &step_graph));
                graph_loss = std::move(l);
                graph_with_update = optimizer_step;
                fx_ok(fx_graph_launch(c, step_graph));
                return (double)graph_loss->first();
            }
            ++warm_steps;
        }
        graph.zero_gradients();
        NodeId xin;
        if (input_requires_grad) {
            if (!have_input_node) {
                input_node = graph.create_variable(x->clone_storage(), true);
                have_input_node = true;
            }
            xin = input_node;
        } else {
            // the reference clones the batch every step (training.rs:125-126); the fused engine reads it in place
            xin = graph.create_variable(fused ? HipStorage<T>::borrow(*x) : x->clone_storage(), false);
        }
        const NodeId pred = forward(xin);
        NodeId loss;
        if (loss_kind == 1) loss = graph.apply_operation(std::make_unique<Sum<T>>(false), {pred});
        else {
            const NodeId yin = graph.create_variable(fused ? HipStorage<T>::borrow(*y) : y->clone_storage(), false);
            loss = fused ? cce_loss_fused<T>(graph, pred, yin) : cce_loss<T>(graph, pred, yin);
        }
        if (!fused) {
            const T lv = graph.get_tensor(loss)->clone_storage()->first();  // device -> host: the GPU drains here (training.rs:60-64)
            graph.backward(loss);
            if (optimizer_step) opt->step(graph);
            return (double)lv;
        }
        // fused engine: the loss tensor outlives the graph's clean-up and is read after the backward pass and the update are
        // enqueued, so the device never waits for the host in the middle of a step
        Tensor<T> lval;
        graph.backward(loss, &lval);
        if (optimizer_step) opt->step(graph);
        return (double)lval->first();
    }
    void get_param(int i, void* host) const override {
        std::vector<T> v = graph.get_tensor(params.at(i))->to_vec();
        std::memcpy(host, v.data(), v.size() * sizeof(T));
    }
    void get_grad(int i, void* host) const override {
        const HipStorage<T>* g = graph.get_gradient(params.at(i));
        if (!g) throw Error("no gradient for parameter " + std::to_string(i));
        std::vector<T> v = g->to_vec();
        std::memcpy(host, v.data(), v.size() * sizeof(T));
    }
    int64_t output_numel() override {
        enter();
        const NodeId xin = graph.create_variable(x->clone_storage(), false);
        const NodeId pred = forward(xin);
        return (int64_t)graph.get_tensor(pred)->size();
    }
    void forward_only(void* host_out) override {
        enter();
        const NodeId xin = graph.create_variable(x->clone_storage(), false);
        const NodeId pred = forward(xin);
        std::vector<T> v = graph.get_tensor(pred)->to_vec();
        std::memcpy(host_out, v.data(), v.size() * sizeof(T));
    }
};

template <typename F> int guarded(F&& f) {
    try {
        f();
        return 0;
    } catch (const std::exception& e) {
        g_err = e.what();
        return 1;
    }
}
}  // namespace

extern "C" {

const char* fxh_last_error(void) { return g_err.c_str(); }

int fxh_init(int device, int conv_grad_mode, const fx_pool_config* cfg) {
    return guarded([&] {
        BackendManager::get().init(device, cfg);
        BackendManager::get().conv_grad_mode = conv_grad_mode;
    });
}
void fxh_shutdown(void) { BackendManager::get().shutdown(); }
// 0 = mathematical conv gradients, 1 = the CPU backend's literal arithmetic; read by every later deconv2d / cross_correlation2d
// 1 (default): clones made by the op-by-op engines share their block; 0: they are device-to-device copies as in the reference
void fxh_set_share_clones(int on) { g_share_clones = on != 0; }
int fxh_set_conv_grad_mode(int mode) {
    return guarded([&] {
        if (mode != 0 && mode != 1) throw Error("conv gradient mode must be 0 or 1");
        BackendManager::get().conv_grad_mode = mode;
    });
}

void* fxh_model_create(int dtype, const char* spec, const char* optimizer, int literal_engine /* engine mode 0, 1 or 2 */, const void* const* params, int n_params) {
    ModelBase* m = nullptr;
    const int rc = guarded([&] {
        if (dtype == FX_F32) m = new Model<float>(spec, optimizer, literal_engine, params, n_params);
        else if (dtype == FX_F64) m = new Model<double>(spec, optimizer, literal_engine, params, n_params);
        else throw Error("unknown dtype");
    });
    return rc ? nullptr : m;
}
void fxh_model_destroy(void* m) { delete static_cast<ModelBase*>(m); }
int fxh_model_num_params(void* m) { return static_cast<ModelBase*>(m)->num_params(); }
int64_t fxh_model_param_numel(void* m, int i) {
    int64_t n = -1;
    guarded([&] { n = static_cast<ModelBase*>(m)->param_numel(i); });
    return n;
}
int fxh_model_set_batch(void* m, const void* x, const int64_t* xshape, int xnd, const void* y, const int64_t* yshape, int ynd) {
    return guarded([&] {
        Shape xs(xshape, xshape + xnd), ys(yshape, yshape + ynd);
        static_cast<ModelBase*>(m)->set_batch(x, xs, y, ys);
    });
}
int fxh_model_train_step(void* m, double* loss) {
    return guarded([&] { *loss = static_cast<ModelBase*>(m)->train_step(true); });
}
// loss_kind 0 = CCELoss, 1 = Sum over the prediction; input_requires_grad: the batch is a leaf with a gradient
int fxh_model_configure(void* m, int loss_kind, int input_requires_grad) {
    return guarded([&] { static_cast<ModelBase*>(m)->configure(loss_kind, input_requires_grad != 0); });
}
// zero_gradients -> forward -> loss -> backward, no optimizer step
int fxh_model_backward(void* m, double* loss) {
    return guarded([&] { *loss = static_cast<ModelBase*>(m)->train_step(false); });
}
// parameters idx[0..n) leave their groups for a new one; lr / weight_decay / momentum are NaN where the group sets none
int fxh_model_add_param_group(void* m, const int* idx, int n, double lr, double weight_decay, double momentum) {
    return guarded([&] { static_cast<ModelBase*>(m)->add_param_group(idx, n, lr, weight_decay, momentum); });
}
int64_t fxh_model_input_numel(void* m) { return static_cast<ModelBase*>(m)->input_numel(); }
int fxh_model_get_input_grad(void* m, void* host) {
    return guarded([&] { static_cast<ModelBase*>(m)->get_input_grad(host); });
}
// n steps back to back; wall time covers forward + backward + optimizer step of every step and one final sync
// Later steps are recorded once and replayed as one graph launch where the model allows it (see Model::graph_on).
int fxh_model_enable_graph(void* m, int on) {
    return guarded([&] { static_cast<ModelBase*>(m)->enable_graph(on != 0); });
}
// nodes / kernel nodes / pool blocks of the recorded step (zeros while there is none)
int fxh_model_graph_info(void* m, int64_t* nodes, int64_t* kernels, int64_t* held) {
    return guarded([&] { static_cast<ModelBase*>(m)->graph_info(nodes, kernels, held); });
}
int fxh_model_train_steps(void* m, int n, double* last_loss, double* total_ms) {
    return guarded([&] {
        fx_ok(fx_sync(BackendManager::get().ctx()));
        const auto t0 = std::chrono::steady_clock::now();
        for (int i = 0; i < n; ++i) *last_loss = static_cast<ModelBase*>(m)->train_step(true);
        fx_ok(fx_sync(BackendManager::get().ctx()));
        *total_ms = std::chrono::duration<double, std::milli>(std::chrono::steady_clock::now() - t0).count();
    });
}
int fxh_model_get_param(void* m, int i, void* host) {
    return guarded([&] { static_cast<ModelBase*>(m)->get_param(i, host); });
}
int fxh_model_get_grad(void* m, int i, void* host) {
    return guarded([&] { static_cast<ModelBase*>(m)->get_grad(i, host); });
}
int64_t fxh_model_output_numel(void* m) {
    int64_t n = -1;
    guarded([&] { n = static_cast<ModelBase*>(m)->output_numel(); });
    return n;
}
int fxh_model_forward(void* m, void* host_out) {
    return guarded([&] { static_cast<ModelBase*>(m)->forward_only(host_out); });
}
// training / evaluation mode of every layer (BatchNorm statistics, Dropout), Module::set_training
int fxh_model_set_training(void* m, int training) {
    return guarded([&] { static_cast<ModelBase*>(m)->set_training(training != 0); });
}
// persistent non-parameter tensors in layer order (BatchNorm: running mean, running variance)
int fxh_model_num_state(void* m) { return static_cast<ModelBase*>(m)->num_state(); }
int64_t fxh_model_state_numel(void* m, int i) {
    int64_t n = -1;
    guarded([&] { n = static_cast<ModelBase*>(m)->state_numel(i); });
    return n;
}
int fxh_model_get_state(void* m, int i, void* host) {
    return guarded([&] { static_cast<ModelBase*>(m)->get_state(i, host); });
}
// Optimizer::state_dict().save_to_bytes(): the moments are copied from the device; *bytes is malloc'ed, release it with fxh_free
int fxh_model_optimizer_state(void* m, uint8_t** bytes, int64_t* len) {
    return guarded([&] {
        const std::vector<uint8_t> v = static_cast<ModelBase*>(m)->optimizer_state();
        *bytes = static_cast<uint8_t*>(std::malloc(v.size() ? v.size() : 1));
        if (!*bytes) throw Error("out of host memory");
        std::memcpy(*bytes, v.data(), v.size());
        *len = (int64_t)v.size();
    });
}
void fxh_free(void* p) { std::free(p); }
// OptimizerStateDict::load_from_bytes + Optimizer::load_state_dict
int fxh_model_load_optimizer_state(void* m, const uint8_t* bytes, int64_t len) {
    return guarded([&] {
        if (len < 0 || (!bytes && len)) throw Error("bad buffer");
        static_cast<ModelBase*>(m)->load_optimizer_state(bytes, (size_t)len);
    });
}
int fxh_pool_stats(int dtype, fx_pool_stats* out) {
    return guarded([&] { fx_ok(fx_pool_stats_get(BackendManager::get().ctx(), dtype, out)); });
}

}  // extern "C"
