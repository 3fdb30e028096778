"""End-to-end parity of the mirrored host stack (HipStorage + autograd tape + layers + loss + optimizer) running on
libferrox_hip.so against the CPU oracle's training step, on the MLP (config 2) and CNN (config 5) shapes:
loss, every parameter gradient and the updated parameters, f32 within rel 1e-5 and f64 within rel 1e-12."""
import numpy as np
import pytest

pytestmark = pytest.mark.gpu

MLP_SMALL = "linear 20 16; relu; linear 16 12; relu; linear 12 5"
CNN_SMALL = "conv 3 4 3 1 1; relu; conv 4 6 3 2 1; relu; flatten; linear 96 5"
CNN_POOL = "conv 3 8 3 1 1; relu; maxpool 2 2 0; conv 8 8 3 1 1; relu; avgpool 3 2 1; flatten; linear 128 5"
# the block order of the reference's CNNClassifier (examples/common/models.rs:200-318): conv, BatchNorm, ReLU twice,
# GlobalAvgPool2d, Flatten, Linear, ReLU, Dropout(0.3), Linear; the second is its 32x32 RGB instance
CNN_CLS_SMALL = ("conv 3 8 3 1 1; bn 8 0.001 0.1; relu; conv 8 16 3 1 1; bn 16 0.001 0.1; relu; gap; flatten; "
                 "linear 16 12; relu; dropout 0.3 17; linear 12 5")
CNN_CLS = ("conv 3 32 3 1 1; bn 32 0.001 0.1; relu; conv 32 64 3 1 1; bn 64 0.001 0.1; relu; gap; flatten; "
           "linear 64 64; relu; dropout 0.3 23; linear 64 10")
MLP_C2 = "linear 784 256; relu; linear 256 128; relu; linear 128 10"
CNN_C5 = "conv 3 32 3 1 1; relu; conv 32 64 3 2 1; relu; flatten; linear 16384 10"
import parity
from parity import TOL


@pytest.fixture(scope="module")
def host():
    from ferrox_amd import host_api
    host_api.init(0, 0)
    yield host_api
    host_api.shutdown()


def kaiming_uniform_problem(spec, in_shape, n_classes, seed, dtype):
    rng = np.random.default_rng(seed)
    params = []
    for tok in [t.strip() for t in spec.split(";") if t.strip()]:
        p = tok.split()
        if p[0] == "linear":
            i, o = int(p[1]), int(p[2])
            lim = np.sqrt(6.0 / i)
            params += [rng.uniform(-lim, lim, (o, i)).astype(dtype), np.zeros(o, dtype)]
        elif p[0] == "conv":
            ci, co, k = int(p[1]), int(p[2]), int(p[3])
            lim = np.sqrt(6.0 / (ci * k * k))
            params += [rng.uniform(-lim, lim, (co, ci, k, k)).astype(dtype), np.zeros(co, dtype)]
        elif p[0] == "bn":
            params += [rng.uniform(0.8, 1.2, int(p[1])).astype(dtype), rng.uniform(-0.1, 0.1, int(p[1])).astype(dtype)]
    x = rng.standard_normal(in_shape).astype(dtype)
    y = np.eye(n_classes, dtype=dtype)[rng.integers(0, n_classes, in_shape[0])]
    return params, x, y


def bias_before_batchnorm(spec):
    """Indices of conv / linear biases that feed a BatchNorm directly: their gradient is exactly zero in exact
    arithmetic (the layer subtracts the batch mean), so both sides hold rounding noise only."""
    toks = [t.strip().split() for t in spec.split(";") if t.strip()]
    out, pi = set(), 0
    for k, t in enumerate(toks):
        if t[0] in ("conv", "linear", "bn"):
            if t[0] != "bn" and k + 1 < len(toks) and toks[k + 1][0] == "bn":
                out.add(pi + 1)
            pi += 2
    return out


def close(got, ref, tol):
    ref64 = np.asarray(ref, np.float64)
    return np.abs(np.asarray(got, np.float64) - ref64).max() <= tol * max(1e-30, np.abs(ref64).max())


CASES = [
    ("mlp_small", MLP_SMALL, (9, 20), 5, "sgd 0.01", 3),
    ("cnn_small", CNN_SMALL, (5, 3, 8, 8), 5, "adam 0.001 0.9 0.999 1e-08 0", 3),
    ("cnn_pool", CNN_POOL, (4, 3, 16, 16), 5, "sgd 0.05", 2),
    ("cnn_cls_small", CNN_CLS_SMALL, (6, 3, 8, 8), 5, "sgd 0.05", 3),
    ("cnn_cls", CNN_CLS, (64, 3, 32, 32), 10, "adam 0.001 0.9 0.999 1e-08 0", 1),
    ("mlp_c2", MLP_C2, (256, 784), 10, "sgd 0.01", 1),
    ("cnn_c5", CNN_C5, (256, 3, 32, 32), 10, "adam 0.001 0.9 0.999 1e-08 0", 1),
    # the optimizer options of the reference's training example (examples/common/training.rs:99-111)
    ("mlp_small_momentum", MLP_SMALL, (9, 20), 5, "sgd 0.05 0.9 0 0", 3),
    ("cnn_small_nesterov_wd", CNN_SMALL, (5, 3, 8, 8), 5, "sgd 0.05 0.9 0.0005 1", 3),
    ("cnn_small_amsgrad_wd", CNN_SMALL, (5, 3, 8, 8), 5, "adam 0.001 0.9 0.999 1e-08 0.01 1", 3),
]


def oracle_optimizer(optspec, groups=None):
    from oracle import train as otrain
    kind, *nums = optspec.split()
    v = [float(t) for t in nums]
    if kind == "sgd":
        v += [0.0] * (4 - len(v))
        return otrain.SGD(v[0], v[1], v[2], bool(v[3]), groups=groups)
    v += [0.0] * (6 - len(v))
    return otrain.Adam(v[0], v[1], v[2], v[3], v[4], bool(v[5]), groups=groups)


@pytest.mark.parametrize("dtype", [np.float32, np.float64])
@pytest.mark.parametrize("case", CASES, ids=[c[0] for c in CASES])
@pytest.mark.parametrize("engine", ["literal", "lean", "fused"])
def test_train_step_matches_oracle(host, case, dtype, engine):
    """engine: the reference's op sequence with / without its per-node clones, or the fused layers, loss and
    optimizer; all three must reproduce the composed CPU oracle."""
    from oracle import train as otrain
    name, spec, in_shape, ncls, optspec, steps = case
    literal_engine = engine == "literal"
    tol = TOL[np.dtype(dtype)]
    noise_only = bias_before_batchnorm(spec)
    params, x, y = kaiming_uniform_problem(spec, in_shape, ncls, 5, dtype)
    ref = otrain.Sequential(spec, params, dtype, conv_mode=0)
    # ground truth for f32: the same composed step carried out in float64 on the same f32-valued parameters and batch; for f64
    # the f64 oracle itself (two f64 evaluation orders differ by ~1e-15, far inside 1e-12)
    truth = otrain.Sequential(spec, params, np.float64, conv_mode=0) if dtype == np.float32 else None
    kind, *nums = optspec.split()
    ropt = oracle_optimizer(optspec)
    model = host.Model(spec, params, optspec, dtype, literal_engine=literal_engine, fused=engine == "fused")
    try:
        model.set_batch(x, y)
        for step in range(steps):
            rloss, rgrads = ref.loss_and_grads(x, y)
            tloss, tgrads = truth.loss_and_grads(x.astype(np.float64), y.astype(np.float64)) if truth else (rloss, rgrads)
            ropt.step(ref, rgrads)
            gloss = model.train_step()
            tag = (name, engine, step)
            parity.check("train step loss", np.array([gloss]), np.array([tloss], np.float64), dtype,
                         oracle=np.array([rloss]) if truth else None, case=tag)
            for i, rg in enumerate(rgrads):
                if i in noise_only:
                    assert np.abs(model.grad(i)).max() <= tol * 1e-2 and np.abs(rg).max() <= tol * 1e-2, (name, step, "grad", i)
                    continue
                parity.check("train step grad", model.grad(i), tgrads[i], dtype, oracle=rg if truth else None, case=tag + (i,), kink=True)
            for i, rp in enumerate(ref.params):
                got = model.param(i).astype(np.float64)
                if kind == "sgd":
                    assert np.abs(got - rp).max() <= tol * max(1.0, np.abs(rp).max()), (name, step, "param", i)
                    continue
                # Adam's first steps move every weight by ~lr whatever the gradient's size, so where the gradient is
                # rounding noise around zero the update's sign is noise too (bounded by lr per step); everywhere else
                # the step taken (parameter delta) must equal the oracle's to a small fraction of lr
                lr = float(nums[0])
                assert np.abs(got - rp).max() <= 2.5 * lr * (step + 1), (name, step, "param", i)
                if step == 0 and i not in noise_only:
                    clear = np.abs(rgrads[i]) > 1e-3 * np.abs(rgrads[i]).max()
                    d_gpu = (got - np.asarray(params[i], np.float64))[clear]
                    d_ref = (rp.astype(np.float64) - np.asarray(params[i], np.float64))[clear]
                    assert clear.any() and np.abs(d_gpu - d_ref).max() <= 0.05 * lr, (name, "param delta", i)
                    assert np.abs(d_ref).min() >= 0.5 * lr, (name, "oracle did not move", i)
            # the next step starts from the GPU's parameters on every side, so each step's gradients are compared on
            # identical parameters (Adam's sign noise on near-zero gradients would otherwise grow from step to step)
            for i in range(len(ref.params)):
                cur = model.param(i)
                ref.params[i] = np.ascontiguousarray(cur, dtype=dtype).reshape(ref.params[i].shape).copy()
                if truth:
                    truth.params[i] = np.ascontiguousarray(cur, dtype=np.float64).reshape(truth.params[i].shape).copy()
    finally:
        model.close()


@pytest.mark.parametrize("dtype", [np.float32, np.float64])
@pytest.mark.parametrize("case", [c for c in CASES if c[0] in ("cnn_small", "cnn_cls_small", "mlp_small_momentum", "cnn_small_amsgrad_wd")],
                         ids=["cnn_small", "cnn_cls_small", "mlp_small_momentum", "cnn_small_amsgrad_wd"])
@pytest.mark.parametrize("engine", ["literal", "lean"])
def test_shared_clones_cannot_be_told_from_copied_ones(host, case, dtype, engine):
    """clone_storage() as a second owner of the block (the default of the op-by-op engines) against the device copy the
    reference makes: loss, every gradient, every parameter and the optimizer's moments after several steps, bit for bit; and the
    shared form asks the pool for fewer blocks."""
    name, spec, in_shape, ncls, optspec, steps = case
    params, x, y = kaiming_uniform_problem(spec, in_shape, ncls, 11, dtype)
    runs = {}
    try:
        for share in (True, False):
            host.set_share_clones(share)
            model = host.Model(spec, params, optspec, dtype, literal_engine=engine == "literal", fused=False)
            try:
                model.set_batch(x, y)
                st0 = host.pool_stats(dtype)
                losses = [model.train_step() for _ in range(steps + 1)]
                st1 = host.pool_stats(dtype)
                runs[share] = (losses, [model.grad(i).copy() for i in range(len(params))], [model.param(i).copy() for i in range(len(params))],
                               [s.copy() for s in model.state()] + [np.frombuffer(model.optimizer_state(), np.uint8).copy()], (st1["pool_hits"] + st1["pool_misses"]) - (st0["pool_hits"] + st0["pool_misses"]))
            finally:
                model.close()
    finally:
        host.set_share_clones(True)
    a, b = runs[True], runs[False]
    assert a[0] == b[0], (name, "loss", a[0], b[0])
    for k in (1, 2, 3):
        assert len(a[k]) == len(b[k])
        for i, (u, v) in enumerate(zip(a[k], b[k])):
            assert np.array_equal(u, v), (name, ("grad", "param", "state")[k - 1], i)
    assert a[4] < b[4], (name, "pool requests", a[4], b[4])


@pytest.mark.parametrize("dtype", [np.float32, np.float64])
@pytest.mark.parametrize("case", [c for c in CASES if c[0] in ("cnn_small", "cnn_c5")], ids=["cnn_small", "cnn_c5"])
@pytest.mark.parametrize("engine", ["literal", "lean", "fused"])
def test_train_step_with_cpu_literal_conv_gradients(host, case, dtype, engine):
    """The same step with the conv gradients in the CPU backend's literal arithmetic (gradient mode 1: grad_output re-read
    as [Cout, B*L], batch-major col2im): what the reference's CPU backend returns for batch > 1."""
    from oracle import train as otrain
    name, spec, in_shape, ncls, optspec, _ = case
    tol = TOL[np.dtype(dtype)]
    params, x, y = kaiming_uniform_problem(spec, in_shape, ncls, 15, dtype)
    ref = otrain.Sequential(spec, params, dtype, conv_mode=1)
    rloss, rgrads = ref.loss_and_grads(x, y)
    if dtype == np.float32:  # truth: the literal arithmetic carried out in float64
        tloss, tgrads = otrain.Sequential(spec, params, np.float64, conv_mode=1).loss_and_grads(x.astype(np.float64), y.astype(np.float64))
    else:
        tloss, tgrads = rloss, rgrads
    correct = otrain.Sequential(spec, params, dtype, conv_mode=0).loss_and_grads(x, y)[1]
    host.set_conv_grad_mode(1)
    model = host.Model(spec, params, optspec, dtype, literal_engine=engine == "literal", fused=engine == "fused")
    try:
        model.set_batch(x, y)
        gloss = model.backward()
        assert abs(gloss - tloss) <= tol * abs(tloss)
        for i, rg in enumerate(rgrads):
            parity.check("train step grad, literal conv gradients", model.grad(i), tgrads[i], dtype,
                         oracle=rg if dtype == np.float32 else None, case=(name, engine, i), kink=True)
        # the first layer's weight gradient passes through both literal gradients: it must differ from the mathematical one
        assert not close(model.grad(0), correct[0], 1e-3)
    finally:
        model.close()
        host.set_conv_grad_mode(0)


@pytest.mark.parametrize("dtype", [np.float32, np.float64])
@pytest.mark.parametrize("optspec", ["sgd 0.05 0.9 0.0005 0", "adam 0.001 0.9 0.999 1e-08 0.01 0"])
@pytest.mark.parametrize("engine", ["literal", "fused"])
def test_parameter_group_overrides(host, dtype, optspec, engine):
    """The last layer's weight and bias move into a group with its own lr / weight decay (and no momentum for SGD):
    ParameterGroup, src/nn/optim/mod.rs:203-258, read by sgd.rs:103-114 / adam.rs:128-134."""
    from oracle import train as otrain
    tol = TOL[np.dtype(dtype)]
    params, x, y = kaiming_uniform_problem(MLP_SMALL, (9, 20), 5, 21, dtype)
    override = (0.2, 0.0, 0.0) if optspec.startswith("sgd") else (0.01, 0.0, None)
    ref = otrain.Sequential(MLP_SMALL, params, dtype)
    ropt = oracle_optimizer(optspec, groups={4: override, 5: override})
    model = host.Model(MLP_SMALL, params, optspec, dtype, literal_engine=engine == "literal", fused=engine == "fused")
    try:
        model.add_param_group([4, 5], *override)
        model.set_batch(x, y)
        for step in range(3):
            _, rgrads = ref.loss_and_grads(x, y)
            ropt.step(ref, rgrads)
            model.train_step()
        for i, rp in enumerate(ref.params):
            if optspec.startswith("sgd"):
                assert close(model.param(i), rp, tol * 64), i
            else:
                assert np.abs(model.param(i).astype(np.float64) - rp).max() <= 0.05 * (0.01 if i >= 4 else 0.001) * 3, i
        # the override took effect: the grouped parameters moved on the group's scale, not the optimizer's
        moved = np.abs(model.param(4) - params[4]).max()
        assert moved > (0.02 if optspec.startswith("adam") else 0.0)
    finally:
        model.close()


C1_SPEC = "conv 1 8 3 1 1; relu"


@pytest.mark.parametrize("dtype", [np.float32, np.float64])
@pytest.mark.parametrize("conv_mode", [0, 1])
@pytest.mark.parametrize("engine", ["literal", "lean", "fused"])
def test_conv_plumbing_relu_sum_backward(host, dtype, conv_mode, engine):
    """The conv plumbing configuration end to end: x U(-1,1) [32,1,28,28], Kaiming-normal W [8,1,3,3], zero bias,
    sum(relu(conv(x) + b)).backward(); loss, input, weight and bias gradients against the oracle in both gradient modes
    (Conv2dOp src/ops/batched.rs:154-217, bias reduction src/ops/basic.rs:10-53, Sum src/ops/reduction.rs:52-140,
    backward src/graph/mod.rs:700-783)."""
    from oracle import train as otrain
    tol = TOL[np.dtype(dtype)]
    rng = np.random.default_rng(1)
    x = rng.uniform(-1, 1, (32, 1, 28, 28)).astype(dtype)
    w = (rng.standard_normal((8, 1, 3, 3)) * np.sqrt(2.0 / 9.0)).astype(dtype)
    b = np.zeros(8, dtype)
    ref = otrain.Sequential(C1_SPEC, [w, b], dtype, conv_mode=conv_mode)
    rloss, rgrads, rgx = ref.loss_and_grads(x, None, loss_kind="sum", want_input_grad=True)
    if dtype == np.float32:  # truth: the same arithmetic (either gradient mode) in float64 on the same f32 values
        t = otrain.Sequential(C1_SPEC, [w, b], np.float64, conv_mode=conv_mode)
        tloss, tgrads, tgx = t.loss_and_grads(x.astype(np.float64), None, loss_kind="sum", want_input_grad=True)
    else:
        tloss, tgrads, tgx = rloss, rgrads, rgx
    orc_of = (lambda a: a) if dtype == np.float32 else (lambda a: None)
    host.set_conv_grad_mode(conv_mode)
    model = host.Model(C1_SPEC, [w, b], "sgd 0.01", dtype, literal_engine=engine == "literal", fused=engine == "fused")
    try:
        model.configure(loss="sum", input_requires_grad=True)
        model.set_batch(x, np.zeros((32, 1), dtype))
        for _ in range(2):  # the second pass reuses the persistent input leaf and the pool's blocks
            gloss = model.backward()
            tag = ("C1", engine, conv_mode)
            parity.check("plumbing loss", np.array([gloss]), np.array([tloss], np.float64), dtype, oracle=orc_of(np.array([rloss])), case=tag)
            parity.check("plumbing input grad", model.input_grad(x.shape), tgx, dtype, oracle=orc_of(rgx), case=tag)
            parity.check("plumbing weight grad", model.grad(0), tgrads[0], dtype, oracle=orc_of(rgrads[0]), case=tag)
            parity.check("plumbing bias grad", model.grad(1), tgrads[1], dtype, oracle=orc_of(rgrads[1]), case=tag)
        assert np.array_equal(model.param(0), w) and np.array_equal(model.param(1), b)  # no optimizer step was taken
    finally:
        model.close()
        host.set_conv_grad_mode(0)


@pytest.mark.parametrize("dtype", [np.float32, np.float64])
@pytest.mark.parametrize("engine", ["literal", "lean", "fused"])
def test_batchnorm_running_statistics_and_evaluation_forward(host, dtype, engine):
    """Two training steps update the running mean / variance like the oracle; in evaluation mode the forward pass
    uses them and skips dropout."""
    from oracle import train as otrain
    tol = TOL[np.dtype(dtype)]
    params, x, y = kaiming_uniform_problem(CNN_CLS_SMALL, (6, 3, 8, 8), 5, 9, dtype)
    ref = otrain.Sequential(CNN_CLS_SMALL, params, dtype)
    ropt = otrain.SGD(0.05)
    model = host.Model(CNN_CLS_SMALL, params, "sgd 0.05", dtype, literal_engine=engine == "literal", fused=engine == "fused")
    try:
        model.set_batch(x, y)
        for _ in range(2):
            _, rg = ref.loss_and_grads(x, y)
            ropt.step(ref, rg)
            model.train_step()
        state = model.state()
        rstate = [a for li in sorted(ref.running) for a in ref.running[li]]
        assert len(state) == len(rstate) == 4
        for got, want in zip(state, rstate):
            assert close(got, want, 16 * tol)
        ref.training = False
        model.set_training(False)
        want, _ = ref.forward(x)
        assert close(model.forward().reshape(want.shape), want, 64 * tol)
        model.set_training(True)
        ref.training = True
        rloss, _ = ref.loss_and_grads(x, y)
        assert abs(model.train_step() - rloss) <= 64 * tol * abs(rloss)
    finally:
        model.close()


def test_adam_update_matches_oracle_given_same_gradient_sign_structure(host):
    """For Adam compare the update where the gradient is well away from zero (|g| > 1e-3 max|g|): there the
    parameter delta must match the oracle tightly."""
    from oracle import train as otrain
    dtype = np.float32
    params, x, y = kaiming_uniform_problem(CNN_SMALL, (5, 3, 8, 8), 5, 6, dtype)
    ref = otrain.Sequential(CNN_SMALL, params, dtype)
    ropt = otrain.Adam(1e-3)
    model = host.Model(CNN_SMALL, params, "adam 0.001 0.9 0.999 1e-08 0", dtype)
    try:
        model.set_batch(x, y)
        _, rg = ref.loss_and_grads(x, y)
        ropt.step(ref, rg)
        model.train_step()
        for i, (p0, rp, g) in enumerate(zip(params, ref.params, rg)):
            big = np.abs(g) > 1e-3 * np.abs(g).max()
            d_gpu = (model.param(i) - p0)[big]
            d_ref = (rp - p0)[big]
            assert np.abs(d_gpu - d_ref).max() <= 2e-6, i  # lr = 1e-3: updates are ~1e-3, agree to ~1e-3 relative
    finally:
        model.close()


def test_pool_serves_the_training_loop(host):
    """After the first step the same sizes are requested again: the hit counter grows, device allocations level off."""
    dtype = np.float32
    params, x, y = kaiming_uniform_problem(MLP_C2, (256, 784), 10, 7, dtype)
    model = host.Model(MLP_C2, params, "sgd 0.01", dtype)
    try:
        model.set_batch(x, y)
        model.train_step()
        s1 = host.pool_stats(dtype)
        for _ in range(5):
            model.train_step()
        s2 = host.pool_stats(dtype)
        requests = (s2["pool_hits"] + s2["pool_misses"]) - (s1["pool_hits"] + s1["pool_misses"])
        hits = s2["pool_hits"] - s1["pool_hits"]
        assert requests > 0 and hits / requests > 0.85, (s1, s2)
    finally:
        model.close()


def test_error_messages_follow_the_reference(host):
    dtype = np.float32
    params, x, y = kaiming_uniform_problem(MLP_SMALL, (9, 20), 5, 8, dtype)
    model = host.Model(MLP_SMALL, params, "sgd 0.01", dtype)
    try:
        model.set_batch(x[:, :19], y)
        with pytest.raises(host.HostError, match=r"Input shape \[9, 19\] doesn't match expected last dimension 20"):
            model.train_step()
    finally:
        model.close()
