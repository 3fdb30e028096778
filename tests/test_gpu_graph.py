"""Recorded steps (fx_graph_*): a graph replays the calls recorded on a context with the same kernels and arguments, so
every replay must reproduce the eager calls bit for bit -- on the C-ABI with temporaries released while recording, and
for whole training steps of the mirrored host stack (fused engine with SGD and Adam).  Every
graph is launched several times with eager work and waits between the launches, and each launch is checked."""
import ctypes as C

import numpy as np
import pytest

from test_gpu_train import CNN_C5, CNN_CLS_SMALL, CNN_SMALL, MLP_C2, MLP_SMALL, kaiming_uniform_problem

pytestmark = pytest.mark.gpu


@pytest.fixture(scope="module")
def ctx():
    from ferrox_amd import capi
    with capi.Context(0) as c:
        yield c


def chain(ctx, a, b, out):
    """out = sum over axis 1 of relu((a + b) * 0.5 - a), through three temporaries that are released on the way"""
    t1 = ctx.binary("add", a, b)
    t2 = ctx.scalar("mul_scalar", t1, 0.5)
    t1.free()
    t3 = ctx.binary("sub", t2, a)
    t2.free()
    t4 = ctx.unary("relu", t3)
    t3.free()
    ctx.reduce("sum", t4, 1, out=out)
    t4.free()


@pytest.mark.parametrize("dtype", [np.float32, np.float64])
def test_recorded_calls_replay_bit_exact_with_released_temporaries(ctx, dtype):
    rng = np.random.default_rng(3)
    shape = (96, 4100)
    a, b = ctx.upload(rng.standard_normal(shape).astype(dtype)), ctx.upload(rng.standard_normal(shape).astype(dtype))
    out = ctx.empty((shape[0],), dtype)
    chain(ctx, a, b, out)  # eager once: pool, scratch
    before = ctx.pool_stats(dtype)
    ctx.graph_begin()
    chain(ctx, a, b, out)
    g = ctx.graph_end()
    info = ctx.graph_info(g)
    assert info["kernel_nodes"] >= 5 and info["held_blocks"] == 4
    for rep in range(4):
        na, nb = rng.standard_normal(shape).astype(dtype), rng.standard_normal(shape).astype(dtype)
        # new inputs at the recorded addresses; unrelated eager work and a wait between the launches
        from ferrox_amd.capi import check, lib
        check(lib.fx_h2d(ctx.h, a.ptr, na.ctypes.data, na.nbytes))
        check(lib.fx_h2d(ctx.h, b.ptr, nb.ctypes.data, nb.nbytes))
        other = ctx.binary("mul", a, b)          # may not land on a block the graph keeps
        ctx.graph_launch(g)
        got = out.numpy().copy()
        other_host = other.numpy()
        other.free()
        ref = ctx.empty((shape[0],), dtype)
        chain(ctx, a, b, ref)
        assert np.array_equal(got, ref.numpy()), rep
        assert np.array_equal(other_host, na * nb)
        ref.free()
    ctx.graph_destroy(g)
    after = ctx.pool_stats(dtype)
    assert after["active_allocations"] == before["active_allocations"]  # the four temporaries went back to the pool


def test_calls_that_wait_are_refused_while_recording_and_the_recording_survives(ctx):
    from ferrox_amd.capi import FerroxHipError
    a = ctx.upload(np.arange(1024, dtype=np.float32))
    out = ctx.empty((1024,), np.float32)
    ctx.graph_begin()
    ctx.scalar("add_scalar", a, 1.0, out=out)
    with pytest.raises(FerroxHipError, match="recording"):
        out.numpy()  # a device-to-host copy waits for the stream
    with pytest.raises(FerroxHipError, match="recording"):
        ctx.sync()
    g = ctx.graph_end()
    assert ctx.graph_info(g)["kernel_nodes"] == 1
    ctx.graph_launch(g)
    assert np.array_equal(out.numpy(), np.arange(1024, dtype=np.float32) + 1)
    ctx.graph_destroy(g)


@pytest.mark.parametrize("dtype", [np.float32, np.float64])
def test_adam_with_device_bias_corrections_has_the_bits_of_the_scalar_call(ctx, dtype):
    from ferrox_amd.capi import check, lib
    rng = np.random.default_rng(11)
    sfx, ct = ("f32", C.c_float) if dtype == np.float32 else ("f64", C.c_double)
    ns = [5000, 37, 70000]
    host = [[rng.standard_normal(n).astype(dtype) for n in ns] for _ in range(2)]  # p, g
    def run(with_bc):
        p = [ctx.upload(h) for h in host[0]]
        g = [ctx.upload(h) for h in host[1]]
        m = [ctx.fill((n,), 0.0, dtype) for n in ns]
        v = [ctx.fill((n,), 0.0, dtype) for n in ns]
        x = [ctx.fill((n,), 0.0, dtype) for n in ns]
        tab = lambda ts: (C.c_void_p * len(ts))(*[t.ptr for t in ts])
        narr = (C.c_int64 * len(ns))(*ns)
        for step in (1, 2, 3):
            bc1, bc2 = dtype(1) - dtype(0.9) ** step, dtype(1) - dtype(0.999) ** step
            if with_bc:
                bc = ctx.upload(np.array([bc1, bc2], dtype))
                check(getattr(lib, "fx_adam_step_multi_bc_" + sfx)(ctx.h, 3, tab(p), tab(g), tab(m), tab(v), tab(x), narr, ct(1e-3), ct(0.9),
                                                                   ct(0.999), ct(1e-8), ct(0.01), bc.ptr))
                ctx.sync()
                bc.free()
            else:
                check(getattr(lib, "fx_adam_amsgrad_step_multi_" + sfx)(ctx.h, 3, tab(p), tab(g), tab(m), tab(v), tab(x), narr, ct(1e-3),
                                                                        ct(0.9), ct(0.999), ct(1e-8), ct(0.01), ct(bc1), ct(bc2)))
        return [t.numpy().copy() for t in p + m + v + x]
    for a, b in zip(run(True), run(False)):
        assert np.array_equal(a, b)


@pytest.fixture(scope="module")
def host():
    from ferrox_amd import host_api
    host_api.init(0, 0)
    yield host_api
    host_api.shutdown()


GRAPH_CASES = [
    ("mlp_small_fused_sgd", MLP_SMALL, (9, 20), 5, "sgd 0.05 0.9 0.0005 1", "fused"),
    ("cnn_small_fused_sgd", CNN_SMALL, (5, 3, 8, 8), 5, "sgd 0.05", "fused"),
    ("cnn_small_fused_adam_plain", CNN_SMALL, (5, 3, 8, 8), 5, "adam 0.001 0.9 0.999 1e-08 0", "fused"),
    ("cnn_small_fused_adam", CNN_SMALL, (5, 3, 8, 8), 5, "adam 0.001 0.9 0.999 1e-08 0.01 1", "fused"),
    ("mlp_c2_fused_sgd", MLP_C2, (256, 784), 10, "sgd 0.01", "fused"),
    ("cnn_c5_fused_adam", CNN_C5, (256, 3, 32, 32), 10, "adam 0.001 0.9 0.999 1e-08 0", "fused"),
]


@pytest.mark.parametrize("dtype", [np.float32, np.float64])
@pytest.mark.parametrize("case", GRAPH_CASES, ids=[c[0] for c in GRAPH_CASES])
def test_recorded_train_steps_equal_eager_ones_bit_for_bit(host, case, dtype):
    """Seven steps on changing batches: two eager warm-up steps, the recording, four replays; losses, parameters and
    gradients of the model with graphs equal those of the eager model exactly."""
    name, spec, in_shape, ncls, optspec, engine = case
    params, x, y = kaiming_uniform_problem(spec, in_shape, ncls, 7, dtype)
    rng = np.random.default_rng(8)
    batches = [(x, y)] + [(rng.standard_normal(in_shape).astype(dtype), np.eye(ncls, dtype=dtype)[rng.integers(0, ncls, in_shape[0])])
                          for _ in range(6)]
    models = [host.Model(spec, params, optspec, dtype, literal_engine=engine == "literal", fused=engine == "fused") for _ in range(2)]
    models[1].enable_graph()
    for step, (bx, by) in enumerate(batches):
        losses = []
        for m in models:
            m.set_batch(bx, by)
            losses.append(m.train_step())
        assert losses[0] == losses[1], (step, losses)
        info = models[1].graph_info()
        assert (info["kernel_nodes"] > 0) == (step >= 2), (step, info)
        for i in range(len(params)):
            assert np.array_equal(models[0].param(i), models[1].param(i)), (step, i)
            assert np.array_equal(models[0].grad(i), models[1].grad(i)), (step, i)
    for m in models:
        m.close()


def test_models_that_cannot_be_recorded_stay_eager(host):
    """A Dropout layer draws a new mask every step; the op-by-op engines put each updated parameter into a new tensor, which
    a replay would not see: both keep launching their kernels one by one, with unchanged results."""
    for spec, in_shape, optspec, engine in ((CNN_CLS_SMALL, (6, 3, 8, 8), "sgd 0.05", "fused"),
                                            (MLP_SMALL, (9, 20), "sgd 0.01", "lean"),
                                            (MLP_SMALL, (9, 20), "adam 0.001 0.9 0.999 1e-08 0", "literal")):
        params, x, y = kaiming_uniform_problem(spec, in_shape, 5, 9, np.float32)
        models = [host.Model(spec, params, optspec, np.float32, literal_engine=engine == "literal", fused=engine == "fused") for _ in range(2)]
        models[1].enable_graph()
        for step in range(4):
            losses = []
            for m in models:
                m.set_batch(x, y)
                losses.append(m.train_step())
            assert losses[0] == losses[1]
        assert models[1].graph_info()["kernel_nodes"] == 0
        for i in range(len(params)):
            assert np.array_equal(models[0].param(i), models[1].param(i))
        for m in models:
            m.close()


def test_input_leaf_with_gradient_follows_the_batch_with_graphs_enabled(host):
    """A model whose batch enters as a leaf with a gradient is never recorded; with graphs enabled it must still read each
    new batch (not the copy of the first one) and hand out the gradient of that batch."""
    spec, in_shape = MLP_SMALL, (9, 20)
    params, x, y = kaiming_uniform_problem(spec, in_shape, 5, 9, np.float32)
    rng = np.random.default_rng(21)
    models = [host.Model(spec, params, "sgd 0.05", np.float32, literal_engine=False, fused=True) for _ in range(2)]
    for m in models:
        m.configure("cce", input_requires_grad=True)
    models[1].enable_graph()
    for step in range(4):
        bx = rng.standard_normal(in_shape).astype(np.float32)
        losses, grads = [], []
        for m in models:
            m.set_batch(bx, y)
            losses.append(m.train_step())
            grads.append(m.input_grad(in_shape))
        assert losses[0] == losses[1], step
        assert np.array_equal(grads[0], grads[1]), step
        if step:
            assert losses[0] != first  # the batch did change what the model saw
        first = losses[0]
    assert models[1].graph_info()["kernel_nodes"] == 0
    for m in models:
        m.close()


@pytest.mark.parametrize("optspec", ["adam 0.001 0.9 0.999 1e-08 0.01 1", "sgd 0.05 0.9 0.0005 1"])
def test_a_recording_is_dropped_when_the_state_it_holds_changes(host, optspec):
    """Loading optimizer state, adding a parameter group, switching the training mode or the loss after a step was recorded:
    the recording holds the old moment buffers, learning rates and kernel sequence, so the model must record again.  Checked
    against an eager model that gets the same calls: losses, parameters, gradients and the saved optimizer state stay equal."""
    spec, in_shape, ncls = CNN_SMALL, (5, 3, 8, 8), 5
    params, x, y = kaiming_uniform_problem(spec, in_shape, ncls, 7, np.float32)
    rng = np.random.default_rng(31)
    models = [host.Model(spec, params, optspec, np.float32, literal_engine=False, fused=True) for _ in range(2)]
    models[1].enable_graph()

    def steps(n):
        for _ in range(n):
            bx = rng.standard_normal(in_shape).astype(np.float32)
            by = np.eye(ncls, dtype=np.float32)[rng.integers(0, ncls, in_shape[0])]
            losses = []
            for m in models:
                m.set_batch(bx, by)
                losses.append(m.train_step())
            assert losses[0] == losses[1]
        for i in range(len(params)):
            assert np.array_equal(models[0].param(i), models[1].param(i)), i
            assert np.array_equal(models[0].grad(i), models[1].grad(i)), i
        assert models[0].optimizer_state() == models[1].optimizer_state()

    steps(4)
    assert models[1].graph_info()["kernel_nodes"] > 0
    saved = models[0].optimizer_state()
    steps(2)
    for m in models:
        m.load_optimizer_state(saved)          # moments back to the state two steps ago, in new tensors
    assert models[1].graph_info()["kernel_nodes"] == 0
    steps(4)
    assert models[1].graph_info()["kernel_nodes"] > 0
    for m in models:
        m.add_param_group([0, 1], lr=0.01, weight_decay=0.0)
    assert models[1].graph_info()["kernel_nodes"] == 0
    steps(4)
    assert models[1].graph_info()["kernel_nodes"] > 0
    for m in models:
        m.set_training(False)
    assert models[1].graph_info()["kernel_nodes"] == 0
    for m in models:
        m.set_training(True)
    steps(3)
    for m in models:
        m.close()


def test_scratch_that_grows_after_a_recording_is_parked_not_freed(ctx):
    """A recorded split reduction keeps the scratch address of its recording.  A later, larger eager request must leave
    that region alive (parked) until the graph is destroyed; the replay after the growth still gives the eager bits.
    Host-side checks of the region bookkeeping; every kernel runs on valid memory either way."""
    rng = np.random.default_rng(5)
    a = ctx.upload(rng.standard_normal((64, 70000)).astype(np.float32))
    out = ctx.empty((70000,), np.float32)
    ctx.reduce("sum", a, 0, out=out)            # eager once: sizes the scratch region for this call
    ref = out.numpy().copy()
    before = ctx.scratch_info()
    ctx.graph_begin()
    ctx.reduce("sum", a, 0, out=out)
    g = ctx.graph_end()
    assert ctx.scratch_info()["live_graphs"] == before["live_graphs"] + 1
    # a larger request: maxima with positions along axis 0 of [64, 100000 * k] leave 2 slices x 12 bytes per column
    k = 1
    while 2 * 100000 * k * 12 <= before["bytes"]:
        k *= 2
    big = ctx.fill((64, 100000 * k), 1.0, np.float32)
    need_more, _ = ctx.reduce("max", big, 0, want_idx=True)
    grown = ctx.scratch_info()
    assert grown["bytes"] > before["bytes"]
    assert grown["parked_regions"] == before["parked_regions"] + 1 and grown["current"] != before["current"]
    ctx.unary("neg", out, out=out)
    ctx.graph_launch(g)
    assert np.array_equal(out.numpy(), ref)
    ctx.graph_destroy(g)
    after = ctx.scratch_info()
    assert after["live_graphs"] == before["live_graphs"]
    if after["live_graphs"] == 0:
        assert after["parked_regions"] == 0
    assert np.array_equal(need_more.numpy(), np.ones(big.shape[1], np.float32))
    big.free()
