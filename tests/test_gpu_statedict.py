"""Optimizer state on disk (OptimizerStateDict, src/nn/optim/mod.rs:263-326) through the mirrored host stack on the GPU:
the moments are copied from the device (the reference skips device tensors when it saves), written in the bincode-2
layout, read back by an independent reader, and a model restored from the bytes continues training with exactly the
bits of the uninterrupted run."""
import numpy as np
import pytest

pytestmark = pytest.mark.gpu

SPEC = "conv 3 4 3 1 1; relu; conv 4 6 3 2 1; relu; flatten; linear 96 5"
ADAM = "adam 0.001 0.9 0.999 1e-08 0.01"


@pytest.fixture(scope="module")
def host():
    from ferrox_amd import host_api
    host_api.init(0, 0)
    yield host_api
    host_api.shutdown()


def problem(dtype, seed=11):
    rng = np.random.default_rng(seed)
    params = [rng.standard_normal((4, 3, 3, 3)).astype(dtype) * 0.3, np.zeros(4, dtype),
              rng.standard_normal((6, 4, 3, 3)).astype(dtype) * 0.3, np.zeros(6, dtype),
              rng.standard_normal((5, 96)).astype(dtype) * 0.2, np.zeros(5, dtype)]
    x = rng.standard_normal((5, 3, 8, 8)).astype(dtype)
    y = np.eye(5, dtype=dtype)[rng.integers(0, 5, 5)]
    return params, x, y


@pytest.mark.parametrize("dtype", [np.float32, np.float64])
@pytest.mark.parametrize("fused", [False, True])
def test_adam_state_saves_device_moments_and_resumes_bit_exactly(host, dtype, fused):
    from oracle import bincode2 as bc
    from oracle import train as otrain
    params, x, y = problem(dtype)
    a = host.Model(SPEC, params, ADAM, dtype, literal_engine=False, fused=fused)
    ref = otrain.Sequential(SPEC, params, dtype)
    ropt = otrain.Adam(1e-3, 0.9, 0.999, 1e-8, 0.01)
    b = None
    try:
        a.set_batch(x, y)
        for _ in range(3):
            a.train_step()
            _, rg = ref.loss_and_grads(x, y)
            ropt.step(ref, rg)
        raw = a.optimizer_state()
        sd = bc.decode_state_dict(raw)                              # independent reader
        assert sd["optimizer_type"] == "Adam" and sd["step_count"] == 3
        hp = sd["hyperparameters"]
        assert hp["beta1"] == float(dtype(0.9)) and hp["beta2"] == float(dtype(0.999)) and hp["amsgrad"] == 0.0
        assert hp["lr"] == float(dtype(1e-3)) and hp["eps"] == float(dtype(1e-8)) and hp["weight_decay"] == float(dtype(0.01))
        assert len(sd["parameter_groups"]) == 1 and sd["parameter_groups"][0]["name"] == "default"
        ids = sd["parameter_groups"][0]["params"]
        assert len(ids) == 6 and ids == sorted(ids)
        assert len(sd["parameter_buffers"]) == 12
        tol = 1e-5 if dtype == np.float32 else 1e-12
        for i, node in enumerate(ids):                               # parameters were created in this order
            for kind, rbuf in (("first_moment", ropt.m[i]), ("second_moment", ropt.v[i])):
                buf = sd["parameter_buffers"][f"{node}_{kind}"]
                assert buf["node_id"] == node and buf["buffer_type"] == kind and buf["device"] == 0
                assert buf["shape"] == list(params[i].shape) and buf["data"].dtype == np.dtype(dtype)
                got = buf["data"].reshape(params[i].shape)
                assert np.abs(got - rbuf).max() <= 64 * tol * max(1e-30, np.abs(rbuf).max()), (i, kind)
        assert bc.encode_state_dict(sd) == raw                      # both writers emit sorted maps: same bytes
        # a second model that starts from a's parameters and the saved state continues exactly like a
        b = host.Model(SPEC, [a.param(i) for i in range(6)], "adam 0.5 0.5 0.5 0.5 0", dtype, literal_engine=False, fused=fused)
        b.load_optimizer_state(raw)
        b.set_batch(x, y)
        for _ in range(2):
            la, lb = a.train_step(), b.train_step()
            assert la == lb
        for i in range(6):
            assert np.array_equal(a.param(i), b.param(i)), i
        assert b.optimizer_state() == a.optimizer_state()
        # bytes written by the independent writer load as well (maps in another order)
        sd2 = bc.decode_state_dict(a.optimizer_state())
        sd2["parameter_buffers"] = dict(reversed(list(sd2["parameter_buffers"].items())))
        b.load_optimizer_state(bc.encode_state_dict(sd2))
        assert b.optimizer_state() == a.optimizer_state()
    finally:
        a.close()
        if b is not None:
            b.close()


def test_state_dict_errors_follow_the_reference(host):
    from oracle import bincode2 as bc
    params, x, y = problem(np.float32)
    adam = host.Model(SPEC, params, ADAM, np.float32)
    sgd = host.Model(SPEC, params, "sgd 0.05", np.float32)
    adam64 = host.Model(SPEC, params, ADAM, np.float64)
    try:
        for m in (adam, sgd, adam64):
            m.set_batch(x, y)
            m.train_step()
        sd = bc.decode_state_dict(sgd.optimizer_state())
        assert sd["optimizer_type"] == "SGD" and sd["step_count"] == 0 and sd["parameter_buffers"] == {}
        assert sd["hyperparameters"] == {"lr": float(np.float32(0.05)), "momentum": 0.0, "weight_decay": 0.0, "nesterov": 0.0}
        # SGD::new stores the optimizer's values in its default group (sgd.rs:28-45)
        grp = sd["parameter_groups"][0]
        assert (grp["lr"], grp["weight_decay"], grp["momentum"]) == (float(np.float32(0.05)), 0.0, 0.0)
        with pytest.raises(host.HostError, match="Expected Adam state dict, got SGD"):
            adam.load_optimizer_state(sgd.optimizer_state())
        with pytest.raises(host.HostError, match="Expected SGD state dict, got Adam"):
            sgd.load_optimizer_state(adam.optimizer_state())
        with pytest.raises(host.HostError, match="Expected f64 data"):
            adam64.load_optimizer_state(adam.optimizer_state())
        raw = adam.optimizer_state()
        for bad in (raw[:-3], raw + b"\x00", b"", b"\xff" + raw[1:]):
            with pytest.raises(host.HostError):
                adam.load_optimizer_state(bad)
        adam.load_optimizer_state(raw)                             # and the model still works afterwards
        adam.train_step()
    finally:
        for m in (adam, sgd, adam64):
            m.close()


@pytest.mark.parametrize("dtype", [np.float32, np.float64])
@pytest.mark.parametrize("fused", [False, True])
@pytest.mark.parametrize("optspec,kinds", [("sgd 0.05 0.9 0.0005 1", ["momentum"]),
                                           ("adam 0.001 0.9 0.999 1e-08 0.01 1", ["first_moment", "second_moment", "max_second_moment"])])
def test_momentum_and_amsgrad_buffers_are_saved_and_resume_bit_exactly(host, dtype, fused, optspec, kinds):
    """SGD's momentum buffers (sgd.rs:278-360) and Adam's AMSGrad maxima (adam.rs:448-461, 540-553) go through the state
    dictionary: a fresh model built with other hyper-parameters continues exactly like the uninterrupted one."""
    from oracle import bincode2 as bc
    params, x, y = problem(dtype, seed=13)
    a = host.Model(SPEC, params, optspec, dtype, literal_engine=False, fused=fused)
    other = "sgd 0.5" if optspec.startswith("sgd") else "adam 0.5 0.5 0.5 0.5 0"
    b = None
    try:
        a.add_param_group([4, 5], 0.02, 0.0, None)
        a.set_batch(x, y)
        for _ in range(3):
            a.train_step()
        raw = a.optimizer_state()
        sd = bc.decode_state_dict(raw)
        assert sorted({v["buffer_type"] for v in sd["parameter_buffers"].values()}) == sorted(kinds)
        assert len(sd["parameter_buffers"]) == 6 * len(kinds)
        assert [g["name"] for g in sd["parameter_groups"]] == ["default", "group1"]
        assert len(sd["parameter_groups"][0]["params"]) == 4 and len(sd["parameter_groups"][1]["params"]) == 2
        assert sd["parameter_groups"][1]["lr"] == float(dtype(0.02)) and sd["parameter_groups"][1]["momentum"] is None
        assert bc.encode_state_dict(sd) == raw
        b = host.Model(SPEC, [a.param(i) for i in range(6)], other, dtype, literal_engine=False, fused=fused)
        b.load_optimizer_state(raw)
        b.set_batch(x, y)
        for _ in range(2):
            assert a.train_step() == b.train_step()
        for i in range(6):
            assert np.array_equal(a.param(i), b.param(i)), i
        assert b.optimizer_state() == a.optimizer_state()
    finally:
        a.close()
        if b is not None:
            b.close()


@pytest.mark.parametrize("fused", [False, True])
def test_state_from_another_model_is_refused(host, fused):
    """A state dictionary whose buffers do not belong to this model's parameters: a node id that no restored group names is
    refused when the state is loaded; a buffer of another shape when the parameter is next updated (the fused update
    would otherwise read and write past the end of the buffer)."""
    from oracle import bincode2 as bc
    params, x, y = problem(np.float32, seed=17)
    m = host.Model(SPEC, params, ADAM, np.float32, literal_engine=False, fused=fused)
    try:
        m.set_batch(x, y)
        m.train_step()
        good = m.optimizer_state()
        sd = bc.decode_state_dict(good)
        ids = sd["parameter_groups"][0]["params"]
        # (a) a buffer names a node that is in no group
        bad = bc.decode_state_dict(good)
        key = f"{ids[0]}_first_moment"
        buf = bad["parameter_buffers"].pop(key)
        buf["node_id"] = 9999
        bad["parameter_buffers"]["9999_first_moment"] = buf
        with pytest.raises(host.HostError, match="names node 9999, which is in no parameter group"):
            m.load_optimizer_state(bc.encode_state_dict(bad))
        # (b) the moments of the first conv weight [4,3,3,3] and of its bias [4] trade places
        bad = bc.decode_state_dict(good)
        for kind in ("first_moment", "second_moment"):
            b0, b1 = bad["parameter_buffers"][f"{ids[0]}_{kind}"], bad["parameter_buffers"][f"{ids[1]}_{kind}"]
            b0["node_id"], b1["node_id"] = ids[1], ids[0]
            bad["parameter_buffers"][f"{ids[0]}_{kind}"], bad["parameter_buffers"][f"{ids[1]}_{kind}"] = b1, b0
        m.load_optimizer_state(bc.encode_state_dict(bad))
        with pytest.raises(host.HostError, match=r"buffer 'first_moment' of node \d+ has shape \[4\], the parameter has \[4, 3, 3, 3\]"):
            m.train_step()
        m.load_optimizer_state(good)          # the model recovers with a matching state
        m.train_step()
    finally:
        m.close()
