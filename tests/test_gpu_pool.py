"""The hipMalloc caching allocator behind fx_alloc/fx_free, replaying the traces of tests/test_pool_oracle.py on
the GPU and checking every counter against the oracle state machine step by step."""
import ctypes as C
import random

import numpy as np
import pytest

pytestmark = pytest.mark.gpu


def make_cfg(capi, buckets, literal):
    cfg = capi.PoolConfig()
    cfg.n_buckets = len(buckets)
    cfg.literal_ids = int(literal)
    cfg.best_fit = 0   # the reference's pop-most-recent policy, which is what the oracle state machine restates
    for i, (lo, hi, cap, ev, th) in enumerate(buckets):
        cfg.buckets[i] = capi.BucketConfig(lo, hi, cap, ev, th)
    return cfg


class GpuPool:
    """fx_alloc/fx_free through the raw C ABI, f32 pool."""

    def __init__(self, capi, buckets, literal):
        self.capi = capi
        self.ctx = capi.Context(0, make_cfg(capi, buckets, literal) if buckets is not None else None)

    def alloc(self, n):
        capi = self.capi
        ptr, granted, aid = C.c_void_p(), C.c_int64(0), C.c_uint64(0)
        capi.check(capi.lib.fx_alloc(self.ctx.h, capi.FX_F32, n, C.byref(ptr), C.byref(granted), C.byref(aid)))
        return ptr.value, granted.value, aid.value

    def free(self, ptr, aid):
        self.capi.check(self.capi.lib.fx_free(self.ctx.h, self.capi.FX_F32, ptr, aid))

    def stats(self):
        return self.ctx.pool_stats()

    def close(self):
        self.ctx.close()


SMALL = [(1, 10, 3, 2, -1), (11, 100, 2, 1, -1)]
KEYS = ("total_allocations", "active_allocations", "pool_hits", "pool_misses", "underflow_misses", "active_table_len",
        "device_allocs", "device_frees")


@pytest.mark.parametrize("literal", [True, False])
def test_random_trace_matches_oracle_counters(literal):
    import oracle as orc
    from ferrox_amd import capi
    rng = random.Random(7)
    gp = GpuPool(capi, SMALL, literal)
    op = orc.Pool(SMALL, literal=literal)
    live = []  # (ptr, granted, gpu_id, oracle_id)
    try:
        for step in range(400):
            if live and rng.random() < 0.5:
                ptr, granted, gid, oid = live.pop(rng.randrange(len(live)))
                gp.free(ptr, gid)
                op.free(granted, oid)
            else:
                n = rng.choice([1, 2, 5, 9, 10, 11, 40, 100])
                ptr, granted, gid = gp.alloc(n)
                og, oid = op.alloc(n)
                assert (granted, gid) == (og, oid), step
                live.append((ptr, granted, gid, oid))
            gs, os_ = gp.stats(), op.stats()
            assert {k: gs[k] for k in KEYS} == {k: os_[k] for k in KEYS}, step
            for b in range(2):
                gb, ob = gp.ctx.bucket_stats(b), op.bucket_stats(b)
                assert (gb["pooled_blocks"], gb["total_allocations"], gb["total_evictions"], gb["av_allocations"],
                        gb["max_allocations"]) == (ob["pooled"], ob["total_allocations"], ob["total_evictions"],
                                                   ob["av_allocations"], ob["max_allocations"]), (step, b)
    finally:
        gp.close()


def test_zero_size_and_unroutable_size_are_errors():
    from ferrox_amd import capi
    gp = GpuPool(capi, SMALL, False)
    try:
        with pytest.raises(capi.FerroxHipError, match="Cannot allocate zero-sized CUDA memory"):
            gp.alloc(0)
        with pytest.raises(capi.FerroxHipError, match="No bucket configured for allocation size 101"):
            gp.alloc(101)
        with pytest.raises(capi.FerroxHipError, match="not owned by this pool"):
            gp.free(12345, 1)
        with pytest.raises(capi.FerroxHipError, match="exceed the address space"):
            gp.alloc(1 << 62)
        # a second release of the same block is refused instead of freeing memory that sits in the pool
        ptr, _, aid = gp.alloc(7)
        gp.free(ptr, aid)
        with pytest.raises(capi.FerroxHipError, match="already released"):
            gp.free(ptr, aid)
        again, _, aid2 = gp.alloc(7)
        assert again == ptr   # the block is still pooled and usable
        gp.free(again, aid2)
    finally:
        gp.close()


def test_default_config_hit_rate_in_a_training_like_loop():
    """Steady-state reuse with the default buckets: released in reverse creation order (LIFO) every request is a
    hit after the first pass; released in creation order the reference's pop-most-recent policy produces underflow
    misses inside a bucket, exactly as the oracle state machine predicts."""
    import oracle as orc
    from ferrox_amd import capi
    sizes = [10, 256 * 10, 256 * 128, 256 * 256, 784 * 256, 256 * 16384]
    ctx = capi.Context(0)
    try:
        for it in range(20):
            bufs = [ctx.empty((n,)) for n in sizes]
            for b in reversed(bufs):
                b.free()
        st = ctx.pool_stats()
        assert st["pool_misses"] == len(sizes) and st["pool_hits"] == 19 * len(sizes) and st["underflow_misses"] == 0
        assert st["device_allocs"] == len(sizes) and st["bytes_in_use"] == 0
        ctx.pool_cleanup()
        st = ctx.pool_stats()
        assert st["bytes_pooled"] == 0 and st["device_frees"] == len(sizes)
        assert [ctx.bucket_stats(b)["max_allocations"] for b in range(4)] == [4096, 1024, 256, 16]
    finally:
        ctx.close()
    ctx = capi.Context(0, make_cfg(capi, orc.DEFAULT_BUCKETS, False))
    op = orc.Pool(literal=False)
    try:
        for it in range(10):
            bufs = [ctx.empty((n,)) for n in sizes]
            obufs = [op.alloc(n) for n in sizes]
            for b, (og, oid) in zip(bufs, obufs):
                assert b.granted == og
                b.free()
                op.free(og, oid)
        gs, os_ = ctx.pool_stats(), op.stats()
        assert {k: gs[k] for k in KEYS} == {k: os_[k] for k in KEYS}
        assert gs["underflow_misses"] > 0
    finally:
        ctx.close()
    # the library default (best fit inside the bucket) serves the same creation-order loop without underflows
    ctx = capi.Context(0)
    try:
        for it in range(10):
            bufs = [ctx.empty((n,)) for n in sizes]
            for b in bufs:
                b.free()
        st = ctx.pool_stats()
        assert st["underflow_misses"] == 0 and st["pool_misses"] == len(sizes) and st["pool_hits"] == 9 * len(sizes)
    finally:
        ctx.close()


def test_reused_block_is_not_zeroed_but_usable():
    from ferrox_amd import capi
    with capi.Context(0) as ctx:
        a = ctx.upload(np.arange(1000, dtype=np.float32))
        ptr = a.ptr
        a.free()
        b = ctx.empty((1000,))
        assert b.ptr == ptr                          # LIFO reuse of the most recently returned block
        assert np.array_equal(b.numpy(), np.arange(1000, dtype=np.float32))  # dirty on purpose (context.rs:72-73)
        c = ctx.fill((1000,), 3.0)
        assert np.all(c.numpy() == 3.0)


def test_entry_points_are_thread_safe():
    """Ferrox's own tests run on parallel threads against one process-wide backend (manager.rs:343-353): calls from
    several threads into one context - pool traffic plus kernels that share the library scratch (split-K partial
    sums, weight images, reduction partials) - must give the single-threaded results bit for bit."""
    import threading
    from ferrox_amd import capi
    ctx = capi.Context(0)
    try:
        rng = np.random.default_rng(90)
        x = rng.uniform(-1, 1, (4, 32, 12, 56)).astype(np.float32)
        w = (rng.standard_normal((96, 32, 3, 3)) * 0.06).astype(np.float32)
        g = rng.standard_normal((4, 96, 12, 56)).astype(np.float32)
        m = rng.standard_normal((512, 2048)).astype(np.float32)
        dx_, dw_, dg_, dm_ = ctx.upload(x), ctx.upload(w), ctx.upload(g), ctx.upload(m)
        dgam0 = ctx.upload(np.ones(96, np.float32))
        dgs_ = ctx.upload(rng.standard_normal((4, 96, 6, 28)).astype(np.float32))

        def work():
            y = ctx.conv2d_fwd(dx_, dw_, (1, 1), (1, 1)).numpy()
            dw = ctx.conv2d_wgrad(dx_, dg_, w.shape, (1, 1), (1, 1)).numpy()
            dxx = ctx.conv2d_dgrad(dg_, dw_, x.shape, (1, 1), (1, 1)).numpy()
            s0 = ctx.reduce("sum", dm_, 0).numpy()
            mx = ctx.reduce("max", dm_, 1).numpy()
            bg = ctx.bias_grad(dg_, 4, 96, 12 * 56).numpy()
            mean, var = ctx.batchnorm_stats(dg_)                      # partial moments in the shared scratch
            _, dgam, dbet = ctx.batchnorm_bwd(dg_, dg_, mean, var, dgam0, 1e-5, need_dx=False)
            sdx = ctx.conv2d_dgrad(dgs_, dw_, x.shape, (2, 2), (1, 1)).numpy()   # class sub-filters in the scratch
            mm = ctx.gemm(dm_, dm_, False, True).numpy()                # split-K partial sums
            return y, dw, dxx, s0, mx, bg, mean.numpy(), var.numpy(), dgam.numpy(), dbet.numpy(), sdx, mm

        want = work()
        results, errors = {}, []

        def runner(i):
            try:
                for _ in range(6):
                    results[i] = work()
            except Exception as e:  # noqa: BLE001
                errors.append(repr(e))

        threads = [threading.Thread(target=runner, args=(i,)) for i in range(6)]
        for t in threads:
            t.start()
        for t in threads:
            t.join()
        assert not errors, errors
        for i, got in results.items():
            for a, b in zip(got, want):
                assert np.array_equal(a, b), i
        st = ctx.pool_stats(np.float32)
        assert st["active_allocations"] >= 4
    finally:
        ctx.close()
