"""fx_reduce_max_noalloc_f32 (slice partials in the library's fixed device array) against fx_reduce_max_f32."""
import numpy as np
import pytest

from ferrox_amd import capi

pytestmark = pytest.mark.gpu


def _both(ctx, a_host, axis):
    a = ctx.upload(a_host)
    ref, ref_idx = ctx.reduce("max", a, axis, want_idx=True)
    oshape = a_host.shape[:axis] + a_host.shape[axis + 1:]
    n_out = max(1, int(np.prod(oshape, dtype=np.int64)))
    out = ctx.empty((n_out,), np.float32)
    idx = capi._RawI64(ctx, n_out)
    ctx.reduce_max_noalloc(a, axis, out, idx)
    got, got_idx = out.numpy().reshape(oshape), idx.numpy().reshape(oshape)
    np.testing.assert_array_equal(got, ref.numpy().reshape(oshape))
    np.testing.assert_array_equal(got_idx, ref_idx)
    # and against numpy: exact maxima, first index attaining them
    np.testing.assert_array_equal(got, a_host.max(axis=axis))
    np.testing.assert_array_equal(got_idx, a_host.argmax(axis=axis))


def test_noalloc_reduce_max_two_calls_second_smaller():
    rng = np.random.default_rng(11)
    with capi.Context(0) as ctx:
        # split column reduction (24 slices of partials), then a smaller one that reuses the same array,
        # then split row reductions (one long run; a few long rows)
        big = rng.standard_normal((2048, 4096)).astype(np.float32)
        big[5, 7] = big[900, 7] = 9.0  # a tie: the first index wins
        _both(ctx, big, 0)
        small = rng.standard_normal((300, 1024)).astype(np.float32)
        _both(ctx, small, 0)
        _both(ctx, big.reshape(-1), 0)
        _both(ctx, small.reshape(-1), 0)
        _both(ctx, big[:3], 1)
        _both(ctx, small, 1)


def test_noalloc_reduce_max_allocates_nothing_on_a_fresh_context():
    """On a context that has never run a split reduction the library's growing scratch region does not exist yet: the
    no-alloc call must leave it that way (its partials go to the fixed array), take nothing from the driver and nothing new
    from the pool; the ordinary entry point on the same shape then does create the region."""
    rng = np.random.default_rng(12)
    a_host = rng.standard_normal((2048, 4096)).astype(np.float32)
    with capi.Context(0) as ctx:
        a = ctx.upload(a_host)
        out = ctx.empty((4096,), np.float32)
        idx = capi._RawI64(ctx, 4096)
        ctx.sync()
        assert ctx.scratch_info()["bytes"] == 0
        pool_before, mem_before = ctx.pool_stats(np.float32), ctx.device_mem_info()["free"]
        ctx.reduce_max_noalloc(a, 0, out, idx)             # 24 slices of partials: a split reduction
        ctx.reduce_max_noalloc(a.reshape(a.size), 0, out, idx)  # one long run: 768 slices
        ctx.sync()
        pool_after, mem_after = ctx.pool_stats(np.float32), ctx.device_mem_info()["free"]
        assert ctx.scratch_info()["bytes"] == 0 and ctx.scratch_info()["current"] == 0
        assert mem_after == mem_before
        for key in ("device_allocs", "active_allocations", "total_allocations"):
            if key in pool_before:
                assert pool_after[key] == pool_before[key], key
        ctx.reduce_max_noalloc(a, 0, out, idx)
        np.testing.assert_array_equal(out.numpy(), a_host.max(axis=0))
        np.testing.assert_array_equal(idx.numpy(), a_host.argmax(axis=0))
        ref, _ = ctx.reduce("max", a, 0, want_idx=True)    # the ordinary entry point grows the context's region
        assert ctx.scratch_info()["bytes"] > 0
        np.testing.assert_array_equal(ref.numpy(), a_host.max(axis=0))


def test_noalloc_reduce_max_refuses_oversized_partials():
    with capi.Context(0) as ctx:
        # [32768, 512] along axis 0: two column tiles, so the axis is split into 1024 slices whose partials
        # (1024 * 512 values + indices = 6.3 MB) exceed the fixed array
        outer, axis, inner = 1, 32768, 512
        a = ctx.fill((outer * axis * inner,), 1.0, np.float32)
        out = ctx.empty((outer * inner,), np.float32)
        idx = capi._RawI64(ctx, outer * inner)
        with pytest.raises(capi.FerroxHipError) as e:
            capi.check(capi.lib.fx_reduce_max_noalloc_f32(ctx.h, a.ptr, out.ptr, idx.ptr, outer, axis, inner))
        assert e.value.code == 4 and "fixed scratch" in e.value.message
        # without the positions the partials are the values alone (2.1 MB): they fit, and the maxima come out
        capi.check(capi.lib.fx_reduce_max_noalloc_f32(ctx.h, a.ptr, out.ptr, None, outer, axis, inner))
        np.testing.assert_array_equal(out.numpy(), np.ones(outer * inner, np.float32))
