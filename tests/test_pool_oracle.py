"""Scripted traces through the allocator state machine with hand-computed counters
(CudaMemoryPool::allocate/deallocate, src/backend/memory/cuda.rs:55-134; PoolBucket, memory/mod.rs:225-359).
The same traces are replayed on the GPU allocator in tests/test_gpu_pool.py."""
import pytest

import oracle as orc

SMALL = [(1, 10, 3, 2, -1), (11, 100, 2, 1, -1)]   # two buckets: cap 3 evict 2, cap 2 evict 1


def test_zero_size_and_no_bucket():
    p = orc.Pool(SMALL)
    with pytest.raises(ValueError, match="zero-sized"):
        p.alloc(0)
    with pytest.raises(ValueError, match="No bucket"):
        p.alloc(101)


def test_miss_then_hit_then_underflow_literal():
    p = orc.Pool(SMALL, literal=True)
    g1, id1 = p.alloc(4)                # miss #1
    assert (g1, id1) == (4, 1)
    assert p.free(4, id1) == 1          # goes back to bucket 0
    g2, id2 = p.alloc(3)                # pops the 4-block: hit, granted 4, OLD id kept (cuda.rs:79-86)
    assert (g2, id2) == (4, 1)
    st = p.stats()
    assert (st["pool_hits"], st["pool_misses"], st["underflow_misses"]) == (1, 1, 0)
    assert st["total_allocations"] == 1 and st["active_allocations"] == 1   # +1 miss, -1 free, +1 hit
    assert st["active_table_len"] == 1  # id 2 was recorded, id 1 was removed by the first free
    # second release of the reused block: id 1 is unknown now -> dropped (freed), not pooled
    assert p.free(4, id2) == 0
    assert p.bucket_stats(0)["pooled"] == 0 and p.stats()["device_frees"] == 1
    assert p.stats()["active_allocations"] == 1   # the dropped release is not counted: the counter drifts upward
    # underflow: pooled block too small
    g3, id3 = p.alloc(2)                # miss #2 (id 3)
    assert p.free(2, id3) == 1
    g4, id4 = p.alloc(9)                # pops the 2-block, too small -> underflow, pushed back; new block (miss #3)
    assert (g4, id4) == (9, 4)
    st = p.stats()
    assert (st["pool_hits"], st["pool_misses"], st["underflow_misses"]) == (1, 3, 1)
    assert p.bucket_stats(0)["pooled"] == 1


def test_fixed_mode_keeps_cycling():
    p = orc.Pool(SMALL, literal=False)
    _, i1 = p.alloc(5)
    for _ in range(10):
        assert p.free(5, i1) == 1
        g, i1 = p.alloc(5)
        assert g == 5
    st = p.stats()
    assert (st["pool_hits"], st["pool_misses"]) == (10, 1) and st["device_allocs"] == 1 and st["device_frees"] == 0
    assert st["active_allocations"] == 1 and st["active_table_len"] == 1


def test_lru_eviction_when_bucket_full():
    p = orc.Pool(SMALL, literal=False)
    ids = [p.alloc(5)[1] for _ in range(4)]          # 4 misses
    for k, i in enumerate(ids[:3]):
        p.tick()
        assert p.free(5, i) == 1
    assert p.bucket_stats(0)["pooled"] == 3          # bucket now at capacity 3
    p.tick()
    p.free(5, ids[3])                                # full: evict the 2 oldest, then push -> 2 pooled
    bs = p.bucket_stats(0)
    assert bs["pooled"] == 2 and bs["total_evictions"] == 2 and bs["av_allocations"] == 1 and bs["total_allocations"] == 2
    assert p.stats()["device_frees"] == 2
    # the survivors are the most recently returned ones: LIFO pop returns ids[3]'s block first
    p.cleanup()
    assert p.bucket_stats(0)["pooled"] == 0 and p.stats()["device_frees"] == 4


def test_age_eviction_threshold():
    p = orc.Pool([(1, 10, 2, 1, 5)], literal=False)   # threshold 5 ticks
    a, b, c = (p.alloc(3)[1] for _ in range(3))
    p.free(3, a)
    p.tick(10)
    p.free(3, b)
    p.tick(1)
    p.free(3, c)                                      # full (2): evict older than 5 -> drops a's block only
    bs = p.bucket_stats(0)
    assert bs["pooled"] == 2 and bs["total_evictions"] == 1


def test_reset_clears_counters():
    p = orc.Pool(SMALL, literal=True)
    i = p.alloc(5)[1]
    p.free(5, i)
    p.reset()
    st = p.stats()
    assert all(st[k] == 0 for k in ("total_allocations", "active_allocations", "pool_hits", "pool_misses", "underflow_misses",
                                    "active_table_len"))
    assert p.alloc(5) == (5, 1)                       # counter restarted


def test_default_buckets_route_sizes():
    p = orc.Pool(literal=False)
    sizes = [1, 1024, 1025, 262144, 262145, 16777216, 16777217]
    ids = [p.alloc(s)[1] for s in sizes]
    for s, i in zip(sizes, ids):
        p.free(s, i)
    assert [p.bucket_stats(b)["pooled"] for b in range(4)] == [2, 2, 2, 1]
