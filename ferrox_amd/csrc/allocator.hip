// Bucketed hipMalloc caching allocator: the HIP replacement for CudaMemoryPool
// (src/backend/memory/cuda.rs:20-202) and PoolBucket (src/backend/memory/mod.rs:225-359).
//
// Semantics kept from the reference:
//  * sizes are ELEMENTS of the pool's dtype; four default buckets (mod.rs:50-82);
//  * allocate(): the most recently returned block of the bucket is popped; if it is large enough it is a hit
//    (and may be larger than requested), otherwise it is an underflow miss, the block goes back to the bucket
//    and a fresh device allocation is made (a miss);
//  * deallocate(): an id found in the active table sends the block back to its bucket with a timestamp; when the
//    bucket is full the `to_evict` least recently returned blocks (or those older than the threshold) are freed
//    first; an id NOT in the active table means the block is simply freed;
//  * cleanup() frees every pooled block; reset() also clears counters and the active table;
//  * PoolStats / BucketStats counters are updated at the same points as the reference.
// Differences: new device memory is not zeroed (the reference's alloc_zeros, cuda.rs:47-51, zeroes only fresh
// blocks, and reused blocks are dirty there too); with literal_ids = 0 (default) a reused block is registered
// under the id handed to the caller, so it keeps cycling through the pool instead of being freed on its
// second release.
#include <algorithm>
#include <chrono>
#include <climits>
#include <unordered_map>
#include <vector>

#include "common.hpp"

namespace fx {

struct Block {
    void* ptr;
    i64 elems;
    uint64_t id;
    uint64_t ts_ms;
    uint64_t seq;  // tie-break so that equal millisecond stamps keep return order (stable sort in the reference)
};

struct Bucket {
    fx_bucket_config cfg;
    std::vector<Block> blocks;
    i64 st_total = 0, st_evictions = 0, st_avail = 0;
};

struct Pool {
    std::mutex mu;
    int elem_size = 4;
    int literal_ids = 0;
    int best_fit = 0;
    hipStream_t stream = nullptr;  // work that may still touch a block is queued here
    const bool* recording = nullptr;  // the owning context's flag: nothing is evicted (it would wait for the stream) while it is set
    std::vector<Bucket> buckets;
    std::unordered_map<uint64_t, int> active;         // allocation id -> bucket index
    struct Live { i64 elems; bool held; };            // held: handed to a caller (not sitting in a bucket)
    std::unordered_map<void*, Live> live;             // every device block this pool owns
    uint64_t counter = 0, seq = 0;
    fx_pool_stats st{};
};

static uint64_t now_ms() {
    using namespace std::chrono;
    return (uint64_t)duration_cast<milliseconds>(system_clock::now().time_since_epoch()).count();
}

// `drained`: one stream wait covers every block freed in the same batch -- the blocks sit in the pool, so only work
// queued before the batch began can still touch them -- and the caller keeps one flag per batch.
static void device_free(Pool* p, const Block& b, bool& drained) {
    if (!drained) {
        (void)hipStreamSynchronize(p->stream);  // kernels already queued may still use the block
        drained = true;
    }
    (void)hipFree(b.ptr);
    p->live.erase(b.ptr);
    p->st.device_frees += 1;
    p->st.bytes_pooled -= b.elems * p->elem_size;
}

// PoolBucket::return_allocation, mod.rs:263-288
static void bucket_return(Pool* p, Bucket& b, Block blk) {
    const i64 cur = (i64)b.blocks.size();
    bool drained = false;
    if (cur >= b.cfg.max_blocks && !(p->recording && *p->recording)) {
        if (b.cfg.eviction_threshold_ms >= 0) {  // evict_older_than, mod.rs:307-320
            const uint64_t now = now_ms();
            std::vector<Block> keep;
            for (auto& x : b.blocks) {
                if ((now > x.ts_ms ? now - x.ts_ms : 0) <= (uint64_t)b.cfg.eviction_threshold_ms) keep.push_back(x);
                else device_free(p, x, drained);
            }
            b.blocks.swap(keep);
        } else {  // evict_lru, mod.rs:291-305
            const i64 n = std::min<i64>(b.cfg.to_evict, (i64)b.blocks.size());
            if (n > 0) {
                std::stable_sort(b.blocks.begin(), b.blocks.end(), [](const Block& x, const Block& y) {
                    return x.ts_ms != y.ts_ms ? x.ts_ms < y.ts_ms : x.seq < y.seq;
                });
                for (i64 i = 0; i < n; ++i) device_free(p, b.blocks[i], drained);
                b.blocks.erase(b.blocks.begin(), b.blocks.begin() + n);
            }
        }
    }
    b.st_evictions += cur - (i64)b.blocks.size();
    b.st_total = (i64)b.blocks.size() + 1;
    b.st_avail = std::max<i64>(0, b.cfg.max_blocks - ((i64)b.blocks.size() + 1));
    blk.ts_ms = now_ms();
    blk.seq = ++p->seq;
    b.blocks.push_back(blk);
}

Pool* pool_create(const fx_pool_config* cfg, int elem_size, hipStream_t stream, const bool* recording) {
    Pool* p = new Pool();
    p->elem_size = elem_size;
    p->stream = stream;
    p->recording = recording;
    fx_pool_config def{};
    if (!cfg || cfg->n_buckets == 0) {
        // The four size classes of PoolConfig::default (mod.rs:50-82) with block counts sized for 288 GB of HBM:
        // the reference's 500/50/10/2 blocks (chosen for a 4-8 GB card) evict and re-allocate on every step of
        // the CNN config, where more than ten 1-32 MiB activations are alive at once.
        def.n_buckets = 4;
        def.literal_ids = cfg ? cfg->literal_ids : 0;
        def.best_fit = cfg ? cfg->best_fit : 1;
        def.buckets[0] = {1, 1024, 4096, 512, -1};
        def.buckets[1] = {1025, 262144, 1024, 128, -1};
        def.buckets[2] = {262145, 16777216, 256, 32, -1};
        def.buckets[3] = {16777217, INT64_MAX, 16, 4, -1};
        cfg = &def;
    }
    if (cfg->n_buckets < 0 || cfg->n_buckets > FX_MAX_BUCKETS) {
        set_error("pool config: n_buckets %d out of range", cfg->n_buckets);
        delete p;
        return nullptr;
    }
    p->literal_ids = cfg->literal_ids;
    p->best_fit = cfg->best_fit;
    for (int i = 0; i < cfg->n_buckets; ++i) {
        Bucket b;
        b.cfg = cfg->buckets[i];
        b.st_avail = b.cfg.max_blocks;
        p->buckets.push_back(b);
    }
    return p;
}

void pool_destroy(Pool* p) {
    if (!p) return;
    for (auto& kv : p->live) (void)hipFree(kv.first);
    delete p;
}

static void note_peak(Pool* p) {
    p->st.peak_bytes = std::max(p->st.peak_bytes, p->st.bytes_in_use + p->st.bytes_pooled);
}

}  // namespace fx

using namespace fx;

static Pool* get_pool(fx_ctx* c, int dtype) {
    if (!c || (dtype != FX_F32 && dtype != FX_F64)) return nullptr;
    return c->pools[dtype];
}

extern "C" {

// CudaMemoryPool::allocate, cuda.rs:56-101
int fx_alloc(fx_ctx* c, int dtype, int64_t n, void** ptr, int64_t* granted, uint64_t* id_out) {
    FX_CHECK_CTX(c);
    Pool* p = get_pool(c, dtype);
    FX_REQUIRE(p != nullptr, "fx_alloc: unknown dtype %d", dtype);
    FX_REQUIRE(ptr && granted && id_out, "fx_alloc: null output");
    FX_REQUIRE(n != 0, "Cannot allocate zero-sized CUDA memory");
    FX_REQUIRE(n > 0, "fx_alloc: negative size");
    FX_REQUIRE(n <= (INT64_MAX >> 4), "fx_alloc: %lld elements exceed the address space", (long long)n);
    std::lock_guard<std::mutex> lk(p->mu);
    p->counter += 1;
    const uint64_t id = p->counter;
    int bi = -1;
    for (size_t i = 0; i < p->buckets.size(); ++i)
        if (n >= p->buckets[i].cfg.min_elems && n <= p->buckets[i].cfg.max_elems) { bi = (int)i; break; }
    if (bi < 0) {  // the reference panics here (cuda.rs:65-74); an error code is the C-ABI equivalent
        set_error("No bucket configured for allocation size %lld", (long long)n);
        p->counter -= 1;
        return FX_ERR_INVALID;
    }
    p->active[id] = bi;
    Bucket& b = p->buckets[bi];
    if (!b.blocks.empty()) {
        size_t pick = b.blocks.size() - 1;  // reference policy: the most recently returned block
        if (p->best_fit) {                   // smallest block that fits; ties go to the most recently returned
            i64 best = -1;
            for (size_t i = b.blocks.size(); i-- > 0;)
                if (b.blocks[i].elems >= n && (best < 0 || b.blocks[i].elems < best)) { best = b.blocks[i].elems; pick = i; }
        }
        Block blk = b.blocks[pick];
        b.blocks.erase(b.blocks.begin() + pick);
        if (blk.elems >= n) {
            p->st.pool_hits += 1;
            p->st.active_allocations += 1;
            if (!p->literal_ids) blk.id = id;
            p->st.bytes_pooled -= blk.elems * p->elem_size;
            p->st.bytes_in_use += blk.elems * p->elem_size;
            p->live[blk.ptr].held = true;
            *ptr = blk.ptr; *granted = blk.elems; *id_out = blk.id;
            return FX_OK;
        }
        p->st.underflow_misses += 1;
        bucket_return(p, b, blk);
    }
    void* d = nullptr;
    hipError_t e = hipMalloc(&d, (size_t)n * (size_t)p->elem_size);
    if (e != hipSuccess && !c->capturing) {
        // one retry after releasing everything cached
        bool drained = false;
        for (auto& bk : p->buckets) { for (auto& x : bk.blocks) device_free(p, x, drained); bk.blocks.clear(); }
        e = hipMalloc(&d, (size_t)n * (size_t)p->elem_size);
    }
    if (e != hipSuccess) {
        (void)hipGetLastError();
        p->active.erase(id);
        set_error("Failed to allocate GPU memory: %s (%lld elements)", hipGetErrorString(e), (long long)n);
        return FX_ERR_OOM;
    }
    p->live[d] = Pool::Live{n, true};
    p->st.device_allocs += 1;
    p->st.pool_misses += 1;  // update_stats, cuda.rs:188-192
    p->st.total_allocations += 1;
    p->st.active_allocations += 1;
    p->st.bytes_in_use += n * p->elem_size;
    note_peak(p);
    *ptr = d; *granted = n; *id_out = id;
    return FX_OK;
}

// CudaMemoryPool::deallocate, cuda.rs:103-111
int fx_free(fx_ctx* c, int dtype, void* ptr, uint64_t id) {
    FX_CHECK_CTX(c);
    Pool* p = get_pool(c, dtype);
    FX_REQUIRE(p != nullptr, "fx_free: unknown dtype %d", dtype);
    std::lock_guard<std::mutex> lk(p->mu);
    auto lv = p->live.find(ptr);
    FX_REQUIRE(lv != p->live.end(), "fx_free: pointer %p is not owned by this pool", ptr);
    FX_REQUIRE(lv->second.held, "fx_free: pointer %p was already released", ptr);
    if (c->capturing) {
        // the graph being recorded will use this address at every launch: the block goes back to the pool when the graph
        // is destroyed (fx_graph_destroy), not now
        for (const auto& h : c->capture_held) FX_REQUIRE(h.ptr != ptr, "fx_free: pointer %p was already released", ptr);
        c->capture_held.push_back(fx_ctx::Held{dtype, ptr, id});
        return FX_OK;
    }
    lv->second.held = false;
    const i64 elems = lv->second.elems;
    p->st.bytes_in_use -= elems * p->elem_size;
    auto it = p->active.find(id);
    if (it != p->active.end()) {
        const int bi = it->second;
        p->active.erase(it);
        p->st.active_allocations -= 1;
        p->st.bytes_pooled += elems * p->elem_size;
        // Kernels already queued may still read the block; reuse happens on the same stream, so order is kept.
        bucket_return(p, p->buckets[bi], Block{ptr, elems, id, 0, 0});
    } else {
        // unknown id: the reference drops the allocation, i.e. frees the device memory
        p->st.bytes_pooled += elems * p->elem_size;  // device_free subtracts it again
        bool drained = false;
        device_free(p, Block{ptr, elems, id, 0, 0}, drained);
    }
    note_peak(p);
    return FX_OK;
}

int fx_pool_cleanup(fx_ctx* c, int dtype) {  // cuda.rs:113-119
    FX_CHECK_CTX(c);
    FX_NOT_RECORDING(c, "fx_pool_cleanup");
    Pool* p = get_pool(c, dtype);
    FX_REQUIRE(p != nullptr, "fx_pool_cleanup: unknown dtype %d", dtype);
    FX_HIP_CHECK(hipStreamSynchronize(c->stream));
    std::lock_guard<std::mutex> lk(p->mu);
    bool drained = false;  // waits once more under the lock: another thread may have returned a block since the wait above
    for (auto& b : p->buckets) { for (auto& x : b.blocks) device_free(p, x, drained); b.blocks.clear(); }
    return FX_OK;
}

int fx_pool_reset(fx_ctx* c, int dtype) {  // cuda.rs:125-133
    FX_CHECK_CTX(c);
    FX_NOT_RECORDING(c, "fx_pool_reset");
    Pool* p = get_pool(c, dtype);
    FX_REQUIRE(p != nullptr, "fx_pool_reset: unknown dtype %d", dtype);
    FX_HIP_CHECK(hipStreamSynchronize(c->stream));
    std::lock_guard<std::mutex> lk(p->mu);
    bool drained = false;  // waits once more under the lock: another thread may have returned a block since the wait above
    for (auto& b : p->buckets) { for (auto& x : b.blocks) device_free(p, x, drained); b.blocks.clear(); }
    p->active.clear();
    p->counter = 0;
    const i64 in_use = p->st.bytes_in_use, allocs = p->st.device_allocs, frees = p->st.device_frees;
    p->st = fx_pool_stats{};
    p->st.bytes_in_use = in_use;  // blocks still held by the caller stay owned by the pool's live table
    p->st.device_allocs = allocs;
    p->st.device_frees = frees;
    return FX_OK;
}

int fx_pool_stats_get(fx_ctx* c, int dtype, fx_pool_stats* out) {
    FX_CHECK_CTX(c);
    Pool* p = get_pool(c, dtype);
    FX_REQUIRE(p != nullptr && out != nullptr, "fx_pool_stats_get: bad arguments");
    std::lock_guard<std::mutex> lk(p->mu);
    *out = p->st;
    out->allocation_counter = (i64)p->counter;
    out->active_table_len = (i64)p->active.size();
    return FX_OK;
}

int fx_pool_bucket_stats_get(fx_ctx* c, int dtype, int bucket, fx_bucket_stats* out) {
    FX_CHECK_CTX(c);
    Pool* p = get_pool(c, dtype);
    FX_REQUIRE(p != nullptr && out != nullptr, "fx_pool_bucket_stats_get: bad arguments");
    std::lock_guard<std::mutex> lk(p->mu);
    FX_REQUIRE(bucket >= 0 && bucket < (int)p->buckets.size(), "fx_pool_bucket_stats_get: bucket %d out of range", bucket);
    const Bucket& b = p->buckets[bucket];
    out->pooled_blocks = (i64)b.blocks.size();
    out->total_allocations = b.st_total;
    out->total_evictions = b.st_evictions;
    out->av_allocations = b.st_avail;
    out->max_allocations = b.cfg.max_blocks;
    return FX_OK;
}

}  // extern "C"
