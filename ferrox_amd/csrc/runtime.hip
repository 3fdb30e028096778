// Context, stream, copies, timing and error reporting of libferrox_hip.so.
// Replaces CudaContextManager (src/backend/cuda/context.rs:30-175) and the named-stream StreamManager
// (src/backend/cuda/stream_manager.rs:97-103): one compute stream, synchronous copies ordered on it.
#include <cstdarg>
#include <cstdlib>
#include <cstring>

#include "common.hpp"

namespace fx {
static thread_local char g_err[512] = "";
void set_error(const char* fmt, ...) {
    va_list ap;
    va_start(ap, fmt);
    vsnprintf(g_err, sizeof(g_err), fmt, ap);
    va_end(ap);
}
int bind_device(int device) {
    int cur = -1;
    if (hipGetDevice(&cur) == hipSuccess && cur == device) return FX_OK;
    FX_HIP_CHECK(hipSetDevice(device));
    return FX_OK;
}
Pool* pool_create(const fx_pool_config* cfg, int elem_size, hipStream_t stream, const bool* recording);
int static_scratch_init(int device);  // reduce.hip
int copy_kernel(fx_ctx* c, void* dst, const void* src, i64 bytes);  // elementwise.hip
void pool_destroy(Pool* p);
}  // namespace fx

void* fx_ctx::get_scratch(i64 bytes) {
    if (bytes <= scratch_bytes) return scratch;
    if (capturing) {  // growing means waiting for the stream and freeing a region the recorded kernels point into
        fx::set_error("the library's scratch region would have to grow to %lld bytes while a graph is being recorded: run the same "
                      "calls once before fx_graph_begin", (long long)bytes);
        return nullptr;
    }
    // Work already queued on the stream may still use the old region.
    if (scratch) {
        if (live_graphs > 0) {
            parked_scratch.push_back(scratch);  // a recorded graph still points into it
        } else {
            if (hipStreamSynchronize(stream) != hipSuccess) return nullptr;
            (void)hipFree(scratch);
        }
        scratch = nullptr;
        scratch_bytes = 0;
    }
    i64 want = std::max<i64>(bytes, 1 << 20);
    want = (want + 255) & ~i64(255);
    if (hipMalloc(&scratch, (size_t)want) != hipSuccess) {
        fx::set_error("scratch allocation of %lld bytes failed", (long long)want);
        scratch = nullptr;
        return nullptr;
    }
    scratch_bytes = want;
    return scratch;
}

extern "C" {

const char* fx_last_error(void) { return fx::g_err; }

int fx_init(int device, const fx_pool_config* cfg, fx_ctx** out) {
    FX_REQUIRE(out != nullptr, "fx_init: out is null");
    int count = 0;
    FX_HIP_CHECK(hipGetDeviceCount(&count));
    FX_REQUIRE(device >= 0 && device < count, "fx_init: device %d out of range (%d visible)", device, count);
    FX_HIP_CHECK(hipSetDevice(device));
    hipDeviceProp_t prop;
    FX_HIP_CHECK(hipGetDeviceProperties(&prop, device));
    if (strncmp(prop.gcnArchName, "gfx950", 6) != 0) {
        fx::set_error("fx_init: this library holds gfx950 code only; device %d is %s", device, prop.gcnArchName);
        return FX_ERR_UNSUPPORTED;
    }
    if (int rc = fx::static_scratch_init(device)) return rc;
    fx_ctx* c = new fx_ctx();
    c->device = device;
    c->name = prop.name[0] ? prop.name : prop.gcnArchName;
    c->num_cus = prop.multiProcessorCount;
    hipError_t e = hipStreamCreate(&c->stream);
    if (e == hipSuccess) e = hipEventCreate(&c->ev_start);
    if (e == hipSuccess) e = hipEventCreate(&c->ev_stop);
    if (e == hipSuccess) {
        c->pools[FX_F32] = fx::pool_create(cfg, 4, c->stream, &c->capturing);
        c->pools[FX_F64] = fx::pool_create(cfg, 8, c->stream, &c->capturing);
    }
    if (e != hipSuccess || !c->pools[0] || !c->pools[1]) {
        if (e != hipSuccess) fx::set_error("fx_init: %s", hipGetErrorString(e));  // else pool_create has set the message
        fx::pool_destroy(c->pools[0]);
        fx::pool_destroy(c->pools[1]);
        if (c->ev_start) (void)hipEventDestroy(c->ev_start);
        if (c->ev_stop) (void)hipEventDestroy(c->ev_stop);
        if (c->stream) (void)hipStreamDestroy(c->stream);
        delete c;
        return e != hipSuccess ? FX_ERR_HIP : FX_ERR_INVALID;
    }
    *out = c;
    return FX_OK;
}

int fx_destroy(fx_ctx* c) {
    FX_CHECK_CTX(c);
    (void)hipSetDevice(c->device);
    (void)hipStreamSynchronize(c->stream);
    fx::pool_destroy(c->pools[0]);
    fx::pool_destroy(c->pools[1]);
    if (c->scratch) (void)hipFree(c->scratch);
    for (void* p : c->parked_scratch) (void)hipFree(p);
    (void)hipEventDestroy(c->ev_start);
    (void)hipEventDestroy(c->ev_stop);
    for (hipEvent_t e : c->ev_tune)
        if (e) (void)hipEventDestroy(e);
    (void)hipStreamDestroy(c->stream);
    delete c;
    return FX_OK;
}

int fx_sync(fx_ctx* c) {
    FX_CHECK_CTX(c);
    FX_NOT_RECORDING(c, "fx_sync");
    FX_HIP_CHECK(hipStreamSynchronize(c->stream));
    return FX_OK;
}

int fx_device_name(fx_ctx* c, char* buf, int64_t len) {
    FX_CHECK_CTX(c);
    FX_REQUIRE(buf && len > 0, "fx_device_name: empty buffer");
    snprintf(buf, (size_t)len, "%s", c->name.c_str());
    return FX_OK;
}

void* fx_stream(fx_ctx* c) { return c ? (void*)c->stream : nullptr; }

int fx_timer_start(fx_ctx* c) {
    FX_CHECK_CTX(c);
    FX_NOT_RECORDING(c, "fx_timer_start");
    FX_HIP_CHECK(hipEventRecord(c->ev_start, c->stream));
    return FX_OK;
}

int fx_timer_stop(fx_ctx* c, float* ms) {
    FX_CHECK_CTX(c);
    FX_NOT_RECORDING(c, "fx_timer_stop");
    FX_REQUIRE(ms != nullptr, "fx_timer_stop: null output");
    FX_HIP_CHECK(hipEventRecord(c->ev_stop, c->stream));
    FX_HIP_CHECK(hipEventSynchronize(c->ev_stop));
    FX_HIP_CHECK(hipEventElapsedTime(ms, c->ev_start, c->ev_stop));
    return FX_OK;
}

int fx_h2d(fx_ctx* c, void* dst, const void* src, int64_t bytes) {
    FX_CHECK_CTX(c);
    FX_NOT_RECORDING(c, "fx_h2d");
    FX_REQUIRE(bytes >= 0 && (bytes == 0 || (dst && src)), "fx_h2d: bad arguments");
    if (bytes == 0) return FX_OK;
    FX_HIP_CHECK(hipMemcpyAsync(dst, src, (size_t)bytes, hipMemcpyHostToDevice, c->stream));
    FX_HIP_CHECK(hipStreamSynchronize(c->stream));
    return FX_OK;
}

int fx_d2h(fx_ctx* c, void* dst, const void* src, int64_t bytes) {
    FX_CHECK_CTX(c);
    FX_NOT_RECORDING(c, "fx_d2h");
    FX_REQUIRE(bytes >= 0 && (bytes == 0 || (dst && src)), "fx_d2h: bad arguments");
    if (bytes == 0) return FX_OK;
    FX_HIP_CHECK(hipMemcpyAsync(dst, src, (size_t)bytes, hipMemcpyDeviceToHost, c->stream));
    FX_HIP_CHECK(hipStreamSynchronize(c->stream));
    return FX_OK;
}

int fx_h2d_async(fx_ctx* c, void* dst, const void* src_pinned, int64_t bytes) {
    FX_CHECK_CTX(c);
    FX_REQUIRE(bytes >= 0 && (bytes == 0 || (dst && src_pinned)), "fx_h2d_async: bad arguments");
    if (bytes == 0) return FX_OK;
    FX_HIP_CHECK(hipMemcpyAsync(dst, src_pinned, (size_t)bytes, hipMemcpyHostToDevice, c->stream));
    return FX_OK;
}

int fx_host_alloc(fx_ctx* c, int64_t bytes, void** out) {
    FX_CHECK_CTX(c);
    FX_REQUIRE(out && bytes > 0, "fx_host_alloc: bad arguments");
    FX_HIP_CHECK(hipHostMalloc(out, (size_t)bytes, hipHostMallocDefault));
    return FX_OK;
}

int fx_host_free(fx_ctx* c, void* p) {
    FX_CHECK_CTX(c);
    FX_NOT_RECORDING(c, "fx_host_free");
    if (!p) return FX_OK;
    FX_HIP_CHECK(hipStreamSynchronize(c->stream));  // a queued copy may still read it
    FX_HIP_CHECK(hipHostFree(p));
    return FX_OK;
}

// ---- step graphs ---------------------------------------------------------------------------------------------------
struct fx_graph {
    hipGraph_t graph = nullptr;
    hipGraphExec_t exec = nullptr;
    std::vector<fx_ctx::Held> held;  // blocks released while recording: the graph's temporaries
    int64_t kernel_nodes = 0, nodes = 0;
};

int fx_graph_begin(fx_ctx* c) {
    FX_CHECK_CTX(c);
    FX_REQUIRE(!c->capturing, "fx_graph_begin: a graph is already being recorded on this context");
    // relaxed: a pool miss may still call hipMalloc while recording (it does not touch the stream)
    FX_HIP_CHECK(hipStreamBeginCapture(c->stream, hipStreamCaptureModeRelaxed));
    c->capturing = true;
    c->capture_held.clear();
    return FX_OK;
}

static int release_held(fx_ctx* c, std::vector<fx_ctx::Held>& held) {
    int rc = FX_OK;
    for (const auto& h : held) {
        const int r = fx_free(c, h.dtype, h.ptr, h.id);
        if (r != FX_OK) rc = r;
    }
    held.clear();
    return rc;
}

int fx_graph_end(fx_ctx* c, fx_graph** out) {
    FX_CHECK_CTX(c);
    FX_REQUIRE(c->capturing, "fx_graph_end: no graph is being recorded");
    c->capturing = false;
    hipGraph_t g = nullptr;
    const hipError_t e = hipStreamEndCapture(c->stream, &g);
    std::vector<fx_ctx::Held> held;
    held.swap(c->capture_held);
    if (e != hipSuccess || !g || !out) {
        (void)hipGetLastError();
        if (g) (void)hipGraphDestroy(g);
        release_held(c, held);  // nothing was queued, the blocks are free
        fx::set_error("fx_graph_end: recording failed (%s): a call between fx_graph_begin and fx_graph_end waited for the stream, "
                      "or the output pointer is null", e != hipSuccess ? hipGetErrorString(e) : "no graph");
        return e != hipSuccess ? FX_ERR_HIP : FX_ERR_INVALID;
    }
    fx_graph* fg = new fx_graph();
    fg->graph = g;
    fg->held.swap(held);
    size_t n = 0;
    if (hipGraphGetNodes(g, nullptr, &n) == hipSuccess && n > 0) {
        std::vector<hipGraphNode_t> nodes(n);
        if (hipGraphGetNodes(g, nodes.data(), &n) == hipSuccess) {
            fg->nodes = (int64_t)n;
            for (size_t i = 0; i < n; ++i) {
                hipGraphNodeType t;
                if (hipGraphNodeGetType(nodes[i], &t) == hipSuccess && t == hipGraphNodeTypeKernel) fg->kernel_nodes += 1;
            }
        }
    }
    const hipError_t ei = hipGraphInstantiate(&fg->exec, g, nullptr, nullptr, 0);
    if (ei != hipSuccess) {
        (void)hipGetLastError();
        (void)hipGraphDestroy(g);
        release_held(c, fg->held);
        delete fg;
        fx::set_error("fx_graph_end: hipGraphInstantiate failed: %s", hipGetErrorString(ei));
        return FX_ERR_HIP;
    }
    c->live_graphs += 1;
    *out = fg;
    return FX_OK;
}

int fx_graph_launch(fx_ctx* c, fx_graph* g) {
    FX_CHECK_CTX(c);
    FX_REQUIRE(g && g->exec, "fx_graph_launch: null graph");
    FX_REQUIRE(!c->capturing, "fx_graph_launch: a graph is being recorded on this context");
    FX_HIP_CHECK(hipGraphLaunch(g->exec, c->stream));
    return FX_OK;
}

int fx_scratch_info(fx_ctx* c, void** current, int64_t* bytes, int64_t* parked_regions, int64_t* live_graphs) {
    FX_REQUIRE(c != nullptr, "null context");
    if (current) *current = c->scratch;
    if (bytes) *bytes = c->scratch_bytes;
    if (parked_regions) *parked_regions = (int64_t)c->parked_scratch.size();
    if (live_graphs) *live_graphs = c->live_graphs;
    return FX_OK;
}

int fx_device_mem_info(fx_ctx* c, int64_t* free_bytes, int64_t* total_bytes) {
    FX_CHECK_CTX(c);
    size_t f = 0, t = 0;
    FX_HIP_CHECK(hipMemGetInfo(&f, &t));
    if (free_bytes) *free_bytes = (int64_t)f;
    if (total_bytes) *total_bytes = (int64_t)t;
    return FX_OK;
}

int fx_graph_info(fx_graph* g, int64_t* nodes, int64_t* kernel_nodes, int64_t* held_blocks) {
    if (!g) return FX_ERR_INVALID;
    if (nodes) *nodes = g->nodes;
    if (kernel_nodes) *kernel_nodes = g->kernel_nodes;
    if (held_blocks) *held_blocks = (int64_t)g->held.size();
    return FX_OK;
}

int fx_graph_destroy(fx_ctx* c, fx_graph* g) {
    FX_CHECK_CTX(c);
    FX_NOT_RECORDING(c, "fx_graph_destroy");
    if (!g) return FX_OK;
    FX_HIP_CHECK(hipStreamSynchronize(c->stream));  // a launch may still be running
    if (g->exec) (void)hipGraphExecDestroy(g->exec);
    if (g->graph) (void)hipGraphDestroy(g->graph);
    const int rc = release_held(c, g->held);
    delete g;
    if (--c->live_graphs <= 0) {  // the stream is idle (synchronised above): nothing uses the parked regions any more
        c->live_graphs = 0;
        for (void* p : c->parked_scratch) (void)hipFree(p);
        c->parked_scratch.clear();
    }
    return rc;
}

int fx_d2d(fx_ctx* c, void* dst, const void* src, int64_t bytes) {
    FX_CHECK_CTX(c);
    FX_REQUIRE(bytes >= 0 && (bytes == 0 || (dst && src)), "fx_d2d: bad arguments");
    if (bytes == 0) return FX_OK;
    // blocks up to 32 MiB go through the library's own streaming kernel (half the stream time of a runtime copy at these
    // sizes); larger ones and odd sizes / alignments through the runtime
    if (bytes <= (32ll << 20)) {
        const int rc = fx::copy_kernel(c, dst, src, bytes);
        if (rc != FX_ERR_UNSUPPORTED) return rc;
    }
    FX_HIP_CHECK(hipMemcpyAsync(dst, src, (size_t)bytes, hipMemcpyDeviceToDevice, c->stream));
    return FX_OK;
}

}  // extern "C"
