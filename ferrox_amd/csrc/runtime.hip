// Context, stream, copies, timing and error reporting of libferrox_hip.so.
// Replaces CudaContextManager (src/backend/cuda/context.rs:30-175) and the named-stream StreamManager
// (src/backend/cuda/stream_manager.rs:97-103): one compute stream, synchronous copies ordered on it.
#include <cstdarg>
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
Pool* pool_create(const fx_pool_config* cfg, int elem_size, hipStream_t stream);
int static_scratch_init(int device);  // reduce.hip
void pool_destroy(Pool* p);
}  // namespace fx

void* fx_ctx::get_scratch(i64 bytes) {
    if (bytes <= scratch_bytes) return scratch;
    // Work already queued on the stream may still use the old region.
    if (scratch) {
        if (hipStreamSynchronize(stream) != hipSuccess) return nullptr;
        (void)hipFree(scratch);
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
        c->pools[FX_F32] = fx::pool_create(cfg, 4, c->stream);
        c->pools[FX_F64] = fx::pool_create(cfg, 8, c->stream);
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
    FX_HIP_CHECK(hipEventRecord(c->ev_start, c->stream));
    return FX_OK;
}

int fx_timer_stop(fx_ctx* c, float* ms) {
    FX_CHECK_CTX(c);
    FX_REQUIRE(ms != nullptr, "fx_timer_stop: null output");
    FX_HIP_CHECK(hipEventRecord(c->ev_stop, c->stream));
    FX_HIP_CHECK(hipEventSynchronize(c->ev_stop));
    FX_HIP_CHECK(hipEventElapsedTime(ms, c->ev_start, c->ev_stop));
    return FX_OK;
}

int fx_h2d(fx_ctx* c, void* dst, const void* src, int64_t bytes) {
    FX_CHECK_CTX(c);
    FX_REQUIRE(bytes >= 0 && (bytes == 0 || (dst && src)), "fx_h2d: bad arguments");
    if (bytes == 0) return FX_OK;
    FX_HIP_CHECK(hipMemcpyAsync(dst, src, (size_t)bytes, hipMemcpyHostToDevice, c->stream));
    FX_HIP_CHECK(hipStreamSynchronize(c->stream));
    return FX_OK;
}

int fx_d2h(fx_ctx* c, void* dst, const void* src, int64_t bytes) {
    FX_CHECK_CTX(c);
    FX_REQUIRE(bytes >= 0 && (bytes == 0 || (dst && src)), "fx_d2h: bad arguments");
    if (bytes == 0) return FX_OK;
    FX_HIP_CHECK(hipMemcpyAsync(dst, src, (size_t)bytes, hipMemcpyDeviceToHost, c->stream));
    FX_HIP_CHECK(hipStreamSynchronize(c->stream));
    return FX_OK;
}

int fx_d2d(fx_ctx* c, void* dst, const void* src, int64_t bytes) {
    FX_CHECK_CTX(c);
    FX_REQUIRE(bytes >= 0 && (bytes == 0 || (dst && src)), "fx_d2d: bad arguments");
    if (bytes == 0) return FX_OK;
    FX_HIP_CHECK(hipMemcpyAsync(dst, src, (size_t)bytes, hipMemcpyDeviceToDevice, c->stream));
    return FX_OK;
}

}  // extern "C"
