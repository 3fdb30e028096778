// Shared internals of libferrox_hip.so: context object, error reporting, launch helpers.
#pragma once
#include <hip/hip_runtime.h>
#include <array>
#include <cstdint>
#include <map>
#include <cstdio>
#include <mutex>
#include <string>
#include <vector>

#include "../../include/ferrox_hip.h"

typedef int64_t i64;

namespace fx {

struct Pool;  // allocator.hip

void set_error(const char* fmt, ...);
int bind_device(int device);  // runtime.hip

#define FX_HIP_CHECK(expr)                                                                                  \
    do {                                                                                                    \
        hipError_t _e = (expr);                                                                             \
        if (_e != hipSuccess) {                                                                             \
            fx::set_error("%s failed: %s (%s:%d)", #expr, hipGetErrorString(_e), __FILE__, __LINE__);       \
            return FX_ERR_HIP;                                                                              \
        }                                                                                                   \
    } while (0)

#define FX_REQUIRE(cond, ...)                                                                               \
    do {                                                                                                    \
        if (!(cond)) {                                                                                      \
            fx::set_error(__VA_ARGS__);                                                                     \
            return FX_ERR_INVALID;                                                                          \
        }                                                                                                   \
    } while (0)

// Every entry point starts here: a valid context, and its device current on the calling thread (the current device is
// per thread in HIP; a context created on one thread may be used from any other).
#define FX_CHECK_CTX(ctx)                                                                                   \
    do {                                                                                                    \
        FX_REQUIRE((ctx) != nullptr, "null context");                                                       \
        if (int _rc = fx::bind_device((ctx)->device)) return _rc;                                           \
    } while (0)

// Checks the launch itself (bad configuration shows up here, not at the next sync).
// Calls that wait for the stream refuse to run while it records a graph (the wait would invalidate the recording).
#define FX_NOT_RECORDING(c, what)                                                                           \
    FX_REQUIRE(!(c)->capturing, "%s waits for the stream, which is recording a graph (fx_graph_begin): call it before "  \
               "fx_graph_begin or after fx_graph_end", what)

#define FX_LAUNCH_CHECK()                                                                                   \
    do {                                                                                                    \
        hipError_t _e = hipGetLastError();                                                                  \
        if (_e != hipSuccess) {                                                                             \
            fx::set_error("kernel launch failed: %s (%s:%d)", hipGetErrorString(_e), __FILE__, __LINE__);   \
            return FX_ERR_HIP;                                                                              \
        }                                                                                                   \
    } while (0)

// Kernel launch, dynamic LDS and register-pinning statements go through these macros so that the same sources also build as
// plain host C++ (FX_HOST_EMULATION, with a stand-in for <hip/hip_runtime.h>): a test harness then runs every thread of every
// block of a launch on the CPU, with the tensors and the LDS between guard pages, and an access outside them faults there.
#ifndef FX_HOST_EMULATION
// FX_LAUNCH(grid, block, dynamic LDS bytes, stream, (arguments), kernel<template arguments>)
#define FX_LAUNCH(grid, block, smem, stream, args, ...) __VA_ARGS__<<<(grid), (block), (smem), (stream)>>> args
#define FX_DYNAMIC_SMEM(T, name) extern __shared__ __align__(16) T name[]
// empty asm statements that make the compiler re-form a value at this point (vector / scalar register) instead of keeping
// it alive, and that touch the accumulation registers
#define FX_PIN_VGPR(a) asm volatile("" : "+v"(a))
#define FX_PIN_VGPR2(a, b) asm volatile("" : "+v"(a), "+v"(b))
#define FX_PIN_SGPR(a) asm volatile("" : "+s"(a))
#define FX_TOUCH_AGPR(z) asm volatile("; accumulators in AGPRs %0" : "+a"(z))
#else
#define FX_LAUNCH(grid, block, smem, stream, args, ...) fxemu::launch((grid), (block), (size_t)(smem), [&] { __VA_ARGS__ args; })
#define FX_DYNAMIC_SMEM(T, name) T* name = reinterpret_cast<T*>(fxemu::dynamic_smem())
#define FX_PIN_VGPR(a) ((void)(a))
#define FX_PIN_VGPR2(a, b) ((void)(a), (void)(b))
#define FX_PIN_SGPR(a) ((void)(a))
#define FX_TOUCH_AGPR(z) ((void)(z))
#endif

inline i64 ceil_div(i64 a, i64 b) { return (a + b - 1) / b; }
inline bool aligned16(const void* p) { return (reinterpret_cast<uintptr_t>(p) & 15u) == 0; }

}  // namespace fx

struct fx_ctx {
    int device = 0;
    hipStream_t stream = nullptr;
    hipEvent_t ev_start = nullptr, ev_stop = nullptr;
    std::string name;
    int num_cus = 0;
    fx::Pool* pools[2] = {nullptr, nullptr};
    // library-owned scratch (split-K partials, reduction partials, permuted weights); grows on demand
    void* scratch = nullptr;
    i64 scratch_bytes = 0;
    // Recorded graphs keep the scratch address of their recording in their kernel arguments.  While any such graph is alive
    // (fx_graph_end .. fx_graph_destroy) a region that has to grow is parked here instead of freed, so a later launch of the
    // graph still finds its region; the parked regions are freed when the last graph is destroyed (or with the context).
    const char* last_conv_path = "";  // which kernel family the last convolution call took (fx_conv2d_last_path)
    int live_graphs = 0;
    std::vector<void*> parked_scratch;
    std::mutex launch_mutex;
    // tile shape that measured fastest per convolution layer shape (conv_patch.hpp); used under launch_mutex
    std::map<std::array<i64, 14>, int> conv_tile_cache;
    bool conv_retune = false;  // set by fx_conv2d_tune around its call: time the shapes again even when the cache has an entry
    // Between fx_graph_begin and fx_graph_end the stream records instead of running: blocks released meanwhile stay out of
    // the pool (the graph keeps using their addresses at every launch) and nothing may wait for the stream.
    bool capturing = false;
    struct Held { int dtype; void* ptr; uint64_t id; };
    std::vector<Held> capture_held;
    hipEvent_t ev_tune[2] = {nullptr, nullptr};
    // returns a scratch region of at least `bytes` (256-byte aligned); nullptr + error on failure
    void* get_scratch(i64 bytes);
};
