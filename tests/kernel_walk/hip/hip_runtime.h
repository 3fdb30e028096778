// Stand-in for <hip/hip_runtime.h> when the kernel sources are built as plain host C++ (FX_HOST_EMULATION): test
// infrastructure, never part of the library.  It gives the sources what they use of HIP -- qualifiers, vector types, index
// variables, the few runtime calls, the wave and MFMA builtins -- in a form that lets a CPU thread run the code of ONE GPU
// thread from start to end:
//   * __syncthreads and the scheduling builtins do nothing; shuffles return the caller's own value; an MFMA only folds its two
//     operands into the accumulator, so that every LDS read that feeds it stays live.  The values computed are therefore
//     meaningless -- what is exercised is every address the thread forms: none of the kernels' addresses depends on loaded data.
//   * fxemu::launch runs all threads of all blocks of a launch one after the other; the dynamic LDS of a block is a buffer of
//     exactly the launch's size between inaccessible pages (fxemu::GuardedBuffer), as the harness makes every tensor.
// An access outside a tensor, the workspace or the dynamic LDS therefore faults in the harness instead of on a GPU.
#pragma once
#ifndef FX_HOST_EMULATION
#error "this header only stands in for the HIP runtime in the host-emulation build of the kernel sources"
#endif
#include <sys/mman.h>
#include <unistd.h>

#include <algorithm>
#include <cmath>
#include <cstdarg>
#include <cstddef>
#include <cstdint>
#include <cstdio>
#include <cstdlib>
#include <cstring>

#define __global__ inline
#define __device__
#define __host__
#define __forceinline__ inline __attribute__((always_inline))
#define __launch_bounds__(...)
#define __shared__ static
#define __align__(n) __attribute__((aligned(n)))

struct dim3 {
    unsigned x, y, z;
    constexpr dim3(unsigned x_ = 1, unsigned y_ = 1, unsigned z_ = 1) : x(x_), y(y_), z(z_) {}
};
inline dim3 threadIdx, blockIdx, blockDim, gridDim;

// The GPU's 8- and 16-byte global accesses only need the alignment of their elements (rows of W % 4 != 0 floats are read with
// 16-byte loads that start at any float), so the vector types carry element alignment here and the host never emits an
// aligned vector move for them; the same for the ext_vector_type typedefs of the sources.
struct float2 { float x, y; };
struct float4 { float x, y, z, w; };
struct double2 { double x, y; };
#define ext_vector_type(n) ext_vector_type(n), aligned(4)
inline float2 make_float2(float x, float y) { return float2{x, y}; }
inline float4 make_float4(float x, float y, float z, float w) { return float4{x, y, z, w}; }
inline double2 make_double2(double x, double y) { return double2{x, y}; }

// ---- the runtime calls the sources make -----------------------------------------------------------------------------------
typedef int hipError_t;
constexpr hipError_t hipSuccess = 0, hipErrorOutOfMemory = 2;
typedef void* hipStream_t;
typedef void* hipEvent_t;
typedef int hipFuncAttribute;
constexpr hipFuncAttribute hipFuncAttributeMaxDynamicSharedMemorySize = 8;
inline const char* hipGetErrorString(hipError_t) { return "host emulation"; }
inline hipError_t hipGetLastError() { return hipSuccess; }
inline hipError_t hipFuncSetAttribute(const void*, hipFuncAttribute, int) { return hipSuccess; }
inline hipError_t hipEventCreate(hipEvent_t* e) { *e = (void*)1; return hipSuccess; }
inline hipError_t hipEventRecord(hipEvent_t, hipStream_t) { return hipSuccess; }
inline hipError_t hipEventSynchronize(hipEvent_t) { return hipSuccess; }
inline hipError_t hipEventElapsedTime(float* ms, hipEvent_t, hipEvent_t) { *ms = 1.f; return hipSuccess; }
inline hipError_t hipStreamSynchronize(hipStream_t) { return hipSuccess; }
inline hipError_t hipMalloc(void** p, size_t n) { *p = calloc(1, n); return *p ? hipSuccess : 2; }
inline hipError_t hipFree(void* p) { free(p); return hipSuccess; }
inline hipError_t hipMemsetAsync(void* p, int v, size_t n, hipStream_t) { memset(p, v, n); return hipSuccess; }

// ---- device-side builtins ---------------------------------------------------------------------------------------------------
inline void __syncthreads() {}
#define __builtin_amdgcn_sched_barrier(x) ((void)0)
#define __builtin_amdgcn_wave_barrier() ((void)0)
#define __builtin_amdgcn_s_setprio(x) ((void)0)
#define __builtin_amdgcn_s_waitcnt(x) ((void)0)
#define __builtin_amdgcn_readfirstlane(x) (x)
template <typename T> inline T __shfl_xor(T v, int, int = 64) { return v; }
template <typename T> inline T __shfl_down(T v, int, int = 64) { return v; }
template <typename T> inline T __shfl_up(T v, int, int = 64) { return v; }
template <typename T> inline T __shfl(T v, int, int = 64) { return v; }
inline uint32_t __umulhi(uint32_t a, uint32_t b) { return (uint32_t)(((uint64_t)a * b) >> 32); }
template <typename V> inline V fxemu_mfma(double a, double b, V c) { c[0] += (decltype(c[0] + 0))(a * b); return c; }
#define __builtin_amdgcn_mfma_f32_32x32x2f32(a, b, c, x, y, z) fxemu_mfma((a), (b), (c))
#define __builtin_amdgcn_mfma_f32_16x16x4f32(a, b, c, x, y, z) fxemu_mfma((a), (b), (c))
#define __builtin_amdgcn_mfma_f64_16x16x4f64(a, b, c, x, y, z) fxemu_mfma((a), (b), (c))
using std::max;
using std::min;
inline long long min(long long a, int b) { return a < b ? a : b; }
inline long long min(int a, long long b) { return a < b ? a : b; }
inline long long max(long long a, int b) { return a > b ? a : b; }
inline long long max(int a, long long b) { return a > b ? a : b; }

// ---- running a launch on the CPU ----------------------------------------------------------------------------------------------
namespace fxemu {
// `bytes` accessible bytes between two inaccessible regions.  at_end: the buffer ends where the upper region begins (an access
// past the end faults at once; one before the start has up to a page of slack), else it starts where the lower region ends.
struct GuardedBuffer {
    static constexpr size_t GUARD = size_t(64) << 20;
    char* map = nullptr;
    size_t map_bytes = 0;
    char* ptr = nullptr;
    GuardedBuffer() = default;
    GuardedBuffer(const GuardedBuffer&) = delete;
    GuardedBuffer& operator=(const GuardedBuffer&) = delete;
    void reset(size_t bytes, bool at_end) {
        release();
        const size_t page = (size_t)sysconf(_SC_PAGESIZE);
        const size_t body = (std::max<size_t>(bytes, 1) + page - 1) / page * page;
        map_bytes = 2 * GUARD + body;
        map = (char*)mmap(nullptr, map_bytes, PROT_NONE, MAP_PRIVATE | MAP_ANONYMOUS | MAP_NORESERVE, -1, 0);
        if (map == MAP_FAILED) { perror("mmap"); abort(); }
        if (mprotect(map + GUARD, body, PROT_READ | PROT_WRITE) != 0) { perror("mprotect"); abort(); }
        ptr = at_end ? map + GUARD + body - bytes : map + GUARD;
        // 16-byte vector accesses need the alignment the allocator of the library gives (256 bytes): sizes are padded by
        // the callers to a multiple of 16 where the end is what is checked
    }
    void release() {
        if (map) munmap(map, map_bytes);
        map = ptr = nullptr;
    }
    ~GuardedBuffer() { release(); }
};

inline GuardedBuffer g_smem;
inline bool g_at_end = true;  // which edge of every buffer is exact in this pass
inline void* dynamic_smem() { return g_smem.ptr; }
inline unsigned long long g_threads_run = 0, g_launches = 0;
inline size_t g_lds_shrink = 0;  // the detector's self-test: bytes taken off every dynamic LDS request larger than that
inline const char* g_what = "";

template <class F> inline void launch(dim3 grid, dim3 block, size_t smem_bytes, F&& body) {
    g_smem.reset(smem_bytes > 4 * g_lds_shrink ? smem_bytes - g_lds_shrink : smem_bytes, g_at_end);
    gridDim = grid;
    blockDim = block;
    ++g_launches;
    for (unsigned bz = 0; bz < grid.z; ++bz)
        for (unsigned by = 0; by < grid.y; ++by)
            for (unsigned bx = 0; bx < grid.x; ++bx) {
                blockIdx = dim3(bx, by, bz);
                for (unsigned tz = 0; tz < block.z; ++tz)
                    for (unsigned ty = 0; ty < block.y; ++ty)
                        for (unsigned tx = 0; tx < block.x; ++tx) {
                            threadIdx = dim3(tx, ty, tz);
                            body();
                            ++g_threads_run;
                        }
            }
}
}  // namespace fxemu
