// CPU walk of the matrix-product path: test infrastructure, the twin of walk.cpp for gemm.hip.  The library's own gemm.hip
// (dispatch, planners, the slab / thin / small / general-tile kernels and their ordered sums) is compiled as host C++ against
// the stand-in HIP header of this directory and every thread of every launch runs on the CPU; A, B, C, the bias, the column
// sums and the library scratch are buffers of exactly their size between inaccessible pages, so a load or store that leaves
// them faults here.  Each case runs twice: with the END of every buffer against a guard page, then with the START.
//
// usage: walk_gemm < cases    with one case per line:
//   <name> <f32|f64> M N K
// Every case runs all four transpose forms of fx_gemm and of fx_gemm_bias_act (bias + ReLU), and fx_gemm_tn_colsum and
// fx_linear_bwd on the same sizes.
#define FX_HOST_EMULATION 1
#include "../../ferrox_amd/csrc/gemm.hip"

#include <csignal>
#include <iostream>
#include <sstream>
#include <string>

// ---- what gemm.hip expects from the rest of the library (elementwise passes: their own files, not walked here) ---------------
namespace fx {
void set_error(const char* fmt, ...) {
    va_list ap;
    va_start(ap, fmt);
    vfprintf(stderr, fmt, ap);
    fputc('\n', stderr);
    va_end(ap);
}
int bind_device(int) { return FX_OK; }
}  // namespace fx
extern "C" int fx_bias_act_f32(fx_ctx*, float*, const float*, int64_t, int64_t, int64_t, int) { return FX_OK; }
extern "C" int fx_bias_act_f64(fx_ctx*, double*, const double*, int64_t, int64_t, int64_t, int) { return FX_OK; }
extern "C" int fx_bias_grad_f32(fx_ctx*, const float*, float*, int64_t, int64_t, int64_t) { return FX_OK; }
extern "C" int fx_bias_grad_f64(fx_ctx*, const double*, double*, int64_t, int64_t, int64_t) { return FX_OK; }
extern "C" int fx_relu_bwd_f32(fx_ctx*, const float*, const float*, float*, int64_t) { return FX_OK; }
extern "C" int fx_relu_bwd_f64(fx_ctx*, const double*, const double*, double*, int64_t) { return FX_OK; }

static fxemu::GuardedBuffer g_scratch;
void* fx_ctx::get_scratch(i64 bytes) {
    g_scratch.reset((size_t)bytes, fxemu::g_at_end);
    return g_scratch.ptr;
}

namespace {
const char* g_shrink = "";
struct Buf {
    fxemu::GuardedBuffer b;
    template <typename T> T* get(i64 elems, const char* name = "") {
        size_t bytes = (size_t)elems * sizeof(T);
        if (*name && strcmp(name, g_shrink) == 0 && bytes > 16) bytes -= 16;
        b.reset(bytes, fxemu::g_at_end);
        char* p = b.ptr;
        p -= (uintptr_t)p & 15;  // the 16-byte alignment every allocation of the library has
        return reinterpret_cast<T*>(p);
    }
};

std::string g_case;
void on_fault(int) {
    const char* a = "\nFAULT (signal) while walking: ";
    (void)!write(2, a, strlen(a));
    (void)!write(2, g_case.c_str(), g_case.size());
    (void)!write(2, "\n", 1);
    _exit(3);
}
int check(int rc, const char* what) {
    if (rc != FX_OK) {
        fprintf(stderr, "%s returned %d for %s\n", what, rc, g_case.c_str());
        exit(4);
    }
    return rc;
}

template <typename T> struct Entry;
template <> struct Entry<float> {
    static int gemm(fx_ctx* c, int ta, int tb, i64 M, i64 N, i64 K, const float* A, const float* B, float* C) { return fx_gemm_f32(c, ta, tb, M, N, K, A, B, C); }
    static int gemm_bias(fx_ctx* c, int ta, int tb, i64 M, i64 N, i64 K, const float* A, const float* B, const float* b, float* C) {
        return fx_gemm_bias_act_f32(c, ta, tb, M, N, K, A, B, b, C, 1);
    }
    static int tn_colsum(fx_ctx* c, i64 M, i64 N, i64 K, const float* A, const float* B, float* C, float* s) { return fx_gemm_tn_colsum_f32(c, M, N, K, A, B, C, s); }
};
template <> struct Entry<double> {
    static int gemm(fx_ctx* c, int ta, int tb, i64 M, i64 N, i64 K, const double* A, const double* B, double* C) { return fx_gemm_f64(c, ta, tb, M, N, K, A, B, C); }
    static int gemm_bias(fx_ctx* c, int ta, int tb, i64 M, i64 N, i64 K, const double* A, const double* B, const double* b, double* C) {
        return fx_gemm_bias_act_f64(c, ta, tb, M, N, K, A, B, b, C, 1);
    }
    static int tn_colsum(fx_ctx* c, i64 M, i64 N, i64 K, const double* A, const double* B, double* C, double* s) { return fx_gemm_tn_colsum_f64(c, M, N, K, A, B, C, s); }
};

template <typename T> void walk_case(fx_ctx* c, i64 M, i64 N, i64 K) {
    typedef Entry<T> E;
    Buf ba, bb, bc, bbias, bsum;
    T* A = ba.get<T>(M * K, "a");
    T* B = bb.get<T>(K * N, "b");
    T* C = bc.get<T>(M * N, "c");
    T* bias = bbias.get<T>(N);
    T* sums = bsum.get<T>(M);
    for (int ta = 0; ta < 2; ++ta)
        for (int tb = 0; tb < 2; ++tb) {
            check(E::gemm(c, ta, tb, M, N, K, A, B, C), "fx_gemm");
            check(E::gemm_bias(c, ta, tb, M, N, K, A, B, bias, C), "fx_gemm_bias_act");
        }
    check(E::tn_colsum(c, M, N, K, A, B, C, sums), "fx_gemm_tn_colsum");
}
}  // namespace

int main() {
    if (!getenv("FX_WALK_RAW_FAULT")) {
        signal(SIGSEGV, on_fault);
        signal(SIGBUS, on_fault);
    }
    if (const char* v = getenv("FX_WALK_SHRINK")) g_shrink = v;
    fx_ctx ctx;
    ctx.device = 0;
    ctx.num_cus = 256;
    std::string line;
    int ncases = 0;
    while (std::getline(std::cin, line)) {
        if (line.empty() || line[0] == '#') continue;
        std::istringstream ss(line);
        std::string name, dt;
        i64 M, N, K;
        ss >> name >> dt >> M >> N >> K;
        if (!ss) {
            fprintf(stderr, "bad case line: %s\n", line.c_str());
            return 2;
        }
        for (int pass = 0; pass < 2; ++pass) {
            fxemu::g_at_end = pass == 0;
            g_case = line + (pass == 0 ? "  [ends exact]" : "  [starts exact]");
            printf("walking %s\n", g_case.c_str());
            fflush(stdout);
            if (dt == "f64") walk_case<double>(&ctx, M, N, K);
            else walk_case<float>(&ctx, M, N, K);
        }
        ++ncases;
    }
    printf("walked %d cases, %llu launches, %llu threads: every access stayed inside its buffer\n", ncases, fxemu::g_launches, fxemu::g_threads_run);
    return 0;
}
