// CPU walk of the convolution path: test infrastructure.  The library's own conv.hip (dispatch, planners, every patch /
// image-layer / stride-2 / implicit-GEMM kernel it launches) is compiled here as host C++ against the stand-in HIP header of
// this directory; every launch then runs all its threads on the CPU (hip/hip_runtime.h: fxemu::launch).  Every tensor, the
// workspace / library scratch and the dynamic LDS of a block are buffers of exactly their size between inaccessible pages, so a
// load or store that leaves them faults here.  Each case is run twice: once with the END of every buffer against a guard
// page (over-reads fault), once with the START (under-reads fault).  The program prints the case before it runs it, so the
// last line of its output names the case that faulted.
//
// usage: walk < cases    with one case per line:
//   <name> <f32|f64> B Cin H W Cout kh kw sh sw ph pw
// FX_WALK_SHRINK=<x|w|y|g|dx|dw|act|ws|lds> makes that buffer 16 bytes shorter than the code is entitled to: the self-test of
// the detector (the walk must then fault).
#define FX_HOST_EMULATION 1
#include "../../ferrox_amd/csrc/conv.hip"

#include <csignal>
#include <iostream>
#include <sstream>
#include <string>

// ---- what conv.hip expects from the rest of the library ----------------------------------------------------------------------
namespace fx {
void set_error(const char* fmt, ...) {
    va_list ap;
    va_start(ap, fmt);
    vfprintf(stderr, fmt, ap);
    fputc('\n', stderr);
    va_end(ap);
}
int bind_device(int) { return FX_OK; }
int col2im_f32(fx_ctx*, const float*, float*, i64, i64, i64, i64, i64, i64, i64, i64, i64, i64, int) { abort(); }
int col2im_f64(fx_ctx*, const double*, double*, i64, i64, i64, i64, i64, i64, i64, i64, i64, i64, int) { abort(); }
}  // namespace fx
extern "C" int fx_gemm_f32(fx_ctx*, int, int, int64_t, int64_t, int64_t, const float*, const float*, float*) { abort(); }
extern "C" int fx_gemm_f64(fx_ctx*, int, int, int64_t, int64_t, int64_t, const double*, const double*, double*) { abort(); }

// the library's growing scratch region: here a fresh buffer of exactly the requested size per request
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
        // keep the 16-byte alignment every allocation of the library has: with the end exact, the start moves down to it
        char* p = b.ptr;
        p -= (uintptr_t)p & 15;
        return reinterpret_cast<T*>(p);
    }
};

std::string g_case;
void on_fault(int sig) {
    // async-signal-safe output of the case that was running
    const char* a = "\nFAULT (signal) while walking: ";
    (void)!write(2, a, strlen(a));
    (void)!write(2, g_case.c_str(), g_case.size());
    (void)!write(2, "\n", 1);
    _exit(3);
}

template <typename T> struct Entry;
template <> struct Entry<float> {
    static constexpr int DT = FX_F32;
    static int fwd(fx_ctx* c, const float* x, const float* w, float* y, const i64* d, void* ws, i64 wsb) {
        return fx_conv2d_fwd_f32(c, x, w, y, d[0], d[1], d[2], d[3], d[4], d[5], d[6], d[7], d[8], d[9], d[10], ws, wsb);
    }
    static int fwd_bias(fx_ctx* c, const float* x, const float* w, const float* b, float* y, const i64* d, int act) {
        return fx_conv2d_fwd_bias_act_f32(c, x, w, b, y, d[0], d[1], d[2], d[3], d[4], d[5], d[6], d[7], d[8], d[9], d[10], act, nullptr, 0);
    }
    static int dgrad(fx_ctx* c, const float* g, const float* w, float* dx, const i64* d, void* ws, i64 wsb) {
        return fx_conv2d_dgrad_f32(c, g, w, dx, d[0], d[1], d[2], d[3], d[4], d[5], d[6], d[7], d[8], d[9], d[10], 0, ws, wsb);
    }
    static int wgrad(fx_ctx* c, const float* x, const float* g, float* dw, const i64* d, void* ws, i64 wsb) {
        return fx_conv2d_wgrad_f32(c, x, g, dw, d[0], d[1], d[2], d[3], d[4], d[5], d[6], d[7], d[8], d[9], d[10], 0, ws, wsb);
    }
    static int wgrad_relu(fx_ctx* c, const float* x, const float* g, const float* a, float* dw, float* db, const i64* d) {
        return fx_conv2d_wgrad_relu_bias_f32(c, x, g, a, dw, db, d[0], d[1], d[2], d[3], d[4], d[5], d[6], d[7], d[8], d[9], d[10], nullptr, 0);
    }
    static int dgrad_relu(fx_ctx* c, const float* g, const float* a, const float* w, float* dx, const i64* d) {
        return fx_conv2d_dgrad_relu_f32(c, g, a, w, dx, d[0], d[1], d[2], d[3], d[4], d[5], d[6], d[7], d[8], d[9], d[10]);
    }
};
template <> struct Entry<double> {
    static constexpr int DT = FX_F64;
    static int fwd(fx_ctx* c, const double* x, const double* w, double* y, const i64* d, void* ws, i64 wsb) {
        return fx_conv2d_fwd_f64(c, x, w, y, d[0], d[1], d[2], d[3], d[4], d[5], d[6], d[7], d[8], d[9], d[10], ws, wsb);
    }
    static int fwd_bias(fx_ctx* c, const double* x, const double* w, const double* b, double* y, const i64* d, int act) {
        return fx_conv2d_fwd_bias_act_f64(c, x, w, b, y, d[0], d[1], d[2], d[3], d[4], d[5], d[6], d[7], d[8], d[9], d[10], act, nullptr, 0);
    }
    static int dgrad(fx_ctx* c, const double* g, const double* w, double* dx, const i64* d, void* ws, i64 wsb) {
        return fx_conv2d_dgrad_f64(c, g, w, dx, d[0], d[1], d[2], d[3], d[4], d[5], d[6], d[7], d[8], d[9], d[10], 0, ws, wsb);
    }
    static int wgrad(fx_ctx* c, const double* x, const double* g, double* dw, const i64* d, void* ws, i64 wsb) {
        return fx_conv2d_wgrad_f64(c, x, g, dw, d[0], d[1], d[2], d[3], d[4], d[5], d[6], d[7], d[8], d[9], d[10], 0, ws, wsb);
    }
    static int wgrad_relu(fx_ctx* c, const double* x, const double* g, const double* a, double* dw, double* db, const i64* d) {
        return fx_conv2d_wgrad_relu_bias_f64(c, x, g, a, dw, db, d[0], d[1], d[2], d[3], d[4], d[5], d[6], d[7], d[8], d[9], d[10], nullptr, 0);
    }
    static int dgrad_relu(fx_ctx* c, const double* g, const double* a, const double* w, double* dx, const i64* d) {
        return fx_conv2d_dgrad_relu_f64(c, g, a, w, dx, d[0], d[1], d[2], d[3], d[4], d[5], d[6], d[7], d[8], d[9], d[10]);
    }
};

int check(int rc, const char* what) {
    if (rc != FX_OK) {
        fprintf(stderr, "%s returned %d for %s\n", what, rc, g_case.c_str());
        exit(4);
    }
    return rc;
}

// every tile shape the forward / data-gradient tuner of the 3x3 f32 patch kernel may time and pick for this layer
void walk_patch_candidates(fx_ctx* c, const float* x, const float* w, float* y, const float* bias, const i64* d, i64 oh, i64 ow, bool dgrad) {
    const i64 B = d[0], Cin = d[1], H = d[2], W = d[3], Cout = d[4];
    cpk::Plan cand[cpk::MAX_CAND];
    int n;
    // the tuner only runs for layers the planner accepts (run() is reached through make_plan().ok)
    if (!dgrad) {
        if (!cpk::make_plan(c->num_cus, B, Cin, H, W, Cout, oh, ow, 3, 3, d[7], d[8], d[9], d[10]).ok) return;
        n = cpk::candidates(cand, c->num_cus, B, Cin, H, W, Cout, oh, ow, d[7], d[8], d[9], d[10]);
    } else {
        if (!cpk::make_plan(c->num_cus, B, Cout, oh, ow, Cin, H, W, 3, 3, 1, 1, 2 - d[9], 2 - d[10]).ok) return;
        n = cpk::candidates(cand, c->num_cus, B, Cout, oh, ow, Cin, H, W, 1, 1, 2 - d[9], 2 - d[10]);
    }
    for (int k = 0; k < n; ++k) {
        float* wimg = (float*)c->get_scratch(cpk::workspace_bytes(cand[k], dgrad ? Cin : Cout));
        if (!dgrad) check(cpk::launch_plan(c, cand[k], x, w, y, wimg, 0, Cout, Cin, B, Cin, H, W, Cout, oh, ow, d[7], d[8], d[9], d[10], bias, 1), "candidate fwd");
        else check(cpk::launch_plan(c, cand[k], x, w, y, wimg, 1, Cout, Cin, B, Cout, oh, ow, Cin, H, W, 1, 1, 2 - d[9], 2 - d[10], nullptr, 0), "candidate dgrad");
    }
}

template <typename T> void walk_case(fx_ctx* c, const i64* d) {
    typedef Entry<T> E;
    const i64 B = d[0], Cin = d[1], H = d[2], W = d[3], Cout = d[4], kh = d[5], kw = d[6], sh = d[7], sw = d[8], ph = d[9], pw = d[10];
    const i64 oh = (H + 2 * ph - kh) / sh + 1, ow = (W + 2 * pw - kw) / sw + 1;
    const i64 nx = B * Cin * H * W, ny = B * Cout * oh * ow, nw = Cout * Cin * kh * kw;
    Buf bx, bw, by, bg, bdx, bdw, bact, bbias, bdb, bws;
    T* x = bx.get<T>(nx, "x");
    T* w = bw.get<T>(nw, "w");
    T* y = by.get<T>(ny, "y");
    T* g = bg.get<T>(ny, "g");
    T* dx = bdx.get<T>(nx, "dx");
    T* dw = bdw.get<T>(nw, "dw");
    T* act = bact.get<T>(ny, "act");
    T* bias = bbias.get<T>(Cout);
    T* db = bdb.get<T>(Cout);
    // forward: library scratch, then a caller workspace of exactly the advertised size; bias + ReLU in the store
    check(E::fwd(c, x, w, y, d, nullptr, 0), "fwd");
    i64 need = fx_conv2d_workspace_bytes(FX_CONV_FWD, E::DT, 0, B, Cin, H, W, Cout, kh, kw, sh, sw, ph, pw);
    if (need > 0) check(E::fwd(c, x, w, y, d, bws.get<char>(need, "ws"), need), "fwd with workspace");
    check(E::fwd_bias(c, x, w, bias, y, d, 1), "fwd + bias + relu");
    check(E::dgrad(c, g, w, dx, d, nullptr, 0), "dgrad");
    need = fx_conv2d_workspace_bytes(FX_CONV_DGRAD, E::DT, 0, B, Cin, H, W, Cout, kh, kw, sh, sw, ph, pw);
    if (need > 0) check(E::dgrad(c, g, w, dx, d, bws.get<char>(need, "ws"), need), "dgrad with workspace");
    check(E::wgrad(c, x, g, dw, d, nullptr, 0), "wgrad");
    need = fx_conv2d_workspace_bytes(FX_CONV_WGRAD, E::DT, 0, B, Cin, H, W, Cout, kh, kw, sh, sw, ph, pw);
    if (need > 0) check(E::wgrad(c, x, g, dw, d, bws.get<char>(need, "ws"), need), "wgrad with workspace");
    if (fx_conv2d_bwd_relu_supported(c, FX_CONV_WGRAD, E::DT, B, Cin, H, W, Cout, kh, kw, sh, sw, ph, pw))
        check(E::wgrad_relu(c, x, g, act, dw, db, d), "wgrad from the unmasked gradient");
    if (fx_conv2d_bwd_relu_supported(c, FX_CONV_DGRAD, E::DT, B, Cin, H, W, Cout, kh, kw, sh, sw, ph, pw))
        check(E::dgrad_relu(c, g, act, w, dx, d), "dgrad from the unmasked gradient");
    if constexpr (sizeof(T) == 4) {
        if (kh == 3 && kw == 3) {
            walk_patch_candidates(c, x, w, y, bias, d, oh, ow, false);
            if (sh == 1 && sw == 1 && ph <= 2 && pw <= 2) walk_patch_candidates(c, g, w, dx, nullptr, d, oh, ow, true);
        }
    }
}
}  // namespace

int main() {
    if (!getenv("FX_WALK_RAW_FAULT")) {  // set it to let a sanitizer build print the faulting stack instead
        signal(SIGSEGV, on_fault);
        signal(SIGBUS, on_fault);
    }
    if (const char* v = getenv("FX_WALK_SHRINK")) g_shrink = v;
    fxemu::g_lds_shrink = strcmp(g_shrink, "lds") == 0 ? 16 : 0;
    setenv("FX_CONV_TUNE", "0", 1);  // the tuner's candidates are walked one by one above instead of timed
    fx_ctx ctx;
    ctx.device = 0;
    ctx.num_cus = 256;
    std::string line;
    int ncases = 0;
    while (std::getline(std::cin, line)) {
        if (line.empty() || line[0] == '#') continue;
        std::istringstream ss(line);
        std::string name, dt;
        i64 d[11];
        ss >> name >> dt;
        for (int i = 0; i < 11; ++i) ss >> d[i];
        if (!ss) {
            fprintf(stderr, "bad case line: %s\n", line.c_str());
            return 2;
        }
        for (int pass = 0; pass < 2; ++pass) {
            fxemu::g_at_end = pass == 0;
            g_case = line + (pass == 0 ? "  [ends exact]" : "  [starts exact]");
            printf("walking %s\n", g_case.c_str());
            fflush(stdout);
            if (dt == "f64") walk_case<double>(&ctx, d);
            else walk_case<float>(&ctx, d);
        }
        ++ncases;
    }
    printf("walked %d cases, %llu launches, %llu threads: every access stayed inside its buffer\n", ncases, fxemu::g_launches, fxemu::g_threads_run);
    return 0;
}
