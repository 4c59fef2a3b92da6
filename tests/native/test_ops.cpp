// Native parity test of the stand-alone operators of the C ABI (libmhc_hip.so) against the plain-C
// fp64 oracle, no Python.
//
// Counterparts in the reference: src/csrc/tests/test_sinkhorn_knopp.cu:86-381 (32 x 32 forward
// against sinkhorn_knopp_cpu_reference, batched 4 x 4 and 8 x 8), src/csrc/tests/test_rmsnorm.cu:32-110
// (N = 128, C = 4096, bf16) and src/csrc/tests/test_rmsnorm_backward.cu:41-140 (N = 16, C = 64).
// Same shapes and seeds of that kind; tolerances: 1e-5 (max |got - ref| / max |ref|) for fp32 results,
// 1e-2 for bf16 results (the reference uses 1e-5 .. 1e-4 and 1e-2 .. 2e-2).  The backward of the
// Sinkhorn operator is checked as well (the reference has no numeric test for it).
// Links oracle/mhc_oracle.c (test infrastructure).  Exit code 0 = all passed.
#include <hip/hip_runtime.h>

#include <chrono>
#include <cmath>
#include <cstdint>
#include <cstdio>
#include <cstdlib>
#include <cstring>
#include <random>
#include <vector>

#include "../../include/mhc_hip.h"

extern "C" {
int mhc_oracle_sinkhorn_plain_forward(const double *inp, double *out, int rows, int cols, int T, double eps);
int mhc_oracle_sinkhorn_plain_backward(const double *grad_out, const double *inp, double *d_inp, int rows, int cols,
                                       int T, double eps);
int mhc_oracle_rmsnorm_forward(const double *inp, const double *w, double *out, double *rms, int rows, int C, double eps);
int mhc_oracle_rmsnorm_backward(const double *grad, const double *inp, const double *w, const double *rms, double *d_inp,
                                double *d_w, int rows, int C);
}

#define HIP_OK(e) do { hipError_t _e = (e); if (_e != hipSuccess) { fprintf(stderr, "HIP error %s at line %d\n", hipGetErrorString(_e), __LINE__); exit(2); } } while (0)
#define MHC_OK_(e) do { int _s = (e); if (_s != MHC_OK) { fprintf(stderr, "mhc error %d (%s) at line %d\n", _s, mhc_status_string(_s), __LINE__); exit(2); } } while (0)

static uint16_t to_bf16(float f) { uint32_t u; memcpy(&u, &f, 4); u += 0x7fffu + ((u >> 16) & 1u); return (uint16_t)(u >> 16); }
static float from_bf16(uint16_t h) { uint32_t u = (uint32_t)h << 16; float f; memcpy(&f, &u, 4); return f; }

static int g_fail = 0;
static void report(const char *what, double maxerr, double maxref, double tol) {
    const double rel = maxerr / (maxref > 0 ? maxref : 1.0);
    const bool ok = std::isfinite(rel) && rel <= tol;
    printf("  %-46s rel err %.3e  (tol %.0e)  %s\n", what, rel, tol, ok ? "ok" : "FAILED");
    if (!ok) g_fail++;
}
template <typename T> static T *dev_copy(const std::vector<T> &h) {
    T *p; HIP_OK(hipMalloc(&p, h.size() * sizeof(T) + 16));
    HIP_OK(hipMemcpy(p, h.data(), h.size() * sizeof(T), hipMemcpyHostToDevice));
    return p;
}
static void compare_f32(const char *what, const float *dev, const std::vector<double> &ref, double tol) {
    std::vector<float> got(ref.size());
    HIP_OK(hipMemcpy(got.data(), dev, ref.size() * 4, hipMemcpyDeviceToHost));
    double e = 0, m = 0;
    for (size_t i = 0; i < ref.size(); i++) { e = std::fmax(e, std::fabs((double)got[i] - ref[i])); m = std::fmax(m, std::fabs(ref[i])); }
    report(what, e, m, tol);
}
static void compare_bf16(const char *what, const uint16_t *dev, const std::vector<double> &ref, double tol) {
    std::vector<uint16_t> got(ref.size());
    HIP_OK(hipMemcpy(got.data(), dev, ref.size() * 2, hipMemcpyDeviceToHost));
    double e = 0, m = 0;
    for (size_t i = 0; i < ref.size(); i++) { e = std::fmax(e, std::fabs((double)from_bf16(got[i]) - ref[i])); m = std::fmax(m, std::fabs(ref[i])); }
    report(what, e, m, tol);
}

// ---- Sinkhorn-Knopp ----------------------------------------------------------------------------
static void test_sinkhorn(int batch, int rows, int cols, int T, double eps, unsigned seed) {
    printf("sinkhorn_knopp: batch %d, %d x %d, %d iterations\n", batch, rows, cols, T);
    std::mt19937 g(seed);
    std::uniform_real_distribution<float> u(0.1f, 1.1f);   // positive entries, like the reference's test
    std::normal_distribution<float> nd(0.f, 1.f);
    const size_t sz = (size_t)rows * cols;
    std::vector<float> inp(batch * sz), go(batch * sz);
    for (auto &v : inp) v = u(g);
    for (auto &v : go) v = nd(g);
    std::vector<double> ref(batch * sz), dref(batch * sz);
    for (int b = 0; b < batch; b++) {
        std::vector<double> a(inp.begin() + b * sz, inp.begin() + (b + 1) * sz), gg(go.begin() + b * sz, go.begin() + (b + 1) * sz);
        mhc_oracle_sinkhorn_plain_forward(a.data(), ref.data() + b * sz, rows, cols, T, eps);
        mhc_oracle_sinkhorn_plain_backward(gg.data(), a.data(), dref.data() + b * sz, rows, cols, T, eps);
    }
    float *d_in = dev_copy(inp), *d_go = dev_copy(go), *d_out, *d_din;
    HIP_OK(hipMalloc(&d_out, batch * sz * 4)); HIP_OK(hipMalloc(&d_din, batch * sz * 4));
    MHC_OK_(mhc_sinkhorn_knopp_fwd(d_in, d_out, batch, rows, cols, T, (float)eps, nullptr));
    const size_t wsb = mhc_sinkhorn_knopp_bwd_workspace_bytes(batch, rows, cols, T);
    void *ws; HIP_OK(hipMalloc(&ws, wsb + 256));
    MHC_OK_(mhc_sinkhorn_knopp_bwd(d_go, d_in, d_din, batch, rows, cols, T, (float)eps, ws, wsb, nullptr));
    HIP_OK(hipDeviceSynchronize());
    compare_f32("forward", d_out, ref, 1e-5);
    compare_f32("backward (exact reverse sweep)", d_din, dref, 1e-5);
    if (rows == cols) {  // doubly stochastic after enough iterations (reference :58-84): column sums exact, rows close
        std::vector<float> out(batch * sz);
        HIP_OK(hipMemcpy(out.data(), d_out, batch * sz * 4, hipMemcpyDeviceToHost));
        double ce = 0, re = 0;
        for (int b = 0; b < batch; b++)
            for (int i = 0; i < rows; i++) {
                double cs = 0, rs = 0;
                for (int k = 0; k < rows; k++) { cs += out[b * sz + k * cols + i]; rs += out[b * sz + i * cols + k]; }
                ce = std::fmax(ce, std::fabs(cs - 1)); re = std::fmax(re, std::fabs(rs - 1));
            }
        report("column sums = 1", ce, 1.0, 1e-5);
        if (T >= 10) report("row sums -> 1", re, 1.0, 1e-3);
    }
    // timing, informational (the reference prints the same for its kernels)
    hipEvent_t e0, e1; HIP_OK(hipEventCreate(&e0)); HIP_OK(hipEventCreate(&e1));
    HIP_OK(hipEventRecord(e0));
    for (int i = 0; i < 20; i++) MHC_OK_(mhc_sinkhorn_knopp_fwd(d_in, d_out, batch, rows, cols, T, (float)eps, nullptr));
    HIP_OK(hipEventRecord(e1)); HIP_OK(hipEventSynchronize(e1));
    float ms; HIP_OK(hipEventElapsedTime(&ms, e0, e1));
    printf("  forward: %.2f us per call (20 back-to-back calls)\n", ms * 1e3 / 20);
    HIP_OK(hipFree(d_in)); HIP_OK(hipFree(d_go)); HIP_OK(hipFree(d_out)); HIP_OK(hipFree(d_din)); HIP_OK(hipFree(ws));
}

// ---- RMSNorm --------------------------------------------------------------------------------------
static void test_rmsnorm(int rows, int C, bool bf16, unsigned seed) {
    printf("rmsnorm: %d x %d, %s\n", rows, C, bf16 ? "bf16" : "fp32");
    std::mt19937 g(seed);
    std::uniform_real_distribution<float> u(-1.f, 1.f);
    std::normal_distribution<float> nd(0.f, 0.5f);
    const size_t sz = (size_t)rows * C;
    const double eps = 1e-5;
    std::vector<float> x(sz), w(C), go(sz);
    for (auto &v : x) v = u(g);
    for (auto &v : w) v = 1.0f + 0.25f * u(g);
    for (auto &v : go) v = nd(g);
    if (bf16) {
        for (auto &v : x) v = from_bf16(to_bf16(v));
        for (auto &v : w) v = from_bf16(to_bf16(v));
        for (auto &v : go) v = from_bf16(to_bf16(v));
    }
    std::vector<double> xd(x.begin(), x.end()), wd(w.begin(), w.end()), gd(go.begin(), go.end());
    std::vector<double> out(sz), rms(rows), dx(sz), dw(C);
    mhc_oracle_rmsnorm_forward(xd.data(), wd.data(), out.data(), rms.data(), rows, C, eps);
    mhc_oracle_rmsnorm_backward(gd.data(), xd.data(), wd.data(), rms.data(), dx.data(), dw.data(), rows, C);
    const int dt = bf16 ? MHC_BF16 : MHC_F32;
    const size_t es = bf16 ? 2 : 4;
    void *d_x, *d_w, *d_go, *d_out, *d_dx;
    float *d_rms, *d_dw;
    auto upload = [&](const std::vector<float> &h) {
        void *p; HIP_OK(hipMalloc(&p, h.size() * es + 16));
        if (bf16) { std::vector<uint16_t> t(h.size()); for (size_t i = 0; i < h.size(); i++) t[i] = to_bf16(h[i]);
                    HIP_OK(hipMemcpy(p, t.data(), t.size() * 2, hipMemcpyHostToDevice)); }
        else HIP_OK(hipMemcpy(p, h.data(), h.size() * 4, hipMemcpyHostToDevice));
        return p;
    };
    d_x = upload(x); d_w = upload(w); d_go = upload(go);
    HIP_OK(hipMalloc(&d_out, sz * es)); HIP_OK(hipMalloc(&d_dx, sz * es));
    HIP_OK(hipMalloc(&d_rms, rows * 4)); HIP_OK(hipMalloc(&d_dw, C * 4));
    MHC_OK_(mhc_rmsnorm_fwd(d_x, dt, d_w, dt, d_out, d_rms, rows, C, (float)eps, nullptr));
    const size_t wsb = mhc_rmsnorm_bwd_workspace_bytes(rows, C);
    void *ws; HIP_OK(hipMalloc(&ws, wsb + 256));
    MHC_OK_(mhc_rmsnorm_bwd(d_go, d_x, dt, d_w, dt, d_rms, d_dx, d_dw, rows, C, ws, wsb, nullptr));
    HIP_OK(hipDeviceSynchronize());
    const double tol = bf16 ? 1e-2 : 1e-5;
    if (bf16) { compare_bf16("forward", (const uint16_t *)d_out, out, tol); compare_bf16("d_inp", (const uint16_t *)d_dx, dx, tol); }
    else { compare_f32("forward", (const float *)d_out, out, tol); compare_f32("d_inp", (const float *)d_dx, dx, tol); }
    compare_f32("rms", d_rms, rms, 1e-5);
    compare_f32("d_weight (two-pass column sum, no atomics)", d_dw, dw, bf16 ? 1e-3 : 1e-5);
    HIP_OK(hipFree(d_x)); HIP_OK(hipFree(d_w)); HIP_OK(hipFree(d_go)); HIP_OK(hipFree(d_out)); HIP_OK(hipFree(d_dx));
    HIP_OK(hipFree(d_rms)); HIP_OK(hipFree(d_dw)); HIP_OK(hipFree(ws));
}

int main() {
    test_sinkhorn(1, 32, 32, 10, 1e-8, 42);     // reference test_sinkhorn_knopp.cu:86-140
    test_sinkhorn(64, 4, 4, 20, 1e-8, 43);      // batched n = 4 (:268-330)
    test_sinkhorn(320, 4, 4, 20, 1e-8, 44);
    test_sinkhorn(32, 8, 8, 20, 1e-8, 45);      // batched n = 8
    test_sinkhorn(3, 64, 64, 10, 1e-8, 46);     // 64 x 64 (:142-214: sums only there)
    test_sinkhorn(5, 3, 7, 6, 1e-8, 47);        // rows != cols
    test_sinkhorn(2, 128, 96, 4, 1e-8, 48);     // largest accepted row count
    test_rmsnorm(128, 4096, true, 42);           // reference test_rmsnorm.cu:32-110
    test_rmsnorm(128, 4096, false, 42);
    test_rmsnorm(16, 64, false, 42);             // reference test_rmsnorm_backward.cu:41-140
    test_rmsnorm(16, 64, true, 42);
    test_rmsnorm(7, 1000, false, 7);             // a row length that is not a multiple of 8
    if (g_fail) { printf("%d comparison(s) FAILED\n", g_fail); return 1; }
    printf("all comparisons passed\n");
    return 0;
}
