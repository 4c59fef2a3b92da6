// Native parity test: the C ABI (libmhc_hip.so) against the plain-C fp64 oracle, no Python.
//
// Counterpart of the reference's native layer test (src/csrc/tests/test_mhc_layer.cu:155-327):
// seeded inputs, CPU reference, element-wise comparison - here at the fp32 tier's 1e-5
// (max |got - ref| / max |ref|) for y and every gradient, dynamic and static H, and at the bf16
// tier's 2e-2 (1e-4 for the float32 results) on bf16-rounded inputs (activations, w and phi stored as bfloat16: the matrix-core
// kernels, every backward path: two-launch, tiled, wide).
// Links oracle/mhc_oracle.c (test infrastructure) and libmhc_hip.so.  Exit code 0 = all passed.
#include <hip/hip_runtime.h>

#include <cmath>
#include <cstdio>
#include <cstdint>
#include <cstdlib>
#include <cstring>
#include <random>
#include <vector>

#include "../../include/mhc_hip.h"

extern "C" {
int mhc_oracle_dynamic_forward(const double *x, const double *w, const double *phi, const double *bias,
                               const double *alpha, const double *f_inject, int B, int n, int C, int T, double eps,
                               double *y, double *Hpre_out, double *Hpost_out, double *M_out);
int mhc_oracle_dynamic_backward(const double *x, const double *dy, const double *w, const double *phi,
                                const double *bias, const double *alpha, const double *f_inject, int B, int n, int C,
                                int T, double eps, double *dx, double *df, double *dw, double *dphi, double *dbias,
                                double *dalpha);
int mhc_oracle_static_forward(const double *x, const double *w, const double *logits, const double *f_inject, int B,
                              int n, int C, int T, double eps, double *y, double *Hpre_out, double *Hpost_out,
                              double *M_out);
int mhc_oracle_static_backward(const double *x, const double *dy, const double *w, const double *logits,
                               const double *f_inject, int B, int n, int C, int T, double eps, double *dx, double *df,
                               double *dw, double *dlogits);
}

#define HIP_OK(e) do { hipError_t _e = (e); if (_e != hipSuccess) { fprintf(stderr, "HIP error %s at line %d\n", hipGetErrorString(_e), __LINE__); exit(2); } } while (0)
#define MHC_OK_(e) do { int _s = (e); if (_s != MHC_OK) { fprintf(stderr, "mhc error %d (%s) at line %d\n", _s, mhc_status_string(_s), __LINE__); exit(2); } } while (0)

static std::vector<double> randn(size_t n, double scale, std::mt19937 &g) {
    std::normal_distribution<double> d(0.0, 1.0);
    std::vector<double> v(n);
    for (auto &x : v) x = (double)(float)(scale * d(g));  // exactly representable in fp32
    return v;
}
static float *to_dev(const std::vector<double> &h) {
    std::vector<float> f(h.begin(), h.end());
    float *p;
    HIP_OK(hipMalloc(&p, f.size() * 4 + 16));
    HIP_OK(hipMemcpy(p, f.data(), f.size() * 4, hipMemcpyHostToDevice));
    return p;
}
static float *dev_alloc(size_t n) { float *p; HIP_OK(hipMalloc(&p, n * 4 + 16)); return p; }
static int g_fail = 0;
static void report(const char *what, const std::vector<float> &got, const std::vector<double> &ref, double tol) {
    double maxerr = 0, maxref = 0;
    for (size_t i = 0; i < ref.size(); i++) {
        maxerr = std::fmax(maxerr, std::fabs((double)got[i] - ref[i]));
        maxref = std::fmax(maxref, std::fabs(ref[i]));
    }
    const double rel = maxerr / (maxref > 0 ? maxref : 1.0);
    const bool ok = rel <= tol && std::isfinite(rel);
    printf("    %-8s rel err %.2e %s\n", what, rel, ok ? "ok" : "FAIL");
    if (!ok) g_fail++;
}
static void compare(const char *what, const float *dev, const std::vector<double> &ref, double tol = 1e-5) {
    std::vector<float> got(ref.size());
    HIP_OK(hipMemcpy(got.data(), dev, ref.size() * 4, hipMemcpyDeviceToHost));
    report(what, got, ref, tol);
}

// bfloat16 storage: round to nearest even on the host, so that the oracle sees exactly the stored values
static uint16_t bf16_bits(float f) {
    uint32_t u;
    memcpy(&u, &f, 4);
    u += 0x7fffu + ((u >> 16) & 1u);
    return (uint16_t)(u >> 16);
}
static float bf16_value(uint16_t h) {
    const uint32_t u = (uint32_t)h << 16;
    float f;
    memcpy(&f, &u, 4);
    return f;
}
static void round_to_bf16(std::vector<double> &v) {
    for (auto &x : v) x = (double)bf16_value(bf16_bits((float)x));
}
static uint16_t *to_dev_bf16(const std::vector<double> &h) {
    std::vector<uint16_t> b(h.size());
    for (size_t i = 0; i < h.size(); i++) b[i] = bf16_bits((float)h[i]);
    uint16_t *p;
    HIP_OK(hipMalloc(&p, b.size() * 2 + 16));
    HIP_OK(hipMemcpy(p, b.data(), b.size() * 2, hipMemcpyHostToDevice));
    return p;
}
static uint16_t *dev_alloc_bf16(size_t n) { uint16_t *p; HIP_OK(hipMalloc(&p, n * 2 + 16)); return p; }
static void compare_bf16(const char *what, const uint16_t *dev, const std::vector<double> &ref, double tol) {
    std::vector<uint16_t> raw(ref.size());
    HIP_OK(hipMemcpy(raw.data(), dev, ref.size() * 2, hipMemcpyDeviceToHost));
    std::vector<float> got(ref.size());
    for (size_t i = 0; i < ref.size(); i++) got[i] = bf16_value(raw[i]);
    report(what, got, ref, tol);
}

static void test_dynamic(int B, int n, int C, int T) {
    printf("dynamic H  B=%d n=%d C=%d T=%d\n", B, n, C, T);
    const int nC = n * C, D = n * n + 2 * n;
    const double eps = 1e-6;
    std::mt19937 g(1234 + B + 7 * n + 13 * C);
    auto x = randn((size_t)B * nC, 1.0, g), dy = randn((size_t)B * nC, 1.0, g), w = randn(C, 0.3, g);
    for (auto &v : w) v = (double)(float)(v + 1.0);
    auto phi = randn((size_t)D * nC, 0.05, g), bias = randn(D, 0.3, g);
    std::vector<double> alpha = {(double)0.7f, (double)-0.4f, (double)0.9f};
    std::vector<double> y((size_t)B * nC), Hp(B * n), Ho(B * n), M((size_t)B * n * n), dx((size_t)B * nC), dw(C),
        dphi((size_t)D * nC), dbias(D), dalpha(3);
    if (mhc_oracle_dynamic_forward(x.data(), w.data(), phi.data(), bias.data(), alpha.data(), nullptr, B, n, C, T, eps,
                                   y.data(), Hp.data(), Ho.data(), M.data()) ||
        mhc_oracle_dynamic_backward(x.data(), dy.data(), w.data(), phi.data(), bias.data(), alpha.data(), nullptr, B, n,
                                    C, T, eps, dx.data(), nullptr, dw.data(), dphi.data(), dbias.data(), dalpha.data())) {
        printf("    oracle refused the shape\n"); g_fail++; return;
    }
    float *dx_ = to_dev(x), *ddy = to_dev(dy), *dw_ = to_dev(w), *dphi_ = to_dev(phi), *dbias_ = to_dev(bias),
          *dalpha_ = to_dev(alpha);
    float *y_ = dev_alloc((size_t)B * nC), *Hp_ = dev_alloc(B * n), *Ho_ = dev_alloc(B * n), *M_ = dev_alloc((size_t)B * n * n),
          *P_ = dev_alloc((size_t)B * D), *r_ = dev_alloc(B), *q_ = dev_alloc(B), *gx = dev_alloc((size_t)B * nC),
          *gw = dev_alloc(C), *gphi = dev_alloc((size_t)D * nC), *gb = dev_alloc(D), *ga = dev_alloc(3);
    float *sk_ = dev_alloc(std::max<size_t>(mhc_layer_sinkhorn_state_floats(B, n, T), 1));
    const size_t wsb = mhc_layer_dynamic_workspace_bytes(B, n, C);
    void *ws; HIP_OK(hipMalloc(&ws, wsb + 256));
    MHC_OK_(mhc_layer_fwd_dynamic(dx_, MHC_F32, dw_, MHC_F32, dphi_, MHC_F32, dbias_, dalpha_, nullptr, y_, MHC_F32, Hp_,
                                  Ho_, M_, P_, r_, q_, sk_, B, n, C, T, (float)eps, ws, wsb, nullptr));
    HIP_OK(hipDeviceSynchronize());
    compare("y", y_, y); compare("H_pre", Hp_, Hp); compare("H_post", Ho_, Ho); compare("M", M_, M);
    // the backward once from the saved Sinkhorn denominators, once recomputing the iterations
    for (const float *state : {(const float *)sk_, (const float *)nullptr}) {
        printf("    backward %s\n", state ? "from the saved Sinkhorn state" : "recomputing the Sinkhorn iterations");
        MHC_OK_(mhc_layer_bwd_dynamic(ddy, MHC_F32, dx_, MHC_F32, dw_, MHC_F32, dphi_, MHC_F32, dbias_, dalpha_, nullptr,
                                      Hp_, Ho_, M_, P_, r_, q_, state, gx, nullptr, gw, gphi, gb, ga, B, n, C, T,
                                      (float)eps, ws, wsb, nullptr));
        HIP_OK(hipDeviceSynchronize());
        compare("dx", gx, dx); compare("dw", gw, dw); compare("dphi", gphi, dphi); compare("dbias", gb, dbias);
        compare("dalpha", ga, dalpha);
    }
    for (float *p : {dx_, ddy, dw_, dphi_, dbias_, dalpha_, y_, Hp_, Ho_, M_, P_, r_, q_, sk_, gx, gw, gphi, gb, ga}) (void)hipFree(p);
    (void)hipFree(ws);
}

static void test_static(int B, int n, int C, int T) {
    printf("static H   B=%d n=%d C=%d T=%d\n", B, n, C, T);
    const int nC = n * C, D = n * n + 2 * n;
    const double eps = 1e-6;
    std::mt19937 g(4321 + B + 7 * n + 13 * C);
    auto x = randn((size_t)B * nC, 1.0, g), dy = randn((size_t)B * nC, 1.0, g), w = randn(C, 0.3, g), lg = randn(D, 1.0, g);
    for (auto &v : w) v = (double)(float)(v + 1.0);
    std::vector<double> y((size_t)B * nC), Hp(n), Ho(n), M(n * n), dx((size_t)B * nC), dw(C), dl(D);
    if (mhc_oracle_static_forward(x.data(), w.data(), lg.data(), nullptr, B, n, C, T, eps, y.data(), Hp.data(), Ho.data(), M.data()) ||
        mhc_oracle_static_backward(x.data(), dy.data(), w.data(), lg.data(), nullptr, B, n, C, T, eps, dx.data(), nullptr,
                                   dw.data(), dl.data())) {
        printf("    oracle refused the shape\n"); g_fail++; return;
    }
    float *x_ = to_dev(x), *dy_ = to_dev(dy), *w_ = to_dev(w), *lg_ = to_dev(lg);
    float *y_ = dev_alloc((size_t)B * nC), *Hp_ = dev_alloc(n), *Ho_ = dev_alloc(n), *M_ = dev_alloc(n * n), *q_ = dev_alloc(B),
          *gx = dev_alloc((size_t)B * nC), *gw = dev_alloc(C), *gl = dev_alloc(D);
    const size_t wsb = mhc_layer_static_workspace_bytes(B, n, C);
    void *ws; HIP_OK(hipMalloc(&ws, wsb + 256));
    MHC_OK_(mhc_layer_fwd(x_, MHC_F32, w_, MHC_F32, lg_, lg_ + n, lg_ + 2 * n, nullptr, y_, MHC_F32, Hp_, Ho_, M_, q_, B, n, C,
                          T, (float)eps, ws, wsb, nullptr));
    MHC_OK_(mhc_layer_bwd(dy_, MHC_F32, x_, MHC_F32, w_, MHC_F32, lg_, lg_ + n, lg_ + 2 * n, nullptr, Hp_, Ho_, M_, q_, gx,
                          nullptr, gw, gl, gl + n, gl + 2 * n, B, n, C, T, (float)eps, ws, wsb, nullptr));
    HIP_OK(hipDeviceSynchronize());
    compare("y", y_, y); compare("H_pre", Hp_, Hp); compare("H_post", Ho_, Ho); compare("M", M_, M);
    compare("dx", gx, dx); compare("dw", gw, dw); compare("dlogits", gl, dl);
    for (float *p : {x_, dy_, w_, lg_, y_, Hp_, Ho_, M_, q_, gx, gw, gl}) (void)hipFree(p);
    (void)hipFree(ws);
}

// bf16 tier: activations, w and phi stored as bfloat16 (fp32 accumulation inside), outputs y and dx bfloat16,
// parameter gradients float32; the oracle runs in fp64 on the rounded values.
static void test_dynamic_bf16(int B, int n, int C, int T) {
    printf("dynamic H, bf16 storage  B=%d n=%d C=%d T=%d\n", B, n, C, T);
    const int nC = n * C, D = n * n + 2 * n;
    // y and dx are rounded to bfloat16 on their way out (half an ulp is 4e-3 of the value); the float32
    // results are sums of exact products of the rounded inputs and stay close to the fp64 oracle
    const double eps = 1e-6, tol = 2e-2, tol32 = 1e-4;
    std::mt19937 g(99 + B + 7 * n + 13 * C);
    auto x = randn((size_t)B * nC, 1.0, g), dy = randn((size_t)B * nC, 1.0, g), w = randn(C, 0.3, g);
    for (auto &v : w) v += 1.0;
    auto phi = randn((size_t)D * nC, 0.05, g), bias = randn(D, 0.3, g);
    round_to_bf16(x); round_to_bf16(dy); round_to_bf16(w); round_to_bf16(phi);
    std::vector<double> alpha = {(double)0.7f, (double)-0.4f, (double)0.9f};
    std::vector<double> y((size_t)B * nC), Hp(B * n), Ho(B * n), M((size_t)B * n * n), dx((size_t)B * nC), dw(C),
        dphi((size_t)D * nC), dbias(D), dalpha(3);
    if (mhc_oracle_dynamic_forward(x.data(), w.data(), phi.data(), bias.data(), alpha.data(), nullptr, B, n, C, T, eps,
                                   y.data(), Hp.data(), Ho.data(), M.data()) ||
        mhc_oracle_dynamic_backward(x.data(), dy.data(), w.data(), phi.data(), bias.data(), alpha.data(), nullptr, B, n,
                                    C, T, eps, dx.data(), nullptr, dw.data(), dphi.data(), dbias.data(), dalpha.data())) {
        printf("    oracle refused the shape\n"); g_fail++; return;
    }
    uint16_t *x_ = to_dev_bf16(x), *dy_ = to_dev_bf16(dy), *w_ = to_dev_bf16(w), *phi_ = to_dev_bf16(phi);
    float *bias_ = to_dev(bias), *alpha_ = to_dev(alpha);
    uint16_t *y_ = dev_alloc_bf16((size_t)B * nC), *gx = dev_alloc_bf16((size_t)B * nC);
    float *Hp_ = dev_alloc(B * n), *Ho_ = dev_alloc(B * n), *M_ = dev_alloc((size_t)B * n * n), *P_ = dev_alloc((size_t)B * D),
          *r_ = dev_alloc(B), *q_ = dev_alloc(B), *gw = dev_alloc(C), *gphi = dev_alloc((size_t)D * nC), *gb = dev_alloc(D),
          *ga = dev_alloc(3);
    float *sk_ = dev_alloc(std::max<size_t>(mhc_layer_sinkhorn_state_floats(B, n, T), 1));
    const size_t wsb = mhc_layer_dynamic_workspace_bytes(B, n, C);
    void *ws; HIP_OK(hipMalloc(&ws, wsb + 256));
    MHC_OK_(mhc_layer_fwd_dynamic(x_, MHC_BF16, w_, MHC_BF16, phi_, MHC_BF16, bias_, alpha_, nullptr, y_, MHC_BF16, Hp_, Ho_,
                                  M_, P_, r_, q_, sk_, B, n, C, T, (float)eps, ws, wsb, nullptr));
    MHC_OK_(mhc_layer_bwd_dynamic(dy_, MHC_BF16, x_, MHC_BF16, w_, MHC_BF16, phi_, MHC_BF16, bias_, alpha_, nullptr, Hp_,
                                  Ho_, M_, P_, r_, q_, sk_, gx, nullptr, gw, gphi, gb, ga, B, n, C, T, (float)eps, ws, wsb,
                                  nullptr));
    HIP_OK(hipDeviceSynchronize());
    compare_bf16("y", y_, y, tol); compare("H_pre", Hp_, Hp, tol32); compare("H_post", Ho_, Ho, tol32); compare("M", M_, M, tol32);
    compare_bf16("dx", gx, dx, tol); compare("dw", gw, dw, tol32); compare("dphi", gphi, dphi, tol32);
    compare("dbias", gb, dbias, tol32); compare("dalpha", ga, dalpha, tol32);
    for (void *p : {(void *)x_, (void *)dy_, (void *)w_, (void *)phi_, (void *)bias_, (void *)alpha_, (void *)y_, (void *)gx,
                    (void *)Hp_, (void *)Ho_, (void *)M_, (void *)P_, (void *)r_, (void *)q_, (void *)gw, (void *)gphi,
                    (void *)gb, (void *)ga, (void *)sk_, ws})
        (void)hipFree(p);
}

static void test_static_bf16(int B, int n, int C, int T) {
    printf("static H, bf16 storage   B=%d n=%d C=%d T=%d\n", B, n, C, T);
    const int nC = n * C, D = n * n + 2 * n;
    const double eps = 1e-6, tol = 2e-2, tol32 = 1e-4;
    std::mt19937 g(77 + B + 7 * n + 13 * C);
    auto x = randn((size_t)B * nC, 1.0, g), dy = randn((size_t)B * nC, 1.0, g), w = randn(C, 0.3, g), lg = randn(D, 1.0, g);
    for (auto &v : w) v += 1.0;
    round_to_bf16(x); round_to_bf16(dy); round_to_bf16(w);
    std::vector<double> y((size_t)B * nC), Hp(n), Ho(n), M(n * n), dx((size_t)B * nC), dw(C), dl(D);
    if (mhc_oracle_static_forward(x.data(), w.data(), lg.data(), nullptr, B, n, C, T, eps, y.data(), Hp.data(), Ho.data(), M.data()) ||
        mhc_oracle_static_backward(x.data(), dy.data(), w.data(), lg.data(), nullptr, B, n, C, T, eps, dx.data(), nullptr,
                                   dw.data(), dl.data())) {
        printf("    oracle refused the shape\n"); g_fail++; return;
    }
    uint16_t *x_ = to_dev_bf16(x), *dy_ = to_dev_bf16(dy), *w_ = to_dev_bf16(w);
    float *lg_ = to_dev(lg);
    uint16_t *y_ = dev_alloc_bf16((size_t)B * nC), *gx = dev_alloc_bf16((size_t)B * nC);
    float *Hp_ = dev_alloc(n), *Ho_ = dev_alloc(n), *M_ = dev_alloc(n * n), *q_ = dev_alloc(B), *gw = dev_alloc(C), *gl = dev_alloc(D);
    const size_t wsb = mhc_layer_static_workspace_bytes(B, n, C);
    void *ws; HIP_OK(hipMalloc(&ws, wsb + 256));
    MHC_OK_(mhc_layer_fwd(x_, MHC_BF16, w_, MHC_BF16, lg_, lg_ + n, lg_ + 2 * n, nullptr, y_, MHC_BF16, Hp_, Ho_, M_, q_, B, n, C,
                          T, (float)eps, ws, wsb, nullptr));
    MHC_OK_(mhc_layer_bwd(dy_, MHC_BF16, x_, MHC_BF16, w_, MHC_BF16, lg_, lg_ + n, lg_ + 2 * n, nullptr, Hp_, Ho_, M_, q_, gx,
                          nullptr, gw, gl, gl + n, gl + 2 * n, B, n, C, T, (float)eps, ws, wsb, nullptr));
    HIP_OK(hipDeviceSynchronize());
    compare_bf16("y", y_, y, tol); compare("M", M_, M, tol32);
    compare_bf16("dx", gx, dx, tol); compare("dw", gw, dw, tol32); compare("dlogits", gl, dl, tol32);
    for (void *p : {(void *)x_, (void *)dy_, (void *)w_, (void *)lg_, (void *)y_, (void *)gx, (void *)Hp_, (void *)Ho_, (void *)M_,
                    (void *)q_, (void *)gw, (void *)gl, ws})
        (void)hipFree(p);
}

int main() {
    printf("mHC layer native parity test (C ABI version %d vs fp64 C oracle; tolerance 1e-5 for fp32 storage; bf16 storage: 2e-2 for y and dx, 1e-4 for the float32 results)\n", mhc_abi_version());
    const int shapes[][3] = {{8, 4, 128}, {5, 3, 72}, {4, 8, 64}, {3, 16, 40}, {2, 32, 32}, {37, 4, 20}};
    for (auto &s : shapes) test_dynamic(s[0], s[1], s[2], 20);
    for (auto &s : shapes) test_static(s[0], s[1], s[2], 20);
    test_dynamic(4, 4, 64, 3);
    // bf16 storage: two-launch backward (n <= 8), tiled backward (n <= 4, B > 768), 8 x 8, the projection
    // products apart (n = 12), wide projection with the dx workgroups beside the coefficient launch (n = 20, 32)
    const int shapes16[][3] = {{64, 4, 256}, {1300, 4, 64}, {40, 8, 128}, {33, 12, 64}, {48, 20, 64}, {24, 32, 64}, {7, 3, 40}};
    for (auto &s : shapes16) test_dynamic_bf16(s[0], s[1], s[2], 20);
    for (auto &s : shapes16) test_static_bf16(s[0], s[1], s[2], 20);
    printf(g_fail ? "FAILED: %d comparisons\n" : "all comparisons passed\n", g_fail);
    return g_fail ? 1 : 0;
}
