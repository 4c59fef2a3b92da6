// Native benchmark of the mHC layer over the C ABI (libmhc_hip.so): no Python, no PyTorch.
//
//   bench_mhc_layer [--batch B] [--hidden C] [--expansion n] [--iters T] [--runs R] [--warmup W]
//                   [--static] [--fp32] [--all-configs]
//   bench_mhc_layer --ops [--runs R] [--warmup W]
//
// Counterpart of the reference's native layer benchmark (src/csrc/benchmarks/bench_mhc_layer.cu:
// warm-up, an L2 / cache flush before every timed run, event timing, bytes-moved bandwidth) for
// this library's entry points.  Times the forward and the backward call separately with HIP
// events, flushing 512 MiB before each timed call, and prints microseconds and the achieved
// fraction of the configuration's algorithmic HBM bytes at 8 TB/s.
// --ops: the two stand-alone operators at the shapes of the reference's per-operator benchmarks
// (src/csrc/benchmarks/bench_rmsnorm.cu:104-107, bench_rmsnorm_backward.cu:17-20,
// bench_sinkhorn_knopp.cu:117-120, bench_sinkhorn_knopp_backward.cu:23-25; CMake targets
// src/csrc/CMakeLists.txt:38-48), same protocol, bytes as those benchmarks count them.
#include <hip/hip_runtime.h>

#include <algorithm>
#include <cmath>
#include <cstdint>
#include <cstdio>
#include <cstdlib>
#include <cstring>
#include <random>
#include <vector>

#include "../../include/mhc_hip.h"


#define HIP_OK(e)                                                                      \
    do {                                                                               \
        hipError_t _e = (e);                                                           \
        if (_e != hipSuccess) {                                                        \
            fprintf(stderr, "HIP error %s at %s:%d\n", hipGetErrorString(_e), __FILE__, __LINE__); \
            exit(1);                                                                   \
        }                                                                              \
    } while (0)
#define MHC_OK_(e)                                                                     \
    do {                                                                               \
        int _s = (e);                                                                  \
        if (_s != MHC_OK) {                                                            \
            fprintf(stderr, "mhc error %d (%s) at %s:%d\n", _s, mhc_status_string(_s), __FILE__, __LINE__); \
            exit(1);                                                                   \
        }                                                                              \
    } while (0)

static uint16_t to_bf16(float f) {
    uint32_t u;
    memcpy(&u, &f, 4);
    u += 0x7fffu + ((u >> 16) & 1u);
    return (uint16_t)(u >> 16);
}

struct DeviceBuf {
    void *p = nullptr;
    size_t bytes = 0;
    explicit DeviceBuf(size_t b) : bytes(b) { HIP_OK(hipMalloc(&p, b ? b : 16)); }
    ~DeviceBuf() { (void)hipFree(p); }
    DeviceBuf(const DeviceBuf &) = delete;
};

static void upload(DeviceBuf &d, const std::vector<float> &h, bool bf16) {
    if (bf16) {
        std::vector<uint16_t> t(h.size());
        for (size_t i = 0; i < h.size(); i++) t[i] = to_bf16(h[i]);
        HIP_OK(hipMemcpy(d.p, t.data(), t.size() * 2, hipMemcpyHostToDevice));
    } else {
        HIP_OK(hipMemcpy(d.p, h.data(), h.size() * 4, hipMemcpyHostToDevice));
    }
}

static std::vector<float> randn(size_t n, float scale, std::mt19937 &g) {
    std::normal_distribution<float> d(0.f, 1.f);
    std::vector<float> v(n);
    for (auto &x : v) x = scale * d(g);
    return v;
}

static float trimmed_mean(std::vector<float> t) {
    std::sort(t.begin(), t.end());
    const size_t k = t.size() / 10;
    double s = 0;
    for (size_t i = k; i < t.size() - k; i++) s += t[i];
    return (float)(s / (double)(t.size() - 2 * k));
}

static void run_config(int B, int C, int n, int T, bool dynamic, bool bf16, int warmup, int runs) {
    const size_t BnC = (size_t)B * n * C, nC = (size_t)n * C, D = (size_t)n * n + 2 * n;
    const size_t es = bf16 ? 2 : 4;
    const int act = bf16 ? MHC_BF16 : MHC_F32;
    std::mt19937 gen(0);
    DeviceBuf x(BnC * es), dy(BnC * es), y(BnC * es), dx(BnC * es), w(C * es), dw(C * 4);
    upload(x, randn(BnC, 1.f, gen), bf16);
    upload(dy, randn(BnC, 1.f, gen), bf16);
    upload(w, std::vector<float>(C, 1.f), bf16);
    DeviceBuf Hp((dynamic ? B : 1) * n * 4), Ho((dynamic ? B : 1) * n * 4), M((dynamic ? B : 1) * n * n * 4);
    DeviceBuf q(B * 4), r(B * 4), P(B * D * 4);
    DeviceBuf sk(std::max<size_t>(mhc_layer_sinkhorn_state_floats(B, n, T), 4) * 4);
    DeviceBuf phi(dynamic ? D * nC * es : 16), dphi(dynamic ? D * nC * 4 : 16), bias(D * 4), dbias(D * 4);
    DeviceBuf alpha(16), dalpha(16), logits(D * 4), dlogits(D * 4);
    if (dynamic) {
        upload(phi, randn(D * nC, 0.02f, gen), bf16);
        upload(bias, std::vector<float>(D, 0.f), false);
        upload(alpha, std::vector<float>(3, 0.01f), false);
    } else {
        upload(logits, randn(D, 1.f, gen), false);
    }
    const size_t wsb = dynamic ? mhc_layer_dynamic_workspace_bytes(B, n, C) : mhc_layer_static_workspace_bytes(B, n, C);
    DeviceBuf ws(wsb);
    DeviceBuf flush(512u << 20);
    const float eps = 1e-6f;
    float *lg = (float *)logits.p, *dlg = (float *)dlogits.p;

    auto fwd = [&]() {
        if (dynamic)
            MHC_OK_(mhc_layer_fwd_dynamic(x.p, act, w.p, act, phi.p, act, (float *)bias.p, (float *)alpha.p, nullptr,
                                          y.p, act, (float *)Hp.p, (float *)Ho.p, (float *)M.p, (float *)P.p,
                                          (float *)r.p, (float *)q.p, (float *)sk.p, B, n, C, T, eps, ws.p, wsb, nullptr));
        else
            MHC_OK_(mhc_layer_fwd(x.p, act, w.p, act, lg, lg + n, lg + 2 * n, nullptr, y.p, act, (float *)Hp.p,
                                  (float *)Ho.p, (float *)M.p, (float *)q.p, B, n, C, T, eps, ws.p, wsb, nullptr));
    };
    auto bwd = [&]() {
        if (dynamic)
            MHC_OK_(mhc_layer_bwd_dynamic(dy.p, act, x.p, act, w.p, act, phi.p, act, (float *)bias.p, (float *)alpha.p,
                                          nullptr, (float *)Hp.p, (float *)Ho.p, (float *)M.p, (float *)P.p,
                                          (float *)r.p, (float *)q.p, (float *)sk.p, dx.p, nullptr, (float *)dw.p, (float *)dphi.p,
                                          (float *)dbias.p, (float *)dalpha.p, B, n, C, T, eps, ws.p, wsb, nullptr));
        else
            MHC_OK_(mhc_layer_bwd(dy.p, act, x.p, act, w.p, act, lg, lg + n, lg + 2 * n, nullptr, (float *)Hp.p,
                                  (float *)Ho.p, (float *)M.p, (float *)q.p, dx.p, nullptr, (float *)dw.p, dlg,
                                  dlg + n, dlg + 2 * n, B, n, C, T, eps, ws.p, wsb, nullptr));
    };
    hipEvent_t e0, e1;
    HIP_OK(hipEventCreate(&e0));
    HIP_OK(hipEventCreate(&e1));
    auto time_it = [&](auto &&fn) {
        std::vector<float> t;
        for (int i = 0; i < warmup + runs; i++) {
            HIP_OK(hipMemsetAsync(flush.p, i & 0xff, flush.bytes, nullptr));
            HIP_OK(hipEventRecord(e0, nullptr));
            fn();
            HIP_OK(hipEventRecord(e1, nullptr));
            HIP_OK(hipEventSynchronize(e1));
            float ms;
            HIP_OK(hipEventElapsedTime(&ms, e0, e1));
            if (i >= warmup) t.push_back(ms * 1e3f);
        }
        return trimmed_mean(t);
    };
    fwd();
    const float tf = time_it(fwd), tb = time_it(bwd);
    const double phib = dynamic ? 2.0 * nC * D : 0.0;
    const double fb = 2.0 * es * BnC + phib, bb = 3.0 * es * BnC + 3.0 * phib;
    printf("%-7s %-4s %6d %6d %4d %10.1f %10.1f %9.0f %9.0f %7.1f%% %7.1f%%\n", dynamic ? "dynamic" : "static",
           bf16 ? "bf16" : "fp32", B, C, n, tf, tb, fb / tf * 1e-3, bb / tb * 1e-3, fb / tf * 1e-3 / 80.0,
           bb / tb * 1e-3 / 80.0);
    HIP_OK(hipEventDestroy(e0));
    HIP_OK(hipEventDestroy(e1));
}

template <typename F> static float time_cold(F &&fn, DeviceBuf &flush, int warmup, int runs) {
    hipEvent_t e0, e1;
    HIP_OK(hipEventCreate(&e0));
    HIP_OK(hipEventCreate(&e1));
    std::vector<float> t;
    for (int i = 0; i < warmup + runs; i++) {
        HIP_OK(hipMemsetAsync(flush.p, i & 0xff, flush.bytes, nullptr));
        HIP_OK(hipEventRecord(e0, nullptr));
        fn();
        HIP_OK(hipEventRecord(e1, nullptr));
        HIP_OK(hipEventSynchronize(e1));
        float ms;
        HIP_OK(hipEventElapsedTime(&ms, e0, e1));
        if (i >= warmup) t.push_back(ms * 1e3f);
    }
    HIP_OK(hipEventDestroy(e0));
    HIP_OK(hipEventDestroy(e1));
    return trimmed_mean(t);
}

static void run_ops(int warmup, int runs) {
    DeviceBuf flush(512u << 20);
    std::mt19937 gen(0);
    printf("\nRMSNorm (bf16 rows, bf16 weight; bytes = rows read + written [+ gradient read])\n");
    printf("%6s %6s %10s %9s %10s %9s\n", "N", "C", "fwd us", "fwd GB/s", "bwd us", "bwd GB/s");
    const int rc[7][2] = {{128, 4096}, {256, 4096}, {512, 4096}, {1024, 4096}, {2048, 4096}, {1024, 8192}, {2048, 8192}};
    for (auto &c : rc) {
        const int N = c[0], C = c[1];
        const size_t NC = (size_t)N * C;
        DeviceBuf inp(NC * 2), out(NC * 2), grad(NC * 2), dinp(NC * 2), w(C * 2), rms(N * 4), dw(C * 4);
        upload(inp, randn(NC, 1.f, gen), true);
        upload(grad, randn(NC, 1.f, gen), true);
        upload(w, std::vector<float>(C, 1.f), true);
        const size_t wsb = mhc_rmsnorm_bwd_workspace_bytes(N, C);
        DeviceBuf ws(wsb);
        auto fwd = [&]() { MHC_OK_(mhc_rmsnorm_fwd(inp.p, MHC_BF16, w.p, MHC_BF16, out.p, (float *)rms.p, N, C, 1e-5f, nullptr)); };
        auto bwd = [&]() {
            MHC_OK_(mhc_rmsnorm_bwd(grad.p, inp.p, MHC_BF16, w.p, MHC_BF16, (const float *)rms.p, dinp.p, (float *)dw.p, N, C,
                                    ws.p, wsb, nullptr));
        };
        fwd();
        const float tf = time_cold(fwd, flush, warmup, runs), tb = time_cold(bwd, flush, warmup, runs);
        printf("%6d %6d %10.1f %9.0f %10.1f %9.0f\n", N, C, tf, 2.0 * NC * 2 / tf * 1e-3, tb, 3.0 * NC * 2 / tb * 1e-3);
    }
    printf("\nSinkhorn-Knopp, one fp32 matrix (threshold form, eps = 1e-8)\n");
    printf("%6s %6s %6s %10s %12s %10s %12s\n", "M", "N", "iters", "fwd us", "fwd us/iter", "bwd us", "bwd us/iter");
    const int sc[9][3] = {{32, 32, 5}, {32, 32, 10}, {32, 32, 20}, {64, 64, 5}, {64, 64, 10}, {64, 64, 20},
                          {128, 128, 5}, {128, 128, 10}, {128, 128, 20}};
    for (auto &c : sc) {
        const int M = c[0], N = c[1], it = c[2];
        const size_t MN = (size_t)M * N;
        DeviceBuf inp(MN * 4), out(MN * 4), grad(MN * 4), dinp(MN * 4);
        std::vector<float> h = randn(MN, 1.f, gen);
        for (auto &v : h) v = std::fabs(v) + 0.1f;  // positive entries, like the reference's benchmark input
        upload(inp, h, false);
        upload(grad, randn(MN, 1.f, gen), false);
        const size_t wsb = mhc_sinkhorn_knopp_bwd_workspace_bytes(1, M, N, it);
        DeviceBuf ws(wsb);
        auto fwd = [&]() { MHC_OK_(mhc_sinkhorn_knopp_fwd((const float *)inp.p, (float *)out.p, 1, M, N, it, 1e-8f, nullptr)); };
        auto bwd = [&]() {
            MHC_OK_(mhc_sinkhorn_knopp_bwd((const float *)grad.p, (const float *)inp.p, (float *)dinp.p, 1, M, N, it, 1e-8f, ws.p,
                                           wsb, nullptr));
        };
        const float tf = time_cold(fwd, flush, warmup, runs), tb = time_cold(bwd, flush, warmup, runs);
        printf("%6d %6d %6d %10.1f %12.2f %10.1f %12.2f\n", M, N, it, tf, tf / it, tb, tb / it);
    }
}

int main(int argc, char **argv) {
    int B = 320, C = 1280, n = 4, T = 20, runs = 50, warmup = 5;
    bool dynamic = true, bf16 = true, all = false, ops = false;
    for (int i = 1; i < argc; i++) {
        auto is = [&](const char *s) { return strcmp(argv[i], s) == 0; };
        if (is("--batch") && i + 1 < argc) B = atoi(argv[++i]);
        else if (is("--hidden") && i + 1 < argc) C = atoi(argv[++i]);
        else if (is("--expansion") && i + 1 < argc) n = atoi(argv[++i]);
        else if (is("--iters") && i + 1 < argc) T = atoi(argv[++i]);
        else if (is("--runs") && i + 1 < argc) runs = atoi(argv[++i]);
        else if (is("--warmup") && i + 1 < argc) warmup = atoi(argv[++i]);
        else if (is("--static")) dynamic = false;
        else if (is("--fp32")) bf16 = false;
        else if (is("--all-configs")) all = true;
        else if (is("--ops")) ops = true;
        else { fprintf(stderr, "unknown argument %s\n", argv[i]); return 2; }
    }
    printf("mHC layer native benchmark over the C ABI (ABI version %d); cold caches (512 MiB flush per call)\n",
           mhc_abi_version());
    if (ops) {
        run_ops(warmup, runs);
        return 0;
    }
    printf("%-7s %-4s %6s %6s %4s %10s %10s %9s %9s %8s %8s\n", "H", "act", "batch", "hidden", "n", "fwd us", "bwd us",
           "fwd GB/s", "bwd GB/s", "fwd roof", "bwd roof");
    if (all) {
        const int cfg[9][3] = {{320, 1280, 4}, {512, 1920, 4}, {1280, 2560, 4}, {2560, 1280, 4}, {128, 1280, 8},
                               {256, 1280, 8}, {32, 1280, 32}, {64, 1280, 32}, {128, 1280, 32}};
        for (int d = 0; d < 2; d++)
            for (auto &c : cfg) run_config(c[0], c[1], c[2], T, d == 1, bf16, warmup, runs);
    } else {
        run_config(B, C, n, T, dynamic, bf16, warmup, runs);
    }
    return 0;
}
