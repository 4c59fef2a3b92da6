// Prints the in-kernel phase timeline of the fused forward kernel and of the slab backward kernel.
//
//   phase_profile [--batch B] [--hidden C] [--expansion n]          (C % 8 == 0, bf16;
//                                                                    n > 4: projection backward instead of the slab kernel;
//                                                                    n > 8: the two coefficient kernels only)
//
// Links libmhc_hip_profile.so (python mhc.cu_amd/build.py --profile), the build of the library with
// csrc/phase_profiler.h compiled in.  Counterpart of the reference's HostProfiler::print_summary
// (src/csrc/include/utils.cuh:305-347): per phase the mean / 10th / 90th percentile over the
// recorded workgroups, in shader-clock ticks (s_memtime) and as a share of the workgroup's life.
#include <hip/hip_runtime.h>

#include <algorithm>
#include <cstdint>
#include <cstdio>
#include <cstdlib>
#include <cstring>
#include <random>
#include <vector>

#include "../../include/mhc_hip.h"

extern "C" int mhc_phase_read(int kernel, unsigned long long *host, int workgroups);
extern "C" int mhc_tuning_set(int key, int value);  // launch-heuristic override; the profile build has it (csrc/tuning.h)

#define HIP_OK(e) do { hipError_t _e = (e); if (_e != hipSuccess) { fprintf(stderr, "HIP error %s at line %d\n", hipGetErrorString(_e), __LINE__); exit(1); } } while (0)
#define MHC_OK_(e) do { int _s = (e); if (_s != MHC_OK) { fprintf(stderr, "mhc error %d (%s) at line %d\n", _s, mhc_status_string(_s), __LINE__); exit(1); } } while (0)

static uint16_t to_bf16(float f) { uint32_t u; memcpy(&u, &f, 4); u += 0x7fffu + ((u >> 16) & 1u); return (uint16_t)(u >> 16); }
static void *dev_bf16(size_t n, float scale, std::mt19937 &g) {
    std::normal_distribution<float> d(0.f, 1.f);
    std::vector<uint16_t> h(n);
    for (auto &v : h) v = to_bf16(scale * d(g));
    void *p; HIP_OK(hipMalloc(&p, n * 2 + 16)); HIP_OK(hipMemcpy(p, h.data(), n * 2, hipMemcpyHostToDevice));
    return p;
}
static float *dev_f32(size_t n, float val) {
    std::vector<float> h(n, val);
    float *p; HIP_OK(hipMalloc(&p, n * 4 + 16)); HIP_OK(hipMemcpy(p, h.data(), n * 4, hipMemcpyHostToDevice));
    return p;
}

static bool phase_slot_used(int kernel) {
    std::vector<unsigned long long> t(8 * 8);
    if (mhc_phase_read(kernel, t.data(), 8) != 0) return false;
    return std::any_of(t.begin(), t.end(), [](unsigned long long v) { return v != 0; });
}

static void summary(const char *title, int kernel, int wgs, const std::vector<const char *> &names, bool stamps) {
    constexpr int M = 8;
    std::vector<unsigned long long> t((size_t)wgs * M);
    if (mhc_phase_read(kernel, t.data(), wgs) != 0) { printf("%s: read failed\n", title); return; }
    // a kernel that the library did not launch for this shape left no stamps: no table
    if (std::all_of(t.begin(), t.end(), [](unsigned long long v) { return v == 0; })) return;
    printf("\n%s (first %d workgroups of the grid, shader-clock ticks)\n", title, wgs);
    printf("%-34s %10s %10s %10s %7s\n", "phase", "mean", "p10", "p90", "share");
    const int np = (int)names.size();
    std::vector<std::vector<double>> d(np);
    std::vector<double> life;
    for (int w = 0; w < wgs; w++) {
        double total = 0;
        for (int i = 0; i < np; i++) {
            const double v = stamps ? (double)(t[(size_t)w * M + i + 1] - t[(size_t)w * M + i]) : (double)t[(size_t)w * M + i];
            d[i].push_back(v);
            if (names[i][0] != ' ') total += v;  // indented lines break a phase down and are not added again
        }
        life.push_back(total);
    }
    double life_mean = 0;
    for (double v : life) life_mean += v;
    life_mean /= wgs;
    for (int i = 0; i < np; i++) {
        std::sort(d[i].begin(), d[i].end());
        double mean = 0;
        for (double v : d[i]) mean += v;
        mean /= wgs;
        printf("%-34s %10.0f %10.0f %10.0f %6.1f%%\n", names[i], mean, d[i][wgs / 10], d[i][wgs * 9 / 10], 100.0 * mean / life_mean);
    }
    printf("%-34s %10.0f\n", "workgroup life", life_mean);
}

int main(int argc, char **argv) {
    int B = 1280, C = 2560, n = 4, T = 20;
    for (int i = 1; i < argc; i++) {
        auto is = [&](const char *s) { return strcmp(argv[i], s) == 0; };
        if (is("--batch") && i + 1 < argc) B = atoi(argv[++i]);
        else if (is("--hidden") && i + 1 < argc) C = atoi(argv[++i]);
        else if (is("--expansion") && i + 1 < argc) n = atoi(argv[++i]);
        else if (is("--tune") && i + 2 < argc) { mhc_tuning_set(atoi(argv[i + 1]), atoi(argv[i + 2])); i += 2; }
        else { fprintf(stderr, "unknown argument %s\n", argv[i]); return 2; }
    }
    if (n > 32 || C % 8) { fprintf(stderr, "the instrumented kernels serve n <= 32 with C %% 8 == 0\n"); return 2; }
    const size_t BnC = (size_t)B * n * C, nC = (size_t)n * C, D = (size_t)n * n + 2 * n;
    std::mt19937 g(0);
    void *x = dev_bf16(BnC, 1.f, g), *dy = dev_bf16(BnC, 1.f, g), *phi = dev_bf16(D * nC, 0.02f, g), *w = dev_bf16(C, 0.f, g);
    { std::vector<uint16_t> one(C, to_bf16(1.f)); HIP_OK(hipMemcpy(w, one.data(), C * 2, hipMemcpyHostToDevice)); }
    void *y, *dx; HIP_OK(hipMalloc(&y, BnC * 2)); HIP_OK(hipMalloc(&dx, BnC * 2));
    float *bias = dev_f32(D, 0.f), *alpha = dev_f32(3, 0.01f), *Hp = dev_f32((size_t)B * n, 0.f), *Ho = dev_f32((size_t)B * n, 0.f),
          *M = dev_f32((size_t)B * n * n, 0.f), *P = dev_f32(B * D, 0.f), *r = dev_f32(B, 0.f), *q = dev_f32(B, 0.f),
          *dw = dev_f32(C, 0.f), *dphi = dev_f32(D * nC, 0.f), *dbias = dev_f32(D, 0.f), *dalpha = dev_f32(3, 0.f);
    float *sk = dev_f32(mhc_layer_sinkhorn_state_floats(B, n, T), 0.f);
    const size_t wsb = mhc_layer_dynamic_workspace_bytes(B, n, C);
    void *ws; HIP_OK(hipMalloc(&ws, wsb + 256));
    for (int it = 0; it < 3; it++) {
        MHC_OK_(mhc_layer_fwd_dynamic(x, MHC_BF16, w, MHC_BF16, phi, MHC_BF16, bias, alpha, nullptr, y, MHC_BF16, Hp, Ho, M, P, r,
                                      q, sk, B, n, C, T, 1e-6f, ws, wsb, nullptr));
        MHC_OK_(mhc_layer_bwd_dynamic(dy, MHC_BF16, x, MHC_BF16, w, MHC_BF16, phi, MHC_BF16, bias, alpha, nullptr, Hp, Ho, M, P, r, q,
                                      sk, dx, nullptr, dw, dphi, dbias, dalpha, B, n, C, T, 1e-6f, ws, wsb, nullptr));
        HIP_OK(hipDeviceSynchronize());
    }
    printf("phase profile: dynamic H, bf16, B=%d C=%d n=%d (last of 3 warm calls)\n", B, C, n);
    if (n > 8) {
        summary("coefficient forward kernel (n > 8), one workgroup per sample", 7, std::min(B, 4096),
                {"split-K partial sums of the projection arrive", "logits, activations, stream tile requested",
                 "Sinkhorn iterations", "M and Sinkhorn state stores issued", "stream tile arrives, aggregate, RMS"}, true);
        summary("coefficient backward kernel (n > 8), one workgroup per sample", 8, std::min(B, 4096),
                {"inputs requested, Sinkhorn state loaded (or recomputed)", "Gram parts arrive, summed, parked",
                 "dHpre / dHpost / s1", "Sinkhorn reverse sweep", "dt / dP stores issued"}, true);
        return 0;
    }
    if (n <= 4 && (n * C) % 64 == 0) {
        const int G = std::min(16, std::max(1, (B + 255) / 256));
        summary("one-launch forward kernel, one workgroup per G samples (wave 0 of each)", 6, std::min((B + G - 1) / G, 4096),
                {"phase A: stream x and phi, project", "wait for the other waves", "activations",
                 "Sinkhorn (wave 0) while the other waves aggregate", "RMS", "mix pass, stores issued"}, true);
    }
    summary("fused forward kernel, one workgroup per sample", 0, std::min(B, 4096),
            {"issue loads (early half: tile too)", "coefficient inputs arrive", "activations + Sinkhorn", "tile request (late half), barrier", "tile arrives, aggregate, RMS",
             "mix, stores issued"}, true);
    {
        const int tiles = (B + 31) / 32;
        summary("narrow projection kernel, one workgroup per (32 samples, K slab), wave 0 of each", 3, std::min(tiles * 16, 4096),
                {"start, first chunk requested", "waits for chunks, parks (all chunks)", "fragments, matrix cores (all chunks)",
                 "cross-wave sum, partial stores"}, false);
    }
    // Which backward ran shows in the stamps: the tiled path leaves the slab (n <= 4) or the projection-backward
    // table, the two-launch path neither.  Both use slots 4 and 5, for different kernels.
    const bool tiled = phase_slot_used(n > 4 ? 2 : 1);
    if (tiled) {
        summary("channel sums + coefficient backward kernel, one workgroup per sample", 4, std::min(B, 4096),
                {"start: coefficient inputs, Sinkhorn state (wave 0)", "streaming loop (wave 0's steps)",
                 "workgroup sums", "coefficient backward (all of it: the three lines below)",
                 "  channel-sum vectors, dHpre / dHpost", "  Sinkhorn reverse sweep", "  dt / dP stores, alpha sums"}, false);
    } else {
        summary("sample-resident backward kernel, one workgroup per sample: its coefficient wave (wave 0)", 4, std::min(B, 4096),
                {"start: coefficient inputs, Sinkhorn state", "waits for the tile waves' Gram sums",
                 "workgroup sums", "coefficient backward (all of it: the three lines below)",
                 "  channel-sum vectors, dHpre / dHpost", "  Sinkhorn reverse sweep", "  dt / dP stores, alpha sums"}, false);
        summary("sample-resident backward kernel: the first tile wave of each workgroup", 5, std::min(B, 4096),
                {"loads requested", "tile arrives, Gram sums, slots written", "two barriers (workgroup sums between them)",
                 "dxp / u computed, stores issued"}, false);
        summary("column-slab kernel, one workgroup per 32 columns of x_flat, all samples (wave 0 of each)", 9,
                std::min((int)(nC / 32), 4096),
                {"prologue: phi slab and the first two blocks requested, slab staged",
                 "operands and x block arrive, block staged, barrier (all blocks)", "matrix cores: dphi and dP phi (all blocks)",
                 "epilogue: dx completed and stored, next loads requested (all)", "dphi summed over the waves and stored"}, false);
        return 0;
    }
    if (n > 4) {
        summary("dx kernel (generic, one wave per workgroup)", 5, std::min(B * ((C / 4 + 63) / 64), 4096),
                {"start: coefficients and all loads requested", "data arrives, df / a / da", "mixing, dx stores issued", "dw / dt partial sums"}, false);
        summary("projection backward kernel, one workgroup per 32 columns of x_flat", 2, std::min((int)(nC / 32), 4096),
                {"prologue (phi slab, first x block requested)", "operands requested, x block parked (all blocks)",
                 "fragments, dphi on the matrix cores (all)", "dxflat on the matrix cores, stores (all)", "dphi stores"}, false);
        return 0;
    }
    const int slabs = (C + 63) / 64;
    summary("slab backward kernel, one workgroup per (64 channels, batch split)", 1, std::min(slabs * 4, 4096),
            {"prologue (phi slab, first loads)", "tile loads, LDS, barrier (all tiles)", "matrix cores, barrier (all tiles)",
             "coefficients, mixing, stores (all)", "epilogue: dphi partial stores", "epilogue: dw / dbias partial sums"}, false);
    return 0;
}
