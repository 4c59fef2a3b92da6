// C ABI of libmhc_hip.so (declared in include/mhc_hip.h): argument validation, workspace
// carving and the launch sequence of each entry point.  No allocation, no synchronisation,
// no global state; every call only enqueues kernels on the caller's stream.  The one exception
// is mhc_layer_fwd_dynamic_static_scratch at the end of this file, whose scratch memory is a
// device array owned by the library.
#include "../../include/mhc_hip.h"

#include "launchers.h"
#include "phase_profiler.h"
#include "tuning.h"

#include <mutex>
#include <stdint.h>

using namespace mhc;

#ifdef MHC_TUNING
namespace mhc {
int g_tuning[kTuneCount];
}
#endif

namespace {

struct Carver {
    char *base;
    size_t off = 0;
    explicit Carver(void *p) : base(static_cast<char *>(p)) {}
    float *floats(size_t count) {
        float *p = base ? reinterpret_cast<float *>(base + off) : nullptr;
        off += (count * sizeof(float) + 255) / 256 * 256;
        return p;
    }
};

inline bool aligned16(const void *p) { return (reinterpret_cast<uintptr_t>(p) & 15u) == 0; }
inline bool valid_dtype(int d) { return d == MHC_F32 || d == MHC_BF16; }
inline bool valid_io(int x_dtype, int y_dtype) {
    // activations in / out: (f32, f32), (bf16, bf16), (bf16 in, f32 out), (f32 consumed as bf16 in, f32 out)
    return (x_dtype == MHC_F32 && y_dtype == MHC_F32) || (x_dtype == MHC_BF16 && valid_dtype(y_dtype)) ||
           (x_dtype == MHC_F32_AS_BF16 && y_dtype == MHC_F32);
}

int check_shape(int B, int n, int C, int iters) {
    if (n < 1 || n > MHC_MAX_N) return MHC_ERR_BAD_N;
    if (B < 1 || C < 1 || iters < 0 || iters > max_layer_sinkhorn_iters(n)) return MHC_ERR_BAD_SHAPE;
    if ((long long)B * n * C > (1ll << 40)) return MHC_ERR_BAD_SHAPE;
    if (C > MHC_MAX_C) return MHC_ERR_BAD_SHAPE;       // the generic kernels keep a [C] float row in LDS
    return MHC_OK;
}

int ws_check(void *ws, size_t have, size_t need) {
    if (need == 0) return MHC_OK;
    if (!ws || (reinterpret_cast<uintptr_t>(ws) & 255u) != 0 || have < need) return MHC_ERR_WORKSPACE;
    return MHC_OK;
}

#define MHC_LAUNCH(expr)                              \
    do {                                              \
        if ((expr) != hipSuccess) return MHC_ERR_LAUNCH; \
    } while (0)

// ---- dynamic workspace layout ----------------------------------------------------------------
struct DynFwdWs { float *Ppart, *ssqpart, *agg; size_t bytes; };
struct DynBwdWs { float *dt, *dP, *cx, *s1, *u, *dtpart, *raw, *s1part, *dx_part, *dphi_part; unsigned short *dPb, *dPT; int BP; size_t bytes; };

// Whether the sample-resident backward (bwd_resident.hip + the column-slab kernel without batch split)
// is taken where it is supported.  Its second launch walks all samples of a column slab in one
// workgroup, which stops paying once the batch is large enough to fill the chip with batch splits.
// Measured, backward in graphs of ten, slab / Gram path -> resident path (us):
//   n=4 C=1280: B=64 17.1 -> 9.2, 128 17.2 -> 9.7, 320 19.1 -> 14.9, 512 23.6 -> 19.0, 768 25.1 -> 24.3,
//               1024 29.8 -> 29.6, 1536 35.7 -> 39.4, 2560 46.2 -> 62.5;  n=4 C=2048: B=768 33.5 -> 30.3, 1024 35.1 -> 41.2
//   n=4 C=2560: B=256 23.9 -> 17.8, 512 32.0 -> 26.9, 768 36.3 -> 35.9, 1280 42.4 -> 53.9;  n=2 C=1280: B=1024 23.7 -> 28.8
//   n=8 C=1280: B=128 25.1 -> 16.9, 256 30.5 -> 22.0, 512 46.1 -> 36.1, 1024 77.3 -> 62.7
// n = 5 .. 8 with short rows and a large batch: a workgroup per sample then has too little to do, and the
// tiled path (several samples per workgroup) wins:
//   n=8 C=256: B=512 30.9 -> 23.8, 1024 39.9 -> 41.3, 2048 59.8 -> 73.4, 4096 94.0 -> 137.7;  C=128: B=8192 139.7 -> 261.4
//   n=8 C=512: B=1024 43.7 -> 45.7, 2048 74.0 -> 83.1, 4096 124.2 -> 157.7;  C=1024: 1024 61.1 -> 51.6, 4096 182.2 -> 179.3
//   n=6 C=512: B=1024 40.1 -> 43.5, 4096 113.0 -> 149.8;  n=5 C=384: B=3000 85.2 -> 97.8
// Experiment hook: 1 = never, 2 = always.
bool bwd_resident_preferred(int B, int n, int C) {
    if (const int hook = tuning_get(kTuneResident)) return hook == 2;
    if (n > 4) return !(B >= 1024 && C <= 512);
    return B <= 768;
}

// Shapes for which the dynamic entry points take fp32 activations that are consumed as bf16
// (MHC_F32_AS_BF16): the kernels that load fp32 storage directly are the narrow projection, the fused
// n <= 8 forward and the two launches of the sample-resident backward.  That backward is taken for fp32
// storage at every batch size, also where the tiled path is faster on bf16 storage: the alternative is
// a cast pass over x on top of the tiled path (through the module, fp32 tensors, forward + backward:
// B=1280 C=2560 n=4 186 -> 184 us, B=2560 C=1280 184 -> 176, B=1024 C=1280 111 -> 100).
bool f32_as_bf16_accepted(int B, int n, int C, int iters) {
    return n <= 8 && layer_fwd_fused_supported(n, C, kF32) &&
           bwd_resident_supported(kF32AsBF16, kF32, kBF16, n, C, iters) && proj_bwd_addx_supported(n);
}

int max_ksplit(int B, int n, int C) {
    const int a = proj_fwd_ksplit(kBF16, kBF16, B, n, C), b = proj_fwd_ksplit(kF32, kF32, B, n, C);
    return a > b ? a : b;
}

DynFwdWs carve_dyn_fwd(void *ws, int B, int n, int C) {
    Carver c(ws);
    const int ks = max_ksplit(B, n, C);
    DynFwdWs w;
    w.Ppart = c.floats((size_t)ks * B * padded_D(n));
    w.ssqpart = c.floats((size_t)ks * B);
    w.agg = c.floats(n > 8 ? (size_t)B * C : 0);  // stream aggregate of the matrix-core mix
    w.bytes = c.off;
    return w;
}

// Wide projections (n > 18) without batch split of dphi: four launches, see mhc_layer_bwd_dynamic.
// Up to 16 M activation elements: the fp32 hand-over costs 4 more bytes per element than completing dx
// in place, which the shorter chain repays only while the coefficient launch leaves CUs idle
// (backward us, four launches | five: B=128 n=32 C=1280 92 | 100, 384 n=32 C=1280 214 | 215,
//  512 n=32 C=1280 283 | 269, 256 n=32 C=2560 338 | 312).
bool wide_dx_beside(int B, int n, int C) {
    return proj_bwd_is_wide(n) && C % 8 == 0 && proj_bwd_batch_splits(B, n, C) == 1 &&
           (long long)B * n * C <= (16ll << 20);
}

DynBwdWs carve_dyn_bwd(void *ws, int B, int n, int C) {
    Carver c(ws);
    const int D = n * n + 2 * n, nC = n * C;
    DynBwdWs w;
    w.dt = c.floats((size_t)B * (D + 3));
    w.dP = c.floats((size_t)B * padded_D(n));
    w.cx = c.floats(B);
    w.s1 = c.floats(B);
    w.u = c.floats((size_t)B * C);
    w.dtpart = c.floats((size_t)B * (D + 3));
    w.raw = c.floats(bwd_reduce_raw_floats(B, n, C));
    w.s1part = c.floats(n > 8 ? (size_t)B * bwd_reduce_parts(B, n, C) : 0);
    // wide projections: the part of dx that is formed beside the coefficient backward, fp32
    w.dx_part = c.floats(wide_dx_beside(B, n, C) ? (size_t)B * nC : 0);
    int bs = dphi_batch_splits(B, n, C);
    const int bs2 = proj_bwd_batch_splits(B, n, C);
    if (bs2 > bs) bs = bs2;
    const int bs3 = n <= 4 ? bwd_slab_batch_splits(B, n, C) : 1;
    if (bs3 > bs) bs = bs3;
    w.dphi_part = c.floats(bs > 1 ? (size_t)bs * D * nC : 0);
    w.BP = (B + 31) / 32 * 32;
    w.dPb = reinterpret_cast<unsigned short *>(c.floats(((size_t)w.BP * padded_D(n) + 1) / 2));
    w.dPT = reinterpret_cast<unsigned short *>(c.floats((size_t)padded_D(n) * w.BP));  // two bf16 planes
    w.bytes = c.off;
    return w;
}

// ---- static workspace layout -----------------------------------------------------------------
struct StaFwdWs { float *Hpre, *Hpost, *M, *q, *agg; size_t bytes; };
struct StaBwdWs { float *red, *s1, *u, *red_sum, *raw, *sk, *s1part; size_t bytes; };

StaFwdWs carve_sta_fwd(void *ws, int B, int n, int C) {
    Carver c(ws);
    StaFwdWs w;
    w.Hpre = c.floats(n); w.Hpost = c.floats(n); w.M = c.floats((size_t)n * n); w.q = c.floats(B);
    w.agg = c.floats(n > 8 ? (size_t)B * C : 0);
    w.bytes = c.off;
    return w;
}

StaBwdWs carve_sta_bwd(void *ws, int B, int n, int C) {
    Carver c(ws);
    const int D = n * n + 2 * n;
    StaBwdWs w;
    w.red = c.floats((size_t)B * (D + 3));
    w.s1 = c.floats(B);
    w.u = c.floats((size_t)B * C);
    w.red_sum = c.floats(D + 3);
    w.raw = c.floats(n > 8 ? bwd_reduce_raw_floats(B, n, C) : 0);
    w.sk = c.floats(n > 8 ? (size_t)(2 * max_layer_sinkhorn_iters(n) + 2) * 32 : 0);
    w.s1part = c.floats(n > 16 ? (size_t)B * bwd_reduce_parts(B, n, C) : 0);  // Sinkhorn denominators of the shared logits
    w.bytes = c.off;
    return w;
}

}  // namespace

#ifdef MHC_PHASE_PROFILE
namespace mhc {
__device__ unsigned long long g_phase[kPhaseKernels][kPhaseMaxWg][kPhaseMaxMarks];
}
#endif

extern "C" {

#ifdef MHC_PHASE_PROFILE
// Profile build only (declared in csrc/phase_profiler.h's host interface, not in the product header):
// copies the stamp table of one instrumented kernel to host memory; returns the HIP status.
__attribute__((visibility("default"))) int mhc_phase_read(int kernel, unsigned long long *host, int workgroups) {
    if (kernel < 0 || kernel >= mhc::kPhaseKernels || workgroups > mhc::kPhaseMaxWg) return -1;
    return (int)hipMemcpyFromSymbol(host, HIP_SYMBOL(mhc::g_phase),
                                    sizeof(unsigned long long) * mhc::kPhaseMaxMarks * workgroups,
                                    sizeof(unsigned long long) * mhc::kPhaseMaxMarks * mhc::kPhaseMaxWg * kernel);
}
#endif

int mhc_abi_version(void) { return MHC_ABI_VERSION; }

#ifdef MHC_TUNING
// Experiment hooks (csrc/tuning.h): only in the -DMHC_TUNING build, never in the product library.
__attribute__((visibility("default"))) int mhc_tuning_set(int key, int value) {
    if (key < 0 || key >= kTuneCount) return -1;
    g_tuning[key] = value;
    return 0;
}
__attribute__((visibility("default"))) int mhc_tuning_get(int key) {
    return (key < 0 || key >= kTuneCount) ? -1 : g_tuning[key];
}
#endif

int mhc_max_sinkhorn_iters(int n) { return (n < 1 || n > MHC_MAX_N) ? 0 : max_layer_sinkhorn_iters(n); }

int mhc_layer_dynamic_accepts_f32_as_bf16(int B, int n, int C, int iters) {
    return check_shape(B, n, C, iters) == MHC_OK && f32_as_bf16_accepted(B, n, C, iters) ? 1 : 0;
}

const char *mhc_status_string(int status) {
    switch (status) {
        case MHC_OK: return "ok";
        case MHC_ERR_NULL_POINTER: return "a required pointer is NULL";
        case MHC_ERR_BAD_N: return "expansion rate n must be in 1..32";
        case MHC_ERR_BAD_SHAPE:
            return "B, C or iters out of range (C <= 32768; B * n * C <= 2^40; iters <= mhc_max_sinkhorn_iters(n))";
        case MHC_ERR_BAD_DTYPE: return "unsupported dtype combination";
        case MHC_ERR_MISALIGNED: return "tensor base pointer is not 16-byte aligned";
        case MHC_ERR_WORKSPACE: return "workspace NULL, not 256-byte aligned or too small";
        case MHC_ERR_LAUNCH: return "HIP kernel launch failed";
        case MHC_ERR_SCRATCH_LIMIT:
            return "shape needs more scratch than the library's static array holds (mhc_static_scratch_capacity)";
        default: return "unknown status";
    }
}

// ===============================================================================================
// dynamic H
// ===============================================================================================
size_t mhc_layer_dynamic_workspace_bytes(int B, int n, int C) {
    if (check_shape(B, n, C, 0) != MHC_OK) return 0;
    const size_t f = carve_dyn_fwd(nullptr, B, n, C).bytes;
    const size_t b = carve_dyn_bwd(nullptr, B, n, C).bytes;
    return f > b ? f : b;
}

size_t mhc_layer_sinkhorn_state_floats(int B, int n, int iters) {
    if (n < 1 || n > MHC_MAX_N || B < 1 || iters < 0) return 0;
    return (size_t)B * (iters + 1) * 2 * sinkhorn_state_np(n);
}

int mhc_layer_fwd_dynamic(const void *x, int x_dtype, const void *w, int w_dtype, const void *phi,
                          int phi_dtype, const float *bias, const float *alpha,
                          const void *f_inject, void *y, int y_dtype, float *H_pre, float *H_post,
                          float *M, float *P, float *r, float *q, float *sk_state, int B, int n, int C,
                          int iters, float eps, void *workspace, size_t workspace_bytes, void *stream) {
    if (int s = check_shape(B, n, C, iters)) return s;
    if (!x || !phi || !bias || !alpha || !y || !H_pre || !H_post || !M || !P || !r || !q)
        return MHC_ERR_NULL_POINTER;
    if (!f_inject && !w) return MHC_ERR_NULL_POINTER;
    if (!valid_io(x_dtype, y_dtype) || !valid_dtype(phi_dtype) || (w && !valid_dtype(w_dtype)))
        return MHC_ERR_BAD_DTYPE;
    if (x_dtype == MHC_F32_AS_BF16 && (phi_dtype != MHC_BF16 || !f32_as_bf16_accepted(B, n, C, iters)))
        return MHC_ERR_BAD_DTYPE;
    if (!aligned16(x) || !aligned16(y) || !aligned16(phi) || (f_inject && !aligned16(f_inject)))
        return MHC_ERR_MISALIGNED;
    const DynFwdWs ws = carve_dyn_fwd(workspace, B, n, C);
    if (int s = ws_check(workspace, workspace_bytes, ws.bytes)) return s;
    hipStream_t st = static_cast<hipStream_t>(stream);
    if (layer_fwd_onepass_supported(x_dtype, phi_dtype, B, n, C)) {
        // projection, coefficients and mix in one launch; x crosses HBM once
        MHC_LAUNCH(launch_layer_fwd_onepass(x, w, w_dtype, f_inject, y, y_dtype, phi, alpha, bias, H_pre, H_post,
                                            M, P, r, q, sk_state, B, n, C, iters, eps, st));
        return MHC_OK;
    }
    const int KS = proj_fwd_ksplit(x_dtype, phi_dtype, B, n, C);
    MHC_LAUNCH(launch_proj_fwd(x, x_dtype, phi, phi_dtype, ws.Ppart, ws.ssqpart, KS, B, n, C, st));
    if (layer_fwd_fused_supported(n, C, x_dtype)) {
        MHC_LAUNCH(launch_layer_fwd_fused(x, x_dtype, w, w_dtype, f_inject, y, y_dtype, ws.Ppart,
                                          ws.ssqpart, KS, padded_D(n), alpha, bias, bias + n,
                                          bias + 2 * n, H_pre, H_post, M, P, r, q, sk_state, B, n, C, iters,
                                          eps, st));
        return MHC_OK;
    }
    // n > 8 in the bf16 tier: the coefficient launch also forms the stream aggregate and its RMS
    const bool agg = !f_inject && ws.agg && coef_fwd_aggregates(n, C, x_dtype);
    MHC_LAUNCH(launch_coef_fwd(ws.Ppart, ws.ssqpart, KS, padded_D(n), alpha, bias, bias + n,
                               bias + 2 * n, H_pre, H_post, M, P, r, B, n, n * C, iters, eps,
                               x_dtype == kF32, agg ? x : nullptr, ws.agg, q, sk_state, st));
    MHC_LAUNCH(launch_mix_fwd(x, x_dtype, w, w_dtype, f_inject, y, y_dtype, H_pre, H_post, M, n, q,
                              ws.agg, B, n, C, eps, agg, st));
    return MHC_OK;
}

int mhc_layer_bwd_dynamic(const void *dy, int y_dtype, const void *x, int x_dtype, const void *w,
                          int w_dtype, const void *phi, int phi_dtype, const float *bias,
                          const float *alpha, const void *f_inject, const float *H_pre,
                          const float *H_post, const float *M, const float *P, const float *r,
                          const float *q, const float *sk_state, void *dx, void *df, float *dw, float *dphi,
                          float *dbias, float *dalpha, int B, int n, int C, int iters, float eps,
                          void *workspace, size_t workspace_bytes, void *stream) {
    if (int s = check_shape(B, n, C, iters)) return s;
    if (!dy || !x || !phi || !bias || !alpha || !H_pre || !H_post || !M || !P || !r || !q || !dx ||
        !dphi || !dbias || !dalpha)
        return MHC_ERR_NULL_POINTER;
    if (!f_inject && (!w || !dw)) return MHC_ERR_NULL_POINTER;
    if (!valid_io(x_dtype, y_dtype) || !valid_dtype(phi_dtype) || (w && !valid_dtype(w_dtype)))
        return MHC_ERR_BAD_DTYPE;
    if (x_dtype == MHC_F32_AS_BF16 && (phi_dtype != MHC_BF16 || !f32_as_bf16_accepted(B, n, C, iters)))
        return MHC_ERR_BAD_DTYPE;
    if (!aligned16(dy) || !aligned16(x) || !aligned16(dx) || !aligned16(phi) || !aligned16(dphi) ||
        (f_inject && !aligned16(f_inject)) || (df && !aligned16(df)))
        return MHC_ERR_MISALIGNED;
    const DynBwdWs ws = carve_dyn_bwd(workspace, B, n, C);
    if (int s = ws_check(workspace, workspace_bytes, ws.bytes)) return s;
    hipStream_t st = static_cast<hipStream_t>(stream);
    const int D = n * n + 2 * n, DP = padded_D(n);
    const bool mfma = proj_bwd_mfma_supported(x_dtype == kF32AsBF16 ? kBF16 : x_dtype, phi_dtype, C);
    BwdCoefOut out{ws.dt, ws.dP, ws.cx, ws.s1, nullptr, mfma ? ws.dPb : nullptr, ws.dPT, ws.BP};
    if (mfma && bwd_resident_supported(x_dtype, y_dtype, phi_dtype, n, C, iters) && proj_bwd_addx_supported(n) &&
        (bwd_resident_preferred(B, n, C) || x_dtype == kF32AsBF16)) {
        // two launches: (1) one workgroup per sample keeps the sample's rows of dy and x in registers for
        // the channel sums, the coefficient backward and the mixing part of dx; (2) a column-slab
        // kernel over all samples adds dP phi - cx x, finishes dphi without batch-split partial sums
        // and sums dw, dbias and dalpha in a few extra workgroups
        BwdCoefOut out2 = out;
        out2.dP = nullptr;  // the second launch takes dP as matrix-core operands only
        MHC_LAUNCH(launch_bwd_resident(dy, x, x_dtype, w, w_dtype, f_inject, H_pre, H_post, M, q, P, r, alpha, bias + 2 * n,
                                       sk_state, out2, dx, df, ws.u, B, n, C, iters, eps, st));
        const BatchSumArgs sums = make_batch_sums(ws.u, B, C, f_inject ? nullptr : dw, ws.dt, B, D, dbias, dalpha);
        bool tail_taken = false;
        MHC_LAUNCH(launch_proj_bwd_addx(x, x_dtype, phi, ws.dPb, ws.dPT, ws.BP, ws.cx, dphi, dx, B, n, C,
                                        tuning_get(kTuneSeparateFinalize) == 1 ? nullptr : &sums, &tail_taken, st));
        if (!tail_taken)
            MHC_LAUNCH(launch_finalize(ws.u, B, C, f_inject ? nullptr : dw, ws.dt, B, D, dbias, dalpha, nullptr, 1,
                                       0, nullptr, st));
        return MHC_OK;
    }
    if (x_dtype == kF32AsBF16) return MHC_ERR_BAD_DTYPE;  // not reached: accepted shapes take the path above
    if (mfma && x_dtype == kBF16 && y_dtype == kBF16 && wide_dx_beside(B, n, C) && tuning_get(kTuneWideDxBeside) != 1) {
        // wide projection (n > 18), four launches.  The coefficient backward is one workgroup per sample,
        // all dependent chains; the part of dx that needs none of its results (M^T dy + Hpre (x) da,
        // with s1 from the channel sums) runs beside it in the same launch and is handed over in fp32;
        // the dP phi kernel then completes dx (+ dP phi - cx x, one rounding); dphi comes last and carries
        // the batch sums.
        // B=128 n=32 C=1280, backward in graphs of ten, same box: five launches 99.8 us, these four 93.0 us
        MHC_LAUNCH(launch_mix_bwd_reduce_with_dx(dy, x, w, w_dtype, f_inject, H_pre, H_post, M, n, q, P, r, alpha,
                                                 bias + 2 * n, sk_state, out, ws.raw, ws.s1part, ws.dx_part, df, ws.u, B, n, C,
                                                 iters, eps, st));
        MHC_LAUNCH(launch_dxflat_wide(phi, ws.dPb, ws.BP, dx, x, ws.cx, ws.dx_part, B, n, C, st));
        const BatchSumArgs sums = make_batch_sums(ws.u, B, C, f_inject ? nullptr : dw, ws.dt, B, D, dbias, dalpha);
        bool tail_taken = false;
        MHC_LAUNCH(launch_dphi_large(x, ws.dPT, ws.BP, dphi, 1, B, n, C,
                                     tuning_get(kTuneSeparateFinalize) != 1 ? &sums : nullptr, &tail_taken, st));
        if (!tail_taken)
            MHC_LAUNCH(launch_finalize(ws.u, B, C, f_inject ? nullptr : dw, ws.dt, B, D, dbias, dalpha, nullptr, 1,
                                       (size_t)D * n * C, dphi, st));
        return MHC_OK;
    }
    MHC_LAUNCH(launch_mix_bwd_reduce(dy, y_dtype, x, x_dtype, w, w_dtype, f_inject, H_pre, H_post, M,
                                     n, q, P, r, alpha, bias + 2 * n, sk_state, out, ws.raw, B, n, C, iters, eps,
                                     st));
    if (mfma && bwd_slab_supported(x_dtype, y_dtype, phi_dtype, n, C)) {
        // n <= 4: one slab kernel finishes dx and produces every batch-split partial sum
        const int S = bwd_slab_batch_splits(B, n, C);
        MHC_LAUNCH(launch_bwd_slab(dy, y_dtype, x, w, w_dtype, f_inject, phi, H_pre, H_post, M, q, ws.s1,
                                   ws.cx, ws.dPb, ws.dPT, ws.BP, ws.dt, dx, df,
                                   S > 1 ? ws.dphi_part : dphi, ws.u, ws.dtpart, S, B, n, C, st));
        MHC_LAUNCH(launch_finalize(ws.u, S, C, f_inject ? nullptr : dw, ws.dtpart, S, D, dbias, dalpha,
                                   ws.dphi_part, S, (size_t)D * n * C, dphi, st));
        return MHC_OK;
    }
    const int spg = bwd_dx_samples_per_group(B, n);
    const int groups = (B + spg - 1) / spg;
    int S = 1;
    if (mfma) {
        // matrix cores: dphi and the projection term of dx (written into dx, then completed in place)
        S = proj_bwd_batch_splits(B, n, C);
        // From D > 128 on the two products run as launches of their own (they share no operand but dP
        // and no output): dP phi first, then the dx kernel that consumes it, dphi = dP^T x last.  The
        // last launch carries the batch sums (dw, dbias, dalpha) in an extra row of workgroups, which
        // run in the shadow of the dphi stores instead of as a launch of their own.  Measured on whole
        // steps, graphs of ten (one launch for both products + finalize launch -> apart + carried sums):
        //   B=256 n=8   47.7 -> 48.8 us (not taken)    B=256 n=10   79.8 -> 80.0 (not taken)
        //   B=512 n=12 126.6 -> 125.9    B=256 n=13 101.6 -> 96.6    B=256 n=16 111.9 -> 104.4
        //   B=256 n=18 127.5 -> 119.0    B=128 n=32 148.6 -> 145.8 (always two product kernels; sums carried)
        const bool wide = proj_bwd_is_wide(n);
        const int hook = tuning_get(kTuneProjApart);
        const bool apart = wide || (hook ? hook == 2 : proj_bwd_products_apart(n));
        if (apart) {
            if (wide) MHC_LAUNCH(launch_dxflat_wide(phi, ws.dPb, ws.BP, dx, nullptr, nullptr, nullptr, B, n, C, st));
            else MHC_LAUNCH(launch_proj_bwd_mfma(x, phi, ws.dPb, ws.dPT, ws.BP, dphi, ws.dphi_part, dx, B, n, C, st, kProjPartDx));
        } else {
            MHC_LAUNCH(launch_proj_bwd_mfma(x, phi, ws.dPb, ws.dPT, ws.BP, dphi, ws.dphi_part, dx, B, n, C, st));
        }
        MHC_LAUNCH(launch_mix_bwd_dx(dy, y_dtype, x, x_dtype, w, w_dtype, f_inject, H_pre, H_post, M,
                                     n, q, ws.s1, ws.cx, ws.dP, DP, nullptr, 0, dx, dx, df, ws.u, ws.dt,
                                     ws.dtpart, spg, B, n, C, st));
        if (apart) {
            const BatchSumArgs sums = make_batch_sums(ws.u, groups, C, f_inject ? nullptr : dw, ws.dtpart, groups,
                                                      D, dbias, dalpha);
            const BatchSumArgs *tail = S == 1 && tuning_get(kTuneSeparateFinalize) != 1 ? &sums : nullptr;
            bool tail_taken = false;
            if (wide) MHC_LAUNCH(launch_dphi_large(x, ws.dPT, ws.BP, S > 1 ? ws.dphi_part : dphi, S, B, n, C, tail, &tail_taken, st));
            else MHC_LAUNCH(launch_proj_bwd_mfma(x, phi, ws.dPb, ws.dPT, ws.BP, dphi, ws.dphi_part, dx, B, n, C, st,
                                                 kProjPartDphi, tail, &tail_taken));
            if (tail_taken) return MHC_OK;
        }
    } else if (gemm_f32_supported(x_dtype, phi_dtype, n, C)) {
        // exact float32 tier, wide projection: both products on the fp32 matrix cores; the projection
        // term of dx is written into dx and completed in place
        MHC_LAUNCH(launch_gemm_f32_dxflat(ws.dP, static_cast<const float *>(phi), static_cast<float *>(dx), B, n, C, st));
        MHC_LAUNCH(launch_mix_bwd_dx(dy, y_dtype, x, x_dtype, w, w_dtype, f_inject, H_pre, H_post, M,
                                     n, q, ws.s1, ws.cx, ws.dP, DP, nullptr, 0, dx, dx, df, ws.u, ws.dt,
                                     ws.dtpart, spg, B, n, C, st));
        MHC_LAUNCH(launch_gemm_f32_dphi(ws.dP, static_cast<const float *>(x), dphi, B, n, C, st));
    } else {
        MHC_LAUNCH(launch_mix_bwd_dx(dy, y_dtype, x, x_dtype, w, w_dtype, f_inject, H_pre, H_post, M,
                                     n, q, ws.s1, ws.cx, ws.dP, DP, phi, phi_dtype, nullptr, dx, df,
                                     ws.u, ws.dt, ws.dtpart, spg, B, n, C, st));
        MHC_LAUNCH(launch_dphi(x, x_dtype, ws.dP, DP, dphi, B, n, C, ws.dphi_part, st));
    }
    MHC_LAUNCH(launch_finalize(ws.u, groups, C, f_inject ? nullptr : dw, ws.dtpart, groups, D, dbias,
                               dalpha, ws.dphi_part, S, (size_t)D * n * C, dphi, st));
    return MHC_OK;
}

int mhc_pack_dynamic_params(const void *phi_pre, const void *phi_post, const void *phi_res, int src_dtype,
                            const float *b_pre, const float *b_post, const float *b_res,
                            const float *alpha_pre, const float *alpha_post, const float *alpha_res,
                            void *phi, int phi_dtype, float *bias, float *alpha, int n, int C, void *stream) {
    if (n < 1 || n > MHC_MAX_N) return MHC_ERR_BAD_N;
    if (C < 1 || C > MHC_MAX_C) return MHC_ERR_BAD_SHAPE;
    if (!phi_pre || !phi_post || !phi_res || !b_pre || !b_post || !b_res || !alpha_pre || !alpha_post ||
        !alpha_res || !phi || !bias || !alpha)
        return MHC_ERR_NULL_POINTER;
    if (!valid_dtype(src_dtype) || !valid_dtype(phi_dtype)) return MHC_ERR_BAD_DTYPE;
    MHC_LAUNCH(launch_pack_params(phi_pre, phi_post, phi_res, src_dtype, b_pre, b_post, b_res, alpha_pre,
                                  alpha_post, alpha_res, phi, phi_dtype, bias, alpha, n, C,
                                  static_cast<hipStream_t>(stream)));
    return MHC_OK;
}

// ===============================================================================================
// static H
// ===============================================================================================
size_t mhc_layer_static_workspace_bytes(int B, int n, int C) {
    if (check_shape(B, n, C, 0) != MHC_OK) return 0;
    const size_t f = carve_sta_fwd(nullptr, B, n, C).bytes;
    const size_t b = carve_sta_bwd(nullptr, B, n, C).bytes;
    return f > b ? f : b;
}

int mhc_layer_fwd(const void *x, int x_dtype, const void *w, int w_dtype,
                  const float *H_pre_logits, const float *H_post_logits,
                  const float *H_res_logits, const void *f_inject, void *y, int y_dtype,
                  float *H_pre, float *H_post, float *M, float *q, int B, int n, int C, int iters,
                  float eps, void *workspace, size_t workspace_bytes, void *stream) {
    if (int s = check_shape(B, n, C, iters)) return s;
    if (!x || !H_pre_logits || !H_post_logits || !H_res_logits || !y) return MHC_ERR_NULL_POINTER;
    if (!f_inject && !w) return MHC_ERR_NULL_POINTER;
    if (!valid_io(x_dtype, y_dtype) || (w && !valid_dtype(w_dtype))) return MHC_ERR_BAD_DTYPE;
    if (!aligned16(x) || !aligned16(y) || (f_inject && !aligned16(f_inject))) return MHC_ERR_MISALIGNED;
    hipStream_t st = static_cast<hipStream_t>(stream);
    if (layer_fwd_fused_supported(n, C, x_dtype)) {
        // one launch; every workgroup derives the shared coefficients itself, none need storing
        MHC_LAUNCH(launch_layer_fwd_fused(x, x_dtype, w, w_dtype, f_inject, y, y_dtype, nullptr, nullptr,
                                          0, 0, nullptr, H_pre_logits, H_post_logits, H_res_logits,
                                          H_pre, H_post, M, nullptr, nullptr, q, nullptr, B, n, C, iters, eps,
                                          st));
        return MHC_OK;
    }
    const StaFwdWs ws = carve_sta_fwd(workspace, B, n, C);
    const bool need_ws = !H_pre || !H_post || !M || !q || n > 8;
    if (need_ws)
        if (int s = ws_check(workspace, workspace_bytes, ws.bytes)) return s;
    float *hp = H_pre ? H_pre : ws.Hpre, *ho = H_post ? H_post : ws.Hpost;
    float *m = M ? M : ws.M, *qq = q ? q : ws.q;
    // n > 8, up to two samples per CU: the coefficient launch runs once per sample, each workgroup with
    // the shared Sinkhorn chain and its sample's aggregate and RMS under it, instead of one workgroup
    // followed by an aggregate launch (forward, cold, B=128 n=32 C=1280: 26 -> 20 us)
    const bool agg = !f_inject && n > 8 && B <= 512 && coef_fwd_aggregates(n, C, x_dtype);
    MHC_LAUNCH(launch_coef_fwd(nullptr, nullptr, 0, 0, nullptr, H_pre_logits, H_post_logits,
                               H_res_logits, hp, ho, m, nullptr, nullptr, agg ? B : 1, n, n * C, iters, eps,
                               x_dtype == kF32, agg ? x : nullptr, agg ? ws.agg : nullptr, agg ? qq : nullptr,
                               nullptr, st));
    MHC_LAUNCH(launch_mix_fwd(x, x_dtype, w, w_dtype, f_inject, y, y_dtype, hp, ho, m, 0, qq,
                              n > 8 ? ws.agg : nullptr, B, n, C, eps, agg, st));
    return MHC_OK;
}

int mhc_layer_bwd(const void *dy, int y_dtype, const void *x, int x_dtype, const void *w,
                  int w_dtype, const float *H_pre_logits, const float *H_post_logits,
                  const float *H_res_logits, const void *f_inject, const float *H_pre,
                  const float *H_post, const float *M, const float *q, void *dx, void *df,
                  float *dw, float *dH_pre, float *dH_post, float *dH_res, int B, int n, int C,
                  int iters, float eps, void *workspace, size_t workspace_bytes, void *stream) {
    if (int s = check_shape(B, n, C, iters)) return s;
    if (!dy || !x || !H_pre_logits || !H_post_logits || !H_res_logits || !H_pre || !H_post || !M ||
        !q || !dx || !dH_pre || !dH_post || !dH_res)
        return MHC_ERR_NULL_POINTER;
    if (!f_inject && (!w || !dw)) return MHC_ERR_NULL_POINTER;
    if (!valid_io(x_dtype, y_dtype) || (w && !valid_dtype(w_dtype))) return MHC_ERR_BAD_DTYPE;
    if (!aligned16(dy) || !aligned16(x) || !aligned16(dx) || (f_inject && !aligned16(f_inject)) ||
        (df && !aligned16(df)))
        return MHC_ERR_MISALIGNED;
    const StaBwdWs ws = carve_sta_bwd(workspace, B, n, C);
    if (int s = ws_check(workspace, workspace_bytes, ws.bytes)) return s;
    hipStream_t st = static_cast<hipStream_t>(stream);
    BwdCoefOut out{nullptr, nullptr, nullptr, ws.s1, ws.red, nullptr, nullptr, 0};
    if (bwd_resident_supported(x_dtype, y_dtype, kBF16, n, C, 0) && tuning_get(kTuneResident) != 1) {
        // bf16 activations, n <= 8: with shared coefficients nothing of dx depends on a batch-wide
        // result, so ONE pass over dy and x (a workgroup keeps its sample's rows in registers) forms
        // the channel sums, the sample's raw coefficient gradients and the complete dx
        MHC_LAUNCH(launch_bwd_resident_static(dy, x, w, w_dtype, f_inject, H_pre, H_post, M, q, out, dx, df, ws.u,
                                              B, n, C, st));
        MHC_LAUNCH(launch_finalize_static(ws.u, B, C, f_inject ? nullptr : dw, ws.red, B, ws.red_sum, H_pre, H_post,
                                          H_res_logits, dH_pre, dH_post, dH_res, n, iters, eps, st));
        return MHC_OK;
    }
    if (n > 16 && x_dtype == kBF16 && y_dtype == kBF16 && C % 8 == 0) {
        // three launches: channel sums (+ the Sinkhorn forward recompute), the per-sample coefficient sums
        // with the complete dx beside them, batch sums + coefficient backward
        // (cold, B=128 n=32 C=1280: 44.7 us -> see profiles/native_bench_all_configs.txt)
        MHC_LAUNCH(launch_mix_bwd_reduce_with_dx_static(dy, x, w, w_dtype, f_inject, H_pre, H_post, M, q, out, ws.raw,
                                                        ws.s1part, dx, df, ws.u, B, n, C, iters, eps, st, H_res_logits,
                                                        ws.sk));
        MHC_LAUNCH(launch_finalize_static(ws.u, B, C, f_inject ? nullptr : dw, ws.red, B, ws.red_sum, H_pre, H_post,
                                          H_res_logits, dH_pre, dH_post, dH_res, n, iters, eps, st, ws.sk));
        return MHC_OK;
    }
    MHC_LAUNCH(launch_mix_bwd_reduce(dy, y_dtype, x, x_dtype, w, w_dtype, f_inject, H_pre, H_post, M,
                                     0, q, nullptr, nullptr, nullptr, nullptr, nullptr, out, n > 8 ? ws.raw : nullptr,
                                     B, n, C, iters, eps, st, H_res_logits, n > 8 ? ws.sk : nullptr));
    // samples per workgroup of the dx kernel: with a large batch a workgroup adds up the dw terms of a
    // few samples itself, so that the batch-sum launch reads fewer rows
    const int hook = tuning_get(kTuneStaticSpg);
    // (measured cold, bf16: B=1280 C=2560 n=4 60.5 -> 58.6 us with four; B=1024 n=8 and small batches lose)
    const int spg = n > 8 ? 1 : (hook > 0 ? hook : (n <= 4 && B >= 1024 ? 4 : 1));
    const int groups = (B + spg - 1) / spg;
    MHC_LAUNCH(launch_mix_bwd_dx(dy, y_dtype, x, x_dtype, w, w_dtype, f_inject, H_pre, H_post, M, 0,
                                 q, ws.s1, nullptr, nullptr, 0, nullptr, 0, nullptr, dx, df, ws.u, nullptr,
                                 nullptr, spg, B, n, C, st));
    // the batch sums (dw = sum_b u, sum_b red) and the coefficient backward on them: one launch for
    // n <= 8, two beyond
    MHC_LAUNCH(launch_finalize_static(ws.u, groups, C, f_inject ? nullptr : dw, ws.red, B, ws.red_sum, H_pre, H_post,
                                      H_res_logits, dH_pre, dH_post, dH_res, n, iters, eps, st, n > 8 ? ws.sk : nullptr));
    return MHC_OK;
}

// ===============================================================================================
// stand-alone operators
// ===============================================================================================
int mhc_sinkhorn_knopp_fwd(const float *inp, float *out, int batch, int rows, int cols, int iters,
                           float eps, void *stream) {
    if (!inp || !out) return MHC_ERR_NULL_POINTER;
    if (batch < 1 || rows < 1 || cols < 1 || rows > 128 || cols > 128 || iters < 0 || iters > 1024)
        return MHC_ERR_BAD_SHAPE;
    MHC_LAUNCH(launch_sinkhorn_plain_fwd(inp, out, batch, rows, cols, iters, eps,
                                         static_cast<hipStream_t>(stream)));
    return MHC_OK;
}

size_t mhc_sinkhorn_knopp_bwd_workspace_bytes(int batch, int rows, int cols, int iters) {
    if (batch < 1 || rows < 1 || cols < 1 || rows > 128 || cols > 128 || iters < 0 || iters > 1024)
        return 0;
    return ((size_t)batch * (iters > 0 ? iters : 1) * 2 * 128 * sizeof(float) + 255) / 256 * 256;
}

int mhc_sinkhorn_knopp_bwd(const float *grad_out, const float *inp, float *d_inp, int batch,
                           int rows, int cols, int iters, float eps, void *workspace,
                           size_t workspace_bytes, void *stream) {
    if (!grad_out || !inp || !d_inp) return MHC_ERR_NULL_POINTER;
    const size_t need = mhc_sinkhorn_knopp_bwd_workspace_bytes(batch, rows, cols, iters);
    if (need == 0) return MHC_ERR_BAD_SHAPE;
    if (int s = ws_check(workspace, workspace_bytes, need)) return s;
    MHC_LAUNCH(launch_sinkhorn_plain_bwd(grad_out, inp, d_inp, batch, rows, cols, iters, eps,
                                         static_cast<float *>(workspace),
                                         static_cast<hipStream_t>(stream)));
    return MHC_OK;
}

int mhc_rmsnorm_fwd(const void *inp, int dtype, const void *w, int w_dtype, void *out, float *rms,
                    int rows, int C, float eps, void *stream) {
    if (!inp || !w || !out) return MHC_ERR_NULL_POINTER;
    if (rows < 1 || C < 1) return MHC_ERR_BAD_SHAPE;
    if (!valid_dtype(dtype) || !valid_dtype(w_dtype)) return MHC_ERR_BAD_DTYPE;
    MHC_LAUNCH(launch_rmsnorm_fwd(inp, dtype, w, w_dtype, out, rms, rows, C, eps,
                                  static_cast<hipStream_t>(stream)));
    return MHC_OK;
}

size_t mhc_rmsnorm_bwd_workspace_bytes(int rows, int C) {
    if (rows < 1 || C < 1) return 0;
    Carver c(nullptr);
    c.floats((size_t)(rows + 3) * C);  // dw terms: a row per input row, or per row slot of the persistent kernel
    c.floats(colsum_workspace_floats(rows + 3, C));
    return c.off;
}

int mhc_rmsnorm_bwd(const void *grad_out, const void *inp, int dtype, const void *w, int w_dtype,
                    const float *rms, void *d_inp, float *d_w, int rows, int C, void *workspace,
                    size_t workspace_bytes, void *stream) {
    if (!grad_out || !inp || !w || !rms || !d_inp || !d_w) return MHC_ERR_NULL_POINTER;
    if (rows < 1 || C < 1) return MHC_ERR_BAD_SHAPE;
    if (!valid_dtype(dtype) || !valid_dtype(w_dtype)) return MHC_ERR_BAD_DTYPE;
    if (int s = ws_check(workspace, workspace_bytes, mhc_rmsnorm_bwd_workspace_bytes(rows, C))) return s;
    Carver c(workspace);
    float *u = c.floats((size_t)(rows + 3) * C);
    float *part = c.floats(colsum_workspace_floats(rows + 3, C));
    hipStream_t st = static_cast<hipStream_t>(stream);
    int u_rows = rows;  // rows of u whose column sums are dw (fewer when the kernel sums its own rows)
    MHC_LAUNCH(launch_rmsnorm_bwd(grad_out, inp, dtype, w, w_dtype, rms, d_inp, u, rows, C, &u_rows, st));
    MHC_LAUNCH(launch_colsum(u, u_rows, C, C, d_w, part, st));
    return MHC_OK;
}

}  // extern "C"

// ===============================================================================================
// Dynamic forward for callers that cannot allocate (HIP graph capture, serving loops, harnesses
// that forbid hipMalloc): the scratch of the split-K projection lives in a device array of this
// library instead of a caller workspace.  Every GPU holds its own copy of the array at its own
// address; the address is looked up once per device and only that pointer is handed to kernels
// (the array's name is a host-side stand-in, not a device address).
// ===============================================================================================
static __device__ __align__(256) unsigned char scratch[MHC_STATIC_SCRATCH_BYTES];

namespace {

constexpr int kMaxDevices = 64;
std::mutex g_scratch_mutex;
void *g_scratch_ptr[kMaxDevices];  // device address of `scratch` per device, nullptr until looked up

int static_scratch_pointer(void **out) {
    int dev = -1;
    if (hipGetDevice(&dev) != hipSuccess || dev < 0 || dev >= kMaxDevices) return MHC_ERR_LAUNCH;
    std::lock_guard<std::mutex> lock(g_scratch_mutex);
    if (!g_scratch_ptr[dev]) {
        void *p = nullptr;
        if (hipGetSymbolAddress(&p, HIP_SYMBOL(scratch)) != hipSuccess || !p) return MHC_ERR_LAUNCH;
        g_scratch_ptr[dev] = p;
    }
    *out = g_scratch_ptr[dev];
    return MHC_OK;
}

}  // namespace

extern "C" {

size_t mhc_static_scratch_capacity(void) { return MHC_STATIC_SCRATCH_BYTES; }

size_t mhc_layer_fwd_dynamic_scratch_bytes(int B, int n, int C) {
    if (check_shape(B, n, C, 0) != MHC_OK) return 0;
    return carve_dyn_fwd(nullptr, B, n, C).bytes;
}

int mhc_static_scratch_init(void) {
    void *p = nullptr;
    return static_scratch_pointer(&p);
}

int mhc_layer_fwd_dynamic_static_scratch(const void *x, int x_dtype, const void *w, int w_dtype,
                                         const void *phi, int phi_dtype, const float *bias,
                                         const float *alpha, const void *f_inject, void *y, int y_dtype,
                                         float *H_pre, float *H_post, float *M, float *P, float *r,
                                         float *q, float *sk_state, int B, int n, int C, int iters, float eps,
                                         void *stream) {
    if (int s = check_shape(B, n, C, iters)) return s;
    // every byte the kernels touch lies below `need`; nothing has to start at zero (the projection
    // writes each partial sum that the coefficient step reads), so the contents left by the last call
    // are simply overwritten
    const size_t need = carve_dyn_fwd(nullptr, B, n, C).bytes;
    if (need > MHC_STATIC_SCRATCH_BYTES) return MHC_ERR_SCRATCH_LIMIT;
    void *ptr = nullptr;
    if (int s = static_scratch_pointer(&ptr)) return s;
    return mhc_layer_fwd_dynamic(x, x_dtype, w, w_dtype, phi, phi_dtype, bias, alpha, f_inject, y, y_dtype,
                                 H_pre, H_post, M, P, r, q, sk_state, B, n, C, iters, eps, ptr,
                                 MHC_STATIC_SCRATCH_BYTES, stream);
}

}  // extern "C"
