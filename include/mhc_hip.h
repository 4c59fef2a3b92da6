/*
 * mhc_hip.h - C ABI of the MI355X (gfx950) mHC layer library, libmhc_hip.so.
 *
 * Plain pointers and sizes only.  Every pointer is a DEVICE pointer unless stated otherwise;
 * every call only enqueues work on `stream` (a hipStream_t passed as void*, NULL = the
 * default stream) and returns a status immediately.  The library keeps no global mutable
 * state, never allocates, never synchronises, never prints and never exits: the caller owns
 * all memory, including the scratch `workspace` (size from the *_workspace_bytes queries,
 * 256-byte aligned).  (One documented exception at the end of this header: the entry point
 * that takes no workspace uses a device array owned by the library and remembers its address.)  Calls are re-entrant across streams as long as each in-flight call has
 * its own workspace.
 *
 * Each entry point names the interface of the reference (AndreSlavescu/mHC.cu) that it
 * replaces; paths are relative to the reference tree.
 *
 * Tensor layouts (row-major, contiguous):
 *   x, y, dy, dx      [B, n, C]     activations, dtype MHC_F32 or MHC_BF16
 *   f, df             [B, C]        same dtype as x
 *   w (rmsnorm)       [C]           MHC_F32 or MHC_BF16
 *   phi, dphi         [D, nC]       D = n*n + 2n, rows [pre(n) | post(n) | res(n*n, i*n+j)];
 *                                   phi MHC_F32 or MHC_BF16, dphi always fp32
 *   bias, dbias       [D]   fp32    same row order (b_pre | b_post | b_res)
 *   alpha, dalpha     [3]   fp32    (alpha_pre, alpha_post, alpha_res), read on the device
 *   H_pre, H_post     [B, n] fp32   activated coefficients (static H: [n])
 *   M                 [B, n, n] fp32 Sinkhorn-normalised mixing matrix (static H: [n, n])
 *   P                 [B, D] fp32   rows of RMSNorm(x_flat) @ phi^T (before alpha and bias)
 *   r, q              [B]   fp32    r = rms of x_flat, q = rms of the aggregated stream
 *   sk_state          [B, iters + 1, 2, NP] fp32  row and column denominators of every Sinkhorn
 *                                   iteration, then one slot the library keeps for itself (NP = n rounded
 *                                   up to 4, 8, 16 or 32); optional, see below
 */
#ifndef MHC_HIP_H
#define MHC_HIP_H

#include <stddef.h>

#ifdef __cplusplus
extern "C" {
#endif

#if defined(__GNUC__)
#define MHC_API __attribute__((visibility("default")))
#else
#define MHC_API
#endif

#define MHC_ABI_VERSION 2
#define MHC_MAX_N 32
#define MHC_MAX_C 32768 /* largest hidden size C of the layer entry points (a [C] float row is kept in LDS) */

/*
 * MHC_F32_AS_BF16: fp32 storage that the kernels consume as bf16 - every kernel rounds the values to
 * bf16 (nearest even) in registers as it loads them and then computes exactly as for MHC_BF16, so no
 * cast pass over the tensor is needed.  This is the reference's default contract (float32
 * activations in and out around a bf16 kernel path: src/python/mhc/ops.py:129,404,
 * src/python/bindings.cu:280,421-423,462).  Accepted as x_dtype by mhc_layer_fwd_dynamic and
 * mhc_layer_bwd_dynamic only, with y_dtype = MHC_F32 (y, dy and dx are then fp32; an injected f and df
 * are fp32 like x), phi in bf16, and only for the shapes mhc_layer_dynamic_accepts_f32_as_bf16()
 * reports; MHC_ERR_BAD_DTYPE otherwise.
 */
enum mhc_dtype { MHC_F32 = 0, MHC_BF16 = 1, MHC_F32_AS_BF16 = 2 };

enum mhc_status {
    MHC_OK = 0,
    MHC_ERR_NULL_POINTER = 1,   /* a required pointer is NULL */
    MHC_ERR_BAD_N = 2,          /* expansion rate outside 1..MHC_MAX_N */
    MHC_ERR_BAD_SHAPE = 3,      /* B, C or iters not positive / too large (C <= MHC_MAX_C, B * n * C <= 2^40) */
    MHC_ERR_BAD_DTYPE = 4,      /* unknown or unsupported dtype combination */
    MHC_ERR_MISALIGNED = 5,     /* a tensor base pointer is not 16-byte aligned */
    MHC_ERR_WORKSPACE = 6,      /* workspace NULL, misaligned or too small */
    MHC_ERR_LAUNCH = 7,         /* the HIP runtime refused a kernel launch */
    MHC_ERR_SCRATCH_LIMIT = 8   /* the shape needs more than MHC_STATIC_SCRATCH_BYTES of scratch */
};

/* Version of this header the library was built from (== MHC_ABI_VERSION). */
MHC_API int mhc_abi_version(void);

/* Static, NUL-terminated description of a status code (host pointer). */
MHC_API const char *mhc_status_string(int status);

/*
 * Largest `iters` the layer entry points below accept for expansion rate n (0 for an invalid n):
 * 256 for every n in 1..32.  The exact Sinkhorn backward keeps the scalings of every iteration in
 * LDS, which bounds the count; its float32 round-off does not grow with it (about 2e-7 relative to
 * float64 on the bias gradients from 20 to 256 iterations).  The reference's interface states no bound
 * (sinkhorn_iters of mhc.MHCLayer, src/python/mhc/layer.py:21-29, default 20).
 * The stand-alone mhc_sinkhorn_knopp_* take up to 1024 iterations for any shape.
 */
MHC_API int mhc_max_sinkhorn_iters(int n);

/*
 * 1 when the two dynamic-H entry points below take x_dtype = MHC_F32_AS_BF16 for this shape (the
 * kernels that load fp32 storage directly serve n <= 8, C % 8 == 0, C <= 2560 and up to 32 Sinkhorn
 * iterations, at every batch size), else 0: the caller then rounds x to bf16 itself, as the reference
 * does (src/python/bindings.cu:421-423).
 */
MHC_API int mhc_layer_dynamic_accepts_f32_as_bf16(int B, int n, int C, int iters);

/* ------------------------------------------------------------------------------------------
 * Dynamic-H layer.  Replaces mhc_cuda.mhc_layer_fwd_dynamic / mhc_layer_bwd_dynamic
 * (src/python/bindings.cu:405-481, :483-542) together with the part of the backward that the
 * reference runs as torch code (src/python/mhc/ops.py:276-361).
 * ---------------------------------------------------------------------------------------- */

/* Scratch bytes needed by one dynamic forward or backward call of this shape. */
MHC_API size_t mhc_layer_dynamic_workspace_bytes(int B, int n, int C);

/* Floats of the optional sk_state tensor of the two calls below (0 for invalid arguments). */
MHC_API size_t mhc_layer_sinkhorn_state_floats(int B, int n, int iters);

/*
 * y = M_b x_b + H_post_b (x) f_b with per-sample coefficients computed from x.
 * f_inject == NULL: f = RMSNorm(sum_i H_pre[b,i] x[b,i,:]) * w  (the layer).
 * f_inject != NULL: f is that [B, C] tensor (kernel-level view; w is ignored, may be NULL).
 * H_pre, H_post, M, P, r, q are outputs kept for the backward call; all six are required.
 * sk_state (may be NULL) receives the Sinkhorn denominators of every iteration: handed to the
 * backward call it saves that call the forward recompute of the iterations (the reference's backward
 * kernel re-runs the forward as well, src/csrc/kernels/sinkhorn_knopp.cuh:587-690).
 */
MHC_API int mhc_layer_fwd_dynamic(const void *x, int x_dtype, const void *w, int w_dtype,
                          const void *phi, int phi_dtype, const float *bias, const float *alpha,
                          const void *f_inject, void *y, int y_dtype, float *H_pre, float *H_post,
                          float *M, float *P, float *r, float *q, float *sk_state, int B, int n, int C,
                          int iters, float eps, void *workspace, size_t workspace_bytes, void *stream);

/*
 * Gradients of the call above for upstream gradient dy (dtype y_dtype).
 * dx has x's dtype.  df (x's dtype) is written only when f_inject != NULL and df != NULL;
 * dw [C] fp32 is written only when f_inject == NULL.  dphi [D, nC], dbias [D], dalpha [3] fp32.
 * Every output is fully overwritten (no pre-zeroing needed); sums are order-deterministic.
 * sk_state: the tensor written by the forward call, or NULL (the iterations are then recomputed).
 */
MHC_API int mhc_layer_bwd_dynamic(const void *dy, int y_dtype, const void *x, int x_dtype, const void *w,
                          int w_dtype, const void *phi, int phi_dtype, const float *bias,
                          const float *alpha, const void *f_inject, const float *H_pre,
                          const float *H_post, const float *M, const float *P, const float *r,
                          const float *q, const float *sk_state, void *dx, void *df, float *dw, float *dphi,
                          float *dbias, float *dalpha, int B, int n, int C, int iters, float eps,
                          void *workspace, size_t workspace_bytes, void *stream);

/*
 * Gathers the parameters as mhc.MHCLayer stores them (src/python/mhc/layer.py:44-54: phi_pre,
 * phi_post [n, nC], phi_res [n*n, nC] in src_dtype; b_pre, b_post [n], b_res [n, n] fp32; the three
 * alpha scalars, fp32, on the device) into phi [D, nC] (phi_dtype), bias [D] and alpha [3] as the two
 * calls above take them, in one launch.  Replaces the torch.cat(...).bfloat16() and the three
 * .item() host synchronisations of every reference forward call (src/python/mhc/ops.py:172-188).
 */
MHC_API int mhc_pack_dynamic_params(const void *phi_pre, const void *phi_post, const void *phi_res, int src_dtype,
                            const float *b_pre, const float *b_post, const float *b_res,
                            const float *alpha_pre, const float *alpha_post, const float *alpha_res,
                            void *phi, int phi_dtype, float *bias, float *alpha, int n, int C, void *stream);

/*
 * mhc_layer_fwd_dynamic for callers that cannot allocate device memory or pass a workspace: code
 * under HIP graph capture, tight serving loops, harnesses that forbid hipMalloc.  It has no
 * counterpart in the reference.  Same arguments and results as mhc_layer_fwd_dynamic minus the
 * workspace: the scratch is a device array of MHC_STATIC_SCRATCH_BYTES inside the library (held by
 * every GPU the library runs on until the process ends).  The call allocates nothing.  Shapes whose
 * scratch need (mhc_layer_fwd_dynamic_scratch_bytes) exceeds the array return
 * MHC_ERR_SCRATCH_LIMIT before any launch.  All calls on one GPU share that GPU's array: calls that
 * overlap on one GPU (different streams or threads) race; order them on one stream.
 * mhc_static_scratch_init looks up the array's address for the current device (the first call on a
 * device does the same); call it once per device before capturing a graph.
 */
#define MHC_STATIC_SCRATCH_BYTES (32u << 20)
MHC_API size_t mhc_static_scratch_capacity(void);
MHC_API size_t mhc_layer_fwd_dynamic_scratch_bytes(int B, int n, int C);
MHC_API int mhc_static_scratch_init(void);
MHC_API int mhc_layer_fwd_dynamic_static_scratch(const void *x, int x_dtype, const void *w, int w_dtype,
                                         const void *phi, int phi_dtype, const float *bias,
                                         const float *alpha, const void *f_inject, void *y, int y_dtype,
                                         float *H_pre, float *H_post, float *M, float *P, float *r,
                                         float *q, float *sk_state, int B, int n, int C, int iters, float eps,
                                         void *stream);

/* ------------------------------------------------------------------------------------------
 * Static-H layer.  Replaces mhc_cuda.mhc_layer_fwd / mhc_layer_fwd_inference / mhc_layer_bwd
 * (src/python/bindings.cu:264-328, :221-262, :330-401).
 * ---------------------------------------------------------------------------------------- */

MHC_API size_t mhc_layer_static_workspace_bytes(int B, int n, int C);

/*
 * H_pre_logits, H_post_logits [n], H_res_logits [n, n] fp32 are the raw parameters.
 * Outputs H_pre, H_post [n], M [n, n] (activated) and q [B] may each be NULL (inference):
 * they are then kept in the workspace only.
 */
MHC_API int mhc_layer_fwd(const void *x, int x_dtype, const void *w, int w_dtype,
                  const float *H_pre_logits, const float *H_post_logits,
                  const float *H_res_logits, const void *f_inject, void *y, int y_dtype,
                  float *H_pre, float *H_post, float *M, float *q, int B, int n, int C,
                  int iters, float eps, void *workspace, size_t workspace_bytes, void *stream);

/* dH_pre, dH_post [n], dH_res [n, n] fp32 are gradients w.r.t. the raw logits. */
MHC_API int mhc_layer_bwd(const void *dy, int y_dtype, const void *x, int x_dtype, const void *w,
                  int w_dtype, const float *H_pre_logits, const float *H_post_logits,
                  const float *H_res_logits, const void *f_inject, const float *H_pre,
                  const float *H_post, const float *M, const float *q, void *dx, void *df,
                  float *dw, float *dH_pre, float *dH_post, float *dH_res, int B, int n, int C,
                  int iters, float eps, void *workspace, size_t workspace_bytes, void *stream);

/* ------------------------------------------------------------------------------------------
 * Stand-alone operators.  Replace mhc_cuda.sinkhorn_knopp_fwd / _bwd and rmsnorm_fwd / _bwd
 * (src/python/bindings.cu:115-164).
 * ---------------------------------------------------------------------------------------- */

/*
 * `batch` independent rows x cols fp32 matrices (rows, cols <= 128).  No exp; a row / column
 * is divided by its sum only when the sum exceeds eps
 * (src/csrc/tests/test_sinkhorn_knopp.cu:16-47).
 */
MHC_API int mhc_sinkhorn_knopp_fwd(const float *inp, float *out, int batch, int rows, int cols, int iters,
                           float eps, void *stream);

/* Exact gradient of the call above w.r.t. inp (recomputes the iterates from inp).  float32 round-off
 * relative to float64 grows by about 1e-7 per iteration (1e-5 at 100, 1e-4 at the limit of 1024). */
MHC_API int mhc_sinkhorn_knopp_bwd(const float *grad_out, const float *inp, float *d_inp, int batch,
                           int rows, int cols, int iters, float eps, void *workspace,
                           size_t workspace_bytes, void *stream);
MHC_API size_t mhc_sinkhorn_knopp_bwd_workspace_bytes(int batch, int rows, int cols, int iters);

/* out = inp / sqrt(mean(inp^2) + eps) * w, row-wise over [rows, C]; rms [rows] fp32 (may be NULL). */
MHC_API int mhc_rmsnorm_fwd(const void *inp, int dtype, const void *w, int w_dtype, void *out,
                    float *rms, int rows, int C, float eps, void *stream);

/* d_inp has inp's dtype; d_w [C] fp32 (deterministic two-pass column sum through workspace). */
MHC_API int mhc_rmsnorm_bwd(const void *grad_out, const void *inp, int dtype, const void *w, int w_dtype,
                    const float *rms, void *d_inp, float *d_w, int rows, int C, void *workspace,
                    size_t workspace_bytes, void *stream);
MHC_API size_t mhc_rmsnorm_bwd_workspace_bytes(int rows, int C);

#ifdef __cplusplus
}
#endif
#endif /* MHC_HIP_H */
