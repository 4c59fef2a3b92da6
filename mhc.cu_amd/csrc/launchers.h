// Host-side launch functions of the individual kernels (internal to the library).
// Every function only enqueues work on `stream` and returns hipGetLastError().
#pragma once

#include <hip/hip_runtime.h>
#include <stddef.h>

#include "batch_sums.h"

namespace mhc {

// kF32AsBF16: stored as fp32, consumed as bf16 - the kernels round the values to bf16 (nearest even) as
// they load them and compute as for bf16 storage (MHC_F32_AS_BF16 of the C ABI).
enum DType { kF32 = 0, kBF16 = 1, kF32AsBF16 = 2 };

inline size_t dtype_size(int dt) { return dt == kBF16 ? 2 : 4; }

// Largest Sinkhorn iteration count of the layer entry points for this n: the per-iteration
// denominators of the backward sweep live in LDS (160 KB per CU).
inline int max_layer_sinkhorn_iters(int) { return 256; }

// Dynamic LDS above 64 KB has to be enabled per kernel before the launch.
template <typename K> inline hipError_t allow_dynamic_lds(K kernel, size_t bytes) {
    if (bytes <= 64 * 1024) return hipSuccess;
    return hipFuncSetAttribute(reinterpret_cast<const void *>(kernel),
                               hipFuncAttributeMaxDynamicSharedMemorySize, (int)bytes);
}

// Projection row count padded to whole 32-wide MFMA tiles.
inline int padded_D(int n) { return ((n * n + 2 * n) + 31) / 32 * 32; }

// ---- forward ---------------------------------------------------------------------------------

// Number of K-splits launch_proj_fwd produces for this shape and dtype pair (never more than
// kMaxKSplit, which sizes the workspace).
constexpr int kMaxKSplit = 64;
int proj_fwd_ksplit(int x_dtype, int phi_dtype, int B, int n, int C);

// Ppart[ks][b][d] = sum over K-slab ks of x_flat[b,k] * phi[d,k]   (d < D; padded rows zero)
// ssqpart[ks][b]  = sum over the slab of x_flat[b,k]^2
hipError_t launch_proj_fwd(const void *x, int x_dtype, const void *phi, int phi_dtype, float *Ppart,
                           float *ssqpart, int KS, int B, int n, int C, hipStream_t stream);

// Coefficients from projection partials (dynamic: Ppart != nullptr) or logits (static: B == 1).
hipError_t launch_coef_fwd(const float *Ppart, const float *ssqpart, int KS, int DP,
                           const float *alpha, const float *b_pre, const float *b_post,
                           const float *b_res, float *Hpre, float *Hpost, float *M, float *P,
                           float *r, int B, int n, int nC, int T, float eps, bool precise,
                           const void *x_agg, float *a_ws, float *q, float *sk_state, hipStream_t stream);
// sk_state (dynamic H, optional): [B][T + 1][2][NP] floats, NP = sinkhorn_state_np(n): the row and column
// denominators of every Sinkhorn iteration and, in slot T for n > 8, the final row and column scalings,
// kept for the backward call (which otherwise recomputes the forward iterations to get them).
inline int sinkhorn_state_np(int n) { return n <= 4 ? 4 : (n <= 8 ? 8 : (n <= 16 ? 16 : 32)); }
// x_agg != nullptr (only where coef_fwd_aggregates() holds): the launch also writes the stream
// aggregate a = Hpre^T x (a_ws, fp32 [B, C]) and its RMS q, which launch_mix_fwd then takes as given
// (have_agg).
bool coef_fwd_aggregates(int n, int C, int x_dtype);
// precise: IEEE divisions in the n > 8 Sinkhorn (fp32 parity tier); otherwise v_rcp_f32

// y = M x + Hpost (x) f, f = RMSNorm(Hpre . x) * w or f_inject.  hstride = n (per-sample
// coefficients) or 0 (shared); the M stride is hstride * n.
hipError_t launch_mix_fwd(const void *x, int x_dtype, const void *w, int w_dtype,
                          const void *f_inject, void *y, int y_dtype, const float *Hpre,
                          const float *Hpost, const float *M, int hstride, float *q, float *a_ws,
                          int B, int n, int C, float eps, bool have_agg, hipStream_t stream);
// a_ws: scratch of B * C floats, needed (with q) by the matrix-core path, see mix_fwd_large_supported
bool mix_fwd_large_supported(int n, int C, int x_dtype);

// Fused coefficients + mix for n <= 8 when the sample's tile fits in registers
// (layer_fwd_fused_supported).  Ppart == nullptr selects static H (logits in b_pre/b_post/b_res,
// outputs Hpre/Hpost/M shared and optional).
bool layer_fwd_fused_supported(int n, int C, int x_dtype);
hipError_t launch_layer_fwd_fused(const void *x, int x_dtype, const void *w, int w_dtype,
                                  const void *f_inject, void *y, int y_dtype, const float *Ppart,
                                  const float *ssqpart, int KS, int DP, const float *alpha,
                                  const float *b_pre, const float *b_post, const float *b_res,
                                  float *Hpre, float *Hpost, float *M, float *P, float *r, float *q,
                                  float *sk_state, int B, int n, int C, int T, float eps, hipStream_t stream);

// Whole dynamic-H forward in one launch (bf16 x and phi, n <= 4, n*C % 64 == 0): projection,
// coefficients and mix with the samples' rows resident in LDS.  bias = [pre | post | res].
bool layer_fwd_onepass_supported(int x_dtype, int phi_dtype, int B, int n, int C);
hipError_t launch_layer_fwd_onepass(const void *x, const void *w, int w_dtype, const void *f_inject, void *y,
                                    int y_dtype, const void *phi, const float *alpha, const float *bias,
                                    float *Hpre, float *Hpost, float *M, float *P, float *r, float *q,
                                    float *sk_state, int B, int n, int C, int T, float eps, hipStream_t stream);

// fp32 matrix-core GEMMs of the exact float32 tier (wide projections): see gemm_f32.hip.
bool gemm_f32_supported(int x_dtype, int phi_dtype, int n, int C);
int gemm_f32_proj_ksplit(int B, int n, int C, int max_splits);
hipError_t launch_gemm_f32_proj(const float *x, const float *phi, float *Ppart, float *ssqpart, int KS,
                                int B, int n, int C, hipStream_t stream);
hipError_t launch_gemm_f32_dphi(const float *dP, const float *x, float *dphi, int B, int n, int C,
                                hipStream_t stream);
hipError_t launch_gemm_f32_dxflat(const float *dP, const float *phi, float *dxflat, int B, int n, int C,
                                  hipStream_t stream);

// ---- backward --------------------------------------------------------------------------------

struct BwdCoefOut {
    float *dt;    // [B, D+3] dL/dlogits per sample, then sum_d dt_d p_d per alpha group (dynamic only)
    float *dP;    // [B, DP]  dL/d(raw dot product) = dt * alpha_g / r, zero padded (dynamic only)
    float *cx;    // [B]      sum_d dt_d alpha_g p_d / (nC r^2)                    (dynamic only)
    float *s1;    // [B]      sum_c df_c w_c a_c
    float *red;   // [B, n*n + 2n + 3] raw per-sample (dM | dHpre | dHpost | 3 unused)   (static only)
    unsigned short *dPb;  // BP * DP bf16, dP in MFMA fragment order (frag_dpb), or nullptr
    unsigned short *dPT;  // 2 planes of DP * BP bf16, dP^T in fragment order (frag_dpt): value, remainder
    int BP;               // row pitch of dPT, a multiple of 32 that is >= B
};

// Per-sample reductions over c (dM, dHpost, dHpre, s1) and, for dynamic H, the coefficient
// backward (activation derivatives + exact Sinkhorn backward) in the same launch.
hipError_t launch_mix_bwd_reduce(const void *dy, int y_dtype, const void *x, int x_dtype,
                                 const void *w, int w_dtype, const void *f_inject,
                                 const float *Hpre, const float *Hpost, const float *M, int hstride,
                                 const float *q, const float *P, const float *r, const float *alpha,
                                 const float *b_res, const float *sk_state, BwdCoefOut out, float *raw, int B,
                                 int n, int C, int T, float eps, hipStream_t stream,
                                 const float *static_logits = nullptr, float *static_state = nullptr);
// static_logits / static_state (optional, static H, n > 8): the channel-sum launch also recomputes the
// Sinkhorn forward of the shared logits and leaves its denominators in static_state ((2 T + 2) * 32 floats)
// for launch_finalize_static.
// raw (optional, dynamic H, n <= 8): scratch of B * bwd_reduce_parts() * (NP*NP + 3*NP + 1) floats;
// when given, the channel sums and the coefficient backward run as two launches.
int bwd_reduce_parts(int B, int n, int C);
size_t bwd_reduce_raw_floats(int B, int n, int C);  // size of `raw` (required for n > 8)
// n > 16, dynamic H, bf16 dy and x: the same two launches, the second also holding the workgroups of
// the matrix-core dx kernel in the form that needs no result of the coefficient backward
// (dxp = M^T dy + Hpre (x) da into `dxp`, fp32 [B][n][C]; df or the dw rows u); they run beside the
// coefficient workgroups, which are one per sample.  s1part: B * bwd_reduce_parts() floats of scratch.
hipError_t launch_mix_bwd_reduce_with_dx(const void *dy, const void *x, const void *w, int w_dtype, const void *f_inject,
                                         const float *Hpre, const float *Hpost, const float *M, int hstride,
                                         const float *q, const float *P, const float *r, const float *alpha,
                                         const float *b_res, const float *sk_state, BwdCoefOut out, float *raw,
                                         float *s1part, float *dxp, void *df, float *u, int B, int n, int C, int T,
                                         float eps, hipStream_t stream);
// Static H, n > 16, bf16: the dx workgroups beside the coefficient launch write the final dx.
hipError_t launch_mix_bwd_reduce_with_dx_static(const void *dy, const void *x, const void *w, int w_dtype,
                                                const void *f_inject, const float *Hpre, const float *Hpost,
                                                const float *M, const float *q, BwdCoefOut out, float *raw,
                                                float *s1part, void *dx, void *df, float *u, int B, int n, int C,
                                                int T, float eps, hipStream_t stream, const float *static_logits,
                                                float *static_state);

// dx = M^T dy + Hpre (x) da - cx * x  [+ dP phi when phi != nullptr] [+ dx_in when != nullptr;
// may alias dx], df, and u = df * a / q (the per-sample summand of dw).
hipError_t launch_mix_bwd_dx(const void *dy, int y_dtype, const void *x, int x_dtype, const void *w,
                             int w_dtype, const void *f_inject, const float *Hpre,
                             const float *Hpost, const float *M, int hstride, const float *q,
                             const float *s1, const float *cx, const float *dP, int DP,
                             const void *phi, int phi_dtype, const void *dx_in, void *dx, void *df,
                             float *u, const float *dt, float *dtpart, int spg, int B, int n, int C,
                             hipStream_t stream);

// Slab kernel for n <= 4 in the bf16 tier: dx (complete), df, and the batch-split partial sums of
// dphi [S][D][nC], dw [S][C] and dt [S][D+3] in one pass over dy and x.  With S == 1 pass the final
// dphi as dphi_part.
bool bwd_slab_supported(int x_dtype, int y_dtype, int phi_dtype, int n, int C);
int bwd_slab_batch_splits(int B, int n, int C);
hipError_t launch_bwd_slab(const void *dy, int y_dtype, const void *x, const void *w, int w_dtype,
                           const void *f_inject, const void *phi, const float *Hpre,
                           const float *Hpost, const float *M, const float *q, const float *s1,
                           const float *cx, const void *dPb, const void *dPT, int BP, const float *dt,
                           void *dx, void *df, float *dphi_part, float *dw_part, float *dt_part, int S,
                           int B, int n, int C, hipStream_t stream);

// Samples per workgroup of launch_mix_bwd_dx and the resulting row count of u / dtpart.
int bwd_dx_samples_per_group(int B, int n);

// One launch for all remaining batch sums: u [rows_u, C] -> dw (skipped when dw == nullptr),
// dt [rows_dt, D+3] -> dbias, dalpha, and (S > 1) dphi_part [S, dphi_elems] -> dphi.
hipError_t launch_finalize(const float *u, int rows_u, int C, float *dw, const float *dt, int rows_dt,
                           int D, float *dbias, float *dalpha, const float *dphi_part, int S,
                           size_t dphi_elems, float *dphi, hipStream_t stream);

// Matrix-core projection backward (x and phi bf16, C % 8 == 0): dphi = dP^T x_flat and
// dxflat = dP phi (bf16 [B, nC]) in one pass over x and phi.  With S = proj_bwd_batch_splits() > 1
// the S partial copies land in dphi_part and the caller's finalize launch sums them.
bool proj_bwd_mfma_supported(int x_dtype, int phi_dtype, int C);
int proj_bwd_batch_splits(int B, int n, int C);
// part: both products in one launch, or one of them (they share no operand but dP and no output, so a
// caller may launch them apart, e.g. around the dx kernel that consumes dxflat).  `tail` (optional,
// with kProjPartDphi): batch sums that a few extra workgroups of the dphi launch compute beside the
// product; they must depend on nothing that is still running.  *tail_taken tells whether the launch
// had room for them (if not, the caller's finalize launch does them).
enum ProjBwdPart { kProjPartBoth = 0, kProjPartDphi = 1, kProjPartDx = 2 };
hipError_t launch_proj_bwd_mfma(const void *x, const void *phi, const void *dPb, const void *dPT,
                                int BP, float *dphi, float *dphi_part, void *dxflat, int B, int n,
                                int C, hipStream_t stream, int part = kProjPartBoth,
                                const BatchSumArgs *tail = nullptr, bool *tail_taken = nullptr);

// Sample-resident first launch of the n <= 8 bf16 backward: channel sums, coefficient backward (all
// outputs of launch_mix_bwd_reduce) and dxp = M^T dy + Hpre (x) da from ONE pass over dy and x, one
// workgroup per sample; u [B, C] = the samples' summands of dw, df with an injected f.
bool bwd_resident_supported(int x_dtype, int y_dtype, int phi_dtype, int n, int C, int T);
hipError_t launch_bwd_resident(const void *dy, const void *x, int x_dtype, const void *w, int w_dtype, const void *f_inject,
                               const float *Hpre, const float *Hpost, const float *M, const float *q,
                               const float *P, const float *r, const float *alpha, const float *b_res,
                               const float *sk_state, BwdCoefOut out, void *dxp, void *df, float *u, int B, int n,
                               int C, int T, float eps, hipStream_t stream);
// Static H (bf16 dy and x, bwd_resident_supported with any T): the complete dx from that one pass, u, and
// per sample out.red [B, D+3] = raw (dM | dHpre | dHpost) and out.s1.
hipError_t launch_bwd_resident_static(const void *dy, const void *x, const void *w, int w_dtype, const void *f_inject,
                                      const float *Hpre, const float *Hpost, const float *M, const float *q,
                                      BwdCoefOut out, void *dx, void *df, float *u, int B, int n, int C,
                                      hipStream_t stream);
// Second and last launch of that backward (D <= 96): a column slab for all samples per workgroup;
// dphi = dP^T x_flat without batch split, dx completed in place (dx = dxp + dP phi - cx x), and `tail`
// (dw, dbias, dalpha) summed by extra workgroups when the grid has room (*tail_taken).
bool proj_bwd_addx_supported(int n);
hipError_t launch_proj_bwd_addx(const void *x, int x_dtype, const void *phi, const void *dPb, const void *dPT, int BP,
                                const float *cx, float *dphi, void *dx, int B, int n, int C, const BatchSumArgs *tail,
                                bool *tail_taken, hipStream_t stream);
// n <= 18: whether the two products are faster apart (measured: from D > 128 on)
bool proj_bwd_products_apart(int n);
// Wide projections (more than 12 row tiles of 32, n > 18) always run the two products as two GEMM
// kernels, launched through the two functions below; tail as above.
bool proj_bwd_is_wide(int n);
// x, cx, dx_part: all nullptr, or the inputs of the completion dxflat = dx_part + dP phi - cx x
// (dx_part: fp32 [B][nC], the part of dx that an earlier launch left), rounded once.
hipError_t launch_dxflat_wide(const void *phi, const void *dPb, int BP, void *dxflat, const void *x, const float *cx,
                              const float *dx_part, int B, int n, int C, hipStream_t stream);
hipError_t launch_dphi_large(const void *x, const void *dPT, int BP, float *dphi_out, int S, int B, int n,
                             int C, const BatchSumArgs *tail, bool *tail_taken, hipStream_t stream);

// dphi[d, k] = sum_b dP[b, d] * x_flat[b, k].  `partial` holds dphi_batch_splits() copies of
// dphi when that is > 1.
int dphi_batch_splits(int B, int n, int C);
hipError_t launch_dphi(const void *x, int x_dtype, const float *dP, int DP, float *dphi, int B,
                       int n, int C, float *partial, hipStream_t stream);

// out[j] = sum_b in[b * ld + j] for j < cols  (deterministic two-level sum through `partial`,
// colsum_workspace_floats() floats).  The _split form sends columns >= split_col to out2.
size_t colsum_workspace_floats(int rows, int cols);
hipError_t launch_colsum(const float *in, int rows, int cols, int ld, float *out, float *partial,
                         hipStream_t stream);
hipError_t launch_colsum_split(const float *in, int rows, int cols, int ld, float *out, float *out2,
                               int split_col, float *partial, hipStream_t stream);

// Static H: coefficient backward on the sample-summed raw gradients.
hipError_t launch_coef_bwd_static(const float *red_sum, const float *Hpre, const float *Hpost,
                                  const float *H_res_logits, float *dH_pre, float *dH_post,
                                  float *dH_res, int n, int T, float eps, hipStream_t stream, const float *state = nullptr);
hipError_t launch_finalize_static(const float *u, int rows_u, int C, float *dw, const float *red, int rows,
                                  float *red_sum, const float *Hpre, const float *Hpost,
                                  const float *H_res_logits, float *dH_pre, float *dH_post, float *dH_res, int n,
                                  int T, float eps, hipStream_t stream, const float *static_state = nullptr);

// phi [D, nC] (out_dtype) = rows [pre | post | res] of the three parameter matrices (src_dtype),
// bias [D] and alpha [3] likewise, in one launch.
hipError_t launch_pack_params(const void *phi_pre, const void *phi_post, const void *phi_res, int src_dtype,
                              const float *b_pre, const float *b_post, const float *b_res,
                              const float *alpha_pre, const float *alpha_post, const float *alpha_res,
                              void *phi_out, int out_dtype, float *bias, float *alpha, int n, int C,
                              hipStream_t stream);

// ---- stand-alone operators -------------------------------------------------------------------
hipError_t launch_sinkhorn_plain_fwd(const float *inp, float *out, int batch, int rows, int cols,
                                     int T, float eps, hipStream_t stream);
hipError_t launch_sinkhorn_plain_bwd(const float *grad, const float *inp, float *d_inp, int batch,
                                     int rows, int cols, int T, float eps, float *scal,
                                     hipStream_t stream);
hipError_t launch_rmsnorm_fwd(const void *inp, int dtype, const void *w, int w_dtype, void *out,
                              float *rms, int rows, int C, float eps, hipStream_t stream);
hipError_t launch_rmsnorm_bwd(const void *grad, const void *inp, int dtype, const void *w,
                              int w_dtype, const float *rms, void *d_inp, float *u, int rows, int C,
                              int *u_rows, hipStream_t stream);  // u: (rows + 3) * C floats

}  // namespace mhc
