// Parameter gradients that sum over the batch: dphi = dP^T x_flat (reference ops.py:332-334),
// dbias / dalpha (ops.py:319-325), dw (reference rmsnorm.cuh:282-294, without its atomics) and the
// static-H coefficient backward (reference bindings.cu:372-396).  All sums are order-deterministic:
// per-split partial sums followed by a second pass, no atomics.
#include "launchers.h"
#include "sinkhorn_device.h"

namespace mhc {

// --------------------------------------------------------------------------------------------
// column sums: out[j] = sum_b in[b * ld + j]
// --------------------------------------------------------------------------------------------
__global__ __launch_bounds__(256) void colsum_kernel(const float *__restrict__ in, int rows, int cols,
                                                     int ld, int rows_per_split,
                                                     float *__restrict__ out, float *__restrict__ out2,
                                                     int split_col) {
    const int j = blockIdx.x * 256 + threadIdx.x;
    if (j >= cols) return;
    const int r0 = blockIdx.y * rows_per_split;
    const int r1 = min(rows, r0 + rows_per_split);
    float a0 = 0.f, a1 = 0.f, a2 = 0.f, a3 = 0.f;
    int r = r0;
    for (; r + 3 < r1; r += 4) {
        a0 += in[(size_t)r * ld + j];
        a1 += in[(size_t)(r + 1) * ld + j];
        a2 += in[(size_t)(r + 2) * ld + j];
        a3 += in[(size_t)(r + 3) * ld + j];
    }
    for (; r < r1; r++) a0 += in[(size_t)r * ld + j];
    const float v = (a0 + a1) + (a2 + a3);
    if (gridDim.y > 1) out[(size_t)blockIdx.y * cols + j] = v;   // partial [split][cols]
    else if (j < split_col) out[j] = v;
    else out2[j - split_col] = v;
}

static int colsum_splits(int rows, int cols) {
    const int col_blocks = (cols + 255) / 256;
    int rs = 256 / col_blocks;
    if (rs > rows / 8) rs = rows / 8;
    if (rs > 64) rs = 64;
    if (rs < 1) rs = 1;
    return rs;
}

size_t colsum_workspace_floats(int rows, int cols) {
    const int rs = colsum_splits(rows, cols);
    return rs > 1 ? (size_t)rs * cols : 0;
}

// out2 / split_col: columns >= split_col go to out2[j - split_col] (pass cols and nullptr for none)
static hipError_t colsum2(const float *in, int rows, int cols, int ld, float *out, float *out2,
                          int split_col, float *partial, hipStream_t stream) {
    const int rs = colsum_splits(rows, cols);
    const int cb = (cols + 255) / 256;
    if (rs == 1) {
        colsum_kernel<<<dim3(cb, 1), 256, 0, stream>>>(in, rows, cols, ld, rows, out, out2, split_col);
        return hipGetLastError();
    }
    const int rps = (rows + rs - 1) / rs;
    colsum_kernel<<<dim3(cb, rs), 256, 0, stream>>>(in, rows, cols, ld, rps, partial, nullptr, cols);
    hipError_t e = hipGetLastError();
    if (e != hipSuccess) return e;
    colsum_kernel<<<dim3(cb, 1), 256, 0, stream>>>(partial, rs, cols, cols, rs, out, out2, split_col);
    return hipGetLastError();
}

hipError_t launch_colsum(const float *in, int rows, int cols, int ld, float *out, float *partial,
                         hipStream_t stream) {
    return colsum2(in, rows, cols, ld, out, nullptr, cols, partial, stream);
}

hipError_t launch_colsum_split(const float *in, int rows, int cols, int ld, float *out, float *out2,
                               int split_col, float *partial, hipStream_t stream) {
    return colsum2(in, rows, cols, ld, out, out2, split_col, partial, stream);
}

// --------------------------------------------------------------------------------------------
// dphi, generic path: thread = one column k of x_flat, 32 projection rows per workgroup,
// batch optionally split (partials summed by colsum).
// --------------------------------------------------------------------------------------------
constexpr int kDphiDB = 32;

template <typename TX>
__global__ __launch_bounds__(256) void dphi_generic_kernel(const TX *__restrict__ x,
                                                           const float *__restrict__ dP, int DP,
                                                           float *__restrict__ out, int B, int D,
                                                           int nC, int b_per_split) {
    const int k = blockIdx.x * 256 + threadIdx.x;
    const int d0 = blockIdx.y * kDphiDB;
    const int b0 = blockIdx.z * b_per_split, b1 = min(B, b0 + b_per_split);
    if (k >= nC) return;
    float acc[kDphiDB];
#pragma unroll
    for (int j = 0; j < kDphiDB; j++) acc[j] = 0.f;
    for (int b = b0; b < b1; b++) {
        const float xv = to_f32<TX>(x[(size_t)b * nC + k]);
        const float *dPb = dP + (size_t)b * DP + d0;  // padded rows of dP are zero
#pragma unroll
        for (int j = 0; j < kDphiDB; j++) acc[j] += dPb[j] * xv;
    }
    float *o = out + (size_t)blockIdx.z * D * nC;
#pragma unroll
    for (int j = 0; j < kDphiDB; j++)
        if (d0 + j < D) o[(size_t)(d0 + j) * nC + k] = acc[j];
}

int dphi_batch_splits(int B, int n, int C) {
    const int nC = n * C, D = n * n + 2 * n;
    const int wgs = ((nC + 255) / 256) * ((D + kDphiDB - 1) / kDphiDB);
    int bs = 512 / wgs;
    if (bs > B / 16) bs = B / 16;
    if (bs > 16) bs = 16;
    if (bs < 1) bs = 1;
    return bs;
}

hipError_t launch_dphi(const void *x, int x_dtype, const float *dP, int DP, float *dphi, int B,
                       int n, int C, float *partial, hipStream_t stream) {
    const int nC = n * C, D = n * n + 2 * n;
    const int bs = dphi_batch_splits(B, n, C);
    const int bps = (B + bs - 1) / bs;
    dim3 grid((nC + 255) / 256, (D + kDphiDB - 1) / kDphiDB, bs);
    float *out = bs > 1 ? partial : dphi;
    if (x_dtype == kBF16)
        dphi_generic_kernel<bf16_t><<<grid, 256, 0, stream>>>(static_cast<const bf16_t *>(x), dP, DP, out, B, D, nC, bps);
    else
        dphi_generic_kernel<float><<<grid, 256, 0, stream>>>(static_cast<const float *>(x), dP, DP, out, B, D, nC, bps);
    hipError_t e = hipGetLastError();
    if (e != hipSuccess || bs == 1) return e;
    const int cols = D * nC;
    colsum_kernel<<<dim3((cols + 255) / 256, 1), 256, 0, stream>>>(partial, bs, cols, cols, bs, dphi, nullptr, cols);
    return hipGetLastError();
}


// --------------------------------------------------------------------------------------------
// finalize: every remaining batch reduction of the dynamic backward in ONE launch.
//   blocks [0, nblk_a): 64 columns x 16 row groups of the virtual matrix [u | dt]
//       u  [rows_u,  C]    -> dw[C]
//       dt [rows_dt, D+3]  -> dbias[D], dalpha[3]
//   blocks [nblk_a, ...): 1024 columns each of the dphi batch-split partials [S, D*nC] -> dphi
// --------------------------------------------------------------------------------------------
struct FinalizeArgs {
    BatchSumArgs sums;
    const float *dphi_part; int S; size_t dphi_elems; float *dphi;
};

__global__ __launch_bounds__(1024) void finalize_kernel(FinalizeArgs a) {
    __shared__ double red[16 * 65];
    const int tid = threadIdx.x;
    if ((int)blockIdx.x < a.sums.nblk) {
        batch_sum_block<16>(a.sums, blockIdx.x, tid, red);
        return;
    }
    // dphi partial sums: one float per thread per 1024-column block (coalesced)
    const size_t e = (size_t)(blockIdx.x - a.sums.nblk) * 1024 + tid;
    if (e < a.dphi_elems) {
        // all copies requested together (sixteen per round: one round trip for the usual 8 to 13
        // splits), added in split order
        float v = 0.f;
        for (int s0 = 0; s0 < a.S; s0 += 16) {
            float t[16];
#pragma unroll
            for (int u = 0; u < 16; u++) {
                const int s = s0 + u < a.S ? s0 + u : a.S - 1;
                t[u] = __builtin_nontemporal_load(a.dphi_part + (size_t)s * a.dphi_elems + e);
            }
#pragma unroll
            for (int u = 0; u < 16; u++) v += s0 + u < a.S ? t[u] : 0.f;
        }
        a.dphi[e] = v;
    }
}

hipError_t launch_finalize(const float *u, int rows_u, int C, float *dw, const float *dt, int rows_dt,
                           int D, float *dbias, float *dalpha, const float *dphi_part, int S,
                           size_t dphi_elems, float *dphi, hipStream_t stream) {
    const BatchSumArgs sums = make_batch_sums(u, rows_u, C, dw, dt, rows_dt, D, dbias, dalpha);
    const int nblk_a = sums.nblk;
    const int nblk_b = S > 1 ? (int)((dphi_elems + 1023) / 1024) : 0;
    FinalizeArgs a{sums, dphi_part, S, dphi_elems, dphi};
    finalize_kernel<<<nblk_a + nblk_b, 1024, 0, stream>>>(a);
    return hipGetLastError();
}

// --------------------------------------------------------------------------------------------
// static H: coefficient backward on the batch-summed raw gradients (one wave)
//   red_sum = (dM [n*n] | dHpre [n] | dHpost [n])
// --------------------------------------------------------------------------------------------
template <int NP>
__global__ __launch_bounds__(256) void coef_bwd_static_kernel(const float *__restrict__ red_sum,
                                                              const float *__restrict__ Hpre,
                                                              const float *__restrict__ Hpost,
                                                              const float *__restrict__ H_res_logits,
                                                              float *__restrict__ dH_pre,
                                                              float *__restrict__ dH_post,
                                                              float *__restrict__ dH_res, int n, int T,
                                                              float eps, const float *__restrict__ state) {
    // one workgroup, the matrix spread over the registers of its 256 threads (IEEE divisions: this
    // kernel serves both precision tiers and runs once per backward call).  state: the denominators of
    // the forward iterations as an earlier launch of the same backward call left them (SkWg::save_state);
    // without it the forward is recomputed here
    using SK = SkWg<NP>;
    extern __shared__ __align__(16) float lds[];  // SK::lds_floats(T)
    const int tid = threadIdx.x;
    if (tid < n) {
        const float hp = Hpre[tid], ho = Hpost[tid];
        dH_pre[tid] = red_sum[n * n + tid] * hp * (1.0f - hp);
        dH_post[tid] = red_sum[n * n + n + tid] * ho * (1.0f - 0.5f * ho);
    }
    const int r0 = SK::row(tid), c0 = SK::col0(tid);
    float E[SK::EPL], d[SK::EPL], u, v[SK::EPL];
#pragma unroll
    for (int e = 0; e < SK::EPL; e++) {
        const bool ok = r0 < n && c0 + e < n;
        E[e] = ok ? expf(H_res_logits[r0 * n + c0 + e]) : 0.f;
        d[e] = ok ? red_sum[r0 * n + c0 + e] : 0.f;
    }
    if (state) SK::load_state(state, u, v, T, lds, tid);
    else SK::template forward<true>(E, u, v, n, T, eps, lds, tid);
    SK::template backward<true>(E, d, u, v, T, lds, tid);
#pragma unroll
    for (int e = 0; e < SK::EPL; e++)
        if (r0 < n && c0 + e < n) dH_res[r0 * n + c0 + e] = d[e];  // gradient of the logits
}

// n <= 8: one wave, one element per lane (SkSmall): the chain of an iteration is a dozen dependent
// instructions instead of the LDS exchanges of the workgroup layout (10.7 -> about 4 us per call).
template <int NP>
__global__ __launch_bounds__(64) void coef_bwd_static_small_kernel(const float *__restrict__ red_sum,
                                                                   const float *__restrict__ Hpre,
                                                                   const float *__restrict__ Hpost,
                                                                   const float *__restrict__ H_res_logits,
                                                                   float *__restrict__ dH_pre,
                                                                   float *__restrict__ dH_post,
                                                                   float *__restrict__ dH_res, int n, int T,
                                                                   float eps) {
    using SK = SkSmall<NP>;
    extern __shared__ float sc[];  // SK::scaling_floats(T)
    const int lane = threadIdx.x, g = lane % SK::kGroup;
    const bool first = lane < SK::kGroup;  // a 4 x 4 matrix takes 16 lanes: the other groups compute copies
    if (first && g < n) {
        const float hp = Hpre[g], ho = Hpost[g];
        dH_pre[g] = red_sum[n * n + g] * hp * (1.0f - hp);
        dH_post[g] = red_sum[n * n + n + g] * ho * (1.0f - 0.5f * ho);
    }
    const int r0 = SK::row(g), c0 = SK::col0(g);
    const bool ok = r0 < n && c0 < n;
    float m[1] = {ok ? expf(H_res_logits[r0 * n + c0]) : 0.f};
    float d[1] = {ok ? red_sum[r0 * n + c0] : 0.f};
    SK::template forward<true>(m, g, n, T, eps, sc, lane);
    SK::template backward<true>(d, m, T, sc, lane);
    if (first && ok) dH_res[r0 * n + c0] = d[0];  // gradient of the logits
}

hipError_t launch_coef_bwd_static(const float *red_sum, const float *Hpre, const float *Hpost,
                                  const float *H_res_logits, float *dH_pre, float *dH_post,
                                  float *dH_res, int n, int T, float eps, hipStream_t stream, const float *state) {
    if (n <= 8) {
        if (n <= 4) {
            const size_t smem = sizeof(float) * SkSmall<4>::scaling_floats(T);
            if (hipError_t e = allow_dynamic_lds(&coef_bwd_static_small_kernel<4>, smem); e != hipSuccess) return e;
            coef_bwd_static_small_kernel<4><<<1, 64, smem, stream>>>(red_sum, Hpre, Hpost, H_res_logits, dH_pre, dH_post, dH_res, n, T, eps);
        } else {
            const size_t smem = sizeof(float) * SkSmall<8>::scaling_floats(T);
            if (hipError_t e = allow_dynamic_lds(&coef_bwd_static_small_kernel<8>, smem); e != hipSuccess) return e;
            coef_bwd_static_small_kernel<8><<<1, 64, smem, stream>>>(red_sum, Hpre, Hpost, H_res_logits, dH_pre, dH_post, dH_res, n, T, eps);
        }
    } else if (n <= 16) {
        const size_t smem = sizeof(float) * SkWg<16>::lds_floats(T);
        if (hipError_t e = allow_dynamic_lds(&coef_bwd_static_kernel<16>, smem); e != hipSuccess) return e;
        coef_bwd_static_kernel<16><<<1, 256, smem, stream>>>(red_sum, Hpre, Hpost, H_res_logits, dH_pre, dH_post, dH_res, n, T, eps, state);
    } else {
        const size_t smem = sizeof(float) * SkWg<32>::lds_floats(T);
        if (hipError_t e = allow_dynamic_lds(&coef_bwd_static_kernel<32>, smem); e != hipSuccess) return e;
        coef_bwd_static_kernel<32><<<1, 256, smem, stream>>>(red_sum, Hpre, Hpost, H_res_logits, dH_pre, dH_post, dH_res, n, T, eps, state);
    }
    return hipGetLastError();
}

// n <= 8: the batch sums of the static backward and the coefficient backward on them in ONE launch.
//   blocks [0, nblk_u): dw = column sums of u, 32 columns each (none with an injected f)
//   last block: the D columns of `red` (per-sample raw gradients dM | dHpre | dHpost, row pitch D + 3)
//       summed over the batch in float64 by waves 1 .. 15 while wave 0 recomputes the Sinkhorn forward;
//       wave 0 then runs the sigmoid derivatives and the exact Sinkhorn backward on the sums, which
//       never leave the workgroup.
struct FinalizeStaticArgs {
    BatchSumArgs sums;  // u -> dw only
    const float *red; int rows, n, T; float eps;
    const float *Hpre, *Hpost, *H_res_logits;
    float *dH_pre, *dH_post, *dH_res;
};

template <int NP>
__global__ __launch_bounds__(1024) void finalize_static_kernel(FinalizeStaticArgs a) {
    using SK = SkSmall<NP>;
    __shared__ double red[32 * 33];
    __shared__ float sum_s[128];
    extern __shared__ float sc[];  // SK::scaling_floats(T)
    const int tid = threadIdx.x;
    if ((int)blockIdx.x < a.sums.nblk) {
        batch_sum_block<32, 32>(a.sums, blockIdx.x, tid, red);
        return;
    }
    const int n = a.n, D = n * n + 2 * n, ld = D + 3;
    // Wave 0 recomputes the Sinkhorn forward (the denominators that its backward needs) from the logits,
    // which needs none of the sums, while waves 1 .. 15 sum the columns of `red`.
    const int lane = tid & 63, g = lane % SK::kGroup;
    const bool first = lane < SK::kGroup;  // a 4 x 4 matrix takes 16 lanes: the other groups compute copies
    const int r0 = SK::row(g), c0 = SK::col0(g);
    const bool ok = r0 < n && c0 < n;
    float m[1] = {0.f};
    if (tid < 64) {
        m[0] = ok ? expf(a.H_res_logits[r0 * n + c0]) : 0.f;
        SK::template forward<true>(m, g, n, a.T, a.eps, sc, lane);
    } else {
        // `red` as one flat array: thread t of the 960 takes element t of every pass of RP whole rows, so a
        // pass is one contiguous piece of memory and a thread stays on its column
        const int t = tid - 64, RP = 896 / ld;  // ld <= 83: at least 10 rows per pass
        if (t < RP * ld) {
            const float *src = a.red + t;
            const size_t step = (size_t)RP * ld;
            const int rs = t / ld;
            double a0 = 0.0, a1 = 0.0, a2 = 0.0, a3 = 0.0;
            int r = rs;
            for (; r + 15 * RP < a.rows; r += 16 * RP, src += 16 * step) {  // sixteen loads in flight
                float v[16];
#pragma unroll
                for (int k = 0; k < 16; k++) v[k] = src[k * step];
#pragma unroll
                for (int k = 0; k < 16; k += 4) {
                    a0 += (double)v[k]; a1 += (double)v[k + 1]; a2 += (double)v[k + 2]; a3 += (double)v[k + 3];
                }
            }
            for (; r < a.rows; r += RP, src += step) a0 += (double)*src;
            red[t] = (a0 + a1) + (a2 + a3);  // [row slot][column]
        }
    }
    __syncthreads();
    if (tid >= 64 && tid < 64 + D) {
        const int RP = 896 / ld;
        double v = 0.0;
        for (int i = 0; i < RP; i++) v += red[i * ld + tid - 64];
        sum_s[tid - 64] = (float)v;
    }
    __syncthreads();
    if (tid >= 64) return;  // the chain below is one wave's (no barrier follows)
    if (first && g < n) {
        const float hp = a.Hpre[g], ho = a.Hpost[g];
        a.dH_pre[g] = sum_s[n * n + g] * hp * (1.0f - hp);
        a.dH_post[g] = sum_s[n * n + n + g] * ho * (1.0f - 0.5f * ho);
    }
    float d[1] = {ok ? sum_s[r0 * n + c0] : 0.f};
    SK::template backward<true>(d, m, a.T, sc, lane);
    if (first && ok) a.dH_res[r0 * n + c0] = d[0];  // gradient of the logits
}

// Batch sums + coefficient backward of the static path.  n <= 8: one launch (above); wider matrices: the
// finalize launch writes the sums to red_sum [D + 3] and the workgroup-wide Sinkhorn kernel follows.
hipError_t launch_finalize_static(const float *u, int rows_u, int C, float *dw, const float *red, int rows,
                                  float *red_sum, const float *Hpre, const float *Hpost,
                                  const float *H_res_logits, float *dH_pre, float *dH_post, float *dH_res, int n,
                                  int T, float eps, hipStream_t stream, const float *static_state) {
    const int D = n * n + 2 * n;
    if (n > 8) {
        if (hipError_t e = launch_finalize(u, rows_u, C, dw, red, rows, D, red_sum, red_sum + D, nullptr, 1, 0,
                                           nullptr, stream); e != hipSuccess)
            return e;
        return launch_coef_bwd_static(red_sum, Hpre, Hpost, H_res_logits, dH_pre, dH_post, dH_res, n, T, eps, stream,
                                      static_state);
    }
    FinalizeStaticArgs a{make_batch_sums(u, rows_u, C, dw, nullptr, 0, 0, nullptr, nullptr), red, rows, n, T, eps,
                         Hpre, Hpost, H_res_logits, dH_pre, dH_post, dH_res};
    a.sums.nblk = dw ? (C + 31) / 32 : 0;  // blocks of 32 columns
    if (n <= 4) {
        const size_t smem = sizeof(float) * SkSmall<4>::scaling_floats(T);
        if (hipError_t e = allow_dynamic_lds(&finalize_static_kernel<4>, smem); e != hipSuccess) return e;
        finalize_static_kernel<4><<<a.sums.nblk + 1, 1024, smem, stream>>>(a);
    } else {
        const size_t smem = sizeof(float) * SkSmall<8>::scaling_floats(T);
        if (hipError_t e = allow_dynamic_lds(&finalize_static_kernel<8>, smem); e != hipSuccess) return e;
        finalize_static_kernel<8><<<a.sums.nblk + 1, 1024, smem, stream>>>(a);
    }
    return hipGetLastError();
}

}  // namespace mhc
