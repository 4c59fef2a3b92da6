// Batch sums of the dynamic backward that no kernel can finish by itself: the column sums of the
// virtual matrix [u | dt],
//     u  [rows_u,  C]    -> dw[C]                 (skipped when dw == nullptr)
//     dt [rows_dt, D+3]  -> dbias[D], dalpha[3]
// as a device routine, so that they can run either as blocks of the finalize launch or as a few extra
// workgroups of a large kernel that comes last in the stream anyway.  One block = 64 columns x RG
// row groups; float64 accumulation: dalpha is a sum of B * n^2 terms of mixed sign whose total can be a
// hundred times smaller than the terms, and a float32 running sum loses what the 1e-5 parity tier
// needs.  The terms themselves stay float32.
#pragma once
#include <hip/hip_runtime.h>

namespace mhc {

struct BatchSumArgs {
    const float *u; int rows_u, C; float *dw;
    const float *dt; int rows_dt, D; float *dbias, *dalpha;
    int nblk;  // blocks of 64 columns
};

inline BatchSumArgs make_batch_sums(const float *u, int rows_u, int C, float *dw, const float *dt, int rows_dt,
                                    int D, float *dbias, float *dalpha) {
    const int ncols = (dw ? C : 0) + (dt ? D + 3 : 0);  // dt == nullptr: the u columns only
    return BatchSumArgs{u, rows_u, C, dw, dt, rows_dt, D, dbias, dalpha, (ncols + 63) / 64};
}

// red: RG * (CW + 1) doubles of LDS; called by all CW * RG threads of the workgroup (contains a barrier).
// CW = columns per block: 64, or 32 (still whole 128-byte lines per row) where twice the blocks are
// wanted; a.nblk must count blocks of CW columns.
template <int RG, int CW = 64>
__device__ __forceinline__ void batch_sum_block(const BatchSumArgs &a, int blk, int tid, double *red) {
    const int cl = tid % CW, rg = tid / CW;
    const int col = blk * CW + cl;
    const int ncol_u = a.dw ? a.C : 0;
    const int ncols = ncol_u + (a.dt ? a.D + 3 : 0);
    double acc = 0.0;
    if (col < ncols) {
        const bool is_u = col < ncol_u;
        const float *src = is_u ? a.u + col : a.dt + (col - ncol_u);
        const int ld = is_u ? a.C : a.D + 3;
        const int rows = is_u ? a.rows_u : a.rows_dt;
        double a0 = 0.0, a1 = 0.0, a2 = 0.0, a3 = 0.0;
        int r = rg;
        // many rows (per-sample rows of a large batch): sixteen loads in flight, the round trips decide
        for (; r + 15 * RG < rows; r += 16 * RG) {
            float t[16];
#pragma unroll
            for (int k = 0; k < 16; k++) t[k] = src[(size_t)(r + k * RG) * ld];
#pragma unroll
            for (int k = 0; k < 16; k += 4) {
                a0 += (double)t[k]; a1 += (double)t[k + 1]; a2 += (double)t[k + 2]; a3 += (double)t[k + 3];
            }
        }
        for (; r + 3 * RG < rows; r += 4 * RG) {
            const float t0 = src[(size_t)r * ld], t1 = src[(size_t)(r + RG) * ld];
            const float t2 = src[(size_t)(r + 2 * RG) * ld], t3 = src[(size_t)(r + 3 * RG) * ld];
            a0 += (double)t0; a1 += (double)t1; a2 += (double)t2; a3 += (double)t3;
        }
        for (; r < rows; r += RG) a0 += (double)src[(size_t)r * ld];
        acc = (a0 + a1) + (a2 + a3);
    }
    red[rg * (CW + 1) + cl] = acc;
    __syncthreads();
    if (rg == 0 && col < ncols) {
        double v = 0.0;
#pragma unroll
        for (int i = 0; i < RG; i++) v += red[i * (CW + 1) + cl];
        if (col < ncol_u) a.dw[col] = (float)v;
        else if (col - ncol_u < a.D) a.dbias[col - ncol_u] = (float)v;
        else a.dalpha[col - ncol_u - a.D] = (float)v;
    }
}

}  // namespace mhc
