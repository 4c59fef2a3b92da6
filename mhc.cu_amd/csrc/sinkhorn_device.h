// Sinkhorn-Knopp on one n x n matrix (n <= 32), forward and exact backward, as device routines.
//
// Semantics (reference: src/python/benchmarks/bench_layer.py:48-53 / :112-117): start from
// E = exp(logits); T times: divide every row by (row sum + eps), then every column by
// (column sum + eps).  The backward is the exact reverse sweep through all T iterations; the
// per-iteration denominators rho_t[r], s_t[c] are kept in LDS during the forward recompute.
//
// Two layouts:
//   SkSmall<NP> (NP = 4, 8): a matrix lives in the registers of 16 consecutive lanes
//       (NP*NP/16 elements per lane); all reductions are DPP moves, no LDS traffic on the
//       forward path.  Four matrices per wave.
//   SkWg<NP>    (NP = 16, 32): one 256-thread workgroup per matrix, everything in registers,
//       iterate kept in scaling form diag(u) E diag(v).
#pragma once

#include "mhc_common.h"

namespace mhc {

// =============================================================================================
// SkSmall
// =============================================================================================
template <int NP> struct SkSmall {
    static_assert(NP == 4 || NP == 8, "SkSmall handles 4x4 and 8x8 tiles");
    static constexpr int EPL = NP * NP / 16;  // elements per lane (contiguous columns of one row)
    static constexpr int LPR = NP / EPL;      // lanes per row
    static constexpr int kGroup = 16;         // lanes per matrix

    __device__ static __forceinline__ int row(int g) { return g / LPR; }
    __device__ static __forceinline__ int col0(int g) { return (g % LPR) * EPL; }

    // sum over the lanes that hold the same row
    __device__ static __forceinline__ float row_allreduce(float v) {
        v += dpp_mov<kDppQuadXor1>(v);
        if constexpr (NP == 4) v += dpp_mov<kDppQuadXor2>(v);
        return v;
    }
    // sum over the lanes that hold the same columns
    __device__ static __forceinline__ float col_allreduce(float v) {
        if constexpr (NP == 8) v += dpp_mov<kDppQuadXor2>(v);
        v += dpp_mov<kDppRowRor4>(v);
        v += dpp_mov<kDppRowRor8>(v);
        return v;
    }

    // m: in = exp(logits) (0 outside n x n), out = final iterate.
    // sc != nullptr: keep, per iteration t and lane, the row denominator, and per element the
    // column denominator, the row-normalised iterate R_t and the iterate after the column step:
    //   sc[(t * kRec + k) * 64 + lane], k = 0: rho | 1..EPL: s | EPL+1..2EPL: R | 2EPL+1..3EPL: Out
    // PRECISE selects IEEE divisions (fp32 parity tier) instead of v_rcp_f32.
    static constexpr int kRec = 1 + 3 * EPL;
    template <bool PRECISE = false>
    __device__ static __forceinline__ void forward(float (&m)[EPL], int g, int n, int T, float eps,
                                                   float *sc, int lane) {
        const bool rv = row(g) < n;
        bool cv[EPL];
#pragma unroll
        for (int e = 0; e < EPL; e++) cv[e] = col0(g) + e < n;
        for (int t = 0; t < T; t++) {
            float rs = 0.f;
#pragma unroll
            for (int e = 0; e < EPL; e++) rs += m[e];
            rs = row_allreduce(rs) + eps;
            rs = rv ? rs : 1.0f;
            const float rinv = PRECISE ? 1.0f / rs : fast_rcp(rs);
            if (sc) sc[(t * kRec) * kWave + lane] = PRECISE ? rs : rinv;  // fast tier keeps 1/rho
#pragma unroll
            for (int e = 0; e < EPL; e++) {
                m[e] = PRECISE ? m[e] / rs : m[e] * rinv;
                float cs = col_allreduce(m[e]) + eps;
                cs = cv[e] ? cs : 1.0f;
                const float cinv = PRECISE ? 0.f : fast_rcp(cs);
                if (sc) {
                    sc[(t * kRec + 1 + e) * kWave + lane] = PRECISE ? cs : cinv;  // fast tier keeps 1/s
                    sc[(t * kRec + 1 + EPL + e) * kWave + lane] = m[e];
                }
                m[e] = PRECISE ? m[e] / cs : m[e] * cinv;
                if (sc) sc[(t * kRec + 1 + 2 * EPL + e) * kWave + lane] = m[e];
            }
        }
    }

    // d: in = dL/dM, out = dL/dE.  sc as written by forward (the saved iterates are used as they
    // were computed, exactly like reverse-mode autodiff of the forward loop).
    template <bool PRECISE = false>
    __device__ static __forceinline__ void backward(float (&d)[EPL], int T, const float *sc, int lane) {
        for (int t = T - 1; t >= 0; t--) {
            const float rs = sc[(t * kRec) * kWave + lane];
            float rdot = 0.f;
            float dR[EPL];
#pragma unroll
            for (int e = 0; e < EPL; e++) {
                const float cs = sc[(t * kRec + 1 + e) * kWave + lane];
                const float R = sc[(t * kRec + 1 + EPL + e) * kWave + lane];
                const float Out = sc[(t * kRec + 1 + 2 * EPL + e) * kWave + lane];
                const float cdot = col_allreduce(d[e] * Out);
                dR[e] = PRECISE ? (d[e] - cdot) / cs : (d[e] - cdot) * cs;  // fast tier: cs holds 1/s
                rdot += dR[e] * R;
            }
            rdot = row_allreduce(rdot);
#pragma unroll
            for (int e = 0; e < EPL; e++) d[e] = PRECISE ? (dR[e] - rdot) / rs : (dR[e] - rdot) * rs;
        }
    }
    __host__ __device__ static constexpr int scaling_floats(int T) { return T * kRec * kWave; }
};

// =============================================================================================
// SkWg: one 256-thread workgroup per matrix, NP = 16 or 32.  Thread t owns EPL consecutive
// columns of row t / LPR of E and of the running gradient in registers; the iterate is kept in
// scaling form diag(u) E diag(v) (u replicated over the lanes of a row, v over the rows).  A
// half-step is one cross-lane reduction: rows inside a DPP row, columns inside the wave and then
// across the 4 waves through a double-buffered LDS slot (one barrier per iteration).
// The denominators rho/s of every iteration are kept in LDS for the backward sweep, which unwinds
// the scalings (u *= rho, v *= s) instead of storing iterates.  Every thread of the workgroup must
// call forward/backward.
// =============================================================================================
template <int NP> struct SkWg {
    static_assert(NP == 16 || NP == 32, "SkWg handles 16x16 and 32x32 tiles");
    static constexpr int EPL = NP * NP / 256;  // 1 or 4
    static constexpr int LPR = NP / EPL;       // lanes per row: 16 or 8
    // LDS floats: cw [2][4][NP] | rho [T][NP] | s [T][NP]
    __host__ __device__ static constexpr int lds_floats(int T) { return 8 * NP + 2 * T * NP; }
    __device__ static __forceinline__ int row(int tid) { return tid / LPR; }
    __device__ static __forceinline__ int col0(int tid) { return (tid % LPR) * EPL; }

    __device__ static __forceinline__ float row_allreduce(float x) {
        x += dpp_mov<kDppQuadXor1>(x);
        x += dpp_mov<kDppQuadXor2>(x);
        if constexpr (LPR == 8) {
            x += dpp_mov<0x141>(x);  // row_half_mirror: lane i <-> 7 - i, i.e. the other quad
        } else {
            x += dpp_mov<kDppRowRor4>(x);
            x += dpp_mov<kDppRowRor8>(x);
        }
        return x;
    }
    // sum over all NP rows of per-column values; cw_t = this iteration's LDS slot [4][NP]
    __device__ static __forceinline__ void col_allreduce(float (&x)[EPL], float *cw_t, int tid) {
        const int lane = tid & 63, wave = tid >> 6;
#pragma unroll
        for (int e = 0; e < EPL; e++) {
            if constexpr (LPR == 8) x[e] += dpp_mov<kDppRowRor8>(x[e]);
            x[e] = xor16_add(x[e]);
            x[e] = xor32_add(x[e]);
        }
        if (lane < LPR) {
#pragma unroll
            for (int e = 0; e < EPL; e++) cw_t[wave * NP + lane * EPL + e] = x[e];
        }
        __syncthreads();
        const int c0 = col0(tid);
#pragma unroll
        for (int e = 0; e < EPL; e++)
            x[e] = (cw_t[c0 + e] + cw_t[NP + c0 + e]) + (cw_t[2 * NP + c0 + e] + cw_t[3 * NP + c0 + e]);
    }

    // E: exp(logits), 0 outside n x n.  On return M = u * E[e] * v[e]; rho/s hold the denominators.
    // PRECISE selects IEEE divisions (fp32 parity tier) instead of v_rcp_f32 (1 ulp).
    template <bool PRECISE = true>
    __device__ static __forceinline__ void forward(const float (&E)[EPL], float &u, float (&v)[EPL],
                                                   int n, int T, float eps, float *lds, int tid) {
        float *cw = lds, *rho = lds + 8 * NP, *s = rho + T * NP;
        const int r = row(tid), c0 = col0(tid);
        u = 1.0f;
#pragma unroll
        for (int e = 0; e < EPL; e++) v[e] = 1.0f;
        for (int t = 0; t < T; t++) {
            float p = 0.f;
#pragma unroll
            for (int e = 0; e < EPL; e++) p += E[e] * v[e];
            p = row_allreduce(p);
            const float rr = r < n ? u * p + eps : 1.0f;
            u = PRECISE ? u / rr : u * fast_rcp(rr);
            if ((tid % LPR) == 0) rho[t * NP + r] = rr;
            float q[EPL];
#pragma unroll
            for (int e = 0; e < EPL; e++) q[e] = E[e] * u;
            col_allreduce(q, cw + (t & 1) * 4 * NP, tid);
#pragma unroll
            for (int e = 0; e < EPL; e++) {
                const float sc = c0 + e < n ? v[e] * q[e] + eps : 1.0f;
                v[e] = PRECISE ? v[e] / sc : v[e] * fast_rcp(sc);
                if (r == 0) s[t * NP + c0 + e] = sc;
            }
        }
        __syncthreads();  // rho / s visible to every thread
    }

    // d: in = dL/dM, out = dL/dE.  u, v: final scalings from forward (destroyed).
    template <bool PRECISE = true>
    __device__ static __forceinline__ void backward(const float (&E)[EPL], float (&d)[EPL], float u,
                                                    float (&v)[EPL], int T, float *lds, int tid) {
        float *cw = lds;
        const float *rho = lds + 8 * NP, *s = rho + T * NP;
        const int r = row(tid), c0 = col0(tid);
        for (int t = T - 1; t >= 0; t--) {
            // column dots with the iterate after column step t: Out = u E v
            float cd[EPL];
#pragma unroll
            for (int e = 0; e < EPL; e++) cd[e] = d[e] * u * E[e];
            col_allreduce(cd, cw + (t & 1) * 4 * NP, tid);
            float z = 0.f, sc[EPL];
#pragma unroll
            for (int e = 0; e < EPL; e++) {
                sc[e] = s[t * NP + c0 + e];
                d[e] -= cd[e] * v[e];
                z += d[e] * E[e] * v[e];
            }
            const float rdot = u * row_allreduce(z);
            const float rr = rho[t * NP + r];
            const float rri = PRECISE ? 0.f : fast_rcp(rr);
#pragma unroll
            for (int e = 0; e < EPL; e++) {
                d[e] = PRECISE ? (d[e] / sc[e] - rdot) / rr : (d[e] * fast_rcp(sc[e]) - rdot) * rri;
                v[e] *= sc[e];
            }
            u *= rr;
        }
    }
};

}  // namespace mhc
