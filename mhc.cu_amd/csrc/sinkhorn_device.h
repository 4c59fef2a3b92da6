// Sinkhorn-Knopp on one n x n matrix (n <= 32), forward and exact backward, as device routines.
//
// Semantics (reference: src/python/benchmarks/bench_layer.py:48-53 / :112-117): start from
// E = exp(logits); T times: divide every row by (row sum + eps), then every column by
// (column sum + eps).  The backward is the exact reverse sweep through all T iterations (carried on the
// product gradient x iterate, which needs no division); only the
// per-iteration denominators rho_t[r], s_t[c] are kept in LDS during the forward recompute, and
// the iterates are rebuilt from them by undoing the scalings.
//
// Two layouts:
//   SkSmall<NP> (NP = 4, 8): one element per lane, a matrix lives in NP*NP consecutive lanes (four
//       4x4 matrices per wave, or one 8x8 matrix); all reductions are DPP moves and lane swaps, no
//       LDS traffic on the forward path.  The chain of an iteration is then about a dozen
//       dependent instructions for either size (with four elements per lane an 8x8 iteration
//       issued some 60 instructions on a wave that has the SIMD to itself).
//   SkWg<NP>    (NP = 16, 32): one 256-thread workgroup per matrix, everything in registers,
//       iterate kept in scaling form diag(u) E diag(v).
#pragma once

#include "mhc_common.h"

namespace mhc {

// a * b + c with the product rounded before the sum (the compiler fuses the plain expression)
__device__ __forceinline__ float mul_add_unfused(float a, float b, float c) {
#pragma clang fp contract(off)
    const float t = a * b;
    return t + c;
}

// =============================================================================================
// SkSmall
// =============================================================================================
// The serial chains below run on one wave while the other waves of the CU stream; the chain's wave
// asks for issue priority while it lasts (B=1280, C=2560, n=4, five workgroups per CU: -0.5 us per step).
__device__ __forceinline__ void sk_chain_begin() { __builtin_amdgcn_s_setprio(3); }
__device__ __forceinline__ void sk_chain_end() { __builtin_amdgcn_s_setprio(0); }

template <int NP> struct SkSmall {
    static_assert(NP == 4 || NP == 8, "SkSmall handles 4x4 and 8x8 tiles");
    static constexpr int EPL = 1;               // elements per lane
    static constexpr int kGroup = NP * NP;      // lanes per matrix: 16 or the whole wave
    static constexpr int kPerWave = kWave / kGroup;  // matrices per wave

    __device__ static __forceinline__ int row(int g) { return g / NP; }
    __device__ static __forceinline__ int col0(int g) { return g % NP; }

    // sum over the NP consecutive lanes that hold a row
    __device__ static __forceinline__ float row_allreduce(float v) {
        v += dpp_mov<kDppQuadXor1>(v);
        v += dpp_mov<kDppQuadXor2>(v);
        if constexpr (NP == 8) v += dpp_mov<kDppRowHalfMirror>(v);  // the other quad of the 8 lanes
        return v;
    }
    // sum over the lanes that hold a column (stride NP)
    __device__ static __forceinline__ float col_allreduce(float v) {
        if constexpr (NP == 4) {
            v += dpp_mov<kDppRowRor4>(v);
            v += dpp_mov<kDppRowRor8>(v);
        } else {
            v += dpp_mov<kDppRowRor8>(v);
            v = xor16_add(v);
            v = xor32_add(v);
        }
        return v;
    }
    // sum over all lanes of the matrix
    __device__ static __forceinline__ float group_allreduce(float v) { return col_allreduce(row_allreduce(v)); }

    // m: in = exp(logits) (0 outside n x n), out = final iterate.
    // RECORD: keep, per iteration t and lane, the row denominator and per element the column
    // denominator:  sc[(t * kRec + k) * 64 + lane], k = 0: rho | 1..EPL: s  (a compile-time switch:
    // a test of the pointer stays in the loop as two branches per iteration)
    // PRECISE selects IEEE divisions (fp32 parity tier) instead of v_rcp_f32.
    static constexpr int kRec = 1 + EPL;
    template <bool PRECISE = false, bool RECORD = true>
    __device__ static __forceinline__ void forward(float (&m)[EPL], int g, int n, int T, float eps,
                                                   float *sc, int lane) {
        // rows and columns beyond n hold zeros: their denominator is made 1 (not eps, which may be
        // 0) by the constant that is added, so the dependent chain carries no select
        const float eps_r = row(g) < n ? eps : 1.0f;
        float eps_c[EPL];
#pragma unroll
        for (int e = 0; e < EPL; e++) eps_c[e] = col0(g) + e < n ? eps : 1.0f;
        sk_chain_begin();
        for (int t = 0; t < T; t++) {
            float rs = 0.f;
#pragma unroll
            for (int e = 0; e < EPL; e++) rs += m[e];
            rs = row_allreduce(rs) + eps_r;
            const float rinv = PRECISE ? 1.0f / rs : fast_rcp(rs);
            if constexpr (RECORD) sc[(t * kRec) * kWave + lane] = rs;
#pragma unroll
            for (int e = 0; e < EPL; e++) {
                m[e] = PRECISE ? m[e] / rs : m[e] * rinv;
                const float cs = col_allreduce(m[e]) + eps_c[e];
                if constexpr (RECORD) sc[(t * kRec + 1 + e) * kWave + lane] = cs;
                m[e] = PRECISE ? m[e] / cs : m[e] * fast_rcp(cs);
            }
        }
        sk_chain_end();
    }

    // The same forward, keeping the denominators of every iteration in GLOBAL memory for the backward
    // call: st[(t * 2 + 0) * NP + row] = rho_t[row], st[(t * 2 + 1) * NP + col] = s_t[col] (every lane
    // of a row / column writes the same value).  2 T NP floats per matrix.
    template <bool PRECISE = false>
    __device__ static __forceinline__ void forward_save(float (&m)[EPL], int g, int n, int T, float eps, float *st) {
        static_assert(EPL == 1, "one element per lane");
        const int r = row(g), c = col0(g);
        const float eps_r = r < n ? eps : 1.0f, eps_c = c < n ? eps : 1.0f;
        sk_chain_begin();
        for (int t = 0; t < T; t++) {
            const float rs = row_allreduce(m[0]) + eps_r;
            st[(t * 2) * NP + r] = rs;
            m[0] = PRECISE ? m[0] / rs : m[0] * fast_rcp(rs);
            const float cs = col_allreduce(m[0]) + eps_c;
            st[(t * 2 + 1) * NP + c] = cs;
            m[0] = PRECISE ? m[0] / cs : m[0] * fast_rcp(cs);
        }
        sk_chain_end();
    }
    // Denominators saved by forward_save() -> the per-lane LDS layout that backward() reads.  The
    // loads of 24 iterations are requested together (one round trip for the usual 20).
    __device__ static __forceinline__ void load_state(const float *st, int g, int T, float *sc, int lane) {
        constexpr int kBatch = 24;
        const float *pr = st + row(g), *pc = st + NP + col0(g);
        for (int t0 = 0; t0 < T; t0 += kBatch) {
            float rs[kBatch], cs[kBatch];
#pragma unroll
            for (int u = 0; u < kBatch; u++) {
                const int t = t0 + u < T ? t0 + u : T - 1;
                rs[u] = pr[t * 2 * NP];
                cs[u] = pc[t * 2 * NP];
            }
#pragma unroll
            for (int u = 0; u < kBatch; u++) {
                if (t0 + u < T) {
                    sc[((t0 + u) * kRec) * kWave + lane] = rs[u];
                    sc[((t0 + u) * kRec + 1) * kWave + lane] = cs[u];
                }
            }
        }
    }
    // one footprint for every layout: [T + 1][2][NP] (slot T is used by SkWg only)
    __host__ __device__ static constexpr int state_floats(int T) { return 2 * (T + 1) * NP; }

    // d: in = dL/dM, out = dL/dlogits (= dL/dE o E).  m: the final iterate from forward (destroyed).
    // The reverse sweep runs on the PRODUCT p = (gradient o iterate) instead of on the gradient: through
    // a normalisation Y = X / (sum X + eps) the gradient is dX = (dY - sum(dY o Y)) / den, and the product
    // with the iterate before it is dX o X = (dY - sum(dY o Y)) o Y = p - sum(p) Y.  So one half-step is
    //     p <- p - allreduce(p) * iterate
    // with no division and no reciprocal; the iterates are rebuilt by undoing the scalings with the saved
    // denominators (Out_t = m, R_t = Out_t s_t, Out_{t-1} = R_t rho_t), a chain of its own beside the
    // one that carries p.  The dependent chain of an iteration is two all-reduces and two fused
    // multiply-adds.  After the last step the iterate is E itself and p = dL/dE o E, which is what every
    // caller wants.  PRECISE is kept for the callers' template argument; both tiers compute the same.
    template <bool PRECISE = false>
    __device__ static __forceinline__ void backward(float (&d)[EPL], float (&m)[EPL], int T,
                                                    const float *sc, int lane) {
        static_assert(EPL == 1, "one element per lane");
        // The denominators of an iteration are requested one iteration ahead of their use (two
        // register pairs, alternating), so that the LDS round trip stays off the dependent chain.
        auto fetch = [&](int t, float &rs, float &cs) {
            t = t < 0 ? 0 : t;
            rs = sc[(t * kRec) * kWave + lane];
            cs = sc[(t * kRec + 1) * kWave + lane];
        };
        float p = d[0] * m[0];
        auto step = [&](float rs, float cs) {
            p = __builtin_fmaf(-col_allreduce(p), m[0], p);  // through the column normalisation: Out_t
            m[0] *= cs;                                      // R_t
            p = __builtin_fmaf(-row_allreduce(p), m[0], p);  // through the row normalisation
            m[0] *= rs;                                      // Out_{t-1}
        };
        float rs0, cs0, rs1, cs1;
        int t = T - 1;
        sk_chain_begin();
        fetch(t, rs0, cs0);
        if (T & 1) {  // an odd count: one step ahead of the pairs
            step(rs0, cs0);
            fetch(--t, rs0, cs0);
        }
        for (; t >= 1; t -= 2) {
            fetch(t - 1, rs1, cs1);
            step(rs0, cs0);
            fetch(t - 2, rs0, cs0);
            step(rs1, cs1);
        }
        sk_chain_end();
        d[0] = p;
    }
    __host__ __device__ static constexpr int scaling_floats(int T) { return T * kRec * kWave; }
};

// =============================================================================================
// SkWg: one 256-thread workgroup per matrix, NP = 16 or 32, iterate kept in scaling form
// diag(u) E diag(v) with E constant in registers: thread t owns E[a][b0 .. b0+EPL) with
// (a, b0) = (t / LPR, (t % LPR) * EPL), and the running gradient there.
//
// forward(): every thread also holds the transposed elements E[b0 .. b0+EPL)[a] (copied once
// through LDS), so both the row sums and the column sums are an in-register dot product plus a
// reduction over the LPR lanes of a DPP row; only the vectors u and v travel through LDS (one
// barrier per half-step).  The denominators rho/s of every iteration stay in LDS.
// backward(): one copy of the product gradient x iterate; row sums inside a DPP row, column sums inside the wave
// (DPP, v_permlane*_swap) and then across the 4 waves through a double-buffered LDS slot (one
// barrier per iteration; keeping a transposed copy of the gradient as well needs two barriers and
// measured 50 % slower); the scalings are unwound with the saved denominators (u *= rho, v *= s)
// instead of storing iterates.  Against float64 the backward stays at ~2e-7 for every iteration count
// once the forward's denominators are computed without a fused multiply-add (see forward()); with it
// the error grew by ~2e-8 per iteration.  Every thread of the workgroup must call forward/backward;
// `lds` must be 16-byte aligned.
// =============================================================================================
template <int NP> struct SkWg {
    static_assert(NP == 16 || NP == 32, "SkWg handles 16x16 and 32x32 tiles");
    static constexpr int EPL = NP * NP / 256;  // 1 or 4
    static constexpr int LPR = NP / EPL;       // lanes per row: 16 or 8
    static constexpr int kTile = NP * (NP + 1);
    // LDS floats: transpose tile (later the column slots [2][4][NP]) | u | v | rho [T][NP] | s [T][NP]
    __host__ __device__ static constexpr int lds_floats(int T) { return kTile + 2 * NP + 2 * T * NP; }
    __device__ static __forceinline__ int row(int tid) { return tid / LPR; }
    __device__ static __forceinline__ int col0(int tid) { return (tid % LPR) * EPL; }

    // sum over the LPR lanes that share tid / LPR
    __device__ static __forceinline__ float seg_allreduce(float x) {
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
    // EPL consecutive floats at a 16-byte aligned LDS address
    __device__ static __forceinline__ void ld_vec(const float *p, float (&x)[EPL]) {
        if constexpr (EPL == 4) {
            const float4 t = *reinterpret_cast<const float4 *>(p);
            x[0] = t.x; x[1] = t.y; x[2] = t.z; x[3] = t.w;
        } else {
#pragma unroll
            for (int e = 0; e < EPL; e++) x[e] = p[e];
        }
    }
    // a[e] = A[a][b0+e]  ->  at[e] = A[b0+e][a]
    __device__ static __forceinline__ void transpose(const float (&a)[EPL], float (&at)[EPL], float *tile,
                                                     int tid) {
        const int r = row(tid), c0 = col0(tid);
#pragma unroll
        for (int e = 0; e < EPL; e++) tile[r * (NP + 1) + c0 + e] = a[e];
        __syncthreads();
#pragma unroll
        for (int e = 0; e < EPL; e++) at[e] = tile[(c0 + e) * (NP + 1) + r];
        __syncthreads();
    }

    // E: exp(logits), 0 outside n x n.  On return M = u * E[e] * v[e]; rho/s hold the denominators.
    // PRECISE selects IEEE divisions (fp32 parity tier) instead of v_rcp_f32 (1 ulp).
    template <bool PRECISE = true>
    __device__ static __forceinline__ void forward(const float (&E)[EPL], float &u, float (&v)[EPL], int n,
                                                   int T, float eps, float *lds, int tid) {
        float *ub = lds + kTile, *vb = ub + NP, *rho = vb + NP, *s = rho + T * NP;
        const int a = row(tid), b0 = col0(tid);
        const bool head = (tid % LPR) == 0, live = a < n;
        float ET[EPL];
        transpose(E, ET, lds, tid);
        u = 1.0f;
        float vc = 1.0f;  // v[a]: this thread's column in the transposed role
#pragma unroll
        for (int e = 0; e < EPL; e++) v[e] = 1.0f;
        for (int t = 0; t < T; t++) {
            float p = 0.f;
#pragma unroll
            for (int e = 0; e < EPL; e++) p += E[e] * v[e];
            p = seg_allreduce(p);
            // fp32 tier: product and sum rounded separately.  With a fused multiply-add the converged
            // denominators settle one ulp off 1 on some rows and columns (u and v keep drifting against
            // each other), and the reverse sweep, which divides by them in every iteration, drifts away
            // from the float64 result by ~2e-8 per iteration; rounded separately they settle at exactly 1.
            const float rr = live ? (PRECISE ? mul_add_unfused(u, p, eps) : u * p + eps) : 1.0f;
            u = PRECISE ? u / rr : u * fast_rcp(rr);
            if (head) { rho[t * NP + a] = rr; ub[a] = u; }
            __syncthreads();
            float uc[EPL], q = 0.f;
            ld_vec(ub + b0, uc);
#pragma unroll
            for (int e = 0; e < EPL; e++) q += ET[e] * uc[e];
            q = seg_allreduce(q);
            const float sc = live ? (PRECISE ? mul_add_unfused(vc, q, eps) : vc * q + eps) : 1.0f;
            vc = PRECISE ? vc / sc : vc * fast_rcp(sc);
            if (head) { s[t * NP + a] = sc; vb[a] = vc; }
            __syncthreads();
            ld_vec(vb + b0, v);
        }
    }

    // Copies what forward() left behind to global memory for the backward call:
    // st[(t * 2 + 0) * NP + a] = rho_t[a], st[(t * 2 + 1) * NP + a] = s_t[a] for t < T, and in slot T
    // the final scalings u[a], v[a] (which the reverse sweep starts from).  Every thread calls it.
    __device__ static __forceinline__ void save_state(const float *lds, int T, float *st, int tid, float u,
                                                      const float (&v)[EPL]) {
        const float *rho = lds + kTile + 2 * NP, *s = rho + T * NP;
        for (int e = tid; e < T * NP; e += 256) {
            const int t = e / NP, a = e % NP;
            st[(t * 2) * NP + a] = rho[e];
            st[(t * 2 + 1) * NP + a] = s[e];
        }
        if (tid % LPR == 0) st[2 * T * NP + row(tid)] = u;
        if (tid < LPR) {
#pragma unroll
            for (int e = 0; e < EPL; e++) st[(2 * T + 1) * NP + col0(tid) + e] = v[e];
        }
    }
    // The inverse: puts the saved denominators where backward() expects them and hands back the final
    // scalings, so that backward() can follow without the forward recompute.  All loads are requested
    // before the first is used.  Every thread calls it; ends on a barrier.
    __device__ static __forceinline__ void load_state(const float *st, float &u, float (&v)[EPL], int T, float *lds,
                                                      int tid) {
        float *rho = lds + kTile + 2 * NP, *s = rho + T * NP;
        const int total = 2 * T * NP;  // [t][rho | s][a]
        u = st[total + row(tid)];
#pragma unroll
        for (int e = 0; e < EPL; e++) v[e] = st[total + NP + col0(tid) + e];
        for (int e0 = 0; e0 < total; e0 += 256 * 8) {
            float tv[8];
#pragma unroll
            for (int k = 0; k < 8; k++) {
                const int e = e0 + tid + 256 * k;
                tv[k] = st[e < total ? e : 0];
            }
#pragma unroll
            for (int k = 0; k < 8; k++) {
                const int e = e0 + tid + 256 * k;
                if (e < total) {
                    const int t = e / (2 * NP), a = e % NP;
                    ((e / NP) & 1 ? s : rho)[t * NP + a] = tv[k];
                }
            }
        }
        __syncthreads();
    }
    __host__ __device__ static constexpr int state_floats(int T) { return 2 * (T + 1) * NP; }

    // d: in = dL/dM, out = dL/dlogits (= dL/dE o E).  E, u, v, LDS contents: as left by forward() (u and
    // v are destroyed).  Product form as in SkSmall::backward: p = gradient o iterate, one half-step is
    // p <- p - allreduce(p) * iterate, no divisions; the iterate u E v is unwound with the saved
    // denominators (v *= s, u *= rho).  Both tiers compute the same.
    template <bool PRECISE = true>
    __device__ static __forceinline__ void backward(const float (&E)[EPL], float (&d)[EPL], float u,
                                                    float (&v)[EPL], int T, float *lds, int tid) {
        float *cw = lds;  // the transpose tile is dead after forward()
        const float *rho = lds + kTile + 2 * NP, *s = rho + T * NP;
        const int r = row(tid), c0 = col0(tid);
        float p[EPL], W[EPL];  // W = E v: the iterate without its row scaling
#pragma unroll
        for (int e = 0; e < EPL; e++) {
            W[e] = E[e] * v[e];
            p[e] = d[e] * (u * W[e]);
        }
        for (int t = T - 1; t >= 0; t--) {
            float sc[EPL];
            ld_vec(s + t * NP + c0, sc);
            const float rr = rho[t * NP + r];
            // through column step t: iterate Out = u E v
            float cd[EPL], out[EPL];
#pragma unroll
            for (int e = 0; e < EPL; e++) { cd[e] = p[e]; out[e] = u * W[e]; W[e] *= sc[e]; }
            col_allreduce(cd, cw + (t & 1) * 4 * NP, tid);
            float z = 0.f, rt[EPL];
#pragma unroll
            for (int e = 0; e < EPL; e++) {
                p[e] = __builtin_fmaf(-cd[e], out[e], p[e]);
                rt[e] = u * W[e];  // through row step t: iterate R = u E (v s)
                z += p[e];
            }
            const float rdot = seg_allreduce(z);
#pragma unroll
            for (int e = 0; e < EPL; e++) p[e] = __builtin_fmaf(-rdot, rt[e], p[e]);
            u *= rr;
        }
#pragma unroll
        for (int e = 0; e < EPL; e++) d[e] = p[e];
    }
};

}  // namespace mhc
