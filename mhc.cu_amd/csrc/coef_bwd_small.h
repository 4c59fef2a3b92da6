// Pieces shared by the kernels that run the n <= 8 coefficient backward inside a larger workgroup
// (channel sums in mix_bwd_reduce.hip, the sample-resident backward in bwd_resident.hip): the argument
// block, the writer of dP in every layout later kernels read, and the coefficient backward itself.
#pragma once
#include "launchers.h"
#include "phase_profiler.h"
#include "sinkhorn_device.h"

namespace mhc {

struct BwdReduceArgs {
    const void *dy, *x, *w, *f_inject;
    const float *Hpre, *Hpost, *M, *q, *P, *r, *alpha, *b_res;
    const float *sk_state;  // dynamic: Sinkhorn denominators saved by the forward ([B][T + 1][2][NP]) or nullptr
    BwdCoefOut out;
    int hstride, w_bf16, B, n, C, T, DP;
    float eps;
    float *raw;   // n <= 8: when set, write the raw channel sums [B][parts][K] and stop
    int parts;    // column parts per sample (gridDim.y)
    float *s1part = nullptr;  // n > 8: when set, the Gram launch also writes s1 = Hpost^T W1 Hpre of every part, [B][parts]
    // static H, n > 8: the channel-sum launch carries one more workgroup that recomputes the Sinkhorn forward
    // of the shared logits (IEEE divisions) and leaves its denominators here for the static coefficient
    // backward, which then has half its chain left (SkWg::save_state layout, (2 T + 2) * NP floats)
    const float *static_logits = nullptr;
    float *static_state = nullptr;
};

// Where the weight of the W1 = dy diag(w) x^T Gram matrix comes from: an injected f [B, C] (W1 = dy [f; 0 ..]^T),
// or the RMSNorm weight in bf16 / fp32.
enum { kGramInject = 0, kGramWBf16 = 1, kGramWF32 = 2 };

__device__ __forceinline__ float load_w_(const void *w, int w_bf16, int c) {
    return w_bf16 ? bf16_to_f32(static_cast<const bf16_t *>(w)[c]) : static_cast<const float *>(w)[c];
}

// Sum over the 16 lanes of a DPP row; every lane of the row gets the total.
__device__ __forceinline__ float row16_allreduce(float v) {
    v += dpp_mov<kDppQuadXor1>(v);
    v += dpp_mov<kDppQuadXor2>(v);
    v += dpp_mov<kDppRowRor4>(v);
    v += dpp_mov<kDppRowRor8>(v);
    return v;
}

// Writes dP[b, d] in every layout the later kernels read: fp32 [B, DP] (generic kernels),
// and two bf16 copies in fragment-major order (frag_dpb / frag_dpt: MFMA A operands; for the
// transpose, plane 0 = value rounded to bf16, plane 1 = the rounding remainder, so that dphi
// keeps ~16 mantissa bits of dP).  Padded
// rows d >= D and, from the last sample's workgroup, padded columns b >= B are zeroed.
struct DPWriter {
    BwdCoefOut o;
    int b, B, DP;
    __device__ __forceinline__ void put(int d, float v) const {
        if (o.dP) o.dP[(size_t)b * DP + d] = v;  // fp32 copy: only the kernels without matrix-core operands read it
        if (o.dPb) {
            const bf16_t h = f32_to_bf16(v);
            const size_t plane = (size_t)DP * o.BP;
            o.dPb[frag_dpb(b, d, DP)] = h;
            o.dPT[frag_dpt(d, b, o.BP)] = h;
            o.dPT[plane + frag_dpt(d, b, o.BP)] = f32_to_bf16(v - bf16_to_f32(h));
            if (b == B - 1)
                for (int bb = B; bb < o.BP; bb++) {
                    o.dPT[frag_dpt(d, bb, o.BP)] = 0;
                    o.dPT[plane + frag_dpt(d, bb, o.BP)] = 0;
                }
        }
    }
    __device__ __forceinline__ void pad(int D, int first, int step) const {
        for (int d = D + first; d < DP; d += step) {
            if (o.dP) o.dP[(size_t)b * DP + d] = 0.f;
            if (o.dPb) {
                const size_t plane = (size_t)DP * o.BP;
                o.dPb[frag_dpb(b, d, DP)] = 0;
                o.dPT[frag_dpt(d, b, o.BP)] = 0;
                o.dPT[plane + frag_dpt(d, b, o.BP)] = 0;
                if (b == B - 1)
                    for (int bb = B; bb < o.BP; bb++) {
                        o.dPT[frag_dpt(d, bb, o.BP)] = 0;
                        o.dPT[plane + frag_dpt(d, bb, o.BP)] = 0;
                    }
            }
        }
    }
};

// =============================================================================================
// n <= 8, dynamic H: coefficient backward of one sample on the lanes of one SkSmall group (16 lanes
// for 4x4, a wave for 8x8).  Input: channel sums of the sample, `parts` blocks of K floats, in
// global memory or in LDS:
//   GRAM:  dM | W1 | XX (NP x NP each, K = 3 NP^2)
//   else:  dM | dHpost | A1 | A2 | s1 (K = NP^2 + 3 NP + 1)
// prefetch() asks for everything else the sample needs (P, H, r, q, alpha, b_res), so that a caller
// with other work to do first has those values waiting; run() then forms dHpre / dHpost, the sigmoid
// derivatives, the exact Sinkhorn backward, dP = dt * alpha / r in all three layouts, and cx.
// =============================================================================================
// STATIC (with GRAM): shared coefficients - prefetch() takes H from the [n] vectors and nothing else, and
// run() stops after the channel-sum vectors: it writes the sample's raw gradients (dM | dHpre | dHpost)
// as a row of `red` for the batch-sum launch; the Sinkhorn backward then runs once on the batch total.
template <int NP, bool PRECISE, bool GRAM, bool STATIC = false> struct CoefBwdSmall {
    using SK = SkSmall<NP>;
    static constexpr int K = GRAM ? 3 * NP * NP : NP * NP + 3 * NP + 1;
    // LDS floats next to the Sinkhorn denominators, per group: the column results of the Gram sums
    static constexpr int kXch = GRAM ? 3 * NP : 0;

    int r0, c0, gc;
    bool inject, mv;
    float qinv, rinv, inv_c, inv_nc, al0, al1, al2, pres, bres, hp, ho, ppre, ppost, hpre_r, hpost_r;
    float m_fin;  // the final Sinkhorn iterate of this lane's element (forward_recompute)
    float dMe, s_a, s_b, s_c, s_d;  // this lane's channel sums (fetch_sums): GRAM w1, w1t, xx | else dHpost, A1, A2, s1

    __device__ __forceinline__ void prefetch(const BwdReduceArgs &a, int b, int g) {
        const int n = a.n, D = n * n + 2 * n;
        r0 = SK::row(g); c0 = SK::col0(g);
        gc = g < n ? g : 0;  // lanes beyond n alias entry 0 (never used): no branch around loads
        mv = r0 < n && c0 < n;
        inject = a.f_inject != nullptr;
        // PRECISE keeps IEEE divisions; otherwise v_rcp_f32 / v_exp_f32 (1 ulp) keep the step short
        qinv = inject ? 0.f : (PRECISE ? 1.0f / a.q[b] : fast_rcp(a.q[b]));
        inv_c = 1.0f / (float)a.C; inv_nc = 1.0f / (float)(n * a.C);
        if constexpr (STATIC) {
            hp = a.Hpre[gc]; ho = a.Hpost[gc];
            hpre_r = a.Hpre[r0 < n ? r0 : 0];
            hpost_r = a.Hpost[r0 < n ? r0 : 0];
            rinv = al0 = al1 = al2 = pres = bres = ppre = ppost = 0.f;
            return;
        }
        const float *Pb = a.P + (size_t)b * D;
        al0 = a.alpha[0]; al1 = a.alpha[1]; al2 = a.alpha[2];
        rinv = PRECISE ? 1.0f / a.r[b] : fast_rcp(a.r[b]);
        pres = Pb[mv ? 2 * n + r0 * n + c0 : 0];
        bres = a.b_res[mv ? r0 * n + c0 : 0];
        hp = a.Hpre[(size_t)b * n + gc]; ho = a.Hpost[(size_t)b * n + gc];
        ppre = Pb[gc]; ppost = Pb[n + gc];
        hpre_r = a.Hpre[(size_t)b * n + (r0 < n ? r0 : 0)];
        hpost_r = a.Hpost[(size_t)b * n + (r0 < n ? r0 : 0)];
    }

    // The Sinkhorn forward recompute, which keeps the denominators of every iteration in sc: it needs
    // none of the channel sums, so a caller that produces them itself can run it while they are
    // still on their way.  g: lane within the group; lane: lane within the wave (indexes sc).
    // With the denominators saved by the forward call there is nothing to iterate: they are copied
    // into sc and the final iterate is the saved M.
    __device__ __forceinline__ void forward_recompute(const BwdReduceArgs &a, int b, int g, int lane, float *sc) {
        if (a.sk_state) {
            // every load is requested before the first value (of prefetch() too) is used
            m_fin = a.M[(size_t)b * a.n * a.n + (mv ? r0 * a.n + c0 : 0)];
            SK::load_state(a.sk_state + (size_t)b * SK::state_floats(a.T), g, a.T, sc, lane);
            m_fin = mv ? m_fin : 0.f;
            return;
        }
        const float E = mv ? (PRECISE ? expf(al2 * pres + bres) : exp_fast(al2 * pres + bres)) : 0.f;
        float m[1] = {E};
        SK::template forward<PRECISE>(m, g, a.n, a.T, a.eps, sc, lane);
        m_fin = m[0];
    }

    // This lane's entries of the channel sums, summed over the column parts.
    __device__ __forceinline__ void fetch_sums(const float *sums, int parts) {
        dMe = s_a = s_b = s_c = s_d = 0.f;
        for (int p = 0; p < parts; p++) {
            const float *rp = sums + (size_t)p * K;
            dMe += rp[r0 * NP + c0];
            if constexpr (GRAM) {
                s_a += rp[NP * NP + r0 * NP + c0];
                s_b += rp[NP * NP + c0 * NP + r0];
                s_c += rp[2 * NP * NP + r0 * NP + c0];
            } else {
                s_a += rp[NP * NP + gc]; s_b += rp[NP * NP + NP + gc]; s_c += rp[NP * NP + 2 * NP + gc];
                s_d += rp[K - 1];
            }
        }
    }

    // after fetch_sums() and forward_recompute(); xch: kXch floats of LDS private to the group
    __device__ __forceinline__ void run(const BwdReduceArgs &a, int b, int g, int lane, float *sc, float *xch) {
        const int n = a.n, D = n * n + 2 * n;
        const int pwg_r = blockIdx.y * gridDim.x + blockIdx.x;
        (void)pwg_r;
        MHC_PHASE_BEGIN(rclk);
        float tpost = 0.f, tA1 = 0.f, tA2 = 0.f, s1 = 0.f;
        if constexpr (GRAM) {
            // lane (r0, c0) takes its element of each matrix and the mirrored element of W1, so that
            // every sum below runs down a column:
            //   dHpost[c] = sum_r Hpre[r] W1[c][r] / q        A1[c] = sum_r Hpost[r] W1[r][c]
            //   A2[c] = sum_r Hpre[r] XX[r][c]                s1 = sum_c Hpost[c] (sum_r Hpre[r] W1[c][r])
            // The column results are handed to lanes 0 .. n-1 through LDS (same wave: no barrier).
            const float w1 = s_a, w1t = s_b, xx = s_c;
            const float hr = r0 < n ? hpre_r : 0.f, hor = r0 < n ? hpost_r : 0.f;
            // with an injected f, W1 = dy [f; 0; ...]^T and dHpost is its column 0
            const float sel = inject ? (r0 == 0 ? 1.f : 0.f) : hr;
            const float x0 = SK::col_allreduce(sel * w1t);
            const float x1 = SK::col_allreduce(hor * w1);
            const float x2 = SK::col_allreduce(hr * xx);
            if (r0 == 0) { xch[c0] = x0; xch[NP + c0] = x1; xch[2 * NP + c0] = x2; }
            const float hw = xch[gc];
            if (inject) {
                tpost = hw;
            } else {
                tpost = hw * qinv;
                tA1 = xch[NP + gc];
                tA2 = xch[2 * NP + gc];
                s1 = SK::group_allreduce(g < n ? ho * hw : 0.f);
            }
        } else {
            tpost = s_a; tA1 = s_b; tA2 = s_c; s1 = s_d;
        }
        if (g == 0) a.out.s1[b] = s1;
        if constexpr (STATIC) {
            float *red = a.out.red + (size_t)b * (D + 3);  // rows padded like dt, for the batch-sum launch
            if (mv) red[r0 * n + c0] = dMe;
            if (g < n) {
                red[n * n + g] = inject ? 0.f : tA1 * qinv - s1 * tA2 * qinv * qinv * qinv * inv_c;
                red[n * n + n + g] = tpost;
            }
            return;
        }
        float *dt = a.out.dt + (size_t)b * (D + 3);
        const DPWriter dpw{a.out, b, a.B, a.DP};
        float S0 = 0.f, S1 = 0.f, S2 = 0.f;  // sum_d dt_d p_d per alpha group
        if (g < n) {
            const float dHpost = tpost;
            const float dHpre = inject ? 0.f : tA1 * qinv - s1 * tA2 * qinv * qinv * qinv * inv_c;
            const float dtp = dHpre * hp * (1.0f - hp);
            const float dto = dHpost * ho * (1.0f - 0.5f * ho);
            dt[g] = dtp; dt[n + g] = dto;
            dpw.put(g, dtp * al0 * rinv); dpw.put(n + g, dto * al1 * rinv);
            S0 = dtp * ppre; S1 = dto * ppost;
        }
        float m[1] = {m_fin}, d[1] = {mv ? dMe : 0.f};
        if constexpr (GRAM) MHC_PHASE_ADD(kPhaseGramSmall, pwg_r, 4, rclk);
        SK::template backward<PRECISE>(d, m, a.T, sc, lane);
        if constexpr (GRAM) MHC_PHASE_ADD(kPhaseGramSmall, pwg_r, 5, rclk);
        if (mv) {
            const int di = 2 * n + r0 * n + c0;
            const float dtr = d[0];  // the Sinkhorn backward hands back the gradient of the logits
            dt[di] = dtr;
            dpw.put(di, dtr * al2 * rinv);
            S2 = dtr * pres;
        }
        S0 = SK::group_allreduce(S0); S1 = SK::group_allreduce(S1); S2 = SK::group_allreduce(S2);
        if (g == 0) {
            dt[D] = S0; dt[D + 1] = S1; dt[D + 2] = S2;
            a.out.cx[b] = (al0 * S0 + al1 * S1 + al2 * S2) * rinv * rinv * inv_nc;
        }
        dpw.pad(D, g, SK::kGroup);
        if constexpr (GRAM) MHC_PHASE_ADD(kPhaseGramSmall, pwg_r, 6, rclk);
    }
};

}  // namespace mhc
