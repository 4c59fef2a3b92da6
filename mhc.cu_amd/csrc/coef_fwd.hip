// Coefficient kernel: per-sample H_pre = sigmoid, H_post = 2 sigmoid, M = Sinkhorn(exp(.)) from
// the projection partial sums (dynamic H) or straight from the logits (static H).
//
// Replaces, in one launch: the split-K reduction of the projection, fused_h_activations
// (reference src/csrc/include/utils.cuh:50-126) and sinkhorn_knopp_forward_batched /
// sinkhorn_knopp_forward_fused_exp (src/csrc/kernels/sinkhorn_knopp.cuh:986-1046, :461-519).
#include <type_traits>
#include "launchers.h"
#include "phase_profiler.h"
#include "sinkhorn_device.h"

namespace mhc {

// Logit of projection row d for sample b:  alpha_g * (sum_ks Ppart) / r + bias_d   (dynamic)
//                                          bias_d                                   (static)
struct CoefArgs {
    const float *Ppart;    // [KS][B][DP] raw dot products x_flat . phi_d, or nullptr (static)
    const float *ssqpart;  // [KS][B] partial sums of x_flat^2
    int KS, DP;
    const float *alpha;    // [3]
    const float *b_pre, *b_post, *b_res;
    float *Hpre, *Hpost, *M;  // [B,n], [B,n], [B,n,n]
    float *P, *r;             // [B,D], [B]  (dynamic only)
    int B, n, nC, T;
    float eps;
    // n > 8, bf16 x, one 16-byte chunk of every stream per thread (C <= 2048): the kernel also forms the
    // stream aggregate a = Hpre^T x (fp32 [B, C]) and its RMS q, from loads that fly under the Sinkhorn chain
    const bf16_t *x_agg;
    float *a_ws, *q;
    float *sk_state;  // dynamic: [B][T + 1][2][NP] Sinkhorn denominators kept for the backward, or nullptr
    bool precise;     // fp32 tier: IEEE divisions in the iterations whose denominators are kept
};

// eight loads in flight per round (a plain loop would pay one memory latency per split)
__device__ __forceinline__ float reduce_partials(const float *part, int KS, size_t stride, size_t idx) {
    float acc = 0.f;
    for (int k0 = 0; k0 < KS; k0 += 8) {
        float t[8];
#pragma unroll
        for (int q = 0; q < 8; q++) t[q] = part[(size_t)(k0 + q < KS ? k0 + q : 0) * stride + idx];
#pragma unroll
        for (int q = 0; q < 8; q++) acc += k0 + q < KS ? t[q] : 0.f;
    }
    return acc;
}

template <int NP> __global__ __launch_bounds__(64) void coef_fwd_small_kernel(CoefArgs a) {
    using SK = SkSmall<NP>;
    const int lane = threadIdx.x;
    const int g = lane % SK::kGroup;
    const int b = blockIdx.x * SK::kPerWave + lane / SK::kGroup;
    if (b >= a.B) return;  // whole groups leave together; the reductions never cross groups
    const int n = a.n, D = n * n + 2 * n;
    const bool dyn = a.Ppart != nullptr;
    float rinv = 0.f, al[3] = {0.f, 0.f, 0.f};
    if (dyn) {
        const float ssq = reduce_partials(a.ssqpart, a.KS, a.B, b);
        const float r = sqrtf(ssq / (float)a.nC + a.eps);
        rinv = 1.0f / r;
        al[0] = a.alpha[0]; al[1] = a.alpha[1]; al[2] = a.alpha[2];
        if (g == 0) a.r[b] = r;
    }
    const size_t pstride = (size_t)a.B * a.DP;
    auto logit = [&](int d, float alpha_g, float bias) -> float {
        if (!dyn) return bias;
        const float p = reduce_partials(a.Ppart, a.KS, pstride, (size_t)b * a.DP + d) * rinv;
        a.P[(size_t)b * D + d] = p;
        return alpha_g * p + bias;
    };
    if (g < n) {
        a.Hpre[b * n + g] = sigmoidf_acc(logit(g, al[0], a.b_pre[g]));
        a.Hpost[b * n + g] = 2.0f * sigmoidf_acc(logit(n + g, al[1], a.b_post[g]));
    }
    const int r0 = SK::row(g), c0 = SK::col0(g);
    float m[SK::EPL];
#pragma unroll
    for (int e = 0; e < SK::EPL; e++) {
        const int c = c0 + e;
        m[e] = (r0 < n && c < n) ? expf(logit(2 * n + r0 * n + c, al[2], a.b_res[r0 * n + c])) : 0.f;
    }
    // The backward call rebuilds the iterates by undoing the scalings with the kept denominators
    // (m * s * rho).  After v_rcp_f32 that product is off by the same fraction of an ulp in every
    // iteration once the denominators have converged, which adds up over hundreds of iterations:
    // the fp32 tier divides.
    float *st = a.sk_state ? a.sk_state + (size_t)b * SK::state_floats(a.T) : nullptr;
    if (st && a.precise) SK::template forward_save<true>(m, g, n, a.T, a.eps, st);
    else if (st) SK::template forward_save<false>(m, g, n, a.T, a.eps, st);
    else if (a.precise) SK::template forward<true, false>(m, g, n, a.T, a.eps, nullptr, lane);
    else SK::template forward<false, false>(m, g, n, a.T, a.eps, nullptr, lane);
#pragma unroll
    for (int e = 0; e < SK::EPL; e++) {
        const int c = c0 + e;
        if (r0 < n && c < n) a.M[(size_t)b * n * n + r0 * n + c] = m[e];
    }
}

// One workgroup (4 waves) per sample.  All 256 threads finish the split-K sums (D = n^2 + 2n
// logits, KS partial sums each, eight loads in flight per thread), then run Sinkhorn with the
// matrix spread over their registers (SkWg).
template <int NP, bool PRECISE, bool AGG = false>
__global__ __launch_bounds__(256) void coef_fwd_lds_kernel(CoefArgs a) {
    using SK = SkWg<NP>;
    __shared__ float hp_s[AGG ? 32 : 1];
    __shared__ float red_s[4];
    extern __shared__ __align__(16) float lds[];
    float *lg = lds;                       // [NP*NP + 2*NP] logits: pre | post | res (row-major n x n)
    float *sk_s = lg + NP * NP + 2 * NP;   // SK::lds_floats(T)
    const int tid = threadIdx.x;
    const int b = blockIdx.x;
    const int n = a.n, D = n * n + 2 * n;
    const bool dyn = a.Ppart != nullptr;
    MHC_PHASE(kPhaseCoefFwdWide, b, 0);
    float al[3] = {0.f, 0.f, 0.f};
    // every wave fetches the split sums of x^2 itself (lane = split, KS <= 64): one load in flight
    // together with the partial dot products below instead of a chain of its own
    float ssq_l = 0.f;
    if (dyn) {
        const int lane = tid & 63;
        ssq_l = a.ssqpart[(size_t)(lane < a.KS ? lane : 0) * a.B + b];
        ssq_l = lane < a.KS ? ssq_l : 0.f;
        al[0] = a.alpha[0]; al[1] = a.alpha[1]; al[2] = a.alpha[2];
    }
    const size_t pstride = (size_t)a.B * a.DP;
    // Logits in fours: thread owns the 16-byte columns c4 = tid + 256 m of a partial row (DP / 4 of
    // them: the rows are padded with zeros up to DP).  All splits of a column are requested at once;
    // a wave whose columns lie beyond the row skips the round (the wave index is uniform).
    constexpr int M4 = (NP * NP + 2 * NP + 1023) / 1024;
    const int wave_u = __builtin_amdgcn_readfirstlane(tid >> 6);
    float psum[M4][4], bias[M4][4];
#pragma unroll
    for (int m = 0; m < M4; m++)
#pragma unroll
        for (int j = 0; j < 4; j++) {
            psum[m][j] = 0.f;
            const int d0 = 4 * (tid + 256 * m) + j;
            const int d = d0 < D ? d0 : 0;
            const int grp = alpha_group(d, n);
            bias[m][j] = *(grp == 0 ? a.b_pre + d : (grp == 1 ? a.b_post + (d - n) : a.b_res + (d - 2 * n)));
        }
    if (dyn) {
        const float4 *pb = reinterpret_cast<const float4 *>(a.Ppart + (size_t)b * a.DP);
        const int q4 = a.DP / 4;
        int cm[M4];
#pragma unroll
        for (int m = 0; m < M4; m++) cm[m] = tid + 256 * m < q4 ? tid + 256 * m : 0;
        // splits per round: 16 or 24 (at most 48 loads in flight per thread); the split counts that the
        // projection picks for a full chip are 15 and 24 at the benchmark shapes
        auto sum_splits = [&](auto kb_tag) {
            constexpr int KB = decltype(kb_tag)::value;
            for (int k0 = 0; k0 < a.KS; k0 += KB) {
                float4 tv[M4][KB];
#pragma unroll
                for (int m = 0; m < M4; m++) {
                    if (256 * m + 64 * wave_u >= q4) continue;
#pragma unroll
                    for (int q = 0; q < KB; q++)
                        tv[m][q] = pb[(size_t)(k0 + q < a.KS ? k0 + q : 0) * (pstride / 4) + cm[m]];
                }
#pragma unroll
                for (int m = 0; m < M4; m++) {
                    if (256 * m + 64 * wave_u >= q4) continue;
#pragma unroll
                    for (int q = 0; q < KB; q++) {
                        const bool ok = k0 + q < a.KS;
                        psum[m][0] += ok ? tv[m][q].x : 0.f; psum[m][1] += ok ? tv[m][q].y : 0.f;
                        psum[m][2] += ok ? tv[m][q].z : 0.f; psum[m][3] += ok ? tv[m][q].w : 0.f;
                    }
                }
            }
        };
        if (a.KS <= 16) sum_splits(std::integral_constant<int, 16>{});
        else sum_splits(std::integral_constant<int, 24>{});
    }
    // AGG: this thread's chunk of every stream is requested now and consumed behind the Sinkhorn
    // chain (whose barriers also publish hp_s); streams >= n alias stream 0 and meet Hpre = 0
    constexpr int NS = AGG ? NP : 1;
    RawVec<bf16_t, 8> xr[NS];
    const int C = a.nC / n, nch = C / 8;
    if constexpr (AGG) {
        const bf16_t *xb = a.x_agg + (size_t)b * a.nC + (size_t)(tid < nch ? tid : 0) * 8;
#pragma unroll
        for (int i = 0; i < NS; i++) xr[i].load(xb + (size_t)(i < n ? i : 0) * C);
    }
    MHC_PHASE(kPhaseCoefFwdWide, b, 1);
    float rinv = 0.f;
    if (dyn) {
        // PRECISE keeps the library routines; otherwise v_sqrt_f32 / v_rcp_f32 / v_exp_f32 (1 ulp)
        const float ms = wave_allreduce_sum(ssq_l) / (float)a.nC + a.eps;
        const float r = PRECISE ? sqrtf(ms) : __builtin_amdgcn_sqrtf(ms);
        rinv = PRECISE ? 1.0f / r : fast_rcp(r);
        if (tid == 0) a.r[b] = r;
    }
#pragma unroll
    for (int m = 0; m < M4; m++)
#pragma unroll
        for (int j = 0; j < 4; j++) {
            const int d = 4 * (tid + 256 * m) + j;
            if (d < D) {
                const int grp = alpha_group(d, n);
                float t = bias[m][j];
                if (dyn) {
                    const float p = psum[m][j] * rinv;
                    a.P[(size_t)b * D + d] = p;
                    t = al[grp] * p + bias[m][j];
                }
                lg[d] = t;
            }
        }
    __syncthreads();
    if (tid < n) {
        const float hp = PRECISE ? sigmoidf_acc(lg[tid]) : sigmoid_fast(lg[tid]);
        // static H with the aggregate: every sample's workgroup derives the shared coefficients (for its
        // aggregate), the first one stores them
        if (dyn || b == 0) {
            a.Hpre[(dyn ? b * n : 0) + tid] = hp;
            a.Hpost[(dyn ? b * n : 0) + tid] = 2.0f * (PRECISE ? sigmoidf_acc(lg[n + tid]) : sigmoid_fast(lg[n + tid]));
        }
        if constexpr (AGG) hp_s[tid] = hp;
    } else if (AGG && tid < 32) {
        hp_s[tid] = 0.f;
    }
    const int r0 = SK::row(tid), c0 = SK::col0(tid);
    float E[SK::EPL], u, v[SK::EPL];
#pragma unroll
    for (int e = 0; e < SK::EPL; e++)
        E[e] = (r0 < n && c0 + e < n) ? (PRECISE ? expf(lg[2 * n + r0 * n + c0 + e]) : exp_fast(lg[2 * n + r0 * n + c0 + e])) : 0.f;
    MHC_PHASE(kPhaseCoefFwdWide, b, 2);
    SK::template forward<PRECISE>(E, u, v, n, a.T, a.eps, sk_s, tid);
    MHC_PHASE(kPhaseCoefFwdWide, b, 3);
#pragma unroll
    for (int e = 0; e < SK::EPL; e++)
        if (r0 < n && c0 + e < n && (dyn || b == 0)) a.M[(dyn ? (size_t)b * n * n : 0) + r0 * n + c0 + e] = u * E[e] * v[e];
    if (a.sk_state) SK::save_state(sk_s, a.T, a.sk_state + (size_t)b * SK::state_floats(a.T), tid, u, v);
    MHC_PHASE(kPhaseCoefFwdWide, b, 4);
    if constexpr (AGG) {
        __syncthreads();  // hp_s (with zero iterations the Sinkhorn step has no barrier of its own)
        float acc[8], ssq = 0.f;
#pragma unroll
        for (int k = 0; k < 8; k++) acc[k] = 0.f;
#pragma unroll
        for (int i = 0; i < NS; i++) {
            float xv[8];
            xr[i].get(xv);
            const float hp = hp_s[i];
#pragma unroll
            for (int k = 0; k < 8; k++) acc[k] += hp * xv[k];
        }
        if (tid < nch) {
            store_vec<float, 8>(a.a_ws + (size_t)b * C + tid * 8, acc);
#pragma unroll
            for (int k = 0; k < 8; k++) ssq += acc[k] * acc[k];
        }
        ssq = block_allreduce_sum<256>(ssq, red_s);
        if (tid == 0) a.q[b] = sqrtf(ssq / (float)C + a.eps);
    }
    MHC_PHASE(kPhaseCoefFwdWide, b, 5);
}

hipError_t launch_coef_fwd(const float *Ppart, const float *ssqpart, int KS, int DP,
                           const float *alpha, const float *b_pre, const float *b_post,
                           const float *b_res, float *Hpre, float *Hpost, float *M, float *P,
                           float *r, int B, int n, int nC, int T, float eps, bool precise,
                           const void *x_agg, float *a_ws, float *q, float *sk_state, hipStream_t stream) {
    CoefArgs a{Ppart, ssqpart, KS, DP, alpha, b_pre, b_post, b_res, Hpre, Hpost, M, P, r, B, n, nC, T, eps,
               static_cast<const bf16_t *>(x_agg), a_ws, q, sk_state, precise};
    const bool agg = x_agg != nullptr;  // the caller has checked coef_fwd_aggregates()
    if (n <= 4)
        coef_fwd_small_kernel<4><<<(B + 3) / 4, 64, 0, stream>>>(a);
    else if (n <= 8)
        coef_fwd_small_kernel<8><<<B, 64, 0, stream>>>(a);
    else if (n <= 16) {
        const size_t smem = sizeof(float) * (16 * 16 + 32 + SkWg<16>::lds_floats(T));
        hipError_t e = precise ? allow_dynamic_lds(&coef_fwd_lds_kernel<16, true>, smem)
                               : allow_dynamic_lds(&coef_fwd_lds_kernel<16, false>, smem);
        if (e != hipSuccess) return e;
        if (agg) {
            e = allow_dynamic_lds(&coef_fwd_lds_kernel<16, false, true>, smem);
            if (e != hipSuccess) return e;
            coef_fwd_lds_kernel<16, false, true><<<B, 256, smem, stream>>>(a);
        } else if (precise) coef_fwd_lds_kernel<16, true><<<B, 256, smem, stream>>>(a);
        else coef_fwd_lds_kernel<16, false><<<B, 256, smem, stream>>>(a);
    } else {
        const size_t smem = sizeof(float) * (32 * 32 + 64 + SkWg<32>::lds_floats(T));
        hipError_t e = precise ? allow_dynamic_lds(&coef_fwd_lds_kernel<32, true>, smem)
                               : allow_dynamic_lds(&coef_fwd_lds_kernel<32, false>, smem);
        if (e != hipSuccess) return e;
        if (agg) {
            e = allow_dynamic_lds(&coef_fwd_lds_kernel<32, false, true>, smem);
            if (e != hipSuccess) return e;
            coef_fwd_lds_kernel<32, false, true><<<B, 256, smem, stream>>>(a);
        } else if (precise) coef_fwd_lds_kernel<32, true><<<B, 256, smem, stream>>>(a);
        else coef_fwd_lds_kernel<32, false><<<B, 256, smem, stream>>>(a);
    }
    return hipGetLastError();
}

// Whether launch_coef_fwd can also produce the stream aggregate and its RMS for this shape (n > 8,
// bf16 x, one 16-byte chunk per thread and stream).  With static H every sample's workgroup then
// repeats the shared Sinkhorn chain (they run side by side: worth it while they fit the chip together).
bool coef_fwd_aggregates(int n, int C, int x_dtype) {
    return n > 8 && x_dtype == kBF16 && C % 8 == 0 && C / 8 <= 256;
}

}  // namespace mhc
