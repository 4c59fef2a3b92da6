// Stream-mixing forward: one workgroup per sample computes, in one launch,
//   a = sum_i Hpre_i x_i         (stream aggregate,   reference stream_ops.cuh:27-92, :453-526)
//   f = a / sqrt(mean(a^2)+eps) * w   (inner RMSNorm, reference rmsnorm.cuh:14-165)
//   y_i = sum_j M_ij x_j + Hpost_i f  (distribute+mix, reference stream_ops.cuh:119-152, :504-526)
// a and f never leave the chip; x is fetched from HBM once (the second sweep over the sample's
// tile hits L1/L2).  With an injected f the first sweep is skipped.
#include "launchers.h"
#include "phase_profiler.h"
#include "sinkhorn_device.h"

namespace mhc {

struct MixFwdArgs {
    const void *x, *w, *f_inject;
    void *y;
    const float *Hpre, *Hpost, *M;
    float *q;
    int hstride, w_bf16, B, n, C;
    float eps;
};

__device__ __forceinline__ float load_w(const void *w, int w_bf16, int c) {
    return w_bf16 ? bf16_to_f32(static_cast<const bf16_t *>(w)[c]) : static_cast<const float *>(w)[c];
}

template <typename TX, typename TY, int NP, int V>
__global__ __launch_bounds__(256) void mix_fwd_kernel(MixFwdArgs a) {
    extern __shared__ float smem[];
    float *a_s = smem;                 // [C] aggregate
    float *red = a_s + a.C;            // [4]
    float *M_s = red + 4;              // [NP*NP] (NP >= 16 only)
    const int b = blockIdx.x, n = a.n, C = a.C, tid = threadIdx.x, nt = blockDim.x;
    const TX *__restrict__ xb = static_cast<const TX *>(a.x) + (size_t)b * n * C;
    TY *__restrict__ yb = static_cast<TY *>(a.y) + (size_t)b * n * C;
    const float *__restrict__ Hpre = a.Hpre + (size_t)b * a.hstride;
    const float *__restrict__ Hpost = a.Hpost + (size_t)b * a.hstride;
    const float *__restrict__ M = a.M + (size_t)b * a.hstride * n;
    const bool inject = a.f_inject != nullptr;
    const int nch = C / V;

    float hpre[NP], hpost[NP];
#pragma unroll
    for (int i = 0; i < NP; i++) {
        hpre[i] = i < n ? Hpre[i] : 0.f;
        hpost[i] = i < n ? Hpost[i] : 0.f;
    }
    if constexpr (NP >= 16) {
        for (int e = tid; e < NP * NP; e += nt) {
            const int i = e / NP, j = e % NP;
            M_s[e] = (i < n && j < n) ? M[i * n + j] : 0.f;
        }
    }

    float qinv = 1.0f;
    if (!inject) {
        float ssq = 0.f;
        for (int ch = tid; ch < nch; ch += nt) {
            const int c = ch * V;
            float acc[V];
#pragma unroll
            for (int v = 0; v < V; v++) acc[v] = 0.f;
#pragma unroll
            for (int i = 0; i < NP; i++) {
                // streams >= n alias stream 0 and meet hpre = 0: no branch around the loads, so
                // all of them are in flight together
                float xv[V];
                load_vec<TX, V>(xb + (size_t)(i < n ? i : 0) * C + c, xv);
#pragma unroll
                for (int v = 0; v < V; v++) acc[v] += hpre[i] * xv[v];
            }
#pragma unroll
            for (int v = 0; v < V; v++) {
                a_s[c + v] = acc[v];
                ssq += acc[v] * acc[v];
            }
        }
        // block sum of ssq (also orders the a_s / M_s writes before the second sweep)
        ssq = wave_allreduce_sum(ssq);
        if ((tid & 63) == 0) red[tid >> 6] = ssq;
        __syncthreads();
        float tot = 0.f;
        for (int i = 0; i < (nt >> 6); i++) tot += red[i];
        const float q = sqrtf(tot / (float)C + a.eps);
        qinv = 1.0f / q;
        if (tid == 0 && a.q) a.q[b] = q;
    } else {
        if (tid == 0 && a.q) a.q[b] = 1.0f;
        __syncthreads();
    }

    for (int ch = tid; ch < nch; ch += nt) {
        const int c = ch * V;
        float f[V];
        if (inject) {
            load_vec<TX, V>(static_cast<const TX *>(a.f_inject) + (size_t)b * C + c, f);
        } else {
#pragma unroll
            for (int v = 0; v < V; v++) f[v] = a_s[c + v] * qinv * load_w(a.w, a.w_bf16, c + v);
        }
        float xv[NP][V];
#pragma unroll
        for (int j = 0; j < NP; j++) load_vec<TX, V>(xb + (size_t)(j < n ? j : 0) * C + c, xv[j]);
#pragma unroll
        for (int i = 0; i < NP; i++) {
            if (i < n) {
                float out[V];
#pragma unroll
                for (int v = 0; v < V; v++) out[v] = hpost[i] * f[v];
#pragma unroll
                for (int j = 0; j < NP; j++) {
                    float mij;
                    if constexpr (NP >= 16) mij = M_s[i * NP + j];
                    else mij = j < n ? M[i * n + j] : 0.f;
#pragma unroll
                    for (int v = 0; v < V; v++) out[v] += mij * xv[j][v];
                }
                store_vec<TY, V, true>(yb + (size_t)i * C + c, out);
            }
        }
    }
}

// =============================================================================================
// Fused layer forward for n <= 8: coefficients + mix in one launch, x read from HBM exactly once.
//
// Every workgroup first issues the loads of its sample's whole [n, C] tile (kept in registers),
// then the first lanes of wave 0 (16 for a 4x4 matrix, all 64 for 8x8) turn the projection partial
// sums (dynamic H) or the shared logits (static H) into H_pre, H_post and M - the Sinkhorn chain
// runs while the x loads are in flight - and finally all threads aggregate, normalise and mix out
// of registers.
// Replaces fused_h_activations + sinkhorn_knopp_forward_batched + stream_aggregate +
// rmsnorm_forward_with_rms + stream_distribute_mix_add of the reference
// (bindings.cu:449-477) by one kernel.
// =============================================================================================
struct LayerFwdArgs {
    const void *x, *w, *f_inject;
    void *y;
    const float *Ppart, *ssqpart;   // dynamic: [KS][B][DP], [KS][B]; static: nullptr
    const float *alpha, *b_pre, *b_post, *b_res;
    float *Hpre, *Hpost, *M, *P, *r, *q;  // outputs (static: shared [n], [n], [n,n]; may be null)
    int KS, DP, w_bf16, B, n, C, T;
    float eps;
    float *sk_state;  // dynamic: [B][T + 1][2][NP] Sinkhorn denominators kept for the backward, or nullptr
};

// The values of a loaded chunk, widened to fp32; fp32 storage that is consumed as bf16 is rounded here
// (nearest even), so that the mixing sees what the projection and the backward kernels see.
template <bool ROUND, typename T, int V>
__device__ __forceinline__ void get_act(const RawVec<T, V> &r, float (&v)[V]) {
    r.get(v);
    if constexpr (ROUND && std::is_same<T, float>::value) {
#pragma unroll
        for (int i = 0; i < V; i++) v[i] = bf16_to_f32(f32_to_bf16(v[i]));
    }
}

constexpr int kFwdStaggerMinB = 512;  // two or more workgroups per CU

// RX: fp32 x (and f) consumed as bf16, every value rounded to bf16 as it is unpacked
template <typename TX, typename TY, int NP, int V, int CPT, bool RX = false>
__global__ __launch_bounds__(256, (CPT == 2 && NP == 4 && !std::is_same<TX, float>::value) ? 4 : 1)
void layer_fwd_small_kernel(LayerFwdArgs a) {
    using SK = SkSmall<NP>;
    __shared__ float coef_s[NP * NP + 2 * NP];  // M | Hpre | Hpost
    __shared__ float red[4];
    const int b = blockIdx.x, n = a.n, C = a.C, tid = threadIdx.x;
    const int nt = blockDim.x;  // whole waves, as few as hold the sample's chunks (256 for 8x8: the four waves share the split sums)
    const TX *__restrict__ xb = static_cast<const TX *>(a.x) + (size_t)b * n * C;
    TY *__restrict__ yb = static_cast<TY *>(a.y) + (size_t)b * n * C;
    const bool inject = a.f_inject != nullptr;
    const bool dyn = a.Ppart != nullptr;
    const int nch = C / V;
    MHC_PHASE(kPhaseFwdFused, b, 0);

    // ---- 1. loads.  Wave 0 first asks for the small coefficient inputs (they return ahead of
    // the bulk data, so the Sinkhorn chain below runs while the tile is still streaming in),
    // then every thread issues the loads of the sample's whole tile. ------------------------------
    // Lane g of a group owns matrix element (r0, c0) and, for g < 2n, entry g of the vector (pre | post).
    // The K-split sums are shared four ways: by the four groups of wave 0 (4x4 matrices, combined
    // with lane swaps) or by the four waves (8x8 matrices, a whole wave per group, combined through
    // LDS); the coefficient step itself runs on the first group.
    constexpr int kSplitWaves = SK::kPerWave == 1 ? 4 : 1;
    __shared__ float psum_s[kSplitWaves == 4 ? 4 * 3 * 64 : 1];
    const int g = tid % SK::kGroup, part = (tid / SK::kGroup) % 4;
    const int D = n * n + 2 * n;
    const int r0 = SK::row(g), c0 = SK::col0(g);
    const bool mv = r0 < n && c0 < n, vv = g < 2 * n;
    float al0 = 0.f, al1 = 0.f, al2 = 0.f, bvec = 0.f, bres = 0.f;
    // 4 * SU K-splits are summed from one round of loads (proj_fwd_ksplit caps the split count to
    // match; the two-chunk variant has no registers to spare for more)
    constexpr int SU = (CPT == 1 ? 24 : 16) / 4;
    float t_ssq[SU], t_vec[SU], t_e[SU];
    const size_t ps = (size_t)a.B * a.DP;
    const float *Pb = dyn ? a.Ppart + (size_t)b * a.DP : nullptr;
    // None of these loads sits behind a per-lane branch or is touched before step 2 / step 3: out of
    // range indices alias element 0 and are discarded where the value is used.
    if (tid < 64 * kSplitWaves) {
        if (dyn) { al0 = a.alpha[0]; al1 = a.alpha[1]; al2 = a.alpha[2]; }
        bvec = g < n ? a.b_pre[g] : a.b_post[vv ? g - n : 0];
        bres = a.b_res[mv ? r0 * n + c0 : 0];
        if (dyn) {
#pragma unroll
            for (int u = 0; u < SU; u++) {  // first batch of K-split partials: ks = part*SU + u
                const int ks = part * SU + u;
                const size_t ko = ks < a.KS ? ks : 0;
                t_ssq[u] = a.ssqpart[ko * a.B + b];
                t_vec[u] = Pb[ko * ps + (vv ? g : 0)];
                t_e[u] = Pb[ko * ps + (mv ? 2 * n + r0 * n + c0 : 0)];
            }
        }
    }
    // Every second workgroup of an XCD asks for its tile only after the coefficient step: with all
    // workgroups resident at once they would otherwise move in lockstep (everybody loads, everybody
    // runs the serial Sinkhorn chain with the memory system idle, everybody stores); the two
    // halves now load and store at different times.  With about one workgroup per CU there is no such
    // contention and the delay would only cost time.
    const bool late = a.B >= kFwdStaggerMinB && ((blockIdx.x >> 3) & 1) != 0;
    RawVec<TX, V> xr[CPT][NP];
    RawVec<TX, V> fr[CPT];
    auto issue_tile = [&]() {
#pragma unroll
        for (int k = 0; k < CPT; k++) {
            const int ch = tid + k * nt;
            const TX *xc = xb + (size_t)(ch < nch ? ch : 0) * V;
#pragma unroll
            for (int i = 0; i < NP; i++) xr[k][i].load(xc + (size_t)(i < n ? i : 0) * C);
        }
        if (inject) {
#pragma unroll
            for (int k = 0; k < CPT; k++) {
                const int ch = tid + k * nt;
                fr[k].load(static_cast<const TX *>(a.f_inject) + (size_t)b * C + (size_t)(ch < nch ? ch : 0) * V);
            }
        }
    };
    if (!late) issue_tile();

    MHC_PHASE(kPhaseFwdFused, b, 1);
    // ---- 2. coefficients on wave 0 -----------------------------------------------------------
    float pe = 0.f, pvec = 0.f, ssq = 0.f;
    if (tid < 64 * kSplitWaves && dyn) {
#pragma unroll
        for (int u = 0; u < SU; u++) {
            const bool ok = part * SU + u < a.KS;
            ssq += ok ? t_ssq[u] : 0.f;
            pvec += (ok && vv) ? t_vec[u] : 0.f;
            pe += (ok && mv) ? t_e[u] : 0.f;
        }
        for (int ks0 = (4 + part) * SU; ks0 < a.KS; ks0 += 4 * SU) {  // never with proj_fwd_ksplit's cap
#pragma unroll
            for (int u = 0; u < SU; u++) {
                const int ks = ks0 + u;
                if (ks < a.KS) {
                    ssq += a.ssqpart[(size_t)ks * a.B + b];
                    if (vv) pvec += Pb[ks * ps + g];
                    if (mv) pe += Pb[ks * ps + 2 * n + r0 * n + c0];
                }
            }
        }
        if constexpr (kSplitWaves == 1) {  // the four groups of wave 0 hold a quarter of the splits each
            ssq = xor32_add(xor16_add(ssq));
            pvec = xor32_add(xor16_add(pvec));
            pe = xor32_add(xor16_add(pe));
        } else {
            psum_s[(part * 3 + 0) * 64 + g] = ssq;
            psum_s[(part * 3 + 1) * 64 + g] = pvec;
            psum_s[(part * 3 + 2) * 64 + g] = pe;
        }
    }
    if constexpr (kSplitWaves == 4) {
        if (dyn) {  // uniform over the workgroup
            __syncthreads();
            if (tid < 64) {
                ssq = (psum_s[0 * 64 + g] + psum_s[3 * 64 + g]) + (psum_s[6 * 64 + g] + psum_s[9 * 64 + g]);
                pvec = (psum_s[1 * 64 + g] + psum_s[4 * 64 + g]) + (psum_s[7 * 64 + g] + psum_s[10 * 64 + g]);
                pe = (psum_s[2 * 64 + g] + psum_s[5 * 64 + g]) + (psum_s[8 * 64 + g] + psum_s[11 * 64 + g]);
            }
        }
    }
    if (tid < 64) {
        MHC_PHASE(kPhaseFwdFused, b, 2);
        if (tid < SK::kGroup) {
            // bf16 tier: hardware exp2 / reciprocal / square root (1 ulp) instead of the library routines
            constexpr bool kFast = !std::is_same<TX, float>::value;
            float rinv = 0.f;
            if (dyn) {
                const float ms = ssq * (1.0f / (float)(n * C)) + a.eps;
                const float r = kFast ? __builtin_amdgcn_sqrtf(ms) : sqrtf(ssq / (float)(n * C) + a.eps);
                rinv = kFast ? fast_rcp(r) : 1.0f / r;
                if (g == 0) a.r[b] = r;
            }
            const bool wr = dyn || b == 0;  // static coefficients are written once
            const size_t hs = dyn ? (size_t)b * n : 0, ms = dyn ? (size_t)b * n * n : 0;
            if (vv) {
                const bool pre = g < n;
                const int gi = pre ? g : g - n;
                const float p = pvec * rinv;
                // one sigmoid for both kinds of lane (two would run one after the other)
                const float z = (pre ? al0 : al1) * p + bvec;
                const float sg = kFast ? sigmoid_fast(z) : sigmoidf_acc(z);
                const float h = pre ? sg : 2.0f * sg;
                coef_s[NP * NP + (pre ? 0 : NP) + gi] = h;
                float *dst = pre ? a.Hpre : a.Hpost;
                if (wr && dst) dst[hs + gi] = h;
                if (dyn) a.P[(size_t)b * D + g] = p;
            } else if (g < 2 * NP) {
                // the padded entries of Hpre and Hpost: 2 (NP - n) slots, taken by lanes 2n .. 2NP-1
                const int k = g - 2 * n;
                coef_s[NP * NP + (k < NP - n ? n + k : NP + n + (k - (NP - n)))] = 0.f;
            }
            float m[1];
            if (mv) {
                const float p = pe * rinv;
                if (dyn) a.P[(size_t)b * D + 2 * n + r0 * n + c0] = p;
                m[0] = kFast ? exp_fast(al2 * p + bres) : expf(al2 * p + bres);
            } else {
                m[0] = 0.f;
            }
            // kept denominators: the fp32 tier divides, so that the backward call can undo the
            // scalings (m * s * rho) without a bias that grows with the iteration count
            // (the same arithmetic with and without the state: the dynamic forward result does not depend
            // on whether the caller keeps it; static H has no state to undo and takes the reciprocals)
            if (dyn && a.sk_state) SK::template forward_save<!kFast>(m, g, n, a.T, a.eps, a.sk_state + (size_t)b * SK::state_floats(a.T));
            else if (dyn) SK::template forward<!kFast, false>(m, g, n, a.T, a.eps, nullptr, tid);
            else SK::template forward<false, false>(m, g, n, a.T, a.eps, nullptr, tid);
            coef_s[r0 * NP + c0] = m[0];
            if (wr && a.M && mv) a.M[ms + r0 * n + c0] = m[0];
        }
    }
    MHC_PHASE(kPhaseFwdFused, b, 3);
    if (late) issue_tile();
    __syncthreads();
    MHC_PHASE(kPhaseFwdFused, b, 4);
    float hpre[NP], hpost[NP], Mr[NP][NP];
#pragma unroll
    for (int i = 0; i < NP; i++) {
        hpre[i] = coef_s[NP * NP + i];
        hpost[i] = coef_s[NP * NP + NP + i];
#pragma unroll
        for (int j = 0; j < NP; j++) Mr[i][j] = coef_s[i * NP + j];
    }

    // bf16 x: the per-sample n x n products of steps 3 and 4 run on v_mfma_f32_4x4x4_16b_bf16 (a block
    // = four consecutive lanes, all of the same sample here): the B column of a lane is four streams
    // of one of its channels (two v_perm_b32), the A rows are the sample's coefficients (bf16 value
    // + remainder), the lane receives four output streams of its own channel; for n > 4 the streams
    // form two groups of four and M is 2 x 2 such blocks.  With the products on the VALU this kernel
    // is bound by VALU issue once several workgroups share a CU.
    constexpr bool kMixMfma = std::is_same<TX, bf16_t>::value && V == 8;
    if constexpr (kMixMfma) {
        constexpr int NB = NP / 4;  // stream groups
        const int jq = tid & 3;
        CoefRow cm[NB][NB], ca[NB];  // rows 4J + jq of M, columns 4I ..; [Hpre; 0; 0; 0]
        const bool r0 = jq == 0;
#pragma unroll
        for (int I = 0; I < NB; I++) {
#pragma unroll
            for (int J = 0; J < NB; J++) {
                const float *mr = coef_s + (4 * J + jq) * NP + 4 * I;
                cm[J][I].set(mr[0], mr[1], mr[2], mr[3]);
            }
            ca[I].set(r0 ? hpre[4 * I] : 0.f, r0 ? hpre[4 * I + 1] : 0.f, r0 ? hpre[4 * I + 2] : 0.f,
                      r0 ? hpre[4 * I + 3] : 0.f);
        }
        const f32x4_t zero = {0.f, 0.f, 0.f, 0.f};
        // B operand: streams 4I .. 4I+3 of channel v = 2p + odd of chunk k, p = word of the channel pair
        auto channel = [&](int k, int v, int I) {
            const int p = v >> 1;
            const uint32_t w0 = xr[k][4 * I].w[p], w1 = xr[k][4 * I + 1].w[p], w2 = xr[k][4 * I + 2].w[p],
                           w3 = xr[k][4 * I + 3].w[p];
            return (v & 1) ? streams_of_channel<true>(w0, w1, w2, w3) : streams_of_channel<false>(w0, w1, w2, w3);
        };
        // aggregate of four channels: register 0 of da[v]
        auto aggregate4 = [&](const bf16x4_t (&bx)[NB][4], f32x4_t (&da)[4]) {
#pragma unroll
            for (int v = 0; v < 4; v++) da[v] = mfma4(ca[0].hi, bx[0][v], zero);
#pragma unroll
            for (int v = 0; v < 4; v++) da[v] = mfma4(ca[0].lo, bx[0][v], da[v]);
#pragma unroll
            for (int I = 1; I < NB; I++) {
#pragma unroll
                for (int v = 0; v < 4; v++) da[v] = mfma4(ca[I].hi, bx[I][v], da[v]);
#pragma unroll
                for (int v = 0; v < 4; v++) da[v] = mfma4(ca[I].lo, bx[I][v], da[v]);
            }
        };
        // ---- 3. aggregate + RMS ----------------------------------------------------------------
        // (four channels at a time keep the accumulators small; the aggregate is formed again in
        // step 4 instead of being kept across the barrier: a few cheap instructions per half chunk)
        float qinv = 1.0f;
        if (!inject) {
            float ssq = 0.f;
#pragma unroll
            for (int k = 0; k < CPT; k++) {
                const bool live = tid + k * nt < nch;  // chunks beyond C alias chunk 0: not counted
#pragma unroll
                for (int h = 0; h < 2; h++) {
                    bf16x4_t bx[NB][4];
#pragma unroll
                    for (int I = 0; I < NB; I++)
#pragma unroll
                        for (int v = 0; v < 4; v++) bx[I][v] = channel(k, 4 * h + v, I);
                    f32x4_t da[4];
                    aggregate4(bx, da);
#pragma unroll
                    for (int v = 0; v < 4; v++) ssq += live ? da[v][0] * da[v][0] : 0.f;
                }
            }
            ssq = block_allreduce_sum(ssq, red, nt / kWave);
            const float q = sqrtf(ssq / (float)C + a.eps);
            qinv = 1.0f / q;
            if (tid == 0 && a.q) a.q[b] = q;
        } else if (tid == 0 && a.q) {
            a.q[b] = 1.0f;
        }
        MHC_PHASE(kPhaseFwdFused, b, 5);
        // ---- 4. mix + distribute -----------------------------------------------------------------
#pragma unroll
        for (int k = 0; k < CPT; k++) {
            const int ch = tid + k * nt;
            const int c = (ch < nch ? ch : 0) * V;
            float f[V];
            if (inject) {
                get_act<RX>(fr[k], f);
            } else {
                if (a.w_bf16) load_vec<bf16_t, V>(static_cast<const bf16_t *>(a.w) + c, f);
                else load_vec<float, V>(static_cast<const float *>(a.w) + c, f);
            }
            uint32_t yw[NP][2];  // packed first half (bf16 output), stored with the second
            float yf[NP][4];     // first half (fp32 output)
#pragma unroll
            for (int h = 0; h < 2; h++) {
                bf16x4_t bx[NB][4];
#pragma unroll
                for (int I = 0; I < NB; I++)
#pragma unroll
                    for (int v = 0; v < 4; v++) bx[I][v] = channel(k, 4 * h + v, I);
                f32x4_t d[NB][4], da[4];
#pragma unroll
                for (int J = 0; J < NB; J++) {
#pragma unroll
                    for (int v = 0; v < 4; v++) d[J][v] = mfma4(cm[J][0].hi, bx[0][v], zero);
#pragma unroll
                    for (int v = 0; v < 4; v++) d[J][v] = mfma4(cm[J][0].lo, bx[0][v], d[J][v]);
#pragma unroll
                    for (int I = 1; I < NB; I++) {
#pragma unroll
                        for (int v = 0; v < 4; v++) d[J][v] = mfma4(cm[J][I].hi, bx[I][v], d[J][v]);
#pragma unroll
                        for (int v = 0; v < 4; v++) d[J][v] = mfma4(cm[J][I].lo, bx[I][v], d[J][v]);
                    }
                }
                float fh[4];
                if (inject) {
#pragma unroll
                    for (int v = 0; v < 4; v++) fh[v] = f[4 * h + v];
                } else {
                    aggregate4(bx, da);
#pragma unroll
                    for (int v = 0; v < 4; v++) fh[v] = da[v][0] * qinv * f[4 * h + v];
                }
#pragma unroll
                for (int i = 0; i < NP; i++) {
                    const int J = i >> 2, r = i & 3;
                    const float o0 = d[J][0][r] + hpost[i] * fh[0], o1 = d[J][1][r] + hpost[i] * fh[1];
                    const float o2 = d[J][2][r] + hpost[i] * fh[2], o3 = d[J][3][r] + hpost[i] * fh[3];
                    if constexpr (std::is_same<TY, bf16_t>::value) {
                        if (h == 0) {
                            yw[i][0] = pack_bf16x2(o0, o1); yw[i][1] = pack_bf16x2(o2, o3);
                        } else if (i < n && ch < nch) {
                            st16<true>(yb + (size_t)i * C + c, yw[i][0], yw[i][1], pack_bf16x2(o0, o1), pack_bf16x2(o2, o3));
                        }
                    } else {
                        if (h == 0) {
                            yf[i][0] = o0; yf[i][1] = o1; yf[i][2] = o2; yf[i][3] = o3;
                        } else if (i < n && ch < nch) {
                            const float out[V] = {yf[i][0], yf[i][1], yf[i][2], yf[i][3], o0, o1, o2, o3};
                            store_vec<TY, V, true>(yb + (size_t)i * C + c, out);
                        }
                    }
                }
            }
        }
    } else {
        // ---- 3. aggregate + RMS ------------------------------------------------------------------
        // (VALU path: fp32 x, n > 4, or rows not a multiple of 8.)  The tile stays in registers as raw
        // words; LEAN (two chunks per thread) widens a stream at the point of use instead of holding
        // the fp32 copy of the whole tile, which keeps the register count down; the extra
        // conversions are cheaper than a second round of the grid.
        constexpr bool LEAN = CPT >= 2 && NP <= 4 && !std::is_same<TX, float>::value;
        float xv[LEAN ? 1 : CPT][NP][V];
        if constexpr (!LEAN) {
#pragma unroll
            for (int k = 0; k < CPT; k++)
#pragma unroll
                for (int i = 0; i < NP; i++) get_act<RX>(xr[k][i], xv[k][i]);  // streams >= n meet zero coefficients
        }
        float av[LEAN ? 1 : CPT][V];  // LEAN recomputes the aggregate in step 4 instead of keeping it
        float qinv = 1.0f;
        if (!inject) {
            float ssq = 0.f;
#pragma unroll
            for (int k = 0; k < CPT; k++) {
                const bool live = tid + k * nt < nch;  // chunks beyond C alias chunk 0: not counted
                float s_a[V];
#pragma unroll
                for (int v = 0; v < V; v++) s_a[v] = 0.f;
#pragma unroll
                for (int i = 0; i < NP; i++) {
                    float t[V];
                    if constexpr (LEAN) get_act<RX>(xr[k][i], t);
#pragma unroll
                    for (int v = 0; v < V; v++) s_a[v] += hpre[i] * (LEAN ? t[v] : xv[LEAN ? 0 : k][i][v]);
                }
#pragma unroll
                for (int v = 0; v < V; v++) {
                    if constexpr (!LEAN) av[k][v] = s_a[v];
                    ssq += live ? s_a[v] * s_a[v] : 0.f;
                }
            }
            ssq = block_allreduce_sum(ssq, red, nt / kWave);
            const float q = sqrtf(ssq / (float)C + a.eps);
            qinv = 1.0f / q;
            if (tid == 0 && a.q) a.q[b] = q;
        } else if (tid == 0 && a.q) {
            a.q[b] = 1.0f;
        }

        MHC_PHASE(kPhaseFwdFused, b, 5);
        // ---- 4. mix + distribute -------------------------------------------------------------------
#pragma unroll
        for (int k = 0; k < CPT; k++) {
            const int ch = tid + k * nt;
            if (ch < nch) {
                const int c = ch * V;
                float f[V];
                if (inject) {
                    get_act<RX>(fr[k], f);
                } else {
                    if constexpr (LEAN) {
#pragma unroll
                        for (int v = 0; v < V; v++) f[v] = 0.f;
#pragma unroll
                        for (int i = 0; i < NP; i++) {
                            float t[V];
                            get_act<RX>(xr[k][i], t);
#pragma unroll
                            for (int v = 0; v < V; v++) f[v] += hpre[i] * t[v];
                        }
#pragma unroll
                        for (int v = 0; v < V; v++) f[v] = f[v] * qinv * load_w(a.w, a.w_bf16, c + v);
                    } else {
#pragma unroll
                        for (int v = 0; v < V; v++) f[v] = av[k][v] * qinv * load_w(a.w, a.w_bf16, c + v);
                    }
                }
#pragma unroll
                for (int i = 0; i < NP; i++) {
                    if (i < n) {
                        float out[V];
#pragma unroll
                        for (int v = 0; v < V; v++) out[v] = hpost[i] * f[v];
#pragma unroll
                        for (int j = 0; j < NP; j++) {
                            float t[V];
                            if constexpr (LEAN) get_act<RX>(xr[k][j], t);
                            const float mij = LEAN ? coef_s[i * NP + j] : Mr[i][j];
#pragma unroll
                            for (int v = 0; v < V; v++) out[v] += mij * (LEAN ? t[v] : xv[LEAN ? 0 : k][j][v]);
                        }
                        store_vec<TY, V, true>(yb + (size_t)i * C + c, out);
                    }
                }
            }
        }
    }
    MHC_PHASE(kPhaseFwdFused, b, 6);
}

// Largest CPT instantiated: tiles with more than 4 * 256 vector chunks per stream take the
// two-kernel path (coefficient kernel + streaming mix kernel).
template <typename TX, typename TY, int NP, bool RX = false>
static bool launch_fused_small(const LayerFwdArgs &a, hipStream_t stream, hipError_t *err) {
    constexpr int V = 16 / (int)sizeof(TX);
    if (a.C % V != 0) return false;
    const int nch = a.C / V;
    const int cpt = (nch + 255) / 256;
    // as few whole waves as hold the chunks: a thread without a chunk of its own still runs the loads
    // and the arithmetic on an aliased one (320 chunks on 2 x 256 slots would waste 37 % of both)
    const int per = cpt == 3 ? 4 : cpt;  // chunks per thread of the instantiation that runs
    const int nt = NP == 8 ? 256 : round_up((nch + per - 1) / per, kWave);
    if (cpt == 1) layer_fwd_small_kernel<TX, TY, NP, V, 1, RX><<<a.B, nt, 0, stream>>>(a);
    else if (cpt == 2) layer_fwd_small_kernel<TX, TY, NP, V, 2, RX><<<a.B, nt, 0, stream>>>(a);
    else if (cpt <= 4 && NP == 4) layer_fwd_small_kernel<TX, TY, 4, V, 4, RX><<<a.B, nt, 0, stream>>>(a);
    else return false;
    *err = hipGetLastError();
    return true;
}

bool layer_fwd_fused_supported(int n, int C, int x_dtype) {
    if (n > 8) return false;
    const int V = x_dtype == kBF16 ? 8 : 4;
    if (C % V != 0) return false;
    const int cpt = (C / V + 255) / 256;
    return cpt <= 2 || (cpt <= 4 && n <= 4);
}

hipError_t launch_layer_fwd_fused(const void *x, int x_dtype, const void *w, int w_dtype,
                                  const void *f_inject, void *y, int y_dtype, const float *Ppart,
                                  const float *ssqpart, int KS, int DP, const float *alpha,
                                  const float *b_pre, const float *b_post, const float *b_res,
                                  float *Hpre, float *Hpost, float *M, float *P, float *r, float *q,
                                  float *sk_state, int B, int n, int C, int T, float eps, hipStream_t stream) {
    LayerFwdArgs a{x, w, f_inject, y, Ppart, ssqpart, alpha, b_pre, b_post, b_res, Hpre, Hpost, M, P, r, q,
                   KS, DP, w_dtype == kBF16, B, n, C, T, eps, sk_state};
    hipError_t err = hipErrorInvalidValue;
    bool ok = false;
#define MHC_FUSED(TX, TY)                                                        \
    ok = n <= 4 ? launch_fused_small<TX, TY, 4>(a, stream, &err) : launch_fused_small<TX, TY, 8>(a, stream, &err)
    if (x_dtype == kF32 && y_dtype == kF32) MHC_FUSED(float, float);
    else if (x_dtype == kF32AsBF16 && y_dtype == kF32)  // fp32 storage, values rounded to bf16 on the way in
        ok = n <= 4 ? launch_fused_small<float, float, 4, true>(a, stream, &err)
                    : launch_fused_small<float, float, 8, true>(a, stream, &err);
    else if (x_dtype == kBF16 && y_dtype == kBF16) MHC_FUSED(bf16_t, bf16_t);
    else if (x_dtype == kBF16 && y_dtype == kF32) MHC_FUSED(bf16_t, float);
#undef MHC_FUSED
    return ok ? err : hipErrorInvalidValue;
}

// =============================================================================================
// n > 8, bf16 x: the mix on the matrix cores, in two launches.
//   agg_large_kernel       one workgroup per sample: a = Hpre^T x (fp32, to scratch) and q
//   mix_fwd_large_kernel   workgroup = (128-channel block, sample): y = M x + Hpost (x) f with
//                          A = M as a bf16 pair (rounded value + remainder), B = the x tile read
//                          back transposed from LDS (the contraction runs over streams); the
//                          result goes through LDS to a row-major epilogue with 16-byte stores.
// =============================================================================================
typedef __attribute__((__vector_size__(8 * sizeof(__bf16)))) __bf16 bf16x8_t;
typedef __attribute__((__vector_size__(16 * sizeof(float)))) float f32x16_t;

struct MixLargeArgs {
    const bf16_t *x;
    const void *w;
    const bf16_t *f_inject;
    void *y;
    const float *Hpre, *Hpost, *M;
    float *q, *a_ws;  // a_ws: [B, C] fp32 aggregate (unused with an injected f)
    int hstride, w_bf16, B, n, C;
    float eps;
};

__global__ __launch_bounds__(256) void agg_large_kernel(MixLargeArgs a) {
    __shared__ float hp_s[32];
    __shared__ float red[4];
    const int b = blockIdx.x, n = a.n, C = a.C, tid = threadIdx.x;
    const bf16_t *xb = a.x + (size_t)b * n * C;
    if (tid < 32) hp_s[tid] = tid < n ? a.Hpre[(size_t)b * a.hstride + tid] : 0.f;
    __syncthreads();
    float ssq = 0.f;
    for (int ch = tid; ch < C / 8; ch += 256) {
        float acc[8];
#pragma unroll
        for (int v = 0; v < 8; v++) acc[v] = 0.f;
#pragma unroll
        for (int i0 = 0; i0 < 32; i0 += 16) {  // 16 loads in flight; streams >= n alias stream 0
            RawVec<bf16_t, 8> xr[16];
#pragma unroll
            for (int u = 0; u < 16; u++) xr[u].load(xb + (size_t)(i0 + u < n ? i0 + u : 0) * C + ch * 8);
#pragma unroll
            for (int u = 0; u < 16; u++) {
                float xv[8];
                xr[u].get(xv);
                const float hp = hp_s[i0 + u];
#pragma unroll
                for (int v = 0; v < 8; v++) acc[v] += hp * xv[v];
            }
        }
        store_vec<float, 8>(a.a_ws + (size_t)b * C + ch * 8, acc);
#pragma unroll
        for (int v = 0; v < 8; v++) ssq += acc[v] * acc[v];
    }
    ssq = block_allreduce_sum<256>(ssq, red);
    if (tid == 0) a.q[b] = sqrtf(ssq / (float)C + a.eps);
}

constexpr int kMflCB = 128;           // channels per workgroup
constexpr int kMflLDT = kMflCB + 8;   // LDS pitch of the bf16 tile (elements)
constexpr int kMflLDO = kMflCB + 4;   // LDS pitch of the fp32 output tile

template <typename TY>
__global__ __launch_bounds__(256) void mix_fwd_large_kernel(MixLargeArgs a) {
    extern __shared__ __align__(16) unsigned char mfl_smem[];
    bf16_t *x_s = reinterpret_cast<bf16_t *>(mfl_smem);          // [32][LDT]
    float *o_s = reinterpret_cast<float *>(x_s + 32 * kMflLDT);  // [32][LDO]
    float *ho_s = o_s + 32 * kMflLDO;                            // [32] Hpost (0 beyond n)
    float *m_s = ho_s + 32;                                      // [32][33] M (0 beyond n x n)
    // linear workgroup id = sample * column blocks + column block (one grid dimension: no bound on B)
    const int ncb = (a.C + kMflCB - 1) / kMflCB;
    const int b = blockIdx.x / ncb, cblk = blockIdx.x % ncb;
    const int cb0 = cblk * kMflCB, n = a.n, C = a.C, tid = threadIdx.x;
    const int lane = tid & 63, wave = tid >> 6, row = lane & 31, kh = lane >> 5;
    const bool inject = a.f_inject != nullptr;
    const bf16_t *xb = a.x + (size_t)b * n * C;
    const float *M = a.M + (size_t)b * a.hstride * n;

    // tile loads: thread owns row tid / 8, 16-byte chunks tid % 8 and tid % 8 + 8
    const int trow = tid >> 3;
    RawVec<bf16_t, 8> xr[2];
    bool cok[2];
#pragma unroll
    for (int h = 0; h < 2; h++) {
        const int c = cb0 + ((tid & 7) + 8 * h) * 8;
        cok[h] = c < C;  // C % 8 == 0
        xr[h].load(xb + (size_t)(trow < n ? trow : 0) * C + (cok[h] ? c : 0));
    }
    // M through LDS: the operand layout below has every lane on a different row of M, which is the
    // slow way to read global memory; here 8 lanes share a row (128 contiguous bytes)
    float mraw[4];
#pragma unroll
    for (int i = 0; i < 4; i++) {
        const int k = (tid & 7) * 4 + i;
        mraw[i] = M[(trow < n && k < n) ? trow * n + k : 0];
    }
    if (tid < 32) ho_s[tid] = tid < n ? a.Hpost[(size_t)b * a.hstride + tid] : 0.f;
#pragma unroll
    for (int i = 0; i < 4; i++) {
        const int k = (tid & 7) * 4 + i;
        m_s[trow * 33 + k] = (trow < n && k < n) ? mraw[i] : 0.f;
    }
    if (inject && a.q && cblk == 0 && tid == 0) a.q[b] = 1.0f;  // q is defined as 1 with an injected f
    // f of this lane's channel in the matrix-core phase
    const int cw = cb0 + wave * 32 + row;
    float f = 0.f;
    if (cw < C) {
        if (inject) f = bf16_to_f32(a.f_inject[(size_t)b * C + cw]);
        else f = a.a_ws[(size_t)b * C + cw] * load_w(a.w, a.w_bf16, cw) / a.q[b];
    }
#pragma unroll
    for (int h = 0; h < 2; h++)
        *reinterpret_cast<uint4 *>(x_s + trow * kMflLDT + ((tid & 7) + 8 * h) * 8) =
            make_uint4(xr[h].w[0], xr[h].w[1], xr[h].w[2], xr[h].w[3]);
    __syncthreads();

    // A operand: lane (row i, kg) holds M[i][k], k = ks*16 + kg*8 .. +8, as a bf16 pair
    bf16x8_t mh[2], ml[2];
#pragma unroll
    for (int ks = 0; ks < 2; ks++) {
        float mv[8], lo[8];
        uint32_t hw[4];
#pragma unroll
        for (int i = 0; i < 8; i++) mv[i] = m_s[row * 33 + ks * 16 + kh * 8 + i];
#pragma unroll
        for (int i = 0; i < 4; i++) {
            hw[i] = pack_bf16x2(mv[2 * i], mv[2 * i + 1]);
            lo[2 * i] = mv[2 * i] - bf16lo_to_f32(hw[i]);
            lo[2 * i + 1] = mv[2 * i + 1] - bf16hi_to_f32(hw[i]);
        }
        mh[ks] = __builtin_bit_cast(bf16x8_t, make_uint4(hw[0], hw[1], hw[2], hw[3]));
        ml[ks] = __builtin_bit_cast(bf16x8_t, make_uint4(pack_bf16x2(lo[0], lo[1]), pack_bf16x2(lo[2], lo[3]),
                                                         pack_bf16x2(lo[4], lo[5]), pack_bf16x2(lo[6], lo[7])));
    }
    f32x16_t o;
#pragma unroll
    for (int i = 0; i < 16; i++) o[i] = 0.f;
#pragma unroll
    for (int ks = 0; ks < 2; ks++) {
        // B fragment: lane (c, kg) gets x[ks*16 + kg*8 + i][c], i = 0..7
        const bf16x8_t xf = __builtin_bit_cast(bf16x8_t, lds_frag_tr(x_s, kMflLDT, ks * 16, wave * 32, lane));
        o = __builtin_amdgcn_mfma_f32_32x32x16_bf16(mh[ks], xf, o, 0, 0, 0);
        o = __builtin_amdgcn_mfma_f32_32x32x16_bf16(ml[ks], xf, o, 0, 0, 0);
    }
    // accumulator layout: column = lane & 31, register i -> row 8*(i/4) + 4*(lane/32) + i%4
#pragma unroll
    for (int i = 0; i < 16; i++) {
        const int r = 8 * (i >> 2) + 4 * kh + (i & 3);
        o_s[r * kMflLDO + wave * 32 + row] = o[i] + ho_s[r] * f;
    }
    __syncthreads();
    if (trow < n) {
        TY *yb = static_cast<TY *>(a.y) + (size_t)b * n * C + (size_t)trow * C + cb0;
#pragma unroll
        for (int h = 0; h < 2; h++) {
            if (cok[h]) {
                const int co = ((tid & 7) + 8 * h) * 8;
                const float4 o0 = *reinterpret_cast<const float4 *>(o_s + trow * kMflLDO + co);
                const float4 o1 = *reinterpret_cast<const float4 *>(o_s + trow * kMflLDO + co + 4);
                const float out[8] = {o0.x, o0.y, o0.z, o0.w, o1.x, o1.y, o1.z, o1.w};
                store_vec<TY, 8, true>(yb + co, out);
            }
        }
    }
}

static hipError_t launch_large_mfma(const MixLargeArgs &a, int y_dtype, bool have_agg, hipStream_t stream) {
    if (!a.f_inject && !have_agg) {
        agg_large_kernel<<<a.B, 256, 0, stream>>>(a);
        hipError_t e = hipGetLastError();
        if (e != hipSuccess) return e;
    }
    const size_t smem = sizeof(bf16_t) * 32 * kMflLDT + sizeof(float) * (32 * kMflLDO + 32 + 32 * 33);
    const unsigned grid = (unsigned)((a.C + kMflCB - 1) / kMflCB) * (unsigned)a.B;
    if (y_dtype == kBF16) mix_fwd_large_kernel<bf16_t><<<grid, 256, smem, stream>>>(a);
    else mix_fwd_large_kernel<float><<<grid, 256, smem, stream>>>(a);
    return hipGetLastError();
}

bool mix_fwd_large_supported(int n, int C, int x_dtype) { return n > 8 && x_dtype == kBF16 && C % 8 == 0; }

template <typename TX, typename TY, int NP, int V>
static hipError_t launch_one(const MixFwdArgs &a, hipStream_t stream) {
    const int nch = a.C / V;
    int nt = (nch + 63) / 64 * 64;
    if (nt > 256) nt = 256;
    const size_t smem = sizeof(float) * (a.C + 4 + (NP >= 16 ? NP * NP : 0));
    mix_fwd_kernel<TX, TY, NP, V><<<a.B, nt, smem, stream>>>(a);
    return hipGetLastError();
}

template <typename TX, typename TY, int NP>
static hipError_t launch_np(const MixFwdArgs &a, hipStream_t stream) {
    // widest vector that keeps the per-thread tile in registers; scalar path for ragged C
    constexpr int VMAX = (NP <= 8 ? 16 : (NP == 16 ? 8 : 4)) / (int)sizeof(TX) > 0
                             ? (NP <= 8 ? 16 : (NP == 16 ? 8 : 4)) / (int)sizeof(TX) : 1;
    if (a.C % VMAX == 0) return launch_one<TX, TY, NP, VMAX>(a, stream);
    return launch_one<TX, TY, NP, 1>(a, stream);
}

template <typename TX, typename TY>
static hipError_t launch_t(const MixFwdArgs &a, hipStream_t stream) {
    if (a.n <= 4) return launch_np<TX, TY, 4>(a, stream);
    if (a.n <= 8) return launch_np<TX, TY, 8>(a, stream);
    if (a.n <= 16) return launch_np<TX, TY, 16>(a, stream);
    return launch_np<TX, TY, 32>(a, stream);
}

hipError_t launch_mix_fwd(const void *x, int x_dtype, const void *w, int w_dtype,
                          const void *f_inject, void *y, int y_dtype, const float *Hpre,
                          const float *Hpost, const float *M, int hstride, float *q, float *a_ws,
                          int B, int n, int C, float eps, bool have_agg, hipStream_t stream) {
    if (mix_fwd_large_supported(n, C, x_dtype) && (f_inject || (a_ws && q))) {
        MixLargeArgs la{static_cast<const bf16_t *>(x), w, static_cast<const bf16_t *>(f_inject), y, Hpre, Hpost,
                        M, q, a_ws, hstride, w_dtype == kBF16, B, n, C, eps};
        return launch_large_mfma(la, y_dtype, have_agg, stream);
    }
    MixFwdArgs a{x, w, f_inject, y, Hpre, Hpost, M, q, hstride, w_dtype == kBF16, B, n, C, eps};
    if (x_dtype == kF32 && y_dtype == kF32) return launch_t<float, float>(a, stream);
    if (x_dtype == kBF16 && y_dtype == kBF16) return launch_t<bf16_t, bf16_t>(a, stream);
    if (x_dtype == kBF16 && y_dtype == kF32) return launch_t<bf16_t, float>(a, stream);
    return hipErrorInvalidValue;
}

}  // namespace mhc
