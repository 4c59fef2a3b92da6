// Backward, first launch: every reduction over the channel axis of one sample, plus (dynamic H)
// the whole coefficient backward, in a single workgroup per sample.
//
//   dM[i,j]   = sum_c dy[i,c] x[j,c]          reference stream_ops.cuh:852-927
//   dHpost[i] = sum_c dy[i,c] f[c]            reference stream_ops.cuh:852-927
//   dHpre[j]  = sum_c da[c] x[j,c]            reference stream_ops.cuh:665-703
//   with df = Hpost . dy, da = df w / q - a s1 / (C q^3), s1 = sum_c df w a   (rmsnorm.cuh:234-294)
// da needs s1, a full reduction; writing dHpre = A1/q - s1 A2/(C q^3) with
// A1[j] = sum_c df w x[j,c] and A2[j] = sum_c a x[j,c] lets everything be accumulated in ONE sweep.
// Dynamic H then continues in the same kernel: sigmoid derivatives, exact Sinkhorn backward
// (reference ops.py:297-317 and sinkhorn_knopp.cuh:587-690, which is approximate and not
// followed), and dP = dt alpha / r, cx = sum_d dt alpha p / (nC r^2)  (ops.py:327-349).
//
// Two layouts: n <= 8 keeps n^2+3n+1 running sums per thread (thread = column chunk);
// n > 8 computes three 32x32 Gram matrices per sample on the matrix cores (operands loaded from
// global memory in MFMA layout) from which all the sums above follow.
#include "coef_bwd_small.h"
#include "dx_large.h"
#include "tuning.h"

namespace mhc {

typedef __attribute__((__vector_size__(8 * sizeof(__bf16)))) __bf16 bf16x8_t;
typedef __attribute__((__vector_size__(16 * sizeof(float)))) float f32x16_t;


// =============================================================================================
// n <= 8
// =============================================================================================
template <typename TG, typename TX, int NP, int V>
__global__ __launch_bounds__(256) void mix_bwd_reduce_small_kernel(BwdReduceArgs a) {
    using SK = SkSmall<NP>;
    constexpr int K = NP * NP + 3 * NP + 1;  // dM | dHpost | A1 | A2 | s1
    extern __shared__ float smem[];
    float *slot_s = smem;          // [K][16]  one slot per 16-lane row of the workgroup
    float *tot = slot_s + K * 16;  // [K]
    float *sc = tot + K;           // Sinkhorn denominators, SK::scaling_floats(T)
    const int b = blockIdx.x, n = a.n, C = a.C, tid = threadIdx.x, nt = blockDim.x;
    const TG *__restrict__ gb = static_cast<const TG *>(a.dy) + (size_t)b * n * C;
    const TX *__restrict__ xb = static_cast<const TX *>(a.x) + (size_t)b * n * C;
    const float *__restrict__ Hpre = a.Hpre + (size_t)b * a.hstride;
    const float *__restrict__ Hpost = a.Hpost + (size_t)b * a.hstride;
    const bool inject = a.f_inject != nullptr;
    // q is only requested here: a division in front of the loop would make the wave wait for this
    // round trip before it asks for its data; 1/q is applied to the sums behind the loop instead
    const float qraw = inject ? 1.0f : a.q[b];

    float hpre[NP], hpost[NP];
#pragma unroll
    for (int i = 0; i < NP; i++) {
        hpre[i] = i < n ? Hpre[i] : 0.f;
        hpost[i] = i < n ? Hpost[i] : 0.f;
    }
    float acc[K];
#pragma unroll
    for (int k = 0; k < K; k++) acc[k] = 0.f;

    const int nch = C / V;
    const int part = blockIdx.y, cpp = (nch + a.parts - 1) / a.parts;  // chunks per part
    const int ch_end = min(nch, (part + 1) * cpp);
    for (int ch = part * cpp + tid; ch < ch_end; ch += nt) {
        const int c = ch * V;
        float gv[NP][V], xv[NP][V];
#pragma unroll
        for (int i = 0; i < NP; i++) {
            // streams >= n alias stream 0 (no branch around the loads): their sums land in entries
            // of acc that nobody reads, and they meet zero coefficients everywhere else
            const size_t so = (size_t)(i < n ? i : 0) * C + c;
            load_vec<TG, V>(gb + so, gv[i]);
            load_vec<TX, V>(xb + so, xv[i]);
        }
        float av[V], fv[V], dfw[V];
        if (inject) load_vec<TX, V>(static_cast<const TX *>(a.f_inject) + (size_t)b * C + c, fv);
#pragma unroll
        for (int v = 0; v < V; v++) {
            float s_a = 0.f, s_df = 0.f;
#pragma unroll
            for (int i = 0; i < NP; i++) { s_a += hpre[i] * xv[i][v]; s_df += hpost[i] * gv[i][v]; }
            av[v] = s_a;
            if (inject) {
                dfw[v] = 0.f;
            } else {
                const float wv = load_w_(a.w, a.w_bf16, c + v);
                fv[v] = s_a * wv;  // f * q
                dfw[v] = s_df * wv;
            }
            acc[K - 1] += dfw[v] * s_a;
        }
#pragma unroll
        for (int i = 0; i < NP; i++) {
#pragma unroll
            for (int v = 0; v < V; v++) {
                acc[NP * NP + i] += gv[i][v] * fv[v];
                acc[NP * NP + NP + i] += dfw[v] * xv[i][v];
                acc[NP * NP + 2 * NP + i] += av[v] * xv[i][v];
            }
#pragma unroll
            for (int j = 0; j < NP; j++)
#pragma unroll
                for (int v = 0; v < V; v++) acc[i * NP + j] += gv[i][v] * xv[j][v];
        }
    }

    const float qinv = inject ? 0.f : 1.0f / qraw;
    if (!inject) {
#pragma unroll
        for (int i = 0; i < NP; i++) acc[NP * NP + i] *= qinv;  // dHpost was summed against f * q
    }
    // workgroup sum: DPP within each 16-lane row, one LDS slot per row, then K lanes finish
    const int slot = tid >> 4, nslots = nt >> 4;
#pragma unroll
    for (int k = 0; k < K; k++) {
        const float v = row16_allreduce(acc[k]);
        if ((tid & 15) == 0) slot_s[k * 16 + slot] = v;
    }
    __syncthreads();
    for (int k = tid; k < K; k += nt) {
        float v = 0.f;
        for (int s = 0; s < nslots; s++) v += slot_s[k * 16 + s];
        tot[k] = v;
        if (a.raw) a.raw[((size_t)b * a.parts + blockIdx.y) * K + k] = v;
    }
    if (a.raw) return;  // the coefficient backward runs as its own small launch
    __syncthreads();
    if (tid >= SK::kGroup) return;

    // ---- epilogue on the lanes of one matrix (SkSmall layout) -------------------------------
    const int g = tid;
    const float s1 = tot[K - 1];
    const int D = n * n + 2 * n;
    float dHpre = 0.f, dHpost = 0.f;
    if (g < n) {
        dHpost = tot[NP * NP + g];
        dHpre = inject ? 0.f
                       : tot[NP * NP + NP + g] * qinv -
                             s1 * tot[NP * NP + 2 * NP + g] * qinv * qinv * qinv / (float)C;
    }
    if (g == 0) a.out.s1[b] = s1;
    const int r0 = SK::row(g), c0 = SK::col0(g);
    if (a.hstride == 0) {
        // static H: raw sums only; the coefficient backward runs once on the batch total
        float *red = a.out.red + (size_t)b * (D + 3);  // rows padded like dt, for the batch-sum launch
#pragma unroll
        for (int e = 0; e < SK::EPL; e++)
            if (r0 < n && c0 + e < n) red[r0 * n + c0 + e] = tot[r0 * NP + c0 + e];
        if (g < n) { red[n * n + g] = dHpre; red[n * n + n + g] = dHpost; }
        return;
    }
    const float *Pb = a.P + (size_t)b * D;
    const float al0 = a.alpha[0], al1 = a.alpha[1], al2 = a.alpha[2];
    const float rinv = 1.0f / a.r[b];
    float *dt = a.out.dt + (size_t)b * (D + 3);
    const DPWriter dpw{a.out, b, a.B, a.DP};
    float S0 = 0.f, S1 = 0.f, S2 = 0.f;  // sum_d dt_d p_d per alpha group
    if (g < n) {
        const float hp = Hpre[g], ho = Hpost[g];
        const float dtp = dHpre * hp * (1.0f - hp);
        const float dto = dHpost * ho * (1.0f - 0.5f * ho);
        dt[g] = dtp; dt[n + g] = dto;
        dpw.put(g, dtp * al0 * rinv); dpw.put(n + g, dto * al1 * rinv);
        S0 = dtp * Pb[g]; S1 = dto * Pb[n + g];
    }
    float E[SK::EPL], m[SK::EPL], d[SK::EPL];
#pragma unroll
    for (int e = 0; e < SK::EPL; e++) {
        const int c = c0 + e;
        const bool ok = r0 < n && c < n;
        E[e] = ok ? expf(al2 * Pb[2 * n + r0 * n + c] + a.b_res[r0 * n + c]) : 0.f;
        m[e] = E[e];
        d[e] = ok ? tot[r0 * NP + c] : 0.f;
    }
    SK::template forward<false>(m, g, n, a.T, a.eps, sc, tid);
    SK::template backward<false>(d, m, a.T, sc, tid);
#pragma unroll
    for (int e = 0; e < SK::EPL; e++) {
        const int c = c0 + e;
        if (r0 < n && c < n) {
            const int di = 2 * n + r0 * n + c;
            const float dtr = d[e];  // the Sinkhorn backward hands back the gradient of the logits
            dt[di] = dtr;
            dpw.put(di, dtr * al2 * rinv);
            S2 += dtr * Pb[di];
        }
    }
    S0 = SK::group_allreduce(S0); S1 = SK::group_allreduce(S1); S2 = SK::group_allreduce(S2);
    if (g == 0) {
        dt[D] = S0; dt[D + 1] = S1; dt[D + 2] = S2;
        a.out.cx[b] = (al0 * S0 + al1 * S1 + al2 * S2) * rinv * rinv / (float)(n * C);
    }
    dpw.pad(D, g, SK::kGroup);
}



// The coefficient backward as its own launch: every sample's serial Sinkhorn chain runs concurrently
// (four 4x4 samples or one 8x8 sample per wave) instead of at the tail of a bandwidth-bound workgroup.
// Input: the channel sums written by a kernel above or below ([B][parts][K]).
template <int NP, bool PRECISE, bool GRAM = false>
__global__ __launch_bounds__(64) void coef_bwd_small_kernel(BwdReduceArgs a) {
    using SK = SkSmall<NP>;
    using CB = CoefBwdSmall<NP, PRECISE, GRAM>;
    extern __shared__ float sc[];  // Sinkhorn denominators, SK::scaling_floats(T), then CB::kXch per group
    const int tid = threadIdx.x, g = tid % SK::kGroup;
    const int b = blockIdx.x * SK::kPerWave + tid / SK::kGroup;
    if (b >= a.B) return;  // whole groups leave together; the reductions never cross groups
    CB cb;
    cb.prefetch(a, b, g);
    cb.fetch_sums(a.raw + (size_t)b * a.parts * CB::K, a.parts);  // requested before the chain, used after it
    cb.forward_recompute(a, b, g, tid, sc);
    cb.run(a, b, g, tid, sc, sc + SK::scaling_floats(a.T) + (tid / SK::kGroup) * CB::kXch);
}

// =============================================================================================
// n <= 8, dynamic H, dy and x both bf16: the channel sums as three n x n Gram matrices per sample
//   dM = dy x^T        W1 = dy diag(w) x^T        XX = x x^T
// (the same three products as for n > 8; the coefficient kernel forms dHpost, A1, A2, s1 from them)
// on v_mfma_f32_4x4x4_16b_bf16: one instruction is 16 independent 4x4x4 products, block = lane / 4,
// a lane holding four consecutive channels of stream lane % 4 for both operands - which is how the
// data lies in memory, so the operands are the loaded words themselves.  For n > 4 the streams
// form two groups of four and every Gram matrix is 2 x 2 such products.  A step of a wave covers
// 128 channels of all streams (16 bytes per lane, stream group and tensor); nothing is unpacked
// except dy for the product with w, and the kernel needs far fewer registers than the VALU
// version, which is what lets enough waves be resident to keep the loads flowing.
// With an injected f, W1 = dy [f; 0; ...]^T (its column 0 is dHpost) and XX is not needed.
// Output: raw[b][part][m][i][j] (NP x NP each), m = dM | W1 | XX.
// =============================================================================================

// FUSED (one column part per sample): the first lanes of wave 0 go on with the sample's coefficient
// backward (CoefBwdSmall) as soon as the sums are complete, its other inputs requested at the start;
// with several workgroups per CU the serial Sinkhorn chain of one runs under the loads of the others,
// and the launch of the coefficient kernel is saved.
// STATIC (with FUSED): shared coefficients; the tail only converts the sums into the sample's row of raw
// gradients (see CoefBwdSmall).
template <int NP, int WMODE, bool FUSED, bool STATIC = false>
__global__ __launch_bounds__(256, NP == 4 ? 4 : 1) void gram_small_kernel(BwdReduceArgs a) {
    static_assert(NP == 4 || NP == 8, "stream groups of four");
    static_assert(FUSED || !STATIC, "the static tail runs inside the launch");
    using SK = SkSmall<NP>;
    using CB = CoefBwdSmall<NP, false, true, STATIC>;
    constexpr int NB = NP / 4;            // stream groups
    constexpr int U = 2;                  // steps of a wave in flight
    constexpr int K = 3 * NP * NP;
    constexpr bool inject = WMODE == kGramInject;
    __shared__ float slot_s[K * 16];  // one slot per 16-lane row of the workgroup
    __shared__ float tot_s[FUSED ? K : 1];
    extern __shared__ float sc[];     // FUSED: Sinkhorn denominators, SK::scaling_floats(T), then CB::kXch
    const int b = blockIdx.x, part = blockIdx.y, n = a.n, C = a.C;
    const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
    const int pwg = blockIdx.y * gridDim.x + blockIdx.x;
    (void)pwg;
    MHC_PHASE_ZERO(kPhaseGramSmall, pwg);
    MHC_PHASE_BEGIN(pclk);
    CB cb;
    if constexpr (FUSED) {
        // the Sinkhorn forward recompute needs none of the sums: it runs here, on the first lanes of
        // wave 0, while the other waves already stream (and not at the tail of the workgroup)
        if (tid < SK::kGroup) {
            cb.prefetch(a, b, tid);
            if constexpr (!STATIC) cb.forward_recompute(a, b, tid, tid, sc);
        }
    }
    const int blk = lane >> 2, i = lane & 3;
    const int nsteps = (C + 127) / 128, spp = (nsteps + a.parts - 1) / a.parts;
    const int s_begin = part * spp, s_end = min(nsteps, s_begin + spp);
    const bf16_t *gb[NB], *xb[NB];
    bool sv[NB];
#pragma unroll
    for (int I = 0; I < NB; I++) {
        sv[I] = 4 * I + i < n;  // streams >= n: masked below
        const size_t row = (size_t)b * n * C + (size_t)(sv[I] ? 4 * I + i : 0) * C;
        gb[I] = static_cast<const bf16_t *>(a.dy) + row;
        xb[I] = static_cast<const bf16_t *>(a.x) + row;
    }
    const bf16_t *fb = inject ? static_cast<const bf16_t *>(a.f_inject) + (size_t)b * C : nullptr;

    f32x4_t acc[3][NB][NB];
#pragma unroll
    for (int m = 0; m < 3; m++)
#pragma unroll
        for (int I = 0; I < NB; I++)
#pragma unroll
            for (int J = 0; J < NB; J++) acc[m][I][J] = f32x4_t{0.f, 0.f, 0.f, 0.f};
    MHC_PHASE_ADD(kPhaseGramSmall, pwg, 0, pclk);

    // FUSED: wave 0 is busy with the forward recompute while the others stream, so the steps are
    // shared by waves 1 .. 3 only
    constexpr int SW = FUSED ? 3 : 4;  // streaming waves
    const int sw = FUSED ? wave - 1 : wave;
    for (int s0 = sw >= 0 ? s_begin + sw : s_end; s0 < s_end; s0 += SW * U) {
        uint4 gr[U][NB], xr[U][NB], fr[U];
        RawVec<bf16_t, 8> wb[U];
        RawVec<float, 8> wf[U];
#pragma unroll
        for (int u = 0; u < U; u++) {
            const int c = (s0 + SW * u) * 128 + blk * 8;
            const bool in = s0 + SW * u < s_end && c < C;  // C % 8 == 0: a chunk is inside or outside
            const int cc = in ? c : 0;
#pragma unroll
            for (int I = 0; I < NB; I++) {
                gr[u][I] = load16_masked(reinterpret_cast<const uint4 *>(gb[I] + cc), in && sv[I]);
                xr[u][I] = load16_masked(reinterpret_cast<const uint4 *>(xb[I] + cc), in && sv[I]);
            }
            if constexpr (inject) fr[u] = load16_masked(reinterpret_cast<const uint4 *>(fb + cc), in && i == 0);
            else if constexpr (WMODE == kGramWBf16) wb[u].load(static_cast<const bf16_t *>(a.w) + cc);
            else wf[u].load(static_cast<const float *>(a.w) + cc);
        }
#pragma unroll
        for (int u = 0; u < U; u++) {
            bf16x4_t g0[NB], g1[NB], x0[NB], x1[NB];  // first / second group of four channels
#pragma unroll
            for (int I = 0; I < NB; I++) {
                g0[I] = bf16x4_of(gr[u][I].x, gr[u][I].y); g1[I] = bf16x4_of(gr[u][I].z, gr[u][I].w);
                x0[I] = bf16x4_of(xr[u][I].x, xr[u][I].y); x1[I] = bf16x4_of(xr[u][I].z, xr[u][I].w);
            }
#pragma unroll
            for (int I = 0; I < NB; I++)
#pragma unroll
                for (int J = 0; J < NB; J++) {
                    acc[0][I][J] = mfma4(g0[I], x0[J], acc[0][I][J]);
                    acc[0][I][J] = mfma4(g1[I], x1[J], acc[0][I][J]);
                }
            if constexpr (inject) {
                const bf16x4_t f0 = bf16x4_of(fr[u].x, fr[u].y), f1 = bf16x4_of(fr[u].z, fr[u].w);
#pragma unroll
                for (int I = 0; I < NB; I++) {
                    acc[1][I][0] = mfma4(g0[I], f0, acc[1][I][0]);
                    acc[1][I][0] = mfma4(g1[I], f1, acc[1][I][0]);
                }
            } else {
                float wv[8];
                if constexpr (WMODE == kGramWBf16) wb[u].get(wv);
                else wf[u].get(wv);
#pragma unroll
                for (int I = 0; I < NB; I++) {
                    // dy * w as a bf16 pair (rounded value + remainder): dHpre is a difference of two
                    // sums built on W1, a single rounding of the products is not enough for it
                    const uint32_t gw[4] = {gr[u][I].x, gr[u][I].y, gr[u][I].z, gr[u][I].w};
                    uint32_t hw[4], lw[4];
#pragma unroll
                    for (int k = 0; k < 4; k++) {
                        const float p0 = bf16lo_to_f32(gw[k]) * wv[2 * k], p1 = bf16hi_to_f32(gw[k]) * wv[2 * k + 1];
                        hw[k] = pack_bf16x2(p0, p1);
                        lw[k] = pack_bf16x2(p0 - bf16lo_to_f32(hw[k]), p1 - bf16hi_to_f32(hw[k]));
                    }
#pragma unroll
                    for (int J = 0; J < NB; J++) {
                        acc[1][I][J] = mfma4(bf16x4_of(hw[0], hw[1]), x0[J], acc[1][I][J]);
                        acc[1][I][J] = mfma4(bf16x4_of(hw[2], hw[3]), x1[J], acc[1][I][J]);
                        acc[1][I][J] = mfma4(bf16x4_of(lw[0], lw[1]), x0[J], acc[1][I][J]);
                        acc[1][I][J] = mfma4(bf16x4_of(lw[2], lw[3]), x1[J], acc[1][I][J]);
                        acc[2][I][J] = mfma4(x0[I], x0[J], acc[2][I][J]);
                        acc[2][I][J] = mfma4(x1[I], x1[J], acc[2][I][J]);
                    }
                }
            }
        }
    }

    MHC_PHASE_ADD(kPhaseGramSmall, pwg, 1, pclk);
    // Lane (block, j) holds column j of its block's products, register = row.  Sum over the four
    // blocks of a 16-lane row with DPP, one LDS slot per row, then K threads finish.
    const int slot = tid >> 4;
#pragma unroll
    for (int m = 0; m < 3; m++)
#pragma unroll
        for (int I = 0; I < NB; I++)
#pragma unroll
            for (int J = 0; J < NB; J++)
#pragma unroll
                for (int r = 0; r < 4; r++) {
                    float v = acc[m][I][J][r];
                    v += dpp_mov<kDppRowRor4>(v);
                    v += dpp_mov<kDppRowRor8>(v);
                    if ((tid & 15) < 4)
                        slot_s[(m * NP * NP + (4 * I + r) * NP + 4 * J + (tid & 3)) * 16 + slot] = v;
                }
    __syncthreads();
    if (tid < K) {
        float v = 0.f;
#pragma unroll
        for (int sl = 0; sl < 16; sl++) v += slot_s[tid * 16 + sl];
        if constexpr (FUSED) tot_s[tid] = v;
        else a.raw[((size_t)b * a.parts + part) * K + tid] = v;
    }
    if constexpr (FUSED) {
        __syncthreads();
        MHC_PHASE_ADD(kPhaseGramSmall, pwg, 2, pclk);
        if (tid < SK::kGroup) {
            cb.fetch_sums(tot_s, 1);
            cb.run(a, b, tid, tid, sc, sc + (STATIC ? 0 : SK::scaling_floats(a.T)));
        }
        MHC_PHASE_ADD(kPhaseGramSmall, pwg, 3, pclk);
    }
}

// =============================================================================================
// n > 8: the channel sums as three 32x32 Gram matrices on the matrix cores
//
//   dM = dy x^T          W1 = dy diag(w) x^T          XX = x x^T          (contraction over channels)
// carry everything the coefficient backward needs:
//   dHpost[i] = sum_j Hpre[j] W1[i][j] / q       A1[j] = sum_i Hpost[i] W1[i][j]
//   A2[j] = sum_k Hpre[k] XX[k][j]               s1 = sum_ij Hpost[i] Hpre[j] W1[i][j]
// (with an injected f: W1 is replaced by dy [f; 0 ...]^T, whose column 0 is dHpost; XX is skipped).
// Launch 1 (grid B x parts): a workgroup takes a column part of one sample; its 4 waves take
// k-steps round robin and load their operands straight in MFMA layout (row = stream), several
// steps in flight; the partial Gram matrices go to `raw`.  Both inputs bf16: v_mfma_f32_32x32x16_bf16
// (dy*w as a rounded value plus remainder, two instructions).  Otherwise fp32 MFMAs (32x32x2) with exact products: the fp32 tier.
// Launch 2 (grid B): sums the parts, forms the vectors above, then sigmoid derivatives, exact
// Sinkhorn backward, dP and cx as in the n <= 8 coefficient kernel.
// =============================================================================================
constexpr int kGramMats = 3;
constexpr int kGramFloats = kGramMats * 1024;  // per (sample, part), row-major [m][i][j], 32 x 32

// Static H: one workgroup behind the samples' (blockIdx.x == B) recomputes the Sinkhorn forward of the shared
// logits with IEEE divisions and leaves the denominators of its iterations in a.static_state for the
// static coefficient backward, the last launch of the call, which then has only the reverse sweep left.
// The chain (about 6 us for 20 iterations of a 32 x 32 matrix) runs in the shadow of the channel sums.
template <int NP>
__device__ __forceinline__ void static_sinkhorn_forward_block(const BwdReduceArgs &a, float *smem) {
    using SK = SkWg<NP>;
    const int tid = threadIdx.x, n = a.n;
    const int r0 = SK::row(tid), c0 = SK::col0(tid);
    float E[SK::EPL], u, v[SK::EPL];
#pragma unroll
    for (int e = 0; e < SK::EPL; e++)
        E[e] = (r0 < n && c0 + e < n) ? expf(a.static_logits[r0 * n + c0 + e]) : 0.f;
    SK::template forward<true>(E, u, v, n, a.T, a.eps, smem, tid);
    SK::save_state(smem, a.T, a.static_state, tid, u, v);
}

template <typename TG, typename TX>
__global__ __launch_bounds__(256) void gram_large_kernel(BwdReduceArgs a) {
    constexpr bool kBf16 = std::is_same<TG, bf16_t>::value && std::is_same<TX, bf16_t>::value;
    constexpr int VL = kBf16 ? 8 : 4;  // columns per lane and k-step
    constexpr int SW = 2 * VL;         // columns per k-step (two lane halves)
    constexpr int U = 4;               // k-steps in flight per wave
    extern __shared__ __align__(16) float smem[];
    if ((int)blockIdx.x >= a.B) {  // only launched with a.static_state set
        if (blockIdx.y == 0) {
            if (a.n <= 16) static_sinkhorn_forward_block<16>(a, smem);
            else static_sinkhorn_forward_block<32>(a, smem);
        }
        return;
    }
    float *w_s = smem;  // [cols of this part] fp32 weights (zero beyond C)
    const int b = blockIdx.x, part = blockIdx.y, n = a.n, C = a.C, tid = threadIdx.x;
    const int lane = tid & 63, wave = tid >> 6, row = lane & 31, kh = lane >> 5;
    const bool inject = a.f_inject != nullptr;
    const int nsteps = (C + SW - 1) / SW;
    const int spp = (nsteps + a.parts - 1) / a.parts;
    const int s_begin = part * spp, s_end = min(nsteps, s_begin + spp);
    const int c_begin = s_begin * SW;
    float *xw = w_s + spp * SW;  // cross-wave scratch [3][kGramMats * 16][64]
    for (int cc = tid; cc < spp * SW; cc += 256) {
        const int c = c_begin + cc;
        w_s[cc] = (c < C && !inject) ? load_w_(a.w, a.w_bf16, c) : 0.f;
    }
    // The part's s1 = Hpost^T W1 Hpre (wave 0, at the end): the coefficients that meet this lane's
    // accumulator registers are requested now and used behind the streaming loop (aliased beyond n,
    // masked where they are used).
    const bool want_s1 = a.s1part != nullptr && !inject && wave == 0;
    float hp_c = 0.f, ho_r[16];
#pragma unroll
    for (int i = 0; i < 16; i++) ho_r[i] = 0.f;
    if (want_s1) {
        hp_c = a.Hpre[(size_t)b * a.hstride + (row < n ? row : 0)];
#pragma unroll
        for (int i = 0; i < 16; i++) {
            const int ri = 8 * (i >> 2) + 4 * kh + (i & 3);  // accumulator register i holds row ri
            ho_r[i] = a.Hpost[(size_t)b * a.hstride + (ri < n ? ri : 0)];
        }
    }
    __syncthreads();

    // rows >= n alias row 0: they only produce Gram rows / columns that nobody reads
    const size_t ro = (size_t)(row < n ? row : 0) * C;
    const TG *grow = static_cast<const TG *>(a.dy) + (size_t)b * n * C + ro;
    const TX *xrow = static_cast<const TX *>(a.x) + (size_t)b * n * C + ro;
    const TX *frow = inject ? static_cast<const TX *>(a.f_inject) + (size_t)b * C : xrow;

    f32x16_t acc[kGramMats];
#pragma unroll
    for (int m = 0; m < kGramMats; m++)
#pragma unroll
        for (int i = 0; i < 16; i++) acc[m][i] = 0.f;

    auto mfma3 = [&](const float (&g)[VL], const float (&x)[VL], const float (&gw)[VL],
                     const RawVec<TG, VL> &gr, const RawVec<TX, VL> &xr, bool with_xx) {
        if constexpr (kBf16) {
            const bf16x8_t gb = __builtin_bit_cast(bf16x8_t, make_uint4(gr.w[0], gr.w[1], gr.w[2], gr.w[3]));
            const bf16x8_t xb = __builtin_bit_cast(bf16x8_t, make_uint4(xr.w[0], xr.w[1], xr.w[2], xr.w[3]));
            // dy * w as a bf16 pair (rounded value + remainder): dHpre is a difference of two
            // sums built on W1, a single rounding of the products is not enough for it
            float lo[VL];
            uint32_t hw[VL / 2];
#pragma unroll
            for (int i = 0; i < VL / 2; i++) {
                hw[i] = pack_bf16x2(gw[2 * i], gw[2 * i + 1]);
                lo[2 * i] = gw[2 * i] - bf16lo_to_f32(hw[i]);
                lo[2 * i + 1] = gw[2 * i + 1] - bf16hi_to_f32(hw[i]);
            }
            const bf16x8_t gwb = __builtin_bit_cast(bf16x8_t, make_uint4(hw[0], hw[1], hw[2], hw[3]));
            const bf16x8_t gwl = __builtin_bit_cast(
                bf16x8_t, make_uint4(pack_bf16x2(lo[0], lo[1]), pack_bf16x2(lo[2], lo[3]),
                                     pack_bf16x2(lo[4], lo[5]), pack_bf16x2(lo[6], lo[7])));
            acc[0] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(gb, xb, acc[0], 0, 0, 0);
            acc[1] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(gwb, xb, acc[1], 0, 0, 0);
            acc[1] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(gwl, xb, acc[1], 0, 0, 0);
            if (with_xx) acc[2] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(xb, xb, acc[2], 0, 0, 0);
        } else {
#pragma unroll
            for (int i = 0; i < VL; i++) {
                acc[0] = __builtin_amdgcn_mfma_f32_32x32x2f32(g[i], x[i], acc[0], 0, 0, 0);
                acc[1] = __builtin_amdgcn_mfma_f32_32x32x2f32(gw[i], x[i], acc[1], 0, 0, 0);
                if (with_xx) acc[2] = __builtin_amdgcn_mfma_f32_32x32x2f32(x[i], x[i], acc[2], 0, 0, 0);
            }
        }
    };

    // full k-steps (every column of the step inside C, rows 16-byte aligned)
    const bool vec_ok = C % VL == 0;
    const int s_full = vec_ok ? min(s_end, C / SW) : s_begin;
    int s;
    if constexpr (kBf16) {
        // Chunks of 4 steps (64 channels), one chunk per wave and round: the 32 rows of dy and x are
        // fetched row-contiguously (8 lanes per 128-byte piece, rows lr + 8 j), parked in a wave-private
        // LDS tile (no barrier: a wave's LDS accesses complete in order) and read back in operand
        // layout, the next chunk in flight in registers.  Loading straight in operand layout has
        // every lane on its own row, which the memory pipeline serves at a quarter of the rate.
        constexpr int PITCH = 72;  // 128 data bytes + 16 pad per row (bf16 elements)
        bf16_t *cb = reinterpret_cast<bf16_t *>(xw) + (size_t)wave * (2 * 32 + 1) * PITCH;  // dy rows | x rows | f
        const int lr = lane >> 3, seg = lane & 7;
        const bf16_t *gq_row[4], *xq_row[4];
#pragma unroll
        for (int j = 0; j < 4; j++) {
            const size_t rj = (size_t)(lr + 8 * j < n ? lr + 8 * j : 0) * C;  // rows >= n alias row 0
            gq_row[j] = static_cast<const bf16_t *>(a.dy) + (size_t)b * n * C + rj;
            xq_row[j] = static_cast<const bf16_t *>(a.x) + (size_t)b * n * C + rj;
        }
        const bf16_t *fq_row = static_cast<const bf16_t *>(frow);
        uint32_t gq[4][4], xq[4][4], fq[4];
        auto fetch = [&](int chunk) {
            const int col = c_begin + chunk * 64 + seg * 8;
#pragma unroll
            for (int j = 0; j < 4; j++) {
                const uint4 g4 = *reinterpret_cast<const uint4 *>(gq_row[j] + col);
                const uint4 x4 = *reinterpret_cast<const uint4 *>(xq_row[j] + col);
                gq[j][0] = g4.x; gq[j][1] = g4.y; gq[j][2] = g4.z; gq[j][3] = g4.w;
                xq[j][0] = x4.x; xq[j][1] = x4.y; xq[j][2] = x4.z; xq[j][3] = x4.w;
            }
            if (inject) {
                const uint4 f4 = *reinterpret_cast<const uint4 *>(fq_row + col);
                fq[0] = f4.x; fq[1] = f4.y; fq[2] = f4.z; fq[3] = f4.w;
            }
        };
        auto park = [&]() {
#pragma unroll
            for (int j = 0; j < 4; j++) {
                *reinterpret_cast<uint4 *>(cb + (size_t)(lr + 8 * j) * PITCH + seg * 8) = make_uint4(gq[j][0], gq[j][1], gq[j][2], gq[j][3]);
                *reinterpret_cast<uint4 *>(cb + (size_t)(32 + lr + 8 * j) * PITCH + seg * 8) = make_uint4(xq[j][0], xq[j][1], xq[j][2], xq[j][3]);
            }
            if (inject && lr == 0) *reinterpret_cast<uint4 *>(cb + (size_t)64 * PITCH + seg * 8) = make_uint4(fq[0], fq[1], fq[2], fq[3]);
        };
        const int nchunks = (s_full - s_begin) / 4;
        if (wave < nchunks) fetch(wave);
        for (int chunk = wave; chunk < nchunks; chunk += 4) {
            park();
            // the rows come back in operand layout from this wave's own tile: a wave's LDS accesses
            // complete in order, the fence keeps the compiler from moving the reads above the writes
            __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront");
            __builtin_amdgcn_wave_barrier();
            if (chunk + 4 < nchunks) fetch(chunk + 4);
#pragma unroll
            for (int u = 0; u < 4; u++) {
                RawVec<TG, VL> gr;
                RawVec<TX, VL> xr;
                const uint4 g4 = *reinterpret_cast<const uint4 *>(cb + (size_t)row * PITCH + u * 16 + kh * 8);
                const uint4 x4 = *reinterpret_cast<const uint4 *>(cb + (size_t)(32 + row) * PITCH + u * 16 + kh * 8);
                gr.w[0] = g4.x; gr.w[1] = g4.y; gr.w[2] = g4.z; gr.w[3] = g4.w;
                xr.w[0] = x4.x; xr.w[1] = x4.y; xr.w[2] = x4.z; xr.w[3] = x4.w;
                if (inject) {
                    // B operand = [f; 0; ...]: only lane row 0 carries f, column 0 of the product is dy . f
                    const uint4 f4 = *reinterpret_cast<const uint4 *>(cb + (size_t)64 * PITCH + u * 16 + kh * 8);
                    const bf16x8_t gb = __builtin_bit_cast(bf16x8_t, g4);
                    const bf16x8_t xb = __builtin_bit_cast(bf16x8_t, x4);
                    const bf16x8_t fb = __builtin_bit_cast(
                        bf16x8_t, make_uint4(row == 0 ? f4.x : 0u, row == 0 ? f4.y : 0u, row == 0 ? f4.z : 0u, row == 0 ? f4.w : 0u));
                    acc[0] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(gb, xb, acc[0], 0, 0, 0);
                    acc[1] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(gb, fb, acc[1], 0, 0, 0);
                } else {
                    const int cc = chunk * 64 + u * 16 + kh * 8;  // relative to c_begin
                    float g[VL], x[VL], gw[VL];
                    gr.get(g);
                    xr.get(x);
#pragma unroll
                    for (int i = 0; i < VL; i++) gw[i] = g[i] * w_s[cc + i];
                    mfma3(g, x, gw, gr, xr, true);
                }
            }
        }
        s = s_begin + nchunks * 4 + wave;
        __syncthreads();  // the chunk tiles live in the cross-wave scratch used below
    } else {
    // raw loads in operand layout, U steps in flight, nothing conditional per lane
    s = s_begin + wave;
    for (; s + 4 * (U - 1) < s_full; s += 4 * U) {
        RawVec<TG, VL> gr[U];
        RawVec<TX, VL> xr[U], fr[U];
#pragma unroll
        for (int u = 0; u < U; u++) {
            const int c = (s + 4 * u) * SW + kh * VL;
            gr[u].load(grow + c);
            xr[u].load(xrow + c);
            if (inject) fr[u].load(frow + c);
        }
#pragma unroll
        for (int u = 0; u < U; u++) {
            const int cc = (s + 4 * u) * SW + kh * VL - c_begin;
            float g[VL], x[VL], gw[VL];
            gr[u].get(g);
            xr[u].get(x);
            if (inject) {
                // B operand = [f; 0; ...]: only lane row 0 carries f, column 0 of the product is dy . f
                float f[VL];
                fr[u].get(f);
                RawVec<TX, VL> fz;
#pragma unroll
                for (int i = 0; i < RawVec<TX, VL>::kWords; i++) fz.w[i] = row == 0 ? fr[u].w[i] : 0u;
#pragma unroll
                for (int i = 0; i < VL; i++) f[i] = row == 0 ? f[i] : 0.f;
                if constexpr (kBf16) {
                    const bf16x8_t gb = __builtin_bit_cast(bf16x8_t, make_uint4(gr[u].w[0], gr[u].w[1], gr[u].w[2], gr[u].w[3]));
                    const bf16x8_t xb = __builtin_bit_cast(bf16x8_t, make_uint4(xr[u].w[0], xr[u].w[1], xr[u].w[2], xr[u].w[3]));
                    const bf16x8_t fb = __builtin_bit_cast(bf16x8_t, make_uint4(fz.w[0], fz.w[1], fz.w[2], fz.w[3]));
                    acc[0] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(gb, xb, acc[0], 0, 0, 0);
                    acc[1] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(gb, fb, acc[1], 0, 0, 0);
                } else {
#pragma unroll
                    for (int i = 0; i < VL; i++) {
                        acc[0] = __builtin_amdgcn_mfma_f32_32x32x2f32(g[i], x[i], acc[0], 0, 0, 0);
                        acc[1] = __builtin_amdgcn_mfma_f32_32x32x2f32(g[i], f[i], acc[1], 0, 0, 0);
                    }
                }
            } else {
#pragma unroll
                for (int i = 0; i < VL; i++) gw[i] = g[i] * w_s[cc + i];
                mfma3(g, x, gw, gr[u], xr[u], true);
            }
        }
    }
    }
    // remaining steps of this wave (fewer than U full ones, a ragged last step, unaligned rows):
    // element-wise masked loads, fp32 operands rounded where the bf16 instruction needs them
    for (; s < s_end; s += 4) {
        const int c = s * SW + kh * VL, cc = c - c_begin;
        float g[VL], x[VL], gw[VL], f[VL];
#pragma unroll
        for (int i = 0; i < VL; i++) {
            const bool ok = c + i < C;
            g[i] = ok ? to_f32<TG>(grow[c + i]) : 0.f;
            x[i] = ok ? to_f32<TX>(xrow[c + i]) : 0.f;
            f[i] = (ok && inject && row == 0) ? to_f32<TX>(frow[c + i]) : 0.f;
            gw[i] = inject ? f[i] : g[i] * w_s[cc + i];
        }
        if constexpr (kBf16) {
            auto pack8 = [](const float (&v)[VL]) {
                return __builtin_bit_cast(bf16x8_t, make_uint4(pack_bf16x2(v[0], v[1]), pack_bf16x2(v[2], v[3]),
                                                               pack_bf16x2(v[4], v[5]), pack_bf16x2(v[6], v[7])));
            };
            const bf16x8_t gb = pack8(g), xb = pack8(x), sb = pack8(gw);  // g, x, f came from bf16: exact
            float lo[VL];
#pragma unroll
            for (int i = 0; i < VL; i++) lo[i] = gw[i] - bf16_to_f32(f32_to_bf16(gw[i]));
            if (!inject) acc[1] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(pack8(lo), xb, acc[1], 0, 0, 0);
            if (inject) {
                acc[0] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(gb, xb, acc[0], 0, 0, 0);
                acc[1] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(gb, sb, acc[1], 0, 0, 0);
            } else {
                acc[0] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(gb, xb, acc[0], 0, 0, 0);
                acc[1] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(sb, xb, acc[1], 0, 0, 0);
                acc[2] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(xb, xb, acc[2], 0, 0, 0);
            }
        } else {
#pragma unroll
            for (int i = 0; i < VL; i++) {
                acc[0] = __builtin_amdgcn_mfma_f32_32x32x2f32(g[i], x[i], acc[0], 0, 0, 0);
                if (inject) {
                    acc[1] = __builtin_amdgcn_mfma_f32_32x32x2f32(g[i], gw[i], acc[1], 0, 0, 0);
                } else {
                    acc[1] = __builtin_amdgcn_mfma_f32_32x32x2f32(gw[i], x[i], acc[1], 0, 0, 0);
                    acc[2] = __builtin_amdgcn_mfma_f32_32x32x2f32(x[i], x[i], acc[2], 0, 0, 0);
                }
            }
        }
    }

    // cross-wave sum in LDS, then wave 0 writes the part's Gram matrices row-major
    if (wave > 0) {
        float *dst = xw + (size_t)(wave - 1) * kGramMats * 16 * 64;
#pragma unroll
        for (int m = 0; m < kGramMats; m++)
#pragma unroll
            for (int i = 0; i < 16; i++) dst[(m * 16 + i) * 64 + lane] = acc[m][i];
    }
    __syncthreads();
    if (wave == 0) {
        float *out = a.raw + ((size_t)b * a.parts + part) * kGramFloats;
        float s1 = 0.f;  // Hpost^T W1 Hpre of this part: this lane's column of W1 against Hpost
#pragma unroll
        for (int m = 0; m < kGramMats; m++)
#pragma unroll
            for (int i = 0; i < 16; i++) {
                float v = acc[m][i];
#pragma unroll
                for (int w = 0; w < 3; w++) v += xw[((size_t)w * kGramMats * 16 + m * 16 + i) * 64 + lane];
                // accumulator layout: column j = lane & 31, register i -> row 8*(i/4) + 4*(lane/32) + i%4
                const int ri = 8 * (i >> 2) + 4 * kh + (i & 3);
                out[m * 1024 + ri * 32 + row] = v;
                if (m == 1 && want_s1) s1 += (ri < n ? ho_r[i] : 0.f) * v;
            }
        if (want_s1) {
            s1 *= row < n ? hp_c : 0.f;  // rows and columns >= n hold aliased garbage
            s1 = wave_allreduce_sum(s1);
            if (lane == 0) a.s1part[(size_t)b * a.parts + part] = s1;
        }
    }
}

// One workgroup (256 threads) of the coefficient launch for n > 8: sample b; smem = coef_bwd_large_lds_floats<NP>(T) floats.
template <int NP>
static size_t coef_bwd_large_lds_floats(int T) { return 3 * 32 * 33 + 64 + 96 + 4 + SkWg<NP>::lds_floats(T); }

template <int NP, bool PRECISE>
__device__ __forceinline__ void coef_bwd_large_block(const BwdReduceArgs &a, const int b, float *smem) {
    using SK = SkWg<NP>;
    float *W_s = smem;                   // [32][33]  W1 (or dy [f;0]^T)
    float *X_s = W_s + 32 * 33;          // [32][33]  XX
    float *M_s = X_s + 32 * 33;          // [32][33]  dM
    float *hp_s = M_s + 32 * 33;         // [32] Hpre
    float *ho_s = hp_s + 32;             // [32] Hpost
    float *vec_s = ho_s + 32;            // [3][32] dHpost | A1 | A2
    float *red_s = vec_s + 96;           // [4]
    float *sk_s = red_s + 4;             // SK::lds_floats(T)
    const int n = a.n, C = a.C, tid = threadIdx.x, lane = tid & 63;
    const bool w0 = tid < 64;
    const bool inject = a.f_inject != nullptr;
    MHC_PHASE(kPhaseCoefBwdWide, b, 0);
    const float qinv = inject ? 0.f : (PRECISE ? 1.0f / a.q[b] : fast_rcp(a.q[b]));
    if (tid < 32) {
        hp_s[tid] = tid < n ? a.Hpre[(size_t)b * a.hstride + tid] : 0.f;
        ho_s[tid] = tid < n ? a.Hpost[(size_t)b * a.hstride + tid] : 0.f;
    }
    // inputs of the Sinkhorn recompute, requested now so that they arrive behind the part sums
    // (out-of-range elements alias element 0 and are masked where they are used)
    const int D = n * n + 2 * n;
    const int r0 = SK::row(tid), c0 = SK::col0(tid);
    const bool dyn = a.hstride != 0;
    // scalars of the coefficient backward, requested with everything else (used after the sums)
    float al0 = 0.f, al1 = 0.f, al2 = 0.f, rinv = 0.f;
    if (dyn) {
        al0 = a.alpha[0]; al1 = a.alpha[1]; al2 = a.alpha[2];
        rinv = PRECISE ? 1.0f / a.r[b] : fast_rcp(a.r[b]);
    }
    float pres[SK::EPL], bres[SK::EPL];
#pragma unroll
    for (int e = 0; e < SK::EPL; e++) {
        const bool ok = dyn && r0 < n && c0 + e < n;
        pres[e] = dyn ? a.P[(size_t)b * D + (ok ? 2 * n + r0 * n + c0 + e : 0)] : 0.f;
        bres[e] = dyn ? a.b_res[ok ? r0 * n + c0 + e : 0] : 0.f;
    }
    // sum the column parts; rows / columns >= n hold aliased garbage and are dropped here.  The
    // first four parts are requested before the Sinkhorn forward recompute (which needs none of
    // them) and collected after it.
    const float *raw = a.raw + (size_t)b * a.parts * kGramFloats;
    constexpr int EPT = kGramFloats / 256;  // 12 elements per thread, all loads of a part in flight
    float t0[4][EPT];
#pragma unroll
    for (int q = 0; q < 4; q++)
#pragma unroll
        for (int k = 0; k < EPT; k++)
            t0[q][k] = raw[(size_t)(q < a.parts ? q : 0) * kGramFloats + tid + 256 * k];
    float E[SK::EPL], u = 1.0f, v[SK::EPL];
    if (dyn) {
#pragma unroll
        for (int e = 0; e < SK::EPL; e++) {
            const bool ok = r0 < n && c0 + e < n;
            pres[e] = ok ? pres[e] : 0.f;
            E[e] = ok ? (PRECISE ? expf(al2 * pres[e] + bres[e]) : exp_fast(al2 * pres[e] + bres[e])) : 0.f;
        }
        if (a.sk_state) SK::load_state(a.sk_state + (size_t)b * SK::state_floats(a.T), u, v, a.T, sk_s, tid);
        else SK::template forward<PRECISE>(E, u, v, n, a.T, a.eps, sk_s, tid);
    }
    MHC_PHASE(kPhaseCoefBwdWide, b, 1);
    {
        float acc[EPT];
#pragma unroll
        for (int k = 0; k < EPT; k++) acc[k] = 0.f;
#pragma unroll
        for (int q = 0; q < 4; q++)
#pragma unroll
            for (int k = 0; k < EPT; k++) acc[k] += q < a.parts ? t0[q][k] : 0.f;
        for (int p0 = 4; p0 < a.parts; p0 += 4) {  // 48 loads in flight; surplus parts alias part 0
            float t[4][EPT];
#pragma unroll
            for (int q = 0; q < 4; q++)
#pragma unroll
                for (int k = 0; k < EPT; k++)
                    t[q][k] = raw[(size_t)(p0 + q < a.parts ? p0 + q : 0) * kGramFloats + tid + 256 * k];
#pragma unroll
            for (int q = 0; q < 4; q++)
#pragma unroll
                for (int k = 0; k < EPT; k++) acc[k] += p0 + q < a.parts ? t[q][k] : 0.f;
        }
#pragma unroll
        for (int k = 0; k < EPT; k++) {
            const int e = tid + 256 * k;
            const int m = e >> 10, i = (e >> 5) & 31, j = e & 31;
            const bool ok = i < n && j < n;
            if (m == 0) M_s[i * 33 + j] = ok ? acc[k] : 0.f;
            else if (m == 1) W_s[i * 33 + j] = (i < n && (j < n || inject)) ? acc[k] : 0.f;
            else X_s[i * 33 + j] = ok ? acc[k] : 0.f;
        }
    }
    __syncthreads();
    MHC_PHASE(kPhaseCoefBwdWide, b, 2);
    {
        // dHpost[i] = sum_j Hpre[j] W1[i][j] / q,  A1[i] = sum_j Hpost[j] W1[j][i],  A2[i] = sum_j Hpre[j] XX[j][i]:
        // thread (i, seg) = (tid / 8, tid % 8) adds four terms of each, the 8 lanes of i finish the sums
        const int i = tid >> 3, seg = tid & 7;
        float dh = 0.f, a1 = 0.f, a2 = 0.f;
#pragma unroll
        for (int k = 0; k < 4; k++) {
            const int j = seg * 4 + k;
            const float hpj = hp_s[j], hoj = ho_s[j];
            dh += hpj * W_s[i * 33 + j];
            a1 += hoj * W_s[j * 33 + i];
            a2 += hpj * X_s[j * 33 + i];
        }
        auto sum8 = [](float x) {
            x += dpp_mov<kDppQuadXor1>(x);
            x += dpp_mov<kDppQuadXor2>(x);
            x += dpp_mov<kDppRowHalfMirror>(x);  // lane i <-> 7 - i: the other quad of the 8 lanes
            return x;
        };
        dh = sum8(dh); a1 = sum8(a1); a2 = sum8(a2);
        if (seg == 0) {
            vec_s[i] = inject ? W_s[i * 33] : dh * qinv;
            vec_s[32 + i] = a1;
            vec_s[64 + i] = a2;
        }
    }
    __syncthreads();
    float s1 = 0.f;
    if (!inject) {  // every wave on its own: lanes 0 .. 31 hold one term each
        s1 = wave_allreduce_sum(lane < 32 ? ho_s[lane] * vec_s[lane] : 0.f);
        s1 = s1 / qinv;  // vec_s holds W1 Hpre / q
    }

    float dHpre = 0.f, dHpost = 0.f;
    if (w0 && lane < n) {
        dHpost = vec_s[lane];
        dHpre = inject ? 0.f
                       : vec_s[32 + lane] * qinv - s1 * vec_s[64 + lane] * qinv * qinv * qinv / (float)C;
    }
    if (tid == 0) a.out.s1[b] = s1;
    if (a.hstride == 0) {
        float *red = a.out.red + (size_t)b * (D + 3);  // rows padded like dt, for the batch-sum launch
        for (int e = tid; e < n * n; e += 256) red[e] = M_s[(e / n) * 33 + (e % n)];
        if (w0 && lane < n) { red[n * n + lane] = dHpre; red[n * n + n + lane] = dHpost; }
        return;
    }
    const float *Pb = a.P + (size_t)b * D;
    float *dt = a.out.dt + (size_t)b * (D + 3);
    const DPWriter dpw{a.out, b, a.B, a.DP};
    float S0 = 0.f, S1 = 0.f, S2 = 0.f;  // sum_d dt_d p_d per alpha group
    if (w0 && lane < n) {
        const float hp = hp_s[lane], ho = ho_s[lane];
        const float dtp = dHpre * hp * (1.0f - hp);
        const float dto = dHpost * ho * (1.0f - 0.5f * ho);
        dt[lane] = dtp; dt[n + lane] = dto;
        dpw.put(lane, dtp * al0 * rinv); dpw.put(n + lane, dto * al1 * rinv);
        S0 = dtp * Pb[lane]; S1 = dto * Pb[n + lane];
    }
    MHC_PHASE(kPhaseCoefBwdWide, b, 3);
    // exact Sinkhorn backward (the forward recompute ran above), the matrix spread over all 256 threads
    float d[SK::EPL];
#pragma unroll
    for (int e = 0; e < SK::EPL; e++) {
        const int c = c0 + e;
        d[e] = (r0 < n && c < n) ? M_s[r0 * 33 + c] : 0.f;
    }
    SK::template backward<PRECISE>(E, d, u, v, a.T, sk_s, tid);
    MHC_PHASE(kPhaseCoefBwdWide, b, 4);
#pragma unroll
    for (int e = 0; e < SK::EPL; e++) {
        const int c = c0 + e;
        if (r0 < n && c < n) {
            const int di = 2 * n + r0 * n + c;
            const float dtr = d[e];  // the Sinkhorn backward hands back the gradient of the logits
            dt[di] = dtr;
            dpw.put(di, dtr * al2 * rinv);
            S2 += dtr * pres[e];
        }
    }
    S2 = block_allreduce_sum<256>(S2, red_s);
    if (w0) {
        S0 = wave_allreduce_sum(S0); S1 = wave_allreduce_sum(S1);
        if (lane == 0) {
            dt[D] = S0; dt[D + 1] = S1; dt[D + 2] = S2;
            a.out.cx[b] = (al0 * S0 + al1 * S1 + al2 * S2) * rinv * rinv / (float)(n * C);
        }
    }
    dpw.pad(D, tid, 256);
    MHC_PHASE(kPhaseCoefBwdWide, b, 5);
}

template <int NP, bool PRECISE>
__global__ __launch_bounds__(256) void coef_bwd_large_kernel(BwdReduceArgs a) {
    extern __shared__ __align__(16) float smem[];
    coef_bwd_large_block<NP, PRECISE>(a, blockIdx.x, smem);
}

// The same launch with the workgroups of the n > 8 dx kernel behind the B coefficient workgroups.  The
// coefficient workgroups are one per sample (half of the CUs at B = 128) and spend their time in
// dependent chains; the dx workgroups given here need nothing that the coefficient workgroups produce
// (d.s1part, no cx, no projection term) and run in their shadow on the rest of the chip.
template <int NP, bool PRECISE>
__global__ __launch_bounds__(256, 4) void coef_bwd_large_dx_kernel(BwdReduceArgs a, BwdDxArgs d) {
    extern __shared__ __align__(16) float smem[];
    if ((int)blockIdx.x < a.B) coef_bwd_large_block<NP, PRECISE>(a, blockIdx.x, smem);
    else dx_large_block(d, blockIdx.x - a.B, reinterpret_cast<unsigned char *>(smem));
}

// =============================================================================================
// launch
// =============================================================================================
// n <= 8, dynamic H, bf16 dy and x, rows 16-byte aligned: Gram matrices on the matrix cores.
static bool gram_small_supported(const BwdReduceArgs &a) { return a.raw != nullptr && a.n <= 8 && a.C % 8 == 0; }

// Column parts of gram_small_kernel: never more than bwd_reduce_parts(), which sizes `raw`.
static int gram_small_parts(int B, int C) { return C >= 1024 && B < 1024 ? 2 : 1; }

// One launch (channel sums, then the coefficient backward at the tail of every workgroup) unless the
// Sinkhorn state would take the LDS that keeps several workgroups per CU resident, or the batch is
// too small to do without column parts.
static bool gram_small_fused(const BwdReduceArgs &a) {
    if (const int hook = tuning_get(kTuneGramFused); hook && a.T <= 32) return hook == 2;  // experiment hook
    // very short rows in a very large batch: the tail of a workgroup (one wave, 2.6 us) outweighs its
    // streaming, and a separate launch packs the chains of four samples into a wave
    // (backward us, one launch | two: B=8192 n=4 C=128 50.3 | 45.2, 6000 C=256 46.7 | 45.4, 4096 C=512 42.4 | 45.5)
    if (a.B >= 6000 && a.C <= 256) return false;
    return a.T <= 32 && (a.B >= 128 || a.C <= 2048);
}

template <int NP, bool FUSED>
static hipError_t launch_gram_small_kernel(const BwdReduceArgs &a, size_t smem, hipStream_t stream) {
    const dim3 grid(a.B, a.parts);
    if (a.f_inject) gram_small_kernel<NP, kGramInject, FUSED><<<grid, 256, smem, stream>>>(a);
    else if (a.w_bf16) gram_small_kernel<NP, kGramWBf16, FUSED><<<grid, 256, smem, stream>>>(a);
    else gram_small_kernel<NP, kGramWF32, FUSED><<<grid, 256, smem, stream>>>(a);
    return hipGetLastError();
}

template <int NP>
static hipError_t launch_gram_small(BwdReduceArgs a, hipStream_t stream) {
    using SK = SkSmall<NP>;
    using CB = CoefBwdSmall<NP, false, true>;
    if (gram_small_fused(a)) {
        a.parts = 1;
        const size_t smem = sizeof(float) * (SK::scaling_floats(a.T) + CB::kXch);  // at most 16 KB + 96 B
        return launch_gram_small_kernel<NP, true>(a, smem, stream);
    }
    a.parts = gram_small_parts(a.B, a.C);
    hipError_t e = launch_gram_small_kernel<NP, false>(a, 0, stream);
    if (e != hipSuccess) return e;
    const size_t smem = sizeof(float) * (SK::scaling_floats(a.T) + SK::kPerWave * CB::kXch);
    e = allow_dynamic_lds(&coef_bwd_small_kernel<NP, false, true>, smem);
    if (e != hipSuccess) return e;
    coef_bwd_small_kernel<NP, false, true><<<(a.B + SK::kPerWave - 1) / SK::kPerWave, 64, smem, stream>>>(a);
    return hipGetLastError();
}

// Static H with bf16 dy and x: the same Gram kernel, one launch, the tail writes the rows of `red`.
template <int NP>
static hipError_t launch_gram_small_static(BwdReduceArgs a, hipStream_t stream) {
    using CB = CoefBwdSmall<NP, false, true, true>;
    a.parts = 1;
    const size_t smem = sizeof(float) * CB::kXch;
    const dim3 grid(a.B, 1);
    if (a.f_inject) gram_small_kernel<NP, kGramInject, true, true><<<grid, 256, smem, stream>>>(a);
    else if (a.w_bf16) gram_small_kernel<NP, kGramWBf16, true, true><<<grid, 256, smem, stream>>>(a);
    else gram_small_kernel<NP, kGramWF32, true, true><<<grid, 256, smem, stream>>>(a);
    return hipGetLastError();
}

template <typename TG, typename TX, int NP, int V>
static hipError_t launch_small(const BwdReduceArgs &a, hipStream_t stream) {
    if constexpr (std::is_same<TG, bf16_t>::value && std::is_same<TX, bf16_t>::value) {
        if (gram_small_supported(a)) return launch_gram_small<NP>(a, stream);
        // static H: worth it once the batch fills the chip (one workgroup per sample)
        if (a.hstride == 0 && a.C % 8 == 0 && a.B >= 128) return launch_gram_small_static<NP>(a, stream);
    }
    const int nch = (a.C / V + a.parts - 1) / a.parts;  // chunks per column part
    // every thread gets the same number of chunks (whole 16-lane rows: the reduction works on them)
    const int rounds = (nch + 255) / 256;
    int nt = round_up((nch + rounds - 1) / rounds, 16);
    if (nt > 256) nt = 256;
    if (nt < SkSmall<NP>::kGroup) nt = SkSmall<NP>::kGroup;  // the epilogue runs on the lanes of one matrix
    constexpr int K = NP * NP + 3 * NP + 1;
    // the Sinkhorn area is only needed when the coefficient backward runs in the same launch
    const size_t smem = sizeof(float) * (K * 16 + K + (a.raw ? 0 : SkSmall<NP>::scaling_floats(a.T)));
    hipError_t e = allow_dynamic_lds(&mix_bwd_reduce_small_kernel<TG, TX, NP, V>, smem);
    if (e != hipSuccess) return e;
    mix_bwd_reduce_small_kernel<TG, TX, NP, V><<<dim3(a.B, a.parts), nt, smem, stream>>>(a);
    e = hipGetLastError();
    if (e != hipSuccess || !a.raw) return e;
    // fp32 activations: the parity tier, IEEE divisions in the Sinkhorn chain
    constexpr bool kPrecise = std::is_same<TX, float>::value;
    const size_t smem2 = sizeof(float) * SkSmall<NP>::scaling_floats(a.T);
    e = allow_dynamic_lds(&coef_bwd_small_kernel<NP, kPrecise>, smem2);
    if (e != hipSuccess) return e;
    coef_bwd_small_kernel<NP, kPrecise><<<(a.B + SkSmall<NP>::kPerWave - 1) / SkSmall<NP>::kPerWave, 64, smem2, stream>>>(a);
    return hipGetLastError();
}

template <typename TG, typename TX, int NP>
static hipError_t launch_small_np(const BwdReduceArgs &a, hipStream_t stream) {
    constexpr int bytes = NP == 4 ? 16 : 8;  // keep the two [NP][V] tiles in registers
    constexpr int szmax = sizeof(TG) > sizeof(TX) ? sizeof(TG) : sizeof(TX);
    constexpr int V = bytes / szmax;
    if (a.C % V == 0) return launch_small<TG, TX, NP, V>(a, stream);
    return launch_small<TG, TX, NP, 1>(a, stream);
}

template <typename TG, typename TX>
static hipError_t launch_large(const BwdReduceArgs &a, hipStream_t stream, const BwdDxArgs *shadow = nullptr) {
    constexpr bool kBf16 = std::is_same<TG, bf16_t>::value && std::is_same<TX, bf16_t>::value;
    constexpr int SW = kBf16 ? 16 : 8;
    const int nsteps = (a.C + SW - 1) / SW;
    const int spp = (nsteps + a.parts - 1) / a.parts;
    // weights of the part | cross-wave scratch, which first holds the four waves' chunk tiles (bf16 path)
    const size_t scratch = sizeof(float) * 3 * kGramMats * 16 * 64, tiles = sizeof(bf16_t) * 4 * (2 * 32 + 1) * 72;
    size_t smem1 = sizeof(float) * (size_t)spp * SW + (kBf16 && tiles > scratch ? tiles : scratch);
    if (a.static_state) {
        const size_t sk = sizeof(float) * (a.n <= 16 ? SkWg<16>::lds_floats(a.T) : SkWg<32>::lds_floats(a.T));
        if (smem1 < sk) smem1 = sk;
    }
    if (smem1 > 64 * 1024) {
        hipError_t e = hipFuncSetAttribute(reinterpret_cast<const void *>(&gram_large_kernel<TG, TX>),
                                           hipFuncAttributeMaxDynamicSharedMemorySize, (int)smem1);
        if (e != hipSuccess) return e;
    }
    gram_large_kernel<TG, TX><<<dim3(a.B + (a.static_state ? 1 : 0), a.parts), 256, smem1, stream>>>(a);
    hipError_t e = hipGetLastError();
    if (e != hipSuccess) return e;
    constexpr bool kPrecise = std::is_same<TX, float>::value;  // fp32 activations: the parity tier
    if constexpr (kBf16) {
        if (shadow) {
            if (a.n <= 16) return hipErrorInvalidValue;
            size_t smem2 = sizeof(float) * coef_bwd_large_lds_floats<32>(a.T);
            if (smem2 < dx_large_lds_bytes()) smem2 = dx_large_lds_bytes();
            e = allow_dynamic_lds(&coef_bwd_large_dx_kernel<32, false>, smem2);
            if (e != hipSuccess) return e;
            const unsigned ncb = (unsigned)((a.C + kDxlCB - 1) / kDxlCB);
            coef_bwd_large_dx_kernel<32, false><<<(unsigned)a.B * (1u + ncb), 256, smem2, stream>>>(a, *shadow);
            return hipGetLastError();
        }
    }
    if (shadow) return hipErrorInvalidValue;
    if (a.n <= 16) {
        const size_t smem2 = sizeof(float) * coef_bwd_large_lds_floats<16>(a.T);
        e = allow_dynamic_lds(&coef_bwd_large_kernel<16, kPrecise>, smem2);
        if (e != hipSuccess) return e;
        coef_bwd_large_kernel<16, kPrecise><<<a.B, 256, smem2, stream>>>(a);
    } else {
        const size_t smem2 = sizeof(float) * coef_bwd_large_lds_floats<32>(a.T);
        e = allow_dynamic_lds(&coef_bwd_large_kernel<32, kPrecise>, smem2);
        if (e != hipSuccess) return e;
        coef_bwd_large_kernel<32, kPrecise><<<a.B, 256, smem2, stream>>>(a);
    }
    return hipGetLastError();
}

// Column parts per sample when the channel sums are a launch of their own.
int bwd_reduce_parts(int B, int n, int C) {
    if (n > 8) {
        // ~512 workgroups, at least ~128 columns per part, at most four parts: the coefficient launch
        // sums the parts of a sample at the head of its chain, and more of them cost it more than the
        // channel-sum kernel gains (backward us, n=32 C=1280: B=64  4 parts 86.3 | 8: 88.6;
        // B=128  4: 92.3 | 6: 99.9; B=32  4: 83.6 | 10: 84.3)
        int parts = (512 + B - 1) / B;
        const int cap = C / 128 > 0 ? C / 128 : 1;
        if (parts > cap) parts = cap;
        if (parts > 4) parts = 4;
        if (parts < 1) parts = 1;
        return parts;
    }
    if (B >= 2048 || C < 1024) return 1;
    return 2;
}

size_t bwd_reduce_raw_floats(int B, int n, int C) {
    if (n > 8) return (size_t)B * bwd_reduce_parts(B, n, C) * kGramFloats;
    return (size_t)B * bwd_reduce_parts(B, n, C) * (3 * 8 * 8);  // Gram input (the VALU sums need 8*8 + 3*8 + 1)
}

hipError_t launch_mix_bwd_reduce(const void *dy, int y_dtype, const void *x, int x_dtype,
                                 const void *w, int w_dtype, const void *f_inject,
                                 const float *Hpre, const float *Hpost, const float *M, int hstride,
                                 const float *q, const float *P, const float *r, const float *alpha,
                                 const float *b_res, const float *sk_state, BwdCoefOut out, float *raw, int B,
                                 int n, int C, int T, float eps, hipStream_t stream, const float *static_logits,
                                 float *static_state) {
    // n <= 8, dynamic H: channel sums per (sample, column part), coefficient backward as a second
    // small launch (static H: everything in the per-sample workgroup).  n > 8: always two launches.
    if (n > 8 && raw == nullptr) return hipErrorInvalidValue;
    const bool split = raw != nullptr && (n > 8 || hstride != 0);
    BwdReduceArgs a{dy, x, w, f_inject, Hpre, Hpost, M, q, P, r, alpha, b_res, sk_state, out,
                    hstride, w_dtype == kBF16, B, n, C, T, padded_D(n), eps,
                    split ? raw : nullptr, split ? bwd_reduce_parts(B, n, C) : 1};
    if (n > 8 && hstride == 0 && static_logits && static_state) {
        a.static_logits = static_logits;
        a.static_state = static_state;
    }
    if (n <= 8) {
#define MHC_SMALL(TG, TX)                                                   \
    return n <= 4 ? launch_small_np<TG, TX, 4>(a, stream) : launch_small_np<TG, TX, 8>(a, stream)
        if (y_dtype == kF32 && x_dtype == kF32) MHC_SMALL(float, float);
        if (y_dtype == kBF16 && x_dtype == kBF16) MHC_SMALL(bf16_t, bf16_t);
        if (y_dtype == kF32 && x_dtype == kBF16) MHC_SMALL(float, bf16_t);
#undef MHC_SMALL
        return hipErrorInvalidValue;
    }
    if (y_dtype == kF32 && x_dtype == kF32) return launch_large<float, float>(a, stream);
    if (y_dtype == kBF16 && x_dtype == kBF16) return launch_large<bf16_t, bf16_t>(a, stream);
    if (y_dtype == kF32 && x_dtype == kBF16) return launch_large<float, bf16_t>(a, stream);
    return hipErrorInvalidValue;
}

// n > 16, dynamic H, bf16 dy and x: the channel sums, then ONE launch that holds the coefficient
// workgroups and, behind them, the workgroups of the matrix-core dx kernel in the form that needs no
// result of the coefficient backward: dxp = M^T dy + Hpre (x) da into `dxp` (fp32), df or the dw rows u.
// s1part: [B][bwd_reduce_parts(B, n, C)] floats of scratch.
hipError_t launch_mix_bwd_reduce_with_dx(const void *dy, const void *x, const void *w, int w_dtype, const void *f_inject,
                                         const float *Hpre, const float *Hpost, const float *M, int hstride,
                                         const float *q, const float *P, const float *r, const float *alpha,
                                         const float *b_res, const float *sk_state, BwdCoefOut out, float *raw,
                                         float *s1part, float *dxp, void *df, float *u, int B, int n, int C, int T,
                                         float eps, hipStream_t stream) {
    if (n <= 16 || raw == nullptr || s1part == nullptr || hstride == 0 || C % 8 != 0) return hipErrorInvalidValue;
    const int parts = bwd_reduce_parts(B, n, C);
    BwdReduceArgs a{dy, x, w, f_inject, Hpre, Hpost, M, q, P, r, alpha, b_res, sk_state, out,
                    hstride, w_dtype == kBF16, B, n, C, T, padded_D(n), eps, raw, parts, s1part};
    BwdDxArgs d{dy, x, w, f_inject, nullptr, nullptr, Hpre, Hpost, M, q, nullptr, nullptr, nullptr, nullptr, df, u,
                nullptr, nullptr, hstride, w_dtype == kBF16, 0, B, n, C, padded_D(n), 1, s1part, parts, dxp};
    return launch_large<bf16_t, bf16_t>(a, stream, &d);
}

// The same for static H (n > 16, bf16 dy and x): with shared coefficients nothing of dx waits for another
// launch, so the dx workgroups beside the coefficient workgroups write the final dx (bf16) themselves.
// static_logits / static_state as in launch_mix_bwd_reduce.
hipError_t launch_mix_bwd_reduce_with_dx_static(const void *dy, const void *x, const void *w, int w_dtype,
                                                const void *f_inject, const float *Hpre, const float *Hpost,
                                                const float *M, const float *q, BwdCoefOut out, float *raw,
                                                float *s1part, void *dx, void *df, float *u, int B, int n, int C,
                                                int T, float eps, hipStream_t stream, const float *static_logits,
                                                float *static_state) {
    if (n <= 16 || raw == nullptr || s1part == nullptr || dx == nullptr || C % 8 != 0) return hipErrorInvalidValue;
    const int parts = bwd_reduce_parts(B, n, C);
    BwdReduceArgs a{dy, x, w, f_inject, Hpre, Hpost, M, q, nullptr, nullptr, nullptr, nullptr, nullptr, out,
                    0, w_dtype == kBF16, B, n, C, T, padded_D(n), eps, raw, parts, s1part};
    if (static_logits && static_state) {
        a.static_logits = static_logits;
        a.static_state = static_state;
    }
    BwdDxArgs d{dy, x, w, f_inject, nullptr, nullptr, Hpre, Hpost, M, q, nullptr, nullptr, nullptr, dx, df, u,
                nullptr, nullptr, 0, w_dtype == kBF16, 0, B, n, C, padded_D(n), 1, s1part, parts, nullptr};
    return launch_large<bf16_t, bf16_t>(a, stream, &d);
}

}  // namespace mhc
