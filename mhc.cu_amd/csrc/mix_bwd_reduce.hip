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
// n > 8 computes dM on the matrix cores (one 32x32 tile per sample, operands loaded from
// global memory in MFMA layout) and the vector sums on the VALU beside it.
#include "launchers.h"
#include "sinkhorn_device.h"

namespace mhc {

typedef __attribute__((__vector_size__(8 * sizeof(__bf16)))) __bf16 bf16x8_t;
typedef __attribute__((__vector_size__(16 * sizeof(float)))) float f32x16_t;

struct BwdReduceArgs {
    const void *dy, *x, *w, *f_inject;
    const float *Hpre, *Hpost, *M, *q, *P, *r, *alpha, *b_res;
    BwdCoefOut out;
    int hstride, w_bf16, B, n, C, T, DP;
    float eps;
    float *raw;   // n <= 8: when set, write the raw channel sums [B][parts][K] and stop
    int parts;    // column parts per sample (gridDim.y)
};

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
        o.dP[(size_t)b * DP + d] = v;
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
            o.dP[(size_t)b * DP + d] = 0.f;
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
    const float qinv = inject ? 0.f : 1.0f / a.q[b];

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
                fv[v] = s_a * qinv * wv;
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
    if (tid >= 16) return;

    // ---- epilogue on one 16-lane group (SkSmall layout) -------------------------------------
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
        float *red = a.out.red + (size_t)b * D;
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
    SK::template backward<false>(d, a.T, sc, tid);
#pragma unroll
    for (int e = 0; e < SK::EPL; e++) {
        const int c = c0 + e;
        if (r0 < n && c < n) {
            const int di = 2 * n + r0 * n + c;
            const float dtr = d[e] * E[e];
            dt[di] = dtr;
            dpw.put(di, dtr * al2 * rinv);
            S2 += dtr * Pb[di];
        }
    }
    S0 = row16_allreduce(S0); S1 = row16_allreduce(S1); S2 = row16_allreduce(S2);
    if (g == 0) {
        dt[D] = S0; dt[D + 1] = S1; dt[D + 2] = S2;
        a.out.cx[b] = (al0 * S0 + al1 * S1 + al2 * S2) * rinv * rinv / (float)(n * C);
    }
    dpw.pad(D, g, 16);
}


// =============================================================================================
// n <= 8, dynamic H: coefficient backward as its own launch - one 16-lane group per sample, four
// samples per wave, so the serial Sinkhorn chain of every sample runs concurrently instead of at
// the tail of a bandwidth-bound workgroup.  Input: the raw channel sums written by the kernel
// above ([B][parts][K], K = NP*NP + 3*NP + 1: dM | dHpost | A1 | A2 | s1).
// =============================================================================================
template <int NP, bool PRECISE>
__global__ __launch_bounds__(64) void coef_bwd_small_kernel(BwdReduceArgs a) {
    using SK = SkSmall<NP>;
    constexpr int K = NP * NP + 3 * NP + 1;
    extern __shared__ float sc[];  // Sinkhorn denominators, SK::scaling_floats(T)
    const int tid = threadIdx.x, g = tid & 15;
    const int b = blockIdx.x * 4 + (tid >> 4);
    if (b >= a.B) return;  // whole 16-lane groups leave together; DPP never crosses groups
    const int n = a.n, C = a.C, D = n * n + 2 * n;
    const bool inject = a.f_inject != nullptr;
    const int r0 = SK::row(g), c0 = SK::col0(g);
    // everything this lane needs from memory, issued up front
    const float *raw = a.raw + (size_t)b * a.parts * K;
    float dMe[SK::EPL], tpost = 0.f, tA1 = 0.f, tA2 = 0.f, s1 = 0.f;
#pragma unroll
    for (int e = 0; e < SK::EPL; e++) dMe[e] = 0.f;
    for (int p = 0; p < a.parts; p++) {
        const float *rp = raw + (size_t)p * K;
#pragma unroll
        for (int e = 0; e < SK::EPL; e++) dMe[e] += rp[r0 * NP + c0 + e];
        if (g < n) { tpost += rp[NP * NP + g]; tA1 += rp[NP * NP + NP + g]; tA2 += rp[NP * NP + 2 * NP + g]; }
        s1 += rp[K - 1];
    }
    const float *Pb = a.P + (size_t)b * D;
    const float al0 = a.alpha[0], al1 = a.alpha[1], al2 = a.alpha[2];
    const float rinv = 1.0f / a.r[b];
    const float qinv = inject ? 0.f : 1.0f / a.q[b];
    float pres[SK::EPL], bres[SK::EPL];
#pragma unroll
    for (int e = 0; e < SK::EPL; e++) {
        const bool ok = r0 < n && c0 + e < n;
        pres[e] = ok ? Pb[2 * n + r0 * n + c0 + e] : 0.f;
        bres[e] = ok ? a.b_res[r0 * n + c0 + e] : 0.f;
    }
    float hp = 0.f, ho = 0.f, ppre = 0.f, ppost = 0.f;
    if (g < n) { hp = a.Hpre[(size_t)b * n + g]; ho = a.Hpost[(size_t)b * n + g]; ppre = Pb[g]; ppost = Pb[n + g]; }

    if (g == 0) a.out.s1[b] = s1;
    float *dt = a.out.dt + (size_t)b * (D + 3);
    const DPWriter dpw{a.out, b, a.B, a.DP};
    float S0 = 0.f, S1 = 0.f, S2 = 0.f;  // sum_d dt_d p_d per alpha group
    if (g < n) {
        const float dHpost = tpost;
        const float dHpre = inject ? 0.f : tA1 * qinv - s1 * tA2 * qinv * qinv * qinv / (float)C;
        const float dtp = dHpre * hp * (1.0f - hp);
        const float dto = dHpost * ho * (1.0f - 0.5f * ho);
        dt[g] = dtp; dt[n + g] = dto;
        dpw.put(g, dtp * al0 * rinv); dpw.put(n + g, dto * al1 * rinv);
        S0 = dtp * ppre; S1 = dto * ppost;
    }
    float E[SK::EPL], m[SK::EPL], d[SK::EPL];
#pragma unroll
    for (int e = 0; e < SK::EPL; e++) {
        const bool ok = r0 < n && c0 + e < n;
        E[e] = ok ? expf(al2 * pres[e] + bres[e]) : 0.f;
        m[e] = E[e];
        d[e] = ok ? dMe[e] : 0.f;
    }
    SK::template forward<PRECISE>(m, g, n, a.T, a.eps, sc, tid);
    SK::template backward<PRECISE>(d, a.T, sc, tid);
#pragma unroll
    for (int e = 0; e < SK::EPL; e++) {
        const int c = c0 + e;
        if (r0 < n && c < n) {
            const int di = 2 * n + r0 * n + c;
            const float dtr = d[e] * E[e];
            dt[di] = dtr;
            dpw.put(di, dtr * al2 * rinv);
            S2 += dtr * pres[e];
        }
    }
    S0 = row16_allreduce(S0); S1 = row16_allreduce(S1); S2 = row16_allreduce(S2);
    if (g == 0) {
        dt[D] = S0; dt[D + 1] = S1; dt[D + 2] = S2;
        a.out.cx[b] = (al0 * S0 + al1 * S1 + al2 * S2) * rinv * rinv / (float)(n * C);
    }
    dpw.pad(D, g, 16);
}

// =============================================================================================
// n > 8: MFMA layout
// =============================================================================================
// One k-step operand pair: VL consecutive columns of row (lane & 31) of dy and of x; the two lane
// halves take adjacent column groups.  Both bf16: one v_mfma_f32_32x32x16_bf16 (exact products,
// fp32 accumulate).  Otherwise VL fp32 MFMAs (32x32x2), bf16 inputs widened exactly.
template <typename TG, typename TX> struct PairStep {
    static constexpr bool kBf16 = std::is_same<TG, bf16_t>::value && std::is_same<TX, bf16_t>::value;
    static constexpr int VL = kBf16 ? 8 : 4;
    float g[VL], x[VL];
    uint4 gbits, xbits;

    __device__ __forceinline__ void load(const TG *gp, const TX *xp, int c, int C, bool rvalid, bool vec_ok) {
        if (rvalid && vec_ok && c + VL <= C) {
            if constexpr (kBf16) {
                gbits = *reinterpret_cast<const uint4 *>(gp + c);
                xbits = *reinterpret_cast<const uint4 *>(xp + c);
                const uint32_t gw[4] = {gbits.x, gbits.y, gbits.z, gbits.w};
                const uint32_t xw[4] = {xbits.x, xbits.y, xbits.z, xbits.w};
#pragma unroll
                for (int i = 0; i < 4; i++) {
                    g[2 * i] = bf16lo_to_f32(gw[i]); g[2 * i + 1] = bf16hi_to_f32(gw[i]);
                    x[2 * i] = bf16lo_to_f32(xw[i]); x[2 * i + 1] = bf16hi_to_f32(xw[i]);
                }
            } else {
                load_vec<TG, VL>(gp + c, g);
                load_vec<TX, VL>(xp + c, x);
            }
        } else {
#pragma unroll
            for (int i = 0; i < VL; i++) {
                const bool ok = rvalid && c + i < C;
                g[i] = ok ? to_f32<TG>(gp[c + i]) : 0.f;
                x[i] = ok ? to_f32<TX>(xp[c + i]) : 0.f;
            }
            if constexpr (kBf16) {
                gbits = make_uint4(pack_bf16x2(g[0], g[1]), pack_bf16x2(g[2], g[3]),
                                   pack_bf16x2(g[4], g[5]), pack_bf16x2(g[6], g[7]));
                xbits = make_uint4(pack_bf16x2(x[0], x[1]), pack_bf16x2(x[2], x[3]),
                                   pack_bf16x2(x[4], x[5]), pack_bf16x2(x[6], x[7]));
            }
        }
    }
    // acc[i][j] += sum_k dy[i,k] x[j,k]
    __device__ __forceinline__ void mfma(f32x16_t &acc) const {
        if constexpr (kBf16) {
            acc = __builtin_amdgcn_mfma_f32_32x32x16_bf16(__builtin_bit_cast(bf16x8_t, gbits),
                                                          __builtin_bit_cast(bf16x8_t, xbits), acc, 0, 0, 0);
        } else {
#pragma unroll
            for (int i = 0; i < VL; i++)
                acc = __builtin_amdgcn_mfma_f32_32x32x2f32(g[i], x[i], acc, 0, 0, 0);
        }
    }
};

constexpr int kLargeCB = 512;  // columns staged per phase

// phase 0 of a column block: a, f, df*w per column into LDS; returns this thread's part of s1
template <typename TG, typename TX, int V>
__device__ __forceinline__ float bwd_large_phase0(const BwdReduceArgs &a, const TG *gb, const TX *xb,
                                                  const float *hp_s, const float *ho_s, float *a_s,
                                                  float *f_s, float *dfw_s, int b, int cb0, int cbn,
                                                  float qinv, bool inject) {
    const int n = a.n, C = a.C;
    float s1 = 0.f;
    for (int cc = threadIdx.x * V; cc < cbn; cc += 256 * V) {
        const int c = cb0 + cc;
        float sa[V], sdf[V];
#pragma unroll
        for (int v = 0; v < V; v++) { sa[v] = 0.f; sdf[v] = 0.f; }
        for (int i0 = 0; i0 < n; i0 += 8) {  // 16 loads in flight; streams >= n alias stream 0
            float xv[8][V], gv[8][V];
#pragma unroll
            for (int u = 0; u < 8; u++) {
                const size_t so = (size_t)(i0 + u < n ? i0 + u : 0) * C + c;
                load_vec<TX, V>(xb + so, xv[u]);
                load_vec<TG, V>(gb + so, gv[u]);
            }
#pragma unroll
            for (int u = 0; u < 8; u++) {
                const float hp = i0 + u < n ? hp_s[i0 + u] : 0.f, ho = i0 + u < n ? ho_s[i0 + u] : 0.f;
#pragma unroll
                for (int v = 0; v < V; v++) { sa[v] += hp * xv[u][v]; sdf[v] += ho * gv[u][v]; }
            }
        }
        float fv[V];
        if (inject) load_vec<TX, V>(static_cast<const TX *>(a.f_inject) + (size_t)b * C + c, fv);
#pragma unroll
        for (int v = 0; v < V; v++) {
            float dfw = 0.f;
            if (!inject) {
                const float wv = load_w_(a.w, a.w_bf16, c + v);
                fv[v] = sa[v] * qinv * wv;
                dfw = sdf[v] * wv;
            }
            a_s[cc + v] = sa[v]; f_s[cc + v] = fv[v]; dfw_s[cc + v] = dfw;
            s1 += dfw * sa[v];
        }
    }
    return s1;
}

template <typename TG, typename TX, int NP>
__global__ __launch_bounds__(256) void mix_bwd_reduce_large_kernel(BwdReduceArgs a) {
    using SK = SkLds<NP>;
    using PS = PairStep<TG, TX>;
    constexpr int VL = PS::VL;
    extern __shared__ float smem[];
    float *a_s = smem;                 // [CB]
    float *f_s = a_s + kLargeCB;       // [CB]
    float *dfw_s = f_s + kLargeCB;     // [CB]
    float *hp_s = dfw_s + kLargeCB;    // [32] Hpre
    float *ho_s = hp_s + 32;           // [32] Hpost
    float *vec_s = ho_s + 32;          // [3][32] dHpost | A1 | A2 totals
    float *red_s = vec_s + 96;         // [8]
    float *xw = red_s + 8;             // cross-wave scratch [3][19][64], later reused by Sinkhorn
    const int b = blockIdx.x, n = a.n, C = a.C, tid = threadIdx.x;
    const int lane = tid & 63, wave = tid >> 6, row = lane & 31, kh = lane >> 5;
    const TG *__restrict__ gb = static_cast<const TG *>(a.dy) + (size_t)b * n * C;
    const TX *__restrict__ xb = static_cast<const TX *>(a.x) + (size_t)b * n * C;
    const bool inject = a.f_inject != nullptr;
    const float qinv = inject ? 0.f : 1.0f / a.q[b];
    if (tid < 32) {
        hp_s[tid] = tid < n ? a.Hpre[(size_t)b * a.hstride + tid] : 0.f;
        ho_s[tid] = tid < n ? a.Hpost[(size_t)b * a.hstride + tid] : 0.f;
    }
    __syncthreads();

    f32x16_t acc;
#pragma unroll
    for (int i = 0; i < 16; i++) acc[i] = 0.f;
    float vpost = 0.f, vA1 = 0.f, vA2 = 0.f, s1 = 0.f;
    const bool rvalid = row < n;
    const bool vec_ok = C % VL == 0;
    const TG *grow = gb + (size_t)(rvalid ? row : 0) * C;
    const TX *xrow = xb + (size_t)(rvalid ? row : 0) * C;

    for (int cb0 = 0; cb0 < C; cb0 += kLargeCB) {
        const int cbn = min(kLargeCB, C - cb0);
        if (C % 2 == 0)
            s1 += bwd_large_phase0<TG, TX, 2>(a, gb, xb, hp_s, ho_s, a_s, f_s, dfw_s, b, cb0, cbn, qinv, inject);
        else
            s1 += bwd_large_phase0<TG, TX, 1>(a, gb, xb, hp_s, ho_s, a_s, f_s, dfw_s, b, cb0, cbn, qinv, inject);
        __syncthreads();
        // phase 1: dM tile on the matrix cores, vector sums beside it
        const int nsteps = (cbn + 2 * VL - 1) / (2 * VL);
        for (int s = wave; s < nsteps; s += 4) {
            const int cc = s * 2 * VL + kh * VL;
            PS ps;
            ps.load(grow, xrow, cb0 + cc, cb0 + cbn, rvalid, vec_ok);
            ps.mfma(acc);
#pragma unroll
            for (int v = 0; v < VL; v++) {
                if (cc + v < cbn) {  // operands beyond the block are zero; LDS beyond it is stale
                    vpost += ps.g[v] * f_s[cc + v];
                    vA1 += ps.x[v] * dfw_s[cc + v];
                    vA2 += ps.x[v] * a_s[cc + v];
                }
            }
        }
        __syncthreads();
    }

    // ---- cross-wave totals (wave 0 finishes; the other waves only keep the barriers) ---------
    vpost += __shfl_xor(vpost, 32, kWave);
    vA1 += __shfl_xor(vA1, 32, kWave);
    vA2 += __shfl_xor(vA2, 32, kWave);
    s1 = wave_allreduce_sum(s1);
    if (wave > 0) {
        float *dst = xw + (size_t)(wave - 1) * 19 * 64;
#pragma unroll
        for (int i = 0; i < 16; i++) dst[i * 64 + lane] = acc[i];
        dst[16 * 64 + lane] = vpost; dst[17 * 64 + lane] = vA1; dst[18 * 64 + lane] = vA2;
    }
    if (lane == 0) red_s[wave] = s1;
    __syncthreads();
    const bool w0 = wave == 0;
    float *Es = xw;                      // [NP][LD]
    float *dO = Es + NP * SK::LD;        // [NP][LD]
    float *u = dO + NP * SK::LD, *v = u + NP, *tmp = v + NP;
    float *rho = tmp + NP, *ssc = rho + a.T * NP;
    if (w0) {
#pragma unroll
        for (int w = 0; w < 3; w++) {
            const float *src = xw + (size_t)w * 19 * 64;
#pragma unroll
            for (int i = 0; i < 16; i++) acc[i] += src[i * 64 + lane];
            vpost += src[16 * 64 + lane]; vA1 += src[17 * 64 + lane]; vA2 += src[18 * 64 + lane];
        }
        s1 = (red_s[0] + red_s[1]) + (red_s[2] + red_s[3]);
        if (lane < 32) { vec_s[lane] = vpost; vec_s[32 + lane] = vA1; vec_s[64 + lane] = vA2; }
    }
    __syncthreads();
    // dM[i][j] sits in acc: j = lane & 31, i = 8*(reg/4) + 4*(lane/32) + reg%4.  Stage it in the
    // Sinkhorn backward buffer (which reuses the cross-wave scratch, now fully consumed).
    if (w0) {
#pragma unroll
        for (int i = 0; i < 16; i++) {
            const int ri = 8 * (i >> 2) + 4 * kh + (i & 3);
            if (ri < NP && row < NP) dO[ri * SK::LD + row] = acc[i];
        }
    }
    __syncthreads();

    const int D = n * n + 2 * n;
    float dHpre = 0.f, dHpost = 0.f;
    if (w0 && lane < n) {
        dHpost = vec_s[lane];
        dHpre = inject ? 0.f
                       : vec_s[32 + lane] * qinv - s1 * vec_s[64 + lane] * qinv * qinv * qinv / (float)C;
    }
    if (tid == 0) a.out.s1[b] = s1;
    if (a.hstride == 0) {
        if (w0) {
            float *red = a.out.red + (size_t)b * D;
            for (int e = lane; e < n * n; e += kWave) red[e] = dO[(e / n) * SK::LD + (e % n)];
            if (lane < n) { red[n * n + lane] = dHpre; red[n * n + n + lane] = dHpost; }
        }
        return;
    }
    const float *Pb = a.P + (size_t)b * D;
    const float al0 = a.alpha[0], al1 = a.alpha[1], al2 = a.alpha[2];
    const float rinv = 1.0f / a.r[b];
    float *dt = a.out.dt + (size_t)b * (D + 3);
    const DPWriter dpw{a.out, b, a.B, a.DP};
    float S0 = 0.f, S1 = 0.f, S2 = 0.f;  // sum_d dt_d p_d per alpha group
    if (w0) {
        if (lane < n) {
            const float hp = hp_s[lane], ho = ho_s[lane];
            const float dtp = dHpre * hp * (1.0f - hp);
            const float dto = dHpost * ho * (1.0f - 0.5f * ho);
            dt[lane] = dtp; dt[n + lane] = dto;
            dpw.put(lane, dtp * al0 * rinv); dpw.put(n + lane, dto * al1 * rinv);
            S0 = dtp * Pb[lane]; S1 = dto * Pb[n + lane];
        }
        for (int e = lane; e < NP * NP; e += kWave) {
            const int r0 = e / NP, c = e % NP;
            Es[r0 * SK::LD + c] =
                (r0 < n && c < n) ? expf(al2 * Pb[2 * n + r0 * n + c] + a.b_res[r0 * n + c]) : 0.f;
        }
    }
    __syncthreads();
    SK::forward(Es, u, v, n, a.T, a.eps, rho, ssc, tid);
    SK::backward(Es, dO, u, v, tmp, n, a.T, rho, ssc, tid);
    if (w0) {
        for (int e = lane; e < n * n; e += kWave) {
            const int r0 = e / n, c = e % n;
            const int di = 2 * n + e;
            const float dtr = dO[r0 * SK::LD + c] * Es[r0 * SK::LD + c];
            dt[di] = dtr;
            dpw.put(di, dtr * al2 * rinv);
            S2 += dtr * Pb[di];
        }
        S0 = wave_allreduce_sum(S0); S1 = wave_allreduce_sum(S1); S2 = wave_allreduce_sum(S2);
        if (lane == 0) {
            dt[D] = S0; dt[D + 1] = S1; dt[D + 2] = S2;
            a.out.cx[b] = (al0 * S0 + al1 * S1 + al2 * S2) * rinv * rinv / (float)(n * C);
        }
        dpw.pad(D, lane, kWave);
    }
}

// =============================================================================================
// launch
// =============================================================================================
template <typename TG, typename TX, int NP, int V>
static hipError_t launch_small(const BwdReduceArgs &a, hipStream_t stream) {
    const int nch = (a.C / V + a.parts - 1) / a.parts;  // chunks per column part
    int nt = (nch + 63) / 64 * 64;
    if (nt > 256) nt = 256;
    constexpr int K = NP * NP + 3 * NP + 1;
    const size_t smem = sizeof(float) * (K * 16 + K + SkSmall<NP>::scaling_floats(a.T));
    mix_bwd_reduce_small_kernel<TG, TX, NP, V><<<dim3(a.B, a.parts), nt, smem, stream>>>(a);
    hipError_t e = hipGetLastError();
    if (e != hipSuccess || !a.raw) return e;
    // fp32 activations: the parity tier, IEEE divisions in the Sinkhorn chain
    constexpr bool kPrecise = std::is_same<TX, float>::value;
    coef_bwd_small_kernel<NP, kPrecise><<<(a.B + 3) / 4, 64, sizeof(float) * SkSmall<NP>::scaling_floats(a.T), stream>>>(a);
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

template <typename TG, typename TX, int NP>
static hipError_t launch_large(const BwdReduceArgs &a, hipStream_t stream) {
    using SK = SkLds<NP>;
    const size_t sk = SK::backward_floats(a.T);
    const size_t xw = 3 * 19 * 64;
    const size_t smem = sizeof(float) * (3 * kLargeCB + 64 + 96 + 8 + (sk > xw ? sk : xw));
    mix_bwd_reduce_large_kernel<TG, TX, NP><<<a.B, 256, smem, stream>>>(a);
    return hipGetLastError();
}

// Column parts per sample when the reduction is split from the coefficient backward.
int bwd_reduce_parts(int B, int n, int C) {
    (void)n;
    if (B >= 2048 || C < 1024) return 1;
    return 2;
}

hipError_t launch_mix_bwd_reduce(const void *dy, int y_dtype, const void *x, int x_dtype,
                                 const void *w, int w_dtype, const void *f_inject,
                                 const float *Hpre, const float *Hpost, const float *M, int hstride,
                                 const float *q, const float *P, const float *r, const float *alpha,
                                 const float *b_res, BwdCoefOut out, float *raw, int B, int n, int C,
                                 int T, float eps, hipStream_t stream) {
    // dynamic H with n <= 8: channel sums per (sample, column part), coefficient backward as a
    // second small launch; otherwise everything in the per-sample workgroup
    const bool split = raw != nullptr && hstride != 0 && n <= 8;
    BwdReduceArgs a{dy, x, w, f_inject, Hpre, Hpost, M, q, P, r, alpha, b_res, out,
                    hstride, w_dtype == kBF16, B, n, C, T, padded_D(n), eps,
                    split ? raw : nullptr, split ? bwd_reduce_parts(B, n, C) : 1};
    if (n <= 8) {
#define MHC_SMALL(TG, TX)                                                   \
    return n <= 4 ? launch_small_np<TG, TX, 4>(a, stream) : launch_small_np<TG, TX, 8>(a, stream)
        if (y_dtype == kF32 && x_dtype == kF32) MHC_SMALL(float, float);
        if (y_dtype == kBF16 && x_dtype == kBF16) MHC_SMALL(bf16_t, bf16_t);
        if (y_dtype == kF32 && x_dtype == kBF16) MHC_SMALL(float, bf16_t);
#undef MHC_SMALL
        return hipErrorInvalidValue;
    }
#define MHC_LARGE(TG, TX)                                                   \
    return n <= 16 ? launch_large<TG, TX, 16>(a, stream) : launch_large<TG, TX, 32>(a, stream)
    if (y_dtype == kF32 && x_dtype == kF32) MHC_LARGE(float, float);
    if (y_dtype == kBF16 && x_dtype == kBF16) MHC_LARGE(bf16_t, bf16_t);
    if (y_dtype == kF32 && x_dtype == kBF16) MHC_LARGE(float, bf16_t);
#undef MHC_LARGE
    return hipErrorInvalidValue;
}

}  // namespace mhc
