// Backward, first launch for n <= 8 in the bf16 tier when a sample's rows fit in the registers of one
// workgroup: dy and x cross HBM ONCE for everything that depends only on the sample itself.
//
// One workgroup per sample: wave 0 runs the coefficient backward, waves 1..4 each keep their share of
// the sample's [n, C] rows of dy and x in registers (a lane holds 8 consecutive channels of one stream,
// four neighbouring lanes hold the four streams of a stream group - the words as they lie in memory,
// which is the operand layout of v_mfma_f32_4x4x4_16b_bf16).
//
//   1. Gram sums on the matrix cores, as in gram_small_kernel:
//        dM = dy x^T     W1 = dy diag(w) x^T     XX = x x^T          reference stream_ops.cuh:852-927
//   2. wave 0: dHpre / dHpost from the sums, sigmoid derivatives, exact Sinkhorn backward, dP in the
//      layouts of the projection backward, cx (CoefBwdSmall)          reference ops.py:297-349
//   3. waves 1..4, meanwhile, from the registers they already hold:
//        dxp[j,c] = sum_i M[i,j] dy[i,c] + Hpre[j] da[c]               reference stream_ops.cuh:761-850, :646-663
//        da = df w / q - a s1 / (C q^3),  df = Hpost . dy, a = Hpre . x   reference rmsnorm.cuh:255-294
//        u[c] = df a / q   (the sample's summand of dw),  df (kernel-level view)
//      s1 = Hpost^T W1 Hpre follows from the Gram sums, so this step does not wait for the serial
//      Sinkhorn chain of step 2: the stores of dxp run under it.
// The terms of dx that need dP (dP phi, reference ops.py:336-338) or cx (-cx x, ops.py:340-349) are
// added by the projection-backward launch that follows (proj_bwd.hip, which owns a column slab for all
// samples and therefore also finishes dphi without batch-split partial sums).
// The mixing uses the VALU with DPP quad broadcasts: the contraction runs over streams, which lie
// across the four lanes of a quad.
#include "coef_bwd_small.h"

#include <type_traits>
#include "tuning.h"

namespace mhc {

struct BwdResidentArgs {
    BwdReduceArgs r;   // inputs and the outputs of the coefficient backward
    void *dxp;         // [B, n, C], stored like x (bf16, or fp32 with F32)
    void *df;          // [B, C] or nullptr (only with r.f_inject), stored like x
    float *u;          // [B, C] (unused with r.f_inject)
};

constexpr int kResTileWaves = 4;                         // waves that hold the tile
constexpr int kResMaxItems = 5;                          // 128-channel steps per tile wave

template <int SEL> __device__ __forceinline__ float quad_bcast(float v) {
    return __int_as_float(__builtin_amdgcn_update_dpp(0, __float_as_int(v), SEL * 0x55, 0xF, 0xF, true));
}
__device__ __forceinline__ float quad_allreduce(float v) {
    v += dpp_mov<kDppQuadXor1>(v);
    v += dpp_mov<kDppQuadXor2>(v);
    return v;
}

// Eight consecutive activation values as four words of bf16 pairs.  bf16 storage: the 16 bytes as
// loaded.  fp32 storage (F32): two 16-byte loads, rounded to bf16 (nearest even) by get() - called
// once all loads of the workgroup have been requested.
template <bool F32> struct Act8;
template <> struct Act8<false> {
    uint4 r;
    __device__ __forceinline__ void load(const void *base, size_t elem, bool ok) {
        r = load16_masked(reinterpret_cast<const uint4 *>(static_cast<const bf16_t *>(base) + (ok ? elem : 0)), ok);
    }
    __device__ __forceinline__ uint4 get() const { return r; }
};
template <> struct Act8<true> {
    uint4 r0, r1;
    __device__ __forceinline__ void load(const void *base, size_t elem, bool ok) {
        const uint4 *p = reinterpret_cast<const uint4 *>(static_cast<const float *>(base) + (ok ? elem : 0));
        r0 = load16_masked(p, ok);
        r1 = load16_masked(p + 1, ok);
    }
    __device__ __forceinline__ uint4 get() const {
        return make_uint4(pack_bf16x2(__uint_as_float(r0.x), __uint_as_float(r0.y)), pack_bf16x2(__uint_as_float(r0.z), __uint_as_float(r0.w)),
                          pack_bf16x2(__uint_as_float(r1.x), __uint_as_float(r1.y)), pack_bf16x2(__uint_as_float(r1.z), __uint_as_float(r1.w)));
    }
};

// F32: dy, x (and an injected f) are stored as fp32 and rounded to bf16 as they are loaded; dxp and df
// are written as fp32.  The arithmetic is the same either way.
// STATIC: shared coefficients ([n] / [n, n] instead of per sample).  There is no projection, so dxp is
// the complete dx; wave 0 only turns the sums into the sample's row of raw coefficient gradients
// (dM | dHpre | dHpost), whose batch sum feeds the one Sinkhorn backward of the static layer.
template <int NP, int WMODE, int ITEMS, bool F32, bool STATIC = false, int TWV = kResTileWaves>
__global__ __launch_bounds__(64 * (TWV + (STATIC ? 0 : 1))) void bwd_resident_kernel(BwdResidentArgs ra) {
    using TS = typename std::conditional<F32, float, bf16_t>::type;  // storage type of the activations
    static_assert(NP == 4 || NP == 8, "stream groups of four");
    using SK = SkSmall<NP>;
    using CB = CoefBwdSmall<NP, false, true, STATIC>;
    constexpr int NB = NP / 4;            // stream groups
    constexpr int K = 3 * NP * NP;
    constexpr int TW = TWV;
    constexpr bool inject = WMODE == kGramInject;
    const BwdReduceArgs &a = ra.r;
    const int hs = STATIC ? 0 : a.n;      // sample stride of Hpre / Hpost (M: hs * n)
    // STATIC has no serial chain to run beside the tile: no coefficient wave, four waves per workgroup
    // (its few coefficient lanes are the first lanes of tile wave 0), so four workgroups fit a CU
    constexpr int CW = STATIC ? 0 : 1;    // coefficient waves in front of the tile waves
    __shared__ float slot_s[K * TW * 4];  // one slot per 16-lane row of the tile waves
    __shared__ float tot_s[K + 1];        // the sums, then s1
    __shared__ float park_s[STATIC ? 1 : SkSmall<NP>::kGroup];  // one value per coefficient lane, see below
    extern __shared__ float sc[];         // Sinkhorn denominators, SK::scaling_floats(T), then CB::kXch
    const int b = blockIdx.x, n = a.n, C = a.C;
    const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
    const int pwg = blockIdx.x;
    (void)pwg;
    MHC_PHASE_ZERO(kPhaseGramSmall, pwg);
    MHC_PHASE_ZERO(kPhaseDxSmall, pwg);   // second timeline: the first tile wave (thread 64)
    MHC_PHASE_BEGIN(pclk);
    MHC_PHASE_BEGIN(tclk);
    CB cb;
    if (tid < SK::kGroup) {
        // everything the coefficient backward needs besides the sums, requested at once
        cb.prefetch(a, b, tid);
        if constexpr (!STATIC) {
            cb.forward_recompute(a, b, tid, tid, sc);
            // The coefficient lanes share their register budget with the tile code below; the final
            // iterate lived across it in scratch memory, and reading it back was a global round trip in
            // front of the serial Sinkhorn sweep: it is parked in LDS instead.
            park_s[tid] = cb.m_fin;
        }
    }
    // the NP^2 threads that will hold the sums of W1 (one DPP row of wave 0 for 4x4, wave 1 for 8x8) ask
    // for their factor of s1 = Hpost^T W1 Hpre now, not behind the barrier
    // (the two factors stay as loaded until then: for 8x8 these threads are a tile wave, and a product
    // here would make it wait for them in front of its tile loads)
    float ho_l = 0.f, hp_l = 0.f;
    bool hohp_ok = false;
    if (!inject && tid >= NP * NP && tid < 2 * NP * NP) {
        const int e = tid - NP * NP, r = e / NP, c = e % NP;
        ho_l = a.Hpost[(size_t)b * hs + (r < n ? r : 0)];
        hp_l = a.Hpre[(size_t)b * hs + (c < n ? c : 0)];
        hohp_ok = r < n && c < n;
    }
    MHC_PHASE_ADD(kPhaseGramSmall, pwg, 0, pclk);
    const int blk = lane >> 2, i = lane & 3;
    const int tw = wave - CW;             // tile wave index, -1 for the coefficient wave
    const bool tile = tw >= 0;

    // ---- tile waves: every load of the sample up front -----------------------------------------
    uint4 gr[ITEMS][NB], xr[ITEMS][NB], fr[ITEMS];
    Act8<F32> graw[ITEMS][NB], xraw[ITEMS][NB], fraw[ITEMS];
    // (the RMSNorm weight chunks stay in registers next to the tile: fetching them again where they are
    // used, one item ahead, to save registers measured slower - B=1280, C=2560 static backward 33.4 -> 34.1 us -
    // and forcing four workgroups per CU made the compiler spill: 50.1 us)
    RawVec<bf16_t, 8> wb[ITEMS];
    RawVec<float, 8> wf[ITEMS];
    bool in[ITEMS], sv[NB];
    float hpre[NB], hpost[NB], Mc[NB][NB][4], qraw = 1.f;
    if (tile) {
        size_t rowoff[NB];
#pragma unroll
        for (int I = 0; I < NB; I++) {
            sv[I] = 4 * I + i < n;  // streams >= n: masked, they alias stream 0
            rowoff[I] = (size_t)b * n * C + (size_t)(sv[I] ? 4 * I + i : 0) * C;
        }
#pragma unroll
        for (int it = 0; it < ITEMS; it++) {
            const int c = (tw + TW * it) * 128 + blk * 8;
            in[it] = c < C;  // C % 8 == 0: a chunk is inside or outside
            const int cc = in[it] ? c : 0;
#pragma unroll
            for (int I = 0; I < NB; I++) {
                graw[it][I].load(a.dy, rowoff[I] + cc, in[it] && sv[I]);
                xraw[it][I].load(a.x, rowoff[I] + cc, in[it] && sv[I]);
            }
            if constexpr (inject) fraw[it].load(a.f_inject, (size_t)b * C + cc, in[it] && i == 0);
            else if constexpr (WMODE == kGramWBf16) wb[it].load(static_cast<const bf16_t *>(a.w) + cc);
            else wf[it].load(static_cast<const float *>(a.w) + cc);
        }
        // this lane's coefficients for step 3 (its own streams j = 4I + i), in flight with the tile
        const float *Hp = a.Hpre + (size_t)b * hs, *Ho = a.Hpost + (size_t)b * hs, *Mb = a.M + (size_t)b * hs * n;
#pragma unroll
        for (int I = 0; I < NB; I++) {
            hpre[I] = Hp[sv[I] ? 4 * I + i : 0];
            hpost[I] = Ho[sv[I] ? 4 * I + i : 0];
#pragma unroll
            for (int J = 0; J < NB; J++)
#pragma unroll
                for (int ii = 0; ii < 4; ii++) {
                    // Mc[I][J][ii] = M[source stream 4J + ii][target stream 4I + i]
                    const bool ok = sv[I] && 4 * J + ii < n;
                    const float m = Mb[ok ? (4 * J + ii) * n + 4 * I + i : 0];
                    Mc[I][J][ii] = ok ? m : 0.f;
                }
        }
        if constexpr (!inject) qraw = a.q[b];
#pragma unroll
        for (int I = 0; I < NB; I++)
            if (!sv[I]) { hpre[I] = 0.f; hpost[I] = 0.f; }
        // every load is requested: from here on the tile is four words of bf16 pairs per chunk
#pragma unroll
        for (int it = 0; it < ITEMS; it++) {
#pragma unroll
            for (int I = 0; I < NB; I++) { gr[it][I] = graw[it][I].get(); xr[it][I] = xraw[it][I].get(); }
            if constexpr (inject) fr[it] = fraw[it].get();
        }
    }

    MHC_PHASE_ADD_BY(64, kPhaseDxSmall, pwg, 0, tclk);
    // ---- 1. Gram sums -------------------------------------------------------------------------------
    if (tile) {
        f32x4_t acc[3][NB][NB];
#pragma unroll
        for (int m = 0; m < 3; m++)
#pragma unroll
            for (int I = 0; I < NB; I++)
#pragma unroll
                for (int J = 0; J < NB; J++) acc[m][I][J] = f32x4_t{0.f, 0.f, 0.f, 0.f};
#pragma unroll
        for (int it = 0; it < ITEMS; it++) {
            bf16x4_t g0[NB], g1[NB], x0[NB], x1[NB];  // first / second group of four channels
#pragma unroll
            for (int I = 0; I < NB; I++) {
                g0[I] = bf16x4_of(gr[it][I].x, gr[it][I].y); g1[I] = bf16x4_of(gr[it][I].z, gr[it][I].w);
                x0[I] = bf16x4_of(xr[it][I].x, xr[it][I].y); x1[I] = bf16x4_of(xr[it][I].z, xr[it][I].w);
            }
#pragma unroll
            for (int I = 0; I < NB; I++)
#pragma unroll
                for (int J = 0; J < NB; J++) {
                    acc[0][I][J] = mfma4(g0[I], x0[J], acc[0][I][J]);
                    acc[0][I][J] = mfma4(g1[I], x1[J], acc[0][I][J]);
                }
            if constexpr (inject) {
                const bf16x4_t f0 = bf16x4_of(fr[it].x, fr[it].y), f1 = bf16x4_of(fr[it].z, fr[it].w);
#pragma unroll
                for (int I = 0; I < NB; I++) {
                    acc[1][I][0] = mfma4(g0[I], f0, acc[1][I][0]);
                    acc[1][I][0] = mfma4(g1[I], f1, acc[1][I][0]);
                }
            } else {
                float wv[8];
                if constexpr (WMODE == kGramWBf16) wb[it].get(wv);
                else wf[it].get(wv);
#pragma unroll
                for (int I = 0; I < NB; I++) {
                    // dy * w as a bf16 pair (rounded value + remainder): dHpre is a difference of two
                    // sums built on W1, a single rounding of the products is not enough for it
                    const uint32_t gw[4] = {gr[it][I].x, gr[it][I].y, gr[it][I].z, gr[it][I].w};
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
        // Lane (block, j) holds column j of its block's products, register = row.  Sum over the four
        // blocks of a 16-lane row with DPP, one LDS slot per row.
        const int slot = (tid - 64 * CW) >> 4;
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
                            slot_s[(m * NP * NP + (4 * I + r) * NP + 4 * J + (tid & 3)) * (TW * 4) + slot] = v;
                    }
    }
    MHC_PHASE_ADD_BY(64, kPhaseDxSmall, pwg, 1, tclk);
    __syncthreads();
    MHC_PHASE_ADD(kPhaseGramSmall, pwg, 1, pclk);
    // K threads finish the sums; the NP^2 threads that hold W1 (one DPP row for 4x4, wave 1 for 8x8)
    // also form s1 = Hpost^T W1 Hpre, which the tile waves need for da
    if (tid < K) {
        float v = 0.f;
#pragma unroll
        for (int sl = 0; sl < TW * 4; sl++) v += slot_s[tid * (TW * 4) + sl];
        tot_s[tid] = v;
        if (!inject && tid >= NP * NP && tid < 2 * NP * NP) {
            float t = hohp_ok ? ho_l * hp_l * v : 0.f;
            if constexpr (NP == 4) t = row16_allreduce(t);
            else t = wave_allreduce_sum(t);
            if (tid == NP * NP) tot_s[K] = t;
        }
    }
    __syncthreads();

    MHC_PHASE_ADD(kPhaseGramSmall, pwg, 2, pclk);
    MHC_PHASE_ADD_BY(64, kPhaseDxSmall, pwg, 2, tclk);
    // ---- 2. coefficient backward on the first lanes of wave 0 -----------------------------------------
    if (tid < SK::kGroup) {
        if constexpr (!STATIC) {
            cb.m_fin = park_s[tid];
        }
        cb.fetch_sums(tot_s, 1);
        cb.run(a, b, tid, tid, sc, sc + (STATIC ? 0 : SK::scaling_floats(a.T)));
    }
    MHC_PHASE_ADD(kPhaseGramSmall, pwg, 3, pclk);
    if (!tile) return;  // the coefficient wave (none with STATIC) is done

    // ---- 3. tile waves: dxp, u, df ---------------------------------------------------------------------
    float qinv = 0.f, k2 = 0.f;
    if constexpr (!inject) {
        qinv = 1.0f / qraw;
        k2 = tot_s[K] * qinv * qinv * qinv / (float)C;
    }
#pragma unroll
    for (int it = 0; it < ITEMS; it++) {
        const int c = (tw + TW * it) * 128 + blk * 8;
        if (!in[it]) continue;  // quads are inside or outside together: the DPP exchanges stay within a quad
        float gv[NB][8], xv[NB][8];
#pragma unroll
        for (int I = 0; I < NB; I++) {
            const uint32_t gw[4] = {gr[it][I].x, gr[it][I].y, gr[it][I].z, gr[it][I].w};
            const uint32_t xw[4] = {xr[it][I].x, xr[it][I].y, xr[it][I].z, xr[it][I].w};
#pragma unroll
            for (int k = 0; k < 4; k++) {
                gv[I][2 * k] = bf16lo_to_f32(gw[k]); gv[I][2 * k + 1] = bf16hi_to_f32(gw[k]);
                xv[I][2 * k] = bf16lo_to_f32(xw[k]); xv[I][2 * k + 1] = bf16hi_to_f32(xw[k]);
            }
        }
        float dfv[8], da[8];
#pragma unroll
        for (int v = 0; v < 8; v++) {
            float pd = 0.f;
#pragma unroll
            for (int I = 0; I < NB; I++) pd += hpost[I] * gv[I][v];
            dfv[v] = quad_allreduce(pd);
        }
        if constexpr (inject) {
#pragma unroll
            for (int v = 0; v < 8; v++) da[v] = 0.f;
            if (ra.df && i == 0) store_vec<TS, 8>(static_cast<TS *>(ra.df) + (size_t)b * C + c, dfv);
        } else {
            float wv[8], uv[8];
            if constexpr (WMODE == kGramWBf16) wb[it].get(wv);
            else wf[it].get(wv);
#pragma unroll
            for (int v = 0; v < 8; v++) {
                float pa = 0.f;
#pragma unroll
                for (int I = 0; I < NB; I++) pa += hpre[I] * xv[I][v];
                const float av = quad_allreduce(pa);
                da[v] = dfv[v] * wv[v] * qinv - av * k2;
                uv[v] = dfv[v] * av * qinv;
            }
            if (i == 0) store_vec<float, 8>(ra.u + (size_t)b * C + c, uv);
        }
#pragma unroll
        for (int I = 0; I < NB; I++) {
            float out[8];
#pragma unroll
            for (int v = 0; v < 8; v++) out[v] = hpre[I] * da[v];
#pragma unroll
            for (int J = 0; J < NB; J++)
#pragma unroll
                for (int v = 0; v < 8; v++) {
                    out[v] += Mc[I][J][0] * quad_bcast<0>(gv[J][v]);
                    out[v] += Mc[I][J][1] * quad_bcast<1>(gv[J][v]);
                    out[v] += Mc[I][J][2] * quad_bcast<2>(gv[J][v]);
                    out[v] += Mc[I][J][3] * quad_bcast<3>(gv[J][v]);
                }
            // plain stores: the projection-backward launch reads dxp back right away
            if (sv[I]) store_vec<TS, 8>(static_cast<TS *>(ra.dxp) + ((size_t)b * n + 4 * I + i) * C + c, out);
        }
    }
    MHC_PHASE_ADD_BY(64, kPhaseDxSmall, pwg, 3, tclk);
}

// The rows of a sample must fit the tile waves' registers; the Sinkhorn state shares the LDS.
// Activations: dy and x both bf16, or both fp32 with x marked as "consumed as bf16".
bool bwd_resident_supported(int x_dtype, int y_dtype, int phi_dtype, int n, int C, int T) {
    const bool io = (x_dtype == kBF16 && y_dtype == kBF16) || (x_dtype == kF32AsBF16 && y_dtype == kF32);
    return io && phi_dtype == kBF16 && n <= 8 && C % 8 == 0 && C <= 128 * kResTileWaves * kResMaxItems && T <= 32;
}

template <int NP, int WMODE, bool F32, bool STATIC, int TW>
static hipError_t launch_items_tw(const BwdResidentArgs &ra, hipStream_t stream) {
    using SK = SkSmall<NP>;
    using CB = CoefBwdSmall<NP, false, true, STATIC>;
    const size_t smem = sizeof(float) * ((STATIC ? 0 : SK::scaling_floats(ra.r.T)) + CB::kXch);
    const int items = (ra.r.C + 128 * TW - 1) / (128 * TW);
    const dim3 grid(ra.r.B);
    const int threads = 64 * (TW + (STATIC ? 0 : 1));
    constexpr int kMaxItems = TW == kResTileWaves ? kResMaxItems : 2;  // wider workgroups are for rows they hold in one or two items
    switch (items) {
        case 1: bwd_resident_kernel<NP, WMODE, 1, F32, STATIC, TW><<<grid, threads, smem, stream>>>(ra); break;
        case 2: bwd_resident_kernel<NP, WMODE, 2, F32, STATIC, TW><<<grid, threads, smem, stream>>>(ra); break;
        case 3: if constexpr (kMaxItems >= 3) { bwd_resident_kernel<NP, WMODE, 3, F32, STATIC, TW><<<grid, threads, smem, stream>>>(ra); break; } return hipErrorInvalidValue;
        case 4: if constexpr (kMaxItems >= 4) { bwd_resident_kernel<NP, WMODE, 4, F32, STATIC, TW><<<grid, threads, smem, stream>>>(ra); break; } return hipErrorInvalidValue;
        case 5: if constexpr (kMaxItems >= 5) { bwd_resident_kernel<NP, WMODE, 5, F32, STATIC, TW><<<grid, threads, smem, stream>>>(ra); break; } return hipErrorInvalidValue;
        default: return hipErrorInvalidValue;
    }
    return hipGetLastError();
}

template <int NP, int WMODE, bool F32, bool STATIC = false>
static hipError_t launch_items(const BwdResidentArgs &ra, hipStream_t stream) {
    // Eight streams, rows of at most 1280 channels: ten tile waves hold the row in one item each
    // instead of four in three - the Gram and mixing products of an 8 x 8 sample are most of such a
    // workgroup's life, and one wave per SIMD has nobody to overlap them with.  Backward at B=256,
    // C=1280, n=8, graphs of ten: 4 tile waves 21.3 us, 5 21.8, 8 21.4, 10 20.8 (n=4, B=320: 15.1 / 14.9 /
    // 15.9 / 15.0: four stay).
    if constexpr (NP == 8 && !F32 && !STATIC) {
        if (ra.r.C <= 1280) return launch_items_tw<NP, WMODE, F32, STATIC, 10>(ra, stream);
    }
    // Four streams: a fifth tile wave where it saves every wave an item (rows of 513..640 and 1025..1280
    // channels: ten 128-channel chunks are 3 + 3 + 2 + 2 on four waves, 2 each on five).  B=320, C=1280,
    // n=4, three runs each: backward 15.15 -> 14.90 us, step 25.53 -> 25.24.
    if constexpr (NP == 4 && !F32 && !STATIC) {
        const int chunks = (ra.r.C + 127) / 128;
        if (ra.r.C <= 1280 && (chunks + 4) / 5 < (chunks + 3) / 4) return launch_items_tw<NP, WMODE, F32, STATIC, 5>(ra, stream);
    }
    return launch_items_tw<NP, WMODE, F32, STATIC, kResTileWaves>(ra, stream);
}

hipError_t launch_bwd_resident(const void *dy, const void *x, int x_dtype, const void *w, int w_dtype, const void *f_inject,
                               const float *Hpre, const float *Hpost, const float *M, const float *q,
                               const float *P, const float *r, const float *alpha, const float *b_res,
                               const float *sk_state, BwdCoefOut out, void *dxp, void *df, float *u, int B, int n,
                               int C, int T, float eps, hipStream_t stream) {
    BwdResidentArgs ra{{dy, x, w, f_inject, Hpre, Hpost, M, q, P, r, alpha, b_res, sk_state, out, n,
                        w_dtype == kBF16, B, n, C, T, padded_D(n), eps, nullptr, 1},
                       dxp, df, u};
#define MHC_RES(NP, F32)                                                                      \
    return f_inject ? launch_items<NP, kGramInject, F32>(ra, stream)                          \
                    : (w_dtype == kBF16 ? launch_items<NP, kGramWBf16, F32>(ra, stream)       \
                                        : launch_items<NP, kGramWF32, F32>(ra, stream))
    if (x_dtype == kF32AsBF16) {
        if (n <= 4) MHC_RES(4, true);
        MHC_RES(8, true);
    }
    if (n <= 4) MHC_RES(4, false);
    MHC_RES(8, false);
#undef MHC_RES
}

// Static H: the same launch with shared coefficients; dxp is the final dx, out.red [B, D+3] receives the
// samples' raw coefficient gradients and out.s1 their s1.
hipError_t launch_bwd_resident_static(const void *dy, const void *x, const void *w, int w_dtype, const void *f_inject,
                                      const float *Hpre, const float *Hpost, const float *M, const float *q,
                                      BwdCoefOut out, void *dx, void *df, float *u, int B, int n, int C,
                                      hipStream_t stream) {
    BwdResidentArgs ra{{dy, x, w, f_inject, Hpre, Hpost, M, q, nullptr, nullptr, nullptr, nullptr, nullptr, out, 0,
                        w_dtype == kBF16, B, n, C, 0, padded_D(n), 0.f, nullptr, 1},
                       dx, df, u};
#define MHC_RES_STATIC(NP)                                                                        \
    return f_inject ? launch_items<NP, kGramInject, false, true>(ra, stream)                      \
                    : (w_dtype == kBF16 ? launch_items<NP, kGramWBf16, false, true>(ra, stream)   \
                                        : launch_items<NP, kGramWF32, false, true>(ra, stream))
    if (n <= 4) MHC_RES_STATIC(4);
    MHC_RES_STATIC(8);
#undef MHC_RES_STATIC
}

}  // namespace mhc
