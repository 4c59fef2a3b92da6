// Backward, second launch: the input gradient, one workgroup per sample, x and dy read once.
//
//   dx[j,c] = sum_i M[i,j] dy[i,c]          (mix,        reference stream_ops.cuh:761-850)
//           + Hpre[j] da[c]                  (aggregate,  reference stream_ops.cuh:646-663)
//           - cx x[j,c]                      (projection RMS term, reference ops.py:340-349)
//           [+ sum_d dP[d] phi[d, jC+c]]     (projection, reference ops.py:336-338; only when the
//                                             caller does not run the tiled projection-backward kernel)
//   da = df w / q - a s1 / (C q^3),  df = sum_i Hpost[i] dy[i,c]      (reference rmsnorm.cuh:255-294)
// Also writes df (kernel-level view) and u[b,c] = df a / q, the per-sample summand of dw.
#include "dx_large.h"
#include "launchers.h"
#include "mhc_common.h"
#include "phase_profiler.h"

namespace mhc {

template <typename TG, typename TX, int NP, int V>
__global__ __launch_bounds__(256) void mix_bwd_dx_kernel(BwdDxArgs a) {
    extern __shared__ float smem[];
    float *M_s = smem;  // [NP*NP] (NP >= 16 only)
    const int grp = blockIdx.x, n = a.n, C = a.C, tid = threadIdx.x, nt = blockDim.x;
    const int pwg = blockIdx.y * gridDim.x + blockIdx.x;
    (void)pwg;
    MHC_PHASE_ZERO(kPhaseDxSmall, pwg);
    MHC_PHASE_BEGIN(pclk);
    const int b_first = grp * a.spg, b_last = min(a.B, b_first + a.spg);
    const bool inject = a.f_inject != nullptr;
    const int D = n * n + 2 * n, nC = n * C;
    if constexpr (NP >= 16) {
        // one sample per workgroup on this path (spg == 1): stage its M once, for all threads
        const float *M0 = a.M + (size_t)b_first * a.hstride * n;
        for (int e = tid; e < NP * NP; e += nt) {
            const int i = e / NP, j = e % NP;
            M_s[e] = (i < n && j < n) ? M0[i * n + j] : 0.f;
        }
        __syncthreads();
    }
    // grid.y workgroups share the channels of a sample group
    const int nch = C / V;
    // The loop runs for whole workgroups (all lanes take part in staging M); a lane without a chunk of
    // its own works on chunk 0 and stores nothing.
    for (int ch0 = blockIdx.y * nt; ch0 < nch; ch0 += nt * gridDim.y) {
      const bool live = ch0 + tid < nch;
      const int ch = live ? ch0 + tid : 0;
      const int c = ch * V;
      float usum[V];
#pragma unroll
      for (int v = 0; v < V; v++) usum[v] = 0.f;
      for (int b = b_first; b < b_last; b++) {
        const TG *__restrict__ gb = static_cast<const TG *>(a.dy) + (size_t)b * n * C;
        const TX *__restrict__ xb = static_cast<const TX *>(a.x) + (size_t)b * n * C;
        TX *__restrict__ dxb = static_cast<TX *>(a.dx) + (size_t)b * n * C;
        const float *__restrict__ Hpre = a.Hpre + (size_t)b * a.hstride;
        const float *__restrict__ Hpost = a.Hpost + (size_t)b * a.hstride;
        const float *__restrict__ M = a.M + (size_t)b * a.hstride * n;
        // The bulk loads come first and nothing is computed from the sample's coefficients until they
        // are all requested (a division on q here would make the wave wait for the coefficient round
        // trip before it asks for its data).  Streams >= n alias stream 0 (no branch around the loads,
        // so all of them are in flight together); they only ever meet zero coefficients.
        RawVec<TG, V> graw[NP];
        RawVec<TX, V> xraw[NP];
#pragma unroll
        for (int i = 0; i < NP; i++) {
            const size_t so = (size_t)(i < n ? i : 0) * C + c;
            graw[i].load(gb + so);
            xraw[i].load(xb + so);
        }
        // dx_in may alias dx, so the compiler cannot move its loads above the stores of earlier
        // rows: request all rows here (every thread reads exactly the elements it later writes)
        RawVec<TX, V> prev[NP];
        if (a.dx_in) {
#pragma unroll
            for (int j = 0; j < NP; j++)
                prev[j].load(static_cast<const TX *>(a.dx_in) + ((size_t)b * n + (j < n ? j : 0)) * C + c);
        }
        // the sample's coefficients.  n <= 8 (one wave per workgroup): M goes through LDS, one load per
        // lane instead of one uniform load per use inside the mixing loops; the wave's own LDS
        // accesses complete in order, so no barrier is involved
        float hpre[NP], hpost[NP];
#pragma unroll
        for (int i = 0; i < NP; i++) {
            hpre[i] = Hpre[i < n ? i : 0];
            hpost[i] = Hpost[i < n ? i : 0];
        }
        if constexpr (NP < 16) {
            const int mi = tid / NP, mj = tid % NP;
            const bool mok = mi < n && mj < n;
            const float mval = M[mok ? mi * n + mj : 0];
            if (tid < NP * NP) M_s[tid] = mok ? mval : 0.f;
        }
        const float qraw = inject ? 1.0f : a.q[b], s1raw = inject ? 0.f : a.s1[b];
        const float cx = a.cx ? a.cx[b] : 0.f;
#pragma unroll
        for (int i = 0; i < NP; i++)
            if (i >= n) { hpre[i] = 0.f; hpost[i] = 0.f; }
        const float qinv = inject ? 0.f : 1.0f / qraw;
        const float k2 = inject ? 0.f : s1raw * qinv * qinv * qinv / (float)C;
        float gv[NP][V], xv[NP][V];
#pragma unroll
        for (int i = 0; i < NP; i++) { graw[i].get(gv[i]); xraw[i].get(xv[i]); }
        MHC_PHASE_ADD(kPhaseDxSmall, pwg, 0, pclk);
        float da[V], dfv[V], uv[V];
#pragma unroll
        for (int v = 0; v < V; v++) {
            float s_a = 0.f, s_df = 0.f;
#pragma unroll
            for (int i = 0; i < NP; i++) { s_a += hpre[i] * xv[i][v]; s_df += hpost[i] * gv[i][v]; }
            dfv[v] = s_df;
            if (inject) {
                da[v] = 0.f; uv[v] = 0.f;
            } else {
                da[v] = s_df * load_w2(a.w, a.w_bf16, c + v) * qinv - s_a * k2;
                uv[v] = s_df * s_a * qinv;
            }
        }
        if (inject) {
            if (a.df && live) store_vec<TX, V>(static_cast<TX *>(a.df) + (size_t)b * C + c, dfv);
        } else {
#pragma unroll
            for (int v = 0; v < V; v++) usum[v] += uv[v];
        }
        MHC_PHASE_ADD(kPhaseDxSmall, pwg, 1, pclk);
#pragma unroll
        for (int j = 0; j < NP; j++) {
            if (j < n) {
                float out[V];
#pragma unroll
                for (int v = 0; v < V; v++) out[v] = hpre[j] * da[v] - cx * xv[j][v];
#pragma unroll
                for (int i = 0; i < NP; i++) {
                    const float mij = M_s[i * NP + j];
#pragma unroll
                    for (int v = 0; v < V; v++) out[v] += mij * gv[i][v];
                }
                if (a.phi) {
                    const float *dPb = a.dP + (size_t)b * a.DP;
                    for (int d = 0; d < D; d++) {
                        const float dp = dPb[d];
                        float pv[V];
                        if (a.phi_bf16)
                            load_vec<bf16_t, V>(static_cast<const bf16_t *>(a.phi) + (size_t)d * nC + j * C + c, pv);
                        else
                            load_vec<float, V>(static_cast<const float *>(a.phi) + (size_t)d * nC + j * C + c, pv);
#pragma unroll
                        for (int v = 0; v < V; v++) out[v] += dp * pv[v];
                    }
                }
                if (a.dx_in) {
                    float pv[V];
                    prev[j].get(pv);
#pragma unroll
                    for (int v = 0; v < V; v++) out[v] += pv[v];
                }
                if (live) store_vec<TX, V, true>(dxb + (size_t)j * C + c, out);
            }
        }
      }
      MHC_PHASE_ADD(kPhaseDxSmall, pwg, 2, pclk);
      if (!inject && a.u && live) store_vec<float, V>(a.u + (size_t)grp * C + c, usum);
    }
    // per-group sums of the logit gradients (feeds dbias / dalpha)
    if (a.dtpart && blockIdx.y == 0) {
        for (int col = tid; col < D + 3; col += nt) {
            double acc = 0.0;  // float64 like the batch sums that follow (finalize_kernel)
            for (int b = b_first; b < b_last; b++) acc += (double)a.dt[(size_t)b * (D + 3) + col];
            a.dtpart[(size_t)grp * (D + 3) + col] = (float)acc;
        }
    }
    MHC_PHASE_ADD(kPhaseDxSmall, pwg, 3, pclk);
}

__global__ __launch_bounds__(256, 5) void mix_bwd_dx_large_kernel(BwdDxArgs a) {
    extern __shared__ __align__(16) unsigned char dxl_smem[];
    dx_large_block(a, blockIdx.x, dxl_smem);
}

static hipError_t launch_large_mfma(const BwdDxArgs &a, hipStream_t stream) {
    const size_t smem = dx_large_lds_bytes();
    mix_bwd_dx_large_kernel<<<(unsigned)((a.C + kDxlCB - 1) / kDxlCB) * (unsigned)a.B, 256, smem, stream>>>(a);
    return hipGetLastError();
}

static int groups_of(const BwdDxArgs &a) { return (a.B + a.spg - 1) / a.spg; }

template <typename TG, typename TX, int NP, int V>
static hipError_t launch_one(const BwdDxArgs &a, hipStream_t stream) {
    const int nch = a.C / V;
    int nt = (nch + 63) / 64 * 64;
    if (nt > 256) nt = 256;
    int ny = 1;
    if (NP <= 8) {
        // one wave per workgroup and one channel chunk per thread: every lane is busy and the grid
        // has enough workgroups to keep loads of many samples in flight on each CU
        nt = 64;
        ny = (nch + 63) / 64;
    }
    const size_t smem = sizeof(float) * NP * NP;
    mix_bwd_dx_kernel<TG, TX, NP, V><<<dim3(groups_of(a), ny), nt, smem, stream>>>(a);
    return hipGetLastError();
}

template <typename TG, typename TX, int NP>
static hipError_t launch_np(const BwdDxArgs &a, hipStream_t stream) {
    constexpr int bytes = NP == 4 ? 16 : (NP == 8 ? 8 : 4);
    constexpr int szmax = sizeof(TG) > sizeof(TX) ? sizeof(TG) : sizeof(TX);
    constexpr int V = bytes / szmax > 0 ? bytes / szmax : 1;
    if (a.C % V == 0) return launch_one<TG, TX, NP, V>(a, stream);
    return launch_one<TG, TX, NP, 1>(a, stream);
}

template <typename TG, typename TX>
static hipError_t launch_t(const BwdDxArgs &a, hipStream_t stream) {
    if (a.n <= 4) return launch_np<TG, TX, 4>(a, stream);
    if (a.n <= 8) return launch_np<TG, TX, 8>(a, stream);
    if (a.n <= 16) return launch_np<TG, TX, 16>(a, stream);
    return launch_np<TG, TX, 32>(a, stream);
}

int bwd_dx_samples_per_group(int B, int n) {
    if (n > 8) return 1;
    int spg = B / 2048;
    if (spg < 1) spg = 1;
    if (spg > 16) spg = 16;
    return spg;
}

hipError_t launch_mix_bwd_dx(const void *dy, int y_dtype, const void *x, int x_dtype, const void *w,
                             int w_dtype, const void *f_inject, const float *Hpre,
                             const float *Hpost, const float *M, int hstride, const float *q,
                             const float *s1, const float *cx, const float *dP, int DP,
                             const void *phi, int phi_dtype, const void *dx_in, void *dx, void *df,
                             float *u, const float *dt, float *dtpart, int spg, int B, int n, int C,
                             hipStream_t stream) {
    if (n > 8) spg = 1;  // the large-n layout stages one sample's M in LDS per workgroup
    BwdDxArgs a{dy, x, w, f_inject, phi, dx_in, Hpre, Hpost, M, q, s1, cx, dP, dx, df, u, dt, dtpart,
                hstride, w_dtype == kBF16, phi_dtype == kBF16, B, n, C, DP, spg};
    if (n > 8 && y_dtype == kBF16 && x_dtype == kBF16 && C % 8 == 0 && phi == nullptr)
        return launch_large_mfma(a, stream);
    if (y_dtype == kF32 && x_dtype == kF32) return launch_t<float, float>(a, stream);
    if (y_dtype == kBF16 && x_dtype == kBF16) return launch_t<bf16_t, bf16_t>(a, stream);
    if (y_dtype == kF32 && x_dtype == kBF16) return launch_t<float, bf16_t>(a, stream);
    return hipErrorInvalidValue;
}

}  // namespace mhc
