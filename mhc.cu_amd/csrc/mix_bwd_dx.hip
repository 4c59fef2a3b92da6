// Backward, second launch: the input gradient, one workgroup per sample, x and dy read once.
//
//   dx[j,c] = sum_i M[i,j] dy[i,c]          (mix,        reference stream_ops.cuh:761-850)
//           + Hpre[j] da[c]                  (aggregate,  reference stream_ops.cuh:646-663)
//           - cx x[j,c]                      (projection RMS term, reference ops.py:340-349)
//           [+ sum_d dP[d] phi[d, jC+c]]     (projection, reference ops.py:336-338; only when the
//                                             caller does not run the tiled projection-backward kernel)
//   da = df w / q - a s1 / (C q^3),  df = sum_i Hpost[i] dy[i,c]      (reference rmsnorm.cuh:255-294)
// Also writes df (kernel-level view) and u[b,c] = df a / q, the per-sample summand of dw.
#include "launchers.h"
#include "mhc_common.h"

namespace mhc {

struct BwdDxArgs {
    const void *dy, *x, *w, *f_inject, *phi, *dx_in;
    const float *Hpre, *Hpost, *M, *q, *s1, *cx, *dP;
    void *dx, *df;
    float *u;            // [G, C] per-group sums of df a / q (the summands of dw)
    const float *dt;     // [B, D+3] per-sample logit gradients (dynamic) or nullptr
    float *dtpart;       // [G, D+3] per-group sums of dt
    int hstride, w_bf16, phi_bf16, B, n, C, DP, spg;  // spg = samples per workgroup
};

__device__ __forceinline__ float load_w2(const void *w, int w_bf16, int c) {
    return w_bf16 ? bf16_to_f32(static_cast<const bf16_t *>(w)[c]) : static_cast<const float *>(w)[c];
}

template <typename TG, typename TX, int NP, int V>
__global__ __launch_bounds__(256) void mix_bwd_dx_kernel(BwdDxArgs a) {
    extern __shared__ float smem[];
    float *M_s = smem;  // [NP*NP] (NP >= 16 only)
    const int grp = blockIdx.x, n = a.n, C = a.C, tid = threadIdx.x, nt = blockDim.x;
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
    const int nch = C / V;
    for (int ch = tid; ch < nch; ch += nt) {
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
        const float qinv = inject ? 0.f : 1.0f / a.q[b];
        const float k2 = inject ? 0.f : a.s1[b] * qinv * qinv * qinv / (float)C;
        const float cx = a.cx ? a.cx[b] : 0.f;
        float hpre[NP], hpost[NP];
#pragma unroll
        for (int i = 0; i < NP; i++) {
            hpre[i] = i < n ? Hpre[i] : 0.f;
            hpost[i] = i < n ? Hpost[i] : 0.f;
        }
        // streams >= n alias stream 0 (no branch around the loads, so all of them are in flight
        // together); they only ever meet zero coefficients
        float gv[NP][V], xv[NP][V];
#pragma unroll
        for (int i = 0; i < NP; i++) {
            const size_t so = (size_t)(i < n ? i : 0) * C + c;
            load_vec<TG, V>(gb + so, gv[i]);
            load_vec<TX, V>(xb + so, xv[i]);
        }
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
            if (a.df) store_vec<TX, V>(static_cast<TX *>(a.df) + (size_t)b * C + c, dfv);
        } else {
#pragma unroll
            for (int v = 0; v < V; v++) usum[v] += uv[v];
        }
#pragma unroll
        for (int j = 0; j < NP; j++) {
            if (j < n) {
                float out[V];
#pragma unroll
                for (int v = 0; v < V; v++) out[v] = hpre[j] * da[v] - cx * xv[j][v];
#pragma unroll
                for (int i = 0; i < NP; i++) {
                    float mij;
                    if constexpr (NP >= 16) mij = M_s[i * NP + j];
                    else mij = (i < n) ? M[i * n + j] : 0.f;
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
                    float prev[V];
                    load_vec<TX, V>(static_cast<const TX *>(a.dx_in) + ((size_t)b * n + j) * C + c, prev);
#pragma unroll
                    for (int v = 0; v < V; v++) out[v] += prev[v];
                }
                store_vec<TX, V>(dxb + (size_t)j * C + c, out);
            }
        }
      }
      if (!inject && a.u) store_vec<float, V>(a.u + (size_t)grp * C + c, usum);
    }
    // per-group sums of the logit gradients (feeds dbias / dalpha)
    if (a.dtpart) {
        for (int col = tid; col < D + 3; col += nt) {
            float acc = 0.f;
            for (int b = b_first; b < b_last; b++) acc += a.dt[(size_t)b * (D + 3) + col];
            a.dtpart[(size_t)grp * (D + 3) + col] = acc;
        }
    }
}

template <typename TG, typename TX, int NP, int V>
static hipError_t launch_one(const BwdDxArgs &a, hipStream_t stream) {
    const int nch = a.C / V;
    int nt = (nch + 63) / 64 * 64;
    if (nt > 256) nt = 256;
    const size_t smem = sizeof(float) * (NP >= 16 ? NP * NP : 1);
    const int groups = (a.B + a.spg - 1) / a.spg;
    mix_bwd_dx_kernel<TG, TX, NP, V><<<groups, nt, smem, stream>>>(a);
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
    if (y_dtype == kF32 && x_dtype == kF32) return launch_t<float, float>(a, stream);
    if (y_dtype == kBF16 && x_dtype == kBF16) return launch_t<bf16_t, bf16_t>(a, stream);
    if (y_dtype == kF32 && x_dtype == kBF16) return launch_t<float, bf16_t>(a, stream);
    return hipErrorInvalidValue;
}

}  // namespace mhc
