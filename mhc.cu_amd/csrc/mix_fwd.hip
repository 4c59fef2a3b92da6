// Stream-mixing forward: one workgroup per sample computes, in one launch,
//   a = sum_i Hpre_i x_i         (stream aggregate,   reference stream_ops.cuh:27-92, :453-526)
//   f = a / sqrt(mean(a^2)+eps) * w   (inner RMSNorm, reference rmsnorm.cuh:14-165)
//   y_i = sum_j M_ij x_j + Hpost_i f  (distribute+mix, reference stream_ops.cuh:119-152, :504-526)
// a and f never leave the chip; x is fetched from HBM once (the second sweep over the sample's
// tile hits L1/L2).  With an injected f the first sweep is skipped.
#include "launchers.h"
#include "mhc_common.h"

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
                if (i < n) {
                    float xv[V];
                    load_vec<TX, V>(xb + (size_t)i * C + c, xv);
#pragma unroll
                    for (int v = 0; v < V; v++) acc[v] += hpre[i] * xv[v];
                }
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
        for (int j = 0; j < NP; j++) {
            if (j < n) {
                load_vec<TX, V>(xb + (size_t)j * C + c, xv[j]);
            } else {
#pragma unroll
                for (int v = 0; v < V; v++) xv[j][v] = 0.f;
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
                    float mij;
                    if constexpr (NP >= 16) mij = M_s[i * NP + j];
                    else mij = j < n ? M[i * n + j] : 0.f;
#pragma unroll
                    for (int v = 0; v < V; v++) out[v] += mij * xv[j][v];
                }
                store_vec<TY, V>(yb + (size_t)i * C + c, out);
            }
        }
    }
}

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
                          const float *Hpost, const float *M, int hstride, float *q, int B, int n,
                          int C, float eps, hipStream_t stream) {
    MixFwdArgs a{x, w, f_inject, y, Hpre, Hpost, M, q, hstride, w_dtype == kBF16, B, n, C, eps};
    if (x_dtype == kF32 && y_dtype == kF32) return launch_t<float, float>(a, stream);
    if (x_dtype == kBF16 && y_dtype == kBF16) return launch_t<bf16_t, bf16_t>(a, stream);
    if (x_dtype == kBF16 && y_dtype == kF32) return launch_t<bf16_t, float>(a, stream);
    return hipErrorInvalidValue;
}

}  // namespace mhc
