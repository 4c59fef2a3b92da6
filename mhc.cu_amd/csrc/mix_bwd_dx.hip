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
#include "phase_profiler.h"

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

// =============================================================================================
// n > 8, bf16 activations: the same dx on the matrix cores.  Workgroup = (128-channel block,
// sample); the [32 streams x 128 channels] tiles of dy and x are fetched row-contiguously, parked
// in LDS and read back transposed (the contraction runs over streams, the strided axis) as B
// operands of v_mfma_f32_32x32x16_bf16; wave w owns channels 32w..32w+32 of the block.
//   O   = M^T dy            A = M^T as a bf16 pair (rounded value + remainder: ~16 mantissa bits)
// df = Hpost^T dy and a = Hpre^T x follow per channel on the VALU from the same LDS tiles (each half
// of the wave sums 16 streams), then da, u = df a / q; O + Hpre (x) da goes through LDS (in the
// memory of the consumed tiles) to a row-major epilogue that subtracts cx x, adds the projection
// term and leaves as 16-byte stores.  95 registers and 17 KB of LDS: five workgroups per CU, so
// the 1280 workgroups of B = 128, C = 1280 are resident in one round.
// =============================================================================================
typedef __attribute__((__vector_size__(8 * sizeof(__bf16)))) __bf16 bf16x8_t;
typedef __attribute__((__vector_size__(16 * sizeof(float)))) float f32x16_t;

constexpr int kDxlCB = 128;           // channels per workgroup
constexpr int kDxlLDT = kDxlCB + 8;   // LDS pitch of the bf16 tiles (elements)
constexpr int kDxlLDO = kDxlCB + 4;   // LDS pitch of the fp32 output tile

// 8 values -> bf16 pair of fragments: hi = rounded, lo = remainder
__device__ __forceinline__ void split_frag(const float (&v)[8], bf16x8_t &hi, bf16x8_t &lo) {
    uint32_t h[4];
    float r[8];
#pragma unroll
    for (int i = 0; i < 4; i++) {
        h[i] = pack_bf16x2(v[2 * i], v[2 * i + 1]);
        r[2 * i] = v[2 * i] - bf16lo_to_f32(h[i]);
        r[2 * i + 1] = v[2 * i + 1] - bf16hi_to_f32(h[i]);
    }
    hi = __builtin_bit_cast(bf16x8_t, make_uint4(h[0], h[1], h[2], h[3]));
    lo = __builtin_bit_cast(bf16x8_t, make_uint4(pack_bf16x2(r[0], r[1]), pack_bf16x2(r[2], r[3]),
                                                 pack_bf16x2(r[4], r[5]), pack_bf16x2(r[6], r[7])));
}

// B fragment (k = stream, column = channel) from a row-major [stream][channel] bf16 tile in LDS:
// lane (c = lane & 31, kg = lane >> 5) gets tile[k0 + kg*8 + i][col0 + c], i = 0..7
__device__ __forceinline__ bf16x8_t dxl_frag_t(const bf16_t *tile, int k0, int col0, int lane) {
    return __builtin_bit_cast(bf16x8_t, lds_frag_tr(tile, kDxlLDT, k0, col0, lane));
}

__global__ __launch_bounds__(256, 5) void mix_bwd_dx_large_kernel(BwdDxArgs a) {
    extern __shared__ __align__(16) unsigned char dxl_smem[];
    bf16_t *g_s = reinterpret_cast<bf16_t *>(dxl_smem);      // [32][LDT] dy tile
    bf16_t *x_s = g_s + 32 * kDxlLDT;                        // [32][LDT] x tile
    float *o_s = reinterpret_cast<float *>(dxl_smem);        // [32][LDO], in the two tiles once they are consumed
    float *hp_s = reinterpret_cast<float *>(x_s + 32 * kDxlLDT);  // [32] Hpre (0 beyond n)
    float *ho_s = hp_s + 32;                                 // [32] Hpost (0 beyond n)
    static_assert(sizeof(float) * 32 * kDxlLDO <= sizeof(bf16_t) * 2 * 32 * kDxlLDT, "output tile must fit in the input tiles");
    // linear workgroup id = sample * column blocks + column block (one grid dimension: no bound on B)
    const int ncb = (a.C + kDxlCB - 1) / kDxlCB;
    const int b = blockIdx.x / ncb, cblk = blockIdx.x % ncb;
    const int cb0 = cblk * kDxlCB, n = a.n, C = a.C, tid = threadIdx.x;
    const int lane = tid & 63, wave = tid >> 6, row = lane & 31, kh = lane >> 5;
    const bool inject = a.f_inject != nullptr;
    const bf16_t *gb = static_cast<const bf16_t *>(a.dy) + (size_t)b * n * C;
    const bf16_t *xb = static_cast<const bf16_t *>(a.x) + (size_t)b * n * C;
    const float *Hpre = a.Hpre + (size_t)b * a.hstride;
    const float *Hpost = a.Hpost + (size_t)b * a.hstride;
    const float *M = a.M + (size_t)b * a.hstride * n;

    // ---- tile loads: thread owns row tid / 8, 16-byte chunks tid % 8 and tid % 8 + 8 ------------
    const int trow = tid >> 3;
    RawVec<bf16_t, 8> gr[2], xr[2], pr[2];
    bool cok[2];
#pragma unroll
    for (int h = 0; h < 2; h++) {
        const int c = cb0 + ((tid & 7) + 8 * h) * 8;
        cok[h] = c < C;  // C % 8 == 0: a chunk is entirely inside or outside
        // rows >= n alias row 0 (they meet zero coefficients), chunks >= C alias chunk 0 (not stored)
        const size_t off = (size_t)(trow < n ? trow : 0) * C + (cok[h] ? c : 0);
        gr[h].load(gb + off);
        xr[h].load(xb + off);
        if (a.dx_in) pr[h].load(static_cast<const bf16_t *>(a.dx_in) + (size_t)b * n * C + off);
    }
    // ---- A operands from the coefficients (overlaps the tile loads) -----------------------------
    // lane (row j, kg): M^T[j][k] = M[k][j], k = ks*16 + kg*8 + i
    bf16x8_t mth[2], mtl[2];
#pragma unroll
    for (int ks = 0; ks < 2; ks++) {
        float mv[8];
#pragma unroll
        for (int i = 0; i < 8; i++) {
            const int k = ks * 16 + kh * 8 + i;
            const bool ok = k < n && row < n;
            const float m = M[ok ? k * n + row : 0];
            mv[i] = ok ? m : 0.f;
        }
        split_frag(mv, mth[ks], mtl[ks]);
    }
    if (tid < 32) hp_s[tid] = tid < n ? Hpre[tid] : 0.f;
    else if (tid < 64) ho_s[tid - 32] = tid - 32 < n ? Hpost[tid - 32] : 0.f;
    const float qinv = inject ? 0.f : 1.0f / a.q[b];
    const float k2 = inject ? 0.f : a.s1[b] * qinv * qinv * qinv / (float)C;
    const float cx = a.cx ? a.cx[b] : 0.f;
    const int cw = cb0 + wave * 32 + row;  // this lane's channel in the matrix-core phase
    const float wv = (!inject && cw < C) ? load_w2(a.w, a.w_bf16, cw) : 0.f;

#pragma unroll
    for (int h = 0; h < 2; h++) {
        const int co = ((tid & 7) + 8 * h) * 8;
        *reinterpret_cast<uint4 *>(g_s + trow * kDxlLDT + co) = make_uint4(gr[h].w[0], gr[h].w[1], gr[h].w[2], gr[h].w[3]);
        *reinterpret_cast<uint4 *>(x_s + trow * kDxlLDT + co) = make_uint4(xr[h].w[0], xr[h].w[1], xr[h].w[2], xr[h].w[3]);
    }
    __syncthreads();

    // ---- matrix cores: O = M^T dy ------------------------------------------------------------------
    f32x16_t o;
#pragma unroll
    for (int i = 0; i < 16; i++) o[i] = 0.f;
#pragma unroll
    for (int ks = 0; ks < 2; ks++) {
        const bf16x8_t gf = dxl_frag_t(g_s, ks * 16, wave * 32, lane);
        o = __builtin_amdgcn_mfma_f32_32x32x16_bf16(mth[ks], gf, o, 0, 0, 0);
        o = __builtin_amdgcn_mfma_f32_32x32x16_bf16(mtl[ks], gf, o, 0, 0, 0);
    }
    // df = Hpost^T dy and a = Hpre^T x of this lane's channel on the VALU, straight from the tiles
    // (fp32 coefficients; each half of the wave sums 16 streams): as matrix-core products they
    // cost 32 more operand registers, and this kernel needs five workgroups per CU to have its
    // whole grid resident at once
    float dfp = 0.f, ap = 0.f;
    {
        const bf16_t *gp = g_s + (size_t)(kh * 16) * kDxlLDT + wave * 32 + row;
        const bf16_t *xp = x_s + (size_t)(kh * 16) * kDxlLDT + wave * 32 + row;
#pragma unroll
        for (int i = 0; i < 16; i++) {
            dfp += ho_s[kh * 16 + i] * bf16_to_f32(gp[i * kDxlLDT]);
            if (!inject) ap += hp_s[kh * 16 + i] * bf16_to_f32(xp[i * kDxlLDT]);
        }
    }
    const float dfc = xor32_add(dfp);
    const float ac = xor32_add(ap);
    __syncthreads();  // the tiles are consumed: their memory becomes the output tile
    const float da = inject ? 0.f : dfc * wv * qinv - ac * k2;
    if (kh == 0 && cw < C) {
        if (inject) {
            if (a.df) static_cast<bf16_t *>(a.df)[(size_t)b * C + cw] = f32_to_bf16(dfc);
        } else if (a.u) {
            a.u[(size_t)b * C + cw] = dfc * ac * qinv;
        }
    }
#pragma unroll
    for (int i = 0; i < 16; i++) {
        const int j = 8 * (i >> 2) + 4 * kh + (i & 3);
        o_s[j * kDxlLDO + wave * 32 + row] = o[i] + hp_s[j] * da;
    }
    __syncthreads();

    // ---- row-major epilogue ---------------------------------------------------------------------------
    if (trow < n) {
#pragma unroll
        for (int h = 0; h < 2; h++) {
            if (cok[h]) {
                const int co = ((tid & 7) + 8 * h) * 8;
                float xv[8], out[8], pv[8];
                xr[h].get(xv);
                const float4 o0 = *reinterpret_cast<const float4 *>(o_s + trow * kDxlLDO + co);
                const float4 o1 = *reinterpret_cast<const float4 *>(o_s + trow * kDxlLDO + co + 4);
                out[0] = o0.x; out[1] = o0.y; out[2] = o0.z; out[3] = o0.w;
                out[4] = o1.x; out[5] = o1.y; out[6] = o1.z; out[7] = o1.w;
#pragma unroll
                for (int v = 0; v < 8; v++) out[v] -= cx * xv[v];
                if (a.dx_in) {
                    pr[h].get(pv);
#pragma unroll
                    for (int v = 0; v < 8; v++) out[v] += pv[v];
                }
                store_vec<bf16_t, 8, true>(static_cast<bf16_t *>(a.dx) + (size_t)b * n * C + (size_t)trow * C + cb0 + co, out);
            }
        }
    }
    // per-sample "group" sums of the logit gradients (one sample per group on this path)
    if (a.dtpart && cblk == 0) {
        const int D = n * n + 2 * n;
        for (int col = tid; col < D + 3; col += 256)
            a.dtpart[(size_t)b * (D + 3) + col] = a.dt[(size_t)b * (D + 3) + col];
    }
}

static hipError_t launch_large_mfma(const BwdDxArgs &a, hipStream_t stream) {
    const size_t smem = sizeof(bf16_t) * 2 * 32 * kDxlLDT + sizeof(float) * 64;
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
