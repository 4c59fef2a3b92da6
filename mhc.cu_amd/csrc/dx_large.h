// Arguments of the dx kernels of the backward, and the body of the n > 8 matrix-core dx kernel as a
// device function, so that its workgroups can also run inside another launch.
#pragma once
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
    // n > 8 matrix-core kernel only: s1 as the per-part sums that the Gram launch leaves
    // ([B][s1parts]) instead of the coefficient launch's s1 [B], so that its workgroups can run beside
    // that launch
    const float *s1part = nullptr;
    int s1parts = 0;
    float *dx_f32 = nullptr;  // when set, the result goes here as fp32 [B][n][C] instead of to dx
};

__device__ __forceinline__ float load_w2(const void *w, int w_bf16, int c) {
    return w_bf16 ? bf16_to_f32(static_cast<const bf16_t *>(w)[c]) : static_cast<const float *>(w)[c];
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

constexpr size_t dx_large_lds_bytes() { return sizeof(bf16_t) * 2 * 32 * kDxlLDT + sizeof(float) * 64; }

// One workgroup (256 threads) of the kernel: `blk` = sample * column blocks + column block;
// dxl_smem = dx_large_lds_bytes() of LDS, 16-byte aligned.
__device__ __forceinline__ void dx_large_block(const BwdDxArgs &a, unsigned blk, unsigned char *dxl_smem) {
    bf16_t *g_s = reinterpret_cast<bf16_t *>(dxl_smem);      // [32][LDT] dy tile
    bf16_t *x_s = g_s + 32 * kDxlLDT;                        // [32][LDT] x tile
    float *o_s = reinterpret_cast<float *>(dxl_smem);        // [32][LDO], in the two tiles once they are consumed
    float *hp_s = reinterpret_cast<float *>(x_s + 32 * kDxlLDT);  // [32] Hpre (0 beyond n)
    float *ho_s = hp_s + 32;                                 // [32] Hpost (0 beyond n)
    static_assert(sizeof(float) * 32 * kDxlLDO <= sizeof(bf16_t) * 2 * 32 * kDxlLDT, "output tile must fit in the input tiles");
    // linear workgroup id = sample * column blocks + column block (one grid dimension: no bound on B)
    const int ncb = (a.C + kDxlCB - 1) / kDxlCB;
    const int b = (int)(blk / ncb), cblk = (int)(blk % ncb);
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
    float s1 = 0.f;
    if (!inject) {
        if (a.s1part) {
            for (int p = 0; p < a.s1parts; p++) s1 += a.s1part[(size_t)b * a.s1parts + p];
        } else {
            s1 = a.s1[b];
        }
    }
    const float k2 = s1 * qinv * qinv * qinv / (float)C;
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
                const size_t off = (size_t)b * n * C + (size_t)trow * C + cb0 + co;
                if (a.dx_f32) store_vec<float, 8>(a.dx_f32 + off, out);  // read again soon: no streaming hint
                else store_vec<bf16_t, 8, true>(static_cast<bf16_t *>(a.dx) + off, out);
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

}  // namespace mhc
