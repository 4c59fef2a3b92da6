// Backward, second launch for n <= 4 in the bf16 tier: everything that needs dP, in ONE pass over
// dy and x.  A workgroup owns a slab of 64 channels (all n streams) and walks the samples of its
// batch split in tiles of 32:
//
//   dx[b,j,c]  = sum_i M_b[i,j] dy[b,i,c] + Hpre_b[j] da[b,c] - cx_b x[b,j,c] + sum_d dP[b,d] phi[d, jC+c]
//   df[b,c]    (kernel-level view)                                   reference stream_ops.cuh:761-850,
//   dphi[d,k] += sum_b dP[b,d] x_flat[b,k]                           :646-663, ops.py:332-351
//   dw[c]     += sum_b df[b,c] a[b,c] / q_b                          reference rmsnorm.cuh:282-294
//   dbias / dalpha partial sums of dt over the split's samples       reference ops.py:319-325
//
// The two projection products run on the matrix cores (v_mfma_f32_32x32x16_bf16): their
// contraction index (b for dphi, d for the dx term) is not the contiguous one in memory, so the
// x tile and the phi slab are staged row-major in LDS and read back transposed; dP arrives from
// the reduce kernel as bf16 [B, DP] and as a transposed hi/lo pair [2][DP][BP].  The projection
// term of dx goes from the accumulators through LDS to the thread that owns (sample, 8 channels)
// of all streams, which finishes dx on the VALU and stores 16 bytes per stream.
// Per tile: two barriers, x and dy read once from HBM, dx written once; no atomics.
#include "launchers.h"

#include <type_traits>
#include "mhc_common.h"
#include "phase_profiler.h"
#include "tuning.h"

namespace mhc {

typedef __attribute__((__vector_size__(8 * sizeof(__bf16)))) __bf16 bf16x8_t;
typedef __attribute__((__vector_size__(16 * sizeof(float)))) float f32x16_t;

constexpr int kSlabCW = 64;                 // channels per slab
constexpr int kSlabNS = 4;                  // streams (padded)
constexpr int kSlabKW = kSlabNS * kSlabCW;  // x_flat columns per slab tile row
constexpr int kSlabLDX = kSlabKW + 8;       // LDS pitch of the bf16 tiles (elements)
constexpr int kSlabLDF = kSlabKW + 4;       // LDS pitch of the fp32 projection-term tile

struct BwdSlabArgs {
    const void *dy;          // TG [B, n, C]
    const bf16_t *x;         // [B, n, C]
    const void *w;           // [C]
    const void *f_inject;    // bf16 [B, C] or nullptr
    const bf16_t *phi;       // [D, nC]
    const float *Hpre, *Hpost, *M, *q, *s1, *cx;  // per sample
    const bf16_t *dPb;       // dP, fragment-major (frag_dpb, DP = 32)
    const bf16_t *dPT;       // dP^T hi/lo planes, fragment-major (frag_dpt), plane stride 32 * BP
    const float *dt;         // [B, D+3]
    bf16_t *dx;              // [B, n, C]
    bf16_t *df;              // [B, C] or nullptr
    float *dphi_part;        // [S][D][nC]
    float *dw_part;          // [S][C]
    float *dt_part;          // [S][D+3]
    int w_bf16, B, BP, n, C, tiles;  // tiles = 32-sample tiles of the batch; split y takes tiles [y T / S, (y + 1) T / S)
};

__device__ __forceinline__ bf16x8_t slab_frag_t(const bf16_t *tile, int k0, int col0, int lane) {
    // lane (n = lane & 31, kg = lane >> 5) gets tile[k0 + kg*8 + i][col0 + n], i = 0..7
    return __builtin_bit_cast(bf16x8_t, lds_frag_tr(tile, kSlabLDX, k0, col0, lane));
}

__device__ __forceinline__ void unpack8(const uint4 &r, float (&v)[8]) {
    v[0] = bf16lo_to_f32(r.x); v[1] = bf16hi_to_f32(r.x);
    v[2] = bf16lo_to_f32(r.y); v[3] = bf16hi_to_f32(r.y);
    v[4] = bf16lo_to_f32(r.z); v[5] = bf16hi_to_f32(r.z);
    v[6] = bf16lo_to_f32(r.w); v[7] = bf16hi_to_f32(r.w);
}

// Eight consecutive values of dy kept as loaded (16 bytes for bf16, 32 for fp32) until they are used.
template <typename T> struct Raw8;
template <> struct Raw8<bf16_t> {
    uint4 r;
    __device__ __forceinline__ void load(const bf16_t *p) { r = *reinterpret_cast<const uint4 *>(p); }
    __device__ __forceinline__ void get(float (&v)[8]) const { unpack8(r, v); }
};
template <> struct Raw8<float> {
    float4 r0, r1;
    __device__ __forceinline__ void load(const float *p) {
        r0 = reinterpret_cast<const float4 *>(p)[0];
        r1 = reinterpret_cast<const float4 *>(p)[1];
    }
    __device__ __forceinline__ void get(float (&v)[8]) const {
        v[0] = r0.x; v[1] = r0.y; v[2] = r0.z; v[3] = r0.w; v[4] = r1.x; v[5] = r1.y; v[6] = r1.z; v[7] = r1.w;
    }
};

template <typename TG>
__global__ __launch_bounds__(256, 2) void bwd_slab_kernel(BwdSlabArgs a) {
    // bf16 dy: the per-sample 4x4 mixing of phase C runs on v_mfma_f32_4x4x4_16b_bf16 (below)
    constexpr bool kMixMfma = std::is_same<TG, bf16_t>::value;
    extern __shared__ float smem_f[];
    float *dxf_s = smem_f;                                                  // [32][LDF] fp32
    bf16_t *x_s = reinterpret_cast<bf16_t *>(dxf_s + 32 * kSlabLDF);         // [32][LDX] bf16
    const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
    const int n = a.n, C = a.C, nC = n * C, D = n * n + 2 * n;
    const int pwg = blockIdx.y * gridDim.x + blockIdx.x;
    (void)pwg;
    MHC_PHASE_ZERO(kPhaseBwdSlab, pwg);
    MHC_PHASE_BEGIN(pclk);
    const int c0 = blockIdx.x * kSlabCW;
    // whole tiles per split, the counts of two splits differing by at most one: any split count up to the
    // tile count can be used, so the grid can be sized to the chip instead of to a divisor of the batch
    const unsigned nsplit = gridDim.y;
    // (tiles <= 2^26 and at most 512 splits: the products fit 32 bits)
    const int b_begin = (int)(blockIdx.y * (unsigned)a.tiles / nsplit) * 32;
    const int b_end = min(a.B, (int)((blockIdx.y + 1) * (unsigned)a.tiles / nsplit) * 32);
    const bool inject = a.f_inject != nullptr;
    const int row = lane & 31, kg = lane >> 5;
    // VALU ownership: sample bl of the tile, channels c0 + ch*8 .. +8 of every stream
    const int bl = tid >> 3, ch = tid & 7;
    const int cth = c0 + ch * 8;
    const bool cok = cth < C;  // C % 8 == 0: a chunk is entirely inside or outside

    // ---- software pipeline: the loads of tile t+1 are issued before the VALU phase of tile t ----
    // raw tile data of this thread (sample slot bl, 8 channels, all streams) and the MFMA operands
    // that come straight from global memory (dP^T hi/lo rows d, dP rows b)
    struct TileRegs {
        uint4 xr[kSlabNS];
        Raw8<TG> gr[kSlabNS];
    };
    // Loads carry no predicate (a predicate would be applied right behind the load and make the
    // prefetch wait): slots beyond the batch, streams >= n and channel chunks >= C alias valid
    // data instead.  Aliased values are finite whenever the real inputs are and only ever meet
    // zero coefficients (dP^T is zero beyond B, H and M are zero beyond n) or land in rows and
    // columns that are never stored.
    auto load_tile = [&](int sb, TileRegs &t) {
        const int b = sb + bl;
        const bool bok = b < b_end && cok;
        const size_t base = bok ? (size_t)b * nC + cth : 0;
        const bf16_t *xb = a.x + base;
        const TG *gb = static_cast<const TG *>(a.dy) + base;
#pragma unroll
        for (int j = 0; j < kSlabNS; j++) {
            const size_t so = j < n ? (size_t)j * C : 0;
            t.xr[j] = *reinterpret_cast<const uint4 *>(xb + so);
            t.gr[j].load(gb + so);
        }
    };
    // ---- phi slab -> LDS (as [32 d][KW]) -> this wave's transposed fragments ----------------
    // wave w owns N-tiles t = 2w, 2w+1; tile t covers stream t/2, channels c0 + (t%2)*32 .. +32
    // The slab is requested first and the first tile right behind it, so that the tile's round
    // trip runs under the staging of the slab.
    bf16_t *phi_s = reinterpret_cast<bf16_t *>(dxf_s);  // staged in the (not yet used) fp32 tile
    constexpr int kPhiIters = 32 * (kSlabKW / 8) / 256;
    static_assert(32 * (kSlabKW / 8) % 256 == 0, "phi slab staging assumes whole rounds of 256 threads");
    uint4 phir[kPhiIters];
#pragma unroll
    for (int i = 0; i < kPhiIters; i++) {
        const int e = tid + i * 256;
        const int d = e / (kSlabKW / 8), chunk = e % (kSlabKW / 8);
        const int j = chunk / (kSlabCW / 8), c = c0 + (chunk % (kSlabCW / 8)) * 8;
        const bool ok = d < D && j < n && c < C;
        phir[i] = load16_masked(
            reinterpret_cast<const uint4 *>(a.phi + (ok ? (size_t)d * nC + (size_t)j * C + c : 0)), ok);
    }
    TileRegs cur, nxt;
    if (b_begin < b_end) load_tile(b_begin, cur);
#pragma unroll
    for (int i = 0; i < kPhiIters; i++) {
        const int e = tid + i * 256;
        const int d = e / (kSlabKW / 8), chunk = e % (kSlabKW / 8);
        *reinterpret_cast<uint4 *>(phi_s + (size_t)d * kSlabLDX + chunk * 8) = phir[i];
    }
    __syncthreads();
    bf16x8_t phif[2][2];
#pragma unroll
    for (int t = 0; t < 2; t++)
#pragma unroll
        for (int ks = 0; ks < 2; ks++) phif[t][ks] = slab_frag_t(phi_s, ks * 16, (2 * wave + t) * 32, lane);
    __syncthreads();  // fragments are in registers; the region becomes dxf_s

    f32x16_t acc[2];
#pragma unroll
    for (int t = 0; t < 2; t++)
#pragma unroll
        for (int i = 0; i < 16; i++) acc[t][i] = 0.f;
    float usum[8];
#pragma unroll
    for (int v = 0; v < 8; v++) usum[v] = 0.f;
    float dtsum = 0.f;  // slab 0 only: thread (col = tid & 31, row group = tid >> 5)

    float wv[8];
#pragma unroll
    for (int v = 0; v < 8; v++)
        wv[v] = (cok && !inject) ? (a.w_bf16 ? bf16_to_f32(static_cast<const bf16_t *>(a.w)[cth + v])
                                              : static_cast<const float *>(a.w)[cth + v]) : 0.f;


    MHC_PHASE_ADD(kPhaseBwdSlab, pwg, 0, pclk);
    // One tile: `cur` holds its data (requested a whole tile earlier); the next tile's loads go to
    // `nxt` right behind this tile's small operand loads and have the three phases to arrive.  The
    // loop alternates the two register sets instead of copying one into the other (a copy waits for
    // the loads it copies).
    auto process_tile = [&](int sb, TileRegs &cur, TileRegs &nxt) {
        const int b = sb + bl;
        const bool bok = b < b_end && cok;
        // MFMA operands that come straight from global memory: dP^T hi/lo (rows d) and dP (rows b);
        // issued first, they arrive while the x tile is written and the barrier is crossed
        uint4 ah[2], al[2], ap2[2];
#pragma unroll
        for (int ks = 0; ks < 2; ks++) {
            const bf16_t *ap = a.dPT + frag_base(0, a.BP >> 4, (sb >> 4) + ks) + lane * 8;
            // splits are whole 32-sample tiles and BP is padded to 32 (dP^T zero beyond B), so every
            // fragment of the tile is inside the buffers; dP rows beyond B only feed unused rows
            ah[ks] = *reinterpret_cast<const uint4 *>(ap);
            al[ks] = *reinterpret_cast<const uint4 *>(ap + (size_t)32 * a.BP);
            ap2[ks] = *reinterpret_cast<const uint4 *>(a.dPb + frag_base(sb >> 5, 2, ks) + lane * 8);
        }
        // this thread's sample coefficients for phase C: asked for here so that they arrive behind
        // the barriers and the matrix-core phase (slots beyond the split alias sample 0, streams
        // >= n alias stream 0; both are discarded below)
        // (matrix-core mixing: a lane only needs column lane & 3 of M)
        constexpr int MC = kMixMfma ? 1 : kSlabNS;
        const int jq = tid & 3;
        float hpre[kSlabNS], hpost[kSlabNS], Mr[kSlabNS][MC], cxv, qv = 1.f, s1v = 0.f;
        {
            // by sample only, whatever the lane's channel chunk: in the matrix-core mixing the four
            // lanes of a block supply each other's coefficient rows
            const size_t bc = b < b_end ? b : 0;
#pragma unroll
            for (int i = 0; i < kSlabNS; i++) {
                hpre[i] = a.Hpre[bc * n + (i < n ? i : 0)];
                hpost[i] = a.Hpost[bc * n + (i < n ? i : 0)];
#pragma unroll
                for (int j = 0; j < MC; j++) {
                    const int jj = kMixMfma ? jq : j;
                    Mr[i][j] = a.M[bc * n * n + ((i < n && jj < n) ? i * n + jj : 0)];
                }
            }
            cxv = a.cx[bc];
            if (!inject) { qv = a.q[bc]; s1v = a.s1[bc]; }
        }
        if (sb + 32 < b_end) load_tile(sb + 32, nxt);
        // x tile -> LDS
#pragma unroll
        for (int j = 0; j < kSlabNS; j++)
            *reinterpret_cast<uint4 *>(x_s + (size_t)bl * kSlabLDX + j * kSlabCW + ch * 8) = cur.xr[j];
        // dt column sums (slab 0): 32 columns x 8 row groups, 4 samples of the tile each
        if (blockIdx.x == 0) {
            const int col = tid & 31, rg = tid >> 5;
            if (col < D + 3) {
#pragma unroll
                for (int rr = 0; rr < 4; rr++) {
                    const int bb = sb + rg * 4 + rr;
                    if (bb < b_end) dtsum += a.dt[(size_t)bb * (D + 3) + col];
                }
            }
        }
        __syncthreads();
        MHC_PHASE_ADD(kPhaseBwdSlab, pwg, 1, pclk);

        // ---- phase B: matrix cores ----------------------------------------------------------------
        {
            // dphi += dP^T(hi + lo) x ; projection term of dx: dP phi
#pragma unroll
            for (int t = 0; t < 2; t++) {
                const int col0 = (2 * wave + t) * 32;
#pragma unroll
                for (int ks = 0; ks < 2; ks++) {
                    const bf16x8_t xf = slab_frag_t(x_s, ks * 16, col0, lane);
                    acc[t] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(__builtin_bit_cast(bf16x8_t, ah[ks]), xf, acc[t], 0, 0, 0);
                    acc[t] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(__builtin_bit_cast(bf16x8_t, al[ks]), xf, acc[t], 0, 0, 0);
                }
                f32x16_t o;
#pragma unroll
                for (int i = 0; i < 16; i++) o[i] = 0.f;
#pragma unroll
                for (int ks = 0; ks < 2; ks++)
                    o = __builtin_amdgcn_mfma_f32_32x32x16_bf16(__builtin_bit_cast(bf16x8_t, ap2[ks]), phif[t][ks], o, 0, 0, 0);
                // accumulator layout: column = lane & 31, register i -> row 8*(i/4) + 4*(lane/32) + i%4
#pragma unroll
                for (int i = 0; i < 16; i++)
                    dxf_s[(size_t)(8 * (i >> 2) + 4 * kg + (i & 3)) * kSlabLDF + col0 + row] = o[i];
            }
        }
        __syncthreads();
        MHC_PHASE_ADD(kPhaseBwdSlab, pwg, 2, pclk);

        // ---- phase C: finish dx ------------------------------------------------------------------
        if constexpr (kMixMfma) {
            // One v_mfma_f32_4x4x4_16b_bf16 is 16 independent 4x4x4 products; a block is four
            // consecutive lanes, here four channel chunks of ONE sample.  With B = the four streams of
            // a lane's channel (column = lane) and A = a coefficient matrix of the sample (row r from
            // lane r of the block), lane l receives column l: the four output streams of its own channel.
            //   D1 = G (M^T dy) + X (-(Hpre Hpre^T k2 + cx I) x)        rows: dx streams (without the
            //   D2 = [Hpost; 0; 0; 0] dy + [0; Hpre; 0; 0] x             projection and da terms)
            //                                                            rows 0, 1: df and the aggregate a
            // Coefficients enter as bf16 value + remainder (two instructions each).  Every lane runs
            // the instructions (lanes beyond the split or the channel range compute on aliased data
            // that is never stored).
            float qinv = 0.f, k2 = 0.f;
            if (!inject) {
                qinv = 1.0f / qv;
                k2 = s1v * qinv * qinv * qinv / (float)C;
            }
#pragma unroll
            for (int i = 0; i < kSlabNS; i++)
                if (i >= n) { hpre[i] = 0.f; hpost[i] = 0.f; }
            float mcol[kSlabNS], xrow[kSlabNS];
            const float hq = jq == 0 ? hpre[0] : (jq == 1 ? hpre[1] : (jq == 2 ? hpre[2] : hpre[3]));  // Hpre[lane & 3]
#pragma unroll
            for (int i = 0; i < kSlabNS; i++) {
                mcol[i] = (i < n && jq < n) ? Mr[i][0] : 0.f;
                xrow[i] = -(hq * hpre[i] * k2 + (i == jq ? cxv : 0.f));
            }
            CoefRow cg, cxr, cdf, caa;
            cg.set(mcol[0], mcol[1], mcol[2], mcol[3]);
            cxr.set(xrow[0], xrow[1], xrow[2], xrow[3]);
            const bool r0 = jq == 0, r1 = jq == 1;
            cdf.set(r0 ? hpost[0] : 0.f, r0 ? hpost[1] : 0.f, r0 ? hpost[2] : 0.f, r0 ? hpost[3] : 0.f);
            caa.set(r1 ? hpre[0] : 0.f, r1 ? hpre[1] : 0.f, r1 ? hpre[2] : 0.f, r1 ? hpre[3] : 0.f);
            const uint32_t gw[kSlabNS][4] = {{cur.gr[0].r.x, cur.gr[0].r.y, cur.gr[0].r.z, cur.gr[0].r.w},
                                             {cur.gr[1].r.x, cur.gr[1].r.y, cur.gr[1].r.z, cur.gr[1].r.w},
                                             {cur.gr[2].r.x, cur.gr[2].r.y, cur.gr[2].r.z, cur.gr[2].r.w},
                                             {cur.gr[3].r.x, cur.gr[3].r.y, cur.gr[3].r.z, cur.gr[3].r.w}};
            const uint32_t xw[kSlabNS][4] = {{cur.xr[0].x, cur.xr[0].y, cur.xr[0].z, cur.xr[0].w},
                                             {cur.xr[1].x, cur.xr[1].y, cur.xr[1].z, cur.xr[1].w},
                                             {cur.xr[2].x, cur.xr[2].y, cur.xr[2].z, cur.xr[2].w},
                                             {cur.xr[3].x, cur.xr[3].y, cur.xr[3].z, cur.xr[3].w}};
            float dfv[8];
            uint32_t dxw[kSlabNS][2];  // packed dx of the first half, stored with the second (16 bytes per stream)
#pragma unroll
            for (int h = 0; h < 2; h++) {  // two halves of four channels keep the accumulators small
                f32x4_t d1[4], d2[4];
                bf16x4_t bg[4], bx[4];
#pragma unroll
                for (int v = 0; v < 4; v++) {
                    const int p = 2 * h + (v >> 1);  // word of the channel pair
                    if (v & 1) {
                        bg[v] = streams_of_channel<true>(gw[0][p], gw[1][p], gw[2][p], gw[3][p]);
                        bx[v] = streams_of_channel<true>(xw[0][p], xw[1][p], xw[2][p], xw[3][p]);
                    } else {
                        bg[v] = streams_of_channel<false>(gw[0][p], gw[1][p], gw[2][p], gw[3][p]);
                        bx[v] = streams_of_channel<false>(xw[0][p], xw[1][p], xw[2][p], xw[3][p]);
                    }
                }
                const f32x4_t zero = {0.f, 0.f, 0.f, 0.f};
#pragma unroll
                for (int v = 0; v < 4; v++) { d1[v] = mfma4(cg.hi, bg[v], zero); d2[v] = mfma4(cdf.hi, bg[v], zero); }
#pragma unroll
                for (int v = 0; v < 4; v++) { d1[v] = mfma4(cg.lo, bg[v], d1[v]); d2[v] = mfma4(cdf.lo, bg[v], d2[v]); }
#pragma unroll
                for (int v = 0; v < 4; v++) { d1[v] = mfma4(cxr.hi, bx[v], d1[v]); d2[v] = mfma4(caa.hi, bx[v], d2[v]); }
#pragma unroll
                for (int v = 0; v < 4; v++) { d1[v] = mfma4(cxr.lo, bx[v], d1[v]); d2[v] = mfma4(caa.lo, bx[v], d2[v]); }
                float dw4[4];  // df * w / q per channel: the da term of dx is Hpre[j] times this
#pragma unroll
                for (int v = 0; v < 4; v++) {
                    const float s_df = d2[v][0], s_a = d2[v][1];
                    dfv[4 * h + v] = s_df;
                    dw4[v] = s_df * wv[4 * h + v] * qinv;
                    usum[4 * h + v] += bok ? s_df * s_a * qinv : 0.f;
                }
                if (bok) {
#pragma unroll
                    for (int j = 0; j < kSlabNS; j++) {
                        if (j < n) {
                            const float4 p0 = *reinterpret_cast<const float4 *>(dxf_s + (size_t)bl * kSlabLDF + j * kSlabCW + ch * 8 + 4 * h);
                            const float out[4] = {p0.x + d1[0][j] + hpre[j] * dw4[0], p0.y + d1[1][j] + hpre[j] * dw4[1],
                                                  p0.z + d1[2][j] + hpre[j] * dw4[2], p0.w + d1[3][j] + hpre[j] * dw4[3]};
                            if (h == 0) {
                                dxw[j][0] = pack_bf16x2(out[0], out[1]);
                                dxw[j][1] = pack_bf16x2(out[2], out[3]);
                            } else {
                                st16<true>(a.dx + (size_t)b * nC + (size_t)j * C + cth, dxw[j][0], dxw[j][1],
                                           pack_bf16x2(out[0], out[1]), pack_bf16x2(out[2], out[3]));
                            }
                        }
                    }
                }
            }
            if (bok && inject && a.df) store_vec<bf16_t, 8>(a.df + (size_t)b * C + cth, dfv);
        } else
        if (bok) {
            float qinv = 0.f, k2 = 0.f;
#pragma unroll
            for (int i = 0; i < kSlabNS; i++) {
                if (i >= n) { hpre[i] = 0.f; hpost[i] = 0.f; }
#pragma unroll
                for (int j = 0; j < kSlabNS; j++)
                    if (i >= n || j >= n) Mr[i][j] = 0.f;
            }
            if (!inject) {
                qinv = 1.0f / qv;
                k2 = s1v * qinv * qinv * qinv / (float)C;
            }
            float dfv[8];
            uint32_t dxw[kSlabNS][2];  // packed dx of the first half, stored with the second (16 bytes per stream)
            // two halves of four channels keep the live unpacked values small
#pragma unroll
            for (int h = 0; h < 2; h++) {
                float xv[kSlabNS][4], gv[kSlabNS][4];
#pragma unroll
                for (int j = 0; j < kSlabNS; j++) {
                    float t8[8];
                    unpack8(cur.xr[j], t8);
#pragma unroll
                    for (int v = 0; v < 4; v++) xv[j][v] = t8[4 * h + v];
                    cur.gr[j].get(t8);
#pragma unroll
                    for (int v = 0; v < 4; v++) gv[j][v] = t8[4 * h + v];
                }
                float da[4];
#pragma unroll
                for (int v = 0; v < 4; v++) {
                    float s_a = 0.f, s_df = 0.f;
#pragma unroll
                    for (int i = 0; i < kSlabNS; i++) { s_a += hpre[i] * xv[i][v]; s_df += hpost[i] * gv[i][v]; }
                    dfv[4 * h + v] = s_df;
                    da[v] = inject ? 0.f : s_df * wv[4 * h + v] * qinv - s_a * k2;
                    usum[4 * h + v] += s_df * s_a * qinv;
                }
#pragma unroll
                for (int j = 0; j < kSlabNS; j++) {
                    if (j < n) {
                        const float4 p0 = *reinterpret_cast<const float4 *>(dxf_s + (size_t)bl * kSlabLDF + j * kSlabCW + ch * 8 + 4 * h);
                        float out[4] = {p0.x, p0.y, p0.z, p0.w};
#pragma unroll
                        for (int v = 0; v < 4; v++) {
                            float sacc = out[v] + hpre[j] * da[v] - cxv * xv[j][v];
#pragma unroll
                            for (int i = 0; i < kSlabNS; i++) sacc += Mr[i][j] * gv[i][v];
                            out[v] = sacc;
                        }
                        if (h == 0) {
                            dxw[j][0] = pack_bf16x2(out[0], out[1]);
                            dxw[j][1] = pack_bf16x2(out[2], out[3]);
                        } else {
                            st16<true>(a.dx + (size_t)b * nC + (size_t)j * C + cth, dxw[j][0], dxw[j][1],
                                       pack_bf16x2(out[0], out[1]), pack_bf16x2(out[2], out[3]));
                        }
                    }
                }
            }
            if (inject && a.df) store_vec<bf16_t, 8>(a.df + (size_t)b * C + cth, dfv);
        }
        // no barrier needed here: the next tile's x_s writes come after barrier 2 of this tile (all
        // fragment reads done) and its dxf_s writes come after its own barrier 1 (all phase C done)
        MHC_PHASE_ADD(kPhaseBwdSlab, pwg, 3, pclk);
    };
    for (int sb = b_begin; sb < b_end; sb += 64) {
        process_tile(sb, cur, nxt);
        if (sb + 32 < b_end) process_tile(sb + 32, nxt, cur);
    }

    // ---- outputs of the split -----------------------------------------------------------------------
    float *dphi_out = a.dphi_part + (size_t)blockIdx.y * D * nC;
#pragma unroll
    for (int t = 0; t < 2; t++) {
        const int tile = 2 * wave + t, j = tile >> 1;
        const int c = c0 + (tile & 1) * 32 + row;
        if (j < n && c < C) {
#pragma unroll
            for (int i = 0; i < 16; i++) {
                const int d = 8 * (i >> 2) + 4 * kg + (i & 3);
                if (d < D) dphi_out[(size_t)d * nC + (size_t)j * C + c] = acc[t][i];
            }
        }
    }
    MHC_PHASE_ADD(kPhaseBwdSlab, pwg, 4, pclk);
    __syncthreads();  // everyone is done with dxf_s; reuse it for the two small reductions
    if (!inject) {
        // dw summands: sum over the 32 sample slots that share a channel chunk
        float *red = dxf_s;  // [32][64 + 1]
#pragma unroll
        for (int v = 0; v < 8; v++) red[bl * 65 + ch * 8 + v] = usum[v];
        __syncthreads();
        if (tid < 64) {
            float s = 0.f;
#pragma unroll
            for (int r = 0; r < 32; r++) s += red[r * 65 + tid];
            if (c0 + tid < C) a.dw_part[(size_t)blockIdx.y * C + c0 + tid] = s;
        }
        __syncthreads();
    }
    if (blockIdx.x == 0) {
        float *red = dxf_s;  // [8][32]
        red[tid] = dtsum;
        __syncthreads();
        if (tid < D + 3 && tid < 32) {
            float s = 0.f;
#pragma unroll
            for (int r = 0; r < 8; r++) s += red[r * 32 + tid];
            a.dt_part[(size_t)blockIdx.y * (D + 3) + tid] = s;
        }
    }
    MHC_PHASE_ADD(kPhaseBwdSlab, pwg, 5, pclk);
}

bool bwd_slab_supported(int x_dtype, int y_dtype, int phi_dtype, int n, int C) {
    (void)y_dtype;
    return x_dtype == kBF16 && phi_dtype == kBF16 && n <= 4 && C % 8 == 0;
}

int bwd_slab_batch_splits(int B, int n, int C) {
    const int slabs = (C + kSlabCW - 1) / kSlabCW;
    const int tiles = (B + 31) / 32;
    if (const int forced = tuning_get(kTuneSlabSplits); forced > 0) {  // experiment hook
        return forced < tiles ? forced : tiles;
    }
    // Two workgroups per CU, all resident at once (one split more than that costs a second round:
    // B=1280 C=2560, 12 splits 42.5 us, 13 splits 48.5).
    int S = 512 / slabs;
    if (S > tiles) S = tiles;
    // the dphi partial copies (written here, read once by the finalize launch) stay below 16 MB or
    // 0.4 of the activation bytes this kernel moves, whichever is larger
    const int D = n * n + 2 * n;
    const double part = 2.0 * 4.0 * D * n * C;  // bytes written + read per split
    double budget = 0.4 * (3.0 * 2.0 * B * n * C);
    if (budget < 16e6) budget = 16e6;
    if (S > (int)(budget / part)) S = (int)(budget / part);
    if (S < 1) S = 1;
    // the longest split decides: the fewest splits that keep its tile count
    // (backward us: B=1024 C=2560  11 splits of 3 tiles 37 | 8 of 4: 40.0;  B=1536 C=1920  16 of 3: 39.4 | 12 of 4: 41.7;
    //  B=800 C=1280  13 of 2: 25.5 | 12 of 2 or 3: 28.8)
    const int tps = (tiles + S - 1) / S;
    S = (tiles + tps - 1) / tps;
    return S;  // <= tiles: every split has at least one tile
}

hipError_t launch_bwd_slab(const void *dy, int y_dtype, const void *x, const void *w, int w_dtype,
                           const void *f_inject, const void *phi, const float *Hpre,
                           const float *Hpost, const float *M, const float *q, const float *s1,
                           const float *cx, const void *dPb, const void *dPT, int BP, const float *dt,
                           void *dx, void *df, float *dphi_part, float *dw_part, float *dt_part, int S,
                           int B, int n, int C, hipStream_t stream) {
    const int tiles = (B + 31) / 32;
    if (S < 1 || S > tiles) return hipErrorInvalidValue;
    BwdSlabArgs a{dy, static_cast<const bf16_t *>(x), w, f_inject, static_cast<const bf16_t *>(phi),
                  Hpre, Hpost, M, q, s1, cx, static_cast<const bf16_t *>(dPb),
                  static_cast<const bf16_t *>(dPT), dt, static_cast<bf16_t *>(dx),
                  static_cast<bf16_t *>(df), dphi_part, dw_part, dt_part, w_dtype == kBF16, B, BP, n, C, tiles};
    const size_t smem = sizeof(float) * 32 * kSlabLDF + sizeof(bf16_t) * 32 * kSlabLDX;
    dim3 grid((C + kSlabCW - 1) / kSlabCW, S);
    if (y_dtype == kBF16) bwd_slab_kernel<bf16_t><<<grid, 256, smem, stream>>>(a);
    else bwd_slab_kernel<float><<<grid, 256, smem, stream>>>(a);
    return hipGetLastError();
}

}  // namespace mhc
