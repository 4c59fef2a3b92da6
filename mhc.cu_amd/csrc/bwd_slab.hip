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
#include "mhc_common.h"
#include "phase_profiler.h"

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
    int w_bf16, B, BP, n, C, b_per_split;
};

__device__ __forceinline__ bf16x8_t slab_frag_t(const bf16_t *tile, int k0, int col0, int lane) {
    // lane (n = lane & 31, kg = lane >> 5) gets tile[k0 + kg*8 + i][col0 + n], i = 0..7
    const bf16_t *p = tile + (size_t)(k0 + (lane >> 5) * 8) * kSlabLDX + col0 + (lane & 31);
    uint32_t wv[4];
#pragma unroll
    for (int i = 0; i < 4; i++) {
        const uint32_t lo = p[(2 * i) * kSlabLDX], hi = p[(2 * i + 1) * kSlabLDX];
        wv[i] = lo | (hi << 16);
    }
    return __builtin_bit_cast(bf16x8_t, make_uint4(wv[0], wv[1], wv[2], wv[3]));
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
    const int b_begin = blockIdx.y * a.b_per_split;
    const int b_end = min(a.B, b_begin + a.b_per_split);
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
    for (int sb = b_begin; sb < b_end; sb += 32) {
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
        float hpre[kSlabNS], hpost[kSlabNS], Mr[kSlabNS][kSlabNS], cxv, qv = 1.f, s1v = 0.f;
        {
            const size_t bc = bok ? b : 0;
#pragma unroll
            for (int i = 0; i < kSlabNS; i++) {
                hpre[i] = a.Hpre[bc * n + (i < n ? i : 0)];
                hpost[i] = a.Hpost[bc * n + (i < n ? i : 0)];
#pragma unroll
                for (int j = 0; j < kSlabNS; j++)
                    Mr[i][j] = a.M[bc * n * n + ((i < n && j < n) ? i * n + j : 0)];
            }
            cxv = a.cx[bc];
            if (!inject) { qv = a.q[bc]; s1v = a.s1[bc]; }
        }
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

        // ---- prefetch the next tile, then phase C: finish dx on the VALU ---------------------------
        const bool more = sb + 32 < b_end;
        if (more) load_tile(sb + 32, nxt);
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
        if (more) cur = nxt;
        MHC_PHASE_ADD(kPhaseBwdSlab, pwg, 3, pclk);
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
    MHC_PHASE_ADD(kPhaseBwdSlab, pwg, 4, pclk);
}

bool bwd_slab_supported(int x_dtype, int y_dtype, int phi_dtype, int n, int C) {
    (void)y_dtype;
    return x_dtype == kBF16 && phi_dtype == kBF16 && n <= 4 && C % 8 == 0;
}

int bwd_slab_batch_splits(int B, int n, int C) {
    const int slabs = (C + kSlabCW - 1) / kSlabCW;
    const int tiles = (B + 31) / 32;
    int S = (512 + slabs - 1) / slabs;  // two workgroups per CU
    if (S > tiles) S = tiles;
    // the dphi partial copies (written here, read once by the finalize launch) stay below 12 MB or
    // ~1/4 of the activation bytes this kernel moves, whichever is larger
    const int D = n * n + 2 * n;
    const double part = 2.0 * 4.0 * D * n * C;  // bytes written + read per split
    double budget = 0.25 * (3.0 * 2.0 * B * n * C);
    if (budget < 12e6) budget = 12e6;
    if (S > (int)(budget / part)) S = (int)(budget / part);
    if (S < 1) S = 1;
    // splits are whole 32-sample tiles: drop the splits that would get none
    const int tps = (tiles + S - 1) / S;
    return (tiles + tps - 1) / tps;
}

hipError_t launch_bwd_slab(const void *dy, int y_dtype, const void *x, const void *w, int w_dtype,
                           const void *f_inject, const void *phi, const float *Hpre,
                           const float *Hpost, const float *M, const float *q, const float *s1,
                           const float *cx, const void *dPb, const void *dPT, int BP, const float *dt,
                           void *dx, void *df, float *dphi_part, float *dw_part, float *dt_part, int S,
                           int B, int n, int C, hipStream_t stream) {
    const int tiles = (B + 31) / 32;
    const int bps = (tiles + S - 1) / S * 32;
    BwdSlabArgs a{dy, static_cast<const bf16_t *>(x), w, f_inject, static_cast<const bf16_t *>(phi),
                  Hpre, Hpost, M, q, s1, cx, static_cast<const bf16_t *>(dPb),
                  static_cast<const bf16_t *>(dPT), dt, static_cast<bf16_t *>(dx),
                  static_cast<bf16_t *>(df), dphi_part, dw_part, dt_part, w_dtype == kBF16, B, BP, n, C, bps};
    const size_t smem = sizeof(float) * 32 * kSlabLDF + sizeof(bf16_t) * 32 * kSlabLDX;
    dim3 grid((C + kSlabCW - 1) / kSlabCW, S);
    if (y_dtype == kBF16) bwd_slab_kernel<bf16_t><<<grid, 256, smem, stream>>>(a);
    else bwd_slab_kernel<float><<<grid, 256, smem, stream>>>(a);
    return hipGetLastError();
}

}  // namespace mhc
