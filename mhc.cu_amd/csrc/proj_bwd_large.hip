// Projection backward for wide projections (D = n^2 + 2n > 384, i.e. n > 18; the n = 32
// configuration has D = 1088): the two products of proj_bwd.hip as two GEMM kernels, because at
// this width they share no operand - dphi = dP^T x_flat streams x and writes dphi, dxflat = dP phi
// streams phi - and separate kernels keep the per-workgroup LDS and register footprints small
// enough for several workgroups per CU, which is what hides the operand-load latency.
//
// Both use v_mfma_f32_32x32x16_bf16 with one operand loaded straight from global memory in MFMA
// layout (dP^T hi/lo rows resp. dP rows, both written by the reduce kernel) and the other staged
// row-major in LDS and read back transposed (x resp. phi, whose contiguous index is not the
// contracted one).
#include "launchers.h"
#include "mhc_common.h"

namespace mhc {

typedef __attribute__((__vector_size__(8 * sizeof(__bf16)))) __bf16 bf16x8_t;
typedef __attribute__((__vector_size__(16 * sizeof(float)))) float f32x16_t;

constexpr int kPL_KW = 128;             // columns per workgroup: wave w owns columns 32w .. 32w+32
constexpr int kPL_LD = kPL_KW + 8;      // LDS row pitch in elements (272 bytes, 16-byte aligned)
constexpr int kPL_SB = 128;             // samples per block of the dphi kernel
constexpr int kPL_TPW = 3;              // dphi row tiles per workgroup (each wave: 3 tiles x its columns)
constexpr int kPL_DC = 64;              // phi rows per LDS chunk of the dxflat kernel

struct ProjBwdLargeArgs {
    const bf16_t *x;     // [B][nC]
    const bf16_t *phi;   // [D][nC]
    const bf16_t *dPb;   // dP, fragment-major (frag_dpb)
    const bf16_t *dPT;   // dP^T hi/lo planes, fragment-major (frag_dpt)
    float *dphi;         // [S][D][nC]
    bf16_t *dxflat;      // [B][nC]
    int B, BP, D, DP, nC, b_per_split;
};

// lane (n = lane & 31, kg = lane >> 5) gets tile[k0 + kg*8 + i][col0 + n], i = 0..7
__device__ __forceinline__ bf16x8_t pl_frag_t(const bf16_t *tile, int k0, int col0, int lane) {
    const bf16_t *p = tile + (size_t)(k0 + (lane >> 5) * 8) * kPL_LD + col0 + (lane & 31);
    uint32_t w[4];
#pragma unroll
    for (int i = 0; i < 4; i++) {
        const uint32_t lo = p[(2 * i) * kPL_LD], hi = p[(2 * i + 1) * kPL_LD];
        w[i] = lo | (hi << 16);
    }
    return __builtin_bit_cast(bf16x8_t, make_uint4(w[0], w[1], w[2], w[3]));
}

// ---------------------------------------------------------------------------------------------
// dphi[d, k] = sum_b dP[b, d] x[b, k]: workgroup = 128 columns k x 3 row tiles of d; the four
// waves share the dP^T operands (L1) and write 512 contiguous bytes per dphi row.
// grid: (column slabs, groups of 3 d-tiles, batch splits)
// ---------------------------------------------------------------------------------------------
__global__ __launch_bounds__(256) void dphi_large_kernel(ProjBwdLargeArgs a) {
    extern __shared__ bf16_t pl_lds[];
    bf16_t *x_s = pl_lds;  // [kPL_SB][kPL_LD]
    const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
    const int row = lane & 31, kg = lane >> 5;
    const int k0 = blockIdx.x * kPL_KW;
    const int NTD = a.DP / 32;
    const int b_begin = blockIdx.z * a.b_per_split;
    const int b_end = min(a.B, b_begin + a.b_per_split);

    f32x16_t acc[kPL_TPW];
#pragma unroll
    for (int m = 0; m < kPL_TPW; m++)
#pragma unroll
        for (int i = 0; i < 16; i++) acc[m][i] = 0.f;

    for (int sb = b_begin; sb < b_end; sb += kPL_SB) {
        if (sb != b_begin) __syncthreads();
        for (int ch = tid; ch < kPL_SB * (kPL_KW / 8); ch += 256) {
            const int bl = ch / (kPL_KW / 8), b = sb + bl, kc = (ch % (kPL_KW / 8)) * 8;
            const bool ok = b < b_end && k0 + kc < a.nC;
            const uint4 v = load16_masked(reinterpret_cast<const uint4 *>(a.x + (ok ? (size_t)b * a.nC + k0 + kc : 0)), ok);
            *reinterpret_cast<uint4 *>(x_s + (size_t)bl * kPL_LD + kc) = v;
        }
        __syncthreads();
        bf16x8_t xf[8];
#pragma unroll
        for (int ks = 0; ks < 8; ks++) xf[ks] = pl_frag_t(x_s, ks * 16, wave * 32, lane);
#pragma unroll
        for (int m = 0; m < kPL_TPW; m++) {
            const int dt = blockIdx.y * kPL_TPW + m;
            if (dt < NTD) {
                const bf16_t *ap = a.dPT + frag_base(dt, a.BP >> 4, sb >> 4) + lane * 8;
                uint4 ah[8], al[8];
#pragma unroll
                for (int ks = 0; ks < 8; ks++) {
                    const bool ok = sb + ks * 16 < b_end;  // pad columns [B, BP) are zero
                    const bf16_t *apk = ok ? ap + ks * 512 : a.dPT;
                    ah[ks] = load16_masked(reinterpret_cast<const uint4 *>(apk), ok);
                    al[ks] = load16_masked(reinterpret_cast<const uint4 *>(apk + (size_t)a.DP * a.BP), ok);
                }
#pragma unroll
                for (int ks = 0; ks < 8; ks++) {
                    acc[m] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(__builtin_bit_cast(bf16x8_t, ah[ks]), xf[ks], acc[m], 0, 0, 0);
                    acc[m] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(__builtin_bit_cast(bf16x8_t, al[ks]), xf[ks], acc[m], 0, 0, 0);
                }
            }
        }
    }
    float *out = a.dphi + (size_t)blockIdx.z * a.D * a.nC;
    const int k = k0 + wave * 32 + row;
#pragma unroll
    for (int m = 0; m < kPL_TPW; m++) {
        const int dt = blockIdx.y * kPL_TPW + m;
        if (dt < NTD && k < a.nC) {
#pragma unroll
            for (int i = 0; i < 16; i++) {
                const int d = dt * 32 + 8 * (i >> 2) + 4 * kg + (i & 3);
                if (d < a.D) out[(size_t)d * a.nC + k] = acc[m][i];
            }
        }
    }
}

// ---------------------------------------------------------------------------------------------
// dxflat[b, k] = sum_d dP[b, d] phi[d, k]: workgroup = 32 samples x 128 columns (wave w: columns
// 32w..), phi streamed through LDS in double-buffered chunks of 64 rows x 256 contiguous bytes.
// grid.x enumerates (sample tile, column slab) with the sample tile fastest and slabs dealt to
// the 8 XCDs so that the workgroups sharing a phi slab run on the same L2.
// ---------------------------------------------------------------------------------------------
__global__ __launch_bounds__(256) void dxflat_large_kernel(ProjBwdLargeArgs a, int tiles_s, int slabs) {
    extern __shared__ bf16_t pl_lds[];
    bf16_t *phi_s0 = pl_lds, *phi_s1 = pl_lds + kPL_DC * kPL_LD;
    const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
    const int row = lane & 31, kg = lane >> 5;
    // id = ((slab / 8) * tiles_s + st) * 8 + slab % 8  ->  XCD (id % 8) is the same for all st
    const int id = blockIdx.x;
    const int slab = (id / (8 * tiles_s)) * 8 + (id & 7);
    const int st = (id >> 3) % tiles_s;
    if (slab >= slabs) return;
    const int k0 = slab * kPL_KW;
    const int nchunks = (a.DP + kPL_DC - 1) / kPL_DC;
    const bf16_t *dprow = a.dPb + frag_base(st, a.DP >> 4, 0) + lane * 8;  // + 512 per k-step

    // this thread's four 16-byte pieces of a phi chunk: rows (tid >> 4) + 16 h, column piece tid & 15.
    // The prefetching loads carry no predicate (it would be applied right behind the load and stall
    // the prefetch): out-of-range pieces alias valid memory and are zeroed when they are parked in
    // LDS; the dP operand then only needs to be finite where phi is zero, so its out-of-range
    // k-steps alias k-step 0.
    auto load_phi = [&](int c, uint4 (&v)[4]) {
#pragma unroll
        for (int h = 0; h < 4; h++) {
            const int d = c * kPL_DC + (tid >> 4) + 16 * h, k = k0 + (tid & 15) * 8;
            const bool ok = d < a.D && k < a.nC;
            v[h] = *reinterpret_cast<const uint4 *>(a.phi + (ok ? (size_t)d * a.nC + k : 0));
        }
    };
    auto store_phi = [&](bf16_t *buf, int c, const uint4 (&v)[4]) {
#pragma unroll
        for (int h = 0; h < 4; h++) {
            const int d = c * kPL_DC + (tid >> 4) + 16 * h, k = k0 + (tid & 15) * 8;
            const bool ok = d < a.D && k < a.nC;
            uint4 t = v[h];
            t.x = ok ? t.x : 0u; t.y = ok ? t.y : 0u; t.z = ok ? t.z : 0u; t.w = ok ? t.w : 0u;
            *reinterpret_cast<uint4 *>(buf + (size_t)((tid >> 4) + 16 * h) * kPL_LD + (tid & 15) * 8) = t;
        }
    };
    auto load_a = [&](int c, uint4 (&v)[4]) {
#pragma unroll
        for (int ks = 0; ks < 4; ks++) {
            const int d0 = c * kPL_DC + ks * 16;
            v[ks] = *reinterpret_cast<const uint4 *>(dprow + (d0 < a.DP ? (size_t)(d0 >> 4) * 512 : 0));
        }
    };

    f32x16_t o;
#pragma unroll
    for (int i = 0; i < 16; i++) o[i] = 0.f;
    uint4 pv[4], av[4], an[4];
    load_phi(0, pv);
    load_a(0, av);
    store_phi(phi_s0, 0, pv);
    __syncthreads();
    for (int c = 0; c < nchunks; c++) {
        const bool more = c + 1 < nchunks;
        bf16_t *cur = (c & 1) ? phi_s1 : phi_s0, *nxt = (c & 1) ? phi_s0 : phi_s1;
        if (more) { load_phi(c + 1, pv); load_a(c + 1, an); }
#pragma unroll
        for (int ks = 0; ks < 4; ks++) {
            const bf16x8_t pf = pl_frag_t(cur, ks * 16, wave * 32, lane);
            o = __builtin_amdgcn_mfma_f32_32x32x16_bf16(__builtin_bit_cast(bf16x8_t, av[ks]), pf, o, 0, 0, 0);
        }
        if (more) {
            store_phi(nxt, c + 1, pv);
#pragma unroll
            for (int ks = 0; ks < 4; ks++) av[ks] = an[ks];
        }
        __syncthreads();
    }
    // accumulator layout: column = lane & 31, register i -> row 8*(i/4) + 4*(lane/32) + i%4.
    // Stage the 32 x 128 tile in LDS as bf16 so that it leaves as 16-byte pieces of 256-byte rows
    // (two-byte scattered stores cost an order of magnitude more write traffic).
    bf16_t *o_s = phi_s0;  // the last loop iteration ended with a barrier: both buffers are free
#pragma unroll
    for (int i = 0; i < 16; i++)
        o_s[(size_t)(8 * (i >> 2) + 4 * kg + (i & 3)) * kPL_LD + wave * 32 + row] = f32_to_bf16(o[i]);
    __syncthreads();
#pragma unroll
    for (int h = 0; h < 2; h++) {
        const int r = (tid >> 4) + 16 * h, kc = (tid & 15) * 8;
        const int bo = st * 32 + r;
        if (bo < a.B && k0 + kc < a.nC)
            *reinterpret_cast<uint4 *>(a.dxflat + (size_t)bo * a.nC + k0 + kc) =
                *reinterpret_cast<const uint4 *>(o_s + (size_t)r * kPL_LD + kc);
    }
}

hipError_t launch_proj_bwd_large(const void *x, const void *phi, const void *dPb, const void *dPT,
                                 int BP, float *dphi_out, void *dxflat, int S, int B, int n, int C,
                                 hipStream_t stream) {
    const int nC = n * C, D = n * n + 2 * n, DP = padded_D(n);
    const int nblocks = (B + kPL_SB - 1) / kPL_SB;
    const int bps = (nblocks + S - 1) / S * kPL_SB;
    ProjBwdLargeArgs a{static_cast<const bf16_t *>(x), static_cast<const bf16_t *>(phi),
                       static_cast<const bf16_t *>(dPb), static_cast<const bf16_t *>(dPT), dphi_out,
                       static_cast<bf16_t *>(dxflat), B, BP, D, DP, nC, bps};
    const int slabs = (nC + kPL_KW - 1) / kPL_KW;
    const int NTD = DP / 32;
    const int tiles_s = (B + 31) / 32;
    const int slab_groups = (slabs + 7) / 8;
    dxflat_large_kernel<<<slab_groups * tiles_s * 8, 256, sizeof(bf16_t) * 2 * kPL_DC * kPL_LD, stream>>>(a, tiles_s, slabs);
    hipError_t e = hipGetLastError();
    if (e != hipSuccess) return e;
    dphi_large_kernel<<<dim3(slabs, (NTD + kPL_TPW - 1) / kPL_TPW, S), 256,
                        sizeof(bf16_t) * kPL_SB * kPL_LD, stream>>>(a);
    return hipGetLastError();
}

}  // namespace mhc
