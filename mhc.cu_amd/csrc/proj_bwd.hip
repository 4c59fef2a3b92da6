// Projection backward on the matrix cores (bf16 tier): for one slab of x_flat / phi columns,
//   dphi[d, k]   = sum_b dP[b, d] x_flat[b, k]        (reference ops.py:332-334)
//   dxflat[b, k] = sum_d dP[b, d] phi[d, k]           (reference ops.py:336-338)
// Both products share the slab's x and phi tiles, so phi and x are read from HBM once here.
//
// A workgroup (4 waves) owns 32*NTK columns k and walks the samples of its batch split in
// blocks of 128/NTK.  v_mfma_f32_32x32x16_bf16 contracts over the index that each lane holds
// 8 consecutive values of; for dphi that index is b and for dxflat it is d, while x and phi are
// stored with k contiguous.  The tiles are therefore staged row-major in LDS with 16-byte
// stores and read back transposed (8 two-byte reads per fragment).  The other operand (dP as
// [B, DP] and as its transpose [DP, BP], both bf16, written by the reduce kernel) is loaded
// straight from global memory in MFMA layout.  dP^T comes as a bf16 high part plus a bf16
// remainder (two MFMAs per step), which keeps dphi at fp32-like accuracy; x is exact in bf16.
#include "launchers.h"

#include <type_traits>
#include "mhc_common.h"
#include "phase_profiler.h"
#include "tuning.h"

namespace mhc {

typedef __attribute__((__vector_size__(8 * sizeof(__bf16)))) __bf16 bf16x8_t;
typedef __attribute__((__vector_size__(16 * sizeof(float)))) float f32x16_t;

struct ProjBwdArgs {
    const bf16_t *x;     // [B][nC]
    const bf16_t *phi;   // [D][nC]
    const bf16_t *dPb;   // dP, fragment-major (frag_dpb); columns >= D are zero
    const bf16_t *dPT;   // dP^T hi and lo bf16 planes, fragment-major (frag_dpt); rows >= D, columns >= B zero
    float *dphi;         // [S][D][nC]  (S = gridDim.y batch splits)
    bf16_t *dxflat;      // [B][nC]
    int B, BP, D, DP, nC, b_per_split;
    int tail_row;        // kProjDphi only: blockIdx.y of the extra row of workgroups that compute `tail` (-1: none)
    BatchSumArgs tail;   // batch sums carried by the dphi launch
};

// Transposed fragment: lane (n = lane & 31, kg = lane >> 5) gets tile[k0 + kg*8 + i][col0 + n], i = 0..7
__device__ __forceinline__ bf16x8_t lds_frag_t(const bf16_t *tile, int ld, int k0, int col0, int lane) {
    return __builtin_bit_cast(bf16x8_t, lds_frag_tr(tile, ld, k0, col0, lane));
}

// WHAT: kProjBoth = both products in one pass; kProjDphi / kProjDx = one of them (they share no
// operand but dP: dphi needs x and dP^T, dxflat needs phi and dP), for callers that launch the two
// apart.
enum { kProjBoth = kProjPartBoth, kProjDphi = kProjPartDphi, kProjDx = kProjPartDx };

template <int NTK, int TPW, bool PHI_REGS, int WHAT = kProjBoth>
__global__ __launch_bounds__(256) void proj_bwd_mfma_kernel(ProjBwdArgs a) {
    constexpr bool DO_DPHI = WHAT != kProjDx, DO_DX = WHAT != kProjDphi;
    constexpr int NSB = 4 / NTK;         // 32-sample tiles per block
    constexpr int KW = 32 * NTK;         // slab width
    constexpr int LD = KW + 8;           // LDS row pitch (elements), keeps 16-byte alignment
    constexpr int SBR = 32 * NSB;        // samples per block
    constexpr int CPR = KW / 8;          // 16-byte chunks per tile row
    extern __shared__ __align__(16) bf16_t lds_bf[];
    bf16_t *phi_s = lds_bf;                       // [DP][LD]
    bf16_t *x_s = phi_s + (size_t)a.DP * LD;      // [SBR][LD]
    const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
    if constexpr (WHAT == kProjDphi) {
        if ((int)blockIdx.y == a.tail_row) {
            // the extra row of the grid: its first workgroups do the batch sums, the others have nothing to do
            if ((int)blockIdx.x < a.tail.nblk) batch_sum_block<4>(a.tail, blockIdx.x, tid, reinterpret_cast<double *>(lds_bf));
            return;
        }
    }
    const int pwg = blockIdx.y * gridDim.x + blockIdx.x;
    (void)pwg;
    MHC_PHASE_ZERO(kPhaseProjBwd, pwg);
    MHC_PHASE_BEGIN(pclk);
    // Workgroup ids go round robin over the 8 XCDs (each with its own L2, 128-byte lines).  A slab
    // row of 32 columns is half a line: neighbouring slabs are given to the same XCD (ids x and
    // x + 8 of a group of 16), otherwise two L2s fetch every line of x and phi.
    int slab = blockIdx.x;
    if constexpr (NTK == 1) slab = (blockIdx.x >> 4) * 16 + (blockIdx.x & 7) * 2 + ((blockIdx.x >> 3) & 1);
    const int k0 = slab * KW;
    if (k0 >= a.nC) return;  // ids of the padded grid; the whole workgroup, before any barrier
    const int nt = wave % NTK, bt = wave / NTK;
    const int NTD = a.DP / 32;
    const int b_begin = blockIdx.y * a.b_per_split;
    const int b_end = min(a.B, b_begin + a.b_per_split);

    // x blocks travel through registers: the first one is requested here, ahead of the phi slab, and
    // the next one as soon as the current one has been parked in LDS
    constexpr int XCH = SBR * CPR / 256;  // 16-byte chunks of a block per thread
    static_assert(SBR * CPR % 256 == 0, "whole rounds of 256 threads");
    uint32_t xr[2][XCH][4];  // two blocks in flight; scalar words: whole-uint4 array elements can end up in scratch
    auto load_x = [&](int sb, auto slot) {
        constexpr int S = decltype(slot)::value;
#pragma unroll
        for (int u = 0; u < XCH; u++) {
            const int ch = tid + u * 256;
            const int bl = ch / CPR, b = sb + bl, k = k0 + (ch % CPR) * 8;
            const bool ok = b < b_end && k < a.nC;
            const uint4 v = load16_masked(reinterpret_cast<const uint4 *>(a.x + (ok ? (size_t)b * a.nC + k : 0)), ok);
            xr[S][u][0] = v.x; xr[S][u][1] = v.y; xr[S][u][2] = v.z; xr[S][u][3] = v.w;
        }
    };
    using Slot0 = std::integral_constant<int, 0>;
    using Slot1 = std::integral_constant<int, 1>;
    if constexpr (DO_DPHI) {
        if (b_begin < b_end) load_x(b_begin, Slot0{});
        if (b_begin + SBR < b_end) load_x(b_begin + SBR, Slot1{});
    }

    // ---- phi slab -> LDS (rows >= D and columns >= nC read as zero) ------------------------
    if constexpr (DO_DX) {
        for (int ch = tid; ch < a.DP * CPR; ch += 256) {
            const int d = ch / CPR, k = k0 + (ch % CPR) * 8;
            const bool ok = d < a.D && k < a.nC;
            const uint4 v = load16_masked(reinterpret_cast<const uint4 *>(a.phi + (ok ? (size_t)d * a.nC + k : 0)), ok);
            *reinterpret_cast<uint4 *>(phi_s + (size_t)d * LD + (ch % CPR) * 8) = v;
        }
        __syncthreads();
    }
    bf16x8_t phif[PHI_REGS ? 2 * TPW * 4 / NTK : 1];  // fragments (nt, ks) for ks < 2*NTD
    if constexpr (PHI_REGS && DO_DX) {
#pragma unroll
        for (int ks = 0; ks < 2 * TPW * 4 / NTK; ks++)
            if (ks < 2 * NTD) phif[ks] = lds_frag_t(phi_s, LD, ks * 16, nt * 32, lane);
    }

    f32x16_t acc[TPW];
#pragma unroll
    for (int m = 0; m < TPW; m++)
#pragma unroll
        for (int i = 0; i < 16; i++) acc[m][i] = 0.f;

    const int row = lane & 31, kg = lane >> 5;
    MHC_PHASE_ADD(kPhaseProjBwd, pwg, 0, pclk);
    auto process_block = [&](int sb, auto slot) {
        constexpr int S = decltype(slot)::value;
        // ---- operands that come straight from global memory (dP^T of the first dphi tile, dP of the
        // dxflat tile): requested before the barriers, they arrive while the x block is parked ------
        const int bs0 = sb + 32 * bt;
        const int b = bs0 + row;
        constexpr bool EARLY = TPW == 1;  // with more dphi tiles per wave the registers are taken by accumulators
        static_assert(!PHI_REGS || EARLY, "the dxflat operands of the phi-in-registers variant are requested early");
        uint4 ah0[EARLY ? 2 * NSB : 1], al0[EARLY ? 2 * NSB : 1], av0[PHI_REGS ? 2 * TPW * 4 / NTK : 1];
        if constexpr (EARLY) {
            if constexpr (DO_DPHI) {
                const int dt = wave / NTK;
                const bf16_t *ap = a.dPT + frag_base(dt < NTD ? dt : 0, a.BP >> 4, sb >> 4) + lane * 8;
#pragma unroll
                for (int ks = 0; ks < 2 * NSB; ks++) {
                    const bool ok = dt < NTD && sb + ks * 16 < b_end;
                    const bf16_t *apk = ok ? ap + ks * 512 : a.dPT;
                    ah0[ks] = load16_masked(reinterpret_cast<const uint4 *>(apk), ok);
                    al0[ks] = load16_masked(reinterpret_cast<const uint4 *>(apk + (size_t)a.DP * a.BP), ok);
                }
            }
            if constexpr (PHI_REGS && DO_DX) {
                const bool ok = bs0 < b_end && b < b_end;
                const bf16_t *dprow = a.dPb + frag_base((ok ? bs0 : 0) >> 5, a.DP >> 4, 0) + lane * 8;  // + 512 per k-step
#pragma unroll
                for (int ks = 0; ks < 2 * TPW * 4 / NTK; ks++)
                    av0[ks] = load16_masked(reinterpret_cast<const uint4 *>(ks < 2 * NTD ? dprow + ks * 512 : a.dPb),
                                            ok && ks < 2 * NTD);
            }
        }
        // ---- x block -> LDS, next block requested ----------------------------------------------
        if constexpr (DO_DPHI) {
        if (sb != b_begin) __syncthreads();  // previous block's fragment reads are done
#pragma unroll
        for (int u = 0; u < XCH; u++) {
            const int ch = tid + u * 256;
            *reinterpret_cast<uint4 *>(x_s + (size_t)(ch / CPR) * LD + (ch % CPR) * 8) =
                make_uint4(xr[S][u][0], xr[S][u][1], xr[S][u][2], xr[S][u][3]);
        }
        __syncthreads();
        if (sb + 2 * SBR < b_end) load_x(sb + 2 * SBR, slot);
        MHC_PHASE_ADD(kPhaseProjBwd, pwg, 1, pclk);

        // ---- dphi tiles of this wave: (dt, nt), dt = (wave + 4m) / NTK -------------------------
        // x fragments of the block once, then per tile all dP^T operands in one batch of loads
        bf16x8_t xf[2 * NSB];
#pragma unroll
        for (int ks = 0; ks < 2 * NSB; ks++) xf[ks] = lds_frag_t(x_s, LD, ks * 16, nt * 32, lane);
#pragma unroll
        for (int m = 0; m < TPW; m++) {
            const int dt = (wave + 4 * m) / NTK;
            if (dt < NTD) {
                // dP^T rows d, 8 consecutive samples; columns beyond the batch are zero padded
                const bf16_t *ap = a.dPT + frag_base(dt, a.BP >> 4, sb >> 4) + lane * 8;
                uint4 ah[2 * NSB], al[2 * NSB];
#pragma unroll
                for (int ks = 0; ks < 2 * NSB; ks++) {
                    if constexpr (EARLY) {  // requested ahead of the barriers
                        ah[ks] = ah0[ks]; al[ks] = al0[ks];
                    } else {
                        const bool ok = sb + ks * 16 < b_end;
                        const bf16_t *apk = ok ? ap + ks * 512 : a.dPT;
                        ah[ks] = load16_masked(reinterpret_cast<const uint4 *>(apk), ok);
                        al[ks] = load16_masked(reinterpret_cast<const uint4 *>(apk + (size_t)a.DP * a.BP), ok);
                    }
                }
#pragma unroll
                for (int ks = 0; ks < 2 * NSB; ks++) {
                    acc[m] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(
                        __builtin_bit_cast(bf16x8_t, ah[ks]), xf[ks], acc[m], 0, 0, 0);
                    acc[m] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(
                        __builtin_bit_cast(bf16x8_t, al[ks]), xf[ks], acc[m], 0, 0, 0);
                }
            }
        }
        }  // DO_DPHI

        MHC_PHASE_ADD(kPhaseProjBwd, pwg, 2, pclk);
        // ---- dxflat tile of this wave: samples sb + 32 bt .. +32, columns nt ------------------
        if (DO_DX && bs0 < b_end) {
            f32x16_t o;
#pragma unroll
            for (int i = 0; i < 16; i++) o[i] = 0.f;
            const bf16_t *dprow = a.dPb + frag_base(bs0 >> 5, a.DP >> 4, 0) + lane * 8;  // + 512 per k-step
            if constexpr (PHI_REGS) {
#pragma unroll
                for (int ks = 0; ks < 2 * TPW * 4 / NTK; ks++) {
                    if (ks < 2 * NTD)
                        o = __builtin_amdgcn_mfma_f32_32x32x16_bf16(__builtin_bit_cast(bf16x8_t, av0[ks]),
                                                                    phif[ks], o, 0, 0, 0);
                }
            } else {
                for (int ks0 = 0; ks0 < 2 * NTD; ks0 += 8) {  // 8 operand loads in flight
                    uint4 av[8];
#pragma unroll
                    for (int u = 0; u < 8; u++)
                    {
                        const bool ok = b < b_end && ks0 + u < 2 * NTD;
                        av[u] = load16_masked(reinterpret_cast<const uint4 *>(ok ? dprow + (ks0 + u) * 512 : a.dPb), ok);
                    }
#pragma unroll
                    for (int u = 0; u < 8; u++) {
                        if (ks0 + u < 2 * NTD) {
                            const bf16x8_t pf = lds_frag_t(phi_s, LD, (ks0 + u) * 16, nt * 32, lane);
                            o = __builtin_amdgcn_mfma_f32_32x32x16_bf16(__builtin_bit_cast(bf16x8_t, av[u]), pf, o, 0, 0, 0);
                        }
                    }
                }
            }
            // accumulator layout: column = lane & 31, register i -> row 8*(i/4) + 4*(lane/32) + i%4
            const int k = k0 + nt * 32 + row;
            if (k < a.nC) {
#pragma unroll
                for (int i = 0; i < 16; i++) {
                    const int bo = bs0 + 8 * (i >> 2) + 4 * kg + (i & 3);
                    if (bo < b_end) a.dxflat[(size_t)bo * a.nC + k] = f32_to_bf16(o[i]);
                }
            }
        }
    };
    for (int sb = b_begin; sb < b_end; sb += 2 * SBR) {
        process_block(sb, Slot0{});
        if (sb + SBR < b_end) process_block(sb + SBR, Slot1{});
    }

    MHC_PHASE_ADD(kPhaseProjBwd, pwg, 3, pclk);
    // ---- dphi out (this split's partial) -------------------------------------------------------
    float *out = a.dphi + (size_t)blockIdx.y * a.D * a.nC;
    const int k = k0 + nt * 32 + row;
#pragma unroll
    for (int m = 0; m < TPW; m++) {
        const int dt = (wave + 4 * m) / NTK;
        if (DO_DPHI && dt < NTD && k < a.nC) {
#pragma unroll
            for (int i = 0; i < 16; i++) {
                const int d = dt * 32 + 8 * (i >> 2) + 4 * kg + (i & 3);
                if (d < a.D) out[(size_t)d * a.nC + k] = acc[m][i];
            }
        }
    }
    MHC_PHASE_ADD(kPhaseProjBwd, pwg, 4, pclk);
}

// --------------------------------------------------------------------------------------------
// shape selection
// --------------------------------------------------------------------------------------------
bool proj_bwd_mfma_supported(int x_dtype, int phi_dtype, int C) {
    return x_dtype == kBF16 && phi_dtype == kBF16 && C % 8 == 0;
}

// Slab width (in 32-column tiles) for this shape.
static int proj_bwd_ntk(int B, int n, int C) {
    (void)B; (void)n; (void)C;
    return 1;
}

int proj_bwd_batch_splits(int B, int n, int C) {
    const int NTK = proj_bwd_ntk(B, n, C);
    const int nC = n * C, D = n * n + 2 * n;
    const int slabs = (nC + 32 * NTK - 1) / (32 * NTK);
    const int sbr = 32 * (4 / NTK);
    const int nblocks = (B + sbr - 1) / sbr;
    int S = (512 + slabs - 1) / slabs;
    if (S > nblocks) S = nblocks;
    // keep the partial sums below ~1/4 of the activation bytes this kernel moves
    const double cap = 0.25 * (2.0 * 2.0 * B * nC) / (4.0 * D * nC);
    if (S > (int)cap) S = (int)cap;
    if (S < 1) S = 1;
    if (const int forced = tuning_get(kTuneSlabSplits); forced > 0) S = forced < nblocks ? forced : nblocks;  // experiment hook
    return S;
}

template <int NTK, int TPW, bool PHI_REGS, int WHAT>
static hipError_t launch_what(const ProjBwdArgs &a, int S, hipStream_t stream) {
    constexpr int LD = 32 * NTK + 8;
    const size_t smem = sizeof(bf16_t) * (size_t)LD * (a.DP + 32 * (4 / NTK));
    auto kern = proj_bwd_mfma_kernel<NTK, TPW, PHI_REGS, WHAT>;
    if (smem > 64 * 1024) {
        hipError_t e = hipFuncSetAttribute(reinterpret_cast<const void *>(kern),
                                           hipFuncAttributeMaxDynamicSharedMemorySize, (int)smem);
        if (e != hipSuccess) return e;
    }
    const int slabs = (a.nC + 32 * NTK - 1) / (32 * NTK);
    dim3 grid(NTK == 1 ? round_up(slabs, 16) : slabs, S + (WHAT == kProjDphi && a.tail_row >= 0 ? 1 : 0));
    kern<<<grid, 256, smem, stream>>>(a);
    return hipGetLastError();
}


bool proj_bwd_products_apart(int n) { return padded_D(n) / 32 > 4; }

hipError_t launch_proj_bwd_mfma(const void *x, const void *phi, const void *dPb, const void *dPT,
                                int BP, float *dphi, float *dphi_part, void *dxflat, int B, int n,
                                int C, hipStream_t stream, int part, const BatchSumArgs *tail, bool *tail_taken) {
    const int nC = n * C, D = n * n + 2 * n, DP = padded_D(n);
    const int S = proj_bwd_batch_splits(B, n, C);
    const int NTK = proj_bwd_ntk(B, n, C);
    const int sbr = 32 * (4 / NTK);
    const int nblocks = (B + sbr - 1) / sbr;
    const int bps = (nblocks + S - 1) / S * sbr;
    ProjBwdArgs a{static_cast<const bf16_t *>(x), static_cast<const bf16_t *>(phi),
                  static_cast<const bf16_t *>(dPb), static_cast<const bf16_t *>(dPT),
                  S > 1 ? dphi_part : dphi, static_cast<bf16_t *>(dxflat), B, BP, D, DP, nC, bps, -1, {}};
    const int NTD = DP / 32;
    hipError_t e;
    if (tail_taken) *tail_taken = false;
    if (NTD <= 12 && part == kProjDphi && tail && tail->nblk <= (nC + 32 * NTK - 1) / (32 * NTK) && NTK == 1) {
        a.tail = *tail;
        a.tail_row = S;
        if (tail_taken) *tail_taken = true;
    }
    // NTK == 1: dphi tiles per wave = ceil(NTD / 4); phi fragments in registers when 2*NTD <= 8.
    // Wide projections (more than 12 row tiles) run as two GEMM kernels that share no operand.
    if (part == kProjDx) { a.b_per_split = B; }
    if (NTD <= 4) e = part == kProjBoth ? launch_what<1, 1, true, kProjBoth>(a, S, stream)
                    : part == kProjDx ? launch_what<1, 1, true, kProjDx>(a, 1, stream)
                                      : launch_what<1, 1, true, kProjDphi>(a, S, stream);
    else if (NTD <= 12) e = part == kProjBoth ? launch_what<1, 3, false, kProjBoth>(a, S, stream)
                            : part == kProjDx ? launch_what<1, 3, false, kProjDx>(a, 1, stream)
                                              : launch_what<1, 3, false, kProjDphi>(a, S, stream);
    else {
        e = launch_dxflat_wide(phi, dPb, BP, dxflat, nullptr, nullptr, nullptr, B, n, C, stream);
        if (e == hipSuccess) e = launch_dphi_large(x, dPT, BP, S > 1 ? dphi_part : dphi, S, B, n, C, nullptr, nullptr, stream);
        (void)part;  // wide shapes: callers that want the products apart use the two launchers themselves
    }
    return e;  // with S > 1 the caller's finalize launch sums the S partial copies
}

}  // namespace mhc
