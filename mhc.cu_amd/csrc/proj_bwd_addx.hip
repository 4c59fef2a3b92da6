// Backward, second (and last) launch behind the sample-resident kernel (bwd_resident.hip), bf16 tier,
// D <= 96 (n <= 8): a workgroup owns a slab of 32 columns of x_flat / phi for ALL samples, so that
//
//   dphi[d, k] = sum_b dP[b, d] x_flat[b, k]                      (reference ops.py:332-334)
//
// is finished here without batch-split partial sums, and completes dx in place,
//
//   dx[b, k] = dxp[b, k] + sum_d dP[b, d] phi[d, k] - cx[b] x_flat[b, k]      (reference ops.py:336-351)
//
// where dxp = M^T dy + Hpre (x) da was left in the dx buffer by the first launch.  A few extra
// workgroups (one more grid row) add up dw, dbias and dalpha (batch_sums.h), so the backward needs no
// third launch.
//
// Samples are walked in blocks of 128, 256 or 384 (4, 8 or 12 waves of 32 samples).  Per block every thread requests its 16-byte
// chunks of x and dxp up front (row-contiguous, next block in flight while this one is worked on); x is
// parked in LDS as [sample][column] and read back transposed as the B operand of
// v_mfma_f32_32x32x16_bf16 (the contraction of dphi runs over samples, the strided axis).  Wave w owns a
// quarter of the block's samples: it accumulates their share of every dphi tile (dP^T from global memory in fragment
// order, rounded value + remainder), forms dP phi for them (phi fragments from the slab in LDS),
// hands the result through a wave-private LDS tile to a row-major epilogue - 16-byte loads of dxp,
// 16-byte stores of dx - and at the very end the four waves' dphi shares are summed through LDS.
#include "launchers.h"

#include <type_traits>
#include "mhc_common.h"
#include "phase_profiler.h"

namespace mhc {

typedef __attribute__((__vector_size__(8 * sizeof(__bf16)))) __bf16 bf16x8_t;
typedef __attribute__((__vector_size__(16 * sizeof(float)))) float f32x16_t;

struct ProjAddxArgs {
    const void *x;       // [B][nC], bf16 or (F32) fp32 rounded to bf16 on its way into LDS
    const bf16_t *phi;   // [D][nC]
    const bf16_t *dPb;   // dP, fragment-major (frag_dpb); columns >= D are zero
    const bf16_t *dPT;   // dP^T hi and lo bf16 planes, fragment-major (frag_dpt); rows >= D, columns >= B zero
    const float *cx;     // [B]
    float *dphi;         // [D][nC]
    void *dx;            // [B][nC]: in dxp, out dx; stored like x
    int B, BP, D, DP, nC;
    int tail_row;        // blockIdx.y of the workgroups that compute `tail` (-1: none)
    BatchSumArgs tail;
};

constexpr int kAxKW = 32;          // slab width (columns)
constexpr int kAxLD = kAxKW + 8;   // LDS pitch of the bf16 tiles (elements): rows stay 16-byte aligned
constexpr int kAxLDO = kAxKW + 4;  // LDS pitch of the fp32 tile of dP phi
constexpr int kAxLDR = 36;         // LDS pitch of the dphi tiles in the final cross-wave sum (rows 16-byte aligned)

// NTD: 32-row tiles of dphi (D <= 32 NTD).  SPW: samples a wave owns per block (32 or 64; a block is
// 4 SPW samples).  PFOP: the dP operands of the next block are requested a block ahead like x and dxp.
// Measured at B=320, C=1280, n=4 (backward, graphs of ten): SPW 32 without / with PFOP 16.1 / 16.1 us,
// SPW 64 without PFOP 19.1 us, with PFOP 23.0 us (registers spill).
// F32: x and dx are stored as fp32 (x is rounded to bf16 for the products and for the -cx x term, as in
// the bf16 storage case; dxp is read and dx written as fp32).
// NW: waves per workgroup (a block is NW * SPW samples).
template <int NTD, int SPW, bool PFOP, bool F32, int NW = 4>
__global__ __launch_bounds__(64 * NW, NW == 4 ? 2 : 1) void proj_bwd_addx_kernel(ProjAddxArgs a) {
    constexpr int NT_ = 64 * NW;  // threads
    using TS = typename std::conditional<F32, float, bf16_t>::type;
    constexpr int AW = F32 ? 8 : 4;  // words of an 8-element chunk as stored
    constexpr int SBR = NW * SPW;  // samples per block
    constexpr int KS = SPW / 16;   // k-steps (16 samples) of a wave per block = its 16-byte chunks of x and of dxp
    constexpr int TT = SPW / 32;   // 32-sample tiles of a wave per block
    extern __shared__ __align__(16) unsigned char ax_smem[];
    bf16_t *phi_s = reinterpret_cast<bf16_t *>(ax_smem);                 // [32 NTD][LD]
    bf16_t *x_s = phi_s + (size_t)32 * NTD * kAxLD;                       // [SBR][LD]
    float *o_s = reinterpret_cast<float *>(x_s + (size_t)SBR * kAxLD);    // [SBR][LDO]
    float *red_s = reinterpret_cast<float *>(ax_smem);                    // final sum: [NW][NTD][32][LDR], over everything
    const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
    if ((int)blockIdx.y == a.tail_row) {
        // the extra row of the grid: its first workgroups do the batch sums, the others have nothing to do
        if ((int)blockIdx.x < a.tail.nblk) batch_sum_block<NW>(a.tail, blockIdx.x, tid, reinterpret_cast<double *>(ax_smem));
        return;
    }
    // Workgroup ids go round robin over the 8 XCDs (each with its own L2, 128-byte lines).  A slab
    // row of 32 columns is half a line: neighbouring slabs are given to the same XCD (ids x and
    // x + 8 of a group of 16), otherwise two L2s fetch every line of x, dxp and phi.
    const int slab = (blockIdx.x >> 4) * 16 + (blockIdx.x & 7) * 2 + ((blockIdx.x >> 3) & 1);
    const int k0 = slab * kAxKW;
    if (k0 >= a.nC) return;  // ids of the padded grid; the whole workgroup, before any barrier
    const int row = lane & 31, kg = lane >> 5;
    const int D = a.D, nC = a.nC, B = a.B;
    const int pwg = slab;
    (void)pwg;
    MHC_PHASE_ZERO(kPhaseColSlab, pwg);
    MHC_PHASE_BEGIN(pclk);

    // ---- per-block loads: x for the LDS tile (thread -> chunks tid + 256 u) and, for the epilogue,
    // the chunks of dxp this thread completes: sample SPW wave + lane / 4 + 16 t, chunk lane % 4 ------
    const int ech = lane & 3, erow = SPW * wave + (lane >> 2);
    const int kc = k0 + ech * 8;
    const bool kok = kc < nC;  // nC % 8 == 0: a chunk is inside or outside
    // dxp of the next block is requested a block ahead like x, except where that costs the registers that
    // keep two workgroups on a CU (fp32 storage with a wide projection): there it is requested at the top
    // of its own block and arrives under the matrix-core phase
    constexpr int PS = (F32 && NTD >= 2) ? 1 : 2;
    uint32_t xr[2][KS][AW], pr[PS][KS][AW];
    float cxr[PS][KS];
    const TS *xg = static_cast<const TS *>(a.x);
    TS *dxg = static_cast<TS *>(a.dx);
    auto load_chunk = [&](const TS *p, uint32_t (&q)[AW], bool ok) {
        const uint4 v = load16_masked(reinterpret_cast<const uint4 *>(p), ok);
        q[0] = v.x; q[1] = v.y; q[2] = v.z; q[3] = v.w;
        if constexpr (F32) {
            const uint4 v2 = load16_masked(reinterpret_cast<const uint4 *>(p) + 1, ok);
            q[4] = v2.x; q[5] = v2.y; q[6] = v2.z; q[7] = v2.w;
        }
    };
    auto load_block = [&](int sb, auto slot) {
        constexpr int S = decltype(slot)::value;
#pragma unroll
        for (int u = 0; u < KS; u++) {
            const int ch = tid + u * NT_;
            const int b = sb + (ch >> 2), k = k0 + (ch & 3) * 8;
            const bool ok = b < B && k < nC;
            load_chunk(xg + (ok ? (size_t)b * nC + k : 0), xr[S][u], ok);
        }
        if constexpr (PS == 2) {
#pragma unroll
            for (int t = 0; t < KS; t++) {
                const int b = sb + erow + 16 * t;
                const bool ok = b < B && kok;
                load_chunk(dxg + (ok ? (size_t)b * nC + kc : 0), pr[S][t], ok);
                cxr[S][t] = a.cx[b < B ? b : 0];
            }
        }
    };
    auto load_prev = [&](int sb) {  // PS == 1: the block's own dxp chunks
#pragma unroll
        for (int t = 0; t < KS; t++) {
            const int b = sb + erow + 16 * t;
            const bool ok = b < B && kok;
            load_chunk(dxg + (ok ? (size_t)b * nC + kc : 0), pr[0][t], ok);
            cxr[0][t] = a.cx[b < B ? b : 0];
        }
    };
    // Operands that come straight from global memory in fragment order: dP^T (rounded value and
    // remainder) of this wave's samples for every dphi tile, and dP of its sample tiles.  Steps and
    // tiles beyond the padded batch read zeros.
    struct Ops {
        uint4 ah[NTD][KS], al[NTD][KS], av[TT][2 * NTD];
    };
    Ops ops[PFOP ? 2 : 1];
    auto load_ops = [&](int sb, Ops &o) {
        const int step0 = (sb >> 4) + KS * wave, nsteps = a.BP >> 4;
#pragma unroll
        for (int m = 0; m < NTD; m++)
#pragma unroll
            for (int ks = 0; ks < KS; ks++) {
                const bool ok = step0 + ks < nsteps;
                const bf16_t *ap = a.dPT + (ok ? frag_base(m, nsteps, step0 + ks) : 0) + lane * 8;
                o.ah[m][ks] = load16_masked(reinterpret_cast<const uint4 *>(ap), ok);
                o.al[m][ks] = load16_masked(reinterpret_cast<const uint4 *>(ap + (size_t)a.DP * a.BP), ok);
            }
#pragma unroll
        for (int t = 0; t < TT; t++) {
            const int tile = (sb >> 5) + TT * wave + t;
            const bool ok = tile < (a.BP >> 5);
#pragma unroll
            for (int ks = 0; ks < 2 * NTD; ks++)
                o.av[t][ks] = load16_masked(
                    reinterpret_cast<const uint4 *>(a.dPb + (ok ? frag_base(tile, a.DP >> 4, ks) : 0) + lane * 8), ok);
        }
    };
    using Slot0 = std::integral_constant<int, 0>;
    using Slot1 = std::integral_constant<int, 1>;

    // ---- every load of the first block (and the next one) is requested before anything is waited for ---
    constexpr int PCH = 32 * NTD * 4;  // 16-byte chunks of the phi slab (rows >= D, columns >= nC read as zero)
    uint4 phir[(PCH + NT_ - 1) / NT_];
#pragma unroll
    for (int u = 0; u < (PCH + NT_ - 1) / NT_; u++) {
        const int ch = tid + u * NT_;
        const int d = ch >> 2, k = k0 + (ch & 3) * 8;
        const bool ok = ch < PCH && d < D && k < nC;
        phir[u] = load16_masked(reinterpret_cast<const uint4 *>(a.phi + (ok ? (size_t)d * nC + k : 0)), ok);
    }
    load_block(0, Slot0{});
    load_ops(0, ops[0]);
    if (SBR < B) {
        load_block(SBR, Slot1{});
        if constexpr (PFOP) load_ops(SBR, ops[1]);
    }
#pragma unroll
    for (int u = 0; u < (PCH + NT_ - 1) / NT_; u++) {
        const int ch = tid + u * NT_;
        if (ch < PCH) *reinterpret_cast<uint4 *>(phi_s + (size_t)(ch >> 2) * kAxLD + (ch & 3) * 8) = phir[u];
    }

    f32x16_t acc[NTD];
#pragma unroll
    for (int m = 0; m < NTD; m++)
#pragma unroll
        for (int i = 0; i < 16; i++) acc[m][i] = 0.f;
    MHC_PHASE_ADD(kPhaseColSlab, pwg, 0, pclk);

    auto process_block = [&](int sb, auto slot) {
        constexpr int S = decltype(slot)::value;
        Ops &op = ops[PFOP ? S : 0];
        constexpr int P = PS == 2 ? S : 0;
        if constexpr (PS == 1) load_prev(sb);
        if (sb != 0) {
            if constexpr (!PFOP) load_ops(sb, op);
            __syncthreads();  // every wave is done with the previous block's tile
        }
        // ---- x block -> LDS (the first barrier also covers the phi slab) -------------------------------
#pragma unroll
        for (int u = 0; u < KS; u++) {
            const int ch = tid + u * NT_;
            uint4 xb;
            if constexpr (F32)
                xb = make_uint4(pack_bf16x2(__uint_as_float(xr[S][u][0]), __uint_as_float(xr[S][u][1])),
                                pack_bf16x2(__uint_as_float(xr[S][u][2]), __uint_as_float(xr[S][u][3])),
                                pack_bf16x2(__uint_as_float(xr[S][u][4]), __uint_as_float(xr[S][u][5])),
                                pack_bf16x2(__uint_as_float(xr[S][u][6]), __uint_as_float(xr[S][u][7])));
            else xb = make_uint4(xr[S][u][0], xr[S][u][1], xr[S][u][2], xr[S][u][3]);
            *reinterpret_cast<uint4 *>(x_s + (size_t)(ch >> 2) * kAxLD + (ch & 3) * 8) = xb;
        }
        __syncthreads();
        MHC_PHASE_ADD(kPhaseColSlab, pwg, 1, pclk);
        // ---- dphi: this wave's samples, every row tile ------------------------------------------------
        {
            bf16x8_t xf[KS];
#pragma unroll
            for (int ks = 0; ks < KS; ks++)
                xf[ks] = __builtin_bit_cast(bf16x8_t, lds_frag_tr(x_s, kAxLD, (KS * wave + ks) * 16, 0, lane));
#pragma unroll
            for (int m = 0; m < NTD; m++)
#pragma unroll
                for (int ks = 0; ks < KS; ks++) {
                    acc[m] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(__builtin_bit_cast(bf16x8_t, op.ah[m][ks]), xf[ks], acc[m], 0, 0, 0);
                    acc[m] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(__builtin_bit_cast(bf16x8_t, op.al[m][ks]), xf[ks], acc[m], 0, 0, 0);
                }
        }
        // ---- dP phi of this wave's sample tiles -> its own rows of o_s (phi fragments from the slab) -----
#pragma unroll
        for (int t = 0; t < TT; t++) {
            f32x16_t o;
#pragma unroll
            for (int i = 0; i < 16; i++) o[i] = 0.f;
#pragma unroll
            for (int ks = 0; ks < 2 * NTD; ks++) {
                const bf16x8_t pf = __builtin_bit_cast(bf16x8_t, lds_frag_tr(phi_s, kAxLD, ks * 16, 0, lane));
                o = __builtin_amdgcn_mfma_f32_32x32x16_bf16(__builtin_bit_cast(bf16x8_t, op.av[t][ks]), pf, o, 0, 0, 0);
            }
            // accumulator layout: column = lane & 31, register i -> row 8*(i/4) + 4*(lane/32) + i%4
#pragma unroll
            for (int i = 0; i < 16; i++)
                o_s[(size_t)(SPW * wave + 32 * t + 8 * (i >> 2) + 4 * kg + (i & 3)) * kAxLDO + row] = o[i];
        }
        MHC_PHASE_ADD(kPhaseColSlab, pwg, 2, pclk);
        // ---- epilogue, row-major: the wave reads back only rows it wrote itself (its LDS accesses
        // complete in order), x from the block's tile ------------------------------------------------------
#pragma unroll
        for (int t = 0; t < KS; t++) {
            const int r = erow + 16 * t, b = sb + r;
            const float4 o0 = *reinterpret_cast<const float4 *>(o_s + (size_t)r * kAxLDO + ech * 8);
            const float4 o1 = *reinterpret_cast<const float4 *>(o_s + (size_t)r * kAxLDO + ech * 8 + 4);
            const uint4 xv = *reinterpret_cast<const uint4 *>(x_s + (size_t)r * kAxLD + ech * 8);
            const float cxv = cxr[P][t];
            const float ov[8] = {o0.x, o0.y, o0.z, o0.w, o1.x, o1.y, o1.z, o1.w};
            const uint32_t xw[4] = {xv.x, xv.y, xv.z, xv.w};
            float res[8];
#pragma unroll
            for (int p = 0; p < 4; p++) {
                const float plo = F32 ? __uint_as_float(pr[P][t][F32 ? 2 * p : p]) : bf16lo_to_f32(pr[P][t][p]);
                const float phi_ = F32 ? __uint_as_float(pr[P][t][F32 ? 2 * p + 1 : p]) : bf16hi_to_f32(pr[P][t][p]);
                res[2 * p] = plo + ov[2 * p] - cxv * bf16lo_to_f32(xw[p]);
                res[2 * p + 1] = phi_ + ov[2 * p + 1] - cxv * bf16hi_to_f32(xw[p]);
            }
            if (b < B && kok) store_vec<TS, 8, true>(dxg + (size_t)b * nC + kc, res);
        }
        if (sb + 2 * SBR < B) {
            load_block(sb + 2 * SBR, slot);
            if constexpr (PFOP) load_ops(sb + 2 * SBR, op);
        }
        MHC_PHASE_ADD(kPhaseColSlab, pwg, 3, pclk);
    };
    for (int sb = 0; sb < B; sb += 2 * SBR) {
        process_block(sb, Slot0{});
        if (sb + SBR < B) process_block(sb + SBR, Slot1{});
    }

    // ---- dphi: sum the four waves' shares through LDS, store row-major --------------------------------
    __syncthreads();  // all tiles consumed; the memory becomes red_s
#pragma unroll
    for (int m = 0; m < NTD; m++)
#pragma unroll
        for (int i = 0; i < 16; i++)
            red_s[((size_t)(wave * NTD + m) * 32 + 8 * (i >> 2) + 4 * kg + (i & 3)) * kAxLDR + row] = acc[m][i];
    __syncthreads();
    for (int e = tid; e < NTD * 32 * 8; e += NT_) {  // four columns per thread: 16-byte LDS reads and stores
        const int d = e >> 3, c = (e & 7) * 4;
        float4 s = make_float4(0.f, 0.f, 0.f, 0.f);
#pragma unroll
        for (int w = 0; w < NW; w++) {
            const float4 v = *reinterpret_cast<const float4 *>(red_s + ((size_t)w * NTD * 32 + d) * kAxLDR + c);
            s.x += v.x; s.y += v.y; s.z += v.z; s.w += v.w;
        }
        // nC % 8 == 0 and k0 % 32 == 0: a quad of columns is inside or outside
        if (d < D && k0 + c < nC) *reinterpret_cast<float4 *>(a.dphi + (size_t)d * nC + k0 + c) = s;
    }
    MHC_PHASE_ADD(kPhaseColSlab, pwg, 4, pclk);
}

bool proj_bwd_addx_supported(int n) { return padded_D(n) / 32 <= 3; }

template <int NTD, int SPW, bool PFOP, bool F32, int NW = 4>
static hipError_t launch_addx(const ProjAddxArgs &a, hipStream_t stream) {
    constexpr int SBR = NW * SPW;
    const size_t tiles = sizeof(bf16_t) * (size_t)kAxLD * (32 * NTD + SBR) + sizeof(float) * SBR * kAxLDO;
    const size_t red = sizeof(float) * NW * NTD * 32 * kAxLDR;  // the final cross-wave sum reuses the tiles' memory
    const size_t smem = tiles > red ? tiles : red;
    hipError_t e = allow_dynamic_lds(&proj_bwd_addx_kernel<NTD, SPW, PFOP, F32, NW>, smem);
    if (e != hipSuccess) return e;
    const int slabs = (a.nC + kAxKW - 1) / kAxKW;
    dim3 grid(round_up(slabs, 16), 1 + (a.tail_row >= 0 ? 1 : 0));
    proj_bwd_addx_kernel<NTD, SPW, PFOP, F32, NW><<<grid, 64 * NW, smem, stream>>>(a);
    return hipGetLastError();
}

hipError_t launch_proj_bwd_addx(const void *x, int x_dtype, const void *phi, const void *dPb, const void *dPT, int BP,
                                const float *cx, float *dphi, void *dx, int B, int n, int C, const BatchSumArgs *tail,
                                bool *tail_taken, hipStream_t stream) {
    const int nC = n * C, D = n * n + 2 * n, DP = padded_D(n), NTD = DP / 32;
    ProjAddxArgs a{x, static_cast<const bf16_t *>(phi), static_cast<const bf16_t *>(dPb),
                   static_cast<const bf16_t *>(dPT), cx, dphi, dx, B, BP, D, DP, nC, -1, {}};
    if (tail_taken) *tail_taken = false;
    if (tail && tail->nblk <= round_up((nC + kAxKW - 1) / kAxKW, 16)) {
        a.tail = *tail;
        a.tail_row = 1;
        if (tail_taken) *tail_taken = true;
    }
    const bool f32 = x_dtype == kF32AsBF16;
    // D <= 32: the workgroup is sized so that it walks its samples in as few blocks as possible (4, 8 or
    // 12 waves of 32 samples; every block costs two barriers and a round of dependent LDS traffic).
    // Backward at B=320, C=1280, n=4, graphs of ten: 4 waves (three blocks) 16.5 us, 8 waves 16.0, 12 waves
    // (one block) 14.9; B=128: 9.5 / 9.9 with 4 / 8 waves; B=512: 19.7 / 19.0 / 19.5.  Wider projections
    // keep four waves: their registers allow two workgroups per CU only that way.
    // More than 256 slabs: workgroups of four waves, of which three fit a CU, keep the grid in one round
    // (B=1280, C=2560, n=4: 24.4 us with 4 waves, 31.7 with 12).
    int nw = 4;
    if (NTD == 1 && (nC + kAxKW - 1) / kAxKW <= 256) {
        int best = (B + 127) / 128;
        if ((B + 255) / 256 < best) { nw = 8; best = (B + 255) / 256; }
        if ((B + 383) / 384 < best) nw = 12;
    }
    switch (NTD) {
        case 1:
            // (fp32 storage needs more registers per wave: eight waves at most)
            if (nw == 12 && !f32) return launch_addx<1, 32, false, false, 12>(a, stream);
            if (nw == 12) return launch_addx<1, 32, false, true, 8>(a, stream);
            if (nw == 8) return f32 ? launch_addx<1, 32, false, true, 8>(a, stream) : launch_addx<1, 32, false, false, 8>(a, stream);
            return f32 ? launch_addx<1, 32, false, true>(a, stream) : launch_addx<1, 32, false, false>(a, stream);
        case 2: return f32 ? launch_addx<2, 32, false, true>(a, stream) : launch_addx<2, 32, false, false>(a, stream);
        case 3: return f32 ? launch_addx<3, 32, false, true>(a, stream) : launch_addx<3, 32, false, false>(a, stream);
        default: return hipErrorInvalidValue;
    }
}

}  // namespace mhc
