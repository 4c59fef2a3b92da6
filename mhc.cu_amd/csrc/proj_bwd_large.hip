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

struct ProjBwdLargeArgs {
    const bf16_t *x;     // [B][nC]
    const bf16_t *phi;   // [D][nC]
    const bf16_t *dPb;   // dP, fragment-major (frag_dpb)
    const bf16_t *dPT;   // dP^T hi/lo planes, fragment-major (frag_dpt)
    float *dphi;         // [S][D][nC]
    bf16_t *dxflat;      // [B][nC]
    int B, BP, D, DP, nC, b_per_split;
    int tpw;             // row tiles per workgroup of the single-block dphi kernel
    int tail_row;        // blockIdx.y of the extra row of workgroups that compute `tail` (-1: none)
    BatchSumArgs tail;   // batch sums carried by the dphi launch (see launch_dphi_large)
    const float *cx = nullptr;     // dxflat kernel: when set, the output is dx = dx_part + dP phi - cx x
    const float *dx_part = nullptr;  // fp32 [B][nC], the part of dx another launch has left (with cx)
};

// lane (n = lane & 31, kg = lane >> 5) gets tile[k0 + kg*8 + i][col0 + n], i = 0..7
__device__ __forceinline__ bf16x8_t pl_frag_t(const bf16_t *tile, int k0, int col0, int lane) {
    return __builtin_bit_cast(bf16x8_t, lds_frag_tr(tile, kPL_LD, k0, col0, lane));
}

// ---------------------------------------------------------------------------------------------
// dphi[d, k] = sum_b dP[b, d] x[b, k]: workgroup = 128 columns k x a group of row tiles of d.
// The [128 samples x 128 columns] block of x is fetched with all of a thread's loads in flight,
// parked in LDS and read back transposed once (the contraction runs over samples); wave w keeps
// the fragments of columns 32w..32w+32 in registers and walks the row tiles of the group: the
// dP^T operands (rounded value + remainder, fragment-major, coalesced) of the next row tile are
// requested before the current tile's MFMAs are issued.  The kernel is bound by the fp32 dphi
// stores (512 contiguous bytes per row and workgroup).
// grid: (column slabs, groups of kPL_TPW row tiles, batch splits)
// ---------------------------------------------------------------------------------------------
// SINGLE: the split holds one sample block, so a row tile is complete (and stored) right after its
// MFMAs and one accumulator is live at a time; otherwise TPW accumulators persist over the blocks.
template <int TPW, bool SINGLE>
__global__ __launch_bounds__(256) void dphi_large_kernel(ProjBwdLargeArgs a) {
    extern __shared__ __align__(16) bf16_t pl_lds[];
    bf16_t *x_s = pl_lds;  // [kPL_SB][kPL_LD]
    const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
    if ((int)blockIdx.y == a.tail_row) {
        // the extra row of the grid: its first workgroups do the batch sums, the others have nothing to do
        if (blockIdx.z == 0 && (int)blockIdx.x < a.tail.nblk)
            batch_sum_block<4>(a.tail, blockIdx.x, tid, reinterpret_cast<double *>(pl_lds));
        return;
    }
    const int row = lane & 31, kg = lane >> 5;
    const int k0 = blockIdx.x * kPL_KW;
    const int NTD = a.DP / 32;
    const int tpw = SINGLE ? a.tpw : TPW;
    const int dt0 = blockIdx.y * tpw, dt1 = min(NTD, dt0 + tpw);
    const int b_begin = blockIdx.z * a.b_per_split;
    const int b_end = min(a.B, b_begin + a.b_per_split);
    float *out = a.dphi + (size_t)blockIdx.z * a.D * a.nC;
    const int k = k0 + wave * 32 + row;
    const size_t plane = (size_t)a.DP * a.BP;

    constexpr int NACC = SINGLE ? 1 : TPW;
    f32x16_t acc[NACC];
#pragma unroll
    for (int m = 0; m < NACC; m++)
#pragma unroll
        for (int i = 0; i < 16; i++) acc[m][i] = 0.f;

    for (int sb = b_begin; sb < b_end; sb += kPL_SB) {
        if (sb != b_begin) __syncthreads();
        // thread owns 16-byte segment tid & 15 of rows (tid >> 4) + 16 q
        const int seg = tid & 15, r0 = tid >> 4;
        const bool kok = k0 + seg * 8 < a.nC;
        RawVec<bf16_t, 8> xr[8];
#pragma unroll
        for (int q = 0; q < 8; q++) {
            const int b = sb + r0 + 16 * q;
            xr[q].load(a.x + ((b < b_end && kok) ? (size_t)b * a.nC + k0 + seg * 8 : 0));
        }
#pragma unroll
        for (int q = 0; q < 8; q++) {
            const bool ok = sb + r0 + 16 * q < b_end && kok;  // rows of other splits must not count
            *reinterpret_cast<uint4 *>(x_s + (size_t)(r0 + 16 * q) * kPL_LD + seg * 8) =
                make_uint4(ok ? xr[q].w[0] : 0u, ok ? xr[q].w[1] : 0u, ok ? xr[q].w[2] : 0u, ok ? xr[q].w[3] : 0u);
        }
        __syncthreads();
        bf16x8_t xf[8];
#pragma unroll
        for (int ks = 0; ks < 8; ks++) xf[ks] = pl_frag_t(x_s, ks * 16, wave * 32, lane);

        // dP^T operands of a row tile: 8 k-steps x (rounded, remainder) x 64 lanes x 16 bytes = 16 KB,
        // contiguous per plane in the fragment-major layout.  All four waves multiply the same
        // operands (they differ in the columns they own), so the workgroup fetches a tile once,
        // 4 x 16 bytes per thread, and shares it through a double-buffered LDS tile; k-steps beyond
        // the padded batch alias k-step 0 of the block and meet zero rows of x.
        // (the operand tiles reuse the LDS of the x block, which is dead once xf is in registers)
        bf16_t *a_s = x_s;  // [2][2 planes][8 k-steps][512]
        uint32_t ar[16];  // scalar words: whole-uint4 array elements can end up in scratch memory
        auto fetch_a = [&](int dt) {
            const bf16_t *ap = a.dPT + frag_base(min(dt, NTD - 1), a.BP >> 4, sb >> 4);
#pragma unroll
            for (int j = 0; j < 2; j++) {
                const int c = tid + 256 * j, ks = c >> 6;  // 16-byte piece c of the plane's 8 KB
                const bf16_t *apk = ap + (sb + ks * 16 < a.BP ? c * 8 : (c & 63) * 8);
                const uint4 h = *reinterpret_cast<const uint4 *>(apk);
                const uint4 l = *reinterpret_cast<const uint4 *>(apk + plane);
                ar[8 * j] = h.x; ar[8 * j + 1] = h.y; ar[8 * j + 2] = h.z; ar[8 * j + 3] = h.w;
                ar[8 * j + 4] = l.x; ar[8 * j + 5] = l.y; ar[8 * j + 6] = l.z; ar[8 * j + 7] = l.w;
            }
        };
        auto park_a = [&](int buf) {
            bf16_t *dst = a_s + (size_t)buf * 2 * 4096;
#pragma unroll
            for (int j = 0; j < 2; j++) {
                *reinterpret_cast<uint4 *>(dst + (tid + 256 * j) * 8) =
                    make_uint4(ar[8 * j], ar[8 * j + 1], ar[8 * j + 2], ar[8 * j + 3]);
                *reinterpret_cast<uint4 *>(dst + 4096 + (tid + 256 * j) * 8) =
                    make_uint4(ar[8 * j + 4], ar[8 * j + 5], ar[8 * j + 6], ar[8 * j + 7]);
            }
        };
        fetch_a(dt0);
        __syncthreads();  // every wave has its x fragments
        park_a(0);
        __syncthreads();
        // one row tile: request the next tile's operands, multiply from LDS, (SINGLE) store, park
        // the next tile, one barrier
        auto do_tile = [&](int m, f32x16_t &am) {
            fetch_a(dt0 + m + 1);  // clamped to the last tile: redundant at the end, never used
            if (SINGLE) {
#pragma unroll
                for (int i = 0; i < 16; i++) am[i] = 0.f;
            }
            const bf16_t *src = a_s + (size_t)(m & 1) * 2 * 4096 + lane * 8;
#pragma unroll
            for (int ks = 0; ks < 8; ks++) {
                const uint4 h = *reinterpret_cast<const uint4 *>(src + ks * 512);
                const uint4 l = *reinterpret_cast<const uint4 *>(src + 4096 + ks * 512);
                am = __builtin_amdgcn_mfma_f32_32x32x16_bf16(__builtin_bit_cast(bf16x8_t, h), xf[ks], am, 0, 0, 0);
                am = __builtin_amdgcn_mfma_f32_32x32x16_bf16(__builtin_bit_cast(bf16x8_t, l), xf[ks], am, 0, 0, 0);
            }
            if (SINGLE && k < a.nC) {
#pragma unroll
                for (int i = 0; i < 16; i++) {
                    const int d = (dt0 + m) * 32 + 8 * (i >> 2) + 4 * kg + (i & 3);
                    if (d < a.D) __builtin_nontemporal_store(am[i], out + (size_t)d * a.nC + k);
                }
            }
            park_a((m + 1) & 1);  // last read two tiles ago, before the previous barrier
            __syncthreads();
        };
        if constexpr (SINGLE) {
#pragma unroll 1
            for (int m = 0; dt0 + m < dt1; m++) do_tile(m, acc[0]);
        } else {
#pragma unroll
            for (int m = 0; m < TPW; m++)
                if (dt0 + m < dt1) do_tile(m, acc[m < NACC ? m : 0]);  // uniform
        }
    }
    if (!SINGLE && k < a.nC) {  // several sample blocks: tiles are complete only now
#pragma unroll
        for (int m = 0; m < NACC; m++) {
            if (dt0 + m < dt1) {
#pragma unroll
                for (int i = 0; i < 16; i++) {
                    const int d = (dt0 + m) * 32 + 8 * (i >> 2) + 4 * kg + (i & 3);
                    if (d < a.D) __builtin_nontemporal_store(acc[m][i], out + (size_t)d * a.nC + k);
                }
            }
        }
    }
}

// ---------------------------------------------------------------------------------------------
// dxflat[b, k] = sum_d dP[b, d] phi[d, k]: workgroup = 128 samples x 64 columns, so a column slab
// of phi is streamed exactly once per 128 samples.  The waves form a (4 / MT) x 2 grid (MT 32-sample
// tiles x 32 columns each).  phi arrives in chunks of 64 rows x 128 contiguous bytes (8 lanes per
// row), two chunks in flight per thread (register FIFO), is parked in a double-buffered LDS tile
// and read back transposed (the contraction runs over d, the strided axis); the dP operand comes
// fragment-major from global memory with fully coalesced 16-byte loads, prefetched with its chunk.
// The result leaves through LDS as 16-byte pieces of 128-byte rows.
// grid: (column slabs of 64, groups of 128 samples)
// ---------------------------------------------------------------------------------------------
constexpr int kDxfCW = 64;            // columns per workgroup
constexpr int kDxfLD = kDxfCW + 8;    // LDS row pitch (elements)
constexpr int kDxfDC = 64;            // phi rows per chunk
constexpr int kDxfLDF = kDxfCW + 4;   // LDS row pitch of the fp32 output tile of the completing form (elements)

// MT = 32-sample tiles per wave: 2 (four waves) or 1 (eight waves; one wave's MFMAs run under
// another's LDS reads on the same SIMD: 3 us faster at B=128 n=32 C=1280).
// FIN: the completing form (a.cx, a.dx_part, a.x set).
template <int MT, bool FIN>
__global__ __launch_bounds__(512 / MT) __attribute__((amdgpu_waves_per_eu(6))) void dxflat_wide_kernel(ProjBwdLargeArgs a) {
    constexpr int NTHR = 512 / MT;
    constexpr int PH = 512 / NTHR;       // 16-byte pieces of a phi chunk per thread (64 rows x 8)
    constexpr int PSTEP = NTHR / 8;      // rows covered by one round of the workgroup's loads
    extern __shared__ bf16_t pl_lds[];  // [2][kDxfDC][kDxfLD]; later the [128][kDxfLD] output tile
    const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
    const int wm = wave >> 1, wn = wave & 1;
    const int k0 = blockIdx.x * kDxfCW;
    const int sg = blockIdx.y;                 // group of 128 samples
    const int tiles_all = a.BP >> 5;
    const int nchunks = (a.DP + kDxfDC - 1) / kDxfDC;

    // phi piece of this thread: rows (tid >> 3) + PSTEP h of the chunk, 16-byte segment tid & 7.
    // Out-of-range rows / columns alias valid memory: rows in [D, DP) meet zero dP, rows >= DP are
    // never multiplied, columns >= nC are never stored.
    const int prow = tid >> 3, pseg = tid & 7;
    const int kc = k0 + pseg * 8 < a.nC ? k0 + pseg * 8 : 0;
    // dP fragments of this wave: sample tiles st0, st0 + 1 (clamped: surplus tiles are not stored)
    const int st0 = sg * 4 + wm * MT;
    const bf16_t *ap[MT];
#pragma unroll
    for (int m = 0; m < MT; m++)
        ap[m] = a.dPb + frag_base(min(st0 + m, tiles_all - 1), a.DP >> 4, 0) + lane * 8;

    // register FIFO of two chunks; a slot holds 2 phi pieces and 2 x 4 dP fragments
    // (RawVec keeps the loaded words as scalars: whole-uint4 copies of an array element can end up in
    // scratch memory, and a scratch store waits for the load it parks)
    struct Slot { RawVec<bf16_t, 8> p[PH]; uint4 f[4 * MT]; };
    auto issue = [&](Slot &sl, int c) {
#pragma unroll
        for (int h = 0; h < PH; h++) {
            const int d = c * kDxfDC + prow + PSTEP * h;
            sl.p[h].load(a.phi + (size_t)(d < a.D ? d : 0) * a.nC + kc);
        }
#pragma unroll
        for (int m = 0; m < MT; m++)
#pragma unroll
            for (int ks = 0; ks < 4; ks++) {
                const int d0 = c * kDxfDC + ks * 16;
                sl.f[m * 4 + ks] = *reinterpret_cast<const uint4 *>(ap[m] + (size_t)(d0 < a.DP ? d0 >> 4 : 0) * 512);
            }
    };
    f32x16_t o[MT];
#pragma unroll
    for (int m = 0; m < MT; m++)
#pragma unroll
        for (int i = 0; i < 16; i++) o[m][i] = 0.f;

    // park the slot's phi pieces in LDS buffer `par`, then multiply the chunk
    auto compute = [&](const Slot &sl, int par, int c) {
        bf16_t *buf = pl_lds + (size_t)par * kDxfDC * kDxfLD;
#pragma unroll
        for (int h = 0; h < PH; h++)
            *reinterpret_cast<uint4 *>(buf + (size_t)(prow + PSTEP * h) * kDxfLD + pseg * 8) =
                make_uint4(sl.p[h].w[0], sl.p[h].w[1], sl.p[h].w[2], sl.p[h].w[3]);
        __syncthreads();
        bf16x8_t pf[4];
#pragma unroll
        for (int ks = 0; ks < 4; ks++) {
            // B fragment: lane (col, kg) gets phi[chunk row ks*16 + kg*8 + i][wn*32 + col]
            pf[ks] = __builtin_bit_cast(bf16x8_t, lds_frag_tr(buf, kDxfLD, ks * 16, wn * 32, lane));
        }
#pragma unroll
        for (int ks = 0; ks < 4; ks++) {
            const bool live = c * kDxfDC + ks * 16 < a.DP;  // uniform; dead k-steps get a zero A operand
#pragma unroll
            for (int m = 0; m < MT; m++) {
                uint4 av = sl.f[m * 4 + ks];
                av.x = live ? av.x : 0u; av.y = live ? av.y : 0u; av.z = live ? av.z : 0u; av.w = live ? av.w : 0u;
                o[m] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(__builtin_bit_cast(bf16x8_t, av), pf[ks], o[m], 0, 0, 0);
            }
        }
    };

    // Completing dx (a.cx set): this thread's pieces of the partial dx (fp32, so that dx is rounded
    // once) and of x are requested behind the loop, in front of the last chunk's products when the
    // chunk count is odd, and arrive under those products and the accumulators' trip through LDS.  Pieces outside the tensor alias piece 0 and are not stored.
    constexpr int NP_OUT = 1024 / NTHR;
    constexpr bool finish = FIN;
    RawVec<float, 8> din[NP_OUT];
    RawVec<bf16_t, 8> xin[NP_OUT];
    float cxv[NP_OUT];
    // (tid_e: the thread index again, made opaque behind the loop, and everything the epilogue derives
    // from it: addresses formed there hold no registers across the loop, which runs at the register
    // count that keeps three workgroups on a CU)
    int tid_e = 0, prow_e = 0, pseg_e = 0;
    auto finish_off = [&](int h, bool &ok) {
        const int bo = sg * 128 + prow_e + PSTEP * h;
        ok = bo < a.B && k0 + pseg_e * 8 < a.nC;
        return ok ? (size_t)bo * a.nC + k0 + pseg_e * 8 : (size_t)0;
    };
    auto issue_finish_x = [&]() {  // 5 registers per piece: fits beside the last chunk's slot
        if constexpr (finish) {
#pragma unroll
            for (int h = 0; h < NP_OUT; h++) {
                bool ok;
                const size_t off = finish_off(h, ok);
                xin[h].load(a.x + off);
                cxv[h] = a.cx[ok ? sg * 128 + prow_e + PSTEP * h : 0];
            }
        }
    };
    auto issue_finish_part = [&]() {  // 8 registers per piece: once the FIFO is empty
        if constexpr (finish) {
#pragma unroll
            for (int h = 0; h < NP_OUT; h++) {
                bool ok;
                din[h].load(a.dx_part + finish_off(h, ok));
            }
        }
    };

    Slot s0, s1;
    issue(s0, 0);
    issue(s1, min(1, nchunks - 1));
    int c = 0;
    for (; c + 2 <= nchunks; c += 2) {
        compute(s0, 0, c);
        issue(s0, min(c + 2, nchunks - 1));
        compute(s1, 1, c + 1);
        issue(s1, min(c + 3, nchunks - 1));
    }
    if (c < nchunks) compute(s0, 0, c);
    tid_e = tid;
    asm volatile("" : "+v"(tid_e) :: "memory");
    prow_e = tid_e >> 3; pseg_e = tid_e & 7;
    const int lane_e = tid_e & 63, wave_e = tid_e >> 6;
    const int row_e = lane_e & 31, kg_e = lane_e >> 5, wm_e = wave_e >> 1, wn_e = wave_e & 1;
    issue_finish_x();  // the FIFO is empty: its registers take the pieces
    issue_finish_part();
    __syncthreads();  // all fragment reads done: the buffers become the output tile

    // accumulator layout: column = lane & 31, register i -> row 8*(i/4) + 4*(lane/32) + i%4.
    if constexpr (finish) {
        // the projection term stays fp32 until the one rounding of dx (the launch sizes the LDS for this tile)
        float *o_s = reinterpret_cast<float *>(pl_lds);  // [128][kDxfLDF]
#pragma unroll
        for (int m = 0; m < MT; m++)
#pragma unroll
            for (int i = 0; i < 16; i++)
                o_s[(size_t)((wm_e * MT + m) * 32 + 8 * (i >> 2) + 4 * kg_e + (i & 3)) * kDxfLDF + wn_e * 32 + row_e] = o[m][i];
        __syncthreads();
#pragma unroll
        for (int h = 0; h < NP_OUT; h++) {
            const int r = prow_e + PSTEP * h;
            const int bo = sg * 128 + r;
            if (bo < a.B && k0 + pseg_e * 8 < a.nC) {
                const float4 p0 = *reinterpret_cast<const float4 *>(o_s + (size_t)r * kDxfLDF + pseg_e * 8);
                const float4 p1 = *reinterpret_cast<const float4 *>(o_s + (size_t)r * kDxfLDF + pseg_e * 8 + 4);
                float pv[8] = {p0.x, p0.y, p0.z, p0.w, p1.x, p1.y, p1.z, p1.w}, dv[8], xv[8];
                din[h].get(dv); xin[h].get(xv);
#pragma unroll
                for (int v = 0; v < 8; v++) pv[v] = dv[v] + pv[v] - cxv[h] * xv[v];
                store_vec<bf16_t, 8, true>(a.dxflat + (size_t)bo * a.nC + k0 + pseg_e * 8, pv);
            }
            __builtin_amdgcn_sched_barrier(0);  // one piece after the other: interleaved they need more registers than the loop
        }
        return;
    }
    bf16_t *o_s = pl_lds;  // [128][kDxfLD]
#pragma unroll
    for (int m = 0; m < MT; m++)
#pragma unroll
        for (int i = 0; i < 16; i++)
            o_s[(size_t)((wm_e * MT + m) * 32 + 8 * (i >> 2) + 4 * kg_e + (i & 3)) * kDxfLD + wn_e * 32 + row_e] = f32_to_bf16(o[m][i]);
    __syncthreads();
#pragma unroll
    for (int h = 0; h < NP_OUT; h++) {
        const int r = prow_e + PSTEP * h;
        const int bo = sg * 128 + r;
        if (bo < a.B && k0 + pseg_e * 8 < a.nC)
            *reinterpret_cast<uint4 *>(a.dxflat + (size_t)bo * a.nC + k0 + pseg_e * 8) =
                *reinterpret_cast<const uint4 *>(o_s + (size_t)r * kDxfLD + pseg_e * 8);
    }
}

bool proj_bwd_is_wide(int n) { return padded_D(n) / 32 > 12; }

// x, cx, dx_part: all nullptr, or the inputs of the completion dxflat = dx_part + dP phi - cx x
// (dx_part fp32 [B][nC]).
hipError_t launch_dxflat_wide(const void *phi, const void *dPb, int BP, void *dxflat, const void *x, const float *cx,
                              const float *dx_part, int B, int n, int C, hipStream_t stream) {
    const int nC = n * C, D = n * n + 2 * n, DP = padded_D(n);
    if ((x == nullptr) != (cx == nullptr) || (x == nullptr) != (dx_part == nullptr)) return hipErrorInvalidValue;
    ProjBwdLargeArgs a{static_cast<const bf16_t *>(x), static_cast<const bf16_t *>(phi), static_cast<const bf16_t *>(dPb), nullptr,
                       nullptr, static_cast<bf16_t *>(dxflat), B, BP, D, DP, nC, B, 0, -1, {}, cx, dx_part};
    // eight waves: 3 us faster than four at B=128 n=32 C=1280
    const size_t lds = cx ? sizeof(float) * 128 * kDxfLDF : sizeof(bf16_t) * 128 * kDxfLD;
    const dim3 grid((nC + kDxfCW - 1) / kDxfCW, (B + 127) / 128);
    if (cx) dxflat_wide_kernel<1, true><<<grid, 512, lds, stream>>>(a);
    else dxflat_wide_kernel<1, false><<<grid, 512, lds, stream>>>(a);
    return hipGetLastError();
}

hipError_t launch_dphi_large(const void *x, const void *dPT, int BP, float *dphi_out, int S, int B, int n,
                             int C, const BatchSumArgs *tail, bool *tail_taken, hipStream_t stream) {
    const int nC = n * C, D = n * n + 2 * n, DP = padded_D(n);
    const int nblocks = (B + kPL_SB - 1) / kPL_SB;
    const int bps = (nblocks + S - 1) / S * kPL_SB;
    ProjBwdLargeArgs a{static_cast<const bf16_t *>(x), nullptr, nullptr, static_cast<const bf16_t *>(dPT),
                       dphi_out, nullptr, B, BP, D, DP, nC, bps, 9, -1, {}};
    const int slabs = (nC + kPL_KW - 1) / kPL_KW;
    const int NTD = DP / 32;
    // the batch sums ride along as one extra row of the grid when that row is long enough for them
    const bool with_tail = tail && tail->nblk <= slabs;
    if (tail_taken) *tail_taken = with_tail;
    if (with_tail) a.tail = *tail;
    const int extra = with_tail ? tail->nblk : 0;
    hipError_t e;
    // the x block, later two operand tiles of 16 KB in the same memory
    const size_t smem = sizeof(bf16_t) * (kPL_SB * kPL_LD > 2 * 2 * 4096 ? kPL_SB * kPL_LD : 2 * 2 * 4096);
    if (bps <= kPL_SB) {
        // one sample block per split: row tiles are stored as they complete.  Tiles per workgroup:
        // the fewest (9, 12, 17, all) with which the grid fits the chip's resident workgroups at once
        // (4 per CU): 1280 workgroups on 1024 slots would run as two rounds, the second a quarter full.
        const int slots = 256 * 4;
        int tpw = NTD;
        for (int cand : {9, 12, 17})
            if (cand < NTD && (long long)slabs * ((NTD + cand - 1) / cand) * S + extra <= slots) { tpw = cand; break; }
        if ((long long)slabs * S > slots) tpw = NTD < 9 ? NTD : 9;  // more than one round anyway
        a.tpw = tpw;
        const int ytiles = (NTD + tpw - 1) / tpw;
        if (with_tail) a.tail_row = ytiles;
        e = allow_dynamic_lds(&dphi_large_kernel<9, true>, smem);
        if (e != hipSuccess) return e;
        dphi_large_kernel<9, true><<<dim3(slabs, ytiles + (with_tail ? 1 : 0), S), 256, smem, stream>>>(a);
    } else {
        const int ytiles = (NTD + 2) / 3;
        if (with_tail) a.tail_row = ytiles;
        e = allow_dynamic_lds(&dphi_large_kernel<3, false>, smem);
        if (e != hipSuccess) return e;
        dphi_large_kernel<3, false><<<dim3(slabs, ytiles + (with_tail ? 1 : 0), S), 256, smem, stream>>>(a);
    }
    return hipGetLastError();
}

}  // namespace mhc
