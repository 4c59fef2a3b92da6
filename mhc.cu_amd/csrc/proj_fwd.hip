// Projection of the dynamic-H path: raw dot products x_flat[b,:] . phi[d,:] for all D = n^2+2n
// rows of phi, plus sum(x_flat^2), as split-K partial sums.  The coefficient kernel finishes
// the reduction, divides by the RMS and applies alpha / bias / activations.
//
// Replaces compute_rms (reference src/csrc/kernels/fused_rmsnorm_matmul.cuh:119-153) and the
// cuBLASLt projection GEMM (src/python/bindings.cu:34-81, :436-443) with one pass over x.
//
// Two kernels:
//   proj_fwd_mfma_kernel    x and phi both bf16, C % 8 == 0: v_mfma_f32_32x32x16_bf16 tiles
//                           (32 samples x 32 projection rows), operands fetched row-contiguously
//                           through a wave-private LDS tile.
//   proj_fwd_generic_kernel any dtype / any C: fp32 FMA, exact products (the fp32 parity tier).
#include "launchers.h"

#include <type_traits>
#include "mhc_common.h"
#include "phase_profiler.h"
#include "tuning.h"

namespace mhc {

typedef __attribute__((__vector_size__(8 * sizeof(__bf16)))) __bf16 bf16x8_t;
typedef __attribute__((__vector_size__(16 * sizeof(float)))) float f32x16_t;

static inline bool use_mfma(int x_dtype, int phi_dtype, int C) {
    return (x_dtype == kBF16 || x_dtype == kF32AsBF16) && phi_dtype == kBF16 && C % 8 == 0;
}

// --------------------------------------------------------------------------------------------
// generic path
// --------------------------------------------------------------------------------------------
constexpr int kGenDB = 16;  // projection rows per workgroup

template <typename TX, typename TP>
__global__ __launch_bounds__(256) void proj_fwd_generic_kernel(const TX *__restrict__ x,
                                                               const TP *__restrict__ phi,
                                                               float *__restrict__ Ppart,
                                                               float *__restrict__ ssqpart, int B,
                                                               int D, int DP, int nC) {
    __shared__ float red[4][kGenDB + 1];
    const int b = blockIdx.x, d0 = blockIdx.y * kGenDB, tid = threadIdx.x;
    const TX *xb = x + (size_t)b * nC;
    float acc[kGenDB], ssq = 0.f;
#pragma unroll
    for (int j = 0; j < kGenDB; j++) acc[j] = 0.f;
    for (int k = tid; k < nC; k += 256) {
        const float xv = to_f32<TX>(xb[k]);
        ssq += xv * xv;
#pragma unroll
        for (int j = 0; j < kGenDB; j++)
            if (d0 + j < D) acc[j] += xv * to_f32<TP>(phi[(size_t)(d0 + j) * nC + k]);
    }
#pragma unroll
    for (int j = 0; j < kGenDB; j++) acc[j] = wave_allreduce_sum(acc[j]);
    ssq = wave_allreduce_sum(ssq);
    if ((tid & 63) == 0) {
#pragma unroll
        for (int j = 0; j < kGenDB; j++) red[tid >> 6][j] = acc[j];
        red[tid >> 6][kGenDB] = ssq;
    }
    __syncthreads();
    if (tid <= kGenDB) {
        const float v = (red[0][tid] + red[1][tid]) + (red[2][tid] + red[3][tid]);
        if (tid < kGenDB) {
            if (d0 + tid < D) Ppart[(size_t)b * DP + d0 + tid] = v;
        } else if (blockIdx.y == 0) {
            ssqpart[b] = v;
        }
    }
}

// --------------------------------------------------------------------------------------------
// MFMA path.  Workgroup = 4 waves on the same 32-sample tile, each wave on its own K sub-slab;
// the four partial tiles are summed through LDS, so one partial per workgroup reaches memory.
// grid.x = sample_tiles * round_up(KS, 8), grid.y = groups of NT projection tiles.  Workgroup ids
// go round robin over the 8 XCDs, each with its own L2: the K slab is chosen by id % 8 (plus 8 per
// full set of sample tiles), so that all sample tiles of a slab run on one XCD and the slab of phi
// is fetched from memory once instead of once per XCD.  Ids whose slab is beyond KS do nothing.
// --------------------------------------------------------------------------------------------
typedef __attribute__((__vector_size__(2 * sizeof(__bf16)))) __bf16 bf16x2_t;
constexpr int kNarrowPitch = 72;  // LDS row of a 64-element chunk: 128 data bytes + 16 pad (bf16 elements)

// XF32: x is stored as fp32 and rounded to bf16 (nearest even) on its way into the LDS tile; everything
// behind the tile, the sum of squares included, sees the rounded values.
template <int NT, bool XF32 = false>
__global__ __launch_bounds__(256) void proj_fwd_mfma_kernel(const void *__restrict__ x_,
                                                            const bf16_t *__restrict__ phi,
                                                            float *__restrict__ Ppart,
                                                            float *__restrict__ ssqpart, int B,
                                                            int D, int DP, int nC, int tiles_s, int KS,
                                                            int sub /* K per wave, multiple of 64 */) {
    extern __shared__ __align__(16) float lds[];  // per wave [(1 + NT) * 32][pitch] bf16; later [4][NT*16 + 1][64] fp32
    using TXS = typename std::conditional<XF32, float, bf16_t>::type;  // storage type of x
    const TXS *__restrict__ x = static_cast<const TXS *>(x_);
    const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
    const int set = (blockIdx.x >> 3) / tiles_s;
    const int st = (blockIdx.x >> 3) % tiles_s, ks = (blockIdx.x & 7) + 8 * set;
    if (ks >= KS) return;  // the whole workgroup, before any barrier
    const int pwg = blockIdx.y * gridDim.x + blockIdx.x;
    (void)pwg;
    MHC_PHASE_ZERO(kPhaseProjFwd, pwg);
    MHC_PHASE_BEGIN(pclk);
    const int row = lane & 31, kh = lane >> 5;
    const int b = st * 32 + row;
    const int dbase = blockIdx.y * NT * 32;
    const int kbeg = (ks * 4 + wave) * sub;
    const int kend = min(kbeg + sub, nC);
    const bool bvalid = b < B;

    // Global loads are row-contiguous (8 lanes per 128-byte row piece, rows lr + 8 j): the operand
    // layout of the matrix cores has every lane on a different row, which the memory pipeline
    // serves at a quarter of this rate.  The chunk goes through a wave-private LDS tile and comes
    // back as fragments; no barrier is involved (a wave's LDS accesses complete in order).
    bf16_t *cb = reinterpret_cast<bf16_t *>(lds) + (size_t)wave * (1 + NT) * 32 * kNarrowPitch;
    const int lr = lane >> 3, seg = lane & 7;
    const TXS *xrow[4];
    const bf16_t *prow[NT][4];
    bool xval[4], pval[NT][4];
#pragma unroll
    for (int j = 0; j < 4; j++) {
        const int bs = st * 32 + lr + 8 * j;
        xval[j] = bs < B;
        xrow[j] = x + (size_t)(xval[j] ? bs : 0) * nC;
#pragma unroll
        for (int t = 0; t < NT; t++) {
            const int d = dbase + t * 32 + lr + 8 * j;
            pval[t][j] = d < D;
            prow[t][j] = phi + (size_t)(pval[t][j] ? d : 0) * nC;
        }
    }
    constexpr int XW = XF32 ? 8 : 4;  // words of a lane's 8 elements of x as loaded
    uint32_t xq[4][XW], pq[NT][4][4];  // scalar words: whole-uint4 array elements can end up in scratch
    auto load_x8 = [&](const TXS *p, uint32_t (&q)[XW], bool ok) {
        const uint4 v = load16_masked(reinterpret_cast<const uint4 *>(p), ok);
        q[0] = v.x; q[1] = v.y; q[2] = v.z; q[3] = v.w;
        if constexpr (XF32) {
            const uint4 v2 = load16_masked(reinterpret_cast<const uint4 *>(p) + 1, ok);
            q[4] = v2.x; q[5] = v2.y; q[6] = v2.z; q[7] = v2.w;
        }
    };
    // Rows beyond B (x) or D (phi) alias row 0: what they produce is finite and is either not stored
    // (samples >= B) or zeroed at the store (projection rows >= D), so only the K tail of the last
    // slab needs a mask - a uniform test per chunk instead of four selects per load (the kernel is
    // bound by VALU issue, not by memory, with four waves per SIMD).
    auto fetch = [&](int k0) {
        const int k = k0 + seg * 8;
        if (k0 + 64 <= kend) {
#pragma unroll
            for (int j = 0; j < 4; j++) {
                if constexpr (XF32) {
                    load_x8(xrow[j] + k, xq[j], true);
                } else {
                    const uint4 v = *reinterpret_cast<const uint4 *>(xrow[j] + k);
                    xq[j][0] = v.x; xq[j][1] = v.y; xq[j][2] = v.z; xq[j][3] = v.w;
                }
#pragma unroll
                for (int t = 0; t < NT; t++) {
                    const uint4 p = *reinterpret_cast<const uint4 *>(prow[t][j] + k);
                    pq[t][j][0] = p.x; pq[t][j][1] = p.y; pq[t][j][2] = p.z; pq[t][j][3] = p.w;
                }
            }
            return;
        }
        const bool kv = k < kend;  // kend and k are multiples of 8
        const int off = kv ? k : 0;
#pragma unroll
        for (int j = 0; j < 4; j++) {
            load_x8(xrow[j] + off, xq[j], kv);
#pragma unroll
            for (int t = 0; t < NT; t++) {
                const uint4 p = load16_masked(reinterpret_cast<const uint4 *>(prow[t][j] + off), kv);
                pq[t][j][0] = p.x; pq[t][j][1] = p.y; pq[t][j][2] = p.z; pq[t][j][3] = p.w;
            }
        }
    };
    auto park = [&]() {
#pragma unroll
        for (int j = 0; j < 4; j++) {
            if constexpr (XF32)
                *reinterpret_cast<uint4 *>(cb + (size_t)(lr + 8 * j) * kNarrowPitch + seg * 8) =
                    make_uint4(pack_bf16x2(__uint_as_float(xq[j][0]), __uint_as_float(xq[j][1])),
                               pack_bf16x2(__uint_as_float(xq[j][2]), __uint_as_float(xq[j][3])),
                               pack_bf16x2(__uint_as_float(xq[j][4]), __uint_as_float(xq[j][5])),
                               pack_bf16x2(__uint_as_float(xq[j][6]), __uint_as_float(xq[j][7])));
            else
            *reinterpret_cast<uint4 *>(cb + (size_t)(lr + 8 * j) * kNarrowPitch + seg * 8) =
                make_uint4(xq[j][0], xq[j][1], xq[j][2], xq[j][3]);
#pragma unroll
            for (int t = 0; t < NT; t++)
                *reinterpret_cast<uint4 *>(cb + (size_t)(32 + t * 32 + lr + 8 * j) * kNarrowPitch + seg * 8) =
                    make_uint4(pq[t][j][0], pq[t][j][1], pq[t][j][2], pq[t][j][3]);
        }
    };

    f32x16_t acc[NT];
#pragma unroll
    for (int t = 0; t < NT; t++)
#pragma unroll
        for (int i = 0; i < 16; i++) acc[t][i] = 0.f;
    float ssq = 0.f;

    if (kbeg < kend) fetch(kbeg);
    MHC_PHASE_ADD(kPhaseProjFwd, pwg, 0, pclk);
    for (int k0 = kbeg; k0 < kend; k0 += 64) {
        park();
        // (a wave's LDS accesses complete in order; the fence keeps the compiler from moving the
        // fragment reads above the writes of its own tile)
        __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront");
        __builtin_amdgcn_wave_barrier();
        MHC_PHASE_ADD(kPhaseProjFwd, pwg, 1, pclk);
        if (k0 + 64 < kend) fetch(k0 + 64);  // in flight while this chunk is multiplied
#pragma unroll
        for (int u = 0; u < 4; u++) {
            // fragment of k-step u: lane (row, kh) holds elements u*16 + kh*8 .. +8 of its row
            const uint4 av = *reinterpret_cast<const uint4 *>(cb + (size_t)row * kNarrowPitch + u * 16 + kh * 8);
            const bf16x8_t af = __builtin_bit_cast(bf16x8_t, av);
#pragma unroll
            for (int t = 0; t < NT; t++) {
                const uint4 bv = *reinterpret_cast<const uint4 *>(cb + (size_t)(32 + t * 32 + row) * kNarrowPitch + u * 16 + kh * 8);
                acc[t] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(af, __builtin_bit_cast(bf16x8_t, bv), acc[t], 0, 0, 0);
            }
            if (blockIdx.y == 0) {  // sum of squares: v_dot2c_f32_bf16, two elements per instruction
                const uint32_t w4[4] = {av.x, av.y, av.z, av.w};
#pragma unroll
                for (int i = 0; i < 4; i++) {
                    const bf16x2_t pr = __builtin_bit_cast(bf16x2_t, w4[i]);
                    ssq = __builtin_amdgcn_fdot2_f32_bf16(pr, pr, ssq, false);
                }
            }
        }
        MHC_PHASE_ADD(kPhaseProjFwd, pwg, 2, pclk);
    }
    __syncthreads();  // every wave is done with its chunk tile: the memory becomes the cross-wave buffer
    ssq = xor32_add(ssq);  // both K halves of the row

    // cross-wave sum: every wave parks its tiles in LDS, then wave w adds and writes accumulator
    // registers 4w .. 4w+3 of every tile (rows 8w + 4 kh .. +3 of the 32 x 32 tile), wave 0 also x^2
    constexpr int R = NT * 16 + 1;
    {
        float *dst = lds + (size_t)wave * R * 64;
#pragma unroll
        for (int t = 0; t < NT; t++)
#pragma unroll
            for (int i = 0; i < 16; i++) dst[(t * 16 + i) * 64 + lane] = acc[t][i];
        dst[(R - 1) * 64 + lane] = ssq;
    }
    __syncthreads();
    // accumulator layout of the 32x32 tile: lane -> column (lane & 31),
    // register i -> row 8 * (i / 4) + 4 * (lane / 32) + (i % 4)
    float *out = Ppart + (size_t)ks * B * DP;
#pragma unroll
    for (int t = 0; t < NT; t++) {
        const int d = dbase + t * 32 + row;
#pragma unroll
        for (int q = 0; q < 4; q++) {
            const int i = 4 * wave + q;
            float v = 0.f;
#pragma unroll
            for (int w = 0; w < 4; w++) v += lds[((size_t)w * R + t * 16 + i) * 64 + lane];
            const int bs = st * 32 + 8 * wave + 4 * kh + q;
            if (bs < B && d < DP) out[(size_t)bs * DP + d] = d < D ? v : 0.f;  // padded rows stay zero
        }
    }
    if (wave == 0 && blockIdx.y == 0 && kh == 0 && bvalid) {
        float v = 0.f;
#pragma unroll
        for (int w = 0; w < 4; w++) v += lds[((size_t)w * R + R - 1) * 64 + lane];
        ssqpart[(size_t)ks * B + b] = v;
    }
    MHC_PHASE_ADD(kPhaseProjFwd, pwg, 3, pclk);
}

// --------------------------------------------------------------------------------------------
// MFMA path for wide projections (phi is the big operand, n > 8).
//
// Loads where every lane addresses a different row (the MFMA operand layout) are served at a
// fraction of the L1 rate, so here both operands are fetched with row-contiguous loads (8 lanes
// per 128-byte line), parked in LDS and read back in MFMA layout.
//   workgroup tile: 128 samples x (NT * 64) projection rows, K chunks of 64 elements
//   NWM x NWN waves: a wave owns 128 / NWM samples x NT*32 rows.  Eight waves (4 x 2, one 32 x 32
//   accumulator tile each at NT = 1) are 12 % faster than four with two tiles each (sixteen waves on
//   a 128 x 128 tile gain another 3 % at D = 1088 with exactly 24 K slabs and lose with any other
//   count; not taken): the kernel is
//   bound by its own pipeline (global loads, LDS parking, LDS reads and MFMAs take turns behind one
//   barrier per chunk), and two waves per SIMD let one wave's MFMAs run under the other's LDS reads.
//   P chunks of global loads are in flight per thread (register FIFO) ahead of the chunk being
//   multiplied; LDS is double-buffered, one barrier per chunk.
// Workgroups that read the same K slab sit on the same XCD (workgroup id modulo 8 selects the
// XCD, every XCD takes the same number of consecutive work items): the slab of x is pulled into that
// L2 once and the other row groups hit it there.
// grid.x = groups * sample_groups * KS rounded up to a multiple of 8
// --------------------------------------------------------------------------------------------
constexpr int kWideLd = 72;  // LDS row stride in bf16 elements: 128 data bytes + 16 pad

template <int NT, int P, int NWM = 2, int NWN = 2>
__global__ __launch_bounds__(64 * NWM * NWN) void proj_fwd_wide_kernel(const bf16_t *__restrict__ x,
                                                            const bf16_t *__restrict__ phi,
                                                            float *__restrict__ Ppart,
                                                            float *__restrict__ ssqpart, int B,
                                                            int D, int DP, int nC, int groups,
                                                            int sgroups, int KS,
                                                            int cpk /* chunks per K slab */) {
    static_assert(P % 2 == 0, "buffer parity is tied to the FIFO slot");
    constexpr int R = NT * 32 * NWN;   // projection rows per workgroup
    constexpr int NTHR = 64 * NWM * NWN;     // NWM x NWN waves: a wave owns 128 / NWM samples x NT*32 rows
    constexpr int MT = 4 / NWM;              // 32-sample tiles per wave
    constexpr int XJ = 128 * 8 / NTHR;       // 16-byte segments of the x tile per thread
    constexpr int PJ = R * 8 / NTHR;         // same for the phi tile
    constexpr int RSTEP = NTHR / 8;          // rows covered by one round of the workgroup's loads
    extern __shared__ __align__(16) bf16_t lds_w[];  // [2][128 + R][kWideLd]
    const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
    const int row = lane & 31, kh = lane >> 5;
    const int wm = wave / NWN, wn = wave % NWN;
    // work item = (K slab, sample group, row group), rows fastest.  Workgroup ids go round the 8 XCDs,
    // so XCD j takes the contiguous items [j * per_xcd, (j + 1) * per_xcd): the same number on every
    // XCD, and the items that share a slab of x sit on one XCD (two where a slab straddles the border).
    const int items = groups * sgroups * KS, per_xcd = (items + 7) >> 3;
    const int item = (blockIdx.x & 7) * per_xcd + (blockIdx.x >> 3);
    if ((int)(blockIdx.x >> 3) >= per_xcd || item >= items) return;  // whole workgroup, before any barrier
    const int group = item % groups;
    const int sg = (item / groups) % sgroups;
    const int ks = item / (groups * sgroups);
    const int nch_all = (nC + 63) / 64;
    const int cbeg = ks * cpk, cend = min(cbeg + cpk, nch_all);
    const bool want_ssq = group == 0;

    // global -> register stage: thread owns segment `seg` of rows lrow + 32 j
    const int lrow = tid >> 3, seg = tid & 7;
    const uint4 *xg[XJ], *pg[PJ];
    bool xv[XJ], pv[PJ];
#pragma unroll
    for (int j = 0; j < XJ; j++) {
        const int b = sg * 128 + lrow + RSTEP * j;
        xv[j] = b < B;
        xg[j] = reinterpret_cast<const uint4 *>(x + (size_t)(xv[j] ? b : 0) * nC) + seg;
    }
#pragma unroll
    for (int j = 0; j < PJ; j++) {
        const int d = group * R + lrow + RSTEP * j;
        pv[j] = d < D;
        pg[j] = reinterpret_cast<const uint4 *>(phi + (size_t)(pv[j] ? d : 0) * nC) + seg;
    }
    // No per-lane predicate on the loads: rows beyond B / D alias row 0 (their products are never
    // stored) and nC % 64 == 0, so a loaded value is not touched until it is parked in LDS and
    // the loads of all P slots stay in flight.
    uint4 rg[P][XJ + PJ];  // per slot: XJ segments of x, then PJ of phi
    auto issue = [&](int slot_, int c) {
#pragma unroll
        for (int j = 0; j < PJ; j++) rg[slot_][XJ + j] = pg[j][c * 8];
#pragma unroll
        for (int j = 0; j < XJ; j++) rg[slot_][j] = xg[j][c * 8];
    };

    f32x16_t acc[MT][NT];
#pragma unroll
    for (int m = 0; m < MT; m++)
#pragma unroll
        for (int t = 0; t < NT; t++)
#pragma unroll
            for (int i = 0; i < 16; i++) acc[m][t][i] = 0.f;
    float ssq[XJ];
#pragma unroll
    for (int j = 0; j < XJ; j++) ssq[j] = 0.f;

    // park slot j in LDS buffer j & 1, then multiply that buffer; with prefetch, `next` is the
    // chunk whose loads refill the slot
    auto step = [&](int j, int next, auto prefetch) {
        bf16_t *xs = lds_w + (size_t)(j & 1) * (128 + R) * kWideLd;
        bf16_t *ps = xs + 128 * kWideLd;
#pragma unroll
        for (int q = 0; q < XJ; q++)
            *reinterpret_cast<uint4 *>(xs + (lrow + RSTEP * q) * kWideLd + seg * 8) = rg[j][q];
#pragma unroll
        for (int q = 0; q < PJ; q++)
            *reinterpret_cast<uint4 *>(ps + (lrow + RSTEP * q) * kWideLd + seg * 8) = rg[j][XJ + q];
        if (want_ssq) {
#pragma unroll
            for (int q = 0; q < XJ; q++) {
                const uint32_t w4[4] = {rg[j][q].x, rg[j][q].y, rg[j][q].z, rg[j][q].w};
#pragma unroll
                for (int i = 0; i < 4; i++) {
                    const float lo = bf16lo_to_f32(w4[i]), hi = bf16hi_to_f32(w4[i]);
                    ssq[q] += lo * lo + hi * hi;
                }
            }
        }
        __syncthreads();
        if constexpr (decltype(prefetch)::value) issue(j, next);
#pragma unroll
        for (int s = 0; s < 4; s++) {
            bf16x8_t af[MT], bfr[NT];
#pragma unroll
            for (int m = 0; m < MT; m++)
                af[m] = *reinterpret_cast<const bf16x8_t *>(
                    xs + (wm * 32 * MT + m * 32 + row) * kWideLd + s * 16 + kh * 8);
#pragma unroll
            for (int t = 0; t < NT; t++)
                bfr[t] = *reinterpret_cast<const bf16x8_t *>(
                    ps + (wn * NT * 32 + t * 32 + row) * kWideLd + s * 16 + kh * 8);
#pragma unroll
            for (int m = 0; m < MT; m++)
#pragma unroll
                for (int t = 0; t < NT; t++)
                    acc[m][t] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(af[m], bfr[t], acc[m][t], 0, 0, 0);
        }
    };

    // prologue: fill the FIFO (indices beyond the slab are clamped: redundant, never consumed)
#pragma unroll
    for (int j = 0; j < P; j++) issue(j, min(cbeg + j, cend - 1));
    int c = cbeg;
    for (; c + P <= cend; c += P) {
#pragma unroll
        for (int j = 0; j < P; j++) step(j, min(c + j + P, cend - 1), std::true_type{});
    }
    const int rem = cend - c;  // < P chunks left, all already in flight
#pragma unroll
    for (int j = 0; j < P - 1; j++)
        if (j < rem) step(j, 0, std::false_type{});

    // accumulator layout of a 32x32 tile: lane -> column (lane & 31),
    // register i -> row 8 * (i / 4) + 4 * (lane / 32) + (i % 4)
    float *out = Ppart + (size_t)ks * B * DP;
#pragma unroll
    for (int m = 0; m < MT; m++)
#pragma unroll
        for (int t = 0; t < NT; t++) {
            const int d = group * R + wn * NT * 32 + t * 32 + row;
#pragma unroll
            for (int i = 0; i < 16; i++) {
                const int bs = sg * 128 + wm * 32 * MT + m * 32 + 8 * (i >> 2) + 4 * kh + (i & 3);
                if (bs < B && d < D) out[(size_t)bs * DP + d] = acc[m][t][i];
            }
        }
    if (want_ssq) {
#pragma unroll
        for (int j = 0; j < XJ; j++) {
            float v = ssq[j];  // the 8 lanes of one row are consecutive
            v += __shfl_xor(v, 1, kWave);
            v += __shfl_xor(v, 2, kWave);
            v += __shfl_xor(v, 4, kWave);
            if (seg == 0 && xv[j]) ssqpart[(size_t)ks * B + sg * 128 + lrow + RSTEP * j] = v;
        }
    }
}

template <int NT, int P, int NWM = 2, int NWN = 2>
static hipError_t launch_wide(const void *x, const void *phi, float *Ppart, float *ssqpart, int KS,
                              int B, int D, int DP, int nC, hipStream_t stream) {
    const int sgroups = (B + 127) / 128;
    constexpr int R = NT * 32 * NWN;
    const int groups = (DP + R - 1) / R;
    const int nch_all = (nC + 63) / 64;
    const int cpk = (nch_all + KS - 1) / KS;
    const int grid = 8 * ((groups * sgroups * KS + 7) / 8);
    const size_t smem = sizeof(bf16_t) * 2 * (128 + R) * kWideLd;
    if (smem > 64 * 1024) {  // above the default dynamic-LDS limit (the CU has 160 KB)
        hipError_t e = hipFuncSetAttribute(reinterpret_cast<const void *>(&proj_fwd_wide_kernel<NT, P, NWM, NWN>),
                                           hipFuncAttributeMaxDynamicSharedMemorySize, (int)smem);
        if (e != hipSuccess) return e;
    }
    proj_fwd_wide_kernel<NT, P, NWM, NWN><<<grid, 64 * NWM * NWN, smem, stream>>>(
        static_cast<const bf16_t *>(x), static_cast<const bf16_t *>(phi), Ppart, ssqpart, B, D, DP,
        nC, groups, sgroups, KS, cpk);
    return hipGetLastError();
}

// --------------------------------------------------------------------------------------------
// shape-dependent split and launch
// --------------------------------------------------------------------------------------------
static int mfma_nt(int n) {
    const int tiles = padded_D(n) / 32;
    return tiles <= 4 ? tiles : 2;
}

// wide projections (more than four 32-row tiles) with whole 64-element K chunks take the
// LDS-staged kernel
static bool use_wide(int n, int C) { return padded_D(n) / 32 > 4 && (n * C) % 64 == 0; }

int proj_fwd_ksplit(int x_dtype, int phi_dtype, int B, int n, int C) {
    // The generic path always uses one split.  MFMA path: enough workgroups to fill 256 CUs
    // several times over (the K loop is latency-bound per wave), at least 64 K elements per wave.
    if (gemm_f32_supported(x_dtype, phi_dtype, n, C)) return gemm_f32_proj_ksplit(B, n, C, kMaxKSplit);
    if (!use_mfma(x_dtype, phi_dtype, C)) return 1;
    const int nC = n * C, DP = padded_D(n);
    if (use_wide(n, C)) {
        // Workgroups = (64-row groups) x (128-sample tiles) x splits.  The chip has 256 CUs and a workgroup
        // (8 waves) loads one: the count that fills every CU once, or twice where that still keeps the
        // splits within the 24 that the coefficient kernel sums in one round of loads, beats the counts in
        // between, which leave some CUs with twice the work of others
        // (forward us, B n C: 128 32 1280  15 splits 41.8 | 24: 43.0 | 30: 44.2 | 16: 48.7;
        //  256 32 1280  15: 62.1 | 12: 66.2 | 7: 67.5;  512 12 512  16: 28.1 | 3: 35.8).
        const int wgs = ((DP + 63) / 64) * ((B + 127) / 128);
        int ks = 512 / wgs <= 24 ? 512 / wgs : 256 / wgs;
        if (ks > 24) ks = 24;
        const int cap_chunks = nC / 64 / 8;  // a slab is at least 8 chunks
        if (ks > cap_chunks) ks = cap_chunks;
        // the partial sums (written here, read by the coefficient kernel) stay below the bytes streamed,
        // unless that would leave half the CUs without a workgroup
        const int cap_bytes = (int)((2.0 * B * nC + 2.0 * DP * nC) / (8.0 * B * DP));
        if (ks > cap_bytes) {
            const int half_chip = (128 + wgs - 1) / wgs;
            ks = cap_bytes > (ks < half_chip ? ks : half_chip) ? cap_bytes : (ks < half_chip ? ks : half_chip);
        }
        if (ks < 1) ks = 1;
        if (const int forced = tuning_get(kTuneSpareB); forced > 0) ks = forced;  // experiment hook
        return ks;
    }
    const int tiles_s = (B + 31) / 32;
    const int groups = DP / 32 / mfma_nt(n);
    int ks = (1024 + tiles_s * groups - 1) / (tiles_s * groups);
    const int cap_slab = nC / 256;
    // partial sums (KS * B * DP fp32) at most ~1/3 of the bytes this kernel streams (x and phi)
    const int cap_bytes = (int)(0.35 * (2.0 * B * nC + 2.0 * DP * nC) / (4.0 * B * DP));
    if (ks > cap_slab) ks = cap_slab;
    if (ks > cap_bytes) ks = cap_bytes;
    // the fused forward kernel (n <= 8) sums up to 24 splits (16 when a thread holds two chunks of
    // the sample, C > 2048) with loads that it issues ahead of the sample's tile; more splits would
    // queue behind the tile
    const int fused_cap = C <= 2048 ? 24 : 16;
    if (n <= 8 && ks > fused_cap) ks = fused_cap;
    if (ks > 64) ks = 64;
    if (ks < 1) ks = 1;
    if (const int forced = tuning_get(kTuneSpareB); forced > 0) ks = forced;  // experiment hook
    // a wave's share is whole 64-element chunks (launch_mfma): with that share fixed, only as many
    // splits as have work (B=1280 n=4 C=2560: 16 splits of 4 x 192 elements would leave the last two
    // and a half empty; 14 do the same work and the forward sums two partial rows fewer per sample)
    const int sub = round_up((nC + ks * 4 - 1) / (ks * 4), 64);
    ks = (nC + 4 * sub - 1) / (4 * sub);
    return ks;
}

template <typename TX, typename TP>
static hipError_t launch_generic(const void *x, const void *phi, float *Ppart, float *ssqpart, int B,
                                 int D, int DP, int nC, hipStream_t stream) {
    dim3 grid(B, (D + kGenDB - 1) / kGenDB);
    proj_fwd_generic_kernel<TX, TP><<<grid, 256, 0, stream>>>(
        static_cast<const TX *>(x), static_cast<const TP *>(phi), Ppart, ssqpart, B, D, DP, nC);
    return hipGetLastError();
}

template <int NT, bool XF32 = false>
static hipError_t launch_mfma(const void *x, const void *phi, float *Ppart, float *ssqpart, int KS,
                              int B, int D, int DP, int nC, hipStream_t stream) {
    const int tiles_s = (B + 31) / 32;
    const int groups = (DP / 32 + NT - 1) / NT;
    const int sub = round_up((nC + KS * 4 - 1) / (KS * 4), 64);  // whole 128-byte lines per lane pair
    dim3 grid(tiles_s * round_up(KS, 8), groups);
    const size_t smem_chunks = sizeof(bf16_t) * 4 * (1 + NT) * 32 * kNarrowPitch;
    const size_t smem_sum = sizeof(float) * 4 * (NT * 16 + 1) * 64;
    const size_t smem = smem_chunks > smem_sum ? smem_chunks : smem_sum;
    if (hipError_t e = allow_dynamic_lds(&proj_fwd_mfma_kernel<NT, XF32>, smem); e != hipSuccess) return e;
    proj_fwd_mfma_kernel<NT, XF32><<<grid, 256, smem, stream>>>(x, static_cast<const bf16_t *>(phi), Ppart,
                                                                 ssqpart, B, D, DP, nC, tiles_s, KS, sub);
    return hipGetLastError();
}

hipError_t launch_proj_fwd(const void *x, int x_dtype, const void *phi, int phi_dtype, float *Ppart,
                           float *ssqpart, int KS, int B, int n, int C, hipStream_t stream) {
    const int nC = n * C, D = n * n + 2 * n, DP = padded_D(n);
    if (use_mfma(x_dtype, phi_dtype, C)) {
        if (x_dtype == kF32AsBF16) {  // fp32 storage, rounded on load: the narrow kernel only (n <= 8)
            switch (use_wide(n, C) ? 0 : mfma_nt(n)) {
                case 1: return launch_mfma<1, true>(x, phi, Ppart, ssqpart, KS, B, D, DP, nC, stream);
                case 2: return launch_mfma<2, true>(x, phi, Ppart, ssqpart, KS, B, D, DP, nC, stream);
                case 3: return launch_mfma<3, true>(x, phi, Ppart, ssqpart, KS, B, D, DP, nC, stream);
                default: return hipErrorInvalidValue;
            }
        }
        if (use_wide(n, C)) return launch_wide<1, 2, 4>(x, phi, Ppart, ssqpart, KS, B, D, DP, nC, stream);
        switch (mfma_nt(n)) {
            case 1: return launch_mfma<1>(x, phi, Ppart, ssqpart, KS, B, D, DP, nC, stream);
            case 2: return launch_mfma<2>(x, phi, Ppart, ssqpart, KS, B, D, DP, nC, stream);
            case 3: return launch_mfma<3>(x, phi, Ppart, ssqpart, KS, B, D, DP, nC, stream);
            default: return launch_mfma<4>(x, phi, Ppart, ssqpart, KS, B, D, DP, nC, stream);
        }
    }
    if (gemm_f32_supported(x_dtype, phi_dtype, n, C))
        return launch_gemm_f32_proj(static_cast<const float *>(x), static_cast<const float *>(phi), Ppart,
                                    ssqpart, KS, B, n, C, stream);
    if (KS != 1) return hipErrorInvalidValue;  // the generic path produces exactly one split
    if (x_dtype == kF32 && phi_dtype == kF32) return launch_generic<float, float>(x, phi, Ppart, ssqpart, B, D, DP, nC, stream);
    if (x_dtype == kF32 && phi_dtype == kBF16) return launch_generic<float, bf16_t>(x, phi, Ppart, ssqpart, B, D, DP, nC, stream);
    if (x_dtype == kBF16 && phi_dtype == kF32) return launch_generic<bf16_t, float>(x, phi, Ppart, ssqpart, B, D, DP, nC, stream);
    return launch_generic<bf16_t, bf16_t>(x, phi, Ppart, ssqpart, B, D, DP, nC, stream);
}

}  // namespace mhc
