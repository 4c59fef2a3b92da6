// Dynamic-H layer forward in ONE launch and one pass over x (bf16 x and phi, n <= 4):
//   projection  P = x_flat phi^T and sum(x_flat^2)    (reference fused_rmsnorm_matmul.cuh:119-153,
//                                                       bindings.cu:34-81, :436-443)
//   coefficients  H_pre, H_post, M = Sinkhorn(exp(.))  (utils.cuh:50-126, sinkhorn_knopp.cuh:828-909)
//   aggregate, inner RMSNorm, distribute + mix         (stream_ops.cuh:453-526, rmsnorm.cuh:14-165)
// i.e. the whole of mhc_layer_fwd_dynamic (bindings.cu:421-477).
//
// A workgroup owns G consecutive samples and keeps their rows [G][nC] in LDS from the first touch
// to the last.  Phase A: every wave streams its share of the K range - the x rows (row-contiguous
// 16-byte loads, parked in LDS) and the same columns of every phi row - and multiplies them on
// v_mfma_f32_16x16x32_bf16 with phi as the A operand (16 projection rows per tile) and the G
// samples as the B columns, read back from the LDS rows the wave has just written (no barrier: a
// wave's LDS accesses complete in order).  phi is re-read by every workgroup, out of the L2 of
// its XCD; the grouping by G samples is what keeps that traffic below the L1 fill rate.
// Phase B: the waves' partial products are summed through LDS and 16 lanes per sample run the
// activations and the Sinkhorn chain (SkSmall).  Phase C: aggregate, RMS and mix straight from
// the LDS rows on v_mfma_f32_4x4x4_16b_bf16, one 16-byte store per stream and 8-channel chunk.
// x is read from HBM once, y written once; nothing else touches memory except the small saved
// tensors (H_pre, H_post, M, P, r, q).
#include "launchers.h"
#include "mhc_common.h"
#include "phase_profiler.h"
#include "sinkhorn_device.h"
#include "tuning.h"

namespace mhc {

typedef __attribute__((__vector_size__(8 * sizeof(__bf16)))) __bf16 bf16x8_t;
typedef __attribute__((__vector_size__(2 * sizeof(__bf16)))) __bf16 bf16x2_t;

struct OnePassArgs {
    const bf16_t *x;
    const void *w;
    const bf16_t *f_inject;
    void *y;
    const bf16_t *phi;
    const float *alpha, *bias;
    float *Hpre, *Hpost, *M, *P, *r, *q;
    int w_bf16, B, n, C, T, G;
    float eps;
    float *sk_state;  // [B][T + 1][2][NP] Sinkhorn denominators kept for the backward, or nullptr
};

constexpr int kOpMaxG = 16;      // samples per workgroup: the columns of one 16-wide tile
constexpr int kOpPadElems = 8;   // LDS row pad (bf16 elements): consecutive rows start 4 banks apart
constexpr int kOpStagePitch = 72;  // staged phi rows: 128 data bytes + 16 pad (bf16 elements)
constexpr int kOpStageBytes = 32 * kOpStagePitch * 2;  // per wave; later its partial products (2 KiB)
constexpr int kOpDepth = 2;      // steps of loads in flight per wave (more changes nothing: the L1 fill rate is the limit)

// LDS layout (bytes), shared by host and device.
struct OnePassLds {
    int pitch;     // bf16 elements per sample row
    size_t stage, ssqw, hpost, pa, pk, ssqi, qinv, total;
    __host__ __device__ OnePassLds(int G, int nC, int nchp, int NW) {
        pitch = nC + kOpPadElems;
        size_t o = (size_t)G * pitch * 2;
        o = (o + 15) / 16 * 16;
        stage = o; o += (size_t)NW * kOpStageBytes;
        ssqw = o;  o += (size_t)NW * 16 * 4;
        hpost = o; o += (size_t)G * 16;
        pa = o;    o += (size_t)G * 16;
        pk = o;    o += (size_t)G * 4 * 16;
        ssqi = o;  o += (size_t)G * nchp * 4;
        qinv = o;  o += (size_t)G * 4;
        total = (o + 15) / 16 * 16;
    }
};

constexpr int kOnePassWaves = 8;  // waves per workgroup (4..7 measured slower at every shape of the sweep)
constexpr int kDppQuadBcast0 = 0x00, kDppQuadBcast1 = 0x55, kDppQuadBcast2 = 0xAA, kDppQuadBcast3 = 0xFF;

template <typename TY, int GH>
__global__ __launch_bounds__(512) void layer_fwd_onepass_kernel(OnePassArgs a) {
    constexpr int NP = 4, DT = 2;
    using SK = SkSmall<NP>;
    extern __shared__ __align__(16) unsigned char op_smem[];
    const int n = a.n, C = a.C, nC = n * C, G = a.G, D = n * n + 2 * n;
    constexpr int NW = kOnePassWaves, NT = NW * 64;  // compile-time: the cross-wave sums below unroll without masks
    const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
    const int b0 = blockIdx.x * G;
    const int Gv = min(G, a.B - b0);
    const int nch = C / 8, nchp = round_up(nch, 4);
    const OnePassLds L(G, nC, nchp, NW);
    bf16_t *xs = reinterpret_cast<bf16_t *>(op_smem);
    bf16_t *ps = reinterpret_cast<bf16_t *>(op_smem + L.stage + (size_t)wave * kOpStageBytes);
    float *red_all = reinterpret_cast<float *>(op_smem + L.stage);  // wave w: + w * kOpStageBytes / 4
    constexpr int kRedStride = kOpStageBytes / 4;
    float *ssq_w = reinterpret_cast<float *>(op_smem + L.ssqw);
    float *hpost_s = reinterpret_cast<float *>(op_smem + L.hpost);
    uint32_t *pa_s = reinterpret_cast<uint32_t *>(op_smem + L.pa);
    uint32_t *pk_s = reinterpret_cast<uint32_t *>(op_smem + L.pk);
    float *ssq_i = reinterpret_cast<float *>(op_smem + L.ssqi);
    float *qinv_s = reinterpret_cast<float *>(op_smem + L.qinv);
    const int pitch = L.pitch;
    const bool inject = a.f_inject != nullptr;
    MHC_PHASE(kPhaseFwdOnepass, blockIdx.x, 0);
    // small inputs of the coefficient step, requested ahead of everything else (lane roles of phase B)
    float c_al, c_al2, c_bvec, c_bres;
    {
        const int g = lane & 15, r0 = SK::row(g), c0 = SK::col0(g);
        const bool mv = r0 < n && c0 < n, vv = g < 2 * n;
        c_al = a.alpha[vv ? (g < n ? 0 : 1) : 2];
        c_al2 = a.alpha[2];
        c_bvec = a.bias[vv ? g : 0];
        c_bres = a.bias[mv ? 2 * n + r0 * n + c0 : 0];
    }

    // ---- phase A: stream x and phi, project ---------------------------------------------------
    {
        const int steps = nC >> 6;  // 64 contraction elements (128 bytes of every row) per step
        // Each workgroup of an XCD (ids 8 apart) walks K from its own starting point: the rows of phi
        // lie a multiple of 4 KiB apart, so at a given k they all sit in the same L2 channel.
        const int rot = (int)(((blockIdx.x >> 3) * (unsigned)steps) >> 5) % steps;
        auto k_of = [&](int st) {
            int p = st + rot;
            p = p >= steps ? p - steps : p;
            return p << 6;
        };
        // Both operands are fetched row-contiguously: 8 lanes per 128-byte row piece, rows r8 + 8j.
        // (Loading phi straight in operand layout, every lane on its own row, costs the L1 one tag
        // lookup per lane: four times the time of these loads.)  x rows beyond the workgroup's samples
        // alias the last valid one and are not parked; phi rows beyond D alias row 0.
        const int r8 = lane >> 3, seg = lane & 7;
        const int dj = (D + 7) >> 3;  // 8-row pieces of phi: 1..3
        const bf16_t *xrow[GH], *prow[3];
        bool xv[GH];
#pragma unroll
        for (int h = 0; h < GH; h++) {
            const int g = r8 + 8 * h;
            xv[h] = g < Gv;
            xrow[h] = a.x + (size_t)(b0 + (xv[h] ? g : Gv - 1)) * nC + seg * 8;
        }
#pragma unroll
        for (int j = 0; j < 3; j++) {
            const int d = j * 8 + r8;
            prow[j] = a.phi + (size_t)(d < D ? d : 0) * nC + seg * 8;
        }
        // operand layout: lane (row, kg) holds k = 16 kg .. 16 kg + 15 of its row; the first 8 feed the
        // first product of the step, the other 8 the second (x follows the same order)
        const int row = lane & 15, kg = lane >> 4;
        const bf16_t *xfrag = xs + (size_t)(row < Gv ? row : Gv - 1) * pitch + kg * 16;
        const bf16_t *pfrag = ps + row * kOpStagePitch + kg * 16;

        // kOpDepth steps in flight per wave (scalar words: whole-uint4 array elements can end up in scratch)
        uint32_t xq[kOpDepth][GH][4], pq[kOpDepth][3][4];
        auto fetch = [&](int slot, int st) {
            const int k0 = k_of(st);
#pragma unroll
            for (int h = 0; h < GH; h++) {
                const uint4 v = *reinterpret_cast<const uint4 *>(xrow[h] + k0);
                xq[slot][h][0] = v.x; xq[slot][h][1] = v.y; xq[slot][h][2] = v.z; xq[slot][h][3] = v.w;
            }
#pragma unroll
            for (int j = 0; j < 3; j++) {
                if (j < dj) {
                    const uint4 v = *reinterpret_cast<const uint4 *>(prow[j] + k0);
                    pq[slot][j][0] = v.x; pq[slot][j][1] = v.y; pq[slot][j][2] = v.z; pq[slot][j][3] = v.w;
                }
            }
        };
        f32x4_t acc[DT];
#pragma unroll
        for (int t = 0; t < DT; t++) acc[t] = f32x4_t{0.f, 0.f, 0.f, 0.f};
        float ssq[GH];
#pragma unroll
        for (int h = 0; h < GH; h++) ssq[h] = 0.f;
        auto process = [&](int slot, int st) {
            const int k0 = k_of(st);
#pragma unroll
            for (int h = 0; h < GH; h++) {
                if (xv[h])
                    *reinterpret_cast<uint4 *>(xs + (size_t)(r8 + 8 * h) * pitch + k0 + seg * 8) =
                        make_uint4(xq[slot][h][0], xq[slot][h][1], xq[slot][h][2], xq[slot][h][3]);
#pragma unroll
                for (int i = 0; i < 4; i++) {
                    const bf16x2_t pr = __builtin_bit_cast(bf16x2_t, xq[slot][h][i]);
                    ssq[h] = __builtin_amdgcn_fdot2_f32_bf16(pr, pr, ssq[h], false);
                }
            }
#pragma unroll
            for (int j = 0; j < 3; j++) {
                if (j < dj)
                    *reinterpret_cast<uint4 *>(ps + (j * 8 + r8) * kOpStagePitch + seg * 8) =
                        make_uint4(pq[slot][j][0], pq[slot][j][1], pq[slot][j][2], pq[slot][j][3]);
            }
            // both come back in operand layout from the lines this wave has just written (a wave's LDS
            // accesses complete in order; the fence keeps the compiler from moving the reads up)
            __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront");
            __builtin_amdgcn_wave_barrier();
            const uint4 x0 = *reinterpret_cast<const uint4 *>(xfrag + k0);
            const uint4 x1 = *reinterpret_cast<const uint4 *>(xfrag + k0 + 8);
#pragma unroll
            for (int t = 0; t < DT; t++) {
                if (t == 0 || D > 16) {
                    const uint4 p0 = *reinterpret_cast<const uint4 *>(pfrag + t * 16 * kOpStagePitch);
                    const uint4 p1 = *reinterpret_cast<const uint4 *>(pfrag + t * 16 * kOpStagePitch + 8);
                    acc[t] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(__builtin_bit_cast(bf16x8_t, p0),
                                                                     __builtin_bit_cast(bf16x8_t, x0), acc[t], 0, 0, 0);
                    acc[t] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(__builtin_bit_cast(bf16x8_t, p1),
                                                                     __builtin_bit_cast(bf16x8_t, x1), acc[t], 0, 0, 0);
                }
            }
            __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "wavefront");
            __builtin_amdgcn_wave_barrier();
        };
        // steps wave, wave + NW, ...: at any time the waves work on neighbouring lines of the same rows
#pragma unroll
        for (int u = 0; u < kOpDepth; u++)
            if (wave + u * NW < steps) fetch(u, wave + u * NW);
        for (int st = wave; st < steps; st += kOpDepth * NW) {
#pragma unroll
            for (int u = 0; u < kOpDepth; u++) {
                const int su = st + u * NW;
                if (su < steps) {
                    process(u, su);
                    if (su + kOpDepth * NW < steps) fetch(u, su + kOpDepth * NW);
                }
            }
        }
        // partial sums into the wave's own (now idle) staging area: accumulator register r of tile t
        // in lane l is row 16t + 4(l / 16) + r, column (sample) l % 16
        float *red = red_all + wave * kRedStride;
#pragma unroll
        for (int t = 0; t < DT; t++)
#pragma unroll
            for (int r = 0; r < 4; r++) red[(t * 4 + r) * 64 + lane] = acc[t][r];
#pragma unroll
        for (int h = 0; h < GH; h++) {
            float v = ssq[h];  // the 8 lanes of a row piece are consecutive
            v += dpp_mov<kDppQuadXor1>(v);
            v += dpp_mov<kDppQuadXor2>(v);
            v += dpp_mov<kDppRowHalfMirror>(v);
            if (seg == 0) ssq_w[wave * 16 + r8 + 8 * h] = v;
        }
        if constexpr (GH == 1) {
            if (lane < 8) ssq_w[wave * 16 + 8 + lane] = 0.f;
        }
    }
    MHC_PHASE(kPhaseFwdOnepass, blockIdx.x, 1);
    __syncthreads();
    MHC_PHASE(kPhaseFwdOnepass, blockIdx.x, 2);

    // ---- phase B: coefficients, 16 lanes per sample.  First the activations (Hpre is all the
    // aggregate pass needs), then the Sinkhorn chain while the other waves run that pass. ----------
    const int ncw = (Gv + SK::kPerWave - 1) / SK::kPerWave;  // waves that hold samples
    const bool coef_wave = wave < ncw;
    const int g = lane & 15, s_c = wave * SK::kPerWave + (lane >> 4);
    const bool sv = coef_wave && s_c < Gv;
    const int sc = s_c < Gv ? s_c : Gv - 1;
    const int r0 = SK::row(g), c0 = SK::col0(g);
    const bool mv = r0 < n && c0 < n, vv = g < 2 * n;
    float m[1] = {0.f};
    if (coef_wave) {  // uniform per wave
        // sums over the waves: all reads issued together (wave slots beyond NW alias the last one)
        const int dv = vv ? g : 0, dm = mv ? 2 * n + r0 * n + c0 : 0;
        auto slot_of = [&](int d) { return ((d >> 4) * 4 + (d & 3)) * 64 + ((d & 15) >> 2) * 16 + sc; };
        const int ov = slot_of(dv), om = slot_of(dm);
        float tv[8], tm[8], ts[8];
#pragma unroll
        for (int w2 = 0; w2 < 8; w2++) {
            const int wc = w2 < NW ? w2 : NW - 1;
            tv[w2] = red_all[wc * kRedStride + ov];
            tm[w2] = red_all[wc * kRedStride + om];
            ts[w2] = ssq_w[wc * 16 + sc];
        }
        float pvec = 0.f, pe = 0.f, ssq = 0.f;
#pragma unroll
        for (int w2 = 0; w2 < 8; w2++) {
            pvec += w2 < NW ? tv[w2] : 0.f;
            pe += w2 < NW ? tm[w2] : 0.f;
            ssq += w2 < NW ? ts[w2] : 0.f;
        }
        const float ms = ssq * (1.0f / (float)nC) + a.eps;
        const float r = __builtin_amdgcn_sqrtf(ms);
        const float rinv = fast_rcp(r);
        const size_t b = (size_t)(b0 + sc);
        if (sv && g == 0) a.r[b] = r;
        float h = 0.f;
        if (vv) {
            const bool pre = g < n;
            const float p = pvec * rinv;
            const float sg = sigmoid_fast(c_al * p + c_bvec);
            h = pre ? sg : 2.0f * sg;
            if (sv) {
                (pre ? a.Hpre : a.Hpost)[b * n + (pre ? g : g - n)] = h;
                a.P[b * D + g] = p;
            }
        }
        // Hpost (zero padded to 4) and Hpre as the A row of the aggregate product: lanes 0..3 of a
        // sample see all four Hpre values through quad broadcasts
        if (sv && g >= n && g < n + NP) hpost_s[sc * NP + (g - n)] = g < 2 * n ? h : 0.f;
        const float hp = g < n ? h : 0.f;
        const float h0 = dpp_mov<kDppQuadBcast0>(hp), h1 = dpp_mov<kDppQuadBcast1>(hp);
        const float h2 = dpp_mov<kDppQuadBcast2>(hp), h3 = dpp_mov<kDppQuadBcast3>(hp);
        if (sv && g == 0) {
            CoefRow ca;
            ca.set(h0, h1, h2, h3);
            const uint2 u0 = __builtin_bit_cast(uint2, ca.hi), u1 = __builtin_bit_cast(uint2, ca.lo);
            *reinterpret_cast<uint4 *>(pa_s + sc * 4) = make_uint4(u0.x, u0.y, u1.x, u1.y);
        }
        if (mv) {
            const float p = pe * rinv;
            if (sv) a.P[b * D + 2 * n + r0 * n + c0] = p;
            m[0] = exp_fast(c_al2 * p + c_bres);
        }
    }
    MHC_PHASE(kPhaseFwdOnepass, blockIdx.x, 3);
    __syncthreads();

    // ---- phase C items = (sample, 8-channel chunk), sample-major with the chunk count padded to a
    // multiple of 4: the four lanes of a 4x4x4 block share their sample. -----------------------------
    const int items = Gv * nchp;
    const f32x4_t zero = {0.f, 0.f, 0.f, 0.f};
    const bool jq0 = (tid & 3) == 0;
    auto load_item = [&](int s, int ch, uint32_t (&xw)[NP][4]) {
        const bf16_t *p = xs + (size_t)s * pitch + (size_t)(ch < nch ? ch : 0) * 8;
#pragma unroll
        for (int i = 0; i < NP; i++) {
            const uint4 v = *reinterpret_cast<const uint4 *>(p + (size_t)(i < n ? i : 0) * C);
            xw[i][0] = v.x; xw[i][1] = v.y; xw[i][2] = v.z; xw[i][3] = v.w;
        }
    };
    auto channel = [&](const uint32_t (&xw)[NP][4], int v) {
        const int p = v >> 1;
        return (v & 1) ? streams_of_channel<true>(xw[0][p], xw[1][p], xw[2][p], xw[3][p])
                       : streams_of_channel<false>(xw[0][p], xw[1][p], xw[2][p], xw[3][p]);
    };
    auto agg_row = [&](int s, bf16x4_t &ahi, bf16x4_t &alo) {  // [Hpre; 0; 0; 0]: lane jq supplies row jq
        const uint4 c1 = *reinterpret_cast<const uint4 *>(pa_s + s * 4);
        ahi = bf16x4_of(jq0 ? c1.x : 0u, jq0 ? c1.y : 0u);
        alo = bf16x4_of(jq0 ? c1.z : 0u, jq0 ? c1.w : 0u);
    };
    // aggregate pass on the waves that hold no samples (on all waves, after the chain, if there are none)
    const int w0 = NW > ncw ? ncw : 0;
    auto aggregate_pass = [&]() {
        const int ht = tid - w0 * 64, hn = NT - w0 * 64;
        int s = 0, ch = ht;
        for (int it = ht; it < items; it += hn, ch += hn) {
            while (ch >= nchp) { ch -= nchp; s++; }
            uint32_t xw[NP][4];
            load_item(s, ch, xw);
            bf16x4_t ahi, alo;
            agg_row(s, ahi, alo);
            float sq = 0.f;
#pragma unroll
            for (int v = 0; v < 8; v++) {
                const bf16x4_t bx = channel(xw, v);
                f32x4_t da = mfma4(ahi, bx, zero);
                da = mfma4(alo, bx, da);
                sq += da[0] * da[0];
            }
            ssq_i[it] = ch < nch ? sq : 0.f;
        }
    };
    if (coef_wave) {
        // (samples beyond the group write the state of the last valid one again: same values)
        if (a.sk_state) SK::template forward_save<false>(m, g, n, a.T, a.eps, a.sk_state + (size_t)(b0 + sc) * SK::state_floats(a.T));
        else SK::template forward<false, false>(m, g, n, a.T, a.eps, nullptr, lane);
        if (sv && mv) a.M[(size_t)(b0 + sc) * n * n + r0 * n + c0] = m[0];
        // row r0 of M as an A row (bf16 value + remainder): the quad that holds the row sees all of it
        const float m0 = dpp_mov<kDppQuadBcast0>(m[0]), m1 = dpp_mov<kDppQuadBcast1>(m[0]);
        const float m2 = dpp_mov<kDppQuadBcast2>(m[0]), m3 = dpp_mov<kDppQuadBcast3>(m[0]);
        if (sv && c0 == 0) {
            CoefRow cm;
            cm.set(m0, m1, m2, m3);
            const uint2 u0 = __builtin_bit_cast(uint2, cm.hi), u1 = __builtin_bit_cast(uint2, cm.lo);
            *reinterpret_cast<uint4 *>(pk_s + (sc * 4 + r0) * 4) = make_uint4(u0.x, u0.y, u1.x, u1.y);
        }
        if (w0 == 0 && !inject) aggregate_pass();
    } else if (!inject) {
        aggregate_pass();
    }
    __syncthreads();
    MHC_PHASE(kPhaseFwdOnepass, blockIdx.x, 4);
    for (int s = wave; s < Gv; s += NW) {
        float q = 1.0f;
        if (!inject) {
            float v = 0.f;
            for (int j = lane; j < nchp; j += 64) v += ssq_i[s * nchp + j];
            v = wave_allreduce_sum(v);
            q = __builtin_amdgcn_sqrtf(v * (1.0f / (float)C) + a.eps);
        }
        if (lane == 0) {
            qinv_s[s] = fast_rcp(q);
            a.q[b0 + s] = q;
        }
    }
    __syncthreads();
    MHC_PHASE(kPhaseFwdOnepass, blockIdx.x, 5);
    {
        int s = 0, ch = tid;
        for (int it = tid; it < items; it += NT, ch += NT) {
            while (ch >= nchp) { ch -= nchp; s++; }
            uint32_t xw[NP][4];
            load_item(s, ch, xw);
            const uint4 c0v = *reinterpret_cast<const uint4 *>(pk_s + (s * 4 + (tid & 3)) * 4);
            const float4 hq = *reinterpret_cast<const float4 *>(hpost_s + s * NP);
            const bf16x4_t mhi = bf16x4_of(c0v.x, c0v.y), mlo = bf16x4_of(c0v.z, c0v.w);
            bf16x4_t ahi, alo;
            agg_row(s, ahi, alo);
            const float hpost[NP] = {hq.x, hq.y, hq.z, hq.w};
            const bool live = ch < nch;
            const int c = (live ? ch : 0) * 8;
            const size_t b = (size_t)(b0 + s);
            float f[8];
            if (inject) {
                load_vec<bf16_t, 8>(a.f_inject + b * C + c, f);
            } else {
                if (a.w_bf16) load_vec<bf16_t, 8>(static_cast<const bf16_t *>(a.w) + c, f);
                else load_vec<float, 8>(static_cast<const float *>(a.w) + c, f);
            }
            const float qinv = qinv_s[s];
            float o[NP][8];
#pragma unroll
            for (int v = 0; v < 8; v++) {
                const bf16x4_t bx = channel(xw, v);
                f32x4_t d = mfma4(mhi, bx, zero);
                d = mfma4(mlo, bx, d);
                float fv;
                if (inject) {
                    fv = f[v];
                } else {
                    f32x4_t da = mfma4(ahi, bx, zero);
                    da = mfma4(alo, bx, da);
                    fv = da[0] * qinv * f[v];
                }
#pragma unroll
                for (int i = 0; i < NP; i++) o[i][v] = d[i] + hpost[i] * fv;
            }
            if (live) {
                TY *yb = static_cast<TY *>(a.y) + b * nC + c;
#pragma unroll
                for (int i = 0; i < NP; i++)
                    if (i < n) store_vec<TY, 8, true>(yb + (size_t)i * C, o[i]);
            }
        }
    }
    MHC_PHASE(kPhaseFwdOnepass, blockIdx.x, 6);
}

// Samples per workgroup: about one workgroup per CU (phi is re-read by every workgroup), bounded by
// the 16 columns of the product tile and by LDS.
static int onepass_group(int B, int n, int C) {
    const int t = tuning_get(kTuneOnepassG);
    int G = t > 0 ? t : (B + 255) / 256;
    if (G > kOpMaxG) G = kOpMaxG;
    if (G < 1) G = 1;
    while (G > 1 && OnePassLds(G, n * C, round_up(C / 8, 4), 8).total > 158 * 1024) G--;
    return G;
}

// Every workgroup streams all of phi out of the L2 (about 90 GB/s per CU in this access pattern, measured
// by a stand-alone loop; more steps in flight change nothing), so phase A costs the kernel start plus
// |phi| / 90 GB/s whatever the batch.  Measured on whole forward+backward steps (graphs of ten steps,
// B = 64 .. 4096, C = 512 .. 4096, n = 2, 3, 4): the one-launch forward wins by 2 - 15 % while phi is
// below ~120 KB; between 120 and 256 KB it wins only around B = 1280 (five samples per workgroup share
// the phi stream: B=1280 C=1280 n=4 47.6 against 48.8 us) and loses at small and very large batches
// (B=320 C=1280 n=4, 240 KB: 31.4 against 30.3 us); beyond 256 KB it loses everywhere (B=1280 C=2560
// n=4: 64.1 against 62.2 us).  Elsewhere the two-launch forward (split-K projection, then the fused mix
// kernel) stays.
bool layer_fwd_onepass_supported(int x_dtype, int phi_dtype, int B, int n, int C) {
    const int mode = tuning_get(kTuneOnepassOff);  // 0 = by cost, 1 = never, 2 = whenever the shape allows
    if (mode == 1) return false;
    if (x_dtype != kBF16 || phi_dtype != kBF16 || n > 4 || C % 8 != 0 || (n * C) % 64 != 0) return false;
    if (OnePassLds(1, n * C, round_up(C / 8, 4), kOnePassWaves).total > 158 * 1024) return false;
    if (mode == 2) return true;
    const long long phi_bytes = 2ll * (n * n + 2 * n) * n * C;
    return phi_bytes <= 120 * 1024 || (phi_bytes <= 256 * 1024 && B >= 1024 && B <= 2048);
}

hipError_t launch_layer_fwd_onepass(const void *x, const void *w, int w_dtype, const void *f_inject, void *y,
                                    int y_dtype, const void *phi, const float *alpha, const float *bias,
                                    float *Hpre, float *Hpost, float *M, float *P, float *r, float *q,
                                    float *sk_state, int B, int n, int C, int T, float eps, hipStream_t stream) {
    const int G = onepass_group(B, n, C);
    constexpr int NW = kOnePassWaves;
    OnePassArgs a{static_cast<const bf16_t *>(x), w, static_cast<const bf16_t *>(f_inject), y,
                  static_cast<const bf16_t *>(phi), alpha, bias, Hpre, Hpost, M, P, r, q,
                  w_dtype == kBF16, B, n, C, T, G, eps, sk_state};
    const size_t smem = OnePassLds(G, n * C, round_up(C / 8, 4), NW).total;
    const int grid = (B + G - 1) / G;
    hipError_t e = hipSuccess;
#define MHC_ONEPASS(TY, GH)                                                                  \
    do {                                                                                     \
        e = allow_dynamic_lds(layer_fwd_onepass_kernel<TY, GH>, smem);                       \
        if (e != hipSuccess) return e;                                                       \
        layer_fwd_onepass_kernel<TY, GH><<<grid, NW * 64, smem, stream>>>(a);                \
    } while (0)
    if (y_dtype == kBF16) {
        if (G <= 8) MHC_ONEPASS(bf16_t, 1); else MHC_ONEPASS(bf16_t, 2);
    } else {
        if (G <= 8) MHC_ONEPASS(float, 1); else MHC_ONEPASS(float, 2);
    }
#undef MHC_ONEPASS
    return hipGetLastError();
}

}  // namespace mhc
