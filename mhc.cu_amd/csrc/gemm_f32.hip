// fp32 GEMM on the matrix cores (v_mfma_f32_32x32x2_f32) for the exact float32 tier of the
// projection: P = x_flat phi^T (split-K, with sum x^2), dphi = dP^T x_flat and dxflat = dP phi.
// Products and sums are IEEE fp32, so the results differ from a sequential fp32 loop only by the
// order of the additions.
//
// Replaces, for float32 activations and parameters, the cuBLASLt projection of the reference
// (src/python/bindings.cu:34-81) and the three torch matmuls of its dynamic backward
// (src/python/mhc/ops.py:332-351).
//
// Workgroup tile 128 x 128, K in slices of 32 through LDS; 4 waves as 2 x 2, each 64 x 64
// (2 x 2 accumulator tiles).  Both operands sit in LDS as [k][row]: an operand whose contiguous
// index is k is fetched row-contiguously (8 lanes per 128-byte line) and transposed on the way in,
// one whose contiguous index is the row goes in as it is.  The next slice is in flight in
// registers while the current one is multiplied.
#include "launchers.h"
#include "mhc_common.h"

namespace mhc {

typedef __attribute__((__vector_size__(16 * sizeof(float)))) float f32x16_t;

constexpr int kGT = 128;        // tile rows = tile columns
constexpr int kGK = 32;         // contraction slice
constexpr int kGLD = kGT + 4;   // LDS pitch (floats); 528 bytes keeps float4 rows 16-byte aligned

struct GemmArgs {
    const float *A, *B;
    float *C;
    int M, N, K;           // C is M x N, contraction length K
    long long lda, ldb, ldc;
    int n_store;           // columns [N, n_store) of C are written as zeros
    int k_per_split;       // multiple of kGK; grid.z splits
    long long c_split;     // elements between the C copies of consecutive splits
    float *ssq;            // optional [splits][M]: sum_k A(m,k)^2 over the split (AK only)
};

// One operand slice in registers: 4 float4 per thread.
struct Slice { float4 v[4]; };

// K-contiguous operand, element (r, k) at P[r * ld + k]: thread = 16-byte segment (tid & 7) of rows
// (tid >> 3) + 32 j.  Rows beyond R alias row R - 1 (their products are never stored); elements
// with k >= K are zeroed.  The row pitch must cover K rounded up to 4.
__device__ __forceinline__ void load_kc(Slice &s, const float *P, long long ld, int r0, int R, int k0,
                                        int K, int tid) {
    const int seg = tid & 7, k = k0 + 4 * seg;
    const bool kin = k < K;
#pragma unroll
    for (int j = 0; j < 4; j++) {
        const int r = min(r0 + (tid >> 3) + 32 * j, R - 1);
        float4 t = *reinterpret_cast<const float4 *>(P + (size_t)r * ld + (kin ? k : 0));
        t.x = k < K ? t.x : 0.f; t.y = k + 1 < K ? t.y : 0.f;
        t.z = k + 2 < K ? t.z : 0.f; t.w = k + 3 < K ? t.w : 0.f;
        s.v[j] = t;
    }
}
__device__ __forceinline__ void park_kc(const Slice &s, float *Xs, int tid) {
    const int seg = tid & 7;
#pragma unroll
    for (int j = 0; j < 4; j++) {
        float *p = Xs + (size_t)(4 * seg) * kGLD + (tid >> 3) + 32 * j;
        p[0] = s.v[j].x; p[kGLD] = s.v[j].y; p[2 * kGLD] = s.v[j].z; p[3 * kGLD] = s.v[j].w;
    }
}

// Row-contiguous operand, element (r, k) at P[k * ld + r]: thread = float4 (tid & 31) of k-rows
// (tid >> 5) + 8 j.  float4s that start at or beyond R alias the tile's first one (never stored);
// k-rows >= K are zeroed.  The k-row pitch must cover R rounded up to 4.
__device__ __forceinline__ void load_rc(Slice &s, const float *P, long long ld, int r0, int R, int k0,
                                        int K, int tid) {
    const int q = tid & 31;
    const int r = r0 + 4 * q < R ? r0 + 4 * q : r0;
#pragma unroll
    for (int j = 0; j < 4; j++) {
        const int k = k0 + (tid >> 5) + 8 * j;
        float4 t = *reinterpret_cast<const float4 *>(P + (size_t)(k < K ? k : 0) * ld + r);
        if (k >= K) t = make_float4(0.f, 0.f, 0.f, 0.f);
        s.v[j] = t;
    }
}
__device__ __forceinline__ void park_rc(const Slice &s, float *Xs, int tid) {
#pragma unroll
    for (int j = 0; j < 4; j++)
        *reinterpret_cast<float4 *>(Xs + (size_t)((tid >> 5) + 8 * j) * kGLD + 4 * (tid & 31)) = s.v[j];
}

// AK / BK: the operand's contiguous index is k.  grid: (N tiles, M tiles, splits)
template <bool AK, bool BK>
__global__ __launch_bounds__(256) void gemm_f32_kernel(GemmArgs a) {
    __shared__ __align__(16) float As[kGK * kGLD];
    __shared__ __align__(16) float Bs[kGK * kGLD];
    const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
    const int wm = wave >> 1, wn = wave & 1;
    const int n0 = blockIdx.x * kGT, m0 = blockIdx.y * kGT;
    const int kbeg = blockIdx.z * a.k_per_split;
    const int kend = min(a.K, kbeg + a.k_per_split);

    f32x16_t acc[2][2];
#pragma unroll
    for (int mt = 0; mt < 2; mt++)
#pragma unroll
        for (int nt = 0; nt < 2; nt++)
#pragma unroll
            for (int i = 0; i < 16; i++) acc[mt][nt][i] = 0.f;
    float ssq[4] = {0.f, 0.f, 0.f, 0.f};
    const bool want_ssq = AK && a.ssq != nullptr && blockIdx.x == 0;

    Slice sa, sb;
    auto fetch = [&](int k0) {
        if constexpr (AK) load_kc(sa, a.A, a.lda, m0, a.M, k0, kend, tid);
        else load_rc(sa, a.A, a.lda, m0, a.M, k0, kend, tid);
        if constexpr (BK) load_kc(sb, a.B, a.ldb, n0, a.N, k0, kend, tid);
        else load_rc(sb, a.B, a.ldb, n0, a.N, k0, kend, tid);
    };
    fetch(kbeg);
    for (int k0 = kbeg; k0 < kend; k0 += kGK) {
        if constexpr (AK) park_kc(sa, As, tid); else park_rc(sa, As, tid);
        if constexpr (BK) park_kc(sb, Bs, tid); else park_rc(sb, Bs, tid);
        if (want_ssq) {
#pragma unroll
            for (int j = 0; j < 4; j++)
                ssq[j] += (sa.v[j].x * sa.v[j].x + sa.v[j].y * sa.v[j].y) + (sa.v[j].z * sa.v[j].z + sa.v[j].w * sa.v[j].w);
        }
        __syncthreads();
        if (k0 + kGK < kend) fetch(k0 + kGK);  // in flight during the multiplications
        // an MFMA contracts two k per call: slice rows kr and kr + 8, whose LDS rows are 32 banks apart,
        // so the two half-waves read disjoint banks
#pragma unroll 4
        for (int kk = 0; kk < kGK / 2; kk++) {
            const int kr = (kk >> 3) * 16 + (kk & 7) + 8 * (lane >> 5);
            const float *ap = As + (size_t)kr * kGLD + wm * 64 + (lane & 31);
            const float *bp = Bs + (size_t)kr * kGLD + wn * 64 + (lane & 31);
            const float a0 = ap[0], a1 = ap[32], b0 = bp[0], b1 = bp[32];
            acc[0][0] = __builtin_amdgcn_mfma_f32_32x32x2f32(a0, b0, acc[0][0], 0, 0, 0);
            acc[0][1] = __builtin_amdgcn_mfma_f32_32x32x2f32(a0, b1, acc[0][1], 0, 0, 0);
            acc[1][0] = __builtin_amdgcn_mfma_f32_32x32x2f32(a1, b0, acc[1][0], 0, 0, 0);
            acc[1][1] = __builtin_amdgcn_mfma_f32_32x32x2f32(a1, b1, acc[1][1], 0, 0, 0);
        }
        __syncthreads();
    }

    // accumulator layout of a 32 x 32 tile: column = lane & 31, register i -> row 8*(i/4) + 4*(lane/32) + i%4
    float *C = a.C + (size_t)blockIdx.z * a.c_split;
#pragma unroll
    for (int mt = 0; mt < 2; mt++)
#pragma unroll
        for (int nt = 0; nt < 2; nt++) {
            const int col = n0 + wn * 64 + nt * 32 + (lane & 31);
#pragma unroll
            for (int i = 0; i < 16; i++) {
                const int row = m0 + wm * 64 + mt * 32 + 8 * (i >> 2) + 4 * (lane >> 5) + (i & 3);
                if (row < a.M && col < a.n_store) C[(size_t)row * a.ldc + col] = col < a.N ? acc[mt][nt][i] : 0.f;
            }
        }
    if (want_ssq) {
#pragma unroll
        for (int j = 0; j < 4; j++) {
            float v = ssq[j];  // the 8 lanes of a row are consecutive
            v += __shfl_xor(v, 1, kWave);
            v += __shfl_xor(v, 2, kWave);
            v += __shfl_xor(v, 4, kWave);
            const int row = m0 + (tid >> 3) + 32 * j;
            if ((tid & 7) == 0 && row < a.M) a.ssq[(size_t)blockIdx.z * a.M + row] = v;
        }
    }
}

template <bool AK, bool BK> static hipError_t launch_gemm(const GemmArgs &a, int splits, hipStream_t stream) {
    dim3 grid((a.n_store + kGT - 1) / kGT, (a.M + kGT - 1) / kGT, splits);
    gemm_f32_kernel<AK, BK><<<grid, 256, 0, stream>>>(a);
    return hipGetLastError();
}

bool gemm_f32_supported(int x_dtype, int phi_dtype, int n, int C) {
    return x_dtype == kF32 && phi_dtype == kF32 && (n * C) % 4 == 0 && n * C >= 256;
}

int gemm_f32_proj_ksplit(int B, int n, int C, int max_splits) {
    const int nC = n * C, DP = padded_D(n);
    const int tiles = ((B + kGT - 1) / kGT) * ((DP + kGT - 1) / kGT);
    int ks = (256 + tiles - 1) / tiles;  // one workgroup per CU; the partial sums stay small
    const int cap = nC / (8 * kGK);  // at least 8 slices per split
    if (ks > cap) ks = cap;
    if (ks > max_splits) ks = max_splits;
    // n <= 8: the fused forward kernel sums at most 24 splits (16 for rows longer than 2048) in its one round of loads
    if (n <= 8 && ks > (C <= 2048 ? 24 : 16)) ks = C <= 2048 ? 24 : 16;
    if (ks < 1) ks = 1;
    // whole slices per split; drop the splits that would get none
    const int kps = ((nC + ks - 1) / ks + kGK - 1) / kGK * kGK;
    return (nC + kps - 1) / kps;
}

hipError_t launch_gemm_f32_proj(const float *x, const float *phi, float *Ppart, float *ssqpart, int KS,
                                int B, int n, int C, hipStream_t stream) {
    const int nC = n * C, D = n * n + 2 * n, DP = padded_D(n);
    const int kps = ((nC + KS - 1) / KS + kGK - 1) / kGK * kGK;
    GemmArgs a{x, phi, Ppart, B, D, nC, nC, nC, DP, DP, kps, (long long)B * DP, ssqpart};
    return launch_gemm<true, true>(a, KS, stream);
}

hipError_t launch_gemm_f32_dphi(const float *dP, const float *x, float *dphi, int B, int n, int C,
                                hipStream_t stream) {
    const int nC = n * C, D = n * n + 2 * n, DP = padded_D(n);
    GemmArgs a{dP, x, dphi, D, nC, B, DP, nC, nC, nC, (B + kGK - 1) / kGK * kGK, 0, nullptr};
    return launch_gemm<false, false>(a, 1, stream);
}

hipError_t launch_gemm_f32_dxflat(const float *dP, const float *phi, float *dxflat, int B, int n, int C,
                                  hipStream_t stream) {
    const int nC = n * C, D = n * n + 2 * n, DP = padded_D(n);
    GemmArgs a{dP, phi, dxflat, B, nC, D, DP, nC, nC, nC, (D + kGK - 1) / kGK * kGK, 0, nullptr};
    return launch_gemm<true, false>(a, 1, stream);
}

}  // namespace mhc
