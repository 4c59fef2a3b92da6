// Stand-alone operators: Sinkhorn-Knopp on plain rows x cols matrices and row-wise RMSNorm,
// forward and backward.  Semantics of the reference's operator-level CPU references:
// src/csrc/tests/test_sinkhorn_knopp.cu:16-47 (no exp; divide only where the sum exceeds eps),
// src/csrc/tests/test_rmsnorm.cu:17-30 and test_rmsnorm_backward.cu:17-39.
#include "launchers.h"
#include "mhc_common.h"
#include "sinkhorn_device.h"

namespace mhc {

constexpr int kSkMax = 128;

// Iterate = diag(u) inp diag(v); a half step only updates u or v.  One workgroup per matrix;
// the matrix itself stays in global memory (L2 resident), u / v / sums live in LDS.
// scal (optional, backward): [batch][T][2][kSkMax] divisors (-1 where the division was skipped).
// A rows x cols matrix with rows != cols has row sums near cols / rows after every column step, so
// the plain scalings would grow like (rows / cols)^t and (cols / rows)^t and leave float32 after a
// few dozen iterations (128 x 3: 25).  The stored u therefore carries an extra factor kappa^t and the
// stored v the factor kappa^-t, kappa = cols / rows: every row step multiplies u by kappa on top of
// its division and every column step finds its sums multiplied by kappa.  The product u v, the
// recorded divisors and the eps test are those of the plain iteration; kappa = 1 for square input.
__global__ __launch_bounds__(256) void sinkhorn_plain_fwd_kernel(const float *__restrict__ inp,
                                                                 float *__restrict__ out, int rows,
                                                                 int cols, int T, float eps,
                                                                 float *__restrict__ scal) {
    __shared__ float u[kSkMax], v[kSkMax];
    const int tid = threadIdx.x;
    const float *A = inp + (size_t)blockIdx.x * rows * cols;
    float *sc = scal ? scal + (size_t)blockIdx.x * T * 2 * kSkMax : nullptr;
    if (tid < kSkMax) { u[tid] = 1.f; v[tid] = 1.f; }
    const float kappa = (float)cols / (float)rows, kappa_inv = (float)rows / (float)cols;
    __syncthreads();
    for (int t = 0; t < T; t++) {
        // rows: two threads per row
        {
            const int r = tid >> 1, h = tid & 1;
            float acc = 0.f;
            if (r < rows)
                for (int c = h; c < cols; c += 2) acc += A[r * cols + c] * v[c];
            acc += __shfl_xor(acc, 1, kWave);
            if (r < rows && h == 0) {
                const float sum = u[r] * acc;
                const bool doit = sum > eps;
                u[r] = doit ? u[r] / sum * kappa : u[r] * kappa;
                if (sc) sc[(t * 2) * kSkMax + r] = doit ? sum : -1.0f;  // negative = skipped
            }
        }
        __syncthreads();
        // columns: two threads per column (coalesced along c within each half)
        {
            const int c = tid & 127, h = tid >> 7;
            float acc = 0.f;
            if (c < cols)
                for (int r = h; r < rows; r += 2) acc += A[r * cols + c] * u[r];
            __shared__ float half_sum[kSkMax];
            if (h == 1) half_sum[c] = acc;
            __syncthreads();
            if (h == 0 && c < cols) {
                const float scaled = v[c] * (acc + half_sum[c]);  // kappa x the column sum
                const float sum = scaled * kappa_inv;
                const bool doit = sum > eps;
                v[c] = doit ? v[c] / scaled : v[c] * kappa_inv;
                if (sc) sc[(t * 2 + 1) * kSkMax + c] = doit ? sum : -1.0f;
            }
        }
        __syncthreads();
    }
    if (out) {
        float *O = out + (size_t)blockIdx.x * rows * cols;
        for (int e = tid; e < rows * cols; e += 256) O[e] = u[e / cols] * A[e] * v[e % cols];
    }
}

// Exact reverse sweep; d_inp doubles as the running gradient buffer.
__global__ __launch_bounds__(256) void sinkhorn_plain_bwd_kernel(const float *__restrict__ grad,
                                                                 const float *__restrict__ inp,
                                                                 float *__restrict__ d_inp, int rows,
                                                                 int cols, int T,
                                                                 const float *__restrict__ scal) {
    __shared__ float u[kSkMax], v[kSkMax], cdot[kSkMax], rdot[kSkMax], half_sum[kSkMax];
    const int tid = threadIdx.x;
    const float *A = inp + (size_t)blockIdx.x * rows * cols;
    const float *G = grad + (size_t)blockIdx.x * rows * cols;
    float *dO = d_inp + (size_t)blockIdx.x * rows * cols;
    const float *sc = scal + (size_t)blockIdx.x * T * 2 * kSkMax;
    // u and v carry kappa^t and kappa^-t like the forward kernel's (see there)
    const float kappa = (float)cols / (float)rows, kappa_inv = (float)rows / (float)cols;
    if (tid < kSkMax) {
        float uu = 1.f, vv = 1.f;
        for (int t = 0; t < T; t++) {
            uu = uu / fabsf(sc[(t * 2) * kSkMax + tid]) * kappa;  // entries beyond rows/cols are masked below
            vv = vv / fabsf(sc[(t * 2 + 1) * kSkMax + tid]) * kappa_inv;
        }
        u[tid] = tid < rows ? uu : 0.f;
        v[tid] = tid < cols ? vv : 0.f;
    }
    for (int e = tid; e < rows * cols; e += 256) dO[e] = G[e];
    __syncthreads();
    for (int t = T - 1; t >= 0; t--) {
        const float *rho = sc + (t * 2) * kSkMax, *s = sc + (t * 2 + 1) * kSkMax;
        // column dots with Out = u A v (skipped columns have divisor 1 and no sum dependence)
        {
            const int c = tid & 127, h = tid >> 7;
            float acc = 0.f;
            if (c < cols)
                for (int r = h; r < rows; r += 2) acc += dO[r * cols + c] * u[r] * A[r * cols + c];
            if (h == 1) half_sum[c] = acc;
            __syncthreads();
            if (h == 0 && c < cols) cdot[c] = s[c] > 0.f ? (acc + half_sum[c]) * v[c] : 0.f;
        }
        __syncthreads();
        // row dots with R = u A v s and dR = (dO - cdot) / s
        {
            const int r = tid >> 1, h = tid & 1;
            float acc = 0.f;
            if (r < rows)
                for (int c = h; c < cols; c += 2) acc += (dO[r * cols + c] - cdot[c]) * A[r * cols + c] * v[c];
            acc += __shfl_xor(acc, 1, kWave);
            if (r < rows && h == 0) rdot[r] = rho[r] > 0.f ? acc * u[r] : 0.f;
        }
        __syncthreads();
        for (int e = tid; e < rows * cols; e += 256) {
            const int r = e / cols, c = e % cols;
            dO[e] = ((dO[e] - cdot[c]) / fabsf(s[c]) - rdot[r]) / fabsf(rho[r]);
        }
        __syncthreads();
        if (tid < rows) u[tid] *= fabsf(rho[tid]) * kappa_inv;
        if (tid < cols) v[tid] *= fabsf(s[tid]) * kappa;
        __syncthreads();
    }
}

// --------------------------------------------------------------------------------------------
// Square matrices up to 8 x 8: one element per lane (four 4 x 4 matrices or one 8 x 8 matrix per wave,
// the lane layout and the DPP reductions of SkSmall), the whole iteration in registers.  Same
// operator: no exp, a row / column is divided only where its sum exceeds eps.  BWD: the forward keeps
// the divisors in LDS (-1 where the division was skipped) and the reverse sweep follows in the same
// launch; it rebuilds the iterates by multiplying the divisors back.
// --------------------------------------------------------------------------------------------
template <int NP, bool BWD>
__global__ __launch_bounds__(64) void sinkhorn_small_kernel(const float *__restrict__ inp, float *__restrict__ out,
                                                            const float *__restrict__ grad, float *__restrict__ d_inp,
                                                            int batch, int n, int T, float eps) {
    using SK = SkSmall<NP>;
    extern __shared__ float sc[];  // BWD: [T][2][64] divisors per lane
    const int lane = threadIdx.x, g = lane % SK::kGroup;
    const int b = blockIdx.x * SK::kPerWave + lane / SK::kGroup;
    const int r = SK::row(g), c = SK::col0(g);
    const bool ok = b < batch && r < n && c < n;  // lanes of absent matrices run on zeros
    const size_t e = ok ? (size_t)b * n * n + r * n + c : 0;
    float m = ok ? inp[e] : 0.f;
    float d = 0.f;
    if constexpr (BWD) d = ok ? grad[e] : 0.f;
    for (int t = 0; t < T; t++) {
        const float rs = SK::row_allreduce(m);
        const bool dr = rs > eps;
        m = dr ? m / rs : m;
        const float cs = SK::col_allreduce(m);
        const bool dc = cs > eps;
        m = dc ? m / cs : m;
        if constexpr (BWD) {
            sc[(t * 2) * 64 + lane] = dr ? rs : -1.0f;
            sc[(t * 2 + 1) * 64 + lane] = dc ? cs : -1.0f;
        }
    }
    if constexpr (!BWD) {
        if (ok) out[e] = m;
        return;
    } else {
        // through column step t: Out = R / s, dR = (dOut - sum_col(dOut Out)) / s; then the row step alike
        for (int t = T - 1; t >= 0; t--) {
            const float rs = sc[(t * 2) * 64 + lane], cs = sc[(t * 2 + 1) * 64 + lane];
            // (selects, not branches: the reductions run on every lane)
            const float cdot = SK::col_allreduce(d * m);
            d = cs > 0.f ? (d - cdot) / cs : d;
            m = cs > 0.f ? m * cs : m;
            const float rdot = SK::row_allreduce(d * m);
            d = rs > 0.f ? (d - rdot) / rs : d;
            m = rs > 0.f ? m * rs : m;
        }
        if (ok) d_inp[e] = d;
    }
}

static bool sinkhorn_small_supported(int rows, int cols, int T) { return rows == cols && rows <= 8 && T <= 96; }

template <bool BWD>
static hipError_t launch_sinkhorn_small(const float *inp, float *out, const float *grad, float *d_inp, int batch,
                                        int n, int T, float eps, hipStream_t stream) {
    const size_t smem = BWD ? sizeof(float) * (size_t)(T > 0 ? T : 1) * 2 * 64 : 0;
    if (n <= 4) {
        sinkhorn_small_kernel<4, BWD><<<(batch + 3) / 4, 64, smem, stream>>>(inp, out, grad, d_inp, batch, n, T, eps);
    } else {
        sinkhorn_small_kernel<8, BWD><<<batch, 64, smem, stream>>>(inp, out, grad, d_inp, batch, n, T, eps);
    }
    return hipGetLastError();
}

hipError_t launch_sinkhorn_plain_fwd(const float *inp, float *out, int batch, int rows, int cols,
                                     int T, float eps, hipStream_t stream) {
    if (sinkhorn_small_supported(rows, cols, T))
        return launch_sinkhorn_small<false>(inp, out, nullptr, nullptr, batch, rows, T, eps, stream);
    sinkhorn_plain_fwd_kernel<<<batch, 256, 0, stream>>>(inp, out, rows, cols, T, eps, nullptr);
    return hipGetLastError();
}

hipError_t launch_sinkhorn_plain_bwd(const float *grad, const float *inp, float *d_inp, int batch,
                                     int rows, int cols, int T, float eps, float *scal,
                                     hipStream_t stream) {
    if (sinkhorn_small_supported(rows, cols, T))
        return launch_sinkhorn_small<true>(inp, nullptr, grad, d_inp, batch, rows, T, eps, stream);
    sinkhorn_plain_fwd_kernel<<<batch, 256, 0, stream>>>(inp, nullptr, rows, cols, T, eps, scal);
    hipError_t e = hipGetLastError();
    if (e != hipSuccess) return e;
    sinkhorn_plain_bwd_kernel<<<batch, 256, 0, stream>>>(grad, inp, d_inp, rows, cols, T, scal);
    return hipGetLastError();
}

// --------------------------------------------------------------------------------------------
// RMSNorm
// --------------------------------------------------------------------------------------------
__device__ __forceinline__ float load_w3(const void *w, int w_bf16, int c) {
    return w_bf16 ? bf16_to_f32(static_cast<const bf16_t *>(w)[c]) : static_cast<const float *>(w)[c];
}

template <typename T>
__global__ __launch_bounds__(256) void rmsnorm_fwd_kernel(const T *__restrict__ inp, const void *w,
                                                          int w_bf16, T *__restrict__ out,
                                                          float *__restrict__ rms, int C, float eps) {
    __shared__ float red[4];
    const int row = blockIdx.x, tid = threadIdx.x;
    const T *x = inp + (size_t)row * C;
    float ssq = 0.f;
    for (int c = tid; c < C; c += 256) { const float v = to_f32<T>(x[c]); ssq += v * v; }
    ssq = block_allreduce_sum<256>(ssq, red);
    const float r = sqrtf(ssq / (float)C + eps);
    if (tid == 0 && rms) rms[row] = r;
    const float rinv = 1.0f / r;
    for (int c = tid; c < C; c += 256)
        out[(size_t)row * C + c] = from_f32<T>(to_f32<T>(x[c]) * rinv * load_w3(w, w_bf16, c));
}

// d_inp = g w / r - x (sum g w x) / (C r^3);  u = g x / r  (column-summed into d_w afterwards)
template <typename T>
__global__ __launch_bounds__(256) void rmsnorm_bwd_kernel(const T *__restrict__ grad,
                                                          const T *__restrict__ inp, const void *w,
                                                          int w_bf16, const float *__restrict__ rms,
                                                          T *__restrict__ d_inp, float *__restrict__ u,
                                                          int C) {
    __shared__ float red[4];
    const int row = blockIdx.x, tid = threadIdx.x;
    const T *x = inp + (size_t)row * C, *g = grad + (size_t)row * C;
    const float rinv = 1.0f / rms[row];
    float dot = 0.f;
    for (int c = tid; c < C; c += 256) dot += to_f32<T>(g[c]) * load_w3(w, w_bf16, c) * to_f32<T>(x[c]);
    dot = block_allreduce_sum<256>(dot, red);
    const float k2 = dot * rinv * rinv * rinv / (float)C;
    for (int c = tid; c < C; c += 256) {
        const float gv = to_f32<T>(g[c]), xv = to_f32<T>(x[c]);
        d_inp[(size_t)row * C + c] = from_f32<T>(gv * load_w3(w, w_bf16, c) * rinv - xv * k2);
        u[(size_t)row * C + c] = gv * xv * rinv;
    }
}

// --------------------------------------------------------------------------------------------
// Rows in registers: TPR threads share a row (64: one wave, four rows per workgroup; 256: the whole
// workgroup), a thread holds VPT 16-byte pieces of it (piece k of thread t = columns (k TPR + t) V ...),
// all requested before the first is used.  One pass over the row: x is read once (forward) and dy and
// x once (backward), 16-byte loads and stores.  Needs C % V == 0, 16-byte aligned rows and
// C <= TPR * V * VPT; other shapes take the kernels above.
// --------------------------------------------------------------------------------------------
template <int V> __device__ __forceinline__ void load_w_vec(const void *w, int w_bf16, int c, float (&wv)[V]) {
    if (w_bf16) load_vec<bf16_t, V>(static_cast<const bf16_t *>(w) + c, wv);
    else load_vec<float, V>(static_cast<const float *>(w) + c, wv);
}

template <int TPR> __device__ __forceinline__ float row_allreduce(float v, float *red) {
    if constexpr (TPR == 64) return wave_allreduce_sum(v);
    else return block_allreduce_sum<256>(v, red);
}

template <typename T, int VPT, int TPR>
__global__ __launch_bounds__(256) void rmsnorm_fwd_rows_kernel(const T *__restrict__ inp, const void *w, int w_bf16,
                                                               T *__restrict__ out, float *__restrict__ rms,
                                                               int rows, int C, float eps) {
    constexpr int V = 16 / (int)sizeof(T), RPW = 256 / TPR;
    __shared__ float red[4];
    const int tid = threadIdx.x, t = tid % TPR;
    const int row = blockIdx.x * RPW + tid / TPR;
    const bool live = row < rows;  // TPR == 64: whole waves; nothing below synchronises across waves
    const T *x = inp + (size_t)(live ? row : 0) * C;
    RawVec<T, V> xr[VPT];
#pragma unroll
    for (int k = 0; k < VPT; k++) {
        const int c = (k * TPR + t) * V;
        xr[k].load(x + (c < C ? c : 0));
    }
    float ssq = 0.f;
#pragma unroll
    for (int k = 0; k < VPT; k++) {
        float v[V];
        xr[k].get(v);
        if ((k * TPR + t) * V < C) {
#pragma unroll
            for (int j = 0; j < V; j++) ssq += v[j] * v[j];
        }
    }
    ssq = row_allreduce<TPR>(ssq, red);
    const float r = sqrtf(ssq / (float)C + eps);
    if (t == 0 && rms && live) rms[row] = r;
    const float rinv = 1.0f / r;
    if (!live) return;
#pragma unroll
    for (int k = 0; k < VPT; k++) {
        const int c = (k * TPR + t) * V;
        if (c < C) {
            float v[V], wv[V];
            xr[k].get(v);
            load_w_vec<V>(w, w_bf16, c, wv);
#pragma unroll
            for (int j = 0; j < V; j++) v[j] = v[j] * rinv * wv[j];
            store_vec<T, V, true>(out + (size_t)row * C + c, v);
        }
    }
}

// Backward, persistent: workgroup g takes the row groups g, g + gridDim.x, ...; a thread keeps the dw
// terms of its own columns in registers over all its rows and writes them once, as row
// (blockIdx.x * RPW + row lane) of `part` [gridDim.x * RPW][C]; a column sum over those rows gives dw.
template <typename T, int VPT, int TPR>
__global__ __launch_bounds__(256) void rmsnorm_bwd_rows_kernel(const T *__restrict__ grad, const T *__restrict__ inp,
                                                               const void *w, int w_bf16, const float *__restrict__ rms,
                                                               T *__restrict__ d_inp, float *__restrict__ part,
                                                               int rows, int C) {
    constexpr int V = 16 / (int)sizeof(T), RPW = 256 / TPR;
    __shared__ float red[4];
    const int tid = threadIdx.x, t = tid % TPR, rl = tid / TPR;
    float acc[VPT][V];
#pragma unroll
    for (int k = 0; k < VPT; k++)
#pragma unroll
        for (int j = 0; j < V; j++) acc[k][j] = 0.f;
    const int ngroups = (rows + RPW - 1) / RPW;
    for (int grp = blockIdx.x; grp < ngroups; grp += gridDim.x) {
        const int row = grp * RPW + rl;
        const bool live = row < rows;
        const size_t base = (size_t)(live ? row : 0) * C;
        RawVec<T, V> xr[VPT], gr[VPT];
#pragma unroll
        for (int k = 0; k < VPT; k++) {
            const int c = (k * TPR + t) * V, cc = c < C ? c : 0;
            xr[k].load(inp + base + cc);
            gr[k].load(grad + base + cc);
        }
        const float rinv = 1.0f / rms[live ? row : 0];
        float dot = 0.f;
#pragma unroll
        for (int k = 0; k < VPT; k++) {
            const int c = (k * TPR + t) * V;
            if (c < C) {
                float xv[V], gv[V], wv[V];
                xr[k].get(xv); gr[k].get(gv);
                load_w_vec<V>(w, w_bf16, c, wv);
#pragma unroll
                for (int j = 0; j < V; j++) dot += gv[j] * wv[j] * xv[j];
            }
        }
        dot = row_allreduce<TPR>(dot, red);  // TPR == 256: every thread of the workgroup gets here (grp is uniform)
        const float k2 = dot * rinv * rinv * rinv / (float)C;
#pragma unroll
        for (int k = 0; k < VPT; k++) {
            const int c = (k * TPR + t) * V;
            if (c < C && live) {
                float xv[V], gv[V], wv[V], dv[V];
                xr[k].get(xv); gr[k].get(gv);
                load_w_vec<V>(w, w_bf16, c, wv);
#pragma unroll
                for (int j = 0; j < V; j++) {
                    dv[j] = gv[j] * wv[j] * rinv - xv[j] * k2;
                    acc[k][j] += gv[j] * xv[j] * rinv;
                }
                store_vec<T, V, true>(d_inp + base + c, dv);
            }
        }
    }
    float *prow = part + (size_t)(blockIdx.x * RPW + rl) * C;
#pragma unroll
    for (int k = 0; k < VPT; k++) {
        const int c = (k * TPR + t) * V;
        if (c < C) store_vec<float, V>(prow + c, acc[k]);
    }
}

// VPT (pieces per thread) and TPR (threads per row) of the row kernels, 0 when the shape does not fit
static int rows_kernel_vpt(int dtype, int C, int max_vpt, int *tpr) {
    const int V = dtype == kBF16 ? 8 : 4;
    if (C % V != 0) return 0;
    const int pieces = C / V;
    *tpr = pieces <= 64 * 4 ? 64 : 256;
    const int need = (pieces + *tpr - 1) / *tpr;
    for (int v : {1, 2, 4, 8, 16})
        if (need <= v) return v <= max_vpt ? v : 0;
    return 0;
}
static bool aligned16_(const void *p) { return (reinterpret_cast<uintptr_t>(p) & 15) == 0; }

// number of partial dw rows the backward row kernel writes (0: the generic kernel runs, rows of u)
int rmsnorm_bwd_partial_rows(int dtype, int rows, int C) {
    int tpr = 0;
    if (rows_kernel_vpt(dtype, C, 8, &tpr) == 0) return 0;
    const int rpw = 256 / tpr, groups = (rows + rpw - 1) / rpw;
    return (groups < 1024 ? groups : 1024) * rpw;
}

hipError_t launch_rmsnorm_fwd(const void *inp, int dtype, const void *w, int w_dtype, void *out,
                              float *rms, int rows, int C, float eps, hipStream_t stream) {
    int tpr = 0;
    const int vpt = rows_kernel_vpt(dtype, C, 16, &tpr);
    if (vpt && aligned16_(inp) && aligned16_(out) && aligned16_(w)) {
        const int wb = w_dtype == kBF16, grid = (rows + 256 / tpr - 1) / (256 / tpr);
#define MHC_RMS_FWD(T, VPT, TPR) \
    rmsnorm_fwd_rows_kernel<T, VPT, TPR><<<grid, 256, 0, stream>>>(static_cast<const T *>(inp), w, wb, static_cast<T *>(out), rms, rows, C, eps)
#define MHC_RMS_FWD_T(T)                                                                  \
    do {                                                                                  \
        if (tpr == 64) { if (vpt == 1) MHC_RMS_FWD(T, 1, 64); else if (vpt == 2) MHC_RMS_FWD(T, 2, 64); else MHC_RMS_FWD(T, 4, 64); } \
        else if (vpt <= 2) MHC_RMS_FWD(T, 2, 256);                                        \
        else if (vpt == 4) MHC_RMS_FWD(T, 4, 256);                                        \
        else if (vpt == 8) MHC_RMS_FWD(T, 8, 256);                                        \
        else MHC_RMS_FWD(T, 16, 256);                                                     \
    } while (0)
        if (dtype == kBF16) MHC_RMS_FWD_T(bf16_t); else MHC_RMS_FWD_T(float);
#undef MHC_RMS_FWD_T
#undef MHC_RMS_FWD
        return hipGetLastError();
    }
    if (dtype == kBF16)
        rmsnorm_fwd_kernel<bf16_t><<<rows, 256, 0, stream>>>(static_cast<const bf16_t *>(inp), w, w_dtype == kBF16,
                                                             static_cast<bf16_t *>(out), rms, C, eps);
    else
        rmsnorm_fwd_kernel<float><<<rows, 256, 0, stream>>>(static_cast<const float *>(inp), w, w_dtype == kBF16,
                                                            static_cast<float *>(out), rms, C, eps);
    return hipGetLastError();
}

// u: rows x C floats of workspace.  *u_rows receives the number of rows of u whose column sums are dw:
// `rows` from the generic kernel, rmsnorm_bwd_partial_rows() from the row kernel.
hipError_t launch_rmsnorm_bwd(const void *grad, const void *inp, int dtype, const void *w,
                              int w_dtype, const float *rms, void *d_inp, float *u, int rows, int C,
                              int *u_rows, hipStream_t stream) {
    int tpr = 0;
    const int vpt = rows_kernel_vpt(dtype, C, 8, &tpr);
    if (vpt && aligned16_(grad) && aligned16_(inp) && aligned16_(d_inp) && aligned16_(w) && aligned16_(u)) {
        const int wb = w_dtype == kBF16, rpw = 256 / tpr;
        const int prow = rmsnorm_bwd_partial_rows(dtype, rows, C), grid = prow / rpw;
        *u_rows = prow;
#define MHC_RMS_BWD(T, VPT, TPR) \
    rmsnorm_bwd_rows_kernel<T, VPT, TPR><<<grid, 256, 0, stream>>>(static_cast<const T *>(grad), static_cast<const T *>(inp), w, wb, rms, static_cast<T *>(d_inp), u, rows, C)
#define MHC_RMS_BWD_T(T)                                                                  \
    do {                                                                                  \
        if (tpr == 64) { if (vpt == 1) MHC_RMS_BWD(T, 1, 64); else if (vpt == 2) MHC_RMS_BWD(T, 2, 64); else MHC_RMS_BWD(T, 4, 64); } \
        else if (vpt <= 2) MHC_RMS_BWD(T, 2, 256);                                        \
        else if (vpt == 4) MHC_RMS_BWD(T, 4, 256);                                        \
        else MHC_RMS_BWD(T, 8, 256);                                                      \
    } while (0)
        if (dtype == kBF16) MHC_RMS_BWD_T(bf16_t); else MHC_RMS_BWD_T(float);
#undef MHC_RMS_BWD_T
#undef MHC_RMS_BWD
        return hipGetLastError();
    }
    *u_rows = rows;
    if (dtype == kBF16)
        rmsnorm_bwd_kernel<bf16_t><<<rows, 256, 0, stream>>>(static_cast<const bf16_t *>(grad),
                                                             static_cast<const bf16_t *>(inp), w, w_dtype == kBF16,
                                                             rms, static_cast<bf16_t *>(d_inp), u, C);
    else
        rmsnorm_bwd_kernel<float><<<rows, 256, 0, stream>>>(static_cast<const float *>(grad),
                                                            static_cast<const float *>(inp), w, w_dtype == kBF16,
                                                            rms, static_cast<float *>(d_inp), u, C);
    return hipGetLastError();
}

}  // namespace mhc
