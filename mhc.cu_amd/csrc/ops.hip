// Stand-alone operators: Sinkhorn-Knopp on plain rows x cols matrices and row-wise RMSNorm,
// forward and backward.  Semantics of the reference's operator-level CPU references:
// src/csrc/tests/test_sinkhorn_knopp.cu:16-47 (no exp; divide only where the sum exceeds eps),
// src/csrc/tests/test_rmsnorm.cu:17-30 and test_rmsnorm_backward.cu:17-39.
#include "launchers.h"
#include "mhc_common.h"

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

hipError_t launch_sinkhorn_plain_fwd(const float *inp, float *out, int batch, int rows, int cols,
                                     int T, float eps, hipStream_t stream) {
    sinkhorn_plain_fwd_kernel<<<batch, 256, 0, stream>>>(inp, out, rows, cols, T, eps, nullptr);
    return hipGetLastError();
}

hipError_t launch_sinkhorn_plain_bwd(const float *grad, const float *inp, float *d_inp, int batch,
                                     int rows, int cols, int T, float eps, float *scal,
                                     hipStream_t stream) {
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

hipError_t launch_rmsnorm_fwd(const void *inp, int dtype, const void *w, int w_dtype, void *out,
                              float *rms, int rows, int C, float eps, hipStream_t stream) {
    if (dtype == kBF16)
        rmsnorm_fwd_kernel<bf16_t><<<rows, 256, 0, stream>>>(static_cast<const bf16_t *>(inp), w, w_dtype == kBF16,
                                                             static_cast<bf16_t *>(out), rms, C, eps);
    else
        rmsnorm_fwd_kernel<float><<<rows, 256, 0, stream>>>(static_cast<const float *>(inp), w, w_dtype == kBF16,
                                                            static_cast<float *>(out), rms, C, eps);
    return hipGetLastError();
}

hipError_t launch_rmsnorm_bwd(const void *grad, const void *inp, int dtype, const void *w,
                              int w_dtype, const float *rms, void *d_inp, float *u, int rows, int C,
                              hipStream_t stream) {
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
