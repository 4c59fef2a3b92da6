// Gathers the dynamic-H parameters of MHCLayer (three phi matrices, three biases, three alpha
// scalars, reference src/python/mhc/layer.py:44-54) into the arrays the layer entry points take:
// phi [D, nC] in the compute dtype, bias [D], alpha [3].  One launch instead of the reference's
// torch.cat(...).bfloat16() and three .item() synchronisations per forward call
// (src/python/mhc/ops.py:172-188).  The rows of the concatenation are contiguous, so phi is the
// plain concatenation of the three flat arrays.
#include "launchers.h"
#include "mhc_common.h"

namespace mhc {

struct PackArgs {
    const void *src[3];
    size_t end[3];  // flat end offset of each source in the concatenation
    const float *b[3];
    int bn[3];
    const float *alpha_in[3];
    void *phi_out;
    float *bias, *alpha;
    size_t total;
};

// Small parameters (biases, alphas): workgroup 0 of either kernel below.
__device__ __forceinline__ void pack_small(const PackArgs &a, int t) {
    if (t < 3) a.alpha[t] = a.alpha_in[t][0];
    for (int i = t; i < a.bn[0] + a.bn[1] + a.bn[2]; i += 256) {
        const int g = i < a.bn[0] ? 0 : (i < a.bn[0] + a.bn[1] ? 1 : 2);
        const int off = g == 0 ? 0 : (g == 1 ? a.bn[0] : a.bn[0] + a.bn[1]);
        a.bias[i] = a.b[g][i - off];
    }
}

template <typename TS, typename TD, int V>
__global__ __launch_bounds__(256) void pack_params_kernel(PackArgs a) {
    const size_t e0 = ((size_t)blockIdx.x * 256 + threadIdx.x) * V;
    if (blockIdx.x == 0) pack_small(a, threadIdx.x);
    if (e0 >= a.total) return;
    // V > 1 only when every source length is a multiple of V: a chunk never straddles two sources
    const int g = e0 < a.end[0] ? 0 : (e0 < a.end[1] ? 1 : 2);
    const size_t base = g == 0 ? 0 : a.end[g - 1];
    const TS *src = static_cast<const TS *>(a.src[g]) + (e0 - base);
    TD *dst = static_cast<TD *>(a.phi_out) + e0;
    float v[V];
    load_vec<TS, V>(src, v);
    store_vec<TD, V>(dst, v);
}

// float32 parameters into a bfloat16 phi, the case of a training step (master weights in fp32, 6 bytes
// moved per element: 267 MB for n = 32, C = 1280).  A lane takes four elements per chunk (a 16-byte
// load, an 8-byte store, both contiguous across the wave), a thread keeps kPackU chunks in flight and
// the grid is a few thousand workgroups that stride over the array; the sources are read once and
// bypass the caches (nontemporal loads), phi stays cached for the projection kernel that follows.
constexpr int kPackU = 8;
__global__ __launch_bounds__(256) void pack_params_stream_kernel(PackArgs a) {
    if (blockIdx.x == 0) pack_small(a, threadIdx.x);
    const size_t chunks = a.total / 4;  // every source length is a multiple of 4
    const size_t per_round = (size_t)gridDim.x * kPackU * 256;
    for (size_t c0 = (size_t)blockIdx.x * kPackU * 256 + threadIdx.x; c0 < chunks; c0 += per_round) {
        uint4 v[kPackU];
#pragma unroll
        for (int u = 0; u < kPackU; u++) {
            const size_t c = c0 + (size_t)u * 256;
            const size_t e = (c < chunks ? c : 0) * 4;
            const int g = e < a.end[0] ? 0 : (e < a.end[1] ? 1 : 2);
            const size_t base = g == 0 ? 0 : a.end[g - 1];
            v[u] = ldg16_stream(reinterpret_cast<const uint4 *>(static_cast<const float *>(a.src[g]) + (e - base)));
        }
#pragma unroll
        for (int u = 0; u < kPackU; u++) {
            const size_t c = c0 + (size_t)u * 256;
            if (c < chunks)
                st8<false>(static_cast<bf16_t *>(a.phi_out) + c * 4,
                           pack_bf16x2(__uint_as_float(v[u].x), __uint_as_float(v[u].y)),
                           pack_bf16x2(__uint_as_float(v[u].z), __uint_as_float(v[u].w)));
        }
    }
}

hipError_t launch_pack_params(const void *phi_pre, const void *phi_post, const void *phi_res, int src_dtype,
                              const float *b_pre, const float *b_post, const float *b_res,
                              const float *alpha_pre, const float *alpha_post, const float *alpha_res,
                              void *phi_out, int out_dtype, float *bias, float *alpha, int n, int C,
                              hipStream_t stream) {
    const size_t nC = (size_t)n * C, rows[3] = {(size_t)n, (size_t)n, (size_t)n * n};
    PackArgs a;
    a.src[0] = phi_pre; a.src[1] = phi_post; a.src[2] = phi_res;
    size_t end = 0;
    for (int i = 0; i < 3; i++) { end += rows[i] * nC; a.end[i] = end; }
    a.b[0] = b_pre; a.b[1] = b_post; a.b[2] = b_res;
    a.bn[0] = n; a.bn[1] = n; a.bn[2] = n * n;
    a.alpha_in[0] = alpha_pre; a.alpha_in[1] = alpha_post; a.alpha_in[2] = alpha_res;
    a.phi_out = phi_out; a.bias = bias; a.alpha = alpha; a.total = end;
    auto al16 = [](const void *p) { return (reinterpret_cast<uintptr_t>(p) & 15u) == 0; };
    // the streaming kernel: fp32 -> bf16, whole 16-byte chunks in every source, enough of them to matter
    if (src_dtype == kF32 && out_dtype == kBF16 && (n * nC) % 4 == 0 && al16(phi_pre) && al16(phi_post) &&
        al16(phi_res) && (reinterpret_cast<uintptr_t>(phi_out) & 7u) == 0 && end >= (size_t)1 << 20) {
        const size_t rounds = (end / 4 + (size_t)kPackU * 256 - 1) / ((size_t)kPackU * 256);
        pack_params_stream_kernel<<<(unsigned)(rounds < 2048 ? rounds : 2048), 256, 0, stream>>>(a);
        return hipGetLastError();
    }
    const bool vec = (n * nC) % 8 == 0 && al16(phi_pre) && al16(phi_post) && al16(phi_res) && al16(phi_out);
    const int V = vec ? 8 : 1;
    const size_t chunks = (end + V - 1) / V;
    const unsigned grid = (unsigned)((chunks + 255) / 256);
#define MHC_PACK(TS, TD)                                                        \
    do {                                                                        \
        if (vec) pack_params_kernel<TS, TD, 8><<<grid, 256, 0, stream>>>(a);    \
        else pack_params_kernel<TS, TD, 1><<<grid, 256, 0, stream>>>(a);        \
    } while (0)
    if (src_dtype == kF32 && out_dtype == kF32) MHC_PACK(float, float);
    else if (src_dtype == kF32 && out_dtype == kBF16) MHC_PACK(float, bf16_t);
    else if (src_dtype == kBF16 && out_dtype == kBF16) MHC_PACK(bf16_t, bf16_t);
    else if (src_dtype == kBF16 && out_dtype == kF32) MHC_PACK(bf16_t, float);
    else return hipErrorInvalidValue;
#undef MHC_PACK
    return hipGetLastError();
}

}  // namespace mhc
