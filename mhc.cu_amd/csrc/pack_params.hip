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

template <typename TS, typename TD, int V>
__global__ __launch_bounds__(256) void pack_params_kernel(PackArgs a) {
    const size_t e0 = ((size_t)blockIdx.x * 256 + threadIdx.x) * V;
    if (blockIdx.x == 0) {
        const int t = threadIdx.x;
        if (t < 3) a.alpha[t] = a.alpha_in[t][0];
        for (int i = t; i < a.bn[0] + a.bn[1] + a.bn[2]; i += 256) {
            const int g = i < a.bn[0] ? 0 : (i < a.bn[0] + a.bn[1] ? 1 : 2);
            const int off = g == 0 ? 0 : (g == 1 ? a.bn[0] : a.bn[0] + a.bn[1]);
            a.bias[i] = a.b[g][i - off];
        }
    }
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
