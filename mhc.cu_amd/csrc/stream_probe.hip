// Streaming kernels that do nothing but move bytes: what this GPU delivers to a read-only, a copy
// and a write-only pass over a large buffer, and what an empty launch costs.  They give the
// memory-bound kernels of the library a measured ceiling next to the published 8 TB/s.  Not part of
// the layer path and not part of libmhc_hip.so: this file is built into its own libmhc_probe.so
// (build.py), which only bench.py --stream-probe and its test load.
#include <hip/hip_runtime.h>
#include <stdint.h>

namespace {

typedef uint32_t u32x4 __attribute__((ext_vector_type(4)));

// grid-stride over 16-byte words, UNROLL independent loads in flight per lane
template <bool NT> __device__ __forceinline__ u32x4 ld(const u32x4 *p) {
    if constexpr (NT) return __builtin_nontemporal_load(p);
    else return *p;
}
template <bool NT> __device__ __forceinline__ void st(u32x4 v, u32x4 *p) {
    if constexpr (NT) __builtin_nontemporal_store(v, p);
    else *p = v;
}

template <int UNROLL, bool NT>
__global__ __launch_bounds__(256) void probe_read_kernel(const u32x4 *__restrict__ src, size_t words, uint32_t *sink) {
    const size_t stride = (size_t)gridDim.x * 256;
    size_t i = (size_t)blockIdx.x * 256 + threadIdx.x;
    uint32_t acc = 0;
    for (; i + (UNROLL - 1) * stride < words; i += UNROLL * stride) {
        u32x4 v[UNROLL];
#pragma unroll
        for (int u = 0; u < UNROLL; u++) v[u] = ld<NT>(src + i + u * stride);
#pragma unroll
        for (int u = 0; u < UNROLL; u++) acc ^= v[u][0] ^ v[u][1] ^ v[u][2] ^ v[u][3];
    }
    for (; i < words; i += stride) {
        const u32x4 v = src[i];
        acc ^= v[0] ^ v[1] ^ v[2] ^ v[3];
    }
    if (acc == 0x9e3779b9u) *sink = acc;  // keeps the loads alive; practically never taken
}

template <int UNROLL, bool NT>
__global__ __launch_bounds__(256) void probe_copy_kernel(const u32x4 *__restrict__ src, u32x4 *__restrict__ dst, size_t words) {
    const size_t stride = (size_t)gridDim.x * 256;
    size_t i = (size_t)blockIdx.x * 256 + threadIdx.x;
    for (; i + (UNROLL - 1) * stride < words; i += UNROLL * stride) {
        u32x4 v[UNROLL];
#pragma unroll
        for (int u = 0; u < UNROLL; u++) v[u] = ld<NT>(src + i + u * stride);
#pragma unroll
        for (int u = 0; u < UNROLL; u++) st<NT>(v[u], dst + i + u * stride);
    }
    for (; i < words; i += stride) dst[i] = src[i];
}

template <bool NT>
__global__ __launch_bounds__(256) void probe_write_kernel(u32x4 *__restrict__ dst, size_t words, uint32_t value) {
    const size_t stride = (size_t)gridDim.x * 256;
    const u32x4 v = {value, value, value, value};
    for (size_t i = (size_t)blockIdx.x * 256 + threadIdx.x; i < words; i += stride) st<NT>(v, dst + i);
}

__global__ void probe_empty_kernel() {}  // launch floor: nothing to do

}  // namespace

// mode 0 = read-only, 1 = copy, 2 = write-only, with the streaming (nt) hint on every access; 3, 4, 5 =
// the same with plain loads and stores; 6 = a kernel that does nothing (launch floor: src, dst, sink and
// bytes unused).  bytes: size of src and of dst, a multiple of 16; blocks = grid size (0: 256 CUs x 8;
// at most 2^20); sink: 4 bytes of device memory (read-only modes).  Pointers a mode dereferences must be
// non-null and 16-byte aligned; everything is checked here, before any launch.  Returns the hipError_t
// of the launch, hipErrorInvalidValue for arguments that do not fit the mode.
extern "C" __attribute__((visibility("default"))) int mhc_stream_probe(int mode, const void *src, void *dst, size_t bytes,
                                                                       int blocks, void *sink, void *stream) {
    if (mode < 0 || mode > 6 || blocks < 0 || blocks > (1 << 20)) return (int)hipErrorInvalidValue;
    const int grid = blocks > 0 ? blocks : 256 * 8;
    hipStream_t st = static_cast<hipStream_t>(stream);
    if (mode == 6) {
        probe_empty_kernel<<<grid, 256, 0, st>>>();
        return (int)hipGetLastError();
    }
    const bool reads = mode == 0 || mode == 1 || mode == 3 || mode == 4, writes = mode != 0 && mode != 3;
    const bool sinks = mode == 0 || mode == 3;
    auto misaligned = [](const void *p) { return (reinterpret_cast<uintptr_t>(p) & 15u) != 0; };
    if (bytes == 0 || bytes % 16) return (int)hipErrorInvalidValue;
    if ((reads && (!src || misaligned(src))) || (writes && (!dst || misaligned(dst))) || (sinks && !sink))
        return (int)hipErrorInvalidValue;
    const size_t words = bytes / 16;
    const u32x4 *s = static_cast<const u32x4 *>(src);
    u32x4 *d = static_cast<u32x4 *>(dst);
    if (mode == 0) probe_read_kernel<8, true><<<grid, 256, 0, st>>>(s, words, static_cast<uint32_t *>(sink));
    else if (mode == 1) probe_copy_kernel<4, true><<<grid, 256, 0, st>>>(s, d, words);
    else if (mode == 2) probe_write_kernel<true><<<grid, 256, 0, st>>>(d, words, 0x3f800000u);
    else if (mode == 3) probe_read_kernel<8, false><<<grid, 256, 0, st>>>(s, words, static_cast<uint32_t *>(sink));
    else if (mode == 4) probe_copy_kernel<4, false><<<grid, 256, 0, st>>>(s, d, words);
    else probe_write_kernel<false><<<grid, 256, 0, st>>>(d, words, 0x3f800000u);
    return (int)hipGetLastError();
}
