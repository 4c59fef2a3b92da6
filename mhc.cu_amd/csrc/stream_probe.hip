// Streaming kernels that do nothing but move bytes: what this GPU delivers to a read-only, a copy
// and a write-only pass over a large buffer.  They give the memory-bound kernels of the library a
// measured ceiling next to the published 8 TB/s.  Not part of the layer path; exported for
// bench.py --stream-probe and --handoff-probe only (no declaration in the public header).
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

__global__ void probe_empty_kernel(uint32_t *sink) {
    if (sink == nullptr) __builtin_trap();  // never: the kernel has nothing to do
}

// Hand-off probe: what it costs to pass data between the workgroups of ONE kernel instead of between
// two kernels.  Every workgroup writes `per` floats, all workgroups meet, every workgroup then sums its
// slice of every workgroup's floats.  ONE: in one kernel - the floats leave with agent-scope relaxed atomic
// stores (write-through, no cache write-back needed), one thread per workgroup counts its arrival with an
// agent-scope atomic and polls the counter, the readers use agent-scope relaxed atomic loads; no fence
// instruction anywhere.  The last workgroup to leave resets the counters, so launches need no host state.
// The wait is bounded: a workgroup that gives up raises sync[2] and the results are garbage, but the kernel
// ends.  PHASE 0 / 1: the same two halves as separate kernels with plain stores and loads.
template <bool ONE, int PHASE>
__global__ __launch_bounds__(256) void probe_handoff_kernel(float *part, float *out, unsigned *sync, int per) {
    const int wg = blockIdx.x, N = gridDim.x, tid = threadIdx.x;
    if (ONE || PHASE == 0) {
        float *mine = part + (size_t)wg * per;
        const float v = (float)(wg + 1);
        for (int i = tid; i < per; i += 256) {
            if (ONE) __hip_atomic_store(mine + i, v, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
            else mine[i] = v;
        }
    }
    if (ONE) {
        __builtin_amdgcn_s_waitcnt(0);  // every store of this wave has been acknowledged
        __syncthreads();
        if (tid == 0) {
            __hip_atomic_fetch_add(sync, 1u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
            unsigned spins = 0;
            while (__hip_atomic_load(sync, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT) < (unsigned)N) {
                __builtin_amdgcn_s_sleep(1);
                if (++spins > 2000000u) { sync[2] = 1; break; }
            }
            if (__hip_atomic_fetch_add(sync + 1, 1u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT) == (unsigned)N - 1) {
                __hip_atomic_store(sync + 1, 0u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
                __hip_atomic_store(sync, 0u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
            }
        }
        __syncthreads();
    }
    if (ONE || PHASE == 1) {
        const int w = per / N;  // this workgroup's slice of every producer: floats [wg*w, wg*w + w)
        float s = 0.f;
        for (int i = tid; i < N * w; i += 256) {
            const float *p = part + (size_t)(i / w) * per + wg * w + i % w;
            s += ONE ? __hip_atomic_load(p, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT) : *p;
        }
        for (int o = 32; o; o >>= 1) s += __shfl_xor(s, o);
        __shared__ float sh[4];
        if ((tid & 63) == 0) sh[tid >> 6] = s;
        __syncthreads();
        if (tid == 0) out[wg] = (sh[0] + sh[1]) + (sh[2] + sh[3]);
    }
}

// Row-piece probe: what one workgroup of 8 waves pulls out of the L2 when every workgroup streams the
// SAME [24][nC] bf16 matrix the way the one-launch forward streams phi: 64 contraction elements per step,
// a wave fetches the step's 24 x 128 bytes row-contiguously (8 lanes per row piece), parks them in its own
// LDS tile and reads them back in operand layout, two steps in flight.  `reps` passes inside one launch, so
// the kernel start is amortised: the figure is the steady streaming rate of a CU, not a kernel time.
__global__ __launch_bounds__(512) void probe_row_pieces_kernel(const unsigned short *phi, int nC, uint32_t *sink, int reps) {
    __shared__ __align__(16) unsigned short tiles[8 * 32 * 72];
    const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
    const int steps = nC >> 6, r8 = lane >> 3, seg = lane & 7;
    const int rot = (int)(((blockIdx.x >> 3) * (unsigned)steps) >> 5) % steps;  // workgroups of an XCD start apart
    unsigned short *ps = tiles + wave * 32 * 72;
    uint32_t acc = 0;
    for (int r = 0; r < reps; r++) {
        uint32_t q[2][3][4];
        auto fetch = [&](int slot, int st) {
            int p = st + rot;
            p = p >= steps ? p - steps : p;
#pragma unroll
            for (int j = 0; j < 3; j++) {
                const uint4 v = *reinterpret_cast<const uint4 *>(phi + (size_t)(j * 8 + r8) * nC + (p << 6) + seg * 8);
                q[slot][j][0] = v.x; q[slot][j][1] = v.y; q[slot][j][2] = v.z; q[slot][j][3] = v.w;
            }
        };
        auto process = [&](int slot) {
#pragma unroll
            for (int j = 0; j < 3; j++)
                *reinterpret_cast<uint4 *>(ps + (j * 8 + r8) * 72 + seg * 8) =
                    make_uint4(q[slot][j][0], q[slot][j][1], q[slot][j][2], q[slot][j][3]);
            __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront");
            __builtin_amdgcn_wave_barrier();
            const uint4 v = *reinterpret_cast<const uint4 *>(ps + (lane & 15) * 72 + (lane >> 4) * 16);
            acc += v.x ^ v.w;
            __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "wavefront");
            __builtin_amdgcn_wave_barrier();
        };
#pragma unroll
        for (int u = 0; u < 2; u++)
            if (wave + u * 8 < steps) fetch(u, wave + u * 8);
        for (int st = wave; st < steps; st += 16) {
#pragma unroll
            for (int u = 0; u < 2; u++) {
                const int su = st + u * 8;
                if (su < steps) {
                    process(u);
                    if (su + 16 < steps) fetch(u, su + 16);
                }
            }
        }
        __syncthreads();
    }
    if (acc == 0x12345678u) *sink = acc;  // never: keeps the reads alive
}

}  // namespace

// mode 0 = read-only, 1 = copy, 2 = write-only, with the streaming (nt) hint on every access; 3, 4, 5 =
// the same with plain loads and stores; 6 = a kernel that does nothing (launch floor); bytes a multiple of 16; blocks = grid size
// (0: 256 CUs x 8).  sink: 4 bytes of device memory.  Returns the hipError_t of the launch.
extern "C" __attribute__((visibility("default"))) int mhc_stream_probe(int mode, const void *src, void *dst, size_t bytes,
                                                                       int blocks, void *sink, void *stream) {
    const size_t words = bytes / 16;
    const int grid = blocks > 0 ? blocks : 256 * 8;
    hipStream_t st = static_cast<hipStream_t>(stream);
    const u32x4 *s = static_cast<const u32x4 *>(src);
    u32x4 *d = static_cast<u32x4 *>(dst);
    if (mode == 0) probe_read_kernel<8, true><<<grid, 256, 0, st>>>(s, words, static_cast<uint32_t *>(sink));
    else if (mode == 1) probe_copy_kernel<4, true><<<grid, 256, 0, st>>>(s, d, words);
    else if (mode == 2) probe_write_kernel<true><<<grid, 256, 0, st>>>(d, words, 0x3f800000u);
    else if (mode == 3) probe_read_kernel<8, false><<<grid, 256, 0, st>>>(s, words, static_cast<uint32_t *>(sink));
    else if (mode == 4) probe_copy_kernel<4, false><<<grid, 256, 0, st>>>(s, d, words);
    else if (mode == 5) probe_write_kernel<false><<<grid, 256, 0, st>>>(d, words, 0x3f800000u);
    else if (mode == 6) probe_empty_kernel<<<grid, 256, 0, st>>>(static_cast<uint32_t *>(sink));  // launch floor
    else if (mode >= 7 && mode <= 9) {
        // hand-off probe: dst = blocks * (bytes / 4) floats of partial data, src = blocks floats of results (written),
        // sink = 3 zeroed words (arrivals, departures, gave-up flag); bytes = per workgroup, a multiple of 4 * blocks;
        // 7 = one kernel (blocks must all be resident: at most 8 per CU), 8 and 9 = its two halves as kernels
        if (blocks <= 0 || blocks > 2048 || bytes % (4 * (size_t)blocks)) return (int)hipErrorInvalidValue;
        float *part = static_cast<float *>(dst), *out = static_cast<float *>(const_cast<void *>(src));
        unsigned *sync = static_cast<unsigned *>(sink);
        const int per = (int)(bytes / 4);
        if (mode == 7) probe_handoff_kernel<true, 0><<<blocks, 256, 0, st>>>(part, out, sync, per);
        else if (mode == 8) probe_handoff_kernel<false, 0><<<blocks, 256, 0, st>>>(part, out, sync, per);
        else probe_handoff_kernel<false, 1><<<blocks, 256, 0, st>>>(part, out, sync, per);
    }
    else if (mode == 10) {
        // row-piece probe: src = [24][nC] bf16, bytes = 24 * nC * 2 (nC a multiple of 64), dst unused; 20 passes per launch
        const int nC = (int)(bytes / 48);
        if (blocks <= 0 || nC <= 0 || nC % 64) return (int)hipErrorInvalidValue;
        probe_row_pieces_kernel<<<blocks, 512, 0, st>>>(static_cast<const unsigned short *>(src), nC, static_cast<uint32_t *>(sink), 20);
    }
    else return (int)hipErrorInvalidValue;
    return (int)hipGetLastError();
}
