// Device-side helpers shared by every kernel of the mHC library (gfx950, wave64).
#pragma once

#include <hip/hip_runtime.h>
#include <stdint.h>
#include <type_traits>

namespace mhc {

typedef uint16_t bf16_t;  // raw bf16 storage; arithmetic is always fp32

constexpr int kWave = 64;

// ---------------------------------------------------------------------------------------------
// bf16 <-> fp32
// ---------------------------------------------------------------------------------------------
__device__ __forceinline__ float bf16_to_f32(bf16_t v) {
    return __uint_as_float(static_cast<uint32_t>(v) << 16);
}
__device__ __forceinline__ float bf16lo_to_f32(uint32_t pair) { return __uint_as_float(pair << 16); }
__device__ __forceinline__ float bf16hi_to_f32(uint32_t pair) {
    return __uint_as_float(pair & 0xffff0000u);
}
// round-to-nearest-even; the compiler selects the gfx950 hardware conversion for __bf16 casts
__device__ __forceinline__ bf16_t f32_to_bf16(float f) {
    __bf16 b = static_cast<__bf16>(f);
    return __builtin_bit_cast(bf16_t, b);
}
__device__ __forceinline__ uint32_t pack_bf16x2(float lo, float hi) {
    return static_cast<uint32_t>(f32_to_bf16(lo)) | (static_cast<uint32_t>(f32_to_bf16(hi)) << 16);
}

template <typename T> __device__ __forceinline__ float to_f32(T v);
template <> __device__ __forceinline__ float to_f32<float>(float v) { return v; }
template <> __device__ __forceinline__ float to_f32<bf16_t>(bf16_t v) { return bf16_to_f32(v); }

template <typename T> __device__ __forceinline__ T from_f32(float v);
template <> __device__ __forceinline__ float from_f32<float>(float v) { return v; }
template <> __device__ __forceinline__ bf16_t from_f32<bf16_t>(float v) { return f32_to_bf16(v); }

// ---------------------------------------------------------------------------------------------
// Vector loads/stores of V consecutive elements (V * sizeof(T) <= 32 bytes), converted to fp32.
// The pointer must be aligned to min(V * sizeof(T), 16) bytes.
// ---------------------------------------------------------------------------------------------
template <typename T, int V>
__device__ __forceinline__ void load_vec(const T *__restrict__ p, float (&out)[V]) {
    if constexpr (std::is_same<T, float>::value) {
        if constexpr (V % 4 == 0) {
#pragma unroll
            for (int i = 0; i < V / 4; i++) {
                float4 t = reinterpret_cast<const float4 *>(p)[i];
                out[4 * i] = t.x; out[4 * i + 1] = t.y; out[4 * i + 2] = t.z; out[4 * i + 3] = t.w;
            }
        } else if constexpr (V == 2) {
            float2 t = *reinterpret_cast<const float2 *>(p);
            out[0] = t.x; out[1] = t.y;
        } else {
#pragma unroll
            for (int i = 0; i < V; i++) out[i] = p[i];
        }
    } else {
        if constexpr (V % 8 == 0) {
#pragma unroll
            for (int i = 0; i < V / 8; i++) {
                uint4 t = reinterpret_cast<const uint4 *>(p)[i];
                out[8 * i] = bf16lo_to_f32(t.x); out[8 * i + 1] = bf16hi_to_f32(t.x);
                out[8 * i + 2] = bf16lo_to_f32(t.y); out[8 * i + 3] = bf16hi_to_f32(t.y);
                out[8 * i + 4] = bf16lo_to_f32(t.z); out[8 * i + 5] = bf16hi_to_f32(t.z);
                out[8 * i + 6] = bf16lo_to_f32(t.w); out[8 * i + 7] = bf16hi_to_f32(t.w);
            }
        } else if constexpr (V == 4) {
            uint2 t = *reinterpret_cast<const uint2 *>(p);
            out[0] = bf16lo_to_f32(t.x); out[1] = bf16hi_to_f32(t.x);
            out[2] = bf16lo_to_f32(t.y); out[3] = bf16hi_to_f32(t.y);
        } else if constexpr (V == 2) {
            uint32_t t = *reinterpret_cast<const uint32_t *>(p);
            out[0] = bf16lo_to_f32(t); out[1] = bf16hi_to_f32(t);
        } else {
#pragma unroll
            for (int i = 0; i < V; i++) out[i] = bf16_to_f32(p[i]);
        }
    }
}

// Raw stores of 16 / 8 / 4 bytes.  STREAM marks the data as written once and not read again soon
// (the `nt` bit of the store): a large output then does not push the operands that other
// workgroups still re-read out of L2.
typedef uint32_t u32x4_t __attribute__((ext_vector_type(4)));
typedef uint32_t u32x2_t __attribute__((ext_vector_type(2)));
template <bool STREAM> __device__ __forceinline__ void st16(void *p, uint32_t a, uint32_t b, uint32_t c, uint32_t d) {
    const u32x4_t v = {a, b, c, d};
    if constexpr (STREAM) __builtin_nontemporal_store(v, reinterpret_cast<u32x4_t *>(p));
    else *reinterpret_cast<u32x4_t *>(p) = v;
}
template <bool STREAM> __device__ __forceinline__ void st8(void *p, uint32_t a, uint32_t b) {
    const u32x2_t v = {a, b};
    if constexpr (STREAM) __builtin_nontemporal_store(v, reinterpret_cast<u32x2_t *>(p));
    else *reinterpret_cast<u32x2_t *>(p) = v;
}
template <bool STREAM> __device__ __forceinline__ void st4(void *p, uint32_t a) {
    if constexpr (STREAM) __builtin_nontemporal_store(a, reinterpret_cast<uint32_t *>(p));
    else *reinterpret_cast<uint32_t *>(p) = a;
}

template <typename T, int V, bool STREAM = false>
__device__ __forceinline__ void store_vec(T *__restrict__ p, const float (&v)[V]) {
    if constexpr (std::is_same<T, float>::value) {
        if constexpr (V % 4 == 0) {
#pragma unroll
            for (int i = 0; i < V / 4; i++)
                st16<STREAM>(p + 4 * i, __float_as_uint(v[4 * i]), __float_as_uint(v[4 * i + 1]),
                             __float_as_uint(v[4 * i + 2]), __float_as_uint(v[4 * i + 3]));
        } else if constexpr (V == 2) {
            st8<STREAM>(p, __float_as_uint(v[0]), __float_as_uint(v[1]));
        } else {
#pragma unroll
            for (int i = 0; i < V; i++) st4<STREAM>(p + i, __float_as_uint(v[i]));
        }
    } else {
        if constexpr (V % 8 == 0) {
#pragma unroll
            for (int i = 0; i < V / 8; i++)
                st16<STREAM>(p + 8 * i, pack_bf16x2(v[8 * i], v[8 * i + 1]), pack_bf16x2(v[8 * i + 2], v[8 * i + 3]),
                             pack_bf16x2(v[8 * i + 4], v[8 * i + 5]), pack_bf16x2(v[8 * i + 6], v[8 * i + 7]));
        } else if constexpr (V == 4) {
            st8<STREAM>(p, pack_bf16x2(v[0], v[1]), pack_bf16x2(v[2], v[3]));
        } else if constexpr (V == 2) {
            st4<STREAM>(p, pack_bf16x2(v[0], v[1]));
        } else {
#pragma unroll
            for (int i = 0; i < V; i++) p[i] = f32_to_bf16(v[i]);
        }
    }
}

// 16-byte load with the streaming (non-temporal) hint.
__device__ __forceinline__ uint4 ldg16_stream(const uint4 *p) {
    const u32x4_t t = __builtin_nontemporal_load(reinterpret_cast<const u32x4_t *>(p));
    return make_uint4(t[0], t[1], t[2], t[3]);
}

// V consecutive elements kept exactly as loaded.  No conversion instruction sits behind the load,
// so a batch of loads stays in flight across whatever code follows (another basic block
// included); get() widens to fp32 at the point of use.  The pointer must be dereferenceable and
// aligned to min(V * sizeof(T), 16) bytes: callers clamp out-of-range indices to a valid element
// instead of branching around the load.
template <typename T, int V> struct RawVec {
    static constexpr int kBytes = V * (int)sizeof(T);
    static constexpr int kWords = (kBytes + 3) / 4;
    uint32_t w[kWords];
    __device__ __forceinline__ void load(const T *__restrict__ p) {
        if constexpr (kBytes % 16 == 0) {
#pragma unroll
            for (int i = 0; i < kBytes / 16; i++) {
                const uint4 t = reinterpret_cast<const uint4 *>(p)[i];
                w[4 * i] = t.x; w[4 * i + 1] = t.y; w[4 * i + 2] = t.z; w[4 * i + 3] = t.w;
            }
        } else if constexpr (kBytes == 8) {
            const uint2 t = *reinterpret_cast<const uint2 *>(p);
            w[0] = t.x; w[1] = t.y;
        } else if constexpr (kBytes == 4) {
            w[0] = *reinterpret_cast<const uint32_t *>(p);
        } else {
            static_assert(kBytes == 2, "unsupported vector width");
            w[0] = *reinterpret_cast<const uint16_t *>(p);
        }
    }
    // The same with the streaming hint (the `nt` bit of the load).  A cold read-only pass over
    // 128-512 MiB runs at 4.7-4.9 TB/s with the hint and at 2.4-3.2 TB/s without it on this GPU, but the
    // hint also keeps the data out of the 256 MB Infinity Cache: with back-to-back steps the 89 MB of
    // phi at n = 32 are partly served from that cache, and the hinted loads made the two kernels that
    // stream phi 15-35 % slower.  Kept for data that is truly read once.  16-byte multiples only.
    __device__ __forceinline__ void load_stream(const T *__restrict__ p) {
        static_assert(kBytes % 16 == 0, "streaming loads are 16-byte loads");
#pragma unroll
        for (int i = 0; i < kBytes / 16; i++) {
            const uint4 t = ldg16_stream(reinterpret_cast<const uint4 *>(p) + i);
            w[4 * i] = t.x; w[4 * i + 1] = t.y; w[4 * i + 2] = t.z; w[4 * i + 3] = t.w;
        }
    }
    __device__ __forceinline__ void get(float (&v)[V]) const {
        if constexpr (std::is_same<T, float>::value) {
#pragma unroll
            for (int i = 0; i < V; i++) v[i] = __uint_as_float(w[i]);
        } else if constexpr (V == 1) {
            v[0] = bf16lo_to_f32(w[0]);
        } else {
#pragma unroll
            for (int i = 0; i < V / 2; i++) { v[2 * i] = bf16lo_to_f32(w[i]); v[2 * i + 1] = bf16hi_to_f32(w[i]); }
        }
    }
};

// 16-byte global load that yields zeros when !ok.  `p` must be dereferenceable either way (callers
// clamp the index): the load is unconditional and the value is masked afterwards, which keeps the
// code free of per-lane branches.  Do NOT write `ok ? *p : zero_variable`: the compiler then selects
// between two addresses (global memory and the variable's stack slot) and emits a flat load that
// waits on both memory counters.
__device__ __forceinline__ uint4 load16_masked(const uint4 *p, bool ok) {
    uint4 v = *p;
    v.x = ok ? v.x : 0u; v.y = ok ? v.y : 0u; v.z = ok ? v.z : 0u; v.w = ok ? v.w : 0u;
    return v;
}

// ---------------------------------------------------------------------------------------------
// v_mfma_f32_4x4x4_16b_bf16: 16 independent 4x4x4 products per instruction.  Block = four
// consecutive lanes; lane r of a block supplies row r of A (four bf16 along k) and column r of B,
// and receives column r of the product (register = row).
// ---------------------------------------------------------------------------------------------
typedef __attribute__((__vector_size__(4 * sizeof(short)))) short bf16x4_t;

// ---------------------------------------------------------------------------------------------
// Transposed MFMA operand from a row-major [k][column] bf16 tile in LDS (pitch ld elements, a
// multiple of 4; col0 a multiple of 4; tile 8-byte aligned): lane (n = lane & 31, kg = lane >> 5)
// receives tile[k0 + kg*8 + i][col0 + n], i = 0..7 - the B (or A) operand of
// v_mfma_f32_32x32x16_bf16 when the contraction index is the strided one in memory.
// Two ds_read_b64_tr_b16: within 16 lanes, lane i receives element i % 4 of the 8 bytes addressed
// by lanes i/4 + 4j (j = 0..3).  So lane q + 4j of a group points at row j, columns 4q .. 4q+3 of
// a 4 x 16 block, and lane i receives column i of the block with its four rows.  Layout checked on
// the device with an index pattern.  (Eight 2-byte reads plus four packs per operand otherwise.)
// ---------------------------------------------------------------------------------------------
typedef short lds_tr_v4i16 __attribute__((ext_vector_type(4)));
__device__ __forceinline__ uint4 lds_frag_tr(const bf16_t *tile, int ld, int k0, int col0, int lane) {
    const int g = lane >> 4, q = lane & 3, j = (lane >> 2) & 3;
    const bf16_t *p = tile + (size_t)(k0 + (g >> 1) * 8 + j) * ld + col0 + (g & 1) * 16 + q * 4;
    typedef __attribute__((address_space(3))) lds_tr_v4i16 *lds_ptr;
    const lds_tr_v4i16 lo = __builtin_amdgcn_ds_read_tr16_b64_v4i16((lds_ptr)p);
    const lds_tr_v4i16 hi = __builtin_amdgcn_ds_read_tr16_b64_v4i16((lds_ptr)(p + 4 * (size_t)ld));
    const uint2 l2 = __builtin_bit_cast(uint2, lo), h2 = __builtin_bit_cast(uint2, hi);
    return make_uint4(l2.x, l2.y, h2.x, h2.y);
}
typedef __attribute__((__vector_size__(4 * sizeof(float)))) float f32x4_t;

__device__ __forceinline__ bf16x4_t bf16x4_of(uint32_t w0, uint32_t w1) {
    return __builtin_bit_cast(bf16x4_t, make_uint2(w0, w1));
}
__device__ __forceinline__ f32x4_t mfma4(bf16x4_t a, bf16x4_t b, f32x4_t c) {
    return __builtin_amdgcn_mfma_f32_4x4x4bf16_1k(a, b, c, 0, 0, 0);
}
// Four fp32 coefficients as two bf16x4 operands: the rounded values and their remainders.
struct CoefRow {
    bf16x4_t hi, lo;
    __device__ __forceinline__ void set(float c0, float c1, float c2, float c3) {
        const uint32_t h0 = pack_bf16x2(c0, c1), h1 = pack_bf16x2(c2, c3);
        const uint32_t l0 = pack_bf16x2(c0 - bf16lo_to_f32(h0), c1 - bf16hi_to_f32(h0));
        const uint32_t l1 = pack_bf16x2(c2 - bf16lo_to_f32(h1), c3 - bf16hi_to_f32(h1));
        hi = bf16x4_of(h0, h1);
        lo = bf16x4_of(l0, l1);
    }
};
// The four streams of one channel as a bf16x4 operand, from the word of each stream that holds the
// channel pair: the low halves (even channel) or the high halves (odd channel).
template <bool ODD>
__device__ __forceinline__ bf16x4_t streams_of_channel(uint32_t w0, uint32_t w1, uint32_t w2, uint32_t w3) {
    constexpr uint32_t sel = ODD ? 0x07060302u : 0x05040100u;
    return bf16x4_of(__builtin_amdgcn_perm(w1, w0, sel), __builtin_amdgcn_perm(w3, w2, sel));
}

// ---------------------------------------------------------------------------------------------
// Cross-lane primitives
// ---------------------------------------------------------------------------------------------
// DPP controls (GFX9 encoding): quad_perm = 8-bit selector, row_ror:n = 0x120 + n
constexpr int kDppQuadXor1 = 0xB1;   // quad_perm:[1,0,3,2]
constexpr int kDppQuadXor2 = 0x4E;   // quad_perm:[2,3,0,1]
constexpr int kDppRowRor4 = 0x124;
constexpr int kDppRowRor8 = 0x128;
constexpr int kDppRowHalfMirror = 0x141;  // lane i <-> 7 - i within each 8 lanes

// All controls used here read a valid lane for every lane, so `old` is irrelevant; passing 0 with
// bound_ctrl lets the compiler fold the move into the consuming VALU instruction (v_add_f32_dpp).
template <int CTRL> __device__ __forceinline__ float dpp_mov(float v) {
    return __int_as_float(__builtin_amdgcn_update_dpp(0, __float_as_int(v), CTRL, 0xF, 0xF, true));
}

// v[lane] + v[lane ^ 16] and v[lane] + v[lane ^ 32] in every lane.  v_permlane16_swap exchanges
// the odd 16-lane rows of its first operand with the even rows of its second, v_permlane32_swap
// the upper half of the first with the lower half of the second; with the same value in both
// operands the two results hold each partner pair, so their sum is the exchange-and-add - one
// VALU instruction instead of a round trip through the LDS crossbar (ds_bpermute).
__device__ __forceinline__ float xor16_add(float v) {
    const unsigned b = __float_as_uint(v);
    const auto r = __builtin_amdgcn_permlane16_swap(b, b, false, false);
    return __uint_as_float(r[0]) + __uint_as_float(r[1]);
}
__device__ __forceinline__ float xor32_add(float v) {
    const unsigned b = __float_as_uint(v);
    const auto r = __builtin_amdgcn_permlane32_swap(b, b, false, false);
    return __uint_as_float(r[0]) + __uint_as_float(r[1]);
}

// Sum over all 64 lanes; every lane gets the total.
__device__ __forceinline__ float wave_allreduce_sum(float v) {
    v += dpp_mov<kDppQuadXor1>(v);
    v += dpp_mov<kDppQuadXor2>(v);
    v += dpp_mov<kDppRowRor4>(v);
    v += dpp_mov<kDppRowRor8>(v);
    v = xor16_add(v);
    v = xor32_add(v);
    return v;
}

// Sum over the whole workgroup (NT threads, multiple of 64); every thread gets the total.
// `red` is LDS scratch of at least NT/64 floats; safe to call repeatedly with the same scratch.
template <int NT> __device__ __forceinline__ float block_allreduce_sum(float v, float *red) {
    v = wave_allreduce_sum(v);
    if constexpr (NT == kWave) return v;
    const int wave = threadIdx.x / kWave;
    __syncthreads();  // previous readers of red are done
    if ((threadIdx.x & (kWave - 1)) == 0) red[wave] = v;
    __syncthreads();
    float total = 0.f;
#pragma unroll
    for (int i = 0; i < NT / kWave; i++) total += red[i];
    return total;
}

// The same for a workgroup of `nwaves` whole waves known only at run time.
__device__ __forceinline__ float block_allreduce_sum(float v, float *red, int nwaves) {
    v = wave_allreduce_sum(v);
    if (nwaves == 1) return v;
    const int wave = threadIdx.x / kWave;
    __syncthreads();  // previous readers of red are done
    if ((threadIdx.x & (kWave - 1)) == 0) red[wave] = v;
    __syncthreads();
    float total = 0.f;
    for (int i = 0; i < nwaves; i++) total += red[i];
    return total;
}

__device__ __forceinline__ float sigmoidf_acc(float t) { return 1.0f / (1.0f + expf(-t)); }

// bf16 tier: exp and sigmoid on the hardware's exp2 and reciprocal (1 ulp each, a handful of
// instructions; the library versions are ~15 and ~30 dependent instructions, which shows on the
// serial coefficient step that every workgroup runs before it can mix its tile).
__device__ __forceinline__ float exp_fast(float t) { return __builtin_amdgcn_exp2f(t * 1.44269504088896341f); }
__device__ __forceinline__ float sigmoid_fast(float t) { return __builtin_amdgcn_rcpf(1.0f + exp_fast(-t)); }

// v_rcp_f32: 1 ulp, one instruction (an IEEE division costs ~10 dependent instructions, which
// matters on the serial Sinkhorn chain).
__device__ __forceinline__ float fast_rcp(float v) { return __builtin_amdgcn_rcpf(v); }

// Index of the alpha group of projection row d: 0 = pre, 1 = post, 2 = res.
__device__ __forceinline__ int alpha_group(int d, int n) { return d < n ? 0 : (d < 2 * n ? 1 : 2); }

__host__ __device__ constexpr int round_up(int v, int m) { return (v + m - 1) / m * m; }

// ---------------------------------------------------------------------------------------------
// MFMA-ready ("fragment-major") storage of the two bf16 copies of dP that the projection
// backward consumes as A operands of v_mfma_f32_32x32x16_bf16.  One fragment = the 64 lanes x 8
// values of one instruction, stored contiguously (1 KiB), so a wave loads it with one fully
// coalesced 16-byte-per-lane access: lane = 32 * kgroup + row, kgroup = (k / 8) % 2.
//   frag_dpt: rows d (tile d / 32), contraction index b (step b / 16); BP = padded batch, % 32 == 0
//   frag_dpb: rows b (tile b / 32), contraction index d (step d / 16); DP = padded D, % 32 == 0
// ---------------------------------------------------------------------------------------------
__host__ __device__ inline size_t frag_base(int tile, int steps_per_tile, int step) {
    return ((size_t)tile * steps_per_tile + step) * 512;  // elements
}
__host__ __device__ inline size_t frag_dpt(int d, int b, int BP) {
    return frag_base(d >> 5, BP >> 4, b >> 4) + (size_t)((((b >> 3) & 1) * 32 + (d & 31)) * 8 + (b & 7));
}
__host__ __device__ inline size_t frag_dpb(int b, int d, int DP) {
    return frag_base(b >> 5, DP >> 4, d >> 4) + (size_t)((((d >> 3) & 1) * 32 + (b & 31)) * 8 + (d & 7));
}

}  // namespace mhc
