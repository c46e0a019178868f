// Shared device helpers for the gfx950 CalibQuant kernels.
#pragma once

#include <hip/hip_runtime.h>
#include <hip/hip_fp16.h>
#include <stdint.h>

#include "calibquant_hip.h"

namespace cq {

constexpr int kWave = 64;

// Last HIP runtime error seen by this host thread (cq_last_hip_error()).
extern thread_local int g_last_hip_error;

inline int hip_fail(hipError_t e) {
    g_last_hip_error = static_cast<int>(e);
    return CQ_ERR_LAUNCH;
}

#define CQ_HIP_CHECK(expr)                                 \
    do {                                                   \
        hipError_t _e = (expr);                            \
        if (_e != hipSuccess) return ::cq::hip_fail(_e);   \
    } while (0)

#define CQ_LAUNCH_CHECK()                                  \
    do {                                                   \
        hipError_t _e = hipGetLastError();                 \
        if (_e != hipSuccess) return ::cq::hip_fail(_e);   \
    } while (0)

inline bool aligned16(const void* p) { return (reinterpret_cast<uintptr_t>(p) & 15u) == 0; }

// ---------------------------------------------------------------- dtypes
struct BF16 {};
struct FP16 {};

__device__ __forceinline__ float bf16_bits_to_float(uint32_t h) { return __uint_as_float(h << 16); }

// fp32 -> bf16 bits, round to nearest even (the hardware conversion of gfx950).
__device__ __forceinline__ uint32_t float_to_bf16_bits(float f) {
    return __builtin_bit_cast(unsigned short, static_cast<__bf16>(f));
}

__device__ __forceinline__ float fp16_bits_to_float(uint32_t h) {
    return __half2float(__ushort_as_half(static_cast<unsigned short>(h)));
}

__device__ __forceinline__ uint32_t float_to_fp16_bits(float f) {
    return static_cast<uint32_t>(__half_as_ushort(__float2half_rn(f)));
}

template <typename DT> struct Cvt;
template <> struct Cvt<BF16> {
    static __device__ __forceinline__ float to_float(uint32_t bits16) { return bf16_bits_to_float(bits16); }
    static __device__ __forceinline__ uint32_t from_float(float f) { return float_to_bf16_bits(f); }
    // low / high halves of a 32-bit word holding two elements
    static __device__ __forceinline__ float lo(uint32_t w) { return __uint_as_float(w << 16); }
    static __device__ __forceinline__ float hi(uint32_t w) { return __uint_as_float(w & 0xffff0000u); }
};
template <> struct Cvt<FP16> {
    static __device__ __forceinline__ float to_float(uint32_t bits16) { return fp16_bits_to_float(bits16); }
    static __device__ __forceinline__ uint32_t from_float(float f) { return float_to_fp16_bits(f); }
    static __device__ __forceinline__ float lo(uint32_t w) { return fp16_bits_to_float(w & 0xffffu); }
    static __device__ __forceinline__ float hi(uint32_t w) { return fp16_bits_to_float(w >> 16); }
};

// Round an fp32 value to the storage dtype and back (one torch op boundary).
template <typename DT>
__device__ __forceinline__ float rnd(float f) { return Cvt<DT>::to_float(Cvt<DT>::from_float(f)); }

// 8 consecutive 16-bit elements (one 16-byte load) -> 8 floats
template <typename DT, typename V16>   // V16: uint4 or a native 4 x uint32 vector
__device__ __forceinline__ void unpack8(const V16& v, float* f) {
    f[0] = Cvt<DT>::lo(v.x); f[1] = Cvt<DT>::hi(v.x);
    f[2] = Cvt<DT>::lo(v.y); f[3] = Cvt<DT>::hi(v.y);
    f[4] = Cvt<DT>::lo(v.z); f[5] = Cvt<DT>::hi(v.z);
    f[6] = Cvt<DT>::lo(v.w); f[7] = Cvt<DT>::hi(v.w);
}

template <typename DT>
__device__ __forceinline__ float load_elem(const void* p, int64_t i) {
    return Cvt<DT>::to_float(static_cast<const uint16_t*>(p)[i]);
}

template <typename DT>
__device__ __forceinline__ void store_elem(void* p, int64_t i, float f) {
    static_cast<uint16_t*>(p)[i] = static_cast<uint16_t>(Cvt<DT>::from_float(f));
}

// Division of indices (< 2^31) by a small run-time constant without the integer-division
// expansion: q = (mulhi(n, mul) + n) >> shift, with mul and shift worked out on the host.
struct FastDiv {
    uint32_t mul, shift, div;
    __host__ void set(uint32_t d) {
        div = d;
        shift = 0;
        while ((1u << shift) < d) ++shift;
        mul = static_cast<uint32_t>(((static_cast<uint64_t>(1) << 32) * ((static_cast<uint64_t>(1) << shift) - d)) / d + 1);
    }
    __device__ __forceinline__ uint32_t quot(uint32_t n) const { return (__umulhi(n, mul) + n) >> shift; }
};

// ------------------------------------------------------- wave reductions
// Cross-lane moves use the data-parallel-primitive modifiers of the VALU (no LDS
// traffic, one instruction per step).  Control codes: quad_perm[1,0,3,2] = 0xB1,
// quad_perm[2,3,0,1] = 0x4E, row_half_mirror = 0x141, row_mirror = 0x140,
// row_bcast:15 = 0x142, row_bcast:31 = 0x143.
template <int CTRL, int ROW_MASK = 0xf>
__device__ __forceinline__ float dpp_move(float v, float inactive) {
    if constexpr (ROW_MASK == 0xf && CTRL < 0x142) {
        // every lane has a source: no fill value needed
        return __builtin_bit_cast(float, __builtin_amdgcn_mov_dpp(__builtin_bit_cast(int, v), CTRL, 0xf, 0xf, true));
    } else {
        return __builtin_bit_cast(float, __builtin_amdgcn_update_dpp(__builtin_bit_cast(int, inactive),
                                                                      __builtin_bit_cast(int, v), CTRL, ROW_MASK,
                                                                      0xf, false));
    }
}
template <int CTRL, int ROW_MASK = 0xf>
__device__ __forceinline__ int dpp_move_i(int v, int inactive) {
    if constexpr (ROW_MASK == 0xf && CTRL < 0x142) {
        return __builtin_amdgcn_mov_dpp(v, CTRL, 0xf, 0xf, true);
    } else {
        return __builtin_amdgcn_update_dpp(inactive, v, CTRL, ROW_MASK, 0xf, false);
    }
}

// Order-preserving map between floats and signed integers (an involution): integer
// max / min then orders like the float one, and fuses with the cross-lane modifiers.
__device__ __forceinline__ int float_key(float f) {
    const int i = __builtin_bit_cast(int, f);
    return i ^ ((i >> 31) & 0x7fffffff);
}
__device__ __forceinline__ float key_float(int k) { return __builtin_bit_cast(float, k ^ ((k >> 31) & 0x7fffffff)); }

// max over aligned groups of 16 lanes / the whole wave, on integer keys
__device__ __forceinline__ int row_max_key(int v) {
    constexpr int lo = static_cast<int>(0x80000000u);
    v = max(v, dpp_move_i<0xB1>(v, lo));
    v = max(v, dpp_move_i<0x4E>(v, lo));
    v = max(v, dpp_move_i<0x141>(v, lo));
    return max(v, dpp_move_i<0x140>(v, lo));
}
__device__ __forceinline__ int wave_max_key(int v) {
    constexpr int lo = static_cast<int>(0x80000000u);
    v = row_max_key(v);
    v = max(v, dpp_move_i<0x142, 0xa>(v, lo));
    v = max(v, dpp_move_i<0x143, 0xc>(v, lo));
    return __builtin_amdgcn_readlane(v, 63);
}

struct OpMin { __device__ __forceinline__ float operator()(float a, float b) const { return fminf(a, b); } };
struct OpMax { __device__ __forceinline__ float operator()(float a, float b) const { return fmaxf(a, b); } };
struct OpSum { __device__ __forceinline__ float operator()(float a, float b) const { return a + b; } };

// Reduce over aligned groups of 4 / 8 / 16 lanes; every lane of the group gets the result.
template <typename Op> __device__ __forceinline__ float quad_reduce(float v, Op op, float id) {
    v = op(v, dpp_move<0xB1>(v, id));
    return op(v, dpp_move<0x4E>(v, id));
}
template <typename Op> __device__ __forceinline__ float oct_reduce(float v, Op op, float id) {
    v = quad_reduce(v, op, id);
    return op(v, dpp_move<0x141>(v, id));
}
template <typename Op> __device__ __forceinline__ float row_reduce(float v, Op op, float id) {
    v = oct_reduce(v, op, id);
    return op(v, dpp_move<0x140>(v, id));
}
// Reduce over the 64 lanes; the result is wave-uniform (scalar register).
template <typename Op> __device__ __forceinline__ float wave_reduce(float v, Op op, float id) {
    v = row_reduce(v, op, id);
    v = op(v, dpp_move<0x142, 0xa>(v, id));
    v = op(v, dpp_move<0x143, 0xc>(v, id));
    return __builtin_bit_cast(float, __builtin_amdgcn_readlane(__builtin_bit_cast(int, v), 63));
}
// The same over N values side by side: the chains are independent, so the cross-lane moves
// of one fill the wait states of the others.
template <int CTRL, int ROW_MASK, int N, typename Op>
__device__ __forceinline__ void reduce_step(float* v, Op op, float id) {
    float t[N];
#pragma unroll
    for (int i = 0; i < N; ++i) t[i] = dpp_move<CTRL, ROW_MASK>(v[i], id);
#pragma unroll
    for (int i = 0; i < N; ++i) v[i] = op(v[i], t[i]);
}
template <int N, typename Op>
__device__ __forceinline__ void wave_reduce_n(float* v, Op op, float id) {
    reduce_step<0xB1, 0xf, N>(v, op, id);
    reduce_step<0x4E, 0xf, N>(v, op, id);
    reduce_step<0x141, 0xf, N>(v, op, id);
    reduce_step<0x140, 0xf, N>(v, op, id);
    reduce_step<0x142, 0xa, N>(v, op, id);
    reduce_step<0x143, 0xc, N>(v, op, id);
#pragma unroll
    for (int i = 0; i < N; ++i) v[i] = __builtin_bit_cast(float, __builtin_amdgcn_readlane(__builtin_bit_cast(int, v[i]), 63));
}
__device__ __forceinline__ float wave_max(float v) { return key_float(wave_max_key(float_key(v))); }
__device__ __forceinline__ float wave_min(float v) { return wave_reduce(v, OpMin(), INFINITY); }
__device__ __forceinline__ float wave_sum(float v) { return wave_reduce(v, OpSum(), 0.0f); }

}  // namespace cq
