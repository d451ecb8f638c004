// Shared device/host helpers for the gfx950 SVDQuant kernels.
#pragma once

#include <hip/hip_runtime.h>
#include <stdint.h>

#include "../../include/svdq_mi355x.h"

namespace svdq {

typedef int v2i __attribute__((ext_vector_type(2)));
typedef int v4i __attribute__((ext_vector_type(4)));
typedef int v8i __attribute__((ext_vector_type(8)));
typedef int v16i __attribute__((ext_vector_type(16)));
typedef float v4f __attribute__((ext_vector_type(4)));
typedef float v16f __attribute__((ext_vector_type(16)));
typedef float v32f __attribute__((ext_vector_type(32)));
typedef __bf16 v8bf __attribute__((ext_vector_type(8)));
typedef _Float16 v8h __attribute__((ext_vector_type(8)));
typedef short v8s __attribute__((ext_vector_type(8)));
typedef short v4s __attribute__((ext_vector_type(4)));
typedef _Float16 v4h __attribute__((ext_vector_type(4)));

#define SVDQ_AS1 __attribute__((address_space(1)))
#define SVDQ_AS3 __attribute__((address_space(3)))

// s_waitcnt immediate (gfx9 encoding): vmcnt in bits [3:0] and [15:14], expcnt [6:4] left at 7, lgkmcnt [11:8]
constexpr int waitcnt_imm(int vm, int lgkm) { return (vm & 0xF) | ((vm >> 4) << 14) | 0x70 | ((lgkm & 0xF) << 8); }

constexpr int GROUP = 64;            // int4 scale group along K
constexpr float RNE_MAGIC = 12582912.0f;  // 1.5 * 2^23: adding it rounds an fp32 at the units place (RNE)
constexpr int RNE_MAGIC_BITS = 0x4B400000;

// ---- 16-bit float types -------------------------------------------------------------------------
struct BF16 {
    static constexpr int code = SVDQ_BF16;
    __device__ static inline float to_f32(uint16_t h) { return __uint_as_float(((uint32_t)h) << 16); }
    // two packed values: low half / high half of a dword
    __device__ static inline float lo_f32(uint32_t w) { return __uint_as_float(w << 16); }
    __device__ static inline float hi_f32(uint32_t w) { return __uint_as_float(w & 0xFFFF0000u); }
    __device__ static inline uint16_t from_f32(float f) {  // round to nearest even (v_cvt_pk_bf16_f32)
        const __bf16 b = (__bf16)f;
        return __builtin_bit_cast(uint16_t, b);
    }
    __device__ static inline uint32_t pack(float lo, float hi) {
        typedef __bf16 bf2 __attribute__((ext_vector_type(2)));
        typedef float f2 __attribute__((ext_vector_type(2)));
        const f2 v = {lo, hi};
        return __builtin_bit_cast(uint32_t, __builtin_convertvector(v, bf2));
    }
    // acc + lo + hi of a packed pair (v_dot2c_f32_bf16 against (1, 1))
    __device__ static inline float sum2(uint32_t w, float acc) {
        typedef __bf16 bf2 __attribute__((ext_vector_type(2)));
        return __builtin_amdgcn_fdot2_f32_bf16(__builtin_bit_cast(bf2, w), __builtin_bit_cast(bf2, 0x3F803F80u), acc, false);
    }
};

struct FP16 {
    static constexpr int code = SVDQ_FP16;
    __device__ static inline float to_f32(uint16_t h) {
        _Float16 v;
        __builtin_memcpy(&v, &h, 2);
        return (float)v;
    }
    __device__ static inline float lo_f32(uint32_t w) { return to_f32((uint16_t)(w & 0xFFFFu)); }
    __device__ static inline float hi_f32(uint32_t w) { return to_f32((uint16_t)(w >> 16)); }
    __device__ static inline uint16_t from_f32(float f) {
        _Float16 v = (_Float16)f;  // v_cvt_f16_f32: round to nearest even
        uint16_t h;
        __builtin_memcpy(&h, &v, 2);
        return h;
    }
    __device__ static inline uint32_t pack(float lo, float hi) {
        typedef _Float16 h2 __attribute__((ext_vector_type(2)));
        typedef float f2 __attribute__((ext_vector_type(2)));
        const f2 v = {lo, hi};
        return __builtin_bit_cast(uint32_t, __builtin_convertvector(v, h2));
    }
    __device__ static inline float sum2(uint32_t w, float acc) {
        typedef _Float16 h2 __attribute__((ext_vector_type(2)));
        return __builtin_amdgcn_fdot2(__builtin_bit_cast(h2, w), __builtin_bit_cast(h2, 0x3C003C00u), acc, false);
    }
};

template <typename T>
__device__ inline uint32_t pack2(float a, float b) {
    return T::pack(a, b);
}

// MFMA on eight 16-bit values per lane (K = 16 for 32x32, K = 32 for 16x16); operands passed as raw bits.
template <typename T>
__device__ inline v16f mfma32_16bit(v4i a, v4i b, v16f c);
template <>
__device__ inline v16f mfma32_16bit<BF16>(v4i a, v4i b, v16f c) {
    return __builtin_amdgcn_mfma_f32_32x32x16_bf16(__builtin_bit_cast(v8bf, a), __builtin_bit_cast(v8bf, b), c, 0, 0, 0);
}
template <>
__device__ inline v16f mfma32_16bit<FP16>(v4i a, v4i b, v16f c) {
    return __builtin_amdgcn_mfma_f32_32x32x16_f16(__builtin_bit_cast(v8h, a), __builtin_bit_cast(v8h, b), c, 0, 0, 0);
}
// The same on four 16-bit values per lane (32x32, K = 8).
template <typename T>
__device__ inline v16f mfma32_16bit_k8(v2i a, v2i b, v16f c);
template <>
__device__ inline v16f mfma32_16bit_k8<BF16>(v2i a, v2i b, v16f c) {
    return __builtin_amdgcn_mfma_f32_32x32x8bf16_1k(__builtin_bit_cast(v4s, a), __builtin_bit_cast(v4s, b), c, 0, 0, 0);
}
template <>
__device__ inline v16f mfma32_16bit_k8<FP16>(v2i a, v2i b, v16f c) {
    return __builtin_amdgcn_mfma_f32_32x32x8f16(__builtin_bit_cast(v4h, a), __builtin_bit_cast(v4h, b), c, 0, 0, 0);
}
template <typename T>
__device__ inline v4f mfma16_16bit(v4i a, v4i b, v4f c);
template <>
__device__ inline v4f mfma16_16bit<BF16>(v4i a, v4i b, v4f c) {
    return __builtin_amdgcn_mfma_f32_16x16x32_bf16(__builtin_bit_cast(v8bf, a), __builtin_bit_cast(v8bf, b), c, 0, 0, 0);
}
template <>
__device__ inline v4f mfma16_16bit<FP16>(v4i a, v4i b, v4f c) {
    return __builtin_amdgcn_mfma_f32_16x16x32_f16(__builtin_bit_cast(v8h, a), __builtin_bit_cast(v8h, b), c, 0, 0, 0);
}

// Value of lane ^ 32 / lane ^ 16 by the lane-swap instructions of gfx950 (vector ALU, no LDS round trip): swapping a
// register with itself leaves every lane's own value in one result and its partner's in the other.
__device__ inline float max_with_lane_xor32(float v) {
    const auto sw = __builtin_amdgcn_permlane32_swap(__float_as_uint(v), __float_as_uint(v), false, false);
    return fmaxf(__uint_as_float(sw[0]), __uint_as_float(sw[1]));
}
__device__ inline float max_with_lane_xor16(float v) {
    const auto sw = __builtin_amdgcn_permlane16_swap(__float_as_uint(v), __float_as_uint(v), false, false);
    return fmaxf(__uint_as_float(sw[0]), __uint_as_float(sw[1]));
}

__device__ inline float gelu_tanh(float x) {
    // 0.5 x (1 + tanh(u)), u = 0.79788456 (x + 0.044715 x^3), which the reference spells 0.5 x (1 + 2 / (1 + exp(-2 u)) - 1)
    // (nunchaku/ops/triton/_common.py:71-78).  That is x / (1 + exp(-2 u)) = x / (1 + 2^(x (c0 + c1 x^2))) with
    // c0 = -2 * 0.79788456 * log2(e), c1 = 0.044715 c0: seven instructions with the hardware exp2 and reciprocal (1 ulp
    // each) instead of 22 for the spelled-out form (an IEEE divide alone is ten), and within a few ulp of fp32 of it, which
    // is also how far exp() implementations differ from each other.
    constexpr float c0 = -2.0f * 0.79788456f * 1.4426950408889634f, c1 = 0.044715f * c0;
    const float p = __builtin_fmaf(x * x, c1, c0);
    return x * __builtin_amdgcn_rcpf(1.0f + __builtin_amdgcn_exp2f(x * p));
}

__device__ inline float silu(float x) { return x / (1.0f + __expf(-x)); }

// ---- host side ------------------------------------------------------------------------------------
void set_error(const char *fmt, ...);
int check_launch(const char *what);

}  // namespace svdq
