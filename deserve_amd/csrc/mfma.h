// MFMA operand helpers and scalar element access shared by the attention
// kernels.  gfx950 (CDNA4) only.
#pragma once

#include "common.h"

namespace dskv {

constexpr float kNegBig = -1.0e30f;   // "minus infinity" that stays finite under subtraction

// 16-bit element traits.  Operands travel as raw 32-bit words (a 16-byte global
// load is a u32x4) and are only reinterpreted at the MFMA call.
template <int DT> struct Elt;

template <> struct Elt<DSKV_BF16> {
    typedef __bf16 v8 __attribute__((ext_vector_type(8)));
    typedef short v4 __attribute__((ext_vector_type(4)));
    typedef __bf16 v2 __attribute__((ext_vector_type(2)));
    typedef float f2 __attribute__((ext_vector_type(2)));
    static __device__ __forceinline__ f32x4 mfma_k32(u32x4 a, u32x4 b, f32x4 c) {
        return __builtin_amdgcn_mfma_f32_16x16x32_bf16(__builtin_bit_cast(v8, a),
                                                        __builtin_bit_cast(v8, b), c, 0, 0, 0);
    }
    static __device__ __forceinline__ f32x4 mfma_k16(u32x2 a, u32x2 b, f32x4 c) {
        return __builtin_amdgcn_mfma_f32_16x16x16bf16_1k(__builtin_bit_cast(v4, a),
                                                          __builtin_bit_cast(v4, b), c, 0, 0, 0);
    }
    static __device__ __forceinline__ uint32_t pack2(float lo, float hi) {
        f2 f = {lo, hi};
        return __builtin_bit_cast(uint32_t, __builtin_convertvector(f, v2));
    }
    static __device__ __forceinline__ float widen(uint16_t h) {
        return __builtin_bit_cast(float, (uint32_t)h << 16);
    }
};

template <> struct Elt<DSKV_F16> {
    typedef _Float16 v8 __attribute__((ext_vector_type(8)));
    typedef _Float16 v4 __attribute__((ext_vector_type(4)));
    typedef _Float16 v2 __attribute__((ext_vector_type(2)));
    typedef float f2 __attribute__((ext_vector_type(2)));
    static __device__ __forceinline__ f32x4 mfma_k32(u32x4 a, u32x4 b, f32x4 c) {
        return __builtin_amdgcn_mfma_f32_16x16x32_f16(__builtin_bit_cast(v8, a),
                                                       __builtin_bit_cast(v8, b), c, 0, 0, 0);
    }
    static __device__ __forceinline__ f32x4 mfma_k16(u32x2 a, u32x2 b, f32x4 c) {
        return __builtin_amdgcn_mfma_f32_16x16x16f16(__builtin_bit_cast(v4, a),
                                                      __builtin_bit_cast(v4, b), c, 0, 0, 0);
    }
    static __device__ __forceinline__ uint32_t pack2(float lo, float hi) {
        f2 f = {lo, hi};
        return __builtin_bit_cast(uint32_t, __builtin_convertvector(f, v2));
    }
    static __device__ __forceinline__ float widen(uint16_t h) {
        return (float)__builtin_bit_cast(_Float16, h);
    }
};

// Scalar element access used by the non-MFMA kernels.
template <int DT> struct LoadElt;
template <> struct LoadElt<DSKV_F32> {
    typedef float T;
    static __device__ __forceinline__ float get(const void *p, long i) { return ((const float *)p)[i]; }
    static __device__ __forceinline__ void put(void *p, long i, float v) { ((float *)p)[i] = v; }
};
template <> struct LoadElt<DSKV_F16> {
    static __device__ __forceinline__ float get(const void *p, long i) {
        return (float)((const _Float16 *)p)[i];
    }
    static __device__ __forceinline__ void put(void *p, long i, float v) {
        ((_Float16 *)p)[i] = (_Float16)v;
    }
};
template <> struct LoadElt<DSKV_BF16> {
    static __device__ __forceinline__ float get(const void *p, long i) {
        return __builtin_bit_cast(float, (uint32_t)((const uint16_t *)p)[i] << 16);
    }
    static __device__ __forceinline__ void put(void *p, long i, float v) {
        ((__bf16 *)p)[i] = (__bf16)v;
    }
};

__device__ __forceinline__ float wave_sum(float v)
{
#pragma unroll
    for (int o = 32; o > 0; o >>= 1) v += __shfl_xor(v, o);
    return v;
}

}  // namespace dskv
