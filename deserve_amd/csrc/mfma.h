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
    static __device__ __forceinline__ f32x16 mfma_32x32(u32x4 a, u32x4 b, f32x16 c) {
        return __builtin_amdgcn_mfma_f32_32x32x16_bf16(__builtin_bit_cast(v8, a),
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
    static __device__ __forceinline__ void unpack2(uint32_t w, float &lo, float &hi) {
        lo = __builtin_bit_cast(float, w << 16);
        hi = __builtin_bit_cast(float, w & 0xFFFF0000u);
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
    static __device__ __forceinline__ f32x16 mfma_32x32(u32x4 a, u32x4 b, f32x16 c) {
        return __builtin_amdgcn_mfma_f32_32x32x16_f16(__builtin_bit_cast(v8, a),
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
    static __device__ __forceinline__ void unpack2(uint32_t w, float &lo, float &hi) {
        const v2 h = __builtin_bit_cast(v2, w);
        lo = (float)h.x;
        hi = (float)h.y;
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

// Exchange between the four lanes that share lane % 16 (lane bits 4 and 5) with
// gfx950's register swaps: after swap_rows16(a, b) on a == b == v, a and b hold
// v of the two lanes that differ in bit 4 (swap_halves32: bit 5).  Pure VALU,
// where __shfl_xor would go through the LDS pipeline.  The s_nop covers the
// wait states the swap needs after a vector write of its operands.
__device__ __forceinline__ void swap_rows16(float &a, float &b)
{
    asm("s_nop 1\n\tv_permlane16_swap_b32 %0, %1" : "+v"(a), "+v"(b));
}
__device__ __forceinline__ void swap_halves32(float &a, float &b)
{
    asm("s_nop 1\n\tv_permlane32_swap_b32 %0, %1" : "+v"(a), "+v"(b));
}
__device__ __forceinline__ float quad_rows_max(float v)
{
    float a = v, b = v;
    swap_rows16(a, b);
    a = b = fmaxf(a, b);
    swap_halves32(a, b);
    return fmaxf(a, b);
}
__device__ __forceinline__ float quad_rows_sum(float v)
{
    float a = v, b = v;
    swap_rows16(a, b);
    a = b = a + b;
    swap_halves32(a, b);
    return a + b;
}

__device__ __forceinline__ float wave_sum(float v)
{
#pragma unroll
    for (int o = 32; o > 0; o >>= 1) v += __shfl_xor(v, o);
    return v;
}

}  // namespace dskv
