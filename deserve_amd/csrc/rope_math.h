// 16-byte chunks of a head row as fp32 lanes, and the adjacent-pair rotation of
// rotary position embedding on them.  Shared by the RoPE kernel and by the decode
// attention kernel's fused form, so both round the same way.
#pragma once

#include "common.h"

#include <math.h>

namespace dskv {

template <int DT> struct Chunk;   // 16 bytes <-> fp32 lanes
template <> struct Chunk<DSKV_F32> {
    static constexpr int kElems = 4;
    static __device__ __forceinline__ void unpack(u32x4 raw, float *f) {
        const f32x4 v = __builtin_bit_cast(f32x4, raw);
        f[0] = v.x;
        f[1] = v.y;
        f[2] = v.z;
        f[3] = v.w;
    }
    static __device__ __forceinline__ u32x4 pack(const float *f) {
        const f32x4 v = {f[0], f[1], f[2], f[3]};
        return __builtin_bit_cast(u32x4, v);
    }
};
template <> struct Chunk<DSKV_F16> {
    static constexpr int kElems = 8;
    typedef _Float16 h8 __attribute__((ext_vector_type(8)));
    typedef float f8 __attribute__((ext_vector_type(8)));
    static __device__ __forceinline__ void unpack(u32x4 raw, float *f) {
        const f8 v = __builtin_convertvector(__builtin_bit_cast(h8, raw), f8);
        f[0] = v.s0; f[1] = v.s1; f[2] = v.s2; f[3] = v.s3;
        f[4] = v.s4; f[5] = v.s5; f[6] = v.s6; f[7] = v.s7;
    }
    static __device__ __forceinline__ u32x4 pack(const float *f) {
        const f8 v = {f[0], f[1], f[2], f[3], f[4], f[5], f[6], f[7]};
        return __builtin_bit_cast(u32x4, __builtin_convertvector(v, h8));
    }
};
template <> struct Chunk<DSKV_BF16> {
    static constexpr int kElems = 8;
    typedef __bf16 b2 __attribute__((ext_vector_type(2)));
    static __device__ __forceinline__ void unpack(u32x4 raw, float *f) {
#pragma unroll
        for (int i = 0; i < 4; i++) {
            f[2 * i] = __builtin_bit_cast(float, raw[i] << 16);
            f[2 * i + 1] = __builtin_bit_cast(float, raw[i] & 0xFFFF0000u);
        }
    }
    static __device__ __forceinline__ u32x4 pack(const float *f) {
        u32x4 r;
#pragma unroll
        for (int i = 0; i < 4; i++) {
            b2 p = {(__bf16)f[2 * i], (__bf16)f[2 * i + 1]};
            r[i] = __builtin_bit_cast(uint32_t, p);
        }
        return r;
    }
};

// cos and sin of pos * theta^(-2*pair/D), evaluated as the reference's table does:
// 1 / theta^(2*pair/D).
__device__ __forceinline__ void rope_angle(float pos, int pair, int head_dim, float theta,
                                           float &cs, float &sn)
{
    const float inv_freq = 1.0f / powf(theta, (float)(2 * pair) / (float)head_dim);
    sincosf(pos * inv_freq, &sn, &cs);
}

// (f[2j], f[2j+1]) rotated by the angle whose cosine and sine are cs[j], sn[j].
template <int kPairs>
__device__ __forceinline__ void rope_rotate(float *f, const float *cs, const float *sn)
{
#pragma unroll
    for (int j = 0; j < kPairs; j++) {
        const float re = f[2 * j], im = f[2 * j + 1];
        f[2 * j] = re * cs[j] - im * sn[j];
        f[2 * j + 1] = re * sn[j] + im * cs[j];
    }
}

}  // namespace dskv
