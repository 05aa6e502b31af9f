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

// The frequencies 1 / theta^(2*pair/D) of the reference's table (execution/exec.py:44 of
// the reference: fp32 power of the fp32 quotient 2*pair/D, fp32 reciprocal), computed once per
// launch on the host and handed to the kernel by value: the angle pos * inv_freq is then the
// same fp32 product everywhere, and no lane evaluates a power.  The power is taken correctly
// rounded to fp32 (evaluated in double): fp32 library powers differ from that, and from each
// other, in the last bit now and then, and at position 4000 one ulp of a frequency is 2e-4 rad.
// Head dims over 256 (more pairs than the table holds) evaluate the power on the device.
constexpr int kRopeTablePairs = 128;
struct RopeFreqs {
    float inv[kRopeTablePairs];
    int pairs;   // entries filled; 0: evaluate on the device
};
static inline RopeFreqs rope_freqs(float theta, int head_dim)
{
    RopeFreqs f;
    f.pairs = head_dim / 2 <= kRopeTablePairs ? head_dim / 2 : 0;
    for (int j = 0; j < kRopeTablePairs; j++)
        f.inv[j] = j < f.pairs
                       ? 1.0f / (float)pow((double)theta, (double)((float)(2 * j) / (float)head_dim))
                       : 0.f;
    return f;
}

// cos and sin of pos * theta^(-2*pair/D).
__device__ __forceinline__ void rope_angle(float pos, int pair, int head_dim, float theta,
                                           const RopeFreqs &freqs, float &cs, float &sn)
{
    const float inv_freq = freqs.pairs > 0 ? freqs.inv[pair]
                                           : 1.0f / powf(theta, (float)(2 * pair) / (float)head_dim);
    // the angle is the rounded fp32 product, as in the reference's table (torch.outer of fp32
    // values): __fmul_rn keeps the compiler from fusing it into the range reduction of sincosf,
    // which it would do in one kernel and not in another
    sincosf(__fmul_rn(pos, inv_freq), &sn, &cs);
}

// (f[2j], f[2j+1]) rotated by the angle whose cosine and sine are cs[j], sn[j].
template <int kPairs>
__device__ __forceinline__ void rope_rotate(float *f, const float *cs, const float *sn)
{
#pragma unroll
    for (int j = 0; j < kPairs; j++) {
        // one product rounded, the other fused, spelled out: left to the compiler, which of the
        // two gets fused differs from kernel to kernel, and the fused decode launch must give
        // the bits of the stand-alone rotation
        const float re = f[2 * j], im = f[2 * j + 1];
        f[2 * j] = __fmaf_rn(re, cs[j], -__fmul_rn(im, sn[j]));
        f[2 * j + 1] = __fmaf_rn(re, sn[j], __fmul_rn(im, cs[j]));
    }
}

}  // namespace dskv
