// Merge pass over the partials of rows cut into a few parts (head_dim 128, 16-bit output):
// shared by the prefill path (tiles cut into parts) and the decode path (requests cut across
// workgroups).
#pragma once

#include "kv_tile.h"

namespace dskv {

// Output row `row`, head qh = sum_i w_i O_i / sum_i w_i l_i over the kParts partials in slots
// first .. first + kParts - 1, w_i = exp2(m_i - max_j m_j).  A thread owns 16 consecutive dims
// of one head and requests the values of all parts at once: one trip to memory per row.
template <int DT, int kParts>
__device__ __forceinline__ void merge_row_parts(uint16_t *__restrict__ out, const float *__restrict__ part_o,
                                                const float *__restrict__ part_ml, long row, long first,
                                                int n_qo_heads)
{
    typedef Elt<DT> E;
    for (int idx = threadIdx.x; idx < n_qo_heads * (kHeadDim / 16); idx += blockDim.x) {
        const int qh = idx / (kHeadDim / 16), d0 = (idx % (kHeadDim / 16)) * 16;
        f32x4 o[kParts][4];
        float m[kParts], l[kParts];
#pragma unroll
        for (int i = 0; i < kParts; i++) {
            const long slot = first + i;
            const float *src = part_o + (slot * n_qo_heads + qh) * kHeadDim + d0;
#pragma unroll
            for (int j = 0; j < 4; j++) o[i][j] = *reinterpret_cast<const f32x4 *>(src + 4 * j);
            const float *ml = part_ml + (slot * n_qo_heads + qh) * 2;
            m[i] = ml[0];
            l[i] = ml[1];
        }
        float m_all = m[0];
#pragma unroll
        for (int i = 1; i < kParts; i++) m_all = fmaxf(m_all, m[i]);
        f32x4 acc[4] = {f32x4{0.f, 0.f, 0.f, 0.f}, f32x4{0.f, 0.f, 0.f, 0.f}, f32x4{0.f, 0.f, 0.f, 0.f},
                        f32x4{0.f, 0.f, 0.f, 0.f}};
        float l_all = 0.f;
#pragma unroll
        for (int i = 0; i < kParts; i++) {
            const float w = __builtin_amdgcn_exp2f(m[i] - m_all);
            l_all += w * l[i];
#pragma unroll
            for (int j = 0; j < 4; j++) acc[j] += w * o[i][j];
        }
        const float inv = l_all > 0.f ? 1.f / l_all : 0.f;
        uint16_t *dst = out + (row * n_qo_heads + qh) * kHeadDim + d0;
#pragma unroll
        for (int j = 0; j < 4; j += 2) {
            const u32x4 w4 = {E::pack2(acc[j][0] * inv, acc[j][1] * inv), E::pack2(acc[j][2] * inv, acc[j][3] * inv),
                              E::pack2(acc[j + 1][0] * inv, acc[j + 1][1] * inv),
                              E::pack2(acc[j + 1][2] * inv, acc[j + 1][3] * inv)};
            *reinterpret_cast<u32x4 *>(dst + 4 * j) = w4;
        }
    }
}

// The same for any number of parts, four at a time under a running maximum.
template <int DT>
__device__ __forceinline__ void merge_row_many_parts(uint16_t *__restrict__ out, const float *__restrict__ part_o,
                                                     const float *__restrict__ part_ml, long row, long first,
                                                     int n, int n_qo_heads)
{
    typedef Elt<DT> E;
    constexpr int kAtOnce = 4;
    for (int idx = threadIdx.x; idx < n_qo_heads * (kHeadDim / 16); idx += blockDim.x) {
        const int qh = idx / (kHeadDim / 16), d0 = (idx % (kHeadDim / 16)) * 16;
        f32x4 acc[4] = {f32x4{0.f, 0.f, 0.f, 0.f}, f32x4{0.f, 0.f, 0.f, 0.f}, f32x4{0.f, 0.f, 0.f, 0.f},
                        f32x4{0.f, 0.f, 0.f, 0.f}};
        float m_all = kNegBig, l_all = 0.f;
        for (int i0 = 0; i0 < n; i0 += kAtOnce) {
            f32x4 o[kAtOnce][4];
            float m[kAtOnce], l[kAtOnce];
#pragma unroll
            for (int i = 0; i < kAtOnce; i++) {
                const long slot = first + min(i0 + i, n - 1);
                const float *src = part_o + (slot * n_qo_heads + qh) * kHeadDim + d0;
#pragma unroll
                for (int j = 0; j < 4; j++) o[i][j] = *reinterpret_cast<const f32x4 *>(src + 4 * j);
                const float *ml = part_ml + (slot * n_qo_heads + qh) * 2;
                m[i] = i0 + i < n ? ml[0] : kNegBig;
                l[i] = i0 + i < n ? ml[1] : 0.f;
            }
            float m_new = m_all;
#pragma unroll
            for (int i = 0; i < kAtOnce; i++) m_new = fmaxf(m_new, m[i]);
            const float keep = __builtin_amdgcn_exp2f(m_all - m_new);
            l_all *= keep;
#pragma unroll
            for (int j = 0; j < 4; j++) acc[j] *= keep;
#pragma unroll
            for (int i = 0; i < kAtOnce; i++) {
                // a part past the row's last one repeats it with weight zero
                const float w = i0 + i < n ? __builtin_amdgcn_exp2f(m[i] - m_new) : 0.f;
                l_all += w * l[i];
#pragma unroll
                for (int j = 0; j < 4; j++) acc[j] += w * o[i][j];
            }
            m_all = m_new;
        }
        const float inv = l_all > 0.f ? 1.f / l_all : 0.f;
        uint16_t *dst = out + (row * n_qo_heads + qh) * kHeadDim + d0;
#pragma unroll
        for (int j = 0; j < 4; j += 2) {
            const u32x4 w4 = {E::pack2(acc[j][0] * inv, acc[j][1] * inv), E::pack2(acc[j][2] * inv, acc[j][3] * inv),
                              E::pack2(acc[j + 1][0] * inv, acc[j + 1][1] * inv),
                              E::pack2(acc[j + 1][2] * inv, acc[j + 1][3] * inv)};
            *reinterpret_cast<u32x4 *>(dst + 4 * j) = w4;
        }
    }
}

// row_parts[2 r] = row r's first slot, row_parts[2 r + 1] = its number of parts (consecutive
// slots); 0: the row was written by the attention kernel itself and is left alone.  One
// workgroup per row; row_map (may be null) names the output row of r.
template <int DT>
__global__ __launch_bounds__(256) void merge_parts_kernel(
    uint16_t *__restrict__ out, const float *__restrict__ part_o, const float *__restrict__ part_ml,
    const int32_t *__restrict__ row_parts, const int32_t *__restrict__ row_map, int max_slots,
    int n_qo_heads)
{
    const long r = blockIdx.x;
    const const_i32_ptr table = as_const(row_parts) + 2 * r;
    const int first = table[0], n = table[1];   // uniform over the workgroup
    if (n <= 0 || first < 0 || first + n > max_slots) return;
    const long row = row_map ? as_const(row_map)[r] : r;
    switch (n) {
    case 1: merge_row_parts<DT, 1>(out, part_o, part_ml, row, first, n_qo_heads); break;
    case 2: merge_row_parts<DT, 2>(out, part_o, part_ml, row, first, n_qo_heads); break;
    case 3: merge_row_parts<DT, 3>(out, part_o, part_ml, row, first, n_qo_heads); break;
    case 4: merge_row_parts<DT, 4>(out, part_o, part_ml, row, first, n_qo_heads); break;
    case 5: merge_row_parts<DT, 5>(out, part_o, part_ml, row, first, n_qo_heads); break;
    case 6: merge_row_parts<DT, 6>(out, part_o, part_ml, row, first, n_qo_heads); break;
    case 7: merge_row_parts<DT, 7>(out, part_o, part_ml, row, first, n_qo_heads); break;
    case 8: merge_row_parts<DT, 8>(out, part_o, part_ml, row, first, n_qo_heads); break;
    default: merge_row_many_parts<DT>(out, part_o, part_ml, row, first, n, n_qo_heads); break;
    }
}

}  // namespace dskv
