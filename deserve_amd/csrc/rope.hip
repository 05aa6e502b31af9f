// Rotary position embedding on the ragged q/k of one step, adjacent-pair
// ("interleaved") convention: (x[2j], x[2j+1]) is rotated by
// pos * theta^(-2j/D) with pos = offsets[request] + index within the request.
// Elementwise, HBM-bound; one workgroup per token.  A thread owns one 16-byte
// chunk column of the head dimension, evaluates its sin/cos once and walks the
// heads, so the transcendental work is per (token, dim pair), not per head.
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

// Where the fused variant puts the rotated K row and the V row of a token: the
// page slot the append would have chosen (see append.hip).
struct AppendTarget {
    char *pages;                 // layer base; nullptr = plain rope (k goes to k_out)
    const char *v;               // (nnz, Hkv, D) values to store next to K
    const int32_t *kv_indices, *kv_indptr, *kv_last;
    int page_size;
};

template <int DT>
__global__ __launch_bounds__(256) void rope_kernel(char *__restrict__ q_out, char *__restrict__ k_out,
                                                   const char *__restrict__ q,
                                                   const char *__restrict__ k,
                                                   const int32_t *__restrict__ qo_indptr,
                                                   const int32_t *__restrict__ offsets, int batch,
                                                   int n_qo_heads, int n_kv_heads, int head_dim,
                                                   float theta, AppendTarget tgt)
{
    typedef Chunk<DT> C;
    constexpr int E = C::kElems;
    const int t = blockIdx.x;
    int lo = 0, hi = batch;   // largest b with qo_indptr[b] <= t
    while (hi - lo > 1) {
        const int mid = (lo + hi) >> 1;
        if (qo_indptr[mid] <= t) lo = mid; else hi = mid;
    }
    if (t >= qo_indptr[lo + 1]) return;   // token not covered by the metadata
    const float pos = (float)(offsets[lo] + (t - qo_indptr[lo]));
    const long kv_row_bytes = (long)n_kv_heads * head_dim * (16 / E);
    char *k_dst = k_out + (long)t * kv_row_bytes;   // rotated K row set of this token
    char *v_dst = nullptr;
    if (tgt.pages) {
        const int page_begin = tgt.kv_indptr[lo];
        const int n_pages = tgt.kv_indptr[lo + 1] - page_begin;
        const long kv_len = (long)(n_pages - 1) * tgt.page_size + tgt.kv_last[lo];
        const long p = kv_len - (qo_indptr[lo + 1] - qo_indptr[lo]) + (t - qo_indptr[lo]);
        if (n_pages <= 0 || p < 0 || p >= kv_len) return;   // malformed metadata: touch nothing
        const long page = tgt.kv_indices[page_begin + (int)(p / tgt.page_size)];
        const long half = (long)tgt.page_size * kv_row_bytes;
        k_dst = tgt.pages + page * 2 * half + (p % tgt.page_size) * kv_row_bytes;
        v_dst = k_dst + half;
    }

    const int cols = head_dim / E;           // 16-byte chunks per head row
    const int col = threadIdx.x % cols;
    const int head_lane = threadIdx.x / cols;
    const int head_lanes = 256 / cols;
    if (head_lane >= head_lanes) return;

    float cs[E / 2], sn[E / 2];
#pragma unroll
    for (int j = 0; j < E / 2; j++) {
        const int pair = col * (E / 2) + j;
        // theta^(-2*pair/D), evaluated as the reference's table does: 1 / theta^(2*pair/D)
        const float inv_freq = 1.0f / powf(theta, (float)(2 * pair) / (float)head_dim);
        sincosf(pos * inv_freq, &sn[j], &cs[j]);
    }
    const long row_bytes = (long)head_dim * (16 / E);
    const int total_heads = n_qo_heads + n_kv_heads;
    for (int h = head_lane; h < total_heads; h += head_lanes) {
        const bool is_q = h < n_qo_heads;
        const long off = is_q ? ((long)t * n_qo_heads + h) * row_bytes
                              : ((long)t * n_kv_heads + (h - n_qo_heads)) * row_bytes;
        const char *src = (is_q ? q : k) + off + col * 16;
        char *dst = is_q ? q_out + off + col * 16
                         : k_dst + (long)(h - n_qo_heads) * row_bytes + col * 16;
        float f[E];
        C::unpack(*reinterpret_cast<const u32x4 *>(src), f);
#pragma unroll
        for (int j = 0; j < E / 2; j++) {
            const float re = f[2 * j], im = f[2 * j + 1];
            f[2 * j] = re * cs[j] - im * sn[j];
            f[2 * j + 1] = re * sn[j] + im * cs[j];
        }
        *reinterpret_cast<u32x4 *>(dst) = C::pack(f);
    }
    if (v_dst) {   // fused append: V rows are copied as they are
        const char *v_src = tgt.v + (long)t * kv_row_bytes;
        for (long off = threadIdx.x * 16L; off < kv_row_bytes; off += 256 * 16)
            *reinterpret_cast<u32x4 *>(v_dst + off) = *reinterpret_cast<const u32x4 *>(v_src + off);
    }
}

static int launch_rope(void *q_out, void *k_out, const void *q, const void *k,
                       const int32_t *qo_indptr, const int32_t *offsets, int32_t batch, int32_t nnz,
                       int32_t n_qo_heads, int32_t n_kv_heads, int32_t head_dim, float rope_theta,
                       int32_t dtype, const AppendTarget &tgt, void *stream, const char *who)
{
    DSKV_REQUIRE(batch >= 0 && nnz >= 0, "%s: negative batch/nnz", who);
    if (batch == 0 || nnz == 0) return 0;
    DSKV_REQUIRE(q_out && q && k && qo_indptr && offsets && (k_out || tgt.pages),
                 "%s: null pointer argument", who);
    DSKV_REQUIRE(dtype == DSKV_F32 || dtype == DSKV_F16 || dtype == DSKV_BF16,
                 "%s: unknown dtype %d", who, dtype);
    const int elems = dtype == DSKV_F32 ? 4 : 8;
    DSKV_REQUIRE(head_dim > 0 && head_dim % elems == 0 && head_dim / elems <= 256,
                 "%s: head_dim %d must be a multiple of %d and at most %d", who, head_dim, elems,
                 256 * elems);
    DSKV_REQUIRE(n_qo_heads > 0 && n_kv_heads > 0, "%s: bad head counts", who);
    DSKV_REQUIRE(rope_theta > 0.f, "%s: rope_theta must be positive", who);
    DSKV_REQUIRE(((uintptr_t)q_out | (uintptr_t)k_out | (uintptr_t)q | (uintptr_t)k |
                  (uintptr_t)tgt.pages | (uintptr_t)tgt.v) % 16 == 0,
                 "%s: tensors must be 16-byte aligned", who);
    hipStream_t s = (hipStream_t)stream;
#define DSKV_LAUNCH_ROPE(DT)                                                                    \
    hipLaunchKernelGGL((rope_kernel<DT>), dim3((unsigned)nnz), dim3(256), 0, s, (char *)q_out,  \
                       (char *)k_out, (const char *)q, (const char *)k, qo_indptr, offsets,     \
                       batch, n_qo_heads, n_kv_heads, head_dim, rope_theta, tgt)
    if (dtype == DSKV_F32) DSKV_LAUNCH_ROPE(DSKV_F32);
    else if (dtype == DSKV_F16) DSKV_LAUNCH_ROPE(DSKV_F16);
    else DSKV_LAUNCH_ROPE(DSKV_BF16);
#undef DSKV_LAUNCH_ROPE
    DSKV_LAUNCH_CHECK("rope_kernel");
    return 0;
}

}  // namespace dskv

extern "C" int dskv_apply_rope(void *q_out, void *k_out, const void *q, const void *k,
                               const int32_t *qo_indptr, const int32_t *offsets, int32_t batch,
                               int32_t nnz, int32_t n_qo_heads, int32_t n_kv_heads,
                               int32_t head_dim, float rope_theta, int32_t dtype, void *stream)
{
    dskv::AppendTarget none = {nullptr, nullptr, nullptr, nullptr, nullptr, 1};
    return dskv::launch_rope(q_out, k_out, q, k, qo_indptr, offsets, batch, nnz, n_qo_heads,
                             n_kv_heads, head_dim, rope_theta, dtype, none, stream, "apply_rope");
}

extern "C" int dskv_rope_append_paged_kv(void *q_out, void *pages_layer, const void *q,
                                         const void *k, const void *v, const int32_t *qo_indptr,
                                         const int32_t *offsets, const int32_t *kv_page_indices,
                                         const int32_t *kv_page_indptr,
                                         const int32_t *kv_last_page_len, int32_t batch,
                                         int32_t nnz, int32_t page_size, int32_t n_qo_heads,
                                         int32_t n_kv_heads, int32_t head_dim, float rope_theta,
                                         int32_t dtype, void *stream)
{
    using namespace dskv;
    if (batch > 0 && nnz > 0) {
        DSKV_REQUIRE(pages_layer && v && kv_page_indices && kv_page_indptr && kv_last_page_len,
                     "rope_append: null pointer argument");
        DSKV_REQUIRE(page_size > 0, "rope_append: page_size must be positive");
    }
    AppendTarget tgt = {(char *)pages_layer, (const char *)v, kv_page_indices, kv_page_indptr,
                        kv_last_page_len, page_size};
    return launch_rope(q_out, nullptr, q, k, qo_indptr, offsets, batch, nnz, n_qo_heads, n_kv_heads,
                       head_dim, rope_theta, dtype, tgt, stream, "rope_append");
}
