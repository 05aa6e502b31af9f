// Rotary position embedding on the ragged q/k of one step, adjacent-pair
// ("interleaved") convention: (x[2j], x[2j+1]) is rotated by
// pos * theta^(-2j/D) with pos = offsets[request] + index within the request.
// Elementwise, HBM-bound; one workgroup per token.  A thread owns one 16-byte
// chunk column of the head dimension, evaluates its sin/cos once and walks the
// heads, so the transcendental work is per (token, dim pair), not per head.
#include "rope_math.h"

namespace dskv {

// Where the fused variant puts the rotated K row and the V row of a token: the
// page slot the append would have chosen (see append.hip).
struct AppendTarget {
    char *pages;                 // layer base; nullptr = plain rope (k goes to k_out)
    const char *v;               // (nnz, Hkv, D) values to store next to K
    const int32_t *kv_indices, *kv_indptr, *kv_last;
    int page_size;
    int num_pages;               // pages in the layer: an id outside [0, num_pages) is never written
};

template <int DT>
__global__ __launch_bounds__(256) void rope_kernel(char *__restrict__ q_out, char *__restrict__ k_out,
                                                   const char *__restrict__ q,
                                                   const char *__restrict__ k,
                                                   const int32_t *__restrict__ qo_indptr,
                                                   const int32_t *__restrict__ offsets, int batch,
                                                   int n_qo_heads, int n_kv_heads, int head_dim,
                                                   float theta, AppendTarget tgt, RopeFreqs freqs)
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
        if (page < 0 || page >= tgt.num_pages) return;      // an id outside the pool: touch nothing
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
    for (int j = 0; j < E / 2; j++) rope_angle(pos, col * (E / 2) + j, head_dim, theta, freqs, cs[j], sn[j]);
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
        rope_rotate<E / 2>(f, cs, sn);
        *reinterpret_cast<u32x4 *>(dst) = C::pack(f);
    }
    if (v_dst) {   // fused append: V rows are copied as they are
        const char *v_src = tgt.v + (long)t * kv_row_bytes;
        for (long off = threadIdx.x * 16L; off < kv_row_bytes; off += 256 * 16)
            *reinterpret_cast<u32x4 *>(v_dst + off) = *reinterpret_cast<const u32x4 *>(v_src + off);
    }
}

// cos | sin of every (request, dim pair) of a decode step: table[b][0 .. D/2) = cos,
// table[b][D/2 .. D) = sin of positions[b] * theta^(-2*pair/D).
__global__ __launch_bounds__(256) void rope_table_kernel(float *__restrict__ table,
                                                         const int32_t *__restrict__ positions,
                                                         int batch, int head_dim, float theta,
                                                         RopeFreqs freqs)
{
    const int pairs = head_dim / 2;
    const long i = (long)blockIdx.x * 256 + threadIdx.x;
    if (i >= (long)batch * pairs) return;
    const int b = (int)(i / pairs), pair = (int)(i - (long)b * pairs);
    float cs, sn;
    rope_angle((float)positions[b], pair, head_dim, theta, freqs, cs, sn);
    table[(long)b * head_dim + pair] = cs;
    table[(long)b * head_dim + pairs + pair] = sn;
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
    const RopeFreqs freqs = rope_freqs(rope_theta, head_dim);
#define DSKV_LAUNCH_ROPE(DT)                                                                    \
    hipLaunchKernelGGL((rope_kernel<DT>), dim3((unsigned)nnz), dim3(256), 0, s, (char *)q_out,  \
                       (char *)k_out, (const char *)q, (const char *)k, qo_indptr, offsets,     \
                       batch, n_qo_heads, n_kv_heads, head_dim, rope_theta, tgt, freqs)
    if (dtype == DSKV_F32) DSKV_LAUNCH_ROPE(DSKV_F32);
    else if (dtype == DSKV_F16) DSKV_LAUNCH_ROPE(DSKV_F16);
    else DSKV_LAUNCH_ROPE(DSKV_BF16);
#undef DSKV_LAUNCH_ROPE
    DSKV_LAUNCH_CHECK("rope_kernel");
    return 0;
}

}  // namespace dskv

extern "C" int dskv_rope_table(float *table, const int32_t *positions, int32_t batch,
                               int32_t head_dim, float rope_theta, void *stream)
{
    using namespace dskv;
    DSKV_REQUIRE(batch >= 0, "rope_table: negative batch");
    if (batch == 0) return 0;
    DSKV_REQUIRE(table && positions, "rope_table: null pointer argument");
    DSKV_REQUIRE(head_dim > 0 && head_dim % 8 == 0, "rope_table: head_dim %d must be a multiple of 8",
                 head_dim);
    DSKV_REQUIRE(rope_theta > 0.f, "rope_table: rope_theta must be positive");
    DSKV_REQUIRE((uintptr_t)table % 16 == 0, "rope_table: the table must be 16-byte aligned");
    const long n = (long)batch * (head_dim / 2);
    hipLaunchKernelGGL(rope_table_kernel, dim3((unsigned)((n + 255) / 256)), dim3(256), 0,
                       (hipStream_t)stream, table, positions, batch, head_dim, rope_theta,
                       rope_freqs(rope_theta, head_dim));
    DSKV_LAUNCH_CHECK("rope_table_kernel");
    return 0;
}

extern "C" int dskv_apply_rope(void *q_out, void *k_out, const void *q, const void *k,
                               const int32_t *qo_indptr, const int32_t *offsets, int32_t batch,
                               int32_t nnz, int32_t n_qo_heads, int32_t n_kv_heads,
                               int32_t head_dim, float rope_theta, int32_t dtype, void *stream)
{
    dskv::AppendTarget none = {nullptr, nullptr, nullptr, nullptr, nullptr, 1, 0};
    return dskv::launch_rope(q_out, k_out, q, k, qo_indptr, offsets, batch, nnz, n_qo_heads,
                             n_kv_heads, head_dim, rope_theta, dtype, none, stream, "apply_rope");
}

extern "C" int dskv_rope_append_paged_kv(void *q_out, void *pages_layer, int32_t num_pages,
                                         const void *q,
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
        DSKV_REQUIRE(num_pages > 0, "rope_append: num_pages must be positive, got %d", num_pages);
    }
    AppendTarget tgt = {(char *)pages_layer, (const char *)v, kv_page_indices, kv_page_indptr,
                        kv_last_page_len, page_size, num_pages};
    return launch_rope(q_out, nullptr, q, k, qo_indptr, offsets, batch, nnz, n_qo_heads, n_kv_heads,
                       head_dim, rope_theta, dtype, tgt, stream, "rope_append");
}
