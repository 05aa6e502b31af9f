// Rotary position embedding on the ragged q/k of one step, adjacent-pair
// ("interleaved") convention: (x[2j], x[2j+1]) is rotated by
// pos * theta^(-2j/D) with pos = offsets[request] + index within the request.
// Elementwise, HBM-bound; one workgroup per token.  The token's sines and cosines are
// evaluated once per (token, dim pair) into LDS; a thread owns one 16-byte chunk column
// of the head dimension and walks the heads.
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

// A chunk's tokens are a few rounds of workgroups on the chip, so the kernel lasts as long as a
// workgroup's chain of dependent loads plus the copy itself.  The chain is kept short as in the
// append kernel: the token's q, k (and v) chunks are requested first (their addresses need no
// metadata: up to kRopeHeadsInFlight heads per thread are held in registers); the request that
// owns the token comes from ONE vector load of qo_indptr and a ballot (lane i holds entry i;
// batches of 64 requests or more take a binary search), with the request's offset, block-table
// range and last-page length fetched by the same lanes at the same time; the page id is the
// last link.
constexpr int kRopeHeadsInFlight = 6;
constexpr int kRopeMaxPairs = 1024;   // head_dim / 2 at most (a head row is at most 256 chunks of 16 bytes)

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
    const int lane = threadIdx.x & 63;
    const int cols = head_dim / E;           // 16-byte chunks per head row
    const int col = threadIdx.x % cols;
    const int head_lane = threadIdx.x / cols;
    const int head_lanes = 256 / cols;
    const bool works = head_lane < head_lanes;   // the last threads of the workgroup may have no column
    const long row_bytes = (long)head_dim * (16 / E);
    const long kv_row_bytes = (long)n_kv_heads * row_bytes;
    const int total_heads = n_qo_heads + n_kv_heads;
    auto src_of = [&](int h) {
        return h < n_qo_heads ? q + ((long)t * n_qo_heads + h) * row_bytes + col * 16
                              : k + ((long)t * n_kv_heads + (h - n_qo_heads)) * row_bytes + col * 16;
    };

    // link 0: the rows themselves
    u32x4 raw[kRopeHeadsInFlight], v_raw = {0, 0, 0, 0};
#pragma unroll
    for (int i = 0; i < kRopeHeadsInFlight; i++) {
        const int h = head_lane + i * head_lanes;
        if (works && h < total_heads) raw[i] = *reinterpret_cast<const u32x4 *>(src_of(h));
    }
    const char *v_src = tgt.pages ? tgt.v + (long)t * kv_row_bytes : nullptr;
    if (v_src && threadIdx.x * 16L < kv_row_bytes) v_raw = *reinterpret_cast<const u32x4 *>(v_src + threadIdx.x * 16L);

    // link 1: the request that owns token t = largest b with qo_indptr[b] <= t
    int b, first, n_b, offset, page_begin = 0, n_pages = 0, last = 0;
    if (batch < 64) {
        const int i = min(lane, batch), j = min(lane, batch - 1);
        const int q_i = qo_indptr[i];
        const int o_i = offsets[j];
        const int p_i = tgt.pages ? tgt.kv_indptr[i] : 0;
        const int l_i = tgt.pages ? tgt.kv_last[j] : 0;
        const unsigned long long le = __ballot(lane <= batch && q_i <= t);
        b = min(__popcll(le) - 1, batch - 1);
        if (b < 0) return;   // qo_indptr[0] > t: malformed
        first = __shfl(q_i, b);
        n_b = __shfl(q_i, b + 1) - first;
        offset = __shfl(o_i, b);
        page_begin = __shfl(p_i, b);
        n_pages = __shfl(p_i, b + 1) - page_begin;
        last = __shfl(l_i, b);
    } else {
        int lo = 0, hi = batch;
        if (t < batch && qo_indptr[t] == t && qo_indptr[t + 1] == t + 1) {
            lo = t;  // one token per request
        } else {
            while (hi - lo > 1) {
                const int mid = (lo + hi) >> 1;
                if (qo_indptr[mid] <= t) lo = mid; else hi = mid;
            }
        }
        b = lo;
        first = qo_indptr[b];
        n_b = qo_indptr[b + 1] - first;
        offset = offsets[b];
        if (tgt.pages) {
            page_begin = tgt.kv_indptr[b];
            n_pages = tgt.kv_indptr[b + 1] - page_begin;
            last = tgt.kv_last[b];
        }
    }
    if (t - first >= n_b) return;   // token not covered by the metadata
    const float pos = (float)(offset + (t - first));
    char *k_dst = k_out + (long)t * kv_row_bytes;   // rotated K row set of this token
    char *v_dst = nullptr;
    if (tgt.pages) {
        const long kv_len = (long)(n_pages - 1) * tgt.page_size + last;
        const long p = kv_len - n_b + (t - first);
        if (n_pages <= 0 || p < 0 || p >= kv_len) return;   // malformed metadata: touch nothing
        // link 2: the page
        const long page = tgt.kv_indices[page_begin + (int)(p / tgt.page_size)];
        if (page < 0 || page >= tgt.num_pages) return;      // an id outside the pool: touch nothing
        const long half = (long)tgt.page_size * kv_row_bytes;
        k_dst = tgt.pages + page * 2 * half + (p % tgt.page_size) * kv_row_bytes;
        v_dst = k_dst + half;
    }
    // cos and sin of the token's head_dim / 2 angles, each evaluated once per workgroup (a thread
    // needs E / 2 of them, the same ones as every other thread of its column: evaluated per
    // thread, the sincosf calls took as long as the kernel's memory traffic)
    __shared__ float cos_of[kRopeMaxPairs], sin_of[kRopeMaxPairs];
    for (int pair = threadIdx.x; pair < head_dim / 2; pair += 256)
        rope_angle(pos, pair, head_dim, theta, freqs, cos_of[pair], sin_of[pair]);
    __syncthreads();   // every exit above is taken by the whole workgroup or by none of it
    if (works) {
        float cs[E / 2], sn[E / 2];
#pragma unroll
        for (int j = 0; j < E / 2; j++) {
            cs[j] = cos_of[col * (E / 2) + j];
            sn[j] = sin_of[col * (E / 2) + j];
        }
        auto rotate_into = [&](int h, const u32x4 &chunk) {
            char *dst = h < n_qo_heads ? q_out + ((long)t * n_qo_heads + h) * row_bytes + col * 16
                                       : k_dst + (long)(h - n_qo_heads) * row_bytes + col * 16;
            float f[E];
            C::unpack(chunk, f);
            rope_rotate<E / 2>(f, cs, sn);
            *reinterpret_cast<u32x4 *>(dst) = C::pack(f);
        };
#pragma unroll
        for (int i = 0; i < kRopeHeadsInFlight; i++) {
            const int h = head_lane + i * head_lanes;
            if (h < total_heads) rotate_into(h, raw[i]);
        }
        for (int h = head_lane + kRopeHeadsInFlight * head_lanes; h < total_heads; h += head_lanes)
            rotate_into(h, *reinterpret_cast<const u32x4 *>(src_of(h)));
    }
    if (v_dst) {   // fused append: V rows are copied as they are
        if (threadIdx.x * 16L < kv_row_bytes) *reinterpret_cast<u32x4 *>(v_dst + threadIdx.x * 16L) = v_raw;
        for (long off = threadIdx.x * 16L + 256 * 16; off < kv_row_bytes; off += 256 * 16)
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
