// KV append: scatter the new K/V rows of a ragged batch into their page slots.
// Pure byte movement (bit-exact by construction); HBM-bound for prefill chunks,
// launch-bound at decode sizes.
//
// Mapping: one 64-lane wavefront per token.  A token's K row set
// (n_kv_heads * head_dim elements, 2 KiB in bf16) is contiguous both in the
// source and in the page slot, so every lane moves 16 bytes per instruction and
// a wavefront moves 1 KiB per load/store pair, fully coalesced.
//
// A chunk of 8192 tokens is one round of waves on the chip (32 per CU), so the
// kernel lasts as long as its chain of dependent loads plus the copy itself.
// The chain is kept at two links: the token's rows are requested first (their
// address needs no metadata); the request that owns the token is found from ONE
// vector load of qo_indptr (lane i holds entry i; the owner is the number of
// entries <= t, a ballot and a popcount) instead of a binary search of
// dependent loads, with kv_page_indptr and kv_last_page_len fetched by the same
// lanes at the same time; the page id is the second link.  Batches over 63
// requests take the binary search.
#include "common.h"

namespace dskv {

constexpr int kAppendWaves = 4;
constexpr int kAppendMaxChunks = 4;   // 16-byte chunks per lane and row set held in registers (row sets <= 4 KiB)

__global__ __launch_bounds__(64 * kAppendWaves) void append_kernel(
    char *__restrict__ pages, const char *__restrict__ k, const char *__restrict__ v,
    const int32_t *__restrict__ qo_indptr, const int32_t *__restrict__ kv_indices,
    const int32_t *__restrict__ kv_indptr, const int32_t *__restrict__ kv_last, int batch, int nnz,
    int page_size, int row_bytes, int num_pages)
{
    const int lane = threadIdx.x & 63;
    const int t = blockIdx.x * kAppendWaves + (threadIdx.x >> 6);
    if (t >= nnz) return;

    // link 0: the rows themselves (row sets beyond 4 KiB are copied after the lookup)
    const char *src_k = k + (long)t * row_bytes;
    const char *src_v = v + (long)t * row_bytes;
    const bool in_regs = row_bytes <= kAppendMaxChunks * 64 * 16;
    u32x4 rk[kAppendMaxChunks], rv[kAppendMaxChunks];
    if (in_regs) {
#pragma unroll
        for (int i = 0; i < kAppendMaxChunks; i++) {
            const int off = (i * 64 + lane) * 16;
            if (off < row_bytes) {
                rk[i] = __builtin_nontemporal_load(reinterpret_cast<const u32x4 *>(src_k + off));
                rv[i] = __builtin_nontemporal_load(reinterpret_cast<const u32x4 *>(src_v + off));
            }
        }
    }

    // link 1: request that owns token t = largest b with qo_indptr[b] <= t
    int b, n_b, first, page_begin, n_pages, last;
    if (batch < 64) {
        const int i = min(lane, batch);
        const int q_i = qo_indptr[i];
        const int p_i = kv_indptr[i];
        const int l_i = kv_last[min(lane, batch - 1)];
        const unsigned long long le = __ballot(lane <= batch && q_i <= t);
        b = min(__popcll(le) - 1, batch - 1);
        if (b < 0) return;   // qo_indptr[0] > t: malformed
        first = __shfl(q_i, b);
        n_b = __shfl(q_i, b + 1) - first;
        page_begin = __shfl(p_i, b);
        n_pages = __shfl(p_i, b + 1) - page_begin;
        last = __shfl(l_i, b);
    } else {
        int lo = 0, hi = batch;  // invariant: qo_indptr[lo] <= t < qo_indptr[hi]
        if (t < batch && qo_indptr[t] == t && qo_indptr[t + 1] == t + 1) {
            lo = t;  // decode: one token per request
        } else {
            while (hi - lo > 1) {
                int mid = (lo + hi) >> 1;
                if (qo_indptr[mid] <= t) lo = mid; else hi = mid;
            }
        }
        b = lo;
        first = qo_indptr[b];
        n_b = qo_indptr[b + 1] - first;
        page_begin = kv_indptr[b];
        n_pages = kv_indptr[b + 1] - page_begin;
        last = kv_last[b];
    }
    const long kv_len = (long)(n_pages - 1) * page_size + last;
    const long pos = kv_len - n_b + (t - first);
    if (n_pages <= 0 || pos < 0 || pos >= kv_len) return;  // malformed metadata: touch nothing
    // link 2: the page
    const long page = kv_indices[page_begin + (int)(pos / page_size)];
    if (page < 0 || page >= num_pages) return;             // an id outside the pool: touch nothing
    const long slot = pos % page_size;

    const long half_bytes = (long)page_size * row_bytes;
    char *dst_k = pages + page * 2 * half_bytes + slot * row_bytes;
    char *dst_v = dst_k + half_bytes;
    if (in_regs) {
#pragma unroll
        for (int i = 0; i < kAppendMaxChunks; i++) {
            const int off = (i * 64 + lane) * 16;
            if (off < row_bytes) {
                __builtin_nontemporal_store(rk[i], reinterpret_cast<u32x4 *>(dst_k + off));
                __builtin_nontemporal_store(rv[i], reinterpret_cast<u32x4 *>(dst_v + off));
            }
        }
    } else {
        for (int off = lane * 16; off < row_bytes; off += 64 * 16) {
            u32x4 a = *reinterpret_cast<const u32x4 *>(src_k + off);
            u32x4 c = *reinterpret_cast<const u32x4 *>(src_v + off);
            *reinterpret_cast<u32x4 *>(dst_k + off) = a;
            *reinterpret_cast<u32x4 *>(dst_v + off) = c;
        }
    }
}

}  // namespace dskv

extern "C" int dskv_append_paged_kv(void *pages_layer, int32_t num_pages, const void *k, const void *v,
                                    const int32_t *qo_indptr, const int32_t *kv_page_indices,
                                    const int32_t *kv_page_indptr, const int32_t *kv_last_page_len,
                                    int32_t batch, int32_t nnz, int32_t page_size,
                                    int32_t n_kv_heads, int32_t head_dim, int32_t elt_bytes,
                                    void *stream)
{
    using namespace dskv;
    DSKV_REQUIRE(batch >= 0 && nnz >= 0, "append: negative batch/nnz (%d, %d)", batch, nnz);
    if (batch == 0 || nnz == 0) return 0;
    DSKV_REQUIRE(pages_layer && k && v && qo_indptr && kv_page_indices && kv_page_indptr &&
                     kv_last_page_len, "append: null pointer argument");
    DSKV_REQUIRE(page_size > 0 && n_kv_heads > 0 && head_dim > 0, "append: bad shape");
    DSKV_REQUIRE(num_pages > 0, "append: num_pages must be positive, got %d", num_pages);
    DSKV_REQUIRE(elt_bytes == 2 || elt_bytes == 4, "append: elt_bytes must be 2 or 4, got %d",
                 elt_bytes);
    const int64_t row_bytes = (int64_t)n_kv_heads * head_dim * elt_bytes;
    DSKV_REQUIRE(row_bytes % 16 == 0 && row_bytes < (1 << 30),
                 "append: a token's row set (%lld bytes) must be a multiple of 16 bytes",
                 (long long)row_bytes);
    DSKV_REQUIRE(((uintptr_t)pages_layer | (uintptr_t)k | (uintptr_t)v) % 16 == 0,
                 "append: pages/k/v must be 16-byte aligned");
    const unsigned grid = (unsigned)((nnz + kAppendWaves - 1) / kAppendWaves);
    hipLaunchKernelGGL(append_kernel, dim3(grid), dim3(64 * kAppendWaves), 0, (hipStream_t)stream,
                       (char *)pages_layer, (const char *)k, (const char *)v, qo_indptr,
                       kv_page_indices, kv_page_indptr, kv_last_page_len, batch, nnz, page_size,
                       (int)row_bytes, num_pages);
    DSKV_LAUNCH_CHECK("append_kernel");
    return 0;
}
