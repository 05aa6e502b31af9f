/*
 * dskv - C ABI of the MI355X (gfx950) KV-cache hot path for one DeServe stage.
 *
 * Every entry point is enqueue-only on the HIP stream it is given (passed as an
 * opaque pointer, i.e. a hipStream_t; NULL is the default stream), takes plain
 * device/host pointers and sizes, never frees caller memory and never throws.
 * Return value: 0 = ok, < 0 = argument error (DSKV_E_*), > 0 = a hipError_t.
 * The message of the last failure on the calling thread is dskv_last_error().
 *
 * Reference interfaces replaced (paths relative to the reference repository's
 * deserve_worker/ package) are cited on each declaration.
 */
#ifndef DSKV_H
#define DSKV_H

#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

#define DSKV_E_INVAL (-1)      /* bad argument / unsupported shape */
#define DSKV_E_NOMEM (-2)      /* caller buffer too small */
#define DSKV_E_STATE (-3)      /* handle used in the wrong state */

/* element types of K/V/Q storage */
#define DSKV_F32 0
#define DSKV_F16 1
#define DSKV_BF16 2

const char *dskv_last_error(void);
/*
 * DSKV_ABI_VERSION of the library that was loaded.  It changes whenever the signature of an
 * exported function changes (the arguments are plain words and pointers: a caller built
 * against another header would pass shifted arguments without any error), so a binding
 * compares it with the value of the header it was written against before its first call.
 */
#define DSKV_ABI_VERSION 3
int dskv_version(void);

/*
 * KV append.  Replaces the call site model/layer/attention.py:175-183
 * (flashinfer.append_paged_kv_cache(xk, xv, indptr, pages, kv_page_indices,
 * kv_page_indptr, kv_last_page_lens)).
 * pages_layer: (num_pages, 2, page_size, n_kv_heads, head_dim) of one layer.
 * k, v: (nnz, n_kv_heads, head_dim) contiguous.  All int32 arrays on device.
 * Token i of request b goes to position kv_len_b - n_b + i of that request.
 * Pure byte copy: elt_bytes is 2 or 4.  A token whose metadata is inconsistent or
 * whose page id lies outside [0, num_pages) is skipped: nothing outside the layer
 * is ever written.
 */
int dskv_append_paged_kv(void *pages_layer, int32_t num_pages, const void *k, const void *v,
                         const int32_t *qo_indptr, const int32_t *kv_page_indices,
                         const int32_t *kv_page_indptr, const int32_t *kv_last_page_len,
                         int32_t batch, int32_t nnz, int32_t page_size, int32_t n_kv_heads,
                         int32_t head_dim, int32_t elt_bytes, void *stream);

/*
 * Page gather / scatter across all layers.  Replace the advanced-index
 * gather of kvcache/manager.py:37-42 (and page_pool.py:78-79) and the indexed
 * assignment of kvcache/manager.py:63-73.
 * pool: base of (n_layers, num_pages, page_bytes) with layer_stride_bytes
 * between layers; chunk: contiguous (n_layers * n_pages, page_bytes), layer
 * major then page_ids order.  page_ids: device int32.  row_begin/row_end select
 * a sub-range of the n_layers*n_pages chunk rows (0, n_layers*n_pages = all);
 * chunk points at row row_begin.
 */
int dskv_gather_pages(void *chunk, const void *pool, const int32_t *page_ids, int32_t n_pages,
                      int32_t n_layers, int64_t layer_stride_bytes, int64_t page_bytes,
                      int64_t row_begin, int64_t row_end, void *stream);
int dskv_scatter_pages(void *pool, const void *chunk, const int32_t *page_ids, int32_t n_pages,
                       int32_t n_layers, int64_t layer_stride_bytes, int64_t page_bytes,
                       int64_t row_begin, int64_t row_end, void *stream);

/*
 * Upload of n_words 32-bit words of per-step metadata from pinned host memory
 * to the device by a kernel on `stream` (no copy engine involved).  Replaces
 * the host-to-device constructions torch.tensor(..., device=main_device) of
 * model/context/flash.py:46-64 and the plan upload inside flashinfer's
 * begin_forward (execution/exec.py:184-192).  src_pinned must be host memory
 * the device can read (hipHostMalloc / a pinned torch tensor) and must keep its
 * contents until the kernel has run; both pointers 16-byte aligned.
 */
int dskv_upload_words(void *dst, const void *src_pinned, int64_t n_words, void *stream);

/*
 * Paged decode attention.  Replaces BatchDecodeWithPagedKVCacheWrapper
 * begin_forward (execution/exec.py:184-192) = dskv_decode_plan, and
 * forward (model/layer/attention.py:185) = dskv_decode_attn.
 *
 * dskv_decode_plan runs on the host from host copies of the CSR metadata.  It
 * lays all requests' 16-token tiles end to end, cuts the sequence into one equal
 * share per workgroup and writes the resulting work list to plan_host (int32
 * words: 4 header words, n_workgroups + 1 share offsets, 2 per request, then 8
 * per item - the variable-length part last, so that the layout depends only on
 * the batch and the number of workgroups); the caller copies it to the device
 * once per step and reuses it for every layer.
 *   target_workgroups:   <= 0 = one per compute unit of the current device.
 *   plan_capacity_words: size of plan_host; dskv_decode_plan_bound(batch,
 *                        total_tokens) words always suffice.
 *   workspace_bytes_out: device scratch dskv_decode_attn needs for the partial
 *                        results of requests that were cut (16-byte aligned).
 */
int64_t dskv_decode_plan_bound(int32_t batch, int64_t total_tokens);
int dskv_decode_plan(const int32_t *kv_page_indptr_host, const int32_t *kv_last_page_len_host,
                     int32_t batch, int32_t page_size, int32_t n_qo_heads, int32_t n_kv_heads,
                     int32_t head_dim, int32_t target_workgroups, int32_t *plan_host,
                     int64_t plan_capacity_words, int32_t *n_items_out, int32_t *n_workgroups_out,
                     int64_t *plan_words_out, int64_t *workspace_bytes_out);

/*
 * out, q: (batch, n_qo_heads, head_dim) of dtype; pages_layer as for append.
 * out[b,h] = softmax_j(q[b,h].K_b[j,h/(Hq/Hkv)] * sm_scale) . V_b[j,h/(Hq/Hkv)]
 * over the kv_len_b tokens fixed at plan time.  fp32 accumulation.
 */
int dskv_decode_attn(void *out, const void *q, const void *pages_layer,
                     const int32_t *kv_page_indices, const int32_t *plan_dev, int32_t n_items,
                     int32_t n_workgroups, void *workspace, int64_t workspace_bytes, int32_t batch,
                     int32_t n_qo_heads, int32_t n_kv_heads, int32_t head_dim, int32_t page_size,
                     float sm_scale, int32_t dtype, void *stream);
/*
 * dskv_decode_attn for callers that cannot allocate device memory (code under HIP graph
 * capture, tight serving loops, harnesses that forbid hipMalloc).  No counterpart in the
 * reference.  Same arguments and result as dskv_decode_attn, bit for bit, minus the
 * workspace: the partial results of cut requests go to an array built into the library
 * (dskv_decode_attn_noalloc_max_bytes() bytes, 32 MiB, one copy per GPU for the life of the
 * process).  Calls no hipMalloc / hipFree.  A plan whose partials do not fit -
 * min(n_items, 2 * (n_items - batch)) * n_qo_heads * (head_dim + 2) * 4 bytes - is refused
 * with DSKV_E_NOMEM.  All calls on one GPU share the array: calls that overlap on one GPU
 * (two streams, two threads) race; calls on one stream do not.  The first call on a device
 * looks the array's address up (hipGetSymbolAddress); make that call outside a capture.
 */
int64_t dskv_decode_attn_noalloc_max_bytes(void);
int dskv_decode_attn_noalloc(void *out, const void *q, const void *pages_layer,
                             const int32_t *kv_page_indices, const int32_t *plan_dev,
                             int32_t n_items, int32_t n_workgroups, int32_t batch,
                             int32_t n_qo_heads, int32_t n_kv_heads, int32_t head_dim,
                             int32_t page_size, float sm_scale, int32_t dtype, void *stream);

/*
 * The same, one pass at a time: phases bit 0 = the split-KV attention pass
 * (writes final rows of uncut requests and the partials of cut ones), bit 1 =
 * the merge pass that combines the partials.  dskv_decode_attn is phases = 3.
 * Lets a caller time or overlap the two passes separately.
 */
int dskv_decode_attn_phases(void *out, const void *q, const void *pages_layer,
                            const int32_t *kv_page_indices, const int32_t *plan_dev,
                            int32_t n_items, int32_t n_workgroups, void *workspace,
                            int64_t workspace_bytes, int32_t batch, int32_t n_qo_heads,
                            int32_t n_kv_heads, int32_t head_dim, int32_t page_size, float sm_scale,
                            int32_t dtype, int32_t phases, void *stream);

/*
 * The decode step's append and attention in one launch (same plan, same result
 * as dskv_append_paged_kv of one token per request followed by
 * dskv_decode_attn; replaces the pair of calls of
 * model/layer/attention.py:174-187 in a decode step).  k_new, v_new:
 * (batch, n_kv_heads, head_dim), the step's token of every request; the plan's
 * kv lengths include it and its page slot exists.  The wave that reads a
 * request's newest row writes it first, so no other launch has to.  phases: 3,
 * or 1 to leave the merge pass to a later dskv_decode_attn_phases(.., 2, ..).  Only for
 * the shapes dskv_decode_append_attn_supported accepts (16-bit, head_dim 128,
 * group <= 16, power-of-two page); others return DSKV_E_INVAL.
 */
int dskv_decode_append_attn_supported(int32_t n_qo_heads, int32_t n_kv_heads, int32_t head_dim,
                                      int32_t page_size, int32_t dtype);
int dskv_decode_append_attn(void *out, const void *q, const void *k_new, const void *v_new,
                            void *pages_layer, const int32_t *kv_page_indices,
                            const int32_t *plan_dev, int32_t n_items, int32_t n_workgroups,
                            void *workspace, int64_t workspace_bytes, int32_t batch,
                            int32_t n_qo_heads, int32_t n_kv_heads, int32_t head_dim,
                            int32_t page_size, float sm_scale, int32_t dtype, int32_t phases,
                            void *stream);

/*
 * The same with the rotary embedding of the step inside the launch: q is
 * rotated as it is loaded and k_new before it is stored, with the adjacent-pair
 * convention and arithmetic of dskv_apply_rope, so a decode step of a layer is
 * this one launch (plus the merge pass) in place of
 * apply_rope + append_paged_kv_cache + forward (model/layer/attention.py:166-187).
 * rope_table: (batch, head_dim) floats, row b = cos | sin of
 * positions[b] * theta^(-2*pair/head_dim) for the head_dim/2 pairs, written by
 * dskv_rope_table from the device array of the new tokens' positions (the
 * reference's ctx.offsets); built once per step, shared by all layers.
 */
int dskv_rope_table(float *table, const int32_t *positions, int32_t batch, int32_t head_dim,
                    float rope_theta, void *stream);
int dskv_decode_rope_append_attn(void *out, const void *q, const void *k_new, const void *v_new,
                                 void *pages_layer, const int32_t *kv_page_indices,
                                 const int32_t *plan_dev, int32_t n_items, int32_t n_workgroups,
                                 void *workspace, int64_t workspace_bytes, int32_t batch,
                                 int32_t n_qo_heads, int32_t n_kv_heads, int32_t head_dim,
                                 int32_t page_size, float sm_scale, int32_t dtype,
                                 const float *rope_table, int32_t phases, void *stream);

/*
 * Paged prefill attention with the end-aligned causal mask.  Replaces
 * BatchPrefillWithPagedKVCacheWrapper.forward(q, pages, causal=True)
 * (model/layer/attention.py:188-192, execution/exec.py:227-236).
 * q, out: (nnz, n_qo_heads, head_dim); qo_indptr (batch+1) device int32.
 * Query i of the n_b queries of request b sees kv positions
 * j <= kv_len_b - n_b + i.
 *
 * dskv_prefill_plan (host; replaces the planning half of begin_forward,
 * execution/exec.py:227-236) cuts the requests' query rows into tiles, one
 * workgroup per tile and kv head, and writes the plan - at most
 * dskv_prefill_plan_bound(batch, nnz) words - that dskv_prefill_attn reads from
 * device memory (plan_dev: the first *plan_words_out words, uploaded by the caller;
 * unused, may be NULL, for fp32).
 * kv_len_host (batch host int32, may be NULL): the requests' kv lengths.  With
 * them the tiles are ordered longest first, which balances a launch over requests
 * of mixed lengths, and tiles are cut into parts (at most 8; every part walks a
 * slice of the tile's K/V as a workgroup of its own and leaves partials in the
 * workspace - *workspace_bytes_out bytes, 16-byte aligned - which dskv_prefill_attn
 * merges in a second pass): all tiles of a batch of few tiles (the 512-token chunks
 * of the reference's scheduler, engine/pipeline/scheduler.py:74,85: 64 workgroups
 * for an 8-kv-head model), so that the launch fills the chip, and any tile whose
 * walk over its keys is long against the launch's fair share per compute unit, so
 * that no single workgroup outlasts the rest.  *n_splits_out: the largest number
 * of parts of any tile (1: no partials, no merge pass).  target_workgroups:
 * workgroups the launch is sized for (0: one per compute unit; negative: never cut
 * a tile).  The result does not depend on the order of the tiles, and on the parts
 * only in the last bits.
 * n_tiles: *n_tiles_out (plan entries: tiles and their parts).
 */
int64_t dskv_prefill_plan_bound(int32_t batch, int64_t nnz);
int dskv_prefill_plan(const int32_t *qo_indptr_host, const int32_t *kv_len_host, int32_t batch,
                      int32_t n_qo_heads, int32_t n_kv_heads, int32_t head_dim,
                      int32_t target_workgroups, int32_t *plan_host, int64_t capacity_words,
                      int32_t *n_tiles_out, int32_t *n_splits_out, int64_t *plan_words_out,
                      int64_t *workspace_bytes_out);
int dskv_prefill_attn(void *out, const void *q, const int32_t *qo_indptr, const void *pages_layer,
                      const int32_t *kv_page_indices, const int32_t *kv_page_indptr,
                      const int32_t *kv_last_page_len, const int32_t *plan_dev, int32_t n_tiles,
                      int32_t n_splits, void *workspace, int64_t workspace_bytes, int32_t batch,
                      int32_t nnz, int32_t n_qo_heads, int32_t n_kv_heads, int32_t head_dim,
                      int32_t page_size, float sm_scale, int32_t causal, int32_t dtype,
                      void *stream);

/*
 * Mixed batches.  The reference sends the WHOLE batch through its prefill wrapper as soon as
 * one task of the step has more than one new token (engine/microbatch/processor.py:116-145),
 * and its decode-first join stage (engine/pipeline/stage/join.py:11-88, 512-token budget)
 * makes that the usual step: dozens of decode rows plus one chunk (benchmark/mixed.py:19-88
 * times exactly this).  dskv_mixed_plan / dskv_mixed_attn are dskv_prefill_plan /
 * dskv_prefill_attn for such batches: a request with ONE query row sees every kv token of
 * its request with or without the causal mask, so it is a decode row - it is planned as
 * split-KV decode items (dskv_decode_plan's work list, its K/V read once at the speed of
 * memory) while the other requests are planned as query tiles; dskv_mixed_attn launches the
 * decode pass over the one-row requests and the tile pass over the rest, and both write
 * their rows of the same ragged `out`.  Routing needs a shape the 16-bit decode kernel
 * takes (head_dim 128, group <= 16, power-of-two page) and route_one_row_requests != 0;
 * otherwise, and for a batch without one-row requests, plan and result are those of
 * dskv_prefill_plan / dskv_prefill_attn.  fp32 data is computed by the generic kernel,
 * whatever the plan routed.
 * With DSKV_ROUTE_AUTO a batch of one-row requests only runs the decode pass alone; a batch
 * of both kinds runs as ONE launch (DSKV_LAYOUT_SHARED: pages of at least 4 tokens, at least
 * 12 one-row requests, which as query tiles of their own would be at least half of the launch's
 * work) in which every compute unit hosts a decode workgroup, which keeps its memory path
 * busy, and tile workgroups beside it, which use its matrix pipeline, followed by one merge
 * pass for both kinds of rows - or, where that launch does not apply or does not pay (a handful
 * of decode rows, a large prefill batch), as tiles only.  The two other modes force a layout
 * (for measurements and tests).
 * The plan (at most dskv_mixed_plan_bound words; upload the first info->plan_words) holds
 * the tile plan (entries, then the rows' parts if a tile is cut), then at word
 * decode_plan_at the decode work list and at row_map_at the query row of every routed request;
 * a DSKV_LAYOUT_SHARED plan ends with the parts of every row of the batch (first slot, parts;
 * the tile parts' slots numbered first), so that ONE merge pass finishes both kinds of rows.
 * workspace: tile_workspace_bytes (partials of tile parts) + decode_workspace_bytes
 * (partials of cut decode rows), 16-byte aligned.
 */
/* route_one_row_requests */
#define DSKV_ROUTE_OFF 0            /* every request as query tiles (the plan of dskv_prefill_plan) */
#define DSKV_ROUTE_AUTO 1           /* the planner chooses (see dskv_mixed_plan) */
#define DSKV_ROUTE_TWO_LAUNCHES 2   /* decode pass, then tile pass */
#define DSKV_ROUTE_SHARED_LAUNCH 3  /* one launch whose decode and tile workgroups share the compute units */
/* dskv_mixed_plan_t.layout */
#define DSKV_LAYOUT_SEPARATE 0      /* tile pass and / or decode pass, workgroups of eight waves */
#define DSKV_LAYOUT_SHARED 1        /* one launch of four-wave workgroups: a decode workgroup on every
                                       compute unit, the tile workgroups beside them */
typedef struct dskv_mixed_plan {
    int32_t n_tiles, n_splits;        /* tile entries (tiles and their parts), most parts of a tile */
    int32_t n_tile_rows;              /* query rows computed by the tile pass */
    int32_t n_decode_rows;            /* one-row requests computed by the decode pass */
    int32_t n_decode_items, n_decode_workgroups;
    int32_t layout, reserved;
    int64_t plan_words;
    int64_t decode_plan_at, row_map_at;
    int64_t tile_workspace_bytes, decode_workspace_bytes;
} dskv_mixed_plan_t;
int64_t dskv_mixed_plan_bound(int32_t batch, int64_t nnz, int64_t total_kv_tokens);
int dskv_mixed_plan(const int32_t *qo_indptr_host, const int32_t *kv_page_indptr_host,
                    const int32_t *kv_last_page_len_host, int32_t batch, int32_t page_size,
                    int32_t n_qo_heads, int32_t n_kv_heads, int32_t head_dim,
                    int32_t target_workgroups, int32_t route_one_row_requests,
                    int32_t *plan_host, int64_t capacity_words, dskv_mixed_plan_t *info);
int dskv_mixed_attn(void *out, const void *q, const int32_t *qo_indptr, const void *pages_layer,
                    const int32_t *kv_page_indices, const int32_t *kv_page_indptr,
                    const int32_t *kv_last_page_len, const int32_t *plan_dev,
                    const dskv_mixed_plan_t *info, void *workspace, int64_t workspace_bytes,
                    int32_t batch, int32_t nnz, int32_t n_qo_heads, int32_t n_kv_heads,
                    int32_t head_dim, int32_t page_size, float sm_scale, int32_t causal,
                    int32_t dtype, void *stream);

/*
 * Rotary embedding, adjacent-pair convention.  Replaces the call site
 * model/layer/attention.py:166-173 (flashinfer.apply_rope(q, k, indptr,
 * offsets, interleave=True, rope_theta=5e5)); maths as in
 * model/layer/attention.py:45-72 with the table of execution/exec.py:25-55.
 * Out of place: q_out/k_out may alias q/k.
 */
int dskv_apply_rope(void *q_out, void *k_out, const void *q, const void *k,
                    const int32_t *qo_indptr, const int32_t *offsets, int32_t batch, int32_t nnz,
                    int32_t n_qo_heads, int32_t n_kv_heads, int32_t head_dim, float rope_theta,
                    int32_t dtype, void *stream);

/*
 * RoPE and KV append in one pass: the two call sites above back to back
 * (model/layer/attention.py:166-183).  q is rotated into q_out; k is rotated and
 * written straight into its page slot, v is copied next to it - the rotated K
 * never makes a round trip through a temporary.  Bit-identical to
 * dskv_apply_rope followed by dskv_append_paged_kv.
 */
int dskv_rope_append_paged_kv(void *q_out, void *pages_layer, int32_t num_pages, const void *q,
                              const void *k, const void *v, const int32_t *qo_indptr, const int32_t *offsets,
                              const int32_t *kv_page_indices, const int32_t *kv_page_indptr,
                              const int32_t *kv_last_page_len, int32_t batch, int32_t nnz,
                              int32_t page_size, int32_t n_qo_heads, int32_t n_kv_heads,
                              int32_t head_dim, float rope_theta, int32_t dtype, void *stream);

/*
 * Bulk swap of one contiguous page slice of every layer.  Replaces
 * swap.swap(d, h0, h1, s0, s1, interval) (kvcache/swap.cpp:9-57, called from
 * kvcache/virtual.py:88-95) with the semantics stated by
 * VirtualPagePool.swap (kvcache/virtual.py:97-113): for every layer, first
 * copy slice -> host_to + layer*slice_bytes, then host_from + layer*slice_bytes
 * -> slice.  Layers [0, L/2) go on stream0, the rest on stream1.  Either host
 * pointer may be NULL to skip that direction.  Host memory must be pinned.
 */
int dskv_swap_slice(void *slice_base, int64_t layer_stride_bytes, int64_t slice_bytes,
                    int32_t n_layers, void *host_to, const void *host_from, void *stream0,
                    void *stream1);

/*
 * Scattered-page swap engine (gather-to-staging + one large async copy per
 * staging chunk, on the engine's own side streams).  Replaces the blocking
 * per-task copies KVCacheManager.copy_gpu_to_cpu / copy_cpu_to_gpu
 * (kvcache/manager.py:24-86); host layout (n_layers*n_pages, page_bytes), layer
 * major then page_ids order.  page_ids is a HOST int32 array (copied at call
 * time, into a ring of 2^20 ids that in-flight calls hold until they have run: a call that
 * finds the ring full is refused with DSKV_E_STATE - nothing in these calls waits); ids
 * outside a layer are refused with DSKV_E_INVAL.  after_stream: work already enqueued
 * there is waited for (on the device) before the pool is touched.  dskv_swap_wait blocks
 * the host until everything enqueued on the handle is done; dskv_swap_fence makes `stream`
 * wait for it instead.
 */
typedef struct dskv_swap dskv_swap_t;
int dskv_swap_create(dskv_swap_t **handle, int64_t staging_bytes);
int dskv_swap_destroy(dskv_swap_t *handle);
int dskv_swap_out_async(dskv_swap_t *handle, void *host_dst, const void *pool,
                        const int32_t *page_ids_host, int32_t n_pages, int32_t n_layers,
                        int64_t layer_stride_bytes, int64_t page_bytes, void *after_stream);
int dskv_swap_in_async(dskv_swap_t *handle, void *pool, const void *host_src,
                       const int32_t *page_ids_host, int32_t n_pages, int32_t n_layers,
                       int64_t layer_stride_bytes, int64_t page_bytes, void *after_stream);
/*
 * Scattered-page counterpart of the microbatch exchange swap.swap performs on a
 * slice (kvcache/swap.cpp:36-56): the named pages go out to host_dst and are then
 * refilled from host_src (same layout), chunk by chunk, with the D2H and H2D
 * traffic on separate streams so both directions of the link are busy.  A chunk
 * is only overwritten after it has been packed for the trip out.
 * host_dst == host_src leaves the pages unchanged (only the dump is done).
 */
int dskv_swap_exchange_async(dskv_swap_t *handle, void *host_dst, const void *host_src, void *pool,
                             const int32_t *page_ids_host, int32_t n_pages, int32_t n_layers,
                             int64_t layer_stride_bytes, int64_t page_bytes, void *after_stream);
int dskv_swap_wait(dskv_swap_t *handle);
int dskv_swap_fence(dskv_swap_t *handle, void *stream);
/* Non-blocking: *done_out = 1 if everything enqueued on the handle has finished, else 0. */
int dskv_swap_query(dskv_swap_t *handle, int32_t *done_out);
/*
 * The two side streams of the engine (hipStream_t): [out] device-to-host, [in]
 * host-to-device.  Lets the bulk slice swap (dskv_swap_slice, the two streams of
 * kvcache/virtual.py:48-49) run on the engine's streams, so that a process holds three
 * streams - compute and these two - and not five.  The handles stay valid until
 * dskv_swap_destroy (after this call dskv_swap_bind_compute_stream no longer replaces them).
 */
int dskv_swap_streams(dskv_swap_t *handle, void **out_stream, void **in_stream);
/*
 * Set-up call (blocks; drains the engine and both streams): makes sure the engine's two
 * streams run beside `compute_stream` and beside each other.  The HIP runtime maps
 * streams onto a few hardware queues whose packets run in order, and which streams
 * share a queue depends on how many streams the process created before - a swap whose
 * stream shares the compute stream's queue does not overlap with compute at all.  The
 * call measures it (an idling kernel on one stream, an empty one on the other) and
 * replaces a stream that serialises by a fresh one, up to eight times.
 * independent_out (may be NULL): 1 if both streams now run beside the compute stream
 * and each other, 0 if no such pair was found (the engine still works, without overlap).
 * No counterpart in the reference, whose two torch streams (kvcache/virtual.py:48-49)
 * are subject to the same sharing.
 * Replacing a stream destroys it: handles obtained from dskv_swap_streams would dangle, so
 * once that call has handed the streams out, binding is refused with DSKV_E_STATE.  Bind
 * first (right after dskv_swap_create), then ask for the streams.
 */
int dskv_swap_bind_compute_stream(dskv_swap_t *handle, void *compute_stream,
                                  int32_t *independent_out);

#ifdef __cplusplus
}
#endif
#endif /* DSKV_H */
