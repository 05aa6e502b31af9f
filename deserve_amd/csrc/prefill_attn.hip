// Paged prefill (multi-query) attention with the end-aligned causal mask:
// query i of the n_b new tokens of request b sees kv positions j <= kv_len_b - n_b + i.
//
// Bound: MFMA for long chunks.  Work decomposition: one workgroup = one kv head x
// one tile of query rows; each of its waves owns 32 columns (kColTiles tiles of
// 32), a column being a (query position, q head of the GQA group) pair, so the
// MFMA N dimension is dense.  The workgroup walks the request's K/V in blocks of
// 32 tokens that its waves load together (each four rows) into LDS stages, so a
// K/V byte crosses the vector memory path once per workgroup instead of once per
// wave: with every wave streaming K/V on its own the kernel was bound by that
// path at a sixth of the MFMA rate.  The rows go from global memory straight into
// LDS (`buffer_load_dwordx4 ... lds`, three blocks ahead of their use), without a
// trip through vector registers; pages shorter than four tokens take the register
// path (load, then ds_write) instead.  The loads are inline assembly with hand-set
// `s_waitcnt vmcnt` and a bare `s_barrier`: through the compiler's builtin every
// barrier and LDS read waited for all loads in flight, which undid the prefetch.
//
// All products use the 32x32x16 MFMA (measured on MI355X at 2.2 PFLOP/s bf16,
// against 1.3 PFLOP/s for 16x16x32).  Per block a wave computes S^T = K.Q^T
// (tokens x columns, K rows from LDS as the A operand), keeps S^T's C layout as
// the B operand P^T, and reads V through the transposing LDS read as the A
// operand of O^T += V^T.P^T.
//
// Workgroup ids are laid out head-fastest: consecutive ids go to different XCDs,
// so (with 8 kv heads) all query tiles of one kv head share one XCD's L2.
//
// A batch of few tiles (one 512-token chunk: 8 tiles x 8 kv heads) would leave most
// of the chip idle.  The plan then cuts every tile's K/V range into parts; a part is
// a workgroup of its own that leaves (maximum, sum, unnormalised O) of its rows in a
// workspace, and a merge pass (one workgroup per query row) turns the parts into the output.
#include "kv_tile.h"
#include "decode_kernel.h"

#include <vector>

#include <algorithm>

#include "prefill_kernel.h"

namespace dskv {

// Generic path (fp32 pools, head_dim != 128, group > 16): one wavefront per
// (query row, q head), plain VALU, sequential over the visible tokens.
template <int DT>
__global__ __launch_bounds__(64) void prefill_attn_generic_kernel(
    void *__restrict__ out, const void *__restrict__ q, const int32_t *__restrict__ qo_indptr,
    const void *__restrict__ pages, const int32_t *__restrict__ kv_indices,
    const int32_t *__restrict__ kv_indptr, const int32_t *__restrict__ kv_last, int batch,
    int n_qo_heads, int n_kv_heads, int head_dim, int page_size, float scale_log2, int causal)
{
    typedef LoadElt<DT> L;
    const int lane = threadIdx.x;
    const int row = blockIdx.x;
    const int qh = blockIdx.y;
    const int kvh = qh / (n_qo_heads / n_kv_heads);
    int lo = 0, hi = batch;   // largest b with qo_indptr[b] <= row
    while (hi - lo > 1) {
        const int mid = (lo + hi) >> 1;
        if (qo_indptr[mid] <= row) lo = mid; else hi = mid;
    }
    const int b = lo;
    if (row >= qo_indptr[b + 1]) return;
    const int n_b = qo_indptr[b + 1] - qo_indptr[b];
    const int page_begin = kv_indptr[b];
    const int n_pages = kv_indptr[b + 1] - page_begin;
    const int kv_len = n_pages > 0 ? (n_pages - 1) * page_size + kv_last[b] : 0;
    int limit = causal ? kv_len - n_b + (row - qo_indptr[b]) + 1 : kv_len;
    limit = min(max(limit, 0), kv_len);
    const long tok_row = (long)n_kv_heads * head_dim;
    const long half = tok_row * page_size;

    float qv[4], acc[4];
#pragma unroll
    for (int i = 0; i < 4; i++) {
        const int d = lane + 64 * i;
        qv[i] = d < head_dim ? L::get(q, ((long)row * n_qo_heads + qh) * head_dim + d) : 0.f;
        acc[i] = 0.f;
    }
    float m_run = kNegBig, l_run = 0.f;
    // kGroup tokens at a time: page ids, K rows and V rows of the group are all requested
    // before the first is used (token by token, every token waited for memory twice)
    constexpr int kGroup = 8;
    for (int t0 = 0; t0 < limit; t0 += kGroup) {
        long base[kGroup];
#pragma unroll
        for (int j = 0; j < kGroup; j++) {
            const int t = min(t0 + j, limit - 1);   // past the limit: the last token again, weight zero
            const long page = kv_indices[page_begin + t / page_size];
            base[j] = page * 2 * half + (long)(t % page_size) * tok_row + (long)kvh * head_dim;
        }
        float kx[kGroup][4], vx[kGroup][4];
#pragma unroll
        for (int j = 0; j < kGroup; j++)
#pragma unroll
            for (int i = 0; i < 4; i++) {
                const int d = lane + 64 * i;
                kx[j][i] = d < head_dim ? L::get(pages, base[j] + d) : 0.f;
            }
#pragma unroll
        for (int j = 0; j < kGroup; j++)
#pragma unroll
            for (int i = 0; i < 4; i++) {
                const int d = lane + 64 * i;
                vx[j][i] = d < head_dim ? L::get(pages, base[j] + half + d) : 0.f;
            }
        float x[kGroup], m_new = m_run;
#pragma unroll
        for (int j = 0; j < kGroup; j++) {
            float dot = 0.f;
#pragma unroll
            for (int i = 0; i < 4; i++) dot += qv[i] * kx[j][i];
            x[j] = t0 + j < limit ? wave_sum(dot) * scale_log2 : kNegBig;
            m_new = fmaxf(m_new, x[j]);
        }
        const float alpha = __builtin_amdgcn_exp2f(m_run - m_new);
        l_run *= alpha;
#pragma unroll
        for (int i = 0; i < 4; i++) acc[i] *= alpha;
#pragma unroll
        for (int j = 0; j < kGroup; j++) {
            const float p = x[j] > kNegBig ? __builtin_amdgcn_exp2f(x[j] - m_new) : 0.f;
            l_run += p;
#pragma unroll
            for (int i = 0; i < 4; i++) acc[i] += p * vx[j][i];
        }
        m_run = m_new;
    }
    const float inv = l_run > 0.f ? 1.f / l_run : 0.f;
#pragma unroll
    for (int i = 0; i < 4; i++) {
        const int d = lane + 64 * i;
        if (d < head_dim) L::put(out, ((long)row * n_qo_heads + qh) * head_dim + d, acc[i] * inv);
    }
}

static int prefill_rows_per_tile(int n_qo_heads, int n_kv_heads, int waves)
{
    const int group = n_qo_heads / n_kv_heads;
    return group <= kWaveCols ? waves * (kWaveCols / group) : 1;
}

// ---------------------------------------------------------------------------
// The mixed launch: decode workgroups and query tiles side by side on every CU.
//
// A compute unit moves at most ~36 GB/s through its vector memory path (measured: one
// decode workgroup of eight, four or two waves per CU streams 37, 35 and 31 GB/s, whatever
// else is free), so the chip's 8 TB/s are only there when EVERY CU has loads in flight -
// and a CU that computes a chunk's query tiles (bound by its matrix pipeline) contributes
// none.  Run one after the other, the decode rows and the chunk of a mixed step (75 rows over
// U[256,4096] tokens + 437 tokens over 2506) take 118 + 47 us; as tiles of one launch, with
// one live row per 64-row tile and the longest rows walked by a single workgroup, 147 us
// (228 us when the chunk follows 8000 tokens).  Here both kinds of work are workgroups of
// FOUR waves (one per SIMD, at most 256 vector registers, half a CU's LDS each), so two fit
// on a CU, and the launch starts with one decode workgroup per CU: the dispatcher places the
// first #CU workgroups of a grid one per CU (measured on the box), so the decode workgroups -
// statically balanced shares that must all start at once - own one slot of every CU for the
// whole launch, while the query tiles pass through the other slot.  Measured: 150 us (175 us
// behind 8000 tokens): the tile workgroups finish within 66 us, the decode workgroups, which
// share the CU's memory path with them meanwhile, after 145 us instead of 113 us alone.
// ---------------------------------------------------------------------------
// Tiles in flight per decode wave of the mixed launch (2, 4 and 5 measured the same).
constexpr int kSharedRing = kStages;
// Wave priority of the tile workgroups.  At equal priority the compute unit serves the older
// waves first, and the decode waves - launched first, never short of a load to issue - kept
// the tile waves' few loads waiting: a tile workgroup took 162 us beside them instead of 38 us
// alone.  With the tile waves ahead (any priority above 0) it takes 66 us.
constexpr int kSharedTilePriority = 3;
struct MixedArgs {
    uint16_t *out;
    const uint16_t *q;
    const char *pages;
    const int32_t *kv_indices;
    int n_qo_heads, n_kv_heads, page_shift;
    float scale_log2;
    // decode side: shares x head groups workgroups come first in the grid
    const Item *items;
    const int32_t *wg_ptr;
    float *dec_part_o, *dec_part_ml;
    int dec_max_slots, n_decode_wgs, head_groups;
    // tile side
    const int32_t *qo_indptr, *kv_indptr, *kv_last, *tile_info;
    float *tile_part_o, *tile_part_ml;
    int tile_max_slots, causal;
};

template <int DT, int kPagesPerTile>
__global__ __launch_bounds__(64 * kSharedWaves, 2) void mixed_attn_kernel(const MixedArgs a)
{
    static_assert(kSharedWaves == kPrefillWavesShared, "both kinds of workgroup have the launch's size");
    static_assert(kPrefillLdsBytes >= kSharedWaves * kVTileBytes, "the LDS is shared by the two bodies");
    __shared__ __align__(16) char lds[kPrefillLdsBytes];
    const int wg = blockIdx.x;
    if (wg < a.n_decode_wgs)
        decode_attn_body<DT, kPagesPerTile, kSharedWaves, kSharedRing>(
            lds, wg / a.head_groups, wg % a.head_groups, a.out, a.q, a.pages, a.kv_indices, a.items, a.wg_ptr,
            a.dec_part_o, a.dec_part_ml, a.dec_max_slots, a.n_qo_heads, a.n_kv_heads, a.page_shift,
            a.scale_log2, nullptr, nullptr, nullptr);
    else {
        __builtin_amdgcn_s_setprio(kSharedTilePriority);
        prefill_attn_body<DT, true, kPrefillWavesShared>(
            lds, wg - a.n_decode_wgs, a.out, a.q, a.qo_indptr, a.pages, a.kv_indices, a.kv_indptr, a.kv_last,
            a.tile_info, a.n_qo_heads, a.n_kv_heads, a.page_shift, a.scale_log2, a.causal,
            a.tile_part_o, a.tile_part_ml, a.tile_max_slots);
    }
}

}  // namespace dskv

namespace dskv {

constexpr int kMaxPrefillSplits = 8;         // parts a tile's K/V range is cut into at most
// a part holds at least this many tokens: with 256, a 512-token chunk without prior context
// took 37 us in two parts instead of 29 us whole; with 1024, chunks over 1-2 k tokens of prior
// context lost a fifth of what the parts buy
constexpr int kMinSplitTokens = 512;
constexpr int kMaxSplitTarget = 1024;        // workgroups a split plan aims at, at most
// a workgroup's start and end, in 32-token blocks of walking (for the fair share of a launch)
constexpr int kTileOverheadBlocks = 4;
constexpr int32_t kWholeRange = 0x7fffffff;  // blk_end of a tile that is not split
// One-row requests of a mixed batch get decode workgroups of their own beside the tiles when
// there are at least this many of them ...
constexpr int kMinSharedLaunchRows = 12;
// ... and when, run as tiles (one live row per tile), they would be most of the launch's work:
// a tile is priced at its 32-token blocks plus this much for its start and end.
constexpr int kTileFixedCostBlocks = 16;

static int compute_units()
{
    int dev = 0, cus = 0;
    if (hipGetDevice(&dev) != hipSuccess ||
        hipDeviceGetAttribute(&cus, hipDeviceAttributeMultiprocessorCount, dev) != hipSuccess || cus <= 0)
        cus = 256;
    (void)hipGetLastError();
    return cus;
}

}  // namespace dskv

extern "C" int64_t dskv_prefill_plan_bound(int32_t batch, int64_t nnz)
{
    using namespace dskv;
    if (batch < 0 || nnz < 0) return 0;
    // entries: one per tile (at most batch + nnz of them), times the parts of those that are
    // cut: filling the chip adds at most 2 * kMaxSplitTarget entries, cutting long walks down
    // to the fair share at most 2 * kMaxSplitTarget more; then two words per query row
    return kTileWords * ((int64_t)batch + nnz + 4 * kMaxSplitTarget + kMaxPrefillSplits) + 2 * nnz;
}

namespace dskv {

// The tile planner.  skip (may be null): requests marked there get no tiles (their single
// row is computed by the decode kernel).  Plan: the tile entries (kTileWords each), then, if
// any tile is cut into parts, two words per query row of the batch (first partial slot,
// number of parts; 0 parts = the row needs no merge).
static int plan_tiles(const int32_t *qo_indptr_host, const int32_t *kv_len_host, const char *skip,
                      int32_t batch, int32_t n_qo_heads, int32_t n_kv_heads, int32_t head_dim,
                      int32_t target_workgroups, int32_t *plan_host, int64_t capacity_words,
                      int32_t *n_tiles_out, int32_t *n_splits_out, int64_t *plan_words_out,
                      int64_t *workspace_bytes_out, int waves = kPrefillWaves, bool cut_long_walks = true)
{
    const int rows = prefill_rows_per_tile(n_qo_heads, n_kv_heads, waves);
    // later query tiles of a request see more keys: they come first within a request
    struct Tile { int32_t b, row, n_rows, parts; int64_t keys, first_slot; };
    std::vector<Tile> tiles;
    int64_t nnz = 0;
    for (int b = 0; b < batch; b++) {
        const int64_t n_b = (int64_t)qo_indptr_host[b + 1] - qo_indptr_host[b];
        DSKV_REQUIRE(n_b >= 0, "prefill_plan: qo_indptr not monotone at %d", b);
        nnz += n_b;
        if (skip && skip[b]) continue;
        for (int64_t i = (n_b + rows - 1) / rows - 1; i >= 0; i--) {
            const int64_t last_row = std::min<int64_t>(i * rows + rows, n_b) - 1;
            const int64_t keys = kv_len_host ? std::max<int64_t>((int64_t)kv_len_host[b] - n_b + last_row + 1, 0) : 0;
            tiles.push_back({b, (int32_t)(i * rows), (int32_t)(last_row + 1 - i * rows), 1, keys, 0});
        }
    }
    DSKV_REQUIRE(tiles.size() < (size_t(1) << 26) && nnz < (int64_t(1) << 31), "prefill_plan: too many tiles");
    // Workgroups are dispatched in plan order and a tile's time grows with the keys its
    // last row sees: longest first, so the short ones fill the end of the launch
    // (request order left a fifth of the wave slots idle on mixed lengths).
    if (kv_len_host && tiles.size() > 1)
        std::stable_sort(tiles.begin(), tiles.end(),
                         [](const Tile &x, const Tile &y) { return x.keys > y.keys; });
    // Parts.  A tile's K/V range can be cut into parts that run as workgroups of their own and
    // leave partials, merged by a second pass - the decode path's way of keeping all compute
    // units busy.  Needs the kv lengths and the 16-bit kernel's head dim.  Two reasons to cut:
    //  * few tiles (a chunk of a few hundred tokens, as the reference's scheduler hands out:
    //    one 512-token chunk of an 8-kv-head model is 64 workgroups) leave most of the chip
    //    idle: every tile is cut into as many parts as fill it;
    //  * a tile whose walk is longer than the launch's fair share per compute unit ends the
    //    launch by itself (a chunk behind 8000 tokens in a step of decode rows: 232 us, with
    //    its tiles cut in two 197 us): it is cut down to that share.  Cutting further does
    //    not pay: with walks of at most half (a quarter of) the share a mixed step of 75
    //    decode rows and a chunk takes 159 (178) us instead of 149 us - the partials cost more
    //    than the shorter tail buys.  For the same reason only outliers are cut: when the
    //    tiles above the share hold more than a quarter of the launch's blocks (one long
    //    prompt of many tiles, the later ones longer), the launch is made of them, every cut
    //    tile would pay for partials, and the longest-first order is left to do its work.
    int max_parts = 1;
    if (kv_len_host && head_dim == kHeadDim && target_workgroups >= 0 && !tiles.empty()) {
        const int64_t target =
            target_workgroups > 0 ? std::min<int64_t>(target_workgroups, kMaxSplitTarget) : compute_units();
        const int64_t wgs = (int64_t)tiles.size() * n_kv_heads;
        int fill = 1;
        if (wgs * 2 <= target) fill = (int)std::min<int64_t>(kMaxPrefillSplits, target / wgs);
        int64_t total_blocks = 0;
        for (const Tile &t : tiles) total_blocks += (t.keys + kBlock - 1) / kBlock + kTileOverheadBlocks;
        // blocks one compute unit walks if the launch is shared out evenly, and the longest
        // walk a single workgroup may then have
        const int64_t share = (total_blocks * n_kv_heads + target - 1) / target;
        const int64_t cap = std::max<int64_t>(kMinSplitTokens / kBlock, share);
        int64_t above = 0;
        for (const Tile &t : tiles)
            if ((t.keys + kBlock - 1) / kBlock > cap) above += (t.keys + kBlock - 1) / kBlock;
        if (above * 4 > total_blocks) cut_long_walks = false;
        for (Tile &t : tiles) {
            const int64_t blocks = (t.keys + kBlock - 1) / kBlock;
            int64_t parts = std::max<int64_t>(fill, cut_long_walks ? (blocks + cap - 1) / cap : 1);
            parts = std::min<int64_t>(parts, kMaxPrefillSplits);
            parts = std::min<int64_t>(parts, std::max<int64_t>(1, t.keys / kMinSplitTokens));
            t.parts = (int32_t)parts;
            max_parts = std::max(max_parts, t.parts);
        }
    }
    int64_t n_entries = 0, n_slots = 0;
    for (Tile &t : tiles) {
        n_entries += t.parts;
        if (t.parts > 1) {
            t.first_slot = n_slots;
            n_slots += (int64_t)t.n_rows * t.parts;
        }
    }
    DSKV_REQUIRE(n_slots < (int64_t(1) << 31), "prefill_plan: too many partial slots");
    const int64_t words = n_entries * kTileWords + (max_parts > 1 ? 2 * nnz : 0);
    if (words > capacity_words) {
        set_error("prefill_plan: plan needs %lld words, buffer has %lld", (long long)words,
                  (long long)capacity_words);
        return DSKV_E_NOMEM;
    }
    int32_t *p = plan_host;
    int32_t *row_parts = plan_host + n_entries * kTileWords;
    if (max_parts > 1) std::fill(row_parts, row_parts + 2 * nnz, 0);
    for (const Tile &t : tiles) {
        // Parts of equal length, in units of four 32-token blocks (the kernel's loop is
        // unrolled by four), measured on the keys the tile sees under the causal mask; the
        // last part is open-ended.  The parts are disjoint and cover all blocks, so they are
        // also right without the mask (the last part then holds the rest of the request); a
        // part that starts past what the tile sees is empty.
        const int64_t blocks = (t.keys + kBlock - 1) / kBlock;
        const int64_t chunk = ((blocks + t.parts - 1) / t.parts + 3) / 4 * 4;
        for (int s = 0; s < t.parts; s++) {
            *p++ = t.b;
            *p++ = t.row;
            *p++ = (int32_t)(s * chunk);
            *p++ = s + 1 < t.parts ? (int32_t)((s + 1) * chunk) : kWholeRange;
            *p++ = t.parts > 1 ? (s | (t.parts << 8)) : -1;
            *p++ = (int32_t)t.first_slot;
        }
        if (t.parts > 1)
            for (int r = 0; r < t.n_rows; r++) {
                const int64_t row = (int64_t)qo_indptr_host[t.b] + t.row + r;
                row_parts[2 * row] = (int32_t)(t.first_slot + (int64_t)r * t.parts);
                row_parts[2 * row + 1] = t.parts;
            }
    }
    *n_tiles_out = (int32_t)n_entries;
    *n_splits_out = max_parts;
    *plan_words_out = words;
    *workspace_bytes_out = n_slots * (int64_t)n_qo_heads * (head_dim + 2) * (int64_t)sizeof(float);
    return 0;
}

}  // namespace dskv

extern "C" int dskv_prefill_plan(const int32_t *qo_indptr_host, const int32_t *kv_len_host,
                                 int32_t batch, int32_t n_qo_heads, int32_t n_kv_heads,
                                 int32_t head_dim, int32_t target_workgroups, int32_t *plan_host,
                                 int64_t capacity_words, int32_t *n_tiles_out,
                                 int32_t *n_splits_out, int64_t *plan_words_out,
                                 int64_t *workspace_bytes_out)
{
    using namespace dskv;
    DSKV_REQUIRE(batch >= 0 && n_tiles_out && n_splits_out && plan_words_out && workspace_bytes_out,
                 "prefill_plan: bad arguments");
    DSKV_REQUIRE(n_qo_heads > 0 && n_kv_heads > 0 && n_qo_heads % n_kv_heads == 0,
                 "prefill_plan: n_qo_heads %d not a multiple of n_kv_heads %d", n_qo_heads,
                 n_kv_heads);
    *n_tiles_out = 0;
    *n_splits_out = 1;
    *plan_words_out = 0;
    *workspace_bytes_out = 0;
    if (batch == 0) return 0;
    DSKV_REQUIRE(qo_indptr_host && plan_host, "prefill_plan: null pointer argument");
    return plan_tiles(qo_indptr_host, kv_len_host, nullptr, batch, n_qo_heads, n_kv_heads, head_dim,
                      target_workgroups, plan_host, capacity_words, n_tiles_out, n_splits_out,
                      plan_words_out, workspace_bytes_out);
}

// ---------------------------------------------------------------------------
// Mixed batches: one-row requests to the decode kernel, the others to query tiles
// ---------------------------------------------------------------------------
extern "C" int64_t dskv_mixed_plan_bound(int32_t batch, int64_t nnz, int64_t total_kv_tokens)
{
    if (batch < 0 || nnz < 0 || total_kv_tokens < 0) return 0;
    // tile entries, padding, the decode plan, the row map, the list of tiled rows and the
    // table of parts per row of a shared launch
    return dskv_prefill_plan_bound(batch, nnz) + 4 + dskv_decode_plan_bound(batch, total_kv_tokens) +
           (int64_t)batch + 3 * nnz + 8;
}

extern "C" int dskv_mixed_plan(const int32_t *qo_indptr_host, const int32_t *kv_page_indptr_host,
                               const int32_t *kv_last_page_len_host, int32_t batch,
                               int32_t page_size, int32_t n_qo_heads, int32_t n_kv_heads,
                               int32_t head_dim, int32_t target_workgroups,
                               int32_t route_one_row_requests, int32_t *plan_host,
                               int64_t capacity_words, dskv_mixed_plan_t *info)
{
    using namespace dskv;
    DSKV_REQUIRE(info, "mixed_plan: null info pointer");
    *info = dskv_mixed_plan_t{};
    info->n_splits = 1;
    DSKV_REQUIRE(batch >= 0, "mixed_plan: negative batch");
    DSKV_REQUIRE(page_size > 0 && n_qo_heads > 0 && n_kv_heads > 0 && head_dim > 0 &&
                     n_qo_heads % n_kv_heads == 0,
                 "mixed_plan: bad shape (page %d, heads %d/%d, dim %d)", page_size, n_qo_heads,
                 n_kv_heads, head_dim);
    if (batch == 0) return 0;
    DSKV_REQUIRE(qo_indptr_host && kv_page_indptr_host && kv_last_page_len_host && plan_host,
                 "mixed_plan: null pointer argument");
    // One query row under the end-aligned mask sees every kv token of its request, with or
    // without the mask: exactly a decode row.  Routed only where the 16-bit decode kernel
    // takes the shape; a request without kv tokens stays with the tiles (a row of zeros).
    DSKV_REQUIRE(route_one_row_requests >= 0 && route_one_row_requests <= DSKV_ROUTE_SHARED_LAUNCH,
                 "mixed_plan: unknown routing mode %d", route_one_row_requests);
    const bool route = route_one_row_requests && decode_mfma_shape(head_dim, n_qo_heads, n_kv_heads, page_size);
    std::vector<int32_t> kv_len(batch);
    std::vector<char> routed(batch, 0);
    std::vector<DecodeRow> rows;
    int64_t n_tile_rows = 0;
    for (int b = 0; b < batch; b++) {
        const int64_t np = (int64_t)kv_page_indptr_host[b + 1] - kv_page_indptr_host[b];
        DSKV_REQUIRE(np >= 0, "mixed_plan: kv_page_indptr not monotone at %d", b);
        const int32_t last = kv_last_page_len_host[b];
        DSKV_REQUIRE(np == 0 || (last >= 1 && last <= page_size),
                     "mixed_plan: kv_last_page_len[%d] = %d outside [1, %d]", b, last, page_size);
        const int64_t len = np > 0 ? (np - 1) * page_size + last : 0;
        DSKV_REQUIRE(len < (int64_t(1) << 30), "mixed_plan: request %d too long", b);
        kv_len[b] = (int32_t)len;
        const int64_t n_b = (int64_t)qo_indptr_host[b + 1] - qo_indptr_host[b];
        DSKV_REQUIRE(n_b >= 0, "mixed_plan: qo_indptr not monotone at %d", b);
        if (route && n_b == 1 && len > 0) {
            routed[b] = 1;
            rows.push_back(DecodeRow{len, kv_page_indptr_host[b], qo_indptr_host[b]});
        } else {
            n_tile_rows += n_b;
        }
    }
    // How the routed rows run.  Without tiled rows: the decode kernel by itself (workgroups of
    // eight waves; 117 us where the same rows take 138 us as tiles).  With both kinds: one
    // launch of four-wave workgroups that share the CUs (pages of at least four tokens: the
    // tile side then loads straight into LDS) and one merge pass for both - if the decode rows
    // are worth it.  As a tile, a decode row is a workgroup with one live row of 64 that walks
    // all of the row's keys by itself; measured over steps of 8 to 75 decode rows beside one to
    // sixteen chunks (bf16, 8 kv heads, groups of 4 and 8), the shared launch wins by 3-40 %
    // where these one-row tiles would be at least half of the launch's tile work (blocks walked
    // plus a fixed cost per tile) and there are a dozen rows or more (75 rows + a 437-token
    // chunk behind 2506 tokens: 147 against 152 us, behind 8000: 171 against 188; 24 rows behind
    // 4096: 86 against 126; 75 rows of at most 300 tokens: 53 against 87), and loses 5-10 %
    // beside a large prefill batch (16 chunks of 512: its four-wave tiles move every K/V row
    // through the CU twice) or with a handful of rows.
    const int rows_per_tile = prefill_rows_per_tile(n_qo_heads, n_kv_heads, kPrefillWaves);
    int64_t decode_cost = 0, tile_cost = 0;
    for (const DecodeRow &r : rows) decode_cost += (r.len + kBlock - 1) / kBlock + kTileFixedCostBlocks;
    for (int b = 0; b < batch; b++) {
        const int64_t n_b = (int64_t)qo_indptr_host[b + 1] - qo_indptr_host[b];
        if (routed[b] || n_b == 0) continue;
        for (int64_t r0 = 0; r0 < n_b; r0 += rows_per_tile) {
            const int64_t keys = std::max<int64_t>(kv_len[b] - n_b + std::min<int64_t>(r0 + rows_per_tile, n_b), 0);
            tile_cost += (keys + kBlock - 1) / kBlock + kTileFixedCostBlocks;
        }
    }
    int layout = DSKV_LAYOUT_SEPARATE;
    if (!rows.empty() && n_tile_rows > 0) {
        const bool can_share = page_size >= 4;
        if (route_one_row_requests == DSKV_ROUTE_SHARED_LAUNCH ||
            (route_one_row_requests == DSKV_ROUTE_AUTO && (int64_t)rows.size() >= kMinSharedLaunchRows &&
             decode_cost >= tile_cost))
            layout = can_share ? DSKV_LAYOUT_SHARED : DSKV_LAYOUT_SEPARATE;
        if (layout != DSKV_LAYOUT_SHARED && route_one_row_requests != DSKV_ROUTE_TWO_LAUNCHES) {
            // not worth it, or not possible: everything as tiles
            rows.clear();
            std::fill(routed.begin(), routed.end(), 0);
            n_tile_rows = qo_indptr_host[batch];
        }
    }
    info->layout = layout;
    const int waves = layout == DSKV_LAYOUT_SHARED ? kPrefillWavesShared : kPrefillWaves;
    int64_t tile_words = 0;
    int rc = plan_tiles(qo_indptr_host, kv_len.data(), rows.empty() ? nullptr : routed.data(), batch,
                        n_qo_heads, n_kv_heads, head_dim, target_workgroups, plan_host, capacity_words,
                        &info->n_tiles, &info->n_splits, &tile_words, &info->tile_workspace_bytes, waves,
                        /* the tiles of a shared launch run beside decode workgroups for its whole length */
                        layout != DSKV_LAYOUT_SHARED);
    if (rc) return rc;
    info->tile_workspace_bytes = (info->tile_workspace_bytes + 255) / 256 * 256;
    info->n_tile_rows = (int32_t)n_tile_rows;
    int64_t at = (tile_words + 3) / 4 * 4;
    info->plan_words = tile_words;
    if (rows.empty()) return 0;
    info->decode_plan_at = at;
    int64_t decode_words = 0;
    if (at > capacity_words) at = capacity_words;   // the decode planner then reports the shortage
    // shared launch: one decode workgroup (a share x a group of four kv heads) per compute unit
    int32_t decode_target = target_workgroups;
    if (layout == DSKV_LAYOUT_SHARED) {
        const int head_groups = (n_kv_heads + kSharedWaves - 1) / kSharedWaves;
        const int cus = target_workgroups > 0 ? std::min<int>(target_workgroups, kMaxWorkgroups) : compute_units();
        decode_target = std::max(1, cus / head_groups);
    }
    rc = plan_decode_rows(rows.data(), (int32_t)rows.size(), n_qo_heads, head_dim, decode_target,
                          plan_host + at, capacity_words - at, &info->n_decode_items,
                          &info->n_decode_workgroups, &decode_words, &info->decode_workspace_bytes);
    if (rc) return rc;
    info->n_decode_rows = (int32_t)rows.size();
    const int32_t *req_parts = plan_host + at + kPlanHeaderWords + info->n_decode_workgroups + 1;
    at += decode_words;
    // a shared launch merges the parts of both kinds of rows in one pass: behind the row map, a
    // table of (first slot, parts) for every row of the batch, the tile parts' slots first
    const int64_t nnz = qo_indptr_host[batch];
    const int64_t total = at + (int64_t)rows.size() + (layout == DSKV_LAYOUT_SHARED ? 2 * nnz : 0);
    if (total > capacity_words) {
        set_error("mixed_plan: plan needs %lld words, buffer has %lld", (long long)total,
                  (long long)capacity_words);
        return DSKV_E_NOMEM;
    }
    info->row_map_at = at;
    for (const DecodeRow &r : rows) plan_host[at++] = r.row;
    if (layout == DSKV_LAYOUT_SHARED) {
        int32_t *table = plan_host + at;
        if (info->n_splits > 1) std::copy_n(plan_host + (int64_t)info->n_tiles * kTileWords, 2 * nnz, table);
        else std::fill_n(table, 2 * nnz, 0);
        const int64_t slot_bytes = (int64_t)n_qo_heads * (head_dim + 2) * (int64_t)sizeof(float);
        const int64_t tile_slots = info->tile_workspace_bytes / slot_bytes;
        for (size_t i = 0; i < rows.size(); i++) {
            const int32_t first = req_parts[2 * i], n = req_parts[2 * i + 1];
            table[2 * (int64_t)rows[i].row] = n > 0 ? (int32_t)(tile_slots + first) : 0;
            table[2 * (int64_t)rows[i].row + 1] = n > 0 ? n : 0;
        }
    }
    info->plan_words = total;
    return 0;
}

namespace dskv {

static int launch_parts_merge(void *out, const float *part_o, const float *part_ml,
                              const int32_t *row_parts, int32_t nnz, int64_t max_slots,
                              int32_t n_qo_heads, int32_t dtype, hipStream_t s);

static bool prefill_mfma_path(int dtype, int head_dim, int n_qo_heads, int n_kv_heads, float scale_log2)
{
    // the MFMA kernel takes maxima before scaling: it needs a positive, sane scale
    return (dtype == DSKV_BF16 || dtype == DSKV_F16) && head_dim == kHeadDim && n_kv_heads > 0 &&
           n_qo_heads / n_kv_heads <= kWaveCols && scale_log2 > 1e-6f && scale_log2 < 1e6f;
}

// some_rows_elsewhere: the tiles do not cover all nnz rows of the batch (the others are the
// decode kernel's); an MFMA-path call with n_tiles == 0 then has nothing to do.
static int prefill_attn_impl(void *out, const void *q, const int32_t *qo_indptr,
                             const void *pages_layer, const int32_t *kv_page_indices,
                             const int32_t *kv_page_indptr, const int32_t *kv_last_page_len,
                             const int32_t *plan_dev, int32_t n_tiles, int32_t n_splits,
                             void *workspace, int64_t workspace_bytes, int32_t batch, int32_t nnz,
                             int32_t n_qo_heads, int32_t n_kv_heads, int32_t head_dim,
                             int32_t page_size, float sm_scale, int32_t causal, int32_t dtype,
                             void *stream, bool some_rows_elsewhere)
{
    DSKV_REQUIRE(batch >= 0 && nnz >= 0 && n_tiles >= 0, "prefill_attn: negative sizes");
    if (batch == 0 || nnz == 0) return 0;
    // kv_page_indices may be null when no request has a page (it is only read for requests that do)
    DSKV_REQUIRE(out && q && qo_indptr && pages_layer && kv_page_indptr && kv_last_page_len,
                 "prefill_attn: null pointer argument");
    DSKV_REQUIRE(dtype == DSKV_F32 || dtype == DSKV_F16 || dtype == DSKV_BF16,
                 "prefill_attn: unknown dtype %d", dtype);
    DSKV_REQUIRE(n_qo_heads > 0 && n_kv_heads > 0 && n_qo_heads % n_kv_heads == 0,
                 "prefill_attn: n_qo_heads %d not a multiple of n_kv_heads %d", n_qo_heads,
                 n_kv_heads);
    DSKV_REQUIRE(head_dim > 0 && head_dim <= 256, "prefill_attn: head_dim %d outside (0, 256]",
                 head_dim);
    DSKV_REQUIRE(page_size > 0, "prefill_attn: page_size must be positive");
    DSKV_REQUIRE(n_qo_heads <= 65535, "prefill_attn: too many heads");
    const float scale_log2 = sm_scale * 1.4426950408889634f;
    hipStream_t s = (hipStream_t)stream;
    const bool mfma = prefill_mfma_path(dtype, head_dim, n_qo_heads, n_kv_heads, scale_log2);
    if (mfma && some_rows_elsewhere && n_tiles == 0) return 0;   // every row went to the decode kernel
    if (mfma) {
        DSKV_REQUIRE(plan_dev && n_tiles > 0, "prefill_attn: missing plan");
        DSKV_REQUIRE(n_splits >= 1 && n_splits <= kMaxPrefillSplits,
                     "prefill_attn: tiles in up to %d parts", n_splits);
        float *part_o = nullptr, *part_ml = nullptr;
        int64_t max_slots = 0;
        if (n_splits > 1) {
            // the plan's partial slots are numbered from 0; the kernels never touch a slot at or
            // beyond max_slots, so a workspace smaller than the plan asked for loses rows, not memory
            const int64_t slot_bytes = (int64_t)n_qo_heads * (head_dim + 2) * (int64_t)sizeof(float);
            DSKV_REQUIRE(workspace && workspace_bytes >= slot_bytes && (uintptr_t)workspace % 16 == 0,
                         "prefill_attn: a plan with tiles in parts needs a 16-byte aligned workspace "
                         "(dskv_prefill_plan says how large), got %lld bytes", (long long)workspace_bytes);
            max_slots = std::min<int64_t>(workspace_bytes / slot_bytes, 1 << 30);
            part_o = reinterpret_cast<float *>(workspace);
            part_ml = part_o + max_slots * n_qo_heads * (int64_t)head_dim;
        }
        DSKV_REQUIRE(((uintptr_t)out | (uintptr_t)q | (uintptr_t)pages_layer) % 16 == 0,
                     "prefill_attn: out/q/pages must be 16-byte aligned");
        DSKV_REQUIRE(is_pow2(page_size),
                     "prefill_attn: 16-bit path needs a power-of-two page size, got %d", page_size);
        DSKV_REQUIRE((int64_t)n_tiles * n_kv_heads < (int64_t(1) << 31), "prefill_attn: too many tiles");
        dim3 grid((unsigned)n_tiles * (unsigned)n_kv_heads);
        dim3 block(64 * kPrefillWaves);
        const int shift = ilog2(page_size);
#define DSKV_LAUNCH_PREFILL(DT, SHARE)                                                          \
    hipLaunchKernelGGL((prefill_attn_mfma_kernel<DT, SHARE>), grid, block, 0, s, (uint16_t *)out, \
                       (const uint16_t *)q, qo_indptr, (const char *)pages_layer,               \
                       kv_page_indices, kv_page_indptr, kv_last_page_len, plan_dev,             \
                       n_qo_heads, n_kv_heads, shift, scale_log2, causal, part_o, part_ml,     \
                       (int)max_slots)
        if (dtype == DSKV_BF16) {
            if (page_size >= 4) DSKV_LAUNCH_PREFILL(DSKV_BF16, true);
            else DSKV_LAUNCH_PREFILL(DSKV_BF16, false);
        } else {
            if (page_size >= 4) DSKV_LAUNCH_PREFILL(DSKV_F16, true);
            else DSKV_LAUNCH_PREFILL(DSKV_F16, false);
        }
#undef DSKV_LAUNCH_PREFILL
        DSKV_LAUNCH_CHECK("prefill_attn_mfma_kernel");
        if (n_splits > 1)   // the parts' partials become the output rows
            return launch_parts_merge(out, part_o, part_ml, plan_dev + (int64_t)n_tiles * kTileWords, nnz,
                                      max_slots, n_qo_heads, dtype, s);
    } else {
        dim3 grid((unsigned)nnz, (unsigned)n_qo_heads);
#define DSKV_LAUNCH_GEN(DT)                                                                      \
    hipLaunchKernelGGL((prefill_attn_generic_kernel<DT>), grid, dim3(64), 0, s, out, q, qo_indptr, \
                       pages_layer, kv_page_indices, kv_page_indptr, kv_last_page_len, batch,    \
                       n_qo_heads, n_kv_heads, head_dim, page_size, scale_log2, causal)
        if (dtype == DSKV_F32) DSKV_LAUNCH_GEN(DSKV_F32);
        else if (dtype == DSKV_F16) DSKV_LAUNCH_GEN(DSKV_F16);
        else DSKV_LAUNCH_GEN(DSKV_BF16);
#undef DSKV_LAUNCH_GEN
        DSKV_LAUNCH_CHECK("prefill_attn_generic_kernel");
    }
    return 0;
}

// Merge pass of a tile plan with parts: one workgroup per query row of the batch (the decode
// path's merge kernel for rows in a few parts, see merge_kernel.h; one wave per (row, head)
// took 11.5 us for the 512 rows of a chunk, this about half); rows without parts return at once.
static int launch_parts_merge(void *out, const float *part_o, const float *part_ml,
                              const int32_t *row_parts, int32_t nnz, int64_t max_slots,
                              int32_t n_qo_heads, int32_t dtype, hipStream_t s)
{
    return launch_partials_merge(out, part_o, part_ml, row_parts, nullptr, (int)max_slots, nnz, n_qo_heads,
                                 kHeadDim, dtype, false, s);
}

// One launch for a batch of decode rows and chunks (layout DSKV_LAYOUT_SHARED), then the two
// merge passes.  The plan info comes from dskv_mixed_plan; everything in it that sizes a
// launch or an array is checked here.
static int mixed_shared_launch(void *out, const void *q, const int32_t *qo_indptr, const void *pages_layer,
                               const int32_t *kv_page_indices, const int32_t *kv_page_indptr,
                               const int32_t *kv_last_page_len, const int32_t *plan_dev,
                               const dskv_mixed_plan_t *info, void *workspace, int64_t workspace_bytes,
                               int32_t batch, int32_t nnz, int32_t n_qo_heads, int32_t n_kv_heads,
                               int32_t head_dim, int32_t page_size, float sm_scale, int32_t causal,
                               int32_t dtype, hipStream_t s)
{
    DSKV_REQUIRE(out && q && qo_indptr && pages_layer && kv_page_indices && kv_page_indptr && kv_last_page_len,
                 "mixed_attn: null pointer argument");
    DSKV_REQUIRE(decode_mfma_shape(head_dim, n_qo_heads, n_kv_heads, page_size) && page_size >= 4 &&
                     (dtype == DSKV_BF16 || dtype == DSKV_F16),
                 "mixed_attn: the shared launch takes 16-bit data, head_dim 128, groups up to 16 and "
                 "power-of-two pages of at least 4 tokens");
    DSKV_REQUIRE(((uintptr_t)out | (uintptr_t)q | (uintptr_t)pages_layer | (uintptr_t)workspace) % 16 == 0,
                 "mixed_attn: out/q/pages/workspace must be 16-byte aligned");
    DSKV_REQUIRE((int64_t)2 * page_size * n_kv_heads * head_dim * 2 < (int64_t(1) << 31),
                 "mixed_attn: a page must be smaller than 2 GiB");
    const int head_groups = (n_kv_heads + kSharedWaves - 1) / kSharedWaves;
    const int32_t n_rows = info->n_decode_rows, n_items = info->n_decode_items, shares = info->n_decode_workgroups;
    DSKV_REQUIRE(n_items >= n_rows && shares >= 1 && shares <= kMaxWorkgroups && info->n_tiles > 0 &&
                     info->n_splits >= 1 && info->n_splits <= kMaxPrefillSplits,
                 "mixed_attn: inconsistent plan (%d items of %d rows in %d shares, %d tile entries in up to %d parts)",
                 n_items, n_rows, shares, info->n_tiles, info->n_splits);
    const int64_t slot_bytes = (int64_t)n_qo_heads * (head_dim + 2) * (int64_t)sizeof(float);
    // workspace: the O partials of the tile parts' slots, then those of the cut decode rows'
    // slots, then the (maximum, sum) pairs in the same order - one numbering of slots, so that
    // one merge pass takes both kinds of rows
    MixedArgs a{};
    const int64_t tile_slots = info->tile_workspace_bytes / slot_bytes;
    const int64_t dec_slots = info->decode_workspace_bytes / slot_bytes;
    const int64_t all_slots = tile_slots + dec_slots;
    DSKV_REQUIRE(all_slots < (int64_t(1) << 30) && all_slots * slot_bytes <= workspace_bytes &&
                     (all_slots == 0 || workspace),
                 "mixed_attn: the plan's %lld partial slots need %lld bytes of workspace, got %lld",
                 (long long)all_slots, (long long)(all_slots * slot_bytes), (long long)workspace_bytes);
    DSKV_REQUIRE(info->n_splits == 1 || tile_slots >= 2, "mixed_attn: tiles in parts without partial slots");
    DSKV_REQUIRE(n_items == n_rows || dec_slots >= 2, "mixed_attn: cut decode rows without partial slots");
    float *const part_o = reinterpret_cast<float *>(workspace);
    float *const part_ml = part_o ? part_o + all_slots * n_qo_heads * (int64_t)head_dim : nullptr;
    a.tile_max_slots = (int)tile_slots;
    a.tile_part_o = part_o;
    a.tile_part_ml = part_ml;
    a.dec_max_slots = (int)dec_slots;
    a.dec_part_o = part_o ? part_o + tile_slots * n_qo_heads * (int64_t)head_dim : nullptr;
    a.dec_part_ml = part_ml ? part_ml + tile_slots * n_qo_heads * 2 : nullptr;
    const int32_t *dplan = plan_dev + info->decode_plan_at;
    a.wg_ptr = dplan + kPlanHeaderWords;
    const int32_t *req_parts = a.wg_ptr + shares + 1;
    a.items = reinterpret_cast<const Item *>(req_parts + 2 * (int64_t)n_rows);
    a.out = (uint16_t *)out;
    a.q = (const uint16_t *)q;
    a.pages = (const char *)pages_layer;
    a.kv_indices = kv_page_indices;
    a.n_qo_heads = n_qo_heads;
    a.n_kv_heads = n_kv_heads;
    a.page_shift = ilog2(page_size);
    a.scale_log2 = sm_scale * 1.4426950408889634f;
    DSKV_REQUIRE(a.scale_log2 > 1e-6f && a.scale_log2 < 1e6f, "mixed_attn: sm_scale out of range");
    a.n_decode_wgs = shares * head_groups;
    a.head_groups = head_groups;
    a.qo_indptr = qo_indptr;
    a.kv_indptr = kv_page_indptr;
    a.kv_last = kv_last_page_len;
    a.tile_info = plan_dev;
    a.causal = causal;
    const int64_t grid = (int64_t)a.n_decode_wgs + (int64_t)info->n_tiles * n_kv_heads;
    DSKV_REQUIRE(grid < (int64_t(1) << 31), "mixed_attn: too many workgroups");
    const dim3 g((unsigned)grid), b(64 * kSharedWaves);
#define DSKV_LAUNCH_MIXED(DT, PPT) hipLaunchKernelGGL((mixed_attn_kernel<DT, PPT>), g, b, 0, s, a)
    if (dtype == DSKV_BF16) {
        if (page_size >= kTile) DSKV_LAUNCH_MIXED(DSKV_BF16, 1);
        else if (page_size == 8) DSKV_LAUNCH_MIXED(DSKV_BF16, 2);
        else DSKV_LAUNCH_MIXED(DSKV_BF16, 0);
    } else {
        if (page_size >= kTile) DSKV_LAUNCH_MIXED(DSKV_F16, 1);
        else if (page_size == 8) DSKV_LAUNCH_MIXED(DSKV_F16, 2);
        else DSKV_LAUNCH_MIXED(DSKV_F16, 0);
    }
#undef DSKV_LAUNCH_MIXED
    DSKV_LAUNCH_CHECK("mixed_attn_kernel");
    // Rows cut into dozens of parts (a few very long decode rows): the decode path's wide merge
    // for them, then the tile parts' own pass.  Otherwise one pass over the table of all rows.
    const bool wide = (int64_t)n_items > 32 * (int64_t)n_rows;
    if (wide) {
        int rc = launch_partials_merge(out, a.dec_part_o, a.dec_part_ml, req_parts, plan_dev + info->row_map_at,
                                       a.dec_max_slots, n_rows, n_qo_heads, head_dim, dtype, true, s);
        if (rc) return rc;
        if (info->n_splits > 1)
            return launch_parts_merge(out, a.tile_part_o, a.tile_part_ml,
                                      plan_dev + (int64_t)info->n_tiles * kTileWords, nnz, a.tile_max_slots,
                                      n_qo_heads, dtype, s);
        return 0;
    }
    if (n_items > n_rows || info->n_splits > 1)
        return launch_parts_merge(out, part_o, part_ml, plan_dev + info->row_map_at + n_rows, nnz, all_slots,
                                  n_qo_heads, dtype, s);
    return 0;
}

}  // namespace dskv

extern "C" int dskv_prefill_attn(void *out, const void *q, const int32_t *qo_indptr,
                                 const void *pages_layer, const int32_t *kv_page_indices,
                                 const int32_t *kv_page_indptr, const int32_t *kv_last_page_len,
                                 const int32_t *plan_dev, int32_t n_tiles, int32_t n_splits,
                                 void *workspace, int64_t workspace_bytes, int32_t batch,
                                 int32_t nnz, int32_t n_qo_heads, int32_t n_kv_heads,
                                 int32_t head_dim, int32_t page_size, float sm_scale,
                                 int32_t causal, int32_t dtype, void *stream)
{
    return dskv::prefill_attn_impl(out, q, qo_indptr, pages_layer, kv_page_indices, kv_page_indptr,
                                   kv_last_page_len, plan_dev, n_tiles, n_splits, workspace,
                                   workspace_bytes, batch, nnz, n_qo_heads, n_kv_heads, head_dim,
                                   page_size, sm_scale, causal, dtype, stream, false);
}

extern "C" int dskv_mixed_attn(void *out, const void *q, const int32_t *qo_indptr,
                               const void *pages_layer, const int32_t *kv_page_indices,
                               const int32_t *kv_page_indptr, const int32_t *kv_last_page_len,
                               const int32_t *plan_dev, const dskv_mixed_plan_t *info,
                               void *workspace, int64_t workspace_bytes, int32_t batch, int32_t nnz,
                               int32_t n_qo_heads, int32_t n_kv_heads, int32_t head_dim,
                               int32_t page_size, float sm_scale, int32_t causal, int32_t dtype,
                               void *stream)
{
    using namespace dskv;
    DSKV_REQUIRE(info, "mixed_attn: null plan info");
    DSKV_REQUIRE(info->n_decode_rows >= 0 && info->n_tile_rows >= 0 && info->n_tiles >= 0 &&
                     info->tile_workspace_bytes >= 0 && info->decode_workspace_bytes >= 0,
                 "mixed_attn: negative sizes in the plan info");
    const bool routed = info->n_decode_rows > 0;
    const float scale_log2 = sm_scale * 1.4426950408889634f;
    // Shapes and types outside the 16-bit kernels: the generic kernel computes every row
    // of the batch by itself, routed or not.
    const bool mfma = n_qo_heads > 0 && n_kv_heads > 0 && n_qo_heads % n_kv_heads == 0 &&
                      prefill_mfma_path(dtype, head_dim, n_qo_heads, n_kv_heads, scale_log2);
    if (!routed || !mfma)
        return prefill_attn_impl(out, q, qo_indptr, pages_layer, kv_page_indices, kv_page_indptr,
                                 kv_last_page_len, plan_dev, info->n_tiles, info->n_splits, workspace,
                                 workspace_bytes, batch, nnz, n_qo_heads, n_kv_heads, head_dim,
                                 page_size, sm_scale, causal, dtype, stream, false);
    DSKV_REQUIRE(plan_dev, "mixed_attn: missing plan");
    DSKV_REQUIRE(info->n_decode_rows + info->n_tile_rows == nnz && info->n_decode_rows <= batch,
                 "mixed_attn: the plan covers %d + %d rows, the batch has %d", info->n_decode_rows,
                 info->n_tile_rows, nnz);
    DSKV_REQUIRE(workspace_bytes >= info->tile_workspace_bytes + info->decode_workspace_bytes &&
                     (workspace || info->tile_workspace_bytes + info->decode_workspace_bytes == 0),
                 "mixed_attn: the plan needs a workspace of %lld bytes, got %lld",
                 (long long)(info->tile_workspace_bytes + info->decode_workspace_bytes),
                 (long long)workspace_bytes);
    if (info->layout == DSKV_LAYOUT_SHARED)
        return mixed_shared_launch(out, q, qo_indptr, pages_layer, kv_page_indices, kv_page_indptr,
                                   kv_last_page_len, plan_dev, info, workspace, workspace_bytes, batch, nnz,
                                   n_qo_heads, n_kv_heads, head_dim, page_size, sm_scale, causal, dtype,
                                   (hipStream_t)stream);
    // The one-row requests: the split-KV decode pass (each K/V byte read once, at the speed
    // of memory) and its merge; their partials lie behind those of the tile parts.
    int rc = decode_rows_attn(out, q, pages_layer, kv_page_indices, plan_dev + info->decode_plan_at,
                              info->n_decode_items, info->n_decode_workgroups,
                              workspace ? (char *)workspace + info->tile_workspace_bytes : nullptr,
                              workspace ? workspace_bytes - info->tile_workspace_bytes : 0,
                              info->n_decode_rows, plan_dev + info->row_map_at, n_qo_heads, n_kv_heads,
                              head_dim, page_size, sm_scale, dtype, (hipStream_t)stream);
    if (rc) return rc;
    // The others: query tiles (and the merge of their parts, over the tiled rows only).
    return prefill_attn_impl(out, q, qo_indptr, pages_layer, kv_page_indices, kv_page_indptr,
                             kv_last_page_len, plan_dev, info->n_tiles, info->n_splits, workspace,
                             info->tile_workspace_bytes, batch, nnz, n_qo_heads, n_kv_heads, head_dim,
                             page_size, sm_scale, causal, dtype, stream, true);
}
