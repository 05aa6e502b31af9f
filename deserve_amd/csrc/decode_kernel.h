// The 16-bit split-KV decode attention kernel (head_dim 128) and the layout of its work
// list: see decode_attn.hip for the decomposition.  Kept in a header because two launches
// use its body: the stand-alone one (workgroups of eight waves) and the mixed launch of
// prefill_attn.hip, whose four-wave workgroups share their compute units with query tiles.
#pragma once

#include "kv_tile.h"
#include "rope_math.h"

namespace dskv {

constexpr int kMaxWaves = 8;         // kv heads per workgroup of the stand-alone launch
constexpr int kSharedWaves = 4;      // ... of a workgroup that shares its compute unit (mixed launch)
#ifndef DSKV_DECODE_STAGES
#define DSKV_DECODE_STAGES 3
#endif
constexpr int kStages = DSKV_DECODE_STAGES;   // tiles in flight per wave (one consumed, the rest loading)
constexpr int kPlanHeaderWords = 4;  // n_items, n_workgroups, n_slots, batch
constexpr int kItemWords = 8;
constexpr int kMaxWorkgroups = 4096;
#ifndef DSKV_DECODE_MIN_TILES
#define DSKV_DECODE_MIN_TILES 4
#endif
constexpr int kMinTilesPerWorkgroup = DSKV_DECODE_MIN_TILES;

// Work item written by the planner.  slot < 0: the item covers its whole request
// and writes the final output row; otherwise it writes partial slot `slot`.
struct Item {
    int32_t b;            // row of q and of the output (the request's index in a decode batch)
    int32_t tok_begin, tok_end, slot;
    int32_t page_begin;   // kv_page_indptr[b]: start of the request's block table
    int32_t tail;         // 1: tok_end is the request's length (the item holds its newest token)
    int32_t reserved[2];
};
static_assert(sizeof(Item) == kItemWords * 4, "plan item layout");

template <int kRing>
__device__ __forceinline__ int padded_end(const Item &it)
{
    const int tiles = (it.tok_end - it.tok_begin + kTile - 1) / kTile;
    return it.tok_begin + (tiles + kRing - 1) / kRing * kRing * kTile;
}

// Position of the load side in this workgroup's tile stream (wave-uniform).
struct LoadCursor {
    Item ahead;                // item next_item, requested when the item before it was entered
    int next_item, item_end;   // next item to enter, one past the workgroup's last
    int t, t_end, t_pad_end;   // next tile, valid end and padded end of the current item
    const_i32_ptr page_ids;    // current item's block table
    long page[2];              // pool pages of tile t (one or two), fetched one tile ahead of their use
};

#ifndef DSKV_DECODE_MIN_WAVES
#define DSKV_DECODE_MIN_WAVES 1
#endif
// The kernel's body for one workgroup: share `share` of the plan, kv heads head_group *
// kWaves .. + kWaves (one per wave); `lds_base`: kWaves * kVTileBytes of the workgroup's LDS.
// A function, so that one launch can hold workgroups of this kind next to others.
//   kPagesPerTile: pages a 16-token tile spans - 1 (pages of 16 tokens or more: one buffer
//     descriptor per tile), 2 (pages of 8 tokens: the two page ids as scalars, selected per
//     lane), 0 (smaller pages: every lane looks its page up itself; with four scalar ids and
//     a four-way selection pages of 4 tokens were slower than that, 130 against 113 us).
//   kRing: tiles in flight per wave (one consumed, the rest loading).
template <int DT, int kPagesPerTile, int kWaves, int kRing = kStages>
__device__ __forceinline__ void decode_attn_body(
    char *lds_base, int share, int head_group, uint16_t *__restrict__ out,
    const uint16_t *__restrict__ q, const char *pages, const int32_t *__restrict__ kv_indices,
    const Item *__restrict__ items, const int32_t *__restrict__ wg_ptr, float *__restrict__ part_o,
    float *__restrict__ part_ml, int max_slots, int n_qo_heads, int n_kv_heads, int page_shift,
    float scale_log2, const uint16_t *__restrict__ k_new, const uint16_t *__restrict__ v_new,
    const float *__restrict__ rope)
{
    typedef Elt<DT> E;
    constexpr bool kPageCoversTile = kPagesPerTile == 1;

    const int wave = threadIdx.x >> 6;
    const int lane = threadIdx.x & 63;
    const int g = lane >> 4;   // 16-lane group
    const int c = lane & 15;   // column within the group
    const int kvh = head_group * kWaves + wave;
    if (kvh >= n_kv_heads) return;
    const int group = n_qo_heads / n_kv_heads;
    // plan and block tables through the constant address space (scalar loads)
    const const_i32_ptr item_words = as_const(reinterpret_cast<const int32_t *>(items));
    auto load_item = [&](int idx) {
        const const_i32_ptr w = item_words + (long)idx * kItemWords;
        return Item{w[0], w[1], w[2], w[3], w[4], w[5], {0, 0}};
    };
    const const_i32_ptr indices_c = as_const(kv_indices);
    const int item_begin = as_const(wg_ptr)[share];
    const int item_end = as_const(wg_ptr)[share + 1];
    if (item_begin >= item_end) return;

    KvView kv;
    kv.pages = pages;
    kv.page_ids = indices_c;   // set per item
    kv.page_shift = page_shift;
    kv.row_bytes = n_kv_heads * kHeadDim * 2;
    kv.half_bytes = kv.row_bytes << page_shift;
    kv.page_bytes = 2L * kv.half_bytes;
    kv.head_off = kvh * (kHeadDim * 2);
    char *lds = lds_base + wave * kVTileBytes;

    // Fused append (k_new != null): the newest token of a request has not been written
    // to its page yet.  The wave that will read it - kv head `kvh` of the item that ends
    // the request - writes its 256 bytes of K and of V first and waits until the cache
    // has them; nobody else reads that row in this launch.
    auto append_new_rows = [&]() {
        for (int idx = item_begin; idx < item_end; idx++) {
            const Item it = load_item(idx);
            if (!it.tail) continue;
            const int tok = it.tok_end - 1;
            const long page = indices_c[it.page_begin + (tok >> page_shift)];
            char *row = const_cast<char *>(pages) + page * kv.page_bytes +
                        (long)(tok & ((1 << page_shift) - 1)) * kv.row_bytes + kv.head_off;
            const long src = ((long)it.b * n_kv_heads + kvh) * kHeadDim;
            if (lane < 16) {
                u32x4 chunk = *reinterpret_cast<const u32x4 *>(k_new + src + lane * 8);
                if (rope) {   // dims 8*lane .. +7 = pairs 4*lane .. +3 of the request's position
                    const float *tab = rope + (long)it.b * kHeadDim + lane * 4;
                    const f32x4 cs = *reinterpret_cast<const f32x4 *>(tab);
                    const f32x4 sn = *reinterpret_cast<const f32x4 *>(tab + kHeadDim / 2);
                    const float c4[4] = {cs[0], cs[1], cs[2], cs[3]}, s4[4] = {sn[0], sn[1], sn[2], sn[3]};
                    float f[8];
                    Chunk<DT>::unpack(chunk, f);
                    rope_rotate<4>(f, c4, s4);
                    chunk = Chunk<DT>::pack(f);
                }
                *reinterpret_cast<u32x4 *>(row + lane * 16) = chunk;
            } else if (lane < 32)
                *reinterpret_cast<u32x4 *>(row + kv.half_bytes + (lane - 16) * 16) =
                    *reinterpret_cast<const u32x4 *>(v_new + src + (lane - 16) * 8);
        }
        asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
    };

    // Q rows of one item as the B operand of the score MFMAs (zero beyond the group), and,
    // with a rope table, the cosines and sines of the lane's 16 dim pairs at the request's
    // position.  finish_q turns the two into the operand once they have arrived.
    struct QRaw {
        u32x4 q[4];
        f32x4 cs[4], sn[4];
    };
    auto load_q = [&](int item_idx, QRaw &dst) {
        const int b = item_words[(long)item_idx * kItemWords];
        const uint16_t *qrow = q + ((long)b * n_qo_heads + (long)kvh * group + c) * kHeadDim + g * 8;
#pragma unroll
        for (int kk = 0; kk < 4; kk++) {
            u32x4 z = {0, 0, 0, 0};
            dst.q[kk] = (c < group) ? *reinterpret_cast<const u32x4 *>(qrow + kk * 32) : z;
        }
        if (rope) {
            const float *tab = rope + (long)b * kHeadDim + g * 4;   // dims 32*kk + 8*g .. +7
#pragma unroll
            for (int kk = 0; kk < 4; kk++) {
                dst.cs[kk] = *reinterpret_cast<const f32x4 *>(tab + kk * 16);
                dst.sn[kk] = *reinterpret_cast<const f32x4 *>(tab + kHeadDim / 2 + kk * 16);
            }
        }
    };
    auto finish_q = [&](const QRaw &raw, u32x4 (&dst)[4]) {
#pragma unroll
        for (int kk = 0; kk < 4; kk++) {
            dst[kk] = raw.q[kk];
            if (rope) {
                const float c4[4] = {raw.cs[kk][0], raw.cs[kk][1], raw.cs[kk][2], raw.cs[kk][3]};
                const float s4[4] = {raw.sn[kk][0], raw.sn[kk][1], raw.sn[kk][2], raw.sn[kk][3]};
                float f[8];
                Chunk<DT>::unpack(raw.q[kk], f);
                rope_rotate<4>(f, c4, s4);
                dst[kk] = Chunk<DT>::pack(f);
            }
        }
    };

    // ---- load side
    LoadCursor cur;
    cur.next_item = item_begin;
    cur.item_end = item_end;
    cur.ahead = load_item(item_begin);
    cur.t = cur.t_end = cur.t_pad_end = 0;
    cur.page_ids = indices_c;
    for (long &pg : cur.page) pg = 0;
    auto fetch_page = [&]() {
        kv.page_ids = cur.page_ids;
        // an exhausted stream (t_end == 0) reads no block table: its descriptors are empty anyway
        if (kPageCoversTile) cur.page[0] = cur.t_end > 0 ? cur.page_ids[page_slot_of(kv, cur.t, cur.t_end)] : 0;
        if (kPagesPerTile > 1) {
            // an exhausted stream (t_end == 0) keeps loading from page 0, which every pool has
#pragma unroll
            for (int j = 0; j < kPagesPerTile; j++)
                cur.page[j] = cur.t_end > 0
                                  ? cur.page_ids[page_slot_of(kv, cur.t + (j << kv.page_shift), cur.t_end)]
                                  : 0;
        }
    };
    auto settle = [&]() {   // step into following items until a tile is available (or none is left)
        while (cur.t >= cur.t_pad_end && cur.next_item < cur.item_end) {
            // the item's words were requested an item ago: entering it costs no round trip in
            // front of the page id; the request for the one after it goes out now
            const Item it = cur.ahead;
            cur.next_item++;
            cur.ahead = load_item(min(cur.next_item, cur.item_end - 1));
            cur.t = it.tok_begin;
            cur.t_end = it.tok_end;
            cur.t_pad_end = padded_end<kRing>(it);
            cur.page_ids = indices_c + it.page_begin;
        }
        if (cur.t >= cur.t_pad_end) cur.t_end = 0;   // stream exhausted: every further tile is empty
        fetch_page();
    };
    auto load_next = [&](TileRegs &r) {
        kv.page_ids = cur.page_ids;
        if (kPageCoversTile) {
            load_kv_tile_in_page<kLoadStreaming>(kv, cur.page[0], cur.t, cur.t_end, g, c, r);
        } else if (kPagesPerTile > 1) {
            long pages_of_tile[kPagesPerTile > 1 ? kPagesPerTile : 1];
#pragma unroll
            for (int j = 0; j < kPagesPerTile; j++) pages_of_tile[j] = cur.page[j];
            load_kv_tile_small_pages<(kPagesPerTile > 1 ? kPagesPerTile : 1), kLoadStreaming>(
                kv, pages_of_tile, cur.t, cur.t_end, g, c, r);
        } else {
            load_kv_tile<false, kLoadStreaming>(kv, cur.t, cur.t_end, g, c, r);
        }
        cur.t += kTile;
        settle();
    };

    u32x4 qreg[4];
    QRaw qnext;
    load_q(item_begin, qnext);
    settle();
    // The new rows are written while the first tiles are already on their way (the chain item
    // -> page id -> store -> acknowledgement then runs beside the first K/V loads instead of
    // in front of them) - unless one of those tiles holds a new row: the first kRing tiles
    // all belong to the workgroup's first item with tiles (items are padded to whole rounds of
    // the ring), so that is the case only if that item ends its request within them.
    // A request without tokens is an item without tiles (it only writes a zero row): the load
    // side steps over it, so "first" means the first item that has tiles.
    bool rows_first = false;
    if (k_new) {
        for (int idx = item_begin; idx < item_end; idx++) {
            const Item it = load_item(idx);
            if (it.tok_end <= it.tok_begin) continue;
            rows_first = it.tail && it.tok_end - 1 < it.tok_begin + kRing * kTile;
            break;
        }
    }
    if (rows_first) append_new_rows();
    TileRegs ring[kRing];
#pragma unroll
    for (int s = 0; s < kRing; s++) load_next(ring[s]);
    if (k_new && !rows_first) append_new_rows();

    // ---- compute side
    Item item_ahead = load_item(item_begin);
    for (int idx = item_begin; idx < item_end; idx++) {
        const Item item = item_ahead;
        item_ahead = load_item(min(idx + 1, item_end - 1));   // for the next turn, like its q rows
        const int t_end = item.tok_end;
        // Q of the following item: issued now, so that it is older than every
        // tile load still in flight when it is needed (no drain at the switch)
        if (idx == item_begin) finish_q(qnext, qreg);
        load_q(min(idx + 1, item_end - 1), qnext);

        f32x4 acc[8];
#pragma unroll
        for (int dt = 0; dt < 8; dt++) acc[dt] = f32x4{0.f, 0.f, 0.f, 0.f};
        float m_run = kNegBig;
        float l_run = 0.f;

        auto compute_tile = [&](int t, const TileRegs &r) {
            // scores: S^T = K . Q^T ; lane holds tokens t + 4g + j of q column c
            f32x4 s = {0.f, 0.f, 0.f, 0.f};
#pragma unroll
            for (int kk = 0; kk < 4; kk++) s = E::mfma_k32(r.k[kk], qreg[kk], s);
            const bool ragged = t + kTile > t_end;   // wave-uniform: last and padding tiles
            float x[4];
#pragma unroll
            for (int j = 0; j < 4; j++) {
                x[j] = s[j] * scale_log2;
                if (ragged && t + 4 * g + j >= t_end) x[j] = kNegBig;
            }
            stage_v_tile<kPageCoversTile>(lds, r, t, t_end, g, c);
            // online softmax (log2 domain)
            float m_tile = fmaxf(fmaxf(x[0], x[1]), fmaxf(x[2], x[3]));
            m_tile = quad_rows_max(m_tile);
            const float m_new = fmaxf(m_run, m_tile);
            const float alpha = __builtin_amdgcn_exp2f(m_run - m_new);
            m_run = m_new;
            float p[4];
            float p_sum = 0.f;
#pragma unroll
            for (int j = 0; j < 4; j++) {
                // x > kNegBig keeps a fully masked tile (padding) at exactly zero weight
                p[j] = x[j] > kNegBig ? __builtin_amdgcn_exp2f(x[j] - m_new) : 0.f;
                p_sum += p[j];
            }
            l_run = l_run * alpha + p_sum;
            const u32x2 pb = {E::pack2(p[0], p[1]), E::pack2(p[2], p[3])};
            // O^T = alpha * O^T + V^T . P^T
#pragma unroll
            for (int dt = 0; dt < 8; dt++)
                acc[dt] = E::mfma_k16(read_v_operand(lds, dt, g, c), pb, acc[dt] * alpha);
            __builtin_amdgcn_wave_barrier();
        };

        // Straight-line body: the compiler can count the loads still in flight
        // and wait only for the tile it is about to consume.
        const int t_pad_end = padded_end<kRing>(item);
        for (int t = item.tok_begin; t < t_pad_end; t += kRing * kTile) {
#pragma unroll
            for (int s = 0; s < kRing; s++) {
                // a padding tile (items are padded to whole rounds of the ring) holds nothing:
                // its loads were issued and fetched nothing, its work is skipped (wave-uniform)
                if (t + s * kTile < t_end) compute_tile(t + s * kTile, ring[s]);
                // keep the scheduler from hoisting a later tile's work (and its
                // wait for younger loads) above this point
                __builtin_amdgcn_sched_barrier(0);
                load_next(ring[s]);
                __builtin_amdgcn_sched_barrier(0);
            }
        }

        // ---- item epilogue
        l_run = quad_rows_sum(l_run);
        if (c < group) {
            const int qh = kvh * group + c;
            if (item.slot < 0) {
                const float inv = l_run > 0.f ? 1.f / l_run : 0.f;
                uint16_t *o = out + ((long)item.b * n_qo_heads + qh) * kHeadDim + 4 * g;
#pragma unroll
                for (int dt = 0; dt < 8; dt++) {
                    u32x2 w = {E::pack2(acc[dt][0] * inv, acc[dt][1] * inv),
                               E::pack2(acc[dt][2] * inv, acc[dt][3] * inv)};
                    *reinterpret_cast<u32x2 *>(o + dt * 16) = w;
                }
            } else if (item.slot < max_slots) {   // a slot beyond the workspace is never written
                float *o = part_o + ((long)item.slot * n_qo_heads + qh) * kHeadDim + 4 * g;
#pragma unroll
                for (int dt = 0; dt < 8; dt++) *reinterpret_cast<f32x4 *>(o + dt * 16) = acc[dt];
                if (g == 0) {
                    float *ml = part_ml + ((long)item.slot * n_qo_heads + qh) * 2;
                    ml[0] = m_run;
                    ml[1] = l_run;
                }
            }
        }
        finish_q(qnext, qreg);
    }
}

template <int DT, int kPagesPerTile>
__global__ __launch_bounds__(64 * kMaxWaves, DSKV_DECODE_MIN_WAVES) void decode_attn_mfma_kernel(
    uint16_t *__restrict__ out, const uint16_t *__restrict__ q, const char *pages,
    const int32_t *__restrict__ kv_indices, const Item *__restrict__ items,
    const int32_t *__restrict__ wg_ptr, float *__restrict__ part_o, float *__restrict__ part_ml,
    int max_slots, int n_qo_heads, int n_kv_heads, int page_shift, float scale_log2,
    const uint16_t *__restrict__ k_new, const uint16_t *__restrict__ v_new,
    const float *__restrict__ rope)
{
    __shared__ __align__(16) char v_lds[kMaxWaves * kVTileBytes];
    decode_attn_body<DT, kPagesPerTile, kMaxWaves>(v_lds, (int)blockIdx.x, (int)blockIdx.y, out, q, pages,
                                                   kv_indices, items, wg_ptr, part_o, part_ml, max_slots,
                                                   n_qo_heads, n_kv_heads, page_shift, scale_log2, k_new,
                                                   v_new, rope);
}

}  // namespace dskv
