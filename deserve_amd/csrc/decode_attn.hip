// Paged decode attention for gfx950: split-KV flash-decoding over 16-token tiles.
//
// Bound: HBM.  Every K and V byte of a request is read exactly once (one
// wavefront owns one kv head and serves its whole GQA group), so the
// algorithmic traffic per layer is sum_b kv_len_b * 2 * Hkv * D * e bytes.
//
// Work decomposition
//   grid.x  = work items {request, token range} produced by the host planner,
//   wave w of a workgroup = kv head w; the 8 waves of a workgroup walk the
//   same pages, so a workgroup streams whole 64 KiB pages (K half, V half).
//
// Per 16-token tile and wave (D = 128, 16-bit elements):
//   S^T[token, qhead] = K_tile (16x128) . Q^T (128x16): four 16x16x32 MFMAs.
//     The A operand wants lane (g = lane/16, c = lane%16) to hold 8 consecutive
//     dims of token-row c - that is exactly one 16-byte global load from the K
//     row, so K goes HBM -> VGPR -> MFMA with no staging.  The B operand is the
//     GQA group's Q rows, zero padded to 16 columns, loaded once per item.
//   Online softmax in the log2 domain on the C layout (4 tokens x 1 q head per
//     lane); the running max is combined across the four 16-lane groups.
//   O^T[dim, qhead] += V_tile^T (128x16) . P^T (16x16): eight 16x16x16 MFMAs.
//     The C layout of S^T (lane holds tokens 4g..4g+3 of column c) is already
//     the B-operand layout, so P never moves.  The A operand needs 4 tokens of
//     ONE dim per lane, which is the transpose of how V lies in memory, so the
//     V tile is staged through LDS: written as loaded (16 B per lane, full rows
//     coalesced) and read back column-wise.  The MFMA row <-> token mapping is
//     permuted (row 4g+r <-> token g+4r, applied consistently to the K rows each
//     lane loads) so that the four lane groups read LDS rows g, g+1, g+2, g+3
//     of a 288-byte-pitch tile: bank-conflict free.
// Each wave keeps its own LDS tile, so there are no workgroup barriers.
//
// Partial results of split requests go to a workspace and a small merge kernel
// combines them; requests that fit one item are written directly.
#include "kv_tile.h"

#include <algorithm>
#include <math.h>
#include <vector>

namespace dskv {

constexpr int kMaxWaves = 8;   // kv heads per workgroup
constexpr int kStages = 3;     // tiles in flight per wave (one consumed, two loading)

// Work item written by the planner: request, [tok_begin, tok_end), partial slot
// (< 0: the item covers the whole request and writes the final output).
struct Item {
    int32_t b, tok_begin, tok_end, slot;
};

template <int DT, bool kPageCoversTile>
__global__ __launch_bounds__(64 * kMaxWaves) void decode_attn_mfma_kernel(
    uint16_t *__restrict__ out, const uint16_t *__restrict__ q, const char *__restrict__ pages,
    const int32_t *__restrict__ kv_indices, const int32_t *__restrict__ kv_indptr,
    const Item *__restrict__ items, float *__restrict__ part_o, float *__restrict__ part_ml,
    int max_slots, int n_qo_heads, int n_kv_heads, int page_shift, float scale_log2)
{
    typedef Elt<DT> E;
    __shared__ __align__(16) char v_lds[kMaxWaves][kVTileBytes];

    const int wave = threadIdx.x >> 6;
    const int lane = threadIdx.x & 63;
    const int g = lane >> 4;   // 16-lane group
    const int c = lane & 15;   // column within the group
    const int kvh = blockIdx.y * kMaxWaves + wave;
    if (kvh >= n_kv_heads) return;
    const int group = n_qo_heads / n_kv_heads;

    const Item item = items[blockIdx.x];
    const int b = item.b;
    const int t_end = item.tok_end;

    KvView kv;
    kv.pages = pages;
    kv.page_ids = kv_indices + kv_indptr[b];
    kv.page_shift = page_shift;
    kv.row_bytes = n_kv_heads * kHeadDim * 2;
    kv.half_bytes = kv.row_bytes << page_shift;
    kv.page_bytes = 2L * kv.half_bytes;
    kv.head_off = kvh * (kHeadDim * 2);

    // B operand of the score MFMAs: Q rows of this kv head's group (zero beyond).
    u32x4 qreg[4];
    {
        const uint16_t *qrow = q + ((long)b * n_qo_heads + (long)kvh * group + c) * kHeadDim + g * 8;
#pragma unroll
        for (int kk = 0; kk < 4; kk++) {
            u32x4 z = {0, 0, 0, 0};
            qreg[kk] = (c < group) ? *reinterpret_cast<const u32x4 *>(qrow + kk * 32) : z;
        }
    }

    f32x4 acc[8];
#pragma unroll
    for (int dt = 0; dt < 8; dt++) acc[dt] = f32x4{0.f, 0.f, 0.f, 0.f};
    float m_run = kNegBig;
    float l_run = 0.f;
    char *lds = v_lds[wave];

    auto compute_tile = [&](int t, const TileRegs &r) {
        // ---- scores: S^T = K . Q^T ; lane holds tokens t + g + 4j of q column c
        f32x4 s = {0.f, 0.f, 0.f, 0.f};
#pragma unroll
        for (int kk = 0; kk < 4; kk++) s = E::mfma_k32(r.k[kk], qreg[kk], s);
        const bool ragged = t + kTile > t_end;   // wave-uniform: only the last tile
        float x[4];
#pragma unroll
        for (int j = 0; j < 4; j++) {
            x[j] = s[j] * scale_log2;
            if (ragged && t + g + 4 * j >= t_end) x[j] = kNegBig;
        }
        stage_v_tile<kPageCoversTile>(lds, r, t, t_end, g, c);
        // ---- online softmax (log2 domain)
        float m_tile = fmaxf(fmaxf(x[0], x[1]), fmaxf(x[2], x[3]));
        m_tile = fmaxf(m_tile, __shfl_xor(m_tile, 16));
        m_tile = fmaxf(m_tile, __shfl_xor(m_tile, 32));
        const float m_new = fmaxf(m_run, m_tile);
        const float alpha = __builtin_amdgcn_exp2f(m_run - m_new);
        m_run = m_new;
        float p[4];
        float p_sum = 0.f;
#pragma unroll
        for (int j = 0; j < 4; j++) {
            p[j] = __builtin_amdgcn_exp2f(x[j] - m_new);
            p_sum += p[j];
        }
        l_run = l_run * alpha + p_sum;
        const u32x2 pb = {E::pack2(p[0], p[1]), E::pack2(p[2], p[3])};
        // ---- O^T = alpha * O^T + V^T . P^T
#pragma unroll
        for (int dt = 0; dt < 8; dt++)
            acc[dt] = E::mfma_k16(read_v_operand(lds, dt, g, c), pb, acc[dt] * alpha);
        __builtin_amdgcn_wave_barrier();
    };

    // ---- main loop: a ring of kStages tile buffers
    TileRegs ring[kStages];
    int t = item.tok_begin;
#pragma unroll
    for (int s = 0; s < kStages; s++)
        load_kv_tile<kPageCoversTile>(kv, t + s * kTile, t_end, g, c, ring[s]);
    // steady state: straight-line body, so the compiler can count the loads
    // still in flight and wait only for the tile it is about to consume
    while (t + (kStages - 1) * kTile < t_end) {
#pragma unroll
        for (int s = 0; s < kStages; s++) {
            compute_tile(t + s * kTile, ring[s]);
            // keep the scheduler from hoisting a later tile's work (and its
            // wait for younger loads) above this point
            __builtin_amdgcn_sched_barrier(0);
            load_kv_tile<kPageCoversTile>(kv, t + (s + kStages) * kTile, t_end, g, c, ring[s]);
            __builtin_amdgcn_sched_barrier(0);
        }
        t += kStages * kTile;
    }
    // tail: fewer than kStages tiles are left, all of them already loaded
#pragma unroll
    for (int s = 0; s < kStages - 1; s++)
        if (t + s * kTile < t_end) compute_tile(t + s * kTile, ring[s]);

    // ---- epilogue
    l_run += __shfl_xor(l_run, 16);
    l_run += __shfl_xor(l_run, 32);
    if (c >= group) return;
    const int qh = kvh * group + c;
    if (item.slot < 0) {
        const float inv = l_run > 0.f ? 1.f / l_run : 0.f;
        uint16_t *o = out + ((long)b * n_qo_heads + qh) * kHeadDim + 4 * g;
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


// ---------------------------------------------------------------------------
// Generic path: any head_dim <= 256, any group size, fp32 or 16-bit storage.
// One wavefront per (item, q head); lanes own dims lane, lane+64, ...; plain
// VALU dot products with a wave reduction per token.  Used for fp32 pools and
// shapes the MFMA kernel is not specialised for.
// ---------------------------------------------------------------------------
template <int DT>
__global__ __launch_bounds__(64) void decode_attn_generic_kernel(
    void *__restrict__ out, const void *__restrict__ q, const void *__restrict__ pages,
    const int32_t *__restrict__ kv_indices, const int32_t *__restrict__ kv_indptr,
    const Item *__restrict__ items, float *__restrict__ part_o, float *__restrict__ part_ml,
    int max_slots, int n_qo_heads, int n_kv_heads, int head_dim, int page_size, float scale_log2)
{
    typedef LoadElt<DT> L;
    const int lane = threadIdx.x;
    const int qh = blockIdx.y;
    const int kvh = qh / (n_qo_heads / n_kv_heads);
    const Item item = items[blockIdx.x];
    const int b = item.b;
    const int page_begin = kv_indptr[b];
    const long row = (long)n_kv_heads * head_dim;
    const long half = row * page_size;

    float qv[4], acc[4];
#pragma unroll
    for (int i = 0; i < 4; i++) {
        const int d = lane + 64 * i;
        qv[i] = d < head_dim ? L::get(q, ((long)b * n_qo_heads + qh) * head_dim + d) : 0.f;
        acc[i] = 0.f;
    }
    float m_run = kNegBig, l_run = 0.f;
    for (int t = item.tok_begin; t < item.tok_end; t++) {
        const long page = kv_indices[page_begin + t / page_size];
        const long base = page * 2 * half + (long)(t % page_size) * row + (long)kvh * head_dim;
        float dot = 0.f;
#pragma unroll
        for (int i = 0; i < 4; i++) {
            const int d = lane + 64 * i;
            if (d < head_dim) dot += qv[i] * L::get(pages, base + d);
        }
        const float x = wave_sum(dot) * scale_log2;
        const float m_new = fmaxf(m_run, x);
        const float alpha = __builtin_amdgcn_exp2f(m_run - m_new);
        const float p = __builtin_amdgcn_exp2f(x - m_new);
        l_run = l_run * alpha + p;
#pragma unroll
        for (int i = 0; i < 4; i++) {
            const int d = lane + 64 * i;
            if (d < head_dim) acc[i] = acc[i] * alpha + p * L::get(pages, base + half + d);
        }
        m_run = m_new;
    }
    if (item.slot < 0) {
        const float inv = l_run > 0.f ? 1.f / l_run : 0.f;
#pragma unroll
        for (int i = 0; i < 4; i++) {
            const int d = lane + 64 * i;
            if (d < head_dim) L::put(out, ((long)b * n_qo_heads + qh) * head_dim + d, acc[i] * inv);
        }
    } else if (item.slot < max_slots) {
        float *o = part_o + ((long)item.slot * n_qo_heads + qh) * head_dim;
#pragma unroll
        for (int i = 0; i < 4; i++) {
            const int d = lane + 64 * i;
            if (d < head_dim) o[d] = acc[i];
        }
        if (lane == 0) {
            float *ml = part_ml + ((long)item.slot * n_qo_heads + qh) * 2;
            ml[0] = m_run;
            ml[1] = l_run;
        }
    }
}

// Combine the partials of split requests.  One wavefront per (request, q head).
template <int DT>
__global__ __launch_bounds__(64) void decode_merge_kernel(void *__restrict__ out,
                                                          const float *__restrict__ part_o,
                                                          const float *__restrict__ part_ml,
                                                          const int32_t *__restrict__ req_parts,
                                                          int max_slots, int n_qo_heads,
                                                          int head_dim)
{
    typedef LoadElt<DT> L;
    const int b = blockIdx.x, qh = blockIdx.y, lane = threadIdx.x;
    const int first = req_parts[2 * b], n = req_parts[2 * b + 1];
    if (n <= 0) return;   // written directly by the attention kernel
    if (first < 0 || first + n > max_slots) return;
    float m = kNegBig;
    for (int s = 0; s < n; s++) m = fmaxf(m, part_ml[((long)(first + s) * n_qo_heads + qh) * 2]);
    float acc[4] = {0.f, 0.f, 0.f, 0.f};
    float l = 0.f;
    for (int s = 0; s < n; s++) {
        const long base = (long)(first + s) * n_qo_heads + qh;
        const float w = __builtin_amdgcn_exp2f(part_ml[base * 2] - m);
        l += w * part_ml[base * 2 + 1];
#pragma unroll
        for (int i = 0; i < 4; i++) {
            const int d = lane + 64 * i;
            if (d < head_dim) acc[i] += w * part_o[base * head_dim + d];
        }
    }
    const float inv = l > 0.f ? 1.f / l : 0.f;
#pragma unroll
    for (int i = 0; i < 4; i++) {
        const int d = lane + 64 * i;
        if (d < head_dim) L::put(out, ((long)b * n_qo_heads + qh) * head_dim + d, acc[i] * inv);
    }
}

static bool mfma_path(int dtype, int head_dim, int n_qo_heads, int n_kv_heads)
{
    return (dtype == DSKV_BF16 || dtype == DSKV_F16) && head_dim == kHeadDim &&
           n_qo_heads / n_kv_heads <= 16;
}

}  // namespace dskv

// ---------------------------------------------------------------------------
// Host planner
// ---------------------------------------------------------------------------
extern "C" int64_t dskv_decode_plan_bound(int32_t batch, int64_t total_tokens)
{
    if (batch < 0 || total_tokens < 0) return 0;
    // every request yields at least one item and at most one per tile
    const int64_t max_items = (int64_t)batch + total_tokens / dskv::kTile + 1;
    return max_items * 4 + (int64_t)batch * 2;
}

extern "C" int dskv_decode_plan(const int32_t *kv_page_indptr_host,
                                const int32_t *kv_last_page_len_host, int32_t batch,
                                int32_t page_size, int32_t n_qo_heads, int32_t n_kv_heads,
                                int32_t head_dim, int32_t target_items, int32_t *plan_host,
                                int64_t plan_capacity_words, int32_t *n_items_out,
                                int64_t *plan_words_out, int64_t *workspace_bytes_out)
{
    using namespace dskv;
    DSKV_REQUIRE(batch >= 0, "decode_plan: negative batch");
    DSKV_REQUIRE(n_items_out && plan_words_out && workspace_bytes_out,
                 "decode_plan: null output pointer");
    DSKV_REQUIRE(page_size > 0 && n_qo_heads > 0 && n_kv_heads > 0 && head_dim > 0 &&
                     n_qo_heads % n_kv_heads == 0,
                 "decode_plan: bad shape (page %d, heads %d/%d, dim %d)", page_size, n_qo_heads,
                 n_kv_heads, head_dim);
    *n_items_out = 0;
    *plan_words_out = 0;
    *workspace_bytes_out = 0;
    if (batch == 0) return 0;
    DSKV_REQUIRE(kv_page_indptr_host && kv_last_page_len_host && plan_host,
                 "decode_plan: null pointer argument");

    std::vector<int64_t> len(batch);
    int64_t total_tiles = 0;
    for (int b = 0; b < batch; b++) {
        const int64_t np = (int64_t)kv_page_indptr_host[b + 1] - kv_page_indptr_host[b];
        DSKV_REQUIRE(np >= 0, "decode_plan: kv_page_indptr not monotone at %d", b);
        const int32_t last = kv_last_page_len_host[b];
        DSKV_REQUIRE(np == 0 || (last >= 1 && last <= page_size),
                     "decode_plan: kv_last_page_len[%d] = %d outside [1, %d]", b, last, page_size);
        len[b] = np > 0 ? (np - 1) * page_size + last : 0;
        DSKV_REQUIRE(len[b] < (int64_t(1) << 30), "decode_plan: request %d too long", b);
        total_tiles += (len[b] + kTile - 1) / kTile;
    }
    // Chunk size: enough items to keep every CU busy with a few waves of
    // workgroups, but never chunks so small that the per-item prologue, the
    // partial write-out and the merge dominate.
    if (target_items <= 0) target_items = 1024;
    const int64_t kMinChunkTiles = 4;
    int64_t chunk_tiles = (total_tiles + target_items - 1) / target_items;
    chunk_tiles = std::max(chunk_tiles, kMinChunkTiles);

    std::vector<Item> items;
    std::vector<int32_t> req(2 * (size_t)batch);
    int32_t n_slots = 0;
    for (int b = 0; b < batch; b++) {
        const int64_t tiles = (len[b] + kTile - 1) / kTile;
        const int64_t parts = std::max<int64_t>(1, (tiles + chunk_tiles - 1) / chunk_tiles);
        if (parts == 1) {
            items.push_back(Item{b, 0, (int32_t)len[b], -1});
            req[2 * b] = 0;
            req[2 * b + 1] = 0;
            continue;
        }
        req[2 * b] = n_slots;
        req[2 * b + 1] = (int32_t)parts;
        int64_t done = 0;
        for (int64_t p = 0; p < parts; p++) {
            const int64_t take = tiles / parts + (p < tiles % parts ? 1 : 0);
            const int64_t begin = done * kTile;
            const int64_t end = std::min<int64_t>((done + take) * kTile, len[b]);
            items.push_back(Item{b, (int32_t)begin, (int32_t)end, n_slots++});
            done += take;
        }
    }
    // longest first: the hardware dispatcher hands out workgroups in order
    std::stable_sort(items.begin(), items.end(), [](const Item &x, const Item &y) {
        return (x.tok_end - x.tok_begin) > (y.tok_end - y.tok_begin);
    });
    const int64_t words = (int64_t)items.size() * 4 + (int64_t)batch * 2;
    if (words > plan_capacity_words) {
        set_error("decode_plan: plan needs %lld words, buffer has %lld", (long long)words,
                  (long long)plan_capacity_words);
        return DSKV_E_NOMEM;
    }
    std::copy(reinterpret_cast<const int32_t *>(items.data()),
              reinterpret_cast<const int32_t *>(items.data()) + items.size() * 4, plan_host);
    std::copy(req.begin(), req.end(), plan_host + items.size() * 4);
    *n_items_out = (int32_t)items.size();
    *plan_words_out = words;
    *workspace_bytes_out = (int64_t)n_slots * n_qo_heads * (head_dim + 2) * (int64_t)sizeof(float);
    return 0;
}

extern "C" int dskv_decode_attn(void *out, const void *q, const void *pages_layer,
                                const int32_t *kv_page_indices, const int32_t *kv_page_indptr,
                                const int32_t *plan_dev, int32_t n_items, void *workspace,
                                int64_t workspace_bytes, int32_t batch, int32_t n_qo_heads,
                                int32_t n_kv_heads, int32_t head_dim, int32_t page_size,
                                float sm_scale, int32_t dtype, void *stream)
{
    using namespace dskv;
    DSKV_REQUIRE(batch >= 0 && n_items >= 0, "decode_attn: negative batch/n_items");
    if (batch == 0 || n_items == 0) return 0;
    DSKV_REQUIRE(out && q && pages_layer && kv_page_indices && kv_page_indptr && plan_dev,
                 "decode_attn: null pointer argument");
    DSKV_REQUIRE(dtype == DSKV_F32 || dtype == DSKV_F16 || dtype == DSKV_BF16,
                 "decode_attn: unknown dtype %d", dtype);
    DSKV_REQUIRE(n_qo_heads > 0 && n_kv_heads > 0 && n_qo_heads % n_kv_heads == 0,
                 "decode_attn: n_qo_heads %d not a multiple of n_kv_heads %d", n_qo_heads,
                 n_kv_heads);
    DSKV_REQUIRE(head_dim > 0 && head_dim <= 256, "decode_attn: head_dim %d outside (0, 256]",
                 head_dim);
    DSKV_REQUIRE(page_size > 0, "decode_attn: page_size must be positive");
    DSKV_REQUIRE(n_items >= batch, "decode_attn: plan has fewer items than requests");
    DSKV_REQUIRE(n_qo_heads <= 65535 && n_kv_heads <= 65535 * kMaxWaves, "decode_attn: too many heads");
    // Partial slots are numbered densely from 0 by the planner.  A plan with
    // n_items items over batch requests has at least n_items - batch + 1 of them
    // when anything is split; the kernels additionally refuse to touch a slot at
    // or beyond max_slots, so an undersized workspace can never be overrun.
    const int64_t slot_bytes = (int64_t)n_qo_heads * (head_dim + 2) * (int64_t)sizeof(float);
    DSKV_REQUIRE(workspace_bytes >= 0, "decode_attn: negative workspace size");
    const int64_t max_slots = std::min<int64_t>(workspace ? workspace_bytes / slot_bytes : 0, 1 << 30);
    DSKV_REQUIRE(n_items == batch || max_slots >= (int64_t)n_items - batch + 1,
                 "decode_attn: workspace (%lld bytes) too small for %d items of %d requests",
                 (long long)workspace_bytes, n_items, batch);

    const Item *items = reinterpret_cast<const Item *>(plan_dev);
    const int32_t *req_parts = plan_dev + (int64_t)n_items * 4;
    // slots are numbered densely from 0, so part_ml can sit after max_slots O blocks
    float *part_o = reinterpret_cast<float *>(workspace);
    float *part_ml = part_o ? part_o + max_slots * n_qo_heads * (int64_t)head_dim : nullptr;
    const float scale_log2 = sm_scale * 1.4426950408889634f;
    hipStream_t s = (hipStream_t)stream;

    if (mfma_path(dtype, head_dim, n_qo_heads, n_kv_heads)) {
        DSKV_REQUIRE(((uintptr_t)out | (uintptr_t)q | (uintptr_t)pages_layer) % 16 == 0,
                     "decode_attn: out/q/pages must be 16-byte aligned");
        DSKV_REQUIRE(is_pow2(page_size), "decode_attn: 16-bit path needs a power-of-two page size, got %d",
                     page_size);
        const int waves = std::min(n_kv_heads, kMaxWaves);
        dim3 grid((unsigned)n_items, (unsigned)((n_kv_heads + kMaxWaves - 1) / kMaxWaves));
        dim3 block(64 * waves);
        const int shift = ilog2(page_size);
#define DSKV_LAUNCH_MFMA(DT, COVER)                                                              \
    hipLaunchKernelGGL((decode_attn_mfma_kernel<DT, COVER>), grid, block, 0, s, (uint16_t *)out, \
                       (const uint16_t *)q, (const char *)pages_layer, kv_page_indices,          \
                       kv_page_indptr, items, part_o, part_ml, (int)max_slots, n_qo_heads,       \
                       n_kv_heads, shift, scale_log2)
        if (dtype == DSKV_BF16) {
            if (page_size >= kTile) DSKV_LAUNCH_MFMA(DSKV_BF16, true);
            else DSKV_LAUNCH_MFMA(DSKV_BF16, false);
        } else {
            if (page_size >= kTile) DSKV_LAUNCH_MFMA(DSKV_F16, true);
            else DSKV_LAUNCH_MFMA(DSKV_F16, false);
        }
#undef DSKV_LAUNCH_MFMA
        DSKV_LAUNCH_CHECK("decode_attn_mfma_kernel");
    } else {
        dim3 grid((unsigned)n_items, (unsigned)n_qo_heads);
#define DSKV_LAUNCH_GEN(DT)                                                                       \
    hipLaunchKernelGGL((decode_attn_generic_kernel<DT>), grid, dim3(64), 0, s, out, q, pages_layer, \
                       kv_page_indices, kv_page_indptr, items, part_o, part_ml, (int)max_slots,   \
                       n_qo_heads, n_kv_heads, head_dim, page_size, scale_log2)
        if (dtype == DSKV_F32) DSKV_LAUNCH_GEN(DSKV_F32);
        else if (dtype == DSKV_F16) DSKV_LAUNCH_GEN(DSKV_F16);
        else DSKV_LAUNCH_GEN(DSKV_BF16);
#undef DSKV_LAUNCH_GEN
        DSKV_LAUNCH_CHECK("decode_attn_generic_kernel");
    }
    if (n_items > batch) {
        dim3 grid((unsigned)batch, (unsigned)n_qo_heads);
        if (dtype == DSKV_F32)
            hipLaunchKernelGGL((decode_merge_kernel<DSKV_F32>), grid, dim3(64), 0, s, out, part_o,
                               part_ml, req_parts, (int)max_slots, n_qo_heads, head_dim);
        else if (dtype == DSKV_F16)
            hipLaunchKernelGGL((decode_merge_kernel<DSKV_F16>), grid, dim3(64), 0, s, out, part_o,
                               part_ml, req_parts, (int)max_slots, n_qo_heads, head_dim);
        else
            hipLaunchKernelGGL((decode_merge_kernel<DSKV_BF16>), grid, dim3(64), 0, s, out, part_o,
                               part_ml, req_parts, (int)max_slots, n_qo_heads, head_dim);
        DSKV_LAUNCH_CHECK("decode_merge_kernel");
    }
    return 0;
}
