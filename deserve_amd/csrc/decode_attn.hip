// Paged decode attention for gfx950: split-KV flash-decoding over 16-token tiles
// with statically balanced, persistent workgroups.
//
// Bound: HBM.  Every K and V byte of a request is read exactly once (one
// wavefront owns one kv head and serves its whole GQA group), so the
// algorithmic traffic per layer is sum_b kv_len_b * 2 * Hkv * D * e bytes.
//
// Work decomposition
//   The host planner lays all requests' tiles end to end and cuts that sequence
//   into one equal share per workgroup (one workgroup per CU by default), so
//   every CU streams the same number of bytes and there is no tail.  A share
//   that crosses request boundaries is a short list of work items {request,
//   token range}; a request cut by share boundaries is merged afterwards from
//   per-item partials (m, l, O).
//   Wave w of a workgroup = kv head w; the 8 waves walk the same pages, so a
//   workgroup streams whole 64 KiB pages (K half, V half).
//   The load side runs ahead of the compute side by kStages tiles THROUGH item
//   boundaries: while the last tiles of one item are consumed, the first tiles
//   of the next one are already in flight, so the memory pipe never drains
//   inside a workgroup.  Items are padded to a multiple of kStages tiles; the
//   padding tiles fetch nothing (empty buffer descriptor) and contribute zero.
//
// Per 16-token tile and wave (D = 128, 16-bit elements):
//   S^T[token, qhead] = K_tile (16x128) . Q^T (128x16): four 16x16x32 MFMAs.
//     The A operand wants lane (g = lane/16, c = lane%16) to hold 8 consecutive
//     dims of token-row c - that is exactly one 16-byte load from the K row, so
//     K goes HBM -> VGPR -> MFMA with no staging.  The B operand is the GQA
//     group's Q rows, zero padded to 16 columns.
//   Online softmax in the log2 domain on the C layout (4 tokens x 1 q head per
//     lane); the running max is combined across the four 16-lane groups.
//   O^T[dim, qhead] += V_tile^T (128x16) . P^T (16x16): eight 16x16x16 MFMAs.
//     The C layout of S^T is already the B-operand layout, so P never moves.  V
//     needs 4 tokens of ONE dim per lane - the transpose of how it lies in
//     memory - so the V tile goes through a wave-private LDS tile.
#include "decode_kernel.h"
#include "merge_kernel.h"

#include <algorithm>
#include <math.h>
#include <mutex>
#include <vector>

#ifndef DSKV_DECODE_STATIC_SCRATCH_BYTES
#define DSKV_DECODE_STATIC_SCRATCH_BYTES (32 << 20)
#endif

namespace dskv {

// ---------------------------------------------------------------------------
// Generic path: any head_dim <= 256, any group size, fp32 or 16-bit storage.
// One wavefront per (item, q head); lanes own dims lane, lane+64, ...; plain
// VALU dot products with a wave reduction per token.  Used for fp32 pools and
// shapes the MFMA kernel is not specialised for.
// ---------------------------------------------------------------------------
template <int DT>
__global__ __launch_bounds__(64) void decode_attn_generic_kernel(
    void *__restrict__ out, const void *__restrict__ q, const void *__restrict__ pages,
    const int32_t *__restrict__ kv_indices, const Item *__restrict__ items,
    float *__restrict__ part_o, float *__restrict__ part_ml, int max_slots, int n_qo_heads,
    int n_kv_heads, int head_dim, int page_size, float scale_log2)
{
    typedef LoadElt<DT> L;
    const int lane = threadIdx.x;
    const int qh = blockIdx.y;
    const int kvh = qh / (n_qo_heads / n_kv_heads);
    const Item item = items[blockIdx.x];
    const int b = item.b;
    const int page_begin = item.page_begin;
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
    // kGroup tokens at a time: their page ids, K rows and V rows are all requested before the
    // first is used, so a wave waits for memory once per group instead of twice per token
    // (token by token the pass over 8 x 512 fp32 tokens took 90 us, all of it latency)
    constexpr int kGroup = 8;
    const int last_tok = item.tok_end - 1;
    for (int t0 = item.tok_begin; t0 < item.tok_end; t0 += kGroup) {
        long base[kGroup];
#pragma unroll
        for (int j = 0; j < kGroup; j++) {
            const int t = min(t0 + j, last_tok);   // past the end: the last token again, weight zero
            const long page = kv_indices[page_begin + t / page_size];
            base[j] = page * 2 * half + (long)(t % page_size) * row + (long)kvh * head_dim;
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
            x[j] = t0 + j <= last_tok ? wave_sum(dot) * scale_log2 : kNegBig;
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

// ---------------------------------------------------------------------------
// Generic path that shares K/V across the GQA group: fp32 or 16-bit storage, head_dim a
// multiple of 8 up to 128, groups of up to 8 q heads.  One wavefront per (item, kv head)
// serves all q heads of the group, so each K/V byte crosses the memory path once (the kernel
// above reads it once per q head).  Lane (g = lane / 16, c = lane % 16) holds dims 8c .. 8c+7
// of tokens t + g, t + 4 + g, ...: a token's row is 16 lanes x 32 (or 16) bytes, contiguous;
// the scores are reduced over the 16 lanes of a row with DPP adds, 16 tokens are in flight per
// iteration, and the per-group partial sums of O are folded across g once, at the end.
// The block table entries of an iteration are fetched an iteration ahead.
// ---------------------------------------------------------------------------
__device__ __forceinline__ float row16_sum(float v)
{
    // quad_perm [1,0,3,2], quad_perm [2,3,0,1], row_half_mirror, row_mirror
    v += __builtin_bit_cast(float, __builtin_amdgcn_mov_dpp(__builtin_bit_cast(int, v), 0xB1, 0xF, 0xF, true));
    v += __builtin_bit_cast(float, __builtin_amdgcn_mov_dpp(__builtin_bit_cast(int, v), 0x4E, 0xF, 0xF, true));
    v += __builtin_bit_cast(float, __builtin_amdgcn_mov_dpp(__builtin_bit_cast(int, v), 0x141, 0xF, 0xF, true));
    v += __builtin_bit_cast(float, __builtin_amdgcn_mov_dpp(__builtin_bit_cast(int, v), 0x140, 0xF, 0xF, true));
    return v;
}

template <int DT>
__device__ __forceinline__ void load_row8(const char *row, bool live, float (&f)[8])
{
    // 8 consecutive elements of a K or V row (zeros for a lane beyond head_dim)
    constexpr int kChunks = 8 / Chunk<DT>::kElems;   // fp32: two 16-byte loads, 16-bit: one
#pragma unroll
    for (int i = 0; i < kChunks; i++) {
        u32x4 raw = {0, 0, 0, 0};
        if (live) raw = *reinterpret_cast<const u32x4 *>(row + 16 * i);
        Chunk<DT>::unpack(raw, f + Chunk<DT>::kElems * i);
    }
}

template <int DT, int kG>   // kG: q heads per kv head the wave carries (group padded to 1, 2, 4, 8)
__global__ __launch_bounds__(64) void decode_attn_gqa_kernel(
    void *__restrict__ out, const void *__restrict__ q, const void *__restrict__ pages,
    const int32_t *__restrict__ kv_indices, const Item *__restrict__ items,
    float *__restrict__ part_o, float *__restrict__ part_ml, int max_slots, int n_qo_heads,
    int n_kv_heads, int head_dim, int page_size, float scale_log2)
{
    typedef LoadElt<DT> L;
    constexpr int kElt = DT == DSKV_F32 ? 4 : 2;
    constexpr int kSub = 4;                     // sub-steps of 4 tokens per iteration: 16 tokens in flight
    const int lane = threadIdx.x, g = lane >> 4, c = lane & 15;
    const int kvh = blockIdx.y;
    const int group = n_qo_heads / n_kv_heads;
    const Item item = items[blockIdx.x];
    const int b = item.b;
    const bool live = c * 8 < head_dim;
    const long row_bytes = (long)n_kv_heads * head_dim * kElt;
    const long half_bytes = row_bytes * page_size;
    const long lane_off = ((long)kvh * head_dim + c * 8) * kElt;
    const char *pool = reinterpret_cast<const char *>(pages);
    const int32_t *table = kv_indices + item.page_begin;

    float qv[kG][8], acc[kG][8], m_run[kG], l_part[kG];
#pragma unroll
    for (int h = 0; h < kG; h++) {
        m_run[h] = kNegBig;
        l_part[h] = 0.f;
#pragma unroll
        for (int i = 0; i < 8; i++) {
            acc[h][i] = 0.f;
            qv[h][i] = (h < group && live)
                           ? L::get(q, ((long)b * n_qo_heads + (long)kvh * group + h) * head_dim + c * 8 + i) * scale_log2
                           : 0.f;
        }
    }
    const int last_tok = item.tok_end - 1;
    // page ids of the lane's tokens of one iteration (past the end: the last token again)
    auto lookup = [&](int t0, long (&page)[kSub]) {
#pragma unroll
        for (int j = 0; j < kSub; j++) page[j] = table[min(t0 + 4 * j + g, last_tok) / page_size];
    };
    long page[kSub];
    if (item.tok_begin < item.tok_end) lookup(item.tok_begin, page);
    for (int t0 = item.tok_begin; t0 < item.tok_end; t0 += 4 * kSub) {
        float kx[kSub][8], vx[kSub][8];
#pragma unroll
        for (int j = 0; j < kSub; j++) {
            const int t = min(t0 + 4 * j + g, last_tok);
            const char *row = pool + page[j] * 2 * half_bytes + (long)(t % page_size) * row_bytes + lane_off;
            load_row8<DT>(row, live, kx[j]);
            load_row8<DT>(row + half_bytes, live, vx[j]);
        }
        if (t0 + 4 * kSub < item.tok_end) lookup(t0 + 4 * kSub, page);   // for the next turn
        float x[kG][kSub], m_new[kG];
#pragma unroll
        for (int h = 0; h < kG; h++) {
            float m = m_run[h];
#pragma unroll
            for (int j = 0; j < kSub; j++) {
                float dot = 0.f;
#pragma unroll
                for (int i = 0; i < 8; i++) dot = __builtin_fmaf(qv[h][i], kx[j][i], dot);
                x[h][j] = t0 + 4 * j + g <= last_tok ? row16_sum(dot) : kNegBig;
                m = fmaxf(m, x[h][j]);
            }
            m_new[h] = quad_rows_max(m);          // over the four token groups
        }
#pragma unroll
        for (int h = 0; h < kG; h++) {
            const float alpha = __builtin_amdgcn_exp2f(m_run[h] - m_new[h]);
            m_run[h] = m_new[h];
            l_part[h] *= alpha;
#pragma unroll
            for (int i = 0; i < 8; i++) acc[h][i] *= alpha;
#pragma unroll
            for (int j = 0; j < kSub; j++) {
                const float p = x[h][j] > kNegBig ? __builtin_amdgcn_exp2f(x[h][j] - m_new[h]) : 0.f;
                l_part[h] += p;
#pragma unroll
                for (int i = 0; i < 8; i++) acc[h][i] = __builtin_fmaf(p, vx[j][i], acc[h][i]);
            }
        }
    }
    // fold the four token groups' partial sums; rows of lanes g == 0 then hold the item's result
#pragma unroll
    for (int h = 0; h < kG; h++) {
        const float l = quad_rows_sum(l_part[h]);
        float o[8];
#pragma unroll
        for (int i = 0; i < 8; i++) o[i] = quad_rows_sum(acc[h][i]);
        if (g != 0 || !live || h >= group) continue;
        const int qh = kvh * group + h;
        if (item.slot < 0) {
            const float inv = l > 0.f ? 1.f / l : 0.f;
#pragma unroll
            for (int i = 0; i < 8; i++) L::put(out, ((long)b * n_qo_heads + qh) * head_dim + c * 8 + i, o[i] * inv);
        } else if (item.slot < max_slots) {
            float *dst = part_o + ((long)item.slot * n_qo_heads + qh) * head_dim + c * 8;
#pragma unroll
            for (int i = 0; i < 8; i++) dst[i] = o[i];
            if (c == 0) {
                float *ml = part_ml + ((long)item.slot * n_qo_heads + qh) * 2;
                ml[0] = m_run[h];
                ml[1] = l;
            }
        }
    }
}

// Combine the partials of split requests.  One workgroup of kWaves wavefronts per
// (request, q head), lane = 2 dims; wave w takes parts w, w + kWaves, ...  Latency-bound,
// so dependent memory round trips are kept few: (m, l) of up to 64 parts are fetched by
// one lane each while the O rows of the first parts are already on their way; weights are
// applied afterwards.  One wave is right for the handful of parts of a batched step; a
// long request cut into hundreds of parts (one request of 32 k tokens: 256) takes eight
// waves, or the merge outlasts the attention pass (34 us against 27 us with one wave, 8 us
// with eight).
template <int DT, int kWaves>
__global__ __launch_bounds__(64 * kWaves) void decode_merge_kernel(
    void *__restrict__ out, const float *__restrict__ part_o, const float *__restrict__ part_ml,
    const int32_t *__restrict__ req_parts, const int32_t *__restrict__ row_map, int max_slots,
    int n_qo_heads, int head_dim)
{
    typedef LoadElt<DT> L;
    constexpr int kBatch = 8;   // O rows in flight per round
    __shared__ float wave_max[kWaves];
    __shared__ float wave_acc[kWaves][4][64];
    __shared__ float wave_l[kWaves];
    const int b = blockIdx.x, qh = blockIdx.y;
    const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
    const int first = req_parts[2 * b], n = req_parts[2 * b + 1];
    if (n <= 0) return;   // written directly by the attention kernel
    // the output row of request b: b itself in a decode batch, an entry of the row map when
    // the requests are the one-row members of a ragged batch
    const long out_row = row_map ? row_map[b] : b;
    if (first < 0 || first + n > max_slots) return;
    const float *ml_base = part_ml + ((long)first * n_qo_heads + qh) * 2;
    const float *o_base = part_o + ((long)first * n_qo_heads + qh) * head_dim;
    const long ml_stride = (long)n_qo_heads * 2, o_stride = (long)n_qo_heads * head_dim;
    // parts of this wave: wave + kWaves * i, i < n_mine
    const int n_mine = (n - wave + kWaves - 1) / kWaves;
    float m = kNegBig;
    for (int i0 = 0; i0 < n_mine; i0 += 64) {
        const int i = i0 + lane;
        float ms = i < n_mine ? ml_base[(long)(wave + kWaves * i) * ml_stride] : kNegBig;
#pragma unroll
        for (int o = 32; o > 0; o >>= 1) ms = fmaxf(ms, __shfl_xor(ms, o));
        m = fmaxf(m, ms);
    }
    if (kWaves > 1) {
        if (lane == 0) wave_max[wave] = m;
        __syncthreads();
#pragma unroll
        for (int w = 0; w < kWaves; w++) m = fmaxf(m, wave_max[w]);
    }
    float acc[4] = {0.f, 0.f, 0.f, 0.f};
    float l = 0.f;
    for (int i0 = 0; i0 < n_mine; i0 += 64) {
        const int i = i0 + lane;
        float w_lane = 0.f, l_lane = 0.f;
        if (i < n_mine) {
            const float *ml = ml_base + (long)(wave + kWaves * i) * ml_stride;
            w_lane = __builtin_amdgcn_exp2f(ml[0] - m);
            l_lane = w_lane * ml[1];
        }
        l += wave_sum(l_lane);
        const int cnt = min(64, n_mine - i0);
        for (int j0 = 0; j0 < cnt; j0 += kBatch) {
            float rows[kBatch][4];
#pragma unroll
            for (int j = 0; j < kBatch; j++) {
                const float *o = o_base + (long)(wave + kWaves * (i0 + min(j0 + j, cnt - 1))) * o_stride;
#pragma unroll
                for (int k = 0; k < 4; k++) {
                    const int d = lane + 64 * k;
                    rows[j][k] = d < head_dim ? o[d] : 0.f;
                }
            }
#pragma unroll
            for (int j = 0; j < kBatch; j++) {
                const float w = (j0 + j < cnt) ? __shfl(w_lane, min(j0 + j, 63)) : 0.f;
#pragma unroll
                for (int k = 0; k < 4; k++) acc[k] += w * rows[j][k];
            }
        }
    }
    if (kWaves > 1) {
#pragma unroll
        for (int k = 0; k < 4; k++) wave_acc[wave][k][lane] = acc[k];
        if (lane == 0) wave_l[wave] = l;
        __syncthreads();
        if (wave != 0) return;
        l = 0.f;
#pragma unroll
        for (int k = 0; k < 4; k++) acc[k] = 0.f;
#pragma unroll
        for (int w = 0; w < kWaves; w++) {
            l += wave_l[w];
#pragma unroll
            for (int k = 0; k < 4; k++) acc[k] += wave_acc[w][k][lane];
        }
    }
    const float inv = l > 0.f ? 1.f / l : 0.f;
#pragma unroll
    for (int k = 0; k < 4; k++) {
        const int d = lane + 64 * k;
        if (d < head_dim) L::put(out, (out_row * n_qo_heads + qh) * head_dim + d, acc[k] * inv);
    }
}

bool decode_mfma_shape(int head_dim, int n_qo_heads, int n_kv_heads, int page_size)
{
    return head_dim == kHeadDim && n_kv_heads > 0 && n_qo_heads % n_kv_heads == 0 &&
           n_qo_heads / n_kv_heads <= 16 && is_pow2(page_size);
}

static bool mfma_path(int dtype, int head_dim, int n_qo_heads, int n_kv_heads)
{
    return (dtype == DSKV_BF16 || dtype == DSKV_F16) && head_dim == kHeadDim &&
           n_qo_heads / n_kv_heads <= 16;
}

// One workgroup per compute unit of the current device (256 on MI355X).
static int default_workgroups()
{
    static int cached = 0;
    if (cached == 0) {
        int dev = 0, cus = 0;
        if (hipGetDevice(&dev) == hipSuccess &&
            hipDeviceGetAttribute(&cus, hipDeviceAttributeMultiprocessorCount, dev) == hipSuccess &&
            cus > 0)
            cached = cus;
        else
            cached = 256;
        (void)hipGetLastError();
    }
    return cached;
}

}  // namespace dskv

// ---------------------------------------------------------------------------
// Host planner
// ---------------------------------------------------------------------------
extern "C" int64_t dskv_decode_plan_bound(int32_t batch, int64_t total_tokens)
{
    using namespace dskv;
    if (batch < 0 || total_tokens < 0) return 0;
    const int64_t max_items = (int64_t)batch + kMaxWorkgroups;
    return kPlanHeaderWords + max_items * kItemWords + (kMaxWorkgroups + 1) + (int64_t)batch * 2;
}

namespace dskv {

// The planner proper.  reqs[i]: tokens, start of the block table and q / output row of
// request i (row i itself for a decode batch).
int plan_decode_rows(const DecodeRow *reqs, int32_t batch, int32_t n_qo_heads, int32_t head_dim,
                     int32_t target_workgroups, int32_t *plan_host, int64_t plan_capacity_words,
                     int32_t *n_items_out, int32_t *n_workgroups_out, int64_t *plan_words_out,
                     int64_t *workspace_bytes_out)
{
    std::vector<int64_t> tiles(batch);
    int64_t total_tiles = 0;
    for (int b = 0; b < batch; b++) {
        DSKV_REQUIRE(reqs[b].len >= 0 && reqs[b].len < (int64_t(1) << 30), "decode_plan: request %d too long", b);
        tiles[b] = (reqs[b].len + kTile - 1) / kTile;
        total_tiles += tiles[b];
    }
    // Workgroup count: one per CU unless told otherwise, fewer when there is so
    // little work that a share would drop below a few tiles.
    int64_t wgs = target_workgroups > 0 ? target_workgroups : default_workgroups();
    wgs = std::min<int64_t>(wgs, kMaxWorkgroups);
    wgs = std::min<int64_t>(wgs, std::max<int64_t>(1, total_tiles / kMinTilesPerWorkgroup));

    // Lay the requests' tiles end to end; workgroup w owns global tiles
    // [w * T / wgs, (w + 1) * T / wgs).  Requests without tokens ride along as
    // empty items (they only write a zero row).
    std::vector<Item> items;
    std::vector<int32_t> wg_ptr(1, 0), req(2 * (size_t)batch, 0);
    int32_t n_slots = 0;
    int64_t w = 0, g0 = 0;                        // current workgroup, global tile index
    auto share_end = [&](int64_t wg) { return (wg + 1) * total_tiles / wgs; };
    for (int b = 0; b < batch; b++) {
        const int64_t len = reqs[b].len;
        if (tiles[b] == 0) {
            items.push_back(Item{reqs[b].row, 0, 0, -1, reqs[b].page_begin, 0, {0, 0}});
            continue;
        }
        const size_t first_item = items.size();
        int64_t done = 0;
        while (done < tiles[b]) {
            while (w + 1 < wgs && g0 >= share_end(w)) {     // this workgroup's share is full
                wg_ptr.push_back((int32_t)items.size());
                w++;
            }
            const int64_t room = (w + 1 < wgs) ? share_end(w) - g0 : tiles[b] - done;
            const int64_t take = std::min(room, tiles[b] - done);
            items.push_back(Item{reqs[b].row, (int32_t)(done * kTile),
                                 (int32_t)std::min<int64_t>((done + take) * kTile, len), -1,
                                 reqs[b].page_begin, done + take == tiles[b], {0, 0}});
            done += take;
            g0 += take;
        }
        const size_t parts = items.size() - first_item;
        if (parts > 1) {
            req[2 * b] = n_slots;
            req[2 * b + 1] = (int32_t)parts;
            for (size_t i = first_item; i < items.size(); i++) items[i].slot = n_slots++;
        }
    }
    while ((int64_t)wg_ptr.size() < wgs + 1) wg_ptr.push_back((int32_t)items.size());
    wg_ptr.back() = (int32_t)items.size();

    const int64_t words = kPlanHeaderWords + (int64_t)items.size() * kItemWords +
                          (int64_t)wg_ptr.size() + (int64_t)batch * 2;
    if (words > plan_capacity_words) {
        set_error("decode_plan: plan needs %lld words, buffer has %lld", (long long)words,
                  (long long)plan_capacity_words);
        return DSKV_E_NOMEM;
    }
    int32_t *p = plan_host;
    *p++ = (int32_t)items.size();
    *p++ = (int32_t)wgs;
    *p++ = n_slots;
    *p++ = batch;
    // the variable-length part (the items) goes last, so that where everything lies
    // depends only on the batch and the number of workgroups: a captured launch
    // stays valid from step to step
    p = std::copy(wg_ptr.begin(), wg_ptr.end(), p);
    p = std::copy(req.begin(), req.end(), p);
    std::copy(reinterpret_cast<const int32_t *>(items.data()),
              reinterpret_cast<const int32_t *>(items.data()) + items.size() * kItemWords, p);
    *n_items_out = (int32_t)items.size();
    *n_workgroups_out = (int32_t)wgs;
    *plan_words_out = words;
    *workspace_bytes_out = (int64_t)n_slots * n_qo_heads * (head_dim + 2) * (int64_t)sizeof(float);
    return 0;
}

}  // namespace dskv

extern "C" int dskv_decode_plan(const int32_t *kv_page_indptr_host,
                                const int32_t *kv_last_page_len_host, int32_t batch,
                                int32_t page_size, int32_t n_qo_heads, int32_t n_kv_heads,
                                int32_t head_dim, int32_t target_workgroups, int32_t *plan_host,
                                int64_t plan_capacity_words, int32_t *n_items_out,
                                int32_t *n_workgroups_out, int64_t *plan_words_out,
                                int64_t *workspace_bytes_out)
{
    using namespace dskv;
    DSKV_REQUIRE(batch >= 0, "decode_plan: negative batch");
    DSKV_REQUIRE(n_items_out && n_workgroups_out && plan_words_out && workspace_bytes_out,
                 "decode_plan: null output pointer");
    DSKV_REQUIRE(page_size > 0 && n_qo_heads > 0 && n_kv_heads > 0 && head_dim > 0 &&
                     n_qo_heads % n_kv_heads == 0,
                 "decode_plan: bad shape (page %d, heads %d/%d, dim %d)", page_size, n_qo_heads,
                 n_kv_heads, head_dim);
    *n_items_out = 0;
    *n_workgroups_out = 0;
    *plan_words_out = 0;
    *workspace_bytes_out = 0;
    if (batch == 0) return 0;
    DSKV_REQUIRE(kv_page_indptr_host && kv_last_page_len_host && plan_host,
                 "decode_plan: null pointer argument");
    std::vector<DecodeRow> reqs(batch);
    for (int b = 0; b < batch; b++) {
        const int64_t np = (int64_t)kv_page_indptr_host[b + 1] - kv_page_indptr_host[b];
        DSKV_REQUIRE(np >= 0, "decode_plan: kv_page_indptr not monotone at %d", b);
        const int32_t last = kv_last_page_len_host[b];
        DSKV_REQUIRE(np == 0 || (last >= 1 && last <= page_size),
                     "decode_plan: kv_last_page_len[%d] = %d outside [1, %d]", b, last, page_size);
        reqs[b] = DecodeRow{np > 0 ? (np - 1) * page_size + last : 0, kv_page_indptr_host[b], b};
    }
    return plan_decode_rows(reqs.data(), batch, n_qo_heads, head_dim, target_workgroups, plan_host,
                            plan_capacity_words, n_items_out, n_workgroups_out, plan_words_out,
                            workspace_bytes_out);
}

namespace dskv {

// k_new / v_new non-null: the fused form, which also writes the step's token of every
// request into its page slot (MFMA path only).
static int decode_attn_impl(void *out, const void *q, const void *pages_layer,
                            const int32_t *kv_page_indices, const int32_t *plan_dev,
                            int32_t n_items, int32_t n_workgroups, void *workspace,
                            int64_t workspace_bytes, int32_t batch, int32_t n_qo_heads,
                            int32_t n_kv_heads, int32_t head_dim, int32_t page_size,
                            float sm_scale, int32_t dtype, int32_t phases, void *stream,
                            const void *k_new, const void *v_new, const float *rope_table,
                            const int32_t *row_map = nullptr)
{
    DSKV_REQUIRE(phases >= 1 && phases <= 3, "decode_attn: phases must be 1, 2 or 3");
    DSKV_REQUIRE(batch >= 0 && n_items >= 0 && n_workgroups >= 0,
                 "decode_attn: negative batch/n_items/n_workgroups");
    if (batch == 0 || n_items == 0) return 0;
    DSKV_REQUIRE(out && q && pages_layer && kv_page_indices && plan_dev,
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
    DSKV_REQUIRE(n_workgroups >= 1 && n_workgroups <= kMaxWorkgroups,
                 "decode_attn: n_workgroups %d outside [1, %d]", n_workgroups, kMaxWorkgroups);
    DSKV_REQUIRE(n_qo_heads <= 65535 && n_kv_heads <= 65535 * kMaxWaves, "decode_attn: too many heads");
    // Partial slots are numbered densely from 0 by the planner.  A plan with
    // n_items items over batch requests has at least n_items - batch + 1 of them
    // when anything is split; the kernels additionally refuse to touch a slot at
    // or beyond max_slots, so an undersized workspace can never be overrun.
    const int64_t slot_bytes = (int64_t)n_qo_heads * (head_dim + 2) * (int64_t)sizeof(float);
    DSKV_REQUIRE(workspace_bytes >= 0, "decode_attn: negative workspace size");
    DSKV_REQUIRE((uintptr_t)workspace % 16 == 0, "decode_attn: the workspace must be 16-byte aligned");
    const int64_t max_slots = std::min<int64_t>(workspace ? workspace_bytes / slot_bytes : 0, 1 << 30);
    DSKV_REQUIRE(n_items == batch || max_slots >= (int64_t)n_items - batch + 1,
                 "decode_attn: workspace (%lld bytes) too small for %d items of %d requests",
                 (long long)workspace_bytes, n_items, batch);

    const int32_t *wg_ptr = plan_dev + kPlanHeaderWords;
    const int32_t *req_parts = wg_ptr + n_workgroups + 1;
    const Item *items = reinterpret_cast<const Item *>(req_parts + 2 * (int64_t)batch);
    // slots are numbered densely from 0, so part_ml can sit after max_slots O blocks
    float *part_o = reinterpret_cast<float *>(workspace);
    float *part_ml = part_o ? part_o + max_slots * n_qo_heads * (int64_t)head_dim : nullptr;
    const float scale_log2 = sm_scale * 1.4426950408889634f;
    hipStream_t s = (hipStream_t)stream;

    DSKV_REQUIRE(!k_new || (mfma_path(dtype, head_dim, n_qo_heads, n_kv_heads) && (phases & 1)),
                 "decode_append_attn: shape or dtype outside the fused kernel (see "
                 "dskv_decode_append_attn_supported); append and attend separately");
    if (!(phases & 1)) {
        // merge only: the split-KV pass of this plan has already been enqueued
    } else if (mfma_path(dtype, head_dim, n_qo_heads, n_kv_heads)) {
        DSKV_REQUIRE(((uintptr_t)out | (uintptr_t)q | (uintptr_t)pages_layer) % 16 == 0,
                     "decode_attn: out/q/pages must be 16-byte aligned");
        DSKV_REQUIRE(is_pow2(page_size), "decode_attn: 16-bit path needs a power-of-two page size, got %d",
                     page_size);
        DSKV_REQUIRE((int64_t)2 * page_size * n_kv_heads * head_dim * 2 < (int64_t(1) << 31),
                     "decode_attn: a page must be smaller than 2 GiB");
        const int waves = std::min(n_kv_heads, kMaxWaves);
        dim3 grid((unsigned)n_workgroups, (unsigned)((n_kv_heads + kMaxWaves - 1) / kMaxWaves));
        dim3 block(64 * waves);
        const int shift = ilog2(page_size);
#define DSKV_LAUNCH_MFMA(DT, COVER)                                                              \
    hipLaunchKernelGGL((decode_attn_mfma_kernel<DT, COVER>), grid, block, 0, s, (uint16_t *)out, \
                       (const uint16_t *)q, (const char *)pages_layer, kv_page_indices, items,   \
                       wg_ptr, part_o, part_ml, (int)max_slots, n_qo_heads, n_kv_heads, shift,   \
                       scale_log2, (const uint16_t *)k_new, (const uint16_t *)v_new, rope_table)
        if (dtype == DSKV_BF16) {
            if (page_size >= kTile) DSKV_LAUNCH_MFMA(DSKV_BF16, 1);
            else if (page_size == 8) DSKV_LAUNCH_MFMA(DSKV_BF16, 2);
            else DSKV_LAUNCH_MFMA(DSKV_BF16, 0);
        } else {
            if (page_size >= kTile) DSKV_LAUNCH_MFMA(DSKV_F16, 1);
            else if (page_size == 8) DSKV_LAUNCH_MFMA(DSKV_F16, 2);
            else DSKV_LAUNCH_MFMA(DSKV_F16, 0);
        }
#undef DSKV_LAUNCH_MFMA
        DSKV_LAUNCH_CHECK("decode_attn_mfma_kernel");
    } else if (n_qo_heads / n_kv_heads <= 8 && head_dim % 8 == 0 && head_dim <= 128 &&
               ((uintptr_t)pages_layer % 16 == 0) && ((int64_t)n_kv_heads * head_dim * (dtype == DSKV_F32 ? 4 : 2)) % 16 == 0) {
        // one wave per (item, kv head) carries the whole GQA group
        const int group = n_qo_heads / n_kv_heads;
        dim3 grid((unsigned)n_items, (unsigned)n_kv_heads);
#define DSKV_LAUNCH_GQA_G(DT, G)                                                                  \
    hipLaunchKernelGGL((decode_attn_gqa_kernel<DT, G>), grid, dim3(64), 0, s, out, q, pages_layer, \
                       kv_page_indices, items, part_o, part_ml, (int)max_slots, n_qo_heads,       \
                       n_kv_heads, head_dim, page_size, scale_log2)
#define DSKV_LAUNCH_GQA(DT)                                  \
    do {                                                     \
        if (group <= 1) DSKV_LAUNCH_GQA_G(DT, 1);            \
        else if (group <= 2) DSKV_LAUNCH_GQA_G(DT, 2);       \
        else if (group <= 4) DSKV_LAUNCH_GQA_G(DT, 4);       \
        else DSKV_LAUNCH_GQA_G(DT, 8);                       \
    } while (0)
        if (dtype == DSKV_F32) DSKV_LAUNCH_GQA(DSKV_F32);
        else if (dtype == DSKV_F16) DSKV_LAUNCH_GQA(DSKV_F16);
        else DSKV_LAUNCH_GQA(DSKV_BF16);
#undef DSKV_LAUNCH_GQA
#undef DSKV_LAUNCH_GQA_G
        DSKV_LAUNCH_CHECK("decode_attn_gqa_kernel");
    } else {
        dim3 grid((unsigned)n_items, (unsigned)n_qo_heads);
#define DSKV_LAUNCH_GEN(DT)                                                                       \
    hipLaunchKernelGGL((decode_attn_generic_kernel<DT>), grid, dim3(64), 0, s, out, q, pages_layer, \
                       kv_page_indices, items, part_o, part_ml, (int)max_slots, n_qo_heads,       \
                       n_kv_heads, head_dim, page_size, scale_log2)
        if (dtype == DSKV_F32) DSKV_LAUNCH_GEN(DSKV_F32);
        else if (dtype == DSKV_F16) DSKV_LAUNCH_GEN(DSKV_F16);
        else DSKV_LAUNCH_GEN(DSKV_BF16);
#undef DSKV_LAUNCH_GEN
        DSKV_LAUNCH_CHECK("decode_attn_generic_kernel");
    }
    if ((phases & 2) && n_items > batch) {
        // many parts per request (long requests, small batch): eight waves share a merge.
        // One wave needs a round trip per 8 parts, eight waves a barrier and a second pass
        // through LDS: they break even at about 32 parts.
        const bool wide = (int64_t)n_items > 32 * (int64_t)batch;
        return launch_partials_merge(out, part_o, part_ml, req_parts, row_map, (int)max_slots, batch,
                                     n_qo_heads, head_dim, dtype, wide, s);
    }
    return 0;
}

int decode_rows_attn(void *out, const void *q, const void *pages_layer,
                     const int32_t *kv_page_indices, const int32_t *plan_dev, int32_t n_items,
                     int32_t n_workgroups, void *workspace, int64_t workspace_bytes, int32_t n_rows,
                     const int32_t *row_map, int32_t n_qo_heads, int32_t n_kv_heads,
                     int32_t head_dim, int32_t page_size, float sm_scale, int32_t dtype,
                     hipStream_t stream)
{
    return decode_attn_impl(out, q, pages_layer, kv_page_indices, plan_dev, n_items, n_workgroups,
                            workspace, workspace_bytes, n_rows, n_qo_heads, n_kv_heads, head_dim,
                            page_size, sm_scale, dtype, 3, stream, nullptr, nullptr, nullptr, row_map);
}

int launch_partials_merge(void *out, const float *part_o, const float *part_ml,
                          const int32_t *row_parts, const int32_t *row_map, int max_slots, int rows,
                          int n_qo_heads, int head_dim, int dtype, bool wide, hipStream_t s)
{
    // rows in a few parts, 16-bit output, head_dim 128: a workgroup per row that requests all
    // parts at once - half the time of a wave per (row, head) on the 512 rows of a chunk, the
    // same 4.7 us on a decode batch's 64 requests in 317 parts (about what any launch that
    // reads what the launch before it wrote takes)
    if (!wide && head_dim == kHeadDim && dtype != DSKV_F32) {
        if (dtype == DSKV_BF16)
            hipLaunchKernelGGL((merge_parts_kernel<DSKV_BF16>), dim3((unsigned)rows), dim3(256), 0, s,
                               (uint16_t *)out, part_o, part_ml, row_parts, row_map, max_slots, n_qo_heads);
        else
            hipLaunchKernelGGL((merge_parts_kernel<DSKV_F16>), dim3((unsigned)rows), dim3(256), 0, s,
                               (uint16_t *)out, part_o, part_ml, row_parts, row_map, max_slots, n_qo_heads);
        DSKV_LAUNCH_CHECK("merge_parts_kernel");
        return 0;
    }
    dim3 grid((unsigned)rows, (unsigned)n_qo_heads);
#define DSKV_LAUNCH_MERGE(DT)                                                                     \
    do {                                                                                          \
        if (wide)                                                                                 \
            hipLaunchKernelGGL((decode_merge_kernel<DT, 8>), grid, dim3(512), 0, s, out, part_o,  \
                               part_ml, row_parts, row_map, max_slots, n_qo_heads, head_dim);     \
        else                                                                                      \
            hipLaunchKernelGGL((decode_merge_kernel<DT, 1>), grid, dim3(64), 0, s, out, part_o,   \
                               part_ml, row_parts, row_map, max_slots, n_qo_heads, head_dim);     \
    } while (0)
    if (dtype == DSKV_F32) DSKV_LAUNCH_MERGE(DSKV_F32);
    else if (dtype == DSKV_F16) DSKV_LAUNCH_MERGE(DSKV_F16);
    else DSKV_LAUNCH_MERGE(DSKV_BF16);
#undef DSKV_LAUNCH_MERGE
    DSKV_LAUNCH_CHECK("decode_merge_kernel");
    return 0;
}

}  // namespace dskv

extern "C" int dskv_decode_attn_phases(void *out, const void *q, const void *pages_layer,
                                       const int32_t *kv_page_indices, const int32_t *plan_dev,
                                       int32_t n_items, int32_t n_workgroups, void *workspace,
                                       int64_t workspace_bytes, int32_t batch, int32_t n_qo_heads,
                                       int32_t n_kv_heads, int32_t head_dim, int32_t page_size,
                                       float sm_scale, int32_t dtype, int32_t phases, void *stream)
{
    return dskv::decode_attn_impl(out, q, pages_layer, kv_page_indices, plan_dev, n_items,
                                  n_workgroups, workspace, workspace_bytes, batch, n_qo_heads,
                                  n_kv_heads, head_dim, page_size, sm_scale, dtype, phases, stream,
                                  nullptr, nullptr, nullptr);
}

extern "C" int dskv_decode_append_attn_supported(int32_t n_qo_heads, int32_t n_kv_heads,
                                                 int32_t head_dim, int32_t page_size, int32_t dtype)
{
    using namespace dskv;
    return n_qo_heads > 0 && n_kv_heads > 0 && n_qo_heads % n_kv_heads == 0 && page_size > 0 &&
           is_pow2(page_size) && mfma_path(dtype, head_dim, n_qo_heads, n_kv_heads);
}

extern "C" int dskv_decode_append_attn(void *out, const void *q, const void *k_new,
                                       const void *v_new, void *pages_layer,
                                       const int32_t *kv_page_indices, const int32_t *plan_dev,
                                       int32_t n_items, int32_t n_workgroups, void *workspace,
                                       int64_t workspace_bytes, int32_t batch, int32_t n_qo_heads,
                                       int32_t n_kv_heads, int32_t head_dim, int32_t page_size,
                                       float sm_scale, int32_t dtype, int32_t phases, void *stream)
{
    using namespace dskv;
    if (batch == 0 || n_items == 0) return 0;
    DSKV_REQUIRE(phases == 1 || phases == 3,
                 "decode_append_attn: the append belongs to the attention pass (phases 1 or 3)");
    DSKV_REQUIRE(k_new && v_new, "decode_append_attn: null k_new / v_new");
    DSKV_REQUIRE(((uintptr_t)k_new | (uintptr_t)v_new) % 16 == 0,
                 "decode_append_attn: k_new / v_new must be 16-byte aligned");
    return decode_attn_impl(out, q, pages_layer, kv_page_indices, plan_dev, n_items, n_workgroups,
                            workspace, workspace_bytes, batch, n_qo_heads, n_kv_heads, head_dim,
                            page_size, sm_scale, dtype, phases, stream, k_new, v_new, nullptr);
}

extern "C" int dskv_decode_rope_append_attn(void *out, const void *q, const void *k_new,
                                            const void *v_new, void *pages_layer,
                                            const int32_t *kv_page_indices, const int32_t *plan_dev,
                                            int32_t n_items, int32_t n_workgroups, void *workspace,
                                            int64_t workspace_bytes, int32_t batch,
                                            int32_t n_qo_heads, int32_t n_kv_heads, int32_t head_dim,
                                            int32_t page_size, float sm_scale, int32_t dtype,
                                            const float *rope_table, int32_t phases, void *stream)
{
    using namespace dskv;
    if (batch == 0 || n_items == 0) return 0;
    DSKV_REQUIRE(phases == 1 || phases == 3,
                 "decode_rope_append_attn: rotation and append belong to the attention pass "
                 "(phases 1 or 3)");
    DSKV_REQUIRE(k_new && v_new && rope_table, "decode_rope_append_attn: null k_new / v_new / table");
    DSKV_REQUIRE(((uintptr_t)k_new | (uintptr_t)v_new | (uintptr_t)rope_table) % 16 == 0,
                 "decode_rope_append_attn: k_new / v_new / table must be 16-byte aligned");
    return decode_attn_impl(out, q, pages_layer, kv_page_indices, plan_dev, n_items, n_workgroups,
                            workspace, workspace_bytes, batch, n_qo_heads, n_kv_heads, head_dim,
                            page_size, sm_scale, dtype, phases, stream, k_new, v_new, rope_table);
}

// ---------------------------------------------------------------------------
// The entry point that allocates nothing: the partial results live in a
// file-scope device array instead of a caller workspace.
// ---------------------------------------------------------------------------
namespace dskv {

constexpr int64_t kStaticScratchBytes = DSKV_DECODE_STATIC_SCRATCH_BYTES;
// Partials (O, m, l) of requests cut by share boundaries.  One copy per GPU, held until the
// process ends.  Never named in a kernel argument or a copy: host code uses the per-device
// address that hipGetSymbolAddress returns (the name is a host-side stand-in only).
static __device__ __align__(256) char scratch[kStaticScratchBytes];

constexpr int kMaxDevices = 64;
static void *g_scratch_ptr[kMaxDevices];   // per device: where that GPU's copy of `scratch` lies
static std::mutex g_scratch_mutex;

// Address of the current device's copy of `scratch`; resolved on the first call per device.
static int static_scratch(void **ptr_out)
{
    int dev = -1;
    DSKV_HIP(hipGetDevice(&dev));
    DSKV_REQUIRE(dev >= 0 && dev < kMaxDevices, "decode_attn_noalloc: device %d outside [0, %d)", dev,
                 kMaxDevices);
    std::lock_guard<std::mutex> lock(g_scratch_mutex);
    if (!g_scratch_ptr[dev]) {
        void *p = nullptr;
        DSKV_HIP(hipGetSymbolAddress(&p, HIP_SYMBOL(scratch)));
        DSKV_REQUIRE(p, "decode_attn_noalloc: the scratch array has no device address");
        g_scratch_ptr[dev] = p;
    }
    *ptr_out = g_scratch_ptr[dev];
    return 0;
}

}  // namespace dskv

extern "C" int64_t dskv_decode_attn_noalloc_max_bytes(void) { return dskv::kStaticScratchBytes; }

extern "C" int dskv_decode_attn_noalloc(void *out, const void *q, const void *pages_layer,
                                        const int32_t *kv_page_indices, const int32_t *plan_dev,
                                        int32_t n_items, int32_t n_workgroups, int32_t batch,
                                        int32_t n_qo_heads, int32_t n_kv_heads, int32_t head_dim,
                                        int32_t page_size, float sm_scale, int32_t dtype,
                                        void *stream)
{
    using namespace dskv;
    if (batch <= 0 || n_items <= 0)
        return decode_attn_impl(out, q, pages_layer, kv_page_indices, plan_dev, n_items,
                                n_workgroups, nullptr, 0, batch, n_qo_heads, n_kv_heads, head_dim,
                                page_size, sm_scale, dtype, 3, stream, nullptr, nullptr, nullptr);
    DSKV_REQUIRE(n_qo_heads > 0 && head_dim > 0, "decode_attn_noalloc: bad shape");
    DSKV_REQUIRE(n_items >= batch, "decode_attn_noalloc: plan has fewer items than requests");
    // Every cut adds one item, and a request cut c times owns c + 1 partial slots: the plan
    // uses at most min(n_items, 2 * (n_items - batch)) slots.
    const int64_t slot_bytes = (int64_t)n_qo_heads * (head_dim + 2) * (int64_t)sizeof(float);
    const int64_t slots = std::min<int64_t>(n_items, 2 * ((int64_t)n_items - batch));
    if (slots * slot_bytes > kStaticScratchBytes) {
        set_error("decode_attn_noalloc: %lld partial slots of %lld bytes exceed the built-in scratch "
                  "of %lld bytes; plan fewer workgroups or pass a workspace to dskv_decode_attn",
                  (long long)slots, (long long)slot_bytes, (long long)kStaticScratchBytes);
        return DSKV_E_NOMEM;
    }
    void *ws = nullptr;
    if (int rc = static_scratch(&ws)) return rc;
    // nothing in the array has to start at zero: every slot the merge pass reads has been
    // written by the attention pass of the same call
    return decode_attn_impl(out, q, pages_layer, kv_page_indices, plan_dev, n_items, n_workgroups,
                            ws, kStaticScratchBytes, batch, n_qo_heads, n_kv_heads, head_dim,
                            page_size, sm_scale, dtype, 3, stream, nullptr, nullptr, nullptr);
}

extern "C" int dskv_decode_attn(void *out, const void *q, const void *pages_layer,
                                const int32_t *kv_page_indices, const int32_t *plan_dev,
                                int32_t n_items, int32_t n_workgroups, void *workspace,
                                int64_t workspace_bytes, int32_t batch, int32_t n_qo_heads,
                                int32_t n_kv_heads, int32_t head_dim, int32_t page_size,
                                float sm_scale, int32_t dtype, void *stream)
{
    return dskv_decode_attn_phases(out, q, pages_layer, kv_page_indices, plan_dev, n_items,
                                   n_workgroups, workspace, workspace_bytes, batch, n_qo_heads,
                                   n_kv_heads, head_dim, page_size, sm_scale, dtype, 3, stream);
}
