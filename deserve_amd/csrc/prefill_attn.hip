// Paged prefill (multi-query) attention with the end-aligned causal mask:
// query i of the n_b new tokens of request b sees kv positions j <= kv_len_b - n_b + i.
//
// Bound: MFMA for long chunks.  Work decomposition: one workgroup = one kv head x
// one tile of query rows; each of its waves owns kColTiles column tiles of 16
// columns, a column being a (query position, q head of the GQA group) pair, so
// the MFMA N dimension is dense.  The workgroup walks the request's K/V in
// blocks of 32 tokens that its waves load together (each a few rows) into a
// double-buffered LDS stage, so a K/V byte crosses the vector memory path once
// per workgroup instead of once per wave: with every wave streaming K/V on its
// own the kernel was bound by that path at a sixth of the MFMA rate.  Per block
// a wave reads K rows from LDS as the A operand of S^T = K.Q^T, keeps S^T's C
// layout as the B operand P^T, and reads V through the transposing LDS read.
//
// Workgroup ids are laid out head-fastest: consecutive ids go to different XCDs,
// so (with 8 kv heads) all query tiles of one kv head share one XCD's L2.
#include "kv_tile.h"

#include <algorithm>

namespace dskv {

#ifndef DSKV_PREFILL_WAVES
#define DSKV_PREFILL_WAVES 8
#endif
#ifndef DSKV_PREFILL_COLTILES
#define DSKV_PREFILL_COLTILES 2
#endif
constexpr int kPrefillWaves = DSKV_PREFILL_WAVES;   // waves per workgroup
constexpr int kColTiles = DSKV_PREFILL_COLTILES;    // column tiles (of 16 columns) per wave
constexpr int kBlock = 2 * kTile;                   // tokens per step
constexpr int kKPitch = 272;                        // bytes per K row in LDS (256 + 16 pad)
constexpr int kStageK = kBlock * kKPitch;
constexpr int kStageBytes = kBlock * (kKPitch + kVPitch);
constexpr int kRowsPerWave = kBlock / kPrefillWaves;   // rows of a block one wave loads
constexpr int kRowGroups = kRowsPerWave / 4;           // in groups of 4 rows (one load each)
static_assert(kRowsPerWave % 4 == 0 && kRowGroups >= 1, "a wave loads whole groups of 4 rows");
// The running maximum of a column is only raised when a block exceeds it by more
// than this (log2 domain): probabilities stay below 2^8, the accumulators are
// rescaled a handful of times per query instead of once per block.
constexpr float kRescaleSlack = 8.f;

struct StageRegs {
    u32x4 k[kRowGroups], v[kRowGroups];
};

template <int DT, bool kRowsSharePage>
__global__ __launch_bounds__(64 * kPrefillWaves) void prefill_attn_mfma_kernel(
    uint16_t *__restrict__ out, const uint16_t *__restrict__ q,
    const int32_t *__restrict__ qo_indptr, const char *__restrict__ pages,
    const int32_t *__restrict__ kv_indices, const int32_t *__restrict__ kv_indptr,
    const int32_t *__restrict__ kv_last, const int32_t *__restrict__ tile_info, int n_qo_heads,
    int n_kv_heads, int page_shift, float scale_log2, int causal)
{
    typedef Elt<DT> E;
    __shared__ __align__(16) char stage[2][kStageBytes];   // per stage: 32 K rows, 32 V rows

    const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
    const int lane = threadIdx.x & 63;
    const int g = lane >> 4;
    const int c = lane & 15;
    const int kvh = blockIdx.x % n_kv_heads;
    const int tile = blockIdx.x / n_kv_heads;
    const int group = n_qo_heads / n_kv_heads;
    const int pos_per_ct = 16 / group;             // query positions per column tile
    const int pos_per_wave = kColTiles * pos_per_ct;

    const int b = tile_info[2 * tile];
    const int q0 = tile_info[2 * tile + 1];        // first query row of the tile within b
    const int q_begin = qo_indptr[b];
    const int n_b = qo_indptr[b + 1] - q_begin;
    const int n_pages = kv_indptr[b + 1] - kv_indptr[b];
    const int kv_len = n_pages > 0 ? ((n_pages - 1) << page_shift) + kv_last[b] : 0;
    const_i32_ptr page_ids = as_const(kv_indices) + kv_indptr[b];
    const int row_bytes = n_kv_heads * kHeadDim * 2;
    const int half_bytes = row_bytes << page_shift;
    const long page_bytes = 2L * half_bytes;
    const int page_mask = (1 << page_shift) - 1;

    // column c of column tile ct: query row wq0 + ct*pos_per_ct + c/group, head c%group
    const int wq0 = q0 + wave * pos_per_wave;
    const int c_pos = c / group;
    const int c_head = c - c_pos * group;
    const bool c_used = c_pos < pos_per_ct;
    int limit[kColTiles];       // number of kv tokens this lane's column may see
    u32x4 qreg[kColTiles][4];
#pragma unroll
    for (int ct = 0; ct < kColTiles; ct++) {
        const int qrow = wq0 + ct * pos_per_ct + c_pos;
        const bool live = c_used && qrow < n_b;
        int lim = causal ? kv_len - n_b + qrow + 1 : kv_len;
        lim = live ? min(max(lim, 0), kv_len) : 0;
        limit[ct] = lim;
        const uint16_t *qrow_p =
            q + ((long)(q_begin + qrow) * n_qo_heads + (long)kvh * group + c_head) * kHeadDim + g * 8;
#pragma unroll
        for (int kk = 0; kk < 4; kk++) {
            u32x4 z = {0, 0, 0, 0};
            qreg[ct][kk] = live ? *reinterpret_cast<const u32x4 *>(qrow_p + kk * 32) : z;
        }
    }
    // Token ranges from scalars only: they steer loops, barriers and page lookups
    // and must be uniform for the compiler too.  The workgroup walks [0, t_end);
    // a wave computes on [0, w_end) and masks from w_mask_from on.
    const int rows_wg = min(kPrefillWaves * pos_per_wave, n_b - q0);          // >= 1 by construction
    const int t_end = min(max(causal ? kv_len - n_b + q0 + rows_wg : kv_len, 0), kv_len);
    const int rows_w = min(pos_per_wave, n_b - wq0);                          // <= 0: idle wave
    const int w_mask_from =
        rows_w > 0 ? min(max(causal ? kv_len - n_b + wq0 + 1 : kv_len, 0), kv_len) : 0;
    const int w_end =
        rows_w > 0 ? min(max(causal ? kv_len - n_b + wq0 + rows_w : kv_len, 0), kv_len) : 0;

    // Start value of a running maximum: far below any scaled score, far above a
    // scaled masked score (kNegBig * scale_log2).
    const float m_floor = 0.5f * kNegBig * scale_log2;
    f32x4 acc[kColTiles][8];
    float m_run[kColTiles], l_run[kColTiles];
#pragma unroll
    for (int ct = 0; ct < kColTiles; ct++) {
        m_run[ct] = m_floor;
        l_run[ct] = 0.f;
#pragma unroll
        for (int dt = 0; dt < 8; dt++) acc[ct][dt] = f32x4{0.f, 0.f, 0.f, 0.f};
    }

    // This wave's share of block [t, t + 32): rows wave*kRowsPerWave .. +kRowsPerWave,
    // lane (g, c) the 16-byte chunk c of row 4i + g.  Rows at or past t_end read as
    // zero (their probabilities are zero, but 0 * garbage is not).
    const int lane_off = g * row_bytes + kvh * (kHeadDim * 2) + c * 16;
    auto load_rows = [&](int t, StageRegs &r) {
#pragma unroll
        for (int i = 0; i < kRowGroups; i++) {
            const int tok0 = t + wave * kRowsPerWave + 4 * i;
            if (kRowsSharePage) {
                // one page holds the 4 rows: descriptors that end after the last
                // valid row make the bounds check free and keep offsets constant
                const int valid = __builtin_amdgcn_readfirstlane(min(max(t_end - tok0, 0), 4));
                const int slot = min(tok0 >> page_shift, max((t_end - 1) >> page_shift, 0));
                const long page = valid > 0 ? page_ids[slot] : 0;   // no lookup past the table
                char *first_row = const_cast<char *>(pages) + page * page_bytes +
                                  (long)(tok0 & page_mask) * row_bytes;
                __amdgpu_buffer_rsrc_t k_rows = __builtin_amdgcn_make_buffer_rsrc(
                    first_row, 0, valid * row_bytes, kBufferFlags);
                __amdgpu_buffer_rsrc_t v_rows = __builtin_amdgcn_make_buffer_rsrc(
                    first_row + half_bytes, 0, valid * row_bytes, kBufferFlags);
                r.k[i] = __builtin_amdgcn_raw_buffer_load_b128(k_rows, lane_off, 0, kLoadCached);
                r.v[i] = __builtin_amdgcn_raw_buffer_load_b128(v_rows, lane_off, 0, kLoadCached);
            } else {
                const int tok = tok0 + g;
                const int tc = min(tok, max(t_end - 1, 0));
                const long page = t_end > 0 ? page_ids[tc >> page_shift] : 0;
                const char *p = pages + page * page_bytes +
                                (long)(tc & page_mask) * row_bytes + (lane_off - g * row_bytes);
                const u32x4 z = {0, 0, 0, 0};
                const u32x4 kk = *reinterpret_cast<const u32x4 *>(p);
                const u32x4 vv = *reinterpret_cast<const u32x4 *>(p + half_bytes);
                r.k[i] = tok < t_end ? kk : z;
                r.v[i] = tok < t_end ? vv : z;
            }
        }
    };
    auto store_rows = [&](char *st, const StageRegs &r) {
#pragma unroll
        for (int i = 0; i < kRowGroups; i++) {
            const int row = wave * kRowsPerWave + 4 * i + g;
            *reinterpret_cast<u32x4 *>(st + row * kKPitch + c * 16) = r.k[i];
            *reinterpret_cast<u32x4 *>(st + kStageK + row * kVPitch + c * 16) = r.v[i];
        }
    };

    // One step: 32 tokens against every column of the wave.  S^T (tokens x columns)
    // comes out of the MFMA with tokens t + 4g + j (low tile) and t + 16 + 4g + j
    // (high tile) in lane (g, c); packed, those eight probabilities are the B
    // operand of a 16x16x32 MFMA whose A operand is the matching eight V rows.
    auto compute_block = [&](int t, const char *st) {
        const bool need_mask = t + kBlock > w_mask_from;   // wave-uniform
        const char *k_lo = st + c * kKPitch + g * 16;
        const char *k_hi = k_lo + kTile * kKPitch;
        const char *v_lo = st + kStageK;
        const char *v_hi = v_lo + kTile * kVPitch;
        u32x4 ka[2][4];
#pragma unroll
        for (int kk = 0; kk < 4; kk++) {
            ka[0][kk] = *reinterpret_cast<const u32x4 *>(k_lo + kk * 64);
            ka[1][kk] = *reinterpret_cast<const u32x4 *>(k_hi + kk * 64);
        }
        u32x4 pb[kColTiles];
#pragma unroll
        for (int ct = 0; ct < kColTiles; ct++) {
            f32x4 s_lo = {0.f, 0.f, 0.f, 0.f}, s_hi = {0.f, 0.f, 0.f, 0.f};
#pragma unroll
            for (int kk = 0; kk < 4; kk++) {
                s_lo = E::mfma_k32(ka[0][kk], qreg[ct][kk], s_lo);
                s_hi = E::mfma_k32(ka[1][kk], qreg[ct][kk], s_hi);
            }
            float x[8];
#pragma unroll
            for (int j = 0; j < 4; j++) {
                x[j] = s_lo[j];
                x[4 + j] = s_hi[j];
            }
            if (need_mask) {
#pragma unroll
                for (int j = 0; j < 4; j++) {
                    if (t + 4 * g + j >= limit[ct]) x[j] = kNegBig;
                    if (t + kTile + 4 * g + j >= limit[ct]) x[4 + j] = kNegBig;
                }
            }
            // scale_log2 > 0: the maximum can be taken before scaling
            float m_blk = fmaxf(fmaxf(fmaxf(x[0], x[1]), fmaxf(x[2], x[3])),
                                fmaxf(fmaxf(x[4], x[5]), fmaxf(x[6], x[7])));
            m_blk = fmaxf(m_blk, __shfl_xor(m_blk, 16));
            m_blk = fmaxf(m_blk, __shfl_xor(m_blk, 32));
            m_blk *= scale_log2;
            if (__builtin_amdgcn_ballot_w64(m_blk > m_run[ct] + kRescaleSlack) != 0) {
                const float m_new = fmaxf(m_run[ct], m_blk);
                const float alpha = __builtin_amdgcn_exp2f(m_run[ct] - m_new);
                m_run[ct] = m_new;
                l_run[ct] *= alpha;
#pragma unroll
                for (int dt = 0; dt < 8; dt++) acc[ct][dt] *= alpha;
            }
            // a masked score is kNegBig and m_run never drops below m_floor, so
            // masked probabilities come out as exp2(-huge) = 0 without a select
            float p[8], p_sum = 0.f;
#pragma unroll
            for (int j = 0; j < 8; j++) {
                p[j] = __builtin_amdgcn_exp2f(__builtin_fmaf(x[j], scale_log2, -m_run[ct]));
                p_sum += p[j];
            }
            l_run[ct] += p_sum;
            pb[ct] = u32x4{E::pack2(p[0], p[1]), E::pack2(p[2], p[3]), E::pack2(p[4], p[5]),
                           E::pack2(p[6], p[7])};
        }
#pragma unroll
        for (int dt = 0; dt < 8; dt++) {
            const u32x2 a_lo = read_v_operand(v_lo, dt, g, c);
            const u32x2 a_hi = read_v_operand(v_hi, dt, g, c);
            const u32x4 va = {a_lo.x, a_lo.y, a_hi.x, a_hi.y};
#pragma unroll
            for (int ct = 0; ct < kColTiles; ct++) acc[ct][dt] = E::mfma_k32(va, pb[ct], acc[ct][dt]);
        }
    };

    // Block n is computed from stage n % 2 while block n + 1 is written to the
    // other stage and block n + 2 is on its way from memory.  One barrier per
    // block: past it every wave has finished reading the stage about to be
    // overwritten and has finished writing the stage about to be read.  Every
    // wave runs every iteration (idle ones only load), so the barriers match.
    StageRegs regs;
    load_rows(0, regs);
    store_rows(stage[0], regs);
    load_rows(kBlock, regs);
    for (int t = 0; t < t_end; t += kBlock) {
        const int cur = (t / kBlock) & 1;
        __syncthreads();
        store_rows(stage[cur ^ 1], regs);
        load_rows(t + 2 * kBlock, regs);
        if (t < w_end) compute_block(t, stage[cur]);
    }

#pragma unroll
    for (int ct = 0; ct < kColTiles; ct++) {
        float l = l_run[ct];
        l += __shfl_xor(l, 16);
        l += __shfl_xor(l, 32);
        const int qrow = wq0 + ct * pos_per_ct + c_pos;
        if (!(c_used && qrow < n_b)) continue;
        const float inv = l > 0.f ? 1.f / l : 0.f;
        uint16_t *o = out + ((long)(q_begin + qrow) * n_qo_heads + (long)kvh * group + c_head) * kHeadDim +
                      4 * g;
#pragma unroll
        for (int dt = 0; dt < 8; dt++) {
            u32x2 w = {E::pack2(acc[ct][dt][0] * inv, acc[ct][dt][1] * inv),
                       E::pack2(acc[ct][dt][2] * inv, acc[ct][dt][3] * inv)};
            *reinterpret_cast<u32x2 *>(o + dt * 16) = w;
        }
    }
}

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
    for (int t = 0; t < limit; t++) {
        const long page = kv_indices[page_begin + t / page_size];
        const long base = page * 2 * half + (long)(t % page_size) * tok_row + (long)kvh * head_dim;
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
    const float inv = l_run > 0.f ? 1.f / l_run : 0.f;
#pragma unroll
    for (int i = 0; i < 4; i++) {
        const int d = lane + 64 * i;
        if (d < head_dim) L::put(out, ((long)row * n_qo_heads + qh) * head_dim + d, acc[i] * inv);
    }
}

static int prefill_rows_per_tile(int n_qo_heads, int n_kv_heads)
{
    const int group = n_qo_heads / n_kv_heads;
    return group <= 16 ? kPrefillWaves * kColTiles * (16 / group) : 1;
}

}  // namespace dskv

extern "C" int64_t dskv_prefill_plan_bound(int32_t batch, int64_t nnz)
{
    if (batch < 0 || nnz < 0) return 0;
    return 2 * ((int64_t)batch + nnz);
}

extern "C" int dskv_prefill_plan(const int32_t *qo_indptr_host, int32_t batch, int32_t n_qo_heads,
                                 int32_t n_kv_heads, int32_t *tile_info_host,
                                 int64_t capacity_words, int32_t *n_tiles_out)
{
    using namespace dskv;
    DSKV_REQUIRE(batch >= 0 && n_tiles_out, "prefill_plan: bad arguments");
    DSKV_REQUIRE(n_qo_heads > 0 && n_kv_heads > 0 && n_qo_heads % n_kv_heads == 0,
                 "prefill_plan: n_qo_heads %d not a multiple of n_kv_heads %d", n_qo_heads,
                 n_kv_heads);
    *n_tiles_out = 0;
    if (batch == 0) return 0;
    DSKV_REQUIRE(qo_indptr_host && tile_info_host, "prefill_plan: null pointer argument");
    const int rows = prefill_rows_per_tile(n_qo_heads, n_kv_heads);
    int64_t n = 0;
    // later query tiles of a request see more keys: emit them first so the
    // longest workgroups start first
    for (int b = 0; b < batch; b++) {
        const int64_t n_b = (int64_t)qo_indptr_host[b + 1] - qo_indptr_host[b];
        DSKV_REQUIRE(n_b >= 0, "prefill_plan: qo_indptr not monotone at %d", b);
        const int64_t tiles = (n_b + rows - 1) / rows;
        if ((n + tiles) * 2 > capacity_words) {
            set_error("prefill_plan: tile list needs more than %lld words", (long long)capacity_words);
            return DSKV_E_NOMEM;
        }
        for (int64_t i = tiles - 1; i >= 0; i--) {
            tile_info_host[2 * n] = b;
            tile_info_host[2 * n + 1] = (int32_t)(i * rows);
            n++;
        }
    }
    DSKV_REQUIRE(n < (int64_t(1) << 31), "prefill_plan: too many tiles");
    *n_tiles_out = (int32_t)n;
    return 0;
}

extern "C" int dskv_prefill_attn(void *out, const void *q, const int32_t *qo_indptr,
                                 const void *pages_layer, const int32_t *kv_page_indices,
                                 const int32_t *kv_page_indptr, const int32_t *kv_last_page_len,
                                 const int32_t *tile_info_dev, int32_t n_tiles, int32_t batch,
                                 int32_t nnz, int32_t n_qo_heads, int32_t n_kv_heads,
                                 int32_t head_dim, int32_t page_size, float sm_scale,
                                 int32_t causal, int32_t dtype, void *stream)
{
    using namespace dskv;
    DSKV_REQUIRE(batch >= 0 && nnz >= 0 && n_tiles >= 0, "prefill_attn: negative sizes");
    if (batch == 0 || nnz == 0) return 0;
    DSKV_REQUIRE(out && q && qo_indptr && pages_layer && kv_page_indices && kv_page_indptr &&
                     kv_last_page_len, "prefill_attn: null pointer argument");
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
    // the MFMA kernel takes maxima before scaling: it needs a positive, sane scale
    const bool mfma = (dtype == DSKV_BF16 || dtype == DSKV_F16) && head_dim == kHeadDim &&
                      n_qo_heads / n_kv_heads <= 16 && scale_log2 > 1e-6f && scale_log2 < 1e6f;
    if (mfma) {
        DSKV_REQUIRE(tile_info_dev && n_tiles > 0, "prefill_attn: missing tile list");
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
                       kv_page_indices, kv_page_indptr, kv_last_page_len, tile_info_dev,        \
                       n_qo_heads, n_kv_heads, shift, scale_log2, causal)
        if (dtype == DSKV_BF16) {
            if (page_size >= 4) DSKV_LAUNCH_PREFILL(DSKV_BF16, true);
            else DSKV_LAUNCH_PREFILL(DSKV_BF16, false);
        } else {
            if (page_size >= 4) DSKV_LAUNCH_PREFILL(DSKV_F16, true);
            else DSKV_LAUNCH_PREFILL(DSKV_F16, false);
        }
#undef DSKV_LAUNCH_PREFILL
        DSKV_LAUNCH_CHECK("prefill_attn_mfma_kernel");
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
