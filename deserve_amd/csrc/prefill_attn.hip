// Paged prefill (multi-query) attention with the end-aligned causal mask:
// query i of the n_b new tokens of request b sees kv positions j <= kv_len_b - n_b + i.
//
// Bound: MFMA for long chunks (every K/V tile is reused by all query columns of
// the wave), L2 for the rest.  Same tile machinery as the decode kernel: K goes
// HBM/L2 -> VGPR -> MFMA A operand, V is transposed through a wave-private LDS
// tile, S^T's C layout is reused as the P^T B operand.
//
// Work decomposition: one wavefront = one kv head x kColTiles column tiles of 16
// columns.  A column is a (query position, q head of the GQA group) pair, so the
// MFMA N dimension is dense: 16/group query positions per column tile.  The 8
// waves of a workgroup are the 8 kv heads of one query tile.
#include "kv_tile.h"

#include <algorithm>

namespace dskv {

#ifndef DSKV_PREFILL_WAVES
#define DSKV_PREFILL_WAVES 8
#endif
#ifndef DSKV_PREFILL_COLTILES
#define DSKV_PREFILL_COLTILES 2
#endif
#ifndef DSKV_PREFILL_STAGES
#define DSKV_PREFILL_STAGES 3
#endif
constexpr int kPrefillStages = DSKV_PREFILL_STAGES; // tiles in flight per wave
constexpr int kPrefillWaves = DSKV_PREFILL_WAVES;   // kv heads per workgroup
constexpr int kColTiles = DSKV_PREFILL_COLTILES;    // column tiles (of 16 columns) per wave

template <int DT, bool kPageCoversTile>
__global__ __launch_bounds__(64 * kPrefillWaves) void prefill_attn_mfma_kernel(
    uint16_t *__restrict__ out, const uint16_t *__restrict__ q,
    const int32_t *__restrict__ qo_indptr, const char *__restrict__ pages,
    const int32_t *__restrict__ kv_indices, const int32_t *__restrict__ kv_indptr,
    const int32_t *__restrict__ kv_last, const int32_t *__restrict__ tile_info, int n_qo_heads,
    int n_kv_heads, int page_shift, float scale_log2, int causal)
{
    typedef Elt<DT> E;
    __shared__ __align__(16) char v_lds[kPrefillWaves][kVTileBytes];

    const int wave = threadIdx.x >> 6;
    const int lane = threadIdx.x & 63;
    const int g = lane >> 4;
    const int c = lane & 15;
    const int kvh = blockIdx.y * kPrefillWaves + wave;
    if (kvh >= n_kv_heads) return;
    const int group = n_qo_heads / n_kv_heads;
    const int pos_per_ct = 16 / group;            // query positions per column tile

    const int b = tile_info[2 * blockIdx.x];
    const int q0 = tile_info[2 * blockIdx.x + 1];   // first query row of the tile within b
    const int q_begin = qo_indptr[b];
    const int n_b = qo_indptr[b + 1] - q_begin;
    const int n_pages = kv_indptr[b + 1] - kv_indptr[b];
    const int kv_len = n_pages > 0 ? ((n_pages - 1) << page_shift) + kv_last[b] : 0;

    KvView kv;
    kv.pages = pages;
    kv.page_ids = as_const(kv_indices) + kv_indptr[b];
    kv.page_shift = page_shift;
    kv.row_bytes = n_kv_heads * kHeadDim * 2;
    kv.half_bytes = kv.row_bytes << page_shift;
    kv.page_bytes = 2L * kv.half_bytes;
    kv.head_off = kvh * (kHeadDim * 2);

    // column c of column tile ct: query row q0 + ct*pos_per_ct + c/group, head c%group
    const int c_pos = c / group;
    const int c_head = c - c_pos * group;
    const bool c_used = c_pos < pos_per_ct;
    int limit[kColTiles];       // number of kv tokens this lane's column may see
    u32x4 qreg[kColTiles][4];
#pragma unroll
    for (int ct = 0; ct < kColTiles; ct++) {
        const int qrow = q0 + ct * pos_per_ct + c_pos;
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
    // Extremes over the tile's live query rows, from scalars only: they steer the
    // loop and the page lookups and must stay wave-uniform for the compiler too.
    const int rows_live = min(kColTiles * pos_per_ct, n_b - q0);            // >= 1 by construction
    const int limit_min = min(max(causal ? kv_len - n_b + q0 + 1 : kv_len, 0), kv_len);
    const int t_end = min(max(causal ? kv_len - n_b + q0 + rows_live : kv_len, 0), kv_len);

    f32x4 acc[kColTiles][8];
    float m_run[kColTiles], l_run[kColTiles];
#pragma unroll
    for (int ct = 0; ct < kColTiles; ct++) {
        m_run[ct] = kNegBig;
        l_run[ct] = 0.f;
#pragma unroll
        for (int dt = 0; dt < 8; dt++) acc[ct][dt] = f32x4{0.f, 0.f, 0.f, 0.f};
    }
    char *lds = v_lds[wave];

    auto compute_tile = [&](int t, const TileRegs &r) {
        stage_v_tile<kPageCoversTile>(lds, r, t, t_end, g, c);
        const bool need_mask = t + kTile > limit_min;   // wave-uniform
        u32x2 pb[kColTiles];
        float alpha[kColTiles];
#pragma unroll
        for (int ct = 0; ct < kColTiles; ct++) {
            f32x4 s = {0.f, 0.f, 0.f, 0.f};
#pragma unroll
            for (int kk = 0; kk < 4; kk++) s = E::mfma_k32(r.k[kk], qreg[ct][kk], s);
            float x[4];
#pragma unroll
            for (int j = 0; j < 4; j++) {
                x[j] = s[j] * scale_log2;
                if (need_mask && t + g + 4 * j >= limit[ct]) x[j] = kNegBig;
            }
            float m_tile = fmaxf(fmaxf(x[0], x[1]), fmaxf(x[2], x[3]));
            m_tile = fmaxf(m_tile, __shfl_xor(m_tile, 16));
            m_tile = fmaxf(m_tile, __shfl_xor(m_tile, 32));
            const float m_new = fmaxf(m_run[ct], m_tile);
            alpha[ct] = __builtin_amdgcn_exp2f(m_run[ct] - m_new);
            m_run[ct] = m_new;
            float p[4], p_sum = 0.f;
#pragma unroll
            for (int j = 0; j < 4; j++) {
                // a fully masked column keeps m at kNegBig: force p to 0 there
                p[j] = x[j] > kNegBig ? __builtin_amdgcn_exp2f(x[j] - m_new) : 0.f;
                p_sum += p[j];
            }
            l_run[ct] = l_run[ct] * alpha[ct] + p_sum;
            pb[ct] = u32x2{E::pack2(p[0], p[1]), E::pack2(p[2], p[3])};
        }
#pragma unroll
        for (int dt = 0; dt < 8; dt++) {
            const u32x2 va = read_v_operand(lds, dt, g, c);
#pragma unroll
            for (int ct = 0; ct < kColTiles; ct++)
                acc[ct][dt] = E::mfma_k16(va, pb[ct], acc[ct][dt] * alpha[ct]);
        }
        __builtin_amdgcn_wave_barrier();
    };

    // A ring of kPrefillStages tile buffers.  The steady-state body is straight
    // line (loads are unconditional; a tile past the end fetches nothing in the
    // page-descriptor path), so the compiler waits only for the tile it consumes.
    TileRegs ring[kPrefillStages];
    int t = 0;
#pragma unroll
    for (int s = 0; s < kPrefillStages; s++)
        load_kv_tile<kPageCoversTile, kLoadCached>(kv, s * kTile, t_end, g, c, ring[s]);
    while (t + (kPrefillStages - 1) * kTile < t_end) {
#pragma unroll
        for (int s = 0; s < kPrefillStages; s++) {
            compute_tile(t + s * kTile, ring[s]);
            __builtin_amdgcn_sched_barrier(0);
            load_kv_tile<kPageCoversTile, kLoadCached>(kv, t + (s + kPrefillStages) * kTile, t_end, g,
                                                        c, ring[s]);
            __builtin_amdgcn_sched_barrier(0);
        }
        t += kPrefillStages * kTile;
    }
#pragma unroll
    for (int s = 0; s < kPrefillStages - 1; s++)
        if (t + s * kTile < t_end) compute_tile(t + s * kTile, ring[s]);

#pragma unroll
    for (int ct = 0; ct < kColTiles; ct++) {
        float l = l_run[ct];
        l += __shfl_xor(l, 16);
        l += __shfl_xor(l, 32);
        const int qrow = q0 + ct * pos_per_ct + c_pos;
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
    return group <= 16 ? kColTiles * (16 / group) : 1;
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
    const bool mfma = (dtype == DSKV_BF16 || dtype == DSKV_F16) && head_dim == kHeadDim &&
                      n_qo_heads / n_kv_heads <= 16;
    if (mfma) {
        DSKV_REQUIRE(tile_info_dev && n_tiles > 0, "prefill_attn: missing tile list");
        DSKV_REQUIRE(((uintptr_t)out | (uintptr_t)q | (uintptr_t)pages_layer) % 16 == 0,
                     "prefill_attn: out/q/pages must be 16-byte aligned");
        DSKV_REQUIRE(is_pow2(page_size),
                     "prefill_attn: 16-bit path needs a power-of-two page size, got %d", page_size);
        const int waves = std::min(n_kv_heads, kPrefillWaves);
        dim3 grid((unsigned)n_tiles, (unsigned)((n_kv_heads + kPrefillWaves - 1) / kPrefillWaves));
        dim3 block(64 * waves);
        const int shift = ilog2(page_size);
#define DSKV_LAUNCH_PREFILL(DT, COVER)                                                          \
    hipLaunchKernelGGL((prefill_attn_mfma_kernel<DT, COVER>), grid, block, 0, s, (uint16_t *)out, \
                       (const uint16_t *)q, qo_indptr, (const char *)pages_layer,               \
                       kv_page_indices, kv_page_indptr, kv_last_page_len, tile_info_dev,        \
                       n_qo_heads, n_kv_heads, shift, scale_log2, causal)
        if (dtype == DSKV_BF16) {
            if (page_size >= kTile) DSKV_LAUNCH_PREFILL(DSKV_BF16, true);
            else DSKV_LAUNCH_PREFILL(DSKV_BF16, false);
        } else {
            if (page_size >= kTile) DSKV_LAUNCH_PREFILL(DSKV_F16, true);
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
