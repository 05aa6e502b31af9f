// The 16-bit paged prefill attention kernel (head_dim 128): see prefill_attn.hip for the
// decomposition.  Kept in a header because two launches use its body: the stand-alone one
// (workgroups of eight waves) and the mixed launch of prefill_attn.hip, whose four-wave
// workgroups share their compute units with decode workgroups.
#pragma once

#include "kv_tile.h"

namespace dskv {

#ifndef DSKV_PREFILL_COLTILES
#define DSKV_PREFILL_COLTILES 1
#endif
constexpr int kPrefillWaves = 8;                    // waves per workgroup of the stand-alone launch
constexpr int kPrefillWavesShared = 4;              // ... of the launch whose workgroups share a CU with decode workgroups
constexpr int kColTiles = DSKV_PREFILL_COLTILES;    // column tiles (of 32 columns) per wave
constexpr int kWaveCols = 32 * kColTiles;           // columns per wave
constexpr int kBlock = 32;                          // tokens per step (one MFMA tile)
constexpr int kTileWords = 6;                       // plan entry: request, first row, block range, part, first slot
// LDS layout of a 32-token block of K (or V) rows of one kv head: eight regions of four rows.
// A region is what one load instruction delivers: 64 lanes x 16 bytes, lane p at byte 16 p.
// Lane p = 4 c + rho fetches the 16-byte chunk c of row rho, so the region holds its rows
// interleaved chunk by chunk ((4 c + rho) * 16); regions are 1088 bytes apart (64 bytes of
// padding).  Operand reads are free of bank conflicts: the 16 lanes of a K-operand read (16
// token rows, one chunk) and the 32 lanes of a transposing V read (4 rows x 4 chunks of a
// region) fall on 16 different 16-byte bank groups each.
constexpr int kRegionBytes = 1088;
constexpr int kStageBytes = (kBlock / 4) * kRegionBytes;
// The running maximum of a column is only raised when a block exceeds it by more
// than this (log2 domain): probabilities stay below 2^8, the accumulators are
// rescaled a handful of times per query instead of once per block.
constexpr float kRescaleSlack = 8.f;
#ifndef DSKV_PREFILL_KPREFETCH
#define DSKV_PREFILL_KPREFETCH 1   // K operands of the next iteration read before its barrier (direct path)
#endif
#ifndef DSKV_PREFILL_KREADS_FIRST
#define DSKV_PREFILL_KREADS_FIRST 0
#endif
#ifndef DSKV_PREFILL_SUM_ON_MFMA
#define DSKV_PREFILL_SUM_ON_MFMA 0
#endif
constexpr bool kSumOnMfma = DSKV_PREFILL_SUM_ON_MFMA;   // row sums of P by the matrix pipeline

// Lane roles of the 32x32x16 MFMA, with h = lane / 32 and r = lane % 32:
//   A operand: row r, k = 8h .. 8h+7.   B operand: column r, k = 8h .. 8h+7.
//   C/D: column r, rows 8i + 4h + j in register 4i + j (i, j = 0..3).
// LDS of one workgroup: four stages of K rows, then four of V rows.
constexpr int kPrefillLdsBytes = 8 * kStageBytes;
struct LdsStages {
    char *base;
    __device__ __forceinline__ char *operator[](int i) const { return base + i * kStageBytes; }
};

// The kernel's body for workgroup `wg` of kWaves waves (a tile of kWaves * 32 / group query
// rows of one kv head); `lds`: kPrefillLdsBytes of the workgroup's LDS.  A function, so that
// one launch can hold workgroups of this kind next to workgroups of another.
template <int DT, bool kRowsSharePage, int kWaves>
__device__ __forceinline__ void prefill_attn_body(
    char *lds_base, int wg, uint16_t *__restrict__ out, const uint16_t *__restrict__ q,
    const int32_t *__restrict__ qo_indptr, const char *__restrict__ pages,
    const int32_t *__restrict__ kv_indices, const int32_t *__restrict__ kv_indptr,
    const int32_t *__restrict__ kv_last, const int32_t *__restrict__ tile_info, int n_qo_heads,
    int n_kv_heads, int page_shift, float scale_log2, int causal,
    float *__restrict__ part_o, float *__restrict__ part_ml, int max_slots)
{
    typedef Elt<DT> E;
    constexpr int kRowsPerWave = kBlock / kWaves;   // rows of a block one wave loads
    constexpr int kRowGroups = kRowsPerWave / 4;    // in groups of 4 rows (one load each)
    static_assert(kRowsPerWave % 4 == 0 && kRowGroups >= 1, "a wave loads whole groups of 4 rows");
    const LdsStages k_stage{lds_base}, v_stage{lds_base + 4 * kStageBytes};

    const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
    const int lane = threadIdx.x & 63;
    const int g = lane >> 4;     // row group / chunk roles of the K/V row movement
    const int c = lane & 15;
    const int h = lane >> 5;     // MFMA roles
    const int r = lane & 31;
    const int kvh = wg % n_kv_heads;
    const int tile = wg / n_kv_heads;
    const int group = n_qo_heads / n_kv_heads;
    const int pos_per_wave = kWaveCols / group;    // query positions per wave

    // plan entry: request, first query row of the tile within it, and the 32-token blocks
    // [blk_begin, blk_end) of the request's K/V that this workgroup walks.  Word 4 is -1 for a
    // tile that walks all of its blocks and writes its output rows itself; for a tile cut
    // into parts (blk_begin a multiple of four) it is part | parts << 8, and word 5 the
    // partial slot of the tile's first row, part 0: row r of the tile, part s, leaves
    // (maximum, sum, unnormalised O) in slot first + (r - q0) * parts + s.
    const const_i32_ptr entry = as_const(tile_info) + (long)tile * kTileWords;
    const int b = entry[0];
    const int q0 = entry[1];
    const int blk_begin = entry[2];
    const int kv_cap_blocks = entry[3];
    const int part_word = entry[4];
    const bool partial = part_word >= 0;
    const int split = part_word & 0xff, tile_parts = part_word >> 8;
    const int first_slot = entry[5];
    const int q_begin = qo_indptr[b];
    const int n_b = qo_indptr[b + 1] - q_begin;
    const int n_pages = kv_indptr[b + 1] - kv_indptr[b];
    const int kv_len = n_pages > 0 ? ((n_pages - 1) << page_shift) + kv_last[b] : 0;
    // tokens this workgroup may look at end here: the request's end, or the end of its part
    const int kv_cap = min(kv_len, kv_cap_blocks < (1 << 25) ? kv_cap_blocks * kBlock : kv_len);
    const_i32_ptr page_ids = as_const(kv_indices) + kv_indptr[b];
    const int row_bytes = n_kv_heads * kHeadDim * 2;
    const int half_bytes = row_bytes << page_shift;
    const long page_bytes = 2L * half_bytes;
    const int page_mask = (1 << page_shift) - 1;

    // column r of column tile ct: query row wq0 + (32 ct + r)/group, head (32 ct + r)%group
    const int wq0 = q0 + wave * pos_per_wave;
    int qrow[kColTiles], c_head[kColTiles], limit[kColTiles];   // limit: kv tokens the column may see
    bool live[kColTiles];
    u32x4 qreg[kColTiles][8];     // dims 16*ks + 8h .. +7 of the column's query
#pragma unroll
    for (int ct = 0; ct < kColTiles; ct++) {
        const int col = 32 * ct + r;
        const int c_pos = col / group;
        c_head[ct] = col - c_pos * group;
        qrow[ct] = wq0 + c_pos;
        live[ct] = c_pos < pos_per_wave && qrow[ct] < n_b;
        const int lim = causal ? kv_len - n_b + qrow[ct] + 1 : kv_len;
        limit[ct] = live[ct] ? min(max(lim, 0), kv_cap) : 0;
        const uint16_t *qrow_p =
            q + ((long)(q_begin + qrow[ct]) * n_qo_heads + (long)kvh * group + c_head[ct]) * kHeadDim + h * 8;
#pragma unroll
        for (int ks = 0; ks < 8; ks++) {
            u32x4 z = {0, 0, 0, 0};
            qreg[ct][ks] = live[ct] ? *reinterpret_cast<const u32x4 *>(qrow_p + ks * 16) : z;
        }
    }
    // Token ranges from scalars only: they steer loops, barriers and page lookups
    // and must be uniform for the compiler too.  The workgroup walks [0, t_end);
    // a wave computes on [0, w_end) and masks from w_mask_from on.
    const int rows_wg = min(kWaves * pos_per_wave, n_b - q0);          // >= 1 by construction
    const int t_first = blk_begin * kBlock;                                   // the walk starts here
    const int t_end = min(max(causal ? kv_len - n_b + q0 + rows_wg : kv_len, 0), kv_cap);
    const int rows_w = min(pos_per_wave, n_b - wq0);                          // <= 0: idle wave
    const int w_mask_from =
        rows_w > 0 ? min(max(causal ? kv_len - n_b + wq0 + 1 : kv_len, 0), kv_cap) : 0;
    int w_end = rows_w > 0 ? min(max(causal ? kv_len - n_b + wq0 + rows_w : kv_len, 0), kv_cap) : 0;
    if (w_end <= t_first) w_end = 0;   // nothing of this part is visible to the wave's rows: idle

    const int n_blocks = (t_end + kBlock - 1) / kBlock;
    // Start value of the running maximum: far below any scaled score, far above a
    // scaled masked score (kNegBig * scale_log2).
    float m_run[kColTiles];
    f32x16 acc[kColTiles][4];     // O^T: dims 32*dt + 8i + 4h + j of column r in acc[ct][dt][4i + j]
    // Row sums of P, optionally on the matrix pipeline: ones(32 x tokens) . P^T - every
    // register of a lane then holds the sum of its column r over the tokens multiplied so
    // far.  It takes 16 additions per block off the vector pipeline and adds two MFMAs;
    // measured on MI355X the kernel takes the same time either way, so the default keeps the
    // sums on the vector pipeline (fewer registers, less matrix work).
    f32x16 l_acc[kColTiles];
    float l_run[kColTiles];       // the same sums kept by the vector pipeline (kSumOnMfma off)
    u32x4 pb[kColTiles][2];       // packed probabilities of the previous block, per k-step
#pragma unroll
    for (int ct = 0; ct < kColTiles; ct++) {
        m_run[ct] = 0.5f * kNegBig * scale_log2;
        l_run[ct] = 0.f;
#pragma unroll
        for (int v = 0; v < 16; v++) l_acc[ct][v] = 0.f;
#pragma unroll
        for (int dt = 0; dt < 4; dt++)
#pragma unroll
            for (int v = 0; v < 16; v++) acc[ct][dt][v] = 0.f;
        pb[ct][0] = pb[ct][1] = u32x4{0, 0, 0, 0};
    }
    const uint32_t one2 = E::pack2(1.f, 1.f);
    const u32x4 ones = {one2, one2, one2, one2};

    // A tile cut into parts: every part leaves (max, sum, unnormalised O) of its rows in the
    // workspace (O blocks of all slots, then their (max, sum) pairs); a part that sees nothing
    // leaves zeros and a maximum below any real one.
    auto store_partial = [&](int ct, float m, float l) {
        const long slot = (long)first_slot + (long)(qrow[ct] - q0) * tile_parts + split;
        if (slot >= max_slots) return;   // a slot beyond the workspace is never written
        const long qh = (long)kvh * group + c_head[ct];
        float *o = part_o + (slot * n_qo_heads + qh) * kHeadDim + 4 * h;
#pragma unroll
        for (int dt = 0; dt < 4; dt++)
#pragma unroll
            for (int i = 0; i < 4; i++)
                *reinterpret_cast<f32x4 *>(o + dt * 32 + 8 * i) =
                    f32x4{acc[ct][dt][4 * i], acc[ct][dt][4 * i + 1], acc[ct][dt][4 * i + 2], acc[ct][dt][4 * i + 3]};
        if (h == 0) {
            float *ml = part_ml + (slot * n_qo_heads + qh) * 2;
            ml[0] = m;
            ml[1] = l;
        }
    };
    // No kv token of this part visible to any row of the tile: the output rows are zero
    // (or the part is empty).  Uniform over the workgroup, and before the first barrier.
    if (t_end <= t_first) {
#pragma unroll
        for (int ct = 0; ct < kColTiles; ct++) {
            if (!live[ct]) continue;
            if (partial) {
                store_partial(ct, m_run[ct], 0.f);
                continue;
            }
            uint16_t *o = out + ((long)(q_begin + qrow[ct]) * n_qo_heads + (long)kvh * group + c_head[ct]) * kHeadDim +
                          4 * h;
#pragma unroll
            for (int i = 0; i < 16; i++) *reinterpret_cast<u32x2 *>(o + 8 * i) = u32x2{0, 0};
        }
        return;
    }

    // This wave's share of the K (or V) rows of block blk: rows wave*kRowsPerWave .. +kRowsPerWave,
    // in groups of four (one region each).  Rows at or past t_end arrive as zeros (their
    // probabilities are zero, but 0 * garbage is not).
    //
    // Pages of at least four tokens (kRowsSharePage): the rows go from memory straight into
    // their LDS region (buffer_load ... lds: lane p's 16 bytes land at region + 16 p, lanes
    // beyond the descriptor's end write zeros), addressed through descriptors that end after
    // the group's last valid row.  Page ids are looked up with a vector load (every lane the
    // same entry; entries past the table read as page 0, whose descriptor is then empty).
    // Smaller pages: every lane resolves its own page, the rows pass through registers.
    typedef __attribute__((address_space(3))) void *lds_ptr;
    const int direct_off = (lane & 3) * row_bytes + kvh * (kHeadDim * 2) + (lane >> 2) * 16;
    const int lane_off = kvh * (kHeadDim * 2) + c * 16;
    // Page ids come through scalar loads (block-table entries past the table are clamped to
    // its last one; their descriptors are empty).  They are consumed at the end of an
    // iteration, when every LDS read of the iteration has been waited for anyway (scalar
    // loads and LDS reads share a counter).
    const int last_entry = max(n_pages - 1, 0);
    auto lookup_pages = [&](int blk, int(&pg)[kRowGroups]) {
        if (!kRowsSharePage) return;
#pragma unroll
        for (int i = 0; i < kRowGroups; i++) {
            const int tok0 = blk * kBlock + wave * kRowsPerWave + 4 * i;
            pg[i] = page_ids[min(tok0 >> page_shift, last_entry)];
        }
    };
    // The descriptors of the rows of block blk (scalar work: page id into an SGPR, base
    // address, valid bytes), prepared an iteration before the loads are issued so that it
    // runs in the shadow of that iteration's MFMAs.
    struct RowDesc {
        u32x4 k[kRowGroups], v[kRowGroups];   // raw buffer descriptors: base, base >> 32, bytes, flags
    };
    auto make_desc = [&](const char *base, int bytes) {
        const uint64_t a = (uint64_t)base;
        return u32x4{(uint32_t)__builtin_amdgcn_readfirstlane((int)(uint32_t)a),
                     (uint32_t)__builtin_amdgcn_readfirstlane((int)((uint32_t)(a >> 32) & 0xFFFFu)),
                     (uint32_t)__builtin_amdgcn_readfirstlane(bytes), (uint32_t)kBufferFlags};
    };
    auto prepare_rows = [&](int blk, const int(&pg)[kRowGroups], RowDesc &d) {
        if (!kRowsSharePage) return;
#pragma unroll
        for (int i = 0; i < kRowGroups; i++) {
            const int tok0 = blk * kBlock + wave * kRowsPerWave + 4 * i;
            // one page holds the 4 rows: descriptors that end after the last
            // valid row make the bounds check free and keep offsets constant
            // (the clamp is selected as a vector instruction: back to a scalar register, the
            // descriptor words must live in SGPRs)
            const int valid = __builtin_amdgcn_readfirstlane(min(max(t_end - tok0, 0), 4));
            const char *first_row = pages + (long)pg[i] * page_bytes + (long)(tok0 & page_mask) * row_bytes;
            d.k[i] = make_desc(first_row, valid * row_bytes);
            d.v[i] = make_desc(first_row + half_bytes, valid * row_bytes);
        }
    };
    auto region_of = [&](char *stage, int i) { return stage + (wave * kRowGroups + i) * kRegionBytes; };
    // Written out as instructions: through the compiler's builtin every later LDS read waits
    // for ALL of these loads (it cannot tell which region a read touches), which would undo
    // requesting them three iterations early.  What it does not know it does not wait for:
    // the waits for these loads are the explicit ones below.
    // M0 is on the clobber list (the compiler reserves it, sets it itself before the few
    // instructions that read it, and must not assume that such a setting survives this one).
#pragma clang diagnostic push
#pragma clang diagnostic ignored "-Winline-asm"
    auto load_direct = [&](const u32x4(&rows)[kRowGroups], char *stage) {
#pragma unroll
        for (int i = 0; i < kRowGroups; i++) {
            const uint32_t lds_addr = (uint32_t)(uintptr_t)(lds_ptr)region_of(stage, i);
            asm volatile("s_mov_b32 m0, %0\n\tbuffer_load_dwordx4 %1, %2, 0 offen lds"
                         :
                         : "s"(lds_addr), "v"(direct_off), "s"(rows[i])
                         : "memory", "m0");
        }
    };
#pragma clang diagnostic pop
    auto load_rows = [&](int blk, u32x4(&k_rows)[kRowGroups], u32x4(&v_rows)[kRowGroups]) {
#pragma unroll
        for (int i = 0; i < kRowGroups; i++) {
            const int tok = blk * kBlock + wave * kRowsPerWave + 4 * i + g;
            const int tc = max(min(tok, t_end - 1), 0);
            const char *p = pages + page_ids[tc >> page_shift] * page_bytes +
                            (long)(tc & page_mask) * row_bytes + lane_off;
            const u32x4 z = {0, 0, 0, 0};
            const u32x4 got_k = *reinterpret_cast<const u32x4 *>(p);
            const u32x4 got_v = *reinterpret_cast<const u32x4 *>(p + half_bytes);
            k_rows[i] = tok < t_end ? got_k : z;
            v_rows[i] = tok < t_end ? got_v : z;
        }
    };
    auto store_rows = [&](char *stage, const u32x4(&rows)[kRowGroups]) {   // lane (g, c): chunk c of row g
#pragma unroll
        for (int i = 0; i < kRowGroups; i++)
            *reinterpret_cast<u32x4 *>(region_of(stage, i) + (c * 4 + g) * 16) = rows[i];
    };
    // Waits until at most n of this wave's vector-memory operations are outstanding (the
    // other counters of s_waitcnt left at "do not wait").
#define DSKV_WAIT_VMEM(n) __builtin_amdgcn_s_waitcnt(((n) & 15) | 0x70 | 0xF00 | (((n) >> 4) << 14))

    // Two score buffers that the iterations use in turn (S(m) is still being turned into
    // P(m) while S(m+1) is computed): the loop is unrolled with static phases, so which
    // buffer is which is known at compile time and no copy is needed.
    f32x16 xs[2][kColTiles];
    // K rows of a block as MFMA operands: token r, dims 16*ks + 8h .. +7.  With the prefetch
    // the operands of K(m+1) are read at the end of iteration m-1 (the block has been published
    // by barrier m-1 then), into the buffer that iteration m's scores use; without, all use [0].
    constexpr bool kKPrefetch = DSKV_PREFILL_KPREFETCH && kRowsSharePage;
    u32x4 ka[kKPrefetch ? 2 : 1][8];
    auto read_k_operands = [&](const char *kst, int kb = 0) {
        // token r = row r & 3 of region r >> 2; chunk 2 ks + h
        const char *k_rows = kst + (r >> 2) * kRegionBytes + h * 64 + (r & 3) * 16;
#pragma unroll
        for (int ks = 0; ks < 8; ks++) ka[kb][ks] = *reinterpret_cast<const u32x4 *>(k_rows + ks * 128);
    };
    auto scores = [&](int buf, int kb = 0) {
#pragma unroll
        for (int ct = 0; ct < kColTiles; ct++)
#pragma unroll
            for (int v = 0; v < 16; v++) xs[buf][ct][v] = 0.f;
#pragma unroll
        for (int ks = 0; ks < 8; ks++)
#pragma unroll
            for (int ct = 0; ct < kColTiles; ct++)
                xs[buf][ct] = E::mfma_32x32(ka[kb][ks], qreg[ct][ks], xs[buf][ct]);
    };
    // Masks block blk's scores (needed from w_mask_from on).  The empty volatile statement
    // keeps this a branch: the compiler otherwise turns it into selects that every block
    // pays for (48 vector instructions), and only the blocks on the diagonal need it.
    auto mask_scores = [&](int blk, int buf) {
        const int t = blk * kBlock;
#pragma unroll
        for (int ct = 0; ct < kColTiles; ct++) {
            asm volatile("" : "+v"(xs[buf][ct]));   // (re)defined here: the selects cannot leave the branch
#pragma unroll
            for (int v = 0; v < 16; v++)
                if (t + 8 * (v >> 2) + 4 * h + (v & 3) >= limit[ct]) xs[buf][ct][v] = kNegBig;
        }
    };
    // Column maximum of the block in xs[buf], and whether the running maximum has to be
    // raised before the block's exponentials.
    float m_blk[kColTiles];
    bool raise = false;
    auto block_max = [&](int buf) {
        raise = false;
#pragma unroll
        for (int ct = 0; ct < kColTiles; ct++) {
            const f32x16 &xc = xs[buf][ct];
            // scale_log2 > 0: the maximum can be taken before scaling.  A chain of
            // three-input maxima: 8 instructions for 16 values.
            float m = fmaxf(fmaxf(xc[0], xc[1]), xc[2]);
#pragma unroll
            for (int v = 3; v < 15; v += 2) m = fmaxf(fmaxf(m, xc[v]), xc[v + 1]);
            m = fmaxf(m, xc[15]);
            float other = m;
            swap_halves32(m, other);
            m_blk[ct] = fmaxf(m, other) * scale_log2;
            raise |= m_blk[ct] > m_run[ct] + kRescaleSlack;
        }
    };

    // Iteration m of the main loop multiplies P(m-1) into V(m-1), turns S(m) into
    // P(m) and computes S(m+1), so that every MFMA of the iteration is independent
    // of its exponentials and the matrix and vector pipelines of a wave overlap.
    // Block j lives in K stage j % 4 and V stage j % 4.  Per iteration one barrier; every
    // wave runs every iteration (idle ones only move rows), so the barriers match.  The loop
    // is unrolled by four so that all stage indices are static.
    //   Direct path: iteration m requests K(m+4) and V(m+2) behind its barrier (K(m+4)
    //   replaces K(m), whose operands were read at the end of iteration m-2; V(m+2) replaces
    //   V(m-2), last read in iteration m-1).  The operands of K(m+1) are read at the END of
    //   iteration m-1, into the registers iteration m's score MFMAs use, so that those MFMAs
    //   start right behind the barrier instead of waiting for LDS (steady state +0.65 %); for
    //   that K(m+2) must have been published by barrier m: it went out two iterations
    //   earlier, and a wave makes sure that its own part of it has landed (at most 3 younger
    //   loads per row group outstanding: V(m), K(m+3), V(m+1)) before it joins that barrier.
    //   The page of block j is looked up in iteration j-6 and its descriptors are built in
    //   iteration j-5, behind that iteration's MFMAs.  (DSKV_PREFILL_KPREFETCH=0: the operands
    //   of K(m+1) are read at the start of iteration m, every request one block nearer.)
    //   Register path: the rows of block m+4 are requested in iteration m and written to
    //   LDS in iteration m+2 (one iteration is shorter than a trip to memory).
    RowDesc desc[4];              // descriptors of block j in desc[j % 4]
    int pg[4][kRowGroups];        // page ids of block j in pg[j % 4]
    struct RowSet {
        u32x4 k[kRowGroups], v[kRowGroups];   // rows on their way to LDS (register path)
    };
    RowSet even, odd;
    {
        const u32x4 z = {0, 0, 0, 0};
        u32x4 zero[kRowGroups];
#pragma unroll
        for (int i = 0; i < kRowGroups; i++) zero[i] = z;
        store_rows(v_stage[3], zero);   // V(-1): multiplied by P(-1) = 0, must be finite
        // the walk starts at block blk_begin, a multiple of four: block j still lives in stage j % 4
        if (kRowsSharePage) {
#pragma unroll
            for (int blk = 0; blk < 4; blk++) lookup_pages(blk_begin + blk, pg[blk]);
#pragma unroll
            for (int blk = 0; blk < 4; blk++) prepare_rows(blk_begin + blk, pg[blk], desc[blk]);
#pragma unroll
            for (int blk = 0; blk < (kKPrefetch ? 4 : 3); blk++) load_direct(desc[blk].k, k_stage[blk]);
#pragma unroll
            for (int blk = 0; blk < 2; blk++) load_direct(desc[blk].v, v_stage[blk]);
            lookup_pages(blk_begin + 4, pg[0]);
            if (kKPrefetch) {   // one block further ahead: block 4's descriptors now, block 5's page
                prepare_rows(blk_begin + 4, pg[0], desc[0]);
                lookup_pages(blk_begin + 5, pg[1]);
            }
            DSKV_WAIT_VMEM(0);
        } else {
            u32x4 first_k[2][kRowGroups], first_v[2][kRowGroups];
#pragma unroll
            for (int blk = 0; blk < 2; blk++) load_rows(blk_begin + blk, first_k[blk], first_v[blk]);
#pragma unroll
            for (int blk = 0; blk < 2; blk++) {
                store_rows(k_stage[blk], first_k[blk]);
                store_rows(v_stage[blk], first_v[blk]);
            }
            load_rows(blk_begin + 2, even.k, even.v);
            load_rows(blk_begin + 3, odd.k, odd.v);
        }
    }
    __syncthreads();
    if (w_end > 0) {
        read_k_operands(k_stage[0], kKPrefetch ? 1 : 0);
        scores(0, kKPrefetch ? 1 : 0);
        if ((blk_begin + 1) * kBlock > w_mask_from) mask_scores(blk_begin, 0);
        block_max(0);
        if (kKPrefetch) read_k_operands(k_stage[1], 0);   // K(blk_begin + 1) for the first iteration
    }
    // V operand: token 16 ks + 8 hi + 4 h + (c >> 2) = row c >> 2 of region 4 ks + 2 hi + h;
    // bytes 64 dt + 32 (g & 1) + 8 (c & 3) of its row = half (c & 1) of chunk 4 dt + 2 (g & 1) + ((c & 3) >> 1)
    const int v_lane_off = h * kRegionBytes + (2 * (g & 1) + ((c & 3) >> 1)) * 64 + (c >> 2) * 16 + (c & 1) * 8;
    auto iteration = [&](int m, int phase, RowSet &rows) {   // phase = m % 4, a literal at each call
        if (kRowsSharePage) {
            // this wave's rows of K(m+1) have landed; then the bare barrier: with the fences of
            // __syncthreads the compiler waits for EVERY load into LDS still on its way, which
            // is the whole point of requesting them early.  Nothing else needs the fences here:
            // the loop of this path writes LDS through these loads only, and the LDS reads of
            // the previous iteration have been consumed.
            // (the empty statements pin the compiler's order of ordinary LDS accesses around the
            // barrier, which the builtin by itself does not: the previous iteration's operand
            // reads stay above it, this iteration's below)
            DSKV_WAIT_VMEM(3 * kRowGroups);
            asm volatile("" ::: "memory");
            __builtin_amdgcn_s_barrier();
            asm volatile("" ::: "memory");
        } else {
            __syncthreads();
        }
        if (kRowsSharePage && kKPrefetch) {
            lookup_pages(m + 6, pg[(phase + 2) & 3]);
            load_direct(desc[phase].k, k_stage[phase]);                       // K(m+4) over K(m), read in iteration m-2
            load_direct(desc[(phase + 2) & 3].v, v_stage[(phase + 2) & 3]);   // V(m+2)
        } else if (kRowsSharePage) {
            lookup_pages(m + 5, pg[(phase + 1) & 3]);
            load_direct(desc[(phase + 3) & 3].k, k_stage[(phase + 3) & 3]);   // K(m+3)
            load_direct(desc[(phase + 2) & 3].v, v_stage[(phase + 2) & 3]);   // V(m+2)
        } else {
            store_rows(k_stage[(phase + 2) & 3], rows.k);                     // K(m+2)
            store_rows(v_stage[(phase + 2) & 3], rows.v);                     // V(m+2)
            load_rows(m + 4, rows.k, rows.v);
        }
        if (!(w_end > 0 && (m - 1) * kBlock < w_end)) {
            if (kKPrefetch) prepare_rows(m + 5, pg[(phase + 1) & 3], desc[(phase + 1) & 3]);
            else prepare_rows(m + 4, pg[phase], desc[phase]);
            return;
        }
        if (__builtin_amdgcn_ballot_w64(raise) != 0) {
            // rare: raise the maximum and bring what was computed under the old
            // one (accumulators, row sum, the pending P(m-1)) to the new scale
#pragma unroll
            for (int ct = 0; ct < kColTiles; ct++) {
                const float m_new = fmaxf(m_run[ct], m_blk[ct]);
                const float alpha = __builtin_amdgcn_exp2f(m_run[ct] - m_new);
                m_run[ct] = m_new;
                if (kSumOnMfma) l_acc[ct] *= alpha;
                else l_run[ct] *= alpha;
#pragma unroll
                for (int dt = 0; dt < 4; dt++) acc[ct][dt] *= alpha;
#pragma unroll
                for (int ks = 0; ks < 2; ks++)
#pragma unroll
                    for (int w = 0; w < 4; w++) {
                        float lo, hi;
                        E::unpack2(pb[ct][ks][w], lo, hi);
                        pb[ct][ks][w] = E::pack2(lo * alpha, hi * alpha);
                    }
            }
        }
        // The rest of the iteration is two straight-line halves, each an MFMA
        // strand with independent vector work in its shadow:
        //   S(m+1) = K(m+1).Q^T     |  P(m) = exp2(S(m) * scale - max), packed; row sum;
        //                           |  V(m-1) operands from LDS
        //   O += P(m-1).V(m-1)      |  maximum of S(m+1)
        // with the masking of S(m+1), where needed, between them.  A masked score
        // is kNegBig and the maximum never drops below its start value, so masked
        // probabilities come out as exp2(-huge) = 0 without a select.
        const int cur = phase & 1, nxt = cur ^ 1;   // xs[cur] = S(m), xs[nxt] receives S(m+1)
        u32x4 pb_prev[kColTiles][2];
#pragma unroll
        for (int ct = 0; ct < kColTiles; ct++) {
            pb_prev[ct][0] = pb[ct][0];
            pb_prev[ct][1] = pb[ct][1];
        }
        // V operand: the transposing read hands each block of 16 lanes four tokens
        // of 16 consecutive dims, lane i of the block supplying the address of dims
        // 4*(i%4) .. +3 of the block's token i/4
        if (!kKPrefetch) read_k_operands(k_stage[(phase + 1) & 3]);      // K(m+1)
#if DSKV_PREFILL_KREADS_FIRST
        __builtin_amdgcn_sched_barrier(0);   // all eight K operands requested before anything else
#endif
        const char *v_rows = v_stage[(phase + 3) & 3] + v_lane_off;        // V(m-1)
        u32x4 va[4][2];
#pragma unroll
        for (int dt = 0; dt < 4; dt++)
#pragma unroll
            for (int ks = 0; ks < 2; ks++) {
                const char *vp = v_rows + ks * 4 * kRegionBytes + dt * 256;
                const u32x2 a_lo = read_transposed(vp);
                const u32x2 a_hi = read_transposed(vp + 2 * kRegionBytes);
                va[dt][ks] = u32x4{a_lo.x, a_lo.y, a_hi.x, a_hi.y};
            }
        scores(nxt, kKPrefetch ? (phase & 1) : 0);
#pragma unroll
        for (int ct = 0; ct < kColTiles; ct++) {
            float p[16], p_sum = 0.f;
#pragma unroll
            for (int v = 0; v < 16; v++) {
                p[v] = __builtin_amdgcn_exp2f(__builtin_fmaf(xs[cur][ct][v], scale_log2, -m_run[ct]));
                if (!kSumOnMfma) p_sum += p[v];
            }
            if (!kSumOnMfma) l_run[ct] += p_sum;
#pragma unroll
            for (int ks = 0; ks < 2; ks++)
                pb[ct][ks] = u32x4{E::pack2(p[8 * ks], p[8 * ks + 1]), E::pack2(p[8 * ks + 2], p[8 * ks + 3]),
                                   E::pack2(p[8 * ks + 4], p[8 * ks + 5]), E::pack2(p[8 * ks + 6], p[8 * ks + 7])};
            // keeps P(m) in this half (it is only consumed by the next iteration)
            asm volatile("" ::"v"(pb[ct][0]), "v"(pb[ct][1]), "v"(l_run[ct]));
        }
        if ((m + 2) * kBlock > w_mask_from) mask_scores(m + 1, nxt);   // wave-uniform

#pragma unroll
        for (int dt = 0; dt < 4; dt++)
#pragma unroll
            for (int ks = 0; ks < 2; ks++)
#pragma unroll
                for (int ct = 0; ct < kColTiles; ct++)
                    acc[ct][dt] = E::mfma_32x32(va[dt][ks], pb_prev[ct][ks], acc[ct][dt]);
        if (kSumOnMfma)
#pragma unroll
            for (int ks = 0; ks < 2; ks++)
#pragma unroll
                for (int ct = 0; ct < kColTiles; ct++)
                    l_acc[ct] = E::mfma_32x32(ones, pb_prev[ct][ks], l_acc[ct]);
        if (kKPrefetch) {
            read_k_operands(k_stage[(phase + 2) & 3], (phase + 1) & 1);   // K(m+2), published by this iteration's barrier
            prepare_rows(m + 5, pg[(phase + 1) & 3], desc[(phase + 1) & 3]);
        } else {
            prepare_rows(m + 4, pg[phase], desc[phase]);   // for the loads of the next iterations
        }
        block_max(nxt);
#pragma unroll
        for (int ct = 0; ct < kColTiles; ct++) asm volatile("" ::"v"(m_blk[ct]));
    };
    for (int m = blk_begin; m <= n_blocks; m += 4) {
        iteration(m, 0, even);
        iteration(m + 1, 1, odd);
        iteration(m + 2, 2, even);
        iteration(m + 3, 3, odd);
    }
    if (kRowsSharePage) DSKV_WAIT_VMEM(0);   // nothing of this wave may still be on its way into LDS
#undef DSKV_WAIT_VMEM

#pragma unroll
    for (int ct = 0; ct < kColTiles; ct++) {
        float l = l_acc[ct][0];   // summed over all tokens by the MFMA (both lane halves)
        if (!kSumOnMfma) {
            float l_other = l_run[ct];
            swap_halves32(l_run[ct], l_other);
            l = l_run[ct] + l_other;
        }
        if (!live[ct]) continue;
        if (partial) {
            store_partial(ct, m_run[ct], l);
            continue;
        }
        const float inv = l > 0.f ? 1.f / l : 0.f;
        uint16_t *o = out + ((long)(q_begin + qrow[ct]) * n_qo_heads + (long)kvh * group + c_head[ct]) * kHeadDim +
                      4 * h;
#pragma unroll
        for (int dt = 0; dt < 4; dt++)
#pragma unroll
            for (int i = 0; i < 4; i++) {
                u32x2 w = {E::pack2(acc[ct][dt][4 * i] * inv, acc[ct][dt][4 * i + 1] * inv),
                           E::pack2(acc[ct][dt][4 * i + 2] * inv, acc[ct][dt][4 * i + 3] * inv)};
                *reinterpret_cast<u32x2 *>(o + dt * 32 + 8 * i) = w;
            }
    }
}

#ifndef DSKV_PREFILL_MIN_WAVES
#define DSKV_PREFILL_MIN_WAVES 1
#endif
template <int DT, bool kRowsSharePage>
__global__ __launch_bounds__(64 * kPrefillWaves, DSKV_PREFILL_MIN_WAVES) void prefill_attn_mfma_kernel(
    uint16_t *__restrict__ out, const uint16_t *__restrict__ q,
    const int32_t *__restrict__ qo_indptr, const char *__restrict__ pages,
    const int32_t *__restrict__ kv_indices, const int32_t *__restrict__ kv_indptr,
    const int32_t *__restrict__ kv_last, const int32_t *__restrict__ tile_info, int n_qo_heads,
    int n_kv_heads, int page_shift, float scale_log2, int causal,
    float *__restrict__ part_o, float *__restrict__ part_ml, int max_slots)
{
    __shared__ __align__(16) char lds[kPrefillLdsBytes];
    prefill_attn_body<DT, kRowsSharePage, kPrefillWaves>(
        lds, (int)blockIdx.x, out, q, qo_indptr, pages, kv_indices, kv_indptr, kv_last, tile_info,
        n_qo_heads, n_kv_heads, page_shift, scale_log2, causal, part_o, part_ml, max_slots);
}

}  // namespace dskv
