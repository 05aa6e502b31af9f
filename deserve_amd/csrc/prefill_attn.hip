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

#include <vector>

#include <algorithm>

namespace dskv {

#ifndef DSKV_PREFILL_WAVES
#define DSKV_PREFILL_WAVES 8
#endif
#ifndef DSKV_PREFILL_COLTILES
#define DSKV_PREFILL_COLTILES 1
#endif
constexpr int kPrefillWaves = DSKV_PREFILL_WAVES;   // waves per workgroup
constexpr int kColTiles = DSKV_PREFILL_COLTILES;    // column tiles (of 32 columns) per wave
constexpr int kWaveCols = 32 * kColTiles;           // columns per wave
constexpr int kBlock = 32;                          // tokens per step (one MFMA tile)
constexpr int kTileWords = 5;                       // plan entry: request, first row, block range, part
constexpr int kRowsPerWave = kBlock / kPrefillWaves;   // rows of a block one wave loads
constexpr int kRowGroups = kRowsPerWave / 4;           // in groups of 4 rows (one load each)
static_assert(kRowsPerWave % 4 == 0 && kRowGroups >= 1, "a wave loads whole groups of 4 rows");
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
template <int DT, bool kRowsSharePage>
#ifndef DSKV_PREFILL_MIN_WAVES
#define DSKV_PREFILL_MIN_WAVES 1
#endif
__global__ __launch_bounds__(64 * kPrefillWaves, DSKV_PREFILL_MIN_WAVES) void prefill_attn_mfma_kernel(
    uint16_t *__restrict__ out, const uint16_t *__restrict__ q,
    const int32_t *__restrict__ qo_indptr, const char *__restrict__ pages,
    const int32_t *__restrict__ kv_indices, const int32_t *__restrict__ kv_indptr,
    const int32_t *__restrict__ kv_last, const int32_t *__restrict__ tile_info, int n_qo_heads,
    int n_kv_heads, int page_shift, float scale_log2, int causal, int n_splits,
    float *__restrict__ part_o, float *__restrict__ part_ml, int max_slots)
{
    typedef Elt<DT> E;
    __shared__ __align__(16) char k_stage[4][kStageBytes];
    __shared__ __align__(16) char v_stage[4][kStageBytes];

    const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
    const int lane = threadIdx.x & 63;
    const int g = lane >> 4;     // row group / chunk roles of the K/V row movement
    const int c = lane & 15;
    const int h = lane >> 5;     // MFMA roles
    const int r = lane & 31;
    const int kvh = blockIdx.x % n_kv_heads;
    const int tile = blockIdx.x / n_kv_heads;
    const int group = n_qo_heads / n_kv_heads;
    const int pos_per_wave = kWaveCols / group;    // query positions per wave

    // plan entry: request, first query row of the tile within it, and the 32-token blocks
    // [blk_begin, blk_end) of the request's K/V that this workgroup walks (all of them unless
    // the plan splits tiles; blk_begin is a multiple of four), as part `split` of n_splits
    const const_i32_ptr entry = as_const(tile_info) + (long)tile * kTileWords;
    const int b = entry[0];
    const int q0 = entry[1];
    const int blk_begin = entry[2];
    const int kv_cap_blocks = entry[3];
    const int split = entry[4];
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
    const int rows_wg = min(kPrefillWaves * pos_per_wave, n_b - q0);          // >= 1 by construction
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

    // A plan that splits tiles: every part leaves (max, sum, unnormalised O) of its rows in
    // slot row * n_splits + split of the workspace (O blocks of all slots, then their (max,
    // sum) pairs); a part that sees nothing leaves zeros and a maximum below any real one.
    auto store_partial = [&](int ct, float m, float l) {
        const long slot = (long)(q_begin + qrow[ct]) * n_splits + split;
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
            if (n_splits > 1) {
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
    u32x4 ka[8];   // K rows of a block as MFMA operands: token r, dims 16*ks + 8h .. +7
    auto read_k_operands = [&](const char *kst) {
        // token r = row r & 3 of region r >> 2; chunk 2 ks + h
        const char *k_rows = kst + (r >> 2) * kRegionBytes + h * 64 + (r & 3) * 16;
#pragma unroll
        for (int ks = 0; ks < 8; ks++) ka[ks] = *reinterpret_cast<const u32x4 *>(k_rows + ks * 128);
    };
    auto scores = [&](int buf) {
#pragma unroll
        for (int ct = 0; ct < kColTiles; ct++)
#pragma unroll
            for (int v = 0; v < 16; v++) xs[buf][ct][v] = 0.f;
#pragma unroll
        for (int ks = 0; ks < 8; ks++)
#pragma unroll
            for (int ct = 0; ct < kColTiles; ct++)
                xs[buf][ct] = E::mfma_32x32(ka[ks], qreg[ct][ks], xs[buf][ct]);
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
    //   Direct path: iteration m requests K(m+3) and V(m+2) behind its barrier (K(m+3)
    //   replaces K(m-1), last read in iteration m-2; V(m+2) replaces V(m-2), last read in
    //   iteration m-1).  K(m+1), which iteration m reads, went out two iterations earlier; a
    //   wave makes sure that its own part of it has landed (at most 3 younger loads per row
    //   group outstanding: V(m), K(m+2), V(m+1)) before it joins the barrier
    //   that publishes the block.  The page of block j is looked up in iteration j-5 and its
    //   descriptors are built in iteration j-4, behind that iteration's MFMAs.
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
            for (int blk = 0; blk < 3; blk++) load_direct(desc[blk].k, k_stage[blk]);
#pragma unroll
            for (int blk = 0; blk < 2; blk++) load_direct(desc[blk].v, v_stage[blk]);
            lookup_pages(blk_begin + 4, pg[0]);
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
        read_k_operands(k_stage[0]);
        scores(0);
        if ((blk_begin + 1) * kBlock > w_mask_from) mask_scores(blk_begin, 0);
        block_max(0);
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
        if (kRowsSharePage) {
            lookup_pages(m + 5, pg[(phase + 1) & 3]);
            load_direct(desc[(phase + 3) & 3].k, k_stage[(phase + 3) & 3]);   // K(m+3)
            load_direct(desc[(phase + 2) & 3].v, v_stage[(phase + 2) & 3]);   // V(m+2)
        } else {
            store_rows(k_stage[(phase + 2) & 3], rows.k);                     // K(m+2)
            store_rows(v_stage[(phase + 2) & 3], rows.v);                     // V(m+2)
            load_rows(m + 4, rows.k, rows.v);
        }
        if (!(w_end > 0 && (m - 1) * kBlock < w_end)) {
            prepare_rows(m + 4, pg[phase], desc[phase]);
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
        read_k_operands(k_stage[(phase + 1) & 3]);                       // K(m+1)
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
        scores(nxt);
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
        prepare_rows(m + 4, pg[phase], desc[phase]);   // for the loads of the next iterations
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
        if (n_splits > 1) {
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

// Merge pass of a plan in parts: output row r, head qh = sum_i w_i O_i / sum_i w_i l_i over
// the n_splits partials of the row (slots r * n_splits + i), w_i = exp2(m_i - max_j m_j).
// One workgroup per query row; a thread owns 16 consecutive dims of one head and requests
// all of its parts' values at once (no block table, no lookup: the slots follow from the
// row).  The decode path's merge kernel, launched with one wave per (row, head) and a table
// of parts per row, took 11.5 us for the 512 rows of a chunk; this one takes about half.
template <int DT, int kParts>
__global__ __launch_bounds__(256) void prefill_merge_parts_kernel(
    uint16_t *__restrict__ out, const float *__restrict__ part_o, const float *__restrict__ part_ml,
    const int32_t *__restrict__ rows, int n_qo_heads)
{
    typedef Elt<DT> E;
    // rows (may be null): the query rows that were computed in parts, when they are not all
    // rows of the batch (the others were left to the decode kernel)
    const long row = rows ? rows[blockIdx.x] : blockIdx.x;
    for (int idx = threadIdx.x; idx < n_qo_heads * (kHeadDim / 16); idx += blockDim.x) {
        const int qh = idx / (kHeadDim / 16), d0 = (idx % (kHeadDim / 16)) * 16;
        f32x4 o[kParts][4];
        float m[kParts], l[kParts];
#pragma unroll
        for (int i = 0; i < kParts; i++) {
            const long slot = row * kParts + i;
            const float *src = part_o + (slot * n_qo_heads + qh) * kHeadDim + d0;
#pragma unroll
            for (int j = 0; j < 4; j++) o[i][j] = *reinterpret_cast<const f32x4 *>(src + 4 * j);
            const float *ml = part_ml + (slot * n_qo_heads + qh) * 2;
            m[i] = ml[0];
            l[i] = ml[1];
        }
        float m_all = m[0];
#pragma unroll
        for (int i = 1; i < kParts; i++) m_all = fmaxf(m_all, m[i]);
        f32x4 acc[4] = {f32x4{0.f, 0.f, 0.f, 0.f}, f32x4{0.f, 0.f, 0.f, 0.f}, f32x4{0.f, 0.f, 0.f, 0.f},
                        f32x4{0.f, 0.f, 0.f, 0.f}};
        float l_all = 0.f;
#pragma unroll
        for (int i = 0; i < kParts; i++) {
            const float w = __builtin_amdgcn_exp2f(m[i] - m_all);
            l_all += w * l[i];
#pragma unroll
            for (int j = 0; j < 4; j++) acc[j] += w * o[i][j];
        }
        const float inv = l_all > 0.f ? 1.f / l_all : 0.f;
        uint16_t *dst = out + (row * n_qo_heads + qh) * kHeadDim + d0;
#pragma unroll
        for (int j = 0; j < 4; j += 2) {
            const u32x4 w4 = {E::pack2(acc[j][0] * inv, acc[j][1] * inv), E::pack2(acc[j][2] * inv, acc[j][3] * inv),
                              E::pack2(acc[j + 1][0] * inv, acc[j + 1][1] * inv),
                              E::pack2(acc[j + 1][2] * inv, acc[j + 1][3] * inv)};
            *reinterpret_cast<u32x4 *>(dst + 4 * j) = w4;
        }
    }
}

static int prefill_rows_per_tile(int n_qo_heads, int n_kv_heads)
{
    const int group = n_qo_heads / n_kv_heads;
    return group <= kWaveCols ? kPrefillWaves * (kWaveCols / group) : 1;
}

}  // namespace dskv

namespace dskv {

constexpr int kMaxPrefillSplits = 8;         // parts a tile's K/V range is cut into at most
// a part holds at least this many tokens: with 256, a 512-token chunk without prior context
// took 37 us in two parts instead of 29 us whole; with 1024, chunks over 1-2 k tokens of prior
// context lost a fifth of what the parts buy
constexpr int kMinSplitTokens = 512;
constexpr int kMaxSplitTarget = 1024;        // workgroups a split plan aims at, at most
constexpr int32_t kWholeRange = 0x7fffffff;  // blk_end of a tile that is not split

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
    // entries: one per tile, or per part of a tile when the plan splits (then there are few
    // tiles: at most 2 * kMaxSplitTarget parts)
    return kTileWords * ((int64_t)batch + nnz + 2 * kMaxSplitTarget);
}

namespace dskv {

// The tile planner.  skip (may be null): requests marked there get no tiles (their single
// row is computed by the decode kernel).
static int plan_tiles(const int32_t *qo_indptr_host, const int32_t *kv_len_host, const char *skip,
                      int32_t batch, int32_t n_qo_heads, int32_t n_kv_heads, int32_t head_dim,
                      int32_t target_workgroups, int32_t *plan_host, int64_t capacity_words,
                      int32_t *n_tiles_out, int32_t *n_splits_out, int64_t *plan_words_out,
                      int64_t *workspace_bytes_out)
{
    const int rows = prefill_rows_per_tile(n_qo_heads, n_kv_heads);
    // later query tiles of a request see more keys: they come first within a request
    struct Tile { int32_t b, row; int64_t keys; };
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
            tiles.push_back({b, (int32_t)(i * rows), keys});
        }
    }
    DSKV_REQUIRE(tiles.size() < (size_t(1) << 26) && nnz < (int64_t(1) << 31), "prefill_plan: too many tiles");
    // Workgroups are dispatched in plan order and a tile's time grows with the keys its
    // last row sees: longest first, so the short ones fill the end of the launch
    // (request order left a fifth of the wave slots idle on mixed lengths).
    if (kv_len_host && tiles.size() > 1)
        std::stable_sort(tiles.begin(), tiles.end(),
                         [](const Tile &x, const Tile &y) { return x.keys > y.keys; });
    // Few tiles (a chunk of a few hundred tokens, as the reference's scheduler hands out:
    // one 512-token chunk of an 8-kv-head model is 64 workgroups) leave most of the chip
    // idle: then every tile's K/V range is cut into parts that run as workgroups of their
    // own and leave partials, merged by a second pass - the decode path's way of keeping
    // all compute units busy.  Needs the kv lengths and the 16-bit kernel's head dim.
    int splits = 1;
    if (kv_len_host && head_dim == kHeadDim && target_workgroups >= 0 && !tiles.empty()) {
        const int64_t target =
            target_workgroups > 0 ? std::min<int64_t>(target_workgroups, kMaxSplitTarget) : compute_units();
        const int64_t wgs = (int64_t)tiles.size() * n_kv_heads;
        if (wgs * 2 <= target) {
            splits = (int)std::min<int64_t>(kMaxPrefillSplits, target / wgs);
            splits = (int)std::min<int64_t>(splits, std::max<int64_t>(1, tiles.front().keys / kMinSplitTokens));
        }
    }
    const int64_t n_entries = (int64_t)tiles.size() * splits;
    const int64_t words = n_entries * kTileWords;
    if (words > capacity_words) {
        set_error("prefill_plan: plan needs %lld words, buffer has %lld", (long long)words,
                  (long long)capacity_words);
        return DSKV_E_NOMEM;
    }
    int32_t *p = plan_host;
    for (const Tile &t : tiles) {
        // Parts of equal length, in units of four 32-token blocks (the kernel's loop is
        // unrolled by four), measured on the keys the tile sees under the causal mask; the
        // last part is open-ended.  The parts are disjoint and cover all blocks, so they are
        // also right without the mask (the last part then holds the rest of the request); a
        // part that starts past what the tile sees is empty.
        const int64_t blocks = (t.keys + kBlock - 1) / kBlock;
        const int64_t chunk = ((blocks + splits - 1) / splits + 3) / 4 * 4;
        for (int s = 0; s < splits; s++) {
            *p++ = t.b;
            *p++ = t.row;
            *p++ = (int32_t)(s * chunk);
            *p++ = s + 1 < splits ? (int32_t)((s + 1) * chunk) : kWholeRange;
            *p++ = s;
        }
    }
    *n_tiles_out = (int32_t)n_entries;
    *n_splits_out = splits;
    *plan_words_out = words;
    *workspace_bytes_out =
        splits > 1 ? nnz * splits * (int64_t)n_qo_heads * (head_dim + 2) * (int64_t)sizeof(float) : 0;
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
    // tile entries, padding, the decode plan, the row map and the list of tiled rows
    return dskv_prefill_plan_bound(batch, nnz) + 4 + dskv_decode_plan_bound(batch, total_kv_tokens) +
           (int64_t)batch + nnz + 8;
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
    const bool route = route_one_row_requests && decode_mfma_shape(head_dim, n_qo_heads, n_kv_heads, page_size);
    std::vector<int32_t> kv_len(batch);
    std::vector<char> routed(batch, 0);
    std::vector<DecodeRow> rows;
    std::vector<int32_t> tile_rows;
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
            for (int64_t i = 0; i < n_b; i++) tile_rows.push_back((int32_t)(qo_indptr_host[b] + i));
        }
    }
    int64_t tile_words = 0;
    int rc = plan_tiles(qo_indptr_host, kv_len.data(), rows.empty() ? nullptr : routed.data(), batch,
                        n_qo_heads, n_kv_heads, head_dim, target_workgroups, plan_host, capacity_words,
                        &info->n_tiles, &info->n_splits, &tile_words, &info->tile_workspace_bytes);
    if (rc) return rc;
    info->tile_workspace_bytes = (info->tile_workspace_bytes + 255) / 256 * 256;
    info->n_tile_rows = (int32_t)tile_rows.size();
    int64_t at = (tile_words + 3) / 4 * 4;
    info->plan_words = tile_words;
    if (rows.empty()) return 0;
    info->decode_plan_at = at;
    int64_t decode_words = 0;
    if (at > capacity_words) at = capacity_words;   // the decode planner then reports the shortage
    rc = plan_decode_rows(rows.data(), (int32_t)rows.size(), n_qo_heads, head_dim, target_workgroups,
                          plan_host + at, capacity_words - at, &info->n_decode_items,
                          &info->n_decode_workgroups, &decode_words, &info->decode_workspace_bytes);
    if (rc) return rc;
    info->n_decode_rows = (int32_t)rows.size();
    at += decode_words;
    const int64_t total = at + (int64_t)rows.size() + (int64_t)tile_rows.size();
    if (total > capacity_words) {
        set_error("mixed_plan: plan needs %lld words, buffer has %lld", (long long)total,
                  (long long)capacity_words);
        return DSKV_E_NOMEM;
    }
    info->row_map_at = at;
    for (const DecodeRow &r : rows) plan_host[at++] = r.row;
    info->tile_rows_at = at;
    std::copy(tile_rows.begin(), tile_rows.end(), plan_host + at);
    info->plan_words = total;
    return 0;
}

namespace dskv {

static bool prefill_mfma_path(int dtype, int head_dim, int n_qo_heads, int n_kv_heads, float scale_log2)
{
    // the MFMA kernel takes maxima before scaling: it needs a positive, sane scale
    return (dtype == DSKV_BF16 || dtype == DSKV_F16) && head_dim == kHeadDim && n_kv_heads > 0 &&
           n_qo_heads / n_kv_heads <= kWaveCols && scale_log2 > 1e-6f && scale_log2 < 1e6f;
}

// merge_rows / n_merge_rows: the query rows the tiles cover when they are not all nnz rows of
// the batch (null: all of them); an MFMA-path call with n_tiles == 0 then has nothing to do.
static int prefill_attn_impl(void *out, const void *q, const int32_t *qo_indptr,
                             const void *pages_layer, const int32_t *kv_page_indices,
                             const int32_t *kv_page_indptr, const int32_t *kv_last_page_len,
                             const int32_t *plan_dev, int32_t n_tiles, int32_t n_splits,
                             void *workspace, int64_t workspace_bytes, int32_t batch, int32_t nnz,
                             int32_t n_qo_heads, int32_t n_kv_heads, int32_t head_dim,
                             int32_t page_size, float sm_scale, int32_t causal, int32_t dtype,
                             void *stream, const int32_t *merge_rows, int32_t n_merge_rows)
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
    if (mfma && merge_rows && n_tiles == 0) return 0;   // every row went to the decode kernel
    if (mfma) {
        DSKV_REQUIRE(plan_dev && n_tiles > 0, "prefill_attn: missing plan");
        DSKV_REQUIRE(n_splits >= 1 && n_splits <= kMaxPrefillSplits && n_tiles % n_splits == 0,
                     "prefill_attn: %d plan entries in %d parts", n_tiles, n_splits);
        float *part_o = nullptr, *part_ml = nullptr;
        int64_t max_slots = 0;
        if (n_splits > 1) {
            const int64_t slot_bytes = (int64_t)n_qo_heads * (head_dim + 2) * (int64_t)sizeof(float);
            DSKV_REQUIRE(workspace && workspace_bytes >= (int64_t)nnz * n_splits * slot_bytes &&
                             (uintptr_t)workspace % 16 == 0,
                         "prefill_attn: a plan in %d parts needs a 16-byte aligned workspace of %lld bytes, got %lld",
                         n_splits, (long long)((int64_t)nnz * n_splits * slot_bytes), (long long)workspace_bytes);
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
                       n_qo_heads, n_kv_heads, shift, scale_log2, causal, n_splits, part_o,     \
                       part_ml, (int)max_slots)
        if (dtype == DSKV_BF16) {
            if (page_size >= 4) DSKV_LAUNCH_PREFILL(DSKV_BF16, true);
            else DSKV_LAUNCH_PREFILL(DSKV_BF16, false);
        } else {
            if (page_size >= 4) DSKV_LAUNCH_PREFILL(DSKV_F16, true);
            else DSKV_LAUNCH_PREFILL(DSKV_F16, false);
        }
#undef DSKV_LAUNCH_PREFILL
        DSKV_LAUNCH_CHECK("prefill_attn_mfma_kernel");
        if (n_splits > 1) {   // the parts' partials become the output rows
#define DSKV_LAUNCH_PARTS(DT, N)                                                                 \
    hipLaunchKernelGGL((prefill_merge_parts_kernel<DT, N>),                                     \
                       dim3((unsigned)(merge_rows ? n_merge_rows : nnz)), dim3(256), 0, s,      \
                       (uint16_t *)out, part_o, part_ml, merge_rows, n_qo_heads)
#define DSKV_LAUNCH_PARTS_N(DT)                                                  \
    switch (n_splits) {                                                          \
    case 2: DSKV_LAUNCH_PARTS(DT, 2); break;                                     \
    case 3: DSKV_LAUNCH_PARTS(DT, 3); break;                                     \
    case 4: DSKV_LAUNCH_PARTS(DT, 4); break;                                     \
    case 5: DSKV_LAUNCH_PARTS(DT, 5); break;                                     \
    case 6: DSKV_LAUNCH_PARTS(DT, 6); break;                                     \
    case 7: DSKV_LAUNCH_PARTS(DT, 7); break;                                     \
    default: DSKV_LAUNCH_PARTS(DT, 8); break;                                    \
    }
            if (dtype == DSKV_BF16) DSKV_LAUNCH_PARTS_N(DSKV_BF16)
            else DSKV_LAUNCH_PARTS_N(DSKV_F16)
#undef DSKV_LAUNCH_PARTS_N
#undef DSKV_LAUNCH_PARTS
            if (!merge_rows || n_merge_rows > 0) DSKV_LAUNCH_CHECK("prefill_merge_parts_kernel");
        }
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
                                   page_size, sm_scale, causal, dtype, stream, nullptr, 0);
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
                                 page_size, sm_scale, causal, dtype, stream, nullptr, 0);
    DSKV_REQUIRE(plan_dev, "mixed_attn: missing plan");
    DSKV_REQUIRE(info->n_decode_rows + info->n_tile_rows == nnz && info->n_decode_rows <= batch,
                 "mixed_attn: the plan covers %d + %d rows, the batch has %d", info->n_decode_rows,
                 info->n_tile_rows, nnz);
    DSKV_REQUIRE(workspace_bytes >= info->tile_workspace_bytes + info->decode_workspace_bytes &&
                     (workspace || info->tile_workspace_bytes + info->decode_workspace_bytes == 0),
                 "mixed_attn: the plan needs a workspace of %lld bytes, got %lld",
                 (long long)(info->tile_workspace_bytes + info->decode_workspace_bytes),
                 (long long)workspace_bytes);
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
                             page_size, sm_scale, causal, dtype, stream, plan_dev + info->tile_rows_at,
                             info->n_tile_rows);
}
