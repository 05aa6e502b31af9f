// 16-token K/V tile movement shared by the decode and prefill attention kernels
// (head_dim 128, 16-bit elements, one wavefront per kv head).
//
// Lane roles, with g = lane / 16 and c = lane % 16:
//   K: lane holds dims kk*32 + g*8 .. +8 (kk = 0..3) of tile token c - the A
//      operand of the 16x16x32 MFMA, so S^T = K.Q^T has tokens 4g..4g+3 of query
//      column c in lane (g, c).
//   V: lane loads the 16-byte chunk c of tile tokens g, g+4, g+8, g+12; the tile
//      is written to LDS row-major (one token per 288-byte row) and read back
//      with the transposing LDS read, which hands lane (g, c) tokens 4g..4g+3 of
//      dim dt*16 + c - the A operand of the P.V MFMA, in the token order S^T has.
#pragma once

#include "mfma.h"

namespace dskv {

constexpr int kTile = 16;                 // tokens per MFMA tile
constexpr int kHeadDim = 128;             // the MFMA kernels are specialised for D = 128
constexpr int kVPitch = 288;              // bytes per V row in LDS (256 + 32 pad)
constexpr int kVTileBytes = kTile * kVPitch;
constexpr int kBufferFlags = 0x00020000;  // raw buffer descriptor word 3 for 32-bit data
// Cache-policy bits of the K/V loads.  Decode uses every K/V byte once, so its
// loads carry the streaming hint (bit 1): measured on MI355X, a 607 MB read with
// the hint runs at 6.9 TB/s against 6.3 TB/s without it.  Prefill re-reads each
// tile from many workgroups and wants it cached, so it loads with policy 0.
constexpr int kLoadStreaming = 2;
constexpr int kLoadCached = 0;

// Block tables and work lists never change while a kernel runs.  Reading them
// through the constant address space tells the compiler so: wave-uniform reads
// become scalar loads (tracked apart from the vector loads of the K/V stream)
// even after the kernel has issued stores.
typedef const __attribute__((address_space(4))) int32_t *const_i32_ptr;
__device__ __forceinline__ const_i32_ptr as_const(const int32_t *p) { return (const_i32_ptr)p; }

struct TileRegs {
    u32x4 k[4];
    u32x4 v[4];
};

// One request's paged K/V of one layer as seen by one wave (one kv head).
struct KvView {
    const char *pages;           // layer base: (num_pages, 2, P, Hkv, 128) 16-bit
    const_i32_ptr page_ids;      // this request's block-table entries
    int page_shift;              // log2(page_size)
    int row_bytes;               // one token, all kv heads
    int half_bytes;              // K half of a page
    long page_bytes;
    int head_off;                // byte offset of this wave's kv head inside a token row
};

// Loads tile [t, t + 16), which lies inside pool page `page`, of a request whose
// valid tokens end at t_end.  The K rows and the V rows of the tile are each
// addressed through a buffer descriptor that ends after the tile's last valid
// row: lanes that hold later rows (or a whole tile past the end) read zero and
// generate no memory traffic, and the per-lane offsets never change.  Always
// issues exactly 8 loads.
template <int kAux>
__device__ __forceinline__ void load_kv_tile_in_page(const KvView &kv, long page, int t, int t_end,
                                                     int g, int c, TileRegs &r)
{
    const int slot = t & ((1 << kv.page_shift) - 1);
    // wave-uniform; the clamp would otherwise be selected as a vector instruction
    const int valid_bytes =
        __builtin_amdgcn_readfirstlane(min(max(t_end - t, 0), kTile)) * kv.row_bytes;
    char *first_row = const_cast<char *>(kv.pages) + page * kv.page_bytes + (long)slot * kv.row_bytes;
    __amdgpu_buffer_rsrc_t k_rows =
        __builtin_amdgcn_make_buffer_rsrc(first_row, 0, valid_bytes, kBufferFlags);
    __amdgpu_buffer_rsrc_t v_rows =
        __builtin_amdgcn_make_buffer_rsrc(first_row + kv.half_bytes, 0, valid_bytes, kBufferFlags);
    const int ko = c * kv.row_bytes + kv.head_off + g * 16;
#pragma unroll
    for (int kk = 0; kk < 4; kk++)
        r.k[kk] = __builtin_amdgcn_raw_buffer_load_b128(k_rows, ko + kk * 64, 0, kAux);
#pragma unroll
    for (int i = 0; i < 4; i++) {
        const int vo = (g + 4 * i) * kv.row_bytes + kv.head_off + c * 16;
        r.v[i] = __builtin_amdgcn_raw_buffer_load_b128(v_rows, vo, 0, kAux);
    }
}

// Index into the request's block table of the page that holds token t, clamped
// to the last page the request owns (a tile past the end still names a valid
// entry; its descriptor is empty anyway).
__device__ __forceinline__ int page_slot_of(const KvView &kv, int t, int t_end)
{
    return min(t >> kv.page_shift, max((t_end - 1) >> kv.page_shift, 0));
}

// Loads tile [t, t + 16) of a request whose valid tokens end at t_end.  Issued
// unconditionally (so the count of loads in flight is static); nothing past
// t_end is fetched.
template <bool kPageCoversTile, int kAux>
__device__ __forceinline__ void load_kv_tile(const KvView &kv, int t, int t_end, int g, int c,
                                             TileRegs &r)
{
    if (kPageCoversTile) {
        load_kv_tile_in_page<kAux>(kv, kv.page_ids[page_slot_of(kv, t, t_end)], t, t_end, g, c, r);
    } else {
        // Pages smaller than a tile: every lane resolves its own page.  Tokens
        // past the end are clamped to the last valid one; the consumer masks
        // their scores and zeroes their V rows.
        const int k_tok = c;
        const int page_mask = (1 << kv.page_shift) - 1;
        const int t_last = max(t_end - 1, 0);
        const int tk = min(t + k_tok, t_last);
        const long kpage = kv.page_ids[tk >> kv.page_shift];
        const char *kp = kv.pages + kpage * kv.page_bytes + (long)(tk & page_mask) * kv.row_bytes +
                         kv.head_off + g * 16;
#pragma unroll
        for (int kk = 0; kk < 4; kk++) r.k[kk] = *reinterpret_cast<const u32x4 *>(kp + kk * 64);
#pragma unroll
        for (int i = 0; i < 4; i++) {
            const int tv = min(t + g + 4 * i, t_last);
            const long vpage = kv.page_ids[tv >> kv.page_shift];
            const char *vp = kv.pages + vpage * kv.page_bytes + kv.half_bytes +
                             (long)(tv & page_mask) * kv.row_bytes + kv.head_off + c * 16;
            r.v[i] = *reinterpret_cast<const u32x4 *>(vp);
        }
    }
}

// Loads tile [t, t + 16) when a page holds fewer tokens than a tile (kPages pages per tile;
// used for pages of 8 tokens, kPages = 2).  The tile's page ids come in as scalars (looked up one
// tile ahead with scalar loads, like the single page of the path above); every lane selects
// the page of its row among them.  Looking the ids up per lane with vector loads instead
// would put a dependent load in front of every tile, and since a wave's vector loads return
// in order, waiting for it means waiting for every tile still in flight: with pages of 8
// tokens the pass took 114 us; this way 100 (98 with pages of 16).  Tokens past the end are clamped to the last
// valid one, as in the per-lane path; page[0] is a valid page of the request also for a tile
// that lies wholly past the end.
template <int kPages, int kAux>
__device__ __forceinline__ void load_kv_tile_small_pages(const KvView &kv, const long (&page)[kPages],
                                                         int t, int t_end, int g, int c, TileRegs &r)
{
    const int page_mask = (1 << kv.page_shift) - 1;
    const int t_last = max(t_end - 1, 0);
    auto row_of = [&](int tok) -> const char * {
        const int tc = min(tok, t_last);
        const int j = max(tc - t, 0) >> kv.page_shift;
        long pg = page[0];
#pragma unroll
        for (int i = 1; i < kPages; i++) pg = j == i ? page[i] : pg;
        return kv.pages + pg * kv.page_bytes + (long)(tc & page_mask) * kv.row_bytes + kv.head_off;
    };
    auto load16 = [](const char *p) {
        const u32x4 *q = reinterpret_cast<const u32x4 *>(p);
        return kAux == kLoadStreaming ? __builtin_nontemporal_load(q) : *q;
    };
    const char *kp = row_of(t + c) + g * 16;
#pragma unroll
    for (int kk = 0; kk < 4; kk++) r.k[kk] = load16(kp + kk * 64);
#pragma unroll
    for (int i = 0; i < 4; i++) r.v[i] = load16(row_of(t + g + 4 * i) + kv.half_bytes + c * 16);
}

// V tile -> this wave's LDS tile.  Rows at or past t_end must be zero (their
// probabilities are zero, but 0 * garbage is not): the buffer-descriptor path
// already delivers zeros, the clamped path zeroes them here.  The tile is
// private to the wave; LDS executes a wave's accesses in order, the barriers
// only pin the compiler's order.
template <bool kPageCoversTile>
__device__ __forceinline__ void stage_v_tile(char *lds, const TileRegs &r, int t, int t_end, int g,
                                             int c)
{
    __builtin_amdgcn_wave_barrier();
#pragma unroll
    for (int i = 0; i < 4; i++) {
        u32x4 vv = r.v[i];
        if (!kPageCoversTile && t + g + 4 * i >= t_end) vv = u32x4{0, 0, 0, 0};
        *reinterpret_cast<u32x4 *>(lds + (g + 4 * i) * kVPitch + c * 16) = vv;
    }
    __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront");
    __builtin_amdgcn_wave_barrier();
}

// The transposing LDS read works on blocks of 16 lanes: lane i of a block
// supplies the address of four consecutive 16-bit values ("its row"), and
// receives value i%4 of the rows supplied by lanes i/4, i/4 + 4, i/4 + 8 and
// i/4 + 12 of its block.
typedef short lds_i16x4 __attribute__((ext_vector_type(4)));
__device__ __forceinline__ u32x2 read_transposed(const char *row)
{
    const lds_i16x4 v = __builtin_amdgcn_ds_read_tr16_b64_v4i16(
        (__attribute__((address_space(3))) lds_i16x4 *)row);
    return __builtin_bit_cast(u32x2, v);
}

// A operand of the 16x16x16 P.V MFMA for dim tile dt: V[token 4g + j][dim dt*16 + c],
// j = 0..3.  Lane (g, i) points at dims dt*16 + 4*(i%4) .. +3 of token 4g + i/4.
__device__ __forceinline__ u32x2 read_v_operand(const char *lds, int dt, int g, int c)
{
    return read_transposed(lds + (4 * g + (c >> 2)) * kVPitch + dt * 32 + (c & 3) * 8);
}

}  // namespace dskv
