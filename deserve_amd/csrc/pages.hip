// Page gather / scatter between the layered pool and a contiguous chunk.
// Pure byte movement; HBM-bound (one read + one write of every byte).
//
// Mapping: chunk row r = layer * n_pages + j holds pool page page_ids[j] of
// that layer.  One 256-thread workgroup moves one 16 KiB part of one row, 16
// bytes per lane per instruction (a wavefront covers 1 KiB contiguous), so a
// 64 KiB bf16 page is four workgroups and a 5000-page x 10-layer microbatch is
// 200 k workgroups - far more than the 256 CUs need to stay busy.
#include "common.h"

namespace dskv {

constexpr int kPartBytes = 16384;

template <bool kGather>
__global__ __launch_bounds__(256) void move_pages_kernel(char *__restrict__ pool,
                                                         char *__restrict__ chunk,
                                                         const int32_t *__restrict__ page_ids,
                                                         int n_pages, long layer_stride,
                                                         long page_bytes, long row_begin)
{
    const long r = row_begin + blockIdx.x;
    const int layer = (int)(r / n_pages);
    const int j = (int)(r - (long)layer * n_pages);
    const long page = page_ids[j];
    // an id outside the layer moves nothing (callers check ids on the host; this keeps a
    // bad id that slipped through from addressing outside the pool)
    if (page < 0 || (page + 1) * page_bytes > layer_stride) return;
    char *p = pool + layer * layer_stride + page * page_bytes;
    char *c = chunk + (long)blockIdx.x * page_bytes;
    const long part_begin = (long)blockIdx.y * kPartBytes;
    const long part_end = min(part_begin + kPartBytes, page_bytes);
    for (long off = part_begin + threadIdx.x * 16; off < part_end; off += 256 * 16) {
        if (kGather)
            *reinterpret_cast<u32x4 *>(c + off) = *reinterpret_cast<const u32x4 *>(p + off);
        else
            *reinterpret_cast<u32x4 *>(p + off) = *reinterpret_cast<const u32x4 *>(c + off);
    }
}

static int move_pages(bool gather, void *pool, void *chunk, const int32_t *page_ids,
                      int32_t n_pages, int32_t n_layers, int64_t layer_stride_bytes,
                      int64_t page_bytes, int64_t row_begin, int64_t row_end, void *stream)
{
    const char *who = gather ? "gather_pages" : "scatter_pages";
    DSKV_REQUIRE(n_pages >= 0 && n_layers >= 0, "%s: negative sizes", who);
    const int64_t rows = (int64_t)n_pages * n_layers;
    DSKV_REQUIRE(0 <= row_begin && row_begin <= row_end && row_end <= rows,
                 "%s: row range [%lld, %lld) outside [0, %lld)", who, (long long)row_begin,
                 (long long)row_end, (long long)rows);
    if (row_end == row_begin) return 0;
    DSKV_REQUIRE(pool && chunk && page_ids, "%s: null pointer argument", who);
    DSKV_REQUIRE(page_bytes > 0 && page_bytes % 16 == 0,
                 "%s: page_bytes (%lld) must be a positive multiple of 16", who,
                 (long long)page_bytes);
    DSKV_REQUIRE(layer_stride_bytes % 16 == 0 && ((uintptr_t)pool | (uintptr_t)chunk) % 16 == 0,
                 "%s: pool/chunk/layer stride must be 16-byte aligned", who);
    DSKV_REQUIRE(row_end - row_begin < (int64_t(1) << 31), "%s: too many rows in one call", who);
    const unsigned parts = (unsigned)((page_bytes + kPartBytes - 1) / kPartBytes);
    DSKV_REQUIRE(parts <= 65535, "%s: page too large", who);
    dim3 grid((unsigned)(row_end - row_begin), parts);
    if (gather)
        hipLaunchKernelGGL(move_pages_kernel<true>, grid, dim3(256), 0, (hipStream_t)stream,
                           (char *)pool, (char *)chunk, page_ids, n_pages, layer_stride_bytes,
                           page_bytes, row_begin);
    else
        hipLaunchKernelGGL(move_pages_kernel<false>, grid, dim3(256), 0, (hipStream_t)stream,
                           (char *)pool, (char *)chunk, page_ids, n_pages, layer_stride_bytes,
                           page_bytes, row_begin);
    DSKV_LAUNCH_CHECK(who);
    return 0;
}

// Small host-to-device upload done by a kernel: every lane reads 16 bytes of
// pinned host memory over the link and stores them to HBM.  For the few tens
// of KiB of per-step metadata this takes microseconds, and unlike an async
// memcpy it stays on the compute queue of the caller's stream: a copy engine
// between two kernels of a stream costs a hand-over to the engine and one
// back, and with a host that runs several steps ahead those hand-overs have
// been measured to stall whole steps.
__global__ __launch_bounds__(256) void upload_words_kernel(uint32_t *__restrict__ dst,
                                                           const uint32_t *__restrict__ src,
                                                           long n_words)
{
    const long quads = n_words / 4;
    const long i = (long)blockIdx.x * 256 + threadIdx.x;
    if (i < quads)
        reinterpret_cast<u32x4 *>(dst)[i] = reinterpret_cast<const u32x4 *>(src)[i];
    else if (i == quads)
        for (long w = quads * 4; w < n_words; w++) dst[w] = src[w];
}

}  // namespace dskv

extern "C" int dskv_upload_words(void *dst, const void *src_pinned, int64_t n_words, void *stream)
{
    DSKV_REQUIRE(n_words >= 0 && n_words <= (int64_t(1) << 28), "upload_words: %lld words out of range",
                 (long long)n_words);
    if (n_words == 0) return 0;
    DSKV_REQUIRE(dst && src_pinned, "upload_words: null pointer");
    DSKV_REQUIRE((uintptr_t)dst % 16 == 0 && (uintptr_t)src_pinned % 16 == 0,
                 "upload_words: both buffers must start on a 16-byte boundary");
    const long quads = n_words / 4;
    hipLaunchKernelGGL(dskv::upload_words_kernel, dim3((unsigned)(quads / 256 + 1)), dim3(256), 0,
                       (hipStream_t)stream, (uint32_t *)dst, (const uint32_t *)src_pinned,
                       (long)n_words);
    DSKV_LAUNCH_CHECK("upload_words");
    return 0;
}

extern "C" int dskv_gather_pages(void *chunk, const void *pool, const int32_t *page_ids,
                                 int32_t n_pages, int32_t n_layers, int64_t layer_stride_bytes,
                                 int64_t page_bytes, int64_t row_begin, int64_t row_end,
                                 void *stream)
{
    return dskv::move_pages(true, const_cast<void *>(pool), chunk, page_ids, n_pages, n_layers,
                            layer_stride_bytes, page_bytes, row_begin, row_end, stream);
}

extern "C" int dskv_scatter_pages(void *pool, const void *chunk, const int32_t *page_ids,
                                  int32_t n_pages, int32_t n_layers, int64_t layer_stride_bytes,
                                  int64_t page_bytes, int64_t row_begin, int64_t row_end,
                                  void *stream)
{
    return dskv::move_pages(false, pool, const_cast<void *>(chunk), page_ids, n_pages, n_layers,
                            layer_stride_bytes, page_bytes, row_begin, row_end, stream);
}
