// KV swap between the HBM page pool and pinned host DRAM.
//
// Bound: the host link (PCIe); HBM-side staging traffic is overhead.
//
// Two forms:
//  * dskv_swap_slice - a contiguous slice of pool pages of every layer; each
//    layer's slice is one contiguous run, so it is one async copy per layer and
//    direction, split over two caller streams.
//  * the scattered-page engine - pages named by a block table are packed by a
//    gather kernel into a contiguous staging buffer and leave in one large
//    async copy per staging chunk (and the reverse for swap-in).  Each direction
//    has ONE stream and one staging buffer: a gather of 128 MiB takes ~1 % of the
//    time of its copy, so serialising them costs nothing measurable, while
//    splitting a direction's copies over two streams made them compete for the
//    link (measured: 41 instead of 47 GB/s each way in an exchange).  The two
//    directions run on their own streams, so D2H and H2D traffic of an exchange
//    use both halves of the full-duplex link.
#include "common.h"

#include <algorithm>
#include <deque>
#include <new>
#include <vector>

struct dskv_swap {
    int device = 0;
    int64_t staging_bytes = 0;
    // [direction: 0 = out (D2H), 1 = in (H2D)]
    hipStream_t stream[2] = {nullptr, nullptr};
    void *staging[2] = {nullptr, nullptr};
    hipEvent_t dir_done[2] = {nullptr, nullptr};
    bool dir_used[2] = {false, false};
    hipEvent_t ready = nullptr;        // caller's stream reached the call
    hipEvent_t ids_ready = nullptr;    // page ids have landed on the device
    hipEvent_t gathered[2] = {nullptr, nullptr};   // exchange: chunk left the pool
    hipEvent_t fence = nullptr;
    // page-id ring: pinned host mirror + device copy.  A call takes the next free stretch;
    // a stretch is free again once the events recorded behind the call's last use of it
    // have completed (checked, never waited for).
    int32_t *ids_host = nullptr;
    int32_t *ids_dev = nullptr;
    int64_t ids_capacity = 0;
    int64_t ids_head = 0;              // where the next stretch starts
    struct IdStretch {
        int64_t begin, end;
        hipEvent_t done[2];            // per direction stream that read it (null = unused)
        bool sealed;                   // every reader's end has been recorded in `done`
    };
    std::deque<IdStretch> ids_pending; // oldest first
    std::vector<hipEvent_t> spare_events;
    bool probed = false;               // streams checked against the caller's compute stream
    bool independent = false;          // ... and found to run beside it
    bool streams_exported = false;     // a caller holds the raw stream handles (dskv_swap_streams)
};

namespace dskv {

constexpr int64_t kIdsCapacity = int64_t(1) << 20;

static int check_geometry(const char *who, int32_t n_pages, int32_t n_layers,
                          int64_t layer_stride_bytes, int64_t page_bytes)
{
    DSKV_REQUIRE(n_pages >= 0 && n_layers >= 0, "%s: negative sizes", who);
    DSKV_REQUIRE(page_bytes > 0 && page_bytes % 16 == 0,
                 "%s: page_bytes (%lld) must be a positive multiple of 16", who,
                 (long long)page_bytes);
    DSKV_REQUIRE(layer_stride_bytes >= page_bytes && layer_stride_bytes % 16 == 0,
                 "%s: bad layer stride %lld", who, (long long)layer_stride_bytes);
    return 0;
}

static void recycle(dskv_swap *h, dskv_swap::IdStretch &st)
{
    for (hipEvent_t &e : st.done)
        if (e) {
            h->spare_events.push_back(e);
            e = nullptr;
        }
}

static int wait_all(dskv_swap *h)
{
    for (int d = 0; d < 2; d++) DSKV_HIP(hipStreamSynchronize(h->stream[d]));
    for (auto &st : h->ids_pending) recycle(h, st);
    h->ids_pending.clear();
    h->ids_head = 0;
    return 0;
}

static int take_event(dskv_swap *h, hipEvent_t *out)
{
    if (!h->spare_events.empty()) {
        *out = h->spare_events.back();
        h->spare_events.pop_back();
        return 0;
    }
    DSKV_HIP(hipEventCreateWithFlags(out, hipEventDisableTiming));
    return 0;
}

// Forget the stretches whose readers have finished (a query, never a wait).
static void retire_ids(dskv_swap *h)
{
    while (!h->ids_pending.empty()) {
        dskv_swap::IdStretch &st = h->ids_pending.front();
        // a stretch whose call did not get as far as recording the end of its readers is
        // only given up by wait_all, which drains both streams
        if (!st.sealed) return;
        for (hipEvent_t e : st.done)
            if (e && hipEventQuery(e) != hipSuccess) {
                (void)hipGetLastError();   // hipErrorNotReady is not a failure
                return;
            }
        recycle(h, st);
        h->ids_pending.pop_front();
    }
    if (h->ids_pending.empty()) h->ids_head = 0;
}

// Copy the caller's page ids into the ring and start their upload on `s`: a kernel
// reading the pinned mirror (stretches are multiples of four words, as it wants), so the
// copy engines carry page data only.  Never blocks: when the ring has no free stretch
// of this size (earlier calls still in flight hold it), the call is refused with
// DSKV_E_STATE and the caller waits (dskv_swap_wait) or retries later.
static int stage_ids(dskv_swap *h, const int32_t *ids, int32_t n, hipStream_t s, int32_t **dev_out)
{
    const int64_t len = ((int64_t)n + 3) / 4 * 4;
    DSKV_REQUIRE(len <= h->ids_capacity, "swap: %d page ids exceed the engine's limit of %lld", n,
                 (long long)h->ids_capacity);
    retire_ids(h);
    // pending stretches occupy [tail, head) of the ring, possibly wrapped
    int64_t begin = h->ids_head;
    const int64_t tail = h->ids_pending.empty() ? begin : h->ids_pending.front().begin;
    const bool wrapped = !h->ids_pending.empty() && tail >= begin;   // free space is [head, tail)
    bool fits;
    if (h->ids_pending.empty()) {
        begin = 0;
        fits = true;
    } else if (wrapped) {
        fits = begin + len <= tail;
    } else if (begin + len <= h->ids_capacity) {
        fits = true;
    } else {
        begin = 0;                                   // wrap: free space is [0, tail)
        fits = len <= tail;
    }
    if (!fits) {
        set_error("swap: the page-id ring (%lld ids) is held by calls still in flight; wait "
                  "(dskv_swap_wait) or retry once they have finished", (long long)h->ids_capacity);
        return DSKV_E_STATE;
    }
    int32_t *host = h->ids_host + begin;
    int32_t *dev = h->ids_dev + begin;
    std::copy(ids, ids + n, host);
    int rc = dskv_upload_words(dev, host, n, s);
    if (rc) return rc;
    h->ids_pending.push_back(dskv_swap::IdStretch{begin, begin + len, {nullptr, nullptr}, false});
    h->ids_head = begin + len;
    *dev_out = dev;
    return 0;
}

// Marks the end of the newest stretch's use on direction `dir` (call after the last kernel
// that reads it has been enqueued there).
static int release_ids_after(dskv_swap *h, int dir)
{
    dskv_swap::IdStretch &st = h->ids_pending.back();
    if (!st.done[dir]) {
        int rc = take_event(h, &st.done[dir]);
        if (rc) return rc;
    }
    DSKV_HIP(hipEventRecord(st.done[dir], h->stream[dir]));
    return 0;
}

// From stage_ids to the end of a call the newest stretch belongs to that call.  A call that
// ends well seals it (the end of every reader is on record in `done`); one that fails on the
// way has already enqueued the id upload and perhaps gather / scatter kernels that read the
// stretch, so the guard records the end of whatever both streams hold now and seals it - or,
// if even that fails, leaves it unsealed, which keeps the stretch (and the pinned mirror
// behind it) out of circulation until dskv_swap_wait has drained the streams.
struct IdsGuard {
    dskv_swap *h;
    bool armed;
    void seal()
    {
        h->ids_pending.back().sealed = true;
        armed = false;
    }
    ~IdsGuard()
    {
        if (!armed || h->ids_pending.empty()) return;
        bool ok = true;
        for (int dir = 0; dir < 2; dir++) ok = release_ids_after(h, dir) == 0 && ok;
        (void)hipGetLastError();
        h->ids_pending.back().sealed = ok;
    }
};

// The gather and scatter kernels index the pool by page id: ids outside a layer are
// refused here, on the host.
static int check_ids(const char *who, const int32_t *ids, int32_t n, int64_t layer_stride_bytes,
                     int64_t page_bytes)
{
    int32_t top = 0;
    for (int32_t i = 0; i < n; i++) {
        DSKV_REQUIRE(ids[i] >= 0, "%s: negative page id %d at %d", who, ids[i], i);
        top = std::max(top, ids[i]);
    }
    DSKV_REQUIRE(((int64_t)top + 1) * page_bytes <= layer_stride_bytes,
                 "%s: page id %d lies outside a layer of %lld bytes", who, top,
                 (long long)layer_stride_bytes);
    return 0;
}

// The stream of direction `dir` waits for: the caller's stream, the id upload,
// and everything previously enqueued in the opposite direction (an earlier
// swap-out may still be reading pages that this swap-in is about to overwrite,
// and the other way round).
static int open_direction(dskv_swap *h, int dir, hipStream_t after, hipStream_t ids_stream)
{
    hipStream_t s = h->stream[dir];
    DSKV_HIP(hipEventRecord(h->ready, after));
    DSKV_HIP(hipStreamWaitEvent(s, h->ready, 0));
    if (s != ids_stream) {
        DSKV_HIP(hipEventRecord(h->ids_ready, ids_stream));
        DSKV_HIP(hipStreamWaitEvent(s, h->ids_ready, 0));
    }
    if (h->dir_used[1 - dir]) DSKV_HIP(hipStreamWaitEvent(s, h->dir_done[1 - dir], 0));
    return 0;
}

static int close_direction(dskv_swap *h, int dir)
{
    DSKV_HIP(hipEventRecord(h->dir_done[dir], h->stream[dir]));
    h->dir_used[dir] = true;
    return release_ids_after(h, dir);
}

// ---- do two streams run side by side?
//
// The HIP runtime maps streams onto a small number of hardware queues (four by default)
// and packets of one queue run in order: a kernel on a stream that shares its queue with
// a copy stream waits for the copy.  Which streams share is decided when they are
// created, from how many streams the process already has - not something a caller can
// see.  So it is measured: a kernel that idles for half a millisecond goes to one
// stream, an empty kernel to the other; if the empty one finishes first, the two streams
// run side by side.
__global__ void idle_kernel(long ticks)
{
    const long t0 = wall_clock64();
    while (wall_clock64() - t0 < ticks) __builtin_amdgcn_s_sleep(64);
}

__global__ void empty_kernel() {}

static int runs_beside(hipStream_t a, hipStream_t b, hipEvent_t ea, hipEvent_t eb, long ticks,
                       bool *beside)
{
    DSKV_HIP(hipStreamSynchronize(a));
    DSKV_HIP(hipStreamSynchronize(b));
    hipLaunchKernelGGL(idle_kernel, dim3(1), dim3(64), 0, a, ticks);
    DSKV_LAUNCH_CHECK("idle_kernel");
    DSKV_HIP(hipEventRecord(ea, a));
    hipLaunchKernelGGL(empty_kernel, dim3(1), dim3(64), 0, b);
    DSKV_LAUNCH_CHECK("empty_kernel");
    DSKV_HIP(hipEventRecord(eb, b));
    DSKV_HIP(hipEventSynchronize(eb));
    const hipError_t q = hipEventQuery(ea);       // still idling = b did not wait for a
    (void)hipGetLastError();
    *beside = q == hipErrorNotReady;
    DSKV_HIP(hipEventSynchronize(ea));
    return 0;
}

}  // namespace dskv

extern "C" int dskv_swap_slice(void *slice_base, int64_t layer_stride_bytes, int64_t slice_bytes,
                               int32_t n_layers, void *host_to, const void *host_from,
                               void *stream0, void *stream1)
{
    using namespace dskv;
    DSKV_REQUIRE(n_layers >= 0 && slice_bytes >= 0, "swap_slice: negative sizes");
    if (n_layers == 0 || slice_bytes == 0 || (!host_to && !host_from)) return 0;
    DSKV_REQUIRE(slice_base, "swap_slice: null slice pointer");
    DSKV_REQUIRE(layer_stride_bytes >= slice_bytes, "swap_slice: layer stride %lld < slice bytes %lld",
                 (long long)layer_stride_bytes, (long long)slice_bytes);
    const int mid = n_layers / 2;
    for (int l = 0; l < n_layers; l++) {
        hipStream_t s = (hipStream_t)(l < mid ? stream0 : stream1);
        char *dev = (char *)slice_base + (int64_t)l * layer_stride_bytes;
        if (host_to)
            DSKV_HIP(hipMemcpyAsync((char *)host_to + (int64_t)l * slice_bytes, dev,
                                    (size_t)slice_bytes, hipMemcpyDeviceToHost, s));
        if (host_from)
            DSKV_HIP(hipMemcpyAsync(dev, (const char *)host_from + (int64_t)l * slice_bytes,
                                    (size_t)slice_bytes, hipMemcpyHostToDevice, s));
    }
    return 0;
}

extern "C" int dskv_swap_create(dskv_swap_t **handle, int64_t staging_bytes)
{
    using namespace dskv;
    DSKV_REQUIRE(handle, "swap_create: null handle pointer");
    DSKV_REQUIRE(staging_bytes >= (1 << 20) && staging_bytes % 16 == 0,
                 "swap_create: staging_bytes (%lld) must be >= 1 MiB and a multiple of 16",
                 (long long)staging_bytes);
    dskv_swap *h = new (std::nothrow) dskv_swap();
    DSKV_REQUIRE(h, "swap_create: out of host memory");
    *handle = nullptr;
#define DSKV_CREATE(expr)                                                   \
    do {                                                                    \
        hipError_t e_ = (expr);                                             \
        if (e_ != hipSuccess) {                                             \
            set_error("%s failed: %s", #expr, hipGetErrorString(e_));       \
            dskv_swap_destroy(h);                                           \
            return (int)e_;                                                 \
        }                                                                   \
    } while (0)
    DSKV_CREATE(hipGetDevice(&h->device));
    h->staging_bytes = staging_bytes;
    for (int d = 0; d < 2; d++) {
        DSKV_CREATE(hipStreamCreateWithFlags(&h->stream[d], hipStreamNonBlocking));
        DSKV_CREATE(hipMalloc(&h->staging[d], (size_t)staging_bytes));
        DSKV_CREATE(hipEventCreateWithFlags(&h->dir_done[d], hipEventDisableTiming));
    }
    DSKV_CREATE(hipEventCreateWithFlags(&h->ready, hipEventDisableTiming));
    DSKV_CREATE(hipEventCreateWithFlags(&h->ids_ready, hipEventDisableTiming));
    DSKV_CREATE(hipEventCreateWithFlags(&h->fence, hipEventDisableTiming));
    for (int i = 0; i < 2; i++)
        DSKV_CREATE(hipEventCreateWithFlags(&h->gathered[i], hipEventDisableTiming));
    h->ids_capacity = kIdsCapacity;
    DSKV_CREATE(hipHostMalloc((void **)&h->ids_host, (size_t)h->ids_capacity * sizeof(int32_t),
                              hipHostMallocDefault));
    DSKV_CREATE(hipMalloc((void **)&h->ids_dev, (size_t)h->ids_capacity * sizeof(int32_t)));
#undef DSKV_CREATE
    *handle = h;
    return 0;
}

extern "C" int dskv_swap_destroy(dskv_swap_t *h)
{
    if (!h) return 0;
    for (int d = 0; d < 2; d++) {
        if (h->stream[d]) {
            (void)hipStreamSynchronize(h->stream[d]);
            (void)hipStreamDestroy(h->stream[d]);
        }
        if (h->staging[d]) (void)hipFree(h->staging[d]);
        if (h->dir_done[d]) (void)hipEventDestroy(h->dir_done[d]);
    }
    if (h->ready) (void)hipEventDestroy(h->ready);
    if (h->ids_ready) (void)hipEventDestroy(h->ids_ready);
    if (h->fence) (void)hipEventDestroy(h->fence);
    for (int i = 0; i < 2; i++)
        if (h->gathered[i]) (void)hipEventDestroy(h->gathered[i]);
    for (auto &st : h->ids_pending)
        for (hipEvent_t e : st.done)
            if (e) (void)hipEventDestroy(e);
    for (hipEvent_t e : h->spare_events) (void)hipEventDestroy(e);
    if (h->ids_host) (void)hipHostFree(h->ids_host);
    if (h->ids_dev) (void)hipFree(h->ids_dev);
    delete h;
    return 0;
}

extern "C" int dskv_swap_out_async(dskv_swap_t *h, void *host_dst, const void *pool,
                                   const int32_t *page_ids_host, int32_t n_pages, int32_t n_layers,
                                   int64_t layer_stride_bytes, int64_t page_bytes,
                                   void *after_stream)
{
    using namespace dskv;
    DSKV_REQUIRE(h, "swap_out: null handle");
    int rc = check_geometry("swap_out", n_pages, n_layers, layer_stride_bytes, page_bytes);
    if (rc) return rc;
    const int64_t rows = (int64_t)n_pages * n_layers;
    if (rows == 0) return 0;
    DSKV_REQUIRE(host_dst && pool && page_ids_host, "swap_out: null pointer argument");
    if ((rc = check_ids("swap_out", page_ids_host, n_pages, layer_stride_bytes, page_bytes))) return rc;
    const int64_t rows_per_chunk = h->staging_bytes / page_bytes;
    DSKV_REQUIRE(rows_per_chunk >= 1, "swap_out: a page (%lld bytes) does not fit the staging buffer",
                 (long long)page_bytes);
    int32_t *ids_dev = nullptr;
    hipStream_t s = h->stream[0];
    if ((rc = stage_ids(h, page_ids_host, n_pages, s, &ids_dev))) return rc;
    IdsGuard ids_guard{h, true};
    if ((rc = open_direction(h, 0, (hipStream_t)after_stream, s))) return rc;
    for (int64_t r0 = 0; r0 < rows; r0 += rows_per_chunk) {
        const int64_t r1 = std::min(rows, r0 + rows_per_chunk);
        if ((rc = dskv_gather_pages(h->staging[0], pool, ids_dev, n_pages, n_layers,
                                    layer_stride_bytes, page_bytes, r0, r1, s)))
            return rc;
        DSKV_HIP(hipMemcpyAsync((char *)host_dst + r0 * page_bytes, h->staging[0],
                                (size_t)((r1 - r0) * page_bytes), hipMemcpyDeviceToHost, s));
    }
    if ((rc = close_direction(h, 0))) return rc;
    ids_guard.seal();
    return 0;
}

extern "C" int dskv_swap_in_async(dskv_swap_t *h, void *pool, const void *host_src,
                                  const int32_t *page_ids_host, int32_t n_pages, int32_t n_layers,
                                  int64_t layer_stride_bytes, int64_t page_bytes,
                                  void *after_stream)
{
    using namespace dskv;
    DSKV_REQUIRE(h, "swap_in: null handle");
    int rc = check_geometry("swap_in", n_pages, n_layers, layer_stride_bytes, page_bytes);
    if (rc) return rc;
    const int64_t rows = (int64_t)n_pages * n_layers;
    if (rows == 0) return 0;
    DSKV_REQUIRE(host_src && pool && page_ids_host, "swap_in: null pointer argument");
    if ((rc = check_ids("swap_in", page_ids_host, n_pages, layer_stride_bytes, page_bytes))) return rc;
    const int64_t rows_per_chunk = h->staging_bytes / page_bytes;
    DSKV_REQUIRE(rows_per_chunk >= 1, "swap_in: a page (%lld bytes) does not fit the staging buffer",
                 (long long)page_bytes);
    int32_t *ids_dev = nullptr;
    hipStream_t s = h->stream[1];
    if ((rc = stage_ids(h, page_ids_host, n_pages, s, &ids_dev))) return rc;
    IdsGuard ids_guard{h, true};
    if ((rc = open_direction(h, 1, (hipStream_t)after_stream, s))) return rc;
    for (int64_t r0 = 0; r0 < rows; r0 += rows_per_chunk) {
        const int64_t r1 = std::min(rows, r0 + rows_per_chunk);
        DSKV_HIP(hipMemcpyAsync(h->staging[1], (const char *)host_src + r0 * page_bytes,
                                (size_t)((r1 - r0) * page_bytes), hipMemcpyHostToDevice, s));
        if ((rc = dskv_scatter_pages(pool, h->staging[1], ids_dev, n_pages, n_layers,
                                     layer_stride_bytes, page_bytes, r0, r1, s)))
            return rc;
    }
    if ((rc = close_direction(h, 1))) return rc;
    ids_guard.seal();
    return 0;
}

extern "C" int dskv_swap_exchange_async(dskv_swap_t *h, void *host_dst, const void *host_src,
                                        void *pool, const int32_t *page_ids_host, int32_t n_pages,
                                        int32_t n_layers, int64_t layer_stride_bytes,
                                        int64_t page_bytes, void *after_stream)
{
    using namespace dskv;
    DSKV_REQUIRE(h, "swap_exchange: null handle");
    int rc = check_geometry("swap_exchange", n_pages, n_layers, layer_stride_bytes, page_bytes);
    if (rc) return rc;
    const int64_t rows = (int64_t)n_pages * n_layers;
    if (rows == 0) return 0;
    DSKV_REQUIRE(host_dst && host_src && pool && page_ids_host,
                 "swap_exchange: null pointer argument");
    if ((rc = check_ids("swap_exchange", page_ids_host, n_pages, layer_stride_bytes, page_bytes)))
        return rc;
    const int64_t rows_per_chunk = h->staging_bytes / page_bytes;
    DSKV_REQUIRE(rows_per_chunk >= 1,
                 "swap_exchange: a page (%lld bytes) does not fit the staging buffer",
                 (long long)page_bytes);
    int32_t *ids_dev = nullptr;
    hipStream_t so = h->stream[0], si = h->stream[1];
    if ((rc = stage_ids(h, page_ids_host, n_pages, so, &ids_dev))) return rc;
    IdsGuard ids_guard{h, true};
    if ((rc = open_direction(h, 0, (hipStream_t)after_stream, so))) return rc;
    if ((rc = open_direction(h, 1, (hipStream_t)after_stream, so))) return rc;
    // host_dst == host_src is a round trip through one buffer (two microbatch
    // rounds share their pinned buffer): dump-then-refill leaves the pages as
    // they were, so only the dump is performed.
    const bool same_buffer = host_dst == host_src;
    int c = 0;
    for (int64_t r0 = 0; r0 < rows; r0 += rows_per_chunk, c ^= 1) {
        const int64_t r1 = std::min(rows, r0 + rows_per_chunk);
        const size_t bytes = (size_t)((r1 - r0) * page_bytes);
        if ((rc = dskv_gather_pages(h->staging[0], pool, ids_dev, n_pages, n_layers,
                                    layer_stride_bytes, page_bytes, r0, r1, so)))
            return rc;
        DSKV_HIP(hipEventRecord(h->gathered[c], so));
        DSKV_HIP(hipMemcpyAsync((char *)host_dst + r0 * page_bytes, h->staging[0], bytes,
                                hipMemcpyDeviceToHost, so));
        if (same_buffer) continue;
        DSKV_HIP(hipMemcpyAsync(h->staging[1], (const char *)host_src + r0 * page_bytes, bytes,
                                hipMemcpyHostToDevice, si));
        DSKV_HIP(hipStreamWaitEvent(si, h->gathered[c], 0));   // pages of this chunk have left
        if ((rc = dskv_scatter_pages(pool, h->staging[1], ids_dev, n_pages, n_layers,
                                     layer_stride_bytes, page_bytes, r0, r1, si)))
            return rc;
    }
    if ((rc = close_direction(h, 0))) return rc;
    if ((rc = close_direction(h, 1))) return rc;
    ids_guard.seal();
    return 0;
}

extern "C" int dskv_swap_streams(dskv_swap_t *h, void **out_stream, void **in_stream)
{
    DSKV_REQUIRE(h && out_stream && in_stream, "swap_streams: null argument");
    *out_stream = h->stream[0];
    *in_stream = h->stream[1];
    h->streams_exported = true;
    return 0;
}

extern "C" int dskv_swap_bind_compute_stream(dskv_swap_t *h, void *compute_stream,
                                             int32_t *independent_out)
{
    using namespace dskv;
    DSKV_REQUIRE(h, "swap_bind_compute_stream: null handle");
    if (h->streams_exported) {
        // binding replaces streams that serialise with the compute stream, which would
        // destroy handles a caller already holds
        set_error("swap_bind_compute_stream: the engine's streams have been handed out "
                  "(dskv_swap_streams); bind before asking for them");
        return DSKV_E_STATE;
    }
    int rc = wait_all(h);
    if (rc) return rc;
    hipStream_t compute = (hipStream_t)compute_stream;
    int khz = 0;
    DSKV_HIP(hipDeviceGetAttribute(&khz, hipDeviceAttributeWallClockRate, h->device));
    const long ticks = (long)(khz > 0 ? khz : 100000) / 2;        // half a millisecond
    hipEvent_t ea = nullptr, eb = nullptr;
    DSKV_HIP(hipEventCreateWithFlags(&ea, hipEventDisableTiming));
    DSKV_HIP(hipEventCreateWithFlags(&eb, hipEventDisableTiming));
    // A stream is good if the compute stream runs beside it, and the second one also runs
    // beside the first (the two directions of an exchange overlap).  Rejected streams
    // stay alive until the search is over: the runtime gives a new stream the least
    // loaded queue, so they steer the next attempt to another queue.
    std::vector<hipStream_t> rejected;
    auto good = [&](hipStream_t s, int dir, bool *ok) -> int {
        bool beside = false;
        int r = runs_beside(s, compute, ea, eb, ticks, &beside);
        if (r) return r;
        if (beside && dir == 1) {
            r = runs_beside(h->stream[0], s, ea, eb, ticks, &beside);
            if (r) return r;
        }
        *ok = beside;
        return 0;
    };
    bool all_good = true;
    for (int dir = 0; dir < 2 && rc == 0; dir++) {
        bool ok = false;
        rc = good(h->stream[dir], dir, &ok);
        for (int attempt = 0; rc == 0 && !ok && attempt < 8; attempt++) {
            hipStream_t fresh = nullptr;
            hipError_t e = hipStreamCreateWithFlags(&fresh, hipStreamNonBlocking);
            if (e != hipSuccess) {
                set_error("swap_bind_compute_stream: hipStreamCreateWithFlags failed: %s",
                          hipGetErrorString(e));
                rc = (int)e;
                break;
            }
            rc = good(fresh, dir, &ok);
            if (rc == 0 && ok) {
                rejected.push_back(h->stream[dir]);
                h->stream[dir] = fresh;
            } else
                rejected.push_back(fresh);
        }
        all_good = all_good && ok;
    }
    for (hipStream_t s : rejected) (void)hipStreamDestroy(s);
    (void)hipEventDestroy(ea);
    (void)hipEventDestroy(eb);
    if (rc) return rc;
    h->probed = true;
    h->independent = all_good;
    h->dir_used[0] = h->dir_used[1] = false;      // everything was drained above
    if (independent_out) *independent_out = all_good ? 1 : 0;
    return 0;
}

extern "C" int dskv_swap_wait(dskv_swap_t *h)
{
    using namespace dskv;
    DSKV_REQUIRE(h, "swap_wait: null handle");
    return wait_all(h);
}

extern "C" int dskv_swap_query(dskv_swap_t *h, int32_t *done_out)
{
    using namespace dskv;
    DSKV_REQUIRE(h && done_out, "swap_query: null argument");
    *done_out = 1;
    for (int d = 0; d < 2; d++) {
        const hipError_t e = hipStreamQuery(h->stream[d]);
        if (e == hipErrorNotReady) {
            (void)hipGetLastError();
            *done_out = 0;
        } else if (e != hipSuccess) {
            set_error("swap_query: hipStreamQuery failed: %s", hipGetErrorString(e));
            return (int)e;
        }
    }
    return 0;
}

extern "C" int dskv_swap_fence(dskv_swap_t *h, void *stream)
{
    using namespace dskv;
    DSKV_REQUIRE(h, "swap_fence: null handle");
    for (int d = 0; d < 2; d++) {
        DSKV_HIP(hipEventRecord(h->fence, h->stream[d]));
        DSKV_HIP(hipStreamWaitEvent((hipStream_t)stream, h->fence, 0));
    }
    return 0;
}
