// Shared helpers of the dskv library: error reporting across the C ABI and
// small device-side vector types.  gfx950 only.
#pragma once

#include <hip/hip_runtime.h>
#include <stdint.h>
#include <stdio.h>

#include "../../include/dskv.h"

namespace dskv {

// Message of the last failure on this thread (returned by dskv_last_error).
void set_error(const char *fmt, ...) __attribute__((format(printf, 1, 2)));

#define DSKV_REQUIRE(cond, ...)                \
    do {                                       \
        if (!(cond)) {                         \
            ::dskv::set_error(__VA_ARGS__);    \
            return DSKV_E_INVAL;               \
        }                                      \
    } while (0)

#define DSKV_HIP(expr)                                                          \
    do {                                                                        \
        hipError_t e_ = (expr);                                                 \
        if (e_ != hipSuccess) {                                                 \
            ::dskv::set_error("%s failed: %s", #expr, hipGetErrorString(e_));   \
            return (int)e_;                                                     \
        }                                                                       \
    } while (0)

// Kernel launches report configuration errors through hipGetLastError.
#define DSKV_LAUNCH_CHECK(name)                                                  \
    do {                                                                         \
        hipError_t e_ = hipGetLastError();                                       \
        if (e_ != hipSuccess) {                                                  \
            ::dskv::set_error("launch of %s failed: %s", name, hipGetErrorString(e_)); \
            return (int)e_;                                                      \
        }                                                                        \
    } while (0)

typedef uint32_t u32x4 __attribute__((ext_vector_type(4)));
typedef uint32_t u32x2 __attribute__((ext_vector_type(2)));
typedef float f32x4 __attribute__((ext_vector_type(4)));
typedef float f32x16 __attribute__((ext_vector_type(16)));

// Merge pass over per-part partials (max, sum, unnormalised O) in a workspace laid out as
// [max_slots x n_qo_heads x head_dim] floats of O followed by [max_slots x n_qo_heads x 2] of
// (max, sum): row r of `out` (rows x n_qo_heads x head_dim, of `dtype`) is merged from the
// row_parts[2r + 1] parts that start at slot row_parts[2r]; rows with no parts are left
// alone.  `wide`: eight waves per (row, head), for rows cut into dozens of parts.  Defined
// beside the decode attention kernels, which write such partials.
// row_map (may be null): request r's output row is row_map[r] instead of r.
int launch_partials_merge(void *out, const float *part_o, const float *part_ml,
                          const int32_t *row_parts, const int32_t *row_map, int max_slots, int rows,
                          int n_qo_heads, int head_dim, int dtype, bool wide, hipStream_t stream);

// The split-KV decode path for requests that are rows of a ragged batch (the one-row
// requests of a prefill batch): request i has `len` kv tokens, its block table starts at
// entry `page_begin` of the table array, and its query and output are row `row` of q and out.
// plan_decode_rows is dskv_decode_plan over such a list (same plan layout, the items name the
// rows); decode_rows_attn is dskv_decode_attn over that plan, with row_map[i] = reqs[i].row on
// the device for the merge pass.  decode_mfma_shape: whether the 16-bit decode kernel takes
// the shape (the routing is only worth it then).
struct DecodeRow {
    int64_t len;
    int32_t page_begin, row;
};
int plan_decode_rows(const DecodeRow *reqs, int32_t batch, int32_t n_qo_heads, int32_t head_dim,
                     int32_t target_workgroups, int32_t *plan_host, int64_t plan_capacity_words,
                     int32_t *n_items_out, int32_t *n_workgroups_out, int64_t *plan_words_out,
                     int64_t *workspace_bytes_out);
int decode_rows_attn(void *out, const void *q, const void *pages_layer,
                     const int32_t *kv_page_indices, const int32_t *plan_dev, int32_t n_items,
                     int32_t n_workgroups, void *workspace, int64_t workspace_bytes, int32_t n_rows,
                     const int32_t *row_map, int32_t n_qo_heads, int32_t n_kv_heads,
                     int32_t head_dim, int32_t page_size, float sm_scale, int32_t dtype,
                     hipStream_t stream);
bool decode_mfma_shape(int head_dim, int n_qo_heads, int n_kv_heads, int page_size);

static inline bool is_pow2(int64_t x) { return x > 0 && (x & (x - 1)) == 0; }
static inline int ilog2(int64_t x) {
    int s = 0;
    while ((int64_t(1) << s) < x) s++;
    return s;
}

}  // namespace dskv
