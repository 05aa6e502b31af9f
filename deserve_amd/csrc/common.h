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
int launch_partials_merge(void *out, const float *part_o, const float *part_ml,
                          const int32_t *row_parts, int max_slots, int rows, int n_qo_heads,
                          int head_dim, int dtype, bool wide, hipStream_t stream);

static inline bool is_pow2(int64_t x) { return x > 0 && (x & (x - 1)) == 0; }
static inline int ilog2(int64_t x) {
    int s = 0;
    while ((int64_t(1) << s) < x) s++;
    return s;
}

}  // namespace dskv
