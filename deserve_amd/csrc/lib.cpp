// Error reporting and version of the dskv C ABI.
#include <stdarg.h>
#include <stdio.h>

#include "../../include/dskv.h"

namespace dskv {

static thread_local char g_error[512] = "";

void set_error(const char *fmt, ...) __attribute__((format(printf, 1, 2)));
void set_error(const char *fmt, ...)
{
    va_list ap;
    va_start(ap, fmt);
    vsnprintf(g_error, sizeof(g_error), fmt, ap);
    va_end(ap);
}

}  // namespace dskv

extern "C" const char *dskv_last_error(void) { return dskv::g_error; }
// Bumped whenever an exported signature changes (2: num_pages argument of the append entry
// points, kv lengths / parts in the prefill plan; 3: plans that route one-row requests of a
// prefill batch to the decode kernel).
extern "C" int dskv_version(void) { return DSKV_ABI_VERSION; }
