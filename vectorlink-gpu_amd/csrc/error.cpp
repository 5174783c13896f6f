// Thread-local error text for the C ABI.
#include "vl_common.h"

static thread_local char g_err[512] = "";

void vl_set_error(const char *fmt, ...) {
    va_list ap;
    va_start(ap, fmt);
    vsnprintf(g_err, sizeof(g_err), fmt, ap);
    va_end(ap);
}

VL_EXPORT const char *vl_last_error(void) { return g_err; }
VL_EXPORT int vl_version(void) { return 1; }
