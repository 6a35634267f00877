// Thread-local last-error string and version of librdkv_hip.so.
#include "rdkv_common.h"

#include <stdarg.h>

static thread_local char g_err[512] = "";

void rdkv_set_error(const char *fmt, ...) {
  va_list ap;
  va_start(ap, fmt);
  vsnprintf(g_err, sizeof(g_err), fmt, ap);
  va_end(ap);
}

RDKV_API int rdkv_version(void) { return 100; }

RDKV_API const char *rdkv_last_error(void) { return g_err; }
