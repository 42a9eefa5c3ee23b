// Thread-local error slot and version of libodmkv.
#include "common.h"

static thread_local char g_err[512] = "";

void odmkv_set_error(const char* fmt, ...) {
    va_list ap;
    va_start(ap, fmt);
    vsnprintf(g_err, sizeof(g_err), fmt, ap);
    va_end(ap);
}

extern "C" int odmkv_version(void) { return ODMKV_VERSION; }
extern "C" const char* odmkv_last_error(void) { return g_err; }
