// Library-level entry points: version and thread-local error string.
#include "common.h"

static thread_local char g_err[512] = "";

int ptj_set_error(int code, const char* fmt, ...) {
    va_list ap;
    va_start(ap, fmt);
    vsnprintf(g_err, sizeof(g_err), fmt, ap);
    va_end(ap);
    return code;
}

extern "C" {
int ptj_version(void) { return 1; }
const char* ptj_last_error(void) { return g_err; }
}
