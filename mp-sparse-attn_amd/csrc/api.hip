// Version and error reporting of libmpsa.
#include "mpsa_common.h"

static thread_local char g_err[512] = "";

int mpsa_fail(int code, const char* fmt, ...) {
    va_list ap;
    va_start(ap, fmt);
    vsnprintf(g_err, sizeof(g_err), fmt, ap);
    va_end(ap);
    return code;
}

extern "C" int mpsa_version(void) { return 100; }
extern "C" const char* mpsa_last_error(void) { return g_err; }
