#include "spinf_tree.h"
#include "common.h"

static thread_local char g_err[512] = "";

int spinf_fail(int code, const char* fmt, ...) {
    va_list ap;
    va_start(ap, fmt);
    vsnprintf(g_err, sizeof(g_err), fmt, ap);
    va_end(ap);
    return code;
}

extern "C" const char* spinf_last_error(void) { return g_err; }
extern "C" int spinf_version(void) { return 1; }
