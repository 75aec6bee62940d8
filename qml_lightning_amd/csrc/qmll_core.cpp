// Error text and version of libqmll (host only).
#include <stdarg.h>
#include <stdio.h>

#include "../../include/qmll.h"

static thread_local char g_err[512] = "";

void qmll_set_error(const char* fmt, ...) {
    va_list ap;
    va_start(ap, fmt);
    vsnprintf(g_err, sizeof(g_err), fmt, ap);
    va_end(ap);
}

extern "C" const char* qmll_last_error(void) { return g_err; }
extern "C" int qmll_version(void) { return 1; }
