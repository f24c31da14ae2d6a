// Error text of the last failed call in this thread; every library links its own copy.
#include "ka_common.h"

#include <stdarg.h>
#include <stdio.h>

static thread_local char g_error[512];

void ka_set_error(const char* fmt, ...) {
    va_list ap;
    va_start(ap, fmt);
    vsnprintf(g_error, sizeof(g_error), fmt, ap);
    va_end(ap);
}

KA_API const char* ka_last_error() { return g_error; }
