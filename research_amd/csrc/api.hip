// Error reporting and small host-only entry points of libpaged_attn.
#include <stdarg.h>
#include <stdio.h>

#include "pa_common.h"

namespace {
thread_local char g_last_error[512] = "";
}

int pa_fail(int code, const char *fmt, ...) {
    va_list ap;
    va_start(ap, fmt);
    vsnprintf(g_last_error, sizeof(g_last_error), fmt, ap);
    va_end(ap);
    return code;
}

void pa_clear_error() { g_last_error[0] = '\0'; }

extern "C" int pa_version(void) { return 6; }

extern "C" const char *pa_last_error(void) { return g_last_error; }

extern "C" int pa_dtype_bytes(int dtype) {
    switch (dtype) {
    case PA_F32: return 4;
    case PA_BF16:
    case PA_F16: return 2;
    case PA_FP8_E4M3: return 1;
    default: return 0;
    }
}
