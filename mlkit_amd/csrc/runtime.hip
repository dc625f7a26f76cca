// Status reporting and version of libmlkit_amd.
#include <cstdarg>
#include <cstdio>

#include "mk_common.h"

namespace {
thread_local char last_error[512] = "";
}

int mk_fail(int code, const char *format, ...) {
    va_list arguments;
    va_start(arguments, format);
    vsnprintf(last_error, sizeof(last_error), format, arguments);
    va_end(arguments);
    return code;
}

extern "C" const char *mk_last_error(void) { return last_error; }

extern "C" const char *mk_version(void) { return "0.1.0"; }
