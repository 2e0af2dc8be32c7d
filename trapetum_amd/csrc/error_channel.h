// The error channel's definitions: include in exactly one source file of each library.
#pragma once
#include "common.h"
#include <string>

static thread_local std::string g_error;
extern "C" const char* tp_last_error() { return g_error.c_str(); }
int tp_fail(const char* fmt, ...) {
    char buf[1024];
    va_list ap; va_start(ap, fmt); vsnprintf(buf, sizeof buf, fmt, ap); va_end(ap);
    g_error = buf;
    return 1;
}
int tp_check_launch(const char* what) {
    hipError_t e = hipGetLastError();
    if (e != hipSuccess) return tp_fail("%s: launch failed: %s", what, hipGetErrorString(e));
    return 0;
}
