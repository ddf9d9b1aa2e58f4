// The error channel and the identification of the library.
#include "common.hpp"

#include <stdarg.h>
#include <stdio.h>

static thread_local char g_error[512] = "";

void pl_set_error(const char* fmt, ...) {
    va_list args;
    va_start(args, fmt);
    vsnprintf(g_error, sizeof(g_error), fmt, args);
    va_end(args);
}

extern "C" const char* pl_last_error() { return g_error; }

// Bumped when an entry point changes its arguments, so that a stale build is rebuilt.
extern "C" int pl_abi_version() { return 1; }
