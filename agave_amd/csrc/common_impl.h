// Definitions that every kernel library carries once: the last-error buffer.
#pragma once
#include <stdarg.h>
#include "common.h"

static thread_local char g_agave_error[512] = "";

void agave_set_error(const char* fmt, ...) {
    va_list ap;
    va_start(ap, fmt);
    vsnprintf(g_agave_error, sizeof(g_agave_error), fmt, ap);
    va_end(ap);
}

extern "C" const char* agave_last_error() { return g_agave_error; }
