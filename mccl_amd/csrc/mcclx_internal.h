// mcclx_internal.h -- shared by the translation units of libmcclx.so only.
#pragma once

// Records the calling thread's error message (what mcclx_last_error() returns)
// and hands back `code`.
extern "C" __attribute__((visibility("hidden"))) int mcclx_fail(int code, const char* fmt, ...)
    __attribute__((format(printf, 2, 3)));
