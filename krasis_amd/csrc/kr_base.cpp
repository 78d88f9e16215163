// kr_base.cpp -- what every part of the library shares: the thread-local error text behind kr_last_error, the version, the allocation counter.
#include "kr_engine_internal.h"

static thread_local std::string g_err;
int kr_fail(int code, const char* fmt, ...) {
    char buf[1024];
    va_list ap; va_start(ap, fmt); vsnprintf(buf, sizeof buf, fmt, ap); va_end(ap);
    g_err = buf;
    return code;
}

extern "C" const char* kr_last_error(void) { return g_err.c_str(); }
extern "C" int kr_version(void) { return 1; }
extern "C" long kr_alloc_count_total(void) { return kr_alloc_count().load(std::memory_order_relaxed); }
