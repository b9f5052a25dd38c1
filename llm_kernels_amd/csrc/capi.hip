// Library-level entry points: version, thread-local error text.
#include "common.hpp"

static thread_local char g_err[512] = "";

void llmk_set_error(const char* fmt, ...) {
    va_list ap;
    va_start(ap, fmt);
    vsnprintf(g_err, sizeof(g_err), fmt, ap);
    va_end(ap);
}

extern "C" int llmk_version(void) { return 100; }

extern "C" const char* llmk_last_error(void) { return g_err; }
