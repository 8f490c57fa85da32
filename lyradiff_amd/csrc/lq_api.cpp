// Error plumbing and version of liblyraquant.
#include <stdarg.h>
#include <stdio.h>

#include "lyraquant.h"

namespace lq {
static thread_local char g_err[512] = "";
void set_error(const char* fmt, ...) {
    va_list ap;
    va_start(ap, fmt);
    vsnprintf(g_err, sizeof(g_err), fmt, ap);
    va_end(ap);
}
}  // namespace lq

extern "C" const char* lq_last_error(void) { return lq::g_err; }
extern "C" int lq_version(void) { return 100; }
