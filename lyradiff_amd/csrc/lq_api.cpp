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

namespace lq {
extern int g_tactic_int8, g_tactic_fp8, g_tactic_w4a4;
}
extern "C" int lq_gemm_set_tactic(lq_weight_kind_t kind, int tactic) {
    switch (kind) {
        case LQ_W_INT8: lq::g_tactic_int8 = tactic; return LQ_OK;
        case LQ_W_FP8: lq::g_tactic_fp8 = tactic; return LQ_OK;
        case LQ_W_INT4: lq::g_tactic_w4a4 = tactic; return LQ_OK;
        default: lq::set_error("lq_gemm_set_tactic: bad kind %d", (int)kind); return LQ_ERR_ARG;
    }
}
