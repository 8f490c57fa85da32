// Error plumbing and version of liblyraquant.
#include <stdarg.h>
#include <stdio.h>

#include <atomic>
#include <map>
#include <mutex>
#include <shared_mutex>
#include <tuple>

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
int g_tactic_int8 = -1, g_tactic_fp8 = -1, g_tactic_w4a4 = -1;  // -1: shape cache, then the built-in table
thread_local int tl_forced_tactic = -1;                         // set by lq_gemm_profile around a timed call

// Per-shape tactic cache (the role of the reference's MNKProfileMap, layers/gemm_utils/GemmProfiler.h:131-251):
// key (kind, m, n, k); a lookup tries the exact m and then m rounded up to a power of two, the bucket the
// reference's getBestConfig uses (GemmProfiler.cc:131-143).  Read-mostly: readers take a shared lock only when the
// cache is not empty.
static std::shared_timed_mutex g_shape_mutex;
static std::map<std::tuple<int, int, int, int>, int> g_shape_tactics;
static std::atomic<int> g_shape_entries{0};

static int next_pow2(int v) {
    int p = 1;
    while (p < v && p < (1 << 30)) p <<= 1;
    return p;
}

int shape_tactic_lookup(int kind, int m, int n, int k) {
    if (g_shape_entries.load(std::memory_order_relaxed) == 0) return -1;
    std::shared_lock<std::shared_timed_mutex> lock(g_shape_mutex);
    auto it = g_shape_tactics.find(std::make_tuple(kind, m, n, k));
    if (it == g_shape_tactics.end()) it = g_shape_tactics.find(std::make_tuple(kind, next_pow2(m), n, k));
    return it == g_shape_tactics.end() ? -1 : it->second;
}
}  // namespace lq

extern "C" int lq_gemm_set_tactic(lq_weight_kind_t kind, int tactic) {
    switch (kind) {
        case LQ_W_INT8: lq::g_tactic_int8 = tactic; return LQ_OK;
        case LQ_W_FP8: lq::g_tactic_fp8 = tactic; return LQ_OK;
        case LQ_W_INT4: lq::g_tactic_w4a4 = tactic; return LQ_OK;
        default: lq::set_error("lq_gemm_set_tactic: bad kind %d", (int)kind); return LQ_ERR_ARG;
    }
}

extern "C" int lq_gemm_set_thread_tactic(int tactic) {
    lq::tl_forced_tactic = tactic < 0 ? -1 : tactic;
    return LQ_OK;
}

extern "C" int lq_gemm_tactic_count(lq_weight_kind_t kind) {
    switch (kind) {
        case LQ_W_INT8: return 8;
        case LQ_W_FP8: return 8;
        case LQ_W_INT4: return 3;
        default: lq::set_error("lq_gemm_tactic_count: bad kind %d", (int)kind); return LQ_ERR_ARG;
    }
}

extern "C" int lq_gemm_set_shape_tactic(lq_weight_kind_t kind, int m, int n, int k, int tactic) {
    const int count = lq_gemm_tactic_count(kind);
    if (count < 0) return count;
    if (tactic >= count || m <= 0 || n <= 0 || k <= 0) {
        lq::set_error("lq_gemm_set_shape_tactic: bad argument (m=%d n=%d k=%d tactic=%d of %d)", m, n, k, tactic, count);
        return LQ_ERR_ARG;
    }
    std::unique_lock<std::shared_timed_mutex> lock(lq::g_shape_mutex);
    const auto key = std::make_tuple((int)kind, m, n, k);
    if (tactic < 0) lq::g_shape_tactics.erase(key);
    else lq::g_shape_tactics[key] = tactic;
    lq::g_shape_entries.store((int)lq::g_shape_tactics.size(), std::memory_order_relaxed);
    return LQ_OK;
}

extern "C" int lq_gemm_get_shape_tactic(lq_weight_kind_t kind, int m, int n, int k) {
    return lq::shape_tactic_lookup((int)kind, m, n, k);
}
