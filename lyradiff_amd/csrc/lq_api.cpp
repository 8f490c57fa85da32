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

// ---- the per-shape cache as a byte string: "LQT1", entry count, then {kind, m, n, k, tactic} as little-endian int32 ----
static const unsigned kTacticsMagic = 0x3154514Cu;  // "LQT1"

extern "C" size_t lq_gemm_tactics_serialized_size(void) {
    std::shared_lock<std::shared_timed_mutex> lock(lq::g_shape_mutex);
    return 8 + lq::g_shape_tactics.size() * 20;
}

extern "C" int lq_gemm_tactics_serialize(void* buffer, size_t buffer_bytes, size_t* written) {
    if (buffer == nullptr) {
        lq::set_error("lq_gemm_tactics_serialize: null buffer");
        return LQ_ERR_ARG;
    }
    std::shared_lock<std::shared_timed_mutex> lock(lq::g_shape_mutex);
    const size_t need = 8 + lq::g_shape_tactics.size() * 20;
    if (buffer_bytes < need) {
        lq::set_error("lq_gemm_tactics_serialize: the buffer holds %zu bytes, %zu are needed", buffer_bytes, need);
        return LQ_ERR_ARG;
    }
    int* out = static_cast<int*>(buffer);
    *out++ = (int)kTacticsMagic;
    *out++ = (int)lq::g_shape_tactics.size();
    for (auto const& e : lq::g_shape_tactics) {
        *out++ = std::get<0>(e.first);
        *out++ = std::get<1>(e.first);
        *out++ = std::get<2>(e.first);
        *out++ = std::get<3>(e.first);
        *out++ = e.second;
    }
    if (written) *written = need;
    return LQ_OK;
}

extern "C" int lq_gemm_tactics_deserialize(const void* data, size_t bytes) {
    const int* in = static_cast<const int*>(data);
    if (data == nullptr || bytes < 8 || (unsigned)in[0] != kTacticsMagic || in[1] < 0 || (size_t)in[1] > (bytes - 8) / 20) {
        lq::set_error("lq_gemm_tactics_deserialize: not a tactic table (%zu bytes)", bytes);
        return LQ_ERR_ARG;
    }
    const int count = in[1];
    for (int i = 0; i < count; ++i) {  // validate everything before anything is stored
        const int* e = in + 2 + 5 * i;
        const int tactics = lq_gemm_tactic_count((lq_weight_kind_t)e[0]);
        if (tactics < 0 || e[1] <= 0 || e[2] <= 0 || e[3] <= 0 || e[4] < 0 || e[4] >= tactics) {
            lq::set_error("lq_gemm_tactics_deserialize: entry %d is invalid (kind %d, m %d, n %d, k %d, tactic %d)", i, e[0], e[1], e[2], e[3], e[4]);
            return LQ_ERR_ARG;
        }
    }
    std::unique_lock<std::shared_timed_mutex> lock(lq::g_shape_mutex);
    for (int i = 0; i < count; ++i) {
        const int* e = in + 2 + 5 * i;
        lq::g_shape_tactics[std::make_tuple(e[0], e[1], e[2], e[3])] = e[4];
    }
    lq::g_shape_entries.store((int)lq::g_shape_tactics.size(), std::memory_order_relaxed);
    return LQ_OK;
}
