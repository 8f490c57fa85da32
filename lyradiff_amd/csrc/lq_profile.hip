// Set-up-time tactic profiler: times every tile configuration of a GEMM on one shape with synthetic
// operands and records the fastest in the per-shape cache.  Stands in for
// GemmPluginProfiler::profileTactics / profileTacticForProblem of lyraDiff
// (layers/gemm_utils/GemmProfiler.cc:78-127,161-265): same idea (warm-up runs, timed runs between two
// events, keep the minimum; here in interleaved rounds), but the caller owns the temporary memory and nothing is allocated here.
#include <algorithm>
#include "lq_common.h"
#include <type_traits>

namespace lq {

// Pseudo-random operand bytes (fp8: never a NaN code, so the timing is not distorted by NaN handling).
__global__ void profile_fill_bytes_kernel(uint8_t* dst, size_t n, int avoid_fp8_nan) {
    for (size_t i = (size_t)blockIdx.x * blockDim.x + threadIdx.x; i < n; i += (size_t)gridDim.x * blockDim.x) {
        u32 h = (u32)i * 2654435761u;
        h ^= h >> 15; h *= 2246822519u; h ^= h >> 13;
        uint8_t b = (uint8_t)(h >> 8);
        if (avoid_fp8_nan && (b & 0x7F) == 0x7F) b ^= 1;
        dst[i] = b;
    }
}
__global__ void profile_fill_f32_kernel(float* dst, size_t n, float v) {
    for (size_t i = (size_t)blockIdx.x * blockDim.x + threadIdx.x; i < n; i += (size_t)gridDim.x * blockDim.x) dst[i] = v;
}
__global__ void profile_fill_u16_kernel(unsigned short* dst, size_t n, unsigned short v) {
    for (size_t i = (size_t)blockIdx.x * blockDim.x + threadIdx.x; i < n; i += (size_t)gridDim.x * blockDim.x) dst[i] = v;
}

static size_t up256(size_t v) { return (v + 255) & ~(size_t)255; }

struct ProfileLayout {
    size_t a, b, c, s0, s1, total;  // byte offsets of A, B, C and the two scale arrays
    size_t a_bytes, b_bytes, s0_elems, s1_elems;
};

static ProfileLayout profile_layout(lq_weight_kind_t kind, int m, int n, int k) {
    ProfileLayout L = {};
    const size_t kb = lq_weight_row_bytes(kind, k);
    L.a_bytes = (size_t)m * kb;
    L.b_bytes = (size_t)n * kb;
    if (kind == LQ_W_INT8) { L.s0_elems = n; L.s1_elems = m; }                      // alpha_col, alpha_row (fp32)
    else if (kind == LQ_W_FP8) { L.s0_elems = 1; L.s1_elems = 1; }                  // a_scale, b_scale (fp32)
    else { L.s0_elems = (size_t)m * (k / 64); L.s1_elems = (size_t)n * (k / 64); }  // group scales (fp16)
    const size_t esz = kind == LQ_W_INT4 ? 2 : 4;
    L.a = 0;
    L.b = L.a + up256(L.a_bytes);
    L.c = L.b + up256(L.b_bytes);
    L.s0 = L.c + up256((size_t)m * n * 2);
    L.s1 = L.s0 + up256(L.s0_elems * esz);
    L.total = L.s1 + up256(L.s1_elems * esz);
    return L;
}

// One wavefront per workgroup reads the shader clock counter (s_memtime: ticks of the clock the compute units run at,
// which follows the power management) and the constant 100 MHz counter (s_memrealtime), idles with s_sleep until
// `realtime_ticks` of the latter have passed, and reads both again.  Launched on one stream while a kernel under study
// runs on another, the ratio of the two differences is the clock that kernel was actually given.
__global__ __launch_bounds__(64) void clock_probe_kernel(unsigned long long* out, unsigned long long realtime_ticks) {
    if (threadIdx.x != 0) return;
    const unsigned long long c0 = __builtin_readcyclecounter(), r0 = wall_clock64();
    unsigned long long r1 = r0;
    for (int spin = 0; spin < (1 << 24) && r1 - r0 < realtime_ticks; ++spin) {  // bounded: ends by itself in any case
        __builtin_amdgcn_s_sleep(32);
        r1 = wall_clock64();
    }
    const unsigned long long c1 = __builtin_readcyclecounter();
    out[2 * blockIdx.x] = c1 - c0;
    out[2 * blockIdx.x + 1] = r1 - r0;
}

}  // namespace lq

using namespace lq;

extern "C" int lq_shader_clock_probe(uint64_t* out_ticks, int probes, unsigned microseconds, lq_stream_t stream) {
    LQ_REQUIRE(out_ticks != nullptr && probes >= 1 && probes <= 1024, LQ_ERR_ARG, "lq_shader_clock_probe: need 1..1024 probes and an output buffer");
    LQ_REQUIRE(microseconds >= 1 && microseconds <= 100000, LQ_ERR_ARG, "lq_shader_clock_probe: 1..100000 microseconds");
    hipLaunchKernelGGL(clock_probe_kernel, dim3((unsigned)probes), dim3(64), 0, as_stream(stream),
                       reinterpret_cast<unsigned long long*>(out_ticks), (unsigned long long)microseconds * 100ull);
    return check_launch("lq_shader_clock_probe");
}

// What the matrix pipes alone sustain: every wavefront (one per SIMD, one workgroup per CU) issues 16 independent
// v_mfma_f32_32x32x64_f8f6f4 per step on operand fragments held in registers -- a 128x128 wavefront tile without any
// memory or LDS traffic.  Two sets of fragments (two k-steps' worth) alternate by unrolled index, so consecutive MFMAs never
// read the same pair of operand registers and nothing is written between them: no instruction of the loop depends on an
// MFMA in flight (an earlier form rotated the fragments' registers with 64 moves per step, whose destinations were sources
// of MFMAs still executing; its matrix pipes were busy three quarters of the time).  With operands drawn from real e4m3
// codes the part is power limited; with zeros it is not.
__global__ __launch_bounds__(256, 1) void mfma_fp8_probe_kernel(float* sink, const uint32_t* __restrict__ src, size_t src_words, int iters) {
    typedef int v8i_t __attribute__((ext_vector_type(8)));
    typedef float v16f_t __attribute__((ext_vector_type(16)));
    v8i_t a[2][4], b[2][4];
    const u32 words = src_words ? (u32)(src_words > 0x40000000u ? 0x40000000u : src_words) : 1u;
    const u32 start = (u32)(((size_t)blockIdx.x * 16384u) % words);
#pragma unroll
    for (int s = 0; s < 2; ++s)
#pragma unroll
        for (int f = 0; f < 4; ++f)
#pragma unroll
            for (int i = 0; i < 8; ++i) {
                // one division per thread (start); the offsets wrap by subtraction -- 128 64-bit divisions per thread took
                // longer than a thousand MFMAs
                u32 ia = start + (u32)s * 8192u + (threadIdx.x + 256u * f) * 8u + i;
                u32 ib = start + (u32)s * 8192u + (threadIdx.x + 256u * (f + 4)) * 8u + i;
                if (src) {
                    while (ia >= words) ia -= words;
                    while (ib >= words) ib -= words;
                }
                a[s][f][i] = src ? (int)src[ia] : 0;
                b[s][f][i] = src ? (int)src[ib] : 0;
            }
    v16f_t acc[16];
#pragma unroll
    for (int t = 0; t < 16; ++t)
#pragma unroll
        for (int i = 0; i < 16; ++i) acc[t][i] = 0.0f;
    auto step = [&](auto set_c) {
        constexpr int s = decltype(set_c)::value;
#pragma unroll
        for (int i = 0; i < 4; ++i)
#pragma unroll
            for (int j = 0; j < 4; ++j)
                acc[i * 4 + j] = __builtin_amdgcn_mfma_scale_f32_32x32x64_f8f6f4(a[s][i], b[s][j], acc[i * 4 + j], 0, 0, 0, 0, 0, 0);
    };
    int it = 0;
    for (; it + 1 < iters; it += 2) {
        step(std::integral_constant<int, 0>{});
        step(std::integral_constant<int, 1>{});
    }
    if (it < iters) step(std::integral_constant<int, 0>{});
    float sum = 0.0f;
#pragma unroll
    for (int t = 0; t < 16; ++t)
#pragma unroll
        for (int i = 0; i < 16; ++i) sum += acc[t][i];
    if (sum == 12345.678f) sink[0] = sum;  // keeps the loop alive; practically never taken
}

extern "C" int lq_mfma_fp8_probe(float* sink, const uint8_t* operand_codes, size_t n_codes, int iters, int* workgroups,
                                 lq_stream_t stream) {
    LQ_REQUIRE(sink != nullptr && iters >= 1 && iters <= (1 << 20), LQ_ERR_ARG, "lq_mfma_fp8_probe: need a sink and 1..2^20 iterations");
    LQ_REQUIRE(operand_codes == nullptr || (n_codes >= 4096 && reinterpret_cast<uintptr_t>(operand_codes) % 4 == 0), LQ_ERR_ARG,
               "lq_mfma_fp8_probe: operand codes must be 4-byte aligned and at least 4096 bytes");
    int dev = 0, cus = 0;
    LQ_REQUIRE(hipGetDevice(&dev) == hipSuccess &&
                   hipDeviceGetAttribute(&cus, hipDeviceAttributeMultiprocessorCount, dev) == hipSuccess && cus > 0,
               LQ_ERR_HIP, "lq_mfma_fp8_probe: cannot read the CU count");
    if (workgroups) *workgroups = cus;
    hipLaunchKernelGGL(mfma_fp8_probe_kernel, dim3((unsigned)cus), dim3(256), 0, as_stream(stream), sink,
                       reinterpret_cast<const uint32_t*>(operand_codes), n_codes / 4, iters);
    return check_launch("lq_mfma_fp8_probe");
}

extern "C" size_t lq_gemm_profile_workspace(lq_weight_kind_t kind, int m, int n, int k) {
    if (m <= 0 || n <= 0 || k <= 0 || lq_gemm_tactic_count(kind) < 0) return 0;
    return profile_layout(kind, m, n, k).total;
}

extern "C" int lq_gemm_profile(lq_weight_kind_t kind, int m, int n, int k, void* workspace, size_t workspace_bytes,
                               int* best_tactic, float* best_us, lq_stream_t stream) {
    const int count = lq_gemm_tactic_count(kind);
    if (count < 0) return count;
    LQ_REQUIRE(m > 0 && n > 0 && k > 0, LQ_ERR_SHAPE, "lq_gemm_profile: bad shape m=%d n=%d k=%d", m, n, k);
    const ProfileLayout L = profile_layout(kind, m, n, k);
    LQ_REQUIRE(workspace != nullptr && workspace_bytes >= L.total && reinterpret_cast<uintptr_t>(workspace) % 256 == 0,
               LQ_ERR_ARG, "lq_gemm_profile: workspace must be 256-byte aligned and hold %zu bytes (got %zu)", L.total,
               workspace_bytes);
    hipStream_t st = as_stream(stream);
    char* base = static_cast<char*>(workspace);
    hipLaunchKernelGGL(profile_fill_bytes_kernel, dim3(1024), dim3(256), 0, st, reinterpret_cast<uint8_t*>(base + L.a),
                       L.a_bytes, kind == LQ_W_FP8);
    hipLaunchKernelGGL(profile_fill_bytes_kernel, dim3(1024), dim3(256), 0, st, reinterpret_cast<uint8_t*>(base + L.b),
                       L.b_bytes, kind == LQ_W_FP8);
    if (kind == LQ_W_INT4) {
        hipLaunchKernelGGL(profile_fill_u16_kernel, dim3(256), dim3(256), 0, st, reinterpret_cast<unsigned short*>(base + L.s0),
                           L.s0_elems, (unsigned short)0x2C00);  // 1/16 as fp16
        hipLaunchKernelGGL(profile_fill_u16_kernel, dim3(256), dim3(256), 0, st, reinterpret_cast<unsigned short*>(base + L.s1),
                           L.s1_elems, (unsigned short)0x2C00);
    } else {
        hipLaunchKernelGGL(profile_fill_f32_kernel, dim3(256), dim3(256), 0, st, reinterpret_cast<float*>(base + L.s0),
                           L.s0_elems, 0.01f);
        hipLaunchKernelGGL(profile_fill_f32_kernel, dim3(256), dim3(256), 0, st, reinterpret_cast<float*>(base + L.s1),
                           L.s1_elems, 0.01f);
    }
    int rc = check_launch("lq_gemm_profile fill");
    if (rc != LQ_OK) return rc;

    auto run_once = [&]() -> int {
        void* C = base + L.c;
        switch (kind) {
            case LQ_W_INT8:
                return lq_gemm_int8(C, LQ_BF16, reinterpret_cast<const int8_t*>(base + L.a), reinterpret_cast<const int8_t*>(base + L.b),
                                    reinterpret_cast<const float*>(base + L.s0), reinterpret_cast<const float*>(base + L.s1), 1,
                                    nullptr, m, n, k, stream);
            case LQ_W_FP8:
                return lq_gemm_fp8(C, LQ_BF16, reinterpret_cast<const uint8_t*>(base + L.a), reinterpret_cast<const uint8_t*>(base + L.b),
                                   reinterpret_cast<const float*>(base + L.s0), reinterpret_cast<const float*>(base + L.s1), nullptr, 0,
                                   nullptr, 0.0f, m, n, k, stream);
            default:
                return lq_gemm_w4a4(C, LQ_BF16, reinterpret_cast<const uint32_t*>(base + L.a), reinterpret_cast<const uint8_t*>(base + L.b),
                                    base + L.s0, base + L.s1, LQ_F16, nullptr, m, n, k, 64, stream);
        }
    };

    hipEvent_t ev0, ev1;
    LQ_REQUIRE(hipEventCreate(&ev0) == hipSuccess && hipEventCreate(&ev1) == hipSuccess, LQ_ERR_HIP,
               "lq_gemm_profile: cannot create events");
    // Candidates are timed in interleaved rounds: on a power-limited part the clock
    // drifts over consecutive launches by more than the candidates differ, and a block of back-to-back runs per
    // candidate would rank them by when they ran.
    // Before that the built-in choice runs until two groups of ten launches agree to 1.5 % (at most 30 ms): from idle the
    // power management needs tens of milliseconds of load to settle, and until then every candidate looks faster than it
    // will be in a running pipeline, the power-hungry ones most of all.  A candidate's figure is the median of its rounds.
    constexpr int kRounds = 5, kRuns = 4, kMaxTactics = 16;
    {
        float prev = 0.0f, spent = 0.0f;
        for (int group = 0; group < 200 && spent < 30.0f; ++group) {
            bool ok = hipEventRecord(ev0, st) == hipSuccess;
            for (int i = 0; i < 10 && ok; ++i) ok = run_once() == LQ_OK;
            float ms = 0.0f;
            ok = ok && hipEventRecord(ev1, st) == hipSuccess && hipEventSynchronize(ev1) == hipSuccess &&
                 hipEventElapsedTime(&ms, ev0, ev1) == hipSuccess;
            if (!ok) { (void)hipGetLastError(); break; }
            spent += ms;
            if (prev > 0.0f && ms < prev * 1.015f && ms > prev * 0.985f) break;
            prev = ms;
        }
    }
    float rounds_of[kMaxTactics][kRounds];
    float best_of[kMaxTactics];
    bool usable[kMaxTactics];
    for (int t = 0; t < kMaxTactics; ++t) { best_of[t] = 0.0f; usable[t] = t < count; }
    for (int round = 0; round < kRounds + 1; ++round) {  // the first pass is the warm-up
        for (int t = 0; t < count && t < kMaxTactics; ++t) {
            if (!usable[t]) continue;
            tl_forced_tactic = t;
            bool ok = hipEventRecord(ev0, st) == hipSuccess;
            for (int i = 0; i < kRuns && ok; ++i) ok = run_once() == LQ_OK;
            if (ok) ok = hipEventRecord(ev1, st) == hipSuccess && hipEventSynchronize(ev1) == hipSuccess;
            float ms = 0.0f;
            if (ok) ok = hipEventElapsedTime(&ms, ev0, ev1) == hipSuccess;
            if (!ok) {
                (void)hipGetLastError();  // a configuration that cannot run this shape is skipped, as in the reference
                usable[t] = false;
                continue;
            }
            if (round > 0) rounds_of[t][round - 1] = ms;
        }
    }
    for (int t = 0; t < count && t < kMaxTactics; ++t) {
        if (!usable[t]) continue;
        std::sort(rounds_of[t], rounds_of[t] + kRounds);
        best_of[t] = rounds_of[t][kRounds / 2];
    }
    int best = -1;
    float best_ms = 0.0f;
    for (int t = 0; t < count && t < kMaxTactics; ++t)
        if (usable[t] && best_of[t] > 0.0f && (best < 0 || best_of[t] < best_ms)) { best = t; best_ms = best_of[t]; }
    tl_forced_tactic = -1;
    (void)hipEventDestroy(ev0);
    (void)hipEventDestroy(ev1);
    LQ_REQUIRE(best >= 0, LQ_ERR_UNSUPPORTED, "lq_gemm_profile: no configuration ran for m=%d n=%d k=%d", m, n, k);
    if (best_tactic) *best_tactic = best;
    if (best_us) *best_us = best_ms * 1000.0f / kRuns;
    return lq_gemm_set_shape_tactic(kind, m, n, k, best);
}
