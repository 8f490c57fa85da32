// FP8 e4m3 GEMM entry point (fp32 accumulation on v_mfma_f32_32x32x64_f8f6f4) with the fused
// per-tensor scale, bias, optional tanh-GELU and residual epilogue.  Reference contract:
// utils/cublasMMWrapper.cc:1104-1274 of lyraDiff (cuBLASLt FP8 matmul with A/B scale pointers and
// BIAS / GELU_BIAS epilogues).
#include "lq_gemm_core.h"

namespace lq {


template <typename OutTag> static constexpr lq_dtype_t out_enum() {
    return std::is_same<OutTag, F16Tag>::value ? LQ_F16 : std::is_same<OutTag, BF16Tag>::value ? LQ_BF16 : LQ_F32;
}

template <typename OutTag> static int run_fp8(GemmParams p, hipStream_t st) {
    int t = requested_tactic(g_tactic_fp8, LQ_W_FP8, p.m, p.n, p.k);
    // scales and bias, and at most the running maximum of the outputs (two instructions per four outputs)
    const bool plain_epilogue = p.gelu == 0 && p.out_scale == nullptr && p.C8 == nullptr && p.gate == nullptr &&
                                p.residual == nullptr && p.addend == nullptr;
    if (t < 0) {
        const long t256 = (long)((p.m + 255) / 256) * ((p.n + 255) / 256);
        const long t128 = (long)((p.m + 127) / 128) * ((p.n + 127) / 128);
        // 256x256 tiles, one wavefront per SIMD, when their last round on the 256 CUs is at least half full (measured on
        // the FLUX shapes at 4608 and 6912 rows, FP8 and INT8: ahead of the others by up to 10 % then, level or up to 4 %
        // behind otherwise); else 128x256 tiles, two workgroups per CU (finer tail, one workgroup's epilogue overlaps the
        // other's MFMA work)
        const long last256 = t256 % 256;
        t = t256 >= 192 ? ((last256 == 0 || last256 >= 128) ? 6 : 4) : (t128 >= 128 ? 2 : 3);  // 128x128 tiles from half a round up (4096x640x2560: 14.5 against 16.3 us with 64x64)
        if (p.k <= 1024 && t128 >= 192) t = 2;  // short K: prologue and epilogue dominate, smaller tiles overlap them better
        // More full 256x256 tiles than CUs and nothing but scales and bias in the epilogue: the persistent form
        // (4608x12288x3072: 134-140 us against 148 with 128x256 tiles, 6912x9216x3072: 156 against 161 with tactic 6)
        if (plain_epilogue && t256 > device_cu_count() && p.m % 256 == 0 && p.n % 256 == 0 && p.kb % 128 == 0 && p.k > 1024 &&
            out_enum<OutTag>() != LQ_F32)
            t = 7;
    }
    if (t == 1 && (p.kb % 128 != 0 || p.a_panel)) t = 0;  // the 128-byte k-tile needs k % 128 == 0 and a row-major activation
    // The per-shape cache is filled by timing the plain epilogue.  With one wavefront per SIMD nothing runs beside tactic 6's
    // epilogue: one that does more than scale and bias (activation, output maximum, codes, gate, residual) costs 13-18 us
    // per 256x256 tile there (transcendentals, or one exposed memory round trip per group of rows) and next to nothing with
    // two wavefronts per SIMD.  Measured at 4608 rows: 12288x3072 with GELU and the output maximum 209-214 us against
    // 153-160 us with tactic 4; 3072x12288 with gate and residual 139 us against 134 us with tactic 0, 3072x3072 55 against
    // 48 us.  A configuration forced by the caller is kept.
    const bool forced = tl_forced_tactic >= 0 || g_tactic_fp8 >= 0;
    if (t == 6 && !forced && p.out_max != nullptr) t = (long)((p.m + 255) / 256) * ((p.n + 255) / 256) > 256 ? 4 : 0;  // outside the persistent form the running maximum takes the activation epilogue
    if ((t == 6 || t == 7) && !forced && !plain_epilogue) t = (long)((p.m + 255) / 256) * ((p.n + 255) / 256) > 256 ? 4 : 0;
    if (t == 7) {  // the persistent form of tactic 6 where it applies, tactic 6 itself elsewhere
        const int rc = launch_persist_fp8(p, out_enum<OutTag>(), st);
        if (rc != 1) return rc;
        t = 6;
    }
    switch (t) {
        case 0: return launch_gemm<K_FP8, OutTag, 256, 256, 64, 2, 4, 3>(p, st);
        case 1: return launch_gemm<K_FP8, OutTag, 256, 256, 128, 2, 4, 2>(p, st);
        case 2: return launch_gemm<K_FP8, OutTag, 128, 128, 64, 2, 2, 3>(p, st);
        case 3: return launch_gemm<K_FP8, OutTag, 64, 64, 64, 2, 2, 3>(p, st);
        case 4: return launch_gemm<K_FP8, OutTag, 128, 256, 64, 2, 2, 3>(p, st);
        case 5: return launch_gemm<K_FP8, OutTag, 256, 128, 64, 2, 2, 3>(p, st);
        case 6: return launch_gemm<K_FP8, OutTag, 256, 256, 64, 2, 2, 4>(p, st);  // one wavefront per SIMD, 128x128 wavefront tiles
        default: set_error("lq_gemm_fp8: unknown tactic %d", t); return LQ_ERR_ARG;
    }
}

}  // namespace lq

using namespace lq;

// LQ_OK: go on; 1: m == 0, nothing to do (pointers of empty tensors may be null); negative: error
static int fp8_check(const char* what, const void* C, const uint8_t* A, const uint8_t* B, const float* a_scale, const float* b_scale,
                     const void* bias, const void* residual, int m, int n, int k) {
    LQ_REQUIRE(m >= 0 && n > 0 && k > 0 && n % 32 == 0 && k % 64 == 0, LQ_ERR_SHAPE,
               "%s: need n %% 32 == 0 and k %% 64 == 0 (m=%d n=%d k=%d)", what, m, n, k);
    if (m == 0) return 1;
    LQ_REQUIRE(A && B && a_scale && b_scale, LQ_ERR_ARG, "%s: null pointer", what);
    LQ_REQUIRE(reinterpret_cast<uintptr_t>(A) % 16 == 0 && reinterpret_cast<uintptr_t>(B) % 16 == 0 &&
                   reinterpret_cast<uintptr_t>(C) % 16 == 0 && reinterpret_cast<uintptr_t>(bias) % 8 == 0 &&
                   reinterpret_cast<uintptr_t>(residual) % 16 == 0,
               LQ_ERR_ARG, "%s: A, B, C, residual must be 16-byte aligned, bias 8-byte aligned", what);
    return LQ_OK;
}

static int fp8_dispatch(const char* what, const GemmParams& p, lq_dtype_t out_dtype, lq_stream_t stream) {
    hipStream_t st = as_stream(stream);
    switch (out_dtype) {
        case LQ_F16: return run_fp8<F16Tag>(p, st);
        case LQ_BF16: return run_fp8<BF16Tag>(p, st);
        case LQ_F32: return run_fp8<F32Tag>(p, st);
        default: set_error("%s: unsupported output dtype %d", what, (int)out_dtype); return LQ_ERR_UNSUPPORTED;
    }
}

extern "C" int lq_gemm_fp8_ex(void* C, lq_dtype_t out_dtype, const uint8_t* A, const uint8_t* B_rows32,
                              const float* a_scale, const float* b_scale, const void* bias, int gelu,
                              const void* residual, float beta, int m, int n, int k, float* out_scale, uint8_t* C_fp8,
                              const float* C_fp8_scale, lq_stream_t stream) {
    int rc = fp8_check("lq_gemm_fp8", C, A, B_rows32, a_scale, b_scale, bias, residual, m, n, k);
    if (rc != LQ_OK) return rc > 0 ? LQ_OK : rc;
    LQ_REQUIRE(C || C_fp8, LQ_ERR_ARG, "lq_gemm_fp8: null pointer");
    LQ_REQUIRE((C_fp8 == nullptr) == (C_fp8_scale == nullptr), LQ_ERR_ARG, "lq_gemm_fp8: C_fp8 and C_fp8_scale go together");
    LQ_REQUIRE(reinterpret_cast<uintptr_t>(C_fp8) % 4 == 0, LQ_ERR_ARG, "lq_gemm_fp8: C_fp8 must be 4-byte aligned");
    LQ_REQUIRE(gelu >= 0 && gelu <= 2, LQ_ERR_ARG, "lq_gemm_fp8: gelu must be 0, 1 or 2");
    if (m == 0) return LQ_OK;
    GemmParams p = {};
    p.C = C; p.A = A; p.B = B_rows32; p.bias = bias; p.a_scale = a_scale; p.b_scale = b_scale;
    p.gelu = gelu; p.residual = (beta != 0.0f) ? residual : nullptr; p.beta = beta;
    p.out_scale = out_scale; p.C8 = C_fp8; p.c8_scale = C_fp8_scale; p.ldc8 = (size_t)n;
    p.m = m; p.n = n; p.k = k; p.kb = k;
    // with out_scale the 16-bit output exists to be cast once with that scale; a large one bypasses the cache on its way out
    p.stream_c = out_scale != nullptr && C != nullptr && (size_t)m * (size_t)n * (out_dtype == LQ_F32 ? 4 : 2) >= kStreamBytes;
    return fp8_dispatch("lq_gemm_fp8", p, out_dtype, stream);
}

extern "C" int lq_gemm_fp8_max(void* C, lq_dtype_t out_dtype, const uint8_t* A, const uint8_t* B_rows32, const float* a_scale,
                               const float* b_scale, const void* bias, int m, int n, int k, float* out_max, lq_stream_t stream) {
    int rc = fp8_check("lq_gemm_fp8_max", C, A, B_rows32, a_scale, b_scale, bias, nullptr, m, n, k);
    if (rc != LQ_OK) return rc > 0 ? LQ_OK : rc;
    LQ_REQUIRE(C && out_max, LQ_ERR_ARG, "lq_gemm_fp8_max: null pointer");
    GemmParams p = {};
    p.C = C; p.A = A; p.B = B_rows32; p.bias = bias; p.a_scale = a_scale; p.b_scale = b_scale;
    p.out_max = out_max; p.ldc8 = (size_t)n;
    p.m = m; p.n = n; p.k = k; p.kb = k;
    // the output exists to be read once by the activation + cast pass; a large one bypasses the cache on its way out (the
    // two-workgroups-per-CU kernels only: the persistent kernel's counted waits do not get along with such stores)
    p.stream_c = (size_t)m * (size_t)n * (out_dtype == LQ_F32 ? 4 : 2) >= kStreamBytes;
    return fp8_dispatch("lq_gemm_fp8_max", p, out_dtype, stream);
}

extern "C" int lq_gemm_fp8_panels(void* C, lq_dtype_t out_dtype, const uint8_t* A_panels, const uint8_t* B_rows32,
                                  const float* a_scale, const float* b_scale, const void* bias, int m, int n, int k,
                                  float* out_max, lq_stream_t stream) {
    int rc = fp8_check("lq_gemm_fp8_panels", C, A_panels, B_rows32, a_scale, b_scale, bias, nullptr, m, n, k);
    if (rc != LQ_OK) return rc > 0 ? LQ_OK : rc;
    LQ_REQUIRE(C, LQ_ERR_ARG, "lq_gemm_fp8_panels: null pointer");
    GemmParams p = {};
    p.C = C; p.A = A_panels; p.B = B_rows32; p.bias = bias; p.a_scale = a_scale; p.b_scale = b_scale;
    p.out_max = out_max; p.ldc8 = (size_t)n;
    p.m = m; p.n = n; p.k = k; p.kb = k;
    p.a_panel = 1;
    p.stream_c = out_max != nullptr && (size_t)m * (size_t)n * (out_dtype == LQ_F32 ? 4 : 2) >= kStreamBytes;  // as lq_gemm_fp8_max
    return fp8_dispatch("lq_gemm_fp8_panels", p, out_dtype, stream);
}

extern "C" int lq_gemm_fp8(void* C, lq_dtype_t out_dtype, const uint8_t* A, const uint8_t* B_rows32,
                           const float* a_scale, const float* b_scale, const void* bias, int gelu,
                           const void* residual, float beta, int m, int n, int k, lq_stream_t stream) {
    LQ_REQUIRE(C != nullptr || m == 0, LQ_ERR_ARG, "lq_gemm_fp8: null pointer");
    return lq_gemm_fp8_ex(C, out_dtype, A, B_rows32, a_scale, b_scale, bias, gelu, residual, beta, m, n, k, nullptr, nullptr,
                          nullptr, stream);
}

static int gemm_fp8_gated(void* C, lq_dtype_t out_dtype, const uint8_t* A, const uint8_t* B_rows32,
                                 const float* a_scale, const float* b_scale, const void* bias, const void* gate,
                                 size_t rows_per_gate, const void* residual, int m, int n, int k, int a_panel, lq_stream_t stream) {
    int rc = fp8_check("lq_gemm_fp8_gated", C, A, B_rows32, a_scale, b_scale, bias, residual, m, n, k);
    if (rc != LQ_OK) return rc > 0 ? LQ_OK : rc;
    LQ_REQUIRE(C && gate && residual, LQ_ERR_ARG, "lq_gemm_fp8_gated: null pointer");
    LQ_REQUIRE(rows_per_gate > 0, LQ_ERR_SHAPE, "lq_gemm_fp8_gated: rows_per_gate must be positive");
    LQ_REQUIRE(reinterpret_cast<uintptr_t>(gate) % 16 == 0, LQ_ERR_ARG, "lq_gemm_fp8_gated: gate must be 16-byte aligned");
    if (m == 0) return LQ_OK;
    GemmParams p = {};
    p.C = C; p.A = A; p.B = B_rows32; p.bias = bias; p.a_scale = a_scale; p.b_scale = b_scale;
    p.residual = residual; p.beta = 1.0f; p.gate = gate; p.gate_rows = rows_per_gate; p.ldc8 = (size_t)n;
    p.m = m; p.n = n; p.k = k; p.kb = k;
    p.a_panel = a_panel;
    return fp8_dispatch("lq_gemm_fp8_gated", p, out_dtype, stream);
}

extern "C" int lq_gemm_fp8_gated(void* C, lq_dtype_t out_dtype, const uint8_t* A, const uint8_t* B_rows32, const float* a_scale,
                                 const float* b_scale, const void* bias, const void* gate, size_t rows_per_gate, const void* residual,
                                 int m, int n, int k, lq_stream_t stream) {
    return gemm_fp8_gated(C, out_dtype, A, B_rows32, a_scale, b_scale, bias, gate, rows_per_gate, residual, m, n, k, 0, stream);
}

extern "C" int lq_gemm_fp8_gated_panels(void* C, lq_dtype_t out_dtype, const uint8_t* A_panels, const uint8_t* B_rows32,
                                        const float* a_scale, const float* b_scale, const void* bias, const void* gate,
                                        size_t rows_per_gate, const void* residual, int m, int n, int k, lq_stream_t stream) {
    return gemm_fp8_gated(C, out_dtype, A_panels, B_rows32, a_scale, b_scale, bias, gate, rows_per_gate, residual, m, n, k, 1, stream);
}

static int gemm_fp8_codes(uint8_t* C_fp8, size_t ldc, const float* C_fp8_scale, lq_dtype_t round_dtype,
                                 const uint8_t* A, const uint8_t* B_rows32, const float* a_scale, const float* b_scale,
                                 const void* bias, int gelu, int m, int n, int k, int panels, lq_stream_t stream) {
    LQ_REQUIRE(gelu >= 0 && gelu <= 2, LQ_ERR_ARG, "lq_gemm_fp8_codes: gelu must be 0, 1 or 2");
    LQ_REQUIRE(ldc >= (size_t)(n > 0 ? n : 0) && ldc % 4 == 0, LQ_ERR_SHAPE, "lq_gemm_fp8_codes: need ldc >= n and ldc %% 4 == 0 (ldc=%zu n=%d)", ldc, n);
    int rc = fp8_check("lq_gemm_fp8_codes", nullptr, A, B_rows32, a_scale, b_scale, bias, nullptr, m, n, k);
    if (rc != LQ_OK) return rc > 0 ? LQ_OK : rc;
    LQ_REQUIRE(C_fp8 && C_fp8_scale, LQ_ERR_ARG, "lq_gemm_fp8_codes: null pointer");
    LQ_REQUIRE(ldc >= (size_t)n && ldc % 4 == 0 && reinterpret_cast<uintptr_t>(C_fp8) % 4 == 0, LQ_ERR_SHAPE,
               "lq_gemm_fp8_codes: need ldc >= n, ldc %% 4 == 0 and a 4-byte aligned destination (ldc=%zu n=%d)", ldc, n);
    GemmParams p = {};
    p.A = A; p.B = B_rows32; p.bias = bias; p.a_scale = a_scale; p.b_scale = b_scale; p.gelu = gelu;
    p.C8 = C_fp8; p.c8_scale = C_fp8_scale; p.ldc8 = ldc;
    p.m = m; p.n = n; p.k = k; p.kb = k;
    p.a_panel = panels;   // both the activation read and the codes written, or neither
    p.c8_panel = panels;
    LQ_REQUIRE(!panels || n % 64 == 0, LQ_ERR_SHAPE, "lq_gemm_fp8_codes_panels: codes in k-panels need n %% 64 == 0 (n=%d)", n);
    return fp8_dispatch("lq_gemm_fp8_codes", p, round_dtype, stream);
}

extern "C" int lq_gemm_fp8_codes(uint8_t* C_fp8, size_t ldc, const float* C_fp8_scale, lq_dtype_t round_dtype, const uint8_t* A,
                                 const uint8_t* B_rows32, const float* a_scale, const float* b_scale, const void* bias, int gelu,
                                 int m, int n, int k, lq_stream_t stream) {
    return gemm_fp8_codes(C_fp8, ldc, C_fp8_scale, round_dtype, A, B_rows32, a_scale, b_scale, bias, gelu, m, n, k, 0, stream);
}

extern "C" int lq_gemm_fp8_codes_panels(uint8_t* C_fp8_panels, const float* C_fp8_scale, lq_dtype_t round_dtype,
                                        const uint8_t* A_panels, const uint8_t* B_rows32, const float* a_scale, const float* b_scale,
                                        const void* bias, int gelu, int m, int n, int k, lq_stream_t stream) {
    return gemm_fp8_codes(C_fp8_panels, (size_t)(n > 0 ? n : 0), C_fp8_scale, round_dtype, A_panels, B_rows32, a_scale, b_scale, bias, gelu,
                          m, n, k, 1, stream);
}
