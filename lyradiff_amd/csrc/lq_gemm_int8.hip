// INT8 W8A8 GEMM entry point (exact int32 accumulation on v_mfma_i32_32x32x32_i8) with the fused
// per-token x per-channel dequant (+ bias) epilogue.  Reference semantics:
// kernels/cutlass_kernels/int8_gemm/int8_gemm_template.h:45-189 and
// kernels/cutlass_extensions/.../epilogue_per_row_per_col_scale.h:239-305 of lyraDiff.
#include "lq_gemm_core.h"

namespace lq {


template <typename OutTag> static constexpr lq_dtype_t out_enum() {
    return std::is_same<OutTag, F16Tag>::value ? LQ_F16 : std::is_same<OutTag, BF16Tag>::value ? LQ_BF16
                                                 : std::is_same<OutTag, F32Tag>::value ? LQ_F32 : LQ_I32;
}

template <typename OutTag> static int run_int8(GemmParams p, hipStream_t st) {
    // static tile table in place of the reference's run-time tactic profiler
    // (layers/gemm_utils/GemmProfiler.cc:78-127): largest tile that still fills the 256 CUs.
    int t = requested_tactic(g_tactic_int8, LQ_W_INT8, p.m, p.n, p.k);
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
        // more full 256x256 tiles than CUs: the persistent form (4608x12288x3072: 153-160 us against 162-165 with 128x256 tiles)
        if (t256 > device_cu_count() && p.m % 256 == 0 && p.n % 256 == 0 && p.kb % 128 == 0 && p.k > 1024 &&
            (out_enum<OutTag>() == LQ_F16 || out_enum<OutTag>() == LQ_BF16))
            t = 7;
    }
    if (t == 1 && (p.kb % 128 != 0 || p.a_panel)) t = 0;  // the 128-byte k-tile needs k % 128 == 0 and a row-major activation
    if (t == 7) {  // the persistent form of tactic 6 where it applies, tactic 6 itself elsewhere
        const int rc = launch_persist_int8(p, out_enum<OutTag>(), st);
        if (rc != 1) return rc;
        t = 6;
    }
    switch (t) {
        case 0: return launch_gemm<K_INT8, OutTag, 256, 256, 64, 2, 4, 3>(p, st);
        case 1: return launch_gemm<K_INT8, OutTag, 256, 256, 128, 2, 4, 2>(p, st);
        case 2: return launch_gemm<K_INT8, OutTag, 128, 128, 64, 2, 2, 3>(p, st);
        case 3: return launch_gemm<K_INT8, OutTag, 64, 64, 64, 2, 2, 3>(p, st);
        case 4: return launch_gemm<K_INT8, OutTag, 128, 256, 64, 2, 2, 3>(p, st);
        case 5: return launch_gemm<K_INT8, OutTag, 256, 128, 64, 2, 2, 3>(p, st);
        case 6: return launch_gemm<K_INT8, OutTag, 256, 256, 64, 2, 2, 4>(p, st);  // one wavefront per SIMD, 128x128 wavefront tiles
        default: set_error("lq_gemm_int8: unknown tactic %d", t); return LQ_ERR_ARG;
    }
}

}  // namespace lq

using namespace lq;

static int gemm_int8(void* C, lq_dtype_t out_dtype, const int8_t* A, const int8_t* B_rows32, const float* alpha_col,
                     const float* alpha_row, int per_token, const void* bias, int m, int n, int k, int a_panel, lq_stream_t stream);

extern "C" int lq_gemm_int8(void* C, lq_dtype_t out_dtype, const int8_t* A, const int8_t* B_rows32,
                            const float* alpha_col, const float* alpha_row, int per_token, const void* bias, int m,
                            int n, int k, lq_stream_t stream) {
    return gemm_int8(C, out_dtype, A, B_rows32, alpha_col, alpha_row, per_token, bias, m, n, k, 0, stream);
}

extern "C" int lq_gemm_int8_panels(void* C, lq_dtype_t out_dtype, const int8_t* A_panels, const int8_t* B_rows32,
                                   const float* alpha_col, const float* alpha_row, int per_token, const void* bias, int m,
                                   int n, int k, lq_stream_t stream) {
    return gemm_int8(C, out_dtype, A_panels, B_rows32, alpha_col, alpha_row, per_token, bias, m, n, k, 1, stream);
}

static int gemm_int8(void* C, lq_dtype_t out_dtype, const int8_t* A, const int8_t* B_rows32, const float* alpha_col,
                     const float* alpha_row, int per_token, const void* bias, int m, int n, int k, int a_panel, lq_stream_t stream) {
    LQ_REQUIRE(C && A && B_rows32, LQ_ERR_ARG, "lq_gemm_int8: null pointer");
    LQ_REQUIRE(out_dtype == LQ_I32 || (alpha_col && alpha_row), LQ_ERR_ARG, "lq_gemm_int8: scale pointers are required");
    LQ_REQUIRE(m >= 0 && n > 0 && k > 0 && n % 32 == 0 && k % 64 == 0, LQ_ERR_SHAPE,
               "lq_gemm_int8: need n %% 32 == 0 and k %% 64 == 0 (m=%d n=%d k=%d)", m, n, k);
    LQ_REQUIRE(reinterpret_cast<uintptr_t>(A) % 16 == 0 && reinterpret_cast<uintptr_t>(B_rows32) % 16 == 0 &&
                   reinterpret_cast<uintptr_t>(C) % 16 == 0 && reinterpret_cast<uintptr_t>(alpha_col) % 16 == 0 &&
                   reinterpret_cast<uintptr_t>(bias) % 8 == 0,
               LQ_ERR_ARG, "lq_gemm_int8: A, B, C, alpha_col must be 16-byte aligned and bias 8-byte aligned");
    if (m == 0) return LQ_OK;
    GemmParams p = {};
    p.C = C; p.A = reinterpret_cast<const uint8_t*>(A); p.B = reinterpret_cast<const uint8_t*>(B_rows32);
    p.bias = bias; p.alpha_col = alpha_col; p.alpha_row = alpha_row; p.per_token = per_token;
    p.m = m; p.n = n; p.k = k; p.kb = k;
    p.a_panel = a_panel;
    hipStream_t st = as_stream(stream);
    switch (out_dtype) {
        case LQ_F16: return run_int8<F16Tag>(p, st);
        case LQ_BF16: return run_int8<BF16Tag>(p, st);
        case LQ_F32: return run_int8<F32Tag>(p, st);
        case LQ_I32: p.bias = nullptr; return run_int8<I32Tag>(p, st);
        default: set_error("lq_gemm_int8: unsupported output dtype %d", (int)out_dtype); return LQ_ERR_UNSUPPORTED;
    }
}
