// W4A4 (group-64 INT4 x INT4) GEMM entry point: nibbles widened to int8 in registers, exact
// int32 group sums on v_mfma_i32_32x32x32_i8, fp32 group-scale accumulation in ascending group
// order.  Reference semantics: kernels/w4a4_gemm/w4a4_gemm.cu:227-512 (group loop :473-506) of
// lyraDiff, without the low-rank branch.
#include "lq_gemm_core.h"

namespace lq {


// Tile configurations.  The kernel is bound by the vector ALU (two or three fp32 operations per output
// per group, plus widening the nibbles), so the wavefront tile is kept at 64x32 or 32x32 outputs: small
// enough for three or four wavefronts per SIMD, which hide each other's LDS and MFMA latencies.
template <int KIND, typename OutTag> static int run_w4a4(GemmParams p, hipStream_t st) {
    int t = requested_tactic(g_tactic_w4a4, LQ_W_INT4, p.m, p.n, p.k);
    if (t < 0) {
        const long tiles = (long)((p.m + 63) / 64) * ((p.n + 127) / 128);
        t = tiles >= 768 ? 0 : 1;  // three workgroups per CU on 256 CUs
        // 16-bit scales, short K: the 128x64 tile (same 64x32 wavefront tile, two rows of wavefronts sharing the weight
        // stage) measured 1-6 % ahead of the 64x128 one at K = 3072 (4608x3072x3072: 91 against 97 us) and 3-4 % behind at
        // K >= 12288; with fp32 scales the two are level
        if (t == 0 && KIND == K_W4A4H && p.k <= 4096) t = 2;
    }
    switch (t) {
        case 0: return launch_gemm<KIND, OutTag, 64, 128, 64, 1, 4, 2>(p, st);
        case 1: return launch_gemm<KIND, OutTag, 64, 64, 64, 2, 2, 2>(p, st);
        case 2: return launch_gemm<KIND, OutTag, 128, 64, 64, 2, 2, 2>(p, st);
        default: set_error("lq_gemm_w4a4: unknown tactic %d", t); return LQ_ERR_ARG;
    }
}

}  // namespace lq

using namespace lq;

extern "C" int lq_gemm_w4a4_ex(void* C, lq_dtype_t out_dtype, const uint32_t* A_words, const uint8_t* B_rows32,
                               const void* sA, const void* sB, lq_dtype_t scale_dtype, const void* bias,
                               const void* lora_act, const void* lora_up, lq_dtype_t lora_dtype, int lora_rank, int m,
                               int n, int k, int group, const lq_epilogue_t* epi, lq_stream_t stream) {
    LQ_REQUIRE((C || (epi && epi->C_fp8)) && A_words && B_rows32 && sA && sB, LQ_ERR_ARG, "lq_gemm_w4a4: null pointer");
    if (epi != nullptr) {
        LQ_REQUIRE(epi->gelu >= 0 && epi->gelu <= 2, LQ_ERR_ARG, "lq_gemm_w4a4: gelu must be 0, 1 or 2");
        LQ_REQUIRE((epi->gate == nullptr) == (epi->residual == nullptr), LQ_ERR_ARG, "lq_gemm_w4a4: gate and residual go together");
        LQ_REQUIRE(epi->gate == nullptr || epi->rows_per_gate > 0, LQ_ERR_SHAPE, "lq_gemm_w4a4: rows_per_gate must be positive");
        LQ_REQUIRE((epi->C_fp8 == nullptr) == (epi->C_fp8_scale == nullptr), LQ_ERR_ARG, "lq_gemm_w4a4: C_fp8 and C_fp8_scale go together");
        LQ_REQUIRE(epi->C_fp8 == nullptr || (epi->ldc_fp8 >= (size_t)(n > 0 ? n : 0) && epi->ldc_fp8 % 4 == 0 &&
                                             reinterpret_cast<uintptr_t>(epi->C_fp8) % 4 == 0),
                   LQ_ERR_SHAPE, "lq_gemm_w4a4: need ldc_fp8 >= n, ldc_fp8 %% 4 == 0 and a 4-byte aligned C_fp8");
        LQ_REQUIRE(reinterpret_cast<uintptr_t>(epi->gate) % 16 == 0 && reinterpret_cast<uintptr_t>(epi->residual) % 16 == 0 &&
                       reinterpret_cast<uintptr_t>(epi->addend) % 16 == 0,
                   LQ_ERR_ARG, "lq_gemm_w4a4: gate, residual and addend must be 16-byte aligned");
    }
    LQ_REQUIRE(group == 64, LQ_ERR_SHAPE, "lq_gemm_w4a4: group=%d, only 64 is supported", group);
    LQ_REQUIRE(scale_dtype == LQ_F32 || scale_dtype == LQ_F16, LQ_ERR_UNSUPPORTED,
               "lq_gemm_w4a4: scale dtype must be F32 or F16");
    LQ_REQUIRE(m >= 0 && n > 0 && k > 0 && n % 32 == 0 && k % 128 == 0, LQ_ERR_SHAPE,
               "lq_gemm_w4a4: need n %% 32 == 0 and k %% 128 == 0 (m=%d n=%d k=%d)", m, n, k);
    LQ_REQUIRE(reinterpret_cast<uintptr_t>(A_words) % 16 == 0 && reinterpret_cast<uintptr_t>(B_rows32) % 16 == 0 &&
                   reinterpret_cast<uintptr_t>(C) % 16 == 0 && reinterpret_cast<uintptr_t>(bias) % 8 == 0,
               LQ_ERR_ARG, "lq_gemm_w4a4: A, B, C must be 16-byte aligned and bias 8-byte aligned");
    LQ_REQUIRE(reinterpret_cast<uintptr_t>(sA) % 4 == 0 && reinterpret_cast<uintptr_t>(sB) % 4 == 0, LQ_ERR_ARG,
               "lq_gemm_w4a4: scale arrays must be 4-byte aligned");
    LQ_REQUIRE((lora_act == nullptr) == (lora_up == nullptr), LQ_ERR_ARG,
               "lq_gemm_w4a4: the low-rank branch needs both lora_act and lora_up");
    if (lora_act != nullptr) {
        LQ_REQUIRE(lora_dtype == LQ_F16 || lora_dtype == LQ_BF16, LQ_ERR_UNSUPPORTED,
                   "lq_gemm_w4a4: low-rank operands must be F16 or BF16");
        LQ_REQUIRE(lora_rank > 0 && lora_rank % 16 == 0, LQ_ERR_SHAPE, "lq_gemm_w4a4: lora_rank=%d must be a multiple of 16", lora_rank);
        LQ_REQUIRE(reinterpret_cast<uintptr_t>(lora_act) % 16 == 0 && reinterpret_cast<uintptr_t>(lora_up) % 16 == 0, LQ_ERR_ARG,
                   "lq_gemm_w4a4: low-rank operands must be 16-byte aligned");
    }
    if (m == 0) return LQ_OK;
    GemmParams p = {};
    p.C = C; p.A = reinterpret_cast<const uint8_t*>(A_words); p.B = B_rows32; p.bias = bias;
    p.sA = sA; p.sB = sB; p.scale_f16 = scale_dtype == LQ_F16;
    p.lora_act = lora_act; p.lora_up = lora_up; p.lora_rank = lora_rank; p.lora_f16 = lora_dtype == LQ_F16;
    p.ldc8 = (size_t)n;
    if (epi != nullptr) {
        p.gelu = epi->gelu; p.addend = epi->addend; p.gate = epi->gate; p.gate_rows = epi->rows_per_gate;
        p.residual = epi->residual; p.beta = 1.0f;
        p.C8 = epi->C_fp8; p.c8_scale = epi->C_fp8_scale;
        if (epi->C_fp8 != nullptr) p.ldc8 = epi->ldc_fp8;
    }
    p.m = m; p.n = n; p.k = k; p.kb = k / 2;
    hipStream_t st = as_stream(stream);
    switch (out_dtype) {
        case LQ_F16: return p.scale_f16 ? run_w4a4<K_W4A4H, F16Tag>(p, st) : run_w4a4<K_W4A4, F16Tag>(p, st);
        case LQ_BF16: return p.scale_f16 ? run_w4a4<K_W4A4H, BF16Tag>(p, st) : run_w4a4<K_W4A4, BF16Tag>(p, st);
        case LQ_F32: return p.scale_f16 ? run_w4a4<K_W4A4H, F32Tag>(p, st) : run_w4a4<K_W4A4, F32Tag>(p, st);
        default: set_error("lq_gemm_w4a4: unsupported output dtype %d", (int)out_dtype); return LQ_ERR_UNSUPPORTED;
    }
}

extern "C" int lq_gemm_w4a4_lora(void* C, lq_dtype_t out_dtype, const uint32_t* A_words, const uint8_t* B_rows32,
                                 const void* sA, const void* sB, lq_dtype_t scale_dtype, const void* bias,
                                 const void* lora_act, const void* lora_up, lq_dtype_t lora_dtype, int lora_rank, int m,
                                 int n, int k, int group, lq_stream_t stream) {
    LQ_REQUIRE(C != nullptr, LQ_ERR_ARG, "lq_gemm_w4a4: null pointer");
    return lq_gemm_w4a4_ex(C, out_dtype, A_words, B_rows32, sA, sB, scale_dtype, bias, lora_act, lora_up, lora_dtype, lora_rank, m, n,
                           k, group, nullptr, stream);
}

extern "C" int lq_gemm_w4a4(void* C, lq_dtype_t out_dtype, const uint32_t* A_words, const uint8_t* B_rows32,
                            const void* sA, const void* sB, lq_dtype_t scale_dtype, const void* bias, int m, int n,
                            int k, int group, lq_stream_t stream) {
    return lq_gemm_w4a4_lora(C, out_dtype, A_words, B_rows32, sA, sB, scale_dtype, bias, nullptr, nullptr, LQ_BF16, 0, m, n, k,
                             group, stream);
}
