// lyradiff_compat.h -- header-only C++ layer that re-creates, on top of the C ABI of lyraquant.h,
// the names and argument meaning of the lyraDiff reference's quantized-linear interfaces, so that
// reference-style call sites compile against liblyraquant.so with `cudaStream_t` spelled
// `hipStream_t`.  Each entity cites what it stands in for (paths relative to the reference's
// src/lyradiff/).  Errors follow the reference's convention: std::runtime_error with a
// "[lyradiff Error][...]" prefix (kernels/cutlass_kernels/int8_gemm/int8_gemm_template.h:169-188).
//
// Differences a maintainer has to know:
//   * the weight operand "B" of every GEMM is the rows32 layout produced once by
//     repackWeight() / lq_repack_rows32 (same byte count as the [N,K] matrix);
//   * workspaces are accepted and ignored; tactics are small integers (tile configurations of the
//     library) and the profiler caches the fastest one per (m bucket, n, k) inside the library;
//   * the W4A4 low-rank down projection overwrites its fp32 output instead of adding into it.
#pragma once

#include <hip/hip_runtime.h>
#include <hip/hip_fp16.h>
#include <hip/hip_bfloat16.h>

#include <cstddef>
#include <cstdint>
#include <memory>
#include <stdexcept>
#include <string>
#include <vector>

#include "lyraquant.h"

namespace lyradiff {

namespace detail {
template <typename T> struct DType;
template <> struct DType<float> { static constexpr lq_dtype_t value = LQ_F32; };
template <> struct DType<__half> { static constexpr lq_dtype_t value = LQ_F16; };
template <> struct DType<hip_bfloat16> { static constexpr lq_dtype_t value = LQ_BF16; };
template <> struct DType<int32_t> { static constexpr lq_dtype_t value = LQ_I32; };
inline void check(int status, const char* what) {
    if (status != LQ_OK)
        throw std::runtime_error(std::string("[lyradiff Error][") + what + "] " + lq_last_error());
}
}  // namespace detail

// ---- utils/quantization.h:9-274 (the subset the quantized-linear path reads) -------------------------
class QuantMode {
public:
    using BaseType = std::uint32_t;
    explicit constexpr QuantMode(BaseType value) noexcept : mValue{value} {}
    QuantMode() noexcept = default;
    static constexpr QuantMode none() noexcept { return QuantMode(0); }
    static constexpr QuantMode int4Weights() noexcept { return QuantMode(1u << 0); }
    static constexpr QuantMode int8Weights() noexcept { return QuantMode(1u << 1); }
    static constexpr QuantMode activations() noexcept { return QuantMode(1u << 2); }
    static constexpr QuantMode perChannelScaling() noexcept { return QuantMode(1u << 3); }
    static constexpr QuantMode perTokenScaling() noexcept { return QuantMode(1u << 4); }
    static constexpr QuantMode perGroupScaling() noexcept { return QuantMode(1u << 5); }
    constexpr BaseType value() const noexcept { return mValue; }
    constexpr bool isSet(QuantMode const& m) const noexcept { return (mValue & m.mValue) == m.mValue; }
    constexpr bool hasInt4Weights() const noexcept { return isSet(int4Weights()); }
    constexpr bool hasInt8Weights() const noexcept { return isSet(int8Weights()); }
    constexpr bool hasActivations() const noexcept { return isSet(activations()); }
    constexpr bool hasPerChannelScaling() const noexcept { return isSet(perChannelScaling()); }
    constexpr bool hasPerTokenScaling() const noexcept { return isSet(perTokenScaling()); }
    constexpr bool hasPerGroupScaling() const noexcept { return isSet(perGroupScaling()); }
    constexpr bool hasStaticActivationScaling() const noexcept { return !hasPerTokenScaling(); }
    static constexpr QuantMode useSmoothQuant(bool perToken = false, bool perChannel = false) {
        return QuantMode((1u << 1) | (1u << 2) | (perChannel ? 1u << 3 : 0u) | (perToken ? 1u << 4 : 0u));
    }
    constexpr bool operator==(QuantMode const& o) const noexcept { return mValue == o.mValue; }
    constexpr bool operator!=(QuantMode const& o) const noexcept { return mValue != o.mValue; }

private:
    BaseType mValue{0};
};

// ---- kernels/quant_kernels/quant_kernels.h:8-37 --------------------------------------------------------
template <typename T>
void invokeSqInputQuant(int8_t* dst, const T* src, const float* pre_quant_scale, const float* input_quant_scale,
                        QuantMode quant_mode, size_t batch_size, size_t seq_len, size_t dim, hipStream_t stream) {
    detail::check(lq_sq_input_quant(dst, src, detail::DType<T>::value, pre_quant_scale, input_quant_scale,
                                    quant_mode.hasPerTokenScaling(), batch_size * seq_len, dim, stream),
                  "invokeSqInputQuant");
}
// dynamic per-token flavour (writes the per-token scales it used); no reference counterpart
template <typename T>
void invokeSqDynamicPerTokenQuant(int8_t* dst, float* token_scale, const T* src, const float* pre_quant_scale,
                                  size_t batch_size, size_t seq_len, size_t dim, hipStream_t stream) {
    detail::check(lq_sq_dynamic_quant(dst, token_scale, src, detail::DType<T>::value, pre_quant_scale,
                                      batch_size * seq_len, dim, stream),
                  "invokeSqDynamicPerTokenQuant");
}
template <typename T>
void invokeSqOutputDequant(T* dst, const int32_t* src, const float* input_quant_scale, const float* weight_quant_scale,
                           QuantMode quant_mode, size_t batch_size, size_t seq_len, size_t dim, hipStream_t stream) {
    detail::check(lq_sq_output_dequant(dst, detail::DType<T>::value, src, input_quant_scale, weight_quant_scale,
                                       quant_mode.hasPerTokenScaling(), batch_size * seq_len, dim, stream),
                  "invokeSqOutputDequant");
}
template <typename T>
void invokeGetINT8WeightScale(float* new_weight_scale, int8_t* quantized_weight, const T* weight,
                              const float* pre_quant_scale, const size_t d_out, const size_t d_in,
                              hipStream_t stream = 0) {
    detail::check(lq_int8_weight_quant(new_weight_scale, quantized_weight, weight, detail::DType<T>::value,
                                       pre_quant_scale, d_out, d_in, stream),
                  "invokeGetINT8WeightScale");
}

// ---- kernels/quant_kernels/ffn_kernels_int8.h:12-21 ----------------------------------------------------
template <typename T>
void invokeFusedAddBiasGegluInt8O(int8_t* dst, const T* hidden_states, const T* bias, const float* pre_quant_scale,
                                  const float* input_quant_scale, const int seq_len, const int dim,
                                  const int batch_size, hipStream_t stream) {
    detail::check(lq_geglu_int8(dst, hidden_states, bias, detail::DType<T>::value, pre_quant_scale, input_quant_scale,
                                (size_t)seq_len * batch_size, dim, stream),
                  "invokeFusedAddBiasGegluInt8O");
}

// ---- kernels/lora/load_lora.h:30-31 and utils/memory_utils.cu:441-446 ------------------------------------
struct fp8_e4m3_t { uint8_t bits; };  // storage type standing in for __nv_fp8_e4m3
template <typename T>
void invokeGetFP8WeightScale(float* new_weight_scale, const T* weight, const size_t size, hipStream_t stream = 0) {
    detail::check(lq_fp8_amax_scale(new_weight_scale, weight, detail::DType<T>::value, size, stream),
                  "invokeGetFP8WeightScale");
}
template <typename T_IN>
void invokeCudaD2DScaleCpyConvert(fp8_e4m3_t* tgt, const T_IN* src, const float* scale, bool invert_scale,
                                  const size_t size, hipStream_t stream) {
    detail::check(lq_fp8_scale_cast(reinterpret_cast<uint8_t*>(tgt), src, detail::DType<T_IN>::value, scale,
                                    invert_scale, size, stream),
                  "invokeCudaD2DScaleCpyConvert");
}

// ---- kernels/quant_kernels/layer_norm_int8.h:8-38 ------------------------------------------------------------
// Static per-tensor scale, as in the reference.  (The C ABI can also produce a dynamic per-token scale.)
template <typename T>
void invokeLayerNormInt8O(int8_t* dst, const T* src, const T* gamma, const T* beta, const float* pre_quant_scale,
                          const float* input_quant_scale, QuantMode /*quant_mode*/, size_t batch_size, size_t channels,
                          size_t nhiddens, hipStream_t stream, const double eps = 1e-6) {
    detail::check(lq_layernorm_int8(dst, nullptr, nullptr, src, nullptr, nullptr, gamma, beta, detail::DType<T>::value,
                                    pre_quant_scale, input_quant_scale, batch_size * channels, nhiddens, (float)eps, stream),
                  "invokeLayerNormInt8O");
}
// dst2 = src + residual + bias (T), dst = int8 of its LayerNorm
template <typename T>
void invokeFusedResidualBiasLayerNormInt8O(int8_t* dst, T* dst2, const T* src, const T* residual, const T* bias, const T* gamma,
                                           const T* beta, const float* pre_quant_scale, const float* input_quant_scale,
                                           QuantMode /*quant_mode*/, size_t batch_size, size_t channels, size_t nhiddens,
                                           hipStream_t stream, const double eps = 1e-6) {
    detail::check(lq_layernorm_int8(dst, nullptr, dst2, src, residual, bias, gamma, beta, detail::DType<T>::value,
                                    pre_quant_scale, input_quant_scale, batch_size * channels, nhiddens, (float)eps, stream),
                  "invokeFusedResidualBiasLayerNormInt8O");
}
// ---- kernels/norms/layer_norm.h:18-27 followed by utils/memory_utils.cu:441-446 in one launch -------------------
// (the two calls of layers/flux_attn_post_processor/FluxAttnPostFP8Processor.cc:125-140: adaLN modulation, then the
// cast to e4m3 with the calibrated static input scale)
template <typename T>
void invokeLayerNormWithShiftAndScaleFP8(fp8_e4m3_t* dst, const T* src, const T* scale, const T* shift, const float* input_scale,
                                         size_t batch_size, size_t channels, size_t nhiddens, hipStream_t stream,
                                         const double eps = 1e-6) {
    detail::check(lq_layernorm_mod_fp8(reinterpret_cast<uint8_t*>(dst), src, scale, shift, detail::DType<T>::value, input_scale,
                                       batch_size, channels, nhiddens, (float)eps, stream),
                  "invokeLayerNormWithShiftAndScaleFP8");
}

// ---- kernels/rope/flux_apply_rope.h:18-28,58-72 ---------------------------------------------------------------
// q/k RMSNorm per head + rotary embedding (+ the [encoder, hidden] concatenation) in front of the attention;
// out / input are [batch, seq, 3, head_num, head_dim], scale is [2 * head_dim] (q then k), rope_emb is indexed per batch.
template <typename T>
void invokeFusedRmsNormAndRope(T* out, const T* input, const T* scale, const T* rope_emb, float eps, int batch_size, int seq_len,
                               int head_num, int head_dim, hipStream_t stream) {
    detail::check(lq_rmsnorm_rope(out, input, nullptr, scale, nullptr, rope_emb, (size_t)seq_len * head_dim * 2,
                                  detail::DType<T>::value, batch_size, seq_len, 0, head_num, head_dim, eps, stream),
                  "invokeFusedRmsNormAndRope");
}
template <typename T>
void invokeFusedRmsNormCatAndRope(T* out, const T* hidden, const T* encoder_hidden, const T* hidden_rms_scale,
                                  const T* encoder_rms_scale, const T* rope_emb, float eps, int batch_size, int hidden_seq_len,
                                  int encoder_seq_len, int head_num, int head_dim, hipStream_t stream) {
    detail::check(lq_rmsnorm_rope(out, hidden, encoder_hidden, hidden_rms_scale, encoder_rms_scale, rope_emb,
                                  (size_t)(hidden_seq_len + encoder_seq_len) * head_dim * 2, detail::DType<T>::value, batch_size,
                                  hidden_seq_len, encoder_seq_len, head_num, head_dim, eps, stream),
                  "invokeFusedRmsNormCatAndRope");
}

// ---- kernels/w4a4_gemm/w4a4_gemm.h:6-30 ------------------------------------------------------------------
// Quantises A [m,k] (bf16) to group-64 int4 words + fp32 group scales and, when Bptr (lora down, bf16
// [n = rank, k]) is given, writes the fp32 down projection A . B^T to Cptr [m, n].  The reference ADDS its
// k-tiles into a Cptr that the caller zeroed (float atomics); here Cptr is simply overwritten with the full sum.
// group_dim: the reference's own call site passes the number of groups in this slot
// (layers/w4a4_gemm_block/W4A4Gemm.cc:127-137); both that and the group size 64 are accepted.
inline void invokeFusedQuantizeAndLoraDownSimple(float* Cptr, uint32_t* quantized_input, float* quantized_scale,
                                                 const void* Aptr /* bf16 [m,k] */, const void* Bptr /* lora down */,
                                                 const float* Smoothptr, int m, int n, int k, int group_dim = 64,
                                                 hipStream_t stream = 0) {
    if (group_dim != 64 && group_dim != k / 64)
        throw std::runtime_error("[lyradiff Error][invokeFusedQuantizeAndLoraDownSimple] only group size 64 is supported");
    if ((Cptr == nullptr) != (Bptr == nullptr))
        throw std::runtime_error("[lyradiff Error][invokeFusedQuantizeAndLoraDownSimple] Cptr and Bptr go together");
    if (Bptr != nullptr)  // one pass over A for both results, as in the reference
        detail::check(lq_w4a4_quantize_lora_down(quantized_input, quantized_scale, LQ_F32, Cptr, LQ_F32, Aptr, LQ_BF16, Smoothptr,
                                                 Bptr, m, k, n, 64, stream),
                      "invokeFusedQuantizeAndLoraDownSimple");
    else
        detail::check(lq_w4a4_quantize(quantized_input, quantized_scale, LQ_F32, Aptr, LQ_BF16, Smoothptr, m, k, 64, stream),
                      "invokeFusedQuantizeAndLoraDownSimple");
}
// utils/memory_utils.cu:398-402, the float -> T instantiations
template <typename T_OUT>
void invokeCudaD2DcpyConvert(T_OUT* tgt, const float* src, const size_t size, hipStream_t stream = 0) {
    detail::check(lq_cast_f32(tgt, detail::DType<T_OUT>::value, src, size, stream), "invokeCudaD2DcpyConvert");
}
// D [m,n] bf16 = W4A4(A, B) + LoraA [m, lora_k] . LoraB [n, lora_k]^T (bf16 operands; both null: no low-rank branch)
inline void invokeFusedW4A4GemmAndLoraUp(void* Dptr /* bf16 [m,n] */, const void* Aptr, const void* Bptr_rows32,
                                         const void* LoraAptr, const void* LoraBptr, const float* AweightScale,
                                         const float* BweightScale, int m, int n, int k, int lora_k, int groups,
                                         hipStream_t stream, const void* bias = nullptr) {
    if (groups != k / 64)
        throw std::runtime_error("[lyradiff Error][invokeFusedW4A4GemmAndLoraUp] groups must equal k / 64");
    detail::check(lq_gemm_w4a4_lora(Dptr, LQ_BF16, static_cast<const uint32_t*>(Aptr), static_cast<const uint8_t*>(Bptr_rows32),
                                    AweightScale, BweightScale, LQ_F32, bias, LoraAptr, LoraBptr, LQ_BF16, lora_k, m, n, k, 64,
                                    stream),
                  "invokeFusedW4A4GemmAndLoraUp");
}

// ---- one-time weight repack (role of kernels/cutlass_kernels/cutlass_preprocessors.cpp:484-530) -----------
inline void repackWeight(void* dst_rows32, const void* src_row_major, lq_weight_kind_t kind, size_t n, size_t k,
                         hipStream_t stream = 0) {
    detail::check(lq_repack_rows32(static_cast<uint8_t*>(dst_rows32), static_cast<const uint8_t*>(src_row_major), n,
                                   lq_weight_row_bytes(kind, k), stream),
                  "repackWeight");
}

// ---- kernels/cutlass_extensions/.../gemm_configs.h:101-130 --------------------------------------------------
// A configuration is one of the library's tile configurations; tile_config = -1 means "choose"
// (ChooseWithHeuristic).  split_k_factor and stages are carried for source compatibility only: the
// reference's launcher never applies split-k either (int8_gemm_template.h:146-148).
// ---- kernels/cutlass_extensions/include/cutlass_extensions/weight_only_quant_op.h:9-25 ------------------------
namespace cutlass {
enum class WeightOnlyQuantOp { UNDEFINED, PER_COLUMN_SCALE_ONLY, FINEGRAINED_SCALE_ONLY, FINEGRAINED_SCALE_AND_ZEROS };
constexpr bool isFinegrained(WeightOnlyQuantOp op) {
    return op == WeightOnlyQuantOp::FINEGRAINED_SCALE_AND_ZEROS || op == WeightOnlyQuantOp::FINEGRAINED_SCALE_ONLY;
}
constexpr bool hasZero(WeightOnlyQuantOp op) { return op == WeightOnlyQuantOp::FINEGRAINED_SCALE_AND_ZEROS; }
struct uint4b_t {};  // tag for 4-bit weights (two per byte); only used as a template argument here
}  // namespace cutlass

namespace cutlass_extensions {
struct CutlassGemmConfig {
    int tile_config = -1;
    int split_k_factor = -1;
    int stages = -1;
    CutlassGemmConfig() {}
    CutlassGemmConfig(int tile_config_, int split_k_factor_, int stages_)
        : tile_config(tile_config_), split_k_factor(split_k_factor_), stages(stages_) {}
};
}  // namespace cutlass_extensions

// ---- kernels/cutlass_kernels/int8_gemm/int8_gemm.h:16-90 ----------------------------------------------------
namespace cutlass_kernels {
class CutlassInt8GemmRunnerInterface {
public:
    virtual ~CutlassInt8GemmRunnerInterface() {}
    virtual void gemm(int8_t const* A, int8_t const* B, QuantMode quantOption, float const* alphaCol,
                      float const* alphaRow, void* C, int m, int n, int k,
                      cutlass_extensions::CutlassGemmConfig gemmConfig, char* workspacePtr, const size_t workspaceBytes,
                      hipStream_t stream) = 0;
    virtual size_t getWorkspaceSize(int const m, int const n, int const k) = 0;
    virtual std::vector<cutlass_extensions::CutlassGemmConfig> getConfigs() const = 0;
};

template <typename T>
class CutlassInt8GemmRunner : public virtual CutlassInt8GemmRunnerInterface {
public:
    // B is the rows32 layout of the [n,k] weight; C[m,n] = T(float(acc) * (alphaCol[n] * alphaRow[m or 0]))
    void gemm(int8_t const* A, int8_t const* B, QuantMode quantOption, float const* alphaCol, float const* alphaRow,
              void* C, int m, int n, int k, cutlass_extensions::CutlassGemmConfig gemmConfig, char* /*workspacePtr*/,
              const size_t /*workspaceBytes*/, hipStream_t stream) override {
        lq_gemm_set_thread_tactic(gemmConfig.tile_config);
        const int status = lq_gemm_int8(C, detail::DType<T>::value, A, B, alphaCol, alphaRow,
                                        quantOption.hasPerTokenScaling(), nullptr, m, n, k, stream);
        lq_gemm_set_thread_tactic(-1);
        detail::check(status, "CutlassInt8GemmRunner::gemm");
    }
    size_t getWorkspaceSize(int const, int const, int const) override { return 0; }
    std::vector<cutlass_extensions::CutlassGemmConfig> getConfigs() const override {
        std::vector<cutlass_extensions::CutlassGemmConfig> configs;
        for (int t = 0; t < lq_gemm_tactic_count(LQ_W_INT8); ++t) configs.emplace_back(t, 1, -1);
        return configs;
    }
};

// ---- kernels/cutlass_kernels/fpA_intB_gemm/fpA_intB_gemm.h:25-180 (weight-only W8A16 / W4A16) ---------------------
// B is the buffer lq_repack_weight_only made from the unprocessed codes (same size as the reference's preprocessed
// weight); scales [n] for PER_COLUMN_SCALE_ONLY, scales and zero points [k / group_size, n] for the FINEGRAINED ops.
// The alpha overloads, the fp8 activation form and the split-k workspace of the reference are not carried.
template <typename ActivationType, typename WeightType, cutlass::WeightOnlyQuantOp QuantOp>
class CutlassFpAIntBGemmRunner {
    static_assert(std::is_same<WeightType, uint8_t>::value || std::is_same<WeightType, cutlass::uint4b_t>::value,
                  "WeightType must be uint8_t or cutlass::uint4b_t");
    static constexpr lq_weight_kind_t kKind = std::is_same<WeightType, uint8_t>::value ? LQ_W_INT8 : LQ_W_INT4;

public:
    void gemm(void const* A, void const* B, void const* weight_scales, void* C, int m, int n, int k,
              cutlass_extensions::CutlassGemmConfig /*gemmConfig*/, char* /*workspace_ptr*/, const size_t /*workspace_bytes*/,
              hipStream_t stream) {
        static_assert(QuantOp == cutlass::WeightOnlyQuantOp::PER_COLUMN_SCALE_ONLY, "per-column overload");
        detail::check(lq_gemm_weight_only(C, A, detail::DType<ActivationType>::value, static_cast<const uint8_t*>(B), kKind,
                                          weight_scales, nullptr, m, n, k, stream),
                      "CutlassFpAIntBGemmRunner::gemm");
    }
    void gemm(void const* A, void const* B, void const* weight_scales, void const* weight_zero_points, void const* biases, void* C,
              int m, int n, int k, int const group_size, cutlass_extensions::CutlassGemmConfig /*gemmConfig*/,
              char* /*workspace_ptr*/, const size_t /*workspace_bytes*/, hipStream_t stream) {
        int status;
        if (QuantOp == cutlass::WeightOnlyQuantOp::PER_COLUMN_SCALE_ONLY)
            status = lq_gemm_weight_only(C, A, detail::DType<ActivationType>::value, static_cast<const uint8_t*>(B), kKind,
                                         weight_scales, biases, m, n, k, stream);
        else
            status = lq_gemm_weight_only_grouped(C, A, detail::DType<ActivationType>::value, static_cast<const uint8_t*>(B), kKind,
                                                 weight_scales,
                                                 QuantOp == cutlass::WeightOnlyQuantOp::FINEGRAINED_SCALE_AND_ZEROS ? weight_zero_points : nullptr,
                                                 biases, m, n, k, group_size, stream);
        detail::check(status, "CutlassFpAIntBGemmRunner::gemm");
    }
    size_t getWorkspaceSize(int const, int const, int const) { return 0; }
    std::vector<cutlass_extensions::CutlassGemmConfig> getConfigs() const { return {cutlass_extensions::CutlassGemmConfig(0, 1, -1)}; }
};
}  // namespace cutlass_kernels

namespace gemm {

// ---- layers/gemm_utils/GemmProfiler.h:36-63,131-251, layers/gemm_utils/SmoothQuantGemm.h:29-48 ---------------
struct GemmDims {
    int minM = 1, maxM = 0, n = 0, k = 0;
    GemmDims() {}
    GemmDims(int minM_, int maxM_, int n_, int k_) : minM(minM_), maxM(maxM_), n(n_), k(k_) {}
};

// Times the library's tile configurations for m = minM rounded up to a power of two, doubling up to
// maxM, plus maxM itself (GemmProfiler.cc:78-127), and leaves the winners in the library's per-shape
// cache, where every later GEMM call of that (m bucket, n, k) finds them.  Temporary device memory
// is allocated for the duration of profileTactics, as the reference's allocateTmpData does.
class SmoothQuantGemmPluginProfiler {
public:
    void setQuantMode(QuantMode const& quantMode) { mQuantMode = quantMode; }
    void setSkip(bool skip) { mSkip = skip; }
    void profileTactics(GemmDims const& dims, hipStream_t stream = 0) {
        if (mSkip || dims.maxM <= 0) return;
        const size_t bytes = lq_gemm_profile_workspace(LQ_W_INT8, dims.maxM, dims.n, dims.k);
        void* tmp = nullptr;
        if (bytes == 0 || hipMalloc(&tmp, bytes) != hipSuccess)
            throw std::runtime_error("[lyradiff Error][profileTactics] Can't allocate tmp workspace for GEMM tactics profiling.");
        int status = LQ_OK;
        auto one = [&](int m) {
            if (status == LQ_OK && lq_gemm_get_shape_tactic(LQ_W_INT8, m, dims.n, dims.k) < 0)
                status = lq_gemm_profile(LQ_W_INT8, m, dims.n, dims.k, tmp, bytes, nullptr, nullptr, stream);
        };
        int m = 1;
        while (m < dims.minM) m *= 2;
        for (; m < dims.maxM; m *= 2) one(m);
        one(dims.maxM);
        (void)hipFree(tmp);
        detail::check(status, "profileTactics");
    }
    // -1: nothing profiled for this shape, the library's built-in table applies
    int getBestConfig(int m, int n, int k) const { return mSkip ? -1 : lq_gemm_get_shape_tactic(LQ_W_INT8, m, n, k); }
    // GemmPluginProfiler::getSerializationSize / serialize / deserialize (layers/gemm_utils/GemmProfiler.cc:26-75): the
    // measured configurations as bytes; the library keeps one table for every shape, so the GEMM id argument of the
    // reference is not needed.  serialize advances `buffer`, deserialize advances `data`, as the reference's do.
    size_t getSerializationSize() const { return lq_gemm_tactics_serialized_size(); }
    void serialize(char*& buffer) const {
        size_t written = 0;
        detail::check(lq_gemm_tactics_serialize(buffer, lq_gemm_tactics_serialized_size(), &written), "GemmPluginProfiler::serialize");
        buffer += written;
    }
    void deserialize(char const*& data, size_t bytes) {
        detail::check(lq_gemm_tactics_deserialize(data, bytes), "GemmPluginProfiler::deserialize");
        data += bytes;
    }
    QuantMode mQuantMode;

private:
    bool mSkip = false;
};

template <typename DataType>
class SmoothQuantGemmPlugin {
public:
    using PluginProfilerPtr = std::shared_ptr<SmoothQuantGemmPluginProfiler>;
    SmoothQuantGemmPlugin() = delete;
    SmoothQuantGemmPlugin(const QuantMode& quantMode, PluginProfilerPtr const& profiler)
        : mQuantMode(quantMode), mPluginProfiler(profiler) {}
    SmoothQuantGemmPlugin<DataType>* clone() { return new SmoothQuantGemmPlugin<DataType>(*this); }
    void configurePlugin(int maxM, int K, int N) { mMaxM = maxM; mK = K; mN = N; }
    int initialize() {  // configGemm(): profile for mDims = {1, maxM, N, K} (layers/gemm_utils/SmoothQuantGemm.cc:86-96,166-170)
        if (mPluginProfiler && mMaxM > 0) mPluginProfiler->profileTactics(GemmDims(1, mMaxM, mN, mK));
        return 0;
    }
    void terminate() {}
    size_t getWorkspaceSize(int, int, int) { return 0; }
    // C[m,n] = T(float(acc) * (alphaCol[n] * alphaRow[m or 0])); B is the rows32 layout of the [n,k] weight
    void RunGemm(int8_t const* A, int8_t const* B, float const* alphaCol, float const* alphaRow, void* C, int m, int n,
                 int k, char* /*workspacePtr*/, hipStream_t stream, const void* bias = nullptr) {
        detail::check(lq_gemm_int8(C, detail::DType<DataType>::value, A, B, alphaCol, alphaRow,
                                   mQuantMode.hasPerTokenScaling(), bias, m, n, k, stream),
                      "SmoothQuantGemmPlugin::RunGemm");
    }
    QuantMode mQuantMode;

private:
    int mMaxM = 0, mK = 0, mN = 0;
    PluginProfilerPtr mPluginProfiler;
};

}  // namespace gemm

// stand-in for the cuBLAS transpose enum in the signature below
enum cublasOperation_t { CUBLAS_OP_N = 0, CUBLAS_OP_T = 1 };

// ---- utils/cublasMMWrapper.h:299-318,354-385 (the two quantized entry points) -----------------------------
// DataType is the activation/output type the wrapper was configured with (setFP16GemmConfig /
// setBF16GemmConfig in the reference).
template <typename DataType>
class cublasMMWrapper {
public:
    explicit cublasMMWrapper(hipStream_t stream, bool per_token_int8 = false)
        : stream_(stream),
          int8_runner_(QuantMode::useSmoothQuant(per_token_int8, true),
                       std::make_shared<gemm::SmoothQuantGemmPluginProfiler>()) {}
    void setStream(hipStream_t s) { stream_ = s; }
    void profileGemmInt8(const int maxM, const int n, const int k) {
        int8_runner_.configurePlugin(maxM, k, n);
        int8_runner_.initialize();
    }
    void runGemmInt8(int8_t const* A, int8_t const* B, float const* alphaCol, float const* alphaRow, void* C, int m,
                     int n, int k, char* workspacePtr, hipStream_t stream) {
        int8_runner_.RunGemm(A, B, alphaCol, alphaRow, C, m, n, k, workspacePtr, stream);
    }
    // The reference calls this in cuBLAS column-major convention with the WEIGHT as "A":
    //   GemmWithResidualAndBias(OP_T, OP_N, m=N_out, n=M_tokens, k, W, lda=k, w_scale, X, ldb=k, x_scale, C, ldc=N_out, ...)
    // (layers/flux_attn_post_processor/FluxAttnPostFP8Processor.cc:146-163), i.e. the row-major product
    // C[tokens, N_out] = X[tokens,k] . W[N_out,k]^T.  Only that (T, N) form exists in the reference's callers.
    void GemmWithResidualAndBias(cublasOperation_t transa, cublasOperation_t transb, const int m, const int n,
                                 const int k, const fp8_e4m3_t* A_weight_rows32, const int lda, const float* a_scale,
                                 const fp8_e4m3_t* B_act, const int ldb, const float* b_scale, void* C, const int ldc,
                                 const void* bias = nullptr, const void* Residual = nullptr, float f_alpha = 1.0f,
                                 float f_beta = 0.0f, const bool is_gelu = false) {
        if (transa != CUBLAS_OP_T || transb != CUBLAS_OP_N || lda != k || ldb != k || ldc != m || f_alpha != 1.0f)
            throw std::runtime_error("[lyradiff Error][GemmWithResidualAndBias] only the (OP_T weight, OP_N activation, "
                                     "lda = ldb = k, ldc = m, alpha = 1) form used by the FP8 blocks is supported");
        if (Residual == nullptr) f_beta = 0.0f;  // utils/cublasMMWrapper.cc:1123-1125
        detail::check(lq_gemm_fp8(C, detail::DType<DataType>::value, reinterpret_cast<const uint8_t*>(B_act),
                                  reinterpret_cast<const uint8_t*>(A_weight_rows32), b_scale, a_scale, bias, is_gelu,
                                  Residual, f_beta, /*tokens*/ n, /*out features*/ m, k, stream_),
                      "GemmWithResidualAndBias");
    }

private:
    hipStream_t stream_;
    gemm::SmoothQuantGemmPlugin<DataType> int8_runner_;
};

}  // namespace lyradiff
