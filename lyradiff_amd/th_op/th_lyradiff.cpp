// torch custom classes `torch.classes.lyradiff.*` for the FLUX blocks, the way the reference's Python reaches them:
//     torch.classes.load_library(os.getenv("LYRA_LIB_PATH"))                      (lyradiff/__init__.py:4-5)
//     torch.classes.lyradiff.FluxTransformerBlockOp("bf16", 3072, 24, 128, 6, quant_level)
// Registered classes and methods follow src/lyradiff/th_op/pybind.cc:66-96 (FluxTransformerBlockOp,
// FluxSingleTransformerBlockOp, LyraDiffCommonContext; constructor arguments with the same names and defaults,
// initialize, forward, load_lora_by_name, clear_lora, reload_model_from_bin, reload_model_from_state_dict) and
// th_op/flux_transformer_block/FluxTransformerBlockOp.h:186-330,
// th_op/flux_single_transformer_block/FluxSingleTransformerBlockOp.h:184-290.
//
// Quant levels 1, 2 (FP8_W8A8, FP8_W8A8_FULL) and 7, 8 (INT4_W4A4, INT4_W4A4_FULL) are built, the levels whose blocks
// consist of quantized linears.  Every quantized linear, adaLN / gate / residual step, activation quantisation, the q/k
// RMSNorm and the rotary embedding run on liblyraquant.so through its C ABI; PyTorch supplies device memory, the current
// stream, the softmax attention between the projections and the 16-bit adaLN matmul of the non-FULL levels.
// This file holds no device code and is compiled with the host compiler.
#include <ATen/ATen.h>
#include <c10/hip/HIPStream.h>
#include <torch/custom_class.h>
#include <torch/script.h>

#include <cstdio>
#include <map>
#include <memory>
#include <mutex>
#include <string>
#include <vector>

#include "lyraquant.h"

namespace th = torch;

namespace torch_ext {

namespace {

lq_stream_t cur_stream() { return reinterpret_cast<lq_stream_t>(c10::hip::getCurrentHIPStream().stream()); }

lq_dtype_t lq_dt(at::ScalarType t) {
    switch (t) {
        case at::kFloat: return LQ_F32;
        case at::kHalf: return LQ_F16;
        case at::kBFloat16: return LQ_BF16;
        default: TORCH_CHECK(false, "unsupported tensor dtype for the quantized-linear library");
    }
}

void* P(const at::Tensor& t) { return t.defined() ? t.data_ptr() : nullptr; }
uint8_t* P8(const at::Tensor& t) { return static_cast<uint8_t*>(P(t)); }
const float* PF(const at::Tensor& t) { return static_cast<const float*>(P(t)); }

void ok(int rc, const char* what) { TORCH_CHECK(rc == LQ_OK, "[lyradiff Error][", what, "] ", lq_last_error()); }

at::TensorOptions on_gpu(at::ScalarType t) { return at::TensorOptions().dtype(t).device(at::kCUDA); }

// ---- where tensors come from: a state dict or the reference's raw .bin files ---------------------------------------
struct Source {
    virtual ~Source() = default;
    // `dtype` is the type the tensor is wanted in; 16-bit members of a .bin directory are stored in the model file type
    virtual at::Tensor get(const std::string& name, at::IntArrayRef shape, at::ScalarType dtype) const = 0;
};

struct DictSource : Source {
    th::Dict<std::string, th::Tensor> d;
    explicit DictSource(th::Dict<std::string, th::Tensor> dict) : d(std::move(dict)) {}
    at::Tensor get(const std::string& name, at::IntArrayRef shape, at::ScalarType dtype) const override {
        TORCH_CHECK(d.contains(name), "Cannot find a tensor of name ", name);  // TensorMap::at of the reference throws likewise
        at::Tensor t = d.at(name);
        int64_t want = 1;
        for (auto s : shape) want *= s;
        TORCH_CHECK(t.numel() == want && t.scalar_type() == dtype, name, ": got ", t.sizes(), " ", t.scalar_type(), ", expected ",
                    shape, " ", dtype);
        return t.reshape(shape).contiguous();
    }
};

// loadWeightFromBin (utils/memory_utils.cu:251-360): a headerless little-endian file of `model_file_type` elements,
// converted to the wanted type with round-to-nearest-even; scales, smoothing vectors and packed codes are always
// stored as fp32 / int8.
struct BinSource : Source {
    at::ScalarType file_type;
    explicit BinSource(const std::string& model_dtype) {
        if (model_dtype == "fp32") file_type = at::kFloat;
        else if (model_dtype == "fp16") file_type = at::kHalf;
        else if (model_dtype == "bf16") file_type = at::kBFloat16;
        else throw std::invalid_argument("wrong model_dtype");
    }
    at::Tensor get(const std::string& name, at::IntArrayRef shape, at::ScalarType dtype) const override {
        const bool sixteen = dtype == at::kHalf || dtype == at::kBFloat16;
        const at::ScalarType in_file = sixteen ? file_type : dtype;
        at::Tensor t = at::empty(shape, at::TensorOptions().dtype(in_file));
        const std::string path = name + ".bin";
        FILE* f = std::fopen(path.c_str(), "rb");
        TORCH_CHECK(f != nullptr, "[lyradiff Error] file ", path, " cannot be opened");
        const size_t bytes = (size_t)t.numel() * t.element_size();
        const size_t got = std::fread(t.data_ptr(), 1, bytes, f);
        const bool more = std::fgetc(f) != EOF;
        std::fclose(f);
        TORCH_CHECK(got == bytes && !more, "[lyradiff Error] file ", path, " does not hold ", t.numel(), " elements of ", in_file);
        return sixteen ? t.to(dtype) : t;
    }
};

// ---- the three kinds of linear ------------------------------------------------------------------------------------
// FP8 e4m3 per-tensor linear, quantised when loaded (MACROLoadFP8WeightFromBin / ...FromCache,
// utils/common_macro_def.h:66-92); the 16-bit host copy stays for LoRA merges (FP8LoraWeight, interface/IFLoraWeight.h:79-128).
struct FP8Linear {
    at::Tensor w_rows32, w_scale, in_scale, bias, master_h;
    int64_t n = 0, k = 0;

    void requantise(const at::Tensor& w16) {
        w_scale.zero_();
        ok(lq_fp8_amax_scale(static_cast<float*>(P(w_scale)), P(w16), lq_dt(w16.scalar_type()), (size_t)w16.numel(), cur_stream()),
           "lq_fp8_amax_scale");
        at::Tensor codes = at::empty({n, k}, on_gpu(at::kByte));
        ok(lq_fp8_scale_cast(P8(codes), P(w16), lq_dt(w16.scalar_type()), PF(w_scale), 1, (size_t)w16.numel(), cur_stream()),
           "lq_fp8_scale_cast");
        ok(lq_repack_rows32(P8(w_rows32), P8(codes), (size_t)n, (size_t)k, cur_stream()), "lq_repack_rows32");
    }
    void load(const Source& src, const std::string& key, int64_t d_out, int64_t d_in, at::ScalarType T) {
        n = d_out, k = d_in;
        master_h = src.get(key + ".weight", {n, k}, T).cpu().clone();
        in_scale = src.get(key + "_input_scale", {1}, at::kFloat).to(at::kCUDA);
        bias = src.get(key + ".bias", {n}, T).to(at::kCUDA);
        w_scale = at::zeros({1}, on_gpu(at::kFloat));
        w_rows32 = at::empty({n, k}, on_gpu(at::kByte));
        requantise(master_h.to(at::kCUDA));
    }
    void load_lora(const at::Tensor& delta, double alpha) {
        at::Tensor w16 = master_h.to(at::kCUDA);
        TORCH_CHECK(delta.numel() == w16.numel(), "lora_weights holds ", delta.numel(), " elements, the weight ", w16.numel());
        at::Tensor dl = delta.to(w16.options()).reshape(w16.sizes()).contiguous();
        ok(lq_load_lora(P(w16), P(dl), lq_dt(w16.scalar_type()), (size_t)w16.numel(), (float)alpha, cur_stream()), "lq_load_lora");
        requantise(w16);
    }
    void clear_lora() { requantise(master_h.to(at::kCUDA)); }

    // FP8 activations inside this file travel as k-panels [K/64][M][64] (lyraquant.h): the quantising kernels write them,
    // the GEMMs fetch them in whole cache lines; codes and outputs are those of the row-major calls.
    at::Tensor cast_input(const at::Tensor& x2) const {  // e4m3 codes of x [M, K] with the calibrated static scale, as k-panels
        at::Tensor q = at::empty({x2.size(1) / 64, x2.size(0), 64}, on_gpu(at::kByte));
        ok(lq_fp8_scale_cast_panels(P8(q), P(x2), lq_dt(x2.scalar_type()), PF(in_scale), 1, (size_t)x2.size(0), (size_t)x2.size(1),
                                    cur_stream()),
           "lq_fp8_scale_cast_panels");
        return q;
    }
    at::Tensor from_panels(const at::Tensor& q, int64_t m, at::ScalarType T) const {
        at::Tensor y = at::empty({m, n}, on_gpu(T));
        ok(lq_gemm_fp8_panels(P(y), lq_dt(T), P8(q), P8(w_rows32), PF(in_scale), PF(w_scale), P(bias), (int)m, (int)n, (int)k, nullptr,
                              cur_stream()),
           "lq_gemm_fp8_panels");
        return y;
    }
    at::Tensor from_panels_gated(const at::Tensor& q, int64_t m, const at::Tensor& gate, int64_t rows_per_gate,
                                 const at::Tensor& residual) const {
        at::Tensor y = at::empty({m, n}, residual.options());
        ok(lq_gemm_fp8_gated_panels(P(y), lq_dt(residual.scalar_type()), P8(q), P8(w_rows32), PF(in_scale), PF(w_scale), P(bias), P(gate),
                                    (size_t)rows_per_gate, P(residual), (int)m, (int)n, (int)k, cur_stream()),
           "lq_gemm_fp8_gated_panels");
        return y;
    }
    // `gate` [B, n] and `residual` [m, n]:  T(T(T(y) * gate) + residual) in the epilogue; row-major codes (written by the W4A4
    // GEMM's epilogue in the INT4 blocks)
    at::Tensor from_codes_gated(const at::Tensor& q, int64_t m, const at::Tensor& gate, int64_t rows_per_gate,
                                const at::Tensor& residual) const {
        at::Tensor y = at::empty({m, n}, residual.options());
        ok(lq_gemm_fp8_gated(P(y), lq_dt(residual.scalar_type()), P8(q), P8(w_rows32), PF(in_scale), PF(w_scale), P(bias), P(gate),
                             (size_t)rows_per_gate, P(residual), (int)m, (int)n, (int)k, cur_stream()),
           "lq_gemm_fp8_gated");
        return y;
    }
};

// W4A4 group-64 linear with its low-rank branch (W4A4GemmWeight.cc:65-83, W4A4Gemm.cc:113-169)
struct W4A4Linear {
    at::Tensor w_rows32, w_scale, smooth, lora_up, lora_down, bias;
    int64_t n = 0, k = 0, rank = 32;

    void load(const Source& src, const std::string& prefix, int64_t d_out, int64_t d_in, bool has_bias, at::ScalarType T) {
        n = d_out, k = d_in;
        at::Tensor packed = src.get(prefix + "packed_weight", {n, k / 2}, at::kChar).to(at::kCUDA);
        w_rows32 = at::empty({n, k / 2}, on_gpu(at::kByte));
        ok(lq_repack_rows32(P8(w_rows32), P8(packed), (size_t)n, (size_t)(k / 2), cur_stream()), "lq_repack_rows32");
        w_scale = src.get(prefix + "weight_scale", {n, k / 64}, at::kFloat).to(at::kCUDA);
        smooth = src.get(prefix + "smooth", {k}, at::kFloat).to(at::kCUDA);
        lora_up = src.get(prefix + "lora_up", {n, rank}, T).to(at::kCUDA);
        lora_down = src.get(prefix + "lora_down", {rank, k}, T).to(at::kCUDA);
        if (has_bias) bias = src.get(prefix + "bias", {n}, T).to(at::kCUDA);
    }
    // quantise + low-rank down + GEMM with the epilogue options of lq_epilogue_t; returns the 16-bit output (undefined
    // when only codes are asked for)
    at::Tensor run(const at::Tensor& x2, const lq_epilogue_t* epi, bool want_output) const {
        const int64_t m = x2.size(0);
        const at::ScalarType T = x2.scalar_type();
        at::Tensor q = at::empty({m, k / 8}, on_gpu(at::kInt)), s = at::empty({m, k / 64}, on_gpu(at::kFloat));
        at::Tensor act = at::empty({m, rank}, on_gpu(T));
        ok(lq_w4a4_quantize_lora_down(static_cast<uint32_t*>(P(q)), P(s), LQ_F32, P(act), lq_dt(T), P(x2), lq_dt(T), PF(smooth),
                                      P(lora_down), (int)m, (int)k, (int)rank, 64, cur_stream()),
           "lq_w4a4_quantize_lora_down");
        at::Tensor y;
        if (want_output) y = at::empty({m, n}, on_gpu(T));
        ok(lq_gemm_w4a4_ex(P(y), lq_dt(T), static_cast<const uint32_t*>(P(q)), P8(w_rows32), P(s), P(w_scale), LQ_F32, P(bias), P(act),
                           P(lora_up), lq_dt(T), (int)rank, (int)m, (int)n, (int)k, 64, epi, cur_stream()),
           "lq_gemm_w4a4_ex");
        return y;
    }
};

// adaLN linear: FP8 at the _FULL levels (AdaFP8LayerNormWeight.cc:36-92), a plain 16-bit linear otherwise (AdaLayerNormWeight)
struct AdaLinear {
    bool fp8 = false;
    FP8Linear q;
    at::Tensor weight, bias;
    void load(const Source& src, const std::string& prefix, int64_t dim, int64_t chunks, bool full, at::ScalarType T) {
        fp8 = full;
        if (full) { q.load(src, prefix + "linear", chunks * dim, dim, T); return; }
        weight = src.get(prefix + "linear.weight", {chunks * dim, dim}, T).to(at::kCUDA);
        bias = src.get(prefix + "linear.bias", {chunks * dim}, T).to(at::kCUDA);
    }
    // msa [chunks, B, D] from the (already SiLU'd) time embedding [B, D]  (AdaFP8LayerNorm.cc:100-175, invokeTranspose102)
    at::Tensor msa(const at::Tensor& temb, int64_t chunks) const {
        const int64_t b = temb.size(0), d = temb.size(1);
        at::Tensor flat = fp8 ? q.from_panels(q.cast_input(temb), b, temb.scalar_type()) : at::linear(temb, weight, bias);
        return b > 1 ? flat.view({b, chunks, d}).transpose(0, 1).contiguous() : flat.view({chunks, 1, d});
    }
};

// (1 + msa[1]) * LayerNorm(x) + msa[0] with the FP8 cast(s) of the consumers fused; x [B, S, D]
at::Tensor adaln_codes(const at::Tensor& x, const at::Tensor& msa, const at::Tensor& in_scale) {  // k-panels [D/64, B*S, 64]
    at::Tensor c = at::empty({x.size(2) / 64, x.size(0) * x.size(1), 64}, on_gpu(at::kByte));
    ok(lq_layernorm_mod_fp8_panels(P8(c), P(x), P(msa[1]), P(msa[0]), lq_dt(x.scalar_type()), PF(in_scale), (size_t)x.size(0),
                                   (size_t)x.size(1), (size_t)x.size(2), 1e-6f, cur_stream()),
       "lq_layernorm_mod_fp8_panels");
    return c;
}
at::Tensor adaln_16(const at::Tensor& x, const at::Tensor& msa) {
    at::Tensor y = at::empty_like(x);
    ok(lq_gate_residual_layernorm_mod(P(y), nullptr, nullptr, nullptr, P(x), P(msa[1]), P(msa[0]), lq_dt(x.scalar_type()),
                                      (size_t)x.size(0), (size_t)x.size(1), (size_t)x.size(2), 1e-6f, cur_stream()),
       "lq_gate_residual_layernorm_mod");
    return y;
}

// q/k RMSNorm + rotary embedding + [text, image] concatenation in one kernel (invokeFusedRmsNormCatAndRope,
// kernels/rope/flux_apply_rope.cu:74-156), then softmax attention on its [B, Sc + S, 3, H, Dh] output.
// Returns [B, Sc + S, D] with the text tokens first.
at::Tensor attention_core(const at::Tensor& qkv, const at::Tensor& ctx_qkv, const at::Tensor& norm_qk, const at::Tensor& norm_added_qk,
                          const at::Tensor& rope, int64_t heads) {
    const int64_t b = qkv.size(0), s = qkv.size(1), d = qkv.size(2) / 3, dh = d / heads;
    const int64_t sc = ctx_qkv.defined() ? ctx_qkv.size(1) : 0;
    const int64_t per_batch = (sc + s) * dh * 2;
    TORCH_CHECK(rope.numel() == per_batch || rope.numel() == b * per_batch, "rope_emb must be [B or 1, ", sc + s, ", ", dh / 2, ", 2, 2]");
    at::Tensor cat = at::empty({b, sc + s, 3, heads, dh}, qkv.options());
    ok(lq_rmsnorm_rope(P(cat), P(qkv), P(ctx_qkv), P(norm_qk), P(norm_added_qk), P(rope), rope.numel() != per_batch ? (size_t)per_batch : 0,
                       lq_dt(qkv.scalar_type()), (int)b, (int)s, (int)sc, (int)heads, (int)dh, 1e-6f, cur_stream()),
       "lq_rmsnorm_rope");
    at::Tensor o = at::scaled_dot_product_attention(cat.select(2, 0).transpose(1, 2), cat.select(2, 1).transpose(1, 2),
                                                    cat.select(2, 2).transpose(1, 2));
    return o.transpose(1, 2).reshape({b, sc + s, d});
}

// FluxAttnPostFP8Processor::forward (FluxAttnPostFP8Processor.cc:93-240) in three launches
struct AttnPostFP8 {
    FP8Linear gelu_proj, ff_linear;
    void load(const Source& src, const std::string& prefix, int64_t dim, at::ScalarType T) {
        gelu_proj.load(src, prefix + "net.0.proj", 4 * dim, dim, T);
        ff_linear.load(src, prefix + "net.2", dim, 4 * dim, T);
    }
    at::Tensor forward(const at::Tensor& x, const at::Tensor& attn, const at::Tensor& msa) const {
        const int64_t b = x.size(0), s = x.size(1), d = x.size(2), m = b * s;
        const lq_dtype_t dt = lq_dt(x.scalar_type());
        at::Tensor q1 = at::empty({d / 64, m, 64}, on_gpu(at::kByte)), hidden = at::empty_like(x);
        ok(lq_gate_residual_layernorm_mod_fp8_panels(P8(q1), P(hidden), P(attn), P(msa[2]), P(x), P(msa[4]), P(msa[3]), dt,
                                                     PF(gelu_proj.in_scale), (size_t)b, (size_t)s, (size_t)d, 1e-6f, cur_stream()),
           "lq_gate_residual_layernorm_mod_fp8_panels");
        at::Tensor q2 = at::empty({4 * d / 64, m, 64}, on_gpu(at::kByte));
        ok(lq_gemm_fp8_codes_panels(P8(q2), PF(ff_linear.in_scale), dt, P8(q1), P8(gelu_proj.w_rows32), PF(gelu_proj.in_scale),
                                    PF(gelu_proj.w_scale), P(gelu_proj.bias), 1, (int)m, (int)(4 * d), (int)d, cur_stream()),
           "lq_gemm_fp8_codes_panels");
        return ff_linear.from_panels_gated(q2, m, msa[5], s, hidden).view({b, s, d});
    }
};

// FluxAttnPostInt4Processor::forward (FluxAttnPostInt4Processor.cc:103-215)
struct AttnPostInt4 {
    W4A4Linear gelu_proj;
    FP8Linear ff_linear;
    void load(const Source& src, const std::string& prefix, int64_t dim, at::ScalarType T) {
        gelu_proj.load(src, prefix + "net.0.proj.", 4 * dim, dim, true, T);
        ff_linear.load(src, prefix + "net.2", dim, 4 * dim, T);
    }
    at::Tensor forward(const at::Tensor& x, const at::Tensor& attn, const at::Tensor& msa) const {
        const int64_t b = x.size(0), s = x.size(1), d = x.size(2), m = b * s;
        at::Tensor norm = at::empty_like(x), hidden = at::empty_like(x);
        ok(lq_gate_residual_layernorm_mod(P(norm), P(hidden), P(attn), P(msa[2]), P(x), P(msa[4]), P(msa[3]), lq_dt(x.scalar_type()),
                                          (size_t)b, (size_t)s, (size_t)d, 1e-6f, cur_stream()),
           "lq_gate_residual_layernorm_mod");
        at::Tensor q2 = at::empty({m, 4 * d}, on_gpu(at::kByte));
        lq_epilogue_t epi = {2, nullptr, nullptr, 1, nullptr, P8(q2), (size_t)(4 * d), PF(ff_linear.in_scale)};
        gelu_proj.run(norm.view({m, d}), &epi, false);
        return ff_linear.from_codes_gated(q2, m, msa[5], s, hidden).view({b, s, d});
    }
};

void check_input(const at::Tensor& t, const char* name, at::ScalarType T) {  // CHECK_TH_CUDA, CHECK_CONTIGUOUS, th_utils.h:14-33
    TORCH_CHECK(t.is_cuda(), name, " must be a CUDA tensor");
    TORCH_CHECK(t.is_contiguous(), name, " must be contiguous");
    TORCH_CHECK(t.scalar_type() == T, name, " dtype should be ", T);
}

struct BlockConfig {
    at::ScalarType T;
    int64_t dim, heads, head_dim, mlp_scale, level;
    bool int4, full;
    BlockConfig(const std::string& inference_dtype, int64_t embedding_dim, int64_t embedding_head_num, int64_t embedding_head_dim,
                int64_t mlp, int64_t quant_level)
        : dim(embedding_dim), heads(embedding_head_num), head_dim(embedding_head_dim), mlp_scale(mlp), level(quant_level) {
        if (inference_dtype == "fp16") T = at::kHalf;
        else if (inference_dtype == "bf16") T = at::kBFloat16;
        else TORCH_CHECK(false, "wrong inference_dtype");  // fp32 blocks hold no quantized linear in the reference either
        TORCH_CHECK(level == 1 || level == 2 || level == 7 || level == 8, "quant level ", level,
                    ": only the FP8 (1, 2) and INT4 (7, 8) blocks are built on this library");
        TORCH_CHECK(dim == heads * head_dim, "embedding_dim must equal embedding_head_num * embedding_head_dim");
        int4 = level >= 7;
        full = level == 2 || level == 8;
    }
};

std::string join(const std::vector<std::string>& parts) {
    std::string s;
    for (size_t i = 0; i < parts.size(); ++i) s += (i ? "." : "") + parts[i];
    return s;
}

}  // namespace

struct LyraDiffCommonContext : th::CustomClassHolder {
    // the reference creates its stream, cuBLAS handles and allocator here (th_op/lyradiff_common_context/
    // LyraDiffCommonContext.h); this library works on PyTorch's current stream and allocator and needs none of it
    LyraDiffCommonContext() = default;
};

// Double-stream block: FluxTransformerFP8Block.cc:159-262 / FluxTransformerInt4Block.cc:159-246
struct FluxTransformerBlockOp : th::CustomClassHolder {
    BlockConfig cfg;
    bool loaded = false;
    std::mutex lock;
    AdaLinear norm1, norm1_context;
    FP8Linear to_qkv, to_added_qkv, to_out, to_add_out;
    W4A4Linear to_qkv4, to_added_qkv4, to_out4, to_add_out4;
    AttnPostFP8 ff, ff_context;
    AttnPostInt4 ff4, ff_context4;
    at::Tensor norm_qk, norm_added_qk;

    FluxTransformerBlockOp(std::string inference_dtype, int64_t embedding_dim, int64_t embedding_head_num, int64_t embedding_head_dim,
                           int64_t mlp_scale, int64_t quant_level)
        : cfg(inference_dtype, embedding_dim, embedding_head_num, embedding_head_dim, mlp_scale, quant_level) {}

    void initialize(const c10::intrusive_ptr<LyraDiffCommonContext>&) {}

    void load(const Source& src, const std::string& p) {
        std::lock_guard<std::mutex> g(lock);
        const at::ScalarType T = cfg.T;
        const int64_t d = cfg.dim;
        norm1.load(src, p + "norm1.", d, 6, cfg.full, T);
        norm1_context.load(src, p + "norm1_context.", d, 6, cfg.full, T);
        if (cfg.int4) {
            to_qkv4.load(src, p + "attn.to_qkv.", 3 * d, d, true, T);
            to_added_qkv4.load(src, p + "attn.to_added_qkv.", 3 * d, d, true, T);
            to_out4.load(src, p + "attn.to_out.0.", d, d, true, T);
            to_add_out4.load(src, p + "attn.to_add_out.", d, d, true, T);
            ff4.load(src, p + "ff.", d, T);
            ff_context4.load(src, p + "ff_context.", d, T);
        } else {
            to_qkv.load(src, p + "attn.to_qkv", 3 * d, d, T);
            to_added_qkv.load(src, p + "attn.to_added_qkv", 3 * d, d, T);
            to_out.load(src, p + "attn.to_out.0", d, d, T);
            to_add_out.load(src, p + "attn.to_add_out", d, d, T);
            ff.load(src, p + "ff.", d, T);
            ff_context.load(src, p + "ff_context.", d, T);
        }
        auto nw = [&](const char* n) { return src.get(p + "attn." + n + ".weight", {cfg.head_dim}, T).to(at::kCUDA); };
        norm_qk = at::cat({nw("norm_q"), nw("norm_k")});
        norm_added_qk = at::cat({nw("norm_added_q"), nw("norm_added_k")});
        loaded = true;
    }
    void reload_model_from_state_dict(std::string prefix, th::Dict<std::string, th::Tensor> weights, std::string /*device*/) {
        load(DictSource(std::move(weights)), prefix);
    }
    void reload_model_from_bin(std::string model_path, std::string model_dtype) { load(BinSource(model_dtype), model_path); }

    std::map<std::string, FP8Linear*> lora_targets() {
        std::map<std::string, FP8Linear*> t = {{"attn.to_qkv", &to_qkv}, {"attn.to_added_qkv", &to_added_qkv},
                                               {"attn.to_out.0", &to_out}, {"attn.to_add_out", &to_add_out},
                                               {"ff.net.0.proj", &ff.gelu_proj}, {"ff.net.2", &ff.ff_linear},
                                               {"ff_context.net.0.proj", &ff_context.gelu_proj}, {"ff_context.net.2", &ff_context.ff_linear}};
        if (norm1.fp8) t["norm1.linear"] = &norm1.q, t["norm1_context.linear"] = &norm1_context.q;
        return t;
    }
    void load_lora_by_name(std::vector<std::string> lora_name, th::Tensor lora_weights, double lora_strength) {
        TORCH_CHECK(loaded, "reload_model_from_state_dict has not been called");
        const std::string key = join(lora_name);
        // the reference's INT4 block weights register no LoRA targets (FluxTransformerInt4BlockWeight.cc:41-45)
        TORCH_CHECK(!cfg.int4, "no LoRA target named ", key, ": the INT4 blocks carry their low-rank branch in the checkpoint");
        auto t = lora_targets();
        auto it = t.find(key);
        TORCH_CHECK(it != t.end(), "no FP8 linear named ", key, " in this block");
        std::lock_guard<std::mutex> g(lock);
        it->second->load_lora(lora_weights, lora_strength);
    }
    void clear_lora() {
        TORCH_CHECK(loaded, "reload_model_from_state_dict has not been called");
        if (cfg.int4) return;
        std::lock_guard<std::mutex> g(lock);
        for (auto& kv : lora_targets()) kv.second->clear_lora();
    }

    std::vector<th::Tensor> forward(th::Tensor hidden_states, th::Tensor encoder_hidden_states, th::Tensor rope_emb, th::Tensor temb_emb) {
        TORCH_CHECK(loaded, "reload_model_from_state_dict has not been called");
        check_input(hidden_states, "hidden_states", cfg.T);
        check_input(encoder_hidden_states, "encoder_hidden_states", cfg.T);
        check_input(rope_emb, "rope_emb", cfg.T);
        check_input(temb_emb, "temb_emb", cfg.T);
        std::lock_guard<std::mutex> g(lock);
        const at::Tensor &x = hidden_states, &c = encoder_hidden_states;
        const int64_t b = x.size(0), s = x.size(1), sc = c.size(1), d = cfg.dim;
        at::Tensor temb = temb_emb.reshape({b, d});
        at::Tensor msa = norm1.msa(temb, 6), cmsa = norm1_context.msa(temb, 6);
        at::Tensor qkv, cqkv;
        if (cfg.int4) {
            qkv = to_qkv4.run(adaln_16(x, msa).view({b * s, d}), nullptr, true).view({b, s, 3 * d});
            cqkv = to_added_qkv4.run(adaln_16(c, cmsa).view({b * sc, d}), nullptr, true).view({b, sc, 3 * d});
        } else {
            qkv = to_qkv.from_panels(adaln_codes(x, msa, to_qkv.in_scale), b * s, cfg.T).view({b, s, 3 * d});
            cqkv = to_added_qkv.from_panels(adaln_codes(c, cmsa, to_added_qkv.in_scale), b * sc, cfg.T).view({b, sc, 3 * d});
        }
        at::Tensor o = attention_core(qkv, cqkv, norm_qk, norm_added_qk, rope_emb, cfg.heads);
        at::Tensor attn = o.slice(1, sc, sc + s).contiguous().view({b * s, d}), cattn = o.slice(1, 0, sc).contiguous().view({b * sc, d});
        if (cfg.int4) {
            at::Tensor a_out = to_out4.run(attn, nullptr, true).view({b, s, d}), c_out = to_add_out4.run(cattn, nullptr, true).view({b, sc, d});
            return {ff4.forward(x, a_out, msa), ff_context4.forward(c, c_out, cmsa)};
        }
        at::Tensor a_out = to_out.from_panels(to_out.cast_input(attn), b * s, cfg.T).view({b, s, d});
        at::Tensor c_out = to_add_out.from_panels(to_add_out.cast_input(cattn), b * sc, cfg.T).view({b, sc, d});
        return {ff.forward(x, a_out, msa), ff_context.forward(c, c_out, cmsa)};
    }
};

// Single-stream block: FluxSingleTransformerFP8Block.cc:163-291 / FluxSingleTransformerInt4Block.cc:178-316
struct FluxSingleTransformerBlockOp : th::CustomClassHolder {
    BlockConfig cfg;
    bool loaded = false;
    std::mutex lock;
    AdaLinear norm;
    FP8Linear to_qkv, proj_mlp, proj_out;
    W4A4Linear to_qkv4, proj_mlp4, proj_out_1, proj_out_2;
    at::Tensor norm_qk;

    FluxSingleTransformerBlockOp(std::string inference_dtype, int64_t embedding_dim, int64_t embedding_head_num,
                                 int64_t embedding_head_dim, int64_t mlp_scale, int64_t quant_level)
        : cfg(inference_dtype, embedding_dim, embedding_head_num, embedding_head_dim, mlp_scale, quant_level) {}

    void initialize(const c10::intrusive_ptr<LyraDiffCommonContext>&) {}

    void load(const Source& src, const std::string& p) {
        std::lock_guard<std::mutex> g(lock);
        const at::ScalarType T = cfg.T;
        const int64_t d = cfg.dim, f = cfg.mlp_scale * cfg.dim;
        norm.load(src, p + "norm.", d, 3, cfg.full, T);
        if (cfg.int4) {
            to_qkv4.load(src, p + "attn.to_qkv.", 3 * d, d, true, T);
            proj_mlp4.load(src, p + "proj_mlp.", f, d, true, T);
            proj_out_1.load(src, p + "proj_out.linears.0.", d, d, true, T);
            proj_out_2.load(src, p + "proj_out.linears.1.linear.", d, f, false, T);
        } else {
            to_qkv.load(src, p + "attn.to_qkv", 3 * d, d, T);
            proj_mlp.load(src, p + "proj_mlp", f, d, T);
            proj_out.load(src, p + "proj_out", d, d + f, T);
        }
        norm_qk = at::cat({src.get(p + "attn.norm_q.weight", {cfg.head_dim}, T).to(at::kCUDA),
                           src.get(p + "attn.norm_k.weight", {cfg.head_dim}, T).to(at::kCUDA)});
        loaded = true;
    }
    void reload_model_from_state_dict(std::string prefix, th::Dict<std::string, th::Tensor> weights, std::string /*device*/) {
        load(DictSource(std::move(weights)), prefix);
    }
    void reload_model_from_bin(std::string model_path, std::string model_dtype) { load(BinSource(model_dtype), model_path); }

    std::map<std::string, FP8Linear*> lora_targets() {
        std::map<std::string, FP8Linear*> t = {{"attn.to_qkv", &to_qkv}, {"proj_mlp", &proj_mlp}, {"proj_out", &proj_out}};
        if (norm.fp8) t["norm.linear"] = &norm.q;
        return t;
    }
    void load_lora_by_name(std::vector<std::string> lora_name, th::Tensor lora_weights, double lora_strength) {
        TORCH_CHECK(loaded, "reload_model_from_state_dict has not been called");
        const std::string key = join(lora_name);
        TORCH_CHECK(!cfg.int4, "no LoRA target named ", key, ": the INT4 blocks carry their low-rank branch in the checkpoint");
        auto t = lora_targets();
        auto it = t.find(key);
        TORCH_CHECK(it != t.end(), "no FP8 linear named ", key, " in this block");
        std::lock_guard<std::mutex> g(lock);
        it->second->load_lora(lora_weights, lora_strength);
    }
    void clear_lora() {
        TORCH_CHECK(loaded, "reload_model_from_state_dict has not been called");
        if (cfg.int4) return;
        std::lock_guard<std::mutex> g(lock);
        for (auto& kv : lora_targets()) kv.second->clear_lora();
    }

    th::Tensor forward(th::Tensor hidden_states, th::Tensor rope_emb, th::Tensor temb_emb) {
        TORCH_CHECK(loaded, "reload_model_from_state_dict has not been called");
        check_input(hidden_states, "hidden_states", cfg.T);
        check_input(rope_emb, "rope_emb", cfg.T);
        check_input(temb_emb, "temb_emb", cfg.T);
        std::lock_guard<std::mutex> g(lock);
        const at::Tensor& x = hidden_states;
        const int64_t b = x.size(0), s = x.size(1), d = cfg.dim, m = b * s, f = cfg.mlp_scale * d;
        const lq_dtype_t dt = lq_dt(cfg.T);
        at::Tensor msa = norm.msa(temb_emb.reshape({b, d}), 3);
        at::Tensor gate = msa[2].contiguous(), none;
        if (cfg.int4) {
            at::Tensor nh = adaln_16(x, msa).view({m, d});
            at::Tensor attn = attention_core(to_qkv4.run(nh, nullptr, true).view({b, s, 3 * d}), none, norm_qk, none, rope_emb, cfg.heads)
                                  .contiguous().view({m, d});
            lq_epilogue_t gelu = {2, nullptr, nullptr, 1, nullptr, nullptr, 0, nullptr};
            at::Tensor mlp = proj_mlp4.run(nh, &gelu, true);
            at::Tensor h1 = proj_out_1.run(attn, nullptr, true);
            lq_epilogue_t tail = {0, P(h1), P(gate), (size_t)s, P(x), nullptr, 0, nullptr};
            return proj_out_2.run(mlp, &tail, true).view({b, s, d});
        }
        // one adaLN read yields the codes for to_qkv and for proj_mlp
        at::Tensor c_qkv = at::empty({d / 64, m, 64}, on_gpu(at::kByte)), c_mlp = at::empty({d / 64, m, 64}, on_gpu(at::kByte));
        ok(lq_layernorm_mod_fp8_dual_panels(P8(c_qkv), PF(to_qkv.in_scale), P8(c_mlp), PF(proj_mlp.in_scale), P(x), P(msa[1]), P(msa[0]),
                                            dt, (size_t)b, (size_t)s, (size_t)d, 1e-6f, cur_stream()),
           "lq_layernorm_mod_fp8_dual_panels");
        at::Tensor attn = attention_core(to_qkv.from_panels(c_qkv, m, cfg.T).view({b, s, 3 * d}), none, norm_qk, none, rope_emb, cfg.heads)
                              .contiguous();
        // proj_out's input [attn | gelu(mlp)] as e4m3 codes in k-panels [(D + F)/64, M, 64]: a block of columns is a run of whole
        // panels, so the attention columns are a cast into the first D/64 panels and the mlp columns come straight from the
        // proj_mlp GEMM's epilogue into the rest (FluxSingleTransformerFP8Block.cc:216-253)
        at::Tensor q2 = at::empty({(d + f) / 64, m, 64}, on_gpu(at::kByte));
        ok(lq_fp8_scale_cast_panels(P8(q2), P(attn), dt, PF(proj_out.in_scale), 1, (size_t)m, (size_t)d, cur_stream()),
           "lq_fp8_scale_cast_panels");
        ok(lq_gemm_fp8_codes_panels(P8(q2) + (size_t)(d / 64) * (size_t)m * 64, PF(proj_out.in_scale), dt, P8(c_mlp), P8(proj_mlp.w_rows32),
                                    PF(proj_mlp.in_scale), PF(proj_mlp.w_scale), P(proj_mlp.bias), 2, (int)m, (int)f, (int)d, cur_stream()),
           "lq_gemm_fp8_codes_panels");
        return proj_out.from_panels_gated(q2, m, gate, s, x.view({m, d})).view({b, s, d});
    }
};

}  // namespace torch_ext

// torch_ops.py registers its operators in the same namespace from Python, so this block is a fragment of it
TORCH_LIBRARY_FRAGMENT(lyradiff, m) {
    m.class_<torch_ext::LyraDiffCommonContext>("LyraDiffCommonContext").def(th::init<>());

    m.class_<torch_ext::FluxTransformerBlockOp>("FluxTransformerBlockOp")
        .def(th::init<std::string, int64_t, int64_t, int64_t, int64_t, int64_t>(), "",
             {th::arg("inference_dtype") = "bf16", th::arg("embedding_dim") = 3072, th::arg("embedding_head_num") = 24,
              th::arg("embedding_head_dim") = 128, th::arg("mlp_scale") = 6, th::arg("quant_level") = 0})
        .def("initialize", &torch_ext::FluxTransformerBlockOp::initialize)
        .def("forward", &torch_ext::FluxTransformerBlockOp::forward)
        .def("load_lora_by_name", &torch_ext::FluxTransformerBlockOp::load_lora_by_name)
        .def("clear_lora", &torch_ext::FluxTransformerBlockOp::clear_lora)
        .def("reload_model_from_bin", &torch_ext::FluxTransformerBlockOp::reload_model_from_bin)
        .def("reload_model_from_state_dict", &torch_ext::FluxTransformerBlockOp::reload_model_from_state_dict);

    m.class_<torch_ext::FluxSingleTransformerBlockOp>("FluxSingleTransformerBlockOp")
        .def(th::init<std::string, int64_t, int64_t, int64_t, int64_t, int64_t>(), "",
             {th::arg("inference_dtype") = "bf16", th::arg("embedding_dim") = 3072, th::arg("embedding_head_num") = 24,
              th::arg("embedding_head_dim") = 128, th::arg("mlp_scale") = 4, th::arg("quant_level") = 0})
        .def("initialize", &torch_ext::FluxSingleTransformerBlockOp::initialize)
        .def("forward", &torch_ext::FluxSingleTransformerBlockOp::forward)
        .def("load_lora_by_name", &torch_ext::FluxSingleTransformerBlockOp::load_lora_by_name)
        .def("clear_lora", &torch_ext::FluxSingleTransformerBlockOp::clear_lora)
        .def("reload_model_from_bin", &torch_ext::FluxSingleTransformerBlockOp::reload_model_from_bin)
        .def("reload_model_from_state_dict", &torch_ext::FluxSingleTransformerBlockOp::reload_model_from_state_dict);
}
