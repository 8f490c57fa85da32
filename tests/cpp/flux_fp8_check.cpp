// Reference-style use of the FP8 FLUX feed-forward types (FluxAttnPostFP8ProcessorWeight / Processor,
// FluxSingleTransformerFP8MlpWeight / Mlp, FP8LoraWeight) on liblyraquant.so.  Each fused forward is compared
// BIT FOR BIT with the reference's own launch sequence run step by step: the library's unfused launchers for the
// casts, the LayerNorm and the GEMMs, host loops (rounding to bf16 after every operation) for the gate/residual
// steps.  Exit code 0 when every check passes; one line per check.  Built by lyradiff_amd/build.py, run by
// tests/test_gpu_compat.py.
#include <cmath>
#include <unistd.h>
#include <cstdio>
#include <cstdlib>
#include <vector>

#include "lyradiff_layers.h"

#define CK(x)                                                                        \
    do {                                                                             \
        hipError_t e = (x);                                                          \
        if (e != hipSuccess) {                                                       \
            std::printf("HIP error %s at line %d\n", hipGetErrorString(e), __LINE__); \
            return 2;                                                                \
        }                                                                            \
    } while (0)

using namespace lyradiff;
typedef hip_bfloat16 bf16;

static float lcg(unsigned& s) { s = s * 1664525u + 1013904223u; return ((s >> 8) & 0xFFFF) / 65536.0f - 0.5f; }
static float r16(float f) { return (float)bf16(f); }

static std::vector<bf16> rand_bf16(size_t n, float scale, unsigned& seed) {
    std::vector<bf16> v(n);
    for (auto& x : v) x = bf16(scale * lcg(seed));
    return v;
}
template <typename U> static U* upload(const std::vector<U>& h) {
    U* d = nullptr;
    if (hipMalloc(reinterpret_cast<void**>(&d), h.size() * sizeof(U)) != hipSuccess) std::abort();
    if (hipMemcpy(d, h.data(), h.size() * sizeof(U), hipMemcpyHostToDevice) != hipSuccess) std::abort();
    return d;
}
template <typename U> static std::vector<U> download(const U* d, size_t n) {
    std::vector<U> h(n);
    if (hipMemcpy(h.data(), d, n * sizeof(U), hipMemcpyDeviceToHost) != hipSuccess) std::abort();
    return h;
}
// out = T( T(x * gate[b]) + res ), the reference's fuseGateAndResidual
static std::vector<bf16> gate_residual(const std::vector<bf16>& x, const std::vector<bf16>& gate, const std::vector<bf16>& res,
                                       size_t batch, size_t seq, size_t d) {
    std::vector<bf16> o(batch * seq * d);
    for (size_t b = 0; b < batch; ++b)
        for (size_t s = 0; s < seq; ++s)
            for (size_t j = 0; j < d; ++j) {
                const size_t i = (b * seq + s) * d + j;
                o[i] = bf16(r16((float)x[i] * (float)gate[b * d + j]) + (float)res[i]);
            }
    return o;
}
static int count_diff(const std::vector<bf16>& a, const std::vector<bf16>& b) {
    int bad = 0;
    for (size_t i = 0; i < a.size(); ++i) bad += (float)a[i] != (float)b[i];
    return bad + (a.size() != b.size());
}

int main() {
    hipStream_t st;
    CK(hipStreamCreate(&st));
    Allocator allocator;
    allocator.setStream(st);
    int failures = 0;
    unsigned seed = 5;
    const lq_dtype_t dt = LQ_BF16;

    // ---------------- FluxAttnPostFP8Processor<bf16> ---------------------------------------------------------------
    {
        const size_t B = 2, S = 70, D = 128, M = B * S;
        auto w1 = rand_bf16(4 * D * D, 0.12f, seed), b1 = rand_bf16(4 * D, 0.3f, seed);
        auto w2 = rand_bf16(4 * D * D, 0.12f, seed), b2 = rand_bf16(D, 0.3f, seed);
        float s_in1 = 5.0f / 448.0f, s_in2 = 1.5f / 448.0f;
        auto x = rand_bf16(M * D, 3.0f, seed), attn = rand_bf16(M * D, 3.0f, seed), msa = rand_bf16(6 * B * D, 1.5f, seed);
        std::unordered_map<std::string, void*> cache = {
            {"blk.ff.net.0.proj.weight", w1.data()}, {"blk.ff.net.0.proj.bias", b1.data()}, {"blk.ff.net.0.proj_input_scale", &s_in1},
            {"blk.ff.net.2.weight", w2.data()},      {"blk.ff.net.2.bias", b2.data()},      {"blk.ff.net.2_input_scale", &s_in2}};
        bf16 *dx = upload(x), *dattn = upload(attn), *dmsa = upload(msa), *dout;
        CK(hipMalloc(&dout, M * D * 2));
        try {
            FluxAttnPostFP8ProcessorWeight<bf16> weights(D, LyraQuantType::FP8_W8A8, &allocator);
            weights.loadWeightsFromCache("blk.ff.", cache, hipMemcpyHostToDevice);
            FluxAttnPostFP8Processor<bf16> proc(D, st, nullptr, &allocator, false);
            TensorMap in({{"input", Tensor(MEMORY_GPU, TYPE_BF16, {B, S, D}, dx)}, {"attn_output", Tensor(MEMORY_GPU, TYPE_BF16, {B, S, D}, dattn)},
                          {"msa_input", Tensor(MEMORY_GPU, TYPE_BF16, {6, B, D}, dmsa)}});
            TensorMap out({{"output", Tensor(MEMORY_GPU, TYPE_BF16, {B, S, D}, dout)}});
            proc.forward(&out, &in, &weights);
            CK(hipStreamSynchronize(st));
            auto got = download(dout, M * D);

            // the reference's sequence, one step at a time
            std::vector<bf16> gate_msa(msa.begin() + 2 * B * D, msa.begin() + 3 * B * D), gate_mlp(msa.begin() + 5 * B * D, msa.end());
            auto hidden = gate_residual(attn, gate_msa, x, B, S, D);
            bf16* dhidden = upload(hidden);
            uint8_t *q1, *q2;
            bf16 *inner, *ff;
            CK(hipMalloc(&q1, M * D)); CK(hipMalloc(&q2, M * 4 * D)); CK(hipMalloc(&inner, M * 4 * D * 2)); CK(hipMalloc(&ff, M * D * 2));
            detail::check(lq_layernorm_mod_fp8(q1, dhidden, dmsa + 4 * B * D, dmsa + 3 * B * D, dt, weights.gelu_proj_input_scale, B, S, D, 1e-6f, st), "ln");
            detail::check(lq_gemm_fp8(inner, dt, q1, reinterpret_cast<const uint8_t*>(weights.gelu_proj_weight), weights.gelu_proj_input_scale,
                                      weights.gelu_proj_weight_scale, weights.gelu_proj_bias, 1, nullptr, 0.f, (int)M, (int)(4 * D), (int)D, st), "up");
            detail::check(lq_fp8_scale_cast(q2, inner, dt, weights.ff_linear_input_scale, 1, M * 4 * D, st), "cast");
            detail::check(lq_gemm_fp8(ff, dt, q2, reinterpret_cast<const uint8_t*>(weights.ff_linear_weight), weights.ff_linear_input_scale,
                                      weights.ff_linear_weight_scale, weights.ff_linear_bias, 0, nullptr, 0.f, (int)M, (int)D, (int)(4 * D), st), "down");
            CK(hipStreamSynchronize(st));
            auto want = gate_residual(download(ff, M * D), gate_mlp, hidden, B, S, D);
            const int bad = count_diff(got, want);
            double energy = 0;
            for (auto v : got) energy += std::fabs((float)v);
            std::printf("FluxAttnPostFP8Processor<bf16>: B=%zu S=%zu D=%zu, mean |out| %.3f, %d mismatches\n", B, S, D, energy / got.size(), bad);
            failures += bad != 0 || !(energy > 0);

            // LoRA: merge a delta into net.2, outputs change; clear it, outputs return bit for bit
            auto delta = rand_bf16(4 * D * D, 0.2f, seed);
            bf16* ddelta = upload(delta);
            weights.lora_weight_map.at("net.2")->load_lora(ddelta, 0.75f, &allocator);
            proc.forward(&out, &in, &weights);
            CK(hipStreamSynchronize(st));
            const int changed = count_diff(download(dout, M * D), got);
            weights.lora_weight_map.at("net.2")->clear_lora(&allocator);
            proc.forward(&out, &in, &weights);
            CK(hipStreamSynchronize(st));
            const int restored = count_diff(download(dout, M * D), got);
            std::printf("FP8LoraWeight load/clear: %d outputs changed by the merge, %d mismatches after clear\n", changed, restored);
            failures += changed == 0 || restored != 0;

            // the same weights from the reference's raw .bin files (loadWeights: MACROLoadFP8WeightFromBin), stored as bf16
            char dir_tmpl[] = "/tmp/lq_fp8_XXXXXX";
            const char* dir = mkdtemp(dir_tmpl);
            if (dir == nullptr) { std::printf("mkdtemp failed\n"); return 2; }
            const std::string fprefix = std::string(dir) + "/ff.";
            const char* names[6] = {"net.0.proj.weight.bin", "net.0.proj.bias.bin", "net.0.proj_input_scale.bin",
                                    "net.2.weight.bin", "net.2.bias.bin", "net.2_input_scale.bin"};
            const void* datas[6] = {w1.data(), b1.data(), &s_in1, w2.data(), b2.data(), &s_in2};
            const size_t sizes[6] = {w1.size() * 2, b1.size() * 2, 4, w2.size() * 2, b2.size() * 2, 4};
            bool wrote = true;
            for (int i = 0; i < 6; ++i) {
                std::FILE* f = std::fopen((fprefix + names[i]).c_str(), "wb");
                wrote = wrote && f != nullptr && std::fwrite(datas[i], 1, sizes[i], f) == sizes[i];
                if (f) std::fclose(f);
            }
            FluxAttnPostFP8ProcessorWeight<bf16> from_files(D, LyraQuantType::FP8_W8A8, &allocator);
            from_files.loadWeights(fprefix, FtCudaDataType::BF16);
            CK(hipMemset(dout, 0, M * D * 2));
            proc.forward(&out, &in, &from_files);
            CK(hipStreamSynchronize(st));
            const int badf = (wrote ? 0 : 1) + count_diff(download(dout, M * D), got);
            std::printf("FluxAttnPostFP8ProcessorWeight::loadWeights from .bin files: %d mismatches\n", badf);
            failures += badf != 0;
            for (int i = 0; i < 6; ++i) std::remove((fprefix + names[i]).c_str());
            rmdir(dir);
        } catch (const std::exception& e) {
            std::printf("exception: %s\n", e.what());
            return 3;
        }
    }

    // ---------------- FluxSingleTransformerFP8Mlp<bf16> ------------------------------------------------------------
    {
        const size_t B = 2, S = 45, D = 128, MS = 4, M = B * S, F = MS * D;
        auto wm = rand_bf16(F * D, 0.12f, seed), bm = rand_bf16(F, 0.3f, seed);
        auto wo = rand_bf16(D * (D + F), 0.12f, seed), bo = rand_bf16(D, 0.3f, seed);
        float s_mlp = 2.0f / 448.0f, s_out = 2.0f / 448.0f;
        auto x = rand_bf16(M * D, 3.0f, seed), norm = rand_bf16(M * D, 3.0f, seed), attn = rand_bf16(M * D, 3.0f, seed);
        auto gate = rand_bf16(B * D, 1.5f, seed);
        std::unordered_map<std::string, void*> cache = {
            {"s.proj_mlp.weight", wm.data()}, {"s.proj_mlp.bias", bm.data()}, {"s.proj_mlp_input_scale", &s_mlp},
            {"s.proj_out.weight", wo.data()}, {"s.proj_out.bias", bo.data()}, {"s.proj_out_input_scale", &s_out}};
        bf16 *dx = upload(x), *dnorm = upload(norm), *dattn = upload(attn), *dgate = upload(gate), *dout;
        CK(hipMalloc(&dout, M * D * 2));
        try {
            FluxSingleTransformerFP8MlpWeight<bf16> weights(D, MS, LyraQuantType::FP8_W8A8, &allocator);
            weights.loadWeightsFromCache("s.", cache, hipMemcpyHostToDevice);
            FluxSingleTransformerFP8Mlp<bf16> mlp(D, MS, st, nullptr, &allocator, false);
            TensorMap in({{"input", Tensor(MEMORY_GPU, TYPE_BF16, {B, S, D}, dx)}, {"norm_hidden", Tensor(MEMORY_GPU, TYPE_BF16, {B, S, D}, dnorm)},
                          {"attn_output", Tensor(MEMORY_GPU, TYPE_BF16, {B, S, D}, dattn)}, {"gate", Tensor(MEMORY_GPU, TYPE_BF16, {B, D}, dgate)}});
            TensorMap out({{"output", Tensor(MEMORY_GPU, TYPE_BF16, {B, S, D}, dout)}});
            mlp.forward(&out, &in, &weights);
            CK(hipStreamSynchronize(st));
            auto got = download(dout, M * D);
            // step by step with the library's own codes for the concatenated input (its GELU is the kernel's own), then the
            // plain GEMM and the host gate/residual
            uint8_t *q1, *cat;
            bf16* o;
            CK(hipMalloc(&q1, M * D)); CK(hipMalloc(&cat, M * (D + F))); CK(hipMalloc(&o, M * D * 2));
            detail::check(lq_fp8_scale_cast(q1, dnorm, dt, weights.proj_mlp_input_scale, 1, M * D, st), "cast");
            detail::check(lq_fp8_scale_cast_2d(cat, D + F, dattn, D, dt, weights.proj_out_input_scale, 1, M, D, st), "cast2d");
            detail::check(lq_gemm_fp8_codes(cat + D, D + F, weights.proj_out_input_scale, dt, q1, reinterpret_cast<const uint8_t*>(weights.proj_mlp_weight),
                                            weights.proj_mlp_input_scale, weights.proj_mlp_weight_scale, weights.proj_mlp_bias, 2, (int)M, (int)F, (int)D, st), "mlp");
            detail::check(lq_gemm_fp8(o, dt, cat, reinterpret_cast<const uint8_t*>(weights.proj_out_weight), weights.proj_out_input_scale,
                                      weights.proj_out_weight_scale, weights.proj_out_bias, 0, nullptr, 0.f, (int)M, (int)D, (int)(D + F), st), "out");
            CK(hipStreamSynchronize(st));
            auto want = gate_residual(download(o, M * D), gate, x, B, S, D);
            const int bad = count_diff(got, want);
            std::printf("FluxSingleTransformerFP8Mlp<bf16>: B=%zu S=%zu D=%zu mlp_scale=%zu, %d mismatches\n", B, S, D, MS, bad);
            failures += bad != 0;
        } catch (const std::exception& e) {
            std::printf("exception: %s\n", e.what());
            return 3;
        }
    }
    // ---------------- invokeFusedRmsNormCatAndRope / invokeFusedRmsNormAndRope -----------------------------------------
    // Exactly checkable cases of the reference call (FluxAttentionFP8Processor.cc:232-245): a quarter-turn rope with unit
    // norm weights swaps each normalised pair (x, y) -> (-y, x); v is copied; the text rows come first; the single-stream
    // launcher agrees with the concatenating one on the same rows.
    {
        const int B = 2, S = 9, SC = 5, H = 3, DH = 128, T = S + SC;
        auto hid = rand_bf16((size_t)B * S * 3 * H * DH, 3.0f, seed), enc = rand_bf16((size_t)B * SC * 3 * H * DH, 3.0f, seed);
        std::vector<bf16> ones(2 * DH, bf16(1.0f)), eye((size_t)B * T * DH * 2), quarter((size_t)B * T * DH * 2);
        for (size_t i = 0; i < eye.size(); i += 4) {
            eye[i] = bf16(1.0f); eye[i + 1] = bf16(0.0f); eye[i + 2] = bf16(0.0f); eye[i + 3] = bf16(1.0f);
            quarter[i] = bf16(0.0f); quarter[i + 1] = bf16(-1.0f); quarter[i + 2] = bf16(1.0f); quarter[i + 3] = bf16(0.0f);
        }
        bf16 *dh = upload(hid), *de = upload(enc), *d1 = upload(ones), *deye = upload(eye), *dq = upload(quarter), *o1, *o2, *o3;
        const size_t n_out = (size_t)B * T * 3 * H * DH;
        CK(hipMalloc(&o1, n_out * 2)); CK(hipMalloc(&o2, n_out * 2)); CK(hipMalloc(&o3, (size_t)B * S * 3 * H * DH * 2));
        try {
            invokeFusedRmsNormCatAndRope<bf16>(o1, dh, de, d1, d1, deye, 1e-6f, B, S, SC, H, DH, st);
            invokeFusedRmsNormCatAndRope<bf16>(o2, dh, de, d1, d1, dq, 1e-6f, B, S, SC, H, DH, st);
            invokeFusedRmsNormAndRope<bf16>(o3, dh, d1, deye, 1e-6f, B, S, H, DH, st);  // rope rows 0..S-1 of each batch: identity too
            CK(hipStreamSynchronize(st));
            auto a = download(o1, n_out), q = download(o2, n_out), single = download(o3, (size_t)B * S * 3 * H * DH);
            int bad = 0;
            for (int b = 0; b < B; ++b)
                for (int t = 0; t < T; ++t)
                    for (int c = 0; c < 3; ++c)
                        for (int h = 0; h < H; ++h)
                            for (int e = 0; e < DH; e += 2) {
                                const size_t o = ((((size_t)b * T + t) * 3 + c) * H + h) * DH + e;
                                const std::vector<bf16>& src = t < SC ? enc : hid;
                                const size_t si = ((((size_t)b * (t < SC ? SC : S) + (t < SC ? t : t - SC)) * 3 + c) * H + h) * DH + e;
                                if (c == 2) {
                                    bad += (float)a[o] != (float)src[si] || (float)a[o + 1] != (float)src[si + 1];
                                } else {
                                    bad += (float)q[o] != -(float)a[o + 1] || (float)q[o + 1] != (float)a[o];
                                    if (t >= SC) {
                                        const size_t so = ((((size_t)b * S + (t - SC)) * 3 + c) * H + h) * DH + e;
                                        bad += (float)single[so] != (float)a[o] || (float)single[so + 1] != (float)a[o + 1];
                                    }
                                }
                            }
            // RMS of a normalised head is 1
            double ss = 0;
            for (int e = 0; e < DH; ++e) ss += (double)(float)a[e] * (float)a[e];
            bad += std::fabs(std::sqrt(ss / DH) - 1.0) > 0.01;
            std::printf("invokeFusedRmsNormCatAndRope<bf16>: B=%d S=%d Sc=%d H=%d Dh=%d, %d mismatches\n", B, S, SC, H, DH, bad);
            failures += bad != 0;
        } catch (const std::exception& e) {
            std::printf("exception: %s\n", e.what());
            return 3;
        }
    }
    return failures == 0 ? 0 : 1;
}
