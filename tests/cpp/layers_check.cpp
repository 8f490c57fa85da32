// Reference-style use of the layer types (Tensor, TensorMap, Allocator, W4A4GemmWeight, W4A4Gemm,
// CutlassInt8GemmRunner + profiler) on liblyraquant.so, checked bit for bit against host loops.
// Exit code 0 when every check passes; one line per check.  Built by lyradiff_amd/build.py, run by
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

static float lcg(unsigned& s) { s = s * 1664525u + 1013904223u; return ((s >> 8) & 0xFFFF) / 65536.0f - 0.5f; }
static float bf16_round(float f) { return (float)hip_bfloat16(f); }

// group-64 int4 quantisation of one row on the host: q in [-8,7], scale = amax/7 (0 for an all-zero group)
static void quant_row(const float* v, int k, std::vector<int>& q, std::vector<float>& s) {
    for (int g = 0; g < k / 64; ++g) {
        float amax = 0.f;
        for (int j = 0; j < 64; ++j) amax = std::fmax(amax, std::fabs(v[g * 64 + j]));
        const float sc = amax / 7.0f;
        s[g] = sc;
        for (int j = 0; j < 64; ++j) {
            float r = sc == 0.f ? 0.f : std::rint(v[g * 64 + j] / sc);
            q[g * 64 + j] = (int)std::fmin(std::fmax(r, -8.f), 7.f);
        }
    }
}

int main() {
    hipStream_t st;
    CK(hipStreamCreate(&st));
    int failures = 0;
    unsigned seed = 11;

    // ---------------- W4A4Gemm<bf16> layer: weights from a host cache, forward through TensorMaps -------------
    {
        const int m = 100, n = 96, k = 256, G = k / 64;
        std::vector<float> w(n * k), x(m * k), smooth(k), biasf(n);
        for (auto& v : w) v = bf16_round(0.1f * lcg(seed));
        for (auto& v : x) v = bf16_round(3.0f * lcg(seed));
        for (auto& v : smooth) v = 1.0f + lcg(seed);
        for (auto& v : biasf) v = bf16_round(lcg(seed));
        // offline weight quantisation on the host: nibble pairs, low nibble first, row-major [n, k/2]
        std::vector<int> wq(n * k);
        std::vector<float> ws(n * G);
        std::vector<int8_t> wpacked(n * k / 2);
        for (int r = 0; r < n; ++r) {
            std::vector<int> q(k);
            std::vector<float> s(G);
            quant_row(&w[r * k], k, q, s);
            for (int j = 0; j < k; ++j) wq[r * k + j] = q[j];
            for (int g = 0; g < G; ++g) ws[r * G + g] = s[g];
            for (int j = 0; j < k / 2; ++j) wpacked[r * k / 2 + j] = (int8_t)((q[2 * j] & 0xF) | ((q[2 * j + 1] & 0xF) << 4));
        }
        std::vector<hip_bfloat16> bias(n), xb(m * k);
        for (int i = 0; i < n; ++i) bias[i] = hip_bfloat16(biasf[i]);
        for (int i = 0; i < m * k; ++i) xb[i] = hip_bfloat16(x[i]);

        Allocator allocator;
        allocator.setStream(st);
        W4A4GemmWeight<hip_bfloat16> weights(n, k, /*lora_rank=*/0, /*has_bias=*/true, 64, LyraQuantType::INT4_W4A4, &allocator);
        std::unordered_map<std::string, void*> cache = {{"blk.packed_weight", wpacked.data()}, {"blk.weight_scale", ws.data()},
                                                        {"blk.smooth", smooth.data()}, {"blk.bias", bias.data()}};
        hip_bfloat16 *dx, *dy;
        CK(hipMalloc(&dx, m * k * 2));
        CK(hipMalloc(&dy, m * n * 2));
        CK(hipMemcpy(dx, xb.data(), m * k * 2, hipMemcpyHostToDevice));
        try {
            weights.loadWeightsFromCache("blk.", cache, hipMemcpyHostToDevice, st);
            W4A4Gemm<hip_bfloat16> layer(n, k, 0, true, 64, st, nullptr, &allocator, false);
            TensorMap in({{"input", Tensor(MEMORY_GPU, TYPE_BF16, {(size_t)m, (size_t)k}, dx)}});
            TensorMap out({{"output", Tensor(MEMORY_GPU, TYPE_BF16, {(size_t)m, (size_t)n}, dy)}});
            layer.forward(&out, &in, &weights);
            layer.forward(&out, &in, &weights);  // second call reuses the named pool buffers
        } catch (const std::exception& e) {
            std::printf("exception: %s\n", e.what());
            return 3;
        }
        CK(hipStreamSynchronize(st));
        std::vector<hip_bfloat16> y(m * n);
        CK(hipMemcpy(y.data(), dy, m * n * 2, hipMemcpyDeviceToHost));
        int bad = 0;
        for (int i = 0; i < m; ++i) {
            std::vector<float> v(k), s(G);
            std::vector<int> q(k);
            for (int j = 0; j < k; ++j) v[j] = x[i * k + j] / smooth[j];
            quant_row(v.data(), k, q, s);
            for (int j = 0; j < n; ++j) {
                float r = 0.f;
                for (int g = 0; g < G; ++g) {
                    int p = 0;
                    for (int t = 0; t < 64; ++t) p += q[g * 64 + t] * wq[j * k + g * 64 + t];
                    const float t1 = (float)p * s[g];
                    r = std::fmaf(t1, ws[j * G + g], r);
                }
                const float t2 = r + biasf[j];
                if (bf16_round(t2) != (float)y[i * n + j]) ++bad;
            }
        }
        std::printf("W4A4Gemm<bf16>::forward (quantize + gemm + bias through TensorMap/Allocator): %d mismatches\n", bad);
        failures += bad != 0;
        const bool pooled = allocator.getAllSize() == (size_t)((4 * m * G + 31) / 32 * 32 + (4 * m * k / 8 + 31) / 32 * 32);
        std::printf("named pool holds exactly the two scratch buffers after two forwards: %s\n", pooled ? "yes" : "no");
        failures += !pooled;
        // ---- the same layer with the rank-32 low-rank branch (SVDQuant): y += bf16(x . down^T) . up^T ----
        {
            const int R = 32;
            std::vector<float> down(R * k), up(n * R);
            for (auto& v : down) v = bf16_round(0.2f * lcg(seed));
            for (auto& v : up) v = bf16_round(0.5f * lcg(seed));
            std::vector<hip_bfloat16> downb(R * k), upb(n * R);
            for (int i = 0; i < R * k; ++i) downb[i] = hip_bfloat16(down[i]);
            for (int i = 0; i < n * R; ++i) upb[i] = hip_bfloat16(up[i]);
            W4A4GemmWeight<hip_bfloat16> wl(n, k, R, true, 64, LyraQuantType::INT4_W4A4, &allocator);
            cache["blk.lora_down"] = downb.data();
            cache["blk.lora_up"] = upb.data();
            try {
                wl.loadWeightsFromCache("blk.", cache, hipMemcpyHostToDevice, st);
                W4A4Gemm<hip_bfloat16> layer(n, k, R, true, 64, st, nullptr, &allocator, false);
                TensorMap in({{"input", Tensor(MEMORY_GPU, TYPE_BF16, {(size_t)m, (size_t)k}, dx)}});
                TensorMap out({{"output", Tensor(MEMORY_GPU, TYPE_BF16, {(size_t)m, (size_t)n}, dy)}});
                layer.forward(&out, &in, &wl);
            } catch (const std::exception& e) {
                std::printf("exception: %s\n", e.what());
                return 3;
            }
            CK(hipStreamSynchronize(st));
            CK(hipMemcpy(y.data(), dy, m * n * 2, hipMemcpyDeviceToHost));
            int outliers = 0;
            for (int i = 0; i < m; ++i) {
                std::vector<float> v(k), s(G);
                std::vector<int> q(k);
                for (int j = 0; j < k; ++j) v[j] = x[i * k + j] / smooth[j];
                quant_row(v.data(), k, q, s);
                std::vector<double> ld(R);
                for (int r = 0; r < R; ++r) {
                    double acc = 0;
                    for (int j = 0; j < k; ++j) acc += (double)x[i * k + j] * (double)down[r * k + j];
                    ld[r] = (double)bf16_round((float)acc);
                }
                for (int j = 0; j < n; ++j) {
                    float r32 = 0.f;
                    for (int g = 0; g < G; ++g) {
                        int p = 0;
                        for (int t = 0; t < 64; ++t) p += q[g * 64 + t] * wq[j * k + g * 64 + t];
                        r32 = std::fmaf((float)p * s[g], ws[j * G + g], r32);
                    }
                    double ref = (double)r32 + (double)biasf[j], mag = std::fabs(ref);
                    for (int r = 0; r < R; ++r) { ref += ld[r] * (double)up[j * R + r]; mag += std::fabs(ld[r] * (double)up[j * R + r]); }
                    // bf16 output (8 bits) plus one bf16 ULP of each low-rank activation, whose fp32 sum order is free
                    if (std::fabs((double)(float)y[i * n + j] - ref) > 0.01 * std::fabs(ref) + 0.01 * mag * 0.5 + 1e-3) ++outliers;
                }
            }
            std::printf("W4A4Gemm<bf16>::forward with the low-rank branch: %d outliers\n", outliers);
            failures += outliers != 0;
            // ---- the same weights from the reference's raw .bin files (W4A4GemmWeight::loadWeights): the 16-bit members
            // are stored as fp32 files and converted on the way in; the forward must equal the cache-loaded layer's, bit for bit
            {
                char dir_tmpl[] = "/tmp/lq_w4a4_XXXXXX";
                const char* dir = mkdtemp(dir_tmpl);
                if (dir == nullptr) { std::printf("mkdtemp failed\n"); return 2; }
                const std::string prefix = std::string(dir) + "/blk.";
                auto dump = [&](const char* name, const void* data, size_t bytes) {
                    std::FILE* f = std::fopen((prefix + name).c_str(), "wb");
                    bool ok = f != nullptr && std::fwrite(data, 1, bytes, f) == bytes;
                    if (f) std::fclose(f);
                    return ok;
                };
                bool wrote = dump("packed_weight.bin", wpacked.data(), wpacked.size()) && dump("weight_scale.bin", ws.data(), ws.size() * 4) &&
                             dump("smooth.bin", smooth.data(), smooth.size() * 4) && dump("bias.bin", biasf.data(), biasf.size() * 4) &&
                             dump("lora_down.bin", down.data(), down.size() * 4) && dump("lora_up.bin", up.data(), up.size() * 4);
                std::vector<hip_bfloat16> y2(m * n);
                bool missing_throws = false;
                try {
                    W4A4GemmWeight<hip_bfloat16> wf(n, k, R, true, 64, LyraQuantType::INT4_W4A4, &allocator);
                    wf.loadWeights(prefix, FtCudaDataType::FP32);
                    W4A4Gemm<hip_bfloat16> layer(n, k, R, true, 64, st, nullptr, &allocator, false);
                    TensorMap in({{"input", Tensor(MEMORY_GPU, TYPE_BF16, {(size_t)m, (size_t)k}, dx)}});
                    TensorMap out({{"output", Tensor(MEMORY_GPU, TYPE_BF16, {(size_t)m, (size_t)n}, dy)}});
                    CK(hipMemset(dy, 0, m * n * 2));
                    layer.forward(&out, &in, &wf);
                    CK(hipStreamSynchronize(st));
                    CK(hipMemcpy(y2.data(), dy, m * n * 2, hipMemcpyDeviceToHost));
                    try {
                        wf.loadWeights(prefix + "absent.", FtCudaDataType::FP32);
                    } catch (const LyraException&) {
                        missing_throws = true;
                    }
                } catch (const std::exception& e) {
                    std::printf("exception: %s\n", e.what());
                    return 3;
                }
                int badf = wrote ? 0 : 1;
                for (int i = 0; i < m * n; ++i) badf += (float)y2[i] != (float)y[i];
                std::printf("W4A4GemmWeight::loadWeights from .bin files: %d mismatches, a missing file raises LyraException: %s\n",
                            badf, missing_throws ? "yes" : "no");
                failures += badf != 0 || !missing_throws;
                for (const char* nm : {"packed_weight.bin", "weight_scale.bin", "smooth.bin", "bias.bin", "lora_down.bin", "lora_up.bin"})
                    std::remove((prefix + nm).c_str());
                rmdir(dir);
            }
            allocator.freeWithName("W4A4Gemm_lora_down_res_buffer2");
        }
        bool threw = false;
        try {
            TensorMap in({{"inputs", Tensor(MEMORY_GPU, TYPE_BF16, {(size_t)m, (size_t)k}, dx)}});
            in.at("input");
        } catch (const LyraException& e) {
            threw = std::string(e.what()).find("Cannot find a tensor of name input") != std::string::npos;
        }
        std::printf("TensorMap::at on a missing key raises LyraException naming the key: %s\n", threw ? "yes" : "no");
        failures += !threw;
    }

    // ---------------- CutlassInt8GemmRunner<half>: every configuration gives the same exact result -----------------
    {
        const int m = 200, n = 160, k = 192;
        std::vector<int8_t> a(m * k), w(n * k);
        std::vector<float> ac(n), ar(m);
        for (auto& v : a) v = (int8_t)(254.0f * lcg(seed));
        for (auto& v : w) v = (int8_t)(254.0f * lcg(seed));
        for (auto& v : ac) v = 0.005f + 0.004f * lcg(seed);
        for (auto& v : ar) v = 0.05f + 0.04f * lcg(seed);
        int8_t *da, *dw, *dwp;
        float *dac, *dar;
        __half* dc;
        CK(hipMalloc(&da, m * k)); CK(hipMalloc(&dw, n * k)); CK(hipMalloc(&dwp, n * k));
        CK(hipMalloc(&dac, n * 4)); CK(hipMalloc(&dar, m * 4)); CK(hipMalloc(&dc, m * n * 2));
        CK(hipMemcpy(da, a.data(), m * k, hipMemcpyHostToDevice));
        CK(hipMemcpy(dw, w.data(), n * k, hipMemcpyHostToDevice));
        CK(hipMemcpy(dac, ac.data(), n * 4, hipMemcpyHostToDevice));
        CK(hipMemcpy(dar, ar.data(), m * 4, hipMemcpyHostToDevice));
        std::vector<float> ref(m * n);
        for (int i = 0; i < m; ++i)
            for (int j = 0; j < n; ++j) {
                int acc = 0;
                for (int p = 0; p < k; ++p) acc += (int)a[i * k + p] * (int)w[j * k + p];
                ref[i * n + j] = __half2float(__float2half((float)acc * (ac[j] * ar[i])));
            }
        int bad = 0, nconf = 0;
        try {
            repackWeight(dwp, dw, LQ_W_INT8, n, k, st);
            cutlass_kernels::CutlassInt8GemmRunner<__half> runner;
            std::vector<__half> c(m * n);
            for (auto cfg : runner.getConfigs()) {
                CK(hipMemsetAsync(dc, 0, m * n * 2, st));
                runner.gemm(da, dwp, QuantMode::useSmoothQuant(true, true), dac, dar, dc, m, n, k, cfg, nullptr, 0, st);
                CK(hipStreamSynchronize(st));
                CK(hipMemcpy(c.data(), dc, m * n * 2, hipMemcpyDeviceToHost));
                for (int i = 0; i < m * n; ++i) bad += __half2float(c[i]) != ref[i];
                ++nconf;
            }
            // profiler: fills the library's per-shape cache, the plugin then runs the cached configuration
            auto profiler = std::make_shared<gemm::SmoothQuantGemmPluginProfiler>();
            gemm::SmoothQuantGemmPlugin<__half> plugin(QuantMode::useSmoothQuant(true, true), profiler);
            plugin.configurePlugin(/*maxM=*/m, k, n);
            plugin.initialize();
            const int best = profiler->getBestConfig(m, n, k);
            std::printf("profiler picked configuration %d for m=%d n=%d k=%d\n", best, m, n, k);
            failures += best < 0 || best >= nconf;
            CK(hipMemsetAsync(dc, 0, m * n * 2, st));
            plugin.RunGemm(da, dwp, dac, dar, dc, m, n, k, nullptr, st);
            CK(hipStreamSynchronize(st));
            CK(hipMemcpy(c.data(), dc, m * n * 2, hipMemcpyDeviceToHost));
            for (int i = 0; i < m * n; ++i) bad += __half2float(c[i]) != ref[i];
        } catch (const std::exception& e) {
            std::printf("exception: %s\n", e.what());
            return 3;
        }
        std::printf("CutlassInt8GemmRunner<half>: %d configurations + profiled plugin run, %d mismatches\n", nconf, bad);
        failures += bad != 0 || nconf != lq_gemm_tactic_count(LQ_W_INT8);
    }
    return failures == 0 ? 0 : 1;
}
