// Reference-style C++ call sites (names of lyraDiff's quant-linear API) running on liblyraquant.so.
// Exit code 0 when the INT8 path is bit-exact against a host triple loop and the FP8 path is within
// tolerance; prints one line per check.  Built by lyradiff_amd/build.py, run by tests/test_gpu_compat.py.
#include <cmath>
#include <cstdio>
#include <cstdlib>
#include <vector>

#include "lyradiff_compat.h"

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

int main() {
    const int m = 96, n = 64, k = 128;
    unsigned seed = 7;
    hipStream_t st;
    CK(hipStreamCreate(&st));
    // ---------------- INT8: dynamic per-token quant -> repack -> runGemmInt8 (fp16 out) ----------------
    std::vector<__half> hx(m * k);
    std::vector<float> fx(m * k), pre(k), wscale(n);
    std::vector<int8_t> hw(n * k);
    for (auto& v : fx) v = 4.0f * lcg(seed);
    for (int i = 0; i < m * k; ++i) { hx[i] = __float2half(fx[i]); fx[i] = __half2float(hx[i]); }
    for (auto& v : pre) v = 1.0f + lcg(seed);
    for (auto& v : wscale) v = 0.005f + 0.004f * lcg(seed);
    for (auto& v : hw) v = (int8_t)(254.0f * lcg(seed));
    __half *dx, *dy;
    int8_t *dq, *dw, *dwp;
    float *dpre, *dscale, *dws;
    CK(hipMalloc(&dx, m * k * 2)); CK(hipMalloc(&dy, m * n * 2)); CK(hipMalloc(&dq, m * k)); CK(hipMalloc(&dw, n * k));
    CK(hipMalloc(&dwp, n * k)); CK(hipMalloc(&dpre, k * 4)); CK(hipMalloc(&dscale, m * 4)); CK(hipMalloc(&dws, n * 4));
    CK(hipMemcpy(dx, hx.data(), m * k * 2, hipMemcpyHostToDevice));
    CK(hipMemcpy(dw, hw.data(), n * k, hipMemcpyHostToDevice));
    CK(hipMemcpy(dpre, pre.data(), k * 4, hipMemcpyHostToDevice));
    CK(hipMemcpy(dws, wscale.data(), n * 4, hipMemcpyHostToDevice));
    try {
        invokeSqDynamicPerTokenQuant<__half>(dq, dscale, dx, dpre, 1, m, k, st);
        repackWeight(dwp, dw, LQ_W_INT8, n, k, st);
        cublasMMWrapper<__half> wrapper(st, /*per_token_int8=*/true);
        wrapper.profileGemmInt8(16384, n, k);
        wrapper.runGemmInt8(dq, dwp, dws, dscale, dy, m, n, k, nullptr, st);
    } catch (const std::exception& e) {
        std::printf("exception: %s\n", e.what());
        return 3;
    }
    CK(hipStreamSynchronize(st));
    std::vector<__half> hy(m * n);
    std::vector<int8_t> hq(m * k);
    std::vector<float> hs(m);
    CK(hipMemcpy(hy.data(), dy, m * n * 2, hipMemcpyDeviceToHost));
    CK(hipMemcpy(hq.data(), dq, m * k, hipMemcpyDeviceToHost));
    CK(hipMemcpy(hs.data(), dscale, m * 4, hipMemcpyDeviceToHost));
    int bad = 0;
    for (int i = 0; i < m; ++i) {
        float amax = 0.f;
        for (int j = 0; j < k; ++j) amax = std::fmax(amax, std::fabs(fx[i * k + j] * pre[j]));
        float s = amax / 127.0f;
        if (s != hs[i]) ++bad;
        for (int j = 0; j < k; ++j) {
            float r = std::rint((fx[i * k + j] * pre[j]) / s);
            r = std::fmin(std::fmax(r, -128.f), 127.f);
            if ((int8_t)r != hq[i * k + j]) ++bad;
        }
        for (int j = 0; j < n; ++j) {
            int acc = 0;
            for (int p = 0; p < k; ++p) acc += (int)hq[i * k + p] * (int)hw[j * k + p];
            float y = (float)acc * (wscale[j] * s);
            if (__half2float(__float2half(y)) != __half2float(hy[i * n + j])) ++bad;
        }
    }
    std::printf("int8 path (invokeSqDynamicPerTokenQuant + runGemmInt8): %d mismatches\n", bad);
    // ---------------- INT8 loader route: invokeGetINT8WeightScale, then the unfused invokeSqOutputDequant -------------
    std::vector<__half> hwf(n * k);
    std::vector<float> fwf(n * k);
    for (int i = 0; i < n * k; ++i) { hwf[i] = __float2half(0.2f * lcg(seed)); fwf[i] = __half2float(hwf[i]); }
    for (int j = 0; j < k; ++j) { hwf[5 * k + j] = __float2half(0.0f); fwf[5 * k + j] = 0.0f; }  // a zero row: scale 0, codes 0
    __half *dwf, *ddq;
    int8_t* dwq;
    float* dwqs;
    int32_t* dacc;
    CK(hipMalloc(&dwf, n * k * 2)); CK(hipMalloc(&dwq, n * k)); CK(hipMalloc(&dwqs, n * 4));
    CK(hipMalloc(&dacc, m * n * 4)); CK(hipMalloc(&ddq, m * n * 2));
    CK(hipMemcpy(dwf, hwf.data(), n * k * 2, hipMemcpyHostToDevice));
    std::vector<int32_t> hacc(m * n);
    for (int i = 0; i < m * n; ++i) hacc[i] = (int32_t)(6.0e6f * lcg(seed));
    CK(hipMemcpy(dacc, hacc.data(), m * n * 4, hipMemcpyHostToDevice));
    try {
        invokeGetINT8WeightScale<__half>(dwqs, dwq, dwf, dpre, n, k, st);
        invokeSqOutputDequant<__half>(ddq, dacc, dscale, dws, QuantMode::useSmoothQuant(true, true), 1, m, n, st);
    } catch (const std::exception& e) {
        std::printf("exception: %s\n", e.what());
        return 3;
    }
    CK(hipStreamSynchronize(st));
    std::vector<int8_t> hwq(n * k);
    std::vector<float> hwqs(n);
    std::vector<__half> hdq(m * n);
    CK(hipMemcpy(hwq.data(), dwq, n * k, hipMemcpyDeviceToHost));
    CK(hipMemcpy(hwqs.data(), dwqs, n * 4, hipMemcpyDeviceToHost));
    CK(hipMemcpy(hdq.data(), ddq, m * n * 2, hipMemcpyDeviceToHost));
    int badw = 0;
    for (int i = 0; i < n; ++i) {
        float amax = 0.f;
        for (int j = 0; j < k; ++j) amax = std::fmax(amax, std::fabs(fwf[i * k + j] / pre[j]));
        float s = amax / 127.0f;
        if (s != hwqs[i]) ++badw;
        for (int j = 0; j < k; ++j) {
            float r = std::rint((fwf[i * k + j] / pre[j]) / s);
            int want = std::isnan(r) ? 0 : (int)std::fmin(std::fmax(r, -128.f), 127.f);
            if (want != (int)hwq[i * k + j]) ++badw;
        }
    }
    for (int i = 0; i < m; ++i)
        for (int j = 0; j < n; ++j) {
            float y = ((float)hacc[i * n + j] * hs[i]) * wscale[j];
            if (__half2float(__float2half(y)) != __half2float(hdq[i * n + j])) ++badw;
        }
    std::printf("int8 loader route (invokeGetINT8WeightScale + invokeSqOutputDequant): %d mismatches\n", badw);
    // ---------------- FP8: weight scale + cast + GemmWithResidualAndBias (bf16 out) ----------------------
    std::vector<hip_bfloat16> bx(m * k), bw(n * k);
    std::vector<float> fbx(m * k), fbw(n * k);
    for (int i = 0; i < m * k; ++i) { bx[i] = hip_bfloat16(2.0f * lcg(seed)); fbx[i] = (float)bx[i]; }
    for (int i = 0; i < n * k; ++i) { bw[i] = hip_bfloat16(0.1f * lcg(seed)); fbw[i] = (float)bw[i]; }
    hip_bfloat16 *dbx, *dbw, *dby;
    fp8_e4m3_t *qx, *qw, *qwp;
    float *sx, *sw;
    CK(hipMalloc(&dbx, m * k * 2)); CK(hipMalloc(&dbw, n * k * 2)); CK(hipMalloc(&dby, m * n * 2));
    CK(hipMalloc(&qx, m * k)); CK(hipMalloc(&qw, n * k)); CK(hipMalloc(&qwp, n * k));
    CK(hipMalloc(&sx, 4)); CK(hipMalloc(&sw, 4));
    CK(hipMemcpy(dbx, bx.data(), m * k * 2, hipMemcpyHostToDevice));
    CK(hipMemcpy(dbw, bw.data(), n * k * 2, hipMemcpyHostToDevice));
    CK(hipMemsetAsync(sx, 0, 4, st)); CK(hipMemsetAsync(sw, 0, 4, st));
    try {
        invokeGetFP8WeightScale(sw, dbw, (size_t)n * k, st);
        invokeCudaD2DScaleCpyConvert(qw, dbw, sw, true, (size_t)n * k, st);
        invokeGetFP8WeightScale(sx, dbx, (size_t)m * k, st);
        invokeCudaD2DScaleCpyConvert(qx, dbx, sx, true, (size_t)m * k, st);
        repackWeight(qwp, qw, LQ_W_FP8, n, k, st);
        cublasMMWrapper<hip_bfloat16> wrapper(st);
        wrapper.GemmWithResidualAndBias(CUBLAS_OP_T, CUBLAS_OP_N, n, m, k, qwp, k, sw, qx, k, sx, dby, n);
    } catch (const std::exception& e) {
        std::printf("exception: %s\n", e.what());
        return 3;
    }
    CK(hipStreamSynchronize(st));
    std::vector<hip_bfloat16> by(m * n);
    CK(hipMemcpy(by.data(), dby, m * n * 2, hipMemcpyDeviceToHost));
    int bad8 = 0;
    for (int i = 0; i < m; ++i)
        for (int j = 0; j < n; ++j) {
            double ref = 0;
            for (int p = 0; p < k; ++p) ref += (double)fbx[i * k + p] * (double)fbw[j * k + p];
            double got = (double)(float)by[i * n + j];
            if (std::fabs(got - ref) > 0.1 * std::fabs(ref) + 0.05) ++bad8;  // e4m3 operands (3 mantissa bits): noise ~0.01 rms here
        }
    std::printf("fp8 path (GetFP8WeightScale + ScaleCpyConvert + GemmWithResidualAndBias): %d outliers\n", bad8);
    // ---------------- weight-only W4A16 with group-wise scales and zero points: CutlassFpAIntBGemmRunner ----------------
    // (fpA_intB_gemm.h:58-85; every dequantised weight is T(T(q * s) + z) for fp16, so a host loop reproduces it)
    int badwo = 0;
    {
        const int wk = 256, wn = 64, wm = 48, grp = 128;
        std::vector<int8_t> codes(wk * wn / 2);
        std::vector<int> qv(wk * wn);
        for (int i = 0; i < wk * wn; ++i) qv[i] = (int)(15.9f * (lcg(seed) + 0.5f)) - 8;
        for (int r = 0; r < wk; ++r)
            for (int c = 0; c < wn; c += 2)
                codes[r * (wn / 2) + c / 2] = (int8_t)((qv[r * wn + c] & 0xF) | ((qv[r * wn + c + 1] & 0xF) << 4));
        std::vector<__half> hs(wk / grp * wn), hz(wk / grp * wn), ha(wm * wk), hb(wn);
        for (auto& v : hs) v = __float2half(0.01f + 0.02f * (lcg(seed) + 0.5f));
        for (auto& v : hz) v = __float2half(0.1f * lcg(seed));
        for (auto& v : ha) v = __float2half(2.0f * lcg(seed));
        for (auto& v : hb) v = __float2half(lcg(seed));
        int8_t* dcodes; uint8_t* dprep; __half *ds, *dz, *da, *db, *dc;
        CK(hipMalloc(&dcodes, codes.size())); CK(hipMalloc(&dprep, codes.size())); CK(hipMalloc(&ds, hs.size() * 2));
        CK(hipMalloc(&dz, hz.size() * 2)); CK(hipMalloc(&da, ha.size() * 2)); CK(hipMalloc(&db, hb.size() * 2)); CK(hipMalloc(&dc, wm * wn * 2));
        CK(hipMemcpy(dcodes, codes.data(), codes.size(), hipMemcpyHostToDevice));
        CK(hipMemcpy(ds, hs.data(), hs.size() * 2, hipMemcpyHostToDevice)); CK(hipMemcpy(dz, hz.data(), hz.size() * 2, hipMemcpyHostToDevice));
        CK(hipMemcpy(da, ha.data(), ha.size() * 2, hipMemcpyHostToDevice)); CK(hipMemcpy(db, hb.data(), hb.size() * 2, hipMemcpyHostToDevice));
        try {
            detail::check(lq_repack_weight_only(dprep, dcodes, LQ_W_INT4, wk, wn, st), "lq_repack_weight_only");
            cutlass_kernels::CutlassFpAIntBGemmRunner<__half, cutlass::uint4b_t, cutlass::WeightOnlyQuantOp::FINEGRAINED_SCALE_AND_ZEROS> runner;
            runner.gemm(da, dprep, ds, dz, db, dc, wm, wn, wk, grp, runner.getConfigs()[0], nullptr, runner.getWorkspaceSize(wm, wn, wk), st);
        } catch (const std::exception& e) {
            std::printf("exception: %s\n", e.what());
            return 4;
        }
        CK(hipStreamSynchronize(st));
        std::vector<__half> hc(wm * wn);
        CK(hipMemcpy(hc.data(), dc, wm * wn * 2, hipMemcpyDeviceToHost));
        for (int i = 0; i < wm; ++i)
            for (int j = 0; j < wn; ++j) {
                double ref = (double)__half2float(hb[j]), mag = 0;
                for (int p = 0; p < wk; ++p) {
                    const float qs = __half2float(__float2half((float)qv[p * wn + j] * __half2float(hs[(p / grp) * wn + j])));
                    const float w = __half2float(__float2half(qs + __half2float(hz[(p / grp) * wn + j])));
                    ref += (double)__half2float(ha[i * wk + p]) * (double)w;
                    mag += std::fabs((double)__half2float(ha[i * wk + p]) * (double)w);
                }
                if (std::fabs((double)__half2float(hc[i * wn + j]) - ref) > 2e-3 * std::fabs(ref) + 1e-5 * mag + 1e-4) ++badwo;
            }
    }
    std::printf("weight-only path (lq_repack_weight_only + CutlassFpAIntBGemmRunner, group scales and zeros): %d mismatches\n", badwo);
    // ---------------- W4A4: invokeFusedQuantizeAndLoraDownSimple = one pass over A for words, scales and the rank-32 projection ----
    int bad4 = 0;
    {
        const int qm = 70, qk = 384, rank = 32;
        std::vector<hip_bfloat16> ha(qm * qk), hd(rank * qk);
        std::vector<float> hsm(qk);
        for (auto& v : ha) v = hip_bfloat16(6.0f * lcg(seed));
        for (auto& v : hd) v = hip_bfloat16(0.2f * lcg(seed));
        for (auto& v : hsm) v = 0.75f + lcg(seed);
        hip_bfloat16 *da, *dd; float *dsm, *dC, *dC2, *dsc, *dsc2; uint32_t *dwords, *dwords2;
        CK(hipMalloc(&da, ha.size() * 2)); CK(hipMalloc(&dd, hd.size() * 2)); CK(hipMalloc(&dsm, qk * 4));
        CK(hipMalloc(&dC, qm * rank * 4)); CK(hipMalloc(&dC2, qm * rank * 4)); CK(hipMalloc(&dsc, qm * (qk / 64) * 4)); CK(hipMalloc(&dsc2, qm * (qk / 64) * 4));
        CK(hipMalloc(&dwords, qm * (qk / 8) * 4)); CK(hipMalloc(&dwords2, qm * (qk / 8) * 4));
        CK(hipMemcpy(da, ha.data(), ha.size() * 2, hipMemcpyHostToDevice)); CK(hipMemcpy(dd, hd.data(), hd.size() * 2, hipMemcpyHostToDevice));
        CK(hipMemcpy(dsm, hsm.data(), qk * 4, hipMemcpyHostToDevice));
        try {
            invokeFusedQuantizeAndLoraDownSimple(dC, dwords, dsc, da, dd, dsm, qm, rank, qk, qk / 64, st);
            detail::check(lq_w4a4_quantize(dwords2, dsc2, LQ_F32, da, LQ_BF16, dsm, qm, qk, 64, st), "lq_w4a4_quantize");
            detail::check(lq_lora_down(dC2, LQ_F32, da, dd, LQ_BF16, qm, qk, rank, st), "lq_lora_down");
        } catch (const std::exception& e) {
            std::printf("exception: %s\n", e.what());
            return 5;
        }
        CK(hipStreamSynchronize(st));
        std::vector<uint32_t> w1(qm * (qk / 8)), w2(w1.size());
        std::vector<float> s1(qm * (qk / 64)), s2(s1.size()), c1(qm * rank);
        CK(hipMemcpy(w1.data(), dwords, w1.size() * 4, hipMemcpyDeviceToHost)); CK(hipMemcpy(w2.data(), dwords2, w2.size() * 4, hipMemcpyDeviceToHost));
        CK(hipMemcpy(s1.data(), dsc, s1.size() * 4, hipMemcpyDeviceToHost)); CK(hipMemcpy(s2.data(), dsc2, s2.size() * 4, hipMemcpyDeviceToHost));
        CK(hipMemcpy(c1.data(), dC, c1.size() * 4, hipMemcpyDeviceToHost));
        for (size_t i = 0; i < w1.size(); ++i) bad4 += w1[i] != w2[i];
        for (size_t i = 0; i < s1.size(); ++i) bad4 += s1[i] != s2[i];
        for (int i = 0; i < qm; ++i)
            for (int r = 0; r < rank; ++r) {
                double ref = 0, mag = 0;
                for (int p = 0; p < qk; ++p) {
                    const double t = (double)(float)ha[i * qk + p] * (double)(float)hd[r * qk + p];
                    ref += t;
                    mag += std::fabs(t);
                }
                if (std::fabs((double)c1[i * rank + r] - ref) > 1e-6 * mag + 1e-30) ++bad4;
            }
    }
    std::printf("w4a4 quantise + low-rank down in one pass (invokeFusedQuantizeAndLoraDownSimple): %d mismatches\n", bad4);
    // error convention: exception with the reference's prefix
    bool threw = false;
    try {
        cublasMMWrapper<__half> wrapper(st);
        wrapper.runGemmInt8(dq, dwp, dws, dscale, dy, m, 33, k, nullptr, st);
    } catch (const std::runtime_error& e) {
        threw = std::string(e.what()).find("[lyradiff Error]") == 0;
    }
    std::printf("bad shape raises std::runtime_error with the reference's prefix: %s\n", threw ? "yes" : "no");
    return (bad == 0 && badw == 0 && bad8 == 0 && badwo == 0 && bad4 == 0 && threw) ? 0 : 1;
}
