/* CPU oracle, scalar C twin of oracle.py (TEST INFRASTRUCTURE, NOT PRODUCT CODE).
 *
 * Only tests/, __graft_entry__.smoke() and bench.py's cpu_baseline leg may load the library
 * built from this file.  It restates the lyraDiff reference's quantization formulas one
 * element at a time with libm's rintf/fmaf, independently of the vectorised numpy version,
 * so that the two pin each other; where a formula needs a true fused multiply-add chain
 * (W4A4 group accumulation) this file is the bit-exact authority.
 *
 * Build: gcc -O2 -ffp-contract=off -fno-fast-math -shared -fPIC oracle_c.c -lm   (see Makefile)
 * Reference citations are relative to src/lyradiff/ of the reference tree.
 */
#include <math.h>
#include <stdint.h>
#include <stdlib.h>
#include <string.h>

static float bits_f32(uint32_t u) { float f; memcpy(&f, &u, 4); return f; }
static uint32_t f32_bits(float f) { uint32_t u; memcpy(&u, &f, 4); return u; }

/* ---- small float formats -------------------------------------------------------------- */

float oc_bf16_to_f32(uint16_t b) { return bits_f32((uint32_t)b << 16); }

uint16_t oc_f32_to_bf16(float f) { /* RNE */
    uint32_t u = f32_bits(f);
    if (isnan(f)) return (uint16_t)((u >> 16) | 0x40);
    return (uint16_t)((u + 0x7FFFu + ((u >> 16) & 1u)) >> 16);
}

float oc_f16_to_f32(uint16_t h) {
    uint32_t s = (uint32_t)(h & 0x8000) << 16, e = (h >> 10) & 0x1F, m = h & 0x3FF;
    if (e == 0) return (s ? -1.0f : 1.0f) * ldexpf((float)m, -24);
    if (e == 31) return bits_f32(s | 0x7F800000u | (m << 13));
    return bits_f32(s | ((e + 112) << 23) | (m << 13));
}

uint16_t oc_f32_to_f16(float f) { /* RNE, overflow -> inf */
    uint32_t u = f32_bits(f), s = (u >> 16) & 0x8000;
    float a = fabsf(f);
    if (isnan(f)) return (uint16_t)(s | 0x7E00);
    if (a >= 65520.0f) return (uint16_t)(s | 0x7C00);
    if (a < 6.103515625e-05f) /* subnormal half: multiples of 2^-24 */
        return (uint16_t)(s | (uint32_t)rintf(ldexpf(a, 24)));
    int e; float m = frexpf(a, &e); /* a = m * 2^e, m in [0.5,1) */
    uint32_t q = (uint32_t)rintf(ldexpf(m, 11)); /* 1024..2048 */
    e -= 1;
    if (q == 2048) { q = 1024; e += 1; }
    return (uint16_t)(s | ((uint32_t)(e + 15) << 10) | (q - 1024));
}

/* ---- a1: float_to_int8_rn (kernels/quant_kernels/int8_utils.cuh:23-28) ------------------ */

int8_t oc_rne_sat_s8(float x) {
    float r = rintf(x);
    if (isnan(r)) return 0;
    if (r > 127.0f) r = 127.0f;
    if (r < -128.0f) r = -128.0f;
    return (int8_t)r;
}

/* ---- a2/a3: SmoothQuant activation quant (kernels/quant_kernels/quant_kernels.cu:51-115);
 *      dynamic scale formula amax/127 (quant_kernels.cu:207), zero-row rule of the exporter
 *      (lyradiff/convert_model_scripts/convert_sd_quant_model.py:137-150) -------------------- */

void oc_sq_input_quant(int8_t* q, const float* x, const float* pre, const float* scale,
                       int per_token, int m, int k) {
    for (int i = 0; i < m; ++i) {
        float s = per_token ? scale[i] : scale[0];
        for (int j = 0; j < k; ++j) {
            float t = pre ? x[(size_t)i * k + j] * pre[j] : x[(size_t)i * k + j];
            q[(size_t)i * k + j] = oc_rne_sat_s8(t / s);
        }
    }
}

void oc_sq_dynamic_quant(int8_t* q, float* scale, const float* x, const float* pre, int m, int k) {
    for (int i = 0; i < m; ++i) {
        float amax = 0.0f;
        for (int j = 0; j < k; ++j) {
            float t = pre ? x[(size_t)i * k + j] * pre[j] : x[(size_t)i * k + j];
            amax = fmaxf(amax, fabsf(t));
        }
        scale[i] = (amax <= 5.9604644775390625e-08f) ? 1.0f : amax / 127.0f;
    }
    oc_sq_input_quant(q, x, pre, scale, 1, m, k);
}

/* ---- a6/a7: exact int32 GEMM and the per-row x per-col epilogue
 *      (kernels/cutlass_extensions/.../epilogue_per_row_per_col_scale.h:286,301) ------------ */

void oc_gemm_i8(int32_t* acc, const int8_t* a, const int8_t* w, int m, int n, int k) {
    for (int i = 0; i < m; ++i)
        for (int j = 0; j < n; ++j) {
            int32_t s = 0;
            for (int p = 0; p < k; ++p) s += (int32_t)a[(size_t)i * k + p] * (int32_t)w[(size_t)j * k + p];
            acc[(size_t)i * n + j] = s;
        }
}

void oc_int8_epilogue(float* y, const int32_t* acc, const float* alpha_col, const float* alpha_row,
                      int per_token, const float* bias, int m, int n) {
    for (int i = 0; i < m; ++i)
        for (int j = 0; j < n; ++j) {
            float sc = alpha_col[j] * alpha_row[per_token ? i : 0];
            float v = (float)acc[(size_t)i * n + j] * sc;
            if (bias) v = v + bias[j];
            y[(size_t)i * n + j] = v;
        }
}

/* ---- a9: tanh from basic operations only (same recipe as oracle.py tanh_f32) -------------- */

float oc_tanh_f32(float u) {
    static const float c[8] = {1.0f, 0.693147180559945f, 0.240226506959101f, 0.0555041086648216f,
                               0.00961812910762848f, 0.00133335581464284f, 0.000154035303933816f,
                               1.52527338040598e-05f};
    float a = fminf(fabsf(u), 10.0f);
    float t = a * 2.8853900817779268f;
    float n = rintf(t);
    float f = t - n;
    float p = c[7];
    for (int i = 6; i >= 0; --i) { p = p * f; p = p + c[i]; }
    float e = ldexpf(p, (int)n);
    float d = e + 1.0f;
    float r = 1.0f - 2.0f / d;
    return copysignf(r, u);
}

/* ---- a10/a11: e4m3fn codec (saturate-to-finite, RNE; utils/cuda_type_utils.cuh:599-613) --- */

float oc_e4m3_decode(uint8_t c) {
    int e = (c >> 3) & 0xF, m = c & 7;
    float v;
    if ((c & 0x7F) == 0x7F) return NAN;
    v = e == 0 ? ldexpf((float)m, -9) : ldexpf((float)(8 + m), e - 10);
    return (c & 0x80) ? -v : v;
}

uint8_t oc_e4m3_encode(float x) {
    uint8_t s = (f32_bits(x) >> 24) & 0x80;
    float a = fabsf(x);
    if (isnan(x)) return (uint8_t)(s | 0x7F);
    if (a >= 448.0f) return (uint8_t)(s | 0x7E);
    if (a < 0.015625f) /* subnormals: multiples of 2^-9 (rounds up into the first normal) */
        return (uint8_t)(s | (uint8_t)rintf(ldexpf(a, 9)));
    int e; float m = frexpf(a, &e); /* m in [0.5,1) */
    int q = (int)rintf(ldexpf(m, 4)); /* 8..16 */
    e -= 1;
    if (q == 16) { q = 8; e += 1; }
    if (e > 8 || (e == 8 && q > 14)) return (uint8_t)(s | 0x7E);
    return (uint8_t)(s | ((e + 7) << 3) | (q - 8));
}

void oc_fp8_scale_cast(uint8_t* q, const float* x, float scale, int invert, size_t n) {
    float r = invert ? 1.0f / scale : scale; /* utils/memory_utils.cu:434 */
    for (size_t i = 0; i < n; ++i) q[i] = oc_e4m3_encode(x[i] * r);
}

float oc_fp8_scale(const float* x, size_t n) { /* kernels/lora/load_lora.cu:48-54 */
    float amax = 0.0f;
    for (size_t i = 0; i < n; ++i) amax = fmaxf(amax, fabsf(x[i]));
    return amax / 448.0f;
}

/* ---- a13: W4A4 group quant + nibble pack (kernels/w4a4_gemm/w4a4_gemm.cu:206-214,897-930) -- */

static int sat_s4(float v) {
    float r = rintf(v);
    if (isnan(r)) return 0;
    if (r > 7.0f) r = 7.0f;
    if (r < -8.0f) r = -8.0f;
    return (int)r;
}

void oc_w4a4_quant(uint32_t* words, float* scales, const float* x, const float* smooth,
                   int m, int k, int group, int f16_scale) {
    int ng = k / group;
    memset(words, 0, (size_t)m * (k / 8) * sizeof(uint32_t));
    for (int i = 0; i < m; ++i)
        for (int g = 0; g < ng; ++g) {
            float amax = 0.0f;
            for (int j = g * group; j < (g + 1) * group; ++j) {
                float v = smooth ? x[(size_t)i * k + j] / smooth[j] : x[(size_t)i * k + j];
                amax = fmaxf(amax, fabsf(v));
            }
            float s = amax / 7.0f;
            if (f16_scale) s = oc_f16_to_f32(oc_f32_to_f16(s));
            scales[(size_t)i * ng + g] = s;
            for (int j = g * group; j < (g + 1) * group; ++j) {
                float v = smooth ? x[(size_t)i * k + j] / smooth[j] : x[(size_t)i * k + j];
                int q = sat_s4(v / s);
                words[(size_t)i * (k / 8) + j / 8] |= ((uint32_t)q & 0xFu) << (4 * (j % 8));
            }
        }
}

static int nib(const uint32_t* row, int j) {
    int v = (int)((row[j / 8] >> (4 * (j % 8))) & 0xF);
    return v >= 8 ? v - 16 : v;
}

/* ---- a14: W4A4 GEMM, fp32 group accumulation in ascending g with the last multiply-add
 *      fused (kernels/w4a4_gemm/w4a4_gemm.cu:473-506: `dst += float(p) * sA * sB`, which the
 *      CUDA compiler contracts to fmaf(float(p)*sA, sB, dst)).  y is fp32 before the bf16 cast;
 *      p_out (nullable) receives the exact per-group int32 sums [m][n][g]. -------------------- */

void oc_w4a4_gemm(float* y, int32_t* p_out, const uint32_t* qa, const uint32_t* qb,
                  const float* sA, const float* sB, const float* bias, int m, int n, int k, int group) {
    int ng = k / group;
    int8_t* ua = (int8_t*)malloc((size_t)m * k);
    int8_t* ub = (int8_t*)malloc((size_t)n * k);
    for (int i = 0; i < m; ++i)
        for (int t = 0; t < k; ++t) ua[(size_t)i * k + t] = (int8_t)nib(qa + (size_t)i * (k / 8), t);
    for (int j = 0; j < n; ++j)
        for (int t = 0; t < k; ++t) ub[(size_t)j * k + t] = (int8_t)nib(qb + (size_t)j * (k / 8), t);
    for (int i = 0; i < m; ++i)
        for (int j = 0; j < n; ++j) {
            float r = 0.0f;
            const int8_t* pa = ua + (size_t)i * k;
            const int8_t* pb = ub + (size_t)j * k;
            for (int g = 0; g < ng; ++g) {
                int32_t p = 0;
                for (int t = g * group; t < (g + 1) * group; ++t) p += (int32_t)pa[t] * (int32_t)pb[t];
                if (p_out) p_out[((size_t)i * n + j) * ng + g] = p;
                float t1 = (float)p * sA[(size_t)i * ng + g];
                r = fmaf(t1, sB[(size_t)j * ng + g], r);
            }
            if (bias) r = r + bias[j];
            y[(size_t)i * n + j] = r;
        }
    free(ua);
    free(ub);
}
