// W4A4 group-64 INT4 activation quantisation with nibble packing, and the rows32 weight repack.
//
// Quantisation formula follows the lyraDiff reference, kernels/w4a4_gemm/w4a4_gemm.cu:206-214
// (rni + saturate to s4, low nibble first) and :897-930 (v = x / smooth, scale = group absmax / 7,
// q = v / scale).  One 64-lane wavefront owns a row; a lane owns 8 consecutive elements per pass, so
// a group of 64 is 8 adjacent lanes: three cross-lane shuffles give the group absmax, each lane
// emits one packed uint32 (coalesced 256 B per wavefront) and the first lane of a group the scale.
#include "lq_common.h"

namespace lq {

// same argument as quant_div_s8 (see lq_quant_int8.hip), bounds [-8, 7]
__device__ __forceinline__ int quant_div_s4(float t, float s, float r, bool slow) {
    float qa = t * r;
    float fr = __builtin_amdgcn_fractf(qa);
    bool risky = slow || (fabsf(fr - 0.5f) < 2e-4f && fabsf(qa) < 512.0f);
    if (__builtin_expect(risky, 0)) qa = t / s;
    return rne_sat_s4(qa);
}

template <typename Tag> __device__ __forceinline__ void load8w(const void* row_base, int col, float* o) {
    if constexpr (Elem<Tag>::bytes == 2) {
        uint4 v = *reinterpret_cast<const uint4*>(static_cast<const char*>(row_base) + (size_t)col * 2);
        unpack8<Tag>(v, o);
    } else {
        const float4* p = reinterpret_cast<const float4*>(static_cast<const char*>(row_base) + (size_t)col * 4);
        float4 a = p[0], b = p[1];
        o[0] = a.x; o[1] = a.y; o[2] = a.z; o[3] = a.w;
        o[4] = b.x; o[5] = b.y; o[6] = b.z; o[7] = b.w;
    }
}

template <typename Tag, int NP, bool F16_SCALE, bool SMOOTH_REGS>
__global__ __launch_bounds__(256) void w4a4_quant_kernel(u32* __restrict__ q_words, void* __restrict__ scales,
                                                         const void* __restrict__ x,
                                                         const float* __restrict__ smooth, int m, int k) {
    const int lane = threadIdx.x & 63;
    const int wave = blockIdx.x * 4 + (threadIdx.x >> 6);
    const int nwaves = gridDim.x * 4;
    const int ng = k >> 6;
    float sm[SMOOTH_REGS ? NP : 1][8];
    if constexpr (SMOOTH_REGS) {
#pragma unroll
        for (int p = 0; p < NP; ++p) {
            int col = (p * 64 + lane) * 8;
#pragma unroll
            for (int i = 0; i < 8; ++i) sm[p][i] = 1.0f;
            if (smooth != nullptr && col < k) load8w<F32Tag>(smooth, col, sm[p]);
        }
    }
    for (int row = wave; row < m; row += nwaves) {
        const char* rb = static_cast<const char*>(x) + (size_t)row * k * Elem<Tag>::bytes;
        float v[NP][8];
#pragma unroll
        for (int p = 0; p < NP; ++p) {
            int col = (p * 64 + lane) * 8;
            if (col < k) load8w<Tag>(rb, col, v[p]);
            else {
#pragma unroll
                for (int i = 0; i < 8; ++i) v[p][i] = 0.0f;
            }
        }
#pragma unroll
        for (int p = 0; p < NP; ++p) {
            int col = (p * 64 + lane) * 8;
            if (smooth != nullptr) {
                if constexpr (SMOOTH_REGS) {
#pragma unroll
                    for (int i = 0; i < 8; ++i) v[p][i] = v[p][i] / sm[p][i];
                } else if (col < k) {
                    float sv[8];
                    load8w<F32Tag>(smooth, col, sv);
#pragma unroll
                    for (int i = 0; i < 8; ++i) v[p][i] = v[p][i] / sv[i];
                }
            }
            float amax = 0.0f;
#pragma unroll
            for (int i = 0; i < 8; ++i) amax = fmaxf(amax, fabsf(v[p][i]));
            amax = group_max<8>(amax);
            float s = amax / 7.0f;
            if constexpr (F16_SCALE) s = round_through<F16Tag>(s);
            const float r = 1.0f / s;
            const bool slow = !(fabsf(s) >= 1e-30f && fabsf(r) < 1e30f && fabsf(r) >= 1e-30f);
            u32 word = 0;
#pragma unroll
            for (int i = 0; i < 8; ++i) word |= ((u32)quant_div_s4(v[p][i], s, r, slow) & 0xFu) << (4 * i);
            if (col < k) {
                q_words[(size_t)row * (k >> 3) + (col >> 3)] = word;
                if ((lane & 7) == 0) {
                    size_t si = (size_t)row * ng + (col >> 6);
                    if constexpr (F16_SCALE) static_cast<unsigned short*>(scales)[si] = (unsigned short)f32_to_f16_bits(s);
                    else static_cast<float*>(scales)[si] = s;
                }
            }
        }
    }
}

// ---- rows32 repack: dst chunk ((nb*KC + kc)*32 + r) <- src chunk (row nb*32 + r, 16-byte column kc) ----
template <bool INVERSE>
__global__ __launch_bounds__(256) void rows32_kernel(uint4* __restrict__ dst, const uint4* __restrict__ src, size_t n,
                                                     size_t kc_count) {
    const size_t total = n * kc_count;
    for (size_t t = (size_t)blockIdx.x * blockDim.x + threadIdx.x; t < total; t += (size_t)gridDim.x * blockDim.x) {
        size_t r = t & 31, rest = t >> 5;
        size_t kc = rest % kc_count, nb = rest / kc_count;
        size_t plain = (nb * 32 + r) * kc_count + kc;
        if constexpr (INVERSE) dst[plain] = src[t];
        else dst[t] = src[plain];
    }
}

}  // namespace lq

using namespace lq;

extern "C" int lq_w4a4_quantize(uint32_t* q_words, void* scales, lq_dtype_t scale_dtype, const void* x,
                                lq_dtype_t x_dtype, const float* smooth, int m, int k, int group, lq_stream_t stream) {
    LQ_REQUIRE(q_words && scales && x, LQ_ERR_ARG, "lq_w4a4_quantize: null pointer");
    LQ_REQUIRE(group == 64, LQ_ERR_SHAPE, "lq_w4a4_quantize: group=%d, only 64 is supported", group);
    LQ_REQUIRE(m >= 0 && k > 0 && k % 64 == 0 && k <= 16384, LQ_ERR_SHAPE,
               "lq_w4a4_quantize: k=%d must be a positive multiple of 64 and <= 16384", k);
    LQ_REQUIRE(scale_dtype == LQ_F32 || scale_dtype == LQ_F16, LQ_ERR_UNSUPPORTED,
               "lq_w4a4_quantize: scale dtype must be F32 or F16");
    LQ_REQUIRE(reinterpret_cast<uintptr_t>(x) % 16 == 0 && (smooth == nullptr || reinterpret_cast<uintptr_t>(smooth) % 16 == 0),
               LQ_ERR_ARG, "lq_w4a4_quantize: x and smooth must be 16-byte aligned");
    if (m == 0) return LQ_OK;
    const int np = (k + 511) / 512;
    int blocks = (m + 3) / 4;
    if (blocks > 256 * 8) blocks = 256 * 8;
    dim3 grid(blocks), block(256);
    hipStream_t st = as_stream(stream);
    const bool f16s = scale_dtype == LQ_F16;
#define LQ_W4_LAUNCH(TAG, NPV, SR)                                                                                        \
    do {                                                                                                                  \
        if (f16s) hipLaunchKernelGGL((w4a4_quant_kernel<TAG, NPV, true, SR>), grid, block, 0, st, q_words, scales, x, smooth, m, k); \
        else hipLaunchKernelGGL((w4a4_quant_kernel<TAG, NPV, false, SR>), grid, block, 0, st, q_words, scales, x, smooth, m, k);      \
    } while (0)
#define LQ_W4_NP(TAG)                          \
    do {                                       \
        if (np <= 1) LQ_W4_LAUNCH(TAG, 1, true);       \
        else if (np <= 2) LQ_W4_LAUNCH(TAG, 2, true);  \
        else if (np <= 4) LQ_W4_LAUNCH(TAG, 4, true);  \
        else if (np <= 6) LQ_W4_LAUNCH(TAG, 6, true);  \
        else if (np <= 8) LQ_W4_LAUNCH(TAG, 8, true);  \
        else if (np <= 16) LQ_W4_LAUNCH(TAG, 16, false); \
        else LQ_W4_LAUNCH(TAG, 32, false);             \
    } while (0)
    switch (x_dtype) {
        case LQ_F16: LQ_W4_NP(F16Tag); break;
        case LQ_BF16: LQ_W4_NP(BF16Tag); break;
        case LQ_F32: LQ_W4_NP(F32Tag); break;
        default: set_error("lq_w4a4_quantize: unsupported x dtype %d", (int)x_dtype); return LQ_ERR_UNSUPPORTED;
    }
#undef LQ_W4_NP
#undef LQ_W4_LAUNCH
    return check_launch("w4a4_quantize");
}

extern "C" size_t lq_weight_row_bytes(lq_weight_kind_t kind, size_t k) { return kind == LQ_W_INT4 ? k / 2 : k; }

static int rows32_launch(uint8_t* dst, const uint8_t* src, size_t n, size_t row_bytes, lq_stream_t stream, bool inverse) {
    LQ_REQUIRE(dst && src, LQ_ERR_ARG, "lq_repack_rows32: null pointer");
    LQ_REQUIRE(dst != src, LQ_ERR_ARG, "lq_repack_rows32: in-place repack is not supported");
    LQ_REQUIRE(n % 32 == 0 && row_bytes % 16 == 0, LQ_ERR_SHAPE,
               "lq_repack_rows32: n=%zu must be a multiple of 32 and row_bytes=%zu a multiple of 16", n, row_bytes);
    LQ_REQUIRE(reinterpret_cast<uintptr_t>(dst) % 16 == 0 && reinterpret_cast<uintptr_t>(src) % 16 == 0, LQ_ERR_ARG,
               "lq_repack_rows32: buffers must be 16-byte aligned");
    if (n == 0 || row_bytes == 0) return LQ_OK;
    size_t total = n * (row_bytes / 16);
    size_t blocks = (total + 255) / 256;
    if (blocks > 65535) blocks = 65535;
    if (inverse)
        hipLaunchKernelGGL((rows32_kernel<true>), dim3((unsigned)blocks), dim3(256), 0, as_stream(stream),
                           reinterpret_cast<uint4*>(dst), reinterpret_cast<const uint4*>(src), n, row_bytes / 16);
    else
        hipLaunchKernelGGL((rows32_kernel<false>), dim3((unsigned)blocks), dim3(256), 0, as_stream(stream),
                           reinterpret_cast<uint4*>(dst), reinterpret_cast<const uint4*>(src), n, row_bytes / 16);
    return check_launch("rows32");
}

extern "C" int lq_repack_rows32(uint8_t* dst, const uint8_t* src, size_t n, size_t row_bytes, lq_stream_t stream) {
    return rows32_launch(dst, src, n, row_bytes, stream, false);
}
extern "C" int lq_unpack_rows32(uint8_t* dst, const uint8_t* src, size_t n, size_t row_bytes, lq_stream_t stream) {
    return rows32_launch(dst, src, n, row_bytes, stream, true);
}
