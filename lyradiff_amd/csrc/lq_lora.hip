// Low-rank ("SVDQuant") side branch of the W4A4 linear: the down projection
//     out[m, r] = sum_k x[m, k] * down[r, k]        (16-bit float operands, fp32 accumulation)
// that the reference computes inside its quantisation kernel with float atomics
// (kernels/w4a4_gemm/w4a4_gemm.cu:769-953 of lyraDiff, `reduce_add` into a zeroed fp32 buffer, followed by a
// separate float -> T conversion, layers/w4a4_gemm_block/W4A4Gemm.cc:138-150).  Here it is a skinny GEMM of its
// own: a workgroup owns 32 rows and all of K, its eight wavefronts take interleaved 64-wide slices of K, the
// partial 32 x rank blocks meet in LDS and are added in wavefront order -- no atomics, so the result does not
// depend on scheduling -- and the output is written once, already in the requested type.  It reads x from HBM
// only if the quantisation kernel that ran just before did not leave it in the caches.
#include "lq_common.h"

namespace lq {

typedef __bf16 v8bf __attribute__((ext_vector_type(8)));
typedef _Float16 v8h __attribute__((ext_vector_type(8)));
typedef float v16f_t __attribute__((ext_vector_type(16)));

template <bool F16> __device__ __forceinline__ v16f_t mfma16(const v4i& a, const v4i& b, const v16f_t& c) {
    if constexpr (F16) return __builtin_amdgcn_mfma_f32_32x32x16_f16(__builtin_bit_cast(v8h, a), __builtin_bit_cast(v8h, b), c, 0, 0, 0);
    else return __builtin_amdgcn_mfma_f32_32x32x16_bf16(__builtin_bit_cast(v8bf, a), __builtin_bit_cast(v8bf, b), c, 0, 0, 0);
}

// NR: rank / 32.  OUT: 0 fp32, 1 fp16, 2 bf16.
template <bool F16, int NR, int OUT>
__global__ __launch_bounds__(512) void lora_down_kernel(void* __restrict__ out, const unsigned short* __restrict__ x,
                                                        const unsigned short* __restrict__ down, int m, int k) {
    constexpr int W = 8;                    // wavefronts per workgroup, each takes every eighth 64-wide slice of K
    __shared__ float part[W - 1][NR][16][64];  // partial blocks of wavefronts 1..7
    const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
    const int row0 = blockIdx.x * 32;
    const int lr = lane & 31, lh = lane >> 5;
    const unsigned short* xrow = x + (size_t)min(row0 + lr, m - 1) * k + lh * 8;
    const unsigned short* drow = down + (size_t)lr * k + lh * 8;
    v16f_t acc[NR];
#pragma unroll
    for (int r = 0; r < NR; ++r)
#pragma unroll
        for (int v = 0; v < 16; ++v) acc[r][v] = 0.0f;
    // a wavefront's slice: 64 consecutive k (four MFMA steps, one 128-byte line per row), every eighth slice.
    // The operands of the next slice are requested before the matrix instructions of the current one, so the
    // memory latency of a slice is hidden behind the previous slice's arithmetic and the other wavefronts.
    v4i xf[2][4], df[2][NR][4];
    auto load_slice = [&](int k0, int buf) {
#pragma unroll
        for (int s = 0; s < 4; ++s) {
            xf[buf][s] = *reinterpret_cast<const v4i*>(xrow + k0 + s * 16);
#pragma unroll
            for (int r = 0; r < NR; ++r) df[buf][r][s] = *reinterpret_cast<const v4i*>(drow + (size_t)r * 32 * k + k0 + s * 16);
        }
    };
    auto compute_slice = [&](int buf) {
#pragma unroll
        for (int s = 0; s < 4; ++s)
#pragma unroll
            for (int r = 0; r < NR; ++r) acc[r] = mfma16<F16>(df[buf][r][s], xf[buf][s], acc[r]);
    };
    int k0 = wave * 64;
    if (k0 < k) load_slice(k0, 0);
    for (; k0 < k; k0 += 2 * 64 * W) {
        if (k0 + 64 * W < k) load_slice(k0 + 64 * W, 1);
        compute_slice(0);
        if (k0 + 64 * W >= k) break;
        if (k0 + 2 * 64 * W < k) load_slice(k0 + 2 * 64 * W, 0);
        compute_slice(1);
    }
    if (wave != 0) {
#pragma unroll
        for (int r = 0; r < NR; ++r)
#pragma unroll
            for (int v = 0; v < 16; ++v) part[wave - 1][r][v][lane] = acc[r][v];
    }
    __syncthreads();
    if (wave != 0) return;
    const int row = row0 + lr;
#pragma unroll
    for (int r = 0; r < NR; ++r) {
#pragma unroll
        for (int v = 0; v < 16; ++v)
#pragma unroll
            for (int w = 0; w < W - 1; ++w) acc[r][v] += part[w][r][v][lane];  // wavefront order: 0, 1, ..., 7
        if (row < m) {
            // result layout of the 32x32 MFMA: this lane holds row (= x row) lr and rank indices 8*(v/4) + 4*lh + v%4
#pragma unroll
            for (int q4 = 0; q4 < 4; ++q4) {
                const size_t idx = (size_t)row * (NR * 32) + r * 32 + q4 * 8 + lh * 4;
                const float y0 = acc[r][q4 * 4], y1 = acc[r][q4 * 4 + 1], y2 = acc[r][q4 * 4 + 2], y3 = acc[r][q4 * 4 + 3];
                if constexpr (OUT == 0) {
                    *reinterpret_cast<float4*>(static_cast<float*>(out) + idx) = make_float4(y0, y1, y2, y3);
                } else {
                    uint2 o;
                    o.x = OUT == 1 ? pack2_f16(y0, y1) : pack2_bf16(y0, y1);
                    o.y = OUT == 1 ? pack2_f16(y2, y3) : pack2_bf16(y2, y3);
                    *reinterpret_cast<uint2*>(static_cast<unsigned short*>(out) + idx) = o;
                }
            }
        }
    }
}

template <bool F16, int NR> static int launch_lora_down(void* out, lq_dtype_t out_dtype, const void* x, const void* down, int m, int k, hipStream_t st) {
    dim3 grid((unsigned)((m + 31) / 32)), block(512);
    const unsigned short* xs = static_cast<const unsigned short*>(x);
    const unsigned short* ds = static_cast<const unsigned short*>(down);
    switch (out_dtype) {
        case LQ_F32: hipLaunchKernelGGL((lora_down_kernel<F16, NR, 0>), grid, block, 0, st, out, xs, ds, m, k); break;
        case LQ_F16: hipLaunchKernelGGL((lora_down_kernel<F16, NR, 1>), grid, block, 0, st, out, xs, ds, m, k); break;
        case LQ_BF16: hipLaunchKernelGGL((lora_down_kernel<F16, NR, 2>), grid, block, 0, st, out, xs, ds, m, k); break;
        default: set_error("lq_lora_down: unsupported output dtype %d", (int)out_dtype); return LQ_ERR_UNSUPPORTED;
    }
    return check_launch("lq_lora_down");
}

// dst[i] = T(src[i]) for fp32 sources: the float -> T step between the reference's two W4A4 kernels
// (invokeCudaD2DcpyConvert, utils/memory_utils.cu:398-402).
template <int OUT> __global__ void cast_f32_kernel(void* __restrict__ dst, const float* __restrict__ src, size_t n) {
    for (size_t i = (size_t)blockIdx.x * blockDim.x + threadIdx.x; i < n; i += (size_t)gridDim.x * blockDim.x) {
        const float v = src[i];
        if constexpr (OUT == 0) static_cast<float*>(dst)[i] = v;
        else static_cast<unsigned short*>(dst)[i] = (unsigned short)(OUT == 1 ? (pack2_f16(v, 0.0f) & 0xFFFFu) : f32_to_bf16_bits(v));
    }
}

// Merge of a full-rank LoRA delta into a 16/32-bit weight, the first step of re-quantising an FP8 weight
// (loadLora, kernels/lora/load_lora.cu:6-14; FP8LoraWeight::load_lora, interface/IFLoraWeight.h:100-112):
//   dst[i] = T( dst[i] + T( src[i] * T(alpha) ) )
template <typename Tag> __global__ void load_lora_kernel(void* __restrict__ dst, const void* __restrict__ src, size_t n, float alpha) {
    const float a = round_through<Tag>(alpha);
    for (size_t i = (size_t)blockIdx.x * blockDim.x + threadIdx.x; i < n; i += (size_t)gridDim.x * blockDim.x) {
        if constexpr (Elem<Tag>::bytes == 2) {
            unsigned short* d = static_cast<unsigned short*>(dst);
            const float w = Elem<Tag>::load(d[i]), l = Elem<Tag>::load(static_cast<const unsigned short*>(src)[i]);
            d[i] = (unsigned short)Elem<Tag>::store(round_through<Tag>(l * a) + w);
        } else {
            float* d = static_cast<float*>(dst);
            d[i] = d[i] + static_cast<const float*>(src)[i] * a;
        }
    }
}

}  // namespace lq

using namespace lq;

extern "C" int lq_load_lora(void* dst, const void* src, lq_dtype_t dtype, size_t n, float alpha, lq_stream_t stream) {
    LQ_REQUIRE((dst && src) || n == 0, LQ_ERR_ARG, "lq_load_lora: null pointer");
    if (n == 0) return LQ_OK;
    hipStream_t st = as_stream(stream);
    const unsigned blocks = (unsigned)std::min<size_t>((n + 255) / 256, 4096);
    switch (dtype) {
        case LQ_F32: hipLaunchKernelGGL((load_lora_kernel<F32Tag>), dim3(blocks), dim3(256), 0, st, dst, src, n, alpha); break;
        case LQ_F16: hipLaunchKernelGGL((load_lora_kernel<F16Tag>), dim3(blocks), dim3(256), 0, st, dst, src, n, alpha); break;
        case LQ_BF16: hipLaunchKernelGGL((load_lora_kernel<BF16Tag>), dim3(blocks), dim3(256), 0, st, dst, src, n, alpha); break;
        default: set_error("lq_load_lora: unsupported dtype %d", (int)dtype); return LQ_ERR_UNSUPPORTED;
    }
    return check_launch("lq_load_lora");
}

extern "C" int lq_lora_down(void* out, lq_dtype_t out_dtype, const void* x, const void* lora_down, lq_dtype_t dtype,
                            int m, int k, int rank, lq_stream_t stream) {
    LQ_REQUIRE(out && x && lora_down, LQ_ERR_ARG, "lq_lora_down: null pointer");
    LQ_REQUIRE(dtype == LQ_F16 || dtype == LQ_BF16, LQ_ERR_UNSUPPORTED, "lq_lora_down: operands must be F16 or BF16");
    LQ_REQUIRE(m >= 0 && k > 0 && k % 64 == 0 && (rank == 32 || rank == 64), LQ_ERR_SHAPE,
               "lq_lora_down: need k %% 64 == 0 and rank 32 or 64 (m=%d k=%d rank=%d)", m, k, rank);
    LQ_REQUIRE(reinterpret_cast<uintptr_t>(out) % 16 == 0 && reinterpret_cast<uintptr_t>(x) % 16 == 0 &&
                   reinterpret_cast<uintptr_t>(lora_down) % 16 == 0,
               LQ_ERR_ARG, "lq_lora_down: pointers must be 16-byte aligned");
    if (m == 0) return LQ_OK;
    hipStream_t st = as_stream(stream);
    if (dtype == LQ_F16) return rank == 32 ? launch_lora_down<true, 1>(out, out_dtype, x, lora_down, m, k, st)
                                           : launch_lora_down<true, 2>(out, out_dtype, x, lora_down, m, k, st);
    return rank == 32 ? launch_lora_down<false, 1>(out, out_dtype, x, lora_down, m, k, st)
                      : launch_lora_down<false, 2>(out, out_dtype, x, lora_down, m, k, st);
}

extern "C" int lq_cast_f32(void* dst, lq_dtype_t dst_dtype, const float* src, size_t n, lq_stream_t stream) {
    LQ_REQUIRE(dst && src, LQ_ERR_ARG, "lq_cast_f32: null pointer");
    if (n == 0) return LQ_OK;
    hipStream_t st = as_stream(stream);
    const unsigned blocks = (unsigned)std::min<size_t>((n + 255) / 256, 2048);
    switch (dst_dtype) {
        case LQ_F32: hipLaunchKernelGGL((cast_f32_kernel<0>), dim3(blocks), dim3(256), 0, st, dst, src, n); break;
        case LQ_F16: hipLaunchKernelGGL((cast_f32_kernel<1>), dim3(blocks), dim3(256), 0, st, dst, src, n); break;
        case LQ_BF16: hipLaunchKernelGGL((cast_f32_kernel<2>), dim3(blocks), dim3(256), 0, st, dst, src, n); break;
        default: set_error("lq_cast_f32: unsupported dtype %d", (int)dst_dtype); return LQ_ERR_UNSUPPORTED;
    }
    return check_launch("lq_cast_f32");
}
