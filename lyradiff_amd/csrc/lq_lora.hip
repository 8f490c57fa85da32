// Low-rank ("SVDQuant") side branch of the W4A4 linear: the down projection
//     out[m, r] = sum_k x[m, k] * down[r, k]        (16-bit float operands, fp32 accumulation)
// that the reference computes inside its quantisation kernel with float atomics
// (kernels/w4a4_gemm/w4a4_gemm.cu:769-953 of lyraDiff, `reduce_add` into a zeroed fp32 buffer, followed by a
// separate float -> T conversion, layers/w4a4_gemm_block/W4A4Gemm.cc:138-150).  Here it is a skinny GEMM of its
// own: a workgroup owns up to 32 rows and all of K, its eight wavefronts take interleaved 64-wide slices of K, the
// partial 32 x rank blocks meet in LDS and are added in wavefront order -- no atomics, so the result does not
// depend on scheduling -- and the output is written once, already in the requested type.  It reads x from HBM
// only if the quantisation kernel that ran just before did not leave it in the caches.
// The matrix instruction wants a lane to hold eight consecutive k of ONE row, so loading its operands straight
// from memory makes every load instruction touch 32 different cache lines and use a quarter of each; the cache's
// tag rate, not bandwidth or latency, then sets the time (about 10 us whatever m is).  A slice therefore takes the
// coalesced route: a load instruction fetches eight whole 128-byte lines (eight lanes per row), the wavefront
// parks the slice in its private, bank-swizzled LDS block and reads the fragments back from there.  The launch
// spreads the rows over every CU: a workgroup takes ceil(m / CUs) rows when that is fewer than 32 (the unused
// rows of the 32-row matrix instruction repeat the last one, which costs no memory traffic).
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
                                                        const unsigned short* __restrict__ down, int m, int k, int rows_per_wg) {
    constexpr int W = 8;                    // wavefronts per workgroup, each takes every eighth 64-wide slice of K
    constexpr int WAVE_STAGE = (1 + NR) * 4096;  // one slice of x and of `down`: 32 rows x 128 bytes each
    constexpr int PART_BYTES = (W - 1) * NR * 16 * 64 * 4;
    __shared__ __attribute__((aligned(16))) char smem[W * WAVE_STAGE > PART_BYTES ? W * WAVE_STAGE : PART_BYTES];
    const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
    const int row0 = blockIdx.x * rows_per_wg;
    const int lr = lane & 31, lh = lane >> 5;
    char* stage = smem + wave * WAVE_STAGE;
    // memory side: lane -> (row 8*i + lane/8, 16-byte chunk lane%8); LDS side: chunk c of row r sits at chunk
    // slot c ^ ((r >> 1) & 7), which keeps both the 16-lane write groups and the 16-lane read groups conflict-free
    const int gr = lane >> 3, gc = lane & 7;
    const unsigned short* xg[4];
    const unsigned short* dg[4];
    int wofs[4], rofs[4];
#pragma unroll
    for (int i = 0; i < 4; ++i) {
        const int r = i * 8 + gr;
        xg[i] = x + (size_t)min(row0 + min(r, rows_per_wg - 1), m - 1) * k + gc * 8;
        dg[i] = down + (size_t)r * k + gc * 8;
        wofs[i] = r * 128 + ((gc ^ ((r >> 1) & 7)) << 4);
        rofs[i] = lr * 128 + (((2 * i + lh) ^ ((lr >> 1) & 7)) << 4);  // matrix step i: k = 16 i + 8 lh .. + 8
    }
    v16f_t acc[NR];
#pragma unroll
    for (int r = 0; r < NR; ++r)
#pragma unroll
        for (int v = 0; v < 16; ++v) acc[r][v] = 0.0f;
    // The lines of the next slice are requested before the current slice goes through LDS and the matrix
    // instructions, so their latency is hidden behind that work and the other wavefronts.
    constexpr int NBUF = 2;  // the slice on its way through LDS and the one requested behind it (deeper queues measured no faster)
    v4i gx[NBUF][4], gd[NBUF][NR][4];
    auto load_slice = [&](int k0, int buf) {
#pragma unroll
        for (int i = 0; i < 4; ++i) {
            gx[buf][i] = *reinterpret_cast<const v4i*>(xg[i] + k0);
#pragma unroll
            for (int r = 0; r < NR; ++r) gd[buf][r][i] = *reinterpret_cast<const v4i*>(dg[i] + (size_t)r * 32 * k + k0);
        }
    };
    auto compute_slice = [&](int buf) {
#pragma unroll
        for (int i = 0; i < 4; ++i) {
            *reinterpret_cast<v4i*>(stage + wofs[i]) = gx[buf][i];
#pragma unroll
            for (int r = 0; r < NR; ++r) *reinterpret_cast<v4i*>(stage + (1 + r) * 4096 + wofs[i]) = gd[buf][r][i];
        }
        // the wavefront's LDS accesses complete in program order; the fence only keeps the compiler from
        // moving the reads of other lanes' data above the writes
        __builtin_amdgcn_fence(__ATOMIC_ACQ_REL, "wavefront");
        __builtin_amdgcn_wave_barrier();
#pragma unroll
        for (int s = 0; s < 4; ++s) {
            const v4i xf = *reinterpret_cast<const v4i*>(stage + rofs[s]);
#pragma unroll
            for (int r = 0; r < NR; ++r)
                acc[r] = mfma16<F16>(*reinterpret_cast<const v4i*>(stage + (1 + r) * 4096 + rofs[s]), xf, acc[r]);
        }
        __builtin_amdgcn_fence(__ATOMIC_ACQ_REL, "wavefront");
        __builtin_amdgcn_wave_barrier();
    };
    constexpr int STEP = 64 * W;
    int k0 = wave * 64;
#pragma unroll
    for (int b = 0; b < NBUF - 1; ++b)
        if (k0 + b * STEP < k) load_slice(k0 + b * STEP, b);
    // the buffers rotate with a period of NBUF slices; the loop body is unrolled over one period so that every
    // buffer index is a compile-time constant (the lines in flight must stay in registers)
    for (; k0 < k; k0 += NBUF * STEP) {
#pragma unroll
        for (int b = 0; b < NBUF; ++b) {
            if (k0 + b * STEP < k) {
                if (k0 + (b + NBUF - 1) * STEP < k) load_slice(k0 + (b + NBUF - 1) * STEP, (b + NBUF - 1) % NBUF);
                compute_slice(b);
            }
        }
    }
    __syncthreads();  // every wavefront is done with its operand block: the partial sums may overwrite them
    float(*part)[NR][16][64] = reinterpret_cast<float(*)[NR][16][64]>(smem);  // partial blocks of wavefronts 1..7
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
        if (row < m && lr < rows_per_wg) {
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
    static const int num_cu = [] {
        int dev = 0, n = 0;
        if (hipGetDevice(&dev) != hipSuccess || hipDeviceGetAttribute(&n, hipDeviceAttributeMultiprocessorCount, dev) != hipSuccess || n <= 0) n = 256;
        return n;
    }();
    const int rpw = std::min(32, std::max(8, (m + num_cu - 1) / num_cu));
    dim3 grid((unsigned)((m + rpw - 1) / rpw)), block(512);
    const unsigned short* xs = static_cast<const unsigned short*>(x);
    const unsigned short* ds = static_cast<const unsigned short*>(down);
    switch (out_dtype) {
        case LQ_F32: hipLaunchKernelGGL((lora_down_kernel<F16, NR, 0>), grid, block, 0, st, out, xs, ds, m, k, rpw); break;
        case LQ_F16: hipLaunchKernelGGL((lora_down_kernel<F16, NR, 1>), grid, block, 0, st, out, xs, ds, m, k, rpw); break;
        case LQ_BF16: hipLaunchKernelGGL((lora_down_kernel<F16, NR, 2>), grid, block, 0, st, out, xs, ds, m, k, rpw); break;
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
