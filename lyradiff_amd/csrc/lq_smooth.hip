// SmoothQuant smoothing vector on the device (calibration time).  The reference consumes a precomputed
// pre_quant_scale = 1/s from nvidia-modelopt (lyradiff/convert_model_scripts/convert_sd_quant_model.py:199,340); the
// closed form used here is the one its benchmark configuration states:
//     s[k] = max_m |X[m,k]|^alpha / max_n |W[n,k]|^(1-alpha),   pre[k] = 1 / s[k],
// and W is multiplied by s offline (lq_int8_weight_quant divides by pre, kernels/quant_kernels/quant_kernels.cu:197-199).
// lq_col_absmax accumulates the per-column maxima over any number of calibration batches (integer-punned atomic max on
// non-negative floats: exact and order independent); lq_smooth_vector turns two such vectors into s and pre.
#include "lq_common.h"

namespace lq {

// Each thread owns 8 consecutive columns and walks a slab of rows; one atomic per column per workgroup slab.
template <typename Tag>
__global__ __launch_bounds__(256) void col_absmax_kernel(float* __restrict__ out, const void* __restrict__ x, size_t rows, int dim,
                                                         int rows_per_block) {
    const int col = (blockIdx.x * 256 + threadIdx.x) * 8;
    if (col >= dim) return;
    const size_t r0 = (size_t)blockIdx.y * rows_per_block;
    const size_t r1 = r0 + rows_per_block < rows ? r0 + rows_per_block : rows;
    float m[8] = {0, 0, 0, 0, 0, 0, 0, 0};
    for (size_t r = r0; r < r1; ++r) {
        float v[8];
        if constexpr (Elem<Tag>::bytes == 2) {
            unpack8<Tag>(*reinterpret_cast<const uint4*>(static_cast<const unsigned short*>(x) + r * dim + col), v);
        } else {
            const float4 a = *reinterpret_cast<const float4*>(static_cast<const float*>(x) + r * dim + col);
            const float4 b = *reinterpret_cast<const float4*>(static_cast<const float*>(x) + r * dim + col + 4);
            v[0] = a.x; v[1] = a.y; v[2] = a.z; v[3] = a.w; v[4] = b.x; v[5] = b.y; v[6] = b.z; v[7] = b.w;
        }
#pragma unroll
        for (int i = 0; i < 8; ++i) m[i] = fmaxf(m[i], fabsf(v[i]));  // fmaxf drops a NaN operand, as CUDA's max does
    }
#pragma unroll
    for (int i = 0; i < 8; ++i) {
        int* slot = reinterpret_cast<int*>(out + col + i);
        if (__float_as_int(m[i]) > __hip_atomic_load(slot, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT)) atomicMax(slot, __float_as_int(m[i]));
    }
}

__global__ void smooth_vector_kernel(float* __restrict__ pre, float* __restrict__ s_out, const float* __restrict__ ax,
                                     const float* __restrict__ aw, float alpha, int dim) {
    const int k = blockIdx.x * blockDim.x + threadIdx.x;
    if (k >= dim) return;
    const float s = __builtin_powf(ax[k], alpha) / __builtin_powf(aw[k], 1.0f - alpha);
    if (s_out != nullptr) s_out[k] = s;
    pre[k] = 1.0f / s;
}

}  // namespace lq

using namespace lq;

extern "C" int lq_col_absmax(float* out, const void* x, lq_dtype_t dtype, size_t rows, size_t dim, lq_stream_t stream) {
    LQ_REQUIRE(out && (x || rows == 0), LQ_ERR_ARG, "lq_col_absmax: null pointer");
    LQ_REQUIRE(dim > 0 && dim % 8 == 0 && dim <= (1u << 24), LQ_ERR_SHAPE, "lq_col_absmax: need dim %% 8 == 0 (dim=%zu)", dim);
    LQ_REQUIRE(reinterpret_cast<uintptr_t>(x) % 16 == 0, LQ_ERR_ARG, "lq_col_absmax: x must be 16-byte aligned");
    if (rows == 0) return LQ_OK;
    const int rpb = 64;
    dim3 grid((unsigned)((dim / 8 + 255) / 256), (unsigned)std::min<size_t>((rows + rpb - 1) / rpb, 65535)), block(256);
    const int rows_per_block = (int)((rows + grid.y - 1) / grid.y);
    hipStream_t st = as_stream(stream);
    switch (dtype) {
        case LQ_F16: hipLaunchKernelGGL((col_absmax_kernel<F16Tag>), grid, block, 0, st, out, x, rows, (int)dim, rows_per_block); break;
        case LQ_BF16: hipLaunchKernelGGL((col_absmax_kernel<BF16Tag>), grid, block, 0, st, out, x, rows, (int)dim, rows_per_block); break;
        case LQ_F32: hipLaunchKernelGGL((col_absmax_kernel<F32Tag>), grid, block, 0, st, out, x, rows, (int)dim, rows_per_block); break;
        default: set_error("lq_col_absmax: unsupported dtype %d", (int)dtype); return LQ_ERR_UNSUPPORTED;
    }
    return check_launch("lq_col_absmax");
}

extern "C" int lq_smooth_vector(float* pre_quant_scale, float* smooth_out, const float* act_absmax, const float* weight_absmax,
                                float alpha, size_t dim, lq_stream_t stream) {
    LQ_REQUIRE(pre_quant_scale && act_absmax && weight_absmax, LQ_ERR_ARG, "lq_smooth_vector: null pointer");
    LQ_REQUIRE(alpha >= 0.0f && alpha <= 1.0f, LQ_ERR_ARG, "lq_smooth_vector: alpha=%f outside [0,1]", (double)alpha);
    if (dim == 0) return LQ_OK;
    hipLaunchKernelGGL(smooth_vector_kernel, dim3((unsigned)((dim + 255) / 256)), dim3(256), 0, as_stream(stream), pre_quant_scale,
                       smooth_out, act_absmax, weight_absmax, alpha, (int)dim);
    return check_launch("lq_smooth_vector");
}
