// The persistent one-wavefront-per-SIMD INT8 / FP8 GEMM kernels (lq_gemm_persist.h) in a translation unit of their own: the
// instantiations (INT8, FP8, FP8 with the running maximum of the outputs) x (fp16, bf16 output), each with the 256-row and the
// 128-row tile form.
#include "lq_gemm_persist.h"

#include <atomic>

namespace lq {

int device_cu_count() {
    static std::atomic<int> cached[64];
    int dev = 0;
    if (hipGetDevice(&dev) != hipSuccess || dev < 0 || dev >= 64) {
        (void)hipGetLastError();
        return 0;
    }
    int cus = cached[dev].load(std::memory_order_relaxed);
    if (cus > 0) return cus;
    if (hipDeviceGetAttribute(&cus, hipDeviceAttributeMultiprocessorCount, dev) != hipSuccess || cus <= 0) {
        (void)hipGetLastError();
        return 0;
    }
    cached[dev].store(cus, std::memory_order_relaxed);
    return cus;
}

int launch_persist_fp8(const GemmParams& p, lq_dtype_t out_dtype, hipStream_t st) {
    switch (out_dtype) {
        case LQ_F16: return p.out_max ? launch_gemm_persist<K_FP8, F16Tag, true>(p, st) : launch_gemm_persist<K_FP8, F16Tag>(p, st);
        case LQ_BF16: return p.out_max ? launch_gemm_persist<K_FP8, BF16Tag, true>(p, st) : launch_gemm_persist<K_FP8, BF16Tag>(p, st);
        default: return 1;
    }
}

int launch_persist_int8(const GemmParams& p, lq_dtype_t out_dtype, hipStream_t st) {
    switch (out_dtype) {
        case LQ_F16: return launch_gemm_persist<K_INT8, F16Tag>(p, st);
        case LQ_BF16: return launch_gemm_persist<K_INT8, BF16Tag>(p, st);
        default: return 1;
    }
}

}  // namespace lq
