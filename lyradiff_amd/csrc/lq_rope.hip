// Per-head RMSNorm of q and k, rotary embedding and the [text, image] concatenation between the QKV projections and the
// attention of the FLUX blocks: invokeFusedRmsNormCatAndRope / invokeFusedRmsNormAndRope of lyraDiff
// (kernels/rope/flux_apply_rope.cu:74-156,291-319; call sites layers/flux_attention_processor/FluxAttentionFP8Processor.cc:232-245,
// layers/flux_single_attention_processor/FluxSingleAttentionFP8Processor.cc:183-193).
//
//   out[b, s, c, h, :] for c = 0 (q), 1 (k):  n = T(x * rsqrt(mean(x^2) + eps)) * w[c]   (the product in T),
//                                             pair (n0, n1) -> ( T(T(n0*r00) + T(n1*r01)), T(T(n0*r10) + T(n1*r11)) )
//   out[b, s, 2, h, :] = v unchanged;   rows s < context_seq come from context_qkv (text tokens first), the rest from qkv.
//
// One wavefront per (token, head slot): a head of 128 elements is 64 lanes x one pair (head_dim 64: 32 lanes), the same
// two-elements-per-thread mapping the reference uses, so a wavefront reads and writes one contiguous 256-byte line.  The sum of
// squares is reduced across the wavefront in a fixed order; 1/sqrt is the IEEE one (the reference uses the approximate rsqrt).
#include "lq_common.h"

namespace lq {

__device__ __forceinline__ float rope_wave_sum(float v) {
#pragma unroll
    for (int off = 32; off > 0; off >>= 1) v += __shfl_xor(v, off, 64);
    return v;
}

template <typename Tag>
__global__ __launch_bounds__(256) void rmsnorm_rope_kernel(unsigned short* __restrict__ out, const unsigned short* __restrict__ qkv,
                                                           const unsigned short* __restrict__ ctx_qkv,
                                                           const unsigned short* __restrict__ norm_qk,
                                                           const unsigned short* __restrict__ norm_added_qk,
                                                           const unsigned short* __restrict__ rope, size_t rope_batch_stride,
                                                           int batch, int seq, int ctx_seq, int heads, int head_dim, float eps) {
    const int lane = threadIdx.x & 63;
    const int total = seq + ctx_seq, slots = 3 * heads;
    const size_t item = (size_t)blockIdx.x * 4 + (threadIdx.x >> 6);  // (b, s, slot), slot fastest
    if (item >= (size_t)batch * total * slots) return;
    const int slot = (int)(item % slots);
    const size_t bs = item / slots;
    const int s = (int)(bs % total), b = (int)(bs / total);
    const bool active = lane * 2 < head_dim;
    const bool is_ctx = s < ctx_seq;
    const unsigned short* src = is_ctx ? ctx_qkv + ((size_t)b * ctx_seq + s) * slots * head_dim
                                       : qkv + ((size_t)b * seq + (s - ctx_seq)) * slots * head_dim;
    u32 w = 0;
    if (active) w = *reinterpret_cast<const u32*>(src + (size_t)slot * head_dim + lane * 2);
    unsigned short* dst = out + (((size_t)b * total + s) * slots + slot) * head_dim + lane * 2;
    if (slot >= 2 * heads) {  // v: copied as it is
        if (active) *reinterpret_cast<u32*>(dst) = w;
        return;
    }
    const float x0 = Elem<Tag>::load(w & 0xFFFFu), x1 = Elem<Tag>::load(w >> 16);
    const float ss = rope_wave_sum(x0 * x0 + x1 * x1);  // inactive lanes contribute zeros
    if (!active) return;
    const float inv = 1.0f / __builtin_sqrtf(ss / (float)head_dim + eps);
    const unsigned short* wn = (is_ctx ? norm_added_qk : norm_qk) + (slot >= heads ? head_dim : 0) + lane * 2;
    const u32 wv = *reinterpret_cast<const u32*>(wn);
    const uint2 rv = *reinterpret_cast<const uint2*>(rope + (size_t)b * rope_batch_stride + ((size_t)s * head_dim + lane * 2) * 2);
    float n0 = x0 * inv, n1 = x1 * inv;
    round_through2<Tag>(n0, n1);
    n0 = n0 * Elem<Tag>::load(wv & 0xFFFFu);
    n1 = n1 * Elem<Tag>::load(wv >> 16);
    round_through2<Tag>(n0, n1);
    float a0 = n0 * Elem<Tag>::load(rv.x & 0xFFFFu), a1 = n1 * Elem<Tag>::load(rv.x >> 16);
    float c0 = n0 * Elem<Tag>::load(rv.y & 0xFFFFu), c1 = n1 * Elem<Tag>::load(rv.y >> 16);
    round_through2<Tag>(a0, a1);
    round_through2<Tag>(c0, c1);
    float y0 = a0 + a1, y1 = c0 + c1;
    asm volatile("" : "+v"(y0), "+v"(y1));  // the sums are rounded to fp32 before the conversion to T
    *reinterpret_cast<u32*>(dst) = Elem<Tag>::store(y0) | (Elem<Tag>::store(y1) << 16);
}

}  // namespace lq

using namespace lq;

extern "C" int lq_rmsnorm_rope(void* out, const void* qkv, const void* context_qkv, const void* norm_qk, const void* norm_added_qk,
                               const void* rope, size_t rope_batch_stride, lq_dtype_t dtype, int batch, int seq, int context_seq,
                               int heads, int head_dim, float eps, lq_stream_t stream) {
    LQ_REQUIRE(dtype == LQ_F16 || dtype == LQ_BF16, LQ_ERR_UNSUPPORTED, "lq_rmsnorm_rope: tensors must be F16 or BF16");
    LQ_REQUIRE(batch >= 0 && seq >= 0 && context_seq >= 0 && heads > 0 && (head_dim == 64 || head_dim == 128), LQ_ERR_SHAPE,
               "lq_rmsnorm_rope: need head_dim 64 or 128 (batch=%d seq=%d context_seq=%d heads=%d head_dim=%d)", batch, seq,
               context_seq, heads, head_dim);
    const size_t items = (size_t)batch * ((size_t)seq + context_seq) * 3 * heads;
    if (items == 0) return LQ_OK;
    LQ_REQUIRE(out && norm_qk && rope && (qkv || seq == 0) && (context_seq == 0 || (context_qkv && norm_added_qk)), LQ_ERR_ARG,
               "lq_rmsnorm_rope: null pointer");
    LQ_REQUIRE(reinterpret_cast<uintptr_t>(out) % 4 == 0 && reinterpret_cast<uintptr_t>(qkv) % 4 == 0 &&
                   reinterpret_cast<uintptr_t>(context_qkv) % 4 == 0 && reinterpret_cast<uintptr_t>(norm_qk) % 4 == 0 &&
                   reinterpret_cast<uintptr_t>(norm_added_qk) % 4 == 0 && reinterpret_cast<uintptr_t>(rope) % 8 == 0 &&
                   rope_batch_stride % 4 == 0,
               LQ_ERR_ARG, "lq_rmsnorm_rope: tensors must be 4-byte aligned, rope (and its batch stride) 8-byte aligned");
    LQ_REQUIRE((items + 3) / 4 <= 0x7fffffffu, LQ_ERR_SHAPE, "lq_rmsnorm_rope: too many (token, head) pairs for one launch");
    dim3 grid((unsigned)((items + 3) / 4)), block(256);
    hipStream_t st = as_stream(stream);
    auto us = [](const void* p) { return static_cast<const unsigned short*>(p); };
    if (dtype == LQ_F16)
        hipLaunchKernelGGL((rmsnorm_rope_kernel<F16Tag>), grid, block, 0, st, static_cast<unsigned short*>(out), us(qkv), us(context_qkv),
                           us(norm_qk), us(norm_added_qk), us(rope), rope_batch_stride, batch, seq, context_seq, heads, head_dim, eps);
    else
        hipLaunchKernelGGL((rmsnorm_rope_kernel<BF16Tag>), grid, block, 0, st, static_cast<unsigned short*>(out), us(qkv), us(context_qkv),
                           us(norm_qk), us(norm_added_qk), us(rope), rope_batch_stride, batch, seq, context_seq, heads, head_dim, eps);
    return check_launch("lq_rmsnorm_rope");
}
