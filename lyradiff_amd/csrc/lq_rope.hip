// Per-head RMSNorm of q and k, rotary embedding and the [text, image] concatenation between the QKV projections and the
// attention of the FLUX blocks: invokeFusedRmsNormCatAndRope / invokeFusedRmsNormAndRope of lyraDiff
// (kernels/rope/flux_apply_rope.cu:74-156,291-319; call sites layers/flux_attention_processor/FluxAttentionFP8Processor.cc:232-245,
// layers/flux_single_attention_processor/FluxSingleAttentionFP8Processor.cc:183-193).
//
//   out[b, s, c, h, :] for c = 0 (q), 1 (k):  n = T(x * rsqrt(mean(x^2) + eps)) * w[c]   (the product in T),
//                                             pair (n0, n1) -> ( T(T(n0*r00) + T(n1*r01)), T(T(n0*r10) + T(n1*r11)) )
//   out[b, s, 2, h, :] = v unchanged;   rows s < context_seq come from context_qkv (text tokens first), the rest from qkv.
//
// A workgroup of four wavefronts owns one token.  A lane holds four consecutive elements (two rotation pairs) of a head, so a
// head of 128 elements is half a wavefront (head_dim 64: a quarter) and a wavefront works on two (four) head slots at a time;
// the token's rotation matrices and the norm weights are loaded once per wavefront and reused for all of its slots, and the
// 8-byte loads of up to four slot groups are in flight together.  The sum of squares is reduced across the lanes of a head in
// a fixed order; 1/sqrt is the IEEE one (the reference uses the approximate rsqrt).
#include "lq_common.h"

namespace lq {

template <typename Tag, int LPH>  // LPH = head_dim / 4 lanes per head: 32 or 16
__global__ __launch_bounds__(256) void rmsnorm_rope_kernel(unsigned short* __restrict__ out, const unsigned short* __restrict__ qkv,
                                                           const unsigned short* __restrict__ ctx_qkv,
                                                           const unsigned short* __restrict__ norm_qk,
                                                           const unsigned short* __restrict__ norm_added_qk,
                                                           const unsigned short* __restrict__ rope, size_t rope_batch_stride,
                                                           int seq, int ctx_seq, int heads, float eps) {
    constexpr int DH = LPH * 4, HP = 64 / LPH, U = 4;
    const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
    const int sub = lane / LPH, l = lane % LPH;
    const int total = seq + ctx_seq, slots = 3 * heads;
    const int s = (int)(blockIdx.x % total), b = (int)(blockIdx.x / total);
    const bool is_ctx = s < ctx_seq;
    const unsigned short* src = is_ctx ? ctx_qkv + ((size_t)b * ctx_seq + s) * slots * DH
                                       : qkv + ((size_t)b * seq + (s - ctx_seq)) * slots * DH;
    unsigned short* dst = out + ((size_t)b * total + s) * slots * DH;
    // this lane's two rotation matrices (r00 r01 r10 r11 each) and its four q and four k norm weights
    const uint4 rv = *reinterpret_cast<const uint4*>(rope + (size_t)b * rope_batch_stride + ((size_t)s * DH + l * 4) * 2);
    const unsigned short* wn = is_ctx ? norm_added_qk : norm_qk;
    const uint2 wq = *reinterpret_cast<const uint2*>(wn + l * 4), wk = *reinterpret_cast<const uint2*>(wn + DH + l * 4);
    const u32 rw[4] = {rv.x, rv.y, rv.z, rv.w};
    const int groups = (slots + HP - 1) / HP;  // slot groups of this token; wavefront w takes groups w, w + 4, ...
    for (int g0 = wave; g0 < groups; g0 += 4 * U) {
        uint2 raw[U];
#pragma unroll
        for (int u = 0; u < U; ++u) {
            const int slot = (g0 + 4 * u) * HP + sub;
            raw[u] = make_uint2(0, 0);
            if (g0 + 4 * u < groups && slot < slots) raw[u] = *reinterpret_cast<const uint2*>(src + (size_t)slot * DH + l * 4);
        }
#pragma unroll
        for (int u = 0; u < U; ++u) {
            const int slot = (g0 + 4 * u) * HP + sub;
            const bool live = g0 + 4 * u < groups && slot < slots;
            const u32 xw[2] = {raw[u].x, raw[u].y};
            float x[4];
#pragma unroll
            for (int i = 0; i < 2; ++i) {
                x[2 * i] = Elem<Tag>::load(xw[i] & 0xFFFFu);
                x[2 * i + 1] = Elem<Tag>::load(xw[i] >> 16);
            }
            float ss = (x[0] * x[0] + x[1] * x[1]) + (x[2] * x[2] + x[3] * x[3]);  // lanes without a slot contribute zeros
#pragma unroll
            for (int off = LPH / 2; off > 0; off >>= 1) ss += __shfl_xor(ss, off, 64);  // stays inside the head's lanes
            uint2 o = raw[u];
            if (slot < 2 * heads) {  // q or k
                const float inv = 1.0f / __builtin_sqrtf(ss / (float)DH + eps);
                const uint2 wv = slot < heads ? wq : wk;
                const u32 ww[2] = {wv.x, wv.y};
                u32 ow[2];
#pragma unroll
                for (int i = 0; i < 2; ++i) {  // pair i of this lane
                    float n0 = x[2 * i] * inv, n1 = x[2 * i + 1] * inv;
                    round_through2<Tag>(n0, n1);
                    n0 = n0 * Elem<Tag>::load(ww[i] & 0xFFFFu);
                    n1 = n1 * Elem<Tag>::load(ww[i] >> 16);
                    round_through2<Tag>(n0, n1);
                    float a0 = n0 * Elem<Tag>::load(rw[2 * i] & 0xFFFFu), a1 = n1 * Elem<Tag>::load(rw[2 * i] >> 16);
                    float c0 = n0 * Elem<Tag>::load(rw[2 * i + 1] & 0xFFFFu), c1 = n1 * Elem<Tag>::load(rw[2 * i + 1] >> 16);
                    round_through2<Tag>(a0, a1);
                    round_through2<Tag>(c0, c1);
                    float y0 = a0 + a1, y1 = c0 + c1;
                    asm volatile("" : "+v"(y0), "+v"(y1));  // the sums are rounded to fp32 before the conversion to T
                    ow[i] = Elem<Tag>::store(y0) | (Elem<Tag>::store(y1) << 16);
                }
                o = make_uint2(ow[0], ow[1]);
            }
            if (live) *reinterpret_cast<uint2*>(dst + (size_t)slot * DH + l * 4) = o;
        }
    }
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
    LQ_REQUIRE(reinterpret_cast<uintptr_t>(out) % 8 == 0 && reinterpret_cast<uintptr_t>(qkv) % 8 == 0 &&
                   reinterpret_cast<uintptr_t>(context_qkv) % 8 == 0 && reinterpret_cast<uintptr_t>(norm_qk) % 8 == 0 &&
                   reinterpret_cast<uintptr_t>(norm_added_qk) % 8 == 0 && reinterpret_cast<uintptr_t>(rope) % 16 == 0 &&
                   rope_batch_stride % 8 == 0,
               LQ_ERR_ARG, "lq_rmsnorm_rope: tensors must be 8-byte aligned, rope 16-byte aligned and its batch stride a multiple of 8 elements");
    const size_t tokens = (size_t)batch * ((size_t)seq + context_seq);
    LQ_REQUIRE(tokens <= 0x7fffffffu, LQ_ERR_SHAPE, "lq_rmsnorm_rope: too many tokens for one launch");
    dim3 grid((unsigned)tokens), block(256);
    hipStream_t st = as_stream(stream);
    auto us = [](const void* p) { return static_cast<const unsigned short*>(p); };
#define LQ_ROPE_GO(TAG, LPH)                                                                                              \
    hipLaunchKernelGGL((rmsnorm_rope_kernel<TAG, LPH>), grid, block, 0, st, static_cast<unsigned short*>(out), us(qkv),   \
                       us(context_qkv), us(norm_qk), us(norm_added_qk), us(rope), rope_batch_stride, seq, context_seq, heads, eps)
    if (dtype == LQ_F16) {
        if (head_dim == 128) LQ_ROPE_GO(F16Tag, 32);
        else LQ_ROPE_GO(F16Tag, 16);
    } else {
        if (head_dim == 128) LQ_ROPE_GO(BF16Tag, 32);
        else LQ_ROPE_GO(BF16Tag, 16);
    }
#undef LQ_ROPE_GO
    return check_launch("lq_rmsnorm_rope");
}
