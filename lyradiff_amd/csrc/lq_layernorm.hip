// LayerNorm fused with the activation quantisation that follows it, the step in front of every
// quantized linear of the reference's blocks:
//   * INT8 (SDXL): invokeLayerNormInt8O / invokeFusedResidualBiasLayerNormInt8O
//     (kernels/quant_kernels/layer_norm_int8.cu:102-556,558-679 of lyraDiff):
//       h = src [+ residual + bias]  (kept in T, written to dst2 when the residual is fused)
//       y = T( gamma * ((h - mean) * rstd) + beta ),   q = sat_s8(rne( f32(y) * pre[k] / s ))
//   * FP8 (FLUX): invokeLayerNormWithShiftAndScale followed by invokeCudaD2DScaleCpyConvert
//     (kernels/norms/layer_norm.cu:406-475, layers/flux_attn_post_processor/FluxAttnPostFP8Processor.cc:125-140):
//       y = T( T( T(scale[b,k] + 1) * T((x - mean) * rstd) ) + shift[b,k] ),   q = e4m3( f32(y) * (1/s) )
//     optionally preceded by invokeFusedGateAndResidual (kernels/flux_single_transformer_block/
//     flux_single_transformer_kernels.cu:42-65, FluxAttnPostFP8Processor.cc:112-119):
//       x = T( T(attn * gate[b,k]) + input ), also written out (the block's second residual uses it)
// A row is owned by one wavefront (by one wavefront per 1024 columns when it is longer than 1536): it stays in registers between the statistics and the quantisation, so the
// activation is read once and only the 1-byte codes (and dst2) are written.  Mean and variance are two-pass
// fp32 sums over the registers (the reference runs Welford updates, in T for the INT8 kernels), reduced across
// the 64 lanes in a fixed order; rstd = 1 / sqrt(var + eps) with IEEE sqrt and division.
#include "lq_common.h"

namespace lq {

// Sum over the 64 lanes in a fixed order with DPP operand swizzles only (no LDS round trips, one instruction per step):
// four exchange steps inside each row of 16 lanes, then row_bcast:15 adds the total of rows 0 / 2 into rows 1 / 3 and
// row_bcast:31 the total of rows 0+1 into rows 2 and 3.  The complete sum is in lane 63 ONLY.
template <int CTRL, int ROW_MASK> __device__ __forceinline__ float dpp_f32(float v) {
    return __builtin_bit_cast(float, __builtin_amdgcn_update_dpp(0, __builtin_bit_cast(int, v), CTRL, ROW_MASK, 0xF, false));
}
// RN(s / d) for a small integer d from r = RN(1 / d): product, exact remainder, one corrected step (Markstein).  Exact for
// every finite s of moderate magnitude (no mismatch against IEEE division in 8e8 trials on the CPU over every d = 8 .. 16384,
// random and near-midpoint quotients); zero, tiny, huge and non-finite sums take the true division, three instructions
// instead of eleven otherwise.
__device__ __forceinline__ float div_small_int(float s, float d, float r) {
    const float q = s * r;
    const float rem = __builtin_fmaf(-q, d, s);
    const float q1 = __builtin_fmaf(rem, r, q);
    const float a = fabsf(s);
    if (__builtin_expect(!(a > 0x1p-80f && a < 0x1p80f), 0)) return s / d;
    return q1;
}
__device__ __forceinline__ float wave_sum_lane63(float v) {
    v += dpp_f32<0xB1, 0xF>(v);   // quad_perm [1,0,3,2]
    v += dpp_f32<0x4E, 0xF>(v);   // quad_perm [2,3,0,1]
    v += dpp_f32<0x141, 0xF>(v);  // row_half_mirror
    v += dpp_f32<0x140, 0xF>(v);  // row_mirror: every lane of a row holds the row's total
    v += dpp_f32<0x142, 0xA>(v);  // row_bcast:15 into rows 1 and 3
    v += dpp_f32<0x143, 0xC>(v);  // row_bcast:31 into rows 2 and 3
    return v;
}

__device__ __forceinline__ u32 ln_cvt4_e4m3(float a, float b, float c, float d) {  // finite inputs: saturating RNE
    a = __builtin_amdgcn_fmed3f(a, 448.0f, -448.0f); b = __builtin_amdgcn_fmed3f(b, 448.0f, -448.0f);
    c = __builtin_amdgcn_fmed3f(c, 448.0f, -448.0f); d = __builtin_amdgcn_fmed3f(d, 448.0f, -448.0f);
    u32 w = (u32)__builtin_amdgcn_cvt_pk_fp8_f32(a, b, 0, false);
    return (u32)__builtin_amdgcn_cvt_pk_fp8_f32(c, d, (int)w, true);
}
__device__ __forceinline__ u32 ln_nan_fix(u32 w, const float* y) {  // NaN -> 0x7F | sign, as the cast kernel does
#pragma unroll
    for (int i = 0; i < 4; ++i)
        if (y[i] != y[i]) w = (w & ~(0xFFu << (8 * i))) | ((0x7Fu | ((__float_as_uint(y[i]) >> 24) & 0x80u)) << (8 * i));
    return w;
}

// QMODE 0: int8, static per-tensor scale; 1: int8, dynamic per-token scale (written to scale_out); 2: fp8, static scale;
// 3: no quantisation, y stored as T (the input of a W4A4 linear, which quantises per group and also feeds its low-rank branch).
// MOD false: y = gamma*n + beta (vectors of length dim).  MOD true: y = (1 + scale[b])*n + shift[b], b = row / rows_per_batch.
// RESID 0: h = src.  1: h = T(T(src + residual) + bias).  2: h = T(T(src * gate[b]) + residual), gate passed as `bias`.
// SPLIT false: a workgroup is four wavefronts with a row each (NP passes of 512 columns, rows up to 1536 columns).
// SPLIT true (longer rows): a workgroup owns one row, cut into 1024-column spans with a wavefront each (NP = 2), so a
// wavefront needs about 60 registers whatever the row length and eight of them share a SIMD; the three row reductions
// then take a step through LDS, added in wavefront order.
// FULL (SPLIT only): dim is a multiple of 1024, every lane of every wavefront owns valid columns in both passes: no range
// checks and no zero-filling of unused registers (7 % of the instructions of a kernel that is bound by its vector ALU).
template <typename Tag, int NP, int QMODE, int RESID, bool MOD, bool SPLIT, bool FULL = false, bool STREAM = false>
__global__ __launch_bounds__(SPLIT ? 384 : 256) void ln_quant_rows_kernel(uint8_t* __restrict__ dst, void* __restrict__ dst2,
                                                            float* __restrict__ scale_out, const void* __restrict__ src,
                                                            const void* __restrict__ residual, const void* __restrict__ bias,
                                                            const void* __restrict__ gamma, const void* __restrict__ beta,
                                                            const float* __restrict__ pre, const float* __restrict__ in_scale,
                                                            uint8_t* __restrict__ dst_b, const float* __restrict__ in_scale_b,
                                                            size_t rows, int dim, size_t rows_per_batch, float eps, float rdim, int codes_panel) {
    // codes_panel (fp8 codes only): dst / dst_b are k-panels [dim / 64][rows][64] instead of row-major (a lane's eight codes
    // stay inside one 64-byte segment), the activation layout of lq_gemm_fp8_panels
    __shared__ __attribute__((aligned(16))) float red[3][8];
    const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
    const size_t row = SPLIT ? (size_t)blockIdx.x : (size_t)blockIdx.x * 4 + wave;
    const int cbase = SPLIT ? wave * 1024 : 0;
    if constexpr (SPLIT) {
        if (threadIdx.x < 24) red[threadIdx.x >> 3][threadIdx.x & 7] = 0.0f;
        __syncthreads();
    } else {
        if (row >= rows) return;
    }
    // sum / max over the whole row from per-wavefront results (slot k of the LDS array is used once)
    auto row_sum = [&](float v, int k) -> float {
        v = wave_sum_lane63(v);
        if constexpr (SPLIT) {
            if (lane == 63) red[k][wave] = v;
            __syncthreads();
            const float4 a = *reinterpret_cast<const float4*>(red[k]), b = *reinterpret_cast<const float4*>(red[k] + 4);
            v = ((((a.x + a.y) + a.z) + a.w) + b.x) + b.y;
        } else {
            v = __builtin_bit_cast(float, __builtin_amdgcn_readlane(__builtin_bit_cast(int, v), 63));
        }
        return v;
    };
    auto row_max = [&](float v, int k) -> float {
        v = wave_max(v);
        if constexpr (SPLIT) {
            if (lane == 0) red[k][wave] = v;
            __syncthreads();
            const float4 a = *reinterpret_cast<const float4*>(red[k]), b = *reinterpret_cast<const float4*>(red[k] + 4);
            v = fmaxf(fmaxf(fmaxf(a.x, a.y), fmaxf(a.z, a.w)), fmaxf(b.x, b.y));
        }
        return v;
    };
    const size_t row_off = row * (size_t)dim;
    const unsigned short* xs = static_cast<const unsigned short*>(src) + row_off;
    const size_t mod_off = (MOD || RESID == 2) ? (row / rows_per_batch) * (size_t)dim : 0;
    const unsigned short* gs = static_cast<const unsigned short*>(gamma) + mod_off;
    const unsigned short* bs = static_cast<const unsigned short*>(beta) + mod_off;
    float h[NP][8];
    float sum = 0.0f;
#pragma unroll
    for (int p = 0; p < NP; ++p) {
        const int col = cbase + (p * 64 + lane) * 8;
#pragma unroll
        for (int i = 0; i < 8; ++i) h[p][i] = 0.0f;
        if (FULL || col < dim) {
            unpack8<Tag>(ld16<STREAM>(xs + col), h[p]);
            if constexpr (RESID != 0) {
                float r[8], b[8];
                unpack8<Tag>(*reinterpret_cast<const uint4*>(static_cast<const unsigned short*>(residual) + row_off + col), r);
                if constexpr (RESID == 2) {
                    unpack8<Tag>(*reinterpret_cast<const uint4*>(static_cast<const unsigned short*>(bias) + mod_off + col), b);
#pragma unroll
                    for (int i = 0; i < 8; ++i) h[p][i] = round_through<Tag>(round_through<Tag>(h[p][i] * b[i]) + r[i]);
                } else {
#pragma unroll
                    for (int i = 0; i < 8; ++i) h[p][i] = round_through<Tag>(h[p][i] + r[i]);
                    if (bias != nullptr) {
                        unpack8<Tag>(*reinterpret_cast<const uint4*>(static_cast<const unsigned short*>(bias) + col), b);
#pragma unroll
                        for (int i = 0; i < 8; ++i) h[p][i] = round_through<Tag>(h[p][i] + b[i]);
                    }
                }
                uint4 o;
                u32* ow = reinterpret_cast<u32*>(&o);
#pragma unroll
                for (int i = 0; i < 4; ++i) ow[i] = Elem<Tag>::store(h[p][2 * i]) | (Elem<Tag>::store(h[p][2 * i + 1]) << 16);
                *reinterpret_cast<uint4*>(static_cast<unsigned short*>(dst2) + row_off + col) = o;
            }
#pragma unroll
            for (int i = 0; i < 8; ++i) sum += h[p][i];
        }
    }
    // the modulation vectors are requested before the reductions, whose barriers no load may cross
    // (without them the compiler places these loads itself)
    uint4 graw[NP], braw[NP];
#pragma unroll
    for (int p = 0; p < NP; ++p) {
        const int col = cbase + (p * 64 + lane) * 8;
        graw[p] = braw[p] = make_uint4(0, 0, 0, 0);
        if (SPLIT && (FULL || col < dim)) {
            graw[p] = *reinterpret_cast<const uint4*>(gs + col);
            braw[p] = *reinterpret_cast<const uint4*>(bs + col);
        }
    }
    const float mean = div_small_int(row_sum(sum, 0), (float)dim, rdim);
    float sq = 0.0f;  // from here on h holds the deviations from the mean
#pragma unroll
    for (int p = 0; p < NP; ++p) {
        const int col = cbase + (p * 64 + lane) * 8;
        if (FULL || col < dim) {
#pragma unroll
            for (int i = 0; i < 8; ++i) {
                h[p][i] = h[p][i] - mean;
                sq = __builtin_fmaf(h[p][i], h[p][i], sq);
            }
        }
    }
    const float var = div_small_int(row_sum(sq, 1), (float)dim, rdim);
    const float rstd = 1.0f / __builtin_sqrtf(var + eps);
    // normalise, modulate, round to T; for the int8 modes apply the smoothing vector and collect the row amax
    float amax = 0.0f;
#pragma unroll
    for (int p = 0; p < NP; ++p) {
        const int col = cbase + (p * 64 + lane) * 8;
        if (FULL || col < dim) {
            float g[8], b[8];
            if constexpr (!SPLIT) {
                graw[p] = *reinterpret_cast<const uint4*>(gs + col);
                braw[p] = *reinterpret_cast<const uint4*>(bs + col);
            }
            unpack8<Tag>(graw[p], g);
            unpack8<Tag>(braw[p], b);
#pragma unroll
            for (int i = 0; i < 8; i += 2) {
                float n0 = h[p][i] * rstd, n1 = h[p][i + 1] * rstd;
                float y0, y1;
                if constexpr (MOD) {
                    float a0 = g[i] + 1.0f, a1 = g[i + 1] + 1.0f;
                    round_through2<Tag>(a0, a1);
                    round_through2<Tag>(n0, n1);
                    y0 = a0 * n0, y1 = a1 * n1;
                    round_through2<Tag>(y0, y1);
                    y0 = y0 + b[i], y1 = y1 + b[i + 1];
                } else {
                    y0 = g[i] * n0 + b[i], y1 = g[i + 1] * n1 + b[i + 1];
                }
                round_through2<Tag>(y0, y1);
                h[p][i] = y0;
                h[p][i + 1] = y1;
            }
            if constexpr (QMODE < 2) {
                if (pre != nullptr) {
                    float4 a = *reinterpret_cast<const float4*>(pre + col);
                    float4 c = *reinterpret_cast<const float4*>(pre + col + 4);
                    const float pv[8] = {a.x, a.y, a.z, a.w, c.x, c.y, c.z, c.w};
#pragma unroll
                    for (int i = 0; i < 8; ++i) h[p][i] = h[p][i] * pv[i];
                }
                if constexpr (QMODE == 1) {
#pragma unroll
                    for (int i = 0; i < 8; ++i) amax = fmaxf(amax, fabsf(h[p][i]));
                }
            }
        }
    }
    float s = 1.0f;
    if constexpr (QMODE == 1) {
        amax = row_max(amax, 2);
        s = amax / 127.0f;
        if (amax <= 5.9604644775390625e-08f) s = 1.0f;
        if (threadIdx.x == (SPLIT ? 0 : wave * 64)) scale_out[row] = s;
    } else if constexpr (QMODE != 3) {
        s = in_scale[0];
    }
    if constexpr (QMODE == 3) {
#pragma unroll
        for (int p = 0; p < NP; ++p) {
            const int col = cbase + (p * 64 + lane) * 8;
            if (FULL || col < dim) {
                uint4 o;
                u32* ow = reinterpret_cast<u32*>(&o);
#pragma unroll
                for (int i = 0; i < 4; ++i) ow[i] = Elem<Tag>::store(h[p][2 * i]) | (Elem<Tag>::store(h[p][2 * i + 1]) << 16);
                *reinterpret_cast<uint4*>(reinterpret_cast<unsigned short*>(dst) + row_off + col) = o;
            }
        }
    } else if constexpr (QMODE == 2) {
        // one set of codes per consumer of the normalised tensor (each linear has its own calibrated input scale)
        const int nout = dst_b != nullptr ? 2 : 1;
        for (int o2 = 0; o2 < nout; ++o2) {
        uint8_t* const out = o2 ? dst_b : dst;
        const float inv = 1.0f / (o2 ? in_scale_b[0] : s);
#pragma unroll
        for (int p = 0; p < NP; ++p) {
            const int col = cbase + (p * 64 + lane) * 8;
            if (FULL || col < dim) {
                float v[8];
                float nanp = 0.0f;
#pragma unroll
                for (int i = 0; i < 8; ++i) {
                    v[i] = h[p][i] * inv;
                    nanp = __builtin_fmaf(v[i], 0.0f, nanp);
                }
                uint2 o;
                o.x = ln_cvt4_e4m3(v[0], v[1], v[2], v[3]);
                o.y = ln_cvt4_e4m3(v[4], v[5], v[6], v[7]);
                if (__builtin_expect(!(nanp == 0.0f), 0)) {  // some value is NaN or infinite
                    o.x = ln_nan_fix(o.x, v);
                    o.y = ln_nan_fix(o.y, v + 4);
                }
                st8<STREAM>(out + (codes_panel ? ((size_t)(col >> 6) * rows + row) * 64 + (col & 63) : row_off + col), o);
            }
        }
        }
    } else {
        const float r = fast_recip(s);
        const bool slow = scale_out_of_range(s);
#pragma unroll
        for (int p = 0; p < NP; ++p) {
            const int col = cbase + (p * 64 + lane) * 8;
            if (FULL || col < dim) {
                uint2 o;
                if constexpr (QMODE == 1) o = quant8_pack_unclamped(h[p], s, r, slow);
                else {
                    int q[8];
                    quant8<-128, 127>(h[p], s, r, slow, q);
                    o.x = pack4_s8(q[0], q[1], q[2], q[3]);
                    o.y = pack4_s8(q[4], q[5], q[6], q[7]);
                }
                st8<STREAM>(dst + row_off + col, o);
            }
        }
    }
}

struct LnArgs {
    uint8_t* dst; void* dst2; float* scale_out; const void* src; const void* residual; const void* bias;
    const void* gamma; const void* beta; const float* pre; const float* in_scale; uint8_t* dst_b; const float* in_scale_b;
    size_t rows; int dim; size_t rows_per_batch; float eps; int codes_panel;
};

template <typename Tag, int QMODE, int RESID, bool MOD> static int launch_ln(const LnArgs& a, hipStream_t st) {
    const int np = (a.dim + 511) / 512;
    if (np > 3) {
        LQ_REQUIRE(a.rows <= 0x7fffffffu, LQ_ERR_SHAPE, "layernorm: %zu rows exceed the launch limit", a.rows);
        dim3 grid((unsigned)a.rows), block(64 * ((np + 1) / 2));
        // a large activation is read once and its codes written once: streaming accesses (see ld16 / st8)
        const bool stream_io = QMODE != 3 && a.rows * (size_t)a.dim * 2 >= kStreamQuantBytes;
        if (a.dim % 1024 == 0 && stream_io)
            hipLaunchKernelGGL((ln_quant_rows_kernel<Tag, 2, QMODE, RESID, MOD, true, true, true>), grid, block, 0, st, a.dst, a.dst2, a.scale_out,
                               a.src, a.residual, a.bias, a.gamma, a.beta, a.pre, a.in_scale, a.dst_b, a.in_scale_b, a.rows, a.dim, a.rows_per_batch, a.eps, 1.0f / (float)a.dim, a.codes_panel);
        else if (a.dim % 1024 == 0)
            hipLaunchKernelGGL((ln_quant_rows_kernel<Tag, 2, QMODE, RESID, MOD, true, true>), grid, block, 0, st, a.dst, a.dst2, a.scale_out,
                               a.src, a.residual, a.bias, a.gamma, a.beta, a.pre, a.in_scale, a.dst_b, a.in_scale_b, a.rows, a.dim, a.rows_per_batch, a.eps, 1.0f / (float)a.dim, a.codes_panel);
        else
            hipLaunchKernelGGL((ln_quant_rows_kernel<Tag, 2, QMODE, RESID, MOD, true, false>), grid, block, 0, st, a.dst, a.dst2, a.scale_out,
                               a.src, a.residual, a.bias, a.gamma, a.beta, a.pre, a.in_scale, a.dst_b, a.in_scale_b, a.rows, a.dim, a.rows_per_batch, a.eps, 1.0f / (float)a.dim, a.codes_panel);
        return check_launch("layernorm_quant");
    }
    dim3 grid((unsigned)((a.rows + 3) / 4)), block(256);
#define LQ_LN_CASE(NPV)                                                                                              \
    hipLaunchKernelGGL((ln_quant_rows_kernel<Tag, NPV, QMODE, RESID, MOD, false>), grid, block, 0, st, a.dst, a.dst2, a.scale_out, \
                       a.src, a.residual, a.bias, a.gamma, a.beta, a.pre, a.in_scale, a.dst_b, a.in_scale_b, a.rows, a.dim, a.rows_per_batch, a.eps, 1.0f / (float)a.dim, a.codes_panel)
    if (np <= 1) LQ_LN_CASE(1);
    else if (np <= 2) LQ_LN_CASE(2);
    else LQ_LN_CASE(3);
#undef LQ_LN_CASE
    return check_launch("layernorm_quant");
}

static int check_ln_common(const char* what, const void* dst, const void* src, lq_dtype_t dtype, size_t rows, size_t dim) {
    LQ_REQUIRE((dst && src) || rows == 0, LQ_ERR_ARG, "%s: null pointer", what);
    LQ_REQUIRE(dtype == LQ_F16 || dtype == LQ_BF16, LQ_ERR_UNSUPPORTED, "%s: activations must be F16 or BF16", what);
    LQ_REQUIRE(dim > 0 && dim % 8 == 0 && dim <= 6144, LQ_ERR_SHAPE, "%s: need dim %% 8 == 0 and dim <= 6144 (dim=%zu)", what, dim);
    LQ_REQUIRE(reinterpret_cast<uintptr_t>(dst) % 8 == 0 && reinterpret_cast<uintptr_t>(src) % 16 == 0, LQ_ERR_ARG,
               "%s: src must be 16-byte and dst 8-byte aligned", what);
    return LQ_OK;
}

}  // namespace lq

using namespace lq;

extern "C" int lq_layernorm_int8(int8_t* dst, float* scale_out, void* dst2, const void* src, const void* residual,
                                 const void* bias, const void* gamma, const void* beta, lq_dtype_t dtype,
                                 const float* pre_quant_scale, const float* input_quant_scale, size_t rows, size_t dim,
                                 float eps, lq_stream_t stream) {
    int rc = check_ln_common("lq_layernorm_int8", dst, src, dtype, rows, dim);
    if (rc != LQ_OK) return rc;
    LQ_REQUIRE(gamma && beta, LQ_ERR_ARG, "lq_layernorm_int8: gamma and beta are required");
    LQ_REQUIRE((scale_out != nullptr) != (input_quant_scale != nullptr), LQ_ERR_ARG,
               "lq_layernorm_int8: pass input_quant_scale (static) or scale_out (dynamic per token), not both");
    LQ_REQUIRE(residual != nullptr || bias == nullptr, LQ_ERR_ARG, "lq_layernorm_int8: bias is only added together with a residual");
    LQ_REQUIRE(residual == nullptr || dst2 != nullptr, LQ_ERR_ARG, "lq_layernorm_int8: dst2 is required with a residual");
    LQ_REQUIRE(reinterpret_cast<uintptr_t>(residual) % 16 == 0 && reinterpret_cast<uintptr_t>(dst2) % 16 == 0 &&
                   reinterpret_cast<uintptr_t>(bias) % 16 == 0 && reinterpret_cast<uintptr_t>(gamma) % 16 == 0 &&
                   reinterpret_cast<uintptr_t>(beta) % 16 == 0 && reinterpret_cast<uintptr_t>(pre_quant_scale) % 16 == 0,
               LQ_ERR_ARG, "lq_layernorm_int8: vectors must be 16-byte aligned");
    if (rows == 0) return LQ_OK;
    LnArgs a = {reinterpret_cast<uint8_t*>(dst), dst2, scale_out, src, residual, bias, gamma, beta, pre_quant_scale,
                input_quant_scale, nullptr, nullptr, rows, (int)dim, 1, eps, 0};
    hipStream_t st = as_stream(stream);
    const bool dyn = scale_out != nullptr, res = residual != nullptr, f16 = dtype == LQ_F16;
#define LQ_LN_GO(Tag)                                                                                   \
    (dyn ? (res ? launch_ln<Tag, 1, 1, false>(a, st) : launch_ln<Tag, 1, 0, false>(a, st))       \
         : (res ? launch_ln<Tag, 0, 1, false>(a, st) : launch_ln<Tag, 0, 0, false>(a, st)))
    return f16 ? LQ_LN_GO(F16Tag) : LQ_LN_GO(BF16Tag);
#undef LQ_LN_GO
}

static int lq_layernorm_mod_fp8_impl(uint8_t* dst, const void* src, const void* scale, const void* shift, lq_dtype_t dtype,
                                    const float* input_scale, size_t batch, size_t rows_per_batch, size_t dim, float eps,
                                    lq_stream_t stream, int panels) {
    int rc = check_ln_common("lq_layernorm_mod_fp8", dst, src, dtype, batch * rows_per_batch, dim);
    if (rc != LQ_OK) return rc;
    LQ_REQUIRE(scale && shift && input_scale, LQ_ERR_ARG, "lq_layernorm_mod_fp8: scale, shift and input_scale are required");
    LQ_REQUIRE(reinterpret_cast<uintptr_t>(scale) % 16 == 0 && reinterpret_cast<uintptr_t>(shift) % 16 == 0, LQ_ERR_ARG,
               "lq_layernorm_mod_fp8: scale and shift must be 16-byte aligned");
    if (batch * rows_per_batch == 0) return LQ_OK;
    LQ_REQUIRE(!panels || dim % 64 == 0, LQ_ERR_SHAPE, "layernorm: codes in k-panels need dim %% 64 == 0 (dim=%zu)", dim);
    LnArgs a = {dst, nullptr, nullptr, src, nullptr, nullptr, scale, shift, nullptr, input_scale, nullptr, nullptr,
                batch * rows_per_batch, (int)dim, rows_per_batch, eps, panels};
    hipStream_t st = as_stream(stream);
    return dtype == LQ_F16 ? launch_ln<F16Tag, 2, 0, true>(a, st) : launch_ln<BF16Tag, 2, 0, true>(a, st);
}

extern "C" int lq_layernorm_mod_fp8(uint8_t* dst, const void* src, const void* scale, const void* shift, lq_dtype_t dtype,
                                    const float* input_scale, size_t batch, size_t rows_per_batch, size_t dim, float eps,
                                    lq_stream_t stream) {
    return lq_layernorm_mod_fp8_impl(dst, src, scale, shift, dtype, input_scale, batch, rows_per_batch, dim, eps, stream, 0);
}

extern "C" int lq_layernorm_mod_fp8_panels(uint8_t* dst, const void* src, const void* scale, const void* shift, lq_dtype_t dtype,
                                    const float* input_scale, size_t batch, size_t rows_per_batch, size_t dim, float eps,
                                    lq_stream_t stream) {
    return lq_layernorm_mod_fp8_impl(dst, src, scale, shift, dtype, input_scale, batch, rows_per_batch, dim, eps, stream, 1);
}

static int lq_layernorm_mod_fp8_dual_impl(uint8_t* dst_a, const float* input_scale_a, uint8_t* dst_b, const float* input_scale_b,
                                         const void* src, const void* scale, const void* shift, lq_dtype_t dtype, size_t batch,
                                         size_t rows_per_batch, size_t dim, float eps, lq_stream_t stream, int panels) {
    int rc = check_ln_common("lq_layernorm_mod_fp8_dual", dst_a, src, dtype, batch * rows_per_batch, dim);
    if (rc != LQ_OK) return rc;
    if (batch * rows_per_batch == 0) return LQ_OK;
    LQ_REQUIRE(dst_b && scale && shift && input_scale_a && input_scale_b, LQ_ERR_ARG, "lq_layernorm_mod_fp8_dual: null pointer");
    LQ_REQUIRE(reinterpret_cast<uintptr_t>(scale) % 16 == 0 && reinterpret_cast<uintptr_t>(shift) % 16 == 0 &&
                   reinterpret_cast<uintptr_t>(dst_b) % 8 == 0,
               LQ_ERR_ARG, "lq_layernorm_mod_fp8_dual: scale and shift must be 16-byte, dst_b 8-byte aligned");
    if (batch * rows_per_batch == 0) return LQ_OK;
    LQ_REQUIRE(!panels || dim % 64 == 0, LQ_ERR_SHAPE, "layernorm: codes in k-panels need dim %% 64 == 0 (dim=%zu)", dim);
    LnArgs a = {dst_a, nullptr, nullptr, src, nullptr, nullptr, scale, shift, nullptr, input_scale_a, dst_b, input_scale_b,
                batch * rows_per_batch, (int)dim, rows_per_batch, eps, panels};
    hipStream_t st = as_stream(stream);
    return dtype == LQ_F16 ? launch_ln<F16Tag, 2, 0, true>(a, st) : launch_ln<BF16Tag, 2, 0, true>(a, st);
}

extern "C" int lq_layernorm_mod_fp8_dual(uint8_t* dst_a, const float* input_scale_a, uint8_t* dst_b, const float* input_scale_b,
                                         const void* src, const void* scale, const void* shift, lq_dtype_t dtype, size_t batch,
                                         size_t rows_per_batch, size_t dim, float eps, lq_stream_t stream) {
    return lq_layernorm_mod_fp8_dual_impl(dst_a, input_scale_a, dst_b, input_scale_b, src, scale, shift, dtype, batch, rows_per_batch, dim, eps, stream, 0);
}

extern "C" int lq_layernorm_mod_fp8_dual_panels(uint8_t* dst_a, const float* input_scale_a, uint8_t* dst_b, const float* input_scale_b,
                                         const void* src, const void* scale, const void* shift, lq_dtype_t dtype, size_t batch,
                                         size_t rows_per_batch, size_t dim, float eps, lq_stream_t stream) {
    return lq_layernorm_mod_fp8_dual_impl(dst_a, input_scale_a, dst_b, input_scale_b, src, scale, shift, dtype, batch, rows_per_batch, dim, eps, stream, 1);
}

extern "C" int lq_gate_residual_layernorm_mod(void* dst, void* hidden_out, const void* attn, const void* gate, const void* input,
                                             const void* scale, const void* shift, lq_dtype_t dtype, size_t batch,
                                             size_t rows_per_batch, size_t dim, float eps, lq_stream_t stream) {
    const bool gated = attn != nullptr;
    int rc = check_ln_common("lq_gate_residual_layernorm_mod", dst, input, dtype, batch * rows_per_batch, dim);
    if (rc != LQ_OK) return rc;
    if (batch * rows_per_batch == 0) return LQ_OK;
    LQ_REQUIRE(scale && shift, LQ_ERR_ARG, "lq_gate_residual_layernorm_mod: scale and shift are required");
    LQ_REQUIRE(gated == (gate != nullptr) && gated == (hidden_out != nullptr), LQ_ERR_ARG,
               "lq_gate_residual_layernorm_mod: attn, gate and hidden_out go together");
    LQ_REQUIRE(reinterpret_cast<uintptr_t>(scale) % 16 == 0 && reinterpret_cast<uintptr_t>(shift) % 16 == 0 &&
                   reinterpret_cast<uintptr_t>(gate) % 16 == 0 && reinterpret_cast<uintptr_t>(attn) % 16 == 0 &&
                   reinterpret_cast<uintptr_t>(hidden_out) % 16 == 0 && reinterpret_cast<uintptr_t>(dst) % 16 == 0,
               LQ_ERR_ARG, "lq_gate_residual_layernorm_mod: all tensors must be 16-byte aligned");
    if (batch * rows_per_batch == 0) return LQ_OK;
    hipStream_t st = as_stream(stream);
    if (gated) {
        LnArgs a = {static_cast<uint8_t*>(dst), hidden_out, nullptr, attn, input, gate, scale, shift, nullptr, nullptr, nullptr, nullptr,
                    batch * rows_per_batch, (int)dim, rows_per_batch, eps, 0};
        return dtype == LQ_F16 ? launch_ln<F16Tag, 3, 2, true>(a, st) : launch_ln<BF16Tag, 3, 2, true>(a, st);
    }
    LnArgs a = {static_cast<uint8_t*>(dst), nullptr, nullptr, input, nullptr, nullptr, scale, shift, nullptr, nullptr, nullptr, nullptr,
                batch * rows_per_batch, (int)dim, rows_per_batch, eps, 0};
    return dtype == LQ_F16 ? launch_ln<F16Tag, 3, 0, true>(a, st) : launch_ln<BF16Tag, 3, 0, true>(a, st);
}

static int lq_gate_residual_layernorm_mod_fp8_impl(uint8_t* dst, void* hidden_out, const void* attn, const void* gate,
                                                  const void* input, const void* scale, const void* shift, lq_dtype_t dtype,
                                                  const float* input_scale, size_t batch, size_t rows_per_batch, size_t dim,
                                                  float eps, lq_stream_t stream, int panels) {
    int rc = check_ln_common("lq_gate_residual_layernorm_mod_fp8", dst, attn, dtype, batch * rows_per_batch, dim);
    if (rc != LQ_OK) return rc;
    if (batch * rows_per_batch == 0) return LQ_OK;
    LQ_REQUIRE(hidden_out && gate && input && scale && shift && input_scale, LQ_ERR_ARG,
               "lq_gate_residual_layernorm_mod_fp8: null pointer");
    LQ_REQUIRE(reinterpret_cast<uintptr_t>(scale) % 16 == 0 && reinterpret_cast<uintptr_t>(shift) % 16 == 0 &&
                   reinterpret_cast<uintptr_t>(gate) % 16 == 0 && reinterpret_cast<uintptr_t>(input) % 16 == 0 &&
                   reinterpret_cast<uintptr_t>(hidden_out) % 16 == 0,
               LQ_ERR_ARG, "lq_gate_residual_layernorm_mod_fp8: all tensors must be 16-byte aligned");
    if (batch * rows_per_batch == 0) return LQ_OK;
    LQ_REQUIRE(!panels || dim % 64 == 0, LQ_ERR_SHAPE, "layernorm: codes in k-panels need dim %% 64 == 0 (dim=%zu)", dim);
    LnArgs a = {dst, hidden_out, nullptr, attn, input, gate, scale, shift, nullptr, input_scale, nullptr, nullptr,
                batch * rows_per_batch, (int)dim, rows_per_batch, eps, panels};
    hipStream_t st = as_stream(stream);
    return dtype == LQ_F16 ? launch_ln<F16Tag, 2, 2, true>(a, st) : launch_ln<BF16Tag, 2, 2, true>(a, st);
}

extern "C" int lq_gate_residual_layernorm_mod_fp8(uint8_t* dst, void* hidden_out, const void* attn, const void* gate,
                                                  const void* input, const void* scale, const void* shift, lq_dtype_t dtype,
                                                  const float* input_scale, size_t batch, size_t rows_per_batch, size_t dim,
                                                  float eps, lq_stream_t stream) {
    return lq_gate_residual_layernorm_mod_fp8_impl(dst, hidden_out, attn, gate, input, scale, shift, dtype, input_scale, batch, rows_per_batch, dim, eps, stream, 0);
}

extern "C" int lq_gate_residual_layernorm_mod_fp8_panels(uint8_t* dst, void* hidden_out, const void* attn, const void* gate,
                                                  const void* input, const void* scale, const void* shift, lq_dtype_t dtype,
                                                  const float* input_scale, size_t batch, size_t rows_per_batch, size_t dim,
                                                  float eps, lq_stream_t stream) {
    return lq_gate_residual_layernorm_mod_fp8_impl(dst, hidden_out, attn, gate, input, scale, shift, dtype, input_scale, batch, rows_per_batch, dim, eps, stream, 1);
}
