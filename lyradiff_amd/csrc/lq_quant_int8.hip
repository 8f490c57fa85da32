// INT8 SmoothQuant activation / weight quantisation kernels for gfx950.
//
// Row kernels: one 64-lane wavefront owns one row at a time and keeps the whole row in
// registers (NP passes of 64 lanes x 8 elements), so the dynamic per-token variant reads the
// activation from HBM exactly once: 128-bit loads, wavefront max by cross-lane shuffles,
// 64-bit packed int8 stores.  The per-channel smoothing vector is loaded once per wavefront
// and reused for all of its rows when it fits in registers.
//
// Formulas follow the lyraDiff reference: kernels/quant_kernels/quant_kernels.cu:51-115
// (activation), :173-223 (weights), :117-171 (dequant), kernels/quant_kernels/
// ffn_kernels_int8.cu:102-147 (bias + GEGLU), kernels/quant_kernels/int8_utils.cuh:23-28.
#include <atomic>

#include "lq_common.h"
#include <type_traits>

namespace lq {

// Load 8 consecutive elements (element offset `col` inside the row) as floats.
template <typename Tag> __device__ __forceinline__ void load8(const void* row_base, int col, float* o) {
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

// MODE 0: static per-tensor scale, 1: given per-token scale, 2: dynamic per-token scale.
// The smoothing vector (fp32, twice the bytes of an fp16 row) is staged once per workgroup in LDS
// and shared by the rows its four wavefronts quantise.
template <typename Tag, int NP, int MODE, bool HAS_PRE>
__global__ __launch_bounds__(256) void sq_quant_rows_kernel(int8_t* __restrict__ dst,
                                                            float* __restrict__ scale_out,
                                                            const void* __restrict__ src,
                                                            const float* __restrict__ pre,
                                                            const float* __restrict__ in_scale,
                                                            size_t rows, int dim, int rows_per_wave) {
    extern __shared__ __attribute__((aligned(16))) float s_pre[];
    const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
    const size_t row_bytes = (size_t)dim * Elem<Tag>::bytes;
    if constexpr (HAS_PRE) {
        for (int c = threadIdx.x * 4; c < dim; c += 1024)
            *reinterpret_cast<float4*>(s_pre + c) = *reinterpret_cast<const float4*>(pre + c);
        __syncthreads();
    }
    // Raw row data is double buffered in registers: the loads of the wavefront's next row are in
    // flight while the current row is quantised.
    constexpr int VPP = Elem<Tag>::bytes == 2 ? 1 : 2;  // 16-byte vectors per 8 elements
    auto load_raw = [&](size_t row, uint4 (*raw)[VPP]) {
        const char* rb = static_cast<const char*>(src) + row * row_bytes;
#pragma unroll
        for (int p = 0; p < NP; ++p) {
            int col = (p * 64 + lane) * 8;
#pragma unroll
            for (int u = 0; u < VPP; ++u) {
                raw[p][u] = make_uint4(0, 0, 0, 0);
                if (col < dim) raw[p][u] = *reinterpret_cast<const uint4*>(rb + (size_t)col * Elem<Tag>::bytes + u * 16);
            }
        }
    };
    auto unpack_raw = [&](const uint4* r, float* o) {
        if constexpr (Elem<Tag>::bytes == 2) unpack8<Tag>(r[0], o);
        else {
            o[0] = __uint_as_float(r[0].x); o[1] = __uint_as_float(r[0].y); o[2] = __uint_as_float(r[0].z); o[3] = __uint_as_float(r[0].w);
            o[4] = __uint_as_float(r[VPP - 1].x); o[5] = __uint_as_float(r[VPP - 1].y); o[6] = __uint_as_float(r[VPP - 1].z); o[7] = __uint_as_float(r[VPP - 1].w);
        }
    };
    const size_t row0 = (size_t)blockIdx.x * 4 * rows_per_wave + wave;
    uint4 cur[NP][VPP], nxt[NP][VPP];
    if (row0 < rows) load_raw(row0, cur);
    for (int j = 0; j < rows_per_wave; ++j) {
        const size_t row = row0 + 4 * (size_t)j;
        if (row >= rows) break;
        const bool has_next = j + 1 < rows_per_wave && row + 4 < rows;
        if (has_next) load_raw(row + 4, nxt);
        float t[NP][8];
        float amax = 0.0f;
#pragma unroll
        for (int p = 0; p < NP; ++p) {
            int col = (p * 64 + lane) * 8;
            if constexpr (HAS_PRE) {
                // (a lane outside the row holds zeros and multiplies them by whatever LDS holds at a clamped offset)
                const int pc = col < dim ? col : 0;
                float4 a = *reinterpret_cast<const float4*>(s_pre + pc);
                float4 b = *reinterpret_cast<const float4*>(s_pre + pc + 4);
                const float pv[8] = {a.x, a.y, a.z, a.w, b.x, b.y, b.z, b.w};
                if constexpr (std::is_same<Tag, F16Tag>::value) mul8_f16(cur[p][0], pv, t[p]);
                else {
                    unpack_raw(cur[p], t[p]);
#pragma unroll
                    for (int i = 0; i < 8; ++i) t[p][i] = t[p][i] * pv[i];
                }
            } else {
                unpack_raw(cur[p], t[p]);
            }
            if constexpr (MODE == 2) {
#pragma unroll
                for (int i = 0; i < 8; ++i) amax = fmaxf(amax, fabsf(t[p][i]));
            }
        }
        float s;
        if constexpr (MODE == 2) {
            amax = wave_max(amax);
            s = div_by_const_fast(amax, 127.0f, 0x1.020408p-7f);
            if (scale_out_of_range(s)) s = amax / 127.0f;
            if (amax <= 5.9604644775390625e-08f) s = 1.0f;
            if (lane == 0) scale_out[row] = s;
        } else if constexpr (MODE == 1) {
            s = in_scale[row];
        } else {
            s = in_scale[0];
        }
        const float r = fast_recip(s);
        const bool slow = scale_out_of_range(s);
        int8_t* ob = dst + row * (size_t)dim;
#pragma unroll
        for (int p = 0; p < NP; ++p) {
            int col = (p * 64 + lane) * 8;
            if (col < dim) {
                uint2 o;
                if constexpr (MODE == 2) o = quant8_pack_unclamped(t[p], s, r, slow);
                else {
                    int q[8];
                    quant8<-128, 127>(t[p], s, r, slow, q);
                    o.x = pack4_s8(q[0], q[1], q[2], q[3]);
                    o.y = pack4_s8(q[4], q[5], q[6], q[7]);
                }
                *reinterpret_cast<uint2*>(ob + col) = o;
            }
        }
        if (has_next) {
#pragma unroll
            for (int p = 0; p < NP; ++p)
#pragma unroll
                for (int u = 0; u < VPP; ++u) cur[p][u] = nxt[p][u];
        }
    }
}

// Rows longer than 1536 columns: the row is cut into 1024-column spans, one wavefront each, and a
// workgroup of dim/1024 wavefronts (rounded up) owns one row.  A wavefront then needs at most 64
// registers whatever the row length, so eight of them share a SIMD and the loads of one overlap the
// arithmetic of the others; the dynamic variant exchanges the span maxima through LDS (one barrier).
// A lane outside the row re-reads a valid octet (harmless for the maximum) and stores nothing.
// PANEL: the codes are written as k-panels [dim / 64][rows][64] (byte ((c / 64) * rows + row) * 64 + c % 64) for
// lq_gemm_int8_panels instead of row-major: a lane's eight codes stay inside one 64-byte segment, eight lanes fill it, and
// with two rows per workgroup the two segments of a 128-byte line are written by the same wavefront.
template <typename Tag, int MODE, bool HAS_PRE, int R, bool STREAM = false, bool PANEL = false>
__global__ __launch_bounds__(1024) void sq_quant_split_kernel(int8_t* __restrict__ dst, float* __restrict__ scale_out,
                                                              const void* __restrict__ src,
                                                              const float* __restrict__ pre,
                                                              const float* __restrict__ in_scale, size_t rows, int dim) {
    // R rows per workgroup (1 or 2): with two, a wavefront's share of the smoothing vector -- twice the bytes of its share
    // of an fp16 row -- is loaded once for both rows.
    __shared__ __attribute__((aligned(16))) float red[R][16];
    const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
    const size_t row0 = (size_t)blockIdx.x * R;
    if constexpr (MODE == 2) {
        if (threadIdx.x < 16 * R) red[threadIdx.x / 16][threadIdx.x % 16] = 0.0f;
        __syncthreads();
    }
    constexpr bool kMix = HAS_PRE && std::is_same<Tag, F16Tag>::value;  // fp16 * fp32 in one instruction
    int col[2];
    bool valid[2];
    bool live[R];
    float t[R][2][8];
    uint4 raw[R][2];
    float amax[R];
#pragma unroll
    for (int rr = 0; rr < R; ++rr) {
        live[rr] = row0 + rr < rows;  // the last workgroup of an odd row count repeats its first row (stores masked)
        const char* rb = static_cast<const char*>(src) + (live[rr] ? row0 + rr : row0) * (size_t)dim * Elem<Tag>::bytes;
        amax[rr] = 0.0f;
#pragma unroll
        for (int p = 0; p < 2; ++p) {
            const int c = wave * 1024 + p * 512 + lane * 8;
            valid[p] = c < dim;
            col[p] = valid[p] ? c : 0;
            if constexpr (kMix) raw[rr][p] = ld16<STREAM>(rb + (size_t)col[p] * 2);
            else if constexpr (Elem<Tag>::bytes == 2) unpack8<Tag>(ld16<STREAM>(rb + (size_t)col[p] * 2), t[rr][p]);
            else load8<Tag>(rb, col[p], t[rr][p]);
        }
    }
#pragma unroll
    for (int p = 0; p < 2; ++p) {
        float pv[8];
        if constexpr (HAS_PRE) load8<F32Tag>(pre, col[p], pv);
#pragma unroll
        for (int rr = 0; rr < R; ++rr) {
            if constexpr (HAS_PRE) {
                if constexpr (kMix) mul8_f16(raw[rr][p], pv, t[rr][p]);
                else {
#pragma unroll
                    for (int i = 0; i < 8; ++i) t[rr][p][i] = t[rr][p][i] * pv[i];
                }
            }
            if constexpr (MODE == 2) {
#pragma unroll
                for (int i = 0; i < 8; ++i) amax[rr] = fmaxf(amax[rr], fabsf(t[rr][p][i]));
            }
        }
    }
    float s[R];
    if constexpr (MODE == 2) {
#pragma unroll
        for (int rr = 0; rr < R; ++rr) {
            amax[rr] = wave_max(amax[rr]);
            if (lane == 0) red[rr][wave] = amax[rr];
        }
        __syncthreads();
#pragma unroll
        for (int rr = 0; rr < R; ++rr) {
            const float4 a = *reinterpret_cast<const float4*>(red[rr]);
            float m = fmaxf(fmaxf(a.x, a.y), fmaxf(a.z, a.w));
            if (blockDim.x > 256) {  // more than four wavefronts (the same for the whole workgroup)
                const float4 b = *reinterpret_cast<const float4*>(red[rr] + 4), c = *reinterpret_cast<const float4*>(red[rr] + 8);
                const float4 d = *reinterpret_cast<const float4*>(red[rr] + 12);
                m = fmaxf(fmaxf(m, fmaxf(fmaxf(b.x, b.y), fmaxf(b.z, b.w))),
                          fmaxf(fmaxf(fmaxf(c.x, c.y), fmaxf(c.z, c.w)), fmaxf(fmaxf(d.x, d.y), fmaxf(d.z, d.w))));
            }
            s[rr] = div_by_const_fast(m, 127.0f, 0x1.020408p-7f);
            if (scale_out_of_range(s[rr])) s[rr] = m / 127.0f;
            if (m <= 5.9604644775390625e-08f) s[rr] = 1.0f;
            if (threadIdx.x == 0 && live[rr]) scale_out[row0 + rr] = s[rr];
        }
    } else {
#pragma unroll
        for (int rr = 0; rr < R; ++rr) s[rr] = MODE == 1 ? in_scale[live[rr] ? row0 + rr : row0] : in_scale[0];
    }
#pragma unroll
    for (int rr = 0; rr < R; ++rr) {
        const float r = fast_recip(s[rr]);
        const bool slow = scale_out_of_range(s[rr]);
        int8_t* ob = dst + (row0 + rr) * (size_t)dim;
#pragma unroll
        for (int p = 0; p < 2; ++p) {
            uint2 o;
            if constexpr (MODE == 2) o = quant8_pack_unclamped(t[rr][p], s[rr], r, slow);
            else {
                int q[8];
                quant8<-128, 127>(t[rr][p], s[rr], r, slow, q);
                o.x = pack4_s8(q[0], q[1], q[2], q[3]);
                o.y = pack4_s8(q[4], q[5], q[6], q[7]);
            }
            if constexpr (PANEL) {
                if (valid[p] && live[rr])
                    st8<STREAM>(dst + ((size_t)(col[p] >> 6) * rows + (row0 + rr)) * 64 + (col[p] & 63), o);
            } else {
                if (valid[p] && live[rr]) st8<STREAM>(ob + col[p], o);
            }
        }
    }
}

// Generic (any dim, any alignment) fallback: one workgroup per row, scalar accesses.
template <typename Tag, int MODE>
__global__ __launch_bounds__(256) void sq_quant_generic_kernel(int8_t* __restrict__ dst, float* __restrict__ scale_out,
                                                               const void* __restrict__ src,
                                                               const float* __restrict__ pre,
                                                               const float* __restrict__ in_scale, size_t rows,
                                                               size_t dim) {
    __shared__ float red[4];
    for (size_t row = blockIdx.x; row < rows; row += gridDim.x) {
        const char* rb = static_cast<const char*>(src) + row * dim * Elem<Tag>::bytes;
        auto ld = [&](size_t c) -> float {
            u32 bits;
            if constexpr (Elem<Tag>::bytes == 2) bits = reinterpret_cast<const unsigned short*>(rb)[c];
            else bits = reinterpret_cast<const u32*>(rb)[c];
            float v = Elem<Tag>::load(bits);
            return pre ? v * pre[c] : v;
        };
        float s;
        if constexpr (MODE == 2) {
            float amax = 0.0f;
            for (size_t c = threadIdx.x; c < dim; c += blockDim.x) amax = fmaxf(amax, fabsf(ld(c)));
            amax = wave_max(amax);
            __syncthreads();
            if ((threadIdx.x & 63) == 0) red[threadIdx.x >> 6] = amax;
            __syncthreads();
            amax = fmaxf(fmaxf(red[0], red[1]), fmaxf(red[2], red[3]));
            s = (amax <= 5.9604644775390625e-08f) ? 1.0f : amax / 127.0f;
            if (threadIdx.x == 0) scale_out[row] = s;
        } else if constexpr (MODE == 1) {
            s = in_scale[row];
        } else {
            s = in_scale[0];
        }
        for (size_t c = threadIdx.x; c < dim; c += blockDim.x) dst[row * dim + c] = (int8_t)rne_sat_s8(ld(c) / s);
    }
}

template <typename Tag, int MODE>
static int launch_sq_quant(int8_t* dst, float* scale_out, const void* src, const float* pre, const float* in_scale,
                           size_t rows, size_t dim, hipStream_t st) {
    const bool fast = (dim % 8 == 0) && dim <= 16384 && (reinterpret_cast<uintptr_t>(src) % 16 == 0) &&
                      (reinterpret_cast<uintptr_t>(dst) % 8 == 0) &&
                      (pre == nullptr || reinterpret_cast<uintptr_t>(pre) % 16 == 0);
    if (!fast) {
        unsigned grid = (unsigned)(rows < 65536 ? rows : 65536);
        hipLaunchKernelGGL((sq_quant_generic_kernel<Tag, MODE>), dim3(grid), dim3(256), 0, st, dst, scale_out, src, pre,
                           in_scale, rows, dim);
        return check_launch("sq_quant_generic");
    }
    const int np = (int)((dim + 511) / 512);
    int d = (int)dim;
    if (np > 3) {
        // one wavefront per 1024 columns, one workgroup per row
        LQ_REQUIRE(rows <= 0x7fffffffu, LQ_ERR_SHAPE, "sq_quant: %zu rows exceed the launch limit", rows);
        dim3 block(64 * ((np + 1) / 2));
        const bool stream_io = rows * dim * Elem<Tag>::bytes >= kStreamQuantBytes;  // read-once input, write-once codes
        if (pre && dim >= 2048) {  // long rows with a smoothing vector: two rows per workgroup share its loads
            dim3 grid((unsigned)((rows + 1) / 2));
            if (stream_io) hipLaunchKernelGGL((sq_quant_split_kernel<Tag, MODE, true, 2, true>), grid, block, 0, st, dst, scale_out, src, pre, in_scale, rows, d);
            else hipLaunchKernelGGL((sq_quant_split_kernel<Tag, MODE, true, 2>), grid, block, 0, st, dst, scale_out, src, pre, in_scale, rows, d);
        } else {
            dim3 grid((unsigned)rows);
            if (pre) hipLaunchKernelGGL((sq_quant_split_kernel<Tag, MODE, true, 1>), grid, block, 0, st, dst, scale_out, src, pre, in_scale, rows, d);
            else if (stream_io) hipLaunchKernelGGL((sq_quant_split_kernel<Tag, MODE, false, 1, true>), grid, block, 0, st, dst, scale_out, src, pre, in_scale, rows, d);
            else hipLaunchKernelGGL((sq_quant_split_kernel<Tag, MODE, false, 1>), grid, block, 0, st, dst, scale_out, src, pre, in_scale, rows, d);
        }
        return check_launch("sq_quant_split");
    }
    // four rows per workgroup pass; more rows per wavefront only when there are plenty of rows
    int rpw = (int)(rows / (4 * 768));
    rpw = rpw < 1 ? 1 : (rpw > 8 ? 8 : rpw);
    const size_t blocks = (rows + 4 * (size_t)rpw - 1) / (4 * (size_t)rpw);
    dim3 grid((unsigned)blocks), block(256);
    const size_t lds = pre ? dim * sizeof(float) : 0;
#define LQ_SQ_CASE(NPV)                                                                                             \
    do {                                                                                                            \
        if (pre) hipLaunchKernelGGL((sq_quant_rows_kernel<Tag, NPV, MODE, true>), grid, block, lds, st, dst, scale_out, src, pre, in_scale, rows, d, rpw); \
        else hipLaunchKernelGGL((sq_quant_rows_kernel<Tag, NPV, MODE, false>), grid, block, 0, st, dst, scale_out, src, pre, in_scale, rows, d, rpw);      \
    } while (0)
    if (np <= 1) LQ_SQ_CASE(1);
    else if (np <= 2) LQ_SQ_CASE(2);
    else LQ_SQ_CASE(3);
#undef LQ_SQ_CASE
    return check_launch("sq_quant_rows");
}

template <int MODE>
static int dispatch_sq_quant(int8_t* dst, float* scale_out, const void* src, lq_dtype_t dt, const float* pre,
                             const float* in_scale, size_t rows, size_t dim, hipStream_t st) {
    switch (dt) {
        case LQ_F16: return launch_sq_quant<F16Tag, MODE>(dst, scale_out, src, pre, in_scale, rows, dim, st);
        case LQ_BF16: return launch_sq_quant<BF16Tag, MODE>(dst, scale_out, src, pre, in_scale, rows, dim, st);
        case LQ_F32: return launch_sq_quant<F32Tag, MODE>(dst, scale_out, src, pre, in_scale, rows, dim, st);
        default: set_error("sq_quant: unsupported source dtype %d", (int)dt); return LQ_ERR_UNSUPPORTED;
    }
}

// ---- unfused dequant (quant_kernels.cu:117-171) -------------------------------------------------
template <typename Tag, bool PER_TOKEN>
__global__ __launch_bounds__(256) void sq_dequant_kernel(void* __restrict__ dst, const int32_t* __restrict__ src,
                                                         const float* __restrict__ in_scale,
                                                         const float* __restrict__ w_scale, size_t rows, size_t dim) {
    size_t total = rows * dim;
    for (size_t i = (size_t)blockIdx.x * blockDim.x + threadIdx.x; i < total; i += (size_t)gridDim.x * blockDim.x) {
        size_t r = i / dim, c = i - r * dim;
        float y = ((float)src[i] * in_scale[PER_TOKEN ? r : 0]) * w_scale[c];
        // pin the fp32 product: otherwise the second multiply and the conversion become one mixed-precision
        // instruction that rounds the exact product straight to fp16 (one rounding instead of the specified two)
        asm volatile("" : "+v"(y));
        u32 b = Elem<Tag>::store(y);
        if constexpr (Elem<Tag>::bytes == 2) static_cast<unsigned short*>(dst)[i] = (unsigned short)b;
        else static_cast<u32*>(dst)[i] = b;
    }
}

// ---- per-output-channel weight quantisation (quant_kernels.cu:173-223) -----------------------------
template <typename Tag>
__global__ __launch_bounds__(256) void int8_weight_quant_kernel(float* __restrict__ scale_out, int8_t* __restrict__ q,
                                                                const void* __restrict__ w,
                                                                const float* __restrict__ pre, size_t d_out,
                                                                size_t d_in) {
    __shared__ float red[4];
    for (size_t row = blockIdx.x; row < d_out; row += gridDim.x) {
        const char* rb = static_cast<const char*>(w) + row * d_in * Elem<Tag>::bytes;
        auto ld = [&](size_t c) -> float {
            u32 bits;
            if constexpr (Elem<Tag>::bytes == 2) bits = reinterpret_cast<const unsigned short*>(rb)[c];
            else bits = reinterpret_cast<const u32*>(rb)[c];
            float v = Elem<Tag>::load(bits);
            return pre ? v / pre[c] : v;
        };
        float amax = 0.0f;
        for (size_t c = threadIdx.x; c < d_in; c += blockDim.x) amax = fmaxf(amax, fabsf(ld(c)));
        amax = wave_max(amax);
        __syncthreads();
        if ((threadIdx.x & 63) == 0) red[threadIdx.x >> 6] = amax;
        __syncthreads();
        amax = fmaxf(fmaxf(red[0], red[1]), fmaxf(red[2], red[3]));
        float s = amax / 127.0f;
        if (threadIdx.x == 0) scale_out[row] = s;
        for (size_t c = threadIdx.x; c < d_in; c += blockDim.x) q[row * d_in + c] = (int8_t)rne_sat_s8(ld(c) / s);
    }
}

// ---- bias + GEGLU -> INT8 (ffn_kernels_int8.cu:102-147) ----------------------------------------------
// The gate factor  gate(g) = T( g * T( 0.5 * (1 + tanh(0.79788 * (g + 0.044715 * T(g * T(g*g))))) ) )  depends only on the
// 16-bit value g, and its evaluation (a tanh built from basic IEEE operations, so that a CPU restatement reproduces it bit
// for bit) is about 70 of the kernel's 85 vector instructions per element.  For fp16 and bf16 inputs the factor is
// therefore tabulated: a small kernel, run once per device (ensure_gate_table), evaluates the formula for each 16-bit pattern with
// 2^-12 <= |g| < 8 (30720 fp16 / 3840 bf16 patterns) into a table in device memory, every workgroup of the main kernel copies
// the table into LDS and looks the factor up.  Outside that range the inner factor T(0.5 * (1 + tanh(...))) is a constant:
// 0.5 for |g| < 2^-12 (the deviation from 0.5 is below half a unit in the last place of T), 1 for g >= 8 and 0 for g <= -8
// (the tanh is +-1 in fp32 there), so gate(g) = T(g * c) with that constant -- the formula's own last step; infinities and
// NaN follow the same expressions.  tests/test_oracle_pins.py checks these three constants against the formula for every
// 16-bit pattern outside the table.  The table's contents never change; concurrent first calls that build it write the same bytes.
template <typename Tag> __device__ __forceinline__ float geglu_gate(float g) {
    const float cube = round_through<Tag>(g * round_through<Tag>(g * g));
    const float cdf = 0.5f * (1.0f + tanh_basic(0.7978845608028654f * (g + 0.044715f * cube)));
    return round_through<Tag>(g * round_through<Tag>(cdf));
}
template <typename Tag> struct GateTable;
template <> struct GateTable<F16Tag> { static constexpr u32 LO = 0x0C00u, COUNT = 0x4800u - 0x0C00u; };   // 2^-12 .. 8
template <> struct GateTable<BF16Tag> { static constexpr u32 LO = 0x3980u, COUNT = 0x4100u - 0x3980u; };
__device__ __attribute__((aligned(16))) unsigned short g_gate_table_f16[2 * GateTable<F16Tag>::COUNT];
__device__ __attribute__((aligned(16))) unsigned short g_gate_table_bf16[2 * GateTable<BF16Tag>::COUNT];
template <typename Tag> __device__ __forceinline__ unsigned short* gate_table() {
    if constexpr (std::is_same<Tag, F16Tag>::value) return g_gate_table_f16;
    else return g_gate_table_bf16;
}
template <typename Tag> __global__ __launch_bounds__(256) void geglu_table_kernel() {
    constexpr u32 COUNT = GateTable<Tag>::COUNT;
    const u32 i = blockIdx.x * 256 + threadIdx.x;
    if (i >= 2 * COUNT) return;
    const u32 bits = (GateTable<Tag>::LO + (i % COUNT)) | (i >= COUNT ? 0x8000u : 0u);
    gate_table<Tag>()[i] = (unsigned short)Elem<Tag>::store(geglu_gate<Tag>(Elem<Tag>::load(bits)));
}

// SW wavefronts per row (1, or 2 for wide rows: half the registers per lane, so twice the wavefronts per SIMD); a
// wavefront's share of the row's `dim` products h*g stays in registers (NP passes of 512 columns).  With SW = 2 the two
// halves of a row meet in LDS for the row maximum; the row loop then has the same trip count in every wavefront of the
// workgroup, because it contains a workgroup barrier.
template <typename Tag, int NP, bool DYNAMIC, int THREADS, int SW>
__global__ __launch_bounds__(THREADS, (SW == 2 && THREADS == 512) ? 4 : 1) void geglu_int8_kernel(int8_t* __restrict__ dst, float* __restrict__ scale_out,
                                                         const void* __restrict__ hidden,
                                                         const void* __restrict__ bias,
                                                         const float* __restrict__ pre,
                                                         const float* __restrict__ in_scale, size_t rows, int dim) {
    constexpr bool TABLE = Elem<Tag>::bytes == 2;
    extern __shared__ __attribute__((aligned(16))) unsigned short s_gate[];
    if constexpr (TABLE) {
        const unsigned short* tab = gate_table<Tag>();
        for (u32 i = threadIdx.x * 8; i < 2 * GateTable<Tag>::COUNT; i += blockDim.x * 8)
            *reinterpret_cast<uint4*>(s_gate + i) = *reinterpret_cast<const uint4*>(tab + i);
        __syncthreads();
    }
    __shared__ float s_half_max[2][THREADS / 64];  // SW = 2: each wavefront's maximum over its half row, by loop parity
    const int lane = threadIdx.x & 63, wave_in_wg = threadIdx.x >> 6;
    const size_t wpb = blockDim.x >> 6;  // wavefronts per workgroup; wpb / SW rows in flight
    const size_t team = ((size_t)blockIdx.x * wpb + wave_in_wg) / SW;  // the wavefronts 2t, 2t+1 of a workgroup share a row
    const size_t nteams = (size_t)gridDim.x * wpb / SW;
    const int cbase = (SW == 2 && (wave_in_wg & 1)) ? NP * 512 : 0;
    const size_t trips = (rows + nteams - 1) / nteams;
    for (size_t trip = 0; trip < trips; ++trip) {
        const size_t row = team + trip * nteams;
        const bool live = row < rows;
        if (SW == 1 && !live) break;
        const char* rb = static_cast<const char*>(hidden) + (live ? row : 0) * (size_t)dim * 2 * Elem<Tag>::bytes;
        float t[NP][8];
        float amax = 0.0f;
#pragma unroll
        for (int p = 0; p < NP; ++p) {
            int col = cbase + (p * 64 + lane) * 8;
            if (col < dim && live) {
                float h[8], g[8], pv[8], gel[8];
                load8<Tag>(rb, col, h);
                load8<Tag>(rb, col + dim, g);
                if (bias != nullptr) {
                    float bh[8], bg[8];
                    load8<Tag>(bias, col, bh);
                    load8<Tag>(bias, col + dim, bg);
#pragma unroll
                    for (int i = 0; i < 8; ++i) {
                        h[i] = round_through<Tag>(h[i] + bh[i]);
                        g[i] = round_through<Tag>(g[i] + bg[i]);
                    }
                }
#pragma unroll
                for (int i = 0; i < 8; ++i) pv[i] = 1.0f;
                if (pre != nullptr) load8<F32Tag>(pre, col, pv);
                if constexpr (TABLE) {
                    constexpr u32 LO = GateTable<Tag>::LO, COUNT = GateTable<Tag>::COUNT;
                    bool in[8], all_in = true;
#pragma unroll
                    for (int i = 0; i < 8; ++i) {
                        const u32 bits = Elem<Tag>::store(g[i]);  // exact: g is a T value
                        const u32 off = (bits & 0x7FFFu) - LO;    // wraps to a huge number below the table
                        in[i] = off < COUNT;
                        all_in = all_in && in[i];
                        gel[i] = Elem<Tag>::load(s_gate[(in[i] ? off : 0u) + ((bits & 0x8000u) ? COUNT : 0u)]);
                    }
                    if (__builtin_expect(!all_in, 0)) {  // rare: outside the table the inner factor is a constant
#pragma unroll
                        for (int i = 0; i < 8; ++i) {
                            const float c = fabsf(g[i]) < 1.0f ? 0.5f : (g[i] < 0.0f ? 0.0f : 1.0f);  // below the table : beyond it
                            if (!in[i]) gel[i] = round_through<Tag>(g[i] * c);
                        }
                    }
                } else {
#pragma unroll
                    for (int i = 0; i < 8; ++i) gel[i] = geglu_gate<Tag>(g[i]);
                }
#pragma unroll
                for (int i = 0; i < 8; ++i) {
                    float prod = round_through<Tag>(h[i] * gel[i]);
                    t[p][i] = prod * pv[i];
                    amax = fmaxf(amax, fabsf(t[p][i]));
                }
            } else {
#pragma unroll
                for (int i = 0; i < 8; ++i) t[p][i] = 0.0f;
            }
        }
        float s;
        if constexpr (DYNAMIC) {
            amax = wave_max(amax);
            if constexpr (SW == 2) {
                if (lane == 0) s_half_max[trip & 1][wave_in_wg] = amax;
                __syncthreads();  // one barrier per trip: the next trip writes the other parity
                amax = fmaxf(amax, s_half_max[trip & 1][wave_in_wg ^ 1]);
            }
            s = (amax <= 5.9604644775390625e-08f) ? 1.0f : amax / 127.0f;
            if (lane == 0 && cbase == 0 && live) scale_out[row] = s;
        } else {
            s = in_scale[0];
        }
        const float r = 1.0f / s;
        const bool slow = recip_unsafe(s, r);
        int8_t* ob = dst + (live ? row : 0) * (size_t)dim;
#pragma unroll
        for (int p = 0; p < NP; ++p) {
            int col = cbase + (p * 64 + lane) * 8;
            if (col < dim && live) {
                int q[8];
                quant8<-128, 127>(t[p], s, r, slow, q);
                uint2 o;
                o.x = pack4_s8(q[0], q[1], q[2], q[3]);
                o.y = pack4_s8(q[4], q[5], q[6], q[7]);
                *reinterpret_cast<uint2*>(ob + col) = o;
            }
        }
    }
}

// The gate table holds constants, so it is built once per device and element type: the first call on a device
// launches the table kernel on the caller's stream and waits for it (the only blocking step of the entry point, once
// per process), after which calls on any stream find it complete.  While the stream is being captured into a graph
// nothing may block: the table kernel then simply becomes part of the graph, and the device stays unmarked.
template <typename Tag> static int ensure_gate_table(hipStream_t st) {
    static std::atomic<unsigned> built{0};  // one bit per device ordinal; devices beyond 31 rebuild on every call
    int dev = 0;
    if (hipGetDevice(&dev) != hipSuccess) dev = 32;
    const unsigned bit = (dev >= 0 && dev < 32) ? 1u << dev : 0u;
    if (bit != 0 && (built.load(std::memory_order_acquire) & bit) != 0) return LQ_OK;
    constexpr unsigned entries = 2 * GateTable<Tag>::COUNT;
    hipLaunchKernelGGL((geglu_table_kernel<Tag>), dim3((entries + 255) / 256), dim3(256), 0, st);
    if (int rc = check_launch("geglu_int8 gate table"); rc != LQ_OK) return rc;
    hipStreamCaptureStatus cs = hipStreamCaptureStatusNone;
    if (hipStreamIsCapturing(st, &cs) != hipSuccess) {
        (void)hipGetLastError();  // e.g. the null stream while another stream captures: treat as capturing
        return LQ_OK;
    }
    if (cs != hipStreamCaptureStatusNone || bit == 0) return LQ_OK;
    if (hipStreamSynchronize(st) != hipSuccess) {
        set_error("geglu_int8: waiting for the gate table failed: %s", hipGetErrorString(hipGetLastError()));
        return LQ_ERR_HIP;
    }
    built.fetch_or(bit, std::memory_order_release);
    return LQ_OK;
}

template <typename Tag, bool DYNAMIC>
static int launch_geglu(int8_t* dst, float* scale_out, const void* hidden, const void* bias, const float* pre,
                        const float* in_scale, size_t rows, size_t dim, hipStream_t st) {
    LQ_REQUIRE(dim % 8 == 0 && dim <= 8192, LQ_ERR_SHAPE, "geglu_int8: dim=%zu must be a multiple of 8 and <= 8192", dim);
    LQ_REQUIRE(reinterpret_cast<uintptr_t>(hidden) % 16 == 0 && reinterpret_cast<uintptr_t>(dst) % 8 == 0 &&
                   (bias == nullptr || reinterpret_cast<uintptr_t>(bias) % 16 == 0) &&
                   (pre == nullptr || reinterpret_cast<uintptr_t>(pre) % 16 == 0),
               LQ_ERR_ARG, "geglu_int8: pointers must be 16-byte aligned");
    const int np_row = (int)((dim + 511) / 512);
    // rows of 2561..5120 columns go to two wavefronts each (the 5120-wide rows of SDXL: 10 passes -> 5, half the registers)
    const int sw = (np_row > 5 && np_row <= 10) ? 2 : 1;
    const int np = (np_row + sw - 1) / sw;
    size_t lds = 0, threads = 256, cap = 65535;
    if constexpr (Elem<Tag>::bytes == 2) {
        // every workgroup stages the gate table once, so the grid is a few workgroups per CU that walk the rows.  The
        // fp16 table (60 KB) allows two workgroups per CU: those have eight wavefronts each.
        constexpr unsigned entries = 2 * GateTable<Tag>::COUNT;
        if (int rc = ensure_gate_table<Tag>(st); rc != LQ_OK) return rc;
        lds = entries * sizeof(unsigned short);
        threads = (lds > 32768 && np <= 10) ? 512 : 256;  // (the 16-pass form needs all 256 registers of a 256-thread workgroup)
        // one 16-wavefront workgroup per CU instead of two of eight halves the table traffic; it pays when every CU gets
        // a full workgroup of whole rows (17.2 against 18.1 us at 4096 x 2560) and costs when rows are few or shared
        if (threads == 512 && sw == 1 && np <= 5 && rows >= 256 * 16) threads = 1024;
        cap = 256 * (lds > 32768 ? (threads == 1024 ? 1 : 2) : 8);
    }
    const size_t rows_per_wg = threads / 64 / sw;
    size_t blocks = (rows + rows_per_wg - 1) / rows_per_wg;
    if (blocks > cap) blocks = cap;
    dim3 grid((unsigned)blocks), block((unsigned)threads);
    int d = (int)dim;
#define LQ_GG_CASE(NPV) \
    do {                \
        if (sw == 2) LQ_GG_GO(NPV, ((NPV == 3 || NPV == 5) ? 2 : 1)); /* split rows need 3..5 passes per wavefront */ \
        else LQ_GG_GO(NPV, 1);                                                                                        \
    } while (0)
#define LQ_GG_GO(NPV, SWV)                                                                                               \
    do {                                                                                                                 \
        auto kern = threads == 1024 ? geglu_int8_kernel<Tag, NPV, DYNAMIC, (NPV <= 5 ? 1024 : 256), SWV>                 \
                    : threads == 512 ? geglu_int8_kernel<Tag, NPV, DYNAMIC, (NPV <= 10 ? 512 : 256), SWV>                \
                                     : geglu_int8_kernel<Tag, NPV, DYNAMIC, 256, SWV>;                                   \
        static bool raised_by_size[3] = {false, false, false}; /* one flag per kernel; idempotent, a race only repeats it */ \
        bool& raised = raised_by_size[threads == 1024 ? 2 : threads == 512 ? 1 : 0];                                     \
        if (lds > 48 * 1024 && !raised) {                                                                                \
            hipError_t e = hipFuncSetAttribute(reinterpret_cast<const void*>(kern), hipFuncAttributeMaxDynamicSharedMemorySize, (int)lds); \
            if (e != hipSuccess) {                                                                                       \
                set_error("geglu_int8: cannot raise the LDS limit to %zu bytes: %s", lds, hipGetErrorString(e));         \
                return LQ_ERR_HIP;                                                                                       \
            }                                                                                                            \
            raised = true;                                                                                               \
        }                                                                                                                \
        hipLaunchKernelGGL(kern, grid, block, lds, st, dst, scale_out, hidden, bias, pre, in_scale, rows, d);            \
    } while (0)
    if (np <= 2) LQ_GG_CASE(2);
    else if (np <= 3) LQ_GG_CASE(3);
    else if (np <= 5) LQ_GG_CASE(5);
    else if (np <= 10) LQ_GG_CASE(10);
    else LQ_GG_CASE(16);
#undef LQ_GG_CASE
#undef LQ_GG_GO
    return check_launch("geglu_int8");
}

template <bool DYNAMIC>
static int dispatch_geglu(int8_t* dst, float* scale_out, const void* hidden, const void* bias, lq_dtype_t dt,
                          const float* pre, const float* in_scale, size_t rows, size_t dim, hipStream_t st) {
    switch (dt) {
        case LQ_F16: return launch_geglu<F16Tag, DYNAMIC>(dst, scale_out, hidden, bias, pre, in_scale, rows, dim, st);
        case LQ_BF16: return launch_geglu<BF16Tag, DYNAMIC>(dst, scale_out, hidden, bias, pre, in_scale, rows, dim, st);
        case LQ_F32: return launch_geglu<F32Tag, DYNAMIC>(dst, scale_out, hidden, bias, pre, in_scale, rows, dim, st);
        default: set_error("geglu_int8: unsupported dtype %d", (int)dt); return LQ_ERR_UNSUPPORTED;
    }
}

}  // namespace lq

using namespace lq;

extern "C" int lq_sq_input_quant(int8_t* dst, const void* src, lq_dtype_t src_dtype, const float* pre_quant_scale,
                                 const float* input_quant_scale, int per_token, size_t rows, size_t dim,
                                 lq_stream_t stream) {
    LQ_REQUIRE(dst && src && input_quant_scale, LQ_ERR_ARG, "lq_sq_input_quant: null pointer");
    if (rows == 0 || dim == 0) return LQ_OK;
    if (per_token)
        return dispatch_sq_quant<1>(dst, nullptr, src, src_dtype, pre_quant_scale, input_quant_scale, rows, dim,
                                    as_stream(stream));
    return dispatch_sq_quant<0>(dst, nullptr, src, src_dtype, pre_quant_scale, input_quant_scale, rows, dim,
                                as_stream(stream));
}

extern "C" int lq_sq_dynamic_quant(int8_t* dst, float* scale_out, const void* src, lq_dtype_t src_dtype,
                                   const float* pre_quant_scale, size_t rows, size_t dim, lq_stream_t stream) {
    LQ_REQUIRE(dst && src && scale_out, LQ_ERR_ARG, "lq_sq_dynamic_quant: null pointer");
    if (rows == 0) return LQ_OK;
    LQ_REQUIRE(dim > 0, LQ_ERR_SHAPE, "lq_sq_dynamic_quant: dim must be positive");
    return dispatch_sq_quant<2>(dst, scale_out, src, src_dtype, pre_quant_scale, nullptr, rows, dim, as_stream(stream));
}

// Dynamic per-token quantisation with the codes written as k-panels: the split kernel for every row length (a wavefront per
// 1024 columns), two rows per workgroup when a smoothing vector is given.
template <typename Tag>
static int launch_sq_dynamic_panels(int8_t* dst, float* scale_out, const void* src, const float* pre, size_t rows, size_t dim,
                                    hipStream_t st) {
    const int np = (int)((dim + 511) / 512), d = (int)dim;
    const dim3 block(64 * ((np + 1) / 2));
    const bool stream_io = rows * dim * Elem<Tag>::bytes >= kStreamQuantBytes;
    if (pre) {
        const dim3 grid((unsigned)((rows + 1) / 2));
        if (stream_io) hipLaunchKernelGGL((sq_quant_split_kernel<Tag, 2, true, 2, true, true>), grid, block, 0, st, dst, scale_out, src, pre, nullptr, rows, d);
        else hipLaunchKernelGGL((sq_quant_split_kernel<Tag, 2, true, 2, false, true>), grid, block, 0, st, dst, scale_out, src, pre, nullptr, rows, d);
    } else {
        const dim3 grid((unsigned)rows);
        if (stream_io) hipLaunchKernelGGL((sq_quant_split_kernel<Tag, 2, false, 1, true, true>), grid, block, 0, st, dst, scale_out, src, pre, nullptr, rows, d);
        else hipLaunchKernelGGL((sq_quant_split_kernel<Tag, 2, false, 1, false, true>), grid, block, 0, st, dst, scale_out, src, pre, nullptr, rows, d);
    }
    return check_launch("sq_quant_split(panels)");
}

extern "C" int lq_sq_dynamic_quant_panels(int8_t* dst_panels, float* scale_out, const void* src, lq_dtype_t src_dtype,
                                          const float* pre_quant_scale, size_t rows, size_t dim, lq_stream_t stream) {
    LQ_REQUIRE(dst_panels && src && scale_out, LQ_ERR_ARG, "lq_sq_dynamic_quant_panels: null pointer");
    if (rows == 0) return LQ_OK;
    LQ_REQUIRE(dim > 0 && dim % 64 == 0 && dim <= 16384 && rows <= 0x7fffffffu, LQ_ERR_SHAPE,
               "lq_sq_dynamic_quant_panels: k-panels need dim %% 64 == 0 and dim <= 16384 (rows=%zu dim=%zu)", rows, dim);
    LQ_REQUIRE(reinterpret_cast<uintptr_t>(src) % 16 == 0 && reinterpret_cast<uintptr_t>(dst_panels) % 16 == 0 &&
                   reinterpret_cast<uintptr_t>(pre_quant_scale) % 16 == 0,
               LQ_ERR_ARG, "lq_sq_dynamic_quant_panels: src, dst and pre_quant_scale must be 16-byte aligned");
    hipStream_t st = as_stream(stream);
    switch (src_dtype) {
        case LQ_F16: return launch_sq_dynamic_panels<F16Tag>(dst_panels, scale_out, src, pre_quant_scale, rows, dim, st);
        case LQ_BF16: return launch_sq_dynamic_panels<BF16Tag>(dst_panels, scale_out, src, pre_quant_scale, rows, dim, st);
        case LQ_F32: return launch_sq_dynamic_panels<F32Tag>(dst_panels, scale_out, src, pre_quant_scale, rows, dim, st);
        default: set_error("lq_sq_dynamic_quant_panels: unsupported source dtype %d", (int)src_dtype); return LQ_ERR_UNSUPPORTED;
    }
}

extern "C" int lq_sq_output_dequant(void* dst, lq_dtype_t dst_dtype, const int32_t* src, const float* input_quant_scale,
                                    const float* weight_quant_scale, int per_token, size_t rows, size_t dim,
                                    lq_stream_t stream) {
    LQ_REQUIRE(dst && src && input_quant_scale && weight_quant_scale, LQ_ERR_ARG, "lq_sq_output_dequant: null pointer");
    if (rows == 0 || dim == 0) return LQ_OK;
    size_t total = rows * dim;
    size_t blocks = (total + 255) / 256;
    if (blocks > 256 * 16) blocks = 256 * 16;
    dim3 grid((unsigned)blocks), block(256);
    hipStream_t st = as_stream(stream);
#define LQ_DQ(TAG)                                                                                                    \
    if (per_token) hipLaunchKernelGGL((sq_dequant_kernel<TAG, true>), grid, block, 0, st, dst, src, input_quant_scale, \
                                      weight_quant_scale, rows, dim);                                                 \
    else hipLaunchKernelGGL((sq_dequant_kernel<TAG, false>), grid, block, 0, st, dst, src, input_quant_scale,          \
                            weight_quant_scale, rows, dim)
    switch (dst_dtype) {
        case LQ_F16: LQ_DQ(F16Tag); break;
        case LQ_BF16: LQ_DQ(BF16Tag); break;
        case LQ_F32: LQ_DQ(F32Tag); break;
        default: set_error("lq_sq_output_dequant: unsupported dtype %d", (int)dst_dtype); return LQ_ERR_UNSUPPORTED;
    }
#undef LQ_DQ
    return check_launch("sq_output_dequant");
}

extern "C" int lq_int8_weight_quant(float* scale_out, int8_t* q_out, const void* weight, lq_dtype_t w_dtype,
                                    const float* pre_quant_scale, size_t d_out, size_t d_in, lq_stream_t stream) {
    LQ_REQUIRE(scale_out && q_out && weight, LQ_ERR_ARG, "lq_int8_weight_quant: null pointer");
    if (d_out == 0 || d_in == 0) return LQ_OK;
    dim3 grid((unsigned)(d_out < 65535 ? d_out : 65535)), block(256);
    hipStream_t st = as_stream(stream);
    switch (w_dtype) {
        case LQ_F16: hipLaunchKernelGGL((int8_weight_quant_kernel<F16Tag>), grid, block, 0, st, scale_out, q_out, weight, pre_quant_scale, d_out, d_in); break;
        case LQ_BF16: hipLaunchKernelGGL((int8_weight_quant_kernel<BF16Tag>), grid, block, 0, st, scale_out, q_out, weight, pre_quant_scale, d_out, d_in); break;
        case LQ_F32: hipLaunchKernelGGL((int8_weight_quant_kernel<F32Tag>), grid, block, 0, st, scale_out, q_out, weight, pre_quant_scale, d_out, d_in); break;
        default: set_error("lq_int8_weight_quant: unsupported dtype %d", (int)w_dtype); return LQ_ERR_UNSUPPORTED;
    }
    return check_launch("int8_weight_quant");
}

extern "C" int lq_geglu_int8(int8_t* dst, const void* hidden, const void* bias, lq_dtype_t dtype,
                             const float* pre_quant_scale, const float* input_quant_scale, size_t rows, size_t dim,
                             lq_stream_t stream) {
    LQ_REQUIRE(dst && hidden && input_quant_scale, LQ_ERR_ARG, "lq_geglu_int8: null pointer");
    if (rows == 0) return LQ_OK;
    return dispatch_geglu<false>(dst, nullptr, hidden, bias, dtype, pre_quant_scale, input_quant_scale, rows, dim,
                                 as_stream(stream));
}

extern "C" int lq_geglu_int8_dynamic(int8_t* dst, float* scale_out, const void* hidden, const void* bias,
                                     lq_dtype_t dtype, const float* pre_quant_scale, size_t rows, size_t dim,
                                     lq_stream_t stream) {
    LQ_REQUIRE(dst && hidden && scale_out, LQ_ERR_ARG, "lq_geglu_int8_dynamic: null pointer");
    if (rows == 0) return LQ_OK;
    return dispatch_geglu<true>(dst, scale_out, hidden, bias, dtype, pre_quant_scale, nullptr, rows, dim,
                                as_stream(stream));
}
