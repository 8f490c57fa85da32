// W4A4 group-64 INT4 activation quantisation with nibble packing, and the rows32 weight repack.
//
// Quantisation formula follows the lyraDiff reference, kernels/w4a4_gemm/w4a4_gemm.cu:206-214
// (rni + saturate to s4, low nibble first) and :897-930 (v = x / smooth, scale = group absmax / 7,
// q = v / scale).  One 64-lane wavefront owns a row (or a 1024-column range of a long row); a lane owns
// 8 consecutive elements per pass, so a group of 64 is 8 adjacent lanes: three cross-lane shuffles give the group absmax, each lane
// emits one packed uint32 (coalesced 256 B per wavefront) and the first lane of a group the scale.
#include "lq_common.h"

namespace lq {

// One lane's eight consecutive elements of a group of 64 (eight adjacent lanes hold the group): divides by the smoothing
// divisors (dv, with yv = fl(1/dv); both unused when !SMOOTHED), takes the group's absmax across the eight lanes, and returns
// the packed word; `s` receives the group's scale (already an fp16 value when F16_SCALE).
template <bool F16_SCALE, bool SMOOTHED>
__device__ __forceinline__ u32 w4a4_quant_lane8(float (&v)[8], const float (&dv)[8], const float (&yv)[8], float& s) {
    float amax = 0.0f;
    if constexpr (SMOOTHED) {
        // v = fl(x/d) from the stored reciprocal: q0 = fl(x*y), rem = x - q0*d (exact in one
        // fma), v = fl(q0 + rem*y) is the correctly rounded quotient when y = fl(1/d) and no
        // intermediate leaves the normal range (Markstein).  The range condition is checked
        // on the group's absmax, which is the only magnitude the outputs depend on: elements
        // far below it quantise to 0 whatever their last bit.  The max runs on the bit
        // patterns of |v| so that an inf or NaN anywhere in the group also takes the exact path.
        float xr[8];
        u32 mbits = 0;
#pragma unroll
        for (int i = 0; i < 8; ++i) {
            xr[i] = v[i];
            float q0 = xr[i] * yv[i];
            float rem = __builtin_fmaf(-q0, dv[i], xr[i]);
            v[i] = __builtin_fmaf(rem, yv[i], q0);
            u32 b = __float_as_uint(v[i]) & 0x7FFFFFFFu;
            mbits = b > mbits ? b : mbits;
        }
        float mf = group8_max(__uint_as_float(mbits));  // non-negative patterns order like floats
        mbits = __float_as_uint(mf);
        const bool odd = mbits != 0 && !(mbits >= 0x219392EFu /*1e-18f*/ && mbits <= 0x5D5E0B6Bu /*1e18f*/);
        amax = mf;
        if (__builtin_expect(odd, 0)) {  // uniform over the 8 lanes of the group
            amax = 0.0f;
#pragma unroll
            for (int i = 0; i < 8; ++i) {
                v[i] = xr[i] / dv[i];
                amax = fmaxf(amax, fabsf(v[i]));
            }
            amax = group8_max(amax);
        }
    } else {
#pragma unroll
        for (int i = 0; i < 8; ++i) amax = fmaxf(amax, fabsf(v[i]));
        amax = group8_max(amax);
    }
    s = div_by_const_fast(amax, 7.0f, 0x1.24924ap-3f);
    if constexpr (F16_SCALE) s = round_through<F16Tag>(s);
    const bool slow = scale_out_of_range(s);  // also covers an absmax outside the fast division's range
    if (__builtin_expect(slow, 0)) {
        s = amax / 7.0f;
        if constexpr (F16_SCALE) s = round_through<F16Tag>(s);
    }
    const float r = fast_recip(s);
    int q[8];
    // fp32 scale: s = fl(absmax / 7) bounds every |v / s| by 7.000001, no clamp needed.  An fp16 scale may have been
    // rounded down by a large factor in the subnormal range, so those results are clamped.
    quant8<-8, 7, F16_SCALE>(v, s, r, slow, q);
    // nibble i of the word = low four bits of q[i]: each step shifts the word right by four and
    // enters the next value's low nibble at the top (one v_alignbit_b32 per element)
    u32 word = 0;
#pragma unroll
    for (int i = 0; i < 8; ++i) word = __builtin_amdgcn_alignbit((u32)q[i], word, 4);
    return word;
}

// SMOOTH 0: no smoothing vector; 1: the divisors d of the workgroup's column range and their correctly
// rounded reciprocals y = fl(1/d) are computed once per workgroup into LDS and shared by the rows of
// its four wavefronts.
// WAVES: wavefronts (= rows in flight) per workgroup.  The staging of the smoothing vector costs a workgroup one IEEE division
// per column of its range whatever its size, so sixteen rows per workgroup would pay a quarter of what four pay -- measured
// slower all the same (15.4 against 14.7 us at 4608x3072 from HBM: sixteen wavefronts wait at one barrier for the staging's
// load and division chain, where small workgroups on a CU are in different phases), so four it stays.
// FULL: k is a multiple of the column range, no lane is ever out of range.
template <typename Tag, int NP, bool F16_SCALE, int SMOOTH, int WAVES = 4, bool FULL = false, bool STREAM = false>
__global__ __launch_bounds__(WAVES * 64) void w4a4_quant_kernel(u32* __restrict__ q_words, void* __restrict__ scales,
                                                         const void* __restrict__ x,
                                                         const float* __restrict__ smooth, int m, int k,
                                                         int rows_per_wave, int parts) {
    // A workgroup owns the column range [cbase, cbase + NP*512) of its rows: long rows are split into `parts`
    // ranges (groups of 64 are independent), which keeps the per-wavefront register footprint small enough for
    // eight wavefronts per SIMD.
    extern __shared__ __attribute__((aligned(16))) float s_dy[];  // [NP*512] divisors, then [NP*512] reciprocals
    constexpr int SPAN = NP * 512;
    const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
    const int ng = k >> 6;
    const int part = blockIdx.x % parts, rowblock = blockIdx.x / parts;
    const int cbase = part * SPAN;
    constexpr int VPP = Elem<Tag>::bytes == 2 ? 1 : 2;  // 16-byte vectors per 8 elements
    auto load_raw = [&](int row, uint4 (*raw)[VPP]) {
        const char* rb = static_cast<const char*>(x) + (size_t)row * k * Elem<Tag>::bytes;
#pragma unroll
        for (int p = 0; p < NP; ++p) {
            int col = cbase + (p * 64 + lane) * 8;
#pragma unroll
            for (int u = 0; u < VPP; ++u) {
                if constexpr (!FULL) raw[p][u] = make_uint4(0, 0, 0, 0);
                if (FULL || col < k) raw[p][u] = ld16<STREAM>(rb + (size_t)col * Elem<Tag>::bytes + u * 16);
            }
        }
    };
    // The wavefront's first row is requested before the smoothing vector is staged, so that the two memory latencies
    // (row from HBM, vector from L2) run side by side instead of one after the other.
    const int row0 = rowblock * WAVES * rows_per_wave + wave;
    uint4 cur[NP][VPP], nxt[NP][VPP];
    if (row0 < m) load_raw(row0, cur);
    if constexpr (SMOOTH == 1) {
        for (int c = threadIdx.x * 4; c < SPAN && cbase + c < k; c += WAVES * 256) {
            float4 d = *reinterpret_cast<const float4*>(smooth + cbase + c);
            *reinterpret_cast<float4*>(s_dy + c) = d;
            *reinterpret_cast<float4*>(s_dy + SPAN + c) = make_float4(1.0f / d.x, 1.0f / d.y, 1.0f / d.z, 1.0f / d.w);
        }
        __syncthreads();
    }
    // Raw row data is double buffered in registers: the loads of the wavefront's next row are in
    // flight while the current row is quantised.
    auto unpack_raw = [&](const uint4* r, float* o) {
        if constexpr (Elem<Tag>::bytes == 2) unpack8<Tag>(r[0], o);
        else {
            o[0] = __uint_as_float(r[0].x); o[1] = __uint_as_float(r[0].y); o[2] = __uint_as_float(r[0].z); o[3] = __uint_as_float(r[0].w);
            o[4] = __uint_as_float(r[VPP - 1].x); o[5] = __uint_as_float(r[VPP - 1].y); o[6] = __uint_as_float(r[VPP - 1].z); o[7] = __uint_as_float(r[VPP - 1].w);
        }
    };
    for (int j = 0; j < rows_per_wave; ++j) {
        const int row = row0 + WAVES * j;
        if (row >= m) break;
        const bool has_next = j + 1 < rows_per_wave && row + WAVES < m;
        if (has_next) load_raw(row + WAVES, nxt);
        const char* rb = static_cast<const char*>(x) + (size_t)row * k * Elem<Tag>::bytes;
#pragma unroll
        for (int p = 0; p < NP; ++p) {
            int col = cbase + (p * 64 + lane) * 8;
            float v[8];
            unpack_raw(cur[p], v);
            float dv[8], yv[8];
            if constexpr (SMOOTH == 1) {
                const int cc = (FULL || col < k) ? col - cbase : 0;
                float4 a = *reinterpret_cast<const float4*>(s_dy + cc), b = *reinterpret_cast<const float4*>(s_dy + cc + 4);
                float4 c = *reinterpret_cast<const float4*>(s_dy + SPAN + cc), d = *reinterpret_cast<const float4*>(s_dy + SPAN + cc + 4);
                dv[0] = a.x; dv[1] = a.y; dv[2] = a.z; dv[3] = a.w; dv[4] = b.x; dv[5] = b.y; dv[6] = b.z; dv[7] = b.w;
                yv[0] = c.x; yv[1] = c.y; yv[2] = c.z; yv[3] = c.w; yv[4] = d.x; yv[5] = d.y; yv[6] = d.z; yv[7] = d.w;
            }
            float s;
            const u32 word = w4a4_quant_lane8<F16_SCALE, SMOOTH == 1>(v, dv, yv, s);
            if (FULL || col < k) {
                st4<STREAM>(q_words + (size_t)row * (k >> 3) + (col >> 3), word);
                if ((lane & 7) == 0) {
                    size_t si = (size_t)row * ng + (col >> 6);
                    if constexpr (F16_SCALE) static_cast<unsigned short*>(scales)[si] = (unsigned short)f32_to_f16_bits(s);  // s is already an fp16 value
                    else static_cast<float*>(scales)[si] = s;
                }
            }
        }
        (void)rb;
        if (has_next) {
#pragma unroll
            for (int p = 0; p < NP; ++p)
#pragma unroll
                for (int u = 0; u < VPP; ++u) cur[p][u] = nxt[p][u];
        }
    }
}

// ---- quantisation and the low-rank down projection in one pass over x -----------------------------------------------
// The reference computes both from one read of x (kernels/w4a4_gemm/w4a4_gemm.cu:769-953: the quantising tile also feeds
// the rank-32 product and adds it into a zeroed fp32 buffer with float atomics).  Here a workgroup owns up to 32 rows and all
// of K, its eight wavefronts take interleaved 128-column slices, and a slice is loaded once into registers in the
// quantiser's layout (a lane holds eight consecutive elements, a group of 64 is eight adjacent lanes; a load instruction
// covers four rows x 256 bytes: whole cache lines).  From the registers the slice is (a) quantised exactly as
// w4a4_quant_kernel does it (the same per-lane function, so words and scales are the same bits) and (b) parked in the
// wavefront's private, bank-swizzled LDS block, from which the matrix instruction reads its fragments (it wants a lane to
// hold eight k of ONE row for each of 32 rows).  The slice of `lora_down` takes the same route.  The divisors of a slice and
// their correctly rounded reciprocals are computed by the wavefront itself (two IEEE divisions per lane and slice).  Partial
// 32 x 32 sums of the wavefronts meet in LDS and are added in wavefront order: no atomics, results do not depend on scheduling.
// Rows per workgroup = ceil(m / CUs) when that is below 32, so that every CU gets the same share; rows are loaded four per
// instruction, so 18 rows cost five row-instructions (90 % of the lanes quantise real data).
typedef __bf16 fv8bf __attribute__((ext_vector_type(8)));
typedef _Float16 fv8h __attribute__((ext_vector_type(8)));
typedef float fv16f __attribute__((ext_vector_type(16)));

template <bool F16> __device__ __forceinline__ fv16f fused_mfma(const v4i& a, const v4i& b, const fv16f& c) {
    if constexpr (F16) return __builtin_amdgcn_mfma_f32_32x32x16_f16(__builtin_bit_cast(fv8h, a), __builtin_bit_cast(fv8h, b), c, 0, 0, 0);
    else return __builtin_amdgcn_mfma_f32_32x32x16_bf16(__builtin_bit_cast(fv8bf, a), __builtin_bit_cast(fv8bf, b), c, 0, 0, 0);
}

constexpr int kFusedWaves = 8;
constexpr int kFusedPark = 8192;                              // 32 rows x 256 bytes
constexpr int kFusedWaveStage = 2 * kFusedPark + 1024;        // x, lora_down, then 128 divisors and 128 reciprocals
constexpr int kFusedLds = kFusedWaves * kFusedWaveStage;

// OUT: 0 fp32, 1 fp16, 2 bf16 (type of the low-rank result).
template <bool F16, bool F16_SCALE, int OUT, bool STREAM>
__global__ __launch_bounds__(kFusedWaves * 64) void w4a4_quant_lora_kernel(u32* __restrict__ q_words, void* __restrict__ scales,
                                                                          void* __restrict__ act,
                                                                          const unsigned short* __restrict__ x,
                                                                          const float* __restrict__ smooth,
                                                                          const unsigned short* __restrict__ down, int m, int k,
                                                                          int rows_per_wg) {
    using Tag = typename std::conditional<F16, F16Tag, BF16Tag>::type;
    constexpr int W = kFusedWaves;
    extern __shared__ __attribute__((aligned(16))) char fsmem[];
    const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
    const int row0 = blockIdx.x * rows_per_wg;
    const int rows = min(rows_per_wg, m - row0);
    const int ni = (rows + 3) >> 2;  // row-instructions per slice, at most 8
    char* stage = fsmem + wave * kFusedWaveStage;
    float* s_dy = reinterpret_cast<float*>(stage + 2 * kFusedPark);
    // memory side: lane -> (row 4*i + lane/16, 16-byte chunk lane%16); LDS side: chunk c of row r sits at chunk slot
    // c ^ (r & 15): the sixteen lanes of a write (one row, all chunks) and of a read (sixteen rows, one chunk) both
    // cover all banks
    const int gr = lane >> 4, gc = lane & 15;
    const int lr = lane & 31, lh = lane >> 5;
    u32 xo[8];
#pragma unroll
    for (int i = 0; i < 8; ++i) xo[i] = (u32)(row0 + min(4 * i + gr, rows - 1)) * (u32)k + gc * 8;
    const u32 dofs = (u32)gr * (u32)k + gc * 8;
    const int nsl = k >> 7, ng = k >> 6;
    fv16f acc;
#pragma unroll
    for (int v = 0; v < 16; ++v) acc[v] = 0.0f;
    uint4 gx[8];
    v4i gd[8];
    float2 gs;
    // One set of registers per operand: a slice is parked in LDS first thing and the next slice is requested right behind
    // that, so that the matrix steps and the quantisation of this slice cover the next one's way from memory.
    auto load_slice = [&](int sl) {
        const int k0 = sl << 7;
        gs = *reinterpret_cast<const float2*>(smooth + k0 + 2 * lane);
#pragma unroll
        for (int i = 0; i < 8; ++i)
            if (i < ni) gx[i] = ld16<STREAM>(x + xo[i] + k0);
#pragma unroll
        for (int i = 0; i < 8; ++i) gd[i] = *reinterpret_cast<const v4i*>(down + dofs + (size_t)i * 4 * k + k0);
    };
    if (wave < nsl) load_slice(wave);
    for (int sl = wave; sl < nsl; sl += W) {
        const int k0 = sl << 7;
        *reinterpret_cast<float2*>(s_dy + 2 * lane) = gs;
        *reinterpret_cast<float2*>(s_dy + 128 + 2 * lane) = make_float2(1.0f / gs.x, 1.0f / gs.y);
#pragma unroll
        for (int i = 0; i < 8; ++i) {
            const int r = 4 * i + gr;
            const int wofs = r * 256 + ((gc ^ (r & 15)) << 4);
            if (i < ni) *reinterpret_cast<uint4*>(stage + wofs) = gx[i];
            *reinterpret_cast<v4i*>(stage + kFusedPark + wofs) = gd[i];
        }
        if (sl + W < nsl) load_slice(sl + W);
        // the wavefront's LDS accesses complete in program order; the fence only keeps the compiler from moving the
        // reads of other lanes' data above the writes
        __builtin_amdgcn_fence(__ATOMIC_ACQ_REL, "wavefront");
        __builtin_amdgcn_wave_barrier();
        float dv[8], yv[8];
        {
            const float4 a = *reinterpret_cast<const float4*>(s_dy + gc * 8), b = *reinterpret_cast<const float4*>(s_dy + gc * 8 + 4);
            const float4 c = *reinterpret_cast<const float4*>(s_dy + 128 + gc * 8), d = *reinterpret_cast<const float4*>(s_dy + 128 + gc * 8 + 4);
            dv[0] = a.x; dv[1] = a.y; dv[2] = a.z; dv[3] = a.w; dv[4] = b.x; dv[5] = b.y; dv[6] = b.z; dv[7] = b.w;
            yv[0] = c.x; yv[1] = c.y; yv[2] = c.z; yv[3] = c.w; yv[4] = d.x; yv[5] = d.y; yv[6] = d.z; yv[7] = d.w;
        }
        // rows of the 32-row matrix operand that no row-instruction wrote hold whatever LDS held: they only reach result
        // columns that are never stored
#pragma unroll
        for (int s = 0; s < 8; ++s) {  // matrix step s: k = 16 s + 8 lh .. + 8
            const int rofs = lr * 256 + (((2 * s + lh) ^ (lr & 15)) << 4);
            acc = fused_mfma<F16>(*reinterpret_cast<const v4i*>(stage + kFusedPark + rofs), *reinterpret_cast<const v4i*>(stage + rofs), acc);
        }
        // the quantiser takes its elements back from the parked slice, one row-instruction (four rows) per turn of a real
        // loop: one copy of the code, and no operand register outlives the parking
        uint4 parked = *reinterpret_cast<const uint4*>(stage + gr * 256 + ((gc ^ gr) << 4));
#pragma unroll 1
        for (int i = 0; i < ni; ++i) {
            const int r = 4 * i + gr;
            float v[8];
            unpack8<Tag>(parked, v);
            {  // the next turn's elements are on their way from LDS while this turn's are quantised (the last turn reads a
               // row nobody uses: inside the block all the same)
                const int rn = (r + 4) & 31;
                parked = *reinterpret_cast<const uint4*>(stage + rn * 256 + ((gc ^ (rn & 15)) << 4));
            }
            float s;
            const u32 word = w4a4_quant_lane8<F16_SCALE, true>(v, dv, yv, s);
            if (r < rows) {
                const size_t row = (size_t)(row0 + r);
                st4<STREAM>(q_words + row * (k >> 3) + (k0 >> 3) + gc, word);
                if ((lane & 7) == 0) {
                    const size_t si = row * ng + (k0 >> 6) + (gc >> 3);
                    if constexpr (F16_SCALE) static_cast<unsigned short*>(scales)[si] = (unsigned short)f32_to_f16_bits(s);  // s is already an fp16 value
                    else static_cast<float*>(scales)[si] = s;
                }
            }
        }
        __builtin_amdgcn_fence(__ATOMIC_ACQ_REL, "wavefront");
        __builtin_amdgcn_wave_barrier();
    }
    __syncthreads();  // every wavefront is done with its blocks: the partial sums may overwrite them
    float(*part)[16][64] = reinterpret_cast<float(*)[16][64]>(fsmem);  // partial blocks of wavefronts 1..7
    if (wave != 0) {
#pragma unroll
        for (int v = 0; v < 16; ++v) part[wave - 1][v][lane] = acc[v];
    }
    __syncthreads();
    if (wave != 0) return;
#pragma unroll
    for (int v = 0; v < 16; ++v)
#pragma unroll
        for (int w = 0; w < W - 1; ++w) acc[v] += part[w][v][lane];  // wavefront order: 0, 1, ..., 7
    if (lr < rows) {
        // result layout of the 32x32 matrix instruction: this lane holds x row lr and rank indices 8*(v/4) + 4*lh + v%4
#pragma unroll
        for (int q4 = 0; q4 < 4; ++q4) {
            const size_t idx = (size_t)(row0 + lr) * 32 + q4 * 8 + lh * 4;
            const float y0 = acc[q4 * 4], y1 = acc[q4 * 4 + 1], y2 = acc[q4 * 4 + 2], y3 = acc[q4 * 4 + 3];
            if constexpr (OUT == 0) {
                *reinterpret_cast<float4*>(static_cast<float*>(act) + idx) = make_float4(y0, y1, y2, y3);
            } else {
                uint2 o;
                o.x = OUT == 1 ? pack2_f16(y0, y1) : pack2_bf16(y0, y1);
                o.y = OUT == 1 ? pack2_f16(y2, y3) : pack2_bf16(y2, y3);
                *reinterpret_cast<uint2*>(static_cast<unsigned short*>(act) + idx) = o;
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
    // Column ranges per row: rows longer than 2048 are cut into ranges of 1024 columns (two passes of 512 per
    // wavefront): 64 registers per lane instead of 124 for a 3072-column row, eight wavefronts per SIMD instead of four,
    // and no half-empty second round of wavefronts (measured 10-19 % faster at 4608..6912 x 3072).
    const int np = k > 2048 ? 2 : (k + 511) / 512;  // 1, 2, 3 or 4
    const int parts = (k + np * 512 - 1) / (np * 512);
    // rows per wavefront: enough wavefronts to fill the chip (about 3 per SIMD), then more rows each so
    // that the loads of one row overlap the arithmetic of the previous one
    int rpw = m / (4 * 768);
    rpw = rpw < 1 ? 1 : (rpw > 8 ? 8 : rpw);
    const int blocks = (m + 4 * rpw - 1) / (4 * rpw) * parts;
    dim3 grid(blocks), block(256);
    hipStream_t st = as_stream(stream);
    const bool f16s = scale_dtype == LQ_F16;
    const int smode = smooth == nullptr ? 0 : 1;
    const size_t lds = smode == 1 ? 2 * (size_t)np * 512 * sizeof(float) : 0;
    // long rows whose length is a whole number of column ranges (FLUX: 3072): no range checks
    if (smode == 1 && np == 2 && k % 1024 == 0 && x_dtype != LQ_F32) {
        const bool stream_io = (size_t)m * k * 2 >= kStreamQuantBytes;  // read-once input, write-once codes
#define LQ_W4_FULL(TAG, F16S)                                                                                                          \
    do {                                                                                                                               \
        if (stream_io) hipLaunchKernelGGL((w4a4_quant_kernel<TAG, 2, F16S, 1, 4, true, true>), grid, block, lds, st, q_words, scales, x, smooth, m, k, rpw, parts); \
        else hipLaunchKernelGGL((w4a4_quant_kernel<TAG, 2, F16S, 1, 4, true, false>), grid, block, lds, st, q_words, scales, x, smooth, m, k, rpw, parts);       \
    } while (0)
        if (x_dtype == LQ_F16) { if (f16s) LQ_W4_FULL(F16Tag, true); else LQ_W4_FULL(F16Tag, false); }
        else { if (f16s) LQ_W4_FULL(BF16Tag, true); else LQ_W4_FULL(BF16Tag, false); }
#undef LQ_W4_FULL
        return check_launch("w4a4_quantize");
    }
#define LQ_W4_LAUNCH2(TAG, NPV, F16S, SM) \
    hipLaunchKernelGGL((w4a4_quant_kernel<TAG, NPV, F16S, SM>), grid, block, lds, st, q_words, scales, x, smooth, m, k, rpw, parts)
#define LQ_W4_LAUNCH(TAG, NPV)                                                     \
    do {                                                                           \
        if (f16s) {                                                                \
            if (smode == 0) LQ_W4_LAUNCH2(TAG, NPV, true, 0);                      \
            else LQ_W4_LAUNCH2(TAG, NPV, true, 1);                                 \
        } else {                                                                   \
            if (smode == 0) LQ_W4_LAUNCH2(TAG, NPV, false, 0);                     \
            else LQ_W4_LAUNCH2(TAG, NPV, false, 1);                                \
        }                                                                          \
    } while (0)
#define LQ_W4_NP(TAG)                            \
    do {                                         \
        if (np <= 1) LQ_W4_LAUNCH(TAG, 1);       \
        else if (np <= 2) LQ_W4_LAUNCH(TAG, 2);  \
        else if (np <= 3) LQ_W4_LAUNCH(TAG, 3);  \
        else LQ_W4_LAUNCH(TAG, 4);               \
    } while (0)
    switch (x_dtype) {
        case LQ_F16: LQ_W4_NP(F16Tag); break;
        case LQ_BF16: LQ_W4_NP(BF16Tag); break;
        case LQ_F32: LQ_W4_NP(F32Tag); break;
        default: set_error("lq_w4a4_quantize: unsupported x dtype %d", (int)x_dtype); return LQ_ERR_UNSUPPORTED;
    }
#undef LQ_W4_NP
#undef LQ_W4_LAUNCH
#undef LQ_W4_LAUNCH2
    return check_launch("w4a4_quantize");
}

template <bool F16, bool F16_SCALE, int OUT, bool STREAM>
static int launch_quant_lora(u32* q_words, void* scales, void* act, const void* x, const float* smooth, const void* down, int m, int k,
                             hipStream_t st) {
    static const int num_cu = [] {
        int dev = 0, n = 0;
        if (hipGetDevice(&dev) != hipSuccess || hipDeviceGetAttribute(&n, hipDeviceAttributeMultiprocessorCount, dev) != hipSuccess || n <= 0) n = 256;
        return n;
    }();
    auto kern = w4a4_quant_lora_kernel<F16, F16_SCALE, OUT, STREAM>;
    static bool raised = false;  // idempotent, a race only repeats it
    if (!raised) {
        hipError_t e = hipFuncSetAttribute(reinterpret_cast<const void*>(kern), hipFuncAttributeMaxDynamicSharedMemorySize, kFusedLds);
        if (e != hipSuccess) {
            set_error("lq_w4a4_quantize_lora_down: cannot raise the LDS limit to %d bytes: %s", kFusedLds, hipGetErrorString(e));
            return LQ_ERR_HIP;
        }
        raised = true;
    }
    const int rpw = std::min(32, std::max(4, (m + num_cu - 1) / num_cu));
    hipLaunchKernelGGL(kern, dim3((unsigned)((m + rpw - 1) / rpw)), dim3(kFusedWaves * 64), kFusedLds, st, q_words, scales, act,
                       static_cast<const unsigned short*>(x), smooth, static_cast<const unsigned short*>(down), m, k, rpw);
    return check_launch("w4a4_quantize_lora_down");
}

extern "C" int lq_w4a4_quantize_lora_down(uint32_t* q_words, void* scales, lq_dtype_t scale_dtype, void* lora_act,
                                          lq_dtype_t act_dtype, const void* x, lq_dtype_t x_dtype, const float* smooth,
                                          const void* lora_down, int m, int k, int rank, int group, lq_stream_t stream) {
    if (m == 0) return LQ_OK;
    LQ_REQUIRE(lora_act && lora_down, LQ_ERR_ARG, "lq_w4a4_quantize_lora_down: null pointer");
    LQ_REQUIRE(act_dtype == LQ_F32 || act_dtype == LQ_F16 || act_dtype == LQ_BF16, LQ_ERR_UNSUPPORTED,
               "lq_w4a4_quantize_lora_down: unsupported low-rank result dtype %d", (int)act_dtype);
    const bool one_pass = q_words && scales && x && group == 64 && (x_dtype == LQ_F16 || x_dtype == LQ_BF16) && smooth != nullptr &&
                          rank == 32 && m > 0 && k > 0 && k % 128 == 0 && k <= 16384 && (size_t)m * k < ((size_t)1 << 31) &&
                          (scale_dtype == LQ_F32 || scale_dtype == LQ_F16) && (act_dtype == LQ_F32 || act_dtype == x_dtype) &&
                          reinterpret_cast<uintptr_t>(x) % 16 == 0 && reinterpret_cast<uintptr_t>(smooth) % 16 == 0 &&
                          reinterpret_cast<uintptr_t>(lora_down) % 16 == 0 && reinterpret_cast<uintptr_t>(lora_act) % 16 == 0;
    if (!one_pass) {  // the two kernels one after the other: same results, same argument checks
        int rc = lq_w4a4_quantize(q_words, scales, scale_dtype, x, x_dtype, smooth, m, k, group, stream);
        if (rc != LQ_OK) return rc;
        return lq_lora_down(lora_act, act_dtype, x, lora_down, x_dtype, m, k, rank, stream);
    }
    hipStream_t st = as_stream(stream);
    const bool f16 = x_dtype == LQ_F16, f16s = scale_dtype == LQ_F16, f32act = act_dtype == LQ_F32;
    const bool stream_io = (size_t)m * k * 2 >= kStreamQuantBytes;  // read-once input, write-once codes
#define LQ_QL_GO(F16V, F16S, OUTV)                                                                                         \
    (stream_io ? launch_quant_lora<F16V, F16S, OUTV, true>(q_words, scales, lora_act, x, smooth, lora_down, m, k, st)         \
               : launch_quant_lora<F16V, F16S, OUTV, false>(q_words, scales, lora_act, x, smooth, lora_down, m, k, st))
#define LQ_QL_OUT(F16V, F16S) (f32act ? LQ_QL_GO(F16V, F16S, 0) : LQ_QL_GO(F16V, F16S, (F16V ? 1 : 2)))
    if (f16) return f16s ? LQ_QL_OUT(true, true) : LQ_QL_OUT(true, false);
    return f16s ? LQ_QL_OUT(false, true) : LQ_QL_OUT(false, false);
#undef LQ_QL_OUT
#undef LQ_QL_GO
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
