// Weight-only quantized GEMM (W8A16 / W4A16, per-output-channel scales):
//     C[m,n] = T( scale[n] * sum_k A[m,k] * q[k,n] [+ bias[n]] )
// with 16-bit activations, int8 or int4 weights and fp32 accumulation on v_mfma_f32_32x32x16_{f16,bf16}.
// Reference: CutlassFpAIntBGemmRunner (kernels/cutlass_kernels/fpA_intB_gemm/fpA_intB_gemm.h:27-130 of lyraDiff,
// PER_COLUMN_SCALE_ONLY) on weights produced by symmetric_quantize + preprocess_weights_for_mixed_gemm
// (kernels/cutlass_kernels/cutlass_preprocessors.cpp:484-631).  That preprocessing (row permutation, column-major
// tile interleave, +128/+8 bias, nibble interleave) is specific to NVIDIA's mma fragments; the counterpart here is
// lq_repack_weight_only, which keeps its contract -- a one-time bijection of the [k, n] integer matrix -- and
// produces the layout this kernel reads:
//   * transposed to [n, k] and stored as UNSIGNED codes u = q + 128 (int8) or u = q + 8 (int4), so that a code
//     can be ORed into the mantissa of a 16-bit float (1024 + u is 0x6400 | u in fp16) and the offset removed by
//     one packed subtraction: one or two vector operations per pair of weights instead of a convert per weight;
//   * int4: the eight codes of a dword sit in nibble order k0 k2 k4 k6 k1 k3 k5 k7 (low to high), so that masking
//     with 0x000F000F after shifts of 0/4/8/12 bits yields the pairs (k0,k1) (k2,k3) (k4,k5) (k6,k7) directly;
//   * then the rows32 chunking of the other GEMMs (16-byte chunk c of 32 consecutive output channels contiguous),
//     which makes every LDS fragment read a conflict-free 16-byte access.
// The scale is applied once per output in the epilogue (the reference multiplies every dequantised weight by the
// scale in T inside the main loop, which rounds each weight; results agree to that rounding).
//
// Group-wise ("fine-grained") scales, with or without zero points (FINEGRAINED_SCALE_ONLY / FINEGRAINED_SCALE_AND_ZEROS,
// group 64 or 128 along k, scales and zeros [k / group, n] of T): every dequantised weight is formed in T inside the main
// loop as the reference's MmaTensorOpDequantizer does (cutlass_extensions/gemm/warp/mma_tensorop_dequantizer.h:150-222,
// 370-390): fp16  w = T(T(q * s) + z)  (multiply, then add, one packed instruction each);  bf16  w = T(fma(q, s, z))
// (evaluated in fp32 and rounded once to bf16; q * s is exact in fp32).  The k-tile of 64 lies inside one group; the
// scales (and zeros) of the tile's output channels travel to LDS with the operands (one 4-byte transfer per lane).
//
// Tiling: 256x128 outputs per workgroup of four wavefronts (2x2), 128x64 per wavefront (eight 32x32 MFMA tiles:
// every converted weight fragment is used by four MFMAs), k-tile 64, two LDS stages filled from registers
// (activations XOR-swizzled, weights copied as they lie), the next tile's global loads in flight during the MFMAs.
#include "lq_gemm_core.h"

namespace lq {

typedef _Float16 v8h __attribute__((ext_vector_type(8)));
typedef __bf16 v8bf __attribute__((ext_vector_type(8)));
typedef _Float16 h2_t __attribute__((ext_vector_type(2)));

template <int CH> __device__ __forceinline__ int wo_swizzle(int row) {  // 8 chunks of 16 bytes per activation row
    return ((row >> 1) & 7) ^ ((row & 1) << 2);
}

// eight consecutive-k weights of one output channel as 16-bit floats (one 16-byte MFMA operand), from unsigned codes.
// G = 0: the bare integer values (the per-channel scale is applied to the sums); 1: times the group's scale; 2: times the
// scale plus the zero point.  s2 / z2: the scale and zero of the lane's channel, as a pair of fp16 (fp16 path) or as fp32
// bit patterns (bf16 path).
template <bool F16, bool W4, int G> struct WoCvt;
template <int G> __device__ __forceinline__ int wo_apply_h2(h2_t q, u32 s2, u32 z2) {
    if constexpr (G >= 1) q = q * __builtin_bit_cast(h2_t, s2);   // v_pk_mul_f16: T(q * s)
    if constexpr (G == 2) q = q + __builtin_bit_cast(h2_t, z2);   // v_pk_add_f16: T(. + z)
    return __builtin_bit_cast(int, q);
}
template <int G> __device__ __forceinline__ float wo_apply_f32(float q, u32 s, u32 z) {
    if constexpr (G == 1) return q * __uint_as_float(s);                                      // exact in fp32
    if constexpr (G == 2) return __builtin_fmaf(q, __uint_as_float(s), __uint_as_float(z));
    return q;
}
template <int G> struct WoCvt<true, false, G> {  // fp16 <- uint8: d0 holds k0..k3, d1 holds k4..k7
    static __device__ __forceinline__ v4i run(u32 d0, u32 d1, u32 s2, u32 z2) {
        v4i o;
        const h2_t off = {(_Float16)1152.0f, (_Float16)1152.0f};
        const u32 p[4] = {__builtin_amdgcn_perm(0x64646464u, d0, 0x04010400u), __builtin_amdgcn_perm(0x64646464u, d0, 0x04030402u),
                          __builtin_amdgcn_perm(0x64646464u, d1, 0x04010400u), __builtin_amdgcn_perm(0x64646464u, d1, 0x04030402u)};
#pragma unroll
        for (int i = 0; i < 4; ++i) o[i] = wo_apply_h2<G>(__builtin_bit_cast(h2_t, p[i]) - off, s2, z2);
        return o;
    }
};
template <int G> struct WoCvt<true, true, G> {  // fp16 <- uint4: d0 holds k0..k7 in the interleaved nibble order
    static __device__ __forceinline__ v4i run(u32 d0, u32, u32 s2, u32 z2) {
        v4i o;
        const h2_t off = {(_Float16)1032.0f, (_Float16)1032.0f};
#pragma unroll
        for (int i = 0; i < 4; ++i) {
            const u32 p = ((d0 >> (4 * i)) & 0x000F000Fu) | 0x64006400u;
            o[i] = wo_apply_h2<G>(__builtin_bit_cast(h2_t, p) - off, s2, z2);
        }
        return o;
    }
};
template <int G> struct WoCvt<false, false, G> {  // bf16 <- uint8 (through fp32: bf16 cannot hold 1024 + u)
    static __device__ __forceinline__ v4i run(u32 d0, u32 d1, u32 s, u32 z) {
        v4i o;
        const u32 d[2] = {d0, d1};
#pragma unroll
        for (int i = 0; i < 4; ++i) {
            const u32 w = d[i >> 1] >> (16 * (i & 1));
            o[i] = (int)pack2_bf16(wo_apply_f32<G>((float)(w & 0xFFu) - 128.0f, s, z), wo_apply_f32<G>((float)((w >> 8) & 0xFFu) - 128.0f, s, z));
        }
        return o;
    }
};
template <int G> struct WoCvt<false, true, G> {  // bf16 <- uint4
    static __device__ __forceinline__ v4i run(u32 d0, u32, u32 s, u32 z) {
        v4i o;
#pragma unroll
        for (int i = 0; i < 4; ++i) {
            const u32 w = d0 >> (4 * i);
            o[i] = (int)pack2_bf16(wo_apply_f32<G>((float)(w & 0xFu) - 8.0f, s, z), wo_apply_f32<G>((float)((w >> 16) & 0xFu) - 8.0f, s, z));
        }
        return o;
    }
};

// WN = 2: 256x128 outputs, four wavefronts, two workgroups per CU.  WN = 4: 256x256 outputs, eight wavefronts, one
// workgroup per CU (more operand reuse per LDS byte; the choice for large problems).
// GROUPED 0: scales [n], applied to the sums; 1: scales [k / group, n] applied to every weight; 2: scales and zeros.
template <typename Tag, bool W4, int WN, int NSTAGE, int GROUPED = 0>
__global__ __launch_bounds__(128 * WN, (WN == 2 ? 2 : 1)) void wo_gemm_kernel(void* __restrict__ C, const void* __restrict__ A,
                                                                              const uint8_t* __restrict__ B,
                                                                              const void* __restrict__ scales,
                                                                              const void* __restrict__ zeros,
                                                                              const void* __restrict__ bias, int m, int n, int k,
                                                                              int tiles_m, int tiles_n, int tiles_per_group) {
    constexpr bool F16 = std::is_same<Tag, F16Tag>::value;
    constexpr int NW = 2 * WN, BM = 256, BN = 64 * WN, BK = 64, TM = 128, TN = 64, MT = 4, NT = 2;
    constexpr int A_BYTES = BM * BK * 2;                 // 32 KiB
    constexpr int BCH = W4 ? 2 : 4;                      // 16-byte weight chunks per row per k-tile
    constexpr int B_BYTES = BN * BCH * 16;
    constexpr int SZ_BYTES = GROUPED ? 1024 : 0;          // scales of the tile's BN channels at +0, zeros at +512
    constexpr int STAGE = A_BYTES + B_BYTES + SZ_BYTES;
    constexpr int A_DMA = A_BYTES / 1024 / NW;           // 1 KiB transfers per wavefront per tile
    constexpr int B_DMA = B_BYTES / 1024 / NW;
    constexpr int PER_TILE = A_DMA + B_DMA + GROUPED;     // + one 4-byte-per-lane transfer for the scales, one for the zeros
    static_assert(A_DMA * NW * 1024 == A_BYTES && B_DMA * NW * 1024 == B_BYTES && B_DMA >= 1, "stage / wavefront mismatch");
    static_assert(PER_TILE * NSTAGE < 64, "vmcnt is a 6-bit counter");
    extern __shared__ __attribute__((aligned(16))) char wo_smem[];
    const int tid = threadIdx.x, lane = tid & 63;
    const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
    const int wm = wave / WN, wn = wave % WN;
    // consecutive workgroup ids of one XCD (ids congruent modulo 8) walk down a column of tiles, so that an XCD's
    // L2 keeps one weight panel and streams activations
    int bid = blockIdx.x;
    const int total = tiles_m * tiles_n, per_xcd = total / 8;
    if (bid < per_xcd * 8) bid = (bid & 7) * per_xcd + (bid >> 3);
    const int tm = bid % tiles_m, tn = bid / tiles_m;
    const int m0 = tm * BM, n0 = tn * BN;
    const int ktiles = k / BK;
    const size_t a_pitch = (size_t)k * 2;
    const size_t b_row_bytes = W4 ? (size_t)k / 2 : (size_t)k;
    const size_t b_blk = b_row_bytes * 32;  // bytes per block of 32 output channels
    const int row_last = m - 1 - m0, blk_last = n / 32 - 1 - n0 / 32;
    const u32 smem_base = (u32)(uintptr_t)(__attribute__((address_space(3))) char*)wo_smem;

    // ---- global -> LDS transfers without registers: lane l of a transfer lands at (transfer base) + 16*l, so the
    // XOR swizzle of the activation tile is applied by choosing WHICH global chunk each lane fetches ----------------
    const char* a_tile = static_cast<const char*>(A) + (size_t)m0 * a_pitch;
    const char* b_tile = reinterpret_cast<const char*>(B) + (size_t)(n0 / 32) * b_blk;
    u32 a_voff[A_DMA], b_voff[B_DMA];
#pragma unroll
    for (int i = 0; i < A_DMA; ++i) {
        const int slot = (wave * A_DMA + i) * 64 + lane;  // 16-byte slot of the activation stage: [row][8 chunks]
        const int row = slot >> 3, c = (slot & 7) ^ wo_swizzle<8>(row);
        a_voff[i] = (u32)min(row, row_last) * (u32)a_pitch + c * 16;
    }
#pragma unroll
    for (int i = 0; i < B_DMA; ++i) {
        const int slot = (wave * B_DMA + i) * 64 + lane;  // [block of 32 channels][chunk][row in block], as in memory
        const int blk = slot / (BCH * 32), within = slot % (BCH * 32);
        b_voff[i] = (u32)((size_t)min(blk, blk_last) * b_blk) + within * 16;
    }
    // group scales / zeros: lane l of a transfer fetches the pair of channels (2l, 2l+1) of its half of the tile's
    // columns; BN / 128 wavefronts cover the tile, the others repeat them (same bytes to the same place)
    const int sz_part = BN == 256 ? (wave & 1) : 0;
    const u32 sz_voff = (u32)min(n0 + sz_part * 128 + 2 * lane, n - 2) * 2u;
    // transfers lo..hi-1 of tile kt (activations, weights, then the group scales and zeros); lo and hi are compile-time
    // values after unrolling
    auto issue_range = [&](int kt, int stage, int lo, int hi) {
        const char* ga = a_tile + (size_t)kt * (BK * 2);
        const char* gb = b_tile + (size_t)kt * (BCH * 512);
        const u32 sa = smem_base + stage * STAGE + wave * (A_DMA * 1024);
        const u32 sb = smem_base + stage * STAGE + A_BYTES + wave * (B_DMA * 1024);
#pragma unroll
        for (int d = 0; d < PER_TILE; ++d) {
            if (d < lo || d >= hi) continue;
            if (d < A_DMA) dma16(ga, a_voff[d < A_DMA ? d : 0], sa + d * 1024);
            else if (d < A_DMA + B_DMA) dma16(gb, b_voff[d >= A_DMA && d < A_DMA + B_DMA ? d - A_DMA : 0], sb + (d - A_DMA) * 1024);
            else {
                const size_t grow = (size_t)(kt / tiles_per_group) * (size_t)n * 2;
                const u32 ss = smem_base + stage * STAGE + A_BYTES + B_BYTES + sz_part * 256;
                if (d == A_DMA + B_DMA) dma4(static_cast<const char*>(scales) + grow, sz_voff, ss);
                else dma4(static_cast<const char*>(zeros) + grow, sz_voff, ss + 512);
            }
        }
    };
    auto issue = [&](int kt, int stage) { issue_range(kt, stage, 0, PER_TILE); };

    v16f acc[MT][NT];
#pragma unroll
    for (int i = 0; i < MT; ++i)
#pragma unroll
        for (int j = 0; j < NT; ++j)
#pragma unroll
            for (int v = 0; v < 16; ++v) acc[i][j][v] = 0.0f;

    const int lr = lane & 31, lh = lane >> 5;
    const int xrow = wm * TM + lr;
    const int xsw = wo_swizzle<8>(xrow);  // unchanged by +32*i
    // One k-tile = 16 steps (half, s, i): one 16-byte activation fragment and NT MFMAs each.  Fragments are read two
    // steps ahead of their use and the order "read, NT MFMAs" is pinned with scheduling barriers, so that the matrix
    // pipe does not wait for an LDS round trip at every step; the weights of the second half are converted while
    // the MFMAs of the first half run.
    // (with three stages the transfers of tile kt_next go out one or two at a time between the steps: a wavefront that
    // stalls on a full memory-instruction queue cannot issue its next MFMA)
    auto compute = [&](int stage, int kt_next, int stage_next) {
        const char* sa = wo_smem + stage * STAGE;
        const char* sb = sa + A_BYTES + (wn * NT) * (BCH * 512) + lr * 16;
        auto xptr = [&](int t) -> const v4i* {
            const int half = t >> 3, s2 = (t >> 2) & 1, i = t & 3;
            const int chunk = W4 ? lh * 4 + half * 2 + s2 : half * 4 + lh * 2 + s2;
            return reinterpret_cast<const v4i*>(sa + (xrow + i * 32) * 128 + ((chunk ^ xsw) << 4));
        };
        v4i wraw[2][NT];  // int8: one 16-byte chunk per half; int4: one chunk for the whole tile (kept in wraw[0])
#pragma unroll
        for (int j = 0; j < NT; ++j) {
            if constexpr (W4) wraw[0][j] = *reinterpret_cast<const v4i*>(sb + j * (BCH * 512) + lh * 512);
            else {
                wraw[0][j] = *reinterpret_cast<const v4i*>(sb + j * (BCH * 512) + lh * 512);
                wraw[1][j] = *reinterpret_cast<const v4i*>(sb + j * (BCH * 512) + (2 + lh) * 512);
            }
        }
        // the scale (and zero) of the lane's output channel in each of its NT column tiles: a pair of fp16, or fp32 bits
        u32 gs[NT], gz[NT];
#pragma unroll
        for (int j = 0; j < NT; ++j) {
            gs[j] = gz[j] = 0;
            if constexpr (GROUPED >= 1) {
                const char* szp = sa + A_BYTES + B_BYTES + ((wn * NT + j) * 32 + lr) * 2;
                const u32 sv = *reinterpret_cast<const unsigned short*>(szp);
                gs[j] = F16 ? (sv | (sv << 16)) : (sv << 16);
                if constexpr (GROUPED == 2) {
                    const u32 zv = *reinterpret_cast<const unsigned short*>(szp + 512);
                    gz[j] = F16 ? (zv | (zv << 16)) : (zv << 16);
                }
            }
        }
        v4i xb[3];
        xb[0] = *xptr(0);
        xb[1] = *xptr(1);
        v4i wfrag[2][NT][2];
        auto convert = [&](int half) {
#pragma unroll
            for (int j = 0; j < NT; ++j) {
                if constexpr (W4) {
                    wfrag[half][j][0] = WoCvt<F16, true, GROUPED>::run((u32)(half ? wraw[0][j][2] : wraw[0][j][0]), 0u, gs[j], gz[j]);
                    wfrag[half][j][1] = WoCvt<F16, true, GROUPED>::run((u32)(half ? wraw[0][j][3] : wraw[0][j][1]), 0u, gs[j], gz[j]);
                } else {
                    wfrag[half][j][0] = WoCvt<F16, false, GROUPED>::run((u32)wraw[half][j][0], (u32)wraw[half][j][1], gs[j], gz[j]);
                    wfrag[half][j][1] = WoCvt<F16, false, GROUPED>::run((u32)wraw[half][j][2], (u32)wraw[half][j][3], gs[j], gz[j]);
                }
            }
        };
        convert(0);
#pragma unroll
        for (int t = 0; t < 16; ++t) {
            const int half = t >> 3, s2 = (t >> 2) & 1, i = t & 3;
            if constexpr (NSTAGE >= 3) issue_range(kt_next, stage_next, t * PER_TILE / 16, (t + 1) * PER_TILE / 16);
            if (t + 2 < 16) xb[(t + 2) % 3] = *xptr(t + 2);
            if (t == 2) convert(1);
            const v4i x = xb[t % 3];
#pragma unroll
            for (int j = 0; j < NT; ++j) {
                const v4i w = wfrag[half][j][s2];
                if constexpr (F16)
                    acc[i][j] = __builtin_amdgcn_mfma_f32_32x32x16_f16(__builtin_bit_cast(v8h, w), __builtin_bit_cast(v8h, x), acc[i][j], 0, 0, 0);
                else
                    acc[i][j] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(__builtin_bit_cast(v8bf, w), __builtin_bit_cast(v8bf, x), acc[i][j], 0, 0, 0);
            }
        }
        // pin the order: the weight chunks and the first two fragments, then (NT MFMAs, one LDS read) x 14, then the
        // MFMAs of the last two steps
        __builtin_amdgcn_sched_group_barrier(0x100, (W4 ? NT : 2 * NT) + 2 + GROUPED * NT, 0);  // DS reads
#pragma unroll
        for (int t = 0; t < 14; ++t) {
            __builtin_amdgcn_sched_group_barrier(0x008, NT, 0);  // MFMA
            __builtin_amdgcn_sched_group_barrier(0x100, 1, 0);   // DS read
        }
        __builtin_amdgcn_sched_group_barrier(0x008, 2 * NT, 0);
    };

    // Tile t lives in stage t % NSTAGE.  Every iteration issues exactly one tile of transfers (past the end it
    // re-fetches the last tile into a stage nobody reads again), so the vmcnt threshold is a compile-time value:
    // when at most (NSTAGE-2) tiles of this wavefront's transfers are outstanding, its part of tile kt has landed;
    // after the barrier everybody's has, and everybody has finished reading the stage that is re-armed next.
#pragma unroll
    for (int t = 0; t < NSTAGE - 1; ++t) issue(min(t, ktiles - 1), t);
    for (int kt = 0; kt < ktiles; ++kt) {
        wait_vmcnt<PER_TILE*(NSTAGE - 2)>();
        __syncthreads();
        // two stages: the next tile must be on its way for the whole of this one, so its transfers go out at once
        if constexpr (NSTAGE < 3) issue(min(kt + NSTAGE - 1, ktiles - 1), (kt + NSTAGE - 1) % NSTAGE);
        compute(kt % NSTAGE, min(kt + NSTAGE - 1, ktiles - 1), (kt + NSTAGE - 1) % NSTAGE);
    }
    wait_vmcnt<0>();  // nothing in flight towards LDS when the workgroup ends

    // ---- epilogue: weights were the first MFMA operand, so a lane holds one activation row (lr) and, per tile,
    // four runs of four consecutive output channels: 8-byte stores -------------------------------------------------
    const int mrow0 = m0 + wm * TM + lr;
#pragma unroll
    for (int j = 0; j < NT; ++j) {
        const int nb = n0 + wn * TN + j * 32;
        float sc[16], bs[16];
#pragma unroll
        for (int q4 = 0; q4 < 4; ++q4) {
            const int nn = nb + q4 * 8 + lh * 4;
            const bool ok = nn < n;
            uint2 sv = make_uint2(0, 0), bv = make_uint2(0, 0);
            if (ok && GROUPED == 0) sv = *reinterpret_cast<const uint2*>(static_cast<const unsigned short*>(scales) + nn);
            if (ok && bias != nullptr) bv = *reinterpret_cast<const uint2*>(static_cast<const unsigned short*>(bias) + nn);
            sc[q4 * 4] = Elem<Tag>::load(sv.x & 0xFFFFu); sc[q4 * 4 + 1] = Elem<Tag>::load(sv.x >> 16);
            sc[q4 * 4 + 2] = Elem<Tag>::load(sv.y & 0xFFFFu); sc[q4 * 4 + 3] = Elem<Tag>::load(sv.y >> 16);
            bs[q4 * 4] = Elem<Tag>::load(bv.x & 0xFFFFu); bs[q4 * 4 + 1] = Elem<Tag>::load(bv.x >> 16);
            bs[q4 * 4 + 2] = Elem<Tag>::load(bv.y & 0xFFFFu); bs[q4 * 4 + 3] = Elem<Tag>::load(bv.y >> 16);
        }
#pragma unroll
        for (int i = 0; i < MT; ++i) {
            const int mr = mrow0 + i * 32;
            if (mr >= m) continue;
#pragma unroll
            for (int q4 = 0; q4 < 4; ++q4) {
                const int nn = nb + q4 * 8 + lh * 4;
                if (nn >= n) continue;
                float y[4];
#pragma unroll
                for (int e = 0; e < 4; ++e) {
                    y[e] = GROUPED == 0 ? acc[i][j][q4 * 4 + e] * sc[q4 * 4 + e] : acc[i][j][q4 * 4 + e];
                    if (bias != nullptr) y[e] = y[e] + bs[q4 * 4 + e];
                }
                uint2 o;
                if constexpr (F16) { o.x = pack2_f16(y[0], y[1]); o.y = pack2_f16(y[2], y[3]); }
                else { o.x = pack2_bf16(y[0], y[1]); o.y = pack2_bf16(y[2], y[3]); }
                *reinterpret_cast<uint2*>(static_cast<unsigned short*>(C) + (size_t)mr * n + nn) = o;
            }
        }
    }
}

// ---- one-time weight preparation: [k, n] signed codes (int8, or int4 pairs packed along n, low nibble = even
// column) -> the layout described at the top.  One thread per 16-byte destination chunk. ---------------------------
template <bool W4>
__global__ __launch_bounds__(256) void wo_repack_kernel(uint8_t* __restrict__ dst, const int8_t* __restrict__ src, size_t k, size_t n) {
    const size_t row_bytes = W4 ? k / 2 : k, kc_count = row_bytes / 16, total = n * kc_count;
    for (size_t t = (size_t)blockIdx.x * blockDim.x + threadIdx.x; t < total; t += (size_t)gridDim.x * blockDim.x) {
        const size_t r = t & 31, rest = t >> 5, kc = rest % kc_count, nb = rest / kc_count;
        const size_t col = nb * 32 + r;
        u32 w[4] = {0, 0, 0, 0};
        if constexpr (W4) {
            const size_t kbase = kc * 32;  // 32 weights per chunk
            const uint8_t* s = reinterpret_cast<const uint8_t*>(src) + col / 2;
            const int sh = (col & 1) * 4;
#pragma unroll
            for (int e = 0; e < 32; ++e) {
                const u32 code = ((((u32)s[(kbase + e) * (n / 2)] >> sh) & 0xFu) + 8u) & 0xFu;  // two's complement nibble + 8
                const int j = e & 7, pos = (j & 1) * 4 + (j >> 1);                             // k0 k2 k4 k6 | k1 k3 k5 k7
                w[e >> 3] |= code << (4 * pos);
            }
        } else {
            const size_t kbase = kc * 16;
#pragma unroll
            for (int e = 0; e < 16; ++e) w[e >> 2] |= (u32)(uint8_t)(src[(kbase + e) * n + col] + 128) << (8 * (e & 3));
        }
        *reinterpret_cast<uint4*>(dst + t * 16) = make_uint4(w[0], w[1], w[2], w[3]);
    }
}

}  // namespace lq

using namespace lq;

extern "C" int lq_repack_weight_only(uint8_t* dst, const int8_t* src_kn, lq_weight_kind_t kind, size_t k, size_t n,
                                     lq_stream_t stream) {
    LQ_REQUIRE(dst && src_kn, LQ_ERR_ARG, "lq_repack_weight_only: null pointer");
    LQ_REQUIRE(kind == LQ_W_INT8 || kind == LQ_W_INT4, LQ_ERR_UNSUPPORTED, "lq_repack_weight_only: kind must be INT8 or INT4");
    LQ_REQUIRE(n % 32 == 0 && k % 64 == 0 && n > 0 && k > 0, LQ_ERR_SHAPE,
               "lq_repack_weight_only: need n %% 32 == 0 and k %% 64 == 0 (k=%zu n=%zu)", k, n);
    LQ_REQUIRE(reinterpret_cast<uintptr_t>(dst) % 16 == 0, LQ_ERR_ARG, "lq_repack_weight_only: dst must be 16-byte aligned");
    const size_t chunks = n * ((kind == LQ_W_INT4 ? k / 2 : k) / 16);
    const unsigned blocks = (unsigned)std::min<size_t>((chunks + 255) / 256, 65535);
    if (kind == LQ_W_INT4) hipLaunchKernelGGL((wo_repack_kernel<true>), dim3(blocks), dim3(256), 0, as_stream(stream), dst, src_kn, k, n);
    else hipLaunchKernelGGL((wo_repack_kernel<false>), dim3(blocks), dim3(256), 0, as_stream(stream), dst, src_kn, k, n);
    return check_launch("wo_repack");
}

static int wo_launch(void* C, const void* A, lq_dtype_t dtype, const uint8_t* B_prepared, lq_weight_kind_t kind, const void* scales,
                     const void* zeros, const void* bias, int m, int n, int k, int group_size, lq_stream_t stream) {
    const bool w4 = kind == LQ_W_INT4;
    const int grouped = group_size == 0 ? 0 : (zeros == nullptr ? 1 : 2);
    const int tiles_per_group = group_size == 0 ? 1 : group_size / 64;
    // 256x256 tiles (eight wavefronts, three stages) once they give every CU work; 256x128 tiles otherwise
    // A tile configuration set with lq_gemm_set_thread_tactic wins: 0 = 256x256, 1 = 256x128.
    const long big_tiles = (long)((m + 255) / 256) * ((n + 255) / 256);
    if (tl_forced_tactic > 1) {
        set_error("gemm_weight_only: unknown tile configuration %d (0 = 256x256, 1 = 256x128)", tl_forced_tactic);
        return LQ_ERR_ARG;
    }
    const bool big = tl_forced_tactic >= 0 ? tl_forced_tactic == 0 : big_tiles >= 192;
    hipStream_t st = as_stream(stream);
#define LQ_WO_GO(TAG, W4V, WNV, NST, GRP)                                                                               \
    do {                                                                                                                \
        constexpr size_t lds = (size_t)(NST) * (256 * 64 * 2 + 64 * (WNV) * ((W4V) ? 2 : 4) * 16 + ((GRP) ? 1024 : 0)); \
        static bool attr_done = false;                                                                                  \
        if (!attr_done) {                                                                                               \
            if (hipFuncSetAttribute(reinterpret_cast<const void*>(&wo_gemm_kernel<TAG, W4V, WNV, NST, GRP>),            \
                                    hipFuncAttributeMaxDynamicSharedMemorySize, (int)lds) != hipSuccess) {              \
                set_error("lq_gemm_weight_only: cannot raise the dynamic LDS limit to %zu bytes", lds);                 \
                return LQ_ERR_HIP;                                                                                      \
            }                                                                                                           \
            attr_done = true;                                                                                           \
        }                                                                                                               \
        const int tiles_m = (m + 255) / 256, tiles_n = (n + 64 * (WNV) - 1) / (64 * (WNV));                             \
        hipLaunchKernelGGL((wo_gemm_kernel<TAG, W4V, WNV, NST, GRP>), dim3((unsigned)(tiles_m * tiles_n)),              \
                           dim3(128 * (WNV)), lds, st, C, A, B_prepared, scales, zeros, bias, m, n, k, tiles_m, tiles_n, \
                           tiles_per_group);                                                                            \
    } while (0)
#define LQ_WO_SIZE(TAG, W4V, GRP)                  \
    do {                                           \
        if (big) LQ_WO_GO(TAG, W4V, 4, 3, GRP);    \
        else LQ_WO_GO(TAG, W4V, 2, 2, GRP);        \
    } while (0)
#define LQ_WO_KIND(TAG, GRP)                       \
    do {                                           \
        if (w4) LQ_WO_SIZE(TAG, true, GRP);        \
        else LQ_WO_SIZE(TAG, false, GRP);          \
    } while (0)
#define LQ_WO_GRP(TAG)                             \
    do {                                           \
        if (grouped == 0) LQ_WO_KIND(TAG, 0);      \
        else if (grouped == 1) LQ_WO_KIND(TAG, 1); \
        else LQ_WO_KIND(TAG, 2);                   \
    } while (0)
    if (dtype == LQ_F16) LQ_WO_GRP(F16Tag);
    else LQ_WO_GRP(BF16Tag);
#undef LQ_WO_GRP
#undef LQ_WO_KIND
#undef LQ_WO_SIZE
#undef LQ_WO_GO
    return check_launch("gemm_weight_only");
}

static int wo_check(const char* what, void* C, const void* A, lq_dtype_t dtype, const uint8_t* B_prepared, lq_weight_kind_t kind,
                    const void* scales, const void* zeros, const void* bias, int m, int n, int k) {
    LQ_REQUIRE(C && A && B_prepared && scales, LQ_ERR_ARG, "%s: null pointer", what);
    LQ_REQUIRE(dtype == LQ_F16 || dtype == LQ_BF16, LQ_ERR_UNSUPPORTED, "%s: activations must be F16 or BF16", what);
    LQ_REQUIRE(kind == LQ_W_INT8 || kind == LQ_W_INT4, LQ_ERR_UNSUPPORTED, "%s: kind must be INT8 or INT4", what);
    LQ_REQUIRE(m >= 0 && n > 0 && k > 0 && n % 32 == 0 && k % 64 == 0, LQ_ERR_SHAPE,
               "%s: need n %% 32 == 0 and k %% 64 == 0 (m=%d n=%d k=%d)", what, m, n, k);
    LQ_REQUIRE(reinterpret_cast<uintptr_t>(A) % 16 == 0 && reinterpret_cast<uintptr_t>(B_prepared) % 16 == 0 &&
                   reinterpret_cast<uintptr_t>(C) % 8 == 0 && reinterpret_cast<uintptr_t>(scales) % 8 == 0 &&
                   reinterpret_cast<uintptr_t>(zeros) % 8 == 0 && reinterpret_cast<uintptr_t>(bias) % 8 == 0,
               LQ_ERR_ARG, "%s: A and B must be 16-byte, C, scales, zeros and bias 8-byte aligned", what);
    return LQ_OK;
}

extern "C" int lq_gemm_weight_only(void* C, const void* A, lq_dtype_t dtype, const uint8_t* B_prepared, lq_weight_kind_t kind,
                                   const void* scales, const void* bias, int m, int n, int k, lq_stream_t stream) {
    int rc = wo_check("lq_gemm_weight_only", C, A, dtype, B_prepared, kind, scales, nullptr, bias, m, n, k);
    if (rc != LQ_OK) return rc;
    if (m == 0) return LQ_OK;
    return wo_launch(C, A, dtype, B_prepared, kind, scales, nullptr, bias, m, n, k, 0, stream);
}

extern "C" int lq_gemm_weight_only_grouped(void* C, const void* A, lq_dtype_t dtype, const uint8_t* B_prepared,
                                           lq_weight_kind_t kind, const void* scales, const void* zeros, const void* bias, int m,
                                           int n, int k, int group_size, lq_stream_t stream) {
    int rc = wo_check("lq_gemm_weight_only_grouped", C, A, dtype, B_prepared, kind, scales, zeros, bias, m, n, k);
    if (rc != LQ_OK) return rc;
    LQ_REQUIRE((group_size == 64 || group_size == 128) && k % group_size == 0, LQ_ERR_SHAPE,
               "lq_gemm_weight_only_grouped: group_size must be 64 or 128 and divide k (group_size=%d k=%d)", group_size, k);
    if (m == 0) return LQ_OK;
    return wo_launch(C, A, dtype, B_prepared, kind, scales, zeros, bias, m, n, k, group_size, stream);
}
