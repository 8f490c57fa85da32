// Tiled quantized GEMM core for gfx950 (MI355X): C[M,N] = epilogue( A[M,K] . B[N,K]^T ).
//
// Data flow per workgroup (BM x BN output tile, K walked in steps of BKB bytes):
//   HBM --128-bit loads--> VGPR --ds_write_b128--> LDS (2 stages) --ds_read_b128--> MFMA operands.
//   * B (weights) arrive in the rows32 layout [N/32][Kb/16][32][16]: the bytes a 32x32 MFMA
//     needs for one k-step are 1 KiB contiguous in HBM and in LDS, so a lane's operand is a
//     single 16-byte read at a lane-linear LDS address (conflict free).
//   * A (activations) are row-major [M,Kb]; the LDS tile keeps rows contiguous and XOR-swizzles
//     the 16-byte chunk index with row bits so that both the row-wise stores and the
//     column-wise (32 rows x one chunk) operand reads are conflict free.
//   * The MFMA "A" operand carries 32 weight rows (n) and the "B" operand 32 activation rows
//     (m): a lane then holds, for one m, four consecutive n per register quad, which packs into
//     one 8-byte (16-bit outputs) or 16-byte (32-bit outputs) store.
//   * INT8: v_mfma_i32_32x32x32_i8, FP8: v_mfma_f32_32x32x64_f8f6f4 (both operands e4m3),
//     W4A4: nibbles are widened in registers to int8 values 16x too large (the nibble is moved
//     to the high half of its byte), multiplied on the int8 MFMA per 64-wide group, and the
//     factor 256 is folded into the activation group scale (a power of two, exact).
//   * Workgroup ids are remapped so that the workgroups an XCD receives (ids congruent mod 8)
//     cover a compact block of tiles and share operands through that XCD's L2.
#pragma once

#include <type_traits>

#include "lq_common.h"

namespace lq {

enum GemmKind { K_INT8 = 0, K_FP8 = 1, K_W4A4 = 2 };

struct GemmParams {
    void* C;
    const uint8_t* A;
    const uint8_t* B;
    const void* bias;
    // int8
    const float* alpha_col;
    const float* alpha_row;
    int per_token;
    // fp8
    const float* a_scale;
    const float* b_scale;
    int gelu;
    const void* residual;
    float beta;
    // w4a4
    const void* sA;
    const void* sB;
    int scale_f16;
    int m, n, k;
    int kb;  // bytes per operand row: k (int8/fp8) or k/2 (int4)
    int tiles_m, tiles_n;
};

template <int CH> __device__ __forceinline__ int chunk_swizzle(int row) {
    if constexpr (CH == 4) return ((row >> 2) & 3) ^ (((row >> 1) & 1) << 1);
    else if constexpr (CH == 8) return ((row >> 1) & 7) ^ ((row & 1) << 2);
    else return 0;
}

// Remap the linear workgroup id so that ids congruent modulo 8 (one XCD) get consecutive tile
// numbers, then walk tiles in bands of GROUP_M tile rows (column-major inside a band).
__device__ __forceinline__ void tile_coords(int bid, int tiles_m, int tiles_n, int& tm, int& tn) {
    const int total = tiles_m * tiles_n;
    const int per_xcd = total / 8;
    int pid = bid;
    if (bid < per_xcd * 8) pid = (bid & 7) * per_xcd + (bid >> 3);
    constexpr int GROUP_M = 4;
    const int band = GROUP_M * tiles_n;
    const int first_m = (pid / band) * GROUP_M;
    const int rows = min(tiles_m - first_m, GROUP_M);
    const int in_band = pid % band;
    tm = first_m + in_band % rows;
    tn = in_band / rows;
}

template <typename OutTag> struct OutStore;
template <> struct OutStore<F16Tag> {
    static __device__ __forceinline__ void store4(void* C, size_t idx, const float* y) {
        uint2 o;
        o.x = f32_to_f16_bits(y[0]) | (f32_to_f16_bits(y[1]) << 16);
        o.y = f32_to_f16_bits(y[2]) | (f32_to_f16_bits(y[3]) << 16);
        *reinterpret_cast<uint2*>(static_cast<unsigned short*>(C) + idx) = o;
    }
    static __device__ __forceinline__ void load4(const void* P, size_t idx, float* y) {
        uint2 v = *reinterpret_cast<const uint2*>(static_cast<const unsigned short*>(P) + idx);
        y[0] = f16_bits_to_f32(v.x & 0xFFFF); y[1] = f16_bits_to_f32(v.x >> 16);
        y[2] = f16_bits_to_f32(v.y & 0xFFFF); y[3] = f16_bits_to_f32(v.y >> 16);
    }
};
template <> struct OutStore<BF16Tag> {
    static __device__ __forceinline__ void store4(void* C, size_t idx, const float* y) {
        uint2 o;
        o.x = f32_to_bf16_bits(y[0]) | (f32_to_bf16_bits(y[1]) << 16);
        o.y = f32_to_bf16_bits(y[2]) | (f32_to_bf16_bits(y[3]) << 16);
        *reinterpret_cast<uint2*>(static_cast<unsigned short*>(C) + idx) = o;
    }
    static __device__ __forceinline__ void load4(const void* P, size_t idx, float* y) {
        uint2 v = *reinterpret_cast<const uint2*>(static_cast<const unsigned short*>(P) + idx);
        y[0] = bf16_bits_to_f32(v.x & 0xFFFF); y[1] = bf16_bits_to_f32(v.x >> 16);
        y[2] = bf16_bits_to_f32(v.y & 0xFFFF); y[3] = bf16_bits_to_f32(v.y >> 16);
    }
};
template <> struct OutStore<F32Tag> {
    static __device__ __forceinline__ void store4(void* C, size_t idx, const float* y) {
        *reinterpret_cast<float4*>(static_cast<float*>(C) + idx) = make_float4(y[0], y[1], y[2], y[3]);
    }
    static __device__ __forceinline__ void load4(const void* P, size_t idx, float* y) {
        float4 v = *reinterpret_cast<const float4*>(static_cast<const float*>(P) + idx);
        y[0] = v.x; y[1] = v.y; y[2] = v.z; y[3] = v.w;
    }
};
struct I32Tag {};

// GELU for the fused FP8 epilogue: hardware exp2 / reciprocal (the reference's counterpart is
// cuBLASLt's GELU epilogue, utils/cublasMMWrapper.cc:1195-1199, whose arithmetic is not visible).
__device__ __forceinline__ float gelu_fast(float x) {
    float inner = 0.7978845608028654f * (x + 0.044715f * x * x * x);
    float e = __builtin_amdgcn_exp2f(inner * 2.8853900817779268f);  // exp(2*inner)
    float t = 1.0f - 2.0f * __builtin_amdgcn_rcpf(e + 1.0f);        // tanh(inner); e=inf -> 1
    return 0.5f * x * (1.0f + t);
}

template <int KIND, typename OutTag, int BM, int BN, int BKB, int WM, int WN>
struct GemmKernel {
    static constexpr int THREADS = WM * WN * 64;
    static constexpr int TM = BM / WM, TN = BN / WN;  // wavefront tile
    static constexpr int MT = TM / 32, NT = TN / 32;  // 32x32 MFMA tiles per wavefront
    static constexpr int CH = BKB / 16;               // 16-byte chunks per tile row
    static constexpr int A_BYTES = BM * BKB, B_BYTES = BN * BKB;
    static constexpr int SCALE_BYTES = (KIND == K_W4A4) ? (BM + BN) * (BKB / 32) * 4 : 0;
    static constexpr int STAGE_BYTES = A_BYTES + B_BYTES + SCALE_BYTES;
    static constexpr int SMEM_BYTES = 2 * STAGE_BYTES;
    static constexpr int ACH = A_BYTES / 16 / THREADS, BCH = B_BYTES / 16 / THREADS;
    static_assert(A_BYTES % (16 * THREADS) == 0 && B_BYTES % (16 * THREADS) == 0, "tile/threads mismatch");
    static_assert(TM % 32 == 0 && TN % 32 == 0, "wave tile must be a multiple of 32");
    static_assert(CH == 4 || CH == 8, "BKB must be 64 or 128");
    using AccT = typename std::conditional<KIND == K_FP8, v16f, v16i>::type;

    static __device__ __forceinline__ void run(const GemmParams& p, char* smem) {
        const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
        const int wm = wave / WN, wn = wave % WN;
        int tm, tn;
        tile_coords(blockIdx.x, p.tiles_m, p.tiles_n, tm, tn);
        const int m0 = tm * BM, n0 = tn * BN;
        const int kb = p.kb;
        const int ktiles = kb / BKB;
        const int nb_last = p.n / 32 - 1;
        const size_t b_block_stride = (size_t)(kb / 16) * 512;  // bytes per 32-row block in rows32 layout

        // ---- global -> register staging ------------------------------------------------------
        uint4 ra[ACH], rb[BCH];
        const uint8_t* a_src[ACH];
        const uint8_t* b_src[BCH];
        int a_dst[ACH];
#pragma unroll
        for (int i = 0; i < ACH; ++i) {
            int q = tid + i * THREADS, row = q / CH, c = q % CH;
            int grow = min(m0 + row, p.m - 1);
            a_src[i] = p.A + (size_t)grow * kb + c * 16;
            a_dst[i] = row * BKB + ((c ^ chunk_swizzle<CH>(row)) << 4);
        }
#pragma unroll
        for (int i = 0; i < BCH; ++i) {
            int q = tid + i * THREADS, rblk = q / (BKB * 2), within = q % (BKB * 2);
            int nb = min(n0 / 32 + rblk, nb_last);
            b_src[i] = p.B + (size_t)nb * b_block_stride + within * 16;
        }
        // W4A4 group scales of a k-tile staged as [NGS][BM] then [NGS][BN] floats (int4: one group
        // of 64 values is 32 bytes); the activation scales absorb the 1/256 of the widened nibbles
        constexpr int NGS = BKB / 32;
        constexpr int NS = NGS * (BM + BN);
        constexpr int SCH = (KIND == K_W4A4) ? (NS + THREADS - 1) / THREADS : 1;
        float rs[SCH];
        auto load_scale = [&](const void* base, size_t idx) -> float {
            if (p.scale_f16) return f16_bits_to_f32(static_cast<const unsigned short*>(base)[idx]);
            return static_cast<const float*>(base)[idx];
        };
        auto load_tile = [&](int kt) {
#pragma unroll
            for (int i = 0; i < ACH; ++i) ra[i] = *reinterpret_cast<const uint4*>(a_src[i] + (size_t)kt * BKB);
#pragma unroll
            for (int i = 0; i < BCH; ++i) rb[i] = *reinterpret_cast<const uint4*>(b_src[i] + (size_t)kt * BKB * 32);
            if constexpr (KIND == K_W4A4) {
                const int ng = p.k / 64;
#pragma unroll
                for (int i = 0; i < SCH; ++i) {
                    int s = tid + i * THREADS;
                    rs[i] = 0.0f;
                    if (s < NGS * BM) {
                        int g = s / BM, r = s % BM;
                        int row = min(m0 + r, p.m - 1);
                        rs[i] = load_scale(p.sA, (size_t)row * ng + kt * NGS + g) * 0.00390625f;
                    } else if (s < NS) {
                        int t2 = s - NGS * BM;
                        int g = t2 / BN, r = t2 % BN;
                        int row = min(n0 + r, p.n - 1);
                        rs[i] = load_scale(p.sB, (size_t)row * ng + kt * NGS + g);
                    }
                }
            }
        };
        auto store_tile = [&](int stage) {
            char* sa = smem + stage * STAGE_BYTES;
            char* sb = sa + A_BYTES;
#pragma unroll
            for (int i = 0; i < ACH; ++i) *reinterpret_cast<uint4*>(sa + a_dst[i]) = ra[i];
#pragma unroll
            for (int i = 0; i < BCH; ++i) *reinterpret_cast<uint4*>(sb + (tid + i * THREADS) * 16) = rb[i];
            if constexpr (KIND == K_W4A4) {
#pragma unroll
                for (int i = 0; i < SCH; ++i)
                    if (tid + i * THREADS < NS) reinterpret_cast<float*>(sb + B_BYTES)[tid + i * THREADS] = rs[i];
            }
        };

        // ---- accumulators ----------------------------------------------------------------------
        AccT acc[MT][NT];
        v16f res[KIND == K_W4A4 ? MT : 1][KIND == K_W4A4 ? NT : 1];
#pragma unroll
        for (int i = 0; i < MT; ++i)
#pragma unroll
            for (int j = 0; j < NT; ++j)
#pragma unroll
                for (int v = 0; v < 16; ++v) {
                    acc[i][j][v] = 0;
                    if constexpr (KIND == K_W4A4) res[i][j][v] = 0.0f;
                }

        const int lr = lane & 31, lh = lane >> 5;
        auto compute_tile = [&](int stage) {
            const char* sa = smem + stage * STAGE_BYTES;
            const char* sb = sa + A_BYTES;
            if constexpr (KIND == K_INT8) {
#pragma unroll
                for (int ks = 0; ks < BKB / 32; ++ks) {
                    v4i w[NT], x[MT];
#pragma unroll
                    for (int j = 0; j < NT; ++j)
                        w[j] = *reinterpret_cast<const v4i*>(sb + (wn * NT + j) * (BKB * 32) + ks * 1024 + lane * 16);
#pragma unroll
                    for (int i = 0; i < MT; ++i) {
                        int row = wm * TM + i * 32 + lr, c = 2 * ks + lh;
                        x[i] = *reinterpret_cast<const v4i*>(sa + row * BKB + ((c ^ chunk_swizzle<CH>(row)) << 4));
                    }
#pragma unroll
                    for (int i = 0; i < MT; ++i)
#pragma unroll
                        for (int j = 0; j < NT; ++j)
                            acc[i][j] = __builtin_amdgcn_mfma_i32_32x32x32_i8(w[j], x[i], acc[i][j], 0, 0, 0);
                }
            } else if constexpr (KIND == K_FP8) {
#pragma unroll
                for (int ks = 0; ks < BKB / 64; ++ks) {
                    v8i w[NT], x[MT];
#pragma unroll
                    for (int j = 0; j < NT; ++j) {
                        const char* base = sb + (wn * NT + j) * (BKB * 32) + ks * 2048 + lane * 16;
                        v4i lo = *reinterpret_cast<const v4i*>(base);
                        v4i hi = *reinterpret_cast<const v4i*>(base + 1024);
                        w[j] = v8i{lo[0], lo[1], lo[2], lo[3], hi[0], hi[1], hi[2], hi[3]};
                    }
#pragma unroll
                    for (int i = 0; i < MT; ++i) {
                        int row = wm * TM + i * 32 + lr, c0 = 4 * ks + lh, sw = chunk_swizzle<CH>(row);
                        v4i lo = *reinterpret_cast<const v4i*>(sa + row * BKB + ((c0 ^ sw) << 4));
                        v4i hi = *reinterpret_cast<const v4i*>(sa + row * BKB + (((c0 + 2) ^ sw) << 4));
                        x[i] = v8i{lo[0], lo[1], lo[2], lo[3], hi[0], hi[1], hi[2], hi[3]};
                    }
#pragma unroll
                    for (int i = 0; i < MT; ++i)
#pragma unroll
                        for (int j = 0; j < NT; ++j)
                            acc[i][j] = __builtin_amdgcn_mfma_scale_f32_32x32x64_f8f6f4(w[j], x[i], acc[i][j], 0, 0, 0, 0, 0, 0);
                }
            } else {  // W4A4: one 64-value group = 32 bytes = chunks (2g, 2g+1)
                const float* ssa = reinterpret_cast<const float*>(sb + B_BYTES);  // [NGS][BM]
                const float* ssb = ssa + NGS * BM;                                 // [NGS][BN]
#pragma unroll
                for (int g = 0; g < NGS; ++g) {
                    v4i wq[NT], xq[MT];
#pragma unroll
                    for (int j = 0; j < NT; ++j)
                        wq[j] = *reinterpret_cast<const v4i*>(sb + (wn * NT + j) * (BKB * 32) + g * 1024 + lane * 16);
#pragma unroll
                    for (int i = 0; i < MT; ++i) {
                        int row = wm * TM + i * 32 + lr, c = 2 * g + lh;
                        xq[i] = *reinterpret_cast<const v4i*>(sa + row * BKB + ((c ^ chunk_swizzle<CH>(row)) << 4));
                    }
                    float sa_l[MT];
#pragma unroll
                    for (int i = 0; i < MT; ++i) sa_l[i] = ssa[g * BM + wm * TM + i * 32 + lr];
                    // widen: even nibbles -> (d << 4) & 0xF0F0F0F0, odd nibbles -> d & 0xF0F0F0F0
                    auto widen = [](const v4i& q, int half) -> v4i {
                        int d0 = q[2 * half], d1 = q[2 * half + 1];
                        return v4i{(int)(((u32)d0 << 4) & 0xF0F0F0F0u), (int)((u32)d0 & 0xF0F0F0F0u),
                                   (int)(((u32)d1 << 4) & 0xF0F0F0F0u), (int)((u32)d1 & 0xF0F0F0F0u)};
                    };
#pragma unroll
                    for (int j = 0; j < NT; ++j) {
                        v4i w0 = widen(wq[j], 0), w1 = widen(wq[j], 1);
                        float sbv[16];
#pragma unroll
                        for (int q4 = 0; q4 < 4; ++q4) {
                            float4 t = *reinterpret_cast<const float4*>(ssb + g * BN + wn * TN + j * 32 + q4 * 8 + lh * 4);
                            sbv[q4 * 4] = t.x; sbv[q4 * 4 + 1] = t.y; sbv[q4 * 4 + 2] = t.z; sbv[q4 * 4 + 3] = t.w;
                        }
#pragma unroll
                        for (int i = 0; i < MT; ++i) {
                            v4i x0 = widen(xq[i], 0), x1 = widen(xq[i], 1);
                            v16i pz = {0};
                            pz = __builtin_amdgcn_mfma_i32_32x32x32_i8(w0, x0, pz, 0, 0, 0);
                            pz = __builtin_amdgcn_mfma_i32_32x32x32_i8(w1, x1, pz, 0, 0, 0);
#pragma unroll
                            for (int v = 0; v < 16; ++v)
                                res[i][j][v] = __builtin_fmaf((float)pz[v] * sa_l[i], sbv[v], res[i][j][v]);
                        }
                    }
                }
            }
        };

        // ---- main loop: 2 LDS stages, one barrier per k-tile -------------------------------------
        load_tile(0);
        store_tile(0);
        __syncthreads();
        for (int kt = 0; kt < ktiles; ++kt) {
            if (kt + 1 < ktiles) load_tile(kt + 1);
            compute_tile(kt & 1);
            if (kt + 1 < ktiles) store_tile((kt + 1) & 1);
            __syncthreads();
        }

        // ---- epilogue -------------------------------------------------------------------------------
        float alpha = 1.0f;
        if constexpr (KIND == K_FP8) alpha = p.a_scale[0] * p.b_scale[0];
#pragma unroll
        for (int i = 0; i < MT; ++i) {
            const int m = m0 + wm * TM + i * 32 + lr;
            float arow = 1.0f;
            if constexpr (KIND == K_INT8 && !std::is_same<OutTag, I32Tag>::value)
                arow = p.alpha_row[p.per_token ? min(m, p.m - 1) : 0];
#pragma unroll
            for (int j = 0; j < NT; ++j) {
                const int nbase = n0 + wn * TN + j * 32;
                if (nbase >= p.n || m >= p.m) continue;
#pragma unroll
                for (int q4 = 0; q4 < 4; ++q4) {
                    const int n = nbase + q4 * 8 + lh * 4;
                    const size_t idx = (size_t)m * p.n + n;
                    if constexpr (std::is_same<OutTag, I32Tag>::value) {
                        *reinterpret_cast<int4*>(static_cast<int*>(p.C) + idx) =
                            make_int4(acc[i][j][q4 * 4], acc[i][j][q4 * 4 + 1], acc[i][j][q4 * 4 + 2], acc[i][j][q4 * 4 + 3]);
                    } else {
                        float y[4], b[4] = {0.f, 0.f, 0.f, 0.f};
                        if (p.bias != nullptr) OutStore<OutTag>::load4(p.bias, n, b);
                        if constexpr (KIND == K_INT8) {
                            float4 ac = *reinterpret_cast<const float4*>(p.alpha_col + n);
                            const float acv[4] = {ac.x, ac.y, ac.z, ac.w};
#pragma unroll
                            for (int t = 0; t < 4; ++t) {
                                y[t] = (float)acc[i][j][q4 * 4 + t] * (acv[t] * arow);
                                if (p.bias != nullptr) y[t] = y[t] + b[t];
                            }
                        } else if constexpr (KIND == K_FP8) {
#pragma unroll
                            for (int t = 0; t < 4; ++t) {
                                y[t] = acc[i][j][q4 * 4 + t] * alpha;
                                if (p.bias != nullptr) y[t] = y[t] + b[t];
                                if (p.gelu) y[t] = gelu_fast(y[t]);
                            }
                            if (p.residual != nullptr) {
                                float rr[4];
                                OutStore<OutTag>::load4(p.residual, idx, rr);
#pragma unroll
                                for (int t = 0; t < 4; ++t) y[t] = y[t] + p.beta * rr[t];
                            }
                        } else {
#pragma unroll
                            for (int t = 0; t < 4; ++t) {
                                y[t] = res[i][j][q4 * 4 + t];
                                if (p.bias != nullptr) y[t] = y[t] + b[t];
                            }
                        }
                        OutStore<OutTag>::store4(p.C, idx, y);
                    }
                }
            }
        }
    }
};

template <int KIND, typename OutTag, int BM, int BN, int BKB, int WM, int WN>
__global__ __launch_bounds__(WM* WN * 64) void gemm_kernel(GemmParams p) {
    extern __shared__ __attribute__((aligned(16))) char lq_smem[];
    GemmKernel<KIND, OutTag, BM, BN, BKB, WM, WN>::run(p, lq_smem);
}

template <int KIND, typename OutTag, int BM, int BN, int BKB, int WM, int WN>
static int launch_gemm(GemmParams p, hipStream_t st) {
    using GK = GemmKernel<KIND, OutTag, BM, BN, BKB, WM, WN>;
    p.tiles_m = (p.m + BM - 1) / BM;
    p.tiles_n = (p.n + BN - 1) / BN;
    auto kern = gemm_kernel<KIND, OutTag, BM, BN, BKB, WM, WN>;
    static bool attr_done = false;  // raising the dynamic LDS limit is idempotent; races are benign
    if (!attr_done && GK::SMEM_BYTES > 48 * 1024) {
        hipError_t e = hipFuncSetAttribute(reinterpret_cast<const void*>(kern), hipFuncAttributeMaxDynamicSharedMemorySize,
                                           GK::SMEM_BYTES);
        if (e != hipSuccess) {
            set_error("gemm: cannot raise LDS limit to %d bytes: %s", GK::SMEM_BYTES, hipGetErrorString(e));
            return LQ_ERR_HIP;
        }
        attr_done = true;
    }
    dim3 grid((unsigned)(p.tiles_m * p.tiles_n)), block(GK::THREADS);
    hipLaunchKernelGGL(kern, grid, block, GK::SMEM_BYTES, st, p);
    return check_launch("gemm");
}

}  // namespace lq
