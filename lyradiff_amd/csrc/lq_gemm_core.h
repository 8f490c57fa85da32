// Tiled quantized GEMM core for gfx950 (MI355X): C[M,N] = epilogue( A[M,K] . B[N,K]^T ).
//
// Data flow per workgroup (BM x BN output tile, K walked in steps of BKB bytes):
//   HBM --16 B/lane direct-to-LDS transfers--> LDS (NSTAGE stages) --ds_read_b128--> MFMA operands.
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
#include <utility>

#include "lq_common.h"

namespace lq {

// K_W4A4H: W4A4 whose group scales are 16-bit floats; it converts the int32 group sums for free (see
// compute_tile), which is exact only because three times such a scale is still an fp32 number.
enum GemmKind { K_INT8 = 0, K_FP8 = 1, K_W4A4 = 2, K_W4A4H = 3 };

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
    // fp8 and w4a4: activation, residual, re-quantisation and gate epilogues
    int gelu;
    const void* residual;
    float beta;
    float* out_scale;       // optional: max(out_scale, max|C| / 448), the e4m3 scale of the output for a following cast
    float* out_max;         // optional: max(out_max, max over T(C), 0): the largest output, for an activation + cast pass that
                            // derives its scale from it (non-negative floats order like their bit patterns)
    uint8_t* C8;            // optional: e4m3 codes of C with a given (static) scale, written next to or instead of C
    const float* c8_scale;  // scale of C8: C8 = e4m3(f32(T(y)) * (1 / c8_scale[0]))
    size_t ldc8;            // row pitch of C8 in bytes (n when the codes are dense)
    int c8_panel;           // C8 is written as k-panels [n / 64][m][64] (the next GEMM's activation layout, see a_panel); ldc8 unused
    // C is written with nontemporal stores: set for an output that is read once, by one streaming pass (the cast of a
    // dynamic-scale chain: out_scale given), and is too large to share the 256 MB last-level cache with the operands of
    // the GEMM after it.  Measured on the FLUX MLP chain (113 MB hidden tensor): up + cast + down 340-353 -> 319-330 us
    // together with the nontemporal loads of the cast.
    int stream_c;
    // A is stored as k-panels [kb / 64][m][64] instead of row-major [m][kb]: the 64 bytes a k-tile takes from each of a
    // tile's rows are then contiguous (256 rows = 16 KiB, whole 128-byte cache lines), where a row-major operand gives half
    // a line per row and every line is requested from L2 twice, one k-tile apart (TCP_TCC_READ_REQ per launch at
    // 4608x3072x12288: 16.2 M row-major, 10.6 M = the operand bytes / 128 in panels).  Kernels with 64-byte k-tiles only.
    int a_panel;
    // gelu: 0 none, 1 on the fp32 value, 2 on the value rounded to T first (the activation applied by a separate
    // kernel to a stored T tensor)
    // gate: C = T( T( T(y) * gate[m / gate_rows, n] ) + residual[m, n] ), the roundings of a GEMM that stores T
    // followed by an elementwise multiply and add in T; requires residual, ignores beta
    const void* gate;
    size_t gate_rows;
    // addend (optional, [m, n] of T): y = T( T(y) + addend ) before the gate/residual step -- the sum of two linears'
    // outputs as the reference forms it with invokeFusedBiasAndResidual
    const void* addend;
    // w4a4
    const void* sA;
    const void* sB;
    int scale_f16;
    // w4a4 low-rank branch: C += lora_act[m, rank] . lora_up[n, rank]^T (both 16-bit floats, row-major)
    const void* lora_act;
    const void* lora_up;
    int lora_rank;  // multiple of 16
    int lora_f16;   // element type: 1 = fp16, 0 = bf16
    int m, n, k;
    int kb;  // bytes per operand row: k (int8/fp8) or k/2 (int4)
    int tiles_m, tiles_n;
    // persistent kernel: whole-tile rounds per workgroup and the number of half tiles in its last, split round (0: none)
    int persist_rounds, persist_halves;
};

template <int CH> __device__ __forceinline__ int chunk_swizzle(int row) {
    if constexpr (CH == 4) return ((row >> 2) & 3) ^ (((row >> 1) & 1) << 1);
    else if constexpr (CH == 8) return ((row >> 1) & 7) ^ ((row & 1) << 2);
    else return 0;
}

// Remap the linear workgroup id so that ids congruent modulo 8 (one XCD) get consecutive tile
// numbers, then walk tiles in bands of GROUP_M tile rows (column-major inside a band).
template <int GROUP_M>
__device__ __forceinline__ void tile_coords(int bid, int tiles_m, int tiles_n, int& tm, int& tn) {
    const int total = tiles_m * tiles_n;
    const int per_xcd = total / 8;
    int pid = bid;
    if (bid < per_xcd * 8) pid = (bid & 7) * per_xcd + (bid >> 3);
    const int band = GROUP_M * tiles_n;
    const int first_m = (pid / band) * GROUP_M;
    const int rows = min(tiles_m - first_m, GROUP_M);
    const int in_band = pid % band;
    tm = first_m + in_band % rows;
    tn = in_band / rows;
}

// store4_stream: the same store with the nontemporal hint, for an output that one streaming pass reads once (see
// GemmParams::stream_c): its lines then do not displace the next kernel's operands from the last-level cache
template <typename OutTag> struct OutStore;
template <> struct OutStore<F16Tag> {
    static __device__ __forceinline__ void store4(void* C, size_t idx, const float* y) {
        uint2 o;
        o.x = pack2_f16(y[0], y[1]);
        o.y = pack2_f16(y[2], y[3]);
        *reinterpret_cast<uint2*>(static_cast<unsigned short*>(C) + idx) = o;
    }
    static __device__ __forceinline__ void store4_stream(void* C, size_t idx, const float* y) {
        const u32x2_t o = {pack2_f16(y[0], y[1]), pack2_f16(y[2], y[3])};
        __builtin_nontemporal_store(o, reinterpret_cast<u32x2_t*>(static_cast<unsigned short*>(C) + idx));
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
        o.x = pack2_bf16(y[0], y[1]);
        o.y = pack2_bf16(y[2], y[3]);
        *reinterpret_cast<uint2*>(static_cast<unsigned short*>(C) + idx) = o;
    }
    static __device__ __forceinline__ void store4_stream(void* C, size_t idx, const float* y) {
        const u32x2_t o = {pack2_bf16(y[0], y[1]), pack2_bf16(y[2], y[3])};
        __builtin_nontemporal_store(o, reinterpret_cast<u32x2_t*>(static_cast<unsigned short*>(C) + idx));
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
    static __device__ __forceinline__ void store4_stream(void* C, size_t idx, const float* y) { store4(C, idx, y); }
    static __device__ __forceinline__ void load4(const void* P, size_t idx, float* y) {
        float4 v = *reinterpret_cast<const float4*>(static_cast<const float*>(P) + idx);
        y[0] = v.x; y[1] = v.y; y[2] = v.z; y[3] = v.w;
    }
};
struct I32Tag {};

// The wavefront's largest output (>= 0) joins the running maximum of the call.  Rounding to T is monotone, so the maximum
// of the rounded outputs is the rounded maximum.
template <typename OutTag> __device__ __forceinline__ void publish_out_max(float* out_max, float wave_part, int lane) {
    const float mx = round_through<OutTag>(wave_max(wave_part));
    if (lane == 0) {
        const int cur = __hip_atomic_load(reinterpret_cast<int*>(out_max), __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
        if (__float_as_int(mx) > cur) atomicMax(reinterpret_cast<int*>(out_max), __float_as_int(mx));
    }
}

// Four floats -> four e4m3 codes, round-to-nearest-even, saturating to +-448, NaN -> 0x7F | sign (the cast kernel's rule).
__device__ __forceinline__ u32 e4m3x4(float a, float b, float c, float d) {
    const float v[4] = {a, b, c, d};
    u32 w = (u32)__builtin_amdgcn_cvt_pk_fp8_f32(__builtin_amdgcn_fmed3f(a, 448.0f, -448.0f), __builtin_amdgcn_fmed3f(b, 448.0f, -448.0f), 0, false);
    w = (u32)__builtin_amdgcn_cvt_pk_fp8_f32(__builtin_amdgcn_fmed3f(c, 448.0f, -448.0f), __builtin_amdgcn_fmed3f(d, 448.0f, -448.0f), (int)w, true);
#pragma unroll
    for (int i = 0; i < 4; ++i)
        if (v[i] != v[i]) w = (w & ~(0xFFu << (8 * i))) | ((0x7Fu | ((__float_as_uint(v[i]) >> 24) & 0x80u)) << (8 * i));
    return w;
}

// One 16-byte-per-lane global -> LDS transfer without passing through registers: lane l of the
// wavefront fetches 16 bytes at gbase + voff and the hardware writes them to LDS byte address
// lds_addr + 16*l (lds_addr is wavefront-uniform, carried in M0).  Issued as inline assembly
// because the compiler would otherwise make every later LDS read wait for all such transfers;
// completion is awaited explicitly with wait_vmcnt<N>() before the workgroup barrier.
__device__ __forceinline__ void dma16(const void* gbase, u32 voff, u32 lds_addr) {
    asm volatile("s_mov_b32 m0, %0\n\tglobal_load_lds_dwordx4 %1, %2" ::"s"(lds_addr), "v"(voff), "s"(gbase) : "memory");
}
// Same with 4 bytes per lane (lane l lands at lds_addr + 4*l); used for the W4A4 group scales.
__device__ __forceinline__ void dma4(const void* gbase, u32 voff, u32 lds_addr) {
    asm volatile("s_mov_b32 m0, %0\n\tglobal_load_lds_dword %1, %2" ::"s"(lds_addr), "v"(voff), "s"(gbase) : "memory");
}
template <int N> __device__ __forceinline__ void wait_vmcnt() {
    asm volatile("s_waitcnt vmcnt(%0)" ::"n"(N) : "memory");
}

// Scheduling hint for a region that holds G MFMAs and NP LDS reads: keep them in the interleaved
// order "reads for slot I, then MFMA I" instead of letting the scheduler cluster the reads.
template <int NP, int G, int I> __device__ __forceinline__ void sched_slot() {
    constexpr int n = (I + 1) * NP / G - I * NP / G;
    if constexpr (n > 0) __builtin_amdgcn_sched_group_barrier(0x100, n, 0);  // DS read
    __builtin_amdgcn_sched_group_barrier(0x008, 1, 0);                       // MFMA
}
template <int NP, int G, int... I> __device__ __forceinline__ void sched_interleave(std::integer_sequence<int, I...>) {
    (sched_slot<NP, G, I>(), ...);
}

template <int KIND, typename OutTag, int BM, int BN, int BKB, int WM, int WN, int NSTAGE>
struct GemmKernel {
    static constexpr int NW = WM * WN;
    static constexpr bool W4 = (KIND == K_W4A4 || KIND == K_W4A4H);
    static constexpr int THREADS = NW * 64;
    static constexpr int TM = BM / WM, TN = BN / WN;  // wavefront tile
    static constexpr int MT = TM / 32, NT = TN / 32;  // 32x32 MFMA tiles per wavefront
    static constexpr int CH = BKB / 16;               // 16-byte chunks per tile row
    static constexpr int A_BYTES = BM * BKB, B_BYTES = BN * BKB;
    static constexpr int NGS = BKB / 32;  // W4A4 groups per k-tile (one group of 64 int4 = 32 bytes)
    static constexpr int NS = NGS * (BM + BN);
    static constexpr int S_DMA = W4 ? (NS + 64 * NW - 1) / (64 * NW) : 0;  // 4-byte scale transfers per wavefront per tile
    static constexpr int SCALE_BYTES = S_DMA * NW * 256;  // NS floats, padded to whole transfers
    static constexpr int STAGE_BYTES = A_BYTES + B_BYTES + SCALE_BYTES;
    static constexpr int SMEM_BYTES = NSTAGE * STAGE_BYTES;
    static constexpr int A_DMA = A_BYTES / 1024 / NW, B_DMA = B_BYTES / 1024 / NW;  // transfers per wavefront per tile
    static constexpr int PER_TILE = A_DMA + B_DMA + S_DMA;
    static_assert(A_BYTES % (1024 * NW) == 0 && B_BYTES % (1024 * NW) == 0, "tile/wavefront mismatch");
    static_assert(TM % 32 == 0 && TN % 32 == 0, "wave tile must be a multiple of 32");
    static_assert(CH == 4 || CH == 8, "BKB must be 64 or 128");
    static_assert(!W4 || ((NGS * BM) % 64 == 0 && NGS % 2 == 0), "scale transfer plan");
    static_assert(PER_TILE * NSTAGE < 64, "vmcnt is a 6-bit counter");
    using AccT = typename std::conditional<KIND == K_FP8, v16f, v16i>::type;
    using FragT = typename std::conditional<KIND == K_FP8, v8i, v4i>::type;
    static constexpr int KSTEP = (KIND == K_FP8) ? 64 : 32;  // operand bytes per MFMA k-step
    static constexpr int KS = BKB / KSTEP;

    static __device__ __forceinline__ void run(const GemmParams& p, char* smem) {
        const int tid = threadIdx.x, lane = tid & 63;
        const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
        const int wm = wave / WN, wn = wave % WN;
        int tm, tn;
        // band height chosen so that the workgroups an XCD runs at once cover a roughly square block of C
        tile_coords<(BM >= 256 ? 4 : 8)>(blockIdx.x, p.tiles_m, p.tiles_n, tm, tn);
        const int m0 = tm * BM, n0 = tn * BN;
        const int kb = p.kb;
        const int ktiles = kb / BKB;
        const size_t b_block_stride = (size_t)(kb / 16) * 512;  // bytes per 32-row block in rows32 layout
        const u32 smem_base = (u32)(uintptr_t)(__attribute__((address_space(3))) char*)smem;

        // ---- global -> LDS transfer plan (per lane offsets are fixed; the bases advance with k) ----
        const u32 a_pitch = p.a_panel ? (u32)BKB : (u32)kb;                      // bytes between two rows of A
        const size_t a_kstep = p.a_panel ? (size_t)p.m * BKB : (size_t)BKB;  // bytes between two k-tiles of a row
        const uint8_t* a_base = p.A + (size_t)m0 * a_pitch;
        const uint8_t* b_base = p.B + (size_t)(n0 / 32) * b_block_stride;
        u32 a_voff[A_DMA], b_voff[B_DMA];
        const int row_last = p.m - 1 - m0, blk_last = p.n / 32 - 1 - n0 / 32;
#pragma unroll
        for (int i = 0; i < A_DMA; ++i) {
            int slot = (wave * A_DMA + i) * 64 + lane;  // 16-byte slot inside the A stage
            int row = slot / CH, c = (slot % CH) ^ chunk_swizzle<CH>(row);
            a_voff[i] = (u32)min(row, row_last) * a_pitch + c * 16;
        }
#pragma unroll
        for (int i = 0; i < B_DMA; ++i) {
            int byteoff = (wave * B_DMA + i) * 1024;
            int rblk = byteoff / (BKB * 32), within = byteoff % (BKB * 32);
            b_voff[i] = (u32)((size_t)min(rblk, blk_last) * b_block_stride) + within + lane * 16;
        }
        // W4A4 group scales of a k-tile: [NGS][BM] activation scales then [NGS][BN] weight scales, one
        // 4-byte transfer per scale.  16-bit scales are fetched as the aligned word that holds them (the
        // number of groups per row and per k-tile is even, so the half is fixed per lane); each lane then
        // rewrites the slots its own transfers filled as fp32 -- activation scales times 2^-8, which
        // undoes the widening of both nibble operands -- before the barrier that publishes the stage.
        const int ng = p.k / 64;
        constexpr bool S16 = (KIND == K_W4A4H);
        constexpr int sesz = S16 ? 2 : 4;
        const char* s_base[S_DMA > 0 ? S_DMA : 1];
        u32 s_voff[S_DMA > 0 ? S_DMA : 1];
        if constexpr (W4) {
#pragma unroll
            for (int i = 0; i < S_DMA; ++i) {
                const int first = (wave * S_DMA + i) * 64;  // wavefront-uniform: a transfer is all-A or all-B
                const bool is_a = first < NGS * BM;
                int s = first + lane - (is_a ? 0 : NGS * BM);
                if (!is_a && s >= NGS * BN) s = 0;  // padding slots of the last transfer: fetch something valid
                const int g = is_a ? s / BM : s / BN, r = is_a ? s % BM : s % BN;
                const int row = is_a ? min(r, row_last) : min(r, p.n - 1 - n0);
                s_base[i] = static_cast<const char*>(is_a ? p.sA : p.sB) + (size_t)(is_a ? m0 : n0) * ng * sesz;
                s_voff[i] = ((u32)(row * ng + g) * (u32)sesz) & ~3u;
            }
        }
        auto issue_scales = [&](int kt, int stage) {
            if constexpr (W4) {
                const u32 ss = smem_base + stage * STAGE_BYTES + A_BYTES + B_BYTES + wave * (S_DMA * 256);
#pragma unroll
                for (int i = 0; i < S_DMA; ++i) dma4(s_base[i] + (size_t)kt * NGS * sesz, s_voff[i], ss + i * 256);
            }
        };
        auto convert_scales = [&](int stage) {
            if constexpr (W4) {
                u32* ss = reinterpret_cast<u32*>(smem + stage * STAGE_BYTES + A_BYTES + B_BYTES) + wave * (S_DMA * 64) + lane;
#pragma unroll
                for (int i = 0; i < S_DMA; ++i) {
                    const int first = (wave * S_DMA + i) * 64;
                    const bool is_a = first < NGS * BM;
                    if (!is_a && !S16) continue;
                    const u32 raw = ss[i * 64];
                    const int slot = first + lane - (is_a ? 0 : NGS * BM);
                    const int g = (is_a ? slot / BM : slot / BN) & 1;  // which half of the fetched word
                    float f = S16 ? f16_bits_to_f32((raw >> (16 * g)) & 0xFFFFu) : __uint_as_float(raw);
                    if (is_a) f *= 0.00390625f;
                    ss[i * 64] = __float_as_uint(f);
                }
            }
        };

        auto issue_tile = [&](int kt, int stage) {
            const uint8_t* ga = a_base + (size_t)kt * a_kstep;
            const uint8_t* gb = b_base + (size_t)kt * (BKB * 32);
            const u32 sa = smem_base + stage * STAGE_BYTES + wave * (A_DMA * 1024);
            const u32 sb = smem_base + stage * STAGE_BYTES + A_BYTES + wave * (B_DMA * 1024);
#pragma unroll
            for (int i = 0; i < A_DMA; ++i) dma16(ga, a_voff[i], sa + i * 1024);
#pragma unroll
            for (int i = 0; i < B_DMA; ++i) dma16(gb, b_voff[i], sb + i * 1024);
            issue_scales(kt, stage);
        };
        // Transfers lo..hi-1 of a tile (A first, then B), for main loops that spread a tile's transfers
        // between their MFMAs; lo and hi are compile-time values after unrolling.
        auto issue_range = [&](int kt, int stage, int lo, int hi) {
            const uint8_t* ga = a_base + (size_t)kt * a_kstep;
            const uint8_t* gb = b_base + (size_t)kt * (BKB * 32);
            const u32 sa = smem_base + stage * STAGE_BYTES + wave * (A_DMA * 1024);
            const u32 sb = smem_base + stage * STAGE_BYTES + A_BYTES + wave * (B_DMA * 1024);
#pragma unroll
            for (int d = 0; d < A_DMA + B_DMA; ++d)
                if (d >= lo && d < hi) {
                    if (d < A_DMA) dma16(ga, a_voff[d < A_DMA ? d : 0], sa + d * 1024);
                    else dma16(gb, b_voff[d >= A_DMA ? d - A_DMA : 0], sb + (d - A_DMA) * 1024);
                }
        };
        // ---- accumulators ----------------------------------------------------------------------
        AccT acc[MT][NT];
        v16f res[W4 ? MT : 1][W4 ? NT : 1];
#pragma unroll
        for (int i = 0; i < MT; ++i)
#pragma unroll
            for (int j = 0; j < NT; ++j)
#pragma unroll
                for (int v = 0; v < 16; ++v) {
                    acc[i][j][v] = 0;
                    if constexpr (W4) res[i][j][v] = 0.0f;
                }

        // ---- LDS -> register operand fragments ---------------------------------------------------
        const int lr = lane & 31, lh = lane >> 5;
        const int xrow = wm * TM + lr;           // activation row of this lane inside the tile (+32 per MFMA tile)
        const int xsw = chunk_swizzle<CH>(xrow);  // same for xrow + 32*i (only the low five row bits enter)
        const int w_off = wn * NT * (BKB * 32) + lane * 16;
        auto ldsv = [&](const char* ptr) -> v4i { return *reinterpret_cast<const v4i*>(ptr); };
        auto load_frags = [&](const char* sa, const char* sb, int ks, FragT* w, FragT* x) {
            if constexpr (KIND == K_FP8) {
#pragma unroll
                for (int j = 0; j < NT; ++j) {
                    v4i lo = ldsv(sb + w_off + j * (BKB * 32) + ks * 2048);
                    v4i hi = ldsv(sb + w_off + j * (BKB * 32) + ks * 2048 + 1024);
                    w[j] = v8i{lo[0], lo[1], lo[2], lo[3], hi[0], hi[1], hi[2], hi[3]};
                }
#pragma unroll
                for (int i = 0; i < MT; ++i) {
                    const char* rowp = sa + (xrow + i * 32) * BKB;
                    v4i lo = ldsv(rowp + (((4 * ks + lh) ^ xsw) << 4));
                    v4i hi = ldsv(rowp + (((4 * ks + 2 + lh) ^ xsw) << 4));
                    x[i] = v8i{lo[0], lo[1], lo[2], lo[3], hi[0], hi[1], hi[2], hi[3]};
                }
            } else {
#pragma unroll
                for (int j = 0; j < NT; ++j) w[j] = ldsv(sb + w_off + j * (BKB * 32) + ks * 1024);
#pragma unroll
                for (int i = 0; i < MT; ++i) x[i] = ldsv(sa + (xrow + i * 32) * BKB + (((2 * ks + lh) ^ xsw) << 4));
            }
        };
        auto widen = [](const v4i& q, int half) -> v4i {  // int4 -> int8 * 16: even nibbles, odd nibbles
            int d0 = q[2 * half], d1 = q[2 * half + 1];
            return v4i{(int)(((u32)d0 << 4) & 0xF0F0F0F0u), (int)((u32)d0 & 0xF0F0F0F0u),
                       (int)(((u32)d1 << 4) & 0xF0F0F0F0u), (int)((u32)d1 & 0xF0F0F0F0u)};
        };

        // W4A4: one 64-value group = 32 bytes = two 16-byte chunks = two int8 k-steps.  The work of a
        // stage is a list of (group, n-tile, m-tile) items; the two MFMAs of item t+1 are issued before
        // the 48 scale operations of item t, so the matrix pipe works in the shadow of the VALU, which
        // is the bound of this kernel (cvt + mul + fma per output per group, see the header comment).
        auto compute_tile = [&](int stage) {
            if constexpr (W4) {
                const char* sa = smem + stage * STAGE_BYTES;
                const char* sb = sa + A_BYTES;
                const float* ssa = reinterpret_cast<const float*>(sb + B_BYTES);  // [NGS][BM]
                const float* ssb = ssa + NGS * BM;                                 // [NGS][BN]
                constexpr int PER_GROUP = NT * MT;
                v4i wq[2][NT], xq[2][MT];  // raw nibble fragments of the current and the next group
                v16i pz[2];
                // K_W4A4H: the group sum S (|S| <= 2^20 after widening) is accumulated on top of the bit
                // pattern of 1.5 * 2^23, so the accumulator register READ AS A FLOAT is 12582912 + S and
                // fma(that, sa, -12582912 * sa) = RN(S * sa): the int->float conversion and the first
                // multiplication in one operation, with the same single rounding.  12582912 * sa is exact
                // for a scale of at most 22 significant bits, which every 16-bit float has.
                constexpr int kMagicBits = 0x4B400000;
                constexpr float kMagic = 12582912.0f;
                v16i zinit;
#pragma unroll
                for (int v = 0; v < 16; ++v) zinit[v] = (KIND == K_W4A4H) ? kMagicBits : 0;
                if constexpr (KIND == K_W4A4H) asm volatile("" : "+v"(zinit));  // keep one copy in registers, do not rebuild it per item
                auto issue_item = [&](int g, int t) {  // t: item inside group g
                    const int j = t / MT, i = t % MT;
                    v16i z = zinit;
                    z = __builtin_amdgcn_mfma_i32_32x32x32_i8(widen(wq[g & 1][j], 0), widen(xq[g & 1][i], 0), z, 0, 0, 0);
                    pz[(g * PER_GROUP + t) & 1] =
                        __builtin_amdgcn_mfma_i32_32x32x32_i8(widen(wq[g & 1][j], 1), widen(xq[g & 1][i], 1), z, 0, 0, 0);
                };
                load_frags(sa, sb, 0, wq[0], xq[0]);
                issue_item(0, 0);
#pragma unroll
                for (int g = 0; g < NGS; ++g) {
                    if (g + 1 < NGS) load_frags(sa, sb, g + 1, wq[(g + 1) & 1], xq[(g + 1) & 1]);
                    float sbv[16];
#pragma unroll
                    for (int t = 0; t < PER_GROUP; ++t) {
                        const int j = t / MT, i = t % MT;
                        if (t + 1 < PER_GROUP) issue_item(g, t + 1);
                        else if (g + 1 < NGS) issue_item(g + 1, 0);
                        if (i == 0) {
#pragma unroll
                            for (int q4 = 0; q4 < 4; ++q4) {
                                float4 f = *reinterpret_cast<const float4*>(ssb + g * BN + wn * TN + j * 32 + q4 * 8 + lh * 4);
                                sbv[q4 * 4] = f.x; sbv[q4 * 4 + 1] = f.y; sbv[q4 * 4 + 2] = f.z; sbv[q4 * 4 + 3] = f.w;
                            }
                        }
                        const float sa_l = ssa[g * BM + xrow + i * 32];
                        const float nmagic_sa = -(kMagic * sa_l);
                        const v16i cur = pz[(g * PER_GROUP + t) & 1];
#pragma unroll
                        for (int v = 0; v < 16; ++v) {
                            float t;
                            if constexpr (KIND == K_W4A4H) t = __builtin_fmaf(__int_as_float(cur[v]), sa_l, nmagic_sa);
                            else t = (float)cur[v] * sa_l;
                            res[i][j][v] = __builtin_fmaf(t, sbv[v], res[i][j][v]);
                        }
                    }
                    __builtin_amdgcn_sched_barrier(0);  // keep the next group's reads and widening from piling up
                }
            }
        };

        // ---- main loop ---------------------------------------------------------------------------------
        // Tile t lives in LDS stage t % NSTAGE.  INT8/FP8: operand fragments are double-buffered in
        // registers ACROSS tile boundaries: at the last k-step of tile kt a wavefront waits for its own
        // transfers of tile kt+1, passes the workgroup barrier (after which tile kt+1 is complete and
        // nobody reads stage kt % NSTAGE any more), re-arms that stage with tile kt+NSTAGE, prefetches
        // the first fragments of tile kt+1 and only then issues the MFMAs of the step -- so the matrix
        // pipe always has queued work while wavefronts sit in the barrier.  One barrier per tile.
        // Every iteration issues exactly one tile of transfers (past the end it re-fetches the last
        // tile into a stage nobody reads again), which makes the vmcnt thresholds compile-time values.
        if constexpr (!W4) {
            // Operand fragments as 16-byte pieces (an fp8 fragment is two pieces), so that the LDS reads
            // of the next k-step can be interleaved one by one with the MFMAs of the current step.
            constexpr int PPF = (KIND == K_FP8) ? 2 : 1;
            constexpr int KCH = KSTEP / 16;  // chunks per k-step
            constexpr int NPIECE = (NT + MT) * PPF;
            constexpr int NMFMA = MT * NT;
            v4i wp[2][NT][PPF], xp[2][MT][PPF];
            // piece order follows first use: x0, w0..w(NT-1), x1..x(MT-1)
            auto load_piece = [&](const char* sa, int ks, int buf, int pc) {
                const int f = pc / PPF, h = pc % PPF;
                if (f == 0 || f > NT) {
                    const int i = f == 0 ? 0 : f - NT;
                    xp[buf][i][h] = ldsv(sa + (xrow + i * 32) * BKB + (((KCH * ks + lh + 2 * h) ^ xsw) << 4));
                } else {
                    const int j = f - 1;
                    wp[buf][j][h] = ldsv(sa + A_BYTES + w_off + j * (BKB * 32) + ks * (KSTEP * 32) + h * 1024);
                }
            };
            auto do_mfma = [&](int buf, int idx) {
                const int i = idx / NT, j = idx % NT;
                if constexpr (KIND == K_FP8) {
                    v8i w = __builtin_shufflevector(wp[buf][j][0], wp[buf][j][PPF - 1], 0, 1, 2, 3, 4, 5, 6, 7);
                    v8i x = __builtin_shufflevector(xp[buf][i][0], xp[buf][i][PPF - 1], 0, 1, 2, 3, 4, 5, 6, 7);
                    acc[i][j] = __builtin_amdgcn_mfma_scale_f32_32x32x64_f8f6f4(w, x, acc[i][j], 0, 0, 0, 0, 0, 0);
                } else {
                    acc[i][j] = __builtin_amdgcn_mfma_i32_32x32x32_i8(wp[buf][j][0], xp[buf][i][0], acc[i][j], 0, 0, 0);
                }
            };
            // With three or more stages a tile's transfers are not issued in one burst behind the barrier
            // but spread between the MFMAs: a wavefront stalled on a full memory-instruction queue cannot
            // feed the matrix pipe, and with one wavefront per SIMD nobody else can either.  Tile T's first
            // N_AFTER transfers go out behind the barrier that retires tile T-NSTAGE, between the MFMAs
            // that follow it; the rest between the MFMAs of tile T-NSTAGE+1 ahead of ITS barrier.  At the
            // barrier of tile kt everything up to tile kt+NSTAGE-1 has been issued, so the wait for tile
            // kt+1 leaves the same PER_TILE*(NSTAGE-2) transfers in flight as the burst scheme.
            constexpr bool SPREAD = NSTAGE >= 3;
            constexpr int HPRE = NMFMA / 2, RPOST = NMFMA - HPRE;  // MFMAs of the last k-step ahead of / behind the barrier
            constexpr int NPOS = KS * NMFMA, PRE = NPOS - RPOST;
            constexpr int N_AFTER = SPREAD ? PER_TILE * RPOST / NPOS : PER_TILE, N_BEFORE = PER_TILE - N_AFTER;
            auto tile_iter = [&](int kt, auto parity) {
                constexpr int P = decltype(parity)::value;
                const char* sa = smem + (kt % NSTAGE) * STAGE_BYTES;
                const int t_prev = min(kt + NSTAGE - 1, ktiles - 1), s_prev = (kt + NSTAGE - 1) % NSTAGE;
#pragma unroll
                for (int ks = 0; ks < KS; ++ks) {
                    const int cur = (P + ks) & 1, nxt = cur ^ 1;
                    if (ks + 1 < KS) {
                        // MFMAs of this step interleaved with the fragment reads of the next step
#pragma unroll
                        for (int idx = 0; idx < NMFMA; ++idx) {
                            if constexpr (SPREAD) {
                                const int q = ks * NMFMA + idx;
                                issue_range(t_prev, s_prev, N_AFTER + q * N_BEFORE / PRE, N_AFTER + (q + 1) * N_BEFORE / PRE);
                            }
#pragma unroll
                            for (int pc = idx * NPIECE / NMFMA; pc < (idx + 1) * NPIECE / NMFMA; ++pc)
                                load_piece(sa, ks + 1, nxt, pc);
                            do_mfma(cur, idx);
                            if constexpr (SPREAD) __builtin_amdgcn_sched_barrier(0);
                        }
                        if constexpr (!SPREAD) sched_interleave<NPIECE, NMFMA>(std::make_integer_sequence<int, NMFMA>{});
                    } else {
                        // last step of the tile: half of the MFMAs go ahead of the barrier so that the matrix
                        // pipe has work while the wavefront waits; the other half is interleaved with the first
                        // fragment reads of the next tile.
#pragma unroll
                        for (int idx = 0; idx < HPRE; ++idx) {
                            if constexpr (SPREAD) {
                                const int q = ks * NMFMA + idx;
                                issue_range(t_prev, s_prev, N_AFTER + q * N_BEFORE / PRE, N_AFTER + (q + 1) * N_BEFORE / PRE);
                            }
                            do_mfma(cur, idx);
                            if constexpr (SPREAD) __builtin_amdgcn_sched_barrier(0);
                        }
                        __builtin_amdgcn_sched_barrier(0);
                        wait_vmcnt<PER_TILE*(NSTAGE - 2)>();
                        __syncthreads();
                        const int t_next = min(kt + NSTAGE, ktiles - 1);
                        if constexpr (!SPREAD) issue_tile(t_next, kt % NSTAGE);
                        __builtin_amdgcn_sched_barrier(0);
                        const char* sn = smem + ((kt + 1) % NSTAGE) * STAGE_BYTES;
#pragma unroll
                        for (int idx = 0; idx < RPOST; ++idx) {
                            if constexpr (SPREAD) issue_range(t_next, kt % NSTAGE, idx * N_AFTER / RPOST, (idx + 1) * N_AFTER / RPOST);
#pragma unroll
                            for (int pc = idx * NPIECE / RPOST; pc < (idx + 1) * NPIECE / RPOST; ++pc) load_piece(sn, 0, nxt, pc);
                            do_mfma(cur, HPRE + idx);
                            if constexpr (SPREAD) __builtin_amdgcn_sched_barrier(0);
                        }
                        if constexpr (!SPREAD) sched_interleave<NPIECE, RPOST>(std::make_integer_sequence<int, RPOST>{});
                        __builtin_amdgcn_sched_barrier(0);
                    }
                }
            };
            if constexpr (SPREAD) {
#pragma unroll
                for (int s = 0; s < NSTAGE - 1; ++s) issue_tile(min(s, ktiles - 1), s);
                issue_range(min(NSTAGE - 1, ktiles - 1), NSTAGE - 1, 0, N_AFTER);
                wait_vmcnt<PER_TILE*(NSTAGE - 2) + N_AFTER>();
            } else {
#pragma unroll
                for (int s = 0; s < NSTAGE; ++s) issue_tile(min(s, ktiles - 1), s);
                wait_vmcnt<PER_TILE*(NSTAGE - 1)>();
            }
            __syncthreads();
#pragma unroll
            for (int pc = 0; pc < NPIECE; ++pc) load_piece(smem, 0, 0, pc);
            int kt = 0;
            if constexpr (KS % 2 == 1) {
                for (; kt + 1 < ktiles; kt += 2) {
                    tile_iter(kt, std::integral_constant<int, 0>{});
                    tile_iter(kt + 1, std::integral_constant<int, 1>{});
                }
                if (kt < ktiles) tile_iter(kt, std::integral_constant<int, 0>{});
            } else {
                for (; kt < ktiles; ++kt) tile_iter(kt, std::integral_constant<int, 0>{});
            }
        } else {
            // W4A4: tile kt+NSTAGE-1 is requested right after the barrier that retires tile kt-1; at the
            // end of an iteration a wavefront waits for its own transfers of tile kt+1 and rewrites the
            // scales among them, which the next barrier publishes.
#pragma unroll
            for (int s = 0; s < NSTAGE - 1; ++s) issue_tile(min(s, ktiles - 1), s);
            wait_vmcnt<PER_TILE*(NSTAGE - 2)>();
            convert_scales(0);
            for (int kt = 0; kt < ktiles; ++kt) {
                __syncthreads();
                issue_tile(min(kt + NSTAGE - 1, ktiles - 1), (kt + NSTAGE - 1) % NSTAGE);
                compute_tile(kt % NSTAGE);
                wait_vmcnt<PER_TILE*(NSTAGE - 2)>();
                if (kt + 1 < ktiles) convert_scales((kt + 1) % NSTAGE);
            }
        }
        wait_vmcnt<0>();
        __syncthreads();  // every transfer has landed and nobody reads operands any more: LDS is reusable

        // ---- W4A4 low-rank branch ---------------------------------------------------------------------------
        // res += act[m, 0:rank] . up[n, 0:rank]^T on the 16-bit float matrix instruction, straight onto the fp32
        // accumulators (every 32x32 MFMA has the same result layout).  An operand fragment is the 16 bytes a
        // lane reads from its own row: eight consecutive rank indices, lanes 32..63 the next eight; rows are
        // rank*2 bytes apart, so a wavefront reads one contiguous block per fragment.
        if constexpr (W4) {
            if (p.lora_act != nullptr) {
                typedef __bf16 v8bf __attribute__((ext_vector_type(8)));
                typedef _Float16 v8h __attribute__((ext_vector_type(8)));
                const int rbytes = p.lora_rank * 2;
                const char* up = static_cast<const char*>(p.lora_up) + (lane >> 5) * 16;
                const char* act = static_cast<const char*>(p.lora_act) + (lane >> 5) * 16;
                for (int ks = 0; ks < p.lora_rank / 16; ++ks) {
                    v4i wf[NT], xf[MT];
#pragma unroll
                    for (int j = 0; j < NT; ++j)
                        wf[j] = *reinterpret_cast<const v4i*>(up + (size_t)min(n0 + wn * TN + j * 32 + (lane & 31), p.n - 1) * rbytes + ks * 32);
#pragma unroll
                    for (int i = 0; i < MT; ++i)
                        xf[i] = *reinterpret_cast<const v4i*>(act + (size_t)min(m0 + wm * TM + i * 32 + (lane & 31), p.m - 1) * rbytes + ks * 32);
#pragma unroll
                    for (int i = 0; i < MT; ++i)
#pragma unroll
                        for (int j = 0; j < NT; ++j) {
                            if (p.lora_f16)
                                res[i][j] = __builtin_amdgcn_mfma_f32_32x32x16_f16(__builtin_bit_cast(v8h, wf[j]), __builtin_bit_cast(v8h, xf[i]), res[i][j], 0, 0, 0);
                            else
                                res[i][j] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(__builtin_bit_cast(v8bf, wf[j]), __builtin_bit_cast(v8bf, xf[i]), res[i][j], 0, 0, 0);
                        }
                }
            }
        }

        // ---- epilogue -------------------------------------------------------------------------------------
        // Each wavefront parks one 32-row band of raw 32-bit accumulators at a time in a private LDS
        // strip laid out [row][n] (plus the band's per-token scales in the row padding), reads it back
        // with rows contiguous -- a lane then owns four consecutive n of one row -- applies the dequant
        // scales, bias and activation there and stores whole 128-byte (or longer) row segments.  The
        // per-lane constants (bias, per-channel scales for the lane's four columns) are loaded once,
        // BEFORE the first store: on this architecture loads and stores share one in-order counter, so a
        // load issued after a store would have to wait for that store to be acknowledged by memory.
        constexpr bool kI32 = std::is_same<OutTag, I32Tag>::value;
        constexpr int ESZ = (std::is_same<OutTag, F16Tag>::value || std::is_same<OutTag, BF16Tag>::value) ? 2 : 4;
        constexpr int PITCH = TN * 4 + 16;  // strip row: TN raw values + one 16-byte pad slot
        constexpr int LPR = TN / 4;         // lanes per output row on the way out
        constexpr int RPI = 64 / LPR;       // rows per store instruction
        static_assert(NW * 32 * PITCH <= SMEM_BYTES, "epilogue strip does not fit in the operand stages");
        static_assert(64 % LPR == 0 && 32 % RPI == 0, "wave tile width must be 32, 64, 128 or 256");
        char* strip = smem + wave * (32 * PITCH);
        const int out_row = lane / LPR, out_n = n0 + wn * TN + (lane % LPR) * 4;
        const bool n_ok = out_n < p.n;
        float alpha = 1.0f, bias4[4] = {0.f, 0.f, 0.f, 0.f}, acol4[4] = {0.f, 0.f, 0.f, 0.f}, arow_l[MT];
        float out_amax = 0.0f, out_pmax = 0.0f, c8_inv = 0.0f, gate4[4] = {0.f, 0.f, 0.f, 0.f};
        bool gate_uniform = true;  // every row of the wavefront's tile uses the same gate vector
        // the FP8 and W4A4 linears of the FLUX blocks share the activation / re-quantisation / gate epilogues
        constexpr bool kExtras = (KIND == K_FP8 || W4) && !kI32;
        if constexpr (KIND == K_FP8) alpha = p.a_scale[0] * p.b_scale[0];
        if constexpr (kExtras) {
            if (p.C8 != nullptr) c8_inv = 1.0f / p.c8_scale[0];
            {
                if (p.gate != nullptr) {
                    const size_t r_first = (size_t)(m0 + wm * TM), r_last = (size_t)min(m0 + wm * TM + TM - 1, p.m - 1);
                    const size_t b_first = r_first / p.gate_rows;
                    gate_uniform = b_first == r_last / p.gate_rows;
                    if (gate_uniform && n_ok && r_first < (size_t)p.m) OutStore<OutTag>::load4(p.gate, b_first * (size_t)p.n + out_n, gate4);
                }
            }
        }
        if constexpr (!kI32) {
            if (p.bias != nullptr && n_ok) OutStore<OutTag>::load4(p.bias, out_n, bias4);
            if constexpr (KIND == K_INT8) {
                if (n_ok) {
                    float4 ac = *reinterpret_cast<const float4*>(p.alpha_col + out_n);
                    acol4[0] = ac.x; acol4[1] = ac.y; acol4[2] = ac.z; acol4[3] = ac.w;
                }
#pragma unroll
                for (int i = 0; i < MT; ++i)
                    arow_l[i] = p.alpha_row[p.per_token ? min(m0 + wm * TM + i * 32 + lr, p.m - 1) : 0];
            }
        }
        // The row loop exists in a few specialisations, chosen once per workgroup: which optional steps run
        // (PLAIN: scales and bias; ACT: also GELU and/or the running maximum; CODES: optional GELU, e4m3 codes
        // instead of C; GATED: gate and residual; GENERAL: every option, checked at run time) and whether the tile lies
        // entirely inside C (no bounds checks).  Strip rows are read four at a time so that their LDS latencies
        // overlap, and the specialisations keep the per-row code free of branches.
        constexpr int E_PLAIN = 0, E_ACT = 1, E_CODES = 2, E_GATED = 3, E_GENERAL = 4;
        constexpr bool kSpecialise = kExtras && ESZ == 2;  // fp32 outputs take the general path only (build time)
        int emode = kExtras ? E_GENERAL : E_PLAIN;
        if constexpr (kSpecialise) {
            const bool join = p.addend != nullptr || p.residual != nullptr || p.gate != nullptr;
            if (!join && p.C8 == nullptr && p.C != nullptr) emode = (p.gelu != 0 || p.out_scale != nullptr || p.out_max != nullptr) ? E_ACT : E_PLAIN;
            else if (!join && p.C8 != nullptr && p.C == nullptr && p.out_scale == nullptr) emode = E_CODES;
            else if (p.gate != nullptr && p.residual != nullptr && p.addend == nullptr && p.C8 == nullptr && p.C != nullptr &&
                     p.gelu == 0 && p.out_scale == nullptr) emode = E_GATED;
        }
        const bool tile_full = m0 + BM <= p.m && n0 + BN <= p.n;
        const bool has_bias = p.bias != nullptr;
        auto band_rows = [&](auto i_c, auto mode_c, auto full_c) {
            constexpr int i = decltype(i_c)::value;
            constexpr int MODE = decltype(mode_c)::value;
            constexpr bool FULL = decltype(full_c)::value;
            constexpr bool GEN = MODE == E_GENERAL;
            constexpr int NITER = 32 / RPI, NB = 4;
            static_assert(NITER % NB == 0, "strip rows are processed four at a time");
            const int mrow0 = m0 + wm * TM + i * 32 + out_row;
            const size_t idx0 = (size_t)mrow0 * p.n + out_n, rstep = (size_t)RPI * p.n;
#pragma unroll
            for (int tb = 0; tb < NITER; tb += NB) {
                v4i raw[NB];
                float arv[NB];
#pragma unroll
                for (int u = 0; u < NB; ++u) {
                    const int row = (tb + u) * RPI + out_row;
                    raw[u] = *reinterpret_cast<const v4i*>(strip + row * PITCH + (lane % LPR) * 16);
                    if constexpr (KIND == K_INT8 && !kI32) arv[u] = *reinterpret_cast<const float*>(strip + row * PITCH + TN * 4);
                }
#pragma unroll
                for (int u = 0; u < NB; ++u) {
                    const int t = tb + u;
                    const int mo = mrow0 + t * RPI;
                    const bool ok = FULL || (mo < p.m && n_ok);
                    const size_t idx = idx0 + (size_t)t * rstep;
                    if constexpr (kI32) {
                        if (ok) *reinterpret_cast<v4i*>(static_cast<int*>(p.C) + idx) = raw[u];
                    } else {
                        float y[4];
                        if constexpr (KIND == K_INT8) {
#pragma unroll
                            for (int e = 0; e < 4; ++e) {
                                y[e] = (float)raw[u][e] * (acol4[e] * arv[u]);
                                if (has_bias) y[e] = y[e] + bias4[e];
                            }
                        } else {
#pragma unroll
                            for (int e = 0; e < 4; ++e) {
                                const float vf = __int_as_float(raw[u][e]);
                                y[e] = (KIND == K_FP8) ? vf * alpha : vf;
                                if (has_bias) y[e] = y[e] + bias4[e];
                            }
                        }
                        if constexpr (kExtras && (MODE == E_ACT || MODE == E_CODES || GEN)) {
                            if (p.gelu) {
#pragma unroll
                                for (int e = 0; e < 4; ++e) {
                                    if (p.gelu == 2) y[e] = round_through<OutTag>(y[e]);
                                    y[e] = gelu_fast(y[e]);
                                }
                            }
                        }
                        if constexpr (kExtras && GEN) {
                            if (p.addend != nullptr && ok) {  // T( T(y) + addend ): a second linear's output joined in T
                                float aa[4];
                                OutStore<OutTag>::load4(p.addend, idx, aa);
#pragma unroll
                                for (int e = 0; e < 4; ++e) y[e] = round_through<OutTag>(round_through<OutTag>(y[e]) + aa[e]);
                            }
                        }
                        if constexpr (kExtras && (MODE == E_GATED || GEN)) {
                            if ((MODE == E_GATED || p.residual != nullptr) && ok) {
                                float rr[4];
                                OutStore<OutTag>::load4(p.residual, idx, rr);
                                if (MODE == E_GATED || p.gate != nullptr) {
                                    if (!gate_uniform) OutStore<OutTag>::load4(p.gate, ((size_t)mo / p.gate_rows) * (size_t)p.n + out_n, gate4);
#pragma unroll
                                    for (int e = 0; e < 4; ++e)
                                        y[e] = round_through<OutTag>(round_through<OutTag>(y[e]) * gate4[e]) + rr[e];
                                } else {
#pragma unroll
                                    for (int e = 0; e < 4; ++e) y[e] = y[e] + p.beta * rr[e];
                                }
                            }
                        }
                        if constexpr (kExtras && (MODE == E_ACT || GEN)) {
                            if (ok && p.out_scale != nullptr)
                                out_amax = fmaxf(fmaxf(out_amax, fmaxf(fabsf(y[0]), fabsf(y[1]))), fmaxf(fabsf(y[2]), fabsf(y[3])));
                            if (ok && p.out_max != nullptr) out_pmax = fmaxf(fmaxf(out_pmax, fmaxf(y[0], y[1])), fmaxf(y[2], y[3]));
                        }
                        if constexpr (kExtras && (MODE == E_CODES || GEN)) {
                            if (ok && (MODE == E_CODES || p.C8 != nullptr)) {  // the codes the cast kernel would produce from the T-rounded output
                                float tq[4];
#pragma unroll
                                for (int e = 0; e < 4; ++e) tq[e] = round_through<OutTag>(y[e]) * c8_inv;
                                *reinterpret_cast<u32*>(p.C8 + (p.c8_panel ? ((size_t)(out_n >> 6) * p.m + mo) * 64 + (out_n & 63) : (size_t)mo * p.ldc8 + out_n)) =
                                    e4m3x4(tq[0], tq[1], tq[2], tq[3]);
                            }
                        }
                        if constexpr (GEN) {
                            if (ok && p.C != nullptr) OutStore<OutTag>::store4(p.C, idx, y);
                        } else if constexpr (kExtras && MODE == E_ACT) {
                            if (ok) {
                                if (p.stream_c) OutStore<OutTag>::store4_stream(p.C, idx, y);
                                else OutStore<OutTag>::store4(p.C, idx, y);
                            }
                        } else if constexpr (MODE != E_CODES) {
                            if (ok) OutStore<OutTag>::store4(p.C, idx, y);
                        }
                    }
                }
            }
        };
        // one fully unrolled pass over the wavefront's MT bands per specialisation (the accumulators must stay
        // statically indexed, so the specialisation is chosen outside the band loop)
        auto all_bands = [&](auto mode_c, auto full_c) {
            auto one_band = [&](auto i_c) {
                constexpr int i = decltype(i_c)::value;
#pragma unroll
                for (int j = 0; j < NT; ++j)
#pragma unroll
                    for (int q4 = 0; q4 < 4; ++q4) {
                        char* spot = strip + lr * PITCH + (j * 32 + q4 * 8 + lh * 4) * 4;
                        if constexpr (W4)
                            *reinterpret_cast<float4*>(spot) = make_float4(res[i][j][q4 * 4], res[i][j][q4 * 4 + 1],
                                                                           res[i][j][q4 * 4 + 2], res[i][j][q4 * 4 + 3]);
                        else if constexpr (KIND == K_FP8)
                            *reinterpret_cast<float4*>(spot) = make_float4(acc[i][j][q4 * 4], acc[i][j][q4 * 4 + 1],
                                                                           acc[i][j][q4 * 4 + 2], acc[i][j][q4 * 4 + 3]);
                        else
                            *reinterpret_cast<int4*>(spot) = make_int4(acc[i][j][q4 * 4], acc[i][j][q4 * 4 + 1],
                                                                       acc[i][j][q4 * 4 + 2], acc[i][j][q4 * 4 + 3]);
                    }
                if constexpr (KIND == K_INT8 && !kI32) {
                    if (lh == 0) *reinterpret_cast<float*>(strip + lr * PITCH + TN * 4) = arow_l[i];
                }
                // strip -> registers with rows contiguous, math, store (the wavefront's own LDS accesses
                // complete in order, so no barrier is needed inside the wavefront)
                band_rows(i_c, mode_c, full_c);
            };
            one_band(std::integral_constant<int, 0>{});
            if constexpr (MT > 1) one_band(std::integral_constant<int, 1>{});
            if constexpr (MT > 2) one_band(std::integral_constant<int, 2>{});
            if constexpr (MT > 3) one_band(std::integral_constant<int, 3>{});
            static_assert(MT <= 4, "at most four 32-row bands per wavefront");
        };
        {
            using std::integral_constant;
            if constexpr (kSpecialise) {
                if (emode == E_GENERAL) all_bands(integral_constant<int, E_GENERAL>{}, std::false_type{});
                else if (tile_full) {
                    if (emode == E_PLAIN) all_bands(integral_constant<int, E_PLAIN>{}, std::true_type{});
                    else if (emode == E_ACT) all_bands(integral_constant<int, E_ACT>{}, std::true_type{});
                    else if (emode == E_CODES) all_bands(integral_constant<int, E_CODES>{}, std::true_type{});
                    else all_bands(integral_constant<int, E_GATED>{}, std::true_type{});
                } else {
                    if (emode == E_PLAIN) all_bands(integral_constant<int, E_PLAIN>{}, std::false_type{});
                    else if (emode == E_ACT) all_bands(integral_constant<int, E_ACT>{}, std::false_type{});
                    else if (emode == E_CODES) all_bands(integral_constant<int, E_CODES>{}, std::false_type{});
                    else all_bands(integral_constant<int, E_GATED>{}, std::false_type{});
                }
            } else if constexpr (kExtras) {
                all_bands(integral_constant<int, E_GENERAL>{}, std::false_type{});
            } else {
                if (tile_full) all_bands(integral_constant<int, E_PLAIN>{}, std::true_type{});
                else all_bands(integral_constant<int, E_PLAIN>{}, std::false_type{});
            }
        }
        if constexpr (kExtras) {
            // Rounding to T is monotone, so the maximum of the rounded outputs is the rounded maximum; so is the
            // division by 448: the scale published here is exactly what an amax pass over C would produce.
            if (p.out_scale != nullptr) {
                out_amax = round_through<OutTag>(wave_max(out_amax));
                if (lane == 0) {
                    const float sc = out_amax / 448.0f;
                    int cur = __hip_atomic_load(reinterpret_cast<int*>(p.out_scale), __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
                    if (__float_as_int(sc) > cur) atomicMax(reinterpret_cast<int*>(p.out_scale), __float_as_int(sc));
                }
            }
            if (p.out_max != nullptr) publish_out_max<OutTag>(p.out_max, out_pmax, lane);
        }
    }
};

// 256-thread configurations are meant to run two workgroups per CU (two wavefronts per SIMD), so that
// one workgroup's barrier waits, pipeline fill and epilogue overlap with the other's MFMA work.
// The W4A4 kernel is bound by the vector ALU (three fp32 operations per output per group), so its
// small-tile configurations ask for more resident wavefronts instead.
template <int KIND, int BM, int BN, int BKB, int WM, int WN> constexpr int min_workgroups_per_cu() {
    if ((BM / WM) * (BN / WN) >= 128 * 128) return 1;  // 256 accumulator registers: one wavefront per SIMD, the whole register file
    if (KIND != K_W4A4 && KIND != K_W4A4H) return 2;
    if (WM * WN > 4) return 1;
    const int wave_tile = (BM / WM) * (BN / WN);
    if (wave_tile <= 32 * 32) return 4;
    if (wave_tile <= 64 * 32) return 3;
    return BKB == 128 ? 1 : 2;
}

template <int KIND, typename OutTag, int BM, int BN, int BKB, int WM, int WN, int NSTAGE>
__global__ __launch_bounds__(WM* WN * 64, (min_workgroups_per_cu<KIND, BM, BN, BKB, WM, WN>())) void gemm_kernel(GemmParams p) {
    extern __shared__ __attribute__((aligned(16))) char lq_smem[];
    GemmKernel<KIND, OutTag, BM, BN, BKB, WM, WN, NSTAGE>::run(p, lq_smem);
}

template <int KIND, typename OutTag, int BM, int BN, int BKB, int WM, int WN, int NSTAGE>
static int launch_gemm(GemmParams p, hipStream_t st) {
    using GK = GemmKernel<KIND, OutTag, BM, BN, BKB, WM, WN, NSTAGE>;
    if (p.kb % BKB != 0) {
        set_error("gemm: row length %d bytes is not a multiple of the %d-byte k-tile", p.kb, BKB);
        return LQ_ERR_SHAPE;
    }
    if (p.a_panel && BKB != 64) {
        set_error("gemm: an activation in 64-byte k-panels needs a configuration with 64-byte k-tiles");
        return LQ_ERR_ARG;
    }
    p.tiles_m = (p.m + BM - 1) / BM;
    p.tiles_n = (p.n + BN - 1) / BN;
    auto kern = gemm_kernel<KIND, OutTag, BM, BN, BKB, WM, WN, NSTAGE>;
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

// Persistent one-wavefront-per-SIMD form (lq_gemm_persist.h, compiled in lq_gemm_persist.hip): LQ_OK when launched, 1 when
// the call is not one it implements (shape with partial tiles or an odd number of k-tiles, an epilogue beyond scales and
// bias, an output type other than fp16 / bf16) -- the caller then runs the plain configuration -- negative on an error.
int launch_persist_fp8(const GemmParams& p, lq_dtype_t out_dtype, hipStream_t st);
int launch_persist_int8(const GemmParams& p, lq_dtype_t out_dtype, hipStream_t st);
int device_cu_count();  // compute units of the current device (cached per device)

}  // namespace lq
