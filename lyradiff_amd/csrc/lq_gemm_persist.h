// Persistent form of the one-wavefront-per-SIMD quantized GEMM (INT8 / FP8, 256x256 tiles, four wavefronts of 128x128,
// 64-byte k-tiles, four LDS stages) for problems whose tiles are all full and outnumber the CUs.
//
// A workgroup of the plain kernel (lq_gemm_core.h) computes one output tile: its pipeline fill (the first operand
// transfers have to come back from L2 / the last-level cache before any MFMA can issue), its epilogue's store drain and
// the start-up of the workgroup that replaces it are exposed on every tile, because with the 256 accumulator registers of
// a 128x128 wavefront tile only one wavefront fits a SIMD and nothing else runs beside it.  Here one workgroup per CU
// walks its tiles in one unbroken stream of k-tiles: the direct-to-LDS transfers that run NSTAGE-1 k-tiles ahead of the
// MFMAs simply continue into the next output tile, so that tile's first operands land -- and its first fragments are
// already in registers -- while the current tile's epilogue runs.  The epilogue has an LDS strip of its own (the four
// operand stages stay live), 32 rows x 64 columns per wavefront, XOR-swizzled instead of padded: 4 x 32 KiB of stages and
// 4 x 8 KiB of strips are exactly the 160 KiB of a CU.
//
// Loads and stores share one in-order counter on this architecture.  Waiting for a transfer that was issued before the
// epilogue's stores therefore cannot be expressed once more than 63 operations are younger than it, and waiting for one
// issued after them would wait for the stores' acknowledgements as well.  So a wavefront waits for everything it issued
// before the epilogue once, in the middle of the epilogue ("at most as many operations outstanding as I have stored
// since"), the workgroup barrier of the next iteration publishes that, and the two iterations after an epilogue -- whose
// k-tiles are then known to have landed -- carry no counter wait at all; the third one waits with the usual threshold,
// by which time the stores are long acknowledged.
#pragma once

#include "lq_gemm_core.h"

namespace lq {

// The epilogue is scales and bias only.  Anything heavier (activation, output maximum, codes, gate and residual) is
// vector-ALU work that nothing hides when one wavefront owns a SIMD -- measured on 4608x12288x3072 FP8 with GELU and the
// output maximum: 182 us in this form against 161 us with two 128x256 workgroups per CU, where it costs 134-140 against
// 148 us with the plain epilogue -- so such calls stay with the two-workgroups-per-CU configuration.
// MT: 32-row MFMA blocks per wavefront along M: 4 = 256x256 tiles, 2 = 128x256 tiles (the halves of the leftover tiles, see
// launch_gemm_persist).
// TRACK (FP8): the largest output joins p.out_max.
template <int KIND, typename OutTag, int MT, bool TRACK = false>
struct GemmPersist {
    static_assert(KIND == K_FP8 || KIND == K_INT8, "INT8 and FP8 only");
    static_assert(MT == 4 || MT == 2, "256- or 128-row tiles");
    static constexpr int BM = 64 * MT, BN = 256, BKB = 64, NSTAGE = 4, NW = 4, THREADS = 256;
    static constexpr int TM = 32 * MT, TN = 128, NT = 4, CH = 4;
    static constexpr int A_REGION = 256 * BKB;  // the activation part of a stage is laid out for the tall tile
    static constexpr int A_BYTES = BM * BKB, B_BYTES = BN * BKB, STAGE_BYTES = A_REGION + B_BYTES;
    static constexpr int STRIP_BYTES = 32 * 64 * 4;  // per wavefront: 32 rows x 64 columns of raw 32-bit accumulators
    static constexpr int SMEM_BYTES = NSTAGE * STAGE_BYTES + NW * STRIP_BYTES;
    static constexpr int A_DMA = A_BYTES / 1024 / NW, B_DMA = B_BYTES / 1024 / NW, PER_TILE = A_DMA + B_DMA;
    using AccT = typename std::conditional<KIND == K_FP8, v16f, v16i>::type;
    static constexpr int KSTEP = (KIND == K_FP8) ? 64 : 32;
    static constexpr int KS = BKB / KSTEP;
    static constexpr int PPF = (KIND == K_FP8) ? 2 : 1;
    static constexpr int KCH = KSTEP / 16;
    static constexpr int NPIECE = (NT + MT) * PPF;
    static constexpr int NMFMA = MT * NT;
    static constexpr int HPRE = NMFMA / 2, RPOST = NMFMA - HPRE;
    static constexpr int NPOS = KS * NMFMA, PRE = NPOS - RPOST;
    static constexpr int N_AFTER = PER_TILE * RPOST / NPOS, N_BEFORE = PER_TILE - N_AFTER;

    struct Cursor {  // the k-tile a transfer fetches: wavefront-uniform
        const uint8_t* ga;
        const uint8_t* gb;
        int kt;  // k-tile inside its output tile
        int tj;  // which of this workgroup's output tiles
    };

    // phase 0: this workgroup's whole tiles (id = workgroup + j * grid); phase 1 (MT == 2): one half of a leftover tile.
    static __device__ __forceinline__ void run(const GemmParams& p, char* smem, const int phase) {
        const int tid = threadIdx.x, lane = tid & 63;
        const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
        const int wm = wave >> 1, wn = wave & 1;
        const int kb = p.kb, ktiles = kb / BKB;
        const int total_tiles = p.tiles_m * p.tiles_n;
        const int my_tiles = phase == 1 ? ((int)blockIdx.x < p.persist_halves ? 1 : 0)
                                        : (p.persist_halves > 0 ? p.persist_rounds
                                                                : (total_tiles - (int)blockIdx.x + (int)gridDim.x - 1) / (int)gridDim.x);
        if (my_tiles == 0) return;  // the same for the whole workgroup
        const size_t b_block_stride = (size_t)(kb / 16) * 512;
        const u32 smem_base = (u32)(uintptr_t)(__attribute__((address_space(3))) char*)smem;

        const u32 a_pitch = p.a_panel ? (u32)BKB : (u32)kb;                      // row-major A or k-panels [kb / 64][m][64]
        const size_t a_kstep = p.a_panel ? (size_t)p.m * BKB : (size_t)BKB;
        // per-lane transfer offsets: every tile is full, so they do not depend on the tile
        u32 a_voff[A_DMA], b_voff[B_DMA];
#pragma unroll
        for (int i = 0; i < A_DMA; ++i) {
            const int slot = (wave * A_DMA + i) * 64 + lane;
            const int row = slot / CH, c = (slot % CH) ^ chunk_swizzle<CH>(row);
            a_voff[i] = (u32)row * a_pitch + c * 16;
        }
#pragma unroll
        for (int i = 0; i < B_DMA; ++i) {
            const int byteoff = (wave * B_DMA + i) * 1024;
            const int rblk = byteoff / (BKB * 32), within = byteoff % (BKB * 32);
            b_voff[i] = (u32)((size_t)rblk * b_block_stride) + within + lane * 16;
        }
        auto tile_origin = [&](int tj, int& m0, int& n0) {
            int tm, tn;
            if (phase == 1) {
                // Workgroup b = 8u + x takes half (u & 1) of leftover tile (u >> 1) * 8 + x: the parent keeps the workgroup's
                // residue modulo 8, i.e. its XCD's share of the tile order.
                const int u = (int)blockIdx.x >> 3, x = (int)blockIdx.x & 7;
                tile_coords<4>(p.persist_rounds * (int)gridDim.x + (u >> 1) * 8 + x, p.tiles_m, p.tiles_n, tm, tn);
                m0 = tm * 256 + (u & 1) * 128;
            } else {
                tile_coords<4>((int)blockIdx.x + tj * (int)gridDim.x, p.tiles_m, p.tiles_n, tm, tn);
                m0 = tm * 256;
            }
            n0 = tn * BN;
        };
        auto cursor_at = [&](int tj) -> Cursor {
            int m0, n0;
            tile_origin(tj, m0, n0);
            return Cursor{p.A + (size_t)m0 * a_pitch, p.B + (size_t)(n0 / 32) * b_block_stride, 0, tj};
        };
        auto advance = [&](Cursor& c) {
            if (c.kt + 1 < ktiles) {
                ++c.kt;
                c.ga += a_kstep;
                c.gb += BKB * 32;
            } else if (c.tj + 1 < my_tiles) {
                c = cursor_at(c.tj + 1);
            }  // past the last k-tile of the last tile: stay (the transfer re-fetches it into a stage nobody reads again)
        };
        auto issue = [&](const Cursor& c, int stage, int lo, int hi) {  // transfers lo..hi-1 of the k-tile (A first, then B)
            const u32 sa = smem_base + stage * STAGE_BYTES + wave * (A_DMA * 1024);
            const u32 sb = smem_base + stage * STAGE_BYTES + A_REGION + wave * (B_DMA * 1024);
#pragma unroll
            for (int d = 0; d < PER_TILE; ++d)
                if (d >= lo && d < hi) {
                    if (d < A_DMA) dma16(c.ga, a_voff[d < A_DMA ? d : 0], sa + d * 1024);
                    else dma16(c.gb, b_voff[d >= A_DMA ? d - A_DMA : 0], sb + (d - A_DMA) * 1024);
                }
        };

        AccT acc[MT][NT];  // defined by the first k-tile of every output tile (its MFMAs take a zero C operand)

        // ---- operand fragments ---------------------------------------------------------------------------
        const int lr = lane & 31, lh = lane >> 5;
        const int xrow = wm * TM + lr;
        const int xsw = chunk_swizzle<CH>(xrow);
        const int w_off = wn * NT * (BKB * 32) + lane * 16;
        v4i wp[2][NT][PPF], xp[2][MT][PPF];
        auto ldsv = [&](const char* ptr) -> v4i { return *reinterpret_cast<const v4i*>(ptr); };
        auto load_piece = [&](const char* sa, int ks, int buf, int pc) {  // piece order follows first use: x0, w0..w3, x1..x3
            const int f = pc / PPF, h = pc % PPF;
            if (f == 0 || f > NT) {
                const int i = f == 0 ? 0 : f - NT;
                xp[buf][i][h] = ldsv(sa + (xrow + i * 32) * BKB + (((KCH * ks + lh + 2 * h) ^ xsw) << 4));
            } else {
                const int j = f - 1;
                wp[buf][j][h] = ldsv(sa + A_REGION + w_off + j * (BKB * 32) + ks * (KSTEP * 32) + h * 1024);
            }
        };
        auto do_mfma = [&](int buf, int idx, bool fresh) {  // fresh (a compile-time value after unrolling): C = 0
            const int i = idx / NT, j = idx % NT;
            AccT zero;
#pragma unroll
            for (int v = 0; v < 16; ++v) zero[v] = 0;
            if constexpr (KIND == K_FP8) {
                v8i w = __builtin_shufflevector(wp[buf][j][0], wp[buf][j][PPF - 1], 0, 1, 2, 3, 4, 5, 6, 7);
                v8i x = __builtin_shufflevector(xp[buf][i][0], xp[buf][i][PPF - 1], 0, 1, 2, 3, 4, 5, 6, 7);
                acc[i][j] = __builtin_amdgcn_mfma_scale_f32_32x32x64_f8f6f4(w, x, fresh ? zero : acc[i][j], 0, 0, 0, 0, 0, 0);
            } else {
                acc[i][j] = __builtin_amdgcn_mfma_i32_32x32x32_i8(wp[buf][j][0], xp[buf][i][0], fresh ? zero : acc[i][j], 0, 0, 0);
            }
        };

        // One k-tile: `stage` holds it, c1 is the k-tile NSTAGE-1 ahead (its stage: stage + NSTAGE-1), c2 the one NSTAGE
        // ahead, which goes into `stage` once the barrier has retired it.  P: which fragment buffer holds step 0.
        auto k_tile = [&](auto parity, auto wait_c, auto first_c, int stage, const Cursor& c1, const Cursor& c2) {
            constexpr int P = decltype(parity)::value;
            constexpr bool WAIT = decltype(wait_c)::value;
            constexpr bool FIRST = decltype(first_c)::value;  // first k-tile of an output tile
            const char* sa = smem + stage * STAGE_BYTES;
            const int s1 = (stage + NSTAGE - 1) % NSTAGE;
#pragma unroll
            for (int ks = 0; ks < KS; ++ks) {
                const int cur = (P + ks) & 1, nxt = cur ^ 1;
                if (ks + 1 < KS) {
#pragma unroll
                    for (int idx = 0; idx < NMFMA; ++idx) {
                        const int q = ks * NMFMA + idx;
                        issue(c1, s1, N_AFTER + q * N_BEFORE / PRE, N_AFTER + (q + 1) * N_BEFORE / PRE);
#pragma unroll
                        for (int pc = idx * NPIECE / NMFMA; pc < (idx + 1) * NPIECE / NMFMA; ++pc) load_piece(sa, ks + 1, nxt, pc);
                        do_mfma(cur, idx, FIRST && ks == 0);
                        __builtin_amdgcn_sched_barrier(0);
                    }
                } else {
#pragma unroll
                    for (int idx = 0; idx < HPRE; ++idx) {
                        const int q = ks * NMFMA + idx;
                        issue(c1, s1, N_AFTER + q * N_BEFORE / PRE, N_AFTER + (q + 1) * N_BEFORE / PRE);
                        do_mfma(cur, idx, FIRST && ks == 0);
                        __builtin_amdgcn_sched_barrier(0);
                    }
                    __builtin_amdgcn_sched_barrier(0);
                    if constexpr (WAIT) wait_vmcnt<PER_TILE*(NSTAGE - 2)>();
                    __syncthreads();
                    __builtin_amdgcn_sched_barrier(0);
                    const char* sn = smem + ((stage + 1) % NSTAGE) * STAGE_BYTES;
#pragma unroll
                    for (int idx = 0; idx < RPOST; ++idx) {
                        issue(c2, stage, idx * N_AFTER / RPOST, (idx + 1) * N_AFTER / RPOST);
#pragma unroll
                        for (int pc = idx * NPIECE / RPOST; pc < (idx + 1) * NPIECE / RPOST; ++pc) load_piece(sn, 0, nxt, pc);
                        do_mfma(cur, HPRE + idx, FIRST && ks == 0);
                        __builtin_amdgcn_sched_barrier(0);
                    }
                    __builtin_amdgcn_sched_barrier(0);
                }
            }
        };

        // ---- epilogue --------------------------------------------------------------------------------------------
        char* strip = smem + NSTAGE * STAGE_BYTES + wave * STRIP_BYTES;
        const int srow = lane >> 4, schunk = lane & 15;  // on the way out: 16 lanes per row, four rows per instruction
        float alpha = 1.0f;
        if constexpr (KIND == K_FP8) alpha = p.a_scale[0] * p.b_scale[0];
        const bool has_bias = p.bias != nullptr;
        float out_pmax = 0.0f;  // TRACK: the largest output this lane has stored
        auto epilogue = [&](int tj) {
            int m0, n0;
            tile_origin(tj, m0, n0);
            // per-lane constants of both 64-column halves and the per-token scales of every band: loaded before the first
            // store (a load issued after a store would wait for that store's acknowledgement)
            float bias4[2][4], acol4[2][4];
            int ncol[2];
#pragma unroll
            for (int hj = 0; hj < 2; ++hj) {
                ncol[hj] = n0 + wn * TN + hj * 64 + schunk * 4;
#pragma unroll
                for (int e = 0; e < 4; ++e) bias4[hj][e] = acol4[hj][e] = 0.0f;
                if (has_bias) OutStore<OutTag>::load4(p.bias, ncol[hj], bias4[hj]);
                if constexpr (KIND == K_INT8) {
                    const float4 ac = *reinterpret_cast<const float4*>(p.alpha_col + ncol[hj]);
                    acol4[hj][0] = ac.x; acol4[hj][1] = ac.y; acol4[hj][2] = ac.z; acol4[hj][3] = ac.w;
                }
            }
            float arow_l[MT];  // INT8: the per-token scale of row lr of band i
#pragma unroll
            for (int i = 0; i < MT; ++i) arow_l[i] = (KIND == K_INT8) ? p.alpha_row[p.per_token ? m0 + wm * TM + i * 32 + lr : 0] : 1.0f;
            auto band = [&](auto i_c) {
                constexpr int i = decltype(i_c)::value;
                const float arow = arow_l[i];
#pragma unroll
                for (int hj = 0; hj < 2; ++hj) {
                    // accumulators -> strip: lane (lr, lh) owns row lr, four consecutive columns per register quad; the
                    // 16-byte chunk index is XORed with the row, which keeps both directions free of bank conflicts
#pragma unroll
                    for (int jj = 0; jj < 2; ++jj)
#pragma unroll
                        for (int q4 = 0; q4 < 4; ++q4) {
                            const int j = hj * 2 + jj;
                            const int chunk = (jj * 8 + q4 * 2 + lh) ^ (lr & 15);
                            char* spot = strip + lr * 256 + chunk * 16;
                            if constexpr (KIND == K_FP8)
                                *reinterpret_cast<float4*>(spot) = make_float4(acc[i][j][q4 * 4], acc[i][j][q4 * 4 + 1], acc[i][j][q4 * 4 + 2], acc[i][j][q4 * 4 + 3]);
                            else
                                *reinterpret_cast<int4*>(spot) = make_int4(acc[i][j][q4 * 4], acc[i][j][q4 * 4 + 1], acc[i][j][q4 * 4 + 2], acc[i][j][q4 * 4 + 3]);
                        }
                    // strip -> rows: a lane owns four consecutive columns of one row, sixteen lanes write 128 bytes of it
                    // (the wavefront's own LDS accesses complete in order: no barrier)
#pragma unroll
                    for (int tb = 0; tb < 8; tb += 4) {
                        v4i raw[4];
                        float arv[4];
#pragma unroll
                        for (int u = 0; u < 4; ++u) {
                            const int row = (tb + u) * 4 + srow;
                            raw[u] = *reinterpret_cast<const v4i*>(strip + row * 256 + ((schunk ^ (row & 15)) << 4));
                            if constexpr (KIND == K_INT8)
                                arv[u] = __builtin_bit_cast(float, __builtin_amdgcn_ds_bpermute(row << 2, __builtin_bit_cast(int, arow)));
                        }
#pragma unroll
                        for (int u = 0; u < 4; ++u) {
                            const int row = (tb + u) * 4 + srow;
                            const size_t idx = (size_t)(m0 + wm * TM + i * 32 + row) * p.n + ncol[hj];
                            float y[4];
#pragma unroll
                            for (int e = 0; e < 4; ++e) {
                                if constexpr (KIND == K_INT8) y[e] = (float)raw[u][e] * (acol4[hj][e] * arv[u]);
                                else y[e] = __int_as_float(raw[u][e]) * alpha;
                                if (has_bias) y[e] = y[e] + bias4[hj][e];
                            }
                            // (plain stores also for an output that is read only once: nontemporal ones are acknowledged so
                            // much later that the counted waits behind them stall the operand stream -- 4608x12288x3072: 184-195
                            // against 140 us)
                            if constexpr (TRACK) out_pmax = fmaxf(fmaxf(out_pmax, fmaxf(y[0], y[1])), fmaxf(y[2], y[3]));
                            OutStore<OutTag>::store4(p.C, idx, y);
                        }
                    }
                }
            };
            // A band issues sixteen stores and nothing else to memory.  Everything this wavefront issued before the epilogue
            // (the next tile's operand transfers among it) has landed once at most as many operations are outstanding as
            // the epilogue has stored since; the wait sits as late as the six-bit counter can name it.
            constexpr int WAIT_AFTER = MT - 2;
            auto band_and_wait = [&](auto i_c) {
                constexpr int i = decltype(i_c)::value;
                band(i_c);
                if constexpr (i == WAIT_AFTER) {
                    __builtin_amdgcn_sched_barrier(0);
                    wait_vmcnt<16 * (WAIT_AFTER + 1)>();
                    __builtin_amdgcn_sched_barrier(0);
                }
            };
            band_and_wait(std::integral_constant<int, 0>{});
            band_and_wait(std::integral_constant<int, 1>{});
            if constexpr (MT > 2) {
                band_and_wait(std::integral_constant<int, 2>{});
                band_and_wait(std::integral_constant<int, 3>{});
            }
        };
        // ---- the stream of k-tiles ----------------------------------------------------------------------------------
        Cursor c = cursor_at(0);
#pragma unroll
        for (int s = 0; s < NSTAGE - 1; ++s) {
            issue(c, s, 0, PER_TILE);
            advance(c);
        }
        Cursor c1 = c;
        issue(c1, NSTAGE - 1, 0, N_AFTER);
        Cursor c2 = c1;
        advance(c2);
        wait_vmcnt<0>();  // once per kernel: the first two k-tiles of every output tile run without a counter wait
        __syncthreads();
#pragma unroll
        for (int pc = 0; pc < NPIECE; ++pc) load_piece(smem, 0, 0, pc);

        int stage = 0;
        auto next = [&]() {
            c1 = c2;
            advance(c2);
            stage = (stage + 1) % NSTAGE;
        };
        using std::integral_constant;
        using P0 = integral_constant<int, 0>;
        using P1 = integral_constant<int, KS % 2>;
        // The number of k-tiles per output tile is even (the launcher checks it), so every tile starts with fragment buffer 0.
        // Its first two k-tiles landed before the previous epilogue ended (or in the prologue): no counter wait there.
        for (int tj = 0; tj < my_tiles; ++tj) {
            k_tile(P0{}, std::false_type{}, std::true_type{}, stage, c1, c2);
            next();
            k_tile(P1{}, std::false_type{}, std::false_type{}, stage, c1, c2);
            next();
            for (int kt = 2; kt < ktiles; kt += 2) {
                k_tile(P0{}, std::true_type{}, std::false_type{}, stage, c1, c2);
                next();
                k_tile(P1{}, std::true_type{}, std::false_type{}, stage, c1, c2);
                next();
            }
            epilogue(tj);
        }
        wait_vmcnt<0>();  // the transfers past the end have landed before the LDS is reused or given back
        __syncthreads();
        if constexpr (TRACK) publish_out_max<OutTag>(p.out_max, out_pmax, lane);
    }
};

template <int KIND, typename OutTag, bool TRACK>
__global__ __launch_bounds__(256, 1) void gemm_persist_kernel(GemmParams p) {
    extern __shared__ __attribute__((aligned(16))) char lq_smem[];
    GemmPersist<KIND, OutTag, 4, TRACK>::run(p, lq_smem, 0);
    if (p.persist_halves > 0) GemmPersist<KIND, OutTag, 2, TRACK>::run(p, lq_smem, 1);
}

// True when the persistent kernel implements this call: full 256x256 tiles, an even number of k-tiles, scales and bias only
// (and, for FP8, the running maximum of the outputs, which costs the epilogue two instructions per four outputs).
template <int KIND> static inline bool persist_supports(const GemmParams& p) {
    if (p.m <= 0 || p.m % 256 != 0 || p.n % 256 != 0 || p.kb % 128 != 0) return false;
    if (p.C == nullptr || p.addend != nullptr || p.gate != nullptr || p.residual != nullptr || p.C8 != nullptr || p.gelu != 0 ||
        p.out_scale != nullptr)
        return false;
    if (p.out_max != nullptr && KIND != K_FP8) return false;
    return true;
}

template <int KIND, typename OutTag, bool TRACK = false> static int launch_gemm_persist(GemmParams p, hipStream_t st) {
    using GK = GemmPersist<KIND, OutTag, 4, TRACK>;
    if (!persist_supports<KIND>(p) || TRACK != (p.out_max != nullptr)) return 1;
    p.tiles_m = p.m / 256;
    p.tiles_n = p.n / 256;
    auto kern = gemm_persist_kernel<KIND, OutTag, TRACK>;
    static bool attr_done = false;
    if (!attr_done) {
        hipError_t e = hipFuncSetAttribute(reinterpret_cast<const void*>(kern), hipFuncAttributeMaxDynamicSharedMemorySize, GK::SMEM_BYTES);
        if (e != hipSuccess) {
            set_error("gemm: cannot raise LDS limit to %d bytes: %s", GK::SMEM_BYTES, hipGetErrorString(e));
            return LQ_ERR_HIP;
        }
        attr_done = true;
    }
    const int cus = device_cu_count();
    if (cus <= 0) {
        set_error("gemm: cannot read the device's CU count");
        return LQ_ERR_HIP;
    }
    const int total = p.tiles_m * p.tiles_n;
    int grid = total;
    if (grid > cus) grid = cus - cus % 8;  // a multiple of 8, so that a workgroup's tiles stay on its XCD's share of the tile order
    if (grid <= 0) grid = 1;
    // Tiles that do not fill a last round: when they occupy at most half of the workgroups, each is cut into two 128-row
    // halves for two workgroups (wavefront tiles of 64x128), so the round that is mostly empty takes half as long --
    // 4608x12288 has 864 tiles: three rounds on 256 CUs and 96 left over, 3.5 rounds of work instead of 4 (INT8, same
    // launches otherwise: 162 -> 153 us).
    const int rounds = total / grid, left = total % grid;
    p.persist_rounds = 0;
    p.persist_halves = 0;
    if (rounds >= 1 && left > 0 && 2 * left <= grid && left % 8 == 0 && grid % 8 == 0) {
        p.persist_rounds = rounds;
        p.persist_halves = 2 * left;
    }
    hipLaunchKernelGGL(kern, dim3((unsigned)grid), dim3(GK::THREADS), GK::SMEM_BYTES, st, p);
    return check_launch("gemm_persist");
}

}  // namespace lq
