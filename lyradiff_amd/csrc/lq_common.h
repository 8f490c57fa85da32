// Shared host/device helpers for liblyraquant (gfx950 only).
#pragma once

#include <hip/hip_runtime.h>
#include <stdint.h>
#include <stdio.h>
#include <stdarg.h>
#include <type_traits>

#include "lyraquant.h"

namespace lq {

// A tensor of at least this many bytes that a kernel touches exactly once (the 16-bit output of a GEMM that a cast pass
// consumes, the input of that cast pass) is moved with nontemporal loads / stores: streaming it through the 256 MB last-level
// cache would displace the operands the GEMMs around it re-read.
constexpr size_t kStreamBytes = (size_t)64 << 20;

// ---- error plumbing ---------------------------------------------------------------------------
void set_error(const char* fmt, ...);  // stores the message for lq_last_error() (thread local)
extern int g_tactic_int8, g_tactic_fp8, g_tactic_w4a4;  // process-wide forced tile configuration, -1 = none
extern thread_local int tl_forced_tactic;                // per-thread override used while profiling
int shape_tactic_lookup(int kind, int m, int n, int k);   // per-shape cache, -1 = no entry
// Order of precedence for the tile configuration of one GEMM call; -1 means "use the built-in table".
static inline int requested_tactic(int process_wide, int kind, int m, int n, int k) {
    if (tl_forced_tactic >= 0) return tl_forced_tactic;
    if (process_wide >= 0) return process_wide;
    return shape_tactic_lookup(kind, m, n, k);
}

#define LQ_REQUIRE(cond, code, ...)     \
    do {                                \
        if (!(cond)) {                  \
            lq::set_error(__VA_ARGS__); \
            return (code);              \
        }                               \
    } while (0)

static inline int check_launch(const char* what) {
    hipError_t e = hipGetLastError();
    if (e != hipSuccess) {
        set_error("%s: HIP launch failed: %s", what, hipGetErrorString(e));
        return LQ_ERR_HIP;
    }
    return LQ_OK;
}

// ---- vector types -----------------------------------------------------------------------------
typedef int v4i __attribute__((ext_vector_type(4)));
typedef int v8i __attribute__((ext_vector_type(8)));
typedef int v16i __attribute__((ext_vector_type(16)));
typedef float v4f __attribute__((ext_vector_type(4)));
typedef float v16f __attribute__((ext_vector_type(16)));
typedef unsigned int u32;

// ---- 16-bit float formats (bit level, RNE) ------------------------------------------------------
struct F16Tag {};
struct BF16Tag {};
struct F32Tag {};

__device__ __forceinline__ float bf16_bits_to_f32(u32 b) { return __uint_as_float(b << 16); }
__device__ __forceinline__ u32 f32_to_bf16_bits(float f) {
    return (u32)__builtin_bit_cast(unsigned short, (__bf16)f);  // v_cvt_pk_bf16_f32, RNE
}
typedef __bf16 bf16x2_t __attribute__((ext_vector_type(2)));
typedef float f32x2_t __attribute__((ext_vector_type(2)));
__device__ __forceinline__ u32 pack2_bf16(float a, float b) {  // one v_cvt_pk_bf16_f32
    f32x2_t v = {a, b};
    return __builtin_bit_cast(u32, __builtin_convertvector(v, bf16x2_t));
}
typedef _Float16 f16x2_t __attribute__((ext_vector_type(2)));
__device__ __forceinline__ u32 pack2_f16(float a, float b) {
    f32x2_t v = {a, b};
    return __builtin_bit_cast(u32, __builtin_convertvector(v, f16x2_t));
}
__device__ __forceinline__ float f16_bits_to_f32(u32 h) {
    return (float)__builtin_bit_cast(_Float16, (unsigned short)h);
}
__device__ __forceinline__ u32 f32_to_f16_bits(float f) {
    return (u32)__builtin_bit_cast(unsigned short, (_Float16)f);  // v_cvt_f16_f32, RNE
}

template <typename Tag> struct Elem;
template <> struct Elem<F16Tag> {
    static constexpr int bytes = 2;
    static __device__ __forceinline__ float load(u32 bits) { return f16_bits_to_f32(bits); }
    static __device__ __forceinline__ u32 store(float f) { return f32_to_f16_bits(f); }
};
template <> struct Elem<BF16Tag> {
    static constexpr int bytes = 2;
    static __device__ __forceinline__ float load(u32 bits) { return bf16_bits_to_f32(bits); }
    static __device__ __forceinline__ u32 store(float f) { return f32_to_bf16_bits(f); }
};
template <> struct Elem<F32Tag> {
    static constexpr int bytes = 4;
    static __device__ __forceinline__ float load(u32 bits) { return __uint_as_float(bits); }
    static __device__ __forceinline__ u32 store(float f) { return __float_as_uint(f); }
};
// round an fp32 value to T and bring it back (the "T arithmetic" of the reference's half2 code).
// The empty asm pins the fp32 value: without it the compiler may merge the producing fma/add with
// the conversion into a mixed-precision instruction that rounds the exact result once to 16 bits,
// which differs (rarely) from rounding to fp32 first as the specification of these kernels does.
template <typename Tag> __device__ __forceinline__ float round_through(float f) {
    asm volatile("" : "+v"(f));
    return Elem<Tag>::load(Elem<Tag>::store(f));
}
// two values at once: for bf16 one packed conversion serves both (1.5 instead of 2 instructions per value)
template <typename Tag> __device__ __forceinline__ void round_through2(float& a, float& b) {
    if constexpr (std::is_same<Tag, BF16Tag>::value) {
        asm volatile("" : "+v"(a), "+v"(b));
        const u32 w = pack2_bf16(a, b);
        a = __uint_as_float(w << 16);
        b = __uint_as_float(w & 0xFFFF0000u);
    } else {
        a = round_through<Tag>(a);
        b = round_through<Tag>(b);
    }
}

// Unpack a 16-byte vector of 8 sixteen-bit values / 4 fp32 values to floats.
template <typename Tag> __device__ __forceinline__ void unpack8(const uint4& v, float* o) {
    const u32 w[4] = {v.x, v.y, v.z, v.w};
#pragma unroll
    for (int i = 0; i < 4; ++i) {
        o[2 * i] = Elem<Tag>::load(w[i] & 0xFFFFu);
        o[2 * i + 1] = Elem<Tag>::load(w[i] >> 16);
    }
}

// ---- streaming accesses ---------------------------------------------------------------------------
// Nontemporal 16-byte load / 4-, 8-, 16-byte stores for tensors that a quantisation kernel touches exactly once (its
// activation input, its codes).  Measured on the fp8 amax + cast kernel at 4608x3072 from HBM: the load phase of the
// whole-tensor-at-once access pattern took 7.5 us with plain loads and 6.3 us with these, and the time from launch to
// launch fell by another 1.6 us with the stores marked, because the codes no longer wait dirty in the L2s for the
// write-back at the end of the kernel.  STREAM false gives the plain access (small tensors that the next kernel
// reads straight from L2).
typedef unsigned int u32x4_t __attribute__((ext_vector_type(4)));
typedef unsigned int u32x2_t __attribute__((ext_vector_type(2)));
constexpr size_t kStreamQuantBytes = (size_t)8 << 20;  // inputs from this size on take the streaming forms
template <bool STREAM> __device__ __forceinline__ uint4 ld16(const void* p) {
    if constexpr (STREAM) {
        const u32x4_t v = __builtin_nontemporal_load(static_cast<const u32x4_t*>(p));
        return make_uint4(v.x, v.y, v.z, v.w);
    } else {
        return *static_cast<const uint4*>(p);
    }
}
template <bool STREAM> __device__ __forceinline__ void st16(void* p, const uint4& v) {
    if constexpr (STREAM) {
        const u32x4_t w = {v.x, v.y, v.z, v.w};
        __builtin_nontemporal_store(w, static_cast<u32x4_t*>(p));
    } else {
        *static_cast<uint4*>(p) = v;
    }
}
template <bool STREAM> __device__ __forceinline__ void st8(void* p, const uint2& v) {
    if constexpr (STREAM) {
        const u32x2_t w = {v.x, v.y};
        __builtin_nontemporal_store(w, static_cast<u32x2_t*>(p));
    } else {
        *static_cast<uint2*>(p) = v;
    }
}
template <bool STREAM> __device__ __forceinline__ void st4(void* p, unsigned int v) {
    if constexpr (STREAM) __builtin_nontemporal_store(v, static_cast<unsigned int*>(p));
    else *static_cast<unsigned int*>(p) = v;
}

// ---- wavefront (64 lanes) reductions ------------------------------------------------------------
// Cross-lane steps inside a row of 16 lanes use DPP operand swizzles (no LDS traffic):
// quad_perm [1,0,3,2] and [2,3,0,1] exchange with the lanes at distance 1 and 2, row_half_mirror
// and row_mirror bring in the other quad / the other half of the row.
template <int CTRL> __device__ __forceinline__ int dpp_i32(int v) {
    // every lane has a valid source under these swizzles, so the "old" operand never shows; passing 0 instead of v
    // leaves the move free to fold into the instruction that uses it (v_max_i32_dpp: one instruction per step, not three)
    return __builtin_amdgcn_update_dpp(0, v, CTRL, 0xF, 0xF, true);
}
// max over aligned groups of 8 consecutive lanes of a NON-NEGATIVE float (or +NaN pattern), result in
// every lane of the group.  Non-negative floats order like their bit patterns, so the steps run as
// integer max (no NaN canonicalisation needed around the DPP moves).
__device__ __forceinline__ float group8_max(float v) {
    int x = __builtin_bit_cast(int, v);
    x = max(x, dpp_i32<0xB1>(x));
    x = max(x, dpp_i32<0x4E>(x));
    x = max(x, dpp_i32<0x141>(x));
    return __builtin_bit_cast(float, x);
}
__device__ __forceinline__ float wave_max(float v) {
    v = group8_max(v);
    v = __builtin_bit_cast(float, max(__builtin_bit_cast(int, v), dpp_i32<0x140>(__builtin_bit_cast(int, v))));  // row_mirror
    v = fmaxf(v, __shfl_xor(v, 16, 64));  // across rows
    v = fmaxf(v, __shfl_xor(v, 32, 64));
    return v;
}
// max over aligned groups of G consecutive lanes (G power of two)
template <int G> __device__ __forceinline__ float group_max(float v) {
    if constexpr (G == 8) return group8_max(v);
#pragma unroll
    for (int off = G / 2; off > 0; off >>= 1) v = fmaxf(v, __shfl_xor(v, off, 64));
    return v;
}

// ---- rounding primitives --------------------------------------------------------------------------
// rint + saturate to [-128,127], NaN -> 0 (fmaxf/fminf drop the NaN operand)
__device__ __forceinline__ int rne_sat_s8(float x) {
    float r = __builtin_rintf(x);
    r = fminf(fmaxf(r, -128.0f), 127.0f);
    r = (x != x) ? 0.0f : r;
    return (int)r;
}
__device__ __forceinline__ int rne_sat_s4(float x) {
    float r = __builtin_rintf(x);
    r = fminf(fmaxf(r, -8.0f), 7.0f);
    r = (x != x) ? 0.0f : r;
    return (int)r;
}

// float -> int32 as the hardware defines it: round toward zero, saturate, NaN -> 0 (a C++ cast leaves
// out-of-range and NaN operands undefined)
__device__ __forceinline__ int cvt_i32_sat(float x) {
    int r;
    asm("v_cvt_i32_f32_e32 %0, %1" : "=v"(r) : "v"(x));
    return r;
}

// q[i] = clamp(rint(t[i] / s), LO, HI) (NaN -> 0) for eight values, bit-identical to the IEEE
// division but normally computed from r ~ 1/s (within 1 ulp).  With Q = t/s the exact quotient:
// |fl(t*r) - Q| <= (2^-23 + 2^-24)|Q| (reciprocal error, one rounding) and |fl(t/s) - Q| <= 2^-24 |Q|, together
// 2.4e-7 |Q|.  Only ties up to HI - 0.5 in magnitude can change the clamped result (beyond them both candidates
// saturate to the same bound), and there |Q| <= HI + 1: if t*r is more than tie_margin<HI>() = 2 * 2.4e-7 * (HI + 1)
// away from every tie, the true quotient, its fp32 rounding and t*r all round to the same integer.
// If any of the eight values fails the test (or the caller flags the scale as unsafe for a reciprocal), the whole
// octet is redone with true divisions.  The branch is taken by a wavefront when ANY lane asks for it, so the width
// of the margin is the frequency of the slow path: with the margin of 2e-4 first used here one step in five ran the
// eight divisions (64 lanes x 8 values x 4e-4); with the bound above it is one in 17 for int8 and one in 250 for int4.
// CLAMP false: the caller guarantees |t[i]| <= LIMIT * s * (1 + 2^-20) with LIMIT = HI (a scale derived from the maximum of
// these very values), so rint(t/s) cannot leave [LO, HI] and the clamp is skipped.
template <int HI> __device__ __forceinline__ constexpr float tie_margin() { return 2.0f * 2.4e-7f * (float)(HI + 1); }
template <int LO, int HI, bool CLAMP = true>
__device__ __forceinline__ void quant8(const float* t, float s, float r, bool slow, int* q) {
    float rq[8], dev = 0.0f;
#pragma unroll
    for (int i = 0; i < 8; ++i) {
        float qa = t[i] * r;
        rq[i] = __builtin_rintf(qa);
        dev = fmaxf(dev, fabsf(qa - rq[i]));  // largest distance from an integer (NaN differences drop out)
    }
    const bool risky = slow | !(dev <= 0.5f - tie_margin<HI>());
    if (__builtin_expect(risky, 0)) {
#pragma unroll
        for (int i = 0; i < 8; ++i) rq[i] = __builtin_rintf(t[i] / s);
    }
    // The hardware conversion saturates and turns NaN into 0, which is what the formula asks of a NaN
    // input; +-inf (t*r and t/s alike, r being a normal positive number here) saturates like any large value.
#pragma unroll
    for (int i = 0; i < 8; ++i) {
        const int v = cvt_i32_sat(rq[i]);
        q[i] = CLAMP ? (v < LO ? LO : (v > HI ? HI : v)) : v;
    }
}
// The dynamic per-token case: every |t[i]| <= amax and s = fl(amax / 127), so |t[i] / s| stays below 127.00002
// and nothing needs clamping; the conversion writes its low byte straight into the packed result
// (sub-dword destination select), which saves the clamp and the byte shuffles.  NaN -> 0 as above.
__device__ __forceinline__ uint2 quant8_pack_unclamped(const float* t, float s, float r, bool slow) {
    float rq[8], dev = 0.0f;
#pragma unroll
    for (int i = 0; i < 8; ++i) {
        float qa = t[i] * r;
        rq[i] = __builtin_rintf(qa);
        dev = fmaxf(dev, fabsf(qa - rq[i]));
    }
    const bool risky = slow | !(dev <= 0.5f - tie_margin<127>());
    if (__builtin_expect(risky, 0)) {
#pragma unroll
        for (int i = 0; i < 8; ++i) rq[i] = __builtin_rintf(t[i] / s);
    }
    uint2 o;
    asm("v_cvt_i32_f32_sdwa %0, %1 dst_sel:BYTE_0 dst_unused:UNUSED_PAD src0_sel:DWORD" : "=v"(o.x) : "v"(rq[0]));
    asm("v_cvt_i32_f32_sdwa %0, %1 dst_sel:BYTE_1 dst_unused:UNUSED_PRESERVE src0_sel:DWORD" : "+v"(o.x) : "v"(rq[1]));
    asm("v_cvt_i32_f32_sdwa %0, %1 dst_sel:BYTE_2 dst_unused:UNUSED_PRESERVE src0_sel:DWORD" : "+v"(o.x) : "v"(rq[2]));
    asm("v_cvt_i32_f32_sdwa %0, %1 dst_sel:BYTE_3 dst_unused:UNUSED_PRESERVE src0_sel:DWORD" : "+v"(o.x) : "v"(rq[3]));
    asm("v_cvt_i32_f32_sdwa %0, %1 dst_sel:BYTE_0 dst_unused:UNUSED_PAD src0_sel:DWORD" : "=v"(o.y) : "v"(rq[4]));
    asm("v_cvt_i32_f32_sdwa %0, %1 dst_sel:BYTE_1 dst_unused:UNUSED_PRESERVE src0_sel:DWORD" : "+v"(o.y) : "v"(rq[5]));
    asm("v_cvt_i32_f32_sdwa %0, %1 dst_sel:BYTE_2 dst_unused:UNUSED_PRESERVE src0_sel:DWORD" : "+v"(o.y) : "v"(rq[6]));
    asm("v_cvt_i32_f32_sdwa %0, %1 dst_sel:BYTE_3 dst_unused:UNUSED_PRESERVE src0_sel:DWORD" : "+v"(o.y) : "v"(rq[7]));
    return o;
}
// t[i] = fl(x[i] * f[i]) for the eight fp16 values of a 16-byte vector: the mixed-precision fma reads the
// half operand directly (x*f + 0 rounds once, like convert-then-multiply; a zero product loses its sign,
// which no consumer here looks at).
__device__ __forceinline__ void mul8_f16(const uint4& v, const float* f, float* t) {
    const u32 w[4] = {v.x, v.y, v.z, v.w};
#pragma unroll
    for (int i = 0; i < 4; ++i) {
        asm("v_fma_mix_f32 %0, %1, %2, 0 op_sel_hi:[1,0,0]" : "=v"(t[2 * i]) : "v"(w[i]), "v"(f[2 * i]));
        asm("v_fma_mix_f32 %0, %1, %2, 0 op_sel:[1,0,0] op_sel_hi:[1,0,0]" : "=v"(t[2 * i + 1]) : "v"(w[i]), "v"(f[2 * i + 1]));
    }
}
// true unless |s| lies in [2^-100, 2^100]: zero, subnormal, huge, infinite and NaN scales all take the
// exact-division path (one integer subtract and compare on the exponent field)
__device__ __forceinline__ bool scale_out_of_range(float s) {
    return ((__float_as_uint(s) & 0x7FFFFFFFu) - 0x0D800000u) > (0x71800000u - 0x0D800000u);
}
// fl(a / D) for a compile-time divisor D from its correctly rounded reciprocal (three operations
// instead of the ~12 of an IEEE division): q0 = fl(a*Y), rem = a - q0*D exactly (one fma),
// result = fl(q0 + rem*Y) is the correctly rounded quotient when Y = fl(1/D) and nothing leaves
// the normal range (Markstein).  Callers check the result with scale_out_of_range() and redo the
// division exactly when it fails.
__device__ __forceinline__ float div_by_const_fast(float a, float D, float Y) {
    float q0 = a * Y;
    float rem = __builtin_fmaf(-q0, D, a);
    return __builtin_fmaf(rem, Y, q0);
}
// reciprocal good to 1 ulp (hardware v_rcp_f32): what quant8's error bound assumes
__device__ __forceinline__ float fast_recip(float s) { return __builtin_amdgcn_rcpf(s); }

// true when 1/s cannot be trusted as a reciprocal (zero, subnormal, infinite or NaN scale)
__device__ __forceinline__ bool recip_unsafe(float s, float r) {
    return !(fabsf(s) >= 1e-30f && fabsf(r) < 1e30f && fabsf(r) >= 1e-30f);
}
// four ints in [-128,127] -> packed bytes
__device__ __forceinline__ u32 pack4_s8(int a, int b, int c, int d) {
    u32 lo = __builtin_amdgcn_perm((u32)b, (u32)a, 0x0c0c0400u);  // bytes: a.b0, b.b0, 0, 0
    u32 hi = __builtin_amdgcn_perm((u32)d, (u32)c, 0x04000c0cu);  // bytes: 0, 0, c.b0, d.b0
    return lo | hi;
}

// tanh from basic IEEE operations only (no fused multiply-add), so that a CPU restatement can
// reproduce it bit for bit; accurate to about 2e-7 absolute.
__device__ __forceinline__ float tanh_basic(float u) {
    float a = fminf(fabsf(u), 10.0f);
    float t = a * 2.8853900817779268f;
    float n = __builtin_rintf(t);
    float f = t - n;
    float p = 1.52527338040598e-05f;
    p = p * f; p = p + 0.000154035303933816f;
    p = p * f; p = p + 0.00133335581464284f;
    p = p * f; p = p + 0.00961812910762848f;
    p = p * f; p = p + 0.0555041086648216f;
    p = p * f; p = p + 0.240226506959101f;
    p = p * f; p = p + 0.693147180559945f;
    p = p * f; p = p + 1.0f;
    float e = ldexpf(p, (int)n);
    float d = e + 1.0f;
    float r = 1.0f - 2.0f / d;
    return copysignf(r, u);
}
__device__ __forceinline__ float gelu_tanh(float x) {
    float inner = 0.7978845608028654f * (x + 0.044715f * (x * x * x));
    return x * (0.5f * (1.0f + tanh_basic(inner)));
}

// GELU for the fused FP8 epilogue: hardware exp2 / reciprocal (the reference's counterpart is
// cuBLASLt's GELU epilogue, utils/cublasMMWrapper.cc:1195-1199, whose arithmetic is not visible).
__device__ __forceinline__ float gelu_fast(float x) {
    // 0.5 x (1 + tanh(u)) = x / (1 + exp(-2u)),  u = sqrt(2/pi) (x + 0.044715 x^3);  -2u log2(e) = x (A + B x^2)
    constexpr float A = -2.0f * 0.7978845608028654f * 1.4426950408889634f, B = A * 0.044715f;
    const float t = x * __builtin_fmaf(B, x * x, A);  // one rounding fewer than the separate multiply and add; the result is compared by tolerance
    const float e = __builtin_amdgcn_exp2f(t);             // exp(-2u): 0 for large x, inf for very negative x
    return x * __builtin_amdgcn_rcpf(1.0f + e);            // x, resp. -0
}

static inline hipStream_t as_stream(lq_stream_t s) { return reinterpret_cast<hipStream_t>(s); }

}  // namespace lq
