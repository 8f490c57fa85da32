// Shared host/device helpers for liblyraquant (gfx950 only).
#pragma once

#include <hip/hip_runtime.h>
#include <stdint.h>
#include <stdio.h>
#include <stdarg.h>

#include "lyraquant.h"

namespace lq {

// ---- error plumbing ---------------------------------------------------------------------------
void set_error(const char* fmt, ...);  // stores the message for lq_last_error() (thread local)

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
// round an fp32 value to T and bring it back (the "T arithmetic" of the reference's half2 code)
template <typename Tag> __device__ __forceinline__ float round_through(float f) {
    return Elem<Tag>::load(Elem<Tag>::store(f));
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

// ---- wavefront (64 lanes) reductions ------------------------------------------------------------
__device__ __forceinline__ float wave_max(float v) {
#pragma unroll
    for (int off = 32; off > 0; off >>= 1) v = fmaxf(v, __shfl_xor(v, off, 64));
    return v;
}
// max over aligned groups of G consecutive lanes (G power of two)
template <int G> __device__ __forceinline__ float group_max(float v) {
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

static inline hipStream_t as_stream(lq_stream_t s) { return reinterpret_cast<hipStream_t>(s); }

}  // namespace lq
