// FP8 e4m3 (OCP e4m3fn on gfx950) per-tensor quantisation: amax -> scale, and scale-cast.
//
// Formulas follow the lyraDiff reference: kernels/lora/load_lora.cu:16-23,48-54 (scale =
// max|x| / 448 through an integer-punned atomic max) and utils/memory_utils.cu:431-446
// (dst = e4m3(float(src) * (invert ? 1/scale : scale)), saturating to +-448, RNE).
// Unlike the reference (one atomic per element, 65 536 threads, byte stores) the amax kernel
// reduces in registers -> wavefront shuffles -> LDS and issues one atomic per workgroup, and
// the cast kernel moves 32 B in / 16 B out per lane per step.
#include "lq_common.h"
#include <atomic>
#include <mutex>

namespace lq {

template <typename Tag> struct Chunk16 {  // 16 consecutive elements of a 16-bit type, or 8 of fp32
    static constexpr int elems = Elem<Tag>::bytes == 2 ? 16 : 8;
};

template <typename Tag, bool NT = false>
__device__ __forceinline__ void load_elems(const void* base, size_t idx, float* o) {
    if constexpr (Elem<Tag>::bytes == 2) {
        uint4 a, b;
        if constexpr (NT) {  // read-once input of a large cast: do not keep its lines in the caches
            typedef unsigned int u32x4_t __attribute__((ext_vector_type(4)));
            const u32x4_t* p = reinterpret_cast<const u32x4_t*>(static_cast<const char*>(base) + idx * 2);
            const u32x4_t a4 = __builtin_nontemporal_load(p), b4 = __builtin_nontemporal_load(p + 1);
            a = make_uint4(a4.x, a4.y, a4.z, a4.w), b = make_uint4(b4.x, b4.y, b4.z, b4.w);
        } else {
            const uint4* p = reinterpret_cast<const uint4*>(static_cast<const char*>(base) + idx * 2);
            a = p[0], b = p[1];
        }
        unpack8<Tag>(a, o);
        unpack8<Tag>(b, o + 8);
    } else {
        const float4* p = reinterpret_cast<const float4*>(static_cast<const char*>(base) + idx * 4);
        float4 a = p[0], b = p[1];
        o[0] = a.x; o[1] = a.y; o[2] = a.z; o[3] = a.w;
        o[4] = b.x; o[5] = b.y; o[6] = b.z; o[7] = b.w;
    }
}
template <typename Tag> __device__ __forceinline__ float load_one(const void* base, size_t idx) {
    if constexpr (Elem<Tag>::bytes == 2) return Elem<Tag>::load(static_cast<const unsigned short*>(base)[idx]);
    else return static_cast<const float*>(base)[idx];
}

// saturate-to-finite RNE conversion of two floats into the low or high half of a dword
// (finite inputs and infinities; NaN lanes are patched by the caller)
__device__ __forceinline__ u32 cvt2_e4m3(float a, float b, u32 old, bool hi) {
    float ca = __builtin_amdgcn_fmed3f(a, 448.0f, -448.0f);
    float cb = __builtin_amdgcn_fmed3f(b, 448.0f, -448.0f);
    return hi ? (u32)__builtin_amdgcn_cvt_pk_fp8_f32(ca, cb, (int)old, true)
              : (u32)__builtin_amdgcn_cvt_pk_fp8_f32(ca, cb, (int)old, false);
}
__device__ __forceinline__ u32 nan_code(float v) { return 0x7Fu | ((__float_as_uint(v) >> 24) & 0x80u); }
// four floats -> four e4m3 codes; NaN -> 0x7F with the sign of the NaN (rare: one unordered
// compare per pair decides whether the patch-up path runs at all)
__device__ __forceinline__ u32 cvt4_e4m3(float a, float b, float c, float d) {
    u32 w = cvt2_e4m3(a, b, 0u, false);
    w = cvt2_e4m3(c, d, w, true);
    if (__builtin_expect(__builtin_isunordered(a, b) || __builtin_isunordered(c, d), 0)) {
        if (a != a) w = (w & 0xFFFFFF00u) | nan_code(a);
        if (b != b) w = (w & 0xFFFF00FFu) | (nan_code(b) << 8);
        if (c != c) w = (w & 0xFF00FFFFu) | (nan_code(c) << 16);
        if (d != d) w = (w & 0x00FFFFFFu) | (nan_code(d) << 24);
    }
    return w;
}
__device__ __forceinline__ u32 cvt1_e4m3(float a) { return cvt4_e4m3(a, 0.0f, 0.0f, 0.0f) & 0xFFu; }

// Non-negative floats order like their bit patterns, so an integer atomic max works.  Thousands of
// same-address atomics serialise in L2, so a workgroup first looks at the current value and only
// issues the atomic when it would raise it (after the first few workgroups almost none do).
__device__ __forceinline__ void publish_scale(float* scale, float v) {
    int cur = __hip_atomic_load(reinterpret_cast<int*>(scale), __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
    if (__float_as_int(v) > cur) atomicMax(reinterpret_cast<int*>(scale), __float_as_int(v));
}

template <typename Tag>
__global__ __launch_bounds__(256) void fp8_amax_kernel(float* __restrict__ scale, const void* __restrict__ x, size_t n) {
    constexpr int E = Chunk16<Tag>::elems;
    const size_t nchunks = n / E;
    float amax = 0.0f;
    for (size_t c = (size_t)blockIdx.x * blockDim.x + threadIdx.x; c < nchunks; c += (size_t)gridDim.x * blockDim.x) {
        float v[16];
        load_elems<Tag>(x, c * E, v);
#pragma unroll
        for (int i = 0; i < E; ++i) amax = fmaxf(amax, fabsf(v[i]));
    }
    // tail elements (fewer than E) handled by the first threads of block 0
    if (blockIdx.x == 0) {
        size_t i = nchunks * E + threadIdx.x;
        if (i < n) amax = fmaxf(amax, fabsf(load_one<Tag>(x, i)));
    }
    __shared__ float red[4];
    amax = wave_max(amax);
    if ((threadIdx.x & 63) == 0) red[threadIdx.x >> 6] = amax;
    __syncthreads();
    if (threadIdx.x == 0) {
        amax = fmaxf(fmaxf(red[0], red[1]), fmaxf(red[2], red[3]));
        // non-negative floats order like their bit patterns
        publish_scale(scale, amax / 448.0f);
    }
}

template <typename Tag, bool NT>
__global__ __launch_bounds__(256) void fp8_cast_kernel(uint8_t* __restrict__ dst, const void* __restrict__ src,
                                                       const float* __restrict__ scale, int invert, size_t n) {
    constexpr int E = Chunk16<Tag>::elems;
    const float s = scale[0];
    const float r = invert ? 1.0f / s : s;
    const size_t nchunks = n / E;
    for (size_t c = (size_t)blockIdx.x * blockDim.x + threadIdx.x; c < nchunks; c += (size_t)gridDim.x * blockDim.x) {
        float v[16];
        load_elems<Tag, NT>(src, c * E, v);
        u32 w[4];
#pragma unroll
        for (int i = 0; i < E / 4; ++i)
            w[i] = cvt4_e4m3(v[4 * i] * r, v[4 * i + 1] * r, v[4 * i + 2] * r, v[4 * i + 3] * r);
        if constexpr (E == 16) *reinterpret_cast<uint4*>(dst + c * 16) = make_uint4(w[0], w[1], w[2], w[3]);
        else *reinterpret_cast<uint2*>(dst + c * 8) = make_uint2(w[0], w[1]);
    }
    if (blockIdx.x == 0) {
        size_t i = nchunks * E + threadIdx.x;
        if (i < n) dst[i] = (uint8_t)cvt1_e4m3(load_one<Tag>(src, i) * r);
    }
}

// The same cast for a matrix whose rows are `src_ld` elements apart, written with rows `dst_ld` bytes apart: a block of
// columns of a wider destination (the concatenated input of FLUX's single-block output projection).  cols % E == 0.
template <typename Tag>
__global__ __launch_bounds__(256) void fp8_cast_2d_kernel(uint8_t* __restrict__ dst, size_t dst_ld, const void* __restrict__ src,
                                                          size_t src_ld, const float* __restrict__ scale, int invert,
                                                          size_t rows, size_t cols) {
    constexpr int E = Chunk16<Tag>::elems;
    const float s = scale[0];
    const float r = invert ? 1.0f / s : s;
    const size_t cpr = cols / E, nchunks = rows * cpr;
    for (size_t c = (size_t)blockIdx.x * blockDim.x + threadIdx.x; c < nchunks; c += (size_t)gridDim.x * blockDim.x) {
        const size_t row = c / cpr, cc = c - row * cpr;
        float v[16];
        load_elems<Tag>(src, row * src_ld + cc * E, v);
        u32 w[4];
#pragma unroll
        for (int i = 0; i < E / 4; ++i)
            w[i] = cvt4_e4m3(v[4 * i] * r, v[4 * i + 1] * r, v[4 * i + 2] * r, v[4 * i + 3] * r);
        uint8_t* o = dst + row * dst_ld + cc * E;
        if constexpr (E == 16) *reinterpret_cast<uint4*>(o) = make_uint4(w[0], w[1], w[2], w[3]);
        else *reinterpret_cast<uint2*>(o) = make_uint2(w[0], w[1]);
    }
}

// scalar fallback for unaligned buffers
template <typename Tag>
__global__ __launch_bounds__(256) void fp8_cast_scalar_kernel(uint8_t* __restrict__ dst, const void* __restrict__ src,
                                                              const float* __restrict__ scale, int invert, size_t n) {
    const float s = scale[0];
    const float r = invert ? 1.0f / s : s;
    for (size_t i = (size_t)blockIdx.x * blockDim.x + threadIdx.x; i < n; i += (size_t)gridDim.x * blockDim.x)
        dst[i] = (uint8_t)cvt1_e4m3(load_one<Tag>(src, i) * r);
}
template <typename Tag>
__global__ __launch_bounds__(256) void fp8_amax_scalar_kernel(float* __restrict__ scale, const void* __restrict__ x, size_t n) {
    float amax = 0.0f;
    for (size_t i = (size_t)blockIdx.x * blockDim.x + threadIdx.x; i < n; i += (size_t)gridDim.x * blockDim.x)
        amax = fmaxf(amax, fabsf(load_one<Tag>(x, i)));
    __shared__ float red[4];
    amax = wave_max(amax);
    if ((threadIdx.x & 63) == 0) red[threadIdx.x >> 6] = amax;
    __syncthreads();
    if (threadIdx.x == 0) {
        amax = fmaxf(fmaxf(red[0], red[1]), fmaxf(red[2], red[3]));
        publish_scale(scale, amax / 448.0f);
    }
}

__global__ void fill_f32_kernel(float* p, float v) { p[0] = v; }

// ---- device scratch of the dynamic (amax + cast) quantiser --------------------------------------------------------
// One statically allocated block per GPU (each device that loads this library holds its own copy until the process
// ends): the time-out flag and the barrier slots of the one-launch kernel, and the partial maxima + ticket counter of
// the two-launch kernel pair.  Static device memory starts zeroed, and every user leaves its counters at zero again.
// Host code never uses the array's name as an address: device_scratch() asks the runtime for the device address once
// per device (hipGetSymbolAddress) and the kernels receive that pointer as an argument.
constexpr int kCoopThreads = 512;
constexpr int kCoopMaxBlocks = 1024;
constexpr int kCoopSlots = 16;
constexpr size_t kTicketSlab = 32768;     // elements per workgroup of the partial-maximum pass
constexpr size_t kTicketMaxSlabs = 8192;  // partial maxima the scratch holds => at most 2^28 elements per call
constexpr int kTicketGroups = 16;         // first-level ticket counters, one 128-byte line each
struct CounterLine {  // one counter per 128-byte line: polls of one word must not queue behind atomics on another
    unsigned count;
    unsigned pad[31];
};
struct CoopSlot {
    CounterLine group[8];
    CounterLine top;
    CounterLine flag;
    float partials[kCoopMaxBlocks];
};
struct TicketRegion {
    CounterLine group[kTicketGroups];
    CounterLine top;
    float partials[kTicketMaxSlabs];
};
struct FusedScratch {
    unsigned timeout;
    unsigned pad[63];
    CoopSlot coop[kCoopSlots];
    TicketRegion ticket;
};
static __device__ __align__(256) unsigned char scratch[sizeof(FusedScratch)];

constexpr int kMaxDevices = 64;
static std::atomic<FusedScratch*> g_scratch_ptr[kMaxDevices];
static std::mutex g_scratch_mutex;

// Device address of `scratch` on the current device (nullptr, with the error message set, on failure).
static FusedScratch* device_scratch(int* dev_out = nullptr) {
    int dev = -1;
    if (hipGetDevice(&dev) != hipSuccess || dev < 0 || dev >= kMaxDevices) {
        (void)hipGetLastError();
        set_error("fp8 quantiser: cannot identify the current device (%d)", dev);
        return nullptr;
    }
    if (dev_out) *dev_out = dev;
    FusedScratch* p = g_scratch_ptr[dev].load(std::memory_order_acquire);
    if (p) return p;
    std::lock_guard<std::mutex> lock(g_scratch_mutex);
    p = g_scratch_ptr[dev].load(std::memory_order_relaxed);
    if (p) return p;
    void* addr = nullptr;
    hipError_t e = hipGetSymbolAddress(&addr, HIP_SYMBOL(scratch));
    if (e != hipSuccess || addr == nullptr) {
        (void)hipGetLastError();
        set_error("fp8 quantiser: hipGetSymbolAddress(scratch) failed on device %d: %s", dev, hipGetErrorString(e));
        return nullptr;
    }
    p = static_cast<FusedScratch*>(addr);
    g_scratch_ptr[dev].store(p, std::memory_order_release);
    return p;
}

// A stream owns one barrier slot for the life of the process (work of one stream runs in order, so its launches never
// overlap); streams beyond kCoopSlots get none and use the scratch-free kernel sequence.
struct StreamSlots {
    hipStream_t stream[kCoopSlots];
    int used = 0;
};
static StreamSlots g_stream_slots[kMaxDevices];
static std::mutex g_slot_mutex;
static int slot_for_stream(int dev, hipStream_t st) {
    std::lock_guard<std::mutex> lock(g_slot_mutex);
    StreamSlots& t = g_stream_slots[dev];
    for (int i = 0; i < t.used; ++i)
        if (t.stream[i] == st) return i;
    if (t.used == kCoopSlots) return -1;
    t.stream[t.used] = st;
    return t.used++;
}

// Fused dynamic per-tensor quantisation in ONE launch: every thread keeps up to KEEP 16-element
// chunks of its slice in registers while the tensor-wide absmax is formed (workgroup partials ->
// grid-wide barrier -> every workgroup reduces the partials), then casts from registers, so the
// source is read from HBM once (3 bytes moved per element: the algorithmic minimum).  Chunks
// beyond KEEP are re-read in the second phase (from L2 / Infinity Cache when they fit).
//
// The grid never exceeds what the device holds at once (CUs x resident workgroups), so every workgroup is running when
// the barrier is reached -- provided nothing else occupies the device; when another stream's kernels hold CUs the
// late workgroups start once those retire, and the wait is bounded so that even a starved grid terminates: on
// time-out the kernel raises the time-out flag (lq_fp8_amax_cast_status reports it) and the scale it writes is NaN,
// which poisons the output visibly instead of hanging the device.  The barrier re-arms itself.  Launches that may
// overlap in time use different slots: a slot belongs to one stream, and the path is not taken under stream capture
// (a captured launch could later replay on any stream).

// Two-level arrive counter (workgroup ids congruent modulo 8 share a counter, so at most G/8 atomics
// hit one address; the last arriver of a group bumps the top counter, the last group flips the flag
// everybody polls).  Counters are cleared by their last arriver.  Only relaxed device-scope atomics are used for the
// hand-over -- no release/acquire fences, which on this multi-die part would write back / invalidate whole L2s.  The
// partial maximum is published with a device-scope atomic store and the thread then waits explicitly (s_waitcnt vmcnt(0):
// on this architecture stores count in vmcnt) for its acknowledgement before the arrival is counted.
// Returns false on time-out.
__device__ __forceinline__ bool grid_barrier(CoopSlot* slot, unsigned* timeout, float partial) {
    __shared__ int ok;
    __syncthreads();
    if (threadIdx.x == 0) {
        const unsigned G = gridDim.x, grp = blockIdx.x & 7;
        const unsigned in_group = (G - grp + 7) / 8, ngroups = G < 8 ? G : 8;
        const unsigned f0 = __hip_atomic_load(&slot->flag.count, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
        __hip_atomic_store(&slot->partials[blockIdx.x], partial, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
        asm volatile("s_waitcnt vmcnt(0)" ::: "memory");  // the device-scope (write-through) store has been acknowledged
        unsigned x = __hip_atomic_fetch_add(&slot->group[grp].count, 1u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
        if (x == in_group - 1) {
            __hip_atomic_store(&slot->group[grp].count, 0u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
            unsigned t = __hip_atomic_fetch_add(&slot->top.count, 1u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
            if (t == ngroups - 1) {
                __hip_atomic_store(&slot->top.count, 0u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
                asm volatile("s_waitcnt vmcnt(0)" ::: "memory");  // counters are zero again before anyone is released
                __hip_atomic_store(&slot->flag.count, f0 + 1u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
            }
        }
        int good = 0;
        for (int spin = 0; spin < (1 << 18); ++spin) {
            if (__hip_atomic_load(&slot->flag.count, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT) != f0) {
                good = 1;
                break;
            }
            __builtin_amdgcn_s_sleep(1);
        }
        if (!good) __hip_atomic_store(timeout, 1u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
        ok = good;
    }
    __syncthreads();
    return ok != 0;
}

template <typename Tag, int KEEP>
__global__ __launch_bounds__(kCoopThreads, (KEEP > 8 ? 4 : 1)) void fp8_amax_cast_coop_kernel(uint8_t* __restrict__ dst,
                                                                          float* __restrict__ scale_out,
                                                                          const void* __restrict__ src, size_t n,
                                                                          CoopSlot* slot, unsigned* timeout) {
    constexpr int E = Chunk16<Tag>::elems;
    constexpr int V = 2;  // uint4 vectors per chunk (32 bytes for every element type)
    const size_t nchunks = n / E;
    const size_t stride = (size_t)gridDim.x * blockDim.x;
    const size_t first = (size_t)blockIdx.x * blockDim.x + threadIdx.x;
    uint4 keep[KEEP][V];
    float amax = 0.0f;
    auto chunk_amax = [&](const uint4* v) {
        float f[16];
        if constexpr (Elem<Tag>::bytes == 2) { unpack8<Tag>(v[0], f); unpack8<Tag>(v[1], f + 8); }
        else { f[0] = __uint_as_float(v[0].x); f[1] = __uint_as_float(v[0].y); f[2] = __uint_as_float(v[0].z); f[3] = __uint_as_float(v[0].w);
               f[4] = __uint_as_float(v[1].x); f[5] = __uint_as_float(v[1].y); f[6] = __uint_as_float(v[1].z); f[7] = __uint_as_float(v[1].w); }
#pragma unroll
        for (int i = 0; i < E; ++i) amax = fmaxf(amax, fabsf(f[i]));
    };
#pragma unroll
    for (int it = 0; it < KEEP; ++it) {
        size_t c = first + it * stride;
        keep[it][0] = make_uint4(0, 0, 0, 0);
        keep[it][1] = make_uint4(0, 0, 0, 0);
        if (c < nchunks) {
            const uint4* p = reinterpret_cast<const uint4*>(static_cast<const char*>(src) + c * 32);
            keep[it][0] = p[0];
            keep[it][1] = p[1];
        }
    }
#pragma unroll
    for (int it = 0; it < KEEP; ++it) chunk_amax(keep[it]);
    for (size_t c = first + KEEP * stride; c < nchunks; c += stride) {
        const uint4* p = reinterpret_cast<const uint4*>(static_cast<const char*>(src) + c * 32);
        uint4 v[2] = {p[0], p[1]};
        chunk_amax(v);
    }
    if (blockIdx.x == 0) {
        size_t i = nchunks * E + threadIdx.x;
        if (i < n) amax = fmaxf(amax, fabsf(load_one<Tag>(src, i)));
    }
    __shared__ float red[kCoopThreads / 64];
    amax = wave_max(amax);
    if ((threadIdx.x & 63) == 0) red[threadIdx.x >> 6] = amax;
    __syncthreads();
    float wg_max = 0.0f;
    if (threadIdx.x == 0) {
#pragma unroll
        for (int i = 0; i < kCoopThreads / 64; ++i) wg_max = fmaxf(wg_max, red[i]);
    }
    const bool arrived = grid_barrier(slot, timeout, wg_max);
    // Only the raw 16-byte vectors live across the barrier: the empty asm makes them new values to the compiler, which
    // would otherwise keep the unpacked fp32 copies of the first phase as well (twice the registers, half the occupancy).
#pragma unroll
    for (int it = 0; it < KEEP; ++it)
#pragma unroll
        for (int u = 0; u < V; ++u)
            asm volatile("" : "+v"(keep[it][u].x), "+v"(keep[it][u].y), "+v"(keep[it][u].z), "+v"(keep[it][u].w));
    float m = 0.0f;
    for (int i = threadIdx.x; i < (int)gridDim.x; i += kCoopThreads)
        m = fmaxf(m, __hip_atomic_load(&slot->partials[i], __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT));
    m = wave_max(m);
    __syncthreads();
    if ((threadIdx.x & 63) == 0) red[threadIdx.x >> 6] = m;
    __syncthreads();
    m = 0.0f;
#pragma unroll
    for (int i = 0; i < kCoopThreads / 64; ++i) m = fmaxf(m, red[i]);
    const float s = arrived ? m / 448.0f : __builtin_nanf("");
    if (blockIdx.x == 0 && threadIdx.x == 0) scale_out[0] = s;
    const float r = 1.0f / s;
    auto chunk_cast = [&](const uint4* v, size_t c) {
        float f[16];
        if constexpr (Elem<Tag>::bytes == 2) { unpack8<Tag>(v[0], f); unpack8<Tag>(v[1], f + 8); }
        else { f[0] = __uint_as_float(v[0].x); f[1] = __uint_as_float(v[0].y); f[2] = __uint_as_float(v[0].z); f[3] = __uint_as_float(v[0].w);
               f[4] = __uint_as_float(v[1].x); f[5] = __uint_as_float(v[1].y); f[6] = __uint_as_float(v[1].z); f[7] = __uint_as_float(v[1].w); }
        u32 w[4];
#pragma unroll
        for (int i = 0; i < E / 4; ++i) w[i] = cvt4_e4m3(f[4 * i] * r, f[4 * i + 1] * r, f[4 * i + 2] * r, f[4 * i + 3] * r);
        if constexpr (E == 16) *reinterpret_cast<uint4*>(dst + c * 16) = make_uint4(w[0], w[1], w[2], w[3]);
        else *reinterpret_cast<uint2*>(dst + c * 8) = make_uint2(w[0], w[1]);
    };
#pragma unroll
    for (int it = 0; it < KEEP; ++it) {
        size_t c = first + it * stride;
        if (c < nchunks) chunk_cast(keep[it], c);
    }
    for (size_t c = first + KEEP * stride; c < nchunks; c += stride) {
        const uint4* p = reinterpret_cast<const uint4*>(static_cast<const char*>(src) + c * 32);
        uint4 v[2] = {p[0], p[1]};
        chunk_cast(v, c);
    }
    if (blockIdx.x == 0) {
        size_t i = nchunks * E + threadIdx.x;
        if (i < n) dst[i] = (uint8_t)cvt1_e4m3(load_one<Tag>(src, i) * r);
    }
}

// Returns LQ_OK when the fused launch was issued, 1 when the caller should fall back to the scratch-free
// kernel sequence (unaligned buffers, stream capture, no barrier slot left for this stream, occupancy query failed),
// a negative status on an error.
// KEEP = 8 chunks of 32 bytes (64 registers) stay in each thread's registers across the barrier: with two workgroups
// per CU that holds a tensor of up to 33.5 M sixteen-bit elements on 256 CUs; the rest of a larger one is read twice.
template <typename Tag, int KEEP> struct CoopCapacity {
    int blocks_per_cu = 0, num_cu = 0;
    static const CoopCapacity& get(int dev) {  // queried once (thread-safe initialisation of a function-local static)
        static const CoopCapacity cap = [dev] {
            CoopCapacity c;
            int occ = 0;
            hipDeviceProp_t prop;
            if (hipGetDeviceProperties(&prop, dev) == hipSuccess &&
                hipOccupancyMaxActiveBlocksPerMultiprocessor(&occ, fp8_amax_cast_coop_kernel<Tag, KEEP>, kCoopThreads, 0) == hipSuccess &&
                occ >= 1) {
                c.blocks_per_cu = occ > 2 ? 2 : occ;
                c.num_cu = prop.multiProcessorCount;
            }
            (void)hipGetLastError();
            return c;
        }();
        return cap;
    }
};

template <typename Tag>
static int launch_amax_cast_coop(uint8_t* dst, float* scale_out, const void* src, size_t n, hipStream_t st) {
    if (reinterpret_cast<uintptr_t>(src) % 16 != 0 || reinterpret_cast<uintptr_t>(dst) % 16 != 0) return 1;
    hipStreamCaptureStatus cs = hipStreamCaptureStatusNone;
    if (hipStreamIsCapturing(st, &cs) != hipSuccess || cs != hipStreamCaptureStatusNone) {
        (void)hipGetLastError();
        return 1;
    }
    int dev = 0;
    FusedScratch* ws = device_scratch(&dev);
    if (ws == nullptr) return LQ_ERR_HIP;
    const int slot = slot_for_stream(dev, st);
    if (slot < 0) return 1;
    const CoopCapacity<Tag, 8>& cap = CoopCapacity<Tag, 8>::get(dev);
    const int blocks_per_cu = cap.blocks_per_cu, num_cu = cap.num_cu;
    if (blocks_per_cu == 0) return 1;
    // One workgroup per CU while the tensor fits in their registers (fewer parties at the barrier: 15.4 us against 17.0
    // at 4608x3072), two for a larger one (more of it stays in registers: 39.6 us against 46.3 at 4608x12288).
    size_t need = (n / Chunk16<Tag>::elems + kCoopThreads - 1) / kCoopThreads;
    // A tensor that two workgroups per CU cannot hold with 8 chunks per thread (more than 33.5 M sixteen-bit elements)
    // takes the form with 10 chunks, 80 of the 128 registers a lane may use at that occupancy (12 spill): 42 M elements stay in
    // registers and less of the tensor is read twice.
    if (need > (size_t)8 * 2 * num_cu) {
        const CoopCapacity<Tag, 10>& cap12 = CoopCapacity<Tag, 10>::get(dev);
        if (cap12.blocks_per_cu == 2) {
            int grid = 2 * num_cu;
            if (grid > kCoopMaxBlocks) grid = kCoopMaxBlocks;
            hipLaunchKernelGGL((fp8_amax_cast_coop_kernel<Tag, 10>), dim3(grid), dim3(kCoopThreads), 0, st, dst, scale_out, src, n,
                               &ws->coop[slot], &ws->timeout);
            return check_launch("fp8_amax_cast_fused");
        }
    }
    int grid = (need <= (size_t)8 * num_cu ? 1 : blocks_per_cu) * num_cu;
    if (grid > kCoopMaxBlocks) grid = kCoopMaxBlocks;
    if ((size_t)grid > need) grid = need ? (int)need : 1;
    hipLaunchKernelGGL((fp8_amax_cast_coop_kernel<Tag, 8>), dim3(grid), dim3(kCoopThreads), 0, st, dst, scale_out, src, n,
                       &ws->coop[slot], &ws->timeout);
    return check_launch("fp8_amax_cast_fused");
}

// ---- two launches, no barrier: partial maxima + ticket, then the cast ------------------------------------------------
// Workgroup b reduces elements [b * kTicketSlab, (b+1) * kTicketSlab) to one partial maximum in the scratch block and
// takes a ticket; the workgroup that draws the last ticket reduces all partials, writes scale_out[0] = max / 448 and
// puts the ticket counters back to zero.  Nobody waits for anybody, so the kernel is safe under any scheduling, under
// stream capture and in graph replays; the cast kernel that follows re-reads the source (from the Infinity Cache when
// it fits).  All calls on one device share the one scratch block: calls that overlap in time race.
template <typename Tag>
__global__ __launch_bounds__(256) void fp8_amax_ticket_kernel(TicketRegion* __restrict__ ws, float* __restrict__ scale_out,
                                                              const void* __restrict__ x, size_t n) {
    constexpr int E = Chunk16<Tag>::elems;
    constexpr int PER_THREAD = (int)(kTicketSlab / E / 256);  // chunks per thread: all requested before the first is used
    const size_t nchunks = n / E;
    const size_t c0 = (size_t)blockIdx.x * (kTicketSlab / E) + threadIdx.x;
    uint4 v[PER_THREAD][2];
#pragma unroll
    for (int it = 0; it < PER_THREAD; ++it) {
        const size_t c = c0 + (size_t)it * 256;
        v[it][0] = make_uint4(0, 0, 0, 0);
        v[it][1] = make_uint4(0, 0, 0, 0);
        if (c < nchunks) {
            const uint4* p = reinterpret_cast<const uint4*>(static_cast<const char*>(x) + c * 32);
            v[it][0] = p[0];
            v[it][1] = p[1];
        }
    }
    float amax = 0.0f;
#pragma unroll
    for (int it = 0; it < PER_THREAD; ++it) {
        float f[16];
        if constexpr (Elem<Tag>::bytes == 2) { unpack8<Tag>(v[it][0], f); unpack8<Tag>(v[it][1], f + 8); }
        else { f[0] = __uint_as_float(v[it][0].x); f[1] = __uint_as_float(v[it][0].y); f[2] = __uint_as_float(v[it][0].z); f[3] = __uint_as_float(v[it][0].w);
               f[4] = __uint_as_float(v[it][1].x); f[5] = __uint_as_float(v[it][1].y); f[6] = __uint_as_float(v[it][1].z); f[7] = __uint_as_float(v[it][1].w); }
#pragma unroll
        for (int i = 0; i < E; ++i) amax = fmaxf(amax, fabsf(f[i]));
    }
    if (blockIdx.x == gridDim.x - 1) {  // fewer than E trailing elements
        size_t i = nchunks * E + threadIdx.x;
        if (i < n) amax = fmaxf(amax, fabsf(load_one<Tag>(x, i)));
    }
    __shared__ float red[4];
    __shared__ int last;
    amax = wave_max(amax);
    if ((threadIdx.x & 63) == 0) red[threadIdx.x >> 6] = amax;
    __syncthreads();
    if (threadIdx.x == 0) {
        const float m = fmaxf(fmaxf(red[0], red[1]), fmaxf(red[2], red[3]));
        __hip_atomic_store(&ws->partials[blockIdx.x], m, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
        asm volatile("s_waitcnt vmcnt(0)" ::: "memory");  // acknowledged at device scope before the ticket is drawn
        // two-level ticket (same-address atomics serialise): workgroups congruent modulo kTicketGroups share a counter,
        // the last of a group puts it back to zero and draws from the top counter
        const unsigned G = gridDim.x, grp = blockIdx.x % kTicketGroups;
        const unsigned in_group = (G - grp + kTicketGroups - 1) / kTicketGroups, ngroups = G < kTicketGroups ? G : kTicketGroups;
        int is_last = 0;
        if (__hip_atomic_fetch_add(&ws->group[grp].count, 1u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT) == in_group - 1) {
            __hip_atomic_store(&ws->group[grp].count, 0u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
            is_last = __hip_atomic_fetch_add(&ws->top.count, 1u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT) == ngroups - 1;
        }
        last = is_last;
    }
    __syncthreads();
    if (!last) return;
    float m = 0.0f;
    for (unsigned i = threadIdx.x; i < gridDim.x; i += 256)
        m = fmaxf(m, __hip_atomic_load(&ws->partials[i], __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT));
    m = wave_max(m);
    __syncthreads();
    if ((threadIdx.x & 63) == 0) red[threadIdx.x >> 6] = m;
    __syncthreads();
    if (threadIdx.x == 0) {
        scale_out[0] = fmaxf(fmaxf(red[0], red[1]), fmaxf(red[2], red[3])) / 448.0f;
        __hip_atomic_store(&ws->top.count, 0u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
    }
}

static unsigned stream_grid(size_t n, int elems_per_thread) {
    size_t blocks = (n / elems_per_thread + 255) / 256;
    const size_t cap = 256 * 8;  // 8 workgroups of 4 wavefronts per CU keep HBM busy
    if (blocks > cap) blocks = cap;
    if (blocks == 0) blocks = 1;
    return (unsigned)blocks;
}

template <typename Tag> static int launch_amax(float* scale, const void* x, size_t n, hipStream_t st) {
    if (reinterpret_cast<uintptr_t>(x) % 16 == 0) {
        // 512 workgroups at most: every workgroup ends with one same-address atomic, and those serialise
        unsigned grid = stream_grid(n, Chunk16<Tag>::elems);
        if (grid > 512) grid = 512;
        hipLaunchKernelGGL((fp8_amax_kernel<Tag>), dim3(grid), dim3(256), 0, st, scale, x, n);
    } else {
        hipLaunchKernelGGL((fp8_amax_scalar_kernel<Tag>), dim3(stream_grid(n, 4)), dim3(256), 0, st, scale, x, n);
    }
    return check_launch("fp8_amax");
}
template <typename Tag>
static int launch_cast(uint8_t* dst, const void* src, const float* scale, int invert, size_t n, hipStream_t st) {
    if (reinterpret_cast<uintptr_t>(src) % 16 == 0 && reinterpret_cast<uintptr_t>(dst) % 16 == 0) {
        if (n * Elem<Tag>::bytes >= kStreamBytes)
            hipLaunchKernelGGL((fp8_cast_kernel<Tag, true>), dim3(stream_grid(n, Chunk16<Tag>::elems)), dim3(256), 0, st, dst, src, scale, invert, n);
        else
            hipLaunchKernelGGL((fp8_cast_kernel<Tag, false>), dim3(stream_grid(n, Chunk16<Tag>::elems)), dim3(256), 0, st, dst, src, scale, invert, n);
    } else {
        hipLaunchKernelGGL((fp8_cast_scalar_kernel<Tag>), dim3(stream_grid(n, 4)), dim3(256), 0, st, dst, src, scale, invert, n);
    }
    return check_launch("fp8_cast");
}

// Partial-maximum pass of the two-launch quantiser on the scratch block `ws` (16-byte aligned x).
template <typename Tag>
static int launch_amax_ticket(TicketRegion* ws, float* scale_out, const void* x, size_t n, hipStream_t st) {
    size_t slabs = (n + kTicketSlab - 1) / kTicketSlab;
    if (slabs == 0) slabs = 1;
    hipLaunchKernelGGL((fp8_amax_ticket_kernel<Tag>), dim3((unsigned)slabs), dim3(256), 0, st, ws, scale_out, x, n);
    return check_launch("fp8_amax_ticket");
}

}  // namespace lq

using namespace lq;

extern "C" int lq_fp8_amax_scale(float* scale, const void* x, lq_dtype_t dtype, size_t n, lq_stream_t stream) {
    LQ_REQUIRE(scale && (x || n == 0), LQ_ERR_ARG, "lq_fp8_amax_scale: null pointer");
    if (n == 0) return LQ_OK;
    switch (dtype) {
        case LQ_F16: return launch_amax<F16Tag>(scale, x, n, as_stream(stream));
        case LQ_BF16: return launch_amax<BF16Tag>(scale, x, n, as_stream(stream));
        case LQ_F32: return launch_amax<F32Tag>(scale, x, n, as_stream(stream));
        default: set_error("lq_fp8_amax_scale: unsupported dtype %d", (int)dtype); return LQ_ERR_UNSUPPORTED;
    }
}

extern "C" int lq_fp8_scale_cast(uint8_t* dst, const void* src, lq_dtype_t dtype, const float* scale, int invert,
                                 size_t n, lq_stream_t stream) {
    LQ_REQUIRE(scale && ((dst && src) || n == 0), LQ_ERR_ARG, "lq_fp8_scale_cast: null pointer");
    if (n == 0) return LQ_OK;
    switch (dtype) {
        case LQ_F16: return launch_cast<F16Tag>(dst, src, scale, invert, n, as_stream(stream));
        case LQ_BF16: return launch_cast<BF16Tag>(dst, src, scale, invert, n, as_stream(stream));
        case LQ_F32: return launch_cast<F32Tag>(dst, src, scale, invert, n, as_stream(stream));
        default: set_error("lq_fp8_scale_cast: unsupported dtype %d", (int)dtype); return LQ_ERR_UNSUPPORTED;
    }
}

extern "C" int lq_fp8_scale_cast_2d(uint8_t* dst, size_t dst_ld, const void* src, size_t src_ld, lq_dtype_t dtype,
                                    const float* scale, int invert, size_t rows, size_t cols, lq_stream_t stream) {
    LQ_REQUIRE(scale && ((dst && src) || rows * cols == 0), LQ_ERR_ARG, "lq_fp8_scale_cast_2d: null pointer");
    LQ_REQUIRE(dtype == LQ_F16 || dtype == LQ_BF16 || dtype == LQ_F32, LQ_ERR_UNSUPPORTED, "lq_fp8_scale_cast_2d: unsupported dtype %d", (int)dtype);
    const size_t esz = dtype == LQ_F32 ? 4 : 2, e = dtype == LQ_F32 ? 8 : 16;
    LQ_REQUIRE(cols % 16 == 0 && dst_ld >= cols && src_ld >= cols && dst_ld % 16 == 0 && (src_ld * esz) % 16 == 0 &&
                   reinterpret_cast<uintptr_t>(dst) % 16 == 0 && reinterpret_cast<uintptr_t>(src) % 16 == 0,
               LQ_ERR_SHAPE, "lq_fp8_scale_cast_2d: cols and both row pitches must keep every row 16-byte aligned (cols=%zu dst_ld=%zu src_ld=%zu)",
               cols, dst_ld, src_ld);
    if (rows * cols == 0) return LQ_OK;
    const unsigned grid = stream_grid(rows * cols, (int)e);
    hipStream_t st = as_stream(stream);
    if (dtype == LQ_F16) hipLaunchKernelGGL((fp8_cast_2d_kernel<F16Tag>), dim3(grid), dim3(256), 0, st, dst, dst_ld, src, src_ld, scale, invert, rows, cols);
    else if (dtype == LQ_BF16) hipLaunchKernelGGL((fp8_cast_2d_kernel<BF16Tag>), dim3(grid), dim3(256), 0, st, dst, dst_ld, src, src_ld, scale, invert, rows, cols);
    else hipLaunchKernelGGL((fp8_cast_2d_kernel<F32Tag>), dim3(grid), dim3(256), 0, st, dst, dst_ld, src, src_ld, scale, invert, rows, cols);
    return check_launch("fp8_cast_2d");
}

extern "C" int lq_fp8_amax_cast(uint8_t* dst, float* scale_out, const void* src, lq_dtype_t dtype, size_t n,
                                lq_stream_t stream) {
    LQ_REQUIRE(scale_out && ((dst && src) || n == 0), LQ_ERR_ARG, "lq_fp8_amax_cast: null pointer");
    if (n >= 4096) {
        int rc = 1;
        switch (dtype) {
            case LQ_F16: rc = launch_amax_cast_coop<F16Tag>(dst, scale_out, src, n, as_stream(stream)); break;
            case LQ_BF16: rc = launch_amax_cast_coop<BF16Tag>(dst, scale_out, src, n, as_stream(stream)); break;
            case LQ_F32: rc = launch_amax_cast_coop<F32Tag>(dst, scale_out, src, n, as_stream(stream)); break;
            default: set_error("lq_fp8_amax_cast: unsupported dtype %d", (int)dtype); return LQ_ERR_UNSUPPORTED;
        }
        if (rc <= 0) return rc;
    }
    // scratch-free sequence: safe under stream capture and for any number of concurrent streams
    hipLaunchKernelGGL(fill_f32_kernel, dim3(1), dim3(1), 0, as_stream(stream), scale_out, 0.0f);
    int rc = check_launch("fp8_amax_cast(fill)");
    if (rc != LQ_OK || n == 0) return rc;
    rc = lq_fp8_amax_scale(scale_out, src, dtype, n, stream);
    if (rc != LQ_OK) return rc;
    return lq_fp8_scale_cast(dst, src, dtype, scale_out, 1, n, stream);
}

extern "C" int lq_fp8_amax_cast_static(uint8_t* dst, float* scale_out, const void* src, lq_dtype_t dtype, size_t n,
                                       lq_stream_t stream) {
    LQ_REQUIRE(dst && scale_out && src, LQ_ERR_ARG, "lq_fp8_amax_cast_static: null pointer");
    LQ_REQUIRE(dtype == LQ_F16 || dtype == LQ_BF16 || dtype == LQ_F32, LQ_ERR_UNSUPPORTED,
               "lq_fp8_amax_cast_static: unsupported dtype %d", (int)dtype);
    LQ_REQUIRE(n >= 1 && n <= lq_fp8_amax_cast_static_max_elems(), LQ_ERR_SHAPE,
               "lq_fp8_amax_cast_static: n=%zu outside 1..%zu (the static scratch holds %zu partial maxima of %zu elements)",
               n, lq_fp8_amax_cast_static_max_elems(), kTicketMaxSlabs, kTicketSlab);
    LQ_REQUIRE(reinterpret_cast<uintptr_t>(src) % 16 == 0 && reinterpret_cast<uintptr_t>(dst) % 16 == 0, LQ_ERR_ARG,
               "lq_fp8_amax_cast_static: src and dst must be 16-byte aligned");
    FusedScratch* ws = device_scratch();
    if (ws == nullptr) return LQ_ERR_HIP;
    hipStream_t st = as_stream(stream);
    int rc;
    switch (dtype) {
        case LQ_F16: rc = launch_amax_ticket<F16Tag>(&ws->ticket, scale_out, src, n, st); break;
        case LQ_BF16: rc = launch_amax_ticket<BF16Tag>(&ws->ticket, scale_out, src, n, st); break;
        default: rc = launch_amax_ticket<F32Tag>(&ws->ticket, scale_out, src, n, st); break;
    }
    if (rc != LQ_OK) return rc;
    return lq_fp8_scale_cast(dst, src, dtype, scale_out, 1, n, stream);
}

extern "C" int lq_fp8_amax_cast_slot(lq_stream_t stream) {
    int dev = 0;
    if (device_scratch(&dev) == nullptr) return LQ_ERR_HIP;
    return slot_for_stream(dev, as_stream(stream));
}

extern "C" size_t lq_fp8_amax_cast_static_max_elems(void) { return kTicketSlab * kTicketMaxSlabs; }

extern "C" int lq_fp8_amax_cast_status(void) {
    FusedScratch* ws = device_scratch();
    if (ws == nullptr) return LQ_ERR_HIP;
    unsigned flag = 0;
    hipError_t e = hipMemcpy(&flag, &ws->timeout, sizeof(flag), hipMemcpyDeviceToHost);
    if (e == hipSuccess && flag != 0) {
        const unsigned zero = 0;
        e = hipMemcpy(&ws->timeout, &zero, sizeof(zero), hipMemcpyHostToDevice);
    }
    if (e != hipSuccess) {
        (void)hipGetLastError();
        set_error("lq_fp8_amax_cast_status: %s", hipGetErrorString(e));
        return LQ_ERR_HIP;
    }
    if (flag != 0) {
        set_error("lq_fp8_amax_cast: a one-launch quantisation timed out at its grid barrier since the last status call "
                  "(its scale is NaN); another stream's kernels held the device -- serialise the streams or quantise with "
                  "lq_fp8_amax_scale + lq_fp8_scale_cast");
        return 1;
    }
    return 0;
}
