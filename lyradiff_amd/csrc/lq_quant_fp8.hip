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

// Codes written as k-panels [k / 64][rows][64] instead of row-major [rows][k]: the layout in which the 64 bytes a GEMM
// k-tile takes from each activation row are contiguous over the rows (lq_gemm_fp8_panels).  PanelMap{k = 0} is row-major.
// A kernel that writes panels walks the tensor in blocks of RB rows x KC 64-element chunks, one block per wavefront and
// step, every lane taking E consecutive elements of one row (E = 8 or 16: a 16- or 32-byte read, an 8- or 16-byte
// write): (64 / E) * KC lanes share a row and RB = E / KC rows make a block, so a wavefront reads KC * 64 * sizeof(T)
// contiguous bytes of each of its rows (whole 128-byte lines) and writes RB x 64 contiguous bytes into each of KC panels.
// Blocks are numbered along k first; a wavefront's next block is a fixed number of blocks on (quotient and remainder by
// the blocks per row block come from the host), so the walk costs one 32-bit division per thread.
struct PanelMap {
    unsigned k, rows;
};
struct PanelStep {  // a fixed advance in blocks, as whole row blocks + remainder along k
    unsigned dq, dr;
};
static PanelStep panel_step(size_t blocks, unsigned kcs) { return PanelStep{(unsigned)(blocks / kcs), (unsigned)(blocks % kcs)}; }
template <int E, int KC = 1> struct PanelWalk {  // blocks of RB rows x KC 64-element chunks
    static constexpr int LPR = (64 / E) * KC;  // lanes per row of a block
    static constexpr int RB = 64 / LPR;        // rows per block
    unsigned rb, kc;                           // row block and first 64-element chunk of the wavefront's current block
    unsigned lr, sub, part;                    // this lane's row inside the block, its chunk inside the block's KC, its piece of that chunk
    __device__ __forceinline__ PanelWalk(unsigned wave, unsigned lane, unsigned kcs)
        : rb(wave / (kcs / KC)), kc((wave % (kcs / KC)) * KC), lr(lane / LPR), sub((lane % LPR) / (64 / E)), part(lane % (64 / E)) {}
    __device__ __forceinline__ void step(const PanelStep& d, unsigned kcs) {  // d counts blocks: d.dr blocks along k = d.dr * KC chunks
        kc += d.dr * KC;
        rb += d.dq;
        if (kc >= kcs) { kc -= kcs; ++rb; }
    }
    __device__ __forceinline__ unsigned row() const { return rb * RB + lr; }
    __device__ __forceinline__ size_t src_elem(const PanelMap& pm) const { return (size_t)row() * pm.k + (kc + sub) * 64 + part * E; }
    __device__ __forceinline__ size_t dst_byte(const PanelMap& pm) const { return ((size_t)(kc + sub) * pm.rows + row()) * 64 + part * E; }
};

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

// PANEL: 0 = row-major codes; 1 or 4 = k-panels, walked in blocks of PANEL 64-element chunks per row (PanelWalk)
template <typename Tag, bool NT, int PANEL = 0>
__global__ __launch_bounds__(256) void fp8_cast_kernel(uint8_t* __restrict__ dst, const void* __restrict__ src,
                                                       const float* __restrict__ scale, int invert, size_t n, PanelMap pm = PanelMap{0, 0},
                                                       PanelStep stride = PanelStep{0, 0}) {
    constexpr int E = Chunk16<Tag>::elems;
    const float s = scale[0];
    const float r = invert ? 1.0f / s : s;
    auto chunk = [&](size_t e, uint8_t* o) {  // E elements from element e on -> E codes at o
        float v[16];
        load_elems<Tag, NT>(src, e, v);
        u32 w[4];
#pragma unroll
        for (int i = 0; i < E / 4; ++i)
            w[i] = cvt4_e4m3(v[4 * i] * r, v[4 * i + 1] * r, v[4 * i + 2] * r, v[4 * i + 3] * r);
        if constexpr (E == 16) *reinterpret_cast<uint4*>(o) = make_uint4(w[0], w[1], w[2], w[3]);
        else *reinterpret_cast<uint2*>(o) = make_uint2(w[0], w[1]);
    };
    if constexpr (PANEL != 0) {
        using Walk = PanelWalk<E, PANEL>;
        const unsigned kcs = pm.k / 64, nrb = (pm.rows + Walk::RB - 1) / Walk::RB;
        for (Walk pw((blockIdx.x * blockDim.x + threadIdx.x) >> 6, threadIdx.x & 63, kcs); pw.rb < nrb; pw.step(stride, kcs))
            if (pw.row() < pm.rows) chunk(pw.src_elem(pm), dst + pw.dst_byte(pm));
        return;
    }
    const size_t nchunks = n / E;
    for (size_t c = (size_t)blockIdx.x * blockDim.x + threadIdx.x; c < nchunks; c += (size_t)gridDim.x * blockDim.x) chunk(c * E, dst + c * E);
    if (blockIdx.x == 0) {
        size_t i = nchunks * E + threadIdx.x;
        if (i < n) dst[i] = (uint8_t)cvt1_e4m3(load_one<Tag>(src, i) * r);
    }
}

// Activation and dynamic quantisation of a stored GEMM output in one pass: h = T(gelu(y)) (the tanh-GELU that the reference
// applies to a stored T tensor, invokeFusedBiasAndGelu, kernels/flux_single_transformer_block/flux_single_transformer_kernels.cu:
// 122-141), codes = e4m3(h / scale), scale = max|h| / 448.  The maximum needs no pass over the tensor: the GEMM that wrote y
// also left ymax = max(y, 0) (lq_gemm_fp8_max), T(gelu(.)) is non-decreasing on the values of T from 0 up (checked value by
// value in the tests), so max|h| = h(ymax) as soon as that beats the largest |h| any negative y can give (0.17 at y = -0.75);
// the kernel takes that route from ymax >= 0.5 (h = 0.345).  Below that -- a tensor without a single output of 0.5 or more --
// the scale comes from the bound max(h(ymax), kGeluNegBound) instead of the exact maximum.
constexpr float kGeluNegBound = 0.171875f;  // >= |gelu(y)| for every y < 0; a value of fp16 and bf16
// PANEL: 0 = row-major codes; 1 or 4 = k-panels, walked in blocks of PANEL 64-element chunks per row (PanelWalk)
template <typename Tag, bool NT, bool WANT_H, int PANEL = 0>
__global__ __launch_bounds__(256) void fp8_gelu_cast_kernel(uint8_t* __restrict__ dst, float* __restrict__ scale_out,
                                                            void* __restrict__ h_out, const void* __restrict__ src,
                                                            const float* __restrict__ src_max, float* __restrict__ clear, size_t n,
                                                            PanelMap pm = PanelMap{0, 0}, PanelStep stride = PanelStep{0, 0}) {
    constexpr int E = Chunk16<Tag>::elems;
    if (clear != nullptr && blockIdx.x == 0 && threadIdx.x == 0) clear[0] = 0.0f;  // the next call's slot for a running maximum
    const float ym = round_through<Tag>(fmaxf(src_max[0], 0.0f));
    float amax = round_through<Tag>(gelu_fast(ym));
    if (!(ym >= 0.5f)) amax = fmaxf(amax, kGeluNegBound);
    const float s = amax / 448.0f;
    const float r = 1.0f / s;
    if (blockIdx.x == 0 && threadIdx.x == 0) scale_out[0] = s;
    auto chunk = [&](size_t e, uint8_t* o) {  // E elements from element e on -> h (row-major, optional) and E codes at o
        float v[16];
        load_elems<Tag, NT>(src, e, v);
#pragma unroll
        for (int i = 0; i < E; i += 2) {
            v[i] = gelu_fast(v[i]);
            v[i + 1] = gelu_fast(v[i + 1]);
            round_through2<Tag>(v[i], v[i + 1]);
        }
        if constexpr (WANT_H) {
            char* ho = static_cast<char*>(h_out) + (e / E) * 32;
            if constexpr (Elem<Tag>::bytes == 2) {
                u32 hw[E / 2];
#pragma unroll
                for (int i = 0; i < E / 2; ++i) hw[i] = Elem<Tag>::store(v[2 * i]) | (Elem<Tag>::store(v[2 * i + 1]) << 16);
                *reinterpret_cast<uint4*>(ho) = make_uint4(hw[0], hw[1], hw[2], hw[3]);
                *reinterpret_cast<uint4*>(ho + 16) = make_uint4(hw[4], hw[5], hw[6], hw[7]);
            } else {
                *reinterpret_cast<float4*>(ho) = make_float4(v[0], v[1], v[2], v[3]);
                *reinterpret_cast<float4*>(ho + 16) = make_float4(v[4], v[5], v[6], v[7]);
            }
        }
        u32 w[4];
#pragma unroll
        for (int i = 0; i < E / 4; ++i)
            w[i] = cvt4_e4m3(v[4 * i] * r, v[4 * i + 1] * r, v[4 * i + 2] * r, v[4 * i + 3] * r);
        if constexpr (E == 16) *reinterpret_cast<uint4*>(o) = make_uint4(w[0], w[1], w[2], w[3]);
        else *reinterpret_cast<uint2*>(o) = make_uint2(w[0], w[1]);
    };
    if constexpr (PANEL != 0) {
        using Walk = PanelWalk<E, PANEL>;
        const unsigned kcs = pm.k / 64, nrb = (pm.rows + Walk::RB - 1) / Walk::RB;
        for (Walk pw((blockIdx.x * blockDim.x + threadIdx.x) >> 6, threadIdx.x & 63, kcs); pw.rb < nrb; pw.step(stride, kcs))
            if (pw.row() < pm.rows) chunk(pw.src_elem(pm), dst + pw.dst_byte(pm));
        return;
    }
    const size_t nchunks = n / E;
    for (size_t c = (size_t)blockIdx.x * blockDim.x + threadIdx.x; c < nchunks; c += (size_t)gridDim.x * blockDim.x) chunk(c * E, dst + c * E);
    if (blockIdx.x == 0) {
        size_t i = nchunks * E + threadIdx.x;
        if (i < n) {
            const float h = round_through<Tag>(gelu_fast(load_one<Tag>(src, i)));
            if constexpr (WANT_H) {
                if constexpr (Elem<Tag>::bytes == 2) static_cast<unsigned short*>(h_out)[i] = (unsigned short)Elem<Tag>::store(h);
                else static_cast<float*>(h_out)[i] = h;
            }
            dst[i] = (uint8_t)cvt1_e4m3(h * r);
        }
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
constexpr int kCoopThreads = 1024;
constexpr int kCoopMaxBlocks = 512;
constexpr int kCoopSlots = 16;
constexpr size_t kTicketSlab = 32768;     // elements per workgroup of the partial-maximum pass
constexpr size_t kTicketMaxSlabs = 8192;  // partial maxima the scratch holds => at most 2^28 elements per call
constexpr int kTicketGroups = 16;         // first-level ticket counters, one 128-byte line each
struct CounterLine {  // one counter per 128-byte line: polls of one word must not queue behind atomics on another
    unsigned count;
    unsigned pad[31];
};
struct TaggedLine {  // one {launch number, float bits} word per 128-byte line
    unsigned long long word;
    unsigned long long pad[15];
};
// Barrier state of the one-launch quantiser.  Nothing in it is a counter: every word is {launch number << 32 | float bits},
// written whole by one 8-byte store, so a launch that gives up leaves nothing behind that a later launch could trip over.
struct CoopSlot {
    unsigned long long partial[kCoopMaxBlocks];  // workgroup maxima of the launch named in the upper half
    TaggedLine result[8];                         // the tensor maximum, one copy per group of pollers (workgroup id mod 8)
};
struct TicketRegion {
    CounterLine group[kTicketGroups];
    CounterLine top;
    float partials[kTicketMaxSlabs];
};
struct FusedScratch {
    unsigned timeout;         // a one-launch quantisation gave up at its exchange
    unsigned ticket_overlap;  // the two-launch quantiser drew a ticket that only overlapping calls can produce
    unsigned pad[62];
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

// A stream owns one barrier slot from its first call until lq_fp8_amax_cast_release_slot (work of one stream runs in
// order, so its launches never overlap); streams beyond kCoopSlots get none and use the scratch-free kernel sequence.
// Every launch on a slot carries the slot's next launch number (never 0, the value of untouched memory).
struct StreamSlots {
    hipStream_t stream[kCoopSlots];
    bool taken[kCoopSlots];
    unsigned launches[kCoopSlots];
};
static StreamSlots g_stream_slots[kMaxDevices];
static std::mutex g_slot_mutex;
static int slot_for_stream(int dev, hipStream_t st, unsigned* launch_number = nullptr) {
    std::lock_guard<std::mutex> lock(g_slot_mutex);
    StreamSlots& t = g_stream_slots[dev];
    int slot = -1;
    for (int i = 0; i < kCoopSlots && slot < 0; ++i)
        if (t.taken[i] && t.stream[i] == st) slot = i;
    for (int i = 0; i < kCoopSlots && slot < 0; ++i)
        if (!t.taken[i]) {
            t.taken[i] = true;
            t.stream[i] = st;
            slot = i;
        }
    if (slot >= 0 && launch_number) {
        if (++t.launches[slot] == 0) ++t.launches[slot];
        *launch_number = t.launches[slot];
    }
    return slot;
}
static int release_slot(int dev, hipStream_t st) {
    std::lock_guard<std::mutex> lock(g_slot_mutex);
    StreamSlots& t = g_stream_slots[dev];
    for (int i = 0; i < kCoopSlots; ++i)
        if (t.taken[i] && t.stream[i] == st) {
            t.taken[i] = false;  // the launch counter stays: a later owner continues the numbering
            return i;
        }
    return -1;
}

// Fused dynamic per-tensor quantisation in ONE launch: every thread keeps up to KEEP 32-byte chunks of the tensor in
// registers while the tensor-wide absmax is formed (workgroup maxima -> grid-wide exchange), then casts from
// registers, so the source is read from HBM once (3 bytes moved per element: the algorithmic minimum).  Chunks beyond
// KEEP are re-read in the second phase (from L2 / Infinity Cache when they fit).
//
// Layout: a wavefront owns 2 KiB blocks of the source; lane l holds the 16-byte pieces at l*16 and 1024 + l*16 of a
// block (fully coalesced 1 KiB requests) and writes their codes at the matching output offsets.  Which element a lane
// holds is free: the maximum is a reduction and the cast elementwise.  Kept pieces are fetched with nontemporal loads and
// the codes leave with nontemporal stores: measured at 4608x3072 bf16 from HBM, in-kernel time stamps, one 1024-thread
// workgroup per CU: load phase 7.5 -> 6.3 us with the loads marked, and 12.8 -> 11.1 us from launch to launch with the
// stores marked as well (the 14 MB of codes no longer sit dirty in the L2s for the end-of-kernel write-back).
//
// Exchange: thread 0 of every workgroup stores {launch number, workgroup maximum} as one 8-byte word; workgroup 0
// gathers the words of this launch (one per thread), reduces them and publishes {launch number, tensor maximum} in
// eight copies; the other workgroups poll the copy of their group (workgroup id mod 8) -- 32 pollers per word.  No
// read-modify-write, no counter to re-arm, two stores and two polls on the critical path (1.5 us against 2.2 us for a
// two-level arrival counter with a flag), and every workgroup receives the maximum itself instead of re-reading all
// partial maxima.  Only relaxed device-scope accesses are used -- no release/acquire fences, which on this multi-die part
// would write back / invalidate whole L2s; a word is complete by construction.
//
// The grid never exceeds what the device holds at once (one workgroup per CU), so every workgroup is running when the
// exchange starts -- provided nothing else occupies the device; when another stream's kernels hold CUs the late
// workgroups start once those retire, and every wait is bounded so that even a starved grid terminates: a workgroup that
// gives up raises the time-out flag (lq_fp8_amax_cast_status reports it), casts with a NaN scale and writes NaN to
// scale_out, which poisons the output visibly instead of hanging the device.  Launches that may overlap in time use
// different slots: a slot belongs to one stream, and the path is not taken under stream capture (a captured launch
// could later replay on any stream) nor for the per-thread default stream (one handle, many streams).
__device__ __forceinline__ unsigned long long poll_tagged(const unsigned long long* word, unsigned launch, bool* ok) {
    unsigned long long v = 0;
    int spin = 0;
    for (; spin < (1 << 18); ++spin) {
        v = __hip_atomic_load(word, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
        if ((unsigned)(v >> 32) == launch) break;
        __builtin_amdgcn_s_sleep(1);
    }
    *ok = spin < (1 << 18);
    return v;
}

template <typename Tag, int KEEP, bool PANEL = false>
__global__ __launch_bounds__(kCoopThreads) void fp8_amax_cast_coop_kernel(uint8_t* __restrict__ dst, float* __restrict__ scale_out,
                                                                          const void* __restrict__ src, size_t n, CoopSlot* slot,
                                                                          unsigned launch, unsigned* timeout,
                                                                          unsigned long long* __restrict__ stamps,
                                                                          PanelMap pm = PanelMap{0, 0}, PanelStep round_step = PanelStep{0, 0}) {
    // stamps (NULL in every product launch): four readings of the constant 100 MHz clock per workgroup -- started, partial
    // maximum formed (its loads are back), released from the exchange, stores acknowledged (lq_fp8_amax_cast_timeline)
    if (stamps != nullptr && threadIdx.x == 0) stamps[blockIdx.x * 4] = wall_clock64();
    constexpr int E2 = Elem<Tag>::bytes == 2 ? 8 : 4;  // elements per 16-byte piece
    constexpr int BLK = 128 * E2;                      // elements per 2 KiB block
    typedef unsigned int u32x4_t __attribute__((ext_vector_type(4)));
    typedef unsigned int u32x2_t __attribute__((ext_vector_type(2)));
    const size_t nblocks = n / BLK;
    const int lane = threadIdx.x & 63;
    const size_t wave = ((size_t)blockIdx.x * kCoopThreads + threadIdx.x) >> 6;
    const size_t nwaves = (size_t)gridDim.x * (kCoopThreads / 64);
    const char* in = static_cast<const char*>(src) + lane * 16;
    uint8_t* out = dst + lane * E2;
    // Where this lane's 16-byte piece number j of the wavefront comes from and where its codes go.  Row-major: pieces 2i and
    // 2i + 1 are pieces `lane` and `lane + 64` of the wavefront's block i (2 KiB of consecutive elements; blocks wave,
    // wave + nwaves, ...).  k-panels: piece j lies in the wavefront's j-th block of E2 rows x 64 elements (PanelWalk: 64 / E2
    // lanes share a row, so one load instruction reads whole 128-byte lines and one store writes E2 x 64 contiguous bytes).
    struct Place {
        const char* p;
        uint8_t* o;
        bool ok;
    };
    const unsigned kcs = PANEL ? pm.k / 64 : 1, nrb = PANEL ? (pm.rows + E2 - 1) / E2 : 0;
    PanelWalk<E2> pw((unsigned)wave, (unsigned)lane, kcs);
    auto rewind = [&]() { pw = PanelWalk<E2>((unsigned)wave, (unsigned)lane, kcs); };
    auto place = [&](size_t j) -> Place {  // k-panels: of the walk's current block, which the caller steps once per piece
        if constexpr (PANEL) {
            return Place{static_cast<const char*>(src) + pw.src_elem(pm) * Elem<Tag>::bytes, dst + pw.dst_byte(pm),
                         pw.rb < nrb && pw.row() < pm.rows};
        } else {
            const size_t b = wave + (j >> 1) * nwaves;
            return Place{in + b * 2048 + (j & 1) * 1024, out + b * BLK + (j & 1) * (64 * E2), b < nblocks};
        }
    };
    auto more = [&](size_t j) -> bool {  // pieces left for this wavefront
        if constexpr (PANEL) return pw.rb < nrb;
        else return wave + (j >> 1) * nwaves < nblocks;
    };
    uint4 keep[KEEP][2];
    float amax = 0.0f;
    auto piece_amax = [&](const uint4& v) {
        float f[8];
        if constexpr (E2 == 8) unpack8<Tag>(v, f);
        else { f[0] = __uint_as_float(v.x); f[1] = __uint_as_float(v.y); f[2] = __uint_as_float(v.z); f[3] = __uint_as_float(v.w); }
#pragma unroll
        for (int i = 0; i < E2; ++i) amax = fmaxf(amax, fabsf(f[i]));
    };
#pragma unroll
    for (int j = 0; j < 2 * KEEP; ++j) {
        const Place pl = place(j);
        keep[j >> 1][j & 1] = make_uint4(0, 0, 0, 0);
        if (pl.ok) {
            const u32x4_t a = __builtin_nontemporal_load(reinterpret_cast<const u32x4_t*>(pl.p));
            keep[j >> 1][j & 1] = make_uint4(a.x, a.y, a.z, a.w);
        }
        if constexpr (PANEL) pw.step(round_step, kcs);
    }
#pragma unroll
    for (int it = 0; it < KEEP; ++it) {
        piece_amax(keep[it][0]);
        piece_amax(keep[it][1]);
    }
    for (size_t j = 2 * KEEP; more(j); ++j) {  // what the registers cannot hold is read twice
        const Place pl = place(j);
        if (pl.ok) piece_amax(*reinterpret_cast<const uint4*>(pl.p));
        if constexpr (PANEL) pw.step(round_step, kcs);
    }
    if (!PANEL && blockIdx.x == 0)  // fewer than BLK trailing elements (the blocks of the k-panel walk cover every element)
        for (size_t i = nblocks * BLK + threadIdx.x; i < n; i += kCoopThreads) amax = fmaxf(amax, fabsf(load_one<Tag>(src, i)));
    __shared__ float red[kCoopThreads / 64];
    __shared__ float tensor_max;
    amax = wave_max(amax);
    if (lane == 0) red[threadIdx.x >> 6] = amax;
    __syncthreads();
    if (stamps != nullptr && threadIdx.x == 0) stamps[blockIdx.x * 4 + 1] = wall_clock64();
    if (threadIdx.x == 0) {
        float wg_max = 0.0f;
#pragma unroll
        for (int i = 0; i < kCoopThreads / 64; ++i) wg_max = fmaxf(wg_max, red[i]);
        __hip_atomic_store(&slot->partial[blockIdx.x], ((unsigned long long)launch << 32) | __float_as_uint(wg_max), __ATOMIC_RELAXED,
                           __HIP_MEMORY_SCOPE_AGENT);
    }
    bool ok = true;
    if (blockIdx.x == 0) {
        float m = 0.0f;
        for (unsigned i = threadIdx.x; i < gridDim.x; i += kCoopThreads) {
            bool got;
            m = fmaxf(m, __uint_as_float((unsigned)poll_tagged(&slot->partial[i], launch, &got)));
            ok = ok && got;
        }
        m = wave_max(__syncthreads_and(ok) ? m : __builtin_nanf(""));  // a missing partial maximum makes the result NaN for everybody
        __syncthreads();
        if (lane == 0) red[threadIdx.x >> 6] = m;
        __syncthreads();
        m = red[0];
#pragma unroll
        for (int i = 1; i < kCoopThreads / 64; ++i) m = (m != m || red[i] != red[i]) ? __builtin_nanf("") : fmaxf(m, red[i]);
        if (threadIdx.x < 8)
            __hip_atomic_store(&slot->result[threadIdx.x].word, ((unsigned long long)launch << 32) | __float_as_uint(m), __ATOMIC_RELAXED,
                               __HIP_MEMORY_SCOPE_AGENT);
        if (threadIdx.x == 0) tensor_max = m;
    } else if (threadIdx.x == 0) {
        const unsigned long long v = poll_tagged(&slot->result[blockIdx.x & 7].word, launch, &ok);
        tensor_max = ok ? __uint_as_float((unsigned)v) : __builtin_nanf("");
    }
    __syncthreads();
    if (stamps != nullptr && threadIdx.x == 0) stamps[blockIdx.x * 4 + 2] = wall_clock64();
    const float s = tensor_max / 448.0f;  // NaN after a time-out
    if (threadIdx.x == 0 && s != s) {
        __hip_atomic_store(timeout, 1u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
        scale_out[0] = s;  // long after workgroup 0 wrote its value, if it had one
    }
    if (blockIdx.x == 0 && threadIdx.x == 0) scale_out[0] = s;
    // Only the raw 16-byte vectors live across the exchange: the empty asm makes them new values to the compiler, which
    // would otherwise keep the unpacked fp32 copies of the first phase as well (twice the registers, half the occupancy).
#pragma unroll
    for (int it = 0; it < KEEP; ++it)
#pragma unroll
        for (int u = 0; u < 2; ++u)
            asm volatile("" : "+v"(keep[it][u].x), "+v"(keep[it][u].y), "+v"(keep[it][u].z), "+v"(keep[it][u].w));
    const float r = 1.0f / s;
    auto piece_cast = [&](const uint4& v, uint8_t* o, bool stream_out) {
        float f[8];
        if constexpr (E2 == 8) unpack8<Tag>(v, f);
        else { f[0] = __uint_as_float(v.x); f[1] = __uint_as_float(v.y); f[2] = __uint_as_float(v.z); f[3] = __uint_as_float(v.w); }
        const u32 w0 = cvt4_e4m3(f[0] * r, f[1] * r, f[2] * r, f[3] * r);
        if constexpr (E2 == 8) {
            const u32x2_t w = {w0, cvt4_e4m3(f[4] * r, f[5] * r, f[6] * r, f[7] * r)};
            if (stream_out) __builtin_nontemporal_store(w, reinterpret_cast<u32x2_t*>(o));
            else *reinterpret_cast<u32x2_t*>(o) = w;
        } else {
            if (stream_out) __builtin_nontemporal_store(w0, reinterpret_cast<u32*>(o));
            else *reinterpret_cast<u32*>(o) = w0;
        }
    };
    rewind();
#pragma unroll
    for (int j = 0; j < 2 * KEEP; ++j) {
        const Place pl = place(j);
        if (pl.ok) piece_cast(keep[j >> 1][j & 1], pl.o, true);
        if constexpr (PANEL) pw.step(round_step, kcs);
    }
    for (size_t j = 2 * KEEP; more(j); ++j) {
        const Place pl = place(j);
        if (pl.ok) piece_cast(*reinterpret_cast<const uint4*>(pl.p), pl.o, true);
        if constexpr (PANEL) pw.step(round_step, kcs);
    }
    if (!PANEL && blockIdx.x == 0)
        for (size_t i = nblocks * BLK + threadIdx.x; i < n; i += kCoopThreads) dst[i] = (uint8_t)cvt1_e4m3(load_one<Tag>(src, i) * r);
    if (stamps != nullptr) {
        asm volatile("s_waitcnt vmcnt(0)" ::: "memory");  // this wavefront's stores are acknowledged
        __syncthreads();
        if (threadIdx.x == 0) stamps[blockIdx.x * 4 + 3] = wall_clock64();
    }
}

// Returns LQ_OK when the fused launch was issued, 1 when the caller should fall back to the scratch-free
// kernel sequence (unaligned buffers, stream capture, per-thread default stream, no barrier slot left for this stream,
// occupancy query failed), a negative status on an error.
// One 1024-thread workgroup per CU keeps KEEP = 4, 8 or 10 chunks of 32 bytes per thread across the exchange: 16.7, 33.5 or
// 41.9 M sixteen-bit elements on 256 CUs; the rest of a larger tensor is read twice (10 chunks are 80 of the 128 registers a
// lane has at this occupancy, 6-8 more spill; 12 chunks spilled 60).
template <typename Tag, int KEEP> struct CoopCapacity {
    int num_cu = 0;
    static const CoopCapacity& get(int dev) {  // queried once (thread-safe initialisation of a function-local static)
        static const CoopCapacity cap = [dev] {
            CoopCapacity c;
            int occ = 0;
            hipDeviceProp_t prop;
            if (hipGetDeviceProperties(&prop, dev) == hipSuccess &&
                hipOccupancyMaxActiveBlocksPerMultiprocessor(&occ, fp8_amax_cast_coop_kernel<Tag, KEEP>, kCoopThreads, 0) == hipSuccess &&
                occ >= 1)
                c.num_cu = prop.multiProcessorCount;
            (void)hipGetLastError();
            return c;
        }();
        return cap;
    }
};

template <typename Tag, int KEEP>
static int launch_coop_keep(uint8_t* dst, float* scale_out, const void* src, size_t n, hipStream_t st, int dev, FusedScratch* ws,
                            size_t waves_needed, unsigned long long* stamps, PanelMap pm) {
    const int num_cu = CoopCapacity<Tag, KEEP>::get(dev).num_cu;
    if (num_cu == 0) return 1;
    unsigned launch = 0;
    const int slot = slot_for_stream(dev, st, &launch);
    if (slot < 0) return 1;
    size_t grid = (waves_needed + kCoopThreads / 64 - 1) / (kCoopThreads / 64);
    if (grid > (size_t)num_cu) grid = num_cu;
    if (grid > kCoopMaxBlocks) grid = kCoopMaxBlocks;
    if (grid == 0) grid = 1;
    if (pm.k != 0) {
        if constexpr (KEEP > 8) {  // the k-panel walk's addresses do not fit beside ten kept chunks (53 registers spilled):
            return 1;              // the caller keeps eight and reads the rest twice
        } else {
            const size_t nwaves = grid * (kCoopThreads / 64);
            hipLaunchKernelGGL((fp8_amax_cast_coop_kernel<Tag, KEEP, true>), dim3((unsigned)grid), dim3(kCoopThreads), 0, st, dst,
                               scale_out, src, n, &ws->coop[slot], launch, &ws->timeout, stamps, pm, panel_step(nwaves, pm.k / 64));
        }
    } else {
        hipLaunchKernelGGL((fp8_amax_cast_coop_kernel<Tag, KEEP>), dim3((unsigned)grid), dim3(kCoopThreads), 0, st, dst, scale_out, src,
                           n, &ws->coop[slot], launch, &ws->timeout, stamps);
    }
    return check_launch("fp8_amax_cast_fused");
}

template <typename Tag>
static int launch_amax_cast_coop(uint8_t* dst, float* scale_out, const void* src, size_t n, hipStream_t st,
                                 unsigned long long* stamps = nullptr, PanelMap pm = PanelMap{0, 0}) {
    if (reinterpret_cast<uintptr_t>(src) % 16 != 0 || reinterpret_cast<uintptr_t>(dst) % 16 != 0) return 1;
    if (st == hipStreamPerThread) return 1;  // one handle for every thread's own stream: its launches can overlap
    hipStreamCaptureStatus cs = hipStreamCaptureStatusNone;
    if (hipStreamIsCapturing(st, &cs) != hipSuccess || cs != hipStreamCaptureStatusNone) {
        (void)hipGetLastError();
        return 1;
    }
    int dev = 0;
    FusedScratch* ws = device_scratch(&dev);
    if (ws == nullptr) return LQ_ERR_HIP;
    size_t blocks = n / (Elem<Tag>::bytes == 2 ? 1024 : 512);  // 2 KiB blocks, one per wavefront and kept chunk
    if (pm.k != 0) {  // k-panels: two blocks of 8 (4 for fp32) rows x 64 elements per kept chunk, the last row block may be partial
        const size_t rb = Elem<Tag>::bytes == 2 ? 8 : 4;
        blocks = (((pm.rows + rb - 1) / rb) * (pm.k / 64) + 1) / 2;
    }
    const int num_cu = CoopCapacity<Tag, 4>::get(dev).num_cu;
    if (num_cu == 0) return 1;
    const size_t waves = (size_t)num_cu * (kCoopThreads / 64);
    const size_t per_wave = (blocks + waves - 1) / waves;
    if (per_wave <= 4) return launch_coop_keep<Tag, 4>(dst, scale_out, src, n, st, dev, ws, blocks, stamps, pm);
    if (per_wave <= 8 || pm.k != 0) return launch_coop_keep<Tag, 8>(dst, scale_out, src, n, st, dev, ws, blocks, stamps, pm);
    return launch_coop_keep<Tag, 10>(dst, scale_out, src, n, st, dev, ws, blocks, stamps, pm);
}

// ---- two launches, no barrier: partial maxima + ticket, then the cast ------------------------------------------------
// Workgroup b reduces elements [b * kTicketSlab, (b+1) * kTicketSlab) to one partial maximum in the scratch block and
// takes a ticket; the workgroup that draws the last ticket reduces all partials, writes scale_out[0] = max / 448 and
// puts the ticket counters back to zero.  Nobody waits for anybody, so the kernel is safe under any scheduling, under
// stream capture and in graph replays; the cast kernel that follows re-reads the source (from the Infinity Cache when
// it fits).  All calls on one device share the one scratch block: calls that overlap in time race.
template <typename Tag>
__global__ __launch_bounds__(256) void fp8_amax_ticket_kernel(TicketRegion* __restrict__ ws, float* __restrict__ scale_out,
                                                              const void* __restrict__ x, size_t n, unsigned* __restrict__ overlap) {
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
        const unsigned drawn = __hip_atomic_fetch_add(&ws->group[grp].count, 1u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
        if (drawn == in_group - 1) {
            __hip_atomic_store(&ws->group[grp].count, 0u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
            const unsigned top = __hip_atomic_fetch_add(&ws->top.count, 1u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
            is_last = top == ngroups - 1;
            if (top >= ngroups) __hip_atomic_store(overlap, 1u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
        } else if (drawn >= in_group) {
            // a ticket this launch cannot have issued: another call's workgroups drew from the same counters (calls that
            // overlap on one GPU); the counters are unusable until lq_fp8_amax_cast_static_reset puts them back to zero
            __hip_atomic_store(overlap, 1u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
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
static int launch_cast(uint8_t* dst, const void* src, const float* scale, int invert, size_t n, hipStream_t st,
                       PanelMap pm = PanelMap{0, 0}) {
    if (pm.k != 0) {  // k-panels: the caller has checked the alignment (every piece of 8 or 16 elements stays inside a 64-element chunk)
        const unsigned grid = stream_grid(n, Chunk16<Tag>::elems);
        const bool wide = (pm.k / 64) % 4 == 0, nt = n * Elem<Tag>::bytes >= kStreamBytes;  // block shapes as in launch_gelu_cast
        const PanelStep stride = panel_step((size_t)grid * 4, pm.k / 64 / (wide ? 4 : 1));
        if (wide && nt) hipLaunchKernelGGL((fp8_cast_kernel<Tag, true, 4>), dim3(grid), dim3(256), 0, st, dst, src, scale, invert, n, pm, stride);
        else if (wide) hipLaunchKernelGGL((fp8_cast_kernel<Tag, false, 4>), dim3(grid), dim3(256), 0, st, dst, src, scale, invert, n, pm, stride);
        else if (nt) hipLaunchKernelGGL((fp8_cast_kernel<Tag, true, 1>), dim3(grid), dim3(256), 0, st, dst, src, scale, invert, n, pm, stride);
        else hipLaunchKernelGGL((fp8_cast_kernel<Tag, false, 1>), dim3(grid), dim3(256), 0, st, dst, src, scale, invert, n, pm, stride);
        return check_launch("fp8_cast");
    }
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
static int launch_amax_ticket(TicketRegion* ws, unsigned* overlap, float* scale_out, const void* x, size_t n, hipStream_t st) {
    size_t slabs = (n + kTicketSlab - 1) / kTicketSlab;
    if (slabs == 0) slabs = 1;
    hipLaunchKernelGGL((fp8_amax_ticket_kernel<Tag>), dim3((unsigned)slabs), dim3(256), 0, st, ws, scale_out, x, n, overlap);
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

template <typename Tag>
static int launch_gelu_cast(uint8_t* dst, float* scale_out, void* h_out, const void* src, const float* src_max, float* clear, size_t n,
                            hipStream_t st, PanelMap pm = PanelMap{0, 0}) {
    const dim3 grid(stream_grid(n, Chunk16<Tag>::elems)), block(256);
    const bool nt = n * Elem<Tag>::bytes >= kStreamBytes;
    if (pm.k != 0) {
        // blocks of 4 rows x 256 elements where k allows it (512 contiguous bytes per source row; 4608x12288 bf16: 34.3 us against
        // 35.9 with 16 rows x 64 elements and 33.6 row-major), else 16 rows x 64 elements
        const bool wide = (pm.k / 64) % 4 == 0;
        const PanelStep stride = panel_step((size_t)grid.x * 4, pm.k / 64 / (wide ? 4 : 1));  // a wavefront's next block: one per wavefront of the grid on
        if (wide && nt) hipLaunchKernelGGL((fp8_gelu_cast_kernel<Tag, true, false, 4>), grid, block, 0, st, dst, scale_out, h_out, src, src_max, clear, n, pm, stride);
        else if (wide) hipLaunchKernelGGL((fp8_gelu_cast_kernel<Tag, false, false, 4>), grid, block, 0, st, dst, scale_out, h_out, src, src_max, clear, n, pm, stride);
        else if (nt) hipLaunchKernelGGL((fp8_gelu_cast_kernel<Tag, true, false, 1>), grid, block, 0, st, dst, scale_out, h_out, src, src_max, clear, n, pm, stride);
        else hipLaunchKernelGGL((fp8_gelu_cast_kernel<Tag, false, false, 1>), grid, block, 0, st, dst, scale_out, h_out, src, src_max, clear, n, pm, stride);
    } else if (h_out != nullptr) {
        hipLaunchKernelGGL((fp8_gelu_cast_kernel<Tag, false, true>), grid, block, 0, st, dst, scale_out, h_out, src, src_max, clear, n);
    } else if (nt) {
        hipLaunchKernelGGL((fp8_gelu_cast_kernel<Tag, true, false>), grid, block, 0, st, dst, scale_out, h_out, src, src_max, clear, n);
    } else {
        hipLaunchKernelGGL((fp8_gelu_cast_kernel<Tag, false, false>), grid, block, 0, st, dst, scale_out, h_out, src, src_max, clear, n);
    }
    return check_launch("fp8_gelu_cast");
}

extern "C" int lq_fp8_gelu_cast(uint8_t* dst, float* scale_out, void* h_out, const void* src, lq_dtype_t dtype, size_t n,
                                const float* src_max, float* clear_max, lq_stream_t stream) {
    LQ_REQUIRE(scale_out && src_max && ((dst && src) || n == 0), LQ_ERR_ARG, "lq_fp8_gelu_cast: null pointer");
    LQ_REQUIRE(clear_max != src_max && clear_max != scale_out, LQ_ERR_ARG,
               "lq_fp8_gelu_cast: clear_max must not be the slot this call reads or the scale it writes");
    LQ_REQUIRE(reinterpret_cast<uintptr_t>(src) % 16 == 0 && reinterpret_cast<uintptr_t>(dst) % 16 == 0 &&
                   reinterpret_cast<uintptr_t>(h_out) % 16 == 0,
               LQ_ERR_ARG, "lq_fp8_gelu_cast: src, dst and h_out must be 16-byte aligned");
    if (n == 0) return LQ_OK;
    switch (dtype) {
        case LQ_F16: return launch_gelu_cast<F16Tag>(dst, scale_out, h_out, src, src_max, clear_max, n, as_stream(stream));
        case LQ_BF16: return launch_gelu_cast<BF16Tag>(dst, scale_out, h_out, src, src_max, clear_max, n, as_stream(stream));
        case LQ_F32: return launch_gelu_cast<F32Tag>(dst, scale_out, h_out, src, src_max, clear_max, n, as_stream(stream));
        default: set_error("lq_fp8_gelu_cast: unsupported dtype %d", (int)dtype); return LQ_ERR_UNSUPPORTED;
    }
}

// LQ_OK, or the error for a shape the k-panel layout does not take
static int panels_check(const char* what, const void* dst, const void* src, size_t rows, size_t k) {
    LQ_REQUIRE(k % 64 == 0 && rows * k <= 0xFFFFFFFFull, LQ_ERR_SHAPE,
               "%s: k-panels need k %% 64 == 0 and fewer than 2^32 elements (rows=%zu k=%zu)", what, rows, k);
    LQ_REQUIRE(reinterpret_cast<uintptr_t>(src) % 16 == 0 && reinterpret_cast<uintptr_t>(dst) % 16 == 0, LQ_ERR_ARG,
               "%s: src and dst must be 16-byte aligned", what);
    return LQ_OK;
}

extern "C" int lq_fp8_amax_cast_panels(uint8_t* dst, float* scale_out, const void* src, lq_dtype_t dtype, size_t rows, size_t k,
                                       lq_stream_t stream) {
    const size_t n = rows * k;
    LQ_REQUIRE(scale_out && ((dst && src) || n == 0), LQ_ERR_ARG, "lq_fp8_amax_cast_panels: null pointer");
    LQ_REQUIRE(dtype == LQ_F16 || dtype == LQ_BF16 || dtype == LQ_F32, LQ_ERR_UNSUPPORTED, "lq_fp8_amax_cast_panels: unsupported dtype %d",
               (int)dtype);
    if (n == 0) return lq_fp8_amax_cast(dst, scale_out, src, dtype, 0, stream);
    int rc = panels_check("lq_fp8_amax_cast_panels", dst, src, rows, k);
    if (rc != LQ_OK) return rc;
    const PanelMap pm{(unsigned)k, (unsigned)rows};
    hipStream_t st = as_stream(stream);
    if (n >= 4096) {
        rc = dtype == LQ_F16    ? launch_amax_cast_coop<F16Tag>(dst, scale_out, src, n, st, nullptr, pm)
             : dtype == LQ_BF16 ? launch_amax_cast_coop<BF16Tag>(dst, scale_out, src, n, st, nullptr, pm)
                                : launch_amax_cast_coop<F32Tag>(dst, scale_out, src, n, st, nullptr, pm);
        if (rc <= 0) return rc;
    }
    // scratch-free sequence, as in lq_fp8_amax_cast
    hipLaunchKernelGGL(fill_f32_kernel, dim3(1), dim3(1), 0, st, scale_out, 0.0f);
    rc = check_launch("fp8_amax_cast_panels(fill)");
    if (rc != LQ_OK) return rc;
    rc = lq_fp8_amax_scale(scale_out, src, dtype, n, stream);
    if (rc != LQ_OK) return rc;
    return dtype == LQ_F16    ? launch_cast<F16Tag>(dst, src, scale_out, 1, n, st, pm)
           : dtype == LQ_BF16 ? launch_cast<BF16Tag>(dst, src, scale_out, 1, n, st, pm)
                              : launch_cast<F32Tag>(dst, src, scale_out, 1, n, st, pm);
}

extern "C" int lq_fp8_scale_cast_panels(uint8_t* dst, const void* src, lq_dtype_t dtype, const float* scale, int invert, size_t rows,
                                        size_t k, lq_stream_t stream) {
    const size_t n = rows * k;
    LQ_REQUIRE(scale && ((dst && src) || n == 0), LQ_ERR_ARG, "lq_fp8_scale_cast_panels: null pointer");
    LQ_REQUIRE(dtype == LQ_F16 || dtype == LQ_BF16 || dtype == LQ_F32, LQ_ERR_UNSUPPORTED, "lq_fp8_scale_cast_panels: unsupported dtype %d",
               (int)dtype);
    if (n == 0) return LQ_OK;
    int rc = panels_check("lq_fp8_scale_cast_panels", dst, src, rows, k);
    if (rc != LQ_OK) return rc;
    const PanelMap pm{(unsigned)k, (unsigned)rows};
    hipStream_t st = as_stream(stream);
    return dtype == LQ_F16    ? launch_cast<F16Tag>(dst, src, scale, invert, n, st, pm)
           : dtype == LQ_BF16 ? launch_cast<BF16Tag>(dst, src, scale, invert, n, st, pm)
                              : launch_cast<F32Tag>(dst, src, scale, invert, n, st, pm);
}

extern "C" int lq_fp8_gelu_cast_panels(uint8_t* dst, float* scale_out, const void* src, lq_dtype_t dtype, size_t rows, size_t k,
                                       const float* src_max, float* clear_max, lq_stream_t stream) {
    const size_t n = rows * k;
    LQ_REQUIRE(scale_out && src_max && ((dst && src) || n == 0), LQ_ERR_ARG, "lq_fp8_gelu_cast_panels: null pointer");
    LQ_REQUIRE(clear_max != src_max && clear_max != scale_out, LQ_ERR_ARG,
               "lq_fp8_gelu_cast_panels: clear_max must not be the slot this call reads or the scale it writes");
    LQ_REQUIRE(dtype == LQ_F16 || dtype == LQ_BF16 || dtype == LQ_F32, LQ_ERR_UNSUPPORTED, "lq_fp8_gelu_cast_panels: unsupported dtype %d",
               (int)dtype);
    if (n == 0) return LQ_OK;
    int rc = panels_check("lq_fp8_gelu_cast_panels", dst, src, rows, k);
    if (rc != LQ_OK) return rc;
    const PanelMap pm{(unsigned)k, (unsigned)rows};
    hipStream_t st = as_stream(stream);
    return dtype == LQ_F16    ? launch_gelu_cast<F16Tag>(dst, scale_out, nullptr, src, src_max, clear_max, n, st, pm)
           : dtype == LQ_BF16 ? launch_gelu_cast<BF16Tag>(dst, scale_out, nullptr, src, src_max, clear_max, n, st, pm)
                              : launch_gelu_cast<F32Tag>(dst, scale_out, nullptr, src, src_max, clear_max, n, st, pm);
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

extern "C" int lq_fp8_amax_cast_timeline(uint8_t* dst, float* scale_out, const void* src, lq_dtype_t dtype, size_t n,
                                         unsigned long long* stamps, lq_stream_t stream) {
    LQ_REQUIRE(dst && scale_out && src && stamps, LQ_ERR_ARG, "lq_fp8_amax_cast_timeline: null pointer");
    int rc = 1;
    if (n >= 4096) {
        switch (dtype) {
            case LQ_F16: rc = launch_amax_cast_coop<F16Tag>(dst, scale_out, src, n, as_stream(stream), stamps); break;
            case LQ_BF16: rc = launch_amax_cast_coop<BF16Tag>(dst, scale_out, src, n, as_stream(stream), stamps); break;
            case LQ_F32: rc = launch_amax_cast_coop<F32Tag>(dst, scale_out, src, n, as_stream(stream), stamps); break;
            default: set_error("lq_fp8_amax_cast_timeline: unsupported dtype %d", (int)dtype); return LQ_ERR_UNSUPPORTED;
        }
    }
    if (rc == 1) {
        set_error("lq_fp8_amax_cast_timeline: the one-launch form does not apply to this call (size, alignment, stream or capture)");
        return LQ_ERR_UNSUPPORTED;
    }
    return rc;
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
        case LQ_F16: rc = launch_amax_ticket<F16Tag>(&ws->ticket, &ws->ticket_overlap, scale_out, src, n, st); break;
        case LQ_BF16: rc = launch_amax_ticket<BF16Tag>(&ws->ticket, &ws->ticket_overlap, scale_out, src, n, st); break;
        default: rc = launch_amax_ticket<F32Tag>(&ws->ticket, &ws->ticket_overlap, scale_out, src, n, st); break;
    }
    if (rc != LQ_OK) return rc;
    return lq_fp8_scale_cast(dst, src, dtype, scale_out, 1, n, stream);
}

extern "C" int lq_fp8_amax_cast_slot(lq_stream_t stream) {
    int dev = 0;
    if (device_scratch(&dev) == nullptr) return LQ_ERR_HIP;
    return slot_for_stream(dev, as_stream(stream));
}

extern "C" int lq_fp8_amax_cast_release_slot(lq_stream_t stream) {
    int dev = 0;
    if (device_scratch(&dev) == nullptr) return LQ_ERR_HIP;
    return release_slot(dev, as_stream(stream));
}

extern "C" size_t lq_fp8_amax_cast_static_max_elems(void) { return kTicketSlab * kTicketMaxSlabs; }

namespace lq {
__global__ void ticket_reset_kernel(TicketRegion* ws, unsigned* overlap) {
    if (threadIdx.x < kTicketGroups) ws->group[threadIdx.x].count = 0;
    if (threadIdx.x == kTicketGroups) ws->top.count = 0;
    if (threadIdx.x == kTicketGroups + 1) *overlap = 0;
}
}  // namespace lq

extern "C" int lq_fp8_amax_cast_static_reset(lq_stream_t stream) {
    FusedScratch* ws = device_scratch();
    if (ws == nullptr) return LQ_ERR_HIP;
    hipLaunchKernelGGL(ticket_reset_kernel, dim3(1), dim3(64), 0, as_stream(stream), &ws->ticket, &ws->ticket_overlap);
    return check_launch("fp8_amax_cast_static_reset");
}

extern "C" int lq_fp8_amax_cast_status(void) {
    FusedScratch* ws = device_scratch();
    if (ws == nullptr) return LQ_ERR_HIP;
    unsigned flags[2] = {0, 0};
    hipError_t e = hipMemcpy(flags, &ws->timeout, sizeof(flags), hipMemcpyDeviceToHost);
    if (e == hipSuccess && flags[0] != 0) {
        const unsigned zero = 0;
        e = hipMemcpy(&ws->timeout, &zero, sizeof(zero), hipMemcpyHostToDevice);
    }
    const unsigned flag = flags[0];
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
    if (flags[1] != 0) {
        set_error("lq_fp8_amax_cast_static: calls overlapped on this GPU and left the ticket counters of the static scratch in a "
                  "state no later call can finish from (scales stay unwritten); serialise the calls and run "
                  "lq_fp8_amax_cast_static_reset");
        return 2;
    }
    return 0;
}
