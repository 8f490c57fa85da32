// lyradiff_layers.h -- header-only host-side layer types of the quantized-linear path, over the C ABI
// of lyraquant.h and the launchers of lyradiff_compat.h: the tensor plumbing (Tensor, TensorMap), the
// named scratch pool (IAllocator / Allocator), the W4A4 linear layer with its weight container, the FP8 weight
// that takes LoRA deltas (FP8LoraWeight) and the FP8 feed-forward halves of the FLUX blocks,
// with the reference's names, members and call shapes (paths relative to the reference's
// src/lyradiff/), so that reference-style layer code compiles against liblyraquant.so.
// Weight files: loadWeightFromBin reads the reference's raw .bin files (one tensor per file, elements of the stated
// file type, converted to the member's type on the way in) and every weight class has loadWeights(prefix, file_type)
// next to loadWeightsFromCache.
//
// Not built: the npy/torch tensor readers of Tensor.
#pragma once

#include <cstdlib>
#include <cstring>
#include <fstream>
#include <initializer_list>
#include <sstream>
#include <unordered_map>
#include <utility>

#include "lyradiff_compat.h"

namespace lyradiff {

// ---- utils/cuda_utils.h:128-147 -----------------------------------------------------------------------------------
class LyraException : public std::runtime_error {
public:
    explicit LyraException(const std::string& msg) : std::runtime_error("[lyradiff Error] " + msg) {}
};
#define LYRA_CHECK_WITH_INFO(cond, info)                                                   \
    do {                                                                                   \
        if (!(cond)) throw ::lyradiff::LyraException(std::string("Assertion fail: ") + (info)); \
    } while (0)

// ---- utils/Tensor.h:24-106 ----------------------------------------------------------------------------------------
typedef enum datatype_enum {
    TYPE_INVALID, TYPE_BOOL, TYPE_UINT8, TYPE_UINT16, TYPE_UINT32, TYPE_UINT64, TYPE_INT8, TYPE_INT16, TYPE_INT32,
    TYPE_INT64, TYPE_FP16, TYPE_FP32, TYPE_FP64, TYPE_BYTES, TYPE_BF16, TYPE_FP8_E4M3, TYPE_STR, TYPE_VOID,
} DataType;

template <typename T> DataType getTensorType() {
    using U = typename std::remove_const<T>::type;
    if (std::is_same<U, float>::value) return TYPE_FP32;
    if (std::is_same<U, __half>::value) return TYPE_FP16;
    if (std::is_same<U, hip_bfloat16>::value) return TYPE_BF16;
    if (std::is_same<U, fp8_e4m3_t>::value) return TYPE_FP8_E4M3;
    if (std::is_same<U, int>::value) return TYPE_INT32;
    if (std::is_same<U, int8_t>::value) return TYPE_INT8;
    if (std::is_same<U, unsigned int>::value) return TYPE_UINT32;
    if (std::is_same<U, unsigned long long>::value) return TYPE_UINT64;
    if (std::is_same<U, bool>::value) return TYPE_BOOL;
    if (std::is_same<U, char>::value) return TYPE_BYTES;
    return TYPE_INVALID;
}

inline size_t getTypeSize(DataType type) {
    switch (type) {
        case TYPE_BOOL: case TYPE_UINT8: case TYPE_INT8: case TYPE_BYTES: case TYPE_FP8_E4M3: return 1;
        case TYPE_UINT16: case TYPE_INT16: case TYPE_FP16: case TYPE_BF16: return 2;
        case TYPE_UINT32: case TYPE_INT32: case TYPE_FP32: return 4;
        case TYPE_UINT64: case TYPE_INT64: case TYPE_FP64: return 8;
        default: return 0;
    }
}

typedef enum memorytype_enum { MEMORY_CPU, MEMORY_CPU_PINNED, MEMORY_GPU } MemoryType;

struct Tensor {
    MemoryType where = MEMORY_CPU;
    DataType type = TYPE_INVALID;
    std::vector<size_t> shape;
    const void* data = nullptr;

    Tensor() {}
    Tensor(MemoryType where_, DataType type_, std::vector<size_t> shape_, const void* data_)
        : where(where_), type(type_), shape(std::move(shape_)), data(data_) {}

    size_t size() const {
        if (data == nullptr || shape.empty()) return 0;
        size_t n = 1;
        for (size_t d : shape) n *= d;
        return n;
    }
    size_t sizeBytes() const { return size() * getTypeSize(type); }
    std::string getShapeStr() const {
        std::ostringstream s;
        s << "(";
        for (size_t i = 0; i < shape.size(); ++i) s << shape[i] << (i + 1 < shape.size() ? ", " : "");
        s << ")";
        return s.str();
    }
    // typed access with the reference's check that the element type matches (Tensor.h getPtr)
    template <typename T> T* getPtr() const {
        LYRA_CHECK_WITH_INFO(getTensorType<T>() == type || type == TYPE_VOID || type == TYPE_BYTES,
                             "getPtr: element type mismatch for tensor of shape " + getShapeStr());
        return const_cast<T*>(static_cast<const T*>(data));
    }
};

// ---- utils/Tensor.h:312-405 ---------------------------------------------------------------------------------------
class TensorMap {
public:
    TensorMap() = default;
    TensorMap(std::initializer_list<std::pair<std::string, Tensor>> tensors) {
        for (auto& kv : tensors) insert(kv.first, kv.second);
    }
    size_t size() const { return tensor_map_.size(); }
    bool isExist(const std::string& key) const { return tensor_map_.find(key) != tensor_map_.end(); }
    std::vector<std::string> keys() const {
        std::vector<std::string> k;
        for (auto& kv : tensor_map_) k.push_back(kv.first);
        return k;
    }
    void insert(const std::string& key, const Tensor& value) {
        LYRA_CHECK_WITH_INFO(!isExist(key), "Duplicated key " + key);
        LYRA_CHECK_WITH_INFO(value.size() > 0 && value.data != nullptr,
                             "A none tensor or nullptr is not allowed (key is " + key + ")");
        tensor_map_.insert({key, value});
    }
    Tensor at(int) = delete;  // keep integers from converting to a key
    Tensor at(size_t) = delete;
    Tensor& at(const std::string& key) {
        LYRA_CHECK_WITH_INFO(isExist(key), missing(key));
        return tensor_map_.at(key);
    }
    Tensor at(const std::string& key) const {
        LYRA_CHECK_WITH_INFO(isExist(key), missing(key));
        return tensor_map_.at(key);
    }

private:
    std::string missing(const std::string& key) const {
        std::string all;
        for (auto& k : keys()) all += (all.empty() ? "" : ", ") + k;
        return "Cannot find a tensor of name " + key + " in the tensor map (keys: " + all + ")";
    }
    std::unordered_map<std::string, Tensor> tensor_map_;
};

// ---- utils/allocator.h:50-104,221-242 -----------------------------------------------------------------------------
// Named scratch pool: a buffer requested under a name is created on first use, grown when a later
// request is larger and otherwise reused, so layers that ask for the same name share one buffer.
class IAllocator {
public:
    virtual ~IAllocator() {}
    virtual void* malloc(size_t size, const bool is_set_zero = true) = 0;
    virtual void free(void** ptr) = 0;
    virtual void setStream(hipStream_t stream) = 0;
    virtual hipStream_t returnStream() = 0;
    virtual void memSet(void* ptr, const int val, const size_t size) = 0;
    virtual size_t getAllSize() = 0;
    virtual void freeAllNameBuf() = 0;
    virtual void freeWithName(const std::string& buf_name) = 0;
    virtual void* reMallocWithName(std::string buf_name, size_t size, const bool is_set_zero = true) = 0;
};

class Allocator : public IAllocator {
public:
    explicit Allocator(int device_id = 0) : device_id_(device_id) {}
    ~Allocator() override {
        for (auto& kv : sizes_) (void)hipFree(kv.first);
    }
    void* malloc(size_t size, const bool is_set_zero = true) override {
        if (size == 0) return nullptr;
        void* p = nullptr;
        const size_t rounded = (size + 31) / 32 * 32;
        if (hipMalloc(&p, rounded) != hipSuccess) throw LyraException("Allocator: hipMalloc of " + std::to_string(rounded) + " bytes failed");
        if (is_set_zero && hipMemsetAsync(p, 0, rounded, stream_) != hipSuccess) throw LyraException("Allocator: memset failed");
        sizes_[p] = rounded;
        return p;
    }
    void free(void** ptr) override {
        if (ptr == nullptr || *ptr == nullptr) return;
        auto it = sizes_.find(*ptr);
        LYRA_CHECK_WITH_INFO(it != sizes_.end(), "Allocator::free of a pointer this allocator does not own");
        (void)hipFree(*ptr);
        sizes_.erase(it);
        for (auto n = names_.begin(); n != names_.end();) n = (n->second == *ptr) ? names_.erase(n) : std::next(n);
        *ptr = nullptr;
    }
    void setStream(hipStream_t stream) override { stream_ = stream; }
    hipStream_t returnStream() override { return stream_; }
    void memSet(void* ptr, const int val, const size_t size) override {
        if (hipMemsetAsync(ptr, val, size, stream_) != hipSuccess) throw LyraException("Allocator: memset failed");
    }
    size_t getAllSize() override {
        size_t total = 0;
        for (auto& kv : sizes_) total += kv.second;
        return total;
    }
    void freeAllNameBuf() override {
        while (!names_.empty()) {
            void* p = names_.begin()->second;
            free(&p);
        }
    }
    void freeWithName(const std::string& buf_name) override {
        auto it = names_.find(buf_name);
        if (it == names_.end()) return;
        void* p = it->second;
        free(&p);
    }
    void* reMallocWithName(std::string buf_name, size_t size, const bool is_set_zero = true) override {
        auto it = names_.find(buf_name);
        if (it != names_.end() && sizes_.at(it->second) >= size) return it->second;  // large enough: reuse as is
        if (it != names_.end()) {
            // growing: work queued on the stream may still read the old buffer
            if (hipStreamSynchronize(stream_) != hipSuccess) throw LyraException("Allocator: stream synchronize failed");
            void* old = it->second;
            free(&old);
        }
        void* p = malloc(size, is_set_zero);
        names_[buf_name] = p;
        return p;
    }

private:
    int device_id_;
    hipStream_t stream_ = 0;
    std::unordered_map<void*, size_t> sizes_;
    std::unordered_map<std::string, void*> names_;
};

// ---- utils/cuda_utils.h:45-55 -------------------------------------------------------------------------------------
enum LyraQuantType {
    NONE = 0, FP8_W8A8 = 1, FP8_W8A8_FULL = 2, FP8_WEIGHT_ONLY = 3, INT8_SMOOTH_QUANT_LEVEL1 = 4,
    INT8_SMOOTH_QUANT_LEVEL2 = 5, INT8_SMOOTH_QUANT_LEVEL3 = 6, INT4_W4A4 = 7, INT4_W4A4_FULL = 8,
};

// ---- utils/cuda_utils.h:37-43 and utils/memory_utils.cu:250-360 ------------------------------------------------------
enum FtCudaDataType { FP32 = 0, FP16 = 1, BF16 = 2, INT8 = 3, FP8 = 4 };

namespace detail {
template <typename T> struct HostCast;  // element conversions of loadWeightFromBin (round to nearest even, as the
template <> struct HostCast<float> {    // reference's device-side invokeCudaD2DcpyConvert does)
    static float from(float v) { return v; }
    static float to(float v) { return v; }
};
template <> struct HostCast<__half> {
    static __half from(float v) { return __float2half(v); }
    static float to(__half v) { return __half2float(v); }
};
template <> struct HostCast<hip_bfloat16> {
    static hip_bfloat16 from(float v) { return hip_bfloat16(v); }
    static float to(hip_bfloat16 v) { return static_cast<float>(v); }
};
template <> struct HostCast<int8_t> {  // never converted (INT8 files load into int8_t members only); keeps the generic code well-formed
    static int8_t from(float v) { return static_cast<int8_t>(v); }
    static float to(int8_t v) { return static_cast<float>(v); }
};
template <typename T_IN> inline bool read_bin(const std::string& filename, size_t count, std::vector<T_IN>& host) {
    std::ifstream in(filename, std::ios::in | std::ios::binary);
    if (!in.is_open()) return false;
    host.resize(count);
    in.read(reinterpret_cast<char*>(host.data()), static_cast<std::streamsize>(sizeof(T_IN) * count));
    return static_cast<size_t>(in.gcount()) == sizeof(T_IN) * count;
}
}  // namespace detail

// Reads shape[0] (* shape[1]) elements of `model_file_type` from `filename` into device memory at `ptr`, converting
// them to T (loadWeightFromBin, utils/memory_utils.cu:336-360).  The reference only logs a warning when a file is
// missing or short and leaves the weight unset; here that throws LyraException, since a linear with a missing weight
// cannot produce a valid result.  Synchronous (hipMemcpy), like the reference's cudaH2Dcpy.
template <typename T>
int loadWeightFromBin(T* ptr, std::vector<size_t> shape, std::string filename, FtCudaDataType model_file_type = FtCudaDataType::FP32) {
    LYRA_CHECK_WITH_INFO(shape.size() >= 1 && shape.size() <= 2, "loadWeightFromBin: shape should have one or two dims");
    const size_t count = shape[0] * (shape.size() == 2 ? shape[1] : 1);
    if (count == 0) return 0;
    std::vector<T> out(count);
    auto convert = [&](auto tag) {
        using T_IN = decltype(tag);
        std::vector<T_IN> host;
        LYRA_CHECK_WITH_INFO(detail::read_bin<T_IN>(filename, count, host), "file " + filename + " cannot be opened or is too short, loading model fails");
        if constexpr (std::is_same<T, T_IN>::value) out.swap(host);
        else if constexpr (std::is_same<T, int8_t>::value || std::is_same<T_IN, int8_t>::value)
            LYRA_CHECK_WITH_INFO(false, "loadWeightFromBin: INT8 files load into int8_t members only");
        else
            for (size_t i = 0; i < count; ++i) out[i] = detail::HostCast<T>::from(detail::HostCast<T_IN>::to(host[i]));
    };
    switch (model_file_type) {
        case FtCudaDataType::FP32: convert(float{}); break;
        case FtCudaDataType::FP16: convert(__half{}); break;
        case FtCudaDataType::BF16: convert(hip_bfloat16{}); break;
        case FtCudaDataType::INT8: convert(int8_t{}); break;
        default: LYRA_CHECK_WITH_INFO(false, "loadWeightFromBin: does not support FtCudaDataType=" + std::to_string(static_cast<int>(model_file_type)));
    }
    LYRA_CHECK_WITH_INFO(hipMemcpy(ptr, out.data(), sizeof(T) * count, hipMemcpyHostToDevice) == hipSuccess, "loadWeightFromBin: copy to the device failed");
    return 0;
}

// ---- layers/w4a4_gemm_block/W4A4GemmWeight.h:7-45, W4A4GemmWeight.cc:31-83 -----------------------------------------
// Device-resident weights of one W4A4 linear.  `packed_weight` holds the [d_out, d_in/2] nibble matrix in
// the rows32 layout the GEMM reads; loadWeightsFromCache takes the reference's row-major bytes and
// repacks them once.  lora_rank = 0 leaves the low-rank members null and the layer skips that branch.
template <typename T>
class W4A4GemmWeight {
public:
    int8_t* packed_weight = nullptr;  // d_out * d_in / 2 bytes, rows32 layout
    float* weight_scale = nullptr;    // fp32 [d_out, d_in / group_size]
    T* lora_up = nullptr;
    T* lora_down = nullptr;
    T* bias = nullptr;                // [d_out]
    float* smooth = nullptr;          // fp32 [d_in]

    W4A4GemmWeight() = default;
    W4A4GemmWeight(size_t d_out, size_t d_in, size_t lora_rank = 32, bool has_bias = false, size_t group_size = 64,
                   LyraQuantType quant_level = LyraQuantType::NONE, IAllocator* allocator = nullptr)
        : d_out_(d_out), d_in_(d_in), lora_rank_(lora_rank), group_size_(group_size), group_num_(d_in / group_size),
          has_bias_(has_bias) {
        (void)quant_level;
        (void)allocator;
        LYRA_CHECK_WITH_INFO(group_size == 64 && d_in % 128 == 0 && d_out % 32 == 0,
                             "W4A4GemmWeight: needs group_size 64, d_in % 128 == 0, d_out % 32 == 0");
        LYRA_CHECK_WITH_INFO(lora_rank == 0 || lora_rank == 32 || lora_rank == 64, "W4A4GemmWeight: lora_rank must be 0, 32 or 64");
    }
    W4A4GemmWeight(const W4A4GemmWeight&) = delete;
    W4A4GemmWeight& operator=(const W4A4GemmWeight&) = delete;
    virtual ~W4A4GemmWeight() {
        if (is_maintain_buffer) {
            (void)hipFree(packed_weight);
            (void)hipFree(weight_scale);
            (void)hipFree(smooth);
            (void)hipFree(lora_up);
            (void)hipFree(lora_down);
            if (has_bias_) (void)hipFree(bias);
        }
    }
    virtual void mallocWeights() {
        if (!is_maintain_buffer) {
            dmalloc(&packed_weight, d_out_ * d_in_ / 2);
            dmalloc(&weight_scale, d_out_ * group_num_);
            dmalloc(&smooth, d_in_);
            if (lora_rank_ > 0) {
                dmalloc(&lora_up, d_out_ * lora_rank_);
                dmalloc(&lora_down, d_in_ * lora_rank_);
            }
            if (has_bias_) dmalloc(&bias, d_out_);
        }
        is_maintain_buffer = true;
    }
    // Keys: prefix + "packed_weight" (row-major [d_out, d_in/2] bytes, two int4 per byte, low nibble first),
    // "weight_scale", "smooth", "lora_up" ([d_out, rank]), "lora_down" ([rank, d_in]), "bias" -- the names of
    // the reference's .bin files (W4A4GemmWeight.cc:65-83).
    virtual void loadWeightsFromCache(std::string prefix, std::unordered_map<std::string, void*>& weights,
                                      hipMemcpyKind memcpyKind, hipStream_t stream = 0) {
        if (!is_maintain_buffer) mallocWeights();
        auto get = [&](const char* name) -> void* {
            auto it = weights.find(prefix + name);
            LYRA_CHECK_WITH_INFO(it != weights.end() && it->second != nullptr, "missing weight " + prefix + name);
            return it->second;
        };
        const size_t wbytes = d_out_ * d_in_ / 2;
        void* staging = nullptr;
        LYRA_CHECK_WITH_INFO(hipMalloc(&staging, wbytes) == hipSuccess, "W4A4GemmWeight: staging allocation failed");
        bool ok = hipMemcpyAsync(staging, get("packed_weight"), wbytes, memcpyKind, stream) == hipSuccess;
        ok = ok && lq_repack_rows32(reinterpret_cast<uint8_t*>(packed_weight), static_cast<const uint8_t*>(staging),
                                    d_out_, d_in_ / 2, stream) == LQ_OK;
        ok = ok && hipMemcpyAsync(weight_scale, get("weight_scale"), sizeof(float) * d_out_ * group_num_, memcpyKind, stream) == hipSuccess;
        ok = ok && hipMemcpyAsync(smooth, get("smooth"), sizeof(float) * d_in_, memcpyKind, stream) == hipSuccess;
        if (lora_rank_ > 0) {
            ok = ok && hipMemcpyAsync(lora_up, get("lora_up"), sizeof(T) * d_out_ * lora_rank_, memcpyKind, stream) == hipSuccess;
            ok = ok && hipMemcpyAsync(lora_down, get("lora_down"), sizeof(T) * d_in_ * lora_rank_, memcpyKind, stream) == hipSuccess;
        }
        if (has_bias_) ok = ok && hipMemcpyAsync(bias, get("bias"), sizeof(T) * d_out_, memcpyKind, stream) == hipSuccess;
        ok = ok && hipStreamSynchronize(stream) == hipSuccess;
        (void)hipFree(staging);
        LYRA_CHECK_WITH_INFO(ok, std::string("W4A4GemmWeight::loadWeightsFromCache failed: ") + lq_last_error());
    }
    // The reference's raw files prefix + {packed_weight, weight_scale, lora_up, lora_down, smooth, bias}.bin
    // (W4A4GemmWeight.cc:65-83): int8 / fp32 files as they are, the 16-bit members converted from model_file_type;
    // the nibble matrix is repacked to rows32 once, as loadWeightsFromCache does.
    virtual void loadWeights(const std::string prefix, FtCudaDataType model_file_type) {
        if (!is_maintain_buffer) mallocWeights();
        const size_t wbytes = d_out_ * d_in_ / 2;
        int8_t* staging = nullptr;
        LYRA_CHECK_WITH_INFO(hipMalloc(reinterpret_cast<void**>(&staging), wbytes) == hipSuccess, "W4A4GemmWeight: staging allocation failed");
        try {
            loadWeightFromBin<int8_t>(staging, {wbytes}, prefix + "packed_weight.bin", FtCudaDataType::INT8);
        } catch (...) {
            (void)hipFree(staging);
            throw;
        }
        bool ok = lq_repack_rows32(reinterpret_cast<uint8_t*>(packed_weight), reinterpret_cast<const uint8_t*>(staging), d_out_, d_in_ / 2, 0) == LQ_OK &&
                  hipStreamSynchronize(0) == hipSuccess;
        (void)hipFree(staging);
        LYRA_CHECK_WITH_INFO(ok, std::string("W4A4GemmWeight::loadWeights: repack failed: ") + lq_last_error());
        loadWeightFromBin<float>(weight_scale, {d_out_ * group_num_}, prefix + "weight_scale.bin", FtCudaDataType::FP32);
        if (lora_rank_ > 0) {
            loadWeightFromBin<T>(lora_up, {d_out_ * lora_rank_}, prefix + "lora_up.bin", model_file_type);
            loadWeightFromBin<T>(lora_down, {d_in_ * lora_rank_}, prefix + "lora_down.bin", model_file_type);
        }
        loadWeightFromBin<float>(smooth, {d_in_}, prefix + "smooth.bin", FtCudaDataType::FP32);
        if (has_bias_) loadWeightFromBin<T>(bias, {d_out_}, prefix + "bias.bin", model_file_type);
    }
    size_t lora_rank() const { return lora_rank_; }
    size_t d_out() const { return d_out_; }
    size_t d_in() const { return d_in_; }
    bool has_bias() const { return has_bias_; }

protected:
    bool is_maintain_buffer = false;

private:
    template <typename U> static void dmalloc(U** p, size_t count) {
        LYRA_CHECK_WITH_INFO(hipMalloc(reinterpret_cast<void**>(p), sizeof(U) * count) == hipSuccess, "deviceMalloc failed");
    }
    size_t d_out_ = 0, d_in_ = 0, lora_rank_ = 32, group_size_ = 64, group_num_ = 0;
    bool has_bias_ = true;
};

// ---- layers/w4a4_gemm_block/W4A4Gemm.h:13-52, W4A4Gemm.cc:87-169 ---------------------------------------------------
// forward(): quantise the [m, d_in] input to group-64 int4 words + fp32 group scales in pool buffers
// named as in the reference, then the W4A4 GEMM with the bias fused.  T = __half or hip_bfloat16.
template <typename T>
class W4A4Gemm {
public:
    W4A4Gemm(size_t d_out, size_t d_in, size_t lora_rank, bool has_bias, size_t group_size, hipStream_t stream,
             void* /*cublas_wrapper*/, IAllocator* allocator, const bool is_free_buffer_after_forward,
             const bool /*sparse*/ = false, const LyraQuantType /*quant_level*/ = LyraQuantType::NONE)
        : d_out_(d_out), d_in_(d_in), lora_rank_(lora_rank), group_size_(group_size), group_num_(d_in / group_size),
          has_bias_(has_bias), stream_(stream), allocator_(allocator),
          is_free_buffer_after_forward_(is_free_buffer_after_forward) {
        LYRA_CHECK_WITH_INFO(allocator_ != nullptr, "W4A4Gemm needs an allocator");
        LYRA_CHECK_WITH_INFO(group_size == 64, "W4A4Gemm: only group_size 64 is supported");
    }
    virtual ~W4A4Gemm() {}

    virtual void forward(const TensorMap* output_tensors, const TensorMap* input_tensors, const W4A4GemmWeight<T>* weights) {
        Tensor input_tensor = input_tensors->at("input");
        Tensor output_tensor = output_tensors->at("output");
        LYRA_CHECK_WITH_INFO(input_tensor.shape.size() == 2 && output_tensor.shape.size() == 2, "W4A4Gemm: tensors must be 2-D");
        const size_t m = input_tensor.shape[0], k = input_tensor.shape[1], n = output_tensor.shape[1];
        LYRA_CHECK_WITH_INFO(k == d_in_ && n == d_out_ && output_tensor.shape[0] == m, "W4A4Gemm: shape mismatch");
        const bool low_rank = weights->lora_up != nullptr && weights->lora_down != nullptr;
        LYRA_CHECK_WITH_INFO(!low_rank || weights->lora_rank() == lora_rank_, "W4A4Gemm: lora rank of layer and weights differ");
        allocateBuffer(m);
        if (low_rank)  // one pass over the input: quantised words and scales, and the down projection of the unsmoothed input
                       // written as T directly (no fp32 detour)
            detail::check(lq_w4a4_quantize_lora_down(quantized_input_buffer, input_scale_buffer, LQ_F32, lora_down_res_buffer2,
                                                     detail::DType<T>::value, input_tensor.getPtr<T>(), detail::DType<T>::value,
                                                     weights->smooth, weights->lora_down, (int)m, (int)k, (int)lora_rank_,
                                                     (int)group_size_, stream_),
                          "W4A4Gemm::forward quantize and lora down");
        else
            detail::check(lq_w4a4_quantize(quantized_input_buffer, input_scale_buffer, LQ_F32, input_tensor.getPtr<T>(),
                                           detail::DType<T>::value, weights->smooth, (int)m, (int)k, (int)group_size_, stream_),
                          "W4A4Gemm::forward quantize");
        detail::check(lq_gemm_w4a4_lora(output_tensor.getPtr<T>(), detail::DType<T>::value, quantized_input_buffer,
                                        reinterpret_cast<const uint8_t*>(weights->packed_weight), input_scale_buffer,
                                        weights->weight_scale, LQ_F32, has_bias_ ? weights->bias : nullptr,
                                        low_rank ? lora_down_res_buffer2 : nullptr, low_rank ? weights->lora_up : nullptr,
                                        detail::DType<T>::value, (int)lora_rank_, (int)m, (int)n, (int)k, (int)group_size_, stream_),
                      "W4A4Gemm::forward gemm");
        if (is_free_buffer_after_forward_) freeBuffer();
    }

protected:
    // sizes follow W4A4Gemm.cc:89-92: 4 bytes per 8 inputs, one fp32 scale per group, m x rank low-rank activations
    void allocateBuffer(size_t m) {
        if (lora_rank_ > 0)
            lora_down_res_buffer2 = static_cast<T*>(
                allocator_->reMallocWithName("W4A4Gemm_lora_down_res_buffer2", sizeof(T) * m * lora_rank_, false));
        input_scale_buffer = static_cast<float*>(
            allocator_->reMallocWithName("W4A4Gemm_context_input_scale_buffer", sizeof(float) * m * group_num_, false));
        quantized_input_buffer = static_cast<uint32_t*>(
            allocator_->reMallocWithName("W4A4Gemm_quantized_input_buffer", sizeof(uint32_t) * m * d_in_ / 8, false));
    }
    void freeBuffer() {}  // pool buffers outlive the call, as in the reference

    size_t d_out_, d_in_, lora_rank_ = 32, group_size_ = 64, group_num_ = 0;
    bool has_bias_ = true;
    hipStream_t stream_;
    IAllocator* allocator_;
    bool is_free_buffer_after_forward_;
    float* input_scale_buffer = nullptr;
    uint32_t* quantized_input_buffer = nullptr;
    T* lora_down_res_buffer2 = nullptr;
};

// ---- interface/IFLoraWeight.h:79-128 ------------------------------------------------------------------------------
// One FP8 weight that can take a full-rank LoRA delta: the 16-bit master copy stays on the host, a merge
// re-quantises it with a fresh per-tensor scale.  weight_shape is {d_out, d_in} (the rows32 repack needs both;
// the reference passes the flat element count); `weight` holds rows32 e4m3 codes.
template <typename T>
class FP8LoraWeight {
public:
    FP8LoraWeight() {}
    FP8LoraWeight(const std::vector<size_t> weight_shape, fp8_e4m3_t* weight, float* weight_scale, T* weight_h)
        : weight_shape_(weight_shape), weight_(weight), weight_scale_(weight_scale), weight_h_(weight_h) {
        LYRA_CHECK_WITH_INFO(weight_shape_.size() == 2, "FP8LoraWeight: weight_shape must be {d_out, d_in}");
    }
    virtual ~FP8LoraWeight() {}
    // lora_weight: device pointer to d_out * d_in elements of T
    virtual void load_lora(const T* lora_weight, const float lora_scale, IAllocator* allocator) {
        requantise(lora_weight, lora_scale, allocator);
        loaded_lora = true;
    }
    virtual void clear_lora(IAllocator* allocator) {
        if (!loaded_lora) return;
        requantise(nullptr, 0.0f, allocator);
        loaded_lora = false;
    }
    // quantises the master copy as it is (what the reference's load macros do once at load time)
    void quantise(IAllocator* allocator) { requantise(nullptr, 0.0f, allocator); }

private:
    void requantise(const T* lora_weight, float lora_scale, IAllocator* allocator) {
        const size_t n = weight_shape_[0] * weight_shape_[1];
        hipStream_t st = allocator->returnStream();
        T* tmp = static_cast<T*>(allocator->reMallocWithName("global_shared_weight_buffer_", sizeof(T) * n, false));
        uint8_t* codes = static_cast<uint8_t*>(allocator->reMallocWithName("global_shared_weight_codes_buffer_", n, false));
        LYRA_CHECK_WITH_INFO(hipMemcpyAsync(tmp, weight_h_, sizeof(T) * n, hipMemcpyHostToDevice, st) == hipSuccess,
                             "FP8LoraWeight: upload of the master copy failed");
        if (lora_weight != nullptr)
            detail::check(lq_load_lora(tmp, lora_weight, detail::DType<T>::value, n, lora_scale, st), "FP8LoraWeight load_lora");
        allocator->memSet(weight_scale_, 0, sizeof(float));
        detail::check(lq_fp8_amax_scale(weight_scale_, tmp, detail::DType<T>::value, n, st), "FP8LoraWeight scale");
        detail::check(lq_fp8_scale_cast(codes, tmp, detail::DType<T>::value, weight_scale_, 1, n, st), "FP8LoraWeight cast");
        detail::check(lq_repack_rows32(reinterpret_cast<uint8_t*>(weight_), codes, weight_shape_[0], weight_shape_[1], st),
                      "FP8LoraWeight repack");
    }
    std::vector<size_t> weight_shape_;
    fp8_e4m3_t* weight_ = nullptr;
    float* weight_scale_ = nullptr;
    T* weight_h_ = nullptr;
    bool loaded_lora = false;
};

namespace detail {
// members of one FP8 linear as the reference's weight classes declare them (X_weight, X_bias, X_weight_scale,
// X_input_scale, X_weight_h; layers/flux_attention_processor/FluxAttentionFP8ProcessorWeight.h:19-44)
template <typename T> struct FP8LinearStore {
    fp8_e4m3_t* weight = nullptr;
    T* bias = nullptr;
    float* weight_scale = nullptr;
    float* input_scale = nullptr;
    T* weight_h = nullptr;
    size_t d_out = 0, d_in = 0;
    void alloc(size_t n, size_t k) {
        d_out = n; d_in = k;
        bool ok = hipMalloc(reinterpret_cast<void**>(&weight), n * k) == hipSuccess &&
                  hipMalloc(reinterpret_cast<void**>(&bias), sizeof(T) * n) == hipSuccess &&
                  hipMalloc(reinterpret_cast<void**>(&weight_scale), sizeof(float)) == hipSuccess &&
                  hipMalloc(reinterpret_cast<void**>(&input_scale), sizeof(float)) == hipSuccess;
        weight_h = static_cast<T*>(std::malloc(sizeof(T) * n * k));
        LYRA_CHECK_WITH_INFO(ok && weight_h != nullptr, "FP8 weight allocation failed");
    }
    void release() {
        (void)hipFree(weight); (void)hipFree(bias); (void)hipFree(weight_scale); (void)hipFree(input_scale);
        std::free(weight_h);
        weight = nullptr; bias = nullptr; weight_scale = nullptr; input_scale = nullptr; weight_h = nullptr;
    }
    // MACROLoadFP8WeightFromCache (utils/common_macro_def.h:77-92): keys prefix + name + {".weight", ".bias", "_input_scale"}
    void load(const std::string& prefix, const std::string& name, std::unordered_map<std::string, void*>& weights,
              hipMemcpyKind kind, IAllocator* allocator) {
        auto get = [&](const std::string& key) -> void* {
            auto it = weights.find(key);
            LYRA_CHECK_WITH_INFO(it != weights.end() && it->second != nullptr, "missing weight " + key);
            return it->second;
        };
        hipStream_t st = allocator->returnStream();
        const hipMemcpyKind to_host = kind == hipMemcpyHostToDevice ? hipMemcpyHostToHost : hipMemcpyDeviceToHost;
        bool ok = hipMemcpyAsync(weight_h, get(prefix + name + ".weight"), sizeof(T) * d_out * d_in, to_host, st) == hipSuccess &&
                  hipMemcpyAsync(bias, get(prefix + name + ".bias"), sizeof(T) * d_out, kind, st) == hipSuccess &&
                  hipMemcpyAsync(input_scale, get(prefix + name + "_input_scale"), sizeof(float), kind, st) == hipSuccess &&
                  hipStreamSynchronize(st) == hipSuccess;
        LYRA_CHECK_WITH_INFO(ok, "FP8 weight copy failed for " + prefix + name);
        FP8LoraWeight<T>({d_out, d_in}, weight, weight_scale, weight_h).quantise(allocator);
    }
    // MACROLoadFP8WeightFromBin (utils/common_macro_def.h:66-75): prefix + name + {".weight.bin", ".bias.bin",
    // "_input_scale.bin"}; the 16-bit weight becomes the host master copy and is quantised on the device with a fresh
    // per-tensor scale (the staging buffer of the macro is the pool buffer FP8LoraWeight uses).
    void load_bin(const std::string& prefix, const std::string& name, FtCudaDataType model_file_type, IAllocator* allocator) {
        T* tmp = static_cast<T*>(allocator->reMallocWithName("global_shared_weight_buffer_", sizeof(T) * d_out * d_in, false));
        loadWeightFromBin<T>(tmp, {d_out * d_in}, prefix + name + ".weight.bin", model_file_type);
        LYRA_CHECK_WITH_INFO(hipMemcpy(weight_h, tmp, sizeof(T) * d_out * d_in, hipMemcpyDeviceToHost) == hipSuccess, "FP8 master copy failed for " + prefix + name);
        loadWeightFromBin<T>(bias, {d_out}, prefix + name + ".bias.bin", model_file_type);
        loadWeightFromBin<float>(input_scale, {1}, prefix + name + "_input_scale.bin", FtCudaDataType::FP32);
        FP8LoraWeight<T>({d_out, d_in}, weight, weight_scale, weight_h).quantise(allocator);
    }
};
}  // namespace detail

// ---- layers/flux_attn_post_processor/FluxAttnPostFP8ProcessorWeight.h, .cc:20-116 ------------------------------------
template <typename T>
class FluxAttnPostFP8ProcessorWeight {
public:
    fp8_e4m3_t* gelu_proj_weight = nullptr;  // [4D, D] rows32 e4m3
    T* gelu_proj_bias = nullptr;
    float* gelu_proj_weight_scale = nullptr;
    float* gelu_proj_input_scale = nullptr;
    T* gelu_proj_weight_h = nullptr;
    fp8_e4m3_t* ff_linear_weight = nullptr;  // [D, 4D] rows32 e4m3
    T* ff_linear_bias = nullptr;
    float* ff_linear_weight_scale = nullptr;
    float* ff_linear_input_scale = nullptr;
    T* ff_linear_weight_h = nullptr;
    std::unordered_map<std::string, FP8LoraWeight<T>*> lora_weight_map;

    FluxAttnPostFP8ProcessorWeight(size_t embedding_dim, LyraQuantType quant_level, IAllocator* allocator)
        : embedding_dim_(embedding_dim), allocator_(allocator) {
        (void)quant_level;
        LYRA_CHECK_WITH_INFO(allocator_ != nullptr && embedding_dim % 64 == 0, "FluxAttnPostFP8ProcessorWeight: bad arguments");
    }
    FluxAttnPostFP8ProcessorWeight(const FluxAttnPostFP8ProcessorWeight&) = delete;
    FluxAttnPostFP8ProcessorWeight& operator=(const FluxAttnPostFP8ProcessorWeight&) = delete;
    virtual ~FluxAttnPostFP8ProcessorWeight() {
        if (is_maintain_buffer) {
            gelu_.release();
            ff_.release();
            for (auto& kv : lora_weight_map) delete kv.second;
        }
    }
    virtual void mallocWeights() {
        if (is_maintain_buffer) return;
        gelu_.alloc(embedding_dim_ * 4, embedding_dim_);
        ff_.alloc(embedding_dim_, embedding_dim_ * 4);
        publish();
        lora_weight_map = {{"net.0.proj", new FP8LoraWeight<T>({gelu_.d_out, gelu_.d_in}, gelu_proj_weight, gelu_proj_weight_scale, gelu_proj_weight_h)},
                           {"net.2", new FP8LoraWeight<T>({ff_.d_out, ff_.d_in}, ff_linear_weight, ff_linear_weight_scale, ff_linear_weight_h)}};
        is_maintain_buffer = true;
    }
    virtual void loadWeightsFromCache(std::string prefix, std::unordered_map<std::string, void*>& weights, hipMemcpyKind memcpyKind) {
        if (!is_maintain_buffer) mallocWeights();
        gelu_.load(prefix, "net.0.proj", weights, memcpyKind, allocator_);
        ff_.load(prefix, "net.2", weights, memcpyKind, allocator_);
    }
    // FluxAttnPostFP8ProcessorWeight.cc:70-89: the raw files of the two feed-forward linears
    virtual void loadWeights(const std::string prefix, FtCudaDataType model_file_type) {
        if (!is_maintain_buffer) mallocWeights();
        gelu_.load_bin(prefix, "net.0.proj", model_file_type, allocator_);
        ff_.load_bin(prefix, "net.2", model_file_type, allocator_);
    }
    size_t embedding_dim() const { return embedding_dim_; }

protected:
    bool is_maintain_buffer = false;

private:
    void publish() {
        gelu_proj_weight = gelu_.weight; gelu_proj_bias = gelu_.bias; gelu_proj_weight_scale = gelu_.weight_scale;
        gelu_proj_input_scale = gelu_.input_scale; gelu_proj_weight_h = gelu_.weight_h;
        ff_linear_weight = ff_.weight; ff_linear_bias = ff_.bias; ff_linear_weight_scale = ff_.weight_scale;
        ff_linear_input_scale = ff_.input_scale; ff_linear_weight_h = ff_.weight_h;
    }
    size_t embedding_dim_;
    IAllocator* allocator_;
    detail::FP8LinearStore<T> gelu_, ff_;
};

// ---- layers/flux_attn_post_processor/FluxAttnPostFP8Processor.cc:66-240 ---------------------------------------------
// forward(): inputs "input", "attn_output" [B, S, D] and "msa_input" [6, B, D]; output "output" [B, S, D].
// The reference's seven launches become three: gate+residual+adaLN+cast, the up GEMM whose epilogue writes the
// e4m3 codes of gelu(.) for the down GEMM, and the down GEMM whose epilogue applies gate_mlp and the residual.
template <typename T>
class FluxAttnPostFP8Processor {
public:
    FluxAttnPostFP8Processor(size_t embedding_dim, hipStream_t stream, void* /*cublas_wrapper*/, IAllocator* allocator,
                             const bool is_free_buffer_after_forward, const bool /*sparse*/ = false)
        : embedding_dim_(embedding_dim), stream_(stream), allocator_(allocator),
          is_free_buffer_after_forward_(is_free_buffer_after_forward) {
        LYRA_CHECK_WITH_INFO(allocator_ != nullptr, "FluxAttnPostFP8Processor needs an allocator");
    }
    virtual ~FluxAttnPostFP8Processor() {}

    virtual void forward(const TensorMap* output_tensors, const TensorMap* input_tensors,
                         const FluxAttnPostFP8ProcessorWeight<T>* weights) {
        Tensor input_tensor = input_tensors->at("input");
        Tensor attn_tensor = input_tensors->at("attn_output");
        Tensor msa_tensor = input_tensors->at("msa_input");
        Tensor output_tensor = output_tensors->at("output");
        LYRA_CHECK_WITH_INFO(input_tensor.shape.size() == 3 && input_tensor.shape[2] == embedding_dim_ &&
                                 msa_tensor.shape.size() == 3 && msa_tensor.shape[0] == 6,
                             "FluxAttnPostFP8Processor: input must be [B, S, D] and msa_input [6, B, D]");
        const size_t batch_size = input_tensor.shape[0], seq_len = input_tensor.shape[1], d = embedding_dim_;
        const size_t m = batch_size * seq_len;
        allocateBuffer(batch_size, seq_len);
        T* msa = msa_tensor.getPtr<T>();
        const T* gate_msa = msa + 2 * batch_size * d;
        const T* shift_mlp = msa + 3 * batch_size * d;
        const T* scale_mlp = msa + 4 * batch_size * d;
        const T* gate_mlp = msa + 5 * batch_size * d;
        const lq_dtype_t dt = detail::DType<T>::value;
        // the two FP8 activations (fp8_buffer [D/64][M][64], fp8_buffer2 [4D/64][M][64]) are k-panels: same bytes, whole
        // cache lines for the GEMMs' transfers (lyraquant.h)
        detail::check(lq_gate_residual_layernorm_mod_fp8_panels(reinterpret_cast<uint8_t*>(fp8_buffer), hidden_buffer, attn_tensor.getPtr<T>(),
                                                                gate_msa, input_tensor.getPtr<T>(), scale_mlp, shift_mlp, dt,
                                                                weights->gelu_proj_input_scale, batch_size, seq_len, d, 1e-6f, stream_),
                      "FluxAttnPostFP8Processor norm");
        detail::check(lq_gemm_fp8_codes_panels(reinterpret_cast<uint8_t*>(fp8_buffer2), weights->ff_linear_input_scale, dt,
                                               reinterpret_cast<const uint8_t*>(fp8_buffer),
                                               reinterpret_cast<const uint8_t*>(weights->gelu_proj_weight), weights->gelu_proj_input_scale,
                                               weights->gelu_proj_weight_scale, weights->gelu_proj_bias,
                                               /*gelu=*/1, (int)m, (int)(4 * d), (int)d, stream_),
                      "FluxAttnPostFP8Processor gelu_proj");
        detail::check(lq_gemm_fp8_gated_panels(output_tensor.getPtr<T>(), dt, reinterpret_cast<const uint8_t*>(fp8_buffer2),
                                               reinterpret_cast<const uint8_t*>(weights->ff_linear_weight), weights->ff_linear_input_scale,
                                               weights->ff_linear_weight_scale, weights->ff_linear_bias, gate_mlp, seq_len, hidden_buffer,
                                               (int)m, (int)d, (int)(4 * d), stream_),
                      "FluxAttnPostFP8Processor ff_linear");
        if (is_free_buffer_after_forward_) freeBuffer();
    }

protected:
    void allocateBuffer(size_t batch_size, size_t seq_len) {
        const size_t elems = batch_size * seq_len * embedding_dim_;
        hidden_buffer = static_cast<T*>(allocator_->reMallocWithName("FluxAttnPostProcessor_hidden_buffer", sizeof(T) * elems, false));
        fp8_buffer = static_cast<fp8_e4m3_t*>(allocator_->reMallocWithName("fp8_input_buffer", elems * 4, false));
        fp8_buffer2 = static_cast<fp8_e4m3_t*>(allocator_->reMallocWithName("fp8_input_buffer2", elems * 4, false));
    }
    void freeBuffer() {}

    size_t embedding_dim_;
    hipStream_t stream_;
    IAllocator* allocator_;
    bool is_free_buffer_after_forward_;
    T* hidden_buffer = nullptr;
    fp8_e4m3_t* fp8_buffer = nullptr;
    fp8_e4m3_t* fp8_buffer2 = nullptr;
};

// ---- layers/flux_single_transformer_block/FluxSingleTransformerFP8BlockWeight.cc:60-121 (proj_mlp, proj_out) ---------
template <typename T>
class FluxSingleTransformerFP8MlpWeight {
public:
    fp8_e4m3_t* proj_mlp_weight = nullptr;  // [mlp_scale*D, D]
    T* proj_mlp_bias = nullptr;
    float* proj_mlp_weight_scale = nullptr;
    float* proj_mlp_input_scale = nullptr;
    T* proj_mlp_weight_h = nullptr;
    fp8_e4m3_t* proj_out_weight = nullptr;  // [D, (mlp_scale+1)*D]
    T* proj_out_bias = nullptr;
    float* proj_out_weight_scale = nullptr;
    float* proj_out_input_scale = nullptr;
    T* proj_out_weight_h = nullptr;
    std::unordered_map<std::string, FP8LoraWeight<T>*> lora_weight_map;

    FluxSingleTransformerFP8MlpWeight(size_t embedding_dim, size_t mlp_scale, LyraQuantType quant_level, IAllocator* allocator)
        : embedding_dim_(embedding_dim), mlp_scale_(mlp_scale), allocator_(allocator) {
        (void)quant_level;
        LYRA_CHECK_WITH_INFO(allocator_ != nullptr && embedding_dim % 64 == 0 && mlp_scale > 0, "FluxSingleTransformerFP8MlpWeight: bad arguments");
    }
    FluxSingleTransformerFP8MlpWeight(const FluxSingleTransformerFP8MlpWeight&) = delete;
    FluxSingleTransformerFP8MlpWeight& operator=(const FluxSingleTransformerFP8MlpWeight&) = delete;
    virtual ~FluxSingleTransformerFP8MlpWeight() {
        if (is_maintain_buffer) {
            mlp_.release();
            out_.release();
            for (auto& kv : lora_weight_map) delete kv.second;
        }
    }
    virtual void mallocWeights() {
        if (is_maintain_buffer) return;
        mlp_.alloc(mlp_scale_ * embedding_dim_, embedding_dim_);
        out_.alloc(embedding_dim_, (mlp_scale_ + 1) * embedding_dim_);
        proj_mlp_weight = mlp_.weight; proj_mlp_bias = mlp_.bias; proj_mlp_weight_scale = mlp_.weight_scale;
        proj_mlp_input_scale = mlp_.input_scale; proj_mlp_weight_h = mlp_.weight_h;
        proj_out_weight = out_.weight; proj_out_bias = out_.bias; proj_out_weight_scale = out_.weight_scale;
        proj_out_input_scale = out_.input_scale; proj_out_weight_h = out_.weight_h;
        lora_weight_map = {{"proj_mlp", new FP8LoraWeight<T>({mlp_.d_out, mlp_.d_in}, proj_mlp_weight, proj_mlp_weight_scale, proj_mlp_weight_h)},
                           {"proj_out", new FP8LoraWeight<T>({out_.d_out, out_.d_in}, proj_out_weight, proj_out_weight_scale, proj_out_weight_h)}};
        is_maintain_buffer = true;
    }
    virtual void loadWeightsFromCache(std::string prefix, std::unordered_map<std::string, void*>& weights, hipMemcpyKind memcpyKind) {
        if (!is_maintain_buffer) mallocWeights();
        mlp_.load(prefix, "proj_mlp", weights, memcpyKind, allocator_);
        out_.load(prefix, "proj_out", weights, memcpyKind, allocator_);
    }
    // FluxSingleTransformerFP8BlockWeight.cc:99-122 (the two linears this class owns)
    virtual void loadWeights(const std::string prefix, FtCudaDataType model_file_type) {
        if (!is_maintain_buffer) mallocWeights();
        mlp_.load_bin(prefix, "proj_mlp", model_file_type, allocator_);
        out_.load_bin(prefix, "proj_out", model_file_type, allocator_);
    }
    size_t embedding_dim() const { return embedding_dim_; }
    size_t mlp_scale() const { return mlp_scale_; }

protected:
    bool is_maintain_buffer = false;

private:
    size_t embedding_dim_, mlp_scale_;
    IAllocator* allocator_;
    detail::FP8LinearStore<T> mlp_, out_;
};

// ---- layers/flux_single_transformer_block/FluxSingleTransformerFP8Block.cc:209-290 -----------------------------------
// The part of the single block's forward after the attention: inputs "input", "norm_hidden", "attn_output"
// [B, S, D] and "gate" [B, D] (chunk 2 of the block's msa buffer); output "output" [B, S, D].  The proj_mlp GEMM
// writes the e4m3 codes of gelu(mlp) into the right-hand columns of the concatenated projection input, a strided
// cast fills the attention columns, and the proj_out GEMM applies the gate and the residual in its epilogue.
template <typename T>
class FluxSingleTransformerFP8Mlp {
public:
    FluxSingleTransformerFP8Mlp(size_t embedding_dim, size_t mlp_scale, hipStream_t stream, void* /*cublas_wrapper*/,
                                IAllocator* allocator, const bool is_free_buffer_after_forward)
        : embedding_dim_(embedding_dim), mlp_scale_(mlp_scale), stream_(stream), allocator_(allocator),
          is_free_buffer_after_forward_(is_free_buffer_after_forward) {
        LYRA_CHECK_WITH_INFO(allocator_ != nullptr, "FluxSingleTransformerFP8Mlp needs an allocator");
    }
    virtual ~FluxSingleTransformerFP8Mlp() {}

    virtual void forward(const TensorMap* output_tensors, const TensorMap* input_tensors,
                         const FluxSingleTransformerFP8MlpWeight<T>* weights) {
        Tensor input_tensor = input_tensors->at("input");
        Tensor norm_tensor = input_tensors->at("norm_hidden");
        Tensor attn_tensor = input_tensors->at("attn_output");
        Tensor gate_tensor = input_tensors->at("gate");
        Tensor output_tensor = output_tensors->at("output");
        LYRA_CHECK_WITH_INFO(input_tensor.shape.size() == 3 && input_tensor.shape[2] == embedding_dim_,
                             "FluxSingleTransformerFP8Mlp: input must be [B, S, D]");
        const size_t batch_size = input_tensor.shape[0], seq_len = input_tensor.shape[1], d = embedding_dim_;
        const size_t m = batch_size * seq_len, f = mlp_scale_ * d;
        fp8_buffer1 = static_cast<fp8_e4m3_t*>(allocator_->reMallocWithName("fp8_input_buffer", m * (d + f), false));
        fp8_buffer2 = static_cast<fp8_e4m3_t*>(allocator_->reMallocWithName("fp8_input_buffer2", m * d, false));
        const lq_dtype_t dt = detail::DType<T>::value;
        uint8_t* cat = reinterpret_cast<uint8_t*>(fp8_buffer1);
        // FP8 activations as k-panels (lyraquant.h): fp8_buffer2 [D/64][M][64]; proj_out's concatenated input `cat`
        // [(D + F)/64][M][64], whose two column blocks (attention output, GELU of proj_mlp) are runs of whole panels
        detail::check(lq_fp8_scale_cast_panels(reinterpret_cast<uint8_t*>(fp8_buffer2), norm_tensor.getPtr<T>(), dt, weights->proj_mlp_input_scale,
                                               1, m, d, stream_), "FluxSingleTransformerFP8Mlp cast");
        detail::check(lq_fp8_scale_cast_panels(cat, attn_tensor.getPtr<T>(), dt, weights->proj_out_input_scale, 1, m, d, stream_),
                      "FluxSingleTransformerFP8Mlp attn cast");
        detail::check(lq_gemm_fp8_codes_panels(cat + (d / 64) * m * 64, weights->proj_out_input_scale, dt,
                                               reinterpret_cast<const uint8_t*>(fp8_buffer2),
                                               reinterpret_cast<const uint8_t*>(weights->proj_mlp_weight), weights->proj_mlp_input_scale,
                                               weights->proj_mlp_weight_scale, weights->proj_mlp_bias, /*gelu=*/2, (int)m, (int)f, (int)d, stream_),
                      "FluxSingleTransformerFP8Mlp proj_mlp");
        detail::check(lq_gemm_fp8_gated_panels(output_tensor.getPtr<T>(), dt, cat, reinterpret_cast<const uint8_t*>(weights->proj_out_weight),
                                               weights->proj_out_input_scale, weights->proj_out_weight_scale, weights->proj_out_bias,
                                               gate_tensor.getPtr<T>(), seq_len, input_tensor.getPtr<T>(), (int)m, (int)d, (int)(d + f), stream_),
                      "FluxSingleTransformerFP8Mlp proj_out");
        (void)is_free_buffer_after_forward_;
    }

protected:
    size_t embedding_dim_, mlp_scale_;
    hipStream_t stream_;
    IAllocator* allocator_;
    bool is_free_buffer_after_forward_;
    fp8_e4m3_t* fp8_buffer1 = nullptr;
    fp8_e4m3_t* fp8_buffer2 = nullptr;
};

}  // namespace lyradiff
