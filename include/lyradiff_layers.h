// lyradiff_layers.h -- header-only host-side layer types of the quantized-linear path, over the C ABI
// of lyraquant.h and the launchers of lyradiff_compat.h: the tensor plumbing (Tensor, TensorMap), the
// named scratch pool (IAllocator / Allocator) and the W4A4 linear layer with its weight container,
// with the reference's names, members and call shapes (paths relative to the reference's
// src/lyradiff/), so that reference-style layer code compiles against liblyraquant.so.
//
// Not built: file loading (loadWeights from .bin files) and the npy/torch tensor readers of Tensor.
#pragma once

#include <cstring>
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
        detail::check(lq_w4a4_quantize(quantized_input_buffer, input_scale_buffer, LQ_F32, input_tensor.getPtr<T>(),
                                       detail::DType<T>::value, weights->smooth, (int)m, (int)k, (int)group_size_, stream_),
                      "W4A4Gemm::forward quantize");
        if (low_rank)  // down projection of the unsmoothed input, written as T directly (no fp32 detour)
            detail::check(lq_lora_down(lora_down_res_buffer2, detail::DType<T>::value, input_tensor.getPtr<T>(), weights->lora_down,
                                       detail::DType<T>::value, (int)m, (int)k, (int)lora_rank_, stream_),
                          "W4A4Gemm::forward lora down");
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

}  // namespace lyradiff
