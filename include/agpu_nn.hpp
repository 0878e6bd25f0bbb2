// agpu_nn.hpp — C++17 host layer over the C ABI of libagpu_hip.so, with the names and the
// behaviour of async_gpu's `nn` module (paths relative to the reference checkout,
// crates/core/gpu-host/src/):
//   NnError            nn/error.rs:7-29
//   KernelRegistry     nn/registry.rs:26-144
//   GpuTensor          nn/tensor.rs:45-282
//   GpuArray, Residency  gpu_array.rs:42-385 (crates/core/gpu-host/src/gpu_array.rs)
//   ops::*             nn/ops/{gemm,norm,activation,reshape,attention,quantize}.rs
//   Module, Int4Linear, Linear, LayerNorm, Gelu, Embedding   nn/layers/*.rs
//   Gpt2Config, Int4Gpt2Model                                nn/models/gpt2.rs:20-93,1341-1580,712-783
// Rust's Result<T, NnError> becomes a thrown NnError.  Operators allocate and return their
// output like the reference's do; in-place ones take a non-const reference.  Header only;
// link with -lagpu_hip.
#pragma once

#include <cstdint>
#include <cstring>
#include <memory>
#include <numeric>
#include <optional>
#include <stdexcept>
#include <string>
#include <type_traits>
#include <utility>
#include <vector>

#include "agpu.h"
#include "agpu_gpt2.h"

namespace agpu {
namespace nn {

// ---- NnError (nn/error.rs:7-29) -----------------------------------------------------------
struct NnError : std::runtime_error {
    enum class Kind { ShapeMismatch, DimOutOfRange, KernelNotFound, Hip, Other };
    Kind kind;
    int32_t code;
    NnError(Kind k, int32_t c, const std::string &msg) : std::runtime_error(msg), kind(k), code(c) {}
    static NnError shape_mismatch(const std::string &expected, const std::string &actual) {
        return NnError(Kind::ShapeMismatch, AGPU_ERR_SHAPE_MISMATCH, "shape mismatch: expected " + expected + ", got " + actual);
    }
};

inline NnError::Kind kind_of(int32_t rc) {
    switch (rc) {
        case AGPU_ERR_SHAPE_MISMATCH: return NnError::Kind::ShapeMismatch;
        case AGPU_ERR_DIM_OUT_OF_RANGE: return NnError::Kind::DimOutOfRange;
        case AGPU_ERR_KERNEL_NOT_FOUND: return NnError::Kind::KernelNotFound;
        default: return rc > 0 ? NnError::Kind::Hip : NnError::Kind::Other;
    }
}

// ---- KernelRegistry (nn/registry.rs:26-144): the device handle every operator takes ---------
class KernelRegistry {
public:
    // KernelRegistry::init_default (registry.rs:131-135)
    static std::shared_ptr<KernelRegistry> init_default(int device = 0) {
        agpu_ctx *c = nullptr;
        const int32_t rc = agpu_ctx_create(device, &c);
        if (rc != AGPU_OK) throw NnError(kind_of(rc), rc, "agpu_ctx_create failed");
        return std::shared_ptr<KernelRegistry>(new KernelRegistry(c));
    }
    ~KernelRegistry() { agpu_ctx_destroy(ctx_); }
    KernelRegistry(const KernelRegistry &) = delete;
    KernelRegistry &operator=(const KernelRegistry &) = delete;

    // registry.get(name) (registry.rs:140-144): the entry point serving a reference kernel name.
    std::string get(const char *name) const {
        const char *entry = nullptr;
        check(agpu_kernel_lookup(ctx_, name, &entry));
        return entry;
    }
    agpu_ctx *device() const { return ctx_; }
    void synchronize() const { check(agpu_sync(ctx_)); }
    void check(int32_t rc) const {
        if (rc != AGPU_OK) throw NnError(kind_of(rc), rc, agpu_last_error_string(ctx_));
    }

private:
    explicit KernelRegistry(agpu_ctx *c) : ctx_(c) {}
    agpu_ctx *ctx_;
};
using Registry = std::shared_ptr<KernelRegistry>;

// ---- GpuTensor (nn/tensor.rs:45-282): dense, row-major, fp32, shared storage ----------------
class GpuTensor {
    struct Storage {
        Registry reg;
        void *ptr = nullptr;
        Storage(Registry r, size_t bytes) : reg(std::move(r)) { reg->check(agpu_malloc(reg->device(), bytes ? bytes : 4, &ptr)); }
        ~Storage() { agpu_free(reg->device(), ptr); }
    };

public:
    GpuTensor() = default;
    // alloc_zeros
    static GpuTensor zeros(const std::vector<size_t> &shape, const Registry &reg) {
        GpuTensor t;
        t.shape_ = shape;
        t.store_ = std::make_shared<Storage>(reg, t.numel() * sizeof(float));
        return t;
    }
    // GpuTensor::from_host (tensor.rs:85-106): data length must match the shape
    static GpuTensor from_host(const std::vector<float> &data, const std::vector<size_t> &shape, const Registry &reg) {
        GpuTensor t = zeros(shape, reg);
        if (data.size() != t.numel())
            throw NnError::shape_mismatch(std::to_string(t.numel()) + " elements", std::to_string(data.size()) + " elements");
        reg->check(agpu_memcpy_h2d(reg->device(), t.data(), data.data(), data.size() * sizeof(float)));
        return t;
    }
    std::vector<float> to_host() const {
        std::vector<float> out(numel());
        registry()->check(agpu_memcpy_d2h(registry()->device(), out.data(), data(), out.size() * sizeof(float)));
        return out;
    }
    // reshape shares the storage (tensor.rs:201-222)
    GpuTensor reshape(const std::vector<size_t> &shape) const {
        GpuTensor t = *this;
        t.shape_ = shape;
        if (t.numel() != numel())
            throw NnError::shape_mismatch(std::to_string(numel()) + " elements", std::to_string(t.numel()) + " elements");
        return t;
    }
    // clone_tensor: a device-to-device copy (tensor.rs:270-282)
    GpuTensor clone_tensor() const {
        GpuTensor t = zeros(shape_, registry());
        registry()->check(agpu_memcpy_d2d(registry()->device(), t.data(), data(), numel() * sizeof(float)));
        return t;
    }
    size_t ndim() const { return shape_.size(); }
    const std::vector<size_t> &shape() const { return shape_; }
    size_t dim(size_t i) const {
        if (i >= shape_.size())
            throw NnError(NnError::Kind::DimOutOfRange, AGPU_ERR_DIM_OUT_OF_RANGE,
                          "dimension " + std::to_string(i) + " out of range for tensor with " + std::to_string(shape_.size()) + " dims");
        return shape_[i];
    }
    size_t numel() const { return std::accumulate(shape_.begin(), shape_.end(), size_t(1), std::multiplies<size_t>()); }
    float *data() const { return static_cast<float *>(store_->ptr); }
    const Registry &registry() const { return store_->reg; }

private:
    std::shared_ptr<Storage> store_;
    std::vector<size_t> shape_;
};

// Device buffer of u32 (packed weights, token ids): CudaSlice<u32> in the reference.
class GpuBufferU32 {
public:
    GpuBufferU32() = default;
    GpuBufferU32(const std::vector<uint32_t> &host, const Registry &reg) : t_(GpuTensor::zeros({host.size()}, reg)), n_(host.size()) {
        reg->check(agpu_memcpy_h2d(reg->device(), t_.data(), host.data(), host.size() * sizeof(uint32_t)));
    }
    uint32_t *data() const { return reinterpret_cast<uint32_t *>(t_.data()); }
    size_t len() const { return n_; }

private:
    GpuTensor t_;
    size_t n_ = 0;
};

// ---- GpuArray (gpu_array.rs:42-385): a host vector with a device copy made on demand -----------
// Residency (gpu_array.rs:55-69).
enum class Residency {
    HostOnly,    // data on the host only; no device storage yet
    Synced,      // host and device hold the same data
    DeviceOnly,  // a kernel wrote the device copy: the host copy is stale until read() syncs it back
    HostDirty,   // the host copy was modified: the device copy is stale until ensure_device uploads it
};

// Below this size the device side is pinned host memory that kernels access in place, at or above it separate device
// memory with explicit copies (SIZE_THRESHOLD_BYTES, gpu_array.rs:45-51).
constexpr size_t kGpuArrayMappedThresholdBytes = 64 * 1024;

template <class T>
class GpuArray {
    static_assert(std::is_trivially_copyable<T>::value, "GpuArray elements are copied byte for byte");

public:
    // GpuArray::from_vec (gpu_array.rs:138-150): HostOnly, nothing allocated on the device.
    static GpuArray from_vec(std::vector<T> data) {
        GpuArray a;
        a.len_ = data.size();
        a.host_ = std::move(data);
        return a;
    }
    static GpuArray from_slice(const T *data, size_t n) { return from_vec(std::vector<T>(data, data + n)); }
    static GpuArray zeroed(size_t n) { return from_vec(std::vector<T>(n, T{})); }  // gpu_array.rs:344-351

    GpuArray() = default;
    GpuArray(GpuArray &&o) noexcept { *this = std::move(o); }
    GpuArray &operator=(GpuArray &&o) noexcept {
        if (this != &o) {
            release();
            host_ = std::move(o.host_);
            len_ = o.len_;
            residency_ = o.residency_;
            reg_ = std::move(o.reg_);
            dev_ptr_ = o.dev_ptr_;
            mapped_host_ = o.mapped_host_;
            o.dev_ptr_ = o.mapped_host_ = nullptr;
            o.len_ = 0;
            o.residency_ = Residency::HostOnly;
        }
        return *this;
    }
    GpuArray(const GpuArray &) = delete;  // the reference type is not Clone
    GpuArray &operator=(const GpuArray &) = delete;
    ~GpuArray() { release(); }

    size_t len() const { return len_; }
    bool is_empty() const { return len_ == 0; }
    Residency residency() const { return residency_; }
    bool should_use_mapped() const { return len_ * sizeof(T) < kGpuArrayMappedThresholdBytes; }  // gpu_array.rs:174-176
    bool is_mapped() const { return mapped_host_ != nullptr; }

    // Deref (gpu_array.rs:353-370): the host data, synced back from the device first if a kernel wrote it.
    const std::vector<T> &read() const {
        if (residency_ == Residency::DeviceOnly) sync_to_host();
        return host_;
    }
    const T &operator[](size_t i) const { return read()[i]; }
    // The elements as DerefMut hands them out (gpu_array.rs:372-385): &mut [T], a view of fixed length.  The array's
    // size and its device allocation belong together, so the host data cannot be resized through it.
    class Slice {
      public:
        Slice(T *p, size_t n) : p_(p), n_(n) {}
        T &operator[](size_t i) const { return p_[i]; }
        T *data() const { return p_; }
        size_t size() const { return n_; }
        T *begin() const { return p_; }
        T *end() const { return p_ + n_; }

      private:
        T *p_;
        size_t n_;
    };
    // DerefMut: as read(), then the host copy is the newer one.
    Slice write() {
        if (residency_ == Residency::DeviceOnly) sync_to_host();
        residency_ = Residency::HostDirty;
        return Slice(host_.data(), host_.size());
    }

    // mark_device_dirty (gpu_array.rs:227-240): a kernel wrote the device copy.
    void mark_device_dirty() const {
        if (residency_ == Residency::Synced) residency_ = Residency::DeviceOnly;
    }

    // ensure_device (gpu_array.rs:241-340): the device address of the data, uploaded if the host copy is newer.
    // HostOnly: allocates (mapped below the threshold) and uploads -> Synced.  HostDirty: uploads -> Synced.
    // Synced / DeviceOnly: nothing to do.  An empty array has no storage and the address 0.
    uint64_t ensure_device(const Registry &reg) const {
        switch (residency_) {
            case Residency::HostOnly: {
                if (len_ == 0) {
                    residency_ = Residency::Synced;
                    return 0;
                }
                const size_t bytes = len_ * sizeof(T);
                reg_ = reg;
                if (should_use_mapped()) {
                    reg->check(agpu_host_alloc_mapped(reg->device(), bytes, &mapped_host_, &dev_ptr_));
                    std::memcpy(mapped_host_, host_.data(), bytes);
                } else {
                    reg->check(agpu_malloc(reg->device(), bytes, &dev_ptr_));
                    reg->check(agpu_memcpy_h2d(reg->device(), dev_ptr_, host_.data(), bytes));
                }
                residency_ = Residency::Synced;
                return (uint64_t)(uintptr_t)dev_ptr_;
            }
            case Residency::HostDirty: {
                if (len_ == 0 || !dev_ptr_) {  // modified before the first upload: nothing on the device yet
                    residency_ = Residency::HostOnly;
                    return ensure_device(reg);
                }
                const size_t bytes = len_ * sizeof(T);
                if (mapped_host_) {
                    reg_->check(agpu_sync(reg_->device()));  // no kernel may still be reading the old contents
                    std::memcpy(mapped_host_, host_.data(), bytes);
                } else {
                    reg_->check(agpu_memcpy_h2d(reg_->device(), dev_ptr_, host_.data(), bytes));
                }
                residency_ = Residency::Synced;
                return (uint64_t)(uintptr_t)dev_ptr_;
            }
            default: return (uint64_t)(uintptr_t)dev_ptr_;
        }
    }
    // The typed device pointer for the C ABI (after ensure_device).
    T *device_ptr(const Registry &reg) const { return reinterpret_cast<T *>((uintptr_t)ensure_device(reg)); }

private:
    void sync_to_host() const {  // gpu_array.rs:178-218
        if (len_ != 0 && dev_ptr_) {
            const size_t bytes = len_ * sizeof(T);
            if (mapped_host_) {
                reg_->check(agpu_sync(reg_->device()));  // the kernel that wrote the memory has finished
                std::memcpy(host_.data(), mapped_host_, bytes);
            } else {
                reg_->check(agpu_memcpy_d2h(reg_->device(), host_.data(), dev_ptr_, bytes));
            }
        }
        residency_ = Residency::Synced;
    }
    void release() {
        if (reg_) {
            if (mapped_host_) agpu_host_free_mapped(reg_->device(), mapped_host_);
            else if (dev_ptr_) agpu_free(reg_->device(), dev_ptr_);
        }
        dev_ptr_ = mapped_host_ = nullptr;
    }

    mutable std::vector<T> host_;
    size_t len_ = 0;
    mutable Residency residency_ = Residency::HostOnly;
    mutable Registry reg_;
    mutable void *dev_ptr_ = nullptr;      // device address of the data (either backend)
    mutable void *mapped_host_ = nullptr;  // host address of the pinned mapped backend, else null
};

// ---- ops (nn/ops/*.rs) ------------------------------------------------------------------------
namespace ops {

namespace quantize {
// quantize_weight_int4 (nn/ops/quantize.rs:102-153) on the host: weight_t [K,N] -> (packed, scales)
inline std::pair<std::vector<uint32_t>, std::vector<float>> quantize_weight_int4(const std::vector<float> &weight_t, size_t k,
                                                                                   size_t n, size_t group_size,
                                                                                   int mode = AGPU_QUANT_RUST) {
    if (weight_t.size() != k * n) throw NnError::shape_mismatch("weight_t of [K, N]", std::to_string(weight_t.size()) + " elements");
    if (k % 8 != 0) throw NnError::shape_mismatch("K divisible by 8", "K = " + std::to_string(k));
    std::vector<uint32_t> packed(k / 8 * n);
    std::vector<float> scales((k + group_size - 1) / group_size * n);
    const int32_t rc = agpu_int4_quantize_host(weight_t.data(), packed.data(), scales.data(), (int32_t)k, (int32_t)n,
                                               (int32_t)group_size, mode);
    if (rc != AGPU_OK) throw NnError(kind_of(rc), rc, "quantize_weight_int4 failed");
    return {std::move(packed), std::move(scales)};
}
// unpack_int4 (quantize.rs:158-162)
inline int8_t unpack_int4(uint32_t packed, size_t index) { return (int8_t)((packed >> (index * 4)) & 0xF) - 8; }
}  // namespace quantize

inline size_t rows_of(const GpuTensor &t) { return t.ndim() ? t.numel() / t.shape().back() : 0; }

// ops::layer_norm (norm.rs:14-81)
inline GpuTensor layer_norm(const GpuTensor &x, const GpuTensor &gamma, const GpuTensor &beta, float eps, const Registry &reg) {
    const size_t d = x.shape().back();
    if (gamma.numel() != d || beta.numel() != d)
        throw NnError::shape_mismatch("gamma/beta of " + std::to_string(d), std::to_string(gamma.numel()) + "/" + std::to_string(beta.numel()));
    GpuTensor y = GpuTensor::zeros(x.shape(), reg);
    reg->check(agpu_layer_norm(reg->device(), x.data(), gamma.data(), beta.data(), y.data(), (int32_t)rows_of(x), (int32_t)d, eps));
    return y;
}
// ops::layer_norm_residual_dual (norm.rs:248-400): returns (a + b, LN(a + b))
inline std::pair<GpuTensor, GpuTensor> layer_norm_residual_dual(const GpuTensor &a, const GpuTensor &b, const GpuTensor &gamma,
                                                                 const GpuTensor &beta, float eps, const Registry &reg) {
    if (a.shape() != b.shape()) throw NnError::shape_mismatch("equal shapes", "different shapes");
    const size_t d = a.shape().back();
    GpuTensor s = GpuTensor::zeros(a.shape(), reg), n = GpuTensor::zeros(a.shape(), reg);
    reg->check(agpu_add_layer_norm_dual(reg->device(), a.data(), b.data(), gamma.data(), beta.data(), s.data(), n.data(),
                                        (int32_t)rows_of(a), (int32_t)d, eps));
    return {s, n};
}
// ops::gelu (activation.rs:14-16,79-108); the reference launches the quick form, its CPU references use tanh
inline GpuTensor gelu(const GpuTensor &x, const Registry &reg, int mode = AGPU_GELU_TANH) {
    GpuTensor y = GpuTensor::zeros(x.shape(), reg);
    reg->check(agpu_gelu(reg->device(), x.data(), y.data(), x.numel(), mode));
    return y;
}
// ops::elementwise_add (reshape.rs:161-186): a += b
inline void elementwise_add(GpuTensor &a, const GpuTensor &b, const Registry &reg) {
    if (a.numel() != b.numel()) throw NnError::shape_mismatch(std::to_string(a.numel()) + " elements", std::to_string(b.numel()) + " elements");
    reg->check(agpu_add_inplace(reg->device(), a.data(), b.data(), a.numel()));
}
// ops::bias_add (reshape.rs:112-136)
inline void bias_add(GpuTensor &data, const GpuTensor &bias, const Registry &reg) {
    const size_t n = data.shape().back();
    if (bias.numel() != n) throw NnError::shape_mismatch("bias of " + std::to_string(n), std::to_string(bias.numel()));
    reg->check(agpu_bias_add(reg->device(), data.data(), bias.data(), (int32_t)rows_of(data), (int32_t)n));
}
inline GpuTensor softmax(const GpuTensor &x, const Registry &reg) {
    GpuTensor y = GpuTensor::zeros(x.shape(), reg);
    reg->check(agpu_softmax_rows(reg->device(), x.data(), y.data(), (int32_t)rows_of(x), (int32_t)x.shape().back()));
    return y;
}
// ops::embedding_lookup (reshape.rs:301-335) with forward_tokens_with_offset's position offset
inline GpuTensor embedding_lookup(const GpuBufferU32 &tokens, size_t seq_len, const GpuTensor &wte, const GpuTensor &wpe,
                                  size_t pos_offset, const Registry &reg) {
    const size_t d = wte.dim(1);
    if (seq_len + pos_offset > wpe.dim(0))
        throw NnError(NnError::Kind::DimOutOfRange, AGPU_ERR_DIM_OUT_OF_RANGE, "position beyond n_positions");
    GpuTensor out = GpuTensor::zeros({seq_len, d}, reg);
    reg->check(agpu_embedding(reg->device(), tokens.data(), wte.data(), wpe.data(), out.data(), (int32_t)seq_len, (int32_t)d,
                              (int32_t)pos_offset));
    return out;
}
// ops::split_qkv (attention.rs:105-142): [seq, 3d] -> (Q, K, V) each [H*seq, dh]
inline std::tuple<GpuTensor, GpuTensor, GpuTensor> split_qkv(const GpuTensor &qkv, size_t seq_len, size_t n_heads, size_t d_head,
                                                             const Registry &reg) {
    if (qkv.numel() != seq_len * 3 * n_heads * d_head)
        throw NnError::shape_mismatch("[seq, 3*d_model]", std::to_string(qkv.numel()) + " elements");
    GpuTensor q = GpuTensor::zeros({n_heads * seq_len, d_head}, reg), k = GpuTensor::zeros({n_heads * seq_len, d_head}, reg),
              v = GpuTensor::zeros({n_heads * seq_len, d_head}, reg);
    reg->check(agpu_split_qkv(reg->device(), qkv.data(), q.data(), k.data(), v.data(), (int32_t)seq_len, (int32_t)n_heads, (int32_t)d_head));
    return {q, k, v};
}
// ops::concat_heads (attention.rs:515-549): [H*seq, dh] -> [seq, d]
inline GpuTensor concat_heads(const GpuTensor &x, size_t seq_len, size_t n_heads, size_t d_head, const Registry &reg) {
    GpuTensor out = GpuTensor::zeros({seq_len, n_heads * d_head}, reg);
    reg->check(agpu_concat_heads(reg->device(), x.data(), out.data(), (int32_t)seq_len, (int32_t)n_heads, (int32_t)d_head));
    return out;
}
// ops::multi_head_flash_attention (attention.rs:151-202): causal, all heads in one launch
inline GpuTensor multi_head_flash_attention(const GpuTensor &q, const GpuTensor &k, const GpuTensor &v, size_t seq_len,
                                            size_t n_heads, size_t d_head, bool causal, const Registry &reg) {
    GpuTensor o = GpuTensor::zeros({n_heads * seq_len, d_head}, reg);
    reg->check(agpu_attention(reg->device(), q.data(), k.data(), v.data(), o.data(), (int32_t)n_heads, (int32_t)seq_len, (int32_t)seq_len, 0,
                              (int32_t)seq_len, (int32_t)d_head, causal ? 1 : 0));
    return o;
}
// ops::scaled_dot_product_attention_kv (attention.rs:557-606): one head, q_len new rows against kv_len keys
inline GpuTensor scaled_dot_product_attention_kv(const GpuTensor &q, const GpuTensor &k, const GpuTensor &v, size_t q_len,
                                                 size_t kv_len, size_t q_offset, size_t kv_stride, size_t d_head,
                                                 const Registry &reg) {
    GpuTensor o = GpuTensor::zeros({q_len, d_head}, reg);
    reg->check(agpu_attention(reg->device(), q.data(), k.data(), v.data(), o.data(), 1, (int32_t)q_len, (int32_t)kv_len, (int32_t)q_offset,
                              (int32_t)kv_stride, (int32_t)d_head, 1));
    return o;
}
// ops::matmul (gemm.rs:20-212): C[M,N] = A[M,K] B[K,N]
inline GpuTensor matmul(const GpuTensor &a, const GpuTensor &b, const Registry &reg) {
    if (a.ndim() != 2 || b.ndim() != 2 || a.dim(1) != b.dim(0))
        throw NnError::shape_mismatch("A [M,K] and B [K,N]", "inner dims " + std::to_string(a.shape().back()) + " vs " + std::to_string(b.dim(0)));
    GpuTensor c = GpuTensor::zeros({a.dim(0), b.dim(1)}, reg);
    reg->check(agpu_gemm_f32(reg->device(), a.data(), b.data(), c.data(), (int32_t)a.dim(0), (int32_t)b.dim(1), (int32_t)a.dim(1)));
    return c;
}
// ops::int4_matmul (gemm.rs:1186-1266): quantizes B (group 128) on the fly, then the int4 kernel
inline GpuTensor int4_matmul(const GpuTensor &a, const GpuTensor &b, const Registry &reg, size_t group_size = 128) {
    if (a.ndim() != 2 || b.ndim() != 2 || a.dim(1) != b.dim(0))
        throw NnError::shape_mismatch("A [M,K] and B [K,N]", "inner dims differ");
    const size_t k = b.dim(0), n = b.dim(1);
    if (k % 8 != 0) throw NnError::shape_mismatch("K divisible by 8", "K = " + std::to_string(k));
    GpuTensor packed = GpuTensor::zeros({k / 8, n}, reg), scales = GpuTensor::zeros({(k + group_size - 1) / group_size, n}, reg);
    reg->check(agpu_int4_quantize(reg->device(), b.data(), reinterpret_cast<uint32_t *>(packed.data()), scales.data(), (int32_t)k,
                                  (int32_t)n, (int32_t)group_size, AGPU_QUANT_RUST));
    GpuTensor c = GpuTensor::zeros({a.dim(0), n}, reg);
    reg->check(agpu_int4_linear(reg->device(), a.data(), reinterpret_cast<uint32_t *>(packed.data()), scales.data(), nullptr, nullptr,
                                c.data(), (int32_t)a.dim(0), (int32_t)n, (int32_t)k, (int32_t)group_size, 0));
    return c;
}
inline std::vector<uint32_t> argmax_rows(const GpuTensor &x, const Registry &reg, bool last_index = false) {
    const size_t rows = rows_of(x);
    GpuTensor idx = GpuTensor::zeros({rows}, reg);
    reg->check(agpu_argmax_rows(reg->device(), x.data(), reinterpret_cast<uint32_t *>(idx.data()), (int32_t)rows, (int32_t)x.shape().back(),
                                last_index ? 1 : 0));
    std::vector<uint32_t> out(rows);
    reg->check(agpu_memcpy_d2h(reg->device(), out.data(), idx.data(), rows * sizeof(uint32_t)));
    return out;
}
}  // namespace ops

// SimpleRng (nn/models/gpt2.rs:1000-1023)
class SimpleRng {
public:
    explicit SimpleRng(uint64_t seed) : s_(agpu_simple_rng_new(seed)) {}
    float next_f32() { return agpu_simple_rng_next_f32(&s_); }
    uint64_t *state() { return &s_; }

private:
    uint64_t s_;
};

// top_k_sample (gpt2.rs:1029-1058) on a device logit vector
inline uint32_t top_k_sample(const GpuTensor &logits, size_t k, float temperature, SimpleRng &rng, const Registry &reg) {
    uint32_t tok = 0;
    reg->check(agpu_top_k_sample(reg->device(), logits.data(), (int32_t)logits.numel(), (int32_t)k, temperature, rng.state(), &tok));
    return tok;
}

// ---- layers (nn/layers/*.rs) --------------------------------------------------------------------
struct Module {  // trait Module (layers/mod.rs:36-39)
    virtual ~Module() = default;
    virtual GpuTensor forward(const GpuTensor &input) const = 0;
};

// Int4Linear (layers/int4_linear.rs:18-147)
class Int4Linear : public Module {
public:
    Int4Linear(const std::vector<uint32_t> &packed, const std::vector<float> &scales, const std::optional<std::vector<float>> &bias,
               size_t in_features, size_t out_features, size_t group_size, const Registry &reg)
        : packed_(packed, reg), scales_(GpuTensor::from_host(scales, {scales.size()}, reg)), in_(in_features), out_(out_features),
          group_(group_size), reg_(reg) {
        if (bias) bias_ = GpuTensor::from_host(*bias, {out_features}, reg);
    }
    GpuTensor forward(const GpuTensor &input) const override {
        const size_t ndim = input.ndim();
        const size_t k = ndim ? input.shape().back() : 0;
        if (k != in_) throw NnError::shape_mismatch("last dim = " + std::to_string(in_), "last dim = " + std::to_string(k));
        size_t m = 1;
        for (size_t i = 0; i + 1 < ndim; ++i) m *= input.shape()[i];
        GpuTensor y = GpuTensor::zeros({m, out_}, reg_);
        reg_->check(agpu_int4_linear(reg_->device(), input.data(), packed_.data(), scales_.data(), bias_ ? bias_->data() : nullptr, nullptr,
                                     y.data(), (int32_t)m, (int32_t)out_, (int32_t)in_, (int32_t)group_, 0));
        if (ndim > 2) {
            std::vector<size_t> shape(input.shape().begin(), input.shape().end() - 1);
            shape.push_back(out_);
            return y.reshape(shape);
        }
        return y;
    }
    // memory_bytes (int4_linear.rs:136-146)
    size_t memory_bytes() const {
        return in_ / 8 * out_ * 4 + (in_ + group_ - 1) / group_ * out_ * 4 + (bias_ ? out_ * 4 : 0);
    }

private:
    GpuBufferU32 packed_;
    GpuTensor scales_;
    std::optional<GpuTensor> bias_;
    size_t in_, out_, group_;
    Registry reg_;
};

// Linear (layers/linear.rs:46-88): takes [out, in] like the reference, keeps [in, out] on the device
class Linear : public Module {
public:
    Linear(const std::vector<float> &weight, const std::optional<std::vector<float>> &bias, size_t in_features, size_t out_features,
           const Registry &reg)
        : in_(in_features), out_(out_features), reg_(reg) {
        if (weight.size() != in_features * out_features)
            throw NnError::shape_mismatch("weight of [out, in]", std::to_string(weight.size()) + " elements");
        std::vector<float> wt(weight.size());
        for (size_t o = 0; o < out_features; ++o)
            for (size_t i = 0; i < in_features; ++i) wt[i * out_features + o] = weight[o * in_features + i];
        weight_t_ = GpuTensor::from_host(wt, {in_features, out_features}, reg);
        if (bias) bias_ = GpuTensor::from_host(*bias, {out_features}, reg);
    }
    GpuTensor forward(const GpuTensor &input) const override {
        const size_t k = input.shape().back();
        if (k != in_) throw NnError::shape_mismatch("last dim = " + std::to_string(in_), "last dim = " + std::to_string(k));
        GpuTensor y = ops::matmul(input.reshape({input.numel() / k, k}), weight_t_, reg_);
        if (bias_) ops::bias_add(y, *bias_, reg_);
        return y;
    }

private:
    GpuTensor weight_t_;
    std::optional<GpuTensor> bias_;
    size_t in_, out_;
    Registry reg_;
};

// LayerNorm (layers/norm.rs:15-55)
class LayerNorm : public Module {
public:
    LayerNorm(const std::vector<float> &gamma, const std::vector<float> &beta, float eps, const Registry &reg)
        : gamma_(GpuTensor::from_host(gamma, {gamma.size()}, reg)), beta_(GpuTensor::from_host(beta, {beta.size()}, reg)), eps_(eps), reg_(reg) {}
    GpuTensor forward(const GpuTensor &input) const override { return ops::layer_norm(input, gamma_, beta_, eps_, reg_); }

private:
    GpuTensor gamma_, beta_;
    float eps_;
    Registry reg_;
};

struct Gelu : Module {  // layers/activation.rs
    Registry reg;
    int mode;
    explicit Gelu(const Registry &r, int m = AGPU_GELU_TANH) : reg(r), mode(m) {}
    GpuTensor forward(const GpuTensor &input) const override { return ops::gelu(input, reg, mode); }
};

// Embedding (layers/embedding.rs:14-93)
class Embedding {
public:
    Embedding(const std::vector<float> &wte, const std::vector<float> &wpe, size_t vocab, size_t n_positions, size_t d, const Registry &reg)
        : wte_(GpuTensor::from_host(wte, {vocab, d}, reg)), wpe_(GpuTensor::from_host(wpe, {n_positions, d}, reg)), reg_(reg) {}
    GpuTensor forward_tokens(const GpuBufferU32 &ids, size_t seq_len) const { return ops::embedding_lookup(ids, seq_len, wte_, wpe_, 0, reg_); }
    GpuTensor forward_tokens_with_offset(const GpuBufferU32 &ids, size_t seq_len, size_t pos_offset) const {
        return ops::embedding_lookup(ids, seq_len, wte_, wpe_, pos_offset, reg_);
    }

private:
    GpuTensor wte_, wpe_;
    Registry reg_;
};

// ---- models (nn/models/gpt2.rs) -------------------------------------------------------------------
struct Gpt2Config {  // gpt2.rs:20-93
    size_t n_layer, n_embd, n_head, vocab_size = 50257, n_positions = 1024;
    float layer_norm_epsilon = 1e-5f;
    static Gpt2Config small() { return {12, 768, 12}; }
    static Gpt2Config medium() { return {24, 1024, 16}; }
    static Gpt2Config large() { return {36, 1280, 20}; }
    static Gpt2Config xl() { return {48, 1600, 25}; }
    size_t head_dim() const { return n_embd / n_head; }
    size_t ffn_dim() const { return 4 * n_embd; }
};

// One transformer layer of fp32 weights in the checkpoint's Conv1D [in, out] layout (model.rs:119-155)
struct Gpt2LayerWeights {
    std::vector<float> ln_1_weight, ln_1_bias, c_attn_weight, c_attn_bias, c_proj_weight, c_proj_bias, ln_2_weight, ln_2_bias,
        mlp_fc_weight, mlp_fc_bias, mlp_proj_weight, mlp_proj_bias;
};
struct Gpt2Weights {
    std::vector<float> wte, wpe, ln_f_weight, ln_f_bias;
    std::vector<Gpt2LayerWeights> layers;
};

// Int4Gpt2Model (gpt2.rs:1341-1580) with the cached control flow of gpt2.rs:712-783; the KV cache lives
// on the device inside the model handle (KvCache, gpt2.rs:1064-1117).
class Int4Gpt2Model {
public:
    static constexpr size_t DEFAULT_GROUP_SIZE = 128;  // gpt2.rs:1358

    // from_weights (gpt2.rs:1362-1433): quantizes every dense layer with quantize_weight_int4.
    // lm_head: AGPU_LM_HEAD_F32 reproduces the reference model, AGPU_LM_HEAD_INT4 ties an int4 head.
    static Int4Gpt2Model from_weights(const Gpt2Weights &w, const Gpt2Config &config, size_t group_size, const Registry &reg,
                                      int lm_head = AGPU_LM_HEAD_F32, int quant_mode = AGPU_QUANT_RUST, size_t max_batch = 1) {
        Int4Gpt2Model m(config, group_size, reg, lm_head, max_batch);
        if (w.layers.size() != config.n_layer) throw NnError::shape_mismatch(std::to_string(config.n_layer) + " layers", std::to_string(w.layers.size()));
        reg->check(agpu_gpt2_set_embeddings(m.h_, w.wte.data(), w.wpe.data(), w.ln_f_weight.data(), w.ln_f_bias.data(), 0));
        const int d = (int)config.n_embd, ff = (int)config.ffn_dim();
        for (size_t l = 0; l < w.layers.size(); ++l) {
            const Gpt2LayerWeights &L = w.layers[l];
            reg->check(agpu_gpt2_set_layer_norms(m.h_, (int)l, L.ln_1_weight.data(), L.ln_1_bias.data(), L.ln_2_weight.data(), L.ln_2_bias.data(), 0));
            reg->check(agpu_gpt2_quantize_linear(m.h_, (int)l, AGPU_LINEAR_QKV, L.c_attn_weight.data(), L.c_attn_bias.data(), d, 3 * d, quant_mode, 0));
            reg->check(agpu_gpt2_quantize_linear(m.h_, (int)l, AGPU_LINEAR_PROJ, L.c_proj_weight.data(), L.c_proj_bias.data(), d, d, quant_mode, 0));
            reg->check(agpu_gpt2_quantize_linear(m.h_, (int)l, AGPU_LINEAR_FC, L.mlp_fc_weight.data(), L.mlp_fc_bias.data(), d, ff, quant_mode, 0));
            reg->check(agpu_gpt2_quantize_linear(m.h_, (int)l, AGPU_LINEAR_FC_PROJ, L.mlp_proj_weight.data(), L.mlp_proj_bias.data(), ff, d, quant_mode, 0));
        }
        if (lm_head == AGPU_LM_HEAD_INT4) {
            std::vector<float> wte_t(w.wte.size());
            for (size_t v = 0; v < config.vocab_size; ++v)
                for (size_t j = 0; j < config.n_embd; ++j) wte_t[j * config.vocab_size + v] = w.wte[v * config.n_embd + j];
            reg->check(agpu_gpt2_quantize_linear(m.h_, -1, 0, wte_t.data(), nullptr, d, (int)config.vocab_size, quant_mode, 0));
        }
        return m;
    }
    Int4Gpt2Model(Int4Gpt2Model &&o) noexcept : config_(o.config_), group_(o.group_), reg_(std::move(o.reg_)), h_(o.h_) { o.h_ = nullptr; }
    Int4Gpt2Model(const Int4Gpt2Model &) = delete;
    ~Int4Gpt2Model() {
        if (h_) agpu_gpt2_destroy(h_);
    }

    // forward (gpt2.rs:1522-1533): logits [seq_len, vocab_size], no cache kept from earlier calls
    GpuTensor forward(const GpuBufferU32 &token_ids, size_t seq_len) const {
        reg_->check(agpu_gpt2_reset_cache(h_));
        return forward_cached(token_ids, seq_len);
    }
    // forward_cached (gpt2.rs:712-734): logits [new_len, vocab_size]; the cache grows by new_len
    GpuTensor forward_cached(const GpuBufferU32 &token_ids, size_t new_len) const {
        GpuTensor logits = GpuTensor::zeros({new_len, config_.vocab_size}, reg_);
        reg_->check(agpu_gpt2_forward_cached(h_, token_ids.data(), 1, (int32_t)new_len, logits.data(), 1));
        return logits;
    }
    // forward_profiled (gpt2.rs:529-568): logits [1, vocab_size] of the last position and (stage, milliseconds) per stage
    std::pair<GpuTensor, std::vector<std::pair<std::string, double>>> forward_profiled(const GpuBufferU32 &token_ids, size_t seq_len) const {
        GpuTensor logits = GpuTensor::zeros({1, config_.vocab_size}, reg_);
        std::vector<agpu_gpt2_stage_report> rep(config_.n_layer + 3);
        int32_t n = 0;
        reg_->check(agpu_gpt2_forward_profiled(h_, token_ids.data(), (int32_t)seq_len, logits.data(), rep.data(), (int32_t)rep.size(), &n));
        std::vector<std::pair<std::string, double>> timings;
        for (int32_t i = 0; i < n; ++i) timings.emplace_back(rep[(size_t)i].name, (double)rep[(size_t)i].ms);
        return {std::move(logits), std::move(timings)};
    }
    // forward_diagnostic (gpt2.rs:595-667): the forward with the reference's [diag] lines on stderr; logits [1, vocab_size]
    GpuTensor forward_diagnostic(const GpuBufferU32 &token_ids, size_t seq_len) const {
        GpuTensor logits = GpuTensor::zeros({1, config_.vocab_size}, reg_);
        std::vector<agpu_gpt2_stage_report> rep(config_.n_layer + 3);
        int32_t n = 0;
        uint32_t top_tok[5];
        float top_val[5];
        reg_->check(agpu_gpt2_forward_diagnostic(h_, token_ids.data(), (int32_t)seq_len, logits.data(), rep.data(), (int32_t)rep.size(), &n,
                                                 top_tok, top_val));
        const size_t last = seq_len - 1;
        auto four = [](const float *a) {
            char b[96];
            std::snprintf(b, sizeof(b), "[%.6f, %.6f, %.6f, %.6f]", a[0], a[1], a[2], a[3]);
            return std::string(b);
        };
        for (int32_t i = 0; i < n; ++i) {
            const agpu_gpt2_stage_report &r = rep[(size_t)i];
            const std::string name = r.name;
            if (name == "embedding") {
                std::fprintf(stderr, "[diag] Embedding pos0 first4: %s\n", four(r.pos0_first4).c_str());
                std::fprintf(stderr, "[diag] Embedding pos%zu first4: %s\n", last, four(r.last_first4).c_str());
            } else if (name == "block_0" || name == "block_" + std::to_string(config_.n_layer - 1)) {
                std::fprintf(stderr, "[diag] Layer %s pos%zu first4: %s\n", name.c_str() + 6, last, four(r.last_first4).c_str());
                if (r.non_finite) std::fprintf(stderr, "[diag] WARNING: Layer %s has %d NaN/Inf values!\n", name.c_str() + 6, r.non_finite);
            } else if (name == "ln_f") {
                std::fprintf(stderr, "[diag] Final LN pos%zu first4: %s\n", last, four(r.last_first4).c_str());
            }
        }
        std::fprintf(stderr, "[diag] Top-5 tokens at pos%zu:\n", last);
        for (int i = 0; i < 5; ++i) std::fprintf(stderr, "  token %u: %.4f\n", top_tok[i], top_val[i]);
        return logits;
    }
    size_t cache_len() const { return (size_t)agpu_gpt2_cache_len(h_); }
    void reset_cache() const { reg_->check(agpu_gpt2_reset_cache(h_)); }
    // generate (gpt2.rs:1536-1560)
    std::vector<uint32_t> generate(const std::vector<uint32_t> &prompt, size_t max_new_tokens, int eos = 50256) const {
        std::vector<uint32_t> out(prompt.size() + max_new_tokens);
        int32_t len = 0;
        reg_->check(agpu_gpt2_generate(h_, prompt.data(), (int32_t)prompt.size(), (int32_t)max_new_tokens, eos, out.data(), &len));
        out.resize((size_t)len);
        return out;
    }
    // generate_cached (gpt2.rs:740-783)
    std::vector<uint32_t> generate_cached(const std::vector<uint32_t> &prompt, size_t max_new_tokens, int eos = 50256) const {
        std::vector<uint32_t> out(prompt.size() + max_new_tokens);
        int32_t len = 0;
        reg_->check(agpu_gpt2_generate_cached(h_, prompt.data(), 1, (int32_t)prompt.size(), (int32_t)max_new_tokens, eos, out.data(), &len, nullptr));
        out.resize((size_t)len);
        return out;
    }
    // generate_cached_sampling (gpt2.rs:931-977)
    std::vector<uint32_t> generate_cached_sampling(const std::vector<uint32_t> &prompt, size_t max_new_tokens, size_t top_k,
                                                   float temperature, SimpleRng &rng, int eos = 50256) const {
        std::vector<uint32_t> out(prompt.size() + max_new_tokens);
        int32_t len = 0;
        reg_->check(agpu_gpt2_generate_cached_sampling(h_, prompt.data(), (int32_t)prompt.size(), (int32_t)max_new_tokens, (int32_t)top_k,
                                                       temperature, rng.state(), eos, out.data(), &len));
        out.resize((size_t)len);
        return out;
    }
    // generate_cached_early_exit (gpt2.rs:837-922) -> (tokens, blocks used per step)
    std::pair<std::vector<uint32_t>, std::vector<size_t>> generate_cached_early_exit(const std::vector<uint32_t> &prompt,
                                                                                     size_t max_new_tokens, float threshold,
                                                                                     int eos = 50256) const {
        const size_t rows = max_new_tokens > 0 ? max_new_tokens : 1;
        std::vector<uint32_t> out(prompt.size() + rows);
        std::vector<int32_t> layers(rows);
        int32_t len = 0, steps = 0;
        reg_->check(agpu_gpt2_generate_cached_early_exit(h_, prompt.data(), (int32_t)prompt.size(), (int32_t)max_new_tokens, threshold,
                                                         eos, out.data(), &len, layers.data(), &steps));
        out.resize((size_t)len);
        return {out, std::vector<size_t>(layers.begin(), layers.begin() + steps)};
    }
    // forward_early_exit (gpt2.rs:797-830) -> (logits [seq, vocab], layers used); tokens on the host
    std::pair<GpuTensor, size_t> forward_early_exit(const std::vector<uint32_t> &tokens, float threshold) const {
        void *ids = nullptr;
        reg_->check(agpu_malloc(reg_->device(), tokens.size() * 4, &ids));
        GpuTensor logits = GpuTensor::zeros({tokens.size(), config_.vocab_size}, reg_);
        int32_t used = 0;
        int32_t rc = agpu_memcpy_h2d(reg_->device(), ids, tokens.data(), tokens.size() * 4);
        if (rc == AGPU_OK)
            rc = agpu_gpt2_forward_early_exit(h_, (const uint32_t *)ids, (int32_t)tokens.size(), threshold, logits.data(), &used);
        (void)agpu_free(reg_->device(), ids);
        reg_->check(rc);
        return {logits, (size_t)used};
    }
    // quantized_memory_bytes (gpt2.rs:1565-1577)
    size_t quantized_memory_bytes() const { return (size_t)agpu_gpt2_quantized_memory_bytes(h_); }
    const Gpt2Config &config() const { return config_; }

private:
    Int4Gpt2Model(const Gpt2Config &c, size_t group, const Registry &reg, int lm_head, size_t max_batch) : config_(c), group_(group), reg_(reg) {
        agpu_gpt2_config cc{};
        cc.n_layer = (int)c.n_layer; cc.n_embd = (int)c.n_embd; cc.n_head = (int)c.n_head; cc.vocab_size = (int)c.vocab_size;
        cc.n_positions = (int)c.n_positions; cc.layer_norm_epsilon = c.layer_norm_epsilon; cc.group_size = (int)group;
        cc.max_batch = (int)max_batch; cc.lm_head = lm_head; cc.gelu = AGPU_GELU_TANH; cc.argmax_last = 0;
        reg->check(agpu_gpt2_create(reg->device(), &cc, &h_));
    }
    Gpt2Config config_;
    size_t group_;
    Registry reg_;
    agpu_gpt2 *h_ = nullptr;
};

}  // namespace nn
}  // namespace agpu
