// C++ mirror of the reference's operator surface for the attention path, implemented on the C ABI
// of libvsp_attn.so (include/vsp_attn.h).  Same names, argument meaning and exception types/messages
// as the reference, so that code written against
//   vesper::ops::flash_attention / flash_attention_hip_dispatch   include/vesper/ops/flash_attention.h:34-41,74-78
//   vesper::ops::repeat_kv                                         include/vesper/ops/attention_ops.h:24
//   vesper::nn::functional::scaled_dot_product_attention           include/vesper/nn/functional.h:132-136
//   vesper::nn::KVCache / GQAKVCache                               include/vesper/nn/transformer.h:21-39,
//                                                                  include/vesper/nn/gqa_attention.h:110-163
//   the attention core of GroupedQueryAttention / MultiHeadAttention::forward(x, cache, start_pos)
//                                                                  src/nn/gqa_attention.cpp:128-148, src/nn/transformer.cpp:190-205
// reads the same here.  The Tensor below is the small part of vesper::Tensor those interfaces need
// (a strided view over shared device storage); a maintainer wiring the library into the reference
// itself would instead fill vsp_tensor from vesper::Tensor directly.
// Header-only; link with libvsp_attn.so and the HIP runtime.
#pragma once

#include <hip/hip_runtime.h>

#include <algorithm>
#include <cmath>
#include <cstdint>
#include <map>
#include <memory>
#include <mutex>
#include <stdexcept>
#include <string>
#include <tuple>
#include <unordered_map>
#include <utility>
#include <vector>

#include "../../../include/vsp_attn.h"

namespace vesper_amd {

enum class DType { Float32, BFloat16 };
enum class Device { CPU, HIP };
enum class KVFormat { Float32 = VSP_KV_F32, BFloat16 = VSP_KV_BF16, Q8_0 = VSP_KV_Q8_0 };

inline size_t GetDTypeSize(DType d) { return d == DType::Float32 ? 4 : 2; }

inline void hip_check(hipError_t e, const char* what) {
    if (e != hipSuccess) throw std::runtime_error(std::string(what) + ": " + hipGetErrorString(e));
}

// Maps a vsp_status to the exception the reference throws at the same point
// (std::invalid_argument in the GroupedQueryAttention constructor, std::runtime_error elsewhere).
inline void throw_status(int st) {
    if (st == VSP_OK) return;
    if (st == VSP_ERR_GQA_HEADS || st == VSP_ERR_GQA_EMBED) throw std::invalid_argument(vsp_status_str(st));
    std::string msg = vsp_status_str(st);
    if (st == VSP_ERR_LAUNCH) msg += std::string(": ") + vsp_last_hip_error();
    throw std::runtime_error(msg);
}

// The thread's current stream, like Stream::current(Device::HIP) (src/core/stream.cpp:132-166).
inline hipStream_t& current_stream() {
    thread_local hipStream_t s = nullptr;
    return s;
}

// Device blocks are recycled instead of returned to the driver, like the reference's CachingAllocator
// (include/vesper/core/allocator.h:28-68: "keep a pool of free blocks sorted by size; when freeing, return to pool"):
// after warm-up no call on this path reaches hipMalloc / hipFree (hipFree waits for the device).  A block is handed out
// again only to the stream it was released on, so reuse is ordered behind the work that last touched it and nobody
// has to synchronise before letting a scratch buffer go.
class BlockCache {
public:
    static BlockCache& instance() {
        static BlockCache c;
        return c;
    }
    void* take(size_t bytes, hipStream_t stream) {
        if (bytes == 0) return nullptr;
        const size_t want = round_size(bytes);
        {
            std::lock_guard<std::mutex> lock(mu_);
            bytes_taken_ += want;
            auto range = free_.equal_range(Key{stream, want});
            if (range.first != range.second) {
                void* p = range.first->second;
                free_.erase(range.first);
                return p;
            }
        }
        void* p = nullptr;
        if (hipMalloc(&p, want) != hipSuccess) {
            // out of memory: give the cached free blocks back to the driver and try once more, as the reference's
            // CachingAllocator::allocate does (src/core/allocator.cpp:190-198)
            (void)hipGetLastError();
            empty_cache();
            hip_check(hipMalloc(&p, want), "hipMalloc");
        }
        std::lock_guard<std::mutex> lock(mu_);
        size_[p] = want;
        return p;
    }
    void give(void* p, hipStream_t stream) {
        if (!p) return;
        std::lock_guard<std::mutex> lock(mu_);
        free_.emplace(Key{stream, size_.at(p)}, p);
    }
    // CachingAllocator::empty_cache(): release every free block to the driver (blocks in use stay)
    void empty_cache() {
        std::lock_guard<std::mutex> lock(mu_);
        for (auto& kv : free_) {
            size_.erase(kv.second);
            (void)hipFree(kv.second);
        }
        free_.clear();
    }
    size_t driver_allocations() const {
        std::lock_guard<std::mutex> lock(mu_);
        return size_.size();
    }
    // bytes handed out so far, recycled blocks included: what the calls in between asked for
    size_t bytes_taken() const {
        std::lock_guard<std::mutex> lock(mu_);
        return bytes_taken_;
    }

private:
    using Key = std::pair<hipStream_t, size_t>;
    // sizes are rounded to 512-byte multiples up to 1 MiB and to 2 MiB multiples above, so that buffers whose size
    // drifts slowly (a workspace that follows the context length) keep hitting the same bin
    static size_t round_size(size_t b) {
        const size_t q = b <= (1u << 20) ? 512 : (2u << 20);
        return (b + q - 1) / q * q;
    }
    mutable std::mutex mu_;
    std::multimap<Key, void*> free_;
    std::unordered_map<void*, size_t> size_;
    size_t bytes_taken_ = 0;
};

class Storage {
public:
    explicit Storage(size_t bytes) : bytes_(bytes), stream_(current_stream()) { ptr_ = BlockCache::instance().take(bytes, stream_); }
    ~Storage() { BlockCache::instance().give(ptr_, stream_); }
    Storage(const Storage&) = delete;
    Storage& operator=(const Storage&) = delete;
    void* data() const { return ptr_; }
    size_t bytes() const { return bytes_; }

private:
    void* ptr_ = nullptr;
    size_t bytes_ = 0;
    hipStream_t stream_ = nullptr;
};

// What a Tensor returned by KVCache::update refers to.
struct KVCacheState {
    vsp_kv_cache c{};
    std::shared_ptr<Storage> planes[4];
};

class Tensor {
public:
    Tensor() = default;
    // view over existing storage (offset in elements)
    static Tensor over(std::shared_ptr<Storage> s, DType dt, std::vector<int64_t> shape, std::vector<int64_t> strides,
                       size_t offset = 0) {
        Tensor t;
        t.storage_ = std::move(s);
        t.dtype_ = dt;
        t.shape_ = std::move(shape);
        t.strides_ = std::move(strides);
        t.offset_ = offset;
        return t;
    }
    static std::vector<int64_t> contiguous_strides(const std::vector<int64_t>& shape) {
        std::vector<int64_t> st(shape.size(), 1);
        int64_t s = 1;
        for (int i = (int)shape.size() - 1; i >= 0; --i) {
            st[i] = s;
            s *= shape[i];
        }
        return st;
    }
    const std::vector<int64_t>& shape() const { return shape_; }
    const std::vector<int64_t>& strides() const { return strides_; }
    int64_t ndim() const { return (int64_t)shape_.size(); }
    DType dtype() const { return dtype_; }
    Device device() const { return Device::HIP; }
    size_t offset() const { return offset_; }
    bool defined() const { return storage_ != nullptr; }
    size_t numel() const {
        size_t n = 1;
        for (auto s : shape_) n *= (size_t)s;
        return n;
    }
    bool is_contiguous() const {
        int64_t expect = 1;
        for (int i = (int)shape_.size() - 1; i >= 0; --i) {
            if (shape_[i] != 1 && strides_[i] != expect) return false;
            expect *= shape_[i];
        }
        return true;
    }
    template <typename T>
    T* data_ptr() const {
        return (T*)((char*)storage_->data() + offset_ * GetDTypeSize(dtype_));
    }
    // host <-> device in contiguous (row-major) order of the view; blocking, like the reference's
    void copy_from_host(const void* src) { host_copy(const_cast<void*>(src), true); }
    void copy_to_host(void* dst) const { const_cast<Tensor*>(this)->host_copy(dst, false); }
    // [:, :, start:stop, :] of a 4-D tensor (the only slicing this path needs)
    Tensor slice_seq(int64_t start, int64_t stop) const {
        Tensor t = *this;
        t.shape_[2] = stop - start;
        t.offset_ += (size_t)(start * strides_[2]);
        return t;
    }
    vsp_tensor desc() const {
        vsp_tensor d{};
        d.data = (storage_ && storage_->data()) ? (void*)data_ptr<char>() : nullptr;
        d.dtype = dtype_ == DType::Float32 ? VSP_F32 : VSP_BF16;
        d.ndim = (int32_t)shape_.size();
        for (size_t i = 0; i < shape_.size() && i < 4; ++i) {
            d.shape[i] = shape_[i];
            d.stride[i] = strides_[i];
        }
        return d;
    }

    // set by ops::repeat_kv: logically [B, H*head_rep, S, D], physically the un-repeated tensor
    int64_t head_rep = 1;
    // set by KVCache::update: this tensor is the K (is_v == false) or V side of that cache's context
    // (the cache's state is shared, not copied: cache_len is the context length as of that update, and cache_desc()
    // the descriptor a kernel should see for this handle)
    std::shared_ptr<KVCacheState> cache;
    int32_t cache_len = 0;
    bool is_v = false;
    vsp_kv_cache cache_desc() const {
        vsp_kv_cache c = cache->c;
        c.len = cache_len;
        return c;
    }

private:
    void host_copy(void* host, bool to_device) {
        const size_t esz = GetDTypeSize(dtype_);
        if (numel() == 0) return;
        hipStream_t st = current_stream();
        auto kind = to_device ? hipMemcpyHostToDevice : hipMemcpyDeviceToHost;
        if (is_contiguous()) {
            void* dev = (void*)data_ptr<char>();
            hip_check(hipMemcpyAsync(to_device ? dev : host, to_device ? host : dev, numel() * esz, kind, st), "hipMemcpyAsync");
        } else {
            if (strides_.back() != 1) throw std::runtime_error("copy: innermost stride must be 1");
            const size_t row = (size_t)shape_.back(), rows = numel() / row;
            for (size_t r = 0; r < rows; ++r) {
                size_t rem = r, off = 0;
                for (int d = (int)shape_.size() - 2; d >= 0; --d) {
                    off += (rem % (size_t)shape_[d]) * (size_t)strides_[d];
                    rem /= (size_t)shape_[d];
                }
                void* dev = data_ptr<char>() + off * esz;
                void* h = (char*)host + r * row * esz;
                hip_check(hipMemcpyAsync(to_device ? dev : h, to_device ? h : dev, row * esz, kind, st), "hipMemcpyAsync");
            }
        }
        hip_check(hipStreamSynchronize(st), "hipStreamSynchronize");
    }
    std::shared_ptr<Storage> storage_;
    DType dtype_ = DType::Float32;
    std::vector<int64_t> shape_, strides_;
    size_t offset_ = 0;
};

inline Tensor empty(const std::vector<int64_t>& shape, DType dtype, Device device = Device::HIP) {
    if (device != Device::HIP) throw std::runtime_error("vesper_amd: only Device::HIP tensors exist on this path");
    size_t n = 1;
    for (auto s : shape) n *= (size_t)s;
    return Tensor::over(std::make_shared<Storage>(n * GetDTypeSize(dtype)), dtype, shape, Tensor::contiguous_strides(shape));
}

// ------------------------------------------------------------------------------------------------
namespace nn {

// {cos, sin} of the angles of functional::compute_rope_frequencies (include/vesper/nn/functional.h:148,
// src/nn/functional.cpp:424-443) for absolute positions [0, max_seq_len): computed once on the host by the
// library and kept on the device, instead of the reference's per-call host loop + upload.
class RopeTable {
public:
    RopeTable(int64_t max_seq_len, int64_t head_dim, float theta = 10000.0f)
        : len_(max_seq_len), head_dim_(head_dim), theta_(theta) {
        if (head_dim % 2 != 0) throw std::runtime_error("RoPE error: head_dim must be even for RoPE");  // src/nn/rope.cpp:98
        std::vector<float> host((size_t)(max_seq_len * (head_dim / 2) * 2));
        vsp_rope_fill_table(host.data(), 0, (int32_t)max_seq_len, (int32_t)head_dim, theta);
        store_ = std::make_shared<Storage>(host.size() * sizeof(float));
        hip_check(hipMemcpy(store_->data(), host.data(), host.size() * sizeof(float), hipMemcpyHostToDevice), "RopeTable upload");
    }
    const float* data() const { return (const float*)store_->data(); }
    int64_t length() const { return len_; }
    int64_t head_dim() const { return head_dim_; }
    float theta() const { return theta_; }

private:
    std::shared_ptr<Storage> store_;
    int64_t len_, head_dim_;
    float theta_;
};

// One template for both reference caches: LenT = int for KVCache, int64_t for GQAKVCache.
template <typename LenT>
class KVCacheT {
public:
    KVCacheT(LenT batch_size, LenT num_heads, LenT max_seq_len, LenT head_dim, Device device = Device::HIP,
             KVFormat format = KVFormat::Float32)
        : KVCacheT(batch_size, num_heads, max_seq_len, head_dim, device, format, /*zero=*/true) {}
    // A cache whose planes are left as allocated (no zero fill: one pass over memory saved): for a caller that writes
    // every row before reading it, such as the scratch of a single forward call.
    static KVCacheT uninitialized(LenT batch_size, LenT num_heads, LenT max_seq_len, LenT head_dim, KVFormat format) {
        return KVCacheT(batch_size, num_heads, max_seq_len, head_dim, Device::HIP, format, /*zero=*/false);
    }

private:
    KVCacheT(LenT batch_size, LenT num_heads, LenT max_seq_len, LenT head_dim, Device device, KVFormat format, bool zero)
        : st_(std::make_shared<KVCacheState>()) {
        if (device != Device::HIP) throw std::runtime_error("KVCache: only Device::HIP is implemented here");
        auto& c = st_->c;
        c.format = (int32_t)format;
        c.B = (int32_t)batch_size;
        c.Hkv = (int32_t)num_heads;
        c.S_max = (int32_t)max_seq_len;
        c.D = (int32_t)head_dim;
        for (int p = 0; p < 4; ++p) {
            size_t n = vsp_kv_plane_bytes(c.format, c.B, c.Hkv, c.S_max, c.D, p);
            if (n) st_->planes[p] = std::make_shared<Storage>(n);
        }
        c.k = st_->planes[0] ? st_->planes[0]->data() : nullptr;
        c.v = st_->planes[1] ? st_->planes[1]->data() : nullptr;
        c.k_scale = st_->planes[2] ? st_->planes[2]->data() : nullptr;
        c.v_scale = st_->planes[3] ? st_->planes[3]->data() : nullptr;
        c.len = 0;
        if (zero) throw_status(vsp_kv_cache_reset(&c, current_stream()));  // vesper::zeros in the reference constructor
    }

public:

    // Writes [:, :, start_pos:start_pos+T, :], then returns the active context [:, :, 0:len, :].
    // Float32 storage: the pair are true strided views of the cache planes, as in the reference.
    // Other formats: the pair are handles (shape [B,H,len,D], no dense storage) that
    // scaled_dot_product_attention consumes directly; materialize() makes a real tensor of one.
    std::pair<Tensor, Tensor> update(const Tensor& new_k, const Tensor& new_v, LenT start_pos) {
        vsp_tensor dk = new_k.desc(), dv = new_v.desc();
        throw_status(vsp_kv_append(&st_->c, &dk, &dv, (int64_t)start_pos, nullptr, current_stream()));
        return {view(false), view(true)};
    }
    // Steps 3-4 of the cached forward (src/nn/gqa_attention.cpp:124-130) in one launch: q and new_k rotated at
    // positions start_pos.., new_k/new_v written like update().  q is replaced by its rotated value
    // (`q_dtype`: what the attention kernels should receive).
    std::pair<Tensor, Tensor> rope_update(Tensor& q, const Tensor& new_k, const Tensor& new_v, LenT start_pos,
                                          const RopeTable& rope, DType q_dtype) {
        return rope_update(q, new_k, new_v, start_pos, rope.data(), rope.length(), q_dtype);
    }
    // The same with the table given as rows: row r of `table` rotates the token written at position r, so a table pointer
    // advanced by p rows places tokens at 0.. while rotating them as positions p.. (a scratch cache of T tokens for a
    // call at start_pos > 0).
    std::pair<Tensor, Tensor> rope_update(Tensor& q, const Tensor& new_k, const Tensor& new_v, LenT start_pos, const float* table,
                                          int64_t table_rows, DType q_dtype) {
        Tensor q_out = empty(q.shape(), q_dtype);
        vsp_tensor dq = q.desc(), dk = new_k.desc(), dv = new_v.desc(), dout = q_out.desc();
        throw_status(vsp_rope_kv_append(&st_->c, &dq, &dk, &dv, &dout, table, table_rows, (int64_t)start_pos, nullptr, current_stream()));
        q = q_out;
        return {view(false), view(true)};
    }
    // Chunked prefill: attention of the LAST T tokens of the context (q [B,Hq,T,D], already appended to the cache)
    // with K/V read in place from the planes.  The reference's scaled_dot_product_attention throws for a causal
    // T != L (src/nn/functional.cpp:406-410); the rows returned are [len-T, len) of its full causal forward.
    // A causal chunk of a few tokens (T * query heads per kv head <= 16: speculative verification, multi-token
    // prediction) takes the split-K decode kernels instead (vsp_attn_decode_multi): K and V read once per kv head at the
    // HBM rate, the context split over the chip, where the prefill kernel would walk it with one wavefront per query head.
    Tensor attend(const Tensor& q, bool is_causal = true) const {
        Tensor out = empty(q.shape(), q.dtype());
        vsp_tensor dq = q.desc(), dout = out.desc();
        const int64_t T = q.ndim() == 4 ? q.shape()[2] : 0, D = q.ndim() == 4 ? q.shape()[3] : 0;
        if (is_causal && T > 1 && st_->c.Hkv > 0 && q.shape()[1] % st_->c.Hkv == 0 && T * (q.shape()[1] / st_->c.Hkv) <= 16 &&
            (D == 64 || D == 128) && (int64_t)st_->c.len >= T) {
            const float sc = 1.0f / std::sqrt(static_cast<float>(D));
            const size_t nb = vsp_attn_decode_workspace_bytes((int32_t)(q.shape()[0] * T), (int32_t)q.shape()[1], (int32_t)D,
                                                              (int32_t)st_->c.len);
            Storage ws(nb ? nb : 16);
            throw_status(vsp_attn_decode_multi(&dq, &st_->c, nullptr, 0, &dout, sc, ws.data(), nb, current_stream()));
            return out;
        }
        // the Q8_0 read-out, or the partials of a context split over workgroups (a few query tiles over a long context)
        const size_t ws_bytes = std::max(vsp_attn_prefill_cached_workspace_bytes(&st_->c, 0, 0),
                                         q.ndim() == 4 ? vsp_attn_prefill_cached_split_workspace_bytes(&st_->c, 0, 0, (int32_t)q.shape()[1], (int32_t)T)
                                                       : size_t{0});
        std::shared_ptr<Storage> ws = ws_bytes ? std::make_shared<Storage>(ws_bytes) : nullptr;
        const float scale = 1.0f / std::sqrt(static_cast<float>(q.shape()[3]));
        throw_status(vsp_attn_prefill_cached(&dq, &st_->c, nullptr, 0, nullptr, &dout, nullptr, scale, is_causal ? 1 : 0,
                                             ws ? ws->data() : nullptr, ws_bytes, current_stream()));
        return out;  // the scratch block goes back to the cache; its next user is ordered behind this call on the stream
    }
    void reset() { throw_status(vsp_kv_cache_reset(&st_->c, current_stream())); }
    LenT current_seq_len() const { return (LenT)st_->c.len; }
    LenT get_max_seq_len() const { return (LenT)st_->c.S_max; }  // KVCache spelling
    LenT max_seq_len() const { return (LenT)st_->c.S_max; }      // GQAKVCache spelling
    static float memory_savings(int64_t num_query_heads, int64_t num_kv_heads) {
        return 1.0f - static_cast<float>(num_kv_heads) / num_query_heads;
    }
    KVFormat format() const { return (KVFormat)st_->c.format; }
    const vsp_kv_cache& raw() const { return st_->c; }

private:
    Tensor view(bool is_v) const {
        const auto& c = st_->c;
        Tensor t;
        if (c.format == VSP_KV_F32) {
            std::vector<int64_t> shape = {c.B, c.Hkv, c.S_max, c.D};
            t = Tensor::over(st_->planes[is_v ? 1 : 0], DType::Float32, shape, Tensor::contiguous_strides(shape)).slice_seq(0, c.len);
        } else {
            std::vector<int64_t> shape = {c.B, c.Hkv, c.len, c.D};
            t = Tensor::over(nullptr, DType::BFloat16, shape, Tensor::contiguous_strides(shape));
        }
        t.cache = st_;          // shared state, no copy: the handle keeps the planes alive
        t.cache_len = c.len;    // the context length as of this update
        t.is_v = is_v;
        return t;
    }
    std::shared_ptr<KVCacheState> st_;
};

using KVCache = KVCacheT<int>;
using GQAKVCache = KVCacheT<int64_t>;

// [:, :, 0:len, :] of a cache handle as a real tensor of `dtype` (copy; Q8_0 is dequantised).
inline Tensor materialize(const Tensor& handle, DType dtype) {
    if (!handle.cache || handle.defined()) return handle;
    const vsp_kv_cache c = handle.cache_desc();
    Tensor out = empty({c.B, c.Hkv, c.len, c.D}, dtype);
    vsp_tensor d = out.desc();
    throw_status(vsp_kv_read(&c, 0, c.len, handle.is_v ? nullptr : &d, handle.is_v ? &d : nullptr, current_stream()));
    out.head_rep = handle.head_rep;
    return out;
}

}  // namespace nn

// ------------------------------------------------------------------------------------------------
namespace ops {

// ops::repeat_kv (src/ops/attention_ops.cpp:92-155).  No copy is made: the result remembers n_rep
// and the attention kernels map query head h to kv head h / n_rep (src/ops/attention_ops.cpp:47).
inline Tensor repeat_kv(const Tensor& x, int64_t n_rep) {
    if (n_rep == 1) return x;
    if (x.ndim() != 4) throw std::runtime_error("repeat_kv: input must be 4D [Batch, KV_Heads, SeqLen, HeadDim]");
    Tensor r = x;
    r.head_rep = x.head_rep * n_rep;
    return r;
}

// Process-wide choice for fp32 tensors of head_dim 64 / 128 in flash_attention_hip_dispatch and
// flash_attention_backward_hip_dispatch: false (default) = fp32 matrix cores, bit-level properties of the fp32 algorithm
// kept; true = bf16 matrix cores with every operand as two bf16 terms (vsp_attn_prefill_split,
// vsp_attn_prefill_backward_split), several times faster and inside the reference's 1e-4 tolerance.
inline bool& fp32_on_bf16_matrix_cores() {
    static bool on = false;
    return on;
}

// include/vesper/ops/flash_attention.h:74-78.  output/lse are caller-allocated; lse may be undefined.
inline void flash_attention_hip_dispatch(const Tensor& q, const Tensor& k, const Tensor& v, Tensor& output, Tensor& lse,
                                         float scale, bool is_causal, float dropout_p, bool training,
                                         Tensor* dropout_mask_out) {
    (void)dropout_mask_out;  // only written when training && dropout_p > 0, which this path rejects
    Tensor kk = nn::materialize(k, q.dtype()), vv = nn::materialize(v, q.dtype());
    vsp_tensor dq = q.desc(), dk = kk.desc(), dv = vv.desc(), dout = output.desc(), dl = lse.desc();
    // a repeat_kv'ed operand must expand to exactly q's head count
    if (q.ndim() == 4 && kk.ndim() == 4 && (kk.shape()[1] * kk.head_rep != q.shape()[1] || vv.shape()[1] * vv.head_rep != q.shape()[1]))
        throw_status(VSP_ERR_SHAPE);
    if (fp32_on_bf16_matrix_cores() && q.ndim() == 4 && kk.ndim() == 4 && q.dtype() == DType::Float32 && kk.dtype() == DType::Float32 &&
        vv.dtype() == DType::Float32 && (q.shape()[3] == 64 || q.shape()[3] == 128) && !(training && dropout_p > 0.0f) &&
        q.shape()[2] > 0 && kk.shape()[2] > 0) {
        const size_t ws_bytes = vsp_attn_prefill_split_workspace_bytes((int32_t)q.shape()[0], (int32_t)q.shape()[1], (int32_t)kk.shape()[1],
                                                                       (int32_t)q.shape()[2], (int32_t)kk.shape()[2], (int32_t)q.shape()[3]);
        Storage ws(ws_bytes > 0 ? ws_bytes : 16);
        throw_status(vsp_attn_prefill_split(&dq, &dk, &dv, &dout, lse.defined() ? &dl : nullptr, scale, is_causal ? 1 : 0, ws.data(),
                                            ws_bytes, current_stream()));
        return;
    }
    throw_status(vsp_attn_prefill(&dq, &dk, &dv, &dout, lse.defined() ? &dl : nullptr, scale, is_causal ? 1 : 0, dropout_p,
                                  training ? 1 : 0, current_stream()));
}

// include/vesper/ops/flash_attention.h:34-41.
inline Tensor flash_attention(const Tensor& q, const Tensor& k, const Tensor& v, float scale, bool is_causal = true,
                              float dropout_p = 0.0f, bool training = false) {
    if (q.ndim() != 4 || k.ndim() != 4 || v.ndim() != 4) throw_status(VSP_ERR_NDIM);
    Tensor output = empty(q.shape(), q.dtype());
    Tensor lse = empty({q.shape()[0], q.shape()[1], q.shape()[2]}, DType::Float32);
    flash_attention_hip_dispatch(q, k, v, output, lse, scale, is_causal, dropout_p, training, nullptr);
    return output;
}

// The same op for fp32 tensors at matrix-core speed: every operand taken as two bf16 terms, three MFMAs per product, fp32
// accumulation (vsp_attn_prefill_split); within the reference's 1e-4 of its fp32 result, not bit-close to it.  A caller
// switches a model over by calling this where it called flash_attention with fp32 tensors of head_dim 64 or 128.
inline Tensor flash_attention_split(const Tensor& q, const Tensor& k, const Tensor& v, float scale, bool is_causal = true,
                                    Tensor* lse_out = nullptr) {
    if (q.ndim() != 4 || k.ndim() != 4 || v.ndim() != 4) throw_status(VSP_ERR_NDIM);
    Tensor kk = nn::materialize(k, q.dtype()), vv = nn::materialize(v, q.dtype());
    if (kk.shape()[1] * kk.head_rep != q.shape()[1] || vv.shape()[1] * vv.head_rep != q.shape()[1]) throw_status(VSP_ERR_SHAPE);
    Tensor output = empty(q.shape(), q.dtype());
    Tensor lse = empty({q.shape()[0], q.shape()[1], q.shape()[2]}, DType::Float32);
    const size_t ws_bytes = vsp_attn_prefill_split_workspace_bytes((int32_t)q.shape()[0], (int32_t)q.shape()[1], (int32_t)kk.shape()[1],
                                                                   (int32_t)q.shape()[2], (int32_t)kk.shape()[2], (int32_t)q.shape()[3]);
    Storage ws(ws_bytes > 0 ? ws_bytes : 16);
    vsp_tensor dq = q.desc(), dk = kk.desc(), dv = vv.desc(), dout = output.desc(), dl = lse.desc();
    throw_status(vsp_attn_prefill_split(&dq, &dk, &dv, &dout, &dl, scale, is_causal ? 1 : 0, ws.data(), ws_bytes, current_stream()));
    if (lse_out) *lse_out = lse;
    return output;
}

// bf16 backward: the larger workspace, with which dS is computed once and kept as tiles (about 2 N^2 bytes per query
// head, vsp_attn_backward_fast_workspace_bytes), is taken for contexts of at least backward_fast_min_context() tokens
// (4096: below that recomputing dS measured as fast) when it is no larger than backward_fast_workspace_limit() bytes
// (8 GiB; 0 switches the path off).
inline int64_t& backward_fast_min_context() {
    static int64_t n = 4096;
    return n;
}
inline size_t& backward_fast_workspace_limit() {
    static size_t limit = (size_t)8 << 30;
    return limit;
}

// include/vesper/ops/flash_attention.h:80-92 (defined src/ops/hip/flash_attention.hip:183-299): the gradients are
// caller-allocated.  A dropout mask can only come from a training forward with dropout_p > 0, which this path
// rejects, so a non-null mask with dropout_p > 0 is VSP_ERR_UNSUPPORTED here too.
inline void flash_attention_backward_hip_dispatch(const Tensor& grad_output, const Tensor& q, const Tensor& k, const Tensor& v,
                                                  const Tensor& output, const Tensor& lse, Tensor& grad_q, Tensor& grad_k,
                                                  Tensor& grad_v, float scale, bool is_causal, float dropout_p,
                                                  const Tensor* dropout_mask) {
    if (dropout_p > 0.0f && dropout_mask && dropout_mask->defined()) throw_status(VSP_ERR_UNSUPPORTED);
    if (dropout_p > 0.0f) throw_status(VSP_ERR_UNSUPPORTED);
    vsp_tensor d0 = grad_output.desc(), d1 = q.desc(), d2 = k.desc(), d3 = v.desc(), d4 = output.desc(), d5 = lse.desc();
    vsp_tensor o0 = grad_q.desc(), o1 = grad_k.desc(), o2 = grad_v.desc();
    if (fp32_on_bf16_matrix_cores() && q.ndim() == 4 && k.ndim() == 4 && q.dtype() == DType::Float32 &&
        (q.shape()[3] == 64 || q.shape()[3] == 128) && q.shape()[2] > 0) {   // the switch covers the backward of the same tensors
        const size_t split_bytes = vsp_attn_backward_split_workspace_bytes((int32_t)q.shape()[0], (int32_t)q.shape()[1], (int32_t)k.shape()[1],
                                                                           (int32_t)q.shape()[2], (int32_t)q.shape()[3]);
        Storage split_ws(split_bytes ? split_bytes : 16);
        throw_status(vsp_attn_prefill_backward_split(&d0, &d1, &d2, &d3, &d4, &d5, &o0, &o1, &o2, scale, is_causal ? 1 : 0, split_ws.data(),
                                                     split_bytes, current_stream()));
        return;
    }
    size_t ws_bytes = q.ndim() == 4 ? vsp_attn_backward_workspace_bytes((int32_t)q.shape()[0], (int32_t)q.shape()[1], (int32_t)q.shape()[2]) : 0;
    if (q.ndim() == 4 && q.dtype() == DType::BFloat16 && q.shape()[2] >= backward_fast_min_context()) {   // dS kept instead of recomputed
        const size_t fast = vsp_attn_backward_fast_workspace_bytes((int32_t)q.shape()[0], (int32_t)q.shape()[1], (int32_t)q.shape()[2]);
        if (fast > 0 && fast <= backward_fast_workspace_limit()) ws_bytes = fast;
    }
    Storage ws(ws_bytes ? ws_bytes : 4);
    throw_status(vsp_attn_prefill_backward(&d0, &d1, &d2, &d3, &d4, &d5, &o0, &o1, &o2, scale, is_causal ? 1 : 0, ws.data(), ws_bytes,
                                           current_stream()));
}

// include/vesper/ops/flash_attention.h:61-71, src/ops/flash_attention.cpp:165-216: (grad_q, grad_k, grad_v).
// `output` and `lse` are the forward's results (flash_attention_hip_dispatch writes both).  k and v may carry
// fewer heads than q: their gradients are then already summed over each group's query heads.
inline std::tuple<Tensor, Tensor, Tensor> flash_attention_backward(const Tensor& grad_output, const Tensor& q, const Tensor& k,
                                                                   const Tensor& v, const Tensor& output, const Tensor& lse, float scale,
                                                                   bool is_causal = true, float dropout_p = 0.0f,
                                                                   const Tensor& dropout_mask = Tensor()) {
    if (q.ndim() != 4 || k.ndim() != 4 || v.ndim() != 4) throw_status(VSP_ERR_NDIM);
    Tensor gq = empty(q.shape(), q.dtype()), gk = empty(k.shape(), k.dtype()), gv = empty(v.shape(), v.dtype());
    flash_attention_backward_hip_dispatch(grad_output, q, k, v, output, lse, gq, gk, gv, scale, is_causal, dropout_p,
                                          dropout_mask.defined() ? &dropout_mask : nullptr);
    return {gq, gk, gv};
}

}  // namespace ops

namespace nn {
namespace functional {

// include/vesper/nn/functional.h:132-136, src/nn/functional.cpp:370-422.  One kernel family serves
// every sequence length (the reference's switch at 512 is a speed heuristic of its own back ends):
// The length a per-call decode workspace is sized for: the next power of two at or above the context length, capped
// at the cache's capacity.
inline int32_t ws_len_bound(int32_t len, int32_t s_max) {
    int64_t p = 256;
    while (p < len) p *= 2;
    return (int32_t)std::min<int64_t>(p, std::max<int32_t>(s_max, 1));
}

// T == 1 over a cache handle -> split-K decode; everything else -> the prefill kernel.
inline Tensor scaled_dot_product_attention(const Tensor& query, const Tensor& key, const Tensor& value, bool is_causal = false,
                                           double dropout_p = 0.0) {
    if (dropout_p > 0.0) throw_status(VSP_ERR_UNSUPPORTED);
    if (query.ndim() != 4 || key.ndim() != 4 || value.ndim() != 4) throw_status(VSP_ERR_NDIM);
    const int64_t T = query.shape()[2], L = key.shape()[2], D = query.shape()[3];
    if (is_causal && T != L && T != 1) throw_status(VSP_ERR_BROADCAST);  // [T,T] mask vs [T,L] scores
    const float scale = 1.0f / std::sqrt(static_cast<float>(D));
    if (T == 1 && key.cache && value.cache && !key.is_v && value.is_v) {
        Tensor out = empty(query.shape(), query.dtype());
        const vsp_kv_cache c = key.cache_desc();
        // (sized for the next power of two of the context length: a token loop then keeps taking the same block
        // instead of walking through a bin per 2 MiB of growth)
        const size_t ws_bytes = vsp_attn_decode_workspace_bytes((int32_t)query.shape()[0], (int32_t)query.shape()[1], (int32_t)D,
                                                               ws_len_bound(c.len, c.S_max));
        Storage ws(ws_bytes);  // a recycled block after the first call; released without waiting (see BlockCache)
        vsp_tensor dq = query.desc(), dout = out.desc();
        throw_status(vsp_attn_decode(&dq, &c, nullptr, 0, &dout, scale, ws.data(), ws_bytes, current_stream()));
        return out;
    }
    return ops::flash_attention(query, key, value, scale, is_causal && T > 1);
}

// T == 1 over a cache handle with the module's output projection behind it: what GroupedQueryAttention::forward
// and MultiHeadAttention::forward do after SDPA -- transpose(1,2).reshape({B,T,C}) and wo_ / out_proj
// (src/nn/gqa_attention.cpp:151-152, src/nn/transformer.cpp:207-215) -- in the same call.  wo: the Linear's weight
// [N, C] (include/vesper/nn/linear.h), bias: its bias [N] or nullptr.  Returns [B, 1, N].
inline Tensor decode_attention_proj(const Tensor& query, const Tensor& key, const Tensor& value, const Tensor& wo,
                                    const Tensor* bias = nullptr) {
    if (query.ndim() != 4) throw_status(VSP_ERR_NDIM);
    if (!(key.cache && value.cache && !key.is_v && value.is_v)) throw std::runtime_error("decode_attention_proj: key/value must be cache handles");
    if (wo.ndim() != 2) throw_status(VSP_ERR_NDIM);
    const int64_t B = query.shape()[0], Hq = query.shape()[1], D = query.shape()[3];
    const vsp_kv_cache c = key.cache_desc();
    const float scale = 1.0f / std::sqrt(static_cast<float>(D));
    Tensor y = empty({B, 1, wo.shape()[0]}, query.dtype());
    const size_t ws_bytes = vsp_attn_decode_proj_workspace_bytes((int32_t)B, (int32_t)Hq, (int32_t)D, ws_len_bound(c.len, c.S_max), (int32_t)wo.shape()[0]);
    Storage ws(ws_bytes);
    vsp_tensor dq = query.desc(), dw = wo.desc(), dy = y.desc(), db;
    if (bias) db = bias->desc();
    throw_status(vsp_attn_decode_proj(&dq, &c, nullptr, 0, &dw, bias ? &db : nullptr, &dy, scale, ws.data(), ws_bytes, current_stream()));
    return y;
}

}  // namespace functional

// The attention core shared by GroupedQueryAttention::forward(x, cache, start_pos)
// (src/nn/gqa_attention.cpp:111-159, steps 4-6) and MultiHeadAttention::forward(x, cache, start_pos)
// (src/nn/transformer.cpp:166-216): q [B,Hq,T,D], k/v [B,Hkv,T,D] are what the projections + RoPE
// produced.  The constructor performs the reference constructor's checks and arithmetic.
class GroupedQueryAttentionCore {
public:
    // the reference's parameter list (include/vesper/nn/gqa_attention.h:40-47); max_seq_len and rope_base size its RoPE
    // table, which callers of this core bring themselves (RopeTable), dropout is refused at forward time when training,
    // bias belongs to the projections
    GroupedQueryAttentionCore(int64_t embed_dim, int64_t num_heads, int64_t num_kv_heads, int64_t max_seq_len = 4096,
                              float rope_base = 10000.0f, float dropout = 0.0f, bool bias = false)
        : embed_dim_(embed_dim), num_heads_(num_heads), num_kv_heads_(num_kv_heads), max_seq_len_(max_seq_len),
          rope_base_(rope_base), dropout_(dropout), bias_(bias) {
        if (num_heads % num_kv_heads != 0)
            throw std::invalid_argument("GroupedQueryAttention: num_heads (" + std::to_string(num_heads) +
                                        ") must be divisible by num_kv_heads (" + std::to_string(num_kv_heads) + ")");
        if (embed_dim % num_heads != 0)
            throw std::invalid_argument("GroupedQueryAttention: embed_dim (" + std::to_string(embed_dim) +
                                        ") must be divisible by num_heads (" + std::to_string(num_heads) + ")");
        throw_status(vsp_gqa_config(embed_dim, num_heads, num_kv_heads, &head_dim_, &num_rep_));
    }
    int64_t embed_dim() const { return embed_dim_; }
    int64_t num_heads() const { return num_heads_; }
    int64_t num_kv_heads() const { return num_kv_heads_; }
    int64_t head_dim() const { return head_dim_; }
    int64_t num_rep() const { return num_rep_; }
    int64_t max_seq_len() const { return max_seq_len_; }
    float rope_base() const { return rope_base_; }
    float dropout() const { return dropout_; }
    bool bias() const { return bias_; }
    float kv_cache_ratio() const { return static_cast<float>(num_kv_heads_) / num_heads_; }

    // forward(x, causal) core, src/nn/gqa_attention.cpp:91-96
    Tensor forward(const Tensor& q, const Tensor& k, const Tensor& v, bool causal = true) const {
        return functional::scaled_dot_product_attention(q, ops::repeat_kv(k, num_rep_), ops::repeat_kv(v, num_rep_), causal, 0.0);
    }
    // forward(x, cache, start_pos) core, src/nn/gqa_attention.cpp:128-148
    template <typename CacheT>
    Tensor forward(const Tensor& q, Tensor k, Tensor v, CacheT* cache, int64_t start_pos = 0) const {
        const int64_t T = q.shape()[2];
        if (cache) {
            auto kv = cache->update(k, v, (decltype(cache->current_seq_len()))start_pos);
            k = kv.first;
            v = kv.second;
        }
        k = ops::repeat_kv(k, num_rep_);
        v = ops::repeat_kv(v, num_rep_);
        const bool use_causal = (T > 1);
        return functional::scaled_dot_product_attention(q, k, v, use_causal, 0.0);
    }

    // forward(x, cache, start_pos) from step 3 on, src/nn/gqa_attention.cpp:124-148: q/k/v are the projections'
    // outputs viewed as [B,H,T,D] (any strides), not yet rotated.
    template <typename CacheT>
    Tensor forward_rope(Tensor q, const Tensor& k, const Tensor& v, CacheT* cache, int64_t start_pos, const RopeTable& rope,
                        DType q_dtype) const {
        if (!cache) throw std::runtime_error("forward_rope: a cache is required");
        const int64_t T = q.shape()[2];
        auto kv = cache->rope_update(q, k, v, (decltype(cache->current_seq_len()))start_pos, rope, q_dtype);
        return functional::scaled_dot_product_attention(q, ops::repeat_kv(kv.first, num_rep_), ops::repeat_kv(kv.second, num_rep_), T > 1, 0.0);
    }

    // The same for a chunk that continues a longer context (start_pos > 0, T > 1), which the reference cannot
    // run: RoPE + append, then the chunk attends over the cache planes in place.
    template <typename CacheT>
    Tensor forward_chunk(Tensor q, const Tensor& k, const Tensor& v, CacheT* cache, int64_t start_pos, const RopeTable& rope,
                         DType q_dtype) const {
        if (!cache) throw std::runtime_error("forward_chunk: a cache is required");
        cache->rope_update(q, k, v, (decltype(cache->current_seq_len()))start_pos, rope, q_dtype);
        return cache->attend(q, true);
    }

    // One generated token from step 3 to the module's end (src/nn/gqa_attention.cpp:124-152): RoPE + append, decode over
    // the cache, heads merged, wo_ applied.  q [B,Hq,1,D], k/v [B,Hkv,1,D] not yet rotated; wo_weight [C, C].  -> [B,1,C]
    template <typename CacheT>
    Tensor forward_token_proj(Tensor q, const Tensor& k, const Tensor& v, CacheT* cache, int64_t start_pos, const RopeTable& rope,
                              DType q_dtype, const Tensor& wo_weight, const Tensor* wo_bias = nullptr) const {
        if (!cache) throw std::runtime_error("forward_token_proj: a cache is required");
        if (q.ndim() != 4 || q.shape()[2] != 1) throw_status(VSP_ERR_SHAPE);
        auto kv = cache->rope_update(q, k, v, (decltype(cache->current_seq_len()))start_pos, rope, q_dtype);
        return functional::decode_attention_proj(q, kv.first, kv.second, wo_weight, wo_bias);
    }

private:
    int64_t embed_dim_, num_heads_, num_kv_heads_, head_dim_ = 0, num_rep_ = 0;
    int64_t max_seq_len_;
    float rope_base_, dropout_;
    bool bias_;
};

// The attention core of MultiHeadAttention (include/vesper/nn/transformer.h:41-56, src/nn/transformer.cpp:96-216):
// q, k, v [B,n_head,T,head_dim] are the three slices of c_attn's output viewed per head (:127-129, :182-184; any
// strides, so the .contiguous() transposes can go).  The three overloads keep the reference's semantics:
//   forward(q,k,v)                    = forward(q,k,v,false): NOT causal (:108-110)
//   forward(q,k,v,causal)             RoPE at positions 0.. when use_rope (:132-136), then SDPA (:141)
//   forward(q,k,v,cache,start_pos)    RoPE at start_pos.. (:187-191), cache->update (:193-197), SDPA with
//                                     use_causal_mask = (T > 1) (:202-206)
// dropout > 0 only matters in training mode, which this path does not implement (VSP_ERR_UNSUPPORTED if asked for).
class MultiHeadAttentionCore {
public:
    MultiHeadAttentionCore(int embed_dim, int num_heads, float dropout = 0.0f, bool use_rope = true)
        : n_head(num_heads), n_embd(embed_dim), dropout_(dropout), use_rope_(use_rope) {}

    Tensor forward(const Tensor& q, const Tensor& k, const Tensor& v) { return forward(q, k, v, false); }

    Tensor forward(const Tensor& q, const Tensor& k, const Tensor& v, bool causal) {
        if (training_ && dropout_ > 0.0f) throw_status(VSP_ERR_UNSUPPORTED);
        if (!use_rope_) return functional::scaled_dot_product_attention(q, k, v, causal, 0.0);
        // RoPE without a cache of the caller's: a cache of exactly T tokens holds the rotated K and V for this call
        // (one launch rotates q and k and writes it), then the attention reads it like any other cache
        if (q.ndim() != 4) throw_status(VSP_ERR_NDIM);
        const int64_t B = q.shape()[0], H = k.shape()[1], T = q.shape()[2], D = q.shape()[3];
        const RopeTable& rope = rope_for(T, D);
        // (every row of the scratch is written by the rotation before it is read: no zero fill)
        KVCache scratch = KVCache::uninitialized((int)B, (int)H, (int)T, (int)D, q.dtype() == DType::Float32 ? KVFormat::Float32 : KVFormat::BFloat16);
        Tensor qr = q;
        auto kv = scratch.rope_update(qr, k, v, 0, rope, q.dtype());
        if (q.dtype() == DType::Float32) return functional::scaled_dot_product_attention(qr, kv.first, kv.second, causal, 0.0);
        return scratch.attend(qr, causal);
    }

    Tensor forward(const Tensor& q, Tensor k, Tensor v, KVCache* cache, int start_pos = 0) {
        if (training_ && dropout_ > 0.0f) throw_status(VSP_ERR_UNSUPPORTED);
        if (q.ndim() != 4) throw_status(VSP_ERR_NDIM);
        const int64_t T = q.shape()[2], D = q.shape()[3];
        Tensor qq = q;
        if (cache) {
            std::pair<Tensor, Tensor> kv = use_rope_ ? cache->rope_update(qq, k, v, start_pos, rope_for(start_pos + T, D), q.dtype())
                                                     : cache->update(k, v, start_pos);
            k = kv.first;
            v = kv.second;
        } else if (use_rope_) {
            // no cache: rotate as positions start_pos.. through a scratch of this call's own that holds exactly these T
            // tokens (the table enters advanced by start_pos rows, so the tokens are placed at 0..: what the call
            // writes does not grow with the position), then SDPA over exactly these T keys (:187-191)
            const int64_t B = q.shape()[0], H = k.shape()[1];
            KVCache scratch = KVCache::uninitialized((int)B, (int)H, (int)T, (int)D,
                                                     q.dtype() == DType::Float32 ? KVFormat::Float32 : KVFormat::BFloat16);
            const RopeTable& rope = rope_for(start_pos + T, D);
            scratch.rope_update(qq, k, v, 0, rope.data() + (int64_t)start_pos * D, rope.length() - start_pos, q.dtype());
            Tensor kr = empty(k.shape(), q.dtype()), vr = empty(v.shape(), q.dtype());
            vsp_tensor dk = kr.desc(), dv = vr.desc();
            throw_status(vsp_kv_read(&scratch.raw(), 0, T, &dk, &dv, current_stream()));
            k = kr;
            v = vr;
        }
        const bool use_causal_mask = (T > 1);
        return functional::scaled_dot_product_attention(qq, k, v, use_causal_mask, 0.0);
    }

    void train(bool on = true) { training_ = on; }
    void eval() { training_ = false; }

    int n_head;
    int n_embd;
    float dropout_;
    bool use_rope_;

private:
    const RopeTable& rope_for(int64_t positions, int64_t head_dim) {
        if (!rope_ || rope_->length() < positions || rope_->head_dim() != head_dim) {
            int64_t len = 256;
            while (len < positions) len *= 2;
            rope_ = std::make_unique<RopeTable>(len, head_dim, 10000.0f);  // theta of :133, :188
        }
        return *rope_;
    }
    bool training_ = false;
    std::unique_ptr<RopeTable> rope_;
};

}  // namespace nn
}  // namespace vesper_amd
