// TEST INFRASTRUCTURE ONLY.  Thin extern "C" shim over the *real* reference
// CPU library, compiled from the sources where they lie under /root/reference
// (see oracle/Makefile, target `ref`).  Output goes to oracle/_ref/ only.
// Nothing in the product path loads this; it exists to pin oracle/vsp_oracle.c
// bit-for-bit, to write tests/golden/ fixtures, and as bench.py's CPU baseline.
//
// Every entry point takes plain contiguous host buffers, wraps them in
// reference Tensors (copy_from_host), calls the reference function named in
// its comment, and copies the result back out.  Exceptions are mapped to a
// non-zero return and the message kept in vref_last_error().
#include <vesper/core/tensor.h>
#include <vesper/core/factories.h>
#include <vesper/core/slice.h>
#include <vesper/autograd/guard.h>
#include <vesper/ops/flash_attention.h>
#include <vesper/ops/attention_ops.h>
#include <vesper/nn/functional.h>
#include <vesper/nn/transformer.h>
#include <vesper/nn/gqa_attention.h>
#include <vesper/nn/linear.h>
#include <vesper/core/half.h>

#include <cstring>
#include <string>
#include <vector>

using vesper::Tensor;
using vesper::DType;
using vesper::Device;

namespace {
thread_local std::string g_err;

Tensor from_host(const float* p, std::vector<int64_t> shape) {
    Tensor t = vesper::empty(shape, DType::Float32, Device::CPU);
    t.copy_from_host(p);
    return t;
}
void to_host(const Tensor& t, float* p) {
    Tensor c = t.is_contiguous() ? t : t.contiguous();
    c.copy_to_host(p);
}
template <class F> int guarded(F&& f) {
    try {
        vesper::autograd::NoGradGuard ng;
        f();
        return 0;
    } catch (const std::exception& e) {
        g_err = e.what();
        return 1;
    } catch (...) {
        g_err = "unknown exception";
        return 2;
    }
}
}  // namespace

extern "C" {

const char* vref_last_error() { return g_err.c_str(); }

// ops::flash_attention front-end (src/ops/flash_attention.cpp:42-163); lse is
// obtained from flash_attention_cpu_dispatch (:218-364) on the same inputs.
int vref_flash_attention(const float* q, const float* k, const float* v,
                         float* out, float* lse,
                         int64_t B, int64_t H, int64_t N, int64_t D,
                         float scale, int is_causal) {
    return guarded([&] {
        Tensor tq = from_host(q, {B, H, N, D});
        Tensor tk = from_host(k, {B, H, N, D});
        Tensor tv = from_host(v, {B, H, N, D});
        Tensor o = vesper::ops::flash_attention(tq, tk, tv, scale, is_causal != 0);
        to_host(o, out);
        if (lse) {
            Tensor o2 = vesper::empty({B, H, N, D}, DType::Float32, Device::CPU);
            Tensor l = vesper::empty({B, H, N}, DType::Float32, Device::CPU);
            vesper::ops::flash_attention_cpu_dispatch(tq, tk, tv, o2, l, scale,
                                                      is_causal != 0, 0.0f, false, nullptr);
            to_host(l, lse);
        }
    });
}

// ops::flash_attention_backward (src/ops/flash_attention.cpp:165-216 -> :366-482), no dropout.  out and lse are
// the forward's own results for the same inputs.
int vref_flash_attention_backward(const float* dout, const float* q, const float* k, const float* v,
                                  const float* out, const float* lse, float* dq, float* dk, float* dv,
                                  int64_t B, int64_t H, int64_t N, int64_t D, float scale, int is_causal) {
    return guarded([&] {
        Tensor tdo = from_host(dout, {B, H, N, D}), tq = from_host(q, {B, H, N, D});
        Tensor tk = from_host(k, {B, H, N, D}), tv = from_host(v, {B, H, N, D});
        Tensor to = from_host(out, {B, H, N, D}), tl = from_host(lse, {B, H, N});
        auto g = vesper::ops::flash_attention_backward(tdo, tq, tk, tv, to, tl, scale, is_causal != 0, 0.0f, Tensor());
        to_host(std::get<0>(g), dq);
        to_host(std::get<1>(g), dk);
        to_host(std::get<2>(g), dv);
    });
}

// Same, but with arbitrary (possibly mismatching) shapes so that the
// validation errors of the front-end can be observed.
int vref_flash_attention_shapes(const int64_t* qs, const int64_t* ks, const int64_t* vs,
                                int nq, int nk, int nv, float dropout_p) {
    return guarded([&] {
        Tensor tq = vesper::zeros(std::vector<int64_t>(qs, qs + nq), DType::Float32, Device::CPU);
        Tensor tk = vesper::zeros(std::vector<int64_t>(ks, ks + nk), DType::Float32, Device::CPU);
        Tensor tv = vesper::zeros(std::vector<int64_t>(vs, vs + nv), DType::Float32, Device::CPU);
        (void)vesper::ops::flash_attention(tq, tk, tv, 1.0f, true, dropout_p, false);
    });
}

// ops::repeat_kv (src/ops/attention_ops.cpp:92-155).
int vref_repeat_kv(const float* in, float* out, int64_t B, int64_t Hkv, int64_t S, int64_t D,
                   int64_t n_rep) {
    return guarded([&] {
        Tensor t = from_host(in, {B, Hkv, S, D});
        Tensor r = vesper::ops::repeat_kv(t, n_rep);
        to_host(r, out);
    });
}

// nn::functional::scaled_dot_product_attention (src/nn/functional.cpp:370-422).
// q [B,H,T,D]; k,v [B,H,L,D].  T>=512 routes to flash_attention inside.
int vref_sdpa(const float* q, const float* k, const float* v, float* out,
              int64_t B, int64_t H, int64_t T, int64_t L, int64_t D, int is_causal) {
    return guarded([&] {
        Tensor tq = from_host(q, {B, H, T, D});
        Tensor tk = from_host(k, {B, H, L, D});
        Tensor tv = from_host(v, {B, H, L, D});
        Tensor o = vesper::nn::functional::scaled_dot_product_attention(tq, tk, tv,
                                                                        is_causal != 0, 0.0);
        to_host(o, out);
    });
}

// nn::KVCache (include/vesper/nn/transformer.h:21-39, src/nn/transformer.cpp:32-93).
void* vref_kvcache_new(int B, int H, int S_max, int D) {
    void* p = nullptr;
    guarded([&] { p = new vesper::nn::KVCache(B, H, S_max, D, Device::CPU); });
    return p;
}
void vref_kvcache_free(void* c) { delete static_cast<vesper::nn::KVCache*>(c); }
int vref_kvcache_len(void* c) { return static_cast<vesper::nn::KVCache*>(c)->current_seq_len(); }
int vref_kvcache_max_len(void* c) { return static_cast<vesper::nn::KVCache*>(c)->get_max_seq_len(); }
int vref_kvcache_reset(void* c) {
    return guarded([&] { static_cast<vesper::nn::KVCache*>(c)->reset(); });
}
// update(); the returned views are copied out contiguously as [B,H,len,D]
// (k_view/v_view may be NULL) and their shape/strides/offset reported in
// meta[0..8] = shape[0..3], strides[0..3], offset.
int vref_kvcache_update(void* c, const float* new_k, const float* new_v,
                        int64_t B, int64_t H, int64_t T, int64_t D, int start_pos,
                        float* k_view, float* v_view, int64_t* meta) {
    return guarded([&] {
        auto* cache = static_cast<vesper::nn::KVCache*>(c);
        Tensor tk = from_host(new_k, {B, H, T, D});
        Tensor tv = from_host(new_v, {B, H, T, D});
        auto kv = cache->update(tk, tv, start_pos);
        if (meta) {
            for (int i = 0; i < 4; ++i) {
                meta[i] = kv.first.shape()[i];
                meta[4 + i] = kv.first.strides()[i];
            }
            meta[8] = (int64_t)kv.first.offset();
        }
        if (k_view) to_host(kv.first, k_view);
        if (v_view) to_host(kv.second, v_view);
    });
}

// nn::GQAKVCache (include/vesper/nn/gqa_attention.h:110-163, src/nn/gqa_attention.cpp:165-214).
void* vref_gqacache_new(int64_t B, int64_t H, int64_t S_max, int64_t D) {
    void* p = nullptr;
    guarded([&] { p = new vesper::nn::GQAKVCache(B, H, S_max, D, Device::CPU); });
    return p;
}
void vref_gqacache_free(void* c) { delete static_cast<vesper::nn::GQAKVCache*>(c); }
int64_t vref_gqacache_len(void* c) { return static_cast<vesper::nn::GQAKVCache*>(c)->current_seq_len(); }
int vref_gqacache_reset(void* c) {
    return guarded([&] { static_cast<vesper::nn::GQAKVCache*>(c)->reset(); });
}
int vref_gqacache_update(void* c, const float* new_k, const float* new_v,
                         int64_t B, int64_t H, int64_t T, int64_t D, int64_t start_pos,
                         float* k_view, float* v_view) {
    return guarded([&] {
        auto* cache = static_cast<vesper::nn::GQAKVCache*>(c);
        Tensor tk = from_host(new_k, {B, H, T, D});
        Tensor tv = from_host(new_v, {B, H, T, D});
        auto kv = cache->update(tk, tv, start_pos);
        if (k_view) to_host(kv.first, k_view);
        if (v_view) to_host(kv.second, v_view);
    });
}

// The attention core of GroupedQueryAttention::forward(x, cache, start_pos),
// steps 4-6 (src/nn/gqa_attention.cpp:128-148): cache->update -> repeat_kv x2
// -> scaled_dot_product_attention(use_causal = T > 1).
// One deliberate difference: the cache views are made contiguous before
// repeat_kv, because repeat_kv_cpu_dispatch reads its input through a raw
// pointer as if contiguous (src/ops/attention_ops.cpp:30-57) and would read
// the wrong rows of a partial-length view; with make_contiguous == 0 the
// reference is called exactly as written.
int vref_gqa_core(void* c, const float* q, const float* new_k, const float* new_v,
                  int64_t B, int64_t Hq, int64_t Hkv, int64_t T, int64_t D,
                  int start_pos, int make_contiguous, float* out) {
    return guarded([&] {
        auto* cache = static_cast<vesper::nn::KVCache*>(c);
        Tensor tq = from_host(q, {B, Hq, T, D});
        Tensor k = from_host(new_k, {B, Hkv, T, D});
        Tensor v = from_host(new_v, {B, Hkv, T, D});
        auto kv = cache->update(k, v, start_pos);
        k = kv.first;
        v = kv.second;
        if (make_contiguous) {
            k = k.contiguous();
            v = v.contiguous();
        }
        int64_t n_rep = Hq / Hkv;
        k = vesper::ops::repeat_kv(k, n_rep);
        v = vesper::ops::repeat_kv(v, n_rep);
        bool use_causal = (T > 1);
        Tensor o = vesper::nn::functional::scaled_dot_product_attention(tq, k, v, use_causal, 0.0);
        to_host(o, out);
    });
}

// GroupedQueryAttention constructor validation (src/nn/gqa_attention.cpp:47-57).
int vref_gqa_ctor(int64_t embed_dim, int64_t num_heads, int64_t num_kv_heads, int64_t* head_dim,
                  int64_t* num_rep) {
    return guarded([&] {
        vesper::nn::GroupedQueryAttention m(embed_dim, num_heads, num_kv_heads);
        if (head_dim) *head_dim = m.head_dim();
        if (num_rep) *num_rep = m.num_rep();
    });
}

// functional::compute_rope_frequencies (src/nn/functional.cpp:424-443): angles [seq_len][head_dim/2].
int vref_rope_frequencies(int seq_len, int head_dim, int start_pos, float theta, float* angles) {
    return guarded([&] {
        Tensor f = vesper::nn::functional::compute_rope_frequencies(seq_len, head_dim, start_pos, theta, Device::CPU);
        to_host(f, angles);
    });
}
// functional::apply_rotary_emb (src/nn/functional.cpp:445-494): x [B,H,S,D], angles [S][D/2].
int vref_apply_rotary_emb(const float* x, int64_t B, int64_t H, int64_t S, int64_t D, const float* angles,
                          float* out) {
    return guarded([&] {
        Tensor tx = from_host(x, {B, H, S, D});
        Tensor tf = from_host(angles, {S, D / 2});
        Tensor o = vesper::nn::functional::apply_rotary_emb(tx, tf);
        to_host(o, out);
    });
}
// The attention module's own sequence with a cache (src/nn/gqa_attention.cpp:124-141): RoPE on q and k
// at start_pos, cache update, repeat_kv, attention.  Returns the rotated q and the attention output.
int vref_gqa_rope_core(void* c, const float* q, const float* new_k, const float* new_v,
                       int64_t B, int64_t Hq, int64_t Hkv, int64_t T, int64_t D,
                       int start_pos, float theta, float* q_rot, float* out) {
    return guarded([&] {
        auto* cache = static_cast<vesper::nn::KVCache*>(c);
        Tensor tq = from_host(q, {B, Hq, T, D});
        Tensor k = from_host(new_k, {B, Hkv, T, D});
        Tensor v = from_host(new_v, {B, Hkv, T, D});
        Tensor freqs = vesper::nn::functional::compute_rope_frequencies((int)T, (int)D, start_pos, theta, Device::CPU);
        tq = vesper::nn::functional::apply_rotary_emb(tq, freqs);
        k = vesper::nn::functional::apply_rotary_emb(k, freqs);
        auto kv = cache->update(k, v, start_pos);
        k = kv.first.contiguous();
        v = kv.second.contiguous();
        int64_t n_rep = Hq / Hkv;
        k = vesper::ops::repeat_kv(k, n_rep);
        v = vesper::ops::repeat_kv(v, n_rep);
        Tensor o = vesper::nn::functional::scaled_dot_product_attention(tq, k, v, T > 1, 0.0);
        to_host(tq, q_rot);
        to_host(o, out);
    });
}

// BFloat16(float) / operator float (include/vesper/core/half.h:162-181).
// nn::Linear::forward (src/nn/linear.cpp:41-49) on a 3-D activation [B, T, K], the way the attention modules
// call their output projection (src/nn/gqa_attention.cpp:151-152): weight [N, K], bias [N] or NULL.
int vref_linear(const float* x, const float* w, const float* bias, float* y, int64_t B, int64_t T, int64_t K, int64_t N) {
    return guarded([&] {
        vesper::nn::Linear lin(K, N, bias != nullptr, Device::CPU);
        lin.weight.copy_from_host(w);
        if (bias) lin.bias.copy_from_host(bias);
        Tensor tx = from_host(x, {B, T, K});
        Tensor ty = lin.forward(tx);
        to_host(ty, y);
    });
}

uint16_t vref_f32_to_bf16(float f) { return vesper::BFloat16(f).to_bits(); }
float vref_bf16_to_f32(uint16_t b) { return float(vesper::BFloat16::from_bits(b)); }

}  // extern "C"
