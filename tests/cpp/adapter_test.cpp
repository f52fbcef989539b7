// Exercises the C++ mirror of the reference's operator surface (vesper_amd/csrc/adapter/vesper_adapter.hpp)
// the way the reference's own assert-style tests exercise the original, with the CPU oracle as checker.
//   adapter_test --cpu-only   host-side checks only (no GPU needed)
//   adapter_test              everything (needs a GPU)
#include <cmath>
#include <cstdio>
#include <cstdlib>
#include <cstring>
#include <string>
#include <vector>

#include "../../oracle/vsp_oracle.h"
#include "../../vesper_amd/csrc/adapter/vesper_adapter.hpp"

using namespace vesper_amd;

static int g_fail = 0;
#define CHECK(cond)                                                                  \
    do {                                                                             \
        if (!(cond)) {                                                               \
            std::printf("  CHECK FAILED %s:%d: %s\n", __FILE__, __LINE__, #cond);    \
            ++g_fail;                                                                \
        }                                                                            \
    } while (0)

template <class Ex, class F>
static std::string thrown(F&& f) {
    try {
        f();
    } catch (const Ex& e) {
        return e.what();
    } catch (...) {
        return "<other exception type>";
    }
    return "<nothing thrown>";
}

static std::vector<float> randn(size_t n, uint64_t seed, float scale = 1.0f) {
    std::vector<float> x(n);
    uint64_t s = seed * 0x9E3779B97F4A7C15ull + 1;
    auto next = [&]() {
        s ^= s << 13;
        s ^= s >> 7;
        s ^= s << 17;
        return (double)(s >> 11) / 9007199254740992.0;
    };
    for (size_t i = 0; i < n; i += 2) {
        double u1 = next() + 1e-12, u2 = next();
        double r = std::sqrt(-2.0 * std::log(u1));
        x[i] = (float)(r * std::cos(6.283185307179586 * u2)) * scale;
        if (i + 1 < n) x[i + 1] = (float)(r * std::sin(6.283185307179586 * u2)) * scale;
    }
    return x;
}
static std::vector<float> bf16_round(std::vector<float> x) {
    for (auto& f : x) f = orc_bf16_to_f32(orc_f32_to_bf16(f));
    return x;
}
static Tensor to_dev(const std::vector<float>& x, std::vector<int64_t> shape, DType dt) {
    Tensor t = empty(shape, dt);
    if (dt == DType::Float32) {
        t.copy_from_host(x.data());
    } else {
        std::vector<uint16_t> b(x.size());
        for (size_t i = 0; i < x.size(); ++i) b[i] = orc_f32_to_bf16(x[i]);
        t.copy_from_host(b.data());
    }
    return t;
}
static std::vector<float> to_host(const Tensor& t) {
    std::vector<float> out(t.numel());
    if (t.dtype() == DType::Float32) {
        t.copy_to_host(out.data());
    } else {
        std::vector<uint16_t> b(t.numel());
        t.copy_to_host(b.data());
        for (size_t i = 0; i < b.size(); ++i) out[i] = orc_bf16_to_f32(b[i]);
    }
    return out;
}
static double max_abs_diff(const std::vector<float>& a, const float* b, size_t n) {
    double m = 0;
    for (size_t i = 0; i < n; ++i) m = std::fmax(m, std::fabs((double)a[i] - (double)b[i]));
    return m;
}

// ---- host-only -------------------------------------------------------------------------------------
static void test_gqa_constructor_validation() {
    std::printf("test_gqa_constructor_validation\n");
    nn::GroupedQueryAttentionCore ok(64, 8, 2);
    CHECK(ok.head_dim() == 8 && ok.num_rep() == 4 && std::fabs(ok.kv_cache_ratio() - 0.25f) < 1e-7f);
    // src/nn/gqa_attention.cpp:47-57 messages, std::invalid_argument
    CHECK(thrown<std::invalid_argument>([] { nn::GroupedQueryAttentionCore m(64, 8, 3); }) ==
          "GroupedQueryAttention: num_heads (8) must be divisible by num_kv_heads (3)");
    CHECK(thrown<std::invalid_argument>([] { nn::GroupedQueryAttentionCore m(60, 8, 2); }) ==
          "GroupedQueryAttention: embed_dim (60) must be divisible by num_heads (8)");
    CHECK(std::fabs(nn::GQAKVCache::memory_savings(32, 8) - 0.75f) < 1e-7f);
    int64_t s, n;
    vsp_slice_bounds(10, 8, 12, &s, &n);  // clamped like ops::index
    CHECK(s == 8 && n == 2);
    CHECK(vsp_f32_to_bf16(1.00390625f) == orc_f32_to_bf16(1.00390625f));
}

// ---- GPU -------------------------------------------------------------------------------------------
static void test_kv_cache_basic() {  // reference tests/test_kv_cache.cpp:8-43
    std::printf("test_kv_cache_basic\n");
    const int B = 1, H = 1, S = 10, D = 4;
    nn::KVCache cache(B, H, S, D, Device::HIP);
    std::vector<float> ones(B * H * 2 * D, 1.0f), threes(B * H * 1 * D, 3.0f);
    Tensor k1 = to_dev(ones, {B, H, 2, D}, DType::Float32);
    auto kv1 = cache.update(k1, k1, 0);
    CHECK(cache.current_seq_len() == 2);
    CHECK(kv1.first.shape()[2] == 2);
    Tensor k2 = to_dev(threes, {B, H, 1, D}, DType::Float32);
    auto kv2 = cache.update(k2, k2, 2);
    CHECK(cache.current_seq_len() == 3);
    CHECK(kv2.first.shape()[2] == 3);
    CHECK((kv2.first.strides() == std::vector<int64_t>{H * S * D, S * D, D, 1}) && kv2.first.offset() == 0);
    auto host = to_host(kv2.first);
    CHECK(host[2 * D] == 3.0f && host[0] == 1.0f && host[D] == 1.0f);
    CHECK(cache.get_max_seq_len() == 10);
    // overflow: the reference clamps the slot and copy_from throws
    CHECK(thrown<std::runtime_error>([&] { cache.update(k1, k1, 9); }) == "copy_from: element count mismatch.");
    CHECK(cache.current_seq_len() == 3);
    cache.reset();
    CHECK(cache.current_seq_len() == 0);
}

static void test_flash_attention_against_oracle() {
    std::printf("test_flash_attention_against_oracle\n");
    const int64_t B = 2, H = 4, N = 96, D = 64;
    const float scale = 1.0f / std::sqrt((float)D);
    auto q = randn(B * H * N * D, 1), k = randn(B * H * N * D, 2), v = randn(B * H * N * D, 3);
    std::vector<float> want(q.size()), lse(B * H * N);
    for (int causal = 0; causal < 2; ++causal) {
        orc_flash_attention_f32(q.data(), k.data(), v.data(), want.data(), lse.data(), B, H, N, D, scale, causal);
        Tensor out = ops::flash_attention(to_dev(q, {B, H, N, D}, DType::Float32), to_dev(k, {B, H, N, D}, DType::Float32),
                                          to_dev(v, {B, H, N, D}, DType::Float32), scale, causal != 0);
        CHECK(max_abs_diff(to_host(out), want.data(), want.size()) < 1e-4);
        // the same fp32 tensors through the bf16 matrix cores (two bf16 terms per operand): inside the same bar, with room
        Tensor outs = ops::flash_attention_split(to_dev(q, {B, H, N, D}, DType::Float32), to_dev(k, {B, H, N, D}, DType::Float32),
                                                 to_dev(v, {B, H, N, D}, DType::Float32), scale, causal != 0);
        CHECK(max_abs_diff(to_host(outs), want.data(), want.size()) < 1e-4);
        CHECK(max_abs_diff(to_host(outs), to_host(out).data(), want.size()) < 5e-5);
        // and the process-wide switch that sends the reference-shaped call the same way
        ops::fp32_on_bf16_matrix_cores() = true;
        Tensor outw = ops::flash_attention(to_dev(q, {B, H, N, D}, DType::Float32), to_dev(k, {B, H, N, D}, DType::Float32),
                                           to_dev(v, {B, H, N, D}, DType::Float32), scale, causal != 0);
        ops::fp32_on_bf16_matrix_cores() = false;
        CHECK(max_abs_diff(to_host(outw), to_host(outs).data(), want.size()) == 0.0);
        auto qb = bf16_round(q), kb = bf16_round(k), vb = bf16_round(v);
        orc_flash_attention_f32(qb.data(), kb.data(), vb.data(), want.data(), lse.data(), B, H, N, D, scale, causal);
        Tensor outb = ops::flash_attention(to_dev(qb, {B, H, N, D}, DType::BFloat16), to_dev(kb, {B, H, N, D}, DType::BFloat16),
                                           to_dev(vb, {B, H, N, D}, DType::BFloat16), scale, causal != 0);
        CHECK(max_abs_diff(to_host(outb), want.data(), want.size()) < 2e-2);
    }
    // backward on the forward's own output and log-sum-exp (reference tests/test_flash_attention.cpp:292-340)
    {
        auto dout = randn(B * H * N * D, 4);
        orc_flash_attention_f32(q.data(), k.data(), v.data(), want.data(), lse.data(), B, H, N, D, scale, 1);
        std::vector<float> wq(q.size()), wk(q.size()), wv(q.size());
        orc_flash_attention_backward_f32(dout.data(), q.data(), k.data(), v.data(), want.data(), lse.data(), wq.data(), wk.data(),
                                         wv.data(), B, H, N, D, scale, 1);
        Tensor tq = to_dev(q, {B, H, N, D}, DType::Float32), tk = to_dev(k, {B, H, N, D}, DType::Float32);
        Tensor tv = to_dev(v, {B, H, N, D}, DType::Float32), tdo = to_dev(dout, {B, H, N, D}, DType::Float32);
        Tensor out = empty({B, H, N, D}, DType::Float32), l = empty({B, H, N}, DType::Float32);
        ops::flash_attention_hip_dispatch(tq, tk, tv, out, l, scale, true, 0.0f, false, nullptr);
        auto g = ops::flash_attention_backward(tdo, tq, tk, tv, out, l, scale, true);
        CHECK(max_abs_diff(to_host(std::get<0>(g)), wq.data(), wq.size()) < 2e-4);
        CHECK(max_abs_diff(to_host(std::get<1>(g)), wk.data(), wk.size()) < 2e-4);
        CHECK(max_abs_diff(to_host(std::get<2>(g)), wv.data(), wv.size()) < 2e-4);
        // the process-wide switch sends the same call through the split-operand backward (fp32 tensors, bf16 matrix cores)
        ops::fp32_on_bf16_matrix_cores() = true;
        auto gs = ops::flash_attention_backward(tdo, tq, tk, tv, out, l, scale, true);
        ops::fp32_on_bf16_matrix_cores() = false;
        CHECK(max_abs_diff(to_host(std::get<0>(gs)), wq.data(), wq.size()) < 2e-4);
        CHECK(max_abs_diff(to_host(std::get<1>(gs)), wk.data(), wk.size()) < 2e-4);
        CHECK(max_abs_diff(to_host(std::get<2>(gs)), wv.data(), wv.size()) < 2e-4);
        CHECK(max_abs_diff(to_host(std::get<0>(gs)), to_host(std::get<0>(g)).data(), wq.size()) > 0.0);   // it is the other kernel
    }
    // the reference's validation messages (src/ops/flash_attention.cpp:45-59)
    Tensor a = empty({1, 2, 4, 64}, DType::Float32), b = empty({1, 2, 5, 64}, DType::Float32), c3 = empty({2, 4, 64}, DType::Float32);
    CHECK(thrown<std::runtime_error>([&] { ops::flash_attention(c3, c3, c3, 1.f); }) == "flash_attention: inputs must be 4D [B, H, N, D]");
    CHECK(thrown<std::runtime_error>([&] { ops::flash_attention(a, b, a, 1.f); }) == "flash_attention: Q, K, V must have same shape");
    CHECK(thrown<std::runtime_error>([&] { ops::flash_attention(a, a, empty({1, 2, 4, 64}, DType::BFloat16), 1.f); }) ==
          "flash_attention: Q, K, V must have same dtype");
    CHECK(thrown<std::runtime_error>([&] { ops::flash_attention(a, a, a, 1.f, true, 1.0f); }) == "flash_attention: dropout_p must be in [0, 1)");
}

template <typename CacheT>
static void run_cached_generation(KVFormat fmt, DType dt, double tol, const char* name) {
    // reference tests/test_kv_cache_chapter33.cpp:66-188 and tests/test_gqa_chapter33.cpp:236-271 (intent):
    // prefill 8 tokens through the cache, then decode token by token; every step equals the causal full forward.
    std::printf("test_cached_generation[%s]\n", name);
    const int64_t B = 2, Hq = 8, Hkv = 2, D = 64, T0 = 8, steps = 5, N = T0 + steps, S_max = 32;
    nn::GroupedQueryAttentionCore attn(Hq * D, Hq, Hkv);
    auto q = randn(B * Hq * N * D, 11, 0.5f), k = randn(B * Hkv * N * D, 12, 0.5f), v = randn(B * Hkv * N * D, 13, 0.5f);
    if (dt == DType::BFloat16) q = bf16_round(q), k = bf16_round(k), v = bf16_round(v);
    std::vector<float> kq = k, vq = v;
    if (fmt == KVFormat::Q8_0) {  // the oracle attends over what the cache holds: the dequantised rows
        std::vector<uint16_t> d(k.size() / 32);
        std::vector<int8_t> qs(k.size());
        orc_q8_0_quantize_row(k.data(), (int64_t)k.size(), d.data(), qs.data());
        orc_q8_0_dequantize_row(d.data(), qs.data(), (int64_t)k.size(), kq.data());
        orc_q8_0_quantize_row(v.data(), (int64_t)v.size(), d.data(), qs.data());
        orc_q8_0_dequantize_row(d.data(), qs.data(), (int64_t)v.size(), vq.data());
    }
    // oracle: full causal GQA attention over all N tokens (matmul/softmax branch, N < 512)
    std::vector<float> want(q.size());
    int64_t st[4] = {Hkv * N * D, N * D, D, 1};
    CHECK(orc_gqa_attention_f32(q.data(), kq.data(), st, vq.data(), st, want.data(), B, Hq, N, N, D, Hq / Hkv, 1) == 0);
    auto slice = [&](const std::vector<float>& x, int64_t H, int64_t t0, int64_t t1) {
        std::vector<float> out((size_t)(B * H * (t1 - t0) * D));
        for (int64_t b = 0; b < B; ++b)
            for (int64_t h = 0; h < H; ++h)
                for (int64_t t = t0; t < t1; ++t)
                    std::memcpy(&out[(size_t)(((b * H + h) * (t1 - t0) + (t - t0)) * D)], &x[(size_t)(((b * H + h) * N + t) * D)], D * sizeof(float));
        return out;
    };
    CacheT cache(B, Hkv, S_max, D, Device::HIP, fmt);
    auto step = [&](int64_t t0, int64_t t1) {
        Tensor tq = to_dev(slice(q, Hq, t0, t1), {B, Hq, t1 - t0, D}, dt);
        Tensor tk = to_dev(slice(k, Hkv, t0, t1), {B, Hkv, t1 - t0, D}, dt);
        Tensor tv = to_dev(slice(v, Hkv, t0, t1), {B, Hkv, t1 - t0, D}, dt);
        Tensor out = attn.forward(tq, tk, tv, &cache, t0);
        auto got = to_host(out), w = slice(want, Hq, t0, t1);
        double err = max_abs_diff(got, w.data(), w.size());
        if (!(err < tol)) std::printf("  step [%ld,%ld): max-abs %.3g\n", (long)t0, (long)t1, err);
        CHECK(err < tol);
        CHECK((int64_t)cache.current_seq_len() == t1);
    };
    step(0, T0);
    for (int64_t t = T0; t < N; ++t) step(t, t + 1);
}

template <class CacheT>
static void run_rope_generation(KVFormat fmt, DType qdt, double tol, const char* name) {
    // GroupedQueryAttention::forward(x, cache, start_pos) from RoPE on (src/nn/gqa_attention.cpp:124-148):
    // prefill 8 tokens, then token by token; each step equals the causal full forward over rotated q, k.
    std::printf("test_rope_generation[%s]\n", name);
    const int64_t B = 2, Hq = 8, Hkv = 2, D = 64, T0 = 8, steps = 4, N = T0 + steps, S_max = 32;
    nn::GroupedQueryAttentionCore attn(Hq * D, Hq, Hkv);
    nn::RopeTable rope(S_max, D);
    auto q = randn(B * Hq * N * D, 31, 0.5f), k = randn(B * Hkv * N * D, 32, 0.5f), v = randn(B * Hkv * N * D, 33, 0.5f);
    std::vector<float> ang((size_t)(N * D / 2)), qr(q.size()), kr(k.size());
    orc_rope_angles((int)N, (int)D, 0, 10000.0f, ang.data());
    orc_rope_apply_f32(q.data(), B, Hq, N, D, ang.data(), qr.data());
    orc_rope_apply_f32(k.data(), B, Hkv, N, D, ang.data(), kr.data());
    std::vector<float> want(q.size());
    int64_t st[4] = {Hkv * N * D, N * D, D, 1};
    CHECK(orc_gqa_attention_f32(qr.data(), kr.data(), st, v.data(), st, want.data(), B, Hq, N, N, D, Hq / Hkv, 1) == 0);
    auto slice = [&](const std::vector<float>& x, int64_t H, int64_t t0, int64_t t1) {
        std::vector<float> out((size_t)(B * H * (t1 - t0) * D));
        for (int64_t b = 0; b < B; ++b)
            for (int64_t h = 0; h < H; ++h)
                for (int64_t t = t0; t < t1; ++t)
                    std::memcpy(&out[(size_t)(((b * H + h) * (t1 - t0) + (t - t0)) * D)], &x[(size_t)(((b * H + h) * N + t) * D)], D * sizeof(float));
        return out;
    };
    CacheT cache(B, Hkv, S_max, D, Device::HIP, fmt);
    auto step = [&](int64_t t0, int64_t t1) {
        Tensor tq = to_dev(slice(q, Hq, t0, t1), {B, Hq, t1 - t0, D}, DType::Float32);
        Tensor tk = to_dev(slice(k, Hkv, t0, t1), {B, Hkv, t1 - t0, D}, DType::Float32);
        Tensor tv = to_dev(slice(v, Hkv, t0, t1), {B, Hkv, t1 - t0, D}, DType::Float32);
        Tensor out = attn.forward_rope(tq, tk, tv, &cache, t0, rope, qdt);
        auto got = to_host(out), w = slice(want, Hq, t0, t1);
        double err = max_abs_diff(got, w.data(), w.size());
        if (!(err < tol)) std::printf("  step [%ld,%ld): max-abs %.3g\n", (long)t0, (long)t1, err);
        CHECK(err < tol);
        CHECK((int64_t)cache.current_seq_len() == t1);
    };
    step(0, T0);
    for (int64_t t = T0; t < N; ++t) step(t, t + 1);
    // the same 12 tokens as a prompt processed in chunks of 8 + 4 (start_pos > 0 with T > 1)
    {
        CacheT cc(B, Hkv, S_max, D, Device::HIP, fmt);
        int64_t bounds[3] = {0, 8, N};
        for (int ci = 0; ci < 2; ++ci) {
            const int64_t t0 = bounds[ci], t1 = bounds[ci + 1];
            Tensor tq = to_dev(slice(q, Hq, t0, t1), {B, Hq, t1 - t0, D}, DType::Float32);
            Tensor tk = to_dev(slice(k, Hkv, t0, t1), {B, Hkv, t1 - t0, D}, DType::Float32);
            Tensor tv = to_dev(slice(v, Hkv, t0, t1), {B, Hkv, t1 - t0, D}, DType::Float32);
            Tensor out = attn.forward_chunk(tq, tk, tv, &cc, t0, rope, qdt);
            auto got = to_host(out), w = slice(want, Hq, t0, t1);
            double err = max_abs_diff(got, w.data(), w.size());
            if (!(err < tol)) std::printf("  chunk [%ld,%ld): max-abs %.3g\n", (long)t0, (long)t1, err);
            CHECK(err < tol);
        }
        CHECK((int64_t)cc.current_seq_len() == N);
    }
    // positions outside the table are refused, nothing is written
    nn::RopeTable small(4, D);
    Tensor tq = to_dev(slice(q, Hq, 0, 8), {B, Hq, 8, D}, DType::Float32);
    Tensor tk = to_dev(slice(k, Hkv, 0, 8), {B, Hkv, 8, D}, DType::Float32);
    CacheT c2(B, Hkv, S_max, D, Device::HIP, fmt);
    CHECK(thrown<std::runtime_error>([&] { attn.forward_rope(tq, tk, tk, &c2, 0, small, qdt); }) != "<nothing thrown>");
    CHECK(c2.current_seq_len() == 0);
}

static void run_token_with_output_projection(KVFormat fmt, DType dt, double tol, const char* name) {
    // GroupedQueryAttention::forward(x, cache, start_pos) for one generated token, through wo_ (src/nn/gqa_attention.cpp:124-152):
    // the fused call equals the step-by-step route (attention output, heads merged, Linear::forward by the oracle)
    std::printf("test_token_with_output_projection[%s]\n", name);
    const int64_t B = 3, Hq = 8, Hkv = 2, D = 64, T0 = 9, S_max = 32, C = Hq * D;
    nn::GroupedQueryAttentionCore attn(C, Hq, Hkv);
    nn::RopeTable rope(S_max, D);
    auto round = [&](std::vector<float> x) { return dt == DType::BFloat16 ? bf16_round(std::move(x)) : x; };
    auto q0 = round(randn(B * Hq * T0 * D, 61, 0.5f)), k0 = round(randn(B * Hkv * T0 * D, 62, 0.5f)), v0 = round(randn(B * Hkv * T0 * D, 63, 0.5f));
    auto q1 = round(randn(B * Hq * D, 64, 0.5f)), k1 = round(randn(B * Hkv * D, 65, 0.5f)), v1 = round(randn(B * Hkv * D, 66, 0.5f));
    auto w = round(randn(C * C, 67, 1.0f / std::sqrt((float)C))), bias = round(randn(C, 68, 0.5f));
    Tensor tw = to_dev(w, {C, C}, dt), tb = to_dev(bias, {C}, dt);
    nn::KVCache ca(B, Hkv, S_max, D, Device::HIP, fmt), cb(B, Hkv, S_max, D, Device::HIP, fmt);
    for (nn::KVCache* c : {&ca, &cb})
        attn.forward_rope(to_dev(q0, {B, Hq, T0, D}, dt), to_dev(k0, {B, Hkv, T0, D}, dt), to_dev(v0, {B, Hkv, T0, D}, dt), c, 0, rope, dt);
    Tensor o = attn.forward_rope(to_dev(q1, {B, Hq, 1, D}, dt), to_dev(k1, {B, Hkv, 1, D}, dt), to_dev(v1, {B, Hkv, 1, D}, dt), &ca, T0, rope, dt);
    auto x = to_host(o);  // [B,Hq,1,D] == [B,1,C] once the heads are merged (T == 1)
    for (int with_bias = 0; with_bias < 2; ++with_bias) {
        nn::KVCache cc(B, Hkv, S_max, D, Device::HIP, fmt);
        attn.forward_rope(to_dev(q0, {B, Hq, T0, D}, dt), to_dev(k0, {B, Hkv, T0, D}, dt), to_dev(v0, {B, Hkv, T0, D}, dt), &cc, 0, rope, dt);
        Tensor y = attn.forward_token_proj(to_dev(q1, {B, Hq, 1, D}, dt), to_dev(k1, {B, Hkv, 1, D}, dt), to_dev(v1, {B, Hkv, 1, D}, dt), &cc, T0,
                                           rope, dt, tw, with_bias ? &tb : nullptr);
        CHECK(y.ndim() == 3 && y.shape()[0] == B && y.shape()[1] == 1 && y.shape()[2] == C);
        CHECK((int64_t)cc.current_seq_len() == T0 + 1);
        std::vector<float> want((size_t)(B * C));
        orc_linear_f32(x.data(), w.data(), with_bias ? bias.data() : nullptr, want.data(), B, C, C);
        double err = max_abs_diff(to_host(y), want.data(), want.size());
        if (!(err < tol)) std::printf("  bias %d: max-abs %.3g\n", with_bias, err);
        CHECK(err < tol);
    }
    // a weight whose inner size is not Hq * D is refused with the shape error
    Tensor bad = to_dev(std::vector<float>((size_t)(C * (C - 8))), {C, C - 8}, dt);
    CHECK(thrown<std::runtime_error>([&] {
              attn.forward_token_proj(to_dev(q1, {B, Hq, 1, D}, dt), to_dev(k1, {B, Hkv, 1, D}, dt), to_dev(v1, {B, Hkv, 1, D}, dt), &cb, T0, rope, dt, bad);
          }) != "<nothing thrown>");
}

static void test_sdpa_routing() {
    std::printf("test_sdpa_routing\n");
    const int64_t B = 1, H = 2, D = 64;
    // cross shapes, non-causal (reference tests/test_attention_chapter32.cpp:135-162)
    auto q = randn(B * H * 16 * D, 21), k = randn(B * H * 40 * D, 22), v = randn(B * H * 40 * D, 23);
    std::vector<float> want(q.size());
    orc_sdpa_f32(q.data(), k.data(), v.data(), want.data(), B, H, 16, 40, D, 0);
    Tensor out = nn::functional::scaled_dot_product_attention(to_dev(q, {B, H, 16, D}, DType::Float32), to_dev(k, {B, H, 40, D}, DType::Float32),
                                                              to_dev(v, {B, H, 40, D}, DType::Float32), false);
    CHECK(max_abs_diff(to_host(out), want.data(), want.size()) < 1e-4);
    // causal with T != L does not broadcast in the reference
    CHECK(thrown<std::runtime_error>([&] {
              nn::functional::scaled_dot_product_attention(to_dev(q, {B, H, 16, D}, DType::Float32), to_dev(k, {B, H, 40, D}, DType::Float32),
                                                           to_dev(v, {B, H, 40, D}, DType::Float32), true);
          }) == "causal mask [T, T] cannot be broadcast onto scores [T, L]");
    // repeat_kv head map, reference tests/test_gqa_chapter33.cpp:76-118: constant V per kv head
    std::vector<float> vv(B * 2 * 8 * D);
    for (size_t i = 0; i < vv.size(); ++i) vv[i] = i < vv.size() / 2 ? 1.0f : 3.0f;
    auto q8 = randn(B * 8 * 8 * D, 24), k8 = randn(B * 2 * 8 * D, 25);
    Tensor o8 = nn::functional::scaled_dot_product_attention(to_dev(q8, {B, 8, 8, D}, DType::Float32),
                                                             ops::repeat_kv(to_dev(k8, {B, 2, 8, D}, DType::Float32), 4),
                                                             ops::repeat_kv(to_dev(vv, {B, 2, 8, D}, DType::Float32), 4), true);
    auto h8 = to_host(o8);
    bool ok = true;
    for (int64_t h = 0; h < 8; ++h)
        for (int64_t i = 0; i < 8 * D; ++i) ok = ok && std::fabs(h8[(size_t)(h * 8 * D + i)] - (h < 4 ? 1.0f : 3.0f)) < 1e-5f;
    CHECK(ok);
}

static void test_backward_dispatch_seam() {
    // flash_attention_backward_hip_dispatch with the reference's parameter list (include/vesper/ops/flash_attention.h:80-92):
    // caller-allocated gradients, GQA operands (dk/dv summed over each group's query heads), dropout mask refused.
    std::printf("test_backward_dispatch_seam\n");
    const int64_t B = 1, Hq = 4, Hkv = 2, N = 40, D = 64, n = Hq / Hkv;
    const float scale = 1.0f / std::sqrt((float)D);
    auto q = randn(B * Hq * N * D, 41), k = randn(B * Hkv * N * D, 42), v = randn(B * Hkv * N * D, 43), dout = randn(B * Hq * N * D, 44);
    // oracle on repeated K/V, then the group sums
    std::vector<float> kr(q.size()), vr(q.size()), out(q.size()), lse(B * Hq * N), wq(q.size()), wkr(q.size()), wvr(q.size());
    for (int64_t h = 0; h < Hq; ++h) {
        std::memcpy(&kr[(size_t)(h * N * D)], &k[(size_t)((h / n) * N * D)], N * D * sizeof(float));
        std::memcpy(&vr[(size_t)(h * N * D)], &v[(size_t)((h / n) * N * D)], N * D * sizeof(float));
    }
    orc_flash_attention_f32(q.data(), kr.data(), vr.data(), out.data(), lse.data(), B, Hq, N, D, scale, 1);
    orc_flash_attention_backward_f32(dout.data(), q.data(), kr.data(), vr.data(), out.data(), lse.data(), wq.data(), wkr.data(), wvr.data(),
                                     B, Hq, N, D, scale, 1);
    std::vector<float> wk(k.size(), 0.f), wv(v.size(), 0.f);
    for (int64_t h = 0; h < Hq; ++h)
        for (int64_t i = 0; i < N * D; ++i) {
            wk[(size_t)((h / n) * N * D + i)] += wkr[(size_t)(h * N * D + i)];
            wv[(size_t)((h / n) * N * D + i)] += wvr[(size_t)(h * N * D + i)];
        }
    Tensor tq = to_dev(q, {B, Hq, N, D}, DType::Float32), tk = to_dev(k, {B, Hkv, N, D}, DType::Float32);
    Tensor tv = to_dev(v, {B, Hkv, N, D}, DType::Float32), tdo = to_dev(dout, {B, Hq, N, D}, DType::Float32);
    Tensor o = empty({B, Hq, N, D}, DType::Float32), l = empty({B, Hq, N}, DType::Float32);
    ops::flash_attention_hip_dispatch(tq, ops::repeat_kv(tk, n), ops::repeat_kv(tv, n), o, l, scale, true, 0.0f, false, nullptr);
    Tensor gq = empty({B, Hq, N, D}, DType::Float32), gk = empty({B, Hkv, N, D}, DType::Float32), gv = empty({B, Hkv, N, D}, DType::Float32);
    ops::flash_attention_backward_hip_dispatch(tdo, tq, tk, tv, o, l, gq, gk, gv, scale, true, 0.0f, nullptr);
    CHECK(max_abs_diff(to_host(gq), wq.data(), wq.size()) < 2e-4);
    CHECK(max_abs_diff(to_host(gk), wk.data(), wk.size()) < 4e-4);
    CHECK(max_abs_diff(to_host(gv), wv.data(), wv.size()) < 4e-4);
    // a dropout mask (training with p > 0) is not implemented: refused, as the forward refuses to produce one
    Tensor mask = empty({B, Hq, N, N}, DType::Float32);
    CHECK(thrown<std::runtime_error>([&] { ops::flash_attention_backward_hip_dispatch(tdo, tq, tk, tv, o, l, gq, gk, gv, scale, true, 0.1f, &mask); }) !=
          "<nothing thrown>");
    // the front end with the reference's defaults (is_causal = true, dropout_p = 0, no mask)
    auto g = ops::flash_attention_backward(tdo, tq, tk, tv, o, l, scale);
    CHECK(max_abs_diff(to_host(std::get<0>(g)), wq.data(), wq.size()) < 2e-4);
    // bf16 tensors: with the larger workspace (taken from backward_fast_min_context() tokens on while it stays under
    // backward_fast_workspace_limit()) dS is computed once, with the limit at 0 twice; both inside the bf16 bar against the
    // fp32 oracle, and dK / dV the same
    {
        Tensor bq = to_dev(q, {B, Hq, N, D}, DType::BFloat16), bk = to_dev(k, {B, Hkv, N, D}, DType::BFloat16);
        Tensor bv = to_dev(v, {B, Hkv, N, D}, DType::BFloat16), bdo = to_dev(dout, {B, Hq, N, D}, DType::BFloat16);
        Tensor bo = empty({B, Hq, N, D}, DType::BFloat16), bl = empty({B, Hq, N}, DType::Float32);
        ops::flash_attention_hip_dispatch(bq, ops::repeat_kv(bk, n), ops::repeat_kv(bv, n), bo, bl, scale, true, 0.0f, false, nullptr);
        const int64_t keep_n = ops::backward_fast_min_context();
        ops::backward_fast_min_context() = 1;
        const size_t taken = BlockCache::instance().bytes_taken();
        auto once = ops::flash_attention_backward(bdo, bq, bk, bv, bo, bl, scale);
        CHECK(BlockCache::instance().bytes_taken() - taken >= vsp_attn_backward_fast_workspace_bytes((int32_t)B, (int32_t)Hq, (int32_t)N));
        ops::backward_fast_min_context() = keep_n;
        const size_t keep = ops::backward_fast_workspace_limit();
        ops::backward_fast_workspace_limit() = 0;
        auto twice = ops::flash_attention_backward(bdo, bq, bk, bv, bo, bl, scale);
        ops::backward_fast_workspace_limit() = keep;
        CHECK(max_abs_diff(to_host(std::get<0>(once)), wq.data(), wq.size()) < 3e-2);
        CHECK(max_abs_diff(to_host(std::get<0>(twice)), wq.data(), wq.size()) < 3e-2);
        CHECK(max_abs_diff(to_host(std::get<1>(once)), wk.data(), wk.size()) < 5e-2);
        CHECK(max_abs_diff(to_host(std::get<2>(once)), wv.data(), wv.size()) < 5e-2);
        auto dk1 = to_host(std::get<1>(once)), dk2 = to_host(std::get<1>(twice));
        CHECK(max_abs_diff(dk1, dk2.data(), dk2.size()) < 1e-2);
    }
}

static void test_multi_head_attention_core() {
    // MultiHeadAttention's three forward overloads (src/nn/transformer.cpp:108-216) on the attention core
    std::printf("test_multi_head_attention_core\n");
    const int64_t B = 2, H = 4, T = 24, D = 64;
    auto q = randn(B * H * T * D, 51, 0.5f), k = randn(B * H * T * D, 52, 0.5f), v = randn(B * H * T * D, 53, 0.5f);
    std::vector<float> want(q.size());
    Tensor tq = to_dev(q, {B, H, T, D}, DType::Float32), tk = to_dev(k, {B, H, T, D}, DType::Float32), tv = to_dev(v, {B, H, T, D}, DType::Float32);
    {   // use_rope = false: forward(x) is NOT causal (:108-110); forward(x, true) is
        nn::MultiHeadAttentionCore mha((int)(H * D), (int)H, 0.0f, false);
        orc_sdpa_f32(q.data(), k.data(), v.data(), want.data(), B, H, T, T, D, 0);
        CHECK(max_abs_diff(to_host(mha.forward(tq, tk, tv)), want.data(), want.size()) < 1e-4);
        orc_sdpa_f32(q.data(), k.data(), v.data(), want.data(), B, H, T, T, D, 1);
        CHECK(max_abs_diff(to_host(mha.forward(tq, tk, tv, true)), want.data(), want.size()) < 1e-4);
        // the default really is the non-causal result: it differs from the causal one
        CHECK(max_abs_diff(to_host(mha.forward(tq, tk, tv)), want.data(), want.size()) > 1e-3);
    }
    {   // use_rope = true (the constructor's default): q, k rotated at positions 0.. (:132-136), fp32 and bf16
        nn::MultiHeadAttentionCore mha((int)(H * D), (int)H);
        std::vector<float> ang((size_t)(T * D / 2)), qr(q.size()), kr(k.size());
        orc_rope_angles((int)T, (int)D, 0, 10000.0f, ang.data());
        orc_rope_apply_f32(q.data(), B, H, T, D, ang.data(), qr.data());
        orc_rope_apply_f32(k.data(), B, H, T, D, ang.data(), kr.data());
        for (int causal = 0; causal < 2; ++causal) {
            orc_sdpa_f32(qr.data(), kr.data(), v.data(), want.data(), B, H, T, T, D, causal);
            Tensor got = causal ? mha.forward(tq, tk, tv, true) : mha.forward(tq, tk, tv);
            CHECK(max_abs_diff(to_host(got), want.data(), want.size()) < 1e-4);
        }
        auto qb = bf16_round(q), kb = bf16_round(k), vb = bf16_round(v);
        orc_rope_apply_f32(qb.data(), B, H, T, D, ang.data(), qr.data());
        orc_rope_apply_f32(kb.data(), B, H, T, D, ang.data(), kr.data());
        auto qrb = bf16_round(qr), krb = bf16_round(kr);
        orc_sdpa_f32(qrb.data(), krb.data(), vb.data(), want.data(), B, H, T, T, D, 0);
        Tensor gb = mha.forward(to_dev(qb, {B, H, T, D}, DType::BFloat16), to_dev(kb, {B, H, T, D}, DType::BFloat16),
                                to_dev(vb, {B, H, T, D}, DType::BFloat16));
        CHECK(max_abs_diff(to_host(gb), want.data(), want.size()) < 2e-2);
        // forward(x, cache, start_pos): prefill 16 tokens (causal because T > 1), then token by token (:166-216)
        nn::KVCache cache((int)B, (int)H, 64, (int)D, Device::HIP);
        orc_sdpa_f32(qr.data(), kr.data(), v.data(), want.data(), B, H, T, T, D, 1);  // overwritten below with fp32 rotation
        orc_rope_apply_f32(q.data(), B, H, T, D, ang.data(), qr.data());
        orc_rope_apply_f32(k.data(), B, H, T, D, ang.data(), kr.data());
        orc_sdpa_f32(qr.data(), kr.data(), v.data(), want.data(), B, H, T, T, D, 1);
        auto slice = [&](const std::vector<float>& x, int64_t t0, int64_t t1) {
            std::vector<float> out((size_t)(B * H * (t1 - t0) * D));
            for (int64_t bh = 0; bh < B * H; ++bh)
                for (int64_t t = t0; t < t1; ++t)
                    std::memcpy(&out[(size_t)((bh * (t1 - t0) + (t - t0)) * D)], &x[(size_t)((bh * T + t) * D)], D * sizeof(float));
            return out;
        };
        auto step = [&](int64_t t0, int64_t t1) {
            Tensor out = mha.forward(to_dev(slice(q, t0, t1), {B, H, t1 - t0, D}, DType::Float32),
                                     to_dev(slice(k, t0, t1), {B, H, t1 - t0, D}, DType::Float32),
                                     to_dev(slice(v, t0, t1), {B, H, t1 - t0, D}, DType::Float32), &cache, (int)t0);
            auto w = slice(want, t0, t1);
            CHECK(max_abs_diff(to_host(out), w.data(), w.size()) < 1e-4);
            CHECK(cache.current_seq_len() == (int)t1);
        };
        step(0, 16);
        for (int64_t t = 16; t < T; ++t) step(t, t + 1);
        // forward(x, nullptr, start_pos) with RoPE and no cache (:187-191): rotated as positions start_pos.., attention
        // over exactly these T tokens; and what the call takes from the allocator does not grow with the position
        {
            const int64_t T2 = 16;
            auto check_at = [&](int64_t pos) {
                std::vector<float> a2((size_t)(T2 * D / 2)), q2(B * H * T2 * D), k2(q2.size()), w2(q2.size());
                auto qs = slice(q, 0, T2), ks = slice(k, 0, T2), vs = slice(v, 0, T2);
                orc_rope_angles((int)T2, (int)D, (int)pos, 10000.0f, a2.data());
                orc_rope_apply_f32(qs.data(), B, H, T2, D, a2.data(), q2.data());
                orc_rope_apply_f32(ks.data(), B, H, T2, D, a2.data(), k2.data());
                orc_sdpa_f32(q2.data(), k2.data(), vs.data(), w2.data(), B, H, T2, T2, D, 1);
                const size_t before = BlockCache::instance().bytes_taken();
                Tensor out = mha.forward(to_dev(qs, {B, H, T2, D}, DType::Float32), to_dev(ks, {B, H, T2, D}, DType::Float32),
                                         to_dev(vs, {B, H, T2, D}, DType::Float32), (nn::KVCache*)nullptr, (int)pos);
                const size_t taken = BlockCache::instance().bytes_taken() - before;
                CHECK(max_abs_diff(to_host(out), w2.data(), w2.size()) < 1e-4);
                return taken;
            };
            check_at(3000);  // (builds the RoPE table that covers every position used below)
            const size_t at0 = check_at(0), at3000 = check_at(3000), at7 = check_at(7);
            if (!(at0 == at3000 && at0 == at7)) std::printf("  bytes taken at 0 / 7 / 3000: %zu %zu %zu\n", at0, at7, at3000);
            CHECK(at0 == at3000 && at0 == at7);
        }
        // training-mode attention dropout is not implemented on this path
        nn::MultiHeadAttentionCore drop((int)(H * D), (int)H, 0.1f, false);
        drop.train();
        CHECK(thrown<std::runtime_error>([&] { drop.forward(tq, tk, tv); }) != "<nothing thrown>");
        drop.eval();
        orc_sdpa_f32(q.data(), k.data(), v.data(), want.data(), B, H, T, T, D, 0);
        CHECK(max_abs_diff(to_host(drop.forward(tq, tk, tv)), want.data(), want.size()) < 1e-4);
    }
}

static void test_chunk_of_a_long_prompt_splits_the_context() {
    // KVCache::attend with the last 96 tokens of a 4192-token context (bf16 cache, head_dim 128): 8 workgroups of queries
    // for the whole chip, so attend() brings the split workspace and the library cuts the context into shares.  Expected:
    // the rows of the causal forward over the whole context, in double precision on the values the cache holds.
    std::printf("test_chunk_of_a_long_prompt_splits_the_context\n");
    const int64_t B = 1, Hq = 8, Hkv = 2, D = 128, L = 4192, T = 96, S_max = 4224, n_rep = Hq / Hkv;
    auto k = bf16_round(randn(B * Hkv * L * D, 71, 0.5f)), v = bf16_round(randn(B * Hkv * L * D, 72, 0.5f));
    auto q = bf16_round(randn(B * Hq * T * D, 73, 0.5f));
    nn::GQAKVCache cache(B, Hkv, S_max, D, Device::HIP, KVFormat::BFloat16);
    cache.update(to_dev(k, {B, Hkv, L, D}, DType::BFloat16), to_dev(v, {B, Hkv, L, D}, DType::BFloat16), 0);
    CHECK(vsp_attn_prefill_cached_split_workspace_bytes(&cache.raw(), 0, 0, (int32_t)Hq, (int32_t)T) > 0);
    auto got = to_host(cache.attend(to_dev(q, {B, Hq, T, D}, DType::BFloat16), true));
    const double scale = 1.0 / std::sqrt((double)D);
    double worst = 0;
    std::vector<double> s((size_t)L), o((size_t)D);
    for (int64_t h = 0; h < Hq; ++h)
        for (int64_t t = 0; t < T; t += 5) {  // every fifth row
            const int64_t last = L - T + t;  // keys [0, last]
            const float* qp = &q[(size_t)((h * T + t) * D)];
            const float* kp = &k[(size_t)((h / n_rep) * L * D)];
            const float* vp = &v[(size_t)((h / n_rep) * L * D)];
            double m = -1e300, l = 0;
            for (int64_t j = 0; j <= last; ++j) {
                double d = 0;
                for (int64_t e = 0; e < D; ++e) d += (double)qp[e] * kp[j * D + e];
                s[(size_t)j] = d * scale;
                m = std::fmax(m, s[(size_t)j]);
            }
            std::fill(o.begin(), o.end(), 0.0);
            for (int64_t j = 0; j <= last; ++j) {
                const double p = std::exp(s[(size_t)j] - m);
                l += p;
                for (int64_t e = 0; e < D; ++e) o[(size_t)e] += p * vp[j * D + e];
            }
            for (int64_t e = 0; e < D; ++e) worst = std::fmax(worst, std::fabs(o[(size_t)e] / l - (double)got[(size_t)((h * T + t) * D + e)]));
        }
    if (!(worst < 2e-2)) std::printf("  max-abs %.3g\n", worst);
    CHECK(worst < 2e-2);
}

static void test_token_loop_allocates_nothing_and_keeps_pace() {
    // One decode step of the drop-in layer = forward_rope (RoPE + append, split-K decode + combine).  After warm-up the
    // step must not reach the driver's allocator and must not wait for the stream; its time per token is compared with
    // the same three launches issued straight through the C ABI on preallocated buffers.
    std::printf("test_token_loop_allocates_nothing_and_keeps_pace\n");
    const int64_t B = 32, Hq = 32, Hkv = 8, D = 128, S_max = 4096, L0 = 2048, tokens = 64;
    nn::GroupedQueryAttentionCore attn(Hq * D, Hq, Hkv);
    nn::RopeTable rope(S_max, D);
    nn::GQAKVCache cache(B, Hkv, S_max, D, Device::HIP, KVFormat::BFloat16);
    {   // a context of L0 tokens
        Tensor k0 = to_dev(randn(B * Hkv * L0 * D, 61, 0.5f), {B, Hkv, L0, D}, DType::BFloat16);
        cache.update(k0, k0, 0);
    }
    Tensor tq = to_dev(randn(B * Hq * D, 62, 0.5f), {B, Hq, 1, D}, DType::BFloat16);
    Tensor tk = to_dev(randn(B * Hkv * D, 63, 0.5f), {B, Hkv, 1, D}, DType::BFloat16);
    hipEvent_t e0, e1;
    hip_check(hipEventCreate(&e0), "event");
    hip_check(hipEventCreate(&e1), "event");
    auto adapter_loop = [&](int64_t pos0) {
        for (int64_t t = 0; t < tokens; ++t) (void)attn.forward_rope(tq, tk, tk, &cache, pos0 + t, rope, DType::BFloat16);
    };
    adapter_loop(L0);  // warm-up: fills the block cache
    hip_check(hipStreamSynchronize(current_stream()), "sync");
    const size_t blocks_before = BlockCache::instance().driver_allocations();
    hip_check(hipEventRecord(e0, current_stream()), "record");
    adapter_loop(L0 + tokens);
    hip_check(hipEventRecord(e1, current_stream()), "record");
    hip_check(hipEventSynchronize(e1), "sync");
    float ms_adapter = 0.f;
    hip_check(hipEventElapsedTime(&ms_adapter, e0, e1), "elapsed");
    CHECK(BlockCache::instance().driver_allocations() == blocks_before);  // no hipMalloc inside the timed loop
    // the same launches through the C ABI
    vsp_kv_cache c = cache.raw();
    Tensor q_rot = empty({B, Hq, 1, D}, DType::BFloat16), out = empty({B, Hq, 1, D}, DType::BFloat16);
    const size_t ws_bytes = vsp_attn_decode_workspace_bytes((int32_t)B, (int32_t)Hq, (int32_t)D, (int32_t)S_max);
    Storage ws(ws_bytes);
    vsp_tensor dq = tq.desc(), dk = tk.desc(), dqo = q_rot.desc(), dout = out.desc();
    const float scale = 1.0f / std::sqrt((float)D);
    auto abi_loop = [&](int64_t pos0) {
        for (int64_t t = 0; t < tokens; ++t) {
            c.len = (int32_t)(pos0 + t);
            throw_status(vsp_rope_kv_append(&c, &dq, &dk, &dk, &dqo, rope.data(), rope.length(), pos0 + t, nullptr, current_stream()));
            throw_status(vsp_attn_decode(&dqo, &c, nullptr, 0, &dout, scale, ws.data(), ws_bytes, current_stream()));
        }
    };
    abi_loop(L0 + 2 * tokens);
    hip_check(hipStreamSynchronize(current_stream()), "sync");
    hip_check(hipEventRecord(e0, current_stream()), "record");
    abi_loop(L0 + 3 * tokens);
    hip_check(hipEventRecord(e1, current_stream()), "record");
    hip_check(hipEventSynchronize(e1), "sync");
    float ms_abi = 0.f;
    hip_check(hipEventElapsedTime(&ms_abi, e0, e1), "elapsed");
    std::printf("  %lld tokens, B %lld, context %lld..: adapter %.1f us/token, C ABI %.1f us/token (ratio %.3f)\n", (long long)tokens,
                (long long)B, (long long)(L0 + tokens), 1e3 * ms_adapter / tokens, 1e3 * ms_abi / tokens, ms_adapter / ms_abi);
    CHECK(ms_adapter < 1.25f * ms_abi);  // a loose bound for a shared test machine; the measured ratio is printed above
    (void)hipEventDestroy(e0);
    (void)hipEventDestroy(e1);
}

static void test_gqa_configurations_of_the_reference() {
    // tests/test_gqa_chapter33.cpp:600-627: embed_dim 256 with 8, 16 and 32 query heads (head_dim 32, 16, 8) at every
    // head ratio the reference lists, T = 8; the attention core against the oracle's matmul / softmax route
    std::printf("test_gqa_configurations_of_the_reference\n");
    const int64_t configs[6][2] = {{8, 8}, {8, 4}, {8, 2}, {8, 1}, {16, 4}, {32, 8}};
    const int64_t C = 256, B = 1, T = 8;
    for (auto& cfg : configs) {
        const int64_t Hq = cfg[0], Hkv = cfg[1], D = C / Hq;
        nn::GroupedQueryAttentionCore attn(C, Hq, Hkv, 64);
        CHECK(attn.head_dim() == D && attn.num_rep() == Hq / Hkv);
        auto q = randn(B * Hq * T * D, 500 + (int)Hq, 1.0f), k = randn(B * Hkv * T * D, 501 + (int)Hkv, 1.0f), v = randn(B * Hkv * T * D, 502, 1.0f);
        std::vector<float> want(q.size());
        int64_t st[4] = {Hkv * T * D, T * D, D, 1};
        CHECK(orc_gqa_attention_f32(q.data(), k.data(), st, v.data(), st, want.data(), B, Hq, T, T, D, Hq / Hkv, 1) == 0);
        Tensor out = attn.forward(to_dev(q, {B, Hq, T, D}, DType::Float32), to_dev(k, {B, Hkv, T, D}, DType::Float32),
                                  to_dev(v, {B, Hkv, T, D}, DType::Float32));
        CHECK((out.shape() == std::vector<int64_t>{B, Hq, T, D}));
        auto got = to_host(out);
        const double err = max_abs_diff(got, want.data(), want.size());
        if (!(err < 1e-4)) std::printf("  %lldQ/%lldKV head_dim %lld: max-abs %.3g\n", (long long)Hq, (long long)Hkv, (long long)D, err);
        CHECK(err < 1e-4);
        // and through a cache: prompt of 8, then one token
        nn::KVCache cache((int)B, (int)Hkv, 64, (int)D, Device::HIP);
        Tensor o2 = attn.forward(to_dev(q, {B, Hq, T, D}, DType::Float32), to_dev(k, {B, Hkv, T, D}, DType::Float32),
                                 to_dev(v, {B, Hkv, T, D}, DType::Float32), &cache, 0);
        CHECK(max_abs_diff(to_host(o2), want.data(), want.size()) < 1e-4);
    }
}

int main(int argc, char** argv) {
    const bool cpu_only = argc > 1 && std::string(argv[1]) == "--cpu-only";
    test_gqa_constructor_validation();
    if (!cpu_only) {
        test_kv_cache_basic();
        test_flash_attention_against_oracle();
        run_cached_generation<nn::KVCache>(KVFormat::Float32, DType::Float32, 1e-4, "KVCache fp32");
        run_cached_generation<nn::GQAKVCache>(KVFormat::BFloat16, DType::BFloat16, 2e-2, "GQAKVCache bf16");
        run_cached_generation<nn::GQAKVCache>(KVFormat::Q8_0, DType::BFloat16, 2e-2, "GQAKVCache q8_0");
        run_rope_generation<nn::KVCache>(KVFormat::Float32, DType::Float32, 1e-4, "KVCache fp32");
        run_rope_generation<nn::GQAKVCache>(KVFormat::BFloat16, DType::BFloat16, 2e-2, "GQAKVCache bf16");
        test_sdpa_routing();
        test_backward_dispatch_seam();
        test_multi_head_attention_core();
        test_gqa_configurations_of_the_reference();
        test_chunk_of_a_long_prompt_splits_the_context();
        run_token_with_output_projection(KVFormat::Float32, DType::Float32, 1e-4, "f32");
        run_token_with_output_projection(KVFormat::BFloat16, DType::BFloat16, 1e-2, "bf16");
        test_token_loop_allocates_nothing_and_keeps_pace();
    }
    std::printf(g_fail ? "FAILED: %d check(s)\n" : "all adapter tests passed\n", g_fail);
    return g_fail ? 1 : 0;
}
