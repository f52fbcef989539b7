// Host-side safety net, built with AddressSanitizer + UndefinedBehaviorSanitizer on the host pass (no GPU needed):
//   1. every offset function of vesper_amd/csrc/kv_layout.hpp is a bijection of the logical index space onto
//      [0, plane elements), for the three cache formats, contiguous and paged (brute force over small shapes);
//   2. the host-side format helpers and the validation halves of the entry points run under the sanitizers with the
//      status codes the header documents (every call here returns before any kernel would be launched).
#include <cmath>
#include <cstdio>
#include <cstdlib>
#include <cstring>
#include <numeric>
#include <random>
#include <vector>

#include "../../include/vsp_attn.h"
#include "../../vesper_amd/csrc/kv_layout.hpp"

static int g_fail = 0;
#define CHECK(cond)                                                               \
    do {                                                                          \
        if (!(cond)) {                                                            \
            std::printf("  CHECK FAILED %s:%d: %s\n", __FILE__, __LINE__, #cond); \
            ++g_fail;                                                             \
        }                                                                         \
    } while (0)

using namespace vsp;

// visits[off] counts how often an offset is produced; a bijection onto [0, n) leaves every count at 1
static bool is_bijection(const std::vector<int>& visits) {
    for (int c : visits)
        if (c != 1) return false;
    return true;
}

static void check_layout(int format, int64_t B, int64_t H, int64_t S_max, int64_t D, bool paged, int64_t page_tokens) {
    // physical geometry: a paged cache is laid out like a contiguous one with batch = n_pages, capacity = page_tokens
    const int64_t pages_per_seq = paged ? S_max / page_tokens : 0;
    const int64_t n_pages = paged ? B * pages_per_seq : 0;
    const int64_t PB = paged ? n_pages : B, PS_max = paged ? page_tokens : S_max;
    const int64_t S = kv_s_pad(format, PS_max);
    std::vector<int32_t> table;
    if (paged) {  // a random permutation: every logical page owns one physical page
        table.resize((size_t)n_pages);
        std::iota(table.begin(), table.end(), 0);
        std::mt19937 rng(7);
        std::shuffle(table.begin(), table.end(), rng);
    }
    const int64_t esz = format == VSP_KV_F32 ? 4 : (format == VSP_KV_BF16 ? 2 : 1);
    const size_t n_k = kv_plane_bytes(format, PB, H, PS_max, D, VSP_KV_PLANE_K) / esz;
    const size_t n_v = kv_plane_bytes(format, PB, H, PS_max, D, VSP_KV_PLANE_V) / esz;
    CHECK(n_k == (size_t)(PB * H * S * D) && n_v == n_k);
    std::vector<int> vk(n_k, 0), vv(n_v, 0);
    const bool q8 = format == VSP_KV_Q8_0;
    const size_t n_ks = kv_plane_bytes(format, PB, H, PS_max, D, VSP_KV_PLANE_K_SCALE) / 2;
    const size_t n_vs = kv_plane_bytes(format, PB, H, PS_max, D, VSP_KV_PLANE_V_SCALE) / 2;
    CHECK(q8 ? (n_ks == (size_t)(PB * H * S * (D / kQBlock)) && n_vs == n_ks) : (n_ks == 0 && n_vs == 0));
    std::vector<int> vks(n_ks, 0), vvs(n_vs, 0);
    // logical tokens cover the padded capacity too, so that "onto" is tested, not just "into"
    const int64_t S_log = paged ? S_max : S;
    for (int64_t b = 0; b < B; ++b)
        for (int64_t h = 0; h < H; ++h)
            for (int64_t s = 0; s < S_log; ++s) {
                int64_t pb = b, ps = s;
                kv_locate(paged ? table.data() : nullptr, (int32_t)page_tokens, (int32_t)pages_per_seq, pb, ps);
                CHECK(pb >= 0 && pb < PB && ps >= 0 && ps < S);
                for (int64_t d = 0; d < D; ++d) {
                    const int64_t ok = kv_off_rowmajor(H, S, D, pb, h, ps, d);
                    const int64_t ov = format == VSP_KV_F32 ? ok : kv_off_vblocked(H, S, D, q8 ? kVBlkQ8 : kVBlkBf16, pb, h, ps, d);
                    CHECK(ok >= 0 && (size_t)ok < n_k && ov >= 0 && (size_t)ov < n_v);
                    if ((size_t)ok < n_k) vk[(size_t)ok]++;
                    if ((size_t)ov < n_v) vv[(size_t)ov]++;
                }
                if (q8)
                    for (int64_t blk = 0; blk < D / kQBlock; ++blk) {
                        const int64_t oks = kv_off_kscale(H, S, D, pb, h, ps, blk), ovs = kv_off_vscale(H, S, D, pb, h, ps, blk);
                        CHECK(oks >= 0 && (size_t)oks < n_ks && ovs >= 0 && (size_t)ovs < n_vs);
                        if ((size_t)oks < n_ks) vks[(size_t)oks]++;
                        if ((size_t)ovs < n_vs) vvs[(size_t)ovs]++;
                    }
            }
    CHECK(is_bijection(vk));
    CHECK(is_bijection(vv));
    CHECK(is_bijection(vks));
    CHECK(is_bijection(vvs));
    // the documented closed forms of include/vsp_attn.h, spot-checked against the functions
    if (format == VSP_KV_BF16 && !paged && B > 1 && H > 1 && S > 9 && D > 5)
        CHECK(kv_off_vblocked(H, S, D, 8, 1, 1, 9, 5) == ((((1 * H + 1) * (S / 8) + 9 / 8) * D + 5) * 8 + 9 % 8));
}

static void test_layouts() {
    std::printf("layout bijections\n");
    for (int format : {VSP_KV_F32, VSP_KV_BF16, VSP_KV_Q8_0})
        for (int64_t S_max : {1, 7, 64, 65, 130}) {
            const int64_t D = format == VSP_KV_F32 ? 6 : 64;
            check_layout(format, 2, 3, S_max, D, false, 0);
        }
    for (int format : {VSP_KV_BF16, VSP_KV_Q8_0}) {
        check_layout(format, 3, 2, 256, 64, true, 64);
        check_layout(format, 2, 1, 384, 128, true, 128);
    }
    CHECK(kv_s_pad(VSP_KV_F32, 70) == 70 && kv_s_pad(VSP_KV_BF16, 70) == 128 && kv_s_pad(VSP_KV_Q8_0, 64) == 64);
    CHECK(vsp_kv_plane_bytes(VSP_KV_Q8_0, 2, 3, 70, 64, VSP_KV_PLANE_K_SCALE) == (size_t)2 * 3 * 128 * 2 * 2);
    CHECK(vsp_kv_plane_bytes(VSP_KV_F32, 2, 3, 70, 64, VSP_KV_PLANE_V_SCALE) == 0);
    CHECK(vsp_kv_plane_bytes(VSP_KV_BF16, -1, 3, 70, 64, VSP_KV_PLANE_K) == 0);
}

static vsp_tensor tensor4(void* p, int dtype, int64_t a, int64_t b, int64_t c, int64_t d) {
    vsp_tensor t{};
    t.data = p;
    t.dtype = dtype;
    t.ndim = 4;
    const int64_t sh[4] = {a, b, c, d};
    int64_t st = 1;
    for (int i = 3; i >= 0; --i) {
        t.shape[i] = sh[i];
        t.stride[i] = st;
        st *= sh[i];
    }
    return t;
}

static void test_helpers() {
    std::printf("format helpers\n");
    // fp16 / bf16 round trips over every fp16 bit pattern and a sweep of floats (incl. subnormals, infinities)
    for (uint32_t hbits = 0; hbits < 65536; ++hbits) {
        const float f = vsp_f16_to_f32((uint16_t)hbits);
        if (f == f) CHECK(vsp_f32_to_f16(f) == (uint16_t)hbits);
    }
    std::mt19937 rng(3);
    for (int i = 0; i < 200000; ++i) {
        uint32_t bits = rng();
        float f;
        std::memcpy(&f, &bits, 4);
        if (f != f) continue;
        const uint16_t b = vsp_f32_to_bf16(f);
        const float back = vsp_bf16_to_f32(b);
        CHECK(std::isinf(back) || std::fabs(back - f) <= std::fabs(f) * 0.00390625f + 1e-40f);
        (void)vsp_f32_to_f16(f);
    }
    // Q8_0 rows: lengths that are and are not what a caller should pass; zero rows; extreme values
    std::vector<float> x(256), y(256);
    std::vector<uint16_t> sc(8);
    std::vector<int8_t> qs(256);
    for (int t = 0; t < 50; ++t) {
        for (auto& v : x) v = (float)((int)(rng() % 2001) - 1000) * (t == 7 ? 0.f : (t == 8 ? 1e30f : 0.01f));
        vsp_q8_0_quantize_row(x.data(), 256, sc.data(), qs.data());
        vsp_q8_0_dequantize_row(sc.data(), qs.data(), 256, y.data());
        for (int i = 0; i < 256 && t != 8; ++i) CHECK(std::fabs(y[i] - x[i]) <= 10.0f / 127.0f * 0.5f + 10.0f / 1024.0f + 1e-3f);
    }
    // RoPE table: exactly count * D/2 * 2 floats are written
    std::vector<float> table(5 * 32 * 2 + 1, -7.f);
    vsp_rope_fill_table(table.data(), 3, 5, 64, 10000.0f);
    CHECK(table.back() == -7.f && table[0] == std::cos(3.0f) && table[1] == std::sin(3.0f));
    int64_t s, n;
    vsp_slice_bounds(10, -3, 100, &s, &n);
    CHECK(s == 7 && n == 3);
    vsp_slice_bounds(10, 12, 14, &s, &n);
    CHECK(s == 10 && n == 0);
    int64_t hd, rep;
    CHECK(vsp_gqa_config(4096, 32, 8, &hd, &rep) == VSP_OK && hd == 128 && rep == 4);
    CHECK(vsp_gqa_config(64, 8, 3, &hd, &rep) == VSP_ERR_GQA_HEADS && vsp_gqa_config(60, 8, 2, &hd, &rep) == VSP_ERR_GQA_EMBED);
    for (int c = -1; c < 45; ++c) CHECK(vsp_status_str(c) != nullptr && std::strlen(vsp_status_str(c)) > 0);
}

static void test_validation() {
    std::printf("entry-point validation (no launch)\n");
    alignas(16) static char mem[1 << 16];
    vsp_tensor q = tensor4(mem, VSP_BF16, 1, 4, 8, 64), k = tensor4(mem, VSP_BF16, 1, 2, 8, 64), out = q;
    vsp_tensor q3 = q;
    q3.ndim = 3;
    CHECK(vsp_attn_prefill(&q3, &k, &k, &out, nullptr, 0.1f, 1, 0.f, 0, nullptr) == VSP_ERR_NDIM);
    CHECK(vsp_attn_prefill(nullptr, &k, &k, &out, nullptr, 0.1f, 1, 0.f, 0, nullptr) == VSP_ERR_NULL);
    vsp_tensor k5 = tensor4(mem, VSP_BF16, 1, 3, 8, 64);
    CHECK(vsp_attn_prefill(&q, &k5, &k5, &out, nullptr, 0.1f, 1, 0.f, 0, nullptr) == VSP_ERR_SHAPE);  // 4 heads over 3
    vsp_tensor kf = tensor4(mem, VSP_F32, 1, 2, 8, 64);
    CHECK(vsp_attn_prefill(&q, &kf, &k, &out, nullptr, 0.1f, 1, 0.f, 0, nullptr) == VSP_ERR_DTYPE);
    CHECK(vsp_attn_prefill(&q, &k, &k, &out, nullptr, 0.1f, 1, 1.0f, 0, nullptr) == VSP_ERR_DROPOUT);
    CHECK(vsp_attn_prefill(&q, &k, &k, &out, nullptr, 0.1f, 1, 0.5f, 1, nullptr) == VSP_ERR_UNSUPPORTED);
    CHECK(vsp_attn_prefill(&q, &k, &k, &out, nullptr, 0.0f, 1, 0.f, 0, nullptr) == VSP_ERR_ARG);
    vsp_tensor qs = q;
    qs.stride[3] = 2;
    CHECK(vsp_attn_prefill(&qs, &k, &k, &out, nullptr, 0.1f, 1, 0.f, 0, nullptr) == VSP_ERR_STRIDE);
    vsp_tensor qa = q;
    qa.data = mem + 2;
    CHECK(vsp_attn_prefill(&qa, &k, &k, &out, nullptr, 0.1f, 1, 0.f, 0, nullptr) == VSP_ERR_ALIGN);
    vsp_tensor q48 = tensor4(mem, VSP_BF16, 1, 4, 8, 48), k48 = tensor4(mem, VSP_BF16, 1, 2, 8, 48);
    CHECK(vsp_attn_prefill(&q48, &k48, &k48, &q48, nullptr, 0.1f, 1, 0.f, 0, nullptr) == VSP_ERR_UNSUPPORTED);
    // cache descriptors
    vsp_kv_cache c{};
    c.format = VSP_KV_BF16, c.B = 1, c.Hkv = 2, c.S_max = 64, c.D = 64, c.k = mem, c.v = mem + 32768;
    vsp_tensor nk = tensor4(mem, VSP_BF16, 1, 2, 8, 64);
    CHECK(vsp_kv_append(&c, &nk, &nk, 60, nullptr, nullptr) == VSP_ERR_NUMEL);  // slot clamped to 4 tokens
    CHECK(c.len == 0);
    vsp_kv_cache bad = c;
    bad.D = 96;
    CHECK(vsp_kv_cache_reset(&bad, nullptr) == VSP_ERR_UNSUPPORTED);
    bad = c;
    bad.k = nullptr;
    CHECK(vsp_kv_cache_reset(&bad, nullptr) == VSP_ERR_NULL);
    // fp32 prefill through split bf16 operands: fp32 only, head_dim 64 / 128, workspace for the K and V planes
    {
        vsp_tensor qf = tensor4(mem, VSP_F32, 1, 4, 8, 64), kf = tensor4(mem, VSP_F32, 1, 2, 8, 64), of = qf;
        CHECK(vsp_attn_prefill_split(&qf, &kf, &kf, &of, nullptr, 0.1f, 1, nullptr, 0, nullptr) == VSP_ERR_WORKSPACE);
        CHECK(vsp_attn_prefill_split(&qf, &kf, &kf, &of, nullptr, 0.1f, 1, mem, 64, nullptr) == VSP_ERR_WORKSPACE);
        CHECK(vsp_attn_prefill_split(&q, &k, &k, &out, nullptr, 0.1f, 1, mem, 1 << 16, nullptr) == VSP_ERR_UNSUPPORTED);   // bf16 tensors
        vsp_tensor q32 = tensor4(mem, VSP_F32, 1, 4, 8, 32), k32 = tensor4(mem, VSP_F32, 1, 2, 8, 32), o32 = q32;
        CHECK(vsp_attn_prefill_split(&q32, &k32, &k32, &o32, nullptr, 0.1f, 1, mem, 1 << 16, nullptr) == VSP_ERR_UNSUPPORTED);
        CHECK(vsp_attn_prefill_split(&qf, &kf, &kf, &of, nullptr, 0.0f, 1, mem, 1 << 16, nullptr) == VSP_ERR_ARG);
        CHECK(vsp_attn_prefill_split_workspace_bytes(1, 4, 2, 8, 8, 64) == (size_t)4 * 2048);   // 2 * 8 * 64 elements * 2 bytes, four planes
        CHECK(vsp_attn_prefill_split_workspace_bytes(1, 4, 2, 8, 0, 64) == 0);
    }
    // decode: shapes, head ratio, bounds, workspace
    vsp_tensor dq = tensor4(mem, VSP_BF16, 1, 4, 1, 64), dout = dq;
    c.len = 40;
    CHECK(vsp_attn_decode(&dq, &c, nullptr, 0, &dout, 0.1f, nullptr, 0, nullptr) == VSP_ERR_WORKSPACE);
    CHECK(vsp_attn_decode(&dq, &c, nullptr, 65, &dout, 0.1f, mem, 1 << 16, nullptr) == VSP_ERR_ARG);
    CHECK(vsp_attn_decode(&dq, &c, nullptr, 32, &dout, 0.1f, mem, 1 << 16, nullptr) == VSP_ERR_ARG);  // len 40 above the bound 32
    vsp_tensor dq2 = tensor4(mem, VSP_BF16, 1, 4, 2, 64);
    CHECK(vsp_attn_decode(&dq2, &c, nullptr, 0, &dq2, 0.1f, mem, 1 << 16, nullptr) == VSP_ERR_SHAPE);
    vsp_tensor dq3 = tensor4(mem, VSP_BF16, 1, 3, 1, 64);
    CHECK(vsp_attn_decode(&dq3, &c, nullptr, 0, &dq3, 0.1f, mem, 1 << 16, nullptr) == VSP_ERR_GQA_HEADS);
    CHECK(vsp_attn_decode_workspace_bytes(2, 8, 128, 1000) == (size_t)2 * 8 * 4 * 130 * 4);
    CHECK(vsp_attn_decode_workspace_bytes(0, 8, 128, 1000) == 0);
    // decode + output projection: weight [N, Hq*D], bias [N], y [B,1,N], workspace = merged heads + the partials
    {
        vsp_tensor w{}, bias{}, y{};
        w.data = mem, w.dtype = VSP_BF16, w.ndim = 2, w.shape[0] = 32, w.shape[1] = 256, w.stride[0] = 256, w.stride[1] = 1;
        bias.data = mem, bias.dtype = VSP_BF16, bias.ndim = 1, bias.shape[0] = 32, bias.stride[0] = 1;
        y.data = mem, y.dtype = VSP_BF16, y.ndim = 3, y.shape[0] = 1, y.shape[1] = 1, y.shape[2] = 32;
        y.stride[0] = 32, y.stride[1] = 32, y.stride[2] = 1;
        CHECK(vsp_attn_decode_proj(&dq, &c, nullptr, 0, &w, &bias, &y, 0.1f, nullptr, 0, nullptr) == VSP_ERR_WORKSPACE);
        CHECK(vsp_attn_decode_proj(&dq, &c, nullptr, 0, nullptr, &bias, &y, 0.1f, mem, 1 << 16, nullptr) == VSP_ERR_NULL);
        vsp_tensor w2 = w;
        w2.shape[1] = 128;
        CHECK(vsp_attn_decode_proj(&dq, &c, nullptr, 0, &w2, &bias, &y, 0.1f, mem, 1 << 16, nullptr) == VSP_ERR_SHAPE);
        w2 = w, w2.dtype = VSP_F32;
        CHECK(vsp_attn_decode_proj(&dq, &c, nullptr, 0, &w2, &bias, &y, 0.1f, mem, 1 << 16, nullptr) == VSP_ERR_DTYPE);
        w2 = w, w2.stride[0] = 260;
        CHECK(vsp_attn_decode_proj(&dq, &c, nullptr, 0, &w2, &bias, &y, 0.1f, mem, 1 << 16, nullptr) == VSP_ERR_ALIGN);
        vsp_tensor b2 = bias;
        b2.shape[0] = 31;
        CHECK(vsp_attn_decode_proj(&dq, &c, nullptr, 0, &w, &b2, &y, 0.1f, mem, 1 << 16, nullptr) == VSP_ERR_SHAPE);
        vsp_tensor y2 = y;
        y2.shape[1] = 2;
        CHECK(vsp_attn_decode_proj(&dq, &c, nullptr, 0, &w, &bias, &y2, 0.1f, mem, 1 << 16, nullptr) == VSP_ERR_SHAPE);
        // the attention step's own refusals come through: a length above the bound, a head count the cache does not divide
        CHECK(vsp_attn_decode_proj(&dq, &c, nullptr, 32, &w, &bias, &y, 0.1f, mem, 1 << 16, nullptr) == VSP_ERR_ARG);
        vsp_tensor w3 = w;
        w3.shape[1] = 192, w3.stride[0] = 192;
        CHECK(vsp_attn_decode_proj(&dq3, &c, nullptr, 0, &w3, &bias, &y, 0.1f, mem, 1 << 16, nullptr) == VSP_ERR_GQA_HEADS);
        CHECK(vsp_attn_decode_proj_workspace_bytes(2, 8, 128, 1000, 512) ==
              (size_t)2 * 8 * 128 * 4 + (size_t)8 * 2 * 512 * 4 + (size_t)2 * 8 * 4 * 130 * 4);
        CHECK(vsp_attn_decode_proj_workspace_bytes(0, 8, 128, 1000, 512) == 0);
    }
    // the entry point without a workspace refuses what its fixed array cannot hold, before anything else happens
    vsp_kv_cache big = c;
    big.B = 64, big.Hkv = 8, big.S_max = 65536, big.D = 128, big.len = 65536;
    vsp_tensor bq = tensor4(mem, VSP_BF16, 64, 128, 1, 128);
    CHECK(vsp_attn_decode_noalloc(&bq, &big, nullptr, 0, &bq, 0.1f, nullptr) == VSP_ERR_WORKSPACE);
    // several tokens per sequence through the decode kernels: tokens x heads per kv head <= 16, head_dim 64 / 128
    {
        vsp_tensor q4 = tensor4(mem, VSP_BF16, 1, 4, 4, 64), q9 = tensor4(mem, VSP_BF16, 1, 4, 9, 64);
        const int32_t keep_len = c.len;
        c.len = 8;
        CHECK(vsp_attn_decode(&q4, &c, nullptr, 0, &q4, 0.1f, mem, 1 << 16, nullptr) == VSP_ERR_SHAPE);        // the plain step: T == 1
        CHECK(vsp_attn_decode_multi(&q9, &c, nullptr, 0, &q9, 0.1f, mem, 1 << 16, nullptr) == VSP_ERR_UNSUPPORTED);   // 2 x 9 columns
        CHECK(vsp_attn_decode_multi(&q4, &c, nullptr, 0, &q4, 0.1f, nullptr, 0, nullptr) == VSP_ERR_WORKSPACE);
        vsp_tensor q4s = q4;
        q4s.stride[2] = 68;   // token rows must stay 16-byte aligned
        CHECK(vsp_attn_decode_multi(&q4s, &c, nullptr, 0, &q4, 0.1f, mem, 1 << 16, nullptr) == VSP_ERR_ALIGN);
        c.len = keep_len;
    }
    // backward
    vsp_tensor lse{};
    lse.data = mem, lse.dtype = VSP_F32, lse.ndim = 3, lse.shape[0] = 1, lse.shape[1] = 4, lse.shape[2] = 8;
    lse.stride[0] = 32, lse.stride[1] = 8, lse.stride[2] = 1;
    CHECK(vsp_attn_prefill_backward(&q, &q, &k, &k, &q, &lse, &q, &k, &k, 0.1f, 1, nullptr, 0, nullptr) == VSP_ERR_WORKSPACE);
    CHECK(vsp_attn_prefill_backward(&q, &q, &k5, &k5, &q, &lse, &q, &k5, &k5, 0.1f, 1, mem, 1 << 16, nullptr) == VSP_ERR_SHAPE);
    CHECK(vsp_attn_backward_workspace_bytes(1, 4, 8) == 2u * 4 * 8 * 4);
    // the larger one: the former rounded up to 256 bytes, then one 2 KB tile per (32 queries, 32 keys), key tiles in pairs
    CHECK(vsp_attn_backward_fast_workspace_bytes(1, 4, 8) == 256u + 4u * 1 * 2 * 2048);
    CHECK(vsp_attn_backward_fast_workspace_bytes(2, 4, 100) == 6400u + 2u * 4 * 4 * 4 * 2048);
    CHECK(vsp_attn_backward_fast_workspace_bytes(1, 32, 8192) == 2u * 32 * 8192 * 4 + (size_t)32 * 256 * 256 * 2048);
    CHECK(vsp_attn_backward_fast_workspace_bytes(0, 4, 8) == 0 && vsp_attn_backward_fast_workspace_bytes(1, 4, 0) == 0);
    // backward with split operands: fp32 only, head_dim 64 / 128, workspace for Di, lse and the eight planes
    {
        vsp_tensor qf = tensor4(mem, VSP_F32, 1, 4, 8, 64), kf = tensor4(mem, VSP_F32, 1, 2, 8, 64), k3 = tensor4(mem, VSP_F32, 1, 3, 8, 64);
        CHECK(vsp_attn_prefill_backward_split(&qf, &qf, &kf, &kf, &qf, &lse, &qf, &kf, &kf, 0.1f, 1, nullptr, 0, nullptr) == VSP_ERR_WORKSPACE);
        CHECK(vsp_attn_prefill_backward_split(&qf, &qf, &kf, &kf, &qf, &lse, &qf, &kf, &kf, 0.1f, 1, mem, 64, nullptr) == VSP_ERR_WORKSPACE);
        CHECK(vsp_attn_prefill_backward_split(&q, &q, &k, &k, &q, &lse, &q, &k, &k, 0.1f, 1, mem, 1 << 16, nullptr) == VSP_ERR_UNSUPPORTED);   // bf16
        CHECK(vsp_attn_prefill_backward_split(&qf, &qf, &k3, &k3, &qf, &lse, &qf, &k3, &k3, 0.1f, 1, mem, 1 << 16, nullptr) == VSP_ERR_SHAPE);
        CHECK(vsp_attn_prefill_backward_split(&qf, &qf, &kf, &kf, &qf, &lse, &qf, &kf, &q, 0.1f, 1, mem, 1 << 16, nullptr) == VSP_ERR_SHAPE);   // dv of q's shape
        vsp_tensor q32 = tensor4(mem, VSP_F32, 1, 4, 8, 32), k32 = tensor4(mem, VSP_F32, 1, 2, 8, 32);
        CHECK(vsp_attn_prefill_backward_split(&q32, &q32, &k32, &k32, &q32, &lse, &q32, &k32, &k32, 0.1f, 1, mem, 1 << 16, nullptr) == VSP_ERR_UNSUPPORTED);
        vsp_tensor odd = qf;
        odd.data = (char*)mem + 4;   // rows are read in 8-byte pieces
        CHECK(vsp_attn_prefill_backward_split(&odd, &qf, &kf, &kf, &qf, &lse, &qf, &kf, &kf, 0.1f, 1, mem, 1 << 16, nullptr) == VSP_ERR_ALIGN);
        CHECK(vsp_attn_backward_split_workspace_bytes(1, 4, 2, 8, 64) == 2u * 4 * 8 * 4 + 4u * (4 + 2) * 8 * 64 * 2);
        CHECK(vsp_attn_backward_split_workspace_bytes(1, 4, 0, 8, 64) == 0);
    }
    // cached prefill: the chunk is part of the context, so T = 8 over a context of 4 is a shape error
    c.len = 4;
    CHECK(vsp_attn_prefill_cached(&q, &c, nullptr, 0, nullptr, &out, nullptr, 0.1f, 1, nullptr, 0, nullptr) == VSP_ERR_SHAPE);
    vsp_tensor qf32 = tensor4(mem, VSP_F32, 1, 4, 8, 64);
    c.len = 40;
    CHECK(vsp_attn_prefill_cached(&qf32, &c, nullptr, 0, nullptr, &qf32, nullptr, 0.1f, 1, nullptr, 0, nullptr) == VSP_ERR_DTYPE);
    // a host-side length above the caller's own bound, a negative bound, a bound beyond the capacity
    CHECK(vsp_attn_prefill_cached(&q, &c, nullptr, 39, nullptr, &out, nullptr, 0.1f, 1, nullptr, 0, nullptr) == VSP_ERR_ARG);
    CHECK(vsp_attn_prefill_cached(&q, &c, nullptr, -1, nullptr, &out, nullptr, 0.1f, 1, nullptr, 0, nullptr) == VSP_ERR_ARG);
    CHECK(vsp_attn_prefill_cached(&q, &c, nullptr, c.S_max + 1, nullptr, &out, nullptr, 0.1f, 1, nullptr, 0, nullptr) == VSP_ERR_ARG);
    // the context split is offered for bf16 planes at head_dim 128 when a short grid meets a long context, and only then
    {
        vsp_kv_cache big = c;
        big.format = VSP_KV_BF16;
        big.B = 1;
        big.D = 128;
        big.S_max = 4096;
        big.len = 4096;
        CHECK(vsp_attn_prefill_cached_split_workspace_bytes(&big, 0, 0, 8, 100) == (size_t)1 * 8 * 100 * 8 * 130 * 4);  // 128 tiles / 16
        big.len = 900;
        CHECK(vsp_attn_prefill_cached_split_workspace_bytes(&big, 0, 0, 8, 100) == 0);   // under 32 key tiles
        CHECK(vsp_attn_prefill_cached_split_workspace_bytes(&big, 1, 0, 8, 100) > 0);    // device lengths: the bound is S_max
        CHECK(vsp_attn_prefill_cached_split_workspace_bytes(&big, 1, 900, 8, 100) == 0); // ... unless the caller gives a tighter one
        CHECK(vsp_attn_prefill_cached_split_workspace_bytes(&big, 1, 2048, 8, 100) == (size_t)1 * 8 * 100 * 4 * 130 * 4);  // 64 tiles / 16
        CHECK(vsp_attn_prefill_cached_split_workspace_bytes(&big, 1, -1, 8, 100) == 0);
        big.len = 4096;
        CHECK(vsp_attn_prefill_cached_split_workspace_bytes(&big, 0, 0, 64, 1024) == 0); // 512 workgroups already
        big.D = 64;
        CHECK(vsp_attn_prefill_cached_split_workspace_bytes(&big, 0, 0, 8, 100) == 0);
        big.D = 128;
        big.format = VSP_KV_Q8_0;
        CHECK(vsp_attn_prefill_cached_split_workspace_bytes(&big, 0, 0, 8, 100) == 0);
        CHECK(vsp_attn_prefill_cached_split_workspace_bytes(nullptr, 0, 0, 8, 100) == 0);
        CHECK(vsp_attn_prefill_cached_split_workspace_bytes(&big, 0, 0, 0, 100) == 0);
    }
}

int main() {
    test_layouts();
    test_helpers();
    test_validation();
    std::printf(g_fail ? "FAILED: %d check(s)\n" : "host checks passed\n", g_fail);
    return g_fail ? 1 : 0;
}
