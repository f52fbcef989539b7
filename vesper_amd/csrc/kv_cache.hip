// KV-cache kernels and their C-ABI entry points: reset (zero fill), append (with conversion /
// quantisation on write into the physical layouts of kv_layout.hpp) and read-back.
//
// Replaces, for the cache write, ops::index + Tensor::copy_from + copy_strided_hip_dispatch
// (src/nn/transformer.cpp:56-73, src/ops/view_ops.cpp:246-323, src/ops/hip/copy.hip:16-93).
#include "kv_layout.hpp"
#include "vsp_common.hpp"

namespace vsp {
namespace {

// ---- zero fill (a kernel, not hipMemsetAsync, so that callers may capture it in a graph) ----
__global__ void __launch_bounds__(256) fill_zero_kernel(uint4* __restrict__ p, size_t n16, uint8_t* __restrict__ tail,
                                                        size_t ntail) {
    size_t i = (size_t)blockIdx.x * blockDim.x + threadIdx.x;
    const size_t stride = (size_t)gridDim.x * blockDim.x;
    for (; i < n16; i += stride) p[i] = uint4{0, 0, 0, 0};
    if (blockIdx.x == 0 && threadIdx.x < ntail) tail[threadIdx.x] = 0;
}

int zero_plane(void* p, size_t bytes, hipStream_t st) {
    if (bytes == 0) return VSP_OK;
    if (!p) return VSP_ERR_NULL;
    if (!is_aligned16(p)) return VSP_ERR_ALIGN;
    size_t n16 = bytes / 16, ntail = bytes % 16;
    size_t blocks = (n16 + 255) / 256;
    if (blocks > 8192) blocks = 8192;
    if (blocks == 0) blocks = 1;
    hipLaunchKernelGGL(fill_zero_kernel, dim3((unsigned)blocks), dim3(256), 0, st, (uint4*)p, n16,
                       (uint8_t*)p + n16 * 16, ntail);
    return check_launch();
}

// ---- append ------------------------------------------------------------------------------
struct AppendArgs {
    const void* src_k;
    const void* src_v;
    int64_t sk[3], sv[3];  // source strides of dims 0..2 (elements); innermost stride is 1
    int64_t nB, nH, nT;    // source shape (dims 0..2)
    void* k;
    void* v;
    void* k_scale;
    void* v_scale;
    int64_t B, H, S, D;  // cache logical dims; S = physical token capacity (S_max for F32, S_pad otherwise)
    int64_t slot_start, slot_len;
    const int32_t* start_dev;  // per-batch start positions or nullptr
    int64_t rows;              // B*H*slot_len
    // Rotary embedding fused into the append (ROPE kernels only): K rows are rotated by the table row of
    // their destination position; the same launch rotates Q into q_out.
    const float* table;  // [table_len][D/2][2] = {cos, sin}
    int64_t table_len;
    const void* q;
    void* q_out;
    int64_t sq[3], so[3];  // q / q_out strides of dims 0..2
    int64_t Hq, T;
    int64_t kv_items;      // threads of the K/V part; the Q part follows
    int32_t q_out_bf16;
    // paged cache (kv_locate): table == nullptr for a contiguous one
    const int32_t* page_table;
    int32_t page_tokens, pages_per_seq;
    int64_t S_logical;  // per-sequence token capacity (the bound for device-side positions)
};

template <typename SrcT>
__device__ inline float load_src(const SrcT* p);
template <>
__device__ inline float load_src<float>(const float* p) { return *p; }
template <>
__device__ inline float load_src<uint16_t>(const uint16_t* p) { return bf16_bits_to_f32(*p); }

// apply_rotary_emb (src/nn/functional.cpp:445-494) on N consecutive elements starting at even d0 of a row
// at absolute position pos: pairs (2i, 2i+1), every product and sum rounded on its own as the
// reference's separate elementwise ops do.  Positions past the table are clamped to its last row.
template <int N>
__device__ inline void rope_rotate(float (&x)[N], int64_t d0, int64_t pos, const AppendArgs& a) {
#pragma clang fp contract(off)  // no fused multiply-add: the products are rounded before the sum
    if (pos >= a.table_len) pos = a.table_len - 1;
    if (pos < 0) pos = 0;
    const float2* t = (const float2*)a.table + pos * (a.D / 2) + d0 / 2;
#pragma unroll
    for (int j = 0; j < N / 2; ++j) {
        const float2 cs = t[j];
        const float x0 = x[2 * j], x1 = x[2 * j + 1];
        const float t1 = x0 * cs.x, t2 = x1 * cs.y, t3 = x0 * cs.y, t4 = x1 * cs.x;
        x[2 * j] = t1 - t2;
        x[2 * j + 1] = t3 + t4;
    }
}

// The Q part of the fused launch: item i rotates 8 consecutive d of one query row.
template <typename SrcT>
__device__ inline void rope_q_item(const AppendArgs& a, int64_t i) {
    const int64_t per_row = a.D / 8;
    const int64_t r = i / per_row, d0 = (i % per_row) * 8;
    const int64_t t = r % a.T, bh = r / a.T;
    const int64_t h = bh % a.Hq, b = bh / a.Hq;
    const int64_t start = a.start_dev ? (int64_t)a.start_dev[b] : a.slot_start;
    const SrcT* p = (const SrcT*)a.q + b * a.sq[0] + h * a.sq[1] + t * a.sq[2] + d0;
    float x[8];
#pragma unroll
    for (int j = 0; j < 8; ++j) x[j] = load_src<SrcT>(p + j);
    rope_rotate<8>(x, d0, start + t, a);
    const int64_t o = b * a.so[0] + h * a.so[1] + t * a.so[2] + d0;
    if (a.q_out_bf16) {
        uint16_t* dst = (uint16_t*)a.q_out + o;
#pragma unroll
        for (int j = 0; j < 8; ++j) dst[j] = f32_to_bf16_bits(x[j]);
    } else {
        float* dst = (float*)a.q_out + o;
#pragma unroll
        for (int j = 0; j < 8; ++j) dst[j] = x[j];
    }
}

// Row r of the slot, in the reference's copy order (src/ops/cpu/copy_cpu.cpp:21-37): linear row
// index decomposed by the slot shape on the destination side and by the source shape on the
// source side.
struct RowMap {
    int64_t b, h, s;     // destination coordinates in the planes (page and token within it for a paged cache)
    int64_t pos;         // the token's position in its sequence (what RoPE rotates by); < 0: drop the token
    int64_t src_off_k, src_off_v;
};
__device__ inline RowMap map_row(const AppendArgs& a, int64_t r) {
    RowMap m;
    int64_t t = r % a.slot_len, bh = r / a.slot_len;
    m.h = bh % a.H;
    m.b = bh / a.H;
    int64_t start = a.start_dev ? (int64_t)a.start_dev[m.b] : a.slot_start;
    m.s = start + t;
    m.pos = (m.s >= 0 && m.s < a.S_logical) ? m.s : -1;  // a device-side position outside the cache
    if (m.pos >= 0) kv_locate(a.page_table, a.page_tokens, a.pages_per_seq, m.b, m.s);
    int64_t st = r % a.nT, sbh = r / a.nT;
    int64_t sh = sbh % a.nH, sb = sbh / a.nH;
    m.src_off_k = sb * a.sk[0] + sh * a.sk[1] + st * a.sk[2];
    m.src_off_v = sb * a.sv[0] + sh * a.sv[1] + st * a.sv[2];
    return m;
}

// F32 cache: both planes row-major fp32; a thread moves 4 consecutive d.
template <typename SrcT, bool ROPE>
__global__ void __launch_bounds__(256) append_f32_kernel(AppendArgs a) {
    const int64_t per_row = a.D / 4;
    int64_t i = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
    if constexpr (ROPE) {
        if (i >= a.kv_items) {
            i -= a.kv_items;
            if (i < a.nB * a.Hq * a.T * (a.D / 8)) rope_q_item<SrcT>(a, i);
            return;
        }
    }
    if (i >= a.rows * per_row) return;
    const int64_t r = i / per_row, d0 = (i % per_row) * 4;
    const RowMap m = map_row(a, r);
    if (m.pos < 0) return;  // never write out of bounds
    const SrcT* pk = (const SrcT*)a.src_k + m.src_off_k + d0;
    const SrcT* pv = (const SrcT*)a.src_v + m.src_off_v + d0;
    float* dk = (float*)a.k + kv_off_rowmajor(a.H, a.S, a.D, m.b, m.h, m.s, d0);
    float* dv = (float*)a.v + kv_off_rowmajor(a.H, a.S, a.D, m.b, m.h, m.s, d0);
    float xk[4];
#pragma unroll
    for (int j = 0; j < 4; ++j) xk[j] = load_src<SrcT>(pk + j);
    if constexpr (ROPE) rope_rotate<4>(xk, d0, m.pos, a);
#pragma unroll
    for (int j = 0; j < 4; ++j) {
        dk[j] = xk[j];
        dv[j] = load_src<SrcT>(pv + j);
    }
}

// BF16 cache: K row-major, V token-blocked by 8; a thread converts 8 consecutive d.
template <typename SrcT, bool ROPE>
__global__ void __launch_bounds__(256) append_bf16_kernel(AppendArgs a) {
    const int64_t per_row = a.D / 8;
    int64_t i = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
    if constexpr (ROPE) {
        if (i >= a.kv_items) {
            i -= a.kv_items;
            if (i < a.nB * a.Hq * a.T * (a.D / 8)) rope_q_item<SrcT>(a, i);
            return;
        }
    }
    if (i >= a.rows * per_row) return;
    const int64_t r = i / per_row, d0 = (i % per_row) * 8;
    const RowMap m = map_row(a, r);
    if (m.pos < 0) return;  // never write out of bounds
    const SrcT* pk = (const SrcT*)a.src_k + m.src_off_k + d0;
    const SrcT* pv = (const SrcT*)a.src_v + m.src_off_v + d0;
    uint16_t kb[8], vb[8];
    if constexpr (ROPE) {
        float xk[8];
#pragma unroll
        for (int j = 0; j < 8; ++j) xk[j] = load_src<SrcT>(pk + j);
        rope_rotate<8>(xk, d0, m.pos, a);
#pragma unroll
        for (int j = 0; j < 8; ++j) kb[j] = f32_to_bf16_bits(xk[j]);
    }
#pragma unroll
    for (int j = 0; j < 8; ++j) {
        if constexpr (sizeof(SrcT) == 2) {
            if constexpr (!ROPE) kb[j] = pk[j];
            vb[j] = pv[j];
        } else {
            if constexpr (!ROPE) kb[j] = f32_to_bf16_bits(pk[j]);
            vb[j] = f32_to_bf16_bits(pv[j]);
        }
    }
    uint4 kq;
    kq.x = kb[0] | ((uint32_t)kb[1] << 16);
    kq.y = kb[2] | ((uint32_t)kb[3] << 16);
    kq.z = kb[4] | ((uint32_t)kb[5] << 16);
    kq.w = kb[6] | ((uint32_t)kb[7] << 16);
    *(uint4*)((uint16_t*)a.k + kv_off_rowmajor(a.H, a.S, a.D, m.b, m.h, m.s, d0)) = kq;
    uint16_t* dv = (uint16_t*)a.v + kv_off_vblocked(a.H, a.S, a.D, kVBlkBf16, m.b, m.h, m.s, d0);
#pragma unroll
    for (int j = 0; j < 8; ++j) dv[j * kVBlkBf16] = vb[j];
}

// IEEE fp32 -> fp16 bits, round-to-nearest-even (the hardware conversion is RNE and keeps subnormals).
__device__ inline uint16_t f32_to_f16_bits_dev(float f) {
    _Float16 h = (_Float16)f;
    return __builtin_bit_cast(uint16_t, h);
}

// Q8_0 cache: a thread quantises one block of 32 consecutive d of one row, for K and for V.
// Arithmetic is ggml's block_q8_0, identical to vsp_q8_0_quantize_row: d = amax/127 (fp32 division),
// id = 1/d (fp32 division), q = roundf(x*id) (half away from zero).
__device__ inline void quantize_block(const float* x, int8_t* q, uint16_t* scale_bits) {
    float amax = 0.0f;
#pragma unroll
    for (int j = 0; j < kQBlock; ++j) amax = fmaxf(amax, fabsf(x[j]));
    const float d = __fdiv_rn(amax, 127.0f);
    const float id = d != 0.0f ? __fdiv_rn(1.0f, d) : 0.0f;
    *scale_bits = f32_to_f16_bits_dev(d);
#pragma unroll
    for (int j = 0; j < kQBlock; ++j) q[j] = (int8_t)(int)roundf(__fmul_rn(x[j], id));
}

template <typename SrcT, bool ROPE>
__global__ void __launch_bounds__(128) append_q8_kernel(AppendArgs a) {
    const int64_t per_row = a.D / kQBlock;
    int64_t i = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
    if constexpr (ROPE) {
        if (i >= a.kv_items) {
            i -= a.kv_items;
            if (i < a.nB * a.Hq * a.T * (a.D / 8)) rope_q_item<SrcT>(a, i);
            return;
        }
    }
    if (i >= a.rows * per_row) return;
    const int64_t r = i / per_row, blk = i % per_row, d0 = blk * kQBlock;
    const RowMap m = map_row(a, r);
    if (m.pos < 0) return;  // never write out of bounds
    const SrcT* pk = (const SrcT*)a.src_k + m.src_off_k + d0;
    const SrcT* pv = (const SrcT*)a.src_v + m.src_off_v + d0;
    float x[kQBlock];
    int8_t q[kQBlock];
    uint16_t sc;
    // K: row-major int8, scales [s][blk]
#pragma unroll
    for (int j = 0; j < kQBlock; ++j) x[j] = load_src<SrcT>(pk + j);
    if constexpr (ROPE) rope_rotate<kQBlock>(x, d0, m.pos, a);
    quantize_block(x, q, &sc);
    {
        uint32_t w[8];
#pragma unroll
        for (int j = 0; j < 8; ++j)
            w[j] = (uint32_t)(uint8_t)q[4 * j] | ((uint32_t)(uint8_t)q[4 * j + 1] << 8) |
                   ((uint32_t)(uint8_t)q[4 * j + 2] << 16) | ((uint32_t)(uint8_t)q[4 * j + 3] << 24);
        uint4* dk = (uint4*)((int8_t*)a.k + kv_off_rowmajor(a.H, a.S, a.D, m.b, m.h, m.s, d0));
        dk[0] = uint4{w[0], w[1], w[2], w[3]};
        dk[1] = uint4{w[4], w[5], w[6], w[7]};
        ((uint16_t*)a.k_scale)[kv_off_kscale(a.H, a.S, a.D, m.b, m.h, m.s, blk)] = sc;
    }
    // V: token-blocked by 16, scales [s/16][blk][s%16]
#pragma unroll
    for (int j = 0; j < kQBlock; ++j) x[j] = load_src<SrcT>(pv + j);
    quantize_block(x, q, &sc);
    {
        int8_t* dv = (int8_t*)a.v + kv_off_vblocked(a.H, a.S, a.D, kVBlkQ8, m.b, m.h, m.s, d0);
#pragma unroll
        for (int j = 0; j < kQBlock; ++j) dv[j * kVBlkQ8] = q[j];
        ((uint16_t*)a.v_scale)[kv_off_vscale(a.H, a.S, a.D, m.b, m.h, m.s, blk)] = sc;
    }
}

// ---- read-back ----------------------------------------------------------------------------
struct ReadArgs {
    const void* k;
    const void* v;
    const void* k_scale;
    const void* v_scale;
    int64_t B, H, S, D;
    int64_t start, count;
    void* out_k;
    void* out_v;
    int64_t ok[3], ov[3];  // output strides of dims 0..2 (elements)
    int format;
    const int32_t* page_table;
    int32_t page_tokens, pages_per_seq;
};

template <typename DstT>
__device__ inline void store_dst(DstT* p, float f, uint16_t bf_bits, bool have_bits);
template <>
__device__ inline void store_dst<float>(float* p, float f, uint16_t, bool) { *p = f; }
template <>
__device__ inline void store_dst<uint16_t>(uint16_t* p, float f, uint16_t bf_bits, bool have_bits) {
    *p = have_bits ? bf_bits : f32_to_bf16_bits(f);
}

__device__ inline float f16_bits_to_f32_dev(uint16_t h) { return (float)__builtin_bit_cast(_Float16, h); }

template <typename DstT>
__global__ void __launch_bounds__(256) read_kernel(ReadArgs a) {
    int64_t i = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
    const int64_t total = a.B * a.H * a.count * a.D;
    if (i >= total) return;
    const int64_t d = i % a.D;
    int64_t r = i / a.D;
    const int64_t t = r % a.count;
    r /= a.count;
    const int64_t h = r % a.H, b = r / a.H;
    const int64_t s_seq = a.start + t;
    int64_t pb = b, s = s_seq;  // plane coordinates
    kv_locate(a.page_table, a.page_tokens, a.pages_per_seq, pb, s);
    float fk, fv;
    uint16_t bk = 0, bv = 0;
    bool bits = false;
    if (a.format == VSP_KV_F32) {
        fk = ((const float*)a.k)[kv_off_rowmajor(a.H, a.S, a.D, pb, h, s, d)];
        fv = ((const float*)a.v)[kv_off_rowmajor(a.H, a.S, a.D, pb, h, s, d)];
    } else if (a.format == VSP_KV_BF16) {
        bk = ((const uint16_t*)a.k)[kv_off_rowmajor(a.H, a.S, a.D, pb, h, s, d)];
        bv = ((const uint16_t*)a.v)[kv_off_vblocked(a.H, a.S, a.D, kVBlkBf16, pb, h, s, d)];
        fk = bf16_bits_to_f32(bk);
        fv = bf16_bits_to_f32(bv);
        bits = true;
    } else {
        const int64_t blk = d / kQBlock;
        const float dk = f16_bits_to_f32_dev(((const uint16_t*)a.k_scale)[kv_off_kscale(a.H, a.S, a.D, pb, h, s, blk)]);
        const float dv = f16_bits_to_f32_dev(((const uint16_t*)a.v_scale)[kv_off_vscale(a.H, a.S, a.D, pb, h, s, blk)]);
        fk = __fmul_rn((float)((const int8_t*)a.k)[kv_off_rowmajor(a.H, a.S, a.D, pb, h, s, d)], dk);
        fv = __fmul_rn((float)((const int8_t*)a.v)[kv_off_vblocked(a.H, a.S, a.D, kVBlkQ8, pb, h, s, d)], dv);
    }
    if (a.out_k) store_dst<DstT>((DstT*)a.out_k + b * a.ok[0] + h * a.ok[1] + t * a.ok[2] + d, fk, bk, bits);
    if (a.out_v) store_dst<DstT>((DstT*)a.out_v + b * a.ov[0] + h * a.ov[1] + t * a.ov[2] + d, fv, bv, bits);
}

__global__ void __launch_bounds__(256) read_q8_raw_kernel(const int8_t* __restrict__ qs, const uint16_t* __restrict__ sc,
                                                          int plane, int64_t B, int64_t H, int64_t S, int64_t D,
                                                          int64_t start, int64_t count, int8_t* __restrict__ qs_out,
                                                          uint16_t* __restrict__ sc_out, const int32_t* __restrict__ page_table,
                                                          int32_t page_tokens, int32_t pages_per_seq) {
    int64_t i = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
    if (i >= B * H * count * D) return;
    const int64_t d = i % D;
    int64_t r = i / D;
    const int64_t t = r % count;
    r /= count;
    const int64_t h = r % H;
    int64_t b = r / H, s = start + t;
    kv_locate(page_table, page_tokens, pages_per_seq, b, s);
    if (plane == VSP_KV_PLANE_K) {
        qs_out[i] = qs[kv_off_rowmajor(H, S, D, b, h, s, d)];
        if (d % kQBlock == 0) sc_out[i / kQBlock] = sc[kv_off_kscale(H, S, D, b, h, s, d / kQBlock)];
    } else {
        qs_out[i] = qs[kv_off_vblocked(H, S, D, kVBlkQ8, b, h, s, d)];
        if (d % kQBlock == 0) sc_out[i / kQBlock] = sc[kv_off_vscale(H, S, D, b, h, s, d / kQBlock)];
    }
}

// lens[b] = min(lens[b] + (n_new ? clamp(n_new[b], 0, T) : T), S_max)
__global__ void __launch_bounds__(256) advance_lens_kernel(int32_t* __restrict__ lens, const int32_t* __restrict__ n_new,
                                                           int32_t T, int32_t B, int32_t S_max) {
    const int b = blockIdx.x * blockDim.x + threadIdx.x;
    if (b >= B) return;
    const int n = n_new ? min(max(n_new[b], 0), T) : T;
    lens[b] = min(lens[b] + n, S_max);
}

int check_cache(const vsp_kv_cache* c) {
    if (!c) return VSP_ERR_NULL;
    if (c->format != VSP_KV_F32 && c->format != VSP_KV_BF16 && c->format != VSP_KV_Q8_0) return VSP_ERR_UNSUPPORTED;
    if (c->B < 0 || c->Hkv < 0 || c->S_max < 0 || c->D < 0 || c->len < 0 || c->len > c->S_max) return VSP_ERR_ARG;
    const int64_t n = (int64_t)c->B * c->Hkv * c->S_max * c->D;
    if (n > 0) {
        if (!c->k || !c->v) return VSP_ERR_NULL;
        if (c->format == VSP_KV_Q8_0 && (!c->k_scale || !c->v_scale)) return VSP_ERR_NULL;
        if (!is_aligned16(c->k) || !is_aligned16(c->v)) return VSP_ERR_ALIGN;
        if (c->format == VSP_KV_Q8_0 && (!is_aligned16(c->k_scale) || !is_aligned16(c->v_scale))) return VSP_ERR_ALIGN;
    }
    if (c->format == VSP_KV_F32) {
        if (c->D % 4 != 0) return VSP_ERR_UNSUPPORTED;
    } else if (c->D != 64 && c->D != 128) {
        return VSP_ERR_UNSUPPORTED;
    }
    if (c->page_table) {
        if (c->format == VSP_KV_F32) return VSP_ERR_UNSUPPORTED;
        if (c->page_tokens <= 0 || c->page_tokens % kTokPad != 0 || c->pages_per_seq <= 0 || c->n_pages <= 0) return VSP_ERR_ARG;
        if ((int64_t)c->pages_per_seq * c->page_tokens != c->S_max) return VSP_ERR_ARG;
    } else if (c->page_tokens != 0 || c->pages_per_seq != 0 || c->n_pages != 0) {
        return VSP_ERR_ARG;  // paging fields without a table
    }
    return VSP_OK;
}

}  // namespace

int check_kv_cache(const vsp_kv_cache* c) { return check_cache(c); }
// Physical batch and token capacity of the planes: pages for a paged cache.
int64_t kv_phys_batch(const vsp_kv_cache* c) { return c->page_table ? c->n_pages : c->B; }
int64_t kv_phys_tokens(const vsp_kv_cache* c) { return c->page_table ? c->page_tokens : kv_s_pad(c->format, c->S_max); }

}  // namespace vsp

using namespace vsp;

extern "C" {

int vsp_kv_cache_reset(vsp_kv_cache* cache, void* stream) {
    int rc = check_cache(cache);
    if (rc != VSP_OK) return rc;
    hipStream_t st = (hipStream_t)stream;
    for (int plane = 0; plane < 4; ++plane) {
        size_t bytes = cache->page_table
                           ? kv_plane_bytes(cache->format, cache->n_pages, cache->Hkv, cache->page_tokens, cache->D, plane)
                           : kv_plane_bytes(cache->format, cache->B, cache->Hkv, cache->S_max, cache->D, plane);
        void* p = plane == 0 ? cache->k : plane == 1 ? cache->v : plane == 2 ? cache->k_scale : cache->v_scale;
        rc = zero_plane(p, bytes, st);
        if (rc != VSP_OK) return rc;
    }
    cache->len = 0;
    return VSP_OK;
}

// Shared body of vsp_kv_append and vsp_rope_kv_append (rope != nullptr: rotate K on the way in and Q in
// the tail of the same launch).
struct RopeParams {
    const vsp_tensor* q;
    vsp_tensor* q_out;
    const float* table;
    int64_t table_len;
};

static int append_impl(vsp_kv_cache* cache, const vsp_tensor* new_k, const vsp_tensor* new_v, int64_t start_pos,
                       const int32_t* start_pos_dev, const RopeParams* rope, void* stream) {
    int rc = check_cache(cache);
    if (rc != VSP_OK) return rc;
    if (!new_k || !new_v) return VSP_ERR_NULL;
    if (new_k->ndim != 4 || new_v->ndim != 4) return VSP_ERR_NDIM;
    if (new_k->dtype != new_v->dtype) return VSP_ERR_COPY_DTYPE;
    if (new_k->dtype != VSP_F32 && new_k->dtype != VSP_BF16) return VSP_ERR_UNSUPPORTED;
    for (int i = 0; i < 4; ++i)
        if (new_k->shape[i] < 0 || new_k->shape[i] != new_v->shape[i]) return VSP_ERR_NUMEL;
    const int64_t T = new_k->shape[2];
    if (rope) {
        const vsp_tensor* q = rope->q;
        const vsp_tensor* qo = rope->q_out;
        if (!q || !qo || !rope->table) return VSP_ERR_NULL;
        if (q->ndim != 4 || qo->ndim != 4) return VSP_ERR_NDIM;
        if (q->dtype != new_k->dtype) return VSP_ERR_DTYPE;
        if (qo->dtype != VSP_F32 && qo->dtype != VSP_BF16) return VSP_ERR_UNSUPPORTED;
        for (int i = 0; i < 4; ++i)
            if (q->shape[i] < 0 || q->shape[i] != qo->shape[i]) return VSP_ERR_SHAPE;
        if (q->shape[0] != new_k->shape[0] || q->shape[2] != T || q->shape[3] != new_k->shape[3]) return VSP_ERR_SHAPE;
        // the rotated rows must be the cache's rows: no reshaping copy as in plain append
        if (new_k->shape[0] != cache->B || new_k->shape[1] != cache->Hkv || new_k->shape[3] != cache->D) return VSP_ERR_NUMEL;
        if (cache->D % 8 != 0) return VSP_ERR_UNSUPPORTED;
        if (q->stride[3] != 1 || qo->stride[3] != 1) return VSP_ERR_STRIDE;
        if (((uintptr_t)rope->table & 7) != 0) return VSP_ERR_ALIGN;
        if (rope->table_len <= 0) return VSP_ERR_ARG;
        if (!start_pos_dev && (start_pos < 0 || start_pos + T > rope->table_len)) return VSP_ERR_ARG;
        if (q->shape[0] * q->shape[1] * T * q->shape[3] > 0 && (!q->data || !qo->data)) return VSP_ERR_NULL;
    }
    // the slot [:, :, start_pos:start_pos+T, :] with the reference's clamping
    int64_t slot_start, slot_len;
    if (start_pos_dev) {
        slot_start = 0;
        slot_len = T;
        if (T > cache->S_max) return VSP_ERR_NUMEL;
    } else {
        slice_bounds(cache->S_max, start_pos, start_pos + T, &slot_start, &slot_len);
    }
    const int64_t slot_numel = (int64_t)cache->B * cache->Hkv * slot_len * cache->D;
    const int64_t src_numel = new_k->shape[0] * new_k->shape[1] * new_k->shape[2] * new_k->shape[3];
    if (slot_numel != src_numel) return VSP_ERR_NUMEL;  // copy_from: element count mismatch.
    const int64_t q_items = rope ? rope->q->shape[0] * rope->q->shape[1] * T * (cache->D / 8) : 0;
    if (slot_numel > 0 || q_items > 0) {
        if (slot_numel > 0) {
            if (new_k->shape[3] != cache->D) return VSP_ERR_UNSUPPORTED;  // rows would straddle
            if (!new_k->data || !new_v->data) return VSP_ERR_NULL;
            if (new_k->stride[3] != 1 || new_v->stride[3] != 1) return VSP_ERR_STRIDE;
        }
        AppendArgs a{};
        a.src_k = new_k->data;
        a.src_v = new_v->data;
        for (int i = 0; i < 3; ++i) {
            a.sk[i] = new_k->stride[i];
            a.sv[i] = new_v->stride[i];
        }
        a.nB = new_k->shape[0];
        a.nH = new_k->shape[1];
        a.nT = new_k->shape[2];
        a.k = cache->k;
        a.v = cache->v;
        a.k_scale = cache->k_scale;
        a.v_scale = cache->v_scale;
        a.B = cache->B;
        a.H = cache->Hkv;
        a.S = kv_phys_tokens(cache);
        a.D = cache->D;
        a.page_table = cache->page_table;
        a.page_tokens = cache->page_tokens;
        a.pages_per_seq = cache->pages_per_seq;
        a.S_logical = cache->S_max;
        a.slot_start = slot_start;
        a.slot_len = slot_len;
        a.start_dev = start_pos_dev;
        a.rows = (int64_t)cache->B * cache->Hkv * slot_len;
        if (rope) {
            a.table = rope->table;
            a.table_len = rope->table_len;
            a.q = rope->q->data;
            a.q_out = rope->q_out->data;
            for (int i = 0; i < 3; ++i) {
                a.sq[i] = rope->q->stride[i];
                a.so[i] = rope->q_out->stride[i];
            }
            a.Hq = rope->q->shape[1];
            a.T = T;
            a.q_out_bf16 = rope->q_out->dtype == VSP_BF16;
        }
        hipStream_t st = (hipStream_t)stream;
        const bool f32src = new_k->dtype == VSP_F32;
        const bool r = rope != nullptr;
        auto blocks = [&](int64_t kv_items, int threads) {
            // the Q part starts at a block boundary so that a block never mixes the two item kinds
            a.kv_items = ceil_div(kv_items, threads) * threads;
            return dim3((unsigned)(a.kv_items / threads + ceil_div(q_items, threads)));
        };
        if (cache->format == VSP_KV_F32) {
            dim3 grid = blocks(a.rows * (a.D / 4), 256);
            if (f32src && r) hipLaunchKernelGGL((append_f32_kernel<float, true>), grid, dim3(256), 0, st, a);
            else if (f32src) hipLaunchKernelGGL((append_f32_kernel<float, false>), grid, dim3(256), 0, st, a);
            else if (r) hipLaunchKernelGGL((append_f32_kernel<uint16_t, true>), grid, dim3(256), 0, st, a);
            else hipLaunchKernelGGL((append_f32_kernel<uint16_t, false>), grid, dim3(256), 0, st, a);
        } else if (cache->format == VSP_KV_BF16) {
            dim3 grid = blocks(a.rows * (a.D / 8), 256);
            if (f32src && r) hipLaunchKernelGGL((append_bf16_kernel<float, true>), grid, dim3(256), 0, st, a);
            else if (f32src) hipLaunchKernelGGL((append_bf16_kernel<float, false>), grid, dim3(256), 0, st, a);
            else if (r) hipLaunchKernelGGL((append_bf16_kernel<uint16_t, true>), grid, dim3(256), 0, st, a);
            else hipLaunchKernelGGL((append_bf16_kernel<uint16_t, false>), grid, dim3(256), 0, st, a);
        } else {
            dim3 grid = blocks(a.rows * (a.D / kQBlock), 128);
            if (f32src && r) hipLaunchKernelGGL((append_q8_kernel<float, true>), grid, dim3(128), 0, st, a);
            else if (f32src) hipLaunchKernelGGL((append_q8_kernel<float, false>), grid, dim3(128), 0, st, a);
            else if (r) hipLaunchKernelGGL((append_q8_kernel<uint16_t, true>), grid, dim3(128), 0, st, a);
            else hipLaunchKernelGGL((append_q8_kernel<uint16_t, false>), grid, dim3(128), 0, st, a);
        }
        rc = check_launch();
        if (rc != VSP_OK) return rc;
    }
    if (!start_pos_dev) {
        // current_len_ = max(current_len_, start_pos + T), src/nn/transformer.cpp:73
        int64_t nl = start_pos + T;
        if (nl > cache->len) cache->len = (int32_t)nl;
    }
    return VSP_OK;
}

int vsp_kv_append(vsp_kv_cache* cache, const vsp_tensor* new_k, const vsp_tensor* new_v, int64_t start_pos,
                  const int32_t* start_pos_dev, void* stream) {
    return append_impl(cache, new_k, new_v, start_pos, start_pos_dev, nullptr, stream);
}

int vsp_rope_kv_append(vsp_kv_cache* cache, const vsp_tensor* q, const vsp_tensor* new_k, const vsp_tensor* new_v,
                       vsp_tensor* q_out, const float* rope_table, int64_t table_len, int64_t start_pos,
                       const int32_t* start_pos_dev, void* stream) {
    RopeParams rp{q, q_out, rope_table, table_len};
    return append_impl(cache, new_k, new_v, start_pos, start_pos_dev, &rp, stream);
}

int vsp_seq_lens_advance(int32_t* seq_lens, const int32_t* n_new, int32_t T, int32_t B, int32_t S_max, void* stream) {
    if (B < 0 || T < 0 || S_max < 0) return VSP_ERR_ARG;
    if (B == 0) return VSP_OK;
    if (!seq_lens) return VSP_ERR_NULL;
    hipLaunchKernelGGL(advance_lens_kernel, dim3((unsigned)ceil_div(B, 256)), dim3(256), 0, (hipStream_t)stream, seq_lens,
                       n_new, T, B, S_max);
    return check_launch();
}

int vsp_kv_read(const vsp_kv_cache* cache, int64_t start, int64_t count, vsp_tensor* k_out, vsp_tensor* v_out,
                void* stream) {
    int rc = check_cache(cache);
    if (rc != VSP_OK) return rc;
    if (start < 0 || count < 0 || start + count > cache->S_max) return VSP_ERR_ARG;
    if (!k_out && !v_out) return VSP_ERR_NULL;
    const vsp_tensor* any = k_out ? k_out : v_out;
    ReadArgs a;
    for (const vsp_tensor* t : {(const vsp_tensor*)k_out, (const vsp_tensor*)v_out}) {
        if (!t) continue;
        if (t->ndim != 4) return VSP_ERR_NDIM;
        if (t->shape[0] != cache->B || t->shape[1] != cache->Hkv || t->shape[2] != count || t->shape[3] != cache->D)
            return VSP_ERR_NUMEL;
        if (t->dtype != any->dtype) return VSP_ERR_COPY_DTYPE;
        if (t->dtype != VSP_F32 && t->dtype != VSP_BF16) return VSP_ERR_UNSUPPORTED;
        if (t->stride[3] != 1) return VSP_ERR_STRIDE;
    }
    const int64_t total = (int64_t)cache->B * cache->Hkv * count * cache->D;
    if (total == 0) return VSP_OK;
    if ((k_out && !k_out->data) || (v_out && !v_out->data)) return VSP_ERR_NULL;
    a.k = cache->k;
    a.v = cache->v;
    a.k_scale = cache->k_scale;
    a.v_scale = cache->v_scale;
    a.B = cache->B;
    a.H = cache->Hkv;
    a.S = kv_phys_tokens(cache);
    a.D = cache->D;
    a.page_table = cache->page_table;
    a.page_tokens = cache->page_tokens;
    a.pages_per_seq = cache->pages_per_seq;
    a.start = start;
    a.count = count;
    a.out_k = k_out ? k_out->data : nullptr;
    a.out_v = v_out ? v_out->data : nullptr;
    for (int i = 0; i < 3; ++i) {
        a.ok[i] = k_out ? k_out->stride[i] : 0;
        a.ov[i] = v_out ? v_out->stride[i] : 0;
    }
    a.format = cache->format;
    dim3 grid((unsigned)ceil_div(total, 256));
    if (any->dtype == VSP_F32) hipLaunchKernelGGL(read_kernel<float>, grid, dim3(256), 0, (hipStream_t)stream, a);
    else hipLaunchKernelGGL(read_kernel<uint16_t>, grid, dim3(256), 0, (hipStream_t)stream, a);
    return check_launch();
}

int vsp_kv_read_q8_0(const vsp_kv_cache* cache, int32_t plane, int64_t start, int64_t count, int8_t* qs_out,
                     uint16_t* scale_out, void* stream) {
    int rc = check_cache(cache);
    if (rc != VSP_OK) return rc;
    if (cache->format != VSP_KV_Q8_0) return VSP_ERR_UNSUPPORTED;
    if (plane != VSP_KV_PLANE_K && plane != VSP_KV_PLANE_V) return VSP_ERR_ARG;
    if (start < 0 || count < 0 || start + count > cache->S_max) return VSP_ERR_ARG;
    const int64_t total = (int64_t)cache->B * cache->Hkv * count * cache->D;
    if (total == 0) return VSP_OK;
    if (!qs_out || !scale_out) return VSP_ERR_NULL;
    const bool isk = plane == VSP_KV_PLANE_K;
    hipLaunchKernelGGL(read_q8_raw_kernel, dim3((unsigned)ceil_div(total, 256)), dim3(256), 0, (hipStream_t)stream,
                       (const int8_t*)(isk ? cache->k : cache->v),
                       (const uint16_t*)(isk ? cache->k_scale : cache->v_scale), plane, (int64_t)cache->B,
                       (int64_t)cache->Hkv, kv_phys_tokens(cache), (int64_t)cache->D, start, count, qs_out, scale_out,
                       cache->page_table, cache->page_tokens, cache->pages_per_seq);
    return check_launch();
}

int vsp_kv_view_f32(const vsp_kv_cache* cache, vsp_tensor* k_view, vsp_tensor* v_view) {
    int rc = check_cache(cache);
    if (rc != VSP_OK) return rc;
    if (cache->format != VSP_KV_F32) return VSP_ERR_UNSUPPORTED;
    if (!k_view || !v_view) return VSP_ERR_NULL;
    for (int which = 0; which < 2; ++which) {
        vsp_tensor* t = which ? v_view : k_view;
        t->data = which ? cache->v : cache->k;
        t->dtype = VSP_F32;
        t->ndim = 4;
        t->shape[0] = cache->B;
        t->shape[1] = cache->Hkv;
        t->shape[2] = cache->len;
        t->shape[3] = cache->D;
        t->stride[3] = 1;
        t->stride[2] = cache->D;
        t->stride[1] = (int64_t)cache->S_max * cache->D;
        t->stride[0] = (int64_t)cache->Hkv * cache->S_max * cache->D;
    }
    return VSP_OK;
}

}  // extern "C"
