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
    int32_t q_vec;         // q rows and q_out rows are 16-byte aligned: whole 16-byte loads and stores
    int32_t small_index;   // every item count of the launch is below 2^31
    int64_t blocks_per_row;  // tile kernels: token blocks one (batch row, head) slot can touch
    int64_t q_tblocks;       // tile kernels: workgroups of the Q rotation per (batch row, query head)
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
    // N is a multiple of 4 and d0 of N: two {cos, sin} pairs per 16-byte load
    const float4* t = (const float4*)((const float2*)a.table + pos * (a.D / 2) + d0 / 2);
#pragma unroll
    for (int j = 0; j < N / 4; ++j) {
        const float4 cs = t[j];
        {
            const float x0 = x[4 * j], x1 = x[4 * j + 1];
            const float t1 = x0 * cs.x, t2 = x1 * cs.y, t3 = x0 * cs.y, t4 = x1 * cs.x;
            x[4 * j] = t1 - t2;
            x[4 * j + 1] = t3 + t4;
        }
        {
            const float x0 = x[4 * j + 2], x1 = x[4 * j + 3];
            const float t1 = x0 * cs.z, t2 = x1 * cs.w, t3 = x0 * cs.w, t4 = x1 * cs.z;
            x[4 * j + 2] = t1 - t2;
            x[4 * j + 3] = t3 + t4;
        }
    }
}

template <typename SrcT>
__device__ inline void load8(const SrcT* p, float (&x)[8]) {
    if constexpr (sizeof(SrcT) == 2) {
        const uint4 w = *(const uint4*)p;
        const uint32_t ww[4] = {w.x, w.y, w.z, w.w};
#pragma unroll
        for (int j = 0; j < 4; ++j) {
            x[2 * j] = __builtin_bit_cast(float, ww[j] << 16);
            x[2 * j + 1] = __builtin_bit_cast(float, ww[j] & 0xffff0000u);
        }
    } else {
        const float4 lo = *(const float4*)p, hi = *(const float4*)(p + 4);
        x[0] = lo.x, x[1] = lo.y, x[2] = lo.z, x[3] = lo.w, x[4] = hi.x, x[5] = hi.y, x[6] = hi.z, x[7] = hi.w;
    }
}
// two fp32 -> packed bf16 pair with the reference's rounding (f32_to_bf16_bits): both words are rounded in place and one
// byte permute picks their high halves
__device__ inline uint32_t round_pack_bf16x2(float lo, float hi) {
    uint32_t a = __builtin_bit_cast(uint32_t, lo), b = __builtin_bit_cast(uint32_t, hi);
    a += 0x7FFFu + ((a >> 16) & 1u);
    b += 0x7FFFu + ((b >> 16) & 1u);
    return __builtin_amdgcn_perm(b, a, 0x07060302u);
}
__device__ inline uint4 pack8_bf16(const float (&x)[8]) {
    return uint4{round_pack_bf16x2(x[0], x[1]), round_pack_bf16x2(x[2], x[3]), round_pack_bf16x2(x[4], x[5]), round_pack_bf16x2(x[6], x[7])};
}

// The Q part of the fused launch: 8 consecutive d (from d0) of query row (b, h, t) are rotated into q_out.
template <typename SrcT>
__device__ inline void rope_q_row(const AppendArgs& a, int64_t b, int64_t h, int64_t t, int64_t d0);

// item i of the per-element launches: (row, 8-element piece) in row-major order
template <typename SrcT>
__device__ inline void rope_q_item(const AppendArgs& a, int64_t i) {
    int64_t d0, t, h, b;
    if (a.small_index) {  // every count fits 32 bits: 64-bit divisions cost several times the rest of the item
        const uint32_t per_row = (uint32_t)a.D / 8, ii = (uint32_t)i;
        const uint32_t r = ii / per_row, bh = r / (uint32_t)a.T;
        d0 = (ii % per_row) * 8;
        t = r % (uint32_t)a.T;
        h = bh % (uint32_t)a.Hq;
        b = bh / (uint32_t)a.Hq;
    } else {
        const int64_t per_row = a.D / 8;
        const int64_t r = i / per_row, bh = r / a.T;
        d0 = (i % per_row) * 8;
        t = r % a.T;
        h = bh % a.Hq;
        b = bh / a.Hq;
    }
    rope_q_row<SrcT>(a, b, h, t, d0);
}

template <typename SrcT>
__device__ inline void rope_q_row(const AppendArgs& a, int64_t b, int64_t h, int64_t t, int64_t d0) {
    const int64_t start = a.start_dev ? (int64_t)a.start_dev[b] : a.slot_start;
    const SrcT* p = (const SrcT*)a.q + b * a.sq[0] + h * a.sq[1] + t * a.sq[2] + d0;
    float x[8];
    if (a.q_vec) {
        load8<SrcT>(p, x);
    } else {
#pragma unroll
        for (int j = 0; j < 8; ++j) x[j] = load_src<SrcT>(p + j);
    }
    rope_rotate<8>(x, d0, start + t, a);
    const int64_t o = b * a.so[0] + h * a.so[1] + t * a.so[2] + d0;
    if (a.q_out_bf16) {
        uint16_t* dst = (uint16_t*)a.q_out + o;
        if (a.q_vec) {
            *(uint4*)dst = pack8_bf16(x);
        } else {
#pragma unroll
            for (int j = 0; j < 8; ++j) dst[j] = f32_to_bf16_bits(x[j]);
        }
    } else {
        float* dst = (float*)a.q_out + o;
        if (a.q_vec) {
            *(float4*)dst = float4{x[0], x[1], x[2], x[3]};
            *(float4*)(dst + 4) = float4{x[4], x[5], x[6], x[7]};
        } else {
#pragma unroll
            for (int j = 0; j < 8; ++j) dst[j] = x[j];
        }
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

// ---- appends of eight tokens or more: one workgroup per (batch row, kv head, token block) ---------------------
// The per-element kernels above write the token-blocked V planes two bytes (bf16) or one byte (Q8_0) at a time, 16
// bytes apart.  Here a workgroup owns one token block (8 bf16 / 16 int8 tokens of one head): the rows are loaded and
// converted in 16-byte pieces, V is transposed through LDS, and whole blocks leave as 16-byte stores to consecutive
// addresses.  Blocks the slot covers only partly (its first and last) keep their other tokens: those are written
// element by element.  Same arithmetic as the per-element kernels, so the planes come out bit for bit the same.
// Preconditions (checked on the host): source shape == slot shape, source rows 16-byte aligned.
constexpr int kQPerThread = 4;     // rows of the Q rotation per thread in the token-block launches
constexpr int kQRowsPerPass = 8;   // a workgroup of D threads covers D / (D / 8) = 8 rows at a time
constexpr int kQRows = kQPerThread * kQRowsPerPass;
struct TileRow {
    int64_t pb, ps0;   // plane coordinates of the block's first token (page and token within it when paged)
    int64_t start;     // first position of the slot in this batch row
    int lo, hi;        // tokens [lo, hi) of the block belong to the slot (and to the cache)
};
template <int BLK>
__device__ inline TileRow tile_row(const AppendArgs& a, int64_t b, int64_t j) {
    TileRow r;
    r.start = a.start_dev ? (int64_t)a.start_dev[b] : a.slot_start;
    const int64_t first_blk = r.start >= 0 ? r.start / BLK : -((-r.start + BLK - 1) / BLK);
    const int64_t s0 = (first_blk + j) * BLK;
    const int64_t lo = max(max(r.start, (int64_t)0), s0), hi = min(min(r.start + a.slot_len, a.S_logical), s0 + BLK);
    r.lo = (int)(lo - s0);
    r.hi = (int)(hi - s0);
    r.pb = b;
    r.ps0 = s0;
    if (r.lo < r.hi) kv_locate(a.page_table, a.page_tokens, a.pages_per_seq, r.pb, r.ps0);
    return r;
}

template <typename SrcT, bool ROPE, int D>
__global__ void __launch_bounds__(D) append_bf16_tile_kernel(AppendArgs a, int64_t n_tile_wgs) {
    constexpr int BLK = kVBlkBf16;
    constexpr int CH = D / 8;          // 16-byte pieces per row
    constexpr int PITCH = D + 8;       // LDS row pitch in elements: rows start 16 bytes apart modulo the bank cycle
    __shared__ __attribute__((aligned(16))) uint16_t tile[BLK * PITCH];
    const int tid = threadIdx.x;
    if constexpr (ROPE) {
        if ((int64_t)blockIdx.x >= n_tile_wgs) {
            // a workgroup rotates kQRows consecutive rows of one (batch row, query head): its place is decoded once
            // per workgroup, and every lane has kQPerThread independent 16-byte loads in flight
            const uint32_t qi = (uint32_t)(blockIdx.x - n_tile_wgs), n_tb = (uint32_t)a.q_tblocks;
            const uint32_t bh = qi / n_tb, tb = qi % n_tb;
            const int64_t b = bh / (uint32_t)a.Hq, h = bh % (uint32_t)a.Hq;
#pragma unroll
            for (int u = 0; u < kQPerThread; ++u) {
                const int64_t t = (int64_t)tb * kQRows + u * kQRowsPerPass + tid / (D / 8);
                if (t < a.T) rope_q_row<SrcT>(a, b, h, t, 8 * (tid % (D / 8)));
            }
            return;
        }
    }
    const uint32_t bpr = (uint32_t)a.blocks_per_row, bh = blockIdx.x / bpr;
    const int64_t j = blockIdx.x % bpr, h = bh % (uint32_t)a.H, b = bh / (uint32_t)a.H;
    const TileRow r = tile_row<BLK>(a, b, j);
    if (r.lo >= r.hi) return;  // uniform for the workgroup
    const int tok = tid / CH, d0 = 8 * (tid % CH);
    if (tok >= r.lo && tok < r.hi) {
        const int64_t s = r.ps0 + tok;                                   // token inside its slab
        const int64_t pos = (int64_t)((r.start >= 0 ? r.start / BLK : -((-r.start + BLK - 1) / BLK)) + j) * BLK + tok;  // position in the sequence
        const int64_t t = pos - r.start;
        const SrcT* pk = (const SrcT*)a.src_k + b * a.sk[0] + h * a.sk[1] + t * a.sk[2] + d0;
        const SrcT* pv = (const SrcT*)a.src_v + b * a.sv[0] + h * a.sv[1] + t * a.sv[2] + d0;
        uint4 kq, vq;
        if constexpr (sizeof(SrcT) == 2 && !ROPE) {
            kq = *(const uint4*)pk;  // bf16 to bf16: the bits travel as they are
        } else {
            float xk[8];
            load8<SrcT>(pk, xk);
            if constexpr (ROPE) rope_rotate<8>(xk, d0, pos, a);
            kq = pack8_bf16(xk);
        }
        if constexpr (sizeof(SrcT) == 2) {
            vq = *(const uint4*)pv;
        } else {
            float xv[8];
            load8<SrcT>(pv, xv);
            vq = pack8_bf16(xv);
        }
        *(uint4*)((uint16_t*)a.k + kv_off_rowmajor(a.H, a.S, a.D, r.pb, h, s, d0)) = kq;
        *(uint4*)(tile + tok * PITCH + d0) = vq;
    }
    __syncthreads();
    // thread d owns one row of the transposed block: [d][8 tokens]
    const int d = tid;
    uint16_t* dv = (uint16_t*)a.v + kv_off_vblocked(a.H, a.S, a.D, BLK, r.pb, h, r.ps0, d);
    if (r.lo == 0 && r.hi == BLK) {
        uint32_t w[4];
#pragma unroll
        for (int i = 0; i < 4; ++i) w[i] = tile[(2 * i) * PITCH + d] | ((uint32_t)tile[(2 * i + 1) * PITCH + d] << 16);
        *(uint4*)dv = uint4{w[0], w[1], w[2], w[3]};
    } else {
        for (int i = r.lo; i < r.hi; ++i) dv[i] = tile[i * PITCH + d];
    }
}

// Q8_0: a token block is 16 tokens; thread i < D/2 quantises a 32-wide block of K, thread i >= D/2 one of V.
template <typename SrcT, bool ROPE, int D>
__global__ void __launch_bounds__(D) append_q8_tile_kernel(AppendArgs a, int64_t n_tile_wgs) {
    constexpr int BLK = kVBlkQ8;
    constexpr int NQ = D / kQBlock;    // quantisation blocks per row
    constexpr int PITCH = D + 16;      // bytes
    __shared__ __attribute__((aligned(16))) int8_t tile[BLK * PITCH];
    __shared__ uint16_t tile_sc[NQ * BLK];  // [blk][token], the layout of the V scale plane inside a token block
    const int tid = threadIdx.x;
    if constexpr (ROPE) {
        if ((int64_t)blockIdx.x >= n_tile_wgs) {
            // a workgroup rotates kQRows consecutive rows of one (batch row, query head): its place is decoded once
            // per workgroup, and every lane has kQPerThread independent 16-byte loads in flight
            const uint32_t qi = (uint32_t)(blockIdx.x - n_tile_wgs), n_tb = (uint32_t)a.q_tblocks;
            const uint32_t bh = qi / n_tb, tb = qi % n_tb;
            const int64_t b = bh / (uint32_t)a.Hq, h = bh % (uint32_t)a.Hq;
#pragma unroll
            for (int u = 0; u < kQPerThread; ++u) {
                const int64_t t = (int64_t)tb * kQRows + u * kQRowsPerPass + tid / (D / 8);
                if (t < a.T) rope_q_row<SrcT>(a, b, h, t, 8 * (tid % (D / 8)));
            }
            return;
        }
    }
    const uint32_t bpr = (uint32_t)a.blocks_per_row, bh = blockIdx.x / bpr;
    const int64_t j = blockIdx.x % bpr, h = bh % (uint32_t)a.H, b = bh / (uint32_t)a.H;
    const TileRow r = tile_row<BLK>(a, b, j);
    if (r.lo >= r.hi) return;
    const bool is_v = tid >= D / 2;
    const int item = is_v ? tid - D / 2 : tid;  // BLK tokens x NQ blocks = D / 2 items per plane
    const int tok = item / NQ, blk = item % NQ, d0 = blk * kQBlock;
    if (tok >= r.lo && tok < r.hi) {
        const int64_t s = r.ps0 + tok;
        const int64_t pos = (int64_t)((r.start >= 0 ? r.start / BLK : -((-r.start + BLK - 1) / BLK)) + j) * BLK + tok;
        const int64_t t = pos - r.start;
        const SrcT* p = is_v ? (const SrcT*)a.src_v + b * a.sv[0] + h * a.sv[1] + t * a.sv[2] + d0
                             : (const SrcT*)a.src_k + b * a.sk[0] + h * a.sk[1] + t * a.sk[2] + d0;
        float x[kQBlock];
#pragma unroll
        for (int c = 0; c < kQBlock / 8; ++c) {
            float y[8];
            load8<SrcT>(p + 8 * c, y);
#pragma unroll
            for (int e = 0; e < 8; ++e) x[8 * c + e] = y[e];
        }
        if constexpr (ROPE) {
            if (!is_v) rope_rotate<kQBlock>(x, d0, pos, a);
        }
        int8_t q[kQBlock];
        uint16_t sc;
        quantize_block(x, q, &sc);
        uint32_t w[8];
#pragma unroll
        for (int e = 0; e < 8; ++e)
            w[e] = (uint32_t)(uint8_t)q[4 * e] | ((uint32_t)(uint8_t)q[4 * e + 1] << 8) | ((uint32_t)(uint8_t)q[4 * e + 2] << 16) |
                   ((uint32_t)(uint8_t)q[4 * e + 3] << 24);
        if (!is_v) {
            uint4* dk = (uint4*)((int8_t*)a.k + kv_off_rowmajor(a.H, a.S, a.D, r.pb, h, s, d0));
            dk[0] = uint4{w[0], w[1], w[2], w[3]};
            dk[1] = uint4{w[4], w[5], w[6], w[7]};
            ((uint16_t*)a.k_scale)[kv_off_kscale(a.H, a.S, a.D, r.pb, h, s, blk)] = sc;
        } else {
            uint4* dt = (uint4*)(tile + tok * PITCH + d0);
            dt[0] = uint4{w[0], w[1], w[2], w[3]};
            dt[1] = uint4{w[4], w[5], w[6], w[7]};
            tile_sc[blk * BLK + tok] = sc;
        }
    }
    __syncthreads();
    const int d = tid;  // row d of the transposed block: [d][16 tokens]
    int8_t* dv = (int8_t*)a.v + kv_off_vblocked(a.H, a.S, a.D, BLK, r.pb, h, r.ps0, d);
    uint16_t* ds = (uint16_t*)a.v_scale + kv_off_vscale(a.H, a.S, a.D, r.pb, h, r.ps0, 0);  // NQ x 16 scales, contiguous
    if (r.lo == 0 && r.hi == BLK) {
        uint32_t w[4];
#pragma unroll
        for (int i = 0; i < 4; ++i)
            w[i] = (uint32_t)(uint8_t)tile[(4 * i) * PITCH + d] | ((uint32_t)(uint8_t)tile[(4 * i + 1) * PITCH + d] << 8) |
                   ((uint32_t)(uint8_t)tile[(4 * i + 2) * PITCH + d] << 16) | ((uint32_t)(uint8_t)tile[(4 * i + 3) * PITCH + d] << 24);
        *(uint4*)dv = uint4{w[0], w[1], w[2], w[3]};
        if (tid < NQ * BLK) ds[tid] = tile_sc[tid];
    } else {
        for (int i = r.lo; i < r.hi; ++i) dv[i] = tile[i * PITCH + d];
        if (tid < NQ * BLK && (tid % BLK) >= r.lo && (tid % BLK) < r.hi) ds[tid] = tile_sc[tid];
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
        auto rows_aligned16 = [](const vsp_tensor* t) {
            const int esz = t->dtype == VSP_F32 ? 4 : 2;
            if (!is_aligned16(t->data)) return false;
            for (int i = 0; i < 3; ++i)
                if ((t->stride[i] * esz) % 16 != 0) return false;
            return true;
        };
        if (rope) a.q_vec = rows_aligned16(rope->q) && rows_aligned16(rope->q_out) ? 1 : 0;
        a.small_index = (q_items < INT32_MAX && slot_numel < INT32_MAX) ? 1 : 0;
        // eight tokens or more of the cache's own shape, rows 16-byte aligned: the token-block kernels
        const bool tiles = cache->format != VSP_KV_F32 && (a.D == 64 || a.D == 128) && slot_len >= 8 && a.nB == a.B && a.nH == a.H &&
                           a.nT == slot_len && rows_aligned16(new_k) && rows_aligned16(new_v);
        if (tiles) {
            const int BLK = cache->format == VSP_KV_BF16 ? kVBlkBf16 : kVBlkQ8;
            a.blocks_per_row = ceil_div(slot_len, BLK) + 1;  // a slot that starts inside a block touches one more
            const int64_t n_tile_wgs = a.B * a.H * a.blocks_per_row;
            const int threads = (int)a.D;
            a.q_tblocks = rope ? ceil_div(T, kQRows) : 0;
            const int64_t total = n_tile_wgs + (rope ? a.nB * a.Hq * a.q_tblocks : 0);
            if (total > INT32_MAX) return VSP_ERR_ARG;
            const dim3 grid((unsigned)total), block((unsigned)threads);
#define VSP_LAUNCH_TILE(KERNEL)                                                                                               \
    do {                                                                                                                      \
        if (a.D == 128) {                                                                                                     \
            if (f32src && r) hipLaunchKernelGGL((KERNEL<float, true, 128>), grid, block, 0, st, a, n_tile_wgs);                \
            else if (f32src) hipLaunchKernelGGL((KERNEL<float, false, 128>), grid, block, 0, st, a, n_tile_wgs);               \
            else if (r) hipLaunchKernelGGL((KERNEL<uint16_t, true, 128>), grid, block, 0, st, a, n_tile_wgs);                  \
            else hipLaunchKernelGGL((KERNEL<uint16_t, false, 128>), grid, block, 0, st, a, n_tile_wgs);                        \
        } else {                                                                                                              \
            if (f32src && r) hipLaunchKernelGGL((KERNEL<float, true, 64>), grid, block, 0, st, a, n_tile_wgs);                 \
            else if (f32src) hipLaunchKernelGGL((KERNEL<float, false, 64>), grid, block, 0, st, a, n_tile_wgs);                \
            else if (r) hipLaunchKernelGGL((KERNEL<uint16_t, true, 64>), grid, block, 0, st, a, n_tile_wgs);                   \
            else hipLaunchKernelGGL((KERNEL<uint16_t, false, 64>), grid, block, 0, st, a, n_tile_wgs);                         \
        }                                                                                                                     \
    } while (0)
            if (cache->format == VSP_KV_BF16) VSP_LAUNCH_TILE(append_bf16_tile_kernel);
            else VSP_LAUNCH_TILE(append_q8_tile_kernel);
#undef VSP_LAUNCH_TILE
        } else if (cache->format == VSP_KV_F32) {
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
