// Causal GQA flash-attention prefill for gfx950.
//
// Replaces flash_attention_hip_dispatch (include/vesper/ops/flash_attention.h:74-78,
// src/ops/hip/flash_attention.hip:305-331) with repeat_kv (src/ops/attention_ops.cpp:30-57) folded
// into the head indexing.  Same mathematics as the reference's CPU forward
// (src/ops/flash_attention.cpp:218-364): online softmax over key tiles, O = acc / l,
// LSE = m + log l; the arithmetic is bf16 MFMA with fp32 accumulation (or fp32 MFMA for fp32 inputs).
//
// Two bf16 kernels share the tiles and the fragment layouts described here; prefill_bf16_pipe_kernel (D = 128,
// further down) reorders the work of a wavefront into a three-stage software pipeline and is the one the
// benchmark shapes run, prefill_bf16_kernel serves D = 64 and dense inputs with per-row lengths.
//
// A workgroup of 4 wavefronts owns 128 consecutive queries of one (batch, query head);
// each wavefront owns 32 of them.  Key tiles of 32 go from global memory straight into LDS (buffer
// loads with the LDS modifier, a ring of slots, later tiles in flight while the current one is
// consumed, one barrier per tile).  LDS rows are unpadded; 16-byte chunks are XOR-swizzled so that
// both the ds_read_b128 of K and the transposing reads of V are bank-conflict free.  The vector ALU,
// not the matrix pipe, is what these kernels run out of first (vector-ALU work of one wavefront hardly
// overlaps with MFMAs of another wavefront on the same SIMD), so the loops are written to keep VALU
// instructions per MFMA minimal: addresses live in scalar registers, the mask and the rescale are rare
// branches.  Both GEMMs are computed transposed so that the softmax statistics of a query live in one
// lane (and its partner 32 lanes away):
//   S^T[key][q] = K[key][:] . Q^T[:][q]     32x32x16 MFMA, A = K rows from LDS, B = Q^T held in registers
//   O^T[d][q]  += V^T[d][key] . P^T[key][q]  A = V^T read from the row-major V tile with the
//                                            transposing LDS read, B = P^T straight from the S^T registers
// The exponent uses a per-row reference maximum that is only raised (and the accumulators rescaled)
// when the row has outgrown it by a wide margin; the result is mathematically the same
// softmax, without a rescale per tile.  Key tiles entirely above the causal diagonal are skipped;
// the mask is evaluated only on tiles that straddle it.
#include <math.h>

#include <algorithm>
#include <utility>

#include "kv_layout.hpp"
#include "vsp_common.hpp"

namespace vsp {
namespace {

struct PrefillArgs {
    const void* q;
    const void* k;
    const void* v;
    void* out;
    float* lse;  // nullable
    int64_t sq[3], sk[3], sv[3], so[3];  // strides of dims 0..2 (elements)
    int64_t sl[3];                       // lse strides dims 0..2
    int32_t B, Hq, Hkv, n_rep, T, L;
    int32_t causal;
    int32_t n_qtiles;
    int32_t negate_q;  // scale < 0: flip the sign of Q (exact) and use |scale|
    int32_t s_pad;     // cache-plane mode: padded token capacity of the planes
    const int32_t* seq_lens;  // cache-plane mode: per-batch context lengths (device) or nullptr
    const int32_t* chunk_lens;  // cache-plane mode: per-batch number of valid query rows (device) or nullptr
    const int32_t* page_table;  // cache-plane mode, paged cache: [B][pages_per_seq] page indices (device) or nullptr
    int32_t page_tokens, pages_per_seq;
    float scale_log2;  // |scale| * log2(e) for bf16; scale * log2(e) for fp32
    // split-bf16 kernel (fp32 tensors as hi + lo bf16 terms): k / v above are the hi planes, these the lo planes; q is
    // the caller's fp32 tensor
    const void* k_lo;
    const void* v_lo;
    // cache-plane mode, context split over workgroups (n_splits > 1): split s of a query tile covers key tiles
    // [s * split_tiles, (s + 1) * split_tiles) and writes an unnormalised partial instead of the output, row
    // ((b * Hq + hq) * T + t) * n_splits + s of ws_o [..][D] and ws_ml [..][2] = (m in the log2 domain, l)
    int32_t n_splits, split_tiles;
    float* ws_o;
    float* ws_ml;
    int32_t D_true;  // fp32 kernel: the tensors' head_dim when the kernel's tile is wider (columns past it read as zeros)
    int32_t elementwise;  // fp32 kernel: rows are read element by element (any head_dim, any 4-byte aligned pitch)
};

constexpr int kBM = 128;       // queries per workgroup
[[maybe_unused]] constexpr float kRescaleThreshold = 8.0f;

typedef short s16x4_t __attribute__((ext_vector_type(4)));
typedef __bf16 bf16x2_t __attribute__((ext_vector_type(2)));

__device__ inline uint32_t cvt_pk_bf16(float a, float b) {
    typedef float f32x2_t __attribute__((ext_vector_type(2)));
    typedef __bf16 bf16x2_t __attribute__((ext_vector_type(2)));
    f32x2_t v = {a, b};
    return __builtin_bit_cast(uint32_t, __builtin_convertvector(v, bf16x2_t));
}

// Reductions over the two half-waves (lane l and lane l ^ 32 hold the two halves of a query's keys).
// v_permlane32_swap exchanges the upper half of its first operand with the lower half of its second; with a
// copy of x in a second register both halves end up holding (lo[l], hi[l]) pairs: no LDS round trip.
__device__ inline float half_swap_max(float x) {
    float y;
    // two wait states between a vector-ALU write and a permlane swap that reads it
    asm volatile("v_mov_b32 %1, %0\n\ts_nop 1\n\tv_permlane32_swap_b32 %0, %1" : "+v"(x), "=&v"(y));
    return fmaxf(x, y);
}
__device__ inline float half_swap_sum(float x) { return x + __shfl_xor(x, 32); }

// Transposing LDS read issued through inline asm: the compiler cannot prove that a builtin
// transposing read does not alias an outstanding direct-to-LDS load and would wait for every such
// load before it.  The asm form carries no such wait; tr_wait() below is the matching
// "all my LDS reads have returned" fence, tied to the values by data dependence.
template <int OFFSET_BYTES>
__device__ inline uint2 lds_read_tr16_b64_asm(uint32_t lds_byte_addr) {
    uint2 v;
    asm volatile("ds_read_b64_tr_b16 %0, %1 offset:%2" : "=v"(v) : "v"(lds_byte_addr), "n"(OFFSET_BYTES));
    return v;
}
// `tie` is a value computed just before the point where the wait should sit: without it the compiler is free to
// hoist the wait above independent vector-ALU work, which would expose the LDS latency the early read hides.
__device__ inline void tr_wait(uint32_t& tie, uint2& a0, uint2& a1, uint2& a2, uint2& a3, uint2& a4, uint2& a5, uint2& a6, uint2& a7) {
    asm volatile("s_waitcnt lgkmcnt(0)" : "+v"(tie), "+v"(a0), "+v"(a1), "+v"(a2), "+v"(a3), "+v"(a4), "+v"(a5), "+v"(a6), "+v"(a7));
}
__device__ inline void tr_wait(uint32_t& tie, uint2& a0, uint2& a1, uint2& a2, uint2& a3) {
    asm volatile("s_waitcnt lgkmcnt(0)" : "+v"(tie), "+v"(a0), "+v"(a1), "+v"(a2), "+v"(a3));
}
// Plain 16-byte LDS read through inline asm, for the same reason; lds_wait<N>() waits until at most N of
// this wave's LDS operations are outstanding (they return in order) and ties the wait to a value.
typedef uint32_t u32x4_t __attribute__((ext_vector_type(4)));
template <int OFFSET_BYTES>
__device__ inline u32x4_t lds_read_b128_asm(uint32_t lds_byte_addr) {
    u32x4_t v;
    asm volatile("ds_read_b128 %0, %1 offset:%2" : "=v"(v) : "v"(lds_byte_addr), "n"(OFFSET_BYTES));
    return v;
}
template <int N>
__device__ inline void lds_wait(u32x4_t& a0) {
    asm volatile("s_waitcnt lgkmcnt(%1)" : "+v"(a0) : "n"(N));
}
__device__ inline void lds_wait0(uint32_t& tie, u32x4_t& a0, u32x4_t& a1, u32x4_t& a2, u32x4_t& a3) {
    asm volatile("s_waitcnt lgkmcnt(0)" : "+v"(tie), "+v"(a0), "+v"(a1), "+v"(a2), "+v"(a3));
}
__device__ inline void lds_wait0(uint32_t& tie, u32x4_t& a0, u32x4_t& a1) {
    asm volatile("s_waitcnt lgkmcnt(0)" : "+v"(tie), "+v"(a0), "+v"(a1));
}
template <int... I, class F>
__device__ inline void static_for_impl(std::integer_sequence<int, I...>, F&& f) {
    (f(std::integral_constant<int, I>{}), ...);
}
template <int N, class F>
__device__ inline void static_for(F&& f) {
    static_for_impl(std::make_integer_sequence<int, N>{}, f);
}
__device__ inline uint32_t lds_addr(const void* p) {
    return (uint32_t)(uintptr_t)(__attribute__((address_space(3))) const void*)p;
}

[[maybe_unused]] constexpr int kUnit = 32;  // keys per tile (one LDS ring slot)

// VBLK: K and V are the planes of a bf16 KV cache (K row-major, V token-blocked by 8) instead of dense
// tensors, and the context length may come per batch row from a device array.  With 8 tokens of one d
// contiguous, a V^T operand is a plain 16-byte LDS read (no transposing read, no swizzle); to make the
// softmax registers line up with those 8 consecutive tokens, lane i of the K operand holds key
// (i with bits 2 and 3 swapped) of the tile.
template <int D, bool VBLK>
__global__ void __launch_bounds__(256, 3) prefill_bf16_kernel(PrefillArgs a) {
#if defined(__HIP_DEVICE_COMPILE__)  // the body uses device-only builtins
    constexpr int KS = D / 16;
    constexpr int DB = D / 32;
    constexpr int CPR = D / 8;
    constexpr int RP = 256 / (2 * D);
    constexpr int NR = 1024 / (2 * D);
    constexpr int NGRP = kUnit / NR;
    constexpr int NLD = (NGRP + 3) / 4;
    constexpr int SLOT = kUnit * D;
    constexpr int NKB = kUnit / 32;   // 32-key S^T blocks per tile
    constexpr int NJ = kUnit / 16;    // PV k-steps per tile

    // Ring slots: K0 | K1 | V0 | V1, SLOT elements each.  Every read of them is issued from inline asm with
    // the slot as an immediate offset, so the per-lane read addresses are loop constants.
    __shared__ __attribute__((aligned(1024))) uint16_t smem[4 * SLOT];
    constexpr int SLOTB = 2 * SLOT;  // bytes per slot
    const uint32_t lds0 = lds_addr(smem);

    // Block order: heaviest query tiles first (causal work grows with the tile index).  Within one
    // query-tile row, workgroups are dealt round-robin to the 8 XCDs by the hardware (id % 8); when the
    // number of (batch, kv head) groups is a multiple of 8, all query heads of a kv group are given ids
    // of the same residue, so a group's K/V stays in one XCD's L2 instead of being fetched into all eight.
    const int bid = blockIdx.x;
    const int nbh = a.B * a.Hq;
    const int qt = a.n_qtiles - 1 - bid / nbh;
    const int bh = xcd_grouped_head(bid % nbh, a.B * a.Hkv, a.n_rep);
    const int b = bh / a.Hq, hq = bh % a.Hq, kvh = hq / a.n_rep;
    int L = a.L;
    // cache mode: per-row context length (clamped to the bound a.L) and per-row chunk length n <= T:
    // query t < n sits at absolute position L - n + t; rows t >= n carry no query and their output is unspecified
    const int n_chunk = a.chunk_lens ? min(max(a.chunk_lens[b], 0), a.T) : a.T;
    if (a.seq_lens) L = min(max(a.seq_lens[b], n_chunk), a.L);

    const int tid = threadIdx.x, lane = tid & 63;
    const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
    const int ql = lane & 31, h = lane >> 5;
    const int q0 = qt * kBM + wave * 32;
    const int off = L - n_chunk;
    const int qrow = min(q0 + ql, a.T - 1);

    const uint16_t* Qp = (const uint16_t*)a.q + (int64_t)b * a.sq[0] + (int64_t)hq * a.sq[1];
    const uint16_t* Kp = (const uint16_t*)a.k + (int64_t)b * a.sk[0] + (int64_t)kvh * a.sk[1];
    const uint16_t* Vp = (const uint16_t*)a.v + (int64_t)b * a.sv[0] + (int64_t)kvh * a.sv[1];

    bf16x8_t qf[KS];
#pragma unroll
    for (int ks = 0; ks < KS; ++ks) {
        uint4 w = *(const uint4*)(Qp + (int64_t)qrow * a.sq[2] + 16 * ks + 8 * h);
        if (a.negate_q) {
            w.x ^= 0x80008000u;
            w.y ^= 0x80008000u;
            w.z ^= 0x80008000u;
            w.w ^= 0x80008000u;
        }
        qf[ks] = __builtin_bit_cast(bf16x8_t, w);
    }

    const int wg_qmax = min(qt * kBM + kBM - 1, a.T - 1);
    const int kv_end_wg = a.causal ? min(L, wg_qmax + off + 1) : L;
    const int n_tiles = (kv_end_wg + kUnit - 1) / kUnit;
    const int wave_qmax = min(q0 + 31, a.T - 1);
    const int kv_end_wave = (q0 < a.T) ? (a.causal ? min(L, wave_qmax + off + 1) : L) : 0;

    f32x16_t acc[DB];
#pragma unroll
    for (int i = 0; i < DB; ++i)
#pragma unroll
        for (int j = 0; j < 16; ++j) acc[i][j] = 0.f;
    float m_ref = -INFINITY;
    float l = 0.f;

    // Global -> LDS through buffer loads with the LDS modifier: one wave-wide load fills 1024 contiguous
    // bytes of LDS (lane i -> bytes [16 i, 16 i + 16)), i.e. NR rows; the swizzle is applied by choosing
    // which 16-byte chunk of the global row each lane fetches.  The buffer descriptor is rebuilt per tile on
    // the scalar unit (base = first row of the tile, size = bytes up to the end of the context), so the
    // per-lane offsets are loop constants and rows past the end of the context read as zeros.
    const int ld_row = lane / CPR, ld_pos = lane % CPR;
    uint32_t voffK[NLD], voffV[NLD];
#pragma unroll
    for (int i = 0; i < NLD; ++i) {
        const int r = NR * (wave + 4 * i) + ld_row;
        voffK[i] = (uint32_t)r * (uint32_t)a.sk[2] * 2u + 16u * (uint32_t)(ld_pos ^ ((r / RP) % CPR));
        if constexpr (VBLK) voffV[i] = (uint32_t)(wave + 4 * i) * 1024u + 16u * (uint32_t)lane;  // the tile is contiguous
        else voffV[i] = (uint32_t)r * (uint32_t)a.sv[2] * 2u + 16u * (uint32_t)(ld_pos ^ (((r / RP) % (CPR / 4)) << 2));
    }
    const int64_t rowK = a.sk[2] * 2, rowV = a.sv[2] * 2;  // bytes per key row
    auto load_tile = [&](int t, int slot) {
        const int key0 = t * kUnit;
        int rows = L - key0;  // > 0
        const char* kb = (const char*)Kp;
        const char* vb = (const char*)Vp;
        int local = key0, cap = a.s_pad;  // first token of the tile inside its [cap][D] slab
        if constexpr (VBLK) {
            if (a.page_table) {  // paged cache: a tile (32 tokens) never straddles a page (a multiple of 64 tokens)
                const int pg = key0 / a.page_tokens;
                local = key0 - pg * a.page_tokens;
                cap = a.page_tokens;
                const int64_t slab = (int64_t)a.page_table[(int64_t)b * a.pages_per_seq + pg] * a.Hkv + kvh;
                kb = (const char*)a.k + slab * cap * D * 2;
                vb = (const char*)a.v + slab * cap * D * 2;
                rows = min(rows, cap - local);
            }
        }
        __amdgpu_buffer_rsrc_t rk = __builtin_amdgcn_make_buffer_rsrc((void*)(kb + (int64_t)local * rowK), 0, (int)((int64_t)rows * rowK), 0x00020000);
        // VBLK: 32 tokens = 4 token blocks = kUnit * D contiguous elements; bound = the rest of this head's slab
        const int64_t v_base = VBLK ? (int64_t)local * D * 2 : (int64_t)key0 * rowV;
        const int64_t v_bytes = VBLK ? ((int64_t)cap - local) * D * 2 : (int64_t)rows * rowV;
        __amdgpu_buffer_rsrc_t rv = __builtin_amdgcn_make_buffer_rsrc((void*)(vb + v_base), 0, (int)v_bytes, 0x00020000);
        uint16_t* dstK = smem + slot * SLOT;
        uint16_t* dstV = smem + (2 + slot) * SLOT;
#pragma unroll
        for (int i = 0; i < NLD; ++i) {
            const int grp = wave + 4 * i;
            if (NGRP % 4 != 0 && grp >= NGRP) break;
            __builtin_amdgcn_raw_ptr_buffer_load_lds(rk, (__attribute__((address_space(3))) void*)(dstK + grp * 512), 16, voffK[i], 0, 0, 0);
            __builtin_amdgcn_raw_ptr_buffer_load_lds(rv, (__attribute__((address_space(3))) void*)(dstV + grp * 512), 16, voffV[i], 0, 0, 0);
        }
    };

    // Loop-constant LDS read addresses (slot 0; the slot is an immediate offset on the instruction).
    const int krow = VBLK ? ((ql & ~12) | ((ql & 4) << 1) | ((ql & 8) >> 1)) : ql;  // tile row this lane's S^T row holds
    const int kswz = (krow / RP) % CPR;
    uint32_t kaddr[KS];
#pragma unroll
    for (int ks = 0; ks < KS; ++ks) kaddr[ks] = lds0 + 2u * (uint32_t)(krow * D + 8 * ((2 * ks + h) ^ kswz));
    const int i16 = lane & 15;
    const int vswz = ((i16 >> 2) / RP) % (CPR / 4);
    const int v_lane_off = (4 * h + (i16 >> 2)) * D + 16 * ((lane >> 4) & 1) + 4 * (lane & 3);
    uint32_t va[DB];
#pragma unroll
    for (int db = 0; db < DB; ++db)
        va[db] = VBLK ? lds0 + 16u * (uint32_t)(h * D + ql) : lds0 + 2u * (uint32_t)v_lane_off + 64u * (uint32_t)(db ^ vswz);

    constexpr int PF = 4;  // K fragments in flight

    auto tile_step = [&](int t, auto slot_c) {
        constexpr int slot = decltype(slot_c)::value;
        constexpr int KOFF = slot * SLOTB;
        constexpr int VOFF = (2 + slot) * SLOTB;
        asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
        __syncthreads();
        if (t + 1 < n_tiles) load_tile(t + 1, slot ^ 1);
        const int k0 = t * kUnit;
        if (k0 >= kv_end_wave) return;

        static_assert(NKB == 1, "one 32-key block per tile");
        f32x16_t s[NKB];
#pragma unroll
        for (int j = 0; j < 16; ++j) s[0][j] = 0.f;
        u32x4_t kf[KS];
        static_for<PF>([&](auto i) { kf[i.value] = lds_read_b128_asm<KOFF>(kaddr[i.value]); });
        static_for<KS>([&](auto i) {
            constexpr int ks = i.value;
            constexpr int issued = (ks + PF < KS) ? ks + PF : KS;
            lds_wait<issued - ks - 1>(kf[ks]);
            s[0] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(__builtin_bit_cast(bf16x8_t, kf[ks]), qf[ks], s[0], 0, 0, 0);
            if constexpr (ks + PF < KS) kf[ks + PF] = lds_read_b128_asm<KOFF>(kaddr[ks + PF]);
        });
        // the first V fragments are requested now, so that their LDS latency passes under the softmax
        u32x4_t vcur[DB];
        uint2 tcur[DB][2];
        if constexpr (VBLK) {
            static_for<DB>([&](auto dbc) { vcur[dbc.value] = lds_read_b128_asm<VOFF + 512 * dbc.value>(va[dbc.value]); });
        } else {
#pragma unroll
            for (int db = 0; db < DB; ++db) {
                tcur[db][0] = lds_read_tr16_b64_asm<VOFF>(va[db]);
                tcur[db][1] = lds_read_tr16_b64_asm<VOFF + 8 * D * 2>(va[db]);
            }
        }
        const bool need_mask = (a.causal && k0 + kUnit - 1 > q0 + off) || (k0 + kUnit > L);
        if (need_mask) {
            const int q_abs = q0 + ql + off;
            const int lim = a.causal ? min(q_abs, L - 1) : L - 1;
#pragma unroll
            for (int v = 0; v < 16; ++v) {
                const int key = VBLK ? k0 + 16 * (v >> 3) + 8 * h + (v & 7) : k0 + 8 * (v >> 2) + 4 * h + (v & 3);
                if (key > lim) s[0][v] = -INFINITY;
            }
        }
        // P is taken against the row's reference maximum as it stands, and the row sum says whether that reference
        // has fallen behind: below 2^10 no P of the tile exceeds 2^10, far from overflow in the fp32 accumulators.
        // Otherwise (rare on real data; always for the first tile, which has no reference yet) the true maximum of
        // these scores becomes the reference, what has been accumulated is rescaled and this tile's P is redone.  The
        // mathematics is the reference's online softmax (src/ops/flash_attention.cpp:309-343) with a reference point
        // that moves only when it has to, which takes the per-tile row maximum (16 max + a cross-half exchange) out of
        // the steady state.  The row sum is taken from the rounded bf16 P (packed dot product against (1, 1)): exactly
        // what the PV MFMAs accumulate.
        uint32_t pw[NJ][4];
        float lsum = 0.f;
        auto softmax = [&](float neg_m) {
            lsum = 0.f;
#pragma unroll
            for (int v = 0; v < 16; v += 2) {
                const float p0 = __builtin_amdgcn_exp2f(__builtin_fmaf(s[0][v], a.scale_log2, neg_m));
                const float p1 = __builtin_amdgcn_exp2f(__builtin_fmaf(s[0][v + 1], a.scale_log2, neg_m));
                const uint32_t pk = cvt_pk_bf16(p0, p1);
                pw[v >> 3][(v & 7) >> 1] = pk;
                lsum = __builtin_amdgcn_fdot2_f32_bf16(__builtin_bit_cast(bf16x2_t, pk), __builtin_bit_cast(bf16x2_t, 0x3f803f80u), lsum, false);
            }
        };
        if (t > 0) softmax(m_ref == -INFINITY ? 0.f : -m_ref);
        if (t == 0 || __any(!(lsum < 1024.f))) {
            float mx = s[0][0];
#pragma unroll
            for (int v = 0; v < 16; ++v) mx = fmaxf(mx, s[0][v]);
            mx = half_swap_max(mx) * a.scale_log2;
            const float m_new = fmaxf(m_ref, mx);
            const float alpha = (m_new == -INFINITY || m_ref == -INFINITY) ? 1.f : __builtin_amdgcn_exp2f(m_ref - m_new);
            l *= alpha;
#pragma unroll
            for (int i = 0; i < DB; ++i)
#pragma unroll
                for (int j = 0; j < 16; ++j) acc[i][j] *= alpha;
            m_ref = m_new;
            softmax(m_ref == -INFINITY ? 0.f : -m_ref);
        }
        l += lsum;
        // PV
        if constexpr (VBLK) {
            u32x4_t vnext[DB];
            const bool tail = k0 + kUnit > L;  // the planes hold stale tokens past L: P is 0 there, V must not be NaN
            static_for<NJ>([&](auto jc) {
                constexpr int j = jc.value;
                if constexpr (DB == 4) lds_wait0(pw[j][3], vcur[0], vcur[1], vcur[2], vcur[3]);
                else lds_wait0(pw[j][3], vcur[0], vcur[1]);
                if constexpr (j + 1 < NJ)
                    static_for<DB>([&](auto dbc) {
                        vnext[dbc.value] = lds_read_b128_asm<VOFF + (2 * (j + 1) * D + 32 * dbc.value) * 16>(va[dbc.value]);
                    });
                if (tail) {
                    const int nvalid = L - (k0 + 16 * j + 8 * h);  // slots e >= nvalid are past the context
#pragma unroll
                    for (int db = 0; db < DB; ++db)
#pragma unroll
                        for (int w = 0; w < 4; ++w) {
                            uint32_t x = vcur[db][w];
                            if (2 * w + 1 >= nvalid) x &= 0x0000ffffu;
                            if (2 * w >= nvalid) x = 0;
                            vcur[db][w] = x;
                        }
                }
                const bf16x8_t pf = __builtin_bit_cast(bf16x8_t, uint4{pw[j][0], pw[j][1], pw[j][2], pw[j][3]});
#pragma unroll
                for (int db = 0; db < DB; ++db)
                    acc[db] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(__builtin_bit_cast(bf16x8_t, vcur[db]), pf, acc[db], 0, 0, 0);
                if constexpr (j + 1 < NJ) {
#pragma unroll
                    for (int db = 0; db < DB; ++db) vcur[db] = vnext[db];
                }
            });
            return;
        }
        uint2 tnext[DB][2];
        static_for<NJ>([&](auto jc) {
            constexpr int j = jc.value;
            if constexpr (DB == 4) tr_wait(pw[j][3], tcur[0][0], tcur[0][1], tcur[1][0], tcur[1][1], tcur[2][0], tcur[2][1], tcur[3][0], tcur[3][1]);
            else tr_wait(pw[j][3], tcur[0][0], tcur[0][1], tcur[1][0], tcur[1][1]);
            if constexpr (j + 1 < NJ) {
#pragma unroll
                for (int db = 0; db < DB; ++db) {
                    tnext[db][0] = lds_read_tr16_b64_asm<VOFF + (16 * (j + 1)) * D * 2>(va[db]);
                    tnext[db][1] = lds_read_tr16_b64_asm<VOFF + (16 * (j + 1) + 8) * D * 2>(va[db]);
                }
            }
            const bf16x8_t pf = __builtin_bit_cast(bf16x8_t, uint4{pw[j][0], pw[j][1], pw[j][2], pw[j][3]});
#pragma unroll
            for (int db = 0; db < DB; ++db) {
                const bf16x8_t vf = __builtin_bit_cast(bf16x8_t, uint4{tcur[db][0].x, tcur[db][0].y, tcur[db][1].x, tcur[db][1].y});
                acc[db] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(vf, pf, acc[db], 0, 0, 0);
            }
            if constexpr (j + 1 < NJ) {
#pragma unroll
                for (int db = 0; db < DB; ++db) {
                    tcur[db][0] = tnext[db][0];
                    tcur[db][1] = tnext[db][1];
                }
            }
        });
    };

    if (n_tiles > 0) load_tile(0, 0);
    for (int t = 0; t < n_tiles; t += 2) {
        tile_step(t, std::integral_constant<int, 0>{});
        if (t + 1 < n_tiles) tile_step(t + 1, std::integral_constant<int, 1>{});
    }

    l = half_swap_sum(l);
    const int qi = q0 + ql;
    if (qi < a.T) {
        const float inv_l = l > 0.f ? 1.0f / l : 0.f;  // an empty context (cache mode, length 0) gives zeros
        uint16_t* op = (uint16_t*)a.out + (int64_t)b * a.so[0] + (int64_t)hq * a.so[1] + (int64_t)qi * a.so[2];
#pragma unroll
        for (int db = 0; db < DB; ++db)
#pragma unroll
            for (int vq = 0; vq < 4; ++vq) {
                const int d = 32 * db + 8 * vq + 4 * h;
                uint2 w;
                w.x = cvt_pk_bf16(acc[db][4 * vq] * inv_l, acc[db][4 * vq + 1] * inv_l);  // round-to-nearest-even
                w.y = cvt_pk_bf16(acc[db][4 * vq + 2] * inv_l, acc[db][4 * vq + 3] * inv_l);
                *(uint2*)(op + d) = w;
            }
        if (a.lse && h == 0)
            a.lse[(int64_t)b * a.sl[0] + (int64_t)hq * a.sl[1] + (int64_t)qi * a.sl[2]] = (m_ref + __builtin_amdgcn_logf(l)) * 0.6931471805599453f;
    }
#endif
}

// ---------------------------------------------------------------------------------------------
// fp32 tensors on the bf16 matrix cores.  Every operand x is split into two bf16 terms, x = hi + lo with hi = bf16(x)
// and lo = bf16(x - hi) (16 significant bits between them), and every product is taken as
//     a b  ~  hi_a hi_b + hi_a lo_b + lo_a hi_b          (fp32 accumulation; the dropped lo_a lo_b is 2^-16 of a b)
// for Q K^T and, with P split the same way after the exponential, for P V.  Three bf16 MFMAs per product at 16 times the
// fp32 MFMA rate, against the reference's fp32 arithmetic (src/ops/flash_attention.cpp:218-364) within its 1e-4 bar
// (observed: below 2e-5 of the output's magnitude).  A pre-pass writes the hi / lo planes of K and V, dense, into a
// caller workspace (Q is split by the wavefront that owns the rows); the attention kernel is prefill_bf16_kernel's
// structure over twice the tiles.
// ---------------------------------------------------------------------------------------------
struct SplitPlan {  // K and V
    const float* src[2];
    uint16_t* hi[2];
    uint16_t* lo[2];
    int64_t s0[2], s1[2], s2[2];  // source strides of dims 0..2 (elements)
    int32_t H, N;
    int64_t groups;               // 8-element groups per tensor
    int32_t D;
};

__global__ void __launch_bounds__(256) split_f32_kernel(SplitPlan p) {
    const int t = blockIdx.y;
    const int64_t g = (int64_t)blockIdx.x * 256 + threadIdx.x;
    if (g >= p.groups) return;
    const int per_row = p.D / 8;
    const int d8 = (int)(g % per_row);
    const int64_t row = g / per_row;
    const int n = (int)(row % p.N);
    const int64_t bh = row / p.N;
    const int h = (int)(bh % p.H);
    const int64_t b = bh / p.H;
    const float* src = p.src[t] + b * p.s0[t] + (int64_t)h * p.s1[t] + (int64_t)n * p.s2[t] + 8 * d8;
    const float4 x0 = *(const float4*)src, x1 = *(const float4*)(src + 4);
    const float x[8] = {x0.x, x0.y, x0.z, x0.w, x1.x, x1.y, x1.z, x1.w};
    uint32_t hw[4], lw[4];
#pragma unroll
    for (int i = 0; i < 4; ++i) {
        hw[i] = cvt_pk_bf16(x[2 * i], x[2 * i + 1]);
        const float r0 = x[2 * i] - __uint_as_float(hw[i] << 16), r1 = x[2 * i + 1] - __uint_as_float(hw[i] & 0xffff0000u);
        lw[i] = cvt_pk_bf16(r0, r1);
    }
    *(uint4*)(p.hi[t] + g * 8) = uint4{hw[0], hw[1], hw[2], hw[3]};
    *(uint4*)(p.lo[t] + g * 8) = uint4{lw[0], lw[1], lw[2], lw[3]};
}

template <int D>
__global__ void __launch_bounds__(256, 2) prefill_split_kernel(PrefillArgs a) {
#if defined(__HIP_DEVICE_COMPILE__)  // the body uses device-only builtins
    constexpr int KS = D / 16;
    constexpr int DB = D / 32;
    constexpr int CPR = D / 8;
    constexpr int RP = 256 / (2 * D);
    constexpr int NR = 1024 / (2 * D);
    constexpr int NGRP = kUnit / NR;
    constexpr int NLD = (NGRP + 3) / 4;
    constexpr int SLOT = kUnit * D;
    constexpr int NJ = kUnit / 16;
    constexpr int SLOTB = 2 * SLOT;  // bytes per tile
    // ring slot r holds four tiles: K hi | K lo | V hi | V lo
    __shared__ __attribute__((aligned(1024))) uint16_t smem[8 * SLOT];
    const uint32_t lds0 = lds_addr(smem);

    const int bid = blockIdx.x;
    const int nbh = a.B * a.Hq;
    const int qt = a.n_qtiles - 1 - bid / nbh;  // heaviest query tiles first
    const int bh = xcd_grouped_head(bid % nbh, a.B * a.Hkv, a.n_rep);  // a kv group's query heads share one XCD's L2
    const int b = bh / a.Hq, hq = bh % a.Hq, kvh = hq / a.n_rep;
    const int L = a.L;
    const int tid = threadIdx.x, lane = tid & 63;
    const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
    const int ql = lane & 31, h = lane >> 5;
    const int q0 = qt * kBM + wave * 32;
    const int off = L - a.T;
    const int qrow = min(q0 + ql, a.T - 1);

    const int64_t ko = (int64_t)b * a.sk[0] + (int64_t)kvh * a.sk[1];
    const int64_t vo = (int64_t)b * a.sv[0] + (int64_t)kvh * a.sv[1];
    // Q comes as the caller's fp32 tensor (any strides) and is split here: each row is read by exactly one wavefront
    const float* qp = (const float*)a.q + (int64_t)b * a.sq[0] + (int64_t)hq * a.sq[1] + (int64_t)qrow * a.sq[2];
    bf16x8_t qh[KS], qlo[KS];
#pragma unroll
    for (int ks = 0; ks < KS; ++ks) {
        const float4 x0 = *(const float4*)(qp + 16 * ks + 8 * h), x1 = *(const float4*)(qp + 16 * ks + 8 * h + 4);
        float x[8] = {x0.x, x0.y, x0.z, x0.w, x1.x, x1.y, x1.z, x1.w};
        uint32_t hw[4], lw[4];
#pragma unroll
        for (int i = 0; i < 4; ++i) {
            const float f0 = a.negate_q ? -x[2 * i] : x[2 * i], f1 = a.negate_q ? -x[2 * i + 1] : x[2 * i + 1];  // exact
            hw[i] = cvt_pk_bf16(f0, f1);
            lw[i] = cvt_pk_bf16(f0 - __uint_as_float(hw[i] << 16), f1 - __uint_as_float(hw[i] & 0xffff0000u));
        }
        qh[ks] = __builtin_bit_cast(bf16x8_t, uint4{hw[0], hw[1], hw[2], hw[3]});
        qlo[ks] = __builtin_bit_cast(bf16x8_t, uint4{lw[0], lw[1], lw[2], lw[3]});
    }

    const int wg_qmax = min(qt * kBM + kBM - 1, a.T - 1);
    const int kv_end_wg = a.causal ? min(L, wg_qmax + off + 1) : L;
    const int n_tiles = (kv_end_wg + kUnit - 1) / kUnit;
    const int wave_qmax = min(q0 + 31, a.T - 1);
    const int kv_end_wave = (q0 < a.T) ? (a.causal ? min(L, wave_qmax + off + 1) : L) : 0;

    f32x16_t acc[DB];
#pragma unroll
    for (int i = 0; i < DB; ++i)
#pragma unroll
        for (int j = 0; j < 16; ++j) acc[i][j] = 0.f;
    float m_ref = -INFINITY;
    float l = 0.f;

    // global -> LDS as in prefill_bf16_kernel; the planes are dense, so K and V rows have the same pitch
    const int ld_row = lane / CPR, ld_pos = lane % CPR;
    uint32_t voffK[NLD], voffV[NLD];
#pragma unroll
    for (int i = 0; i < NLD; ++i) {
        const int r = NR * (wave + 4 * i) + ld_row;
        voffK[i] = (uint32_t)r * (uint32_t)(2 * D) + 16u * (uint32_t)(ld_pos ^ ((r / RP) % CPR));
        voffV[i] = (uint32_t)r * (uint32_t)(2 * D) + 16u * (uint32_t)(ld_pos ^ (((r / RP) % (CPR / 4)) << 2));
    }
    auto load_tile = [&](int t, int slot) {
        const int key0 = t * kUnit;
        const int bytes = (L - key0) * 2 * D;  // rows past the context read as zeros
        const char* bases[4] = {(const char*)((const uint16_t*)a.k + ko), (const char*)((const uint16_t*)a.k_lo + ko),
                                (const char*)((const uint16_t*)a.v + vo), (const char*)((const uint16_t*)a.v_lo + vo)};
#pragma unroll
        for (int x = 0; x < 4; ++x) {
            __amdgpu_buffer_rsrc_t rs = __builtin_amdgcn_make_buffer_rsrc((void*)(bases[x] + (int64_t)key0 * 2 * D), 0, bytes, 0x00020000);
            uint16_t* dst = smem + (4 * slot + x) * SLOT;
#pragma unroll
            for (int i = 0; i < NLD; ++i) {
                const int grp = wave + 4 * i;
                if (NGRP % 4 != 0 && grp >= NGRP) break;
                __builtin_amdgcn_raw_ptr_buffer_load_lds(rs, (__attribute__((address_space(3))) void*)(dst + grp * 512), 16, x < 2 ? voffK[i] : voffV[i], 0, 0, 0);
            }
        }
    };

    const int kswz = (ql / RP) % CPR;
    uint32_t kaddr[KS];
#pragma unroll
    for (int ks = 0; ks < KS; ++ks) kaddr[ks] = lds0 + 2u * (uint32_t)(ql * D + 8 * ((2 * ks + h) ^ kswz));
    const int i16 = lane & 15;
    const int vswz = ((i16 >> 2) / RP) % (CPR / 4);
    const int v_lane_off = (4 * h + (i16 >> 2)) * D + 16 * ((lane >> 4) & 1) + 4 * (lane & 3);
    uint32_t va[DB];
#pragma unroll
    for (int db = 0; db < DB; ++db) va[db] = lds0 + 2u * (uint32_t)v_lane_off + 64u * (uint32_t)(db ^ vswz);

    auto tile_step = [&](int t, auto slot_c) {
        constexpr int slot = decltype(slot_c)::value;
        constexpr int KH = (4 * slot) * SLOTB, KL = (4 * slot + 1) * SLOTB, VH = (4 * slot + 2) * SLOTB, VL = (4 * slot + 3) * SLOTB;
        asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
        __syncthreads();
        if (t + 1 < n_tiles) load_tile(t + 1, slot ^ 1);
        const int k0 = t * kUnit;
        if (k0 >= kv_end_wave) return;

        // S^T = K_hi Q_hi^T + K_hi Q_lo^T + K_lo Q_hi^T; the operands of k-step ks + 1 are requested before those of ks are used
        f32x16_t s;
#pragma unroll
        for (int j = 0; j < 16; ++j) s[j] = 0.f;
        u32x4_t kh[KS], kl[KS];
        kh[0] = lds_read_b128_asm<KH>(kaddr[0]);
        kl[0] = lds_read_b128_asm<KL>(kaddr[0]);
        static_for<KS>([&](auto i) {
            constexpr int ks = i.value;
            if constexpr (ks + 1 < KS) {
                kh[ks + 1] = lds_read_b128_asm<KH>(kaddr[ks + 1]);
                kl[ks + 1] = lds_read_b128_asm<KL>(kaddr[ks + 1]);
                lds_wait<3>(kh[ks]);
                lds_wait<2>(kl[ks]);
            } else {
                lds_wait<1>(kh[ks]);
                lds_wait<0>(kl[ks]);
            }
            s = __builtin_amdgcn_mfma_f32_32x32x16_bf16(__builtin_bit_cast(bf16x8_t, kh[ks]), qh[ks], s, 0, 0, 0);
            s = __builtin_amdgcn_mfma_f32_32x32x16_bf16(__builtin_bit_cast(bf16x8_t, kh[ks]), qlo[ks], s, 0, 0, 0);
            s = __builtin_amdgcn_mfma_f32_32x32x16_bf16(__builtin_bit_cast(bf16x8_t, kl[ks]), qh[ks], s, 0, 0, 0);
        });
        const bool need_mask = (a.causal && k0 + kUnit - 1 > q0 + off) || (k0 + kUnit > L);
        if (need_mask) {
            const int q_abs = q0 + ql + off;
            const int lim = a.causal ? min(q_abs, L - 1) : L - 1;
#pragma unroll
            for (int v = 0; v < 16; ++v)
                if (k0 + 8 * (v >> 2) + 4 * h + (v & 3) > lim) s[v] = -INFINITY;
        }
        float mx = s[0];
#pragma unroll
        for (int v = 1; v < 16; ++v) mx = fmaxf(mx, s[v]);
        mx = half_swap_max(mx) * a.scale_log2;
        if (__any(mx > m_ref + kRescaleThreshold)) {  // P stays below 2^8 between raises: nothing to lose in fp32
            const float m_new = fmaxf(m_ref, mx);
            const float alpha = (m_new == -INFINITY || m_ref == -INFINITY) ? (m_ref == -INFINITY ? 0.f : 1.f) : __builtin_amdgcn_exp2f(m_ref - m_new);
            l *= alpha;
#pragma unroll
            for (int i = 0; i < DB; ++i)
#pragma unroll
                for (int j = 0; j < 16; ++j) acc[i][j] *= alpha;
            m_ref = m_new;
        }
        const float neg_m = (m_ref == -INFINITY) ? 0.f : -m_ref;
        // P = exp2(s scale - m) in fp32, summed in fp32, then split like the inputs
        uint32_t ph[NJ][4], pl[NJ][4];
        float lsum = 0.f;
#pragma unroll
        for (int v = 0; v < 16; v += 2) {
            const float p0 = __builtin_amdgcn_exp2f(__builtin_fmaf(s[v], a.scale_log2, neg_m));
            const float p1 = __builtin_amdgcn_exp2f(__builtin_fmaf(s[v + 1], a.scale_log2, neg_m));
            lsum += p0 + p1;
            const uint32_t hw = cvt_pk_bf16(p0, p1);
            ph[v >> 3][(v & 7) >> 1] = hw;
            pl[v >> 3][(v & 7) >> 1] = cvt_pk_bf16(p0 - __uint_as_float(hw << 16), p1 - __uint_as_float(hw & 0xffff0000u));
        }
        l += lsum;
        // O^T += V_hi^T P_hi + V_hi^T P_lo + V_lo^T P_hi, one (key half, d block) at a time, the next operands in flight
        uint2 vh[2], vl[2], nh[2], nl[2];
        vh[0] = lds_read_tr16_b64_asm<VH>(va[0]);
        vh[1] = lds_read_tr16_b64_asm<VH + 8 * D * 2>(va[0]);
        vl[0] = lds_read_tr16_b64_asm<VL>(va[0]);
        vl[1] = lds_read_tr16_b64_asm<VL + 8 * D * 2>(va[0]);
        static_for<NJ * DB>([&](auto ic) {
            constexpr int idx = ic.value, j = idx / DB, db = idx % DB;
            if constexpr (idx + 1 < NJ * DB) {
                constexpr int j2 = (idx + 1) / DB, db2 = (idx + 1) % DB;
                nh[0] = lds_read_tr16_b64_asm<VH + (16 * j2) * D * 2>(va[db2]);
                nh[1] = lds_read_tr16_b64_asm<VH + (16 * j2 + 8) * D * 2>(va[db2]);
                nl[0] = lds_read_tr16_b64_asm<VL + (16 * j2) * D * 2>(va[db2]);
                nl[1] = lds_read_tr16_b64_asm<VL + (16 * j2 + 8) * D * 2>(va[db2]);
                asm volatile("s_waitcnt lgkmcnt(4)" : "+v"(vh[0]), "+v"(vh[1]), "+v"(vl[0]), "+v"(vl[1]));
            } else {
                asm volatile("s_waitcnt lgkmcnt(0)" : "+v"(vh[0]), "+v"(vh[1]), "+v"(vl[0]), "+v"(vl[1]));
            }
            const bf16x8_t pfh = __builtin_bit_cast(bf16x8_t, uint4{ph[j][0], ph[j][1], ph[j][2], ph[j][3]});
            const bf16x8_t pfl = __builtin_bit_cast(bf16x8_t, uint4{pl[j][0], pl[j][1], pl[j][2], pl[j][3]});
            const bf16x8_t vfh = __builtin_bit_cast(bf16x8_t, uint4{vh[0].x, vh[0].y, vh[1].x, vh[1].y});
            const bf16x8_t vfl = __builtin_bit_cast(bf16x8_t, uint4{vl[0].x, vl[0].y, vl[1].x, vl[1].y});
            acc[db] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(vfh, pfh, acc[db], 0, 0, 0);
            acc[db] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(vfh, pfl, acc[db], 0, 0, 0);
            acc[db] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(vfl, pfh, acc[db], 0, 0, 0);
            if constexpr (idx + 1 < NJ * DB) {
                vh[0] = nh[0];
                vh[1] = nh[1];
                vl[0] = nl[0];
                vl[1] = nl[1];
            }
        });
    };

    if (n_tiles > 0) load_tile(0, 0);
    for (int t = 0; t < n_tiles; t += 2) {
        tile_step(t, std::integral_constant<int, 0>{});
        if (t + 1 < n_tiles) tile_step(t + 1, std::integral_constant<int, 1>{});
    }

    l = half_swap_sum(l);
    const int qi = q0 + ql;
    if (qi < a.T) {
        const float inv_l = l > 0.f ? 1.0f / l : 0.f;
        float* op = (float*)a.out + (int64_t)b * a.so[0] + (int64_t)hq * a.so[1] + (int64_t)qi * a.so[2];
#pragma unroll
        for (int db = 0; db < DB; ++db)
#pragma unroll
            for (int vq = 0; vq < 4; ++vq)
                *(float4*)(op + 32 * db + 8 * vq + 4 * h) = float4{acc[db][4 * vq] * inv_l, acc[db][4 * vq + 1] * inv_l, acc[db][4 * vq + 2] * inv_l, acc[db][4 * vq + 3] * inv_l};
        if (a.lse && h == 0)
            a.lse[(int64_t)b * a.sl[0] + (int64_t)hq * a.sl[1] + (int64_t)qi * a.sl[2]] = (m_ref + log2f(l)) * 0.6931471805599453f;
    }
#endif
}

// ---------------------------------------------------------------------------------------------
// Software-pipelined bf16 kernel, D = 128, dense K/V.  Same tiles, fragment layouts and arithmetic as
// prefill_bf16_kernel; what changes is the order of work inside a wavefront.  Step tau of a wavefront issues, as
// three independent instruction streams,
//     S(tau+2) = K(tau+2) Q^T          8 MFMAs into the "next" score registers
//     P(tau+1) = exp2(S(tau+1) - m)    the vector-ALU work, on scores finished one step earlier
//     O       += V(tau)^T P(tau)       8 MFMAs with the P computed one step earlier
// so no MFMA of a step waits for vector-ALU work of the same step and vice versa: the matrix pipe and the vector ALU
// of one SIMD run side by side from a single wavefront's instruction stream.  The 16 MFMAs of a step are "slots";
// each slot is followed by its share of the softmax instructions and by the LDS reads of the operand needed kLead
// slots later (the reads run ahead across step boundaries).  Four ring slots per operand in LDS: the tiles a step
// needs were requested three steps earlier and published by the barrier one step earlier, so neither the barrier nor
// the global loads sit on a wavefront's critical path.
// Vector-ALU instructions of one wavefront hardly overlap with MFMAs of ANOTHER wavefront on the same SIMD (a wavefront
// of nothing but vector-ALU work gets about one instruction in per MFMA of its neighbour), while those that follow an
// MFMA in the same instruction stream are nearly free; hence this structure, and the diet of the softmax stage:
//   - -m / c (m: the row's reference maximum, c = |scale| * log2(e)) enters as the C operand of the first QK^T MFMA,
//     so P is one multiply and one exp2 per score (Q is not pre-multiplied by c: rounding Q * c to bf16 again costs
//     2^-9 of every score, which shows in the output once logits reach the tens);
//   - the row sum uses plain adds (v_dot2c_f32_bf16 occupies the matrix pipe);
//   - no row maximum per tile: m is raised only when the row sum shows that it has fallen behind (rare), and is
//     kept integer-valued (log2 domain) so that the rescale factor is a power of two and the P tile that has been
//     computed but not yet multiplied into O rescales exactly.
// ---------------------------------------------------------------------------------------------
constexpr int kLead = 6;  // LDS operand reads run this many MFMA slots ahead

// MFMA slot order of a step: Q = a QK^T MFMA (k-step index), P = a PV MFMA (index p: key half p / 4, d block p % 4).
// The QK chain finishes at slot 10, so that the row maximum of the new scores is taken under the last PV MFMAs.
constexpr int kSlotIsQ[16] = {1, 1, 0, 1, 1, 0, 1, 1, 0, 1, 1, 0, 0, 0, 0, 0};
[[maybe_unused]] constexpr int kSlotIdx[16] = {0, 1, 0, 2, 3, 1, 4, 5, 2, 6, 7, 3, 4, 5, 6, 7};
// LDS read instructions per operand: one ds_read_b128 for K rows and for V^T taken from a token-blocked plane, two
// transposing reads for V^T taken from row-major V
template <bool VBLK>
constexpr int slot_reads(int s) { return (kSlotIsQ[s & 15] || VBLK) ? 1 : 2; }
// LDS reads issued after the operand of slot s and before the wait at slot s: those of slots s+1 .. s+kLead-1
template <bool VBLK>
constexpr int reads_behind(int s) {
    int n = 0;
    for (int k = 1; k < kLead; ++k) n += slot_reads<VBLK>(s + k);
    return n;
}

struct Frag {  // one MFMA A operand on its way from LDS
    u32x4_t k;     // K rows (ds_read_b128)
    uint2 t0, t1;  // V^T halves (two transposing reads)
};

template <int N>
__device__ inline void frag_wait_k(u32x4_t& k) {
    asm volatile("s_waitcnt lgkmcnt(%1)" : "+v"(k) : "n"(N));
}
template <int N>
__device__ inline void frag_wait_v(uint2& t0, uint2& t1) {
    asm volatile("s_waitcnt lgkmcnt(%2)" : "+v"(t0), "+v"(t1) : "n"(N));
}

// VBLK: K and V are the planes of a bf16 KV cache (K row-major, V token-blocked by 8), possibly paged, with the context
// length per batch row from a device array; see prefill_bf16_kernel for the operand layouts this implies.
template <bool VBLK>
__global__ void __launch_bounds__(256, 2) prefill_bf16_pipe_kernel(PrefillArgs a) {
#if defined(__HIP_DEVICE_COMPILE__)  // the body uses device-only builtins
    constexpr int D = 128;
    constexpr int KS = D / 16;
    constexpr int DB = D / 32;
    constexpr int CPR = D / 8;
    constexpr int RP = 256 / (2 * D);
    constexpr int NR = 1024 / (2 * D);
    constexpr int NGRP = kUnit / NR;
    constexpr int NLD = NGRP / 4;
    constexpr int SLOT = kUnit * D;
    constexpr int SLOTB = 2 * SLOT;
    constexpr int NRING = 4;
    static_assert(KS == 8 && DB == 4 && NLD == 2, "written for D = 128");

    // K ring (4 slots) | V ring (4 slots)
    __shared__ __attribute__((aligned(1024))) uint16_t smem[2 * NRING * SLOT];
    const uint32_t lds0 = lds_addr(smem);

    const int nbh = a.B * a.Hq;
    int bid = blockIdx.x;
    int tile0 = 0;  // first key tile of this workgroup's share of the context (a split context: cache-plane mode only)
    int split = 0;
    if constexpr (VBLK) {
        if (a.n_splits > 1) {
            const int inner = a.n_qtiles * nbh;
            split = bid / inner;
            bid -= split * inner;
            tile0 = split * a.split_tiles;
        }
    }
    const int qt = a.n_qtiles - 1 - bid / nbh;
    const int bh = xcd_grouped_head(bid % nbh, a.B * a.Hkv, a.n_rep);
    const int b = bh / a.Hq, hq = bh % a.Hq, kvh = hq / a.n_rep;
    int L = a.L;
    // cache mode: per-row context length (clamped to the bound a.L) and per-row chunk length n <= T: query t < n sits
    // at absolute position L - n + t; rows t >= n carry no query and their output is unspecified
    int n_chunk = a.T;
    if constexpr (VBLK) {
        if (a.chunk_lens) n_chunk = min(max(a.chunk_lens[b], 0), a.T);
        if (a.seq_lens) L = min(max(a.seq_lens[b], n_chunk), a.L);
    }
    const int tid = threadIdx.x, lane = tid & 63;
    const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
    const int ql = lane & 31, h = lane >> 5;
    const int q0 = qt * kBM + wave * 32;
    const int off = L - n_chunk;
    const int qrow = min(q0 + ql, a.T - 1);

    const uint16_t* Qp = (const uint16_t*)a.q + (int64_t)b * a.sq[0] + (int64_t)hq * a.sq[1];
    const uint16_t* Kp = (const uint16_t*)a.k + (int64_t)b * a.sk[0] + (int64_t)kvh * a.sk[1];
    const uint16_t* Vp = (const uint16_t*)a.v + (int64_t)b * a.sv[0] + (int64_t)kvh * a.sv[1];

    uint4 qraw[KS];
#pragma unroll
    for (int ks = 0; ks < KS; ++ks) qraw[ks] = *(const uint4*)(Qp + (int64_t)qrow * a.sq[2] + 16 * ks + 8 * h);
    bf16x8_t qf[KS];
    // Q goes into the MFMAs as stored (a negative scale flips its sign bits: exact); |scale| * log2(e) multiplies the
    // fp32 scores in front of the exp2, so the scores carry no rounding beyond the fp32 accumulation
    const float cexp = a.scale_log2;
    const float inv_cexp = 1.0f / cexp;
    auto prescale_q = [&]() {
        const uint32_t flip = a.negate_q ? 0x80008000u : 0u;
#pragma unroll
        for (int ks = 0; ks < KS; ++ks) {
            const uint4 w = qraw[ks];
            qf[ks] = __builtin_bit_cast(bf16x8_t, uint4{w.x ^ flip, w.y ^ flip, w.z ^ flip, w.w ^ flip});
        }
    };

    const int wg_qmax = min(qt * kBM + kBM - 1, a.T - 1);
    const int kv_end_wg = a.causal ? min(L, wg_qmax + off + 1) : L;
    int n_tiles = (kv_end_wg + kUnit - 1) / kUnit;  // tiles the workgroup loads
    const int wave_qmax = min(q0 + 31, a.T - 1);
    const int kv_end_wave = (q0 < a.T) ? (a.causal ? min(L, wave_qmax + off + 1) : L) : 0;
    int nt_w = (kv_end_wave + kUnit - 1) / kUnit;  // tiles this wavefront uses
    // first tile of this wavefront that needs the mask (straddles the diagonal or the end of the context)
    int first_masked = min(nt_w, L / kUnit);
    if (a.causal) first_masked = min(first_masked, q0 + off - 31 < 0 ? 0 : (q0 + off - 31) / kUnit + 1);
    if constexpr (VBLK) {
        if (a.n_splits > 1) {  // this workgroup's share: tiles [tile0, tile0 + split_tiles), counted from tile0 below
            n_tiles = max(0, min(n_tiles, tile0 + a.split_tiles) - tile0);
            nt_w = min(max(0, nt_w - tile0), n_tiles);
            first_masked = min(max(0, first_masked - tile0), nt_w);
        }
    }
    const int n_fast = max(0, first_masked - 2);  // steps [0, n_fast): all three stages active, no mask
    const int n_mid = max(0, nt_w - 2);           // steps [0, n_mid): all three stages active

    f32x16_t acc[DB];
#pragma unroll
    for (int i = 0; i < DB; ++i)
#pragma unroll
        for (int j = 0; j < 16; ++j) acc[i][j] = 0.f;
    float m_ref = -INFINITY;
    float l = 0.f;

    // global -> LDS, as in prefill_bf16_kernel
    const int ld_row = lane / CPR, ld_pos = lane % CPR;
    uint32_t voffK[NLD], voffV[NLD];
#pragma unroll
    for (int i = 0; i < NLD; ++i) {
        const int r = NR * (wave + 4 * i) + ld_row;
        voffK[i] = (uint32_t)r * (uint32_t)a.sk[2] * 2u + 16u * (uint32_t)(ld_pos ^ ((r / RP) % CPR));
        if constexpr (VBLK) voffV[i] = (uint32_t)(wave + 4 * i) * 1024u + 16u * (uint32_t)lane;  // the tile is contiguous
        else voffV[i] = (uint32_t)r * (uint32_t)a.sv[2] * 2u + 16u * (uint32_t)(ld_pos ^ (((r / RP) % (CPR / 4)) << 2));
    }
    const int64_t rowK = a.sk[2] * 2, rowV = a.sv[2] * 2;
    // where the 32-token tile starting at key0 lives: the head's slab and the first token inside it (a tile never
    // straddles a page: pages are multiples of 64 tokens)
    auto locate_tile = [&](int key0, const char*& kb, const char*& vb, int& local, int& cap, int& rows) {
        kb = (const char*)Kp;
        vb = (const char*)Vp;
        local = key0;
        cap = a.s_pad;
        rows = L - key0;
        if constexpr (VBLK) {
            if (a.page_table) {
                const int pg = key0 / a.page_tokens;
                local = key0 - pg * a.page_tokens;
                cap = a.page_tokens;
                const int64_t slab = (int64_t)a.page_table[(int64_t)b * a.pages_per_seq + pg] * a.Hkv + kvh;
                kb = (const char*)a.k + slab * cap * D * 2;
                vb = (const char*)a.v + slab * cap * D * 2;
                rows = min(rows, cap - local);
            }
        }
    };
    auto load_k_tile = [&](int t, int slot) {
        const char *kb, *vb;
        int local, cap, rows;
        locate_tile((tile0 + t) * kUnit, kb, vb, local, cap, rows);
        __amdgpu_buffer_rsrc_t rk = __builtin_amdgcn_make_buffer_rsrc((void*)(kb + (int64_t)local * rowK), 0, (int)((int64_t)rows * rowK), 0x00020000);
        uint16_t* dst = smem + slot * SLOT;
#pragma unroll
        for (int i = 0; i < NLD; ++i)
            __builtin_amdgcn_raw_ptr_buffer_load_lds(rk, (__attribute__((address_space(3))) void*)(dst + (wave + 4 * i) * 512), 16, voffK[i], 0, 0, 0);
    };
    auto load_v_tile = [&](int t, int slot) {
        const char *kb, *vb;
        int local, cap, rows;
        locate_tile((tile0 + t) * kUnit, kb, vb, local, cap, rows);
        // VBLK: 32 tokens = 4 token blocks = kUnit * D contiguous elements; bound = the rest of this head's slab
        const int64_t v_base = VBLK ? (int64_t)local * D * 2 : (int64_t)local * rowV;
        const int64_t v_bytes = VBLK ? ((int64_t)cap - local) * D * 2 : (int64_t)rows * rowV;
        __amdgpu_buffer_rsrc_t rv = __builtin_amdgcn_make_buffer_rsrc((void*)(vb + v_base), 0, (int)v_bytes, 0x00020000);
        uint16_t* dst = smem + (NRING + slot) * SLOT;
#pragma unroll
        for (int i = 0; i < NLD; ++i)
            __builtin_amdgcn_raw_ptr_buffer_load_lds(rv, (__attribute__((address_space(3))) void*)(dst + (wave + 4 * i) * 512), 16, voffV[i], 0, 0, 0);
    };

    // loop-constant LDS read addresses (ring slot 0 of each operand; the slot is an immediate offset)
    const int krow = VBLK ? ((ql & ~12) | ((ql & 4) << 1) | ((ql & 8) >> 1)) : ql;  // tile row this lane's S^T row holds
    const int kswz = (krow / RP) % CPR;
    uint32_t kaddr[KS];
#pragma unroll
    for (int ks = 0; ks < KS; ++ks) kaddr[ks] = lds0 + 2u * (uint32_t)(krow * D + 8 * ((2 * ks + h) ^ kswz));
    const int i16 = lane & 15;
    const int vswz = ((i16 >> 2) / RP) % (CPR / 4);
    const int v_lane_off = (4 * h + (i16 >> 2)) * D + 16 * ((lane >> 4) & 1) + 4 * (lane & 3);
    uint32_t va[DB];
#pragma unroll
    for (int db = 0; db < DB; ++db)
        va[db] = VBLK ? lds0 + 16u * (uint32_t)(h * D + ql) : lds0 + 2u * (uint32_t)v_lane_off + 64u * (uint32_t)(db ^ vswz);

    Frag fr[16];         // operand of MFMA slot s of the current step (slots < kLead: already requested)
    // With c = |scale| * log2(e), scores are kept as u = q.k - m / c: -m / c (m = the row's reference maximum in the
    // log2 domain) enters as the C operand of the first QK^T MFMA from a tile of 16 registers that all hold it, and
    // P = exp2(c * u).
    f32x16_t sb[2];      // step tau finishes S'(tau+2) in sb[tau & 1] and consumes S'(tau+1) from sb[(tau+1) & 1]
    uint32_t pb[2][8];   // packed bf16 P: step tau consumes P(tau) from pb[tau & 1] and writes P(tau+1) to pb[(tau+1) & 1]
    f32x16_t negm;       // every element = -m_ref / c of this lane's query
#pragma unroll
    for (int j = 0; j < 16; ++j) negm[j] = 0.f;
    m_ref = 0.f;  // "no reference yet": the first tile sets it

    // Request the operand of MFMA slot S of the step whose ring slot is RS.
    auto request = [&](auto s_c, auto rs_c) {
        constexpr int S = decltype(s_c)::value;
        constexpr int RS = decltype(rs_c)::value;
        if constexpr (kSlotIsQ[S]) {
            constexpr int ks = kSlotIdx[S];
            fr[S].k = lds_read_b128_asm<RS * SLOTB>(kaddr[ks]);
        } else {
            constexpr int p = kSlotIdx[S], j = p / 4, db = p % 4;
            if constexpr (VBLK) {  // token block 2j + h of the tile, rows d = 32 db + ql: one 16-byte read
                fr[S].k = lds_read_b128_asm<(NRING + RS) * SLOTB + (2 * j * D + 32 * db) * 16>(va[db]);
            } else {
                constexpr int VOFF = (NRING + RS) * SLOTB + 16 * j * D * 2;
                fr[S].t0 = lds_read_tr16_b64_asm<VOFF>(va[db]);
                fr[S].t1 = lds_read_tr16_b64_asm<VOFF + 8 * D * 2>(va[db]);
            }
        }
    };

    // One step.  PH = tau & 3 (ring slot of the step's tiles: K(tau+2), V(tau)).  MODE 0: all three stages are active
    // and the new scores need no mask, so the body is one straight line of code; 1: the same with the mask applied
    // under one wavefront-uniform branch; 2: every stage guarded (the first and last steps of a wavefront).
    auto step = [&](int tau, auto ph_c, auto fast_c) {
        constexpr int PH = decltype(ph_c)::value;
        constexpr int MODE = decltype(fast_c)::value;
        constexpr bool FAST = MODE < 2;     // all three stages active: no per-slot guards
        constexpr bool MASK = MODE > 0;     // the new scores may need the mask
        constexpr bool FIRST = MODE == 4;   // step -1: the softmax stage sees tile 0 and sets the reference
        f32x16_t& s_cur = sb[(PH + 1) & 1];
        f32x16_t& s_nxt = sb[PH & 1];
        uint32_t(&p_cur)[8] = pb[PH & 1];
        uint32_t(&p_nxt)[8] = pb[(PH + 1) & 1];

        if constexpr (MODE == 3) asm volatile("s_waitcnt vmcnt(8)" ::: "memory");  // first step: K(1) has landed
        else asm volatile("s_waitcnt vmcnt(4)" ::: "memory");  // the tiles of step tau+1 have landed; those of tau+2 may be in flight
        __builtin_amdgcn_s_barrier();  // waits are explicit: no fence, which would drain every load in flight
        // always four loads per wavefront and step, so that the vmcnt arithmetic holds: past the end the tile index is
        // clamped (the rows fall outside the buffer bound and arrive as zeros, or re-read the last tile; never consumed)
        if constexpr (MODE != 3) {
            load_k_tile(min(tau + 5, n_tiles - 1), (PH + 3) & 3);
            load_v_tile(min(tau + 3, n_tiles - 1), (PH + 3) & 3);
        }

        const bool qk_on = FAST || (tau + 2 < nt_w);
        const bool sm_on = FAST || (tau + 1 >= 0 && tau + 1 < nt_w);
        const bool pv_on = FAST || (tau >= 0 && tau < nt_w);

        float es[16];
        float lsum = 0.f, lsum2 = 0.f;
        // instruction i of the 32 that turn s_cur into p_nxt: per pair of scores 2 exp2, 1 pack, and the row sum.
        // Steady-state steps sum the fp32 values with plain adds (a dot2 occupies the matrix pipe); against the sum of
        // the bf16-rounded P that the PV MFMAs consume this is zero-mean rounding noise of relative size
        // 2^-9 / sqrt(keys), and such steps only exist in contexts of more than a hundred keys.  The first and last
        // steps of a wavefront sum the rounded values themselves (packed dot product against (1, 1)), so that short
        // contexts are normalised by exactly what was accumulated (a single key reproduces V bit for bit).
        auto softmax_op = [&](auto i_c) {
            constexpr int i = decltype(i_c)::value, p = i / 4, k = i % 4;
            if constexpr (k == 0) {  // both multiplies first: neither exp2 waits on the instruction right before it
                es[2 * p] = s_cur[2 * p] * cexp;
                es[2 * p + 1] = s_cur[2 * p + 1] * cexp;
                es[2 * p] = __builtin_amdgcn_exp2f(es[2 * p]);
            } else if constexpr (k == 1) es[2 * p + 1] = __builtin_amdgcn_exp2f(es[2 * p + 1]);
            else if constexpr (k == 2) p_nxt[p] = cvt_pk_bf16(es[2 * p], es[2 * p + 1]);
            else if constexpr (FAST && !MASK) { lsum += es[2 * p]; lsum2 += es[2 * p + 1]; }
            else lsum = __builtin_amdgcn_fdot2_f32_bf16(__builtin_bit_cast(bf16x2_t, p_nxt[p]), __builtin_bit_cast(bf16x2_t, 0x3f803f80u), lsum, false);
        };

        static_for<16>([&](auto s_c) {
            constexpr int S = decltype(s_c)::value;
            // ---- the MFMA of this slot
            if constexpr (kSlotIsQ[S]) {
                constexpr int ks = kSlotIdx[S];
                frag_wait_k<reads_behind<VBLK>(S)>(fr[S].k);
                if (qk_on) {
                    if constexpr (ks == 0) s_nxt = __builtin_amdgcn_mfma_f32_32x32x16_bf16(__builtin_bit_cast(bf16x8_t, fr[S].k), qf[ks], negm, 0, 0, 0);
                    else s_nxt = __builtin_amdgcn_mfma_f32_32x32x16_bf16(__builtin_bit_cast(bf16x8_t, fr[S].k), qf[ks], s_nxt, 0, 0, 0);
                }
            } else {
                constexpr int p = kSlotIdx[S], j = p / 4, db = p % 4;
                if constexpr (VBLK) frag_wait_k<reads_behind<VBLK>(S)>(fr[S].k);
                else frag_wait_v<reads_behind<VBLK>(S)>(fr[S].t0, fr[S].t1);
                if (pv_on) {
                    if constexpr (VBLK && MODE >= 2) {
                        // the planes hold stale tokens past L: P is 0 there, V must not be NaN
                        const int nvalid = L - ((tile0 + tau) * kUnit + 16 * j + 8 * h);  // slots e >= nvalid are past the context
                        if (nvalid < 8) {
#pragma unroll
                            for (int w = 0; w < 4; ++w) {
                                uint32_t x = fr[S].k[w];
                                if (2 * w + 1 >= nvalid) x &= 0x0000ffffu;
                                if (2 * w >= nvalid) x = 0;
                                fr[S].k[w] = x;
                            }
                        }
                    }
                    const bf16x8_t vf = VBLK ? __builtin_bit_cast(bf16x8_t, fr[S].k)
                                             : __builtin_bit_cast(bf16x8_t, uint4{fr[S].t0.x, fr[S].t0.y, fr[S].t1.x, fr[S].t1.y});
                    const bf16x8_t pf = __builtin_bit_cast(bf16x8_t, uint4{p_cur[4 * j], p_cur[4 * j + 1], p_cur[4 * j + 2], p_cur[4 * j + 3]});
                    acc[db] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(vf, pf, acc[db], 0, 0, 0);
                }
            }
            // ---- the operand of the slot kLead ahead (next step's tiles once the index wraps)
            if constexpr (S + kLead < 16) request(std::integral_constant<int, S + kLead>{}, std::integral_constant<int, PH>{});
            else request(std::integral_constant<int, S + kLead - 16>{}, std::integral_constant<int, (PH + 1) & 3>{});
            // ---- this slot's share of the vector-ALU work
            if constexpr (!FIRST) {
                if (sm_on) static_for<2>([&](auto k_c) { softmax_op(std::integral_constant<int, 2 * S + decltype(k_c)::value>{}); });
            }
            if constexpr (MASK && S == 12) {
                if (qk_on) {
                    const int k0 = (tile0 + tau + 2) * kUnit;
                    if ((a.causal && k0 + kUnit - 1 > q0 + off) || (k0 + kUnit > L)) {
                        const int q_abs = q0 + ql + off;
                        const int lim = a.causal ? min(q_abs, L - 1) : L - 1;
#pragma unroll
                        for (int v = 0; v < 16; ++v)
                            if ((VBLK ? k0 + 16 * (v >> 3) + 8 * h + (v & 7) : k0 + 8 * (v >> 2) + 4 * h + (v & 3)) > lim) s_nxt[v] = -INFINITY;
                    }
                }
            }
            __builtin_amdgcn_sched_barrier(0);
        });
        if (sm_on) {
            // A reference that has fallen behind shows in the row sum: below 2^10 no P of the tile exceeds 2^10, far
            // from overflow; otherwise (rare; and always for the first tile, which has no reference yet) take the true
            // maximum of these scores, raise the reference to an integer at or above it (alpha is then a power of
            // two, so everything computed against the old reference rescales exactly) and redo this tile's P.
            constexpr bool first = FIRST;
            if (first || __any(!(lsum + lsum2 < 1024.f))) {
                float mx = s_cur[0];
#pragma unroll
                for (int v = 1; v < 16; ++v) mx = fmaxf(mx, s_cur[v]);
                mx = half_swap_max(mx);
                // raise (first tile: set) the reference by delta, an integer in the log2 domain; the scores move by du
                float delta = (mx == -INFINITY) ? 0.f : ceilf(mx * cexp);
                if (!first) delta = fmaxf(delta, 0.f);
                const float du = delta == 0.f ? 0.f : delta * inv_cexp;  // (a scale in the denormal range has 1 / c = inf)
                if constexpr (!first) {  // nothing has been accumulated before the first tile
                    const float alpha = __builtin_amdgcn_exp2f(-delta);
                    l *= alpha;
#pragma unroll
                    for (int i = 0; i < DB; ++i)
#pragma unroll
                        for (int j = 0; j < 16; ++j) acc[i][j] *= alpha;
                }
                lsum = lsum2 = 0.f;
#pragma unroll
                for (int v = 0; v < 16; ++v) s_cur[v] -= du;
                static_for<32>([&](auto i_c) { softmax_op(i_c); });
                if (qk_on) {
#pragma unroll
                    for (int v = 0; v < 16; ++v) s_nxt[v] -= du;  // finished this step against the old reference
                }
                m_ref += delta;
#pragma unroll
                for (int j = 0; j < 16; ++j) negm[j] = m_ref == 0.f ? 0.f : -m_ref * inv_cexp;
            }
            l += lsum + lsum2;
        }
    };

    using I0 = std::integral_constant<int, 0>;
    using I1 = std::integral_constant<int, 1>;
    using I2 = std::integral_constant<int, 2>;
    using I3 = std::integral_constant<int, 3>;
    using Fast = std::integral_constant<int, 0>;
    using Mid = std::integral_constant<int, 1>;
    using Slow = std::integral_constant<int, 2>;
    using First = std::integral_constant<int, 3>;   // step -2: Slow, and the tiles three steps ahead were requested by the prologue
    using Second = std::integral_constant<int, 4>;  // step -1: Slow, and its softmax stage sets the reference from tile 0

    if (n_tiles > 0) {  // an empty context (cache mode, length 0) has nothing to attend to: zeros below
    // prologue: the tiles of steps -2 and -1 (K(0), K(1)) are requested here, published by the barrier below
    load_k_tile(0, 2);
    load_k_tile(min(1, n_tiles - 1), 3);
    // tiles of steps 0 and 1 (K(2), V(0), K(3), V(1)); from step -1 on every step requests the tiles three steps ahead
    load_k_tile(min(2, n_tiles - 1), 0);
    load_v_tile(0, 0);
    load_k_tile(min(3, n_tiles - 1), 1);
    load_v_tile(min(1, n_tiles - 1), 1);
    prescale_q();
    asm volatile("s_waitcnt vmcnt(10)" ::: "memory");  // K(0) has landed
    __builtin_amdgcn_s_barrier();  // waits are explicit: no fence, which would drain every load in flight
    static_for<kLead>([&](auto s_c) { request(s_c, I2{}); });

    step(-2, I2{}, First{});
    step(-1, I3{}, Second{});
    int tau = 0;
    for (; tau + 4 <= n_fast; tau += 4) {
        step(tau, I0{}, Fast{});
        step(tau + 1, I1{}, Fast{});
        step(tau + 2, I2{}, Fast{});
        step(tau + 3, I3{}, Fast{});
    }
    for (; tau + 4 <= n_mid; tau += 4) {
        step(tau, I0{}, Mid{});
        step(tau + 1, I1{}, Mid{});
        step(tau + 2, I2{}, Mid{});
        step(tau + 3, I3{}, Mid{});
    }
    for (; tau < n_tiles; tau += 4) {
        step(tau, I0{}, Slow{});
        if (tau + 1 < n_tiles) step(tau + 1, I1{}, Slow{});
        if (tau + 2 < n_tiles) step(tau + 2, I2{}, Slow{});
        if (tau + 3 < n_tiles) step(tau + 3, I3{}, Slow{});
    }
    // operands requested for a step that does not exist are still in flight: let them land before the registers die
    asm volatile("s_waitcnt lgkmcnt(0)" ::: "memory");
    } else {
        prescale_q();
    }

    l = half_swap_sum(l);
    const int qi = q0 + ql;
    if constexpr (VBLK) {
        if (a.n_splits > 1) {  // the unnormalised partial of this share of the context; the combine kernel finishes the row
            if (qi < a.T) {
                const int64_t row = (((int64_t)b * a.Hq + hq) * a.T + qi) * a.n_splits + split;
                float* po = a.ws_o + row * D;
#pragma unroll
                for (int db = 0; db < DB; ++db)
#pragma unroll
                    for (int vq = 0; vq < 4; ++vq)
                        *(float4*)(po + 32 * db + 8 * vq + 4 * h) = float4{acc[db][4 * vq], acc[db][4 * vq + 1], acc[db][4 * vq + 2], acc[db][4 * vq + 3]};
                if (h == 0) {  // a row that met no key in this share (masked, or the share lies past its diagonal) says so
                    a.ws_ml[row * 2] = l > 0.f ? m_ref : -INFINITY;
                    a.ws_ml[row * 2 + 1] = l;
                }
            }
            asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
            return;
        }
    }
    if (qi < a.T) {
        const float inv_l = l > 0.f ? 1.0f / l : 0.f;
        uint16_t* op = (uint16_t*)a.out + (int64_t)b * a.so[0] + (int64_t)hq * a.so[1] + (int64_t)qi * a.so[2];
#pragma unroll
        for (int db = 0; db < DB; ++db)
#pragma unroll
            for (int vq = 0; vq < 4; ++vq) {
                const int d = 32 * db + 8 * vq + 4 * h;
                uint2 w;
                w.x = cvt_pk_bf16(acc[db][4 * vq] * inv_l, acc[db][4 * vq + 1] * inv_l);
                w.y = cvt_pk_bf16(acc[db][4 * vq + 2] * inv_l, acc[db][4 * vq + 3] * inv_l);
                *(uint2*)(op + d) = w;
            }
        if (a.lse && h == 0)
            a.lse[(int64_t)b * a.sl[0] + (int64_t)hq * a.sl[1] + (int64_t)qi * a.sl[2]] = (m_ref + __builtin_amdgcn_logf(l)) * 0.6931471805599453f;
    }
    // the clamped tile requests of the last steps write LDS: they have landed before the workgroup gives its LDS back
    asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
#endif
}

// ---------------------------------------------------------------------------------------------
// fp32 kernel (fp32 inputs, fp32 MFMA 32x32x2, fp32 softmax): the precision the reference computes
// in.  One wavefront owns 32 queries, a workgroup 128; key tiles of 32 through LDS.
// GEN: the tensors' head_dim a.D_true is any value up to the tile width D (the reference's forward takes any
// head_dim, src/ops/flash_attention.cpp:235-238): columns past it are zero in the operands (they add nothing to a
// score) and are not stored; rows are read element by element, so they need no 16-byte alignment.
// ---------------------------------------------------------------------------------------------
template <int D, bool GEN>
__global__ void __launch_bounds__(256) prefill_f32_kernel(PrefillArgs a) {
    constexpr int BN = 32;
    constexpr int PITCH = D + 1;  // odd pitch: a column walk hits 32 different banks
    constexpr int DB = D / 32;
    extern __shared__ float smem_f32[];  // K tile | V tile (2 * BN * PITCH floats, sized by the launch)
    float* sK = smem_f32;
    float* sV = smem_f32 + BN * PITCH;
    const int Dt = GEN ? a.D_true : D;

    const int bid = blockIdx.x;
    const int qt = a.n_qtiles - 1 - bid / (a.B * a.Hq);
    const int bh = xcd_grouped_head(bid % (a.B * a.Hq), a.B * a.Hkv, a.n_rep);
    const int b = bh / a.Hq, hq = bh % a.Hq, kvh = hq / a.n_rep;
    const int n_chunk = a.chunk_lens ? min(max(a.chunk_lens[b], 0), a.T) : a.T;  // cache mode, as in the bf16 kernel
    const int L = a.seq_lens ? min(max(a.seq_lens[b], n_chunk), a.L) : a.L;
    const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
    const int ql = lane & 31, h = lane >> 5;
    const int q0 = qt * kBM + wave * 32;
    const int off = L - n_chunk;
    const int qrow = min(q0 + ql, a.T - 1);

    const float* Qp = (const float*)a.q + (int64_t)b * a.sq[0] + (int64_t)hq * a.sq[1] + (int64_t)qrow * a.sq[2];
    const float* Kp = (const float*)a.k + (int64_t)b * a.sk[0] + (int64_t)kvh * a.sk[1];
    const float* Vp = (const float*)a.v + (int64_t)b * a.sv[0] + (int64_t)kvh * a.sv[1];

    // Q^T operands: column ql, contraction slot d = 2*ks + h
    float qf[D / 2];
#pragma unroll
    for (int ks = 0; ks < D / 2; ++ks) qf[ks] = (!GEN || 2 * ks + h < Dt) ? Qp[2 * ks + h] : 0.f;

    const int wg_qmax = min(qt * kBM + kBM - 1, a.T - 1);
    const int kv_end_wg = a.causal ? min(L, wg_qmax + off + 1) : L;
    const int n_tiles = (kv_end_wg + BN - 1) / BN;
    const int wave_qmax = min(q0 + 31, a.T - 1);
    const int kv_end_wave = a.causal ? min(L, wave_qmax + off + 1) : L;

    f32x16_t acc[DB];
#pragma unroll
    for (int i = 0; i < DB; ++i)
#pragma unroll
        for (int j = 0; j < 16; ++j) acc[i][j] = 0.f;
    float m_run = -INFINITY, l = 0.f;

    for (int kt = 0; kt < n_tiles; ++kt) {
        __syncthreads();
        if constexpr (GEN) {
            for (int id = tid; id < BN * D; id += 256) {
                const int row = id / D, col = id % D, key = kt * BN + row;
                const bool ok = key < L && col < Dt;
                sK[row * PITCH + col] = ok ? Kp[(int64_t)key * a.sk[2] + col] : 0.f;
                sV[row * PITCH + col] = ok ? Vp[(int64_t)key * a.sv[2] + col] : 0.f;
            }
        } else
        for (int id = tid; id < BN * (D / 4); id += 256) {  // 16-byte loads (rows are 16-byte aligned), padded LDS rows
            const int row = id / (D / 4), col = 4 * (id % (D / 4)), key = kt * BN + row;
            float4 kk = {0.f, 0.f, 0.f, 0.f}, vv = kk;
            if (key < L) {
                kk = *(const float4*)(Kp + (int64_t)key * a.sk[2] + col);
                vv = *(const float4*)(Vp + (int64_t)key * a.sv[2] + col);
            }
            float* dk = sK + row * PITCH + col;
            float* dv = sV + row * PITCH + col;
            dk[0] = kk.x, dk[1] = kk.y, dk[2] = kk.z, dk[3] = kk.w;
            dv[0] = vv.x, dv[1] = vv.y, dv[2] = vv.z, dv[3] = vv.w;
        }
        __syncthreads();
        const int k0 = kt * BN;
        if (k0 >= kv_end_wave) continue;

        f32x16_t s;
#pragma unroll
        for (int j = 0; j < 16; ++j) s[j] = 0.f;
#pragma unroll
        for (int ks = 0; ks < D / 2; ++ks)
            s = __builtin_amdgcn_mfma_f32_32x32x2f32(sK[ql * PITCH + 2 * ks + h], qf[ks], s, 0, 0, 0);
        const int lim = a.causal ? min(q0 + ql + off, L - 1) : L - 1;
        float mx = -INFINITY;
#pragma unroll
        for (int v = 0; v < 16; ++v) {
            const int key = k0 + 8 * (v >> 2) + 4 * h + (v & 3);
            float t = s[v] * a.scale_log2;
            if (key > lim) t = -INFINITY;
            s[v] = t;
            mx = fmaxf(mx, t);
        }
        mx = half_swap_max(mx);
        const float m_new = fmaxf(m_run, mx);
        const float alpha = (m_new == -INFINITY) ? 1.f : exp2f(m_run - m_new);
        const float sub = (m_new == -INFINITY) ? 0.f : m_new;
        l *= alpha;
#pragma unroll
        for (int i = 0; i < DB; ++i)
#pragma unroll
            for (int j = 0; j < 16; ++j) acc[i][j] *= alpha;
        m_run = m_new;
        float p[16];
#pragma unroll
        for (int v = 0; v < 16; ++v) {
            p[v] = exp2f(s[v] - sub);
            l += p[v];
        }
        // O^T += V^T . P^T : contraction slot h of step v is key 8*(v/4) + 4*h + v%4, the key p[v] belongs to
#pragma unroll
        for (int v = 0; v < 16; ++v) {
            const int krow = 8 * (v >> 2) + 4 * h + (v & 3);
#pragma unroll
            for (int db = 0; db < DB; ++db)
                acc[db] = __builtin_amdgcn_mfma_f32_32x32x2f32(sV[krow * PITCH + 32 * db + ql], p[v], acc[db], 0, 0, 0);
        }
    }
    l = half_swap_sum(l);
    const int qi = q0 + ql;
    if (qi < a.T) {
        const float inv_l = l > 0.f ? 1.0f / l : 0.f;  // an empty context (cache mode, length 0) gives zeros
        float* op = (float*)a.out + (int64_t)b * a.so[0] + (int64_t)hq * a.so[1] + (int64_t)qi * a.so[2];
#pragma unroll
        for (int db = 0; db < DB; ++db)
#pragma unroll
            for (int v = 0; v < 16; ++v) {
                const int d = 32 * db + 8 * (v >> 2) + 4 * h + (v & 3);
                if (!GEN || d < Dt) op[d] = acc[db][v] * inv_l;
            }
        if (a.lse && h == 0)
            a.lse[(int64_t)b * a.sl[0] + (int64_t)hq * a.sl[1] + (int64_t)qi * a.sl[2]] = (m_run + log2f(l)) * 0.6931471805599453f;
    }
}

int check_tensor4(const vsp_tensor* t, int esz) {
    if (t->stride[3] != 1) return VSP_ERR_STRIDE;
    if (!t->data) return VSP_ERR_NULL;
    if (!is_aligned16(t->data)) return VSP_ERR_ALIGN;
    for (int i = 0; i < 3; ++i)
        if ((t->stride[i] * esz) % 16 != 0) return VSP_ERR_ALIGN;
    return VSP_OK;
}

// fp32 tensors whose head_dim is not one of the native tiles: element-wise access, so 4-byte alignment is all it takes
int check_tensor4_any_d(const vsp_tensor* t) {
    if (t->stride[3] != 1) return VSP_ERR_STRIDE;
    if (!t->data) return VSP_ERR_NULL;
    if ((reinterpret_cast<uintptr_t>(t->data) & 3u) != 0) return VSP_ERR_ALIGN;
    return VSP_OK;
}
bool native_head_dim(int dtype, int64_t D) { return D == 64 || D == 128 || (D == 32 && dtype == VSP_F32); }
// the fp32 kernels' tile width for a head_dim they do not hold natively (0: none)
int64_t padded_head_dim(int dtype, int64_t D) {
    if (dtype != VSP_F32 || D < 1 || D > 256) return 0;
    return D <= 32 ? 32 : D <= 64 ? 64 : D <= 128 ? 128 : 256;
}

template <int DP, bool GEN>
int launch_prefill_f32(const PrefillArgs& a, dim3 grid, hipStream_t st) {
    constexpr size_t lds = 2 * 32 * (DP + 1) * sizeof(float);
    if constexpr (lds > 65536) {  // beyond the default limit of a launch: raised once per process
        static const hipError_t e = hipFuncSetAttribute((const void*)prefill_f32_kernel<DP, GEN>, hipFuncAttributeMaxDynamicSharedMemorySize, (int)lds);
        if (e != hipSuccess) {
            set_hip_error(e);
            return VSP_ERR_LAUNCH;
        }
    }
    hipLaunchKernelGGL((prefill_f32_kernel<DP, GEN>), grid, dim3(256), lds, st, a);
    return check_launch();
}

int launch_prefill(const PrefillArgs& a, int dtype, int64_t D, bool cache_planes, void* stream) {
    const int64_t blocks = (int64_t)a.n_qtiles * a.B * a.Hq;
    if (blocks > INT32_MAX) return VSP_ERR_ARG;
    hipStream_t st = (hipStream_t)stream;
    dim3 grid((unsigned)blocks), block(256);
    if (dtype == VSP_BF16) {
        // head_dim 128 has two kernels.  The software-pipelined one (two workgroups per CU) has the faster steady state;
        // the general one (three per CU, no pipeline to fill and drain) has the cheaper workgroup and wins while contexts
        // are short, provided the grid fills its 3 x CUs slots: measured crossover between 2560 and 3072 tokens
        // (+3 % at 2048, +10 % at 1024, +14 % at 512; -2 % at 3072, -3 % at 8192).
        const bool short_ctx = a.L <= 2560 && blocks >= 3 * (int64_t)device_cu_count();
        if (cache_planes) {
            if (D == 128 && !short_ctx) hipLaunchKernelGGL(prefill_bf16_pipe_kernel<true>, grid, block, 0, st, a);
            else if (D == 128) hipLaunchKernelGGL((prefill_bf16_kernel<128, true>), grid, block, 0, st, a);
            else hipLaunchKernelGGL((prefill_bf16_kernel<64, true>), grid, block, 0, st, a);
        } else {
            // the software-pipelined kernel takes one context length for the batch; dense K/V with per-row lengths
            // (a Q8_0 cache read out into the workspace) stay with the general kernel
            if (D == 128 && !a.seq_lens && !a.chunk_lens && !short_ctx) hipLaunchKernelGGL(prefill_bf16_pipe_kernel<false>, grid, block, 0, st, a);
            else if (D == 128) hipLaunchKernelGGL((prefill_bf16_kernel<128, false>), grid, block, 0, st, a);
            else hipLaunchKernelGGL((prefill_bf16_kernel<64, false>), grid, block, 0, st, a);
        }
    } else {
        if (!a.elementwise) {
            if (D == 128) return launch_prefill_f32<128, false>(a, grid, st);
            if (D == 64) return launch_prefill_f32<64, false>(a, grid, st);
            if (D == 32) return launch_prefill_f32<32, false>(a, grid, st);
        }
        switch (padded_head_dim(dtype, D)) {  // a.D_true == D
            case 32: return launch_prefill_f32<32, true>(a, grid, st);
            case 64: return launch_prefill_f32<64, true>(a, grid, st);
            case 128: return launch_prefill_f32<128, true>(a, grid, st);
            case 256: return launch_prefill_f32<256, true>(a, grid, st);
            default: return VSP_ERR_UNSUPPORTED;
        }
    }
    return check_launch();
}

}  // namespace

int check_kv_cache(const vsp_kv_cache* c);  // kv_cache.hip

}  // namespace vsp

using namespace vsp;

namespace {
// Context split for a chunk over a long cached context (bf16 planes, head_dim 128): the grid of a few query tiles
// leaves most of the chip idle while each workgroup walks the whole context, so the context is cut into shares of
// split_tiles key tiles, one workgroup per (query tile, head, share), and the decode step's combine kernel merges the
// partials.  Shares are at least 16 tiles (512 keys) long and as many as it takes to reach two workgroups per CU.
struct SplitChoice {
    int n_splits, split_tiles;
};
SplitChoice plan_context_split(const vsp_kv_cache* cache, int64_t Hq, int64_t T, int64_t L) {
    SplitChoice c{1, 0};
    if (cache->format != VSP_KV_BF16 || cache->D != 128) return c;
    const int64_t inner = ceil_div(T, kBM) * cache->B * Hq;
    const int64_t slots = 2 * (int64_t)device_cu_count();
    const int64_t tiles = ceil_div(L, kUnit);
    if (inner <= 0 || inner * 2 > slots || tiles < 32) return c;
    int64_t n = std::min<int64_t>(ceil_div(slots, inner), tiles / 16);
    n = std::min<int64_t>(n, 64);
    if (n <= 1) return c;
    c.split_tiles = (int)ceil_div(tiles, n);
    c.n_splits = (int)ceil_div(tiles, c.split_tiles);
    return c;
}

// The host-side bound of the context lengths a cached-prefill call is planned on: max_len when given, else the
// cache's own length, or its capacity when the lengths live on the device.
int64_t cached_len_bound(const vsp_kv_cache* cache, bool with_seq_lens, int32_t max_len) {
    if (max_len > 0) return std::min<int64_t>(max_len, cache->S_max);
    return with_seq_lens ? cache->S_max : cache->len;
}
}  // namespace

extern "C" size_t vsp_attn_prefill_cached_split_workspace_bytes(const vsp_kv_cache* cache, int with_seq_lens, int32_t max_len,
                                                                int32_t Hq, int32_t T) {
    if (!cache || Hq <= 0 || T <= 0 || max_len < 0) return 0;
    const int64_t L = cached_len_bound(cache, with_seq_lens != 0, max_len);
    const SplitChoice c = plan_context_split(cache, Hq, T, L);
    if (c.n_splits <= 1) return 0;
    return (size_t)cache->B * (size_t)Hq * (size_t)T * (size_t)c.n_splits * (size_t)(cache->D + 2) * sizeof(float);
}

extern "C" size_t vsp_attn_prefill_cached_workspace_bytes(const vsp_kv_cache* cache, int with_seq_lens, int32_t max_len) {
    if (!cache || cache->format != VSP_KV_Q8_0 || max_len < 0) return 0;
    const int64_t rows = cached_len_bound(cache, with_seq_lens != 0, max_len);
    return (size_t)2 * (size_t)cache->B * (size_t)cache->Hkv * (size_t)rows * (size_t)cache->D * 2;  // K and V, bf16
}

extern "C" int vsp_kv_read(const vsp_kv_cache* cache, int64_t start, int64_t count, vsp_tensor* k_out, vsp_tensor* v_out,
                           void* stream);

extern "C" int vsp_attn_prefill_cached(const vsp_tensor* q, const vsp_kv_cache* cache, const int32_t* seq_lens, int32_t max_len,
                                       const int32_t* chunk_lens, vsp_tensor* out, vsp_tensor* lse, float scale,
                                       int is_causal, void* workspace, size_t workspace_bytes, void* stream) {
    if (!q || !out) return VSP_ERR_NULL;
    int rc = check_kv_cache(cache);
    if (rc != VSP_OK) return rc;
    if (q->ndim != 4 || out->ndim != 4) return VSP_ERR_NDIM;
    const int64_t B = q->shape[0], Hq = q->shape[1], T = q->shape[2], D = q->shape[3];
    const int64_t Hkv = cache->Hkv;
    if (B != cache->B || D != cache->D) return VSP_ERR_SHAPE;
    if (Hkv <= 0 ? Hq != 0 : (Hq % Hkv != 0)) return VSP_ERR_SHAPE;
    // the bound every plan below is made on; device-side lengths are clamped to it inside the kernels, a host-side
    // length above it is a caller error (as in vsp_attn_decode)
    if (max_len < 0 || max_len > cache->S_max) return VSP_ERR_ARG;
    if (!seq_lens && max_len > 0 && cache->len > max_len) return VSP_ERR_ARG;
    const int64_t L = cached_len_bound(cache, seq_lens != nullptr, max_len);
    if (T > L) return VSP_ERR_SHAPE;                          // the chunk is part of the context
    for (int i = 0; i < 4; ++i)
        if (out->shape[i] != q->shape[i]) return VSP_ERR_SHAPE;
    if (out->dtype != q->dtype) return VSP_ERR_DTYPE;
    if (q->dtype != (cache->format == VSP_KV_F32 ? VSP_F32 : VSP_BF16)) return VSP_ERR_DTYPE;
    if (lse) {
        if (lse->ndim != 3 || lse->shape[0] != B || lse->shape[1] != Hq || lse->shape[2] != T) return VSP_ERR_SHAPE;
        if (lse->dtype != VSP_F32) return VSP_ERR_DTYPE;
    }
    if (B * Hq * T * D == 0) return VSP_OK;
    // bf16: head_dim 64 or 128; fp32: any head_dim up to 256 (the native tiles 32 / 64 / 128, or the next one padded)
    const bool native = native_head_dim(q->dtype, D);
    if (!native && !padded_head_dim(q->dtype, D)) return VSP_ERR_UNSUPPORTED;
    if (!(fabsf(scale) > 0.0f) || !(fabsf(scale) < INFINITY)) return VSP_ERR_ARG;
    const int esz = q->dtype == VSP_F32 ? 4 : 2;
    bool elementwise = !native;
    if (native && ((rc = check_tensor4(q, esz)) != VSP_OK || (rc = check_tensor4(out, esz)) != VSP_OK)) {
        if (q->dtype != VSP_F32 || rc != VSP_ERR_ALIGN) return rc;
        elementwise = true;  // fp32 rows that are not 16-byte aligned: the element-wise kernel takes them
    }
    if (elementwise && ((rc = check_tensor4_any_d(q)) != VSP_OK || (rc = check_tensor4_any_d(out)) != VSP_OK)) return rc;
    if (lse && !lse->data) return VSP_ERR_NULL;
    if (T > INT32_MAX / 2) return VSP_ERR_ARG;

    PrefillArgs a{};
    a.D_true = (int)D;
    a.elementwise = elementwise ? 1 : 0;
    a.q = q->data;
    a.k = cache->k;
    a.v = cache->v;
    a.out = out->data;
    a.lse = lse ? (float*)lse->data : nullptr;
    int64_t s_phys = kv_s_pad(cache->format, cache->S_max);
    for (int i = 0; i < 3; ++i) {
        a.sq[i] = q->stride[i];
        a.so[i] = out->stride[i];
        a.sl[i] = lse ? lse->stride[i] : 0;
    }
    if (cache->format == VSP_KV_Q8_0) {
        // Compute-bound path: dequantising inside the MFMA loop would add vector-ALU work to a kernel that is
        // already short of it, while reading the context out once costs ~0.2 % of the attention time.  The rows
        // [0, L) are dequantised to dense bf16 in the workspace and the dense kernel runs over that.
        const size_t need = vsp_attn_prefill_cached_workspace_bytes(cache, seq_lens != nullptr, max_len);
        if (!workspace || workspace_bytes < need) return VSP_ERR_WORKSPACE;
        if (!is_aligned16(workspace)) return VSP_ERR_ALIGN;
        vsp_tensor kt{}, vt{};
        kt.dtype = vt.dtype = VSP_BF16;
        kt.ndim = vt.ndim = 4;
        const int64_t shp[4] = {B, Hkv, L, D};
        for (int i = 0; i < 4; ++i) kt.shape[i] = vt.shape[i] = shp[i];
        kt.stride[3] = vt.stride[3] = 1;
        kt.stride[2] = vt.stride[2] = D;
        kt.stride[1] = vt.stride[1] = L * D;
        kt.stride[0] = vt.stride[0] = Hkv * L * D;
        kt.data = workspace;
        vt.data = (char*)workspace + need / 2;
        if ((rc = vsp_kv_read(cache, 0, L, &kt, &vt, stream)) != VSP_OK) return rc;
        a.k = kt.data;
        a.v = vt.data;
        s_phys = L;
    }
    a.sk[0] = a.sv[0] = Hkv * s_phys * D;
    a.sk[1] = a.sv[1] = s_phys * D;
    a.sk[2] = a.sv[2] = D;
    a.B = (int)B;
    a.Hq = (int)Hq;
    a.Hkv = (int)Hkv;
    a.n_rep = (int)(Hq / Hkv);
    a.T = (int)T;
    a.L = (int)L;
    a.s_pad = (int)s_phys;
    a.seq_lens = seq_lens;
    a.chunk_lens = chunk_lens;
    if (cache->page_table && cache->format == VSP_KV_BF16) {
        a.page_table = cache->page_table;
        a.page_tokens = cache->page_tokens;
        a.pages_per_seq = cache->pages_per_seq;
        a.s_pad = cache->page_tokens;
    }
    a.causal = is_causal ? 1 : 0;
    a.n_qtiles = (int)ceil_div(T, kBM);
    a.negate_q = (q->dtype == VSP_BF16 && scale < 0.0f) ? 1 : 0;
    a.scale_log2 = (q->dtype == VSP_BF16 ? fabsf(scale) : scale) * kLog2e;
    // a caller that brings the workspace of vsp_attn_prefill_cached_split_workspace_bytes gets the context split over
    // workgroups when the grid would otherwise leave the chip idle; the combine kernel finishes the rows (and their lse)
    if (workspace && is_aligned16(workspace)) {
        const SplitChoice c = plan_context_split(cache, Hq, T, L);
        const size_t rows = (size_t)B * (size_t)Hq * (size_t)T * (size_t)c.n_splits;
        if (c.n_splits > 1 && workspace_bytes >= rows * (size_t)(D + 2) * sizeof(float)) {
            a.n_splits = c.n_splits;
            a.split_tiles = c.split_tiles;
            a.ws_o = (float*)workspace;
            a.ws_ml = a.ws_o + rows * (size_t)D;
            const int64_t blocks = (int64_t)a.n_qtiles * B * Hq * c.n_splits;
            if (blocks > INT32_MAX) return VSP_ERR_ARG;
            hipLaunchKernelGGL(prefill_bf16_pipe_kernel<true>, dim3((unsigned)blocks), dim3(256), 0, (hipStream_t)stream, a);
            if ((rc = check_launch()) != VSP_OK) return rc;
            CombineExtra x;
            x.chunk_lens = chunk_lens;
            x.len_floor = (int)T;
            x.lse = a.lse;
            for (int i = 0; i < 3; ++i) x.sl[i] = a.sl[i];
            return launch_split_combine(a.ws_o, a.ws_ml, seq_lens, cache->len, c.split_tiles * kUnit, c.n_splits, B, Hq, T, D, (int)L, out,
                                        (hipStream_t)stream, x);
        }
    }
    return launch_prefill(a, q->dtype, D, cache->format == VSP_KV_BF16, stream);
}

namespace {
// Bytes of the hi / lo bf16 planes of Q, K and V (dense [B,H,N,D] each, 256-byte aligned starts).
size_t split_plane_bytes(int64_t elems) { return (size_t)((elems * 2 + 255) / 256 * 256); }

int prefill_entry(const vsp_tensor* q, const vsp_tensor* k, const vsp_tensor* v, vsp_tensor* out, vsp_tensor* lse, float scale,
                  int is_causal, float dropout_p, int training, bool split, void* workspace, size_t workspace_bytes, void* stream);
}  // namespace

extern "C" int vsp_attn_prefill(const vsp_tensor* q, const vsp_tensor* k, const vsp_tensor* v, vsp_tensor* out,
                                vsp_tensor* lse, float scale, int is_causal, float dropout_p, int training,
                                void* stream) {
    return prefill_entry(q, k, v, out, lse, scale, is_causal, dropout_p, training, false, nullptr, 0, stream);
}

extern "C" size_t vsp_attn_prefill_split_workspace_bytes(int32_t B, int32_t Hq, int32_t Hkv, int32_t T, int32_t L, int32_t D) {
    if (B <= 0 || Hq <= 0 || Hkv <= 0 || T <= 0 || L <= 0 || D <= 0) return 0;
    return 4 * split_plane_bytes((int64_t)B * Hkv * L * D);  // hi and lo planes of K and of V
}

extern "C" int vsp_attn_prefill_split(const vsp_tensor* q, const vsp_tensor* k, const vsp_tensor* v, vsp_tensor* out,
                                      vsp_tensor* lse, float scale, int is_causal, void* workspace, size_t workspace_bytes,
                                      void* stream) {
    return prefill_entry(q, k, v, out, lse, scale, is_causal, 0.0f, 0, true, workspace, workspace_bytes, stream);
}

namespace {
int prefill_entry(const vsp_tensor* q, const vsp_tensor* k, const vsp_tensor* v, vsp_tensor* out, vsp_tensor* lse, float scale,
                  int is_causal, float dropout_p, int training, bool split, void* workspace, size_t workspace_bytes, void* stream) {
    if (!q || !k || !v || !out) return VSP_ERR_NULL;
    // validation in the reference's order, src/ops/flash_attention.cpp:45-59
    if (q->ndim != 4 || k->ndim != 4 || v->ndim != 4) return VSP_ERR_NDIM;
    const int64_t B = q->shape[0], Hq = q->shape[1], T = q->shape[2], D = q->shape[3];
    const int64_t Hkv = k->shape[1], L = k->shape[2];
    for (int i = 0; i < 4; ++i)
        if (k->shape[i] != v->shape[i]) return VSP_ERR_SHAPE;
    if (k->shape[0] != B || k->shape[3] != D) return VSP_ERR_SHAPE;
    if (Hkv <= 0 ? Hq != 0 : (Hq % Hkv != 0)) return VSP_ERR_SHAPE;
    if (is_causal && T > L) return VSP_ERR_SHAPE;
    if (q->dtype != k->dtype || k->dtype != v->dtype) return VSP_ERR_DTYPE;
    if (dropout_p < 0.0f || dropout_p >= 1.0f) return VSP_ERR_DROPOUT;
    // inference only: dropout is active in the reference iff training && dropout_p > 0 (:241)
    if (training && dropout_p > 0.0f) return VSP_ERR_UNSUPPORTED;
    if (out->ndim != 4) return VSP_ERR_NDIM;
    for (int i = 0; i < 4; ++i)
        if (out->shape[i] != q->shape[i]) return VSP_ERR_SHAPE;
    if (out->dtype != q->dtype) return VSP_ERR_DTYPE;
    if (q->dtype != VSP_BF16 && q->dtype != VSP_F32) return VSP_ERR_UNSUPPORTED;
    if (lse) {
        if (lse->ndim != 3 || lse->shape[0] != B || lse->shape[1] != Hq || lse->shape[2] != T) return VSP_ERR_SHAPE;
        if (lse->dtype != VSP_F32) return VSP_ERR_DTYPE;
    }
    if (B * Hq * T * D == 0) return VSP_OK;
    // bf16: head_dim 64 or 128; fp32: any head_dim up to 256, as the reference's forward takes any (:235-238): the native
    // tiles 32 / 64 / 128, or the next one with the columns past head_dim padded with zeros inside the kernel
    const bool native = native_head_dim(q->dtype, D);
    if (!native && (split || !padded_head_dim(q->dtype, D))) return VSP_ERR_UNSUPPORTED;
    if (L == 0) return VSP_ERR_SHAPE;  // softmax over an empty context is undefined
    if (!(fabsf(scale) > 0.0f) || !(fabsf(scale) < INFINITY)) return VSP_ERR_ARG;
    const int esz = q->dtype == VSP_F32 ? 4 : 2;
    int rc;
    bool elementwise = !native;
    if (native && ((rc = check_tensor4(q, esz)) != VSP_OK || (rc = check_tensor4(k, esz)) != VSP_OK ||
                   (rc = check_tensor4(v, esz)) != VSP_OK || (rc = check_tensor4(out, esz)) != VSP_OK)) {
        if (q->dtype != VSP_F32 || split || rc != VSP_ERR_ALIGN) return rc;
        elementwise = true;  // fp32 rows that are not 16-byte aligned: the element-wise kernel takes them
    }
    if (elementwise && ((rc = check_tensor4_any_d(q)) != VSP_OK || (rc = check_tensor4_any_d(k)) != VSP_OK ||
                        (rc = check_tensor4_any_d(v)) != VSP_OK || (rc = check_tensor4_any_d(out)) != VSP_OK))
        return rc;
    if (lse && !lse->data) return VSP_ERR_NULL;
    if (T > INT32_MAX / 2 || L > INT32_MAX / 2) return VSP_ERR_ARG;
    // the tile loads address one head's rows through a 32-bit buffer descriptor
    if (k->stride[2] < 0 || v->stride[2] < 0) return VSP_ERR_STRIDE;
    if (q->dtype == VSP_BF16 && (L * k->stride[2] * 2 > INT32_MAX || L * v->stride[2] * 2 > INT32_MAX)) return VSP_ERR_STRIDE;

    PrefillArgs a{};
    a.D_true = (int)D;
    a.elementwise = elementwise ? 1 : 0;
    a.q = q->data;
    a.k = k->data;
    a.v = v->data;
    a.out = out->data;
    a.lse = lse ? (float*)lse->data : nullptr;
    for (int i = 0; i < 3; ++i) {
        a.sq[i] = q->stride[i];
        a.sk[i] = k->stride[i];
        a.sv[i] = v->stride[i];
        a.so[i] = out->stride[i];
        a.sl[i] = lse ? lse->stride[i] : 0;
    }
    a.B = (int)B;
    a.Hq = (int)Hq;
    a.Hkv = (int)Hkv;
    a.n_rep = (int)(Hq / Hkv);
    a.T = (int)T;
    a.L = (int)L;
    a.causal = is_causal ? 1 : 0;
    a.n_qtiles = (int)ceil_div(T, kBM);
    a.negate_q = (q->dtype == VSP_BF16 && scale < 0.0f) ? 1 : 0;
    a.scale_log2 = (q->dtype == VSP_BF16 ? fabsf(scale) : scale) * kLog2e;
    if (split) {
        // fp32 tensors through the bf16 matrix cores: split planes in the workspace, then the attention kernel over them
        if (q->dtype != VSP_F32 || (D != 64 && D != 128)) return VSP_ERR_UNSUPPORTED;
        const int64_t nk = B * Hkv * L * D;
        if (L * D * 2 > INT32_MAX || nk / 8 > INT32_MAX * 256LL) return VSP_ERR_ARG;
        const size_t need = 4 * split_plane_bytes(nk);
        if (!workspace || workspace_bytes < need) return VSP_ERR_WORKSPACE;
        if (!is_aligned16(workspace)) return VSP_ERR_ALIGN;
        uint16_t* planes[4];
        for (int i = 0; i < 4; ++i) planes[i] = (uint16_t*)((char*)workspace + i * split_plane_bytes(nk));
        SplitPlan sp{};
        const vsp_tensor* src[2] = {k, v};
        for (int t = 0; t < 2; ++t) {
            sp.src[t] = (const float*)src[t]->data;
            sp.hi[t] = planes[2 * t];
            sp.lo[t] = planes[2 * t + 1];
            sp.s0[t] = src[t]->stride[0];
            sp.s1[t] = src[t]->stride[1];
            sp.s2[t] = src[t]->stride[2];
        }
        sp.H = (int)Hkv;
        sp.N = (int)L;
        sp.groups = nk / 8;
        sp.D = (int)D;
        hipStream_t st = (hipStream_t)stream;
        hipLaunchKernelGGL(split_f32_kernel, dim3((unsigned)ceil_div(nk / 8, 256), 2), dim3(256), 0, st, sp);
        rc = check_launch();
        if (rc != VSP_OK) return rc;
        a.k = planes[0];
        a.k_lo = planes[1];
        a.v = planes[2];
        a.v_lo = planes[3];
        a.sk[0] = Hkv * L * D, a.sk[1] = L * D, a.sk[2] = D;
        a.sv[0] = a.sk[0], a.sv[1] = a.sk[1], a.sv[2] = D;
        a.negate_q = scale < 0.0f ? 1 : 0;
        a.scale_log2 = fabsf(scale) * kLog2e;
        const dim3 grid((unsigned)((int64_t)a.n_qtiles * B * Hq));
        if (D == 128) hipLaunchKernelGGL(prefill_split_kernel<128>, grid, dim3(256), 0, st, a);
        else hipLaunchKernelGGL(prefill_split_kernel<64>, grid, dim3(256), 0, st, a);
        return check_launch();
    }
    return launch_prefill(a, q->dtype, D, false, stream);
}
}  // namespace
