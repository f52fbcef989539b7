// Single-token decode over the KV cache: split-K over the context + combine.
//
// Replaces, for T == 1, what the reference runs below its flash threshold
// (src/nn/functional.cpp:397-421: matmul, div, softmax, matmul over a materialised score tensor)
// together with the two repeat_kv copies before it (src/nn/gqa_attention.cpp:140-141).
//
// One workgroup (4 wavefronts) handles one (batch row, kv head, context split).  The n_rep query
// heads that share the kv head ride in the N dimension of 16x16x32 MFMA tiles (padded to 16), so
// K and V are read from HBM exactly once per kv head:
//   S^T[key][head]  = K[key][:] . Q^T[:][head]        A = K rows as they lie in HBM (16-byte loads)
//   O^T[d][head]   += V^T[d][key] . P^T[key][head]    A = V^T, which the token-blocked V plane
//                                                     stores so that 8/16 tokens of one d are one load
// A wavefront consumes 64 keys per iteration.  MFMA row i of S^T tile jj (0..3) is key
// 16*(i/4) + 4*jj + i%4 of the group, which makes the four S values a lane gets from each tile
// line up with the contraction slots of the PV MFMAs (slot (t, g, e) = key 16*g + 8*t + e) without
// any cross-lane movement.  Online softmax in fp32, exp2 with the scale folded in.
#include <stdlib.h>

#include <mutex>

#include "kv_layout.hpp"
#include "vsp_common.hpp"

namespace vsp {
int check_kv_cache(const vsp_kv_cache* c);

namespace {

constexpr int kWaves = 4;
constexpr int kGroup = 64;  // keys per wave iteration

struct DecodeArgs {
    const void* q;
    int64_t sq_b, sq_h, sq_t;  // q strides (elements) of dims 0, 1, 2
    int32_t T;                 // query tokens per sequence: token t sits at position L - T + t and sees the keys up to itself
    const void* k;
    const void* v;
    const void* k_scale;
    const void* v_scale;
    const int32_t* seq_lens;  // device, or nullptr
    int32_t len;              // used when seq_lens == nullptr
    int32_t B, Hq, Hkv, n_rep;
    int64_t S;  // physical token capacity of the planes
    int32_t S_max;  // logical capacity
    int32_t L_cap;  // min(S_max, the host's upper bound of the lengths): every length is clamped to it, because the
                    // grid, max_splits and the workspace are sized from that bound
    int32_t chunk;
    int32_t max_splits;
    float scale_log2;  // scale * log2(e)
    float* ws_o;       // [B][Hq][T][max_splits][D]
    float* ws_ml;      // [B][Hq][T][max_splits][2]  (m in log2 domain, l)
    // paged cache: sequence b's 64-key group starting at token t lives in page page_table[b * pages_per_seq +
    // t / page_tokens] (page_tokens is a multiple of 64, so a group never straddles two pages); S is then the
    // page size.  nullptr for a contiguous cache.
    const int32_t* page_table;
    int32_t page_tokens, pages_per_seq;
    // More than 16 query heads per kv head (one token per sequence): the heads are cut into n_cgroups groups of 16
    // columns, one workgroup per (item, kv head, group); col0 is the group's first head (set by each workgroup).
    int32_t n_cgroups, col0;
};

// Index of the [S][D] slab that holds the 64-key group at token `kbase` of (sequence b, kv head), and the
// group's first token inside that slab.
template <bool PAGED>
__device__ inline int64_t group_slab(const DecodeArgs& a, int b, int kvh, int kbase, int& local) {
    if constexpr (PAGED) {
        const int pg = kbase / a.page_tokens;
        local = kbase - pg * a.page_tokens;
        return (int64_t)a.page_table[(int64_t)b * a.pages_per_seq + pg] * a.Hkv + kvh;
    } else {
        local = kbase;
        return (int64_t)b * a.Hkv + kvh;
    }
}

__device__ inline float wave_max_over_groups(float x) {
    x = fmaxf(x, __shfl_xor(x, 16));
    x = fmaxf(x, __shfl_xor(x, 32));
    return x;
}
__device__ inline float wave_sum_over_groups(float x) {
    x += __shfl_xor(x, 16);
    x += __shfl_xor(x, 32);
    return x;
}

// The 16 MFMA columns of a work item are the (token, query head of the kv head) pairs of the call, token-major:
// column c = t * n_rep + r.  With one token per sequence (the plain decode step) a column is a query head.
struct Column {
    int t, r;
    bool live;
};
// Columns this workgroup owns: all (token, head) pairs, or its group of up to 16 heads.
__device__ inline int column_count(const DecodeArgs& a) { return a.n_cgroups > 1 ? min(16, a.n_rep - a.col0) : a.n_rep * a.T; }
__device__ inline Column column_of(const DecodeArgs& a, int c) {
    const int n = column_count(a), cc = min(c, n - 1);
    if (a.n_cgroups > 1) return Column{0, a.col0 + cc, c < n};
    return Column{cc / a.n_rep, cc % a.n_rep, c < n};
}
// Which (work item, kv head) a workgroup serves.  kv head fastest: every item that exists comes before the first
// surplus workgroup of the grid (which is sized for the longest possible batch), so the surplus ones start, find
// nothing and exit under the tail of the real work.  With column groups, the groups of one (item, kv head) get block
// ids 8 apart: the same XCD (ids are dealt round-robin to the 8 XCDs), so the K/V stream they share is fetched into
// one L2, once, and read from there by the others.
__device__ inline void block_coords(DecodeArgs& a, int& kvh, int& item) {
    int ik = blockIdx.x;
    if (a.n_cgroups > 1) {  // id = ((ik / 8) * n_cgroups + group) * 8 + ik % 8
        const int rest = blockIdx.x >> 3;
        a.col0 = 16 * (rest % a.n_cgroups);
        ik = (rest / a.n_cgroups) * 8 + (blockIdx.x & 7);
    }
    kvh = ik % a.Hkv;
    item = ik / a.Hkv;
}
// Keys [0, limit) are visible to column col: token t of T sits at position L - T + t and attends up to itself.
__device__ inline int column_limit(const DecodeArgs& a, const Column& col, int L, int chunk_end) {
    return min(chunk_end, L - (a.T - 1 - col.t));
}
// Row of the split-K partials that column col of (batch row b, kv head) writes for `split`.
__device__ inline int64_t partial_row(const DecodeArgs& a, int b, int kvh, const Column& col, int split) {
    return (((int64_t)b * a.Hq + kvh * a.n_rep + col.r) * a.T + col.t) * a.max_splits + split;
}

__device__ inline uint4 mask_tail_u16x8(uint4 v, int nvalid) {
    // keep the first nvalid 16-bit elements, zero the rest
    uint32_t w[4] = {v.x, v.y, v.z, v.w};
#pragma unroll
    for (int i = 0; i < 4; ++i) {
        int rem = nvalid - 2 * i;
        w[i] = rem >= 2 ? w[i] : (rem == 1 ? (w[i] & 0xFFFFu) : 0u);
    }
    return uint4{w[0], w[1], w[2], w[3]};
}


// Work items are (batch row, split) pairs packed without gaps: item i belongs to the sequence b with
// offs(b) <= i < offs(b) + nsplits(b), nsplits(b) = ceil(L_b / chunk).  Lengths live on the device, so
// every workgroup locates its item itself: 64 sequences at a time, one per lane, wave-wide prefix sum.
// The grid is sized for the worst case; surplus workgroups sit at the END of the grid and exit at once
// (with the (split, b) grid of a naive mapping the empty workgroups of short sequences would be
// interleaved with real work and cost launch slots all the way through).
__device__ inline bool locate_work(const DecodeArgs& a, int item, int lane, int& b, int& split, int& L) {
    if (!a.seq_lens) {
        L = min(a.len, a.L_cap);
        const int ns = (L + a.chunk - 1) / a.chunk;
        if (ns == 0 || item >= ns * a.B) return false;
        b = item / ns;
        split = item - b * ns;
        return true;
    }
    int base = 0;
    for (int b0 = 0; b0 < a.B; b0 += 64) {
        const int bb = b0 + lane;
        const int Lb = bb < a.B ? min(max(a.seq_lens[bb], 0), a.L_cap) : 0;
        const int ns = (Lb + a.chunk - 1) / a.chunk;
        int incl = ns;
#pragma unroll
        for (int off = 1; off < 64; off <<= 1) {
            const int t = __shfl_up(incl, off);
            if (lane >= off) incl += t;
        }
        const int total = __shfl(incl, 63);
        if (item < base + total) {
            const unsigned long long m = __ballot(base + incl > item);
            const int src = __ffsll((long long)m) - 1;
            b = b0 + src;
            split = item - (base + __shfl(incl, src) - __shfl(ns, src));
            L = __shfl(Lb, src);
            return true;
        }
        base += total;
    }
    return false;
}

// The (m, l, O^T) of a workgroup's four wavefronts, left in LDS per column, merged into one split-K partial per column.
// First, one lane per column: the merged maximum, the four weights 2^(m_w - m), the merged sum and the partial's row
// (once per column, not once per element: the weights are four exp2 and the row takes integer divisions).  Then one
// element per thread: o = sum_w weight_w * O_w in wavefront order.  ZERO_FOR_EMPTY: a wavefront that saw no key of a
// short split, or a column with no key in it, carries m = -inf, l = 0 and zero sums, and gets the weight 0 explicitly;
// otherwise -inf is replaced by 0 as the reference point (a column without a key in this split: zero sums, m = -inf).
template <int D, bool ZERO_FOR_EMPTY>
__device__ inline void merge_waves_and_store(const DecodeArgs& a, const float (&sm_o)[kWaves][16][D + 4], const float (&sm_m)[kWaves][16],
                                             const float (&sm_l)[kWaves][16], int b, int kvh, int split, int tid) {
    __shared__ float sm_f[kWaves][16];
    __shared__ int64_t sm_row[16];
    const int ncol = column_count(a);
    if (tid < ncol) {
        const int hc = tid;
        float mm = sm_m[0][hc];
#pragma unroll
        for (int w = 1; w < kWaves; ++w) mm = fmaxf(mm, sm_m[w][hc]);
        const float mm_ref = mm == -INFINITY ? 0.f : mm;
        float ll = 0.f;
#pragma unroll
        for (int w = 0; w < kWaves; ++w) {
            const float f = ZERO_FOR_EMPTY ? (sm_m[w][hc] == -INFINITY ? 0.f : __builtin_amdgcn_exp2f(sm_m[w][hc] - mm))
                                           : __builtin_amdgcn_exp2f(sm_m[w][hc] - mm_ref);
            sm_f[w][hc] = f;
            ll += f * sm_l[w][hc];
        }
        const int64_t row = partial_row(a, b, kvh, column_of(a, hc), split);
        sm_row[hc] = row;
        a.ws_ml[row * 2] = mm;
        a.ws_ml[row * 2 + 1] = ll;
    }
    __syncthreads();
    for (int i = tid; i < ncol * D; i += 256) {
        const int hc = i / D, d = i % D;
        float o = 0.f;
#pragma unroll
        for (int w = 0; w < kWaves; ++w) o += sm_f[w][hc] * sm_o[w][hc][d];
        a.ws_o[sm_row[hc] * D + d] = o;
    }
}

// ---------------------------------------------------------------------------------------------
// bf16 cache
// ---------------------------------------------------------------------------------------------
template <int D, bool PAGED>
__global__ void __launch_bounds__(256, 2) decode_bf16_kernel(DecodeArgs a) {
    constexpr int KS = D / 32;   // MFMA k-steps over the head dim
    constexpr int DB = D / 16;   // 16-row tiles of O^T
    const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
    int kvh, item;
    block_coords(a, kvh, item);
    int b, split, L;
    if (!locate_work(a, item, lane, b, split, L)) return;
    const int chunk_start = split * a.chunk;
    const int chunk_end = min(L, chunk_start + a.chunk);

    const int c = lane & 15, g = lane >> 4;

    // Q^T operands: column c = (token, query head of this kv head), zero beyond the last one
    const Column col = column_of(a, c);
    const int lim = column_limit(a, col, L, chunk_end);
    bf16x8_t qf[KS];
    {
        const uint16_t* qrow = (const uint16_t*)a.q + (int64_t)b * a.sq_b + (int64_t)(kvh * a.n_rep + col.r) * a.sq_h + (int64_t)col.t * a.sq_t;
#pragma unroll
        for (int ks = 0; ks < KS; ++ks) {
            uint4 w = *(const uint4*)(qrow + 32 * ks + 8 * g);
            if (!col.live) w = uint4{0, 0, 0, 0};
            qf[ks] = __builtin_bit_cast(bf16x8_t, w);
        }
    }
    const int krow = 16 * (c >> 2) + (c & 3);  // this lane's A-operand row: key offset before + 4*jj

    f32x4_t acc[DB];
#pragma unroll
    for (int i = 0; i < DB; ++i) acc[i] = f32x4_t{0.f, 0.f, 0.f, 0.f};
    float m = -INFINITY, l = 0.f;

    // K rows (A operands of S^T) and V^T blocks (A operands of O^T) of one 64-key group.  The loop is
    // rotated: the loads of group i+1 are issued as soon as group i's registers have been consumed
    // (K after the S^T MFMAs, V after the O^T MFMAs), so every wavefront keeps HBM requests in flight
    // while it computes.
    uint4 kf[4][KS];
    uint4 vf[DB][2];
    auto load_k = [&](int kbase) {
        int local;
        const uint16_t* Kp = (const uint16_t*)a.k + group_slab<PAGED>(a, b, kvh, kbase, local) * a.S * D;
#pragma unroll
        for (int jj = 0; jj < 4; ++jj) {
            const uint16_t* kr = Kp + (int64_t)(local + krow + 4 * jj) * D + 8 * g;
#pragma unroll
            for (int ks = 0; ks < KS; ++ks) kf[jj][ks] = *(const uint4*)(kr + 32 * ks);
        }
    };
    auto load_v = [&](int kbase) {
        int local;
        const uint16_t* Vp = (const uint16_t*)a.v + group_slab<PAGED>(a, b, kvh, kbase, local) * a.S * D;
        const uint16_t* vb = Vp + ((int64_t)(local / kVBlkBf16 + 2 * g) * D + c) * kVBlkBf16;
#pragma unroll
        for (int db = 0; db < DB; ++db)
#pragma unroll
            for (int t = 0; t < 2; ++t) vf[db][t] = *(const uint4*)(vb + ((int64_t)t * D + 16 * db) * kVBlkBf16);
    };
    const int kfirst = chunk_start + wave * kGroup;
    if (kfirst < chunk_end) {
        load_k(kfirst);
        load_v(kfirst);
    }
    for (int kbase = kfirst; kbase < chunk_end; kbase += kWaves * kGroup) {
        const int knext = kbase + kWaves * kGroup;
        // ---- S^T
        f32x4_t s[4];
#pragma unroll
        for (int jj = 0; jj < 4; ++jj) {
            s[jj] = f32x4_t{0.f, 0.f, 0.f, 0.f};
#pragma unroll
            for (int ks = 0; ks < KS; ++ks)
                s[jj] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(__builtin_bit_cast(bf16x8_t, kf[jj][ks]), qf[ks], s[jj], 0, 0, 0);
        }
        if (knext < chunk_end) load_k(knext);
        const bool tail = kbase + kGroup > chunk_end;               // keys past the end of the split: stale rows of the planes
        const bool tail_s = kbase + kGroup > chunk_end - (a.T - 1);  // keys past some column's limit
        float mloc = -INFINITY;
#pragma unroll
        for (int jj = 0; jj < 4; ++jj)
#pragma unroll
            for (int v = 0; v < 4; ++v) {
                float t = s[jj][v] * a.scale_log2;
                if (tail_s && kbase + 16 * g + 4 * jj + v >= lim) t = -INFINITY;
                s[jj][v] = t;
                mloc = fmaxf(mloc, t);
            }
        mloc = wave_max_over_groups(mloc);
        const float m_new = fmaxf(m, mloc);
        // -inf while a column has seen no key yet (several tokens per sequence: the last keys of a context lie past the
        // earlier tokens' limits); its sums then stay zero
        const float m_ref = m_new == -INFINITY ? 0.f : m_new;
        const float alpha = __builtin_amdgcn_exp2f(m - m_ref);
        float lsum = 0.f;
        uint32_t pw[2][4];
#pragma unroll
        for (int jj = 0; jj < 4; ++jj) {
            float p0 = __builtin_amdgcn_exp2f(s[jj][0] - m_ref), p1 = __builtin_amdgcn_exp2f(s[jj][1] - m_ref);
            float p2 = __builtin_amdgcn_exp2f(s[jj][2] - m_ref), p3 = __builtin_amdgcn_exp2f(s[jj][3] - m_ref);
            lsum += (p0 + p1) + (p2 + p3);
            pw[jj >> 1][2 * (jj & 1)] = pack_bf16x2(p0, p1);
            pw[jj >> 1][2 * (jj & 1) + 1] = pack_bf16x2(p2, p3);
        }
        l = l * alpha + lsum;
        m = m_new;
        if (tail) {
#pragma unroll
            for (int db = 0; db < DB; ++db)
#pragma unroll
                for (int t = 0; t < 2; ++t) vf[db][t] = mask_tail_u16x8(vf[db][t], chunk_end - (kbase + 16 * g + 8 * t));
        }
        // ---- O^T
#pragma unroll
        for (int db = 0; db < DB; ++db) {
            acc[db] *= alpha;
#pragma unroll
            for (int t = 0; t < 2; ++t) {
                bf16x8_t pf = __builtin_bit_cast(bf16x8_t, uint4{pw[t][0], pw[t][1], pw[t][2], pw[t][3]});
                acc[db] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(__builtin_bit_cast(bf16x8_t, vf[db][t]), pf, acc[db], 0, 0, 0);
            }
        }
        if (knext < chunk_end) load_v(knext);
    }
    l = wave_sum_over_groups(l);

    // ---- combine the four wavefronts through LDS, write one partial per (b, head, split)
    __shared__ float sm_o[kWaves][16][D + 4];
    __shared__ float sm_m[kWaves][16], sm_l[kWaves][16];
    if (col.live) {
#pragma unroll
        for (int db = 0; db < DB; ++db)
#pragma unroll
            for (int v = 0; v < 4; ++v) sm_o[wave][c][16 * db + 4 * g + v] = acc[db][v];
        if (g == 0) {
            sm_m[wave][c] = m;
            sm_l[wave][c] = l;
        }
    }
    __syncthreads();
    merge_waves_and_store<D, false>(a, sm_o, sm_m, sm_l, b, kvh, split, tid);
}

// ---------------------------------------------------------------------------------------------
// Q8_0 cache: int8 payload widened to fp16 in registers and scaled, fp16 MFMA.
// ---------------------------------------------------------------------------------------------
// 4 int8 (one dword, two's complement) -> 4 fp16 holding the same integers.  x ^ 0x80 is the
// biased value u = q + 128; 0x6400 | u is the fp16 1024 + u; subtracting 1152 is exact.
__device__ inline void i8x4_to_f16x4(uint32_t w, f16x2_t& lo, f16x2_t& hi) {
    const uint32_t x = w ^ 0x80808080u;
    const uint32_t a = __builtin_amdgcn_perm(0x64646464u, x, 0x04010400u);
    const uint32_t bq = __builtin_amdgcn_perm(0x64646464u, x, 0x04030402u);
    const f16x2_t bias = {(_Float16)1152.0f, (_Float16)1152.0f};
    lo = __builtin_bit_cast(f16x2_t, a) - bias;
    hi = __builtin_bit_cast(f16x2_t, bq) - bias;
}
__device__ inline uint32_t f16x2_bits(f16x2_t v) { return __builtin_bit_cast(uint32_t, v); }

template <int D, bool PAGED>
__global__ void __launch_bounds__(256, 2) decode_q8_kernel(DecodeArgs a) {
    constexpr int KS = D / 32;
    constexpr int DB = D / 16;
    constexpr int NH = D / 64;  // 16-byte K loads per row per lane
    constexpr int NQ = D / kQBlock;
    const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
    int kvh, item;
    block_coords(a, kvh, item);
    int b, split, L;
    if (!locate_work(a, item, lane, b, split, L)) return;
    const int chunk_start = split * a.chunk;
    const int chunk_end = min(L, chunk_start + a.chunk);

    const int c = lane & 15, g = lane >> 4;

    // Q^T operands in fp16.  Contraction slot (ks, g, e) is head-dim index
    // 64*(ks/2) + 16*g + 8*(ks%2) + e, so that one 16-byte K load (16 int8) feeds two k-steps.
    const Column col = column_of(a, c);
    const int lim = column_limit(a, col, L, chunk_end);
    f16x8_t qf[KS];
    {
        const uint16_t* qrow = (const uint16_t*)a.q + (int64_t)b * a.sq_b + (int64_t)(kvh * a.n_rep + col.r) * a.sq_h + (int64_t)col.t * a.sq_t;
#pragma unroll
        for (int ks = 0; ks < KS; ++ks) {
            uint4 w = *(const uint4*)(qrow + 64 * (ks >> 1) + 16 * g + 8 * (ks & 1));
            const uint32_t ww[4] = {w.x, w.y, w.z, w.w};
#pragma unroll
            for (int i = 0; i < 4; ++i) {
                float lo = bf16_bits_to_f32((uint16_t)(ww[i] & 0xFFFFu)), hi = bf16_bits_to_f32((uint16_t)(ww[i] >> 16));
                lo = fminf(fmaxf(lo, -65504.f), 65504.f);
                hi = fminf(fmaxf(hi, -65504.f), 65504.f);
                if (!col.live) lo = hi = 0.f;
                qf[ks][2 * i] = (_Float16)lo;
                qf[ks][2 * i + 1] = (_Float16)hi;
            }
        }
    }
    const int krow = 16 * (c >> 2) + (c & 3);

    f32x4_t acc[DB];
#pragma unroll
    for (int i = 0; i < DB; ++i) acc[i] = f32x4_t{0.f, 0.f, 0.f, 0.f};
    float m = -INFINITY, l = 0.f;

    // loads of one 64-key group; rotated like the bf16 kernel (K re-issued after S^T, V after O^T)
    uint4 kq[4][NH];
    uint16_t ksc[4][NH];
    uint4 vq[DB];
    uint4 vsc[NQ][2];
    auto load_k = [&](int kbase) {
        int local;
        const int64_t head = group_slab<PAGED>(a, b, kvh, kbase, local);
        const int8_t* Kp = (const int8_t*)a.k + head * a.S * D;
        const uint16_t* KSp = (const uint16_t*)a.k_scale + head * a.S * NQ;
#pragma unroll
        for (int jj = 0; jj < 4; ++jj) {
            const int64_t key = local + krow + 4 * jj;
#pragma unroll
            for (int h = 0; h < NH; ++h) {
                kq[jj][h] = *(const uint4*)(Kp + key * D + 64 * h + 16 * g);
                ksc[jj][h] = KSp[key * NQ + 2 * h + (g >> 1)];
            }
        }
    };
    auto load_v = [&](int kbase) {
        int local;
        const int64_t head = group_slab<PAGED>(a, b, kvh, kbase, local);
        const int8_t* Vp = (const int8_t*)a.v + head * a.S * D;
        const uint16_t* VSp = (const uint16_t*)a.v_scale + head * a.S * NQ;
        const int64_t blk = local / kVBlkQ8 + g;
#pragma unroll
        for (int db = 0; db < DB; ++db) vq[db] = *(const uint4*)(Vp + (blk * D + 16 * db + c) * kVBlkQ8);
#pragma unroll
        for (int qb = 0; qb < NQ; ++qb) {
            const uint4* sp = (const uint4*)(VSp + (blk * NQ + qb) * kVBlkQ8);
            vsc[qb][0] = sp[0];
            vsc[qb][1] = sp[1];
        }
    };
    const int kfirst = chunk_start + wave * kGroup;
    if (kfirst < chunk_end) {
        load_k(kfirst);
        load_v(kfirst);
    }
    for (int kbase = kfirst; kbase < chunk_end; kbase += kWaves * kGroup) {
        const bool tail = kbase + kGroup > chunk_end;
        const bool tail_s = kbase + kGroup > chunk_end - (a.T - 1);
        const int knext = kbase + kWaves * kGroup;
        // ---- S^T
        f32x4_t s[4];
#pragma unroll
        for (int jj = 0; jj < 4; ++jj) {
            s[jj] = f32x4_t{0.f, 0.f, 0.f, 0.f};
#pragma unroll
            for (int h = 0; h < NH; ++h) {
                const _Float16 sc = __builtin_bit_cast(_Float16, ksc[jj][h]);
                const f16x2_t sc2 = {sc, sc};
                const uint32_t w[4] = {kq[jj][h].x, kq[jj][h].y, kq[jj][h].z, kq[jj][h].w};
                uint32_t o[8];
#pragma unroll
                for (int i = 0; i < 4; ++i) {
                    f16x2_t lo, hi;
                    i8x4_to_f16x4(w[i], lo, hi);
                    o[2 * i] = f16x2_bits(lo * sc2);
                    o[2 * i + 1] = f16x2_bits(hi * sc2);
                }
                f16x8_t k0 = __builtin_bit_cast(f16x8_t, uint4{o[0], o[1], o[2], o[3]});
                f16x8_t k1 = __builtin_bit_cast(f16x8_t, uint4{o[4], o[5], o[6], o[7]});
                s[jj] = __builtin_amdgcn_mfma_f32_16x16x32_f16(k0, qf[2 * h], s[jj], 0, 0, 0);
                s[jj] = __builtin_amdgcn_mfma_f32_16x16x32_f16(k1, qf[2 * h + 1], s[jj], 0, 0, 0);
            }
        }
        if (knext < chunk_end) load_k(knext);
        float mloc = -INFINITY;
#pragma unroll
        for (int jj = 0; jj < 4; ++jj)
#pragma unroll
            for (int v = 0; v < 4; ++v) {
                float t = s[jj][v] * a.scale_log2;
                if (tail_s && kbase + 16 * g + 4 * jj + v >= lim) t = -INFINITY;
                s[jj][v] = t;
                mloc = fmaxf(mloc, t);
            }
        mloc = wave_max_over_groups(mloc);
        const float m_new = fmaxf(m, mloc);
        const float m_ref = m_new == -INFINITY ? 0.f : m_new;   // see decode_bf16_kernel
        const float alpha = __builtin_amdgcn_exp2f(m - m_ref);
        float lsum = 0.f;
        f16x8_t pf[2];
#pragma unroll
        for (int jj = 0; jj < 4; ++jj)
#pragma unroll
            for (int v = 0; v < 4; ++v) {
                const float p = __builtin_amdgcn_exp2f(s[jj][v] - m_ref);
                lsum += p;
                pf[jj >> 1][4 * (jj & 1) + v] = (_Float16)p;
            }
        l = l * alpha + lsum;
        m = m_new;
        // ---- O^T: dequantise V^T operands (16 tokens of one d per lane; per-token scales)
#pragma unroll
        for (int db = 0; db < DB; ++db) {
            acc[db] *= alpha;
            const int qb = (16 * db) / kQBlock;
            const uint32_t w[4] = {vq[db].x, vq[db].y, vq[db].z, vq[db].w};
            const uint32_t scw[8] = {vsc[qb][0].x, vsc[qb][0].y, vsc[qb][0].z, vsc[qb][0].w,
                                     vsc[qb][1].x, vsc[qb][1].y, vsc[qb][1].z, vsc[qb][1].w};
            uint32_t o[8];
#pragma unroll
            for (int i = 0; i < 4; ++i) {
                f16x2_t lo, hi;
                i8x4_to_f16x4(w[i], lo, hi);
                o[2 * i] = f16x2_bits(lo * __builtin_bit_cast(f16x2_t, scw[2 * i]));
                o[2 * i + 1] = f16x2_bits(hi * __builtin_bit_cast(f16x2_t, scw[2 * i + 1]));
            }
            uint4 v0 = uint4{o[0], o[1], o[2], o[3]}, v1 = uint4{o[4], o[5], o[6], o[7]};
            if (tail) {
                v0 = mask_tail_u16x8(v0, chunk_end - (kbase + 16 * g));
                v1 = mask_tail_u16x8(v1, chunk_end - (kbase + 16 * g + 8));
            }
            acc[db] = __builtin_amdgcn_mfma_f32_16x16x32_f16(__builtin_bit_cast(f16x8_t, v0), pf[0], acc[db], 0, 0, 0);
            acc[db] = __builtin_amdgcn_mfma_f32_16x16x32_f16(__builtin_bit_cast(f16x8_t, v1), pf[1], acc[db], 0, 0, 0);
        }
        if (knext < chunk_end) load_v(knext);
    }
    l = wave_sum_over_groups(l);

    __shared__ float sm_o[kWaves][16][D + 4];
    __shared__ float sm_m[kWaves][16], sm_l[kWaves][16];
    if (col.live) {
#pragma unroll
        for (int db = 0; db < DB; ++db)
#pragma unroll
            for (int v = 0; v < 4; ++v) sm_o[wave][c][16 * db + 4 * g + v] = acc[db][v];
        if (g == 0) {
            sm_m[wave][c] = m;
            sm_l[wave][c] = l;
        }
    }
    __syncthreads();
    merge_waves_and_store<D, false>(a, sm_o, sm_m, sm_l, b, kvh, split, tid);
}

// ---------------------------------------------------------------------------------------------
// fp32 cache in the reference's own layout, any head size: plain fp32 arithmetic, one workgroup per
// (batch row, group of query heads, split).  Serves what decode_f32_mfma_kernel does not take (D other than 64 / 128,
// more than 16 query heads per kv head).
// ---------------------------------------------------------------------------------------------
// NH query heads of one kv head per workgroup (NH divides n_rep), so that K and V are read n_rep / NH times instead of
// n_rep times; a thread owns a key in the score phase and a (d, key residue) pair in the output phase.
template <int MAXD, int NH>
__global__ void __launch_bounds__(256) decode_f32_kernel(DecodeArgs a, int D) {
    const int tid = threadIdx.x;
    const int hq0 = blockIdx.y * NH;
    int b, split, L;
    if (!locate_work(a, blockIdx.x, tid & 63, b, split, L)) return;
    const int chunk_start = split * a.chunk;
    const int chunk_end = min(L, chunk_start + a.chunk);
    const int n = chunk_end - chunk_start;
    const int kvh = hq0 / a.n_rep;

    extern __shared__ float smem[];
    float* sq = smem;                    // [NH][MAXD]
    float* sp = smem + NH * MAXD;        // [NH][chunk]
    float* red = sp + NH * a.chunk;      // [256]
    for (int i = tid; i < NH * D; i += 256) {
        const int r = i / D, d = i - r * D;
        sq[r * MAXD + d] = ((const float*)a.q + (int64_t)b * a.sq_b + (int64_t)(hq0 + r) * a.sq_h)[d];
    }
    __syncthreads();
    const float* Kp = (const float*)a.k + (((int64_t)b * a.Hkv + kvh) * a.S + chunk_start) * D;
    const float* Vp = (const float*)a.v + (((int64_t)b * a.Hkv + kvh) * a.S + chunk_start) * D;
    float mloc[NH];
#pragma unroll
    for (int r = 0; r < NH; ++r) mloc[r] = -INFINITY;
    for (int j = tid; j < n; j += 256) {
        const float4* kr = (const float4*)(Kp + (int64_t)j * D);
        float s[NH];
#pragma unroll
        for (int r = 0; r < NH; ++r) s[r] = 0.f;
        for (int d4 = 0; d4 < D / 4; ++d4) {
            const float4 kk = kr[d4];
#pragma unroll
            for (int r = 0; r < NH; ++r) {
                const float* qr = sq + r * MAXD + 4 * d4;
                s[r] = fmaf(qr[0], kk.x, s[r]);
                s[r] = fmaf(qr[1], kk.y, s[r]);
                s[r] = fmaf(qr[2], kk.z, s[r]);
                s[r] = fmaf(qr[3], kk.w, s[r]);
            }
        }
#pragma unroll
        for (int r = 0; r < NH; ++r) {
            const float t = s[r] * a.scale_log2;
            sp[r * a.chunk + j] = t;
            mloc[r] = fmaxf(mloc[r], t);
        }
    }
    float m[NH], l[NH];
#pragma unroll
    for (int r = 0; r < NH; ++r) {
        red[tid] = mloc[r];
        __syncthreads();
        for (int st = 128; st > 0; st >>= 1) {
            if (tid < st) red[tid] = fmaxf(red[tid], red[tid + st]);
            __syncthreads();
        }
        m[r] = red[0];
        __syncthreads();
        float lloc = 0.f;
        for (int j = tid; j < n; j += 256) {
            const float p = exp2f(sp[r * a.chunk + j] - m[r]);
            sp[r * a.chunk + j] = p;
            lloc += p;
        }
        red[tid] = lloc;
        __syncthreads();
        for (int st = 128; st > 0; st >>= 1) {
            if (tid < st) red[tid] += red[tid + st];
            __syncthreads();
        }
        l[r] = red[0];
        __syncthreads();
    }
    // PV: thread (d, part) sums keys part, part+P, ...; P = 256 / D' where D' = D rounded up to a power of two
    int Dp = 1;
    while (Dp < D) Dp <<= 1;
    const int P = 256 / Dp > 0 ? 256 / Dp : 1;
    const int d = tid % Dp, part = tid / Dp;
    float o[NH];
#pragma unroll
    for (int r = 0; r < NH; ++r) o[r] = 0.f;
    if (d < D && part < P)
        for (int j = part; j < n; j += P) {
            const float vv = Vp[(int64_t)j * D + d];
#pragma unroll
            for (int r = 0; r < NH; ++r) o[r] = fmaf(sp[r * a.chunk + j], vv, o[r]);
        }
#pragma unroll
    for (int r = 0; r < NH; ++r) {
        __syncthreads();
        red[tid] = o[r];
        __syncthreads();
        if (tid < D && tid < Dp) {
            float t = 0.f;
            for (int p = 0; p < P; ++p) t += red[p * Dp + tid];
            const int64_t row = ((int64_t)b * a.Hq + hq0 + r) * a.max_splits + split;
            a.ws_o[row * D + tid] = t;
            if (tid == 0) {
                a.ws_ml[row * 2] = m[r];
                a.ws_ml[row * 2 + 1] = l[r];
            }
        }
    }
}

// ---------------------------------------------------------------------------------------------
// fp32 cache, D = 64 or 128, n_rep <= 16: the bf16 kernel's structure on fp32 matrix instructions
// (v_mfma_f32_16x16x4_f32), so that the reference's own cache layout is also read once per kv head and at the
// rate HBM delivers it.  One workgroup (4 wavefronts) per (batch row, kv head, context split); a wavefront
// consumes 32 keys per iteration as two 16-key tiles.
//   S^T[key][head] = K[key][:] . Q^T[:][head]: lane (row i, k-slot kk) of the A operand loads the 16 bytes
//     K[key i][16 cc + 4 kk .. + 3] and feeds its four floats to four MFMAs; MFMA (cc, e) contracts over
//     d = 16 cc + 4 kk + e, and the Q^T operand is laid out to match (scale * log2(e) folded in).
//   O^T[d][head] += V^T[d][key] . P^T[key][head]: the S^T result of a lane holds keys 4 g + v of the tile, so
//     k-step v of the PV product takes the keys {4 kk + v}: P needs no cross-lane movement and stays fp32.
//     Lane (row i, kk) loads the 16 bytes V[key 4 kk + v][64 vc + 4 i .. + 3] and feeds them to four MFMAs;
//     tile (vc, e) therefore holds the rows d = 64 vc + 4 i + e.
// Keys past the end of the split are read from the split's last valid row instead (the planes are not padded, and
// rows that were never written may hold anything) and masked in S.
// ---------------------------------------------------------------------------------------------
template <int D>
__global__ void __launch_bounds__(256, 2) decode_f32_mfma_kernel(DecodeArgs a) {
    constexpr int C4 = D / 16;  // 16-byte pieces of a K row per lane
    constexpr int VC = D / 64;  // 16-byte pieces of a V row per lane
    constexpr int KT = 2;       // 16-key tiles per wavefront iteration
    constexpr int GROUP = 16 * KT;
    const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
    int kvh, item;
    block_coords(a, kvh, item);
    int b, split, L;
    if (!locate_work(a, item, lane, b, split, L)) return;
    const int chunk_start = split * a.chunk;
    const int chunk_end = min(L, chunk_start + a.chunk);
    const int c = lane & 15, g = lane >> 4;

    const Column col = column_of(a, c);
    const int lim = column_limit(a, col, L, chunk_end);
    float qf[C4][4];
    {
        const float* qrow = (const float*)a.q + (int64_t)b * a.sq_b + (int64_t)(kvh * a.n_rep + col.r) * a.sq_h + (int64_t)col.t * a.sq_t;
#pragma unroll
        for (int cc = 0; cc < C4; ++cc) {
            const float4 w = *(const float4*)(qrow + 16 * cc + 4 * g);
            const float f = col.live ? a.scale_log2 : 0.f;
            qf[cc][0] = w.x * f, qf[cc][1] = w.y * f, qf[cc][2] = w.z * f, qf[cc][3] = w.w * f;
        }
    }
    const float* Kp = (const float*)a.k + ((int64_t)b * a.Hkv + kvh) * a.S * D;
    const float* Vp = (const float*)a.v + ((int64_t)b * a.Hkv + kvh) * a.S * D;

    f32x4_t acc[VC][4];
#pragma unroll
    for (int i = 0; i < VC; ++i)
#pragma unroll
        for (int e = 0; e < 4; ++e) acc[i][e] = f32x4_t{0.f, 0.f, 0.f, 0.f};
    float m = -INFINITY, l = 0.f;

    float4 kf[KT][C4];
    float4 vf[KT][4][VC];
    const int last = chunk_end - 1;
    auto load_k = [&](int kbase) {
#pragma unroll
        for (int t = 0; t < KT; ++t) {
            const float* kr = Kp + (int64_t)min(kbase + 16 * t + c, last) * D + 4 * g;
#pragma unroll
            for (int cc = 0; cc < C4; ++cc) kf[t][cc] = *(const float4*)(kr + 16 * cc);
        }
    };
    auto load_v = [&](int kbase) {
#pragma unroll
        for (int t = 0; t < KT; ++t)
#pragma unroll
            for (int v = 0; v < 4; ++v) {
                const float* vr = Vp + (int64_t)min(kbase + 16 * t + 4 * g + v, last) * D + 4 * c;
#pragma unroll
                for (int vc = 0; vc < VC; ++vc) vf[t][v][vc] = *(const float4*)(vr + 64 * vc);
            }
    };
    const int kfirst = chunk_start + wave * GROUP;
    if (kfirst < chunk_end) {
        load_k(kfirst);
        load_v(kfirst);
    }
    for (int kbase = kfirst; kbase < chunk_end; kbase += kWaves * GROUP) {
        const int knext = kbase + kWaves * GROUP;
        f32x4_t s[KT];
#pragma unroll
        for (int t = 0; t < KT; ++t) {
            s[t] = f32x4_t{0.f, 0.f, 0.f, 0.f};
#pragma unroll
            for (int cc = 0; cc < C4; ++cc) {
                const float kk[4] = {kf[t][cc].x, kf[t][cc].y, kf[t][cc].z, kf[t][cc].w};
#pragma unroll
                for (int e = 0; e < 4; ++e) s[t] = __builtin_amdgcn_mfma_f32_16x16x4f32(kk[e], qf[cc][e], s[t], 0, 0, 0);
            }
        }
        if (knext < chunk_end) load_k(knext);
        const bool tail_s = kbase + GROUP > chunk_end - (a.T - 1);
        float mloc = -INFINITY;
#pragma unroll
        for (int t = 0; t < KT; ++t)
#pragma unroll
            for (int v = 0; v < 4; ++v) {
                float x = s[t][v];
                if (tail_s && kbase + 16 * t + 4 * g + v >= lim) x = -INFINITY;
                s[t][v] = x;
                mloc = fmaxf(mloc, x);
            }
        mloc = wave_max_over_groups(mloc);
        const float m_new = fmaxf(m, mloc);
        const float m_ref = m_new == -INFINITY ? 0.f : m_new;   // see decode_bf16_kernel
        const float alpha = __builtin_amdgcn_exp2f(m - m_ref);
        float lsum = 0.f;
#pragma unroll
        for (int t = 0; t < KT; ++t)
#pragma unroll
            for (int v = 0; v < 4; ++v) {
                s[t][v] = __builtin_amdgcn_exp2f(s[t][v] - m_ref);
                lsum += s[t][v];
            }
        l = l * alpha + lsum;
        m = m_new;
#pragma unroll
        for (int vc = 0; vc < VC; ++vc)
#pragma unroll
            for (int e = 0; e < 4; ++e) acc[vc][e] *= alpha;
#pragma unroll
        for (int t = 0; t < KT; ++t)
#pragma unroll
            for (int v = 0; v < 4; ++v)
#pragma unroll
                for (int vc = 0; vc < VC; ++vc) {
                    const float vv[4] = {vf[t][v][vc].x, vf[t][v][vc].y, vf[t][v][vc].z, vf[t][v][vc].w};
#pragma unroll
                    for (int e = 0; e < 4; ++e) acc[vc][e] = __builtin_amdgcn_mfma_f32_16x16x4f32(vv[e], s[t][v], acc[vc][e], 0, 0, 0);
                }
        if (knext < chunk_end) load_v(knext);
    }
    l = wave_sum_over_groups(l);

    // ---- combine the four wavefronts through LDS, write one partial per (b, head, split)
    __shared__ float sm_o[kWaves][16][D + 4];
    __shared__ float sm_m[kWaves][16], sm_l[kWaves][16];
    if (col.live) {
#pragma unroll
        for (int vc = 0; vc < VC; ++vc)
#pragma unroll
            for (int e = 0; e < 4; ++e)
#pragma unroll
                for (int v = 0; v < 4; ++v) sm_o[wave][c][64 * vc + 4 * (4 * g + v) + e] = acc[vc][e][v];
        if (g == 0) {
            sm_m[wave][c] = m;
            sm_l[wave][c] = l;
        }
    }
    __syncthreads();
    merge_waves_and_store<D, true>(a, sm_o, sm_m, sm_l, b, kvh, split, tid);
}

// ---------------------------------------------------------------------------------------------
// combine: out[b][h][:] = sum_s w_s O_s / sum_s w_s l_s, w_s = 2^(m_s - max m); fixed order.
// ---------------------------------------------------------------------------------------------
template <typename OutT, int BLK>
__global__ void __launch_bounds__(256) decode_combine_kernel(const float* __restrict__ ws_o, const float* __restrict__ ws_ml,
                                                             const int32_t* __restrict__ seq_lens, int32_t len, int32_t chunk,
                                                             int32_t max_splits, int32_t Hq, int32_t D, OutT* __restrict__ out,
                                                             int64_t so_b, int64_t so_h, int32_t L_cap, int32_t T, int64_t so_t,
                                                             CombineExtra x) {
    const int hq = blockIdx.x / T, t = blockIdx.x % T, b = blockIdx.y, d = threadIdx.x;
    // the producers' clamp: [0, L_cap] in the decode step (locate_work); a chunk of a prompt is part of its context, so
    // there a row is at least as long as its chunk (prefill_bf16_pipe_kernel)
    const int len_floor = x.chunk_lens ? min(max(x.chunk_lens[b], 0), x.len_floor) : x.len_floor;
    const int L = min(max(seq_lens ? seq_lens[b] : len, len_floor), L_cap);
    const int ns = min((L + chunk - 1) / chunk, max_splits);
    const int64_t row0 = (((int64_t)b * Hq + hq) * T + t) * max_splits;
    // One pass over blocks of BLK splits (8, 16 or 32, the smallest that covers the launch's split count): everything a block needs (maxima, sums, partial rows) is requested before any of
    // it is used, so the workgroup pays one memory latency per block instead of one per dependent step; across blocks
    // the reference point moves as in the online softmax.  Within a block and across blocks the sums run over the
    // splits in ascending order: the result does not depend on anything but the inputs.
    float M = -INFINITY, o = 0.f, l = 0.f;
    const float* po = ws_o + row0 * D + (d < D ? d : 0);
    for (int s0 = 0; s0 < ns; s0 += BLK) {
        float x[BLK], ms[BLK], ls[BLK];
#pragma unroll
        for (int i = 0; i < BLK; ++i) {
            const int64_t si = min(s0 + i, ns - 1);
            x[i] = po[si * D];
            ms[i] = ws_ml[(row0 + si) * 2];
            ls[i] = ws_ml[(row0 + si) * 2 + 1];
        }
        float Mb = M;
#pragma unroll
        for (int i = 0; i < BLK; ++i) Mb = fmaxf(Mb, ms[i]);   // indices past the end repeat the last split: harmless in a maximum
        const float keep = exp2f(M - Mb);                      // 0 for the first block (M = -inf, Mb finite)
        o *= keep;
        l *= keep;
        M = Mb;
#pragma unroll
        for (int i = 0; i < BLK; ++i)
            if (s0 + i < ns) {
                const float w = exp2f(ms[i] - M);
                l += w * ls[i];
                o += w * x[i];
            }
    }
    if (d < D) {
        const float r = (ns > 0 && l > 0.f) ? o / l : 0.f;   // l = 0: a token placed before the start of its context
        OutT* p = out + (int64_t)b * so_b + (int64_t)hq * so_h + (int64_t)t * so_t + d;
        if constexpr (sizeof(OutT) == 4) *p = r;
        else *p = f32_to_bf16_bits(r);
    }
    // LSE = m + log l (src/ops/flash_attention.cpp:359), here from the merged (M, l) in the log2 domain; a row that met
    // no key has l = 0 and reads -inf, as the unsplit kernels write it
    if (x.lse && d == 0) x.lse[(int64_t)b * x.sl[0] + (int64_t)hq * x.sl[1] + (int64_t)t * x.sl[2]] = (M + __builtin_amdgcn_logf(l)) * 0.6931471805599453f;
}

// ---------------------------------------------------------------------------------------------
// Output projection behind the combine: y[m][n] = sum_k x[m][k] W[n][k] + bias[n]
// (Linear::forward, src/nn/linear.cpp:41-49, as GroupedQueryAttention applies it to the merged heads,
// src/nn/gqa_attention.cpp:151-152).  x is the decode output [B][Hq*D] left in the workspace, so M = B is small and
// the job is one pass over W at HBM rate.  Workgroup (nb, ks) owns 128 output columns (16 per wavefront) and the
// ks-th of KS equal ranges of K.  Per 512-wide piece of its range every lane first issues its sixteen 16-byte loads
// of W rows (the A operands of 16x16x32 MFMAs, straight from HBM into registers), then the workgroup stages the
// matching piece of x in LDS once for its eight wavefronts (x^T is the B operand; up to MT tiles of 16 batch rows share
// the pass over W).  The fp32 partial tiles go to P[ks][m][n] (through LDS, so that P is written in whole rows);
// proj_reduce_kernel adds the KS partials in index order, the bias, and rounds.  The reduction is a second launch on
// purpose: folding it into the last workgroup to arrive needs device-scope fences, which on this multi-die part write
// back and invalidate the L2 slices and cost several times the whole projection.
// ---------------------------------------------------------------------------------------------
constexpr int kProjWaves = 8;     // wavefronts per workgroup, 16 output columns each
constexpr int kProjCols = 16 * kProjWaves;
constexpr int kProjThreads = 64 * kProjWaves;
constexpr int kProjPiece = 512;   // k values staged in LDS at a time
constexpr int kProjPitch = kProjPiece + 8;  // LDS row pitch (elements): 16 rows of one 16-byte read fall in 64 distinct banks
constexpr int kProjMaxSplit = 8;

template <int MT>
__global__ void __launch_bounds__(kProjThreads) proj_bf16_partial_kernel(const uint16_t* __restrict__ x, const uint16_t* __restrict__ w,
                                                                int64_t w_pitch, float* __restrict__ part, int32_t m0, int32_t M,
                                                                int32_t N, int32_t K, int32_t Kc) {
    __shared__ __attribute__((aligned(16))) uint16_t sx[16 * MT * kProjPitch];
    const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
    const int r = lane & 15, g = lane >> 4;
    const int n0 = blockIdx.x * kProjCols + 16 * wave;
    const int ks = blockIdx.y;
    const int64_t wrow = min(n0 + r, N - 1);  // rows past N are computed from the last row and never stored
    const uint16_t* pw = w + wrow * w_pitch + g * 8;
    const int rows = min(M - m0, 16 * MT);
    f32x4_t acc[MT];
#pragma unroll
    for (int t = 0; t < MT; ++t) acc[t] = f32x4_t{0.f, 0.f, 0.f, 0.f};
    constexpr int kItems = 16 * MT * (kProjPiece / 8) / kProjThreads;  // 16-byte items of x a thread stages per piece
    for (int k0 = ks * Kc; k0 < (ks + 1) * Kc; k0 += kProjPiece) {
        const int piece = min(kProjPiece, (ks + 1) * Kc - k0);  // a multiple of 32
        const int n_slices = piece / 32;
        // x first, W behind it: loads return in order, so x can go to LDS while the W slices are still in flight and
        // the MFMAs start as the slices arrive
        u32x4_t xs[kItems];
#pragma unroll
        for (int i = 0; i < kItems; ++i) {
            const int e = threadIdx.x + i * kProjThreads, row = e / (kProjPiece / 8), c = e % (kProjPiece / 8);
            if (row < rows && 8 * c < piece) xs[i] = *(const u32x4_t*)(x + (int64_t)(m0 + row) * K + k0 + 8 * c);
        }
        bf16x8_t a[16];
#pragma unroll
        for (int u = 0; u < 16; ++u)
            if (u < n_slices) a[u] = *(const bf16x8_t*)(pw + k0 + 32 * u);
        __builtin_amdgcn_s_barrier();  // the previous piece's readers are done with sx (their LDS reads fed MFMAs already issued)
#pragma unroll
        for (int i = 0; i < kItems; ++i) {
            const int e = threadIdx.x + i * kProjThreads, row = e / (kProjPiece / 8), c = e % (kProjPiece / 8);
            if (row < rows && 8 * c < piece) *(u32x4_t*)(sx + row * kProjPitch + 8 * c) = xs[i];
        }
        // LDS writes landed, then the barrier: a fence here would also wait for the W loads
        asm volatile("s_waitcnt lgkmcnt(0)" ::: "memory");
        __builtin_amdgcn_s_barrier();
#pragma unroll
        for (int u = 0; u < 16; ++u) {
            if (u < n_slices) {
#pragma unroll
                for (int t = 0; t < MT; ++t) {
                    // rows past `rows` hold whatever LDS held: they only reach output columns that are never stored
                    const bf16x8_t bx = *(const bf16x8_t*)(sx + (16 * t + r) * kProjPitch + 32 * u + 8 * g);
                    acc[t] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(a[u], bx, acc[t], 0, 0, 0);
                }
            }
        }
    }
    // The partial tile goes through LDS so that P is written in whole rows.  A lane holds batch row r of tile t, output
    // columns 16 wave + 4 g + i of the workgroup's 128.
    constexpr int kTilePitch = kProjCols + 4;  // floats; 16 rows of one 16-byte write fall in 64 distinct banks
    float* tile = (float*)sx;
    __builtin_amdgcn_s_barrier();  // every wavefront's reads of sx have returned (they fed its MFMAs)
#pragma unroll
    for (int t = 0; t < MT; ++t) *(f32x4_t*)(tile + (16 * t + r) * kTilePitch + 16 * wave + 4 * g) = acc[t];
    asm volatile("s_waitcnt lgkmcnt(0)" ::: "memory");
    __builtin_amdgcn_s_barrier();
    const int nb0 = blockIdx.x * kProjCols;
    const bool vec = (N & 3) == 0;  // then a group of four columns is inside the row and 16-byte aligned in P
    for (int e = threadIdx.x; e < rows * (kProjCols / 4); e += kProjThreads) {
        const int m = e / (kProjCols / 4), c = (e % (kProjCols / 4)) * 4, n = nb0 + c;
        const f32x4_t v = *(const f32x4_t*)(tile + m * kTilePitch + c);
        float* dst = part + ((int64_t)ks * M + m0 + m) * N + n;
        if (vec && n < N) *(f32x4_t*)dst = v;
        else
            for (int i = 0; i < 4; ++i)
                if (n + i < N) dst[i] = v[i];
    }
}

// Up to 16 batch rows: one launch.  A workgroup owns 16 output columns; its eight wavefronts take the 32-wide slices of K
// round-robin (slice c goes to wavefront c % 8), x^T comes straight from L2 (16 rows at most: no staging pays), and the
// eight partial tiles meet in LDS, where they are added in wavefront order.  No partial buffer, no second launch.
__global__ void __launch_bounds__(512) proj_bf16_small_kernel(const uint16_t* __restrict__ x, const uint16_t* __restrict__ w,
                                                              int64_t w_pitch, const uint16_t* __restrict__ bias,
                                                              uint16_t* __restrict__ y, int64_t y_pitch, int32_t M, int32_t N,
                                                              int32_t K) {
    __shared__ float part[8][16][17];
    const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
    const int r = lane & 15, g = lane >> 4;
    const int n0 = blockIdx.x * 16;
    const uint16_t* pw = w + (int64_t)min(n0 + r, N - 1) * w_pitch + g * 8;  // rows past N: computed, never stored
    const uint16_t* px = x + (int64_t)min(r, M - 1) * K + g * 8;             // likewise for batch rows past M
    const int n_slices = K / 32;
    f32x4_t acc = {0.f, 0.f, 0.f, 0.f};
    for (int c0 = wave; c0 < n_slices; c0 += 8 * 16) {  // sixteen slices of W (and of x) in flight per lane
        bf16x8_t a[16], b[16];
#pragma unroll
        for (int u = 0; u < 16; ++u)
            if (c0 + 8 * u < n_slices) a[u] = *(const bf16x8_t*)(pw + (int64_t)(c0 + 8 * u) * 32);
#pragma unroll
        for (int u = 0; u < 16; ++u)
            if (c0 + 8 * u < n_slices) b[u] = *(const bf16x8_t*)(px + (int64_t)(c0 + 8 * u) * 32);
#pragma unroll
        for (int u = 0; u < 16; ++u)
            if (c0 + 8 * u < n_slices) acc = __builtin_amdgcn_mfma_f32_16x16x32_bf16(a[u], b[u], acc, 0, 0, 0);
    }
    // the tile a lane holds: batch row r, output columns 4 g + i
#pragma unroll
    for (int i = 0; i < 4; ++i) part[wave][r][4 * g + i] = acc[i];
    __syncthreads();
    if (threadIdx.x < 256) {
        const int m = threadIdx.x >> 4, n = threadIdx.x & 15;
        if (m < M && n0 + n < N) {
            float sum = part[0][m][n];
#pragma unroll
            for (int wv = 1; wv < 8; ++wv) sum += part[wv][m][n];
            if (bias) sum += bf16_bits_to_f32(bias[n0 + n]);
            y[(int64_t)m * y_pitch + n0 + n] = f32_to_bf16_bits(sum);
        }
    }
}

// y[m][n] = round(sum_ks P[ks][m][n] + bias[n]), the partials added in index order.  VEC consecutive outputs per thread
// (4 when N is a multiple of 4, so that a group never straddles two rows).
template <int VEC>
__global__ void __launch_bounds__(256) proj_reduce_kernel(const float* __restrict__ part, const uint16_t* __restrict__ bias,
                                                          uint16_t* __restrict__ y, int64_t y_pitch, int32_t M, int32_t N, int32_t KS) {
    typedef float vec_t __attribute__((ext_vector_type(VEC)));
    const int64_t e = ((int64_t)blockIdx.x * 256 + threadIdx.x) * VEC;
    const int64_t plane = (int64_t)M * N;
    if (e >= plane) return;
    const int m = (int)(e / N), n = (int)(e - (int64_t)m * N);
    vec_t v[kProjMaxSplit];
#pragma unroll
    for (int s = 0; s < kProjMaxSplit; ++s) v[s] = *(const vec_t*)(part + min(s, KS - 1) * plane + e);  // all loads in flight at once
    vec_t sum = v[0];
#pragma unroll
    for (int s = 1; s < kProjMaxSplit; ++s) sum += s < KS ? v[s] : vec_t(0.f);
#pragma unroll
    for (int j = 0; j < VEC; ++j) {
        float f = sum[j];
        if (bias) f += bf16_bits_to_f32(bias[n + j]);
        y[(int64_t)m * y_pitch + n + j] = f32_to_bf16_bits(f);
    }
}

// fp32 operands (the reference's own dtype): one wavefront per output column, lanes stride over k, eight batch rows
// per pass over the row of W.
__global__ void __launch_bounds__(256) proj_f32_kernel(const float* __restrict__ x, const float* __restrict__ w, int64_t w_pitch,
                                                       const float* __restrict__ bias, float* __restrict__ y, int64_t y_pitch,
                                                       int32_t M, int32_t N, int32_t K) {
    const int lane = threadIdx.x & 63;
    const int n = blockIdx.x * kWaves + (threadIdx.x >> 6);
    if (n >= N) return;
    const float* pw = w + (int64_t)n * w_pitch;
    for (int m0 = 0; m0 < M; m0 += 8) {
        float acc[8] = {0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f};
        for (int k = lane; k < K; k += 64) {
            const float wk = pw[k];
#pragma unroll
            for (int j = 0; j < 8; ++j) acc[j] = fmaf(x[(int64_t)min(m0 + j, M - 1) * K + k], wk, acc[j]);
        }
#pragma unroll
        for (int j = 0; j < 8; ++j) {
            float v = acc[j];
#pragma unroll
            for (int off = 32; off > 0; off >>= 1) v += __shfl_xor(v, off);
            if (lane == 0 && m0 + j < M) y[(int64_t)(m0 + j) * y_pitch + n] = bias ? v + bias[n] : v;
        }
    }
}

// Tokens per split.  Every work item pays a fixed cost (locating itself, loading Q, merging four wavefronts, writing a
// partial) and every split is one more row for the combine kernel, so splits should be as long as they can be while
// the launch still spreads over the chip: the largest candidate that yields at least one work item per two CUs
// (counted with the host's upper bound of the lengths).  Measured on small batches, where it matters (one sequence,
// 32k context: 25.6 us with 1024-token splits against 34.6 us with 256-token ones); a large batch reaches the cap
// whatever the threshold.  The quantised kernel has the heavier per-item cost and the lighter stream, hence its larger
// cap; a step of several tokens per sequence writes that many partial rows per split, hence its (+3 % at batch 32,
// four tokens, contexts of 1k-32k).  Workspace sizing assumes >= 256.
int pick_chunk(int format, int64_t B, int64_t Hkv, int64_t max_len, int64_t tokens) {
    const int64_t want = device_cu_count() / 2;
    const int cap = format == VSP_KV_Q8_0 ? 8192 : (tokens > 1 ? 2048 : 1024);
    for (int chunk = cap; chunk > 256; chunk >>= 1) {
        if (B * Hkv * ceil_div(max_len, chunk) >= want) return chunk;
    }
    return 256;
}

}  // namespace

// out[b][h][t][:] from the split-K partials ws_o [B][Hq][T][max_splits][D], ws_ml [..][2] = (m in the log2 domain, l): the
// combine of the decode step, also used by the context-split prefill over a cache.  A row's split count is
// ceil(its length / chunk), its length seq_lens[b] (or len) clamped to [0, L_cap].
int launch_split_combine(const float* ws_o, const float* ws_ml, const int32_t* seq_lens, int32_t len, int32_t chunk, int32_t max_splits,
                         int64_t B, int64_t Hq, int64_t T, int64_t D, int32_t L_cap, vsp_tensor* out, hipStream_t st,
                         const CombineExtra& extra) {
    dim3 cgrid((unsigned)(Hq * T), (unsigned)B);
    const int cthreads = D <= 64 ? 64 : (D <= 128 ? 128 : 256);
    auto combine = [&](auto out_tag, auto blk) {
        using OutT = decltype(out_tag);
        hipLaunchKernelGGL((decode_combine_kernel<OutT, decltype(blk)::value>), cgrid, dim3(cthreads), 0, st, ws_o, ws_ml, seq_lens, len,
                           chunk, max_splits, (int)Hq, (int)D, (OutT*)out->data, out->stride[0], out->stride[1], L_cap, (int)T,
                           out->stride[2], extra);
    };
    auto combine_blk = [&](auto out_tag) {
        if (max_splits <= 8) combine(out_tag, std::integral_constant<int, 8>{});
        else if (max_splits <= 16) combine(out_tag, std::integral_constant<int, 16>{});
        else combine(out_tag, std::integral_constant<int, 32>{});
    };
    if (out->dtype == VSP_F32) combine_blk(float{});
    else combine_blk(uint16_t{});
    return check_launch();
}
}  // namespace vsp

using namespace vsp;

namespace {

// Split-K partials for callers that cannot allocate (vsp_attn_decode_noalloc): one fixed array per GPU, part of
// the library's code object, held until the process ends.  In host code the array's name is only a handle for
// hipGetSymbolAddress; kernels and launches use the per-device address looked up through it.
constexpr size_t kScratchBytes = 32u << 20;
static __device__ __align__(256) unsigned char scratch[kScratchBytes];

constexpr int kMaxDevices = 64;
void* g_scratch_ptr[kMaxDevices];  // per device, filled on the first call on that device
std::mutex g_scratch_mutex;

// Address of the current device's copy of `scratch` (each GPU holds its own at its own address).
int scratch_for_current_device(void** out) {
    int dev = 0;
    hipError_t e = hipGetDevice(&dev);
    if (e != hipSuccess) {
        set_hip_error(e);
        return VSP_ERR_LAUNCH;
    }
    if (dev < 0 || dev >= kMaxDevices) return VSP_ERR_ARG;
    std::lock_guard<std::mutex> lock(g_scratch_mutex);
    if (!g_scratch_ptr[dev]) {
        void* p = nullptr;
        e = hipGetSymbolAddress(&p, HIP_SYMBOL(scratch));
        if (e != hipSuccess || !p) {
            set_hip_error(e);
            return VSP_ERR_LAUNCH;
        }
        g_scratch_ptr[dev] = p;
    }
    *out = g_scratch_ptr[dev];
    return VSP_OK;
}

// Both decode entry points: validation, split sizing and the two launches.  `own_scratch` selects the
// library's fixed per-device array instead of a caller workspace.
int decode_impl(const vsp_tensor* q, const vsp_kv_cache* cache, const int32_t* seq_lens, int32_t max_len, vsp_tensor* out,
                float scale, void* workspace, size_t workspace_bytes, bool own_scratch, void* stream, bool multi = false) {
    if (!q || !out) return VSP_ERR_NULL;
    int rc = check_kv_cache(cache);
    if (rc != VSP_OK) return rc;
    if (q->ndim != 4 || out->ndim != 4) return VSP_ERR_NDIM;
    const int64_t B = q->shape[0], Hq = q->shape[1], T = q->shape[2], D = q->shape[3];
    if ((multi ? T < 1 : T != 1) || B != cache->B || D != cache->D) return VSP_ERR_SHAPE;
    for (int i = 0; i < 4; ++i)
        if (out->shape[i] != q->shape[i]) return VSP_ERR_SHAPE;
    if (cache->Hkv <= 0 || Hq <= 0 || Hq % cache->Hkv != 0) return VSP_ERR_GQA_HEADS;
    const int n_rep = (int)(Hq / cache->Hkv);
    const int want_dtype = cache->format == VSP_KV_F32 ? VSP_F32 : VSP_BF16;
    if (q->dtype != out->dtype) return VSP_ERR_DTYPE;
    if (q->dtype != want_dtype) return VSP_ERR_UNSUPPORTED;
    // bf16 / Q8_0: the query heads of a kv head ride in the 16 columns of the matrix instructions; more than 16 are
    // served in groups of 16 (one token per sequence; ops::repeat_kv takes any n_rep, src/ops/attention_ops.cpp:92-155)
    if (cache->format == VSP_KV_F32 && D > 256) return VSP_ERR_UNSUPPORTED;
    // several tokens per sequence: they and the query heads of a kv head share the 16 columns of the matrix instructions
    if (T > 1 && (n_rep * T > 16 || (D != 64 && D != 128))) return VSP_ERR_UNSUPPORTED;
    if (B == 0) return VSP_OK;
    if (!q->data || !out->data) return VSP_ERR_NULL;
    if (q->stride[3] != 1 || out->stride[3] != 1) return VSP_ERR_STRIDE;
    const int esz = q->dtype == VSP_F32 ? 4 : 2;
    if (!is_aligned16(q->data) || (q->stride[0] * esz) % 16 || (q->stride[1] * esz) % 16 || (T > 1 && (q->stride[2] * esz) % 16))
        return VSP_ERR_ALIGN;
    if (max_len < 0 || max_len > cache->S_max) return VSP_ERR_ARG;
    // a host-side length above the bound the launch is sized from is a caller error; device-side lengths
    // cannot be read here and are clamped to the bound inside the kernels instead
    if (!seq_lens && max_len > 0 && cache->len > max_len) return VSP_ERR_ARG;
    if (max_len == 0) max_len = seq_lens ? cache->S_max : cache->len;
    hipStream_t st = (hipStream_t)stream;

    const int chunk = max_len > 0 ? pick_chunk(cache->format, B, cache->Hkv, max_len, T) : 256;
    const int max_splits = max_len > 0 ? (int)ceil_div(max_len, chunk) : 1;
    const size_t need = (size_t)(B * Hq * T * max_splits * (D + 2) * 4);
    if (own_scratch) {
        if (max_len > 0 && need > kScratchBytes) return VSP_ERR_WORKSPACE;  // an empty context writes no partials
        rc = scratch_for_current_device(&workspace);
        if (rc != VSP_OK) return rc;
    } else if (max_len > 0) {
        if (!workspace || workspace_bytes < need) return VSP_ERR_WORKSPACE;
        if (!is_aligned16(workspace)) return VSP_ERR_ALIGN;
    }
    DecodeArgs a;
    a.q = q->data;
    a.sq_b = q->stride[0];
    a.sq_h = q->stride[1];
    a.sq_t = q->stride[2];
    a.T = (int)T;
    a.k = cache->k;
    a.v = cache->v;
    a.k_scale = cache->k_scale;
    a.v_scale = cache->v_scale;
    a.seq_lens = seq_lens;
    a.len = cache->len;
    a.B = (int)B;
    a.Hq = (int)Hq;
    a.Hkv = cache->Hkv;
    a.n_rep = n_rep;
    a.S = cache->page_table ? cache->page_tokens : kv_s_pad(cache->format, cache->S_max);
    a.S_max = cache->S_max;
    a.L_cap = max_len < cache->S_max ? max_len : cache->S_max;
    a.page_table = cache->page_table;
    a.page_tokens = cache->page_tokens;
    a.pages_per_seq = cache->pages_per_seq;
    a.chunk = chunk;
    a.max_splits = max_splits;
    a.scale_log2 = scale * kLog2e;
    a.ws_o = (float*)workspace;
    a.ws_ml = a.ws_o ? a.ws_o + (size_t)B * Hq * T * max_splits * D : nullptr;
    a.n_cgroups = (cache->format != VSP_KV_F32 && n_rep > 16) ? (n_rep + 15) / 16 : 1;
    a.col0 = 0;
    // (item, kv head) pairs in the grid, and the grid with one workgroup per pair and column group (pairs padded to a
    // multiple of 8 when there are groups: see block_coords)
    const int64_t pairs = (int64_t)max_splits * B * cache->Hkv;
    const int64_t wgs = a.n_cgroups > 1 ? round_up(pairs, 8) * a.n_cgroups : pairs;
    if (wgs > INT32_MAX) return VSP_ERR_ARG;

    if (max_len > 0) {
        if (cache->format == VSP_KV_BF16) {
            dim3 grid((unsigned)wgs);
            if (cache->page_table) {
                if (D == 128) hipLaunchKernelGGL((decode_bf16_kernel<128, true>), grid, dim3(256), 0, st, a);
                else hipLaunchKernelGGL((decode_bf16_kernel<64, true>), grid, dim3(256), 0, st, a);
            } else {
                if (D == 128) hipLaunchKernelGGL((decode_bf16_kernel<128, false>), grid, dim3(256), 0, st, a);
                else hipLaunchKernelGGL((decode_bf16_kernel<64, false>), grid, dim3(256), 0, st, a);
            }
        } else if (cache->format == VSP_KV_Q8_0) {
            dim3 grid((unsigned)wgs);
            if (cache->page_table) {
                if (D == 128) hipLaunchKernelGGL((decode_q8_kernel<128, true>), grid, dim3(256), 0, st, a);
                else hipLaunchKernelGGL((decode_q8_kernel<64, true>), grid, dim3(256), 0, st, a);
            } else {
                if (D == 128) hipLaunchKernelGGL((decode_q8_kernel<128, false>), grid, dim3(256), 0, st, a);
                else hipLaunchKernelGGL((decode_q8_kernel<64, false>), grid, dim3(256), 0, st, a);
            }
        } else if ((D == 64 || D == 128) && n_rep <= 16) {
            dim3 grid((unsigned)(max_splits * B * cache->Hkv));
            if (D == 128) hipLaunchKernelGGL((decode_f32_mfma_kernel<128>), grid, dim3(256), 0, st, a);
            else hipLaunchKernelGGL((decode_f32_mfma_kernel<64>), grid, dim3(256), 0, st, a);
        } else {
            // as many query heads of a kv head per workgroup as divide n_rep (up to four: 16 KB of scores each at chunk 1024)
            const int nh = n_rep % 4 == 0 ? 4 : (n_rep % 2 == 0 ? 2 : 1);
            dim3 grid((unsigned)(max_splits * B), (unsigned)(Hq / nh));
            const size_t smem = ((size_t)nh * 256 + (size_t)nh * chunk + 256) * sizeof(float);
            if (nh == 4) hipLaunchKernelGGL((decode_f32_kernel<256, 4>), grid, dim3(256), smem, st, a, (int)D);
            else if (nh == 2) hipLaunchKernelGGL((decode_f32_kernel<256, 2>), grid, dim3(256), smem, st, a, (int)D);
            else hipLaunchKernelGGL((decode_f32_kernel<256, 1>), grid, dim3(256), smem, st, a, (int)D);
        }
        rc = check_launch();
        if (rc != VSP_OK) return rc;
    }
    // with max_len == 0 every row is empty: the combine kernel reads nothing and writes zeros
    return launch_split_combine(a.ws_o, a.ws_ml, seq_lens, max_len > 0 ? cache->len : 0, chunk, max_splits, B, Hq, T, D, a.L_cap,
                                out, st);
}

// vsp_attn_decode_proj's workspace: the merged heads x [B][Hq*D] (4 bytes an element whatever the dtype), the
// projection's split-K partials [kProjMaxSplit][B][N] fp32, then the attention step's own partials; each part
// rounded up to 256 bytes.
size_t proj_x_bytes(int64_t B, int64_t Hq, int64_t D) { return (size_t)((B * Hq * D * 4 + 255) / 256 * 256); }
size_t proj_part_bytes(int64_t B, int64_t N) { return (size_t)((kProjMaxSplit * B * N * 4 + 255) / 256 * 256); }

// Equal ranges of K per workgroup row: as many as kProjMaxSplit while each stays a whole number of 32-wide slices.
int proj_split(int64_t K) {
    int ks = kProjMaxSplit;
    while (ks > 1 && K % (32 * ks) != 0) ks >>= 1;
    return ks;
}

}  // namespace

extern "C" {

size_t vsp_attn_decode_workspace_bytes(int32_t B, int32_t Hq, int32_t D, int32_t max_len) {
    if (B <= 0 || Hq <= 0 || D <= 0 || max_len <= 0) return 0;
    const int64_t splits = ceil_div(max_len, 256);
    return (size_t)((int64_t)B * Hq * splits * (D + 2) * 4);
}

int vsp_attn_decode(const vsp_tensor* q, const vsp_kv_cache* cache, const int32_t* seq_lens, int32_t max_len,
                    vsp_tensor* out, float scale, void* workspace, size_t workspace_bytes, void* stream) {
    return decode_impl(q, cache, seq_lens, max_len, out, scale, workspace, workspace_bytes, false, stream);
}

int vsp_attn_decode_multi(const vsp_tensor* q, const vsp_kv_cache* cache, const int32_t* seq_lens, int32_t max_len,
                          vsp_tensor* out, float scale, void* workspace, size_t workspace_bytes, void* stream) {
    return decode_impl(q, cache, seq_lens, max_len, out, scale, workspace, workspace_bytes, false, stream, true);
}

int vsp_attn_decode_noalloc(const vsp_tensor* q, const vsp_kv_cache* cache, const int32_t* seq_lens, int32_t max_len,
                            vsp_tensor* out, float scale, void* stream) {
    return decode_impl(q, cache, seq_lens, max_len, out, scale, nullptr, 0, true, stream);
}

size_t vsp_attn_decode_proj_workspace_bytes(int32_t B, int32_t Hq, int32_t D, int32_t max_len, int32_t N) {
    if (B <= 0 || Hq <= 0 || D <= 0 || N < 0) return 0;
    return proj_x_bytes(B, Hq, D) + proj_part_bytes(B, N) + vsp_attn_decode_workspace_bytes(B, Hq, D, max_len);
}

int vsp_attn_decode_proj(const vsp_tensor* q, const vsp_kv_cache* cache, const int32_t* seq_lens, int32_t max_len,
                         const vsp_tensor* wo, const vsp_tensor* bias, vsp_tensor* y, float scale, void* workspace,
                         size_t workspace_bytes, void* stream) {
    if (!q || !wo || !y) return VSP_ERR_NULL;
    if (q->ndim != 4) return VSP_ERR_NDIM;
    if (wo->ndim != 2 || y->ndim != 3 || (bias && bias->ndim != 1)) return VSP_ERR_NDIM;
    const int64_t B = q->shape[0], Hq = q->shape[1], D = q->shape[3];
    const int64_t K = Hq * D, N = wo->shape[0];
    if (wo->shape[1] != K || y->shape[0] != B || y->shape[1] != 1 || y->shape[2] != N) return VSP_ERR_SHAPE;
    if (bias && bias->shape[0] != N) return VSP_ERR_SHAPE;
    if (wo->dtype != q->dtype || y->dtype != q->dtype || (bias && bias->dtype != q->dtype)) return VSP_ERR_DTYPE;
    if (wo->stride[1] != 1 || y->stride[2] != 1 || (bias && bias->stride[0] != 1)) return VSP_ERR_STRIDE;
    const int esz = q->dtype == VSP_F32 ? 4 : 2;
    if (N > 0 && B > 0) {
        if (!wo->data || !y->data || (bias && !bias->data)) return VSP_ERR_NULL;
        if (!is_aligned16(wo->data) || (wo->stride[0] * esz) % 16) return VSP_ERR_ALIGN;
    }
    if (B <= 0 || Hq <= 0 || D <= 0) {
        // shapes the attention step rejects are reported by it (it launches nothing for them); an empty batch has
        // nothing to project
        vsp_tensor none = *q;
        return decode_impl(q, cache, seq_lens, max_len, &none, scale, workspace, workspace_bytes, false, stream);
    }
    if (B > INT32_MAX || N > INT32_MAX || K > INT32_MAX) return VSP_ERR_ARG;  // the projection kernels index with 32 bits
    // the attention step writes the merged heads x [B][Hq][D] (= [B][K]) to the head of the workspace
    const size_t pb_bytes = proj_part_bytes(B, N);
    const size_t xb = proj_x_bytes(B, Hq, D) + pb_bytes;
    if (!workspace || workspace_bytes < xb) return VSP_ERR_WORKSPACE;
    if (!is_aligned16(workspace)) return VSP_ERR_ALIGN;
    vsp_tensor x = *q;
    x.data = workspace;
    x.stride[0] = K;
    x.stride[1] = D;
    x.stride[2] = D;
    x.stride[3] = 1;
    int rc = decode_impl(q, cache, seq_lens, max_len, &x, scale, (char*)workspace + xb, workspace_bytes - xb, false, stream);
    if (rc != VSP_OK || N == 0) return rc;
    hipStream_t st = (hipStream_t)stream;
    if (q->dtype == VSP_F32) {
        hipLaunchKernelGGL(proj_f32_kernel, dim3((unsigned)ceil_div(N, kWaves)), dim3(256), 0, st, (const float*)x.data,
                           (const float*)wo->data, wo->stride[0], bias ? (const float*)bias->data : nullptr,
                           (float*)y->data, y->stride[0], (int)B, (int)N, (int)K);
    } else {
        // K = Hq * D with D 64 or 128 (the bf16 attention kernels' head sizes): a whole number of 32-wide slices
        if (B <= 16) {
            hipLaunchKernelGGL(proj_bf16_small_kernel, dim3((unsigned)ceil_div(N, 16)), dim3(512), 0, st, (const uint16_t*)x.data,
                               (const uint16_t*)wo->data, wo->stride[0], bias ? (const uint16_t*)bias->data : nullptr,
                               (uint16_t*)y->data, y->stride[0], (int)B, (int)N, (int)K);
            return check_launch();
        }
        const int KS = proj_split(K);
        float* part = (float*)((char*)workspace + proj_x_bytes(B, Hq, D));
        const dim3 grid((unsigned)ceil_div(N, kProjCols), (unsigned)KS);
        const uint16_t* px = (const uint16_t*)x.data;
        const uint16_t* pw = (const uint16_t*)wo->data;
        for (int64_t m0 = 0; m0 < B; m0 += 64) {  // 64 batch rows share a pass over W
            const int64_t rows = B - m0;
            if (rows <= 16)
                hipLaunchKernelGGL(proj_bf16_partial_kernel<1>, grid, dim3(kProjThreads), 0, st, px, pw, wo->stride[0], part, (int)m0, (int)B,
                                   (int)N, (int)K, (int)(K / KS));
            else if (rows <= 32)
                hipLaunchKernelGGL(proj_bf16_partial_kernel<2>, grid, dim3(kProjThreads), 0, st, px, pw, wo->stride[0], part, (int)m0, (int)B,
                                   (int)N, (int)K, (int)(K / KS));
            else
                hipLaunchKernelGGL(proj_bf16_partial_kernel<4>, grid, dim3(kProjThreads), 0, st, px, pw, wo->stride[0], part, (int)m0, (int)B,
                                   (int)N, (int)K, (int)(K / KS));
        }
        rc = check_launch();
        if (rc != VSP_OK) return rc;
        const uint16_t* pbias = bias ? (const uint16_t*)bias->data : nullptr;
        if (N % 4 == 0)
            hipLaunchKernelGGL(proj_reduce_kernel<4>, dim3((unsigned)ceil_div(B * N, 1024)), dim3(256), 0, st, part, pbias,
                               (uint16_t*)y->data, y->stride[0], (int)B, (int)N, KS);
        else
            hipLaunchKernelGGL(proj_reduce_kernel<1>, dim3((unsigned)ceil_div(B * N, 256)), dim3(256), 0, st, part, pbias,
                               (uint16_t*)y->data, y->stride[0], (int)B, (int)N, KS);
    }
    return check_launch();
}

}  // extern "C"
