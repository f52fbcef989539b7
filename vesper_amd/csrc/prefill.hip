// Causal GQA flash-attention prefill for gfx950.
//
// Replaces flash_attention_hip_dispatch (include/vesper/ops/flash_attention.h:74-78,
// src/ops/hip/flash_attention.hip:305-331) with repeat_kv (src/ops/attention_ops.cpp:30-57) folded
// into the head indexing.  Same mathematics as the reference's CPU forward
// (src/ops/flash_attention.cpp:218-364): online softmax over key tiles, O = acc / l,
// LSE = m + log l; the arithmetic is bf16 MFMA with fp32 accumulation (or fp32 MFMA for fp32 inputs).
//
// bf16 kernel.  A workgroup of 4 wavefronts owns 128 consecutive queries of one (batch, query head);
// each wavefront owns 32 of them.  Key tiles of 64 go through LDS (register-staged prefetch of the
// next tile while the current one is consumed).  Both GEMMs are computed transposed so that the
// softmax statistics of a query live in one lane (and its partner 32 lanes away):
//   S^T[key][q] = K[key][:] . Q^T[:][q]     32x32x16 MFMA, A = K rows from LDS, B = Q^T held in registers
//   O^T[d][q]  += V^T[d][key] . P^T[key][q]  A = V^T read from the row-major V tile with the
//                                            transposing LDS read, B = P^T straight from the S^T registers
// The exponent uses a per-row reference maximum that is only raised (and the accumulators rescaled)
// when the true running maximum outgrows it by more than 2^8; the result is mathematically the same
// softmax, without a rescale per tile.  Key tiles entirely above the causal diagonal are skipped;
// the mask is evaluated only on tiles that straddle it.
#include <math.h>

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
    float scale_log2;  // |scale| * log2(e) for bf16; scale * log2(e) for fp32
};

constexpr int kBM = 128;       // queries per workgroup
constexpr int kBN = 64;        // keys per tile
constexpr float kRescaleThreshold = 8.0f;

typedef short s16x4_t __attribute__((ext_vector_type(4)));

__device__ inline uint2 lds_read_tr16_b64(const uint16_t* p) {
    s16x4_t v = __builtin_amdgcn_ds_read_tr16_b64_v4i16((s16x4_t __attribute__((address_space(3)))*)p);
    return __builtin_bit_cast(uint2, v);
}

__device__ inline uint32_t cvt_pk_bf16(float a, float b) {
    typedef float f32x2_t __attribute__((ext_vector_type(2)));
    typedef __bf16 bf16x2_t __attribute__((ext_vector_type(2)));
    f32x2_t v = {a, b};
    return __builtin_bit_cast(uint32_t, __builtin_convertvector(v, bf16x2_t));
}

// Reductions over the two half-waves (lane l and lane l ^ 32 hold the two halves of a query's keys).
__device__ inline float half_swap_max(float x) { return fmaxf(x, __shfl_xor(x, 32)); }
__device__ inline float half_swap_sum(float x) { return x + __shfl_xor(x, 32); }

template <int D>
__global__ void __launch_bounds__(256, 2) prefill_bf16_kernel(PrefillArgs a) {
    constexpr int KS = D / 16;      // k-steps of S^T over the head dim
    constexpr int DB = D / 32;      // 32-row tiles of O^T
    constexpr int KPITCH = D + 8;   // LDS row pitch of the K tile (elements): rows shift by 16 B -> ds_read_b128 conflict-free
    constexpr int VPITCH = D + 32;  // V tile: rows shift by 64 B -> the 4-row transposing reads are conflict-free
    constexpr int CPR = D / 8;      // 16-byte chunks per row
    constexpr int NLD = kBN * CPR / 256;  // chunks per thread per tile

    __shared__ __attribute__((aligned(16))) uint16_t sK[kBN * KPITCH];
    __shared__ __attribute__((aligned(16))) uint16_t sV[kBN * VPITCH];

    // heaviest query tiles first (causal work grows with the tile index); heads of one kv group adjacent
    const int bid = blockIdx.x;
    const int qt = a.n_qtiles - 1 - bid / (a.B * a.Hq);
    const int bh = bid % (a.B * a.Hq);
    const int b = bh / a.Hq, hq = bh % a.Hq, kvh = hq / a.n_rep;

    const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
    const int ql = lane & 31, h = lane >> 5;
    const int q0 = qt * kBM + wave * 32;   // first query of this wavefront
    const int off = a.L - a.T;             // key j visible to query t iff j <= t + off
    const int qrow = min(q0 + ql, a.T - 1);

    const uint16_t* Qp = (const uint16_t*)a.q + (int64_t)b * a.sq[0] + (int64_t)hq * a.sq[1];
    const uint16_t* Kp = (const uint16_t*)a.k + (int64_t)b * a.sk[0] + (int64_t)kvh * a.sk[1];
    const uint16_t* Vp = (const uint16_t*)a.v + (int64_t)b * a.sv[0] + (int64_t)kvh * a.sv[1];

    // Q^T operands (B of S^T): column ql, contraction slots d = 16*ks + 8*h + e
    bf16x8_t qf[KS];
#pragma unroll
    for (int ks = 0; ks < KS; ++ks)
    {
        uint4 w = *(const uint4*)(Qp + (int64_t)qrow * a.sq[2] + 16 * ks + 8 * h);
        if (a.negate_q) {
            w.x ^= 0x80008000u;
            w.y ^= 0x80008000u;
            w.z ^= 0x80008000u;
            w.w ^= 0x80008000u;
        }
        qf[ks] = __builtin_bit_cast(bf16x8_t, w);
    }

    // number of key tiles this workgroup / this wavefront needs
    const int wg_qmax = min(qt * kBM + kBM - 1, a.T - 1);
    const int kv_end_wg = a.causal ? min(a.L, wg_qmax + off + 1) : a.L;
    const int n_tiles = (kv_end_wg + kBN - 1) / kBN;
    const int wave_qmax = min(q0 + 31, a.T - 1);
    const int kv_end_wave = a.causal ? min(a.L, wave_qmax + off + 1) : a.L;  // may be <= 0 for waves past T

    f32x16_t acc[DB];
#pragma unroll
    for (int i = 0; i < DB; ++i)
#pragma unroll
        for (int j = 0; j < 16; ++j) acc[i][j] = 0.f;
    float m_ref = -INFINITY;  // reference maximum used in the exponent (log2 domain, scaled)
    float l = 0.f;            // this lane's share of the row sum

    uint4 stage_k[NLD], stage_v[NLD];
    auto load_tile = [&](int kt) {
#pragma unroll
        for (int i = 0; i < NLD; ++i) {
            const int id = tid + 256 * i, row = id / CPR, cc = id % CPR;
            const int key = kt * kBN + row;
            if (key < a.L) {
                stage_k[i] = *(const uint4*)(Kp + (int64_t)key * a.sk[2] + 8 * cc);
                stage_v[i] = *(const uint4*)(Vp + (int64_t)key * a.sv[2] + 8 * cc);
            } else {
                stage_k[i] = uint4{0, 0, 0, 0};
                stage_v[i] = uint4{0, 0, 0, 0};
            }
        }
    };
    auto store_tile = [&]() {
#pragma unroll
        for (int i = 0; i < NLD; ++i) {
            const int id = tid + 256 * i, row = id / CPR, cc = id % CPR;
            *(uint4*)(sK + row * KPITCH + 8 * cc) = stage_k[i];
            *(uint4*)(sV + row * VPITCH + 8 * cc) = stage_v[i];
        }
    };

    if (n_tiles > 0) load_tile(0);
    for (int kt = 0; kt < n_tiles; ++kt) {
        __syncthreads();  // everyone is done reading the previous tile
        store_tile();
        __syncthreads();
        if (kt + 1 < n_tiles) load_tile(kt + 1);  // in flight while this tile is consumed

        const int k0 = kt * kBN;
        if (k0 >= kv_end_wave) continue;  // tile entirely masked for this wavefront (uniform per wave)

        // ---- S^T = K . Q^T for the two 32-key halves of the tile
        f32x16_t s[2];
#pragma unroll
        for (int kb = 0; kb < 2; ++kb) {
#pragma unroll
            for (int j = 0; j < 16; ++j) s[kb][j] = 0.f;
            const uint16_t* kr = sK + (32 * kb + ql) * KPITCH + 8 * h;
#pragma unroll
            for (int ks = 0; ks < KS; ++ks) {
                bf16x8_t kf = __builtin_bit_cast(bf16x8_t, *(const uint4*)(kr + 16 * ks));
                s[kb] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(kf, qf[ks], s[kb], 0, 0, 0);
            }
        }
        // ---- mask (only tiles that straddle the diagonal or the end of the context)
        const int q_abs = q0 + ql + off;  // last visible key of this lane's query
        const bool need_mask = (a.causal && k0 + kBN - 1 > q0 + off) || (k0 + kBN > a.L);
        if (need_mask) {
            const int lim = a.causal ? min(q_abs, a.L - 1) : a.L - 1;
#pragma unroll
            for (int kb = 0; kb < 2; ++kb)
#pragma unroll
                for (int v = 0; v < 16; ++v) {
                    const int key = k0 + 32 * kb + 8 * (v >> 2) + 4 * h + (v & 3);
                    if (key > lim) s[kb][v] = -INFINITY;
                }
        }
        // ---- running maximum (raw scores; scale_log2 > 0 here, a negative scale was folded into Q)
        float mx = s[0][0];
#pragma unroll
        for (int kb = 0; kb < 2; ++kb)
#pragma unroll
            for (int v = 0; v < 16; ++v) mx = fmaxf(mx, s[kb][v]);
        mx = half_swap_max(mx) * a.scale_log2;
        if (__any(mx > m_ref + kRescaleThreshold)) {
            const float m_new = fmaxf(m_ref, mx);
            const float alpha = (m_new == -INFINITY) ? 1.f : __builtin_amdgcn_exp2f(m_ref - m_new);
            l *= alpha;
#pragma unroll
            for (int i = 0; i < DB; ++i)
#pragma unroll
                for (int j = 0; j < 16; ++j) acc[i][j] *= alpha;
            m_ref = m_new;
        }
        // ---- P^T = exp2(S^T * c - m_ref), packed to bf16 as the B operands of the PV MFMAs
        const float neg_m = (m_ref == -INFINITY) ? 0.f : -m_ref;
        uint32_t pw[4][4];
#pragma unroll
        for (int kb = 0; kb < 2; ++kb)
#pragma unroll
            for (int v = 0; v < 16; v += 2) {
                const float p0 = __builtin_amdgcn_exp2f(__builtin_fmaf(s[kb][v], a.scale_log2, neg_m));
                const float p1 = __builtin_amdgcn_exp2f(__builtin_fmaf(s[kb][v + 1], a.scale_log2, neg_m));
                l += p0 + p1;
                pw[2 * kb + (v >> 3)][(v & 7) >> 1] = cvt_pk_bf16(p0, p1);
            }
        // ---- O^T += V^T . P^T
#pragma unroll
        for (int j = 0; j < 4; ++j) {
            const bf16x8_t pf = __builtin_bit_cast(bf16x8_t, uint4{pw[j][0], pw[j][1], pw[j][2], pw[j][3]});
            // transposing read: a 16-lane group reads a 4(keys) x 16(d) patch; lane i of the group gets d = i.
            const uint16_t* vr = sV + (16 * j + 4 * h + ((lane & 15) >> 2)) * VPITCH + 16 * ((lane >> 4) & 1) + 4 * (lane & 3);
#pragma unroll
            for (int db = 0; db < DB; ++db) {
                const uint2 lo = lds_read_tr16_b64(vr + 32 * db);
                const uint2 hi = lds_read_tr16_b64(vr + 8 * VPITCH + 32 * db);
                const bf16x8_t vf = __builtin_bit_cast(bf16x8_t, uint4{lo.x, lo.y, hi.x, hi.y});
                acc[db] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(vf, pf, acc[db], 0, 0, 0);
            }
        }
    }

    // ---- epilogue: O = acc / l, LSE = (m_ref + log2 l) * ln 2
    l = half_swap_sum(l);
    const int qi = q0 + ql;
    if (qi < a.T) {
        const float inv_l = 1.0f / l;
        uint16_t* op = (uint16_t*)a.out + (int64_t)b * a.so[0] + (int64_t)hq * a.so[1] + (int64_t)qi * a.so[2];
#pragma unroll
        for (int db = 0; db < DB; ++db)
#pragma unroll
            for (int vq = 0; vq < 4; ++vq) {
                const int d = 32 * db + 8 * vq + 4 * h;
                uint2 w;
                w.x = (uint32_t)f32_to_bf16_bits(acc[db][4 * vq] * inv_l) | ((uint32_t)f32_to_bf16_bits(acc[db][4 * vq + 1] * inv_l) << 16);
                w.y = (uint32_t)f32_to_bf16_bits(acc[db][4 * vq + 2] * inv_l) | ((uint32_t)f32_to_bf16_bits(acc[db][4 * vq + 3] * inv_l) << 16);
                *(uint2*)(op + d) = w;
            }
        if (a.lse && h == 0)
            a.lse[(int64_t)b * a.sl[0] + (int64_t)hq * a.sl[1] + (int64_t)qi * a.sl[2]] = (m_ref + __builtin_amdgcn_logf(l)) * 0.6931471805599453f;
    }
}

// ---------------------------------------------------------------------------------------------
// fp32 kernel (fp32 inputs, fp32 MFMA 32x32x2, fp32 softmax): the precision the reference computes
// in.  One wavefront owns 32 queries, a workgroup 128; key tiles of 32 through LDS.
// ---------------------------------------------------------------------------------------------
template <int D>
__global__ void __launch_bounds__(256) prefill_f32_kernel(PrefillArgs a) {
    constexpr int BN = 32;
    constexpr int PITCH = D + 1;  // odd pitch: a column walk hits 32 different banks
    constexpr int DB = D / 32;
    __shared__ float sK[BN * PITCH];
    __shared__ float sV[BN * PITCH];

    const int bid = blockIdx.x;
    const int qt = a.n_qtiles - 1 - bid / (a.B * a.Hq);
    const int bh = bid % (a.B * a.Hq);
    const int b = bh / a.Hq, hq = bh % a.Hq, kvh = hq / a.n_rep;
    const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
    const int ql = lane & 31, h = lane >> 5;
    const int q0 = qt * kBM + wave * 32;
    const int off = a.L - a.T;
    const int qrow = min(q0 + ql, a.T - 1);

    const float* Qp = (const float*)a.q + (int64_t)b * a.sq[0] + (int64_t)hq * a.sq[1] + (int64_t)qrow * a.sq[2];
    const float* Kp = (const float*)a.k + (int64_t)b * a.sk[0] + (int64_t)kvh * a.sk[1];
    const float* Vp = (const float*)a.v + (int64_t)b * a.sv[0] + (int64_t)kvh * a.sv[1];

    // Q^T operands: column ql, contraction slot d = 2*ks + h
    float qf[D / 2];
#pragma unroll
    for (int ks = 0; ks < D / 2; ++ks) qf[ks] = Qp[2 * ks + h];

    const int wg_qmax = min(qt * kBM + kBM - 1, a.T - 1);
    const int kv_end_wg = a.causal ? min(a.L, wg_qmax + off + 1) : a.L;
    const int n_tiles = (kv_end_wg + BN - 1) / BN;
    const int wave_qmax = min(q0 + 31, a.T - 1);
    const int kv_end_wave = a.causal ? min(a.L, wave_qmax + off + 1) : a.L;

    f32x16_t acc[DB];
#pragma unroll
    for (int i = 0; i < DB; ++i)
#pragma unroll
        for (int j = 0; j < 16; ++j) acc[i][j] = 0.f;
    float m_run = -INFINITY, l = 0.f;

    for (int kt = 0; kt < n_tiles; ++kt) {
        __syncthreads();
        for (int id = tid; id < BN * D; id += 256) {
            const int row = id / D, col = id % D, key = kt * BN + row;
            sK[row * PITCH + col] = key < a.L ? Kp[(int64_t)key * a.sk[2] + col] : 0.f;
            sV[row * PITCH + col] = key < a.L ? Vp[(int64_t)key * a.sv[2] + col] : 0.f;
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
        const int lim = a.causal ? min(q0 + ql + off, a.L - 1) : a.L - 1;
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
        const float inv_l = 1.0f / l;
        float* op = (float*)a.out + (int64_t)b * a.so[0] + (int64_t)hq * a.so[1] + (int64_t)qi * a.so[2];
#pragma unroll
        for (int db = 0; db < DB; ++db)
#pragma unroll
            for (int v = 0; v < 16; ++v) op[32 * db + 8 * (v >> 2) + 4 * h + (v & 3)] = acc[db][v] * inv_l;
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

}  // namespace
}  // namespace vsp

using namespace vsp;

extern "C" int vsp_attn_prefill(const vsp_tensor* q, const vsp_tensor* k, const vsp_tensor* v, vsp_tensor* out,
                                vsp_tensor* lse, float scale, int is_causal, float dropout_p, int training,
                                void* stream) {
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
    if (D != 64 && D != 128) return VSP_ERR_UNSUPPORTED;
    if (L == 0) return VSP_ERR_SHAPE;  // softmax over an empty context is undefined
    if (!(fabsf(scale) > 0.0f) || !(fabsf(scale) < INFINITY)) return VSP_ERR_ARG;
    const int esz = q->dtype == VSP_F32 ? 4 : 2;
    int rc;
    if ((rc = check_tensor4(q, esz)) != VSP_OK || (rc = check_tensor4(k, esz)) != VSP_OK ||
        (rc = check_tensor4(v, esz)) != VSP_OK || (rc = check_tensor4(out, esz)) != VSP_OK)
        return rc;
    if (lse && !lse->data) return VSP_ERR_NULL;
    if (T > INT32_MAX / 2 || L > INT32_MAX / 2) return VSP_ERR_ARG;

    PrefillArgs a;
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
    const int64_t blocks = (int64_t)a.n_qtiles * B * Hq;
    if (blocks > INT32_MAX) return VSP_ERR_ARG;
    hipStream_t st = (hipStream_t)stream;
    dim3 grid((unsigned)blocks), block(256);
    if (q->dtype == VSP_BF16) {
        if (D == 128) hipLaunchKernelGGL(prefill_bf16_kernel<128>, grid, block, 0, st, a);
        else hipLaunchKernelGGL(prefill_bf16_kernel<64>, grid, block, 0, st, a);
    } else {
        if (D == 128) hipLaunchKernelGGL(prefill_f32_kernel<128>, grid, block, 0, st, a);
        else hipLaunchKernelGGL(prefill_f32_kernel<64>, grid, block, 0, st, a);
    }
    return check_launch();
}
