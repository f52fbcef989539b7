// Flash-attention backward for gfx950.
//
// Replaces flash_attention_backward_hip_dispatch (include/vesper/ops/flash_attention.h:80-92,
// src/ops/hip/flash_attention.hip:183-299) with the mathematics of the reference's CPU backward
// (src/ops/flash_attention.cpp:366-482): with P = exp(scale q.k - lse) recomputed from the forward's
// log-sum-exp,  Di = rowsum(dO * O),  dV = P^T dO,  dP = dO V^T,  dS = P * (dP - Di),
// dQ = scale dS K,  dK = scale dS^T Q.  Differences from the reference's HIP kernel: matrix cores
// instead of scalar FMAs, D in {64, 128} (and 32 for fp32 operands), grouped-query heads folded in
// (dK / dV of a kv head sum over its query heads, the gradient of ops::repeat_kv), and no atomics:
// dQ is produced by one pass that owns query rows, dK / dV by a second pass that owns key rows, so the
// result is bitwise reproducible (the reference accumulates dQ with atomicAdd).  Both passes compute dS; with the
// larger of the two workspaces (bf16 operands) the dK / dV pass runs first and leaves dS behind as bf16 tiles, and dQ is
// one product over those tiles (bwd_rowstats_bf16_kernel, bwd_dkdv_bf16_kernel<D, false, true>, bwd_dq_stream_kernel).
//
// fp32 operands: fp32 MFMA (32x32x2) throughout.  bf16 operands: bf16 MFMA (32x32x16) with fp32 accumulation
// and fp32 softmax algebra; P and dS are rounded to bf16 (round-to-nearest-even) between the products, as P is
// in the forward kernel, and the gradients are rounded to bf16 on store.  The fp32 kernels use plain padded LDS
// tiles filled by ordinary loads; the bf16 kernels use dense XOR-swizzled tiles filled by direct-to-LDS loads
// through a ring of slots (see the comments at bwd_dq_bf16_kernel and bwd_dkdv_bf16_kernel).
#include <math.h>

#include <type_traits>

#include "vsp_common.hpp"

namespace vsp {
namespace {

struct BwdArgs {
    const void *dout, *q, *k, *v, *out;
    const float* lse;
    void *dq, *dk, *dv;
    float* delta;                          // workspace: Di [B][Hq][N]
    float* lse2;                           // workspace: lse * log2(e) [B][Hq][N] (bf16 kernels)
    int64_t s_do[3], s_q[3], s_k[3], s_v[3], s_o[3], s_l[3], s_dq[3], s_dk[3], s_dv[3];
    int32_t B, Hq, Hkv, n_rep, N;
    int32_t causal;
    float scale;
    int64_t lo_q, lo_kv;                   // split operands: elements from a hi plane to its lo plane (q-shaped, kv-shaped)
    int32_t D_true;                        // fp32 kernels: the tensors' head_dim (<= the kernel's tile width; columns past it are zero)
    // bf16, one-pass dS: the dK / dV pass leaves every dS tile (32 keys x 32 queries, bf16, [key][query], 2 KB) in the
    // workspace at [b][hq][query tile][key tile], and dQ is one product over those tiles
    uint16_t* ds_tiles;
    int32_t n_qt32, n_kt32;                // query tiles per head, key tiles per head (an even number: key blocks come in pairs)
};

template <typename T>
__device__ inline float ld(const T* p);
template <>
__device__ inline float ld<float>(const float* p) { return *p; }
template <>
__device__ inline float ld<uint16_t>(const uint16_t* p) { return bf16_bits_to_f32(*p); }
template <typename T>
__device__ inline void st(T* p, float f);
template <>
__device__ inline void st<float>(float* p, float f) { *p = f; }
template <>
__device__ inline void st<uint16_t>(uint16_t* p, float f) { *p = f32_to_bf16_bits(f); }

// Di[b][h][i] = sum_d dO[i][d] * O[i][d]   (src/ops/flash_attention.cpp:416-423); one wavefront per row.
template <typename T>
__global__ void __launch_bounds__(256) bwd_delta_kernel(BwdArgs a, int D) {
    const int lane = threadIdx.x & 63;
    const int64_t row = (int64_t)blockIdx.x * 4 + (threadIdx.x >> 6);
    const int64_t rows = (int64_t)a.B * a.Hq * a.N;
    if (row >= rows) return;
    const int i = (int)(row % a.N);
    const int64_t bh = row / a.N;
    const int h = (int)(bh % a.Hq), b = (int)(bh / a.Hq);
    const T* po = (const T*)a.out + (int64_t)b * a.s_o[0] + (int64_t)h * a.s_o[1] + (int64_t)i * a.s_o[2];
    const T* pd = (const T*)a.dout + (int64_t)b * a.s_do[0] + (int64_t)h * a.s_do[1] + (int64_t)i * a.s_do[2];
    float s = 0.f;
    for (int d = lane; d < D; d += 64) s += ld<T>(pd + d) * ld<T>(po + d);
#pragma unroll
    for (int o = 32; o > 0; o >>= 1) s += __shfl_xor(s, o);
    if (lane == 0) a.delta[row] = s;
}

// bf16 operands: Di as above and lse * log2(e), the two per-row constants of the dK / dV pass, when no dQ pass has
// run before it.  D / 8 lanes per row, 16 bytes of O and dO each.
template <int D>
__global__ void __launch_bounds__(256) bwd_rowstats_bf16_kernel(BwdArgs a) {
    constexpr int LPR = D / 8, RPB = 256 / LPR;
    const int64_t row = (int64_t)blockIdx.x * RPB + threadIdx.x / LPR;
    const int piece = threadIdx.x % LPR;
    const int64_t rows = (int64_t)a.B * a.Hq * a.N;
    const int64_t rr = row < rows ? row : rows - 1;
    const int i = (int)(rr % a.N);
    const int64_t bh = rr / a.N;
    const int h = (int)(bh % a.Hq), b = (int)(bh / a.Hq);
    const uint4 wo = *(const uint4*)((const uint16_t*)a.out + (int64_t)b * a.s_o[0] + (int64_t)h * a.s_o[1] + (int64_t)i * a.s_o[2] + 8 * piece);
    const uint4 wd = *(const uint4*)((const uint16_t*)a.dout + (int64_t)b * a.s_do[0] + (int64_t)h * a.s_do[1] + (int64_t)i * a.s_do[2] + 8 * piece);
    const uint32_t o4[4] = {wo.x, wo.y, wo.z, wo.w}, d4[4] = {wd.x, wd.y, wd.z, wd.w};
    float s = 0.f;
#pragma unroll
    for (int j = 0; j < 4; ++j) {
        s += __uint_as_float(o4[j] << 16) * __uint_as_float(d4[j] << 16);
        s += __uint_as_float(o4[j] & 0xffff0000u) * __uint_as_float(d4[j] & 0xffff0000u);
    }
#pragma unroll
    for (int o = LPR / 2; o > 0; o >>= 1) s += __shfl_xor(s, o);
    if (row < rows && piece == 0) {
        a.delta[row] = s;
        a.lse2[row] = 1.4426950408889634f * a.lse[(int64_t)b * a.s_l[0] + (int64_t)h * a.s_l[1] + (int64_t)i * a.s_l[2]];
    }
}

constexpr int kBQ = 128;  // rows (queries or keys) per workgroup, 32 per wavefront
constexpr int kBT = 32;   // rows of the streamed tile

// ---- dQ: a wavefront owns 32 query rows and walks the key tiles (the forward's structure) ----
//   S^T[key][q]  = K . Q^T      A = K tile (LDS), B = Q^T (registers)
//   dP^T[key][q] = V . dO^T     A = V tile (LDS), B = dO^T (registers)
//   dS^T = exp(scale S^T - lse[q]) * (dP^T - Di[q])        a lane owns one query column: lse, Di are per lane
//   dQ^T[d][q]  += K^T . dS^T   A = K^T (the same tile read column-wise), B = dS^T straight from registers
template <int D, typename T>
__global__ void __launch_bounds__(256) bwd_dq_kernel(BwdArgs a) {
    constexpr int PITCH = D + 1;
    constexpr int DB = D / 32;
    __shared__ float sK[kBT * PITCH];
    __shared__ float sV[kBT * PITCH];
    const int n_qtiles = (a.N + kBQ - 1) / kBQ;
    const int bid = blockIdx.x;
    const int qt = n_qtiles - 1 - bid / (a.B * a.Hq);
    const int bh = xcd_grouped_head(bid % (a.B * a.Hq), a.B * a.Hkv, a.n_rep);  // a kv group's query heads share one XCD's L2
    const int b = bh / a.Hq, hq = bh % a.Hq, kvh = hq / a.n_rep;
    const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
    const int ql = lane & 31, h = lane >> 5;
    const int q0 = qt * kBQ + wave * 32;
    const int qi = q0 + ql;
    const int qrow = min(qi, a.N - 1);

    const T* Qp = (const T*)a.q + (int64_t)b * a.s_q[0] + (int64_t)hq * a.s_q[1] + (int64_t)qrow * a.s_q[2];
    const T* Op = (const T*)a.dout + (int64_t)b * a.s_do[0] + (int64_t)hq * a.s_do[1] + (int64_t)qrow * a.s_do[2];
    const T* Kp = (const T*)a.k + (int64_t)b * a.s_k[0] + (int64_t)kvh * a.s_k[1];
    const T* Vp = (const T*)a.v + (int64_t)b * a.s_v[0] + (int64_t)kvh * a.s_v[1];
    float qf[D / 2], dof[D / 2];
    const int Dt = a.D_true;  // the reference's backward takes any head_dim (src/ops/flash_attention.cpp:366-482)
#pragma unroll
    for (int ks = 0; ks < D / 2; ++ks) {
        qf[ks] = 2 * ks + h < Dt ? ld<T>(Qp + 2 * ks + h) : 0.f;
        dof[ks] = 2 * ks + h < Dt ? ld<T>(Op + 2 * ks + h) : 0.f;
    }
    const float lse_q = a.lse[(int64_t)b * a.s_l[0] + (int64_t)hq * a.s_l[1] + (int64_t)qrow * a.s_l[2]];
    const float di_q = a.delta[((int64_t)b * a.Hq + hq) * a.N + qrow];

    const int wg_qmax = min(qt * kBQ + kBQ - 1, a.N - 1);
    const int kv_end_wg = a.causal ? min(a.N, wg_qmax + 1) : a.N;
    const int n_tiles = (kv_end_wg + kBT - 1) / kBT;
    const int kv_end_wave = (q0 < a.N) ? (a.causal ? min(a.N, min(q0 + 31, a.N - 1) + 1) : a.N) : 0;

    f32x16_t acc[DB];
#pragma unroll
    for (int i = 0; i < DB; ++i)
#pragma unroll
        for (int j = 0; j < 16; ++j) acc[i][j] = 0.f;

    for (int kt = 0; kt < n_tiles; ++kt) {
        __syncthreads();
        for (int id = tid; id < kBT * D; id += 256) {
            const int row = id / D, col = id % D, key = kt * kBT + row;
            const bool ok = key < a.N && col < Dt;
            sK[row * PITCH + col] = ok ? ld<T>(Kp + (int64_t)key * a.s_k[2] + col) : 0.f;
            sV[row * PITCH + col] = ok ? ld<T>(Vp + (int64_t)key * a.s_v[2] + col) : 0.f;
        }
        __syncthreads();
        const int k0 = kt * kBT;
        if (k0 >= kv_end_wave) continue;
        f32x16_t s, dp;
#pragma unroll
        for (int j = 0; j < 16; ++j) s[j] = dp[j] = 0.f;
#pragma unroll
        for (int ks = 0; ks < D / 2; ++ks) {
            s = __builtin_amdgcn_mfma_f32_32x32x2f32(sK[ql * PITCH + 2 * ks + h], qf[ks], s, 0, 0, 0);
            dp = __builtin_amdgcn_mfma_f32_32x32x2f32(sV[ql * PITCH + 2 * ks + h], dof[ks], dp, 0, 0, 0);
        }
        const int lim = a.causal ? min(qi, a.N - 1) : a.N - 1;
        float ds[16];
#pragma unroll
        for (int v = 0; v < 16; ++v) {
            const int key = k0 + 8 * (v >> 2) + 4 * h + (v & 3);
            const float p = key <= lim ? expf(s[v] * a.scale - lse_q) : 0.f;
            ds[v] = p * (dp[v] - di_q);
        }
        // dQ^T += K^T . dS^T : contraction slot h of step v is key 8*(v/4) + 4*h + v%4, the key ds[v] belongs to
#pragma unroll
        for (int v = 0; v < 16; ++v) {
            const int krow = 8 * (v >> 2) + 4 * h + (v & 3);
#pragma unroll
            for (int db = 0; db < DB; ++db)
                acc[db] = __builtin_amdgcn_mfma_f32_32x32x2f32(sK[krow * PITCH + 32 * db + ql], ds[v], acc[db], 0, 0, 0);
        }
    }
    if (qi < a.N) {
        T* op = (T*)a.dq + (int64_t)b * a.s_dq[0] + (int64_t)hq * a.s_dq[1] + (int64_t)qi * a.s_dq[2];
#pragma unroll
        for (int db = 0; db < DB; ++db)
#pragma unroll
            for (int v = 0; v < 16; ++v) {
                const int d = 32 * db + 8 * (v >> 2) + 4 * h + (v & 3);
                if (d < Dt) st<T>(op + d, a.scale * acc[db][v]);
            }
    }
}

// ---- dK, dV: a wavefront owns 32 key rows of one kv head and walks the query heads of the group and their
// query tiles (the forward's structure with the roles of queries and keys exchanged) ----
//   S[q][key]  = Q . K^T        A = Q tile (LDS), B = K^T (registers);  a lane owns one key column
//   dP[q][key] = dO . V^T       A = dO tile (LDS), B = V^T (registers)
//   P = exp(scale S - lse[q]),  dS = P * (dP - Di[q])      lse, Di per row: read from LDS
//   dV^T[d][key] += dO^T . P    A = dO^T (tile read column-wise), B = P from registers
//   dK^T[d][key] += Q^T . dS    A = Q^T, B = dS
template <int D, typename T>
__global__ void __launch_bounds__(256) bwd_dkdv_kernel(BwdArgs a) {
    constexpr int PITCH = D + 1;
    constexpr int DB = D / 32;
    __shared__ float sQ[kBT * PITCH];
    __shared__ float sO[kBT * PITCH];
    __shared__ float sL[kBT], sD[kBT];
    const int n_ktiles = (a.N + kBQ - 1) / kBQ;
    const int bid = blockIdx.x;
    const int kt = bid / (a.B * a.Hkv);  // causal: early key tiles see the most queries -> dispatched first
    const int bh = bid % (a.B * a.Hkv);
    const int b = bh / a.Hkv, kvh = bh % a.Hkv;
    const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
    const int kl = lane & 31, h = lane >> 5;
    const int key0 = kt * kBQ + wave * 32;
    const int ki = key0 + kl;
    const int krow = min(ki, a.N - 1);
    (void)n_ktiles;

    const T* Kp = (const T*)a.k + (int64_t)b * a.s_k[0] + (int64_t)kvh * a.s_k[1] + (int64_t)krow * a.s_k[2];
    const T* Vp = (const T*)a.v + (int64_t)b * a.s_v[0] + (int64_t)kvh * a.s_v[1] + (int64_t)krow * a.s_v[2];
    float kf[D / 2], vf[D / 2];
    const int Dt = a.D_true;
#pragma unroll
    for (int ks = 0; ks < D / 2; ++ks) {
        kf[ks] = 2 * ks + h < Dt ? ld<T>(Kp + 2 * ks + h) : 0.f;
        vf[ks] = 2 * ks + h < Dt ? ld<T>(Vp + 2 * ks + h) : 0.f;
    }
    f32x16_t acck[DB], accv[DB];
#pragma unroll
    for (int i = 0; i < DB; ++i)
#pragma unroll
        for (int j = 0; j < 16; ++j) acck[i][j] = accv[i][j] = 0.f;

    // query tiles that can see any key of this workgroup / of this wavefront
    const int wg_kmin = kt * kBQ;
    const int qt_begin_wg = a.causal ? wg_kmin / kBT : 0;
    const int n_qt = (a.N + kBT - 1) / kBT;
    const int q_begin_wave = a.causal ? key0 : 0;

    for (int r = 0; r < a.n_rep; ++r) {
        const int hq = kvh * a.n_rep + r;
        const T* Qp = (const T*)a.q + (int64_t)b * a.s_q[0] + (int64_t)hq * a.s_q[1];
        const T* Op = (const T*)a.dout + (int64_t)b * a.s_do[0] + (int64_t)hq * a.s_do[1];
        const float* Lp = a.lse + (int64_t)b * a.s_l[0] + (int64_t)hq * a.s_l[1];
        const float* Dp = a.delta + ((int64_t)b * a.Hq + hq) * a.N;
        for (int qt = qt_begin_wg; qt < n_qt; ++qt) {
            __syncthreads();
            for (int id = tid; id < kBT * D; id += 256) {
                const int row = id / D, col = id % D, qi = qt * kBT + row;
                const bool ok = qi < a.N && col < Dt;
                sQ[row * PITCH + col] = ok ? ld<T>(Qp + (int64_t)qi * a.s_q[2] + col) : 0.f;
                sO[row * PITCH + col] = ok ? ld<T>(Op + (int64_t)qi * a.s_do[2] + col) : 0.f;
            }
            if (tid < kBT) {
                const int qi = qt * kBT + tid;
                sL[tid] = qi < a.N ? Lp[(int64_t)qi * a.s_l[2]] : 0.f;
                sD[tid] = qi < a.N ? Dp[qi] : 0.f;
            }
            __syncthreads();
            const int qb = qt * kBT;
            if (key0 >= a.N || qb + kBT - 1 < q_begin_wave) continue;  // no query of this tile sees these keys
            f32x16_t s, dp;
#pragma unroll
            for (int j = 0; j < 16; ++j) s[j] = dp[j] = 0.f;
#pragma unroll
            for (int ks = 0; ks < D / 2; ++ks) {
                s = __builtin_amdgcn_mfma_f32_32x32x2f32(sQ[kl * PITCH + 2 * ks + h], kf[ks], s, 0, 0, 0);
                dp = __builtin_amdgcn_mfma_f32_32x32x2f32(sO[kl * PITCH + 2 * ks + h], vf[ks], dp, 0, 0, 0);
            }
            float p[16], ds[16];
#pragma unroll
            for (int v = 0; v < 16; ++v) {
                const int row = 8 * (v >> 2) + 4 * h + (v & 3);
                const int qi = qb + row;
                const bool ok = qi < a.N && ki < a.N && (!a.causal || ki <= qi);
                p[v] = ok ? expf(s[v] * a.scale - sL[row]) : 0.f;
                ds[v] = p[v] * (dp[v] - sD[row]);
            }
#pragma unroll
            for (int v = 0; v < 16; ++v) {
                const int row = 8 * (v >> 2) + 4 * h + (v & 3);
#pragma unroll
                for (int db = 0; db < DB; ++db) {
                    accv[db] = __builtin_amdgcn_mfma_f32_32x32x2f32(sO[row * PITCH + 32 * db + kl], p[v], accv[db], 0, 0, 0);
                    acck[db] = __builtin_amdgcn_mfma_f32_32x32x2f32(sQ[row * PITCH + 32 * db + kl], ds[v], acck[db], 0, 0, 0);
                }
            }
        }
    }
    if (ki < a.N) {
        T* pk = (T*)a.dk + (int64_t)b * a.s_dk[0] + (int64_t)kvh * a.s_dk[1] + (int64_t)ki * a.s_dk[2];
        T* pv = (T*)a.dv + (int64_t)b * a.s_dv[0] + (int64_t)kvh * a.s_dv[1] + (int64_t)ki * a.s_dv[2];
#pragma unroll
        for (int db = 0; db < DB; ++db)
#pragma unroll
            for (int v = 0; v < 16; ++v) {
                const int d = 32 * db + 8 * (v >> 2) + 4 * h + (v & 3);
                if (d < Dt) {
                    st<T>(pk + d, a.scale * acck[db][v]);
                    st<T>(pv + d, accv[db][v]);
                }
            }
    }
}

// =============================================================================================
// bf16 operands: the same two passes on bf16 matrix cores (v_mfma_f32_32x32x16_bf16), fp32 accumulation and
// fp32 softmax algebra.  Tiles are bf16 in LDS with a padded pitch; the operand that a product contracts
// over rows (K^T, Q^T, dO^T) is fetched with the transposing LDS read, as V^T is in the forward kernel, and
// P / dS go from the accumulator registers into the next MFMA without leaving the lane.
// =============================================================================================
typedef short s16x4b_t __attribute__((ext_vector_type(4)));
typedef __attribute__((address_space(3))) void* lds_ptr_t;

// ---- a [32][D] bf16 tile in LDS ----
// Rows are dense (2 D bytes); the 16-byte chunks of a row are permuted by an XOR that depends on the row, chosen
// so that both access patterns the kernels use are free of bank conflicts: 16 lanes reading the same chunk of
// 16 consecutive rows (the row-major MFMA operand), and a 4-row x 64-byte block (the transposing read).
template <int D>
__device__ inline int tile_swz(int row) {
    return D == 128 ? (((row & 3) << 2) | ((row >> 2) & 3)) : ((((row >> 1) & 1) << 2) | ((row >> 2) & 3));
}
template <int D>
__device__ inline int tile_off(int row, int chunk) { return row * (2 * D) + ((chunk ^ tile_swz<D>(row)) << 4); }
// MFMA operand, contraction over the row's elements: lane (row r = lane % 32, half h) takes elements 16 ks + 8 h ..
template <int D>
__device__ inline bf16x8_t load_row(const uint16_t* tile, int ks, int lane) {
    return __builtin_bit_cast(bf16x8_t, *(const uint4*)((const char*)tile + tile_off<D>(lane & 31, 2 * ks + (lane >> 5))));
}
__device__ inline uint2 lds_tr16(const char* p) {
    s16x4b_t v = __builtin_amdgcn_ds_read_tr16_b64_v4i16((__attribute__((address_space(3))) s16x4b_t*)p);
    return __builtin_bit_cast(uint2, v);
}
// MFMA operand, contraction over the tile's rows: lane (column 32 db + lane % 32, half h) takes, as slot e of
// k-step j, row 16 j + 8 (e / 4) + 4 h + e % 4 - the row that accumulator register 8 j + e of this lane half
// belongs to, so a product's result feeds the next product without leaving the lane.
template <int D>
__device__ inline bf16x8_t load_transposed(const uint16_t* tile, int j, int db, int lane) {
    const int h = lane >> 5, row = 16 * j + 4 * h + ((lane & 15) >> 2);
    const int chunk = 4 * db + 2 * ((lane >> 4) & 1) + ((lane & 3) >> 1), o8 = (lane & 1) * 8;
    const uint2 lo = lds_tr16((const char*)tile + tile_off<D>(row, chunk) + o8);
    const uint2 hi = lds_tr16((const char*)tile + tile_off<D>(row + 8, chunk) + o8);
    return __builtin_bit_cast(bf16x8_t, uint4{lo.x, lo.y, hi.x, hi.y});
}
// Global -> LDS without passing through registers: a wavefront instruction moves 64 x 16 bytes to 1 KB of
// consecutive LDS, so the lane that lands on (row, physical chunk) fetches the row's chunk `physical ^ swizzle`.
// Rows at or past `valid_rows` fall outside the buffer descriptor's range and arrive as zeros.
template <int D>
struct TileDma {
    static constexpr int CPR = D / 8, RPG = 64 / CPR, NLD = CPR / 8;   // chunks per row, rows per instruction, instructions per wavefront
    uint32_t voff[NLD];
    __device__ inline void init(int64_t row_stride, int wave, int lane) {
#pragma unroll
        for (int i = 0; i < NLD; ++i) {
            const int r = (wave + 4 * i) * RPG + lane / CPR;
            voff[i] = (uint32_t)r * (uint32_t)row_stride * 2u + 16u * (uint32_t)((lane % CPR) ^ tile_swz<D>(r));
        }
    }
    __device__ inline void load(uint16_t* dst, const uint16_t* row0, int valid_rows, int64_t row_stride, int wave) const {
        __amdgpu_buffer_rsrc_t rs = __builtin_amdgcn_make_buffer_rsrc((void*)row0, 0, (int)((int64_t)max(valid_rows, 0) * row_stride * 2), 0x00020000);
#pragma unroll
        for (int i = 0; i < NLD; ++i)
            __builtin_amdgcn_raw_ptr_buffer_load_lds(rs, (lds_ptr_t)((char*)dst + (wave + 4 * i) * 1024), 16, voff[i], 0, 0, 0);
    }
};
// One float per lane (element stride `stride`) to 64 consecutive LDS words; lanes at or past `valid` bring zeros.
__device__ inline void row_dma(float* dst, const float* src, int valid, int64_t stride, int lane) {
    __amdgpu_buffer_rsrc_t rs = __builtin_amdgcn_make_buffer_rsrc((void*)src, 0, (int)((int64_t)valid * stride * 4), 0x00020000);
    __builtin_amdgcn_raw_ptr_buffer_load_lds(rs, (lds_ptr_t)dst, 4, (uint32_t)lane * (uint32_t)stride * 4u, 0, 0, 0);
}
__device__ inline void dma_wait_all() { asm volatile("s_waitcnt vmcnt(0)" ::: "memory"); }

constexpr float kLog2e = 1.4426950408889634f;

// two fp32 -> packed bf16x2 (lo = a, hi = b), round-to-nearest-even in one instruction
__device__ inline uint32_t cvt_pk_bf16(float a, float b) {
    typedef float f32x2_t __attribute__((ext_vector_type(2)));
    typedef __bf16 bf16x2_t __attribute__((ext_vector_type(2)));
    f32x2_t v = {a, b};
    return __builtin_bit_cast(uint32_t, __builtin_convertvector(v, bf16x2_t));
}

// four consecutive gradient elements from accumulator registers v .. v + 3: bf16 (rounded to nearest even) or fp32
template <bool F32>
__device__ inline void store4(void* base, int64_t elem, float f, const f32x16_t& acc, int v) {
    if constexpr (F32) {
        *(float4*)((float*)base + elem) = float4{f * acc[v], f * acc[v + 1], f * acc[v + 2], f * acc[v + 3]};
    } else {
        uint2 w;
        w.x = cvt_pk_bf16(f * acc[v], f * acc[v + 1]);
        w.y = cvt_pk_bf16(f * acc[v + 2], f * acc[v + 3]);
        *(uint2*)((uint16_t*)base + elem) = w;
    }
}

// ---- dQ (bf16): the structure of bwd_dq_kernel; K serves both as rows (S^T) and transposed (dQ^T) ----
// SPLIT: fp32 tensors taken as two bf16 terms each (x = hi + lo, planes written by bwd_split_kernel); every product
// is hi hi + hi lo + lo hi, dS is split the same way after the fp32 algebra, Di and lse * log2(e) come from the
// pre-pass, and dQ is stored as fp32.
template <int D, bool SPLIT = false>
__global__ void __launch_bounds__(256, SPLIT ? 1 : 2) bwd_dq_bf16_kernel(BwdArgs a) {
    constexpr int KS = D / 16, DB = D / 32;
    // One variable per ring slot: the compiler then knows that a read of one slot does not touch the slot a
    // direct-to-LDS load in flight is filling, and does not wait for that load.
    __shared__ __attribute__((aligned(1024))) uint16_t sK0[kBT * D], sK1[kBT * D];
    __shared__ __attribute__((aligned(1024))) uint16_t sV0[kBT * D], sV1[kBT * D];
    __shared__ __attribute__((aligned(1024))) uint16_t sKl0[SPLIT ? kBT * D : 8], sKl1[SPLIT ? kBT * D : 8];   // the lo planes' tiles
    __shared__ __attribute__((aligned(1024))) uint16_t sVl0[SPLIT ? kBT * D : 8], sVl1[SPLIT ? kBT * D : 8];
    const int n_qtiles = (a.N + kBQ - 1) / kBQ;
    const int bid = blockIdx.x;
    const int qt = n_qtiles - 1 - bid / (a.B * a.Hq);
    const int bh = xcd_grouped_head(bid % (a.B * a.Hq), a.B * a.Hkv, a.n_rep);  // a kv group's query heads share one XCD's L2
    const int b = bh / a.Hq, hq = bh % a.Hq, kvh = hq / a.n_rep;
    const int tid = threadIdx.x, lane = tid & 63, wave = __builtin_amdgcn_readfirstlane(tid >> 6);
    const int ql = lane & 31, h = lane >> 5;
    const int q0 = qt * kBQ + wave * 32;
    const int qi = q0 + ql;
    const int qrow = min(qi, a.N - 1);

    const uint16_t* Qp = (const uint16_t*)a.q + (int64_t)b * a.s_q[0] + (int64_t)hq * a.s_q[1] + (int64_t)qrow * a.s_q[2];
    const uint16_t* Op = (const uint16_t*)a.dout + (int64_t)b * a.s_do[0] + (int64_t)hq * a.s_do[1] + (int64_t)qrow * a.s_do[2];
    const uint16_t* Kp = (const uint16_t*)a.k + (int64_t)b * a.s_k[0] + (int64_t)kvh * a.s_k[1];
    const uint16_t* Vp = (const uint16_t*)a.v + (int64_t)b * a.s_v[0] + (int64_t)kvh * a.s_v[1];
    bf16x8_t qf[KS], dof[KS], qfl[SPLIT ? KS : 1], dofl[SPLIT ? KS : 1];
#pragma unroll
    for (int ks = 0; ks < KS; ++ks) {
        qf[ks] = __builtin_bit_cast(bf16x8_t, *(const uint4*)(Qp + 16 * ks + 8 * h));
        dof[ks] = __builtin_bit_cast(bf16x8_t, *(const uint4*)(Op + 16 * ks + 8 * h));
        if constexpr (SPLIT) {
            qfl[ks] = __builtin_bit_cast(bf16x8_t, *(const uint4*)(Qp + a.lo_q + 16 * ks + 8 * h));
            dofl[ks] = __builtin_bit_cast(bf16x8_t, *(const uint4*)(Op + a.lo_q + 16 * ks + 8 * h));
        }
    }
    // Di = rowsum(dO * O) of this lane's query: each lane holds half of the row of dO (the operand above) and reads the
    // same half of O; the two halves meet across lane ^ 32.  Every query row belongs to exactly one wavefront of this
    // launch, which also leaves Di and lse * log2(e) in the workspace for the dK/dV pass that follows.
    float di_q = 0.f;
    if constexpr (SPLIT) {
        di_q = a.delta[((int64_t)b * a.Hq + hq) * a.N + qrow];
    } else {
        const uint16_t* Orow = (const uint16_t*)a.out + (int64_t)b * a.s_o[0] + (int64_t)hq * a.s_o[1] + (int64_t)qrow * a.s_o[2];
#pragma unroll
        for (int ks = 0; ks < KS; ++ks) {
            const uint4 wo = *(const uint4*)(Orow + 16 * ks + 8 * h);
            const uint4 wd = __builtin_bit_cast(uint4, dof[ks]);
            const uint32_t o4[4] = {wo.x, wo.y, wo.z, wo.w}, d4[4] = {wd.x, wd.y, wd.z, wd.w};
#pragma unroll
            for (int j = 0; j < 4; ++j) {
                di_q += __uint_as_float(o4[j] << 16) * __uint_as_float(d4[j] << 16);
                di_q += __uint_as_float(o4[j] & 0xffff0000u) * __uint_as_float(d4[j] & 0xffff0000u);
            }
        }
        di_q += __shfl_xor(di_q, 32);
    }
    const float lse_q = SPLIT ? a.lse2[((int64_t)b * a.Hq + hq) * a.N + qrow]
                              : kLog2e * a.lse[(int64_t)b * a.s_l[0] + (int64_t)hq * a.s_l[1] + (int64_t)qrow * a.s_l[2]];
    if (!SPLIT && h == 0 && qi < a.N) {
        a.delta[((int64_t)b * a.Hq + hq) * a.N + qi] = di_q;
        a.lse2[((int64_t)b * a.Hq + hq) * a.N + qi] = lse_q;
    }
    const float scale_log2 = a.scale * kLog2e;

    const int wg_qmax = min(qt * kBQ + kBQ - 1, a.N - 1);
    const int kv_end_wg = a.causal ? min(a.N, wg_qmax + 1) : a.N;
    const int n_tiles = (kv_end_wg + kBT - 1) / kBT;
    const int kv_end_wave = (q0 < a.N) ? (a.causal ? min(a.N, min(q0 + 31, a.N - 1) + 1) : a.N) : 0;
    const int lim = a.causal ? min(qi, a.N - 1) : a.N - 1;

    f32x16_t acc[DB];
#pragma unroll
    for (int i = 0; i < DB; ++i)
#pragma unroll
        for (int j = 0; j < 16; ++j) acc[i][j] = 0.f;

    TileDma<D> dk_, dv_;
    dk_.init(a.s_k[2], wave, lane);
    dv_.init(a.s_v[2], wave, lane);
    auto load = [&](int kt, auto slot) {
        dk_.load(slot.value ? sK1 : sK0, Kp + (int64_t)kt * kBT * a.s_k[2], a.N - kt * kBT, a.s_k[2], wave);
        dv_.load(slot.value ? sV1 : sV0, Vp + (int64_t)kt * kBT * a.s_v[2], a.N - kt * kBT, a.s_v[2], wave);
        if constexpr (SPLIT) {
            dk_.load(slot.value ? sKl1 : sKl0, Kp + a.lo_kv + (int64_t)kt * kBT * a.s_k[2], a.N - kt * kBT, a.s_k[2], wave);
            dv_.load(slot.value ? sVl1 : sVl0, Vp + a.lo_kv + (int64_t)kt * kBT * a.s_v[2], a.N - kt * kBT, a.s_v[2], wave);
        }
    };
    auto step = [&](int kt, auto slot) {
        dma_wait_all();
        __syncthreads();   // tile kt is in LDS; every wavefront has left tile kt - 1, whose slot is refilled now
        if (kt + 1 < n_tiles) load(kt + 1, std::integral_constant<int, 1 - slot.value>{});
        const uint16_t* tK = slot.value ? sK1 : sK0;
        const uint16_t* tV = slot.value ? sV1 : sV0;
        const uint16_t* tKl = slot.value ? sKl1 : sKl0;
        const uint16_t* tVl = slot.value ? sVl1 : sVl0;
        const int k0 = kt * kBT;
        if (k0 >= kv_end_wave) return;
        f32x16_t s, dp;
#pragma unroll
        for (int j = 0; j < 16; ++j) s[j] = dp[j] = 0.f;
#pragma unroll
        for (int ks = 0; ks < KS; ++ks) {
            const bf16x8_t kh = load_row<D>(tK, ks, lane), vh = load_row<D>(tV, ks, lane);
            s = __builtin_amdgcn_mfma_f32_32x32x16_bf16(kh, qf[ks], s, 0, 0, 0);
            dp = __builtin_amdgcn_mfma_f32_32x32x16_bf16(vh, dof[ks], dp, 0, 0, 0);
            if constexpr (SPLIT) {
                s = __builtin_amdgcn_mfma_f32_32x32x16_bf16(kh, qfl[ks], s, 0, 0, 0);
                dp = __builtin_amdgcn_mfma_f32_32x32x16_bf16(vh, dofl[ks], dp, 0, 0, 0);
                s = __builtin_amdgcn_mfma_f32_32x32x16_bf16(load_row<D>(tKl, ks, lane), qf[ks], s, 0, 0, 0);
                dp = __builtin_amdgcn_mfma_f32_32x32x16_bf16(load_row<D>(tVl, ks, lane), dof[ks], dp, 0, 0, 0);
            }
        }
        uint32_t dsw[2][4], dsl[SPLIT ? 2 : 1][4];
        // dS as bf16 pairs; SPLIT: the rounding remainders as a second set of pairs
        auto pack = [&](int v, float d0, float d1) {
            const uint32_t w = cvt_pk_bf16(d0, d1);
            dsw[v >> 3][(v & 7) >> 1] = w;
            if constexpr (SPLIT) dsl[v >> 3][(v & 7) >> 1] = cvt_pk_bf16(d0 - __uint_as_float(w << 16), d1 - __uint_as_float(w & 0xffff0000u));
        };
        if (k0 + kBT - 1 <= min(q0, a.N - 1) || (!a.causal && k0 + kBT <= a.N)) {   // no position of the tile is masked
#pragma unroll
            for (int v = 0; v < 16; v += 2) {
                const float p0 = __builtin_amdgcn_exp2f(fmaf(s[v], scale_log2, -lse_q));
                const float p1 = __builtin_amdgcn_exp2f(fmaf(s[v + 1], scale_log2, -lse_q));
                pack(v, p0 * (dp[v] - di_q), p1 * (dp[v + 1] - di_q));
            }
        } else {
#pragma unroll
            for (int v = 0; v < 16; v += 2) {
                float d2[2];
#pragma unroll
                for (int u = 0; u < 2; ++u) {
                    const int key = k0 + 8 * ((v + u) >> 2) + 4 * h + ((v + u) & 3);
                    const float p = __builtin_amdgcn_exp2f(key <= lim ? fmaf(s[v + u], scale_log2, -lse_q) : -INFINITY);
                    d2[u] = p * (dp[v + u] - di_q);
                }
                pack(v, d2[0], d2[1]);
            }
        }
#pragma unroll
        for (int j = 0; j < 2; ++j) {
            const bf16x8_t dsf = __builtin_bit_cast(bf16x8_t, uint4{dsw[j][0], dsw[j][1], dsw[j][2], dsw[j][3]});
#pragma unroll
            for (int db = 0; db < DB; ++db) {
                const bf16x8_t kt_h = load_transposed<D>(tK, j, db, lane);
                acc[db] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(kt_h, dsf, acc[db], 0, 0, 0);
                if constexpr (SPLIT) {
                    const bf16x8_t dsfl = __builtin_bit_cast(bf16x8_t, uint4{dsl[j][0], dsl[j][1], dsl[j][2], dsl[j][3]});
                    acc[db] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(kt_h, dsfl, acc[db], 0, 0, 0);
                    acc[db] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(load_transposed<D>(tKl, j, db, lane), dsf, acc[db], 0, 0, 0);
                }
            }
        }
    };
    load(0, std::integral_constant<int, 0>{});
    for (int kt = 0; kt < n_tiles; kt += 2) {
        step(kt, std::integral_constant<int, 0>{});
        if (kt + 1 < n_tiles) step(kt + 1, std::integral_constant<int, 1>{});
    }
    if (qi < a.N) {
        const int64_t row = (int64_t)b * a.s_dq[0] + (int64_t)hq * a.s_dq[1] + (int64_t)qi * a.s_dq[2];
#pragma unroll
        for (int db = 0; db < DB; ++db)
#pragma unroll
            for (int vq = 0; vq < 4; ++vq) store4<SPLIT>(a.dq, row + 32 * db + 8 * vq + 4 * h, a.scale, acc[db], 4 * vq);
    }
}

// ---- dK, dV (bf16) ----
// A workgroup owns 64 key rows of one kv head: two blocks of 32, each worked by a pair of wavefronts that share
// the arithmetic of a (query tile, key block) step by product instead of by rows, which halves what each has to
// keep in registers (one of K / V, one of dK / dV):
//   wavefront P:  S = Q K^T  ->  P = exp2(..)  ->  hands P (bf16) to its partner through LDS  ->  dV^T += dO^T P
//   wavefront D:  dP = dO V^T                  ->  takes P  ->  dS = P (dP - Di)               ->  dK^T += Q^T dS
// Both see the same accumulator layout, so lane l of one reads exactly the words lane l of the other wrote.
// The two halves of a step are one iteration apart: while the second products of tile t run, the first products
// of tile t + 1 are issued, and P(t + 1) crosses to the partner over the iteration's only barrier.  A tile is
// therefore live for two iterations and the ring holds three.
constexpr int kBK = 64;   // key rows per workgroup in the bf16 dK / dV pass

// SPLIT: as in bwd_dq_bf16_kernel; P crosses to the partner as fp32, and each wavefront splits what it feeds to its
// own second product (P or dS) into two bf16 terms.
// SPILL: the D wavefront also leaves dS of every (query tile, key block) in the workspace (a.ds_tiles), from where
// bwd_dq_stream_kernel takes dQ with one product instead of the three of bwd_dq_bf16_kernel.
template <int D, bool SPLIT = false, bool SPILL = false>
__global__ void __launch_bounds__(256, SPLIT ? 1 : 2) bwd_dkdv_bf16_kernel(BwdArgs a) {
    constexpr int KS = D / 16, DB = D / 32;
    // One variable per ring slot: the compiler then knows that a read of one slot does not touch the slot a
    // direct-to-LDS load in flight is filling, and does not wait for that load.
    __shared__ __attribute__((aligned(1024))) uint16_t sQ0[kBT * D], sQ1[kBT * D], sQ2[kBT * D];
    __shared__ __attribute__((aligned(1024))) uint16_t sO0[kBT * D], sO1[kBT * D], sO2[kBT * D];
    __shared__ __attribute__((aligned(256))) float sL0[64], sL1[64], sL2[64];   // lse and Di of the tile's rows (32 used; a
    __shared__ __attribute__((aligned(256))) float sD0[64], sD1[64], sD2[64];   // wavefront instruction fills 64 words)
    __shared__ __attribute__((aligned(16))) uint32_t sP[3][2][SPLIT ? 16 : 8][64];   // [ring slot][key block][word][lane]
    __shared__ __attribute__((aligned(1024))) uint16_t sQl0[SPLIT ? kBT * D : 8], sQl1[SPLIT ? kBT * D : 8], sQl2[SPLIT ? kBT * D : 8];   // lo planes
    __shared__ __attribute__((aligned(1024))) uint16_t sOl0[SPLIT ? kBT * D : 8], sOl1[SPLIT ? kBT * D : 8], sOl2[SPLIT ? kBT * D : 8];
    auto tql = [&](auto s) -> uint16_t* { if constexpr (s.value == 0) return sQl0; else if constexpr (s.value == 1) return sQl1; else return sQl2; };
    auto tol = [&](auto s) -> uint16_t* { if constexpr (s.value == 0) return sOl0; else if constexpr (s.value == 1) return sOl1; else return sOl2; };
    auto tq = [&](auto s) -> uint16_t* { if constexpr (s.value == 0) return sQ0; else if constexpr (s.value == 1) return sQ1; else return sQ2; };
    auto to = [&](auto s) -> uint16_t* { if constexpr (s.value == 0) return sO0; else if constexpr (s.value == 1) return sO1; else return sO2; };
    auto tl = [&](auto s) -> float* { if constexpr (s.value == 0) return sL0; else if constexpr (s.value == 1) return sL1; else return sL2; };
    auto td = [&](auto s) -> float* { if constexpr (s.value == 0) return sD0; else if constexpr (s.value == 1) return sD1; else return sD2; };
    const int bid = blockIdx.x;
    const int kt = bid / (a.B * a.Hkv);          // causal work falls with the key tile: heaviest first
    const int bh = bid % (a.B * a.Hkv);
    const int b = bh / a.Hkv, kvh = bh % a.Hkv;
    const int tid = threadIdx.x, lane = tid & 63, wave = __builtin_amdgcn_readfirstlane(tid >> 6);
    const int kb = wave >> 1;
    // which wavefront of a pair takes which role alternates between workgroups, so that the exp-heavy role of two
    // co-resident workgroups does not always fall on the same SIMDs
    const bool role_d = __builtin_amdgcn_readfirstlane((wave ^ __builtin_popcount(bid >> 3)) & 1);
    const int kl = lane & 31, h = lane >> 5;
    const int key0 = kt * kBK + kb * 32;
    const int ki = key0 + kl;
    const int krow = min(ki, a.N - 1);

    // the stationary operand: K rows for the P wavefront, V rows for the D wavefront
    const uint16_t* Xp = role_d ? (const uint16_t*)a.v + (int64_t)b * a.s_v[0] + (int64_t)kvh * a.s_v[1] + (int64_t)krow * a.s_v[2]
                                : (const uint16_t*)a.k + (int64_t)b * a.s_k[0] + (int64_t)kvh * a.s_k[1] + (int64_t)krow * a.s_k[2];
    bf16x8_t xf[KS], xfl[SPLIT ? KS : 1];
#pragma unroll
    for (int ks = 0; ks < KS; ++ks) {
        xf[ks] = __builtin_bit_cast(bf16x8_t, *(const uint4*)(Xp + 16 * ks + 8 * h));
        if constexpr (SPLIT) xfl[ks] = __builtin_bit_cast(bf16x8_t, *(const uint4*)(Xp + a.lo_kv + 16 * ks + 8 * h));
    }
    f32x16_t acc[DB];
#pragma unroll
    for (int i = 0; i < DB; ++i)
#pragma unroll
        for (int j = 0; j < 16; ++j) acc[i][j] = 0.f;

    const int qt_begin = a.causal ? (kt * kBK) / kBT : 0;
    const int n_qt = (a.N + kBT - 1) / kBT - qt_begin;   // query tiles per head
    const int n_it = a.n_rep * n_qt;                     // the loop runs over (head of the group, query tile)
    // SPILL: where the D wavefront leaves its next dS tile; query tiles of a head are n_kt32 tiles apart, heads
    // n_qt32 * n_kt32
    char* ds_tile = nullptr;
    int64_t ds_step_t = 0, ds_step_r = 0;   // to the next query tile; from the last query tile of a head to the first of the next
    if constexpr (SPILL) {
        ds_step_t = -(int64_t)a.n_kt32 * 2048;
        ds_step_r = (int64_t)a.n_qt32 * a.n_kt32 * 2048 - (int64_t)(n_qt - 1) * ds_step_t;
        ds_tile = (char*)a.ds_tiles + ((((int64_t)b * a.Hq + kvh * a.n_rep) * a.n_qt32 + qt_begin + n_qt - 1) * a.n_kt32 + (key0 >> 5)) * 2048 + lane * 16;
    }
    const float scale_log2 = a.scale * kLog2e;

    TileDma<D> dq_, do_;
    dq_.init(a.s_q[2], wave, lane);
    do_.init(a.s_do[2], wave, lane);
    // (head of the group, query tile) of the tile being fetched and of the tile whose first products are due:
    // the loop index split without a division per step
    int ld_r = 0, ld_t = 0, fi_r = 0, fi_t = 0, se_t = 0;
    auto advance = [&](int& r, int& t) {
        if (++t == n_qt) {
            t = 0;
            ++r;
        }
    };
    auto load = [&](int it, auto buf) {
        const int hq = kvh * a.n_rep + ld_r, qb = (qt_begin + (n_qt - 1 - ld_t)) * kBT;   // a head's query tiles from the last one down
        advance(ld_r, ld_t);
        dq_.load(tq(buf), (const uint16_t*)a.q + (int64_t)b * a.s_q[0] + (int64_t)hq * a.s_q[1] + (int64_t)qb * a.s_q[2], a.N - qb,
                 a.s_q[2], wave);
        do_.load(to(buf), (const uint16_t*)a.dout + (int64_t)b * a.s_do[0] + (int64_t)hq * a.s_do[1] + (int64_t)qb * a.s_do[2],
                 a.N - qb, a.s_do[2], wave);
        if constexpr (SPLIT) {
            dq_.load(tql(buf), (const uint16_t*)a.q + a.lo_q + (int64_t)b * a.s_q[0] + (int64_t)hq * a.s_q[1] + (int64_t)qb * a.s_q[2],
                     a.N - qb, a.s_q[2], wave);
            do_.load(tol(buf), (const uint16_t*)a.dout + a.lo_q + (int64_t)b * a.s_do[0] + (int64_t)hq * a.s_do[1] + (int64_t)qb * a.s_do[2],
                     a.N - qb, a.s_do[2], wave);
        }
        if (wave == 0)
            row_dma(tl(buf), a.lse2 + ((int64_t)b * a.Hq + hq) * a.N + qb, min(a.N - qb, kBT), 1, lane);
        else if (wave == 1)
            row_dma(td(buf), a.delta + ((int64_t)b * a.Hq + hq) * a.N + qb, min(a.N - qb, kBT), 1, lane);
    };
    // The loop exists once per role, so that each wavefront's code reads its tiles from named variables.
    auto run = [&](auto role) {
    constexpr bool RD = decltype(role)::value;
    // first products of tile t: S (P wavefront) or dP (D wavefront) into s; the P wavefront goes on to P(t),
    // packed into pw and posted for its partner.  Masked or out-of-range positions get P = 0, so a tile that lies
    // wholly above the diagonal or past the end costs its MFMAs and contributes nothing.
    auto first = [&](int t, auto buf, f32x16_t& s, uint32_t (&pw)[2][4], uint32_t (&pl)[2][4]) {
        const uint16_t *rows, *rows_lo;
        if constexpr (RD) rows = to(buf), rows_lo = tol(buf);
        else rows = tq(buf), rows_lo = tql(buf);
#pragma unroll
        for (int j = 0; j < 16; ++j) s[j] = 0.f;
#pragma unroll
        for (int ks = 0; ks < KS; ++ks) {
            const bf16x8_t rh = load_row<D>(rows, ks, lane);
            s = __builtin_amdgcn_mfma_f32_32x32x16_bf16(rh, xf[ks], s, 0, 0, 0);
            if constexpr (SPLIT) {
                s = __builtin_amdgcn_mfma_f32_32x32x16_bf16(rh, xfl[ks], s, 0, 0, 0);
                s = __builtin_amdgcn_mfma_f32_32x32x16_bf16(load_row<D>(rows_lo, ks, lane), xf[ks], s, 0, 0, 0);
            }
        }
        if constexpr (!RD) {
            const int qb = (qt_begin + (n_qt - 1 - fi_t)) * kBT;
            float lq[16];
#pragma unroll
            for (int g = 0; g < 4; ++g) *(float4*)&lq[4 * g] = *(const float4*)&tl(buf)[8 * g + 4 * h];
            const bool edge = (a.causal && qb < key0 + 31) || qb + kBT > a.N || key0 + 32 > a.N;   // same for the wavefront
            // P as bf16 pairs (SPLIT: the rounding remainders as a second set, and fp32 P posted for the partner)
            auto pack = [&](int v, float p0, float p1) {
                const uint32_t w = cvt_pk_bf16(p0, p1);
                pw[v >> 3][(v & 7) >> 1] = w;
                if constexpr (SPLIT) {
                    pl[v >> 3][(v & 7) >> 1] = cvt_pk_bf16(p0 - __uint_as_float(w << 16), p1 - __uint_as_float(w & 0xffff0000u));
                    sP[buf.value][kb][v][lane] = __float_as_uint(p0);
                    sP[buf.value][kb][v + 1][lane] = __float_as_uint(p1);
                }
            };
            if (!edge) {
#pragma unroll
                for (int v = 0; v < 16; v += 2)
                    pack(v, __builtin_amdgcn_exp2f(fmaf(s[v], scale_log2, -lq[v])), __builtin_amdgcn_exp2f(fmaf(s[v + 1], scale_log2, -lq[v + 1])));
            } else {
#pragma unroll
                for (int v = 0; v < 16; v += 2) {
                    float p2[2];
#pragma unroll
                    for (int u = 0; u < 2; ++u) {
                        const int qi = qb + 8 * ((v + u) >> 2) + 4 * h + ((v + u) & 3);
                        const bool ok = qi < a.N && ki < a.N && (!a.causal || ki <= qi);
                        p2[u] = __builtin_amdgcn_exp2f(ok ? fmaf(s[v + u], scale_log2, -lq[v + u]) : -INFINITY);
                    }
                    pack(v, p2[0], p2[1]);
                }
            }
            if constexpr (!SPLIT) {
#pragma unroll
                for (int j = 0; j < 2; ++j)
#pragma unroll
                    for (int w = 0; w < 4; ++w) sP[buf.value][kb][4 * j + w][lane] = pw[j][w];
            }
            advance(fi_r, fi_t);
        }
    };
    // second products of tile t: dV^T += dO^T P (P wavefront, P from its own registers) or
    // dS = P (dP - Di), dK^T += Q^T dS (D wavefront, P from its partner)
    auto second = [&](int t, auto buf, const f32x16_t& s, uint32_t (&pw)[2][4], uint32_t (&pl)[2][4]) {
        if constexpr (RD) {
            float di[16];
#pragma unroll
            for (int g = 0; g < 4; ++g) *(float4*)&di[4 * g] = *(const float4*)&td(buf)[8 * g + 4 * h];
#pragma unroll
            for (int v = 0; v < 16; v += 2) {
                float p0, p1;
                if constexpr (SPLIT) {
                    p0 = __uint_as_float(sP[buf.value][kb][v][lane]), p1 = __uint_as_float(sP[buf.value][kb][v + 1][lane]);
                } else {
                    const uint32_t w = sP[buf.value][kb][v >> 1][lane];
                    p0 = __uint_as_float(w << 16), p1 = __uint_as_float(w & 0xffff0000u);
                }
                const float d0 = p0 * (s[v] - di[v]), d1 = p1 * (s[v + 1] - di[v + 1]);
                const uint32_t w2 = cvt_pk_bf16(d0, d1);
                pw[v >> 3][(v & 7) >> 1] = w2;
                if constexpr (SPLIT) pl[v >> 3][(v & 7) >> 1] = cvt_pk_bf16(d0 - __uint_as_float(w2 << 16), d1 - __uint_as_float(w2 & 0xffff0000u));
            }
            if constexpr (SPILL) {
                // the tile as this wavefront's registers hold it, [j][lane][4 words]: lane (key kl, half h) holds, in
                // pw[j][2c], pw[j][2c + 1], the queries 16 j + 8 c + 4 h .. + 3.  Two instructions of 1 KB each, written once
                // and read once: kept out of the way of the tiles the L2 is holding.
                u32x4_t* tile = (u32x4_t*)ds_tile;
                if (++se_t == n_qt) {
                    se_t = 0;
                    ds_tile += ds_step_r;
                } else {
                    ds_tile += ds_step_t;
                }
#pragma unroll
                for (int j = 0; j < 2; ++j) __builtin_nontemporal_store(u32x4_t{pw[j][0], pw[j][1], pw[j][2], pw[j][3]}, tile + 64 * j);
            }
        }
        const uint16_t *cols, *cols_lo;
        if constexpr (RD) cols = tq(buf), cols_lo = tql(buf);
        else cols = to(buf), cols_lo = tol(buf);
#pragma unroll
        for (int j = 0; j < 2; ++j) {
            const bf16x8_t bf = __builtin_bit_cast(bf16x8_t, uint4{pw[j][0], pw[j][1], pw[j][2], pw[j][3]});
#pragma unroll
            for (int db = 0; db < DB; ++db) {
                const bf16x8_t ch = load_transposed<D>(cols, j, db, lane);
                acc[db] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(ch, bf, acc[db], 0, 0, 0);
                if constexpr (SPLIT) {
                    const bf16x8_t bl = __builtin_bit_cast(bf16x8_t, uint4{pl[j][0], pl[j][1], pl[j][2], pl[j][3]});
                    acc[db] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(ch, bl, acc[db], 0, 0, 0);
                    acc[db] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(load_transposed<D>(cols_lo, j, db, lane), bf, acc[db], 0, 0, 0);
                }
            }
        }
    };

    f32x16_t s_cur;
    uint32_t pw_cur[2][4], pl_cur[2][4];
    using S0 = std::integral_constant<int, 0>;
    using S1 = std::integral_constant<int, 1>;
    using S2 = std::integral_constant<int, 2>;
    load(0, S0{});
    if (n_it > 1) load(1, S1{});
    dma_wait_all();
    __syncthreads();
    first(0, S0{}, s_cur, pw_cur, pl_cur);
    // one iteration, for tile `it` in ring slot `buf`
    auto step = [&](int it, auto buf) {
        using B1 = std::integral_constant<int, (buf.value + 1) % 3>;
        using B2 = std::integral_constant<int, (buf.value + 2) % 3>;
        // tile it + 1 and P(it) are in LDS; every wavefront has left tile it - 1, whose slot takes tile it + 2
        // (SPILL: the D wavefront's two dS stores of the previous iteration are younger than that tile's requests in
        // its memory queue and need not have been acknowledged)
        if constexpr (RD && SPILL) asm volatile("s_waitcnt vmcnt(2)" ::: "memory");
        else dma_wait_all();
        __syncthreads();
        if (it + 2 < n_it) load(it + 2, B2{});
        // the second products consume s / pw of this tile, then the first products of the next tile refill them
        second(it, buf, s_cur, pw_cur, pl_cur);
        if (it + 1 < n_it) first(it + 1, B1{}, s_cur, pw_cur, pl_cur);
    };
    for (int it = 0; it < n_it; it += 3) {
        step(it, S0{});
        if (it + 1 < n_it) step(it + 1, S1{});
        if (it + 2 < n_it) step(it + 2, S2{});
    }
    };
    if (role_d) run(std::true_type{});
    else run(std::false_type{});
    if (ki < a.N) {
        const float f = role_d ? a.scale : 1.f;
        void* po = role_d ? a.dk : a.dv;
        const int64_t row = role_d ? (int64_t)b * a.s_dk[0] + (int64_t)kvh * a.s_dk[1] + (int64_t)ki * a.s_dk[2]
                                   : (int64_t)b * a.s_dv[0] + (int64_t)kvh * a.s_dv[1] + (int64_t)ki * a.s_dv[2];
#pragma unroll
        for (int db = 0; db < DB; ++db)
#pragma unroll
            for (int vq = 0; vq < 4; ++vq) store4<SPLIT>(po, row + 32 * db + 8 * vq + 4 * h, f, acc[db], 4 * vq);
    }
}

// ---- dQ from the dS tiles the dK / dV pass left behind (bf16) ----
// A wavefront owns 32 query rows and walks the key tiles.  Its own dS tile (2 KB, consecutive key tiles consecutive in
// the workspace) comes straight into registers, several tiles ahead; the workgroup's shared K tile comes through a
// ring of four LDS slots.  The tile is the register image of the wavefront that wrote it (a lane = a key), and this
// product contracts over keys, so it passes through a 2 KB patch of LDS of the wavefront's own: written as it came,
// read back with the transposing read (a lane = a query).  Then dQ^T[d][q] += K^T . dS^T, A = the K tile read
// column-wise.  One product instead of the three of bwd_dq_bf16_kernel: the pass runs at the rate the tiles stream in.
// Masked positions hold zeros in the tiles, so no mask is applied here.
template <int D>
__global__ void __launch_bounds__(256, 2) bwd_dq_stream_kernel(BwdArgs a) {
    constexpr int DB = D / 32;
    constexpr int PER_STAGE = TileDma<D>::NLD + 2;   // memory instructions a wavefront issues per ring stage
    __shared__ __attribute__((aligned(1024))) uint16_t sK0[kBT * D], sK1[kBT * D], sK2[kBT * D], sK3[kBT * D];
    __shared__ __attribute__((aligned(1024))) char sT[4][2048];   // per wavefront
    auto tk = [&](auto s) -> uint16_t* { if constexpr (s.value == 0) return sK0; else if constexpr (s.value == 1) return sK1; else if constexpr (s.value == 2) return sK2; else return sK3; };
    const int n_qtiles = (a.N + kBQ - 1) / kBQ;
    const int bid = blockIdx.x;
    const int qt = n_qtiles - 1 - bid / (a.B * a.Hq);
    const int bh = xcd_grouped_head(bid % (a.B * a.Hq), a.B * a.Hkv, a.n_rep);
    const int b = bh / a.Hq, hq = bh % a.Hq, kvh = hq / a.n_rep;
    const int tid = threadIdx.x, lane = tid & 63, wave = __builtin_amdgcn_readfirstlane(tid >> 6);
    const int ql = lane & 31, h = lane >> 5;
    const int q0 = qt * kBQ + wave * 32;
    const int qi = q0 + ql;

    const int wg_qmax = min(qt * kBQ + kBQ - 1, a.N - 1);
    const int n_tiles = ((a.causal ? wg_qmax + 1 : a.N) + kBT - 1) / kBT;          // key tiles the workgroup walks
    const int nt_w = q0 < a.N ? ((a.causal ? min(q0 + 31, a.N - 1) + 1 : a.N) + kBT - 1) / kBT : 0;   // of which this wavefront uses

    const uint16_t* Kp = (const uint16_t*)a.k + (int64_t)b * a.s_k[0] + (int64_t)kvh * a.s_k[1];
    const u32x4_t* Sp = (const u32x4_t*)((const char*)a.ds_tiles + ((((int64_t)b * a.Hq + hq) * a.n_qt32 + min(q0 >> 5, a.n_qt32 - 1)) * a.n_kt32) * 2048) + lane;
    TileDma<D> dk_;
    dk_.init(a.s_k[2], wave, lane);
    constexpr int NI = 8, AHEAD = 6;   // dS tiles: register ring, and how many tiles ahead they are requested
    u32x4_t img[NI][2];
    // Every step issues the same number of loads, so that the wait counts below hold: past the end the tile index is
    // clamped (the tile is fetched again and not used).
    auto load_k = [&](int t, auto slot) {
        const int kt = min(t, n_tiles - 1);
        dk_.load(tk(slot), Kp + (int64_t)kt * kBT * a.s_k[2], a.N - kt * kBT, a.s_k[2], wave);
    };
    auto load_s = [&](int t, auto islot) {
        const u32x4_t* tile = Sp + (int64_t)min(t, max(nt_w - 1, 0)) * 128;
        img[islot.value][0] = __builtin_nontemporal_load(tile);
        img[islot.value][1] = __builtin_nontemporal_load(tile + 64);
    };
    f32x16_t acc[DB];
#pragma unroll
    for (int i = 0; i < DB; ++i)
#pragma unroll
        for (int j = 0; j < 16; ++j) acc[i][j] = 0.f;
    // The patch holds the image as [j][position of the writing lane][4 words], the lane (key kl, half hh) at position
    // 2 kl + hh, rotated by 128 bytes for j = 1: the 16 lanes of a transposing read then fetch 4 keys x 32 bytes =
    // 128 consecutive bytes, and the four such groups of an instruction fall in different banks.
    char* patch = sT[wave];
    const int wr_off = (2 * ql + h) * 16;
    const int i16 = lane & 15, g4 = (lane >> 4) & 1;
    // k-step j', keys 16 j' + 4 h + (i16 >> 2) (+ 8), queries 16 g4 + 4 (i16 & 3) .. + 3: words 2c, 2c + 1 of the lane
    // (key, hh) with hh = i16 & 1, c = (i16 >> 1) & 1, in half j = g4 of the image
    const int rd_off = 32 * (4 * h + (i16 >> 2)) + 16 * (i16 & 1) + 8 * ((i16 >> 1) & 1);
    auto step = [&](int t, auto idx) {
        using KS = std::integral_constant<int, idx.value % 4>;
        using KL = std::integral_constant<int, (idx.value + 3) % 4>;
        using IL = std::integral_constant<int, (idx.value + AHEAD) % NI>;
        // This wavefront's share of K tile t has landed.  Younger in its memory queue, and possibly still in flight: the
        // dS tile requested right behind it and the two steps' requests since.  No fence: it would drain them.
        asm volatile("s_waitcnt vmcnt(%0)" ::"n"(2 + 2 * PER_STAGE) : "memory");
        __builtin_amdgcn_s_barrier();
        asm volatile("" ::: "memory");
        const u32x4_t i0 = img[idx.value % NI][0], i1 = img[idx.value % NI][1];
        load_k(t + 3, KL{});   // into the slot every wavefront left before this barrier
        load_s(t + AHEAD, IL{});
        if (t >= nt_w) return;
        using slot_t = KS;
        const slot_t slot{};
        const uint16_t* tK = tk(slot);
        *(u32x4_t*)(patch + wr_off) = i0;
        *(u32x4_t*)(patch + 1024 + ((wr_off + 128) & 1023)) = i1;
#pragma unroll
        for (int j = 0; j < 2; ++j) {
            const char* half = patch + 1024 * g4;
            const uint2 lo = lds_tr16(half + ((rd_off + 512 * j + 128 * g4) & 1023));
            const uint2 hi = lds_tr16(half + ((rd_off + 512 * j + 256 + 128 * g4) & 1023));
            const bf16x8_t dsf = __builtin_bit_cast(bf16x8_t, uint4{lo.x, lo.y, hi.x, hi.y});
#pragma unroll
            for (int db = 0; db < DB; ++db) acc[db] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(load_transposed<D>(tK, j, db, lane), dsf, acc[db], 0, 0, 0);
        }
    };
    using I0 = std::integral_constant<int, 0>;
    using I1 = std::integral_constant<int, 1>;
    using I2 = std::integral_constant<int, 2>;
    using I3 = std::integral_constant<int, 3>;
    using I4 = std::integral_constant<int, 4>;
    using I5 = std::integral_constant<int, 5>;
    using I6 = std::integral_constant<int, 6>;
    using I7 = std::integral_constant<int, 7>;
    // the order of the first requests gives every K tile at least as many younger requests as the steady state does
    load_k(0, I0{});
    load_s(0, I0{});
    load_s(1, I1{});
    load_s(2, I2{});
    load_s(3, I3{});
    load_k(1, I1{});
    load_s(4, I4{});
    load_k(2, I2{});
    load_s(5, I5{});
    for (int t = 0; t < n_tiles; t += 8) {
        step(t, I0{});
        if (t + 1 < n_tiles) step(t + 1, I1{});
        if (t + 2 < n_tiles) step(t + 2, I2{});
        if (t + 3 < n_tiles) step(t + 3, I3{});
        if (t + 4 < n_tiles) step(t + 4, I4{});
        if (t + 5 < n_tiles) step(t + 5, I5{});
        if (t + 6 < n_tiles) step(t + 6, I6{});
        if (t + 7 < n_tiles) step(t + 7, I7{});
    }
    dma_wait_all();   // the clamped requests of the last steps write LDS: they land before the workgroup gives it back
    if (qi < a.N) {
        const int64_t row = (int64_t)b * a.s_dq[0] + (int64_t)hq * a.s_dq[1] + (int64_t)qi * a.s_dq[2];
#pragma unroll
        for (int db = 0; db < DB; ++db)
#pragma unroll
            for (int vq = 0; vq < 4; ++vq) store4<false>(a.dq, row + 32 * db + 8 * vq + 4 * h, a.scale, acc[db], 4 * vq);
    }
}

// Instantiated explicitly: the host pass of this compiler drops the implicit instantiation of the launch stubs.
template __global__ void bwd_dkdv_bf16_kernel<128, false, true>(BwdArgs);
template __global__ void bwd_dkdv_bf16_kernel<64, false, true>(BwdArgs);
template __global__ void bwd_dq_stream_kernel<128>(BwdArgs);
template __global__ void bwd_dq_stream_kernel<64>(BwdArgs);
template __global__ void bwd_rowstats_bf16_kernel<128>(BwdArgs);
template __global__ void bwd_rowstats_bf16_kernel<64>(BwdArgs);
template __global__ void bwd_dkdv_bf16_kernel<128, false>(BwdArgs);
template __global__ void bwd_dkdv_bf16_kernel<64, false>(BwdArgs);
template __global__ void bwd_dq_bf16_kernel<128, false>(BwdArgs);
template __global__ void bwd_dq_bf16_kernel<64, false>(BwdArgs);
template __global__ void bwd_dkdv_bf16_kernel<128, true>(BwdArgs);
template __global__ void bwd_dkdv_bf16_kernel<64, true>(BwdArgs);
template __global__ void bwd_dq_bf16_kernel<128, true>(BwdArgs);
template __global__ void bwd_dq_bf16_kernel<64, true>(BwdArgs);

// ---- pre-pass of the split-operand path: every fp32 operand as two bf16 planes, Di and lse * log2(e) ----
struct SplitArgs {
    const float *q, *dout, *out, *k, *v, *lse;
    int64_t s_q[3], s_do[3], s_o[3], s_k[3], s_v[3], s_l[3];
    uint16_t *qh, *doh, *kh, *vh;          // hi planes, dense [B][H][N][D]; the lo plane follows at lo_q / lo_kv elements
    int64_t lo_q, lo_kv;
    float *delta, *lse2;
    int32_t B, Hq, Hkv, N, D;
};
__device__ inline void split_pair(float x0, float x1, uint16_t* hi, uint16_t* lo) {
    const uint32_t h = cvt_pk_bf16(x0, x1);
    *(uint32_t*)hi = h;
    *(uint32_t*)lo = cvt_pk_bf16(x0 - __uint_as_float(h << 16), x1 - __uint_as_float(h & 0xffff0000u));
}
// One wavefront per row: rows [0, B Hq N) are query rows (Q, dO, and Di = rowsum(dO * O) in fp32,
// src/ops/flash_attention.cpp:416-423), the rest are key rows (K, V).
__global__ void __launch_bounds__(256) bwd_split_kernel(SplitArgs a) {
    const int lane = threadIdx.x & 63;
    const int64_t row = (int64_t)blockIdx.x * 4 + (threadIdx.x >> 6);
    const int64_t rows_q = (int64_t)a.B * a.Hq * a.N, rows_kv = (int64_t)a.B * a.Hkv * a.N;
    if (row < rows_q) {
        const int i = (int)(row % a.N);
        const int64_t bh = row / a.N;
        const int h = (int)(bh % a.Hq), b = (int)(bh / a.Hq);
        const float* pq = a.q + (int64_t)b * a.s_q[0] + (int64_t)h * a.s_q[1] + (int64_t)i * a.s_q[2];
        const float* pd = a.dout + (int64_t)b * a.s_do[0] + (int64_t)h * a.s_do[1] + (int64_t)i * a.s_do[2];
        const float* po = a.out + (int64_t)b * a.s_o[0] + (int64_t)h * a.s_o[1] + (int64_t)i * a.s_o[2];
        float di = 0.f;
        for (int d = 2 * lane; d < a.D; d += 128) {
            const float2 xq = *(const float2*)(pq + d), xd = *(const float2*)(pd + d), xo = *(const float2*)(po + d);
            split_pair(xq.x, xq.y, a.qh + row * a.D + d, a.qh + a.lo_q + row * a.D + d);
            split_pair(xd.x, xd.y, a.doh + row * a.D + d, a.doh + a.lo_q + row * a.D + d);
            di += xd.x * xo.x;
            di += xd.y * xo.y;
        }
#pragma unroll
        for (int o = 32; o > 0; o >>= 1) di += __shfl_xor(di, o);
        if (lane == 0) {
            a.delta[row] = di;
            a.lse2[row] = kLog2e * a.lse[(int64_t)b * a.s_l[0] + (int64_t)h * a.s_l[1] + (int64_t)i * a.s_l[2]];
        }
    } else if (row < rows_q + rows_kv) {
        const int64_t r = row - rows_q;
        const int i = (int)(r % a.N);
        const int64_t bh = r / a.N;
        const int h = (int)(bh % a.Hkv), b = (int)(bh / a.Hkv);
        const float* pk = a.k + (int64_t)b * a.s_k[0] + (int64_t)h * a.s_k[1] + (int64_t)i * a.s_k[2];
        const float* pv = a.v + (int64_t)b * a.s_v[0] + (int64_t)h * a.s_v[1] + (int64_t)i * a.s_v[2];
        for (int d = 2 * lane; d < a.D; d += 128) {
            const float2 xk = *(const float2*)(pk + d), xv = *(const float2*)(pv + d);
            split_pair(xk.x, xk.y, a.kh + r * a.D + d, a.kh + a.lo_kv + r * a.D + d);
            split_pair(xv.x, xv.y, a.vh + r * a.D + d, a.vh + a.lo_kv + r * a.D + d);
        }
    }
}

int check4(const vsp_tensor* t, int64_t B, int64_t H, int64_t N, int64_t D, int dtype) {
    if (!t) return VSP_ERR_NULL;
    if (t->ndim != 4) return VSP_ERR_NDIM;
    if (t->shape[0] != B || t->shape[1] != H || t->shape[2] != N || t->shape[3] != D) return VSP_ERR_SHAPE;
    if (t->dtype != dtype) return VSP_ERR_DTYPE;
    if (t->stride[3] != 1) return VSP_ERR_STRIDE;
    if (B * H * N * D > 0 && !t->data) return VSP_ERR_NULL;
    return VSP_OK;
}

template <typename T>
int launch_backward(const BwdArgs& a, int64_t D, hipStream_t st) {
    const int64_t rows = (int64_t)a.B * a.Hq * a.N;
    if constexpr (sizeof(T) != 2) {  // the bf16 dQ pass computes Di itself, in its prologue
        hipLaunchKernelGGL(bwd_delta_kernel<T>, dim3((unsigned)ceil_div(rows, 4)), dim3(256), 0, st, a, (int)D);
        int rc = check_launch();
        if (rc != VSP_OK) return rc;
    }
    const int64_t tiles = ceil_div(a.N, kBQ);
    const dim3 gq((unsigned)(tiles * a.B * a.Hq)), gk((unsigned)(tiles * a.B * a.Hkv));
    if constexpr (sizeof(T) == 2) {
        const dim3 gk((unsigned)(ceil_div(a.N, kBK) * a.B * a.Hkv));
        if (a.ds_tiles) {  // one-pass dS: row constants, dK / dV (leaving the dS tiles), dQ from the tiles
            if (D == 128) {
                hipLaunchKernelGGL((bwd_rowstats_bf16_kernel<128>), dim3((unsigned)ceil_div(rows, 16)), dim3(256), 0, st, a);
                hipLaunchKernelGGL((bwd_dkdv_bf16_kernel<128, false, true>), gk, dim3(256), 0, st, a);
                hipLaunchKernelGGL((bwd_dq_stream_kernel<128>), gq, dim3(256), 0, st, a);
            } else {
                hipLaunchKernelGGL((bwd_rowstats_bf16_kernel<64>), dim3((unsigned)ceil_div(rows, 32)), dim3(256), 0, st, a);
                hipLaunchKernelGGL((bwd_dkdv_bf16_kernel<64, false, true>), gk, dim3(256), 0, st, a);
                hipLaunchKernelGGL((bwd_dq_stream_kernel<64>), gq, dim3(256), 0, st, a);
            }
            return check_launch();
        }
        if (D == 128) {
            hipLaunchKernelGGL((bwd_dq_bf16_kernel<128, false>), gq, dim3(256), 0, st, a);
            hipLaunchKernelGGL((bwd_dkdv_bf16_kernel<128, false>), gk, dim3(256), 0, st, a);
        } else {
            hipLaunchKernelGGL((bwd_dq_bf16_kernel<64, false>), gq, dim3(256), 0, st, a);
            hipLaunchKernelGGL((bwd_dkdv_bf16_kernel<64, false>), gk, dim3(256), 0, st, a);
        }
        return check_launch();
    }
    if (D > 64) {  // the fp32 kernels take any head_dim up to their tile width (a.D_true)
        hipLaunchKernelGGL((bwd_dq_kernel<128, T>), gq, dim3(256), 0, st, a);
        hipLaunchKernelGGL((bwd_dkdv_kernel<128, T>), gk, dim3(256), 0, st, a);
    } else if (D > 32) {
        hipLaunchKernelGGL((bwd_dq_kernel<64, T>), gq, dim3(256), 0, st, a);
        hipLaunchKernelGGL((bwd_dkdv_kernel<64, T>), gk, dim3(256), 0, st, a);
    } else {
        hipLaunchKernelGGL((bwd_dq_kernel<32, T>), gq, dim3(256), 0, st, a);
        hipLaunchKernelGGL((bwd_dkdv_kernel<32, T>), gk, dim3(256), 0, st, a);
    }
    return check_launch();
}

int launch_backward_split(const SplitArgs& sa, const BwdArgs& a, int64_t D, hipStream_t st) {
    const int64_t rows = (int64_t)a.B * (a.Hq + a.Hkv) * a.N;
    hipLaunchKernelGGL(bwd_split_kernel, dim3((unsigned)ceil_div(rows, 4)), dim3(256), 0, st, sa);
    int rc = check_launch();
    if (rc != VSP_OK) return rc;
    const dim3 gq((unsigned)(ceil_div(a.N, kBQ) * a.B * a.Hq)), gk((unsigned)(ceil_div(a.N, kBK) * a.B * a.Hkv));
    if (D == 128) {
        hipLaunchKernelGGL((bwd_dq_bf16_kernel<128, true>), gq, dim3(256), 0, st, a);
        hipLaunchKernelGGL((bwd_dkdv_bf16_kernel<128, true>), gk, dim3(256), 0, st, a);
    } else {
        hipLaunchKernelGGL((bwd_dq_bf16_kernel<64, true>), gq, dim3(256), 0, st, a);
        hipLaunchKernelGGL((bwd_dkdv_bf16_kernel<64, true>), gk, dim3(256), 0, st, a);
    }
    return check_launch();
}

size_t align16(size_t n) { return (n + 15) & ~(size_t)15; }

}  // namespace
}  // namespace vsp

using namespace vsp;

extern "C" size_t vsp_attn_backward_workspace_bytes(int32_t B, int32_t Hq, int32_t N) {
    if (B <= 0 || Hq <= 0 || N <= 0) return 0;
    return 2 * (size_t)B * (size_t)Hq * (size_t)N * sizeof(float);   // Di and the rescaled log-sum-exp
}

extern "C" size_t vsp_attn_backward_fast_workspace_bytes(int32_t B, int32_t Hq, int32_t N) {
    if (B <= 0 || Hq <= 0 || N <= 0) return 0;
    const size_t base = (vsp_attn_backward_workspace_bytes(B, Hq, N) + 255) & ~(size_t)255;
    const size_t n_qt32 = ((size_t)N + 31) / 32, n_kt32 = 2 * (((size_t)N + 63) / 64);
    return base + (size_t)B * (size_t)Hq * n_qt32 * n_kt32 * 2048;   // one 32 x 32 bf16 dS tile per (query tile, key tile)
}

extern "C" int vsp_attn_prefill_backward(const vsp_tensor* dout, const vsp_tensor* q, const vsp_tensor* k,
                                         const vsp_tensor* v, const vsp_tensor* out, const vsp_tensor* lse,
                                         vsp_tensor* dq, vsp_tensor* dk, vsp_tensor* dv, float scale, int is_causal,
                                         void* workspace, size_t workspace_bytes, void* stream) {
    if (!q || !k || !v) return VSP_ERR_NULL;
    if (q->ndim != 4 || k->ndim != 4 || v->ndim != 4) return VSP_ERR_NDIM;
    const int64_t B = q->shape[0], Hq = q->shape[1], N = q->shape[2], D = q->shape[3];
    const int64_t Hkv = k->shape[1];
    if (Hkv <= 0 ? Hq != 0 : (Hq % Hkv != 0)) return VSP_ERR_SHAPE;
    const int dt = q->dtype;
    if (dt != VSP_F32 && dt != VSP_BF16) return VSP_ERR_UNSUPPORTED;
    int rc;
    if ((rc = check4(q, B, Hq, N, D, dt)) || (rc = check4(dout, B, Hq, N, D, dt)) || (rc = check4(out, B, Hq, N, D, dt)) ||
        (rc = check4(dq, B, Hq, N, D, dt)) || (rc = check4(k, B, Hkv, N, D, dt)) || (rc = check4(v, B, Hkv, N, D, dt)) ||
        (rc = check4(dk, B, Hkv, N, D, dt)) || (rc = check4(dv, B, Hkv, N, D, dt)))
        return rc;
    if (!lse) return VSP_ERR_NULL;
    if (lse->ndim != 3 || lse->shape[0] != B || lse->shape[1] != Hq || lse->shape[2] != N) return VSP_ERR_SHAPE;
    if (lse->dtype != VSP_F32) return VSP_ERR_DTYPE;
    if (B * Hq * N * D == 0) return VSP_OK;
    if (!lse->data) return VSP_ERR_NULL;
    // bf16: head_dim 64 or 128; fp32: any head_dim up to 128, as the reference's backward takes any
    if (dt == VSP_BF16 ? (D != 64 && D != 128) : D > 128) return VSP_ERR_UNSUPPORTED;
    if (!(fabsf(scale) < INFINITY)) return VSP_ERR_ARG;
    if (N > INT32_MAX / 2) return VSP_ERR_ARG;
    if (!workspace || workspace_bytes < vsp_attn_backward_workspace_bytes((int32_t)B, (int32_t)Hq, (int32_t)N)) return VSP_ERR_WORKSPACE;
    if (((uintptr_t)workspace & 3) != 0) return VSP_ERR_ALIGN;
    if (dt == VSP_BF16) {  // 16-byte row segments are moved whole
        for (const vsp_tensor* t : {dout, q, k, v, out, (const vsp_tensor*)dq, (const vsp_tensor*)dk, (const vsp_tensor*)dv}) {
            if (!is_aligned16(t->data)) return VSP_ERR_ALIGN;
            for (int i = 0; i < 3; ++i)
                if ((t->stride[i] * 2) % 16 != 0) return VSP_ERR_ALIGN;
            if (t->stride[2] < D) return VSP_ERR_STRIDE;   // whole rows are fetched under a byte-range check
            if ((uint64_t)N * (uint64_t)t->stride[2] * 2u > 0x7fffffffull) return VSP_ERR_STRIDE;
        }
    }

    BwdArgs a{};
    a.dout = dout->data;
    a.q = q->data;
    a.k = k->data;
    a.v = v->data;
    a.out = out->data;
    a.lse = (const float*)lse->data;
    a.dq = dq->data;
    a.dk = dk->data;
    a.dv = dv->data;
    a.delta = (float*)workspace;
    a.lse2 = a.delta + B * Hq * N;
    for (int i = 0; i < 3; ++i) {
        a.s_do[i] = dout->stride[i];
        a.s_q[i] = q->stride[i];
        a.s_k[i] = k->stride[i];
        a.s_v[i] = v->stride[i];
        a.s_o[i] = out->stride[i];
        a.s_l[i] = lse->stride[i];
        a.s_dq[i] = dq->stride[i];
        a.s_dk[i] = dk->stride[i];
        a.s_dv[i] = dv->stride[i];
    }
    a.B = (int)B;
    a.Hq = (int)Hq;
    a.Hkv = (int)Hkv;
    a.n_rep = (int)(Hq / Hkv);
    a.N = (int)N;
    a.causal = is_causal ? 1 : 0;
    a.scale = scale;
    a.D_true = (int)D;
    // bf16 with the larger workspace: dS is computed once (see include/vsp_attn.h)
    if (dt == VSP_BF16 && workspace_bytes >= vsp_attn_backward_fast_workspace_bytes((int32_t)B, (int32_t)Hq, (int32_t)N) && is_aligned16(workspace)) {
        a.ds_tiles = (uint16_t*)((char*)workspace + ((vsp_attn_backward_workspace_bytes((int32_t)B, (int32_t)Hq, (int32_t)N) + 255) & ~(size_t)255));
        a.n_qt32 = (int)ceil_div(N, 32);
        a.n_kt32 = (int)(2 * ceil_div(N, 64));
    }
    return dt == VSP_F32 ? launch_backward<float>(a, D, (hipStream_t)stream) : launch_backward<uint16_t>(a, D, (hipStream_t)stream);
}

// fp32 tensors, the arithmetic on the bf16 matrix cores with every operand as two bf16 terms (see include/vsp_attn.h).
extern "C" size_t vsp_attn_backward_split_workspace_bytes(int32_t B, int32_t Hq, int32_t Hkv, int32_t N, int32_t D) {
    if (B <= 0 || Hq <= 0 || Hkv <= 0 || N <= 0 || D <= 0) return 0;
    const size_t rows_q = (size_t)B * (size_t)Hq * (size_t)N, rows_kv = (size_t)B * (size_t)Hkv * (size_t)N;
    return align16(2 * rows_q * sizeof(float)) + 4 * (rows_q + rows_kv) * (size_t)D * sizeof(uint16_t);   // Q, dO, K, V: hi and lo
}

extern "C" int vsp_attn_prefill_backward_split(const vsp_tensor* dout, const vsp_tensor* q, const vsp_tensor* k,
                                               const vsp_tensor* v, const vsp_tensor* out, const vsp_tensor* lse,
                                               vsp_tensor* dq, vsp_tensor* dk, vsp_tensor* dv, float scale, int is_causal,
                                               void* workspace, size_t workspace_bytes, void* stream) {
    if (!q || !k || !v) return VSP_ERR_NULL;
    if (q->ndim != 4 || k->ndim != 4 || v->ndim != 4) return VSP_ERR_NDIM;
    const int64_t B = q->shape[0], Hq = q->shape[1], N = q->shape[2], D = q->shape[3];
    const int64_t Hkv = k->shape[1];
    if (Hkv <= 0 ? Hq != 0 : (Hq % Hkv != 0)) return VSP_ERR_SHAPE;
    if (q->dtype != VSP_F32) return VSP_ERR_UNSUPPORTED;
    int rc;
    if ((rc = check4(q, B, Hq, N, D, VSP_F32)) || (rc = check4(dout, B, Hq, N, D, VSP_F32)) || (rc = check4(out, B, Hq, N, D, VSP_F32)) ||
        (rc = check4(dq, B, Hq, N, D, VSP_F32)) || (rc = check4(k, B, Hkv, N, D, VSP_F32)) || (rc = check4(v, B, Hkv, N, D, VSP_F32)) ||
        (rc = check4(dk, B, Hkv, N, D, VSP_F32)) || (rc = check4(dv, B, Hkv, N, D, VSP_F32)))
        return rc;
    if (!lse) return VSP_ERR_NULL;
    if (lse->ndim != 3 || lse->shape[0] != B || lse->shape[1] != Hq || lse->shape[2] != N) return VSP_ERR_SHAPE;
    if (lse->dtype != VSP_F32) return VSP_ERR_DTYPE;
    if (B * Hq * N * D == 0) return VSP_OK;
    if (!lse->data) return VSP_ERR_NULL;
    if (D != 64 && D != 128) return VSP_ERR_UNSUPPORTED;
    if (!(fabsf(scale) < INFINITY)) return VSP_ERR_ARG;
    if (N > INT32_MAX / 2 || (uint64_t)N * (uint64_t)D * 2u > 0x7fffffffull) return VSP_ERR_ARG;
    if (!workspace || workspace_bytes < vsp_attn_backward_split_workspace_bytes((int32_t)B, (int32_t)Hq, (int32_t)Hkv, (int32_t)N, (int32_t)D))
        return VSP_ERR_WORKSPACE;
    if (!is_aligned16(workspace)) return VSP_ERR_ALIGN;
    for (const vsp_tensor* t : {dout, q, k, v, out}) {   // rows are read in 8-byte pieces
        if (((uintptr_t)t->data & 7) != 0) return VSP_ERR_ALIGN;
        for (int i = 0; i < 3; ++i)
            if (t->stride[i] % 2 != 0) return VSP_ERR_ALIGN;
    }
    for (const vsp_tensor* t : {(const vsp_tensor*)dq, (const vsp_tensor*)dk, (const vsp_tensor*)dv}) {   // and written in 16-byte ones
        if (!is_aligned16(t->data)) return VSP_ERR_ALIGN;
        for (int i = 0; i < 3; ++i)
            if (t->stride[i] % 4 != 0) return VSP_ERR_ALIGN;
    }

    const int64_t rows_q = B * Hq * N, rows_kv = B * Hkv * N;
    SplitArgs sa{};
    sa.q = (const float*)q->data, sa.dout = (const float*)dout->data, sa.out = (const float*)out->data;
    sa.k = (const float*)k->data, sa.v = (const float*)v->data, sa.lse = (const float*)lse->data;
    for (int i = 0; i < 3; ++i) {
        sa.s_q[i] = q->stride[i], sa.s_do[i] = dout->stride[i], sa.s_o[i] = out->stride[i];
        sa.s_k[i] = k->stride[i], sa.s_v[i] = v->stride[i], sa.s_l[i] = lse->stride[i];
    }
    sa.delta = (float*)workspace;
    sa.lse2 = sa.delta + rows_q;
    sa.qh = (uint16_t*)((char*)workspace + align16(2 * (size_t)rows_q * sizeof(float)));
    sa.doh = sa.qh + 2 * rows_q * D;
    sa.kh = sa.doh + 2 * rows_q * D;
    sa.vh = sa.kh + 2 * rows_kv * D;
    sa.lo_q = rows_q * D, sa.lo_kv = rows_kv * D;
    sa.B = (int)B, sa.Hq = (int)Hq, sa.Hkv = (int)Hkv, sa.N = (int)N, sa.D = (int)D;

    BwdArgs a{};
    a.dout = sa.doh, a.q = sa.qh, a.k = sa.kh, a.v = sa.vh;
    a.dq = dq->data, a.dk = dk->data, a.dv = dv->data;
    a.delta = sa.delta, a.lse2 = sa.lse2;
    const int64_t sq[3] = {Hq * N * D, N * D, D}, skv[3] = {Hkv * N * D, N * D, D};
    for (int i = 0; i < 3; ++i) {
        a.s_do[i] = a.s_q[i] = sq[i];
        a.s_k[i] = a.s_v[i] = skv[i];
        a.s_dq[i] = dq->stride[i], a.s_dk[i] = dk->stride[i], a.s_dv[i] = dv->stride[i];
    }
    a.lo_q = sa.lo_q, a.lo_kv = sa.lo_kv;
    a.B = (int)B, a.Hq = (int)Hq, a.Hkv = (int)Hkv, a.n_rep = (int)(Hq / Hkv), a.N = (int)N;
    a.causal = is_causal ? 1 : 0;
    a.scale = scale;
    return launch_backward_split(sa, a, D, (hipStream_t)stream);
}
