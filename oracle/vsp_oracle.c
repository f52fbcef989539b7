/*
 * vsp_oracle.c — CPU restatement of the reference attention hot path.
 * TEST INFRASTRUCTURE: see vsp_oracle.h for who may use it and how each
 * function is pinned.  Build: make -C oracle oracle  (-O2 -ffp-contract=off).
 */
#include "vsp_oracle.h"

#include <math.h>
#include <stdlib.h>
#include <string.h>

const char* orc_strerror(int code) {
    switch (code) {
        case ORC_OK: return "ok";
        case ORC_ERR_NDIM: return "flash_attention: inputs must be 4D [B, H, N, D]";
        case ORC_ERR_SHAPE: return "flash_attention: Q, K, V must have same shape";
        case ORC_ERR_DTYPE: return "flash_attention: Q, K, V must have same dtype";
        case ORC_ERR_DROPOUT: return "flash_attention: dropout_p must be in [0, 1)";
        case ORC_ERR_NUMEL: return "copy_from: element count mismatch.";
        case ORC_ERR_BROADCAST: return "causal mask [T, T] cannot be broadcast onto scores [T, L]";
        case ORC_ERR_REPEAT_NDIM:
            return "repeat_kv: input must be 4D [Batch, KV_Heads, SeqLen, HeadDim]";
        case ORC_ERR_GQA_HEADS: return "GroupedQueryAttention: num_heads must be divisible by num_kv_heads";
        case ORC_ERR_GQA_EMBED: return "GroupedQueryAttention: embed_dim must be divisible by num_heads";
        case ORC_ERR_STEP: return "Slice step cannot be zero";
    }
    return "unknown";
}

static int64_t min64(int64_t a, int64_t b) { return a < b ? a : b; }
static int64_t max64(int64_t a, int64_t b) { return a > b ? a : b; }

/* ------------------------------------------------------------------------ */
/* src/ops/flash_attention.cpp:45-59: the order of the checks is the order of
 * the throws. */
int orc_flash_attention_check(int q_ndim, const int64_t* q_shape, int k_ndim, const int64_t* k_shape,
                              int v_ndim, const int64_t* v_shape, int q_dtype, int k_dtype,
                              int v_dtype, float dropout_p) {
    if (q_ndim != 4 || k_ndim != 4 || v_ndim != 4) return ORC_ERR_NDIM;
    for (int i = 0; i < 4; ++i)
        if (q_shape[i] != k_shape[i] || k_shape[i] != v_shape[i]) return ORC_ERR_SHAPE;
    if (q_dtype != k_dtype || k_dtype != v_dtype) return ORC_ERR_DTYPE;
    if (dropout_p < 0.0f || dropout_p >= 1.0f) return ORC_ERR_DROPOUT;
    return ORC_OK;
}

/* src/ops/flash_attention.cpp:218-364, inference branch (use_dropout false).
 * BLOCK_M = BLOCK_N = 32 (:252-253). */
void orc_flash_attention_f32(const float* Q, const float* K, const float* V, float* O, float* L,
                             int64_t B, int64_t H, int64_t N, int64_t D, float scale, int is_causal) {
    enum { BLOCK_M = 32, BLOCK_N = 32 };
    float* acc = (float*)malloc(sizeof(float) * BLOCK_M * (size_t)(D > 0 ? D : 1));
    float m_prev[BLOCK_M], l_prev[BLOCK_M];
    float scores[BLOCK_N];

    for (int64_t b = 0; b < B; ++b) {
        for (int64_t h = 0; h < H; ++h) {
            const float* q_ptr = Q + (b * H + h) * N * D;
            const float* k_ptr = K + (b * H + h) * N * D;
            const float* v_ptr = V + (b * H + h) * N * D;
            float* o_ptr = O + (b * H + h) * N * D;
            float* l_ptr = L ? L + (b * H + h) * N : NULL;

            for (int64_t q_start = 0; q_start < N; q_start += BLOCK_M) {
                int64_t q_end = min64(q_start + BLOCK_M, N);
                /* :270-273 */
                for (int64_t i = 0; i < BLOCK_M * D; ++i) acc[i] = 0.0f;
                for (int i = 0; i < BLOCK_M; ++i) {
                    m_prev[i] = -INFINITY;
                    l_prev[i] = 0.0f;
                }
                /* :276 */
                int64_t k_end_limit = is_causal ? min64(q_end, N) : N;

                for (int64_t k_start = 0; k_start < k_end_limit; k_start += BLOCK_N) {
                    int64_t k_end = min64(k_start + BLOCK_N, k_end_limit);
                    int64_t nk = k_end - k_start;

                    for (int64_t qi = q_start; qi < q_end; ++qi) {
                        int qi_local = (int)(qi - q_start);
                        float m_block = -INFINITY;
                        /* :291-306 */
                        for (int64_t ki = k_start; ki < k_end; ++ki) {
                            if (is_causal && ki > qi) {
                                scores[ki - k_start] = -INFINITY;
                                continue;
                            }
                            float score = 0.0f;
                            for (int64_t d = 0; d < D; ++d) score += q_ptr[qi * D + d] * k_ptr[ki * D + d];
                            score *= scale;
                            scores[ki - k_start] = score;
                            m_block = (m_block < score) ? score : m_block; /* std::max */
                        }
                        /* :309 */
                        float m_new = (m_prev[qi_local] < m_block) ? m_block : m_prev[qi_local]; /* std::max */
                        /* :312-331 */
                        float l_block = 0.0f;
                        for (int64_t i = 0; i < nk; ++i) {
                            scores[i] = expf(scores[i] - m_new);
                            l_block += scores[i];
                        }
                        /* :334-335 */
                        float scale_prev = expf(m_prev[qi_local] - m_new);
                        l_prev[qi_local] = l_prev[qi_local] * scale_prev + l_block;
                        /* :338-343 */
                        for (int64_t d = 0; d < D; ++d) {
                            acc[qi_local * D + d] *= scale_prev;
                            for (int64_t ki = k_start; ki < k_end; ++ki)
                                acc[qi_local * D + d] += scores[ki - k_start] * v_ptr[ki * D + d];
                        }
                        m_prev[qi_local] = m_new;
                    }
                }
                /* :350-360 */
                for (int64_t qi = q_start; qi < q_end; ++qi) {
                    int qi_local = (int)(qi - q_start);
                    float inv_l = 1.0f / l_prev[qi_local];
                    for (int64_t d = 0; d < D; ++d) o_ptr[qi * D + d] = acc[qi_local * D + d] * inv_l;
                    if (l_ptr) l_ptr[qi] = m_prev[qi_local] + logf(l_prev[qi_local]);
                }
            }
        }
    }
    free(acc);
}

/* src/ops/attention_ops.cpp:30-57 */
void orc_repeat_kv_f32(const float* in, float* out, int64_t B, int64_t KV_H, int64_t S, int64_t D,
                       int64_t n_rep) {
    int64_t Q_H = KV_H * n_rep;
    for (int64_t b = 0; b < B; ++b)
        for (int64_t q_h = 0; q_h < Q_H; ++q_h) {
            int64_t kv_h = q_h / n_rep;
            for (int64_t s = 0; s < S; ++s)
                for (int64_t d = 0; d < D; ++d) {
                    int64_t in_idx = ((b * KV_H + kv_h) * S + s) * D + d;
                    int64_t out_idx = ((b * Q_H + q_h) * S + s) * D + d;
                    out[out_idx] = in[in_idx];
                }
        }
}

int orc_sdpa_matmul_f32(const float* q, const float* k, const int64_t* ks, const float* v,
                        const int64_t* vs, float* out, int64_t B, int64_t H, int64_t T, int64_t L,
                        int64_t D, int64_t n_rep, int is_causal) {
    /* src/nn/functional.cpp:406-410: mask is [T,T]; adding it to [B,H,T,L]
     * broadcasts only when L == T or T == 1. */
    if (is_causal && T != L && T != 1) return ORC_ERR_BROADCAST;
    float* scores = (float*)malloc(sizeof(float) * (size_t)(T * L > 0 ? T * L : 1));
    float sqrt_dk = sqrtf((float)D); /* :403 */
    for (int64_t b = 0; b < B; ++b) {
        for (int64_t h = 0; h < H; ++h) {
            int64_t kvh = h / n_rep; /* src/ops/attention_ops.cpp:47 */
            const float* qp = q + (b * H + h) * T * D;
            const float* kp = k + b * ks[0] + kvh * ks[1];
            const float* vp = v + b * vs[0] + kvh * vs[1];
            float* op = out + (b * H + h) * T * D;
            /* scores = q @ k^T, src/ops/gemm.cpp:254-279 */
            for (int64_t m = 0; m < T; ++m)
                for (int64_t n = 0; n < L; ++n) {
                    float sum = 0.0f;
                    for (int64_t kk = 0; kk < D; ++kk) sum += qp[m * D + kk] * kp[n * ks[2] + kk * ks[3]];
                    scores[m * L + n] = sum;
                }
            /* scores / sqrt(d_k), src/ops/cpu/elementwise_cpu.cpp:93-95 */
            for (int64_t i = 0; i < T * L; ++i) scores[i] = scores[i] / sqrt_dk;
            /* + mask, src/nn/functional.cpp:36-52 (0 or -inf; T==1 mask is [[0]]) */
            if (is_causal) {
                for (int64_t m = 0; m < T; ++m)
                    for (int64_t n = 0; n < L; ++n) {
                        float mk = (T == 1) ? 0.0f : ((n > m) ? -INFINITY : 0.0f);
                        scores[m * L + n] = scores[m * L + n] + mk;
                    }
            }
            /* softmax(-1), src/ops/normalization.cpp:88-118 */
            for (int64_t m = 0; m < T; ++m) {
                float* row = scores + m * L;
                float max_val = -INFINITY;
                for (int64_t j = 0; j < L; ++j)
                    if (row[j] > max_val) max_val = row[j];
                float sum_exp = 0.0f;
                for (int64_t j = 0; j < L; ++j) sum_exp += expf(row[j] - max_val);
                for (int64_t j = 0; j < L; ++j) row[j] = expf(row[j] - max_val) / sum_exp;
            }
            /* probs @ v, src/ops/gemm.cpp:254-279 */
            for (int64_t m = 0; m < T; ++m)
                for (int64_t n = 0; n < D; ++n) {
                    float sum = 0.0f;
                    for (int64_t kk = 0; kk < L; ++kk) sum += scores[m * L + kk] * vp[kk * vs[2] + n * vs[3]];
                    op[m * D + n] = sum;
                }
        }
    }
    free(scores);
    return ORC_OK;
}

static void contiguous_strides(int64_t H, int64_t L, int64_t D, int64_t* s) {
    s[3] = 1;
    s[2] = D;
    s[1] = L * D;
    s[0] = H * L * D;
}

/* src/nn/functional.cpp:370-422 */
int orc_sdpa_f32(const float* q, const float* k, const float* v, float* out, int64_t B, int64_t H,
                 int64_t T, int64_t L, int64_t D, int is_causal) {
    if (T >= 512) { /* FLASH_ATTENTION_THRESHOLD, :385 */
        if (T != L) return ORC_ERR_SHAPE; /* src/ops/flash_attention.cpp:49-51 */
        float scale = 1.0f / sqrtf((float)D); /* :388 */
        orc_flash_attention_f32(q, k, v, out, NULL, B, H, T, D, scale, is_causal);
        return ORC_OK;
    }
    int64_t s[4];
    contiguous_strides(H, L, D, s);
    return orc_sdpa_matmul_f32(q, k, s, v, s, out, B, H, T, L, D, 1, is_causal);
}

int orc_gqa_attention_f32(const float* q, const float* k, const int64_t* ks, const float* v,
                          const int64_t* vs, float* out, int64_t B, int64_t Hq, int64_t T, int64_t L,
                          int64_t D, int64_t n_rep, int is_causal) {
    if (T < 512) return orc_sdpa_matmul_f32(q, k, ks, v, vs, out, B, Hq, T, L, D, n_rep, is_causal);
    if (T != L) return ORC_ERR_SHAPE;
    /* flash branch: heads are independent, so run it per (b, h) on a
     * contiguous copy of the kv head that repeat_kv would have produced. */
    float scale = 1.0f / sqrtf((float)D);
    float* kc = (float*)malloc(sizeof(float) * (size_t)(L * D));
    float* vc = (float*)malloc(sizeof(float) * (size_t)(L * D));
    for (int64_t b = 0; b < B; ++b)
        for (int64_t h = 0; h < Hq; ++h) {
            int64_t kvh = h / n_rep;
            for (int64_t s = 0; s < L; ++s)
                for (int64_t d = 0; d < D; ++d) {
                    kc[s * D + d] = k[b * ks[0] + kvh * ks[1] + s * ks[2] + d * ks[3]];
                    vc[s * D + d] = v[b * vs[0] + kvh * vs[1] + s * vs[2] + d * vs[3]];
                }
            orc_flash_attention_f32(q + (b * Hq + h) * T * D, kc, vc, out + (b * Hq + h) * T * D, NULL,
                                    1, 1, T, D, scale, is_causal);
        }
    free(kc);
    free(vc);
    return ORC_OK;
}

/* src/nn/gqa_attention.cpp:38-57: head_dim and num_rep are integer divisions
 * made before the divisibility checks. */
int orc_gqa_config(int64_t embed_dim, int64_t num_heads, int64_t num_kv_heads, int64_t* head_dim,
                   int64_t* num_rep) {
    if (num_heads % num_kv_heads != 0) return ORC_ERR_GQA_HEADS;
    if (embed_dim % num_heads != 0) return ORC_ERR_GQA_EMBED;
    if (head_dim) *head_dim = embed_dim / num_heads;
    if (num_rep) *num_rep = num_heads / num_kv_heads;
    return ORC_OK;
}

/* ------------------------------------------------------------------------ */
/* The output projection of the attention modules: out = wo_.forward(out) with out [B, T, C_in]
 * (src/nn/gqa_attention.cpp:151-152, src/nn/transformer.cpp:148-151,207-210).  Linear::forward
 * (src/nn/linear.cpp:41-49) is ops::matmul(input, weight.transpose(0, 1)) followed by ops::add(output, bias);
 * a 3-D input against a 2-D weight takes gemm's batched branch (src/ops/gemm.cpp:130-138), whose CPU loop
 * (:254-279) sums the K products of every output element in index order into one fp32 accumulator.
 * x [M, K] (M = B * T rows), w [N, K] = Linear::weight, bias [N] or NULL, y [M, N]. */
void orc_linear_f32(const float* x, const float* w, const float* bias, float* y, int64_t M, int64_t K, int64_t N) {
    for (int64_t m = 0; m < M; ++m)
        for (int64_t n = 0; n < N; ++n) {
            float sum = 0.0f;
            for (int64_t k = 0; k < K; ++k) sum += x[m * K + k] * w[n * K + k];
            y[m * N + n] = bias ? sum + bias[n] : sum;
        }
}

/* ------------------------------------------------------------------------ */
/* src/ops/view_ops.cpp:266-316 */
int orc_slice_bounds(int64_t dim_size, int has_start, int64_t start_in, int has_stop, int64_t stop_in,
                     int has_step, int64_t step_in, int64_t* out_start, int64_t* out_len) {
    int64_t step = has_step ? step_in : 1;
    if (step == 0) return ORC_ERR_STEP;
    int64_t start = has_start ? start_in : (step > 0 ? 0 : dim_size - 1);
    int64_t stop = has_stop ? stop_in : (step > 0 ? dim_size : -1);
    if (start < 0) start += dim_size;
    if (stop < 0) stop += dim_size;
    int64_t len;
    if (step > 0) {
        start = max64(0, min64(start, dim_size));
        stop = max64(0, min64(stop, dim_size));
        if (start >= stop) {
            *out_start = start;
            *out_len = 0;
            return ORC_OK;
        }
        len = (stop - start + step - 1) / step;
    } else {
        start = max64(0, min64(start, dim_size - 1));
        stop = max64(-1, min64(stop, dim_size - 1));
        if (start <= stop) {
            *out_start = start;
            *out_len = 0;
            return ORC_OK;
        }
        len = (stop - start + step + 1) / step;
    }
    *out_start = start;
    *out_len = len;
    return ORC_OK;
}

orc_kv_cache* orc_kv_new(int64_t B, int64_t H, int64_t S_max, int64_t D) {
    orc_kv_cache* c = (orc_kv_cache*)calloc(1, sizeof(orc_kv_cache));
    size_t n = (size_t)(B * H * S_max * D);
    c->k = (float*)calloc(n ? n : 1, sizeof(float)); /* vesper::zeros, src/nn/transformer.cpp:40-41 */
    c->v = (float*)calloc(n ? n : 1, sizeof(float));
    c->B = B;
    c->H = H;
    c->S_max = S_max;
    c->D = D;
    c->current_len = 0;
    return c;
}
void orc_kv_free(orc_kv_cache* c) {
    if (!c) return;
    free(c->k);
    free(c->v);
    free(c);
}
void orc_kv_reset(orc_kv_cache* c) {
    size_t n = (size_t)(c->B * c->H * c->S_max * c->D);
    c->current_len = 0;
    memset(c->k, 0, n * sizeof(float));
    memset(c->v, 0, n * sizeof(float));
}

/* src/ops/cpu/copy_cpu.cpp:8-76 for a contiguous source and a 4-D strided
 * destination of equal element count: destination element i (row-major over
 * dst_shape) receives source element i. */
static void copy_into_slot(const float* src, float* dst_base, const int64_t* dst_shape,
                           const int64_t* dst_strides) {
    int64_t n = dst_shape[0] * dst_shape[1] * dst_shape[2] * dst_shape[3];
    for (int64_t i = 0; i < n; ++i) {
        int64_t remaining = i, offset_out = 0;
        for (int d = 3; d >= 0; --d) {
            int64_t coord = remaining % dst_shape[d];
            remaining /= dst_shape[d];
            offset_out += coord * dst_strides[d];
        }
        dst_base[offset_out] = src[i];
    }
}

/* src/nn/transformer.cpp:56-93 (KVCache) == src/nn/gqa_attention.cpp:175-207 (GQAKVCache) */
int orc_kv_update(orc_kv_cache* c, const float* new_k, const float* new_v, int64_t nB, int64_t nH,
                  int64_t T, int64_t nD, int64_t start_pos, int64_t* view) {
    int64_t strides[4] = {c->H * c->S_max * c->D, c->S_max * c->D, c->D, 1};
    int64_t s_start, s_len;
    /* selectors {Slice(), Slice(), Slice(start_pos, start_pos+T), Slice()} */
    orc_slice_bounds(c->S_max, 1, start_pos, 1, start_pos + T, 1, 1, &s_start, &s_len);
    int64_t slot_shape[4] = {c->B, c->H, s_len, c->D};
    int64_t slot_numel = c->B * c->H * s_len * c->D;
    /* Tensor::copy_from, src/core/tensor.cpp:198-200 */
    if (slot_numel != nB * nH * T * nD) return ORC_ERR_NUMEL;
    if (slot_numel > 0) {
        int64_t off = s_start * strides[2];
        copy_into_slot(new_k, c->k + off, slot_shape, strides);
        copy_into_slot(new_v, c->v + off, slot_shape, strides);
    }
    /* :73 */
    c->current_len = max64(c->current_len, start_pos + T);
    if (view) {
        int64_t v_start, v_len;
        orc_slice_bounds(c->S_max, 1, 0, 1, c->current_len, 1, 1, &v_start, &v_len);
        view[0] = c->B;
        view[1] = c->H;
        view[2] = v_len;
        view[3] = c->D;
        for (int i = 0; i < 4; ++i) view[4 + i] = strides[i];
        view[8] = v_len > 0 ? v_start * strides[2] : 0;
    }
    return ORC_OK;
}

/* ------------------------------------------------------------------------ */
/* include/vesper/core/half.h:162-173 */
uint16_t orc_f32_to_bf16(float f) {
    uint32_t bits;
    memcpy(&bits, &f, sizeof bits);
    uint32_t rounding_bias = 0x7FFFu + ((bits >> 16) & 1u);
    bits += rounding_bias;
    return (uint16_t)(bits >> 16);
}
/* include/vesper/core/half.h:175-181 */
float orc_bf16_to_f32(uint16_t b) {
    uint32_t bits = (uint32_t)b << 16;
    float r;
    memcpy(&r, &bits, sizeof r);
    return r;
}
void orc_f32_to_bf16_array(const float* in, uint16_t* out, int64_t n) {
    for (int64_t i = 0; i < n; ++i) out[i] = orc_f32_to_bf16(in[i]);
}
void orc_bf16_to_f32_array(const uint16_t* in, float* out, int64_t n) {
    for (int64_t i = 0; i < n; ++i) out[i] = orc_bf16_to_f32(in[i]);
}

/* IEEE 754 binary32 -> binary16, round-to-nearest-even. */
uint16_t orc_f32_to_f16(float f) {
    uint32_t x;
    memcpy(&x, &f, sizeof x);
    uint32_t sign = (x >> 16) & 0x8000u;
    uint32_t exp = (x >> 23) & 0xFFu;
    uint32_t man = x & 0x7FFFFFu;
    if (exp == 0xFFu) return (uint16_t)(sign | 0x7C00u | (man ? (0x200u | (man >> 13)) : 0u));
    int32_t e = (int32_t)exp - 127 + 15;
    if (e >= 31) return (uint16_t)(sign | 0x7C00u); /* overflow -> inf */
    if (e <= 0) {
        if (e < -10) return (uint16_t)sign; /* underflow -> 0 */
        man |= 0x800000u;
        uint32_t shift = (uint32_t)(14 - e); /* 14..24 */
        uint32_t half = man >> shift;
        uint32_t rem = man & ((1u << shift) - 1u);
        uint32_t halfway = 1u << (shift - 1);
        if (rem > halfway || (rem == halfway && (half & 1u))) ++half;
        return (uint16_t)(sign | half);
    }
    uint32_t half = (uint32_t)(e << 10) | (man >> 13);
    uint32_t rem = man & 0x1FFFu;
    if (rem > 0x1000u || (rem == 0x1000u && (half & 1u))) ++half; /* may carry into exponent/inf */
    return (uint16_t)(sign | half);
}
float orc_f16_to_f32(uint16_t h) {
    uint32_t sign = ((uint32_t)h & 0x8000u) << 16;
    uint32_t exp = (h >> 10) & 0x1Fu;
    uint32_t man = h & 0x3FFu;
    uint32_t x;
    if (exp == 0) {
        if (man == 0) {
            x = sign;
        } else {
            int e = -1;
            do {
                ++e;
                man <<= 1;
            } while (!(man & 0x400u));
            man &= 0x3FFu;
            x = sign | (uint32_t)(127 - 15 - e) << 23 | (man << 13);
        }
    } else if (exp == 31) {
        x = sign | 0x7F800000u | (man << 13);
    } else {
        x = sign | ((exp - 15 + 127) << 23) | (man << 13);
    }
    float f;
    memcpy(&f, &x, sizeof f);
    return f;
}

void orc_q8_0_quantize_row(const float* x, int64_t n, uint16_t* d, int8_t* qs) {
    int64_t nb = n / 32;
    for (int64_t i = 0; i < nb; ++i) {
        float amax = 0.0f;
        for (int j = 0; j < 32; ++j) {
            float a = fabsf(x[i * 32 + j]);
            if (a > amax) amax = a;
        }
        float dd = amax / 127.0f;
        float id = dd ? 1.0f / dd : 0.0f;
        d[i] = orc_f32_to_f16(dd);
        for (int j = 0; j < 32; ++j) qs[i * 32 + j] = (int8_t)roundf(x[i * 32 + j] * id);
    }
}
void orc_q8_0_dequantize_row(const uint16_t* d, const int8_t* qs, int64_t n, float* x) {
    int64_t nb = n / 32;
    for (int64_t i = 0; i < nb; ++i) {
        float dd = orc_f16_to_f32(d[i]);
        for (int j = 0; j < 32; ++j) x[i * 32 + j] = (float)qs[i * 32 + j] * dd;
    }
}

/* ---- rotary position embedding ----------------------------------------- */

/* src/nn/functional.cpp:424-443.  `-2.0f * i / dim` is evaluated in float left to right
 * ((-2.0f * (float)i) / (float)dim); std::pow(float, float) is powf; `pos * freq` converts the int
 * position to float. */
void orc_rope_angles(int seq_len, int head_dim, int start_pos, float theta, float* angles) {
    const int half = head_dim / 2;
    for (int m = 0; m < seq_len; ++m) {
        const int pos = start_pos + m;
        for (int i = 0; i < half; ++i) {
            const float freq = powf(theta, -2.0f * (float)i / (float)head_dim);
            angles[(int64_t)m * half + i] = (float)pos * freq;
        }
    }
}

/* src/nn/functional.cpp:445-494. */
void orc_rope_apply_f32(const float* x, int64_t B, int64_t H, int64_t S, int64_t D, const float* angles,
                        float* out) {
    const int64_t half = D / 2;
    for (int64_t bh = 0; bh < B * H; ++bh)
        for (int64_t s = 0; s < S; ++s)
            for (int64_t i = 0; i < half; ++i) {
                const float a = angles[s * half + i];
                const float c = cosf(a), sn = sinf(a);
                const int64_t o = (bh * S + s) * D + 2 * i;
                const float x0 = x[o], x1 = x[o + 1];
                const float t1 = x0 * c, t2 = x1 * sn, t3 = x0 * sn, t4 = x1 * c;
                out[o] = t1 - t2;
                out[o + 1] = t3 + t4;
            }
}

/* ---- attention backward -------------------------------------------------- */

/* src/ops/flash_attention.cpp:366-482, dropout off. */
void orc_flash_attention_backward_f32(const float* dO, const float* Q, const float* K, const float* V,
                                      const float* O, const float* Lse, float* dQ, float* dK, float* dV,
                                      int64_t B, int64_t H, int64_t N, int64_t D, float scale, int is_causal) {
    const int64_t total = B * H * N * D;
    for (int64_t i = 0; i < total; ++i) dQ[i] = dK[i] = dV[i] = 0.0f;
    float* Di = (float*)malloc(sizeof(float) * (size_t)(N > 0 ? N : 1));
    for (int64_t b = 0; b < B; ++b) {
        for (int64_t h = 0; h < H; ++h) {
            const int64_t off = (b * H + h) * N * D;
            const float *q_ptr = Q + off, *k_ptr = K + off, *v_ptr = V + off, *o_ptr = O + off, *do_ptr = dO + off;
            const float* l_ptr = Lse + (b * H + h) * N;
            float *dq_ptr = dQ + off, *dk_ptr = dK + off, *dv_ptr = dV + off;
            for (int64_t i = 0; i < N; ++i) {
                float sum = 0.0f;
                for (int64_t d = 0; d < D; ++d) sum += do_ptr[i * D + d] * o_ptr[i * D + d];
                Di[i] = sum;
            }
            for (int64_t qi = 0; qi < N; ++qi) {
                const float li = l_ptr[qi];
                const int64_t k_end = is_causal ? qi + 1 : N;
                for (int64_t ki = 0; ki < k_end; ++ki) {
                    float score = 0.0f;
                    for (int64_t d = 0; d < D; ++d) score += q_ptr[qi * D + d] * k_ptr[ki * D + d];
                    score *= scale;
                    const float p = expf(score - li);
                    for (int64_t d = 0; d < D; ++d) dv_ptr[ki * D + d] += p * do_ptr[qi * D + d];
                    float dp = 0.0f;
                    for (int64_t d = 0; d < D; ++d) dp += do_ptr[qi * D + d] * v_ptr[ki * D + d];
                    const float ds = p * (dp - Di[qi]);
                    for (int64_t d = 0; d < D; ++d) {
                        dq_ptr[qi * D + d] += scale * ds * k_ptr[ki * D + d];
                        dk_ptr[ki * D + d] += scale * ds * q_ptr[qi * D + d];
                    }
                }
            }
        }
    }
    free(Di);
}
