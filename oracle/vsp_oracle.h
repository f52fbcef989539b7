/*
 * vsp_oracle — CPU restatement of the reference's attention hot path.
 *
 * THIS IS TEST INFRASTRUCTURE.  Only tests/, __graft_entry__.smoke() and the
 * cpu_baseline leg of bench.py may load it, and only as the checker.  The
 * product (libvsp_attn.so and everything under vesper_amd/) never links,
 * imports or calls anything in this directory.
 *
 * Every function follows one reference function operation for operation
 * (same loop nests, same accumulation order, same libm calls) and cites it.
 * Compile with -O2 -ffp-contract=off (see Makefile) so that fp32 results are
 * the bits the reference's own CPU build produces on x86-64.
 *
 * How each function is pinned (tests/test_oracle_*.py):
 *   orc_flash_attention_f32   bit-exact vs oracle/_ref (the compiled reference)
 *                             and vs tests/golden fixtures written from it;
 *                             float64 closed form; the reference tests' known
 *                             answers (identity/causal-prefix/constant-V/...).
 *   orc_sdpa_f32 / _matmul    same.
 *   orc_flash_attention_backward_f32  bit-exact vs oracle/_ref (flash_attention_backward) and a fixture
 *                             written from it; float64 closed-form gradients; central finite
 *                             differences of the forward (the reference's own gradient check).
 *   orc_repeat_kv_f32         bit-exact vs _ref; iota head-map known answer.
 *   orc_gqa_attention_f32     bit-identical to repeat_kv -> sdpa by test.
 *   orc_slice_bounds,
 *   orc_kv_update/_reset      exact vs _ref KVCache and GQAKVCache, the
 *                             reference tests' exact append values, and a
 *                             brute-force 4-D array model.
 *   orc_f32_to_bf16           bit-exact vs _ref BFloat16 and vs an independent
 *                             round-to-nearest-even implementation.
 *   orc_q8_0_*, orc_f32_to_f16,
 *   orc_f16_to_f32            NOT in the reference (it has no quantised cache):
 *                             "parity unpinned" at the reference.  Pinned to the
 *                             published ggml block_q8_0 arithmetic by closed-form
 *                             known answers and to numpy's IEEE float16 cast.
 */
#ifndef VSP_ORACLE_H
#define VSP_ORACLE_H

#include <stddef.h>
#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

/* error codes; orc_strerror() gives the reference's exception text */
enum {
    ORC_OK = 0,
    ORC_ERR_NDIM = 1,        /* "flash_attention: inputs must be 4D [B, H, N, D]" */
    ORC_ERR_SHAPE = 2,       /* "flash_attention: Q, K, V must have same shape" */
    ORC_ERR_DTYPE = 3,       /* "flash_attention: Q, K, V must have same dtype" */
    ORC_ERR_DROPOUT = 4,     /* "flash_attention: dropout_p must be in [0, 1)" */
    ORC_ERR_NUMEL = 5,       /* "copy_from: element count mismatch." */
    ORC_ERR_BROADCAST = 6,   /* causal mask [T,T] does not broadcast onto [T,L] */
    ORC_ERR_REPEAT_NDIM = 7, /* "repeat_kv: input must be 4D [Batch, KV_Heads, SeqLen, HeadDim]" */
    ORC_ERR_GQA_HEADS = 8,   /* num_heads not divisible by num_kv_heads */
    ORC_ERR_GQA_EMBED = 9,   /* embed_dim not divisible by num_heads */
    ORC_ERR_STEP = 10        /* "Slice step cannot be zero" */
};
const char* orc_strerror(int code);

/* ---- attention ---------------------------------------------------------- */

/* ops::flash_attention front-end validation, src/ops/flash_attention.cpp:45-59.
 * shapes are given as (ndim, dims[]) triples; dtype codes are compared only. */
int orc_flash_attention_check(int q_ndim, const int64_t* q_shape, int k_ndim, const int64_t* k_shape,
                              int v_ndim, const int64_t* v_shape, int q_dtype, int k_dtype,
                              int v_dtype, float dropout_p);

/* flash_attention_cpu_dispatch, src/ops/flash_attention.cpp:218-364 (inference:
 * use_dropout == false).  Contiguous [B,H,N,D]; lse [B,H,N] may be NULL. */
void orc_flash_attention_f32(const float* q, const float* k, const float* v, float* out, float* lse,
                             int64_t B, int64_t H, int64_t N, int64_t D, float scale, int is_causal);

/* flash_attention_backward_cpu_dispatch, src/ops/flash_attention.cpp:366-482 (no dropout): contiguous
 * [B,H,N,D] operands, lse [B,H,N]; dq, dk, dv are OVERWRITTEN (the reference allocates them as zeros,
 * :178-181, and accumulates).  Di = rowsum(dO*O); for every (qi, ki <= qi if causal): p = expf(q.k*scale - lse),
 * dV[ki] += p*dO[qi], dP = dO[qi].V[ki], dS = p*(dP - Di), dQ[qi] += scale*dS*K[ki], dK[ki] += scale*dS*Q[qi],
 * all in the reference's loop order. */
void orc_flash_attention_backward_f32(const float* dout, const float* q, const float* k, const float* v,
                                      const float* out, const float* lse, float* dq, float* dk, float* dv,
                                      int64_t B, int64_t H, int64_t N, int64_t D, float scale, int is_causal);

/* ops::repeat_kv, src/ops/attention_ops.cpp:30-57 (CPU dispatch) and :92-155. */
void orc_repeat_kv_f32(const float* in, float* out, int64_t B, int64_t Hkv, int64_t S, int64_t D,
                       int64_t n_rep);

/* The non-flash branch of scaled_dot_product_attention, src/nn/functional.cpp:397-421:
 * scores = q @ k^T (src/ops/gemm.cpp:254-279: k ascending, one accumulator),
 * scores / sqrt(D) (src/ops/cpu/elementwise_cpu.cpp:93-95), + mask[T,T] of 0/-inf
 * (src/nn/functional.cpp:36-52), softmax over the last dim in three passes
 * (src/ops/normalization.cpp:88-118), probs @ v.
 * q is contiguous [B,H,T,D]; k and v are [B,H/n_rep,L,D] addressed through
 * element strides ks[4], vs[4] (so cache views can be passed as they are);
 * query head h reads kv head h / n_rep (repeat_kv folded in, a pure copy).
 * Returns ORC_ERR_BROADCAST when is_causal and T != L and T != 1. */
int orc_sdpa_matmul_f32(const float* q, const float* k, const int64_t* ks, const float* v,
                        const int64_t* vs, float* out, int64_t B, int64_t H, int64_t T, int64_t L,
                        int64_t D, int64_t n_rep, int is_causal);

/* scaled_dot_product_attention, src/nn/functional.cpp:370-422: T >= 512 routes
 * to flash_attention with scale 1/sqrt(D) (needs L == T, else ORC_ERR_SHAPE),
 * otherwise the matmul branch above.  Contiguous q [B,H,T,D], k,v [B,H,L,D]. */
int orc_sdpa_f32(const float* q, const float* k, const float* v, float* out, int64_t B, int64_t H,
                 int64_t T, int64_t L, int64_t D, int is_causal);

/* repeat_kv(k), repeat_kv(v) -> scaled_dot_product_attention, the attention
 * core of GroupedQueryAttention::forward (src/nn/gqa_attention.cpp:91-96 and
 * :140-148), without materialising the repeat.  k,v: [B,Hq/n_rep,L,D] strided.
 * For T >= 512 the flash branch runs on gathered per-head contiguous copies. */
int orc_gqa_attention_f32(const float* q, const float* k, const int64_t* ks, const float* v,
                          const int64_t* vs, float* out, int64_t B, int64_t Hq, int64_t T, int64_t L,
                          int64_t D, int64_t n_rep, int is_causal);

/* GroupedQueryAttention constructor checks, src/nn/gqa_attention.cpp:38-57. */
/* Linear::forward on a 3-D activation (the modules' output projection wo_ / c_proj): y = x w^T + bias,
 * src/nn/linear.cpp:41-49 over src/ops/gemm.cpp:254-279.  Pinned bit-exact to the compiled reference
 * (tests/test_oracle_linear.py) and to a float64 product within rounding. */
void orc_linear_f32(const float* x, const float* w, const float* bias, float* y, int64_t M, int64_t K, int64_t N);

int orc_gqa_config(int64_t embed_dim, int64_t num_heads, int64_t num_kv_heads, int64_t* head_dim,
                   int64_t* num_rep);

/* ---- KV cache ----------------------------------------------------------- */

/* One Slice selector of ops::index, src/ops/view_ops.cpp:266-316.  has_* say
 * whether start/stop/step were given.  Writes the clamped start and the length
 * (0 for an empty slice; start is then left at the clamped value). */
int orc_slice_bounds(int64_t dim_size, int has_start, int64_t start, int has_stop, int64_t stop,
                     int has_step, int64_t step, int64_t* out_start, int64_t* out_len);

/* nn::KVCache / nn::GQAKVCache: fp32 [B,H,S_max,D], zero-initialised, one length
 * for the whole batch (src/nn/transformer.cpp:32-43, src/nn/gqa_attention.cpp:165-173). */
typedef struct {
    float* k;
    float* v;
    int64_t B, H, S_max, D;
    int64_t current_len;
} orc_kv_cache;

orc_kv_cache* orc_kv_new(int64_t B, int64_t H, int64_t S_max, int64_t D);
void orc_kv_free(orc_kv_cache* c);
/* reset(): length 0 and data zeroed, src/nn/transformer.cpp:45-54. */
void orc_kv_reset(orc_kv_cache* c);
/* update(new_k,new_v,start_pos), src/nn/transformer.cpp:56-93: writes
 * [:, :, start_pos:start_pos+T, :] through ops::index + Tensor::copy_from
 * (src/core/tensor.cpp:197-228, src/ops/cpu/copy_cpu.cpp:8-76), then
 * current_len = max(current_len, start_pos+T).  new_* are contiguous
 * [nB,nH,T,D].  On success view[0..3] = shape, view[4..7] = strides (elements),
 * view[8] = offset of the returned [:, :, 0:current_len, :] view.
 * ORC_ERR_NUMEL when the clamped slot does not hold exactly nB*nH*T*D elements. */
int orc_kv_update(orc_kv_cache* c, const float* new_k, const float* new_v, int64_t nB, int64_t nH,
                  int64_t T, int64_t nD, int64_t start_pos, int64_t* view);

/* ---- number formats ----------------------------------------------------- */

/* BFloat16(float), include/vesper/core/half.h:162-173 (device twin
 * src/ops/hip/cast.hip:28-34): bits += 0x7FFF + ((bits >> 16) & 1); >> 16. */
uint16_t orc_f32_to_bf16(float f);
/* BFloat16::operator float, include/vesper/core/half.h:175-181. */
float orc_bf16_to_f32(uint16_t b);
void orc_f32_to_bf16_array(const float* in, uint16_t* out, int64_t n);
void orc_bf16_to_f32_array(const uint16_t* in, float* out, int64_t n);

/* IEEE binary16 <-> binary32, round-to-nearest-even, subnormals kept.
 * (Not the reference's Float16(float), which truncates: half.h:56.) */
uint16_t orc_f32_to_f16(float f);
float orc_f16_to_f32(uint16_t h);

/* Q8_0 rows (ggml block_q8_0 arithmetic; no counterpart in the reference):
 * per 32 consecutive elements amax = max|x|, d = amax/127 (fp32),
 * id = d ? 1/d : 0, q_i = (int8) roundf(x_i * id), scale stored as fp16 RNE(d);
 * dequant x_i = q_i * f16->f32(scale).  n must be a multiple of 32. */
void orc_q8_0_quantize_row(const float* x, int64_t n, uint16_t* d, int8_t* qs);
void orc_q8_0_dequantize_row(const uint16_t* d, const int8_t* qs, int64_t n, float* x);

/* ---- rotary position embedding (the step before the cache append) ------ */

/* compute_rope_frequencies(seq_len, head_dim, start_pos, theta), src/nn/functional.cpp:424-443:
 * angles[m][i] = (float)(start_pos + m) * powf(theta, -2.0f * i / head_dim), i < head_dim/2. */
void orc_rope_angles(int seq_len, int head_dim, int start_pos, float theta, float* angles);
/* apply_rotary_emb(x, freqs), src/nn/functional.cpp:445-494, x [B,H,S,D] contiguous, angles [S][D/2]:
 * pairs (2i, 2i+1); c = cosf(angle), s = sinf(angle) (ops::cos / ops::sin = std::cos / std::sin on
 * float, src/ops/elementwise.cpp:1039-1045); out[2i] = x0*c - x1*s, out[2i+1] = x0*s + x1*c with
 * every product and the sum rounded separately (separate elementwise ops, no fused multiply-add). */
void orc_rope_apply_f32(const float* x, int64_t B, int64_t H, int64_t S, int64_t D, const float* angles,
                        float* out);

#ifdef __cplusplus
}
#endif
#endif /* VSP_ORACLE_H */
