/*
 * vsp_attn.h — C ABI of libvsp_attn.so: the MI355X (gfx950) implementation of
 * the reference's attention hot path (causal GQA flash-attention prefill,
 * single-token decode over the KV cache, KV-cache append/read).
 *
 * The reference (danielmriley/vesper) has no FFI; its operator seam is a set
 * of C++ per-backend dispatch functions declared in public headers.  Each
 * entry point below names the reference interface it replaces (paths relative
 * to the reference tree).  The C++ mirror of those interfaces — same names,
 * argument meaning and exceptions — lives in vesper_amd/csrc/adapter/ and is
 * implemented on top of exactly these calls.
 *
 * Conventions
 *   - plain pointers and sizes only; every pointer in a vsp_tensor / vsp_kv_cache
 *     is DEVICE memory owned by the caller; the library never allocates, never
 *     frees and never keeps a pointer after a call returns;
 *   - all work is enqueued asynchronously on `stream` (a hipStream_t passed as
 *     void*; NULL = the null stream), the way the reference enqueues on
 *     Stream::current(Device::HIP) (src/core/stream.cpp:104-166).  No call
 *     synchronises;
 *   - strides are in ELEMENTS, like Tensor::strides() (include/vesper/core/tensor.h:30);
 *   - every call returns a vsp_status; nothing throws across the boundary.
 *     vsp_status_str() returns, where one exists, the reference's exception text.
 */
#ifndef VSP_ATTN_H
#define VSP_ATTN_H

#include <stddef.h>
#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

#define VSP_ATTN_ABI_VERSION 2

typedef enum {
    VSP_OK = 0,
    /* the reference's own failures (text identical to its exceptions) */
    VSP_ERR_NDIM = 1,        /* flash_attention: inputs must be 4D [B, H, N, D]        (src/ops/flash_attention.cpp:45-47) */
    VSP_ERR_SHAPE = 2,       /* flash_attention: Q, K, V must have same shape          (:49-51; GQA-aware, see vsp_attn_prefill) */
    VSP_ERR_DTYPE = 3,       /* flash_attention: Q, K, V must have same dtype          (:53-55) */
    VSP_ERR_DROPOUT = 4,     /* flash_attention: dropout_p must be in [0, 1)           (:57-59) */
    VSP_ERR_NUMEL = 5,       /* copy_from: element count mismatch.                     (src/core/tensor.cpp:198-200) */
    VSP_ERR_COPY_DTYPE = 6,  /* copy_from: dtype mismatch.                             (src/core/tensor.cpp:201-203) */
    VSP_ERR_REPEAT_NDIM = 7, /* repeat_kv: input must be 4D [...]                      (src/ops/attention_ops.cpp:97-99) */
    VSP_ERR_GQA_HEADS = 8,   /* GroupedQueryAttention: num_heads ... divisible by num_kv_heads (src/nn/gqa_attention.cpp:47-51) */
    VSP_ERR_GQA_EMBED = 9,   /* GroupedQueryAttention: embed_dim ... divisible by num_heads    (:52-56) */
    VSP_ERR_BROADCAST = 10,  /* causal mask [T,T] cannot be added to scores [T,L]      (src/nn/functional.cpp:406-410) */
    /* failures that only exist at this boundary */
    VSP_ERR_NULL = 32,        /* a required pointer is NULL */
    VSP_ERR_UNSUPPORTED = 33, /* dtype/format/head_dim combination the kernels do not implement */
    VSP_ERR_STRIDE = 34,      /* innermost stride != 1, or a stride the kernel cannot address */
    VSP_ERR_ALIGN = 35,       /* a base pointer or row pitch is not 16-byte aligned */
    VSP_ERR_WORKSPACE = 36,   /* workspace missing or smaller than vsp_attn_decode_workspace_bytes() */
    VSP_ERR_ARG = 37,         /* an argument is out of range (negative size, len > S_max, ...) */
    VSP_ERR_LAUNCH = 38       /* the HIP runtime rejected a launch (hipGetLastError text via vsp_last_hip_error) */
} vsp_status;

typedef enum {
    VSP_F32 = 0,  /* DType::Float32  (include/vesper/core/dtype.h:9-16) */
    VSP_BF16 = 1, /* DType::BFloat16: raw bits of include/vesper/core/half.h:157 */
    VSP_F16 = 2,  /* IEEE binary16 (scales of Q8_0 planes only) */
    VSP_I8 = 3,
    VSP_I32 = 4
} vsp_dtype;

/* A strided view, the part of vesper::Tensor a kernel needs
 * (data_ptr() already includes the element offset, include/vesper/core/tensor.h:68-80). */
typedef struct {
    void* data;
    int32_t dtype; /* vsp_dtype */
    int32_t ndim;  /* <= 4 */
    int64_t shape[4];
    int64_t stride[4]; /* elements */
} vsp_tensor;

/* ---- KV cache ---------------------------------------------------------------
 * Replaces the storage of nn::KVCache (include/vesper/nn/transformer.h:21-39,
 * src/nn/transformer.cpp:32-93) and nn::GQAKVCache (include/vesper/nn/gqa_attention.h:110-163).
 * Logical content is the reference's: K and V of shape [B, Hkv, S_max, D], one
 * current length for the whole batch.  Physical layout per format (S_pad =
 * S_max rounded up to a multiple of 64; all planes are zero-initialised by
 * vsp_kv_cache_reset):
 *
 *  VSP_KV_F32   the reference's own layout, both planes fp32 row-major
 *               [B][Hkv][S_max][D]; element (b,h,s,d) at ((b*Hkv+h)*S_max+s)*D+d.
 *  VSP_KV_BF16  k: bf16 row-major [B][Hkv][S_pad][D]
 *               v: bf16 token-blocked, transposed inside the block:
 *                  [B][Hkv][S_pad/8][D][8]; element (b,h,s,d) at
 *                  (((b*Hkv+h)*(S_pad/8) + s/8)*D + d)*8 + s%8.
 *               (PV contracts over tokens; with 8 consecutive tokens of one d
 *               contiguous, a lane's 16-byte load is an MFMA operand as it is.)
 *  VSP_KV_Q8_0  rows quantised in blocks of 32 along D (ggml block_q8_0
 *               arithmetic: d = max|x|/127 stored as fp16 RNE, q = roundf(x/d)).
 *               k:       int8 [B][Hkv][S_pad][D]
 *               k_scale: fp16 [B][Hkv][S_pad][D/32]
 *               v:       int8 [B][Hkv][S_pad/16][D][16]   (token-blocked by 16)
 *               v_scale: fp16 [B][Hkv][S_pad/16][D/32][16]
 * D must be 64 or 128 for BF16/Q8_0.  Plane sizes: vsp_kv_plane_bytes().
 *
 * Paged variant (page_table != NULL; no counterpart in the reference, whose caches are one allocation per
 * batch): the planes hold n_pages pages of page_tokens tokens, each page laid out exactly like one batch
 * row above with S_pad = page_tokens -- [n_pages][Hkv][page_tokens][D] and so on -- and sequence b's tokens
 * [i*page_tokens, (i+1)*page_tokens) live in page page_table[b*pages_per_seq + i] (device int32, values in
 * [0, n_pages), owned and kept consistent by the caller).  BF16 and Q8_0 only; page_tokens a multiple of 64;
 * S_max == pages_per_seq * page_tokens; plane sizes: vsp_kv_plane_bytes(format, n_pages, Hkv, page_tokens, D, plane).
 * Every entry point that takes a cache accepts a paged one.
 */
typedef enum { VSP_KV_F32 = 0, VSP_KV_BF16 = 1, VSP_KV_Q8_0 = 2 } vsp_kv_format;
typedef enum { VSP_KV_PLANE_K = 0, VSP_KV_PLANE_V = 1, VSP_KV_PLANE_K_SCALE = 2, VSP_KV_PLANE_V_SCALE = 3 } vsp_kv_plane;

typedef struct {
    int32_t format; /* vsp_kv_format */
    int32_t B, Hkv, S_max, D;
    void* k;
    void* v;
    void* k_scale; /* Q8_0 only, else NULL */
    void* v_scale; /* Q8_0 only, else NULL */
    int32_t len;   /* the reference's current_len_ (host side, maintained by vsp_kv_append) */
    /* paged variant; all zero / NULL for a contiguous cache */
    const int32_t* page_table; /* device int32 [B][pages_per_seq] */
    int32_t page_tokens, pages_per_seq, n_pages;
} vsp_kv_cache;

/* Bytes the caller must allocate for one plane (0 for planes the format lacks). */
size_t vsp_kv_plane_bytes(int32_t format, int32_t B, int32_t Hkv, int32_t S_max, int32_t D, int32_t plane);

/* KVCache::reset(), src/nn/transformer.cpp:45-54 / GQAKVCache::reset(), src/nn/gqa_attention.cpp:209-214:
 * zero every plane (a fill kernel, not a memset node, so it may be graph-captured) and set len = 0.
 * Also the way a freshly allocated cache reaches the constructor's all-zero state (:40-41). */
int vsp_kv_cache_reset(vsp_kv_cache* cache, void* stream);

/* KVCache::update(new_k,new_v,start_pos) write half, src/nn/transformer.cpp:56-73 (== gqa_attention.cpp:175-194),
 * replacing ops::index + Tensor::copy_from + copy_strided_hip_dispatch (include/vesper/ops/copy.h:12,
 * src/ops/hip/copy.hip:16-93).  new_k/new_v: [B,Hkv,T,D], fp32 or bf16, any strides with stride[3]==1.
 * The slot is [:, :, start_pos:start_pos+T, :] under the reference's Python-slice clamping
 * (src/ops/view_ops.cpp:270-316); if the clamped slot does not hold exactly the elements of
 * new_k -> VSP_ERR_NUMEL, nothing written, len unchanged.  Conversion on write: fp32 -> bf16 is the
 * reference's round-to-nearest-even (include/vesper/core/half.h:162-173); Q8_0 quantises per row.
 * Afterwards len = max(len, start_pos + T).
 * start_pos_dev (nullable): device int32[B], per-sequence start positions for ragged batches
 * (no counterpart in the reference, which has one position for the batch); when given, start_pos
 * is ignored for placement, each row b is written at start_pos_dev[b] (0 <= start_pos_dev[b],
 * start_pos_dev[b]+T <= S_max; tokens that would land outside the planes are dropped) and len is left unchanged. */
int vsp_kv_append(vsp_kv_cache* cache, const vsp_tensor* new_k, const vsp_tensor* new_v, int64_t start_pos,
                  const int32_t* start_pos_dev, void* stream);

/* The step before the cache write in the attention modules, fused with it: rotary position embedding of
 * q and k (functional::compute_rope_frequencies + functional::apply_rotary_emb,
 * src/nn/functional.cpp:424-494, as called at src/nn/gqa_attention.cpp:124-130 and
 * src/nn/transformer.cpp:184-189) followed by KVCache::update's write (above).  One launch replaces the
 * reference's host-side angle table + upload, ~10 elementwise/stack/permute/contiguous launches per
 * tensor, and the strided cache copy.
 *   q [B,Hq,T,D], new_k/new_v [B,Hkv,T,D] (shape must equal the cache's B,Hkv,D): fp32 or bf16, one
 *   dtype, any strides with stride[3]==1 -- so the three can be strided views of one fused projection
 *   output [B,T,(Hq+2Hkv)*D] and the reference's transpose copies (src/nn/gqa_attention.cpp:120-122)
 *   disappear.  q_out [B,Hq,T,D] fp32 or bf16 (may alias q when dtypes match).
 *   rope_table: device float [table_len][D/2][2] = {cos, sin} of the angle of absolute position p and
 *   pair i, filled by vsp_rope_fill_table() (8-byte aligned).  Row b, token t uses position
 *   start_pos + t (or start_pos_dev[b] + t); without start_pos_dev the range must lie inside the
 *   table (else VSP_ERR_ARG); device-side positions past the table are clamped to its last row.
 * Arithmetic: pairs (2i, 2i+1); out[2i] = x0*cos - x1*sin, out[2i+1] = x0*sin + x1*cos in fp32 with each
 * product and sum rounded separately (bit-identical to the reference's separate elementwise ops); bf16
 * inputs are widened exactly first; conversion into the cache format as in vsp_kv_append.  V is not
 * rotated.  Slot placement, clamping, errors and the len update are those of vsp_kv_append. */
int vsp_rope_kv_append(vsp_kv_cache* cache, const vsp_tensor* q, const vsp_tensor* new_k, const vsp_tensor* new_v,
                       vsp_tensor* q_out, const float* rope_table, int64_t table_len, int64_t start_pos,
                       const int32_t* start_pos_dev, void* stream);

/* The read half of KVCache::update, :75-92: the reference returns VIEWS [:, :, 0:len, :] of its fp32
 * storage.  For VSP_KV_F32 the same view can be formed by the caller (vsp_kv_view_f32); for the other
 * formats this call materialises logical rows [start, start+count) into k_out/v_out
 * ([B,Hkv,count,D], fp32 or bf16, strided): bf16 planes are copied bit-for-bit (widened exactly for
 * fp32), Q8_0 planes are dequantised as q * f16->f32(scale).  Used by tests and by callers that
 * need the reference-shaped tensors; the attention kernels read the planes directly. */
int vsp_kv_read(const vsp_kv_cache* cache, int64_t start, int64_t count, vsp_tensor* k_out, vsp_tensor* v_out,
                void* stream);
/* Q8_0 only: the raw logical blocks, for bit-exact packing checks. qs_out int8 [B,Hkv,count,D],
 * scale_out fp16 bits [B,Hkv,count,D/32], both contiguous; plane = VSP_KV_PLANE_K or _V. */
int vsp_kv_read_q8_0(const vsp_kv_cache* cache, int32_t plane, int64_t start, int64_t count, int8_t* qs_out,
                     uint16_t* scale_out, void* stream);
/* VSP_KV_F32: fill k_view/v_view with the reference's view [:, :, 0:len, :] (shape, strides, offset 0). */
int vsp_kv_view_f32(const vsp_kv_cache* cache, vsp_tensor* k_view, vsp_tensor* v_view);

/* ---- prefill ------------------------------------------------------------------
 * Replaces flash_attention_hip_dispatch (include/vesper/ops/flash_attention.h:74-78, defined at
 * src/ops/hip/flash_attention.hip:305-331), with repeat_kv_hip_dispatch
 * (include/vesper/ops/attention_ops.h:35) folded in: q [B,Hq,T,D]; k, v [B,Hkv,L,D] with
 * Hq % Hkv == 0, query head h reading kv head h / (Hq/Hkv) (src/ops/attention_ops.cpp:47).
 * out [B,Hq,T,D] same dtype as q; lse [B,Hq,T] fp32 or NULL (= m + log l, src/ops/flash_attention.cpp:359).
 * dtype bf16 (MFMA, fp32 accumulation) or fp32.  D in {64,128}; fp32 also takes D = 32 (the shapes of the
 * reference's own tests, tests/test_flash_attention.cpp:110-179).  q/k/v/out may be strided
 * (stride[3]==1, rows 16-byte aligned), e.g. VSP_KV_F32 cache views.
 * is_causal: key j visible to query t iff j <= t + (L - T): the reference's mask when T == L
 * (src/ops/flash_attention.cpp:293-296), and its natural extension to a chunk appended at the end
 * of a longer context.  T > L with is_causal -> VSP_ERR_SHAPE.
 * Validation order and codes follow src/ops/flash_attention.cpp:45-59. */
int vsp_attn_prefill(const vsp_tensor* q, const vsp_tensor* k, const vsp_tensor* v, vsp_tensor* out, vsp_tensor* lse,
                     float scale, int is_causal, float dropout_p, int training, void* stream);

/* vsp_attn_prefill for fp32 tensors at matrix-core speed (the reference computes this op in fp32,
 * src/ops/flash_attention.cpp:218-364, and its modules hold fp32 tensors).  Same arguments and semantics as
 * vsp_attn_prefill with q, k, v, out fp32 and D in {64, 128} (else VSP_ERR_UNSUPPORTED), plus a workspace of
 * vsp_attn_prefill_split_workspace_bytes() bytes (16-byte aligned; else VSP_ERR_WORKSPACE).  A pre-pass writes every
 * operand as two bf16 planes x = hi + lo (hi = bf16(x), lo = bf16(x - hi): 16 significant bits) into the workspace; the
 * attention kernel takes each product as hi hi + hi lo + lo hi on the bf16 MFMAs with fp32 accumulation, and splits P the
 * same way after the fp32 exponential.  Results agree with the reference's fp32 arithmetic within its 1e-4 bar
 * (observed below 2e-5 of the output's magnitude) at several times the rate of the fp32-MFMA kernel. */
size_t vsp_attn_prefill_split_workspace_bytes(int32_t B, int32_t Hq, int32_t Hkv, int32_t T, int32_t L, int32_t D);
int vsp_attn_prefill_split(const vsp_tensor* q, const vsp_tensor* k, const vsp_tensor* v, vsp_tensor* out, vsp_tensor* lse,
                           float scale, int is_causal, void* workspace, size_t workspace_bytes, void* stream);

/* ops::flash_attention_backward (include/vesper/ops/flash_attention.h:61-66, src/ops/flash_attention.cpp:165-216)
 * = flash_attention_backward_hip_dispatch (header :80-92, src/ops/hip/flash_attention.hip:183-299), the
 * training-side companion of vsp_attn_prefill; mathematics of the CPU backward, src/ops/flash_attention.cpp:366-482,
 * without dropout: Di = rowsum(dO*O), P = exp(scale q.k - lse), dV = P^T dO, dS = P*(dO V^T - Di), dQ = scale dS K,
 * dK = scale dS^T Q.  dout/q/out/dq [B,Hq,N,D], k/v/dk/dv [B,Hkv,N,D] (Hq % Hkv == 0: dk/dv of a kv head sum over
 * its query heads, the gradient of ops::repeat_kv), lse [B,Hq,N] fp32 as written by vsp_attn_prefill; fp32 or bf16
 * (one dtype).  fp32: fp32 matrix-core arithmetic, any strides with stride[3]==1.  bf16: bf16 matrix cores with fp32
 * accumulation, P and dS rounded to bf16 between the products, gradients rounded to nearest even; base pointers and
 * strides multiples of 16 bytes (VSP_ERR_ALIGN), stride[2] >= D (VSP_ERR_STRIDE).  D in {64,128}, fp32 also 32.  dq/dk/dv are
 * overwritten.  No atomics: results are bitwise reproducible (the reference's
 * HIP kernel accumulates dQ with atomicAdd).  workspace: vsp_attn_backward_workspace_bytes(B, Hq, N) bytes.
 * bf16 with a workspace of at least vsp_attn_backward_fast_workspace_bytes(B, Hq, N) bytes (16-byte aligned; about
 * 2 N^2 bytes per query head on top of the former): dS is computed once instead of twice - the dK / dV pass leaves
 * every 32 x 32 tile of it in the workspace as bf16 and dQ is one product over those tiles - five tile products
 * instead of seven for the price of writing and reading the tiles, which the matrix-core-bound passes have the memory
 * bandwidth for.  Same rounding points (dS enters both of its products as the same bf16 values); still no atomics. */
size_t vsp_attn_backward_workspace_bytes(int32_t B, int32_t Hq, int32_t N);
size_t vsp_attn_backward_fast_workspace_bytes(int32_t B, int32_t Hq, int32_t N);
int vsp_attn_prefill_backward(const vsp_tensor* dout, const vsp_tensor* q, const vsp_tensor* k, const vsp_tensor* v,
                              const vsp_tensor* out, const vsp_tensor* lse, vsp_tensor* dq, vsp_tensor* dk,
                              vsp_tensor* dv, float scale, int is_causal, void* workspace, size_t workspace_bytes,
                              void* stream);

/* vsp_attn_prefill_backward for fp32 tensors at matrix-core speed: the backward companion of vsp_attn_prefill_split
 * (the reference computes this op in fp32, src/ops/flash_attention.cpp:366-482, and its modules hold fp32 tensors).
 * Same arguments and semantics as vsp_attn_prefill_backward with every tensor fp32 and D in {64, 128} (else
 * VSP_ERR_UNSUPPORTED).  A pre-pass writes Q, K, V and dO as two bf16 planes each
 * (x = hi + lo) and Di = rowsum(dO * O) in fp32 into the workspace; the two passes of the bf16 path then take every
 * product as hi hi + hi lo + lo hi with fp32 accumulation, with P and dS split the same way after the fp32 algebra,
 * and store fp32 gradients.  Inputs: base pointers 8-byte aligned, even strides; dq/dk/dv: 16-byte aligned, strides
 * multiples of 4 elements (VSP_ERR_ALIGN).  workspace: vsp_attn_backward_split_workspace_bytes() bytes, 16-byte aligned.
 * Results agree with the reference's fp32 gradients within its 1e-4 bar at several times the rate of the fp32-MFMA path;
 * bitwise reproducible like the other paths. */
size_t vsp_attn_backward_split_workspace_bytes(int32_t B, int32_t Hq, int32_t Hkv, int32_t N, int32_t D);
int vsp_attn_prefill_backward_split(const vsp_tensor* dout, const vsp_tensor* q, const vsp_tensor* k, const vsp_tensor* v,
                                    const vsp_tensor* out, const vsp_tensor* lse, vsp_tensor* dq, vsp_tensor* dk,
                                    vsp_tensor* dv, float scale, int is_causal, void* workspace, size_t workspace_bytes,
                                    void* stream);

/* Chunked / offset prefill straight over the cache planes (no counterpart in the reference, whose causal mask is
 * [T,T] and cannot be added to [T,L] scores, src/nn/functional.cpp:406-410; the semantics are the rows
 * [L-T, L) of the reference's full causal forward over L tokens, src/ops/flash_attention.cpp:218-364):
 * q [B,Hq,T,D] holds the LAST T tokens of each context, whose K/V are already in the cache
 * (vsp_kv_append / vsp_rope_kv_append first).  Context length: cache->len, or seq_lens[b] (device int32[B],
 * T <= seq_lens[b] <= max_len; values are clamped to that range) for ragged batches.  max_len: host-side upper
 * bound of L_b, as in vsp_attn_decode (0 = cache->len if seq_lens is NULL, else S_max): the launch, the Q8_0 read-out
 * and the context split are planned on it, so a batch whose longest row is far below the capacity should say so.
 * max_len < 0 or > S_max, or cache->len > max_len > 0 with seq_lens NULL, is VSP_ERR_ARG.  Query t attends keys
 * j <= L_b - T + t when is_causal, all L_b keys otherwise.
 *   VSP_KV_F32 : q/out fp32, fp32 arithmetic.   VSP_KV_BF16 : q/out bf16; K rows and token-blocked V are
 *   consumed in place (V^T operands are plain 16-byte reads of the blocked plane).
 *   VSP_KV_Q8_0: q/out bf16; rows [0, L) are first dequantised to dense bf16 in `workspace`
 *                (vsp_attn_prefill_cached_workspace_bytes() bytes, 16-byte aligned; else VSP_ERR_WORKSPACE) and
 *                the dense kernel runs over that: prefill is compute-bound, the read-out is ~0.2 % of its time.
 *                The other formats need no workspace (NULL, 0).
 * Tokens past L_b in the planes are never used, whatever they hold.  lse as in vsp_attn_prefill.
 * chunk_lens (nullable): device int32[B], n_b <= T valid query rows per sequence (ragged chunks in one call):
 * query t < n_b sits at position L_b - n_b + t; rows t >= n_b of `out` are unspecified.
 * Context split (VSP_KV_BF16, D = 128): a chunk of a few query tiles over a long context leaves most of
 * the chip idle, each workgroup walking the whole context.  A caller that passes a 16-byte aligned workspace of at
 * least vsp_attn_prefill_cached_split_workspace_bytes(cache, with_seq_lens, max_len, Hq, T) bytes (0 when the grid fills
 * the chip anyway, or the context is short) gets the context cut into shares of at least 512 keys, one workgroup per
 * (query tile, head, share), and the partials merged by the decode step's combine kernel in a fixed order (lse
 * included: the partials carry (m, l)).  Without that workspace the call runs unsplit; the results agree within bf16
 * rounding either way.  The two size functions take the same with_seq_lens (seq_lens != NULL) and max_len as the call. */
size_t vsp_attn_prefill_cached_workspace_bytes(const vsp_kv_cache* cache, int with_seq_lens, int32_t max_len);
size_t vsp_attn_prefill_cached_split_workspace_bytes(const vsp_kv_cache* cache, int with_seq_lens, int32_t max_len, int32_t Hq,
                                                     int32_t T);
int vsp_attn_prefill_cached(const vsp_tensor* q, const vsp_kv_cache* cache, const int32_t* seq_lens, int32_t max_len,
                            const int32_t* chunk_lens, vsp_tensor* out, vsp_tensor* lse, float scale, int is_causal,
                            void* workspace, size_t workspace_bytes, void* stream);

/* Ragged batches keep their lengths on the device (the reference's caches have one host-side length for the
 * whole batch, src/nn/transformer.cpp:73): after vsp_kv_append / vsp_rope_kv_append with start_pos_dev = seq_lens,
 * this advances them in stream order: seq_lens[b] = min(seq_lens[b] + n_b, S_max), n_b = n_new[b] clamped to
 * [0, T], or T when n_new is NULL.  The same array is what vsp_attn_decode and vsp_attn_prefill_cached take. */
int vsp_seq_lens_advance(int32_t* seq_lens, const int32_t* n_new, int32_t T, int32_t B, int32_t S_max, void* stream);

/* ---- decode -------------------------------------------------------------------
 * Replaces, for T == 1, the op chain scaled_dot_product_attention runs below its flash threshold
 * (src/nn/functional.cpp:397-421: gemm_batch_hip_dispatch x2, div_scalar, softmax_hip_dispatch)
 * and the two repeat_kv copies before it (src/nn/gqa_attention.cpp:140-141).
 * q, out: [B,Hq,1,D] bf16 (fp32 for a VSP_KV_F32 cache).  Every query head attends, unmasked, to
 * positions [0, L_b) of its kv head, L_b = seq_lens[b] (device int32[B]) or cache->len when
 * seq_lens is NULL.  L_b == 0 yields zeros.  max_len: host-side upper bound of L_b used to size the
 * launch and the workspace (0 = cache->len if seq_lens is NULL, else S_max).  The bound is enforced: with
 * seq_lens == NULL, cache->len > max_len > 0 is VSP_ERR_ARG; device-side lengths cannot be checked on the
 * host, so seq_lens[b] is clamped to [0, min(max_len, S_max)] inside the kernels and a row longer than the
 * bound attends to its first max_len keys only (the reference's cache length never exceeds what its
 * buffers were sized for, src/nn/transformer.cpp:73-92).
 * Split-K over the context: partial (m, l, acc) per (b, head, split) go to `workspace`
 * (>= vsp_attn_decode_workspace_bytes), then a combine kernel reduces them in a fixed order
 * (bitwise run-to-run deterministic). */
size_t vsp_attn_decode_workspace_bytes(int32_t B, int32_t Hq, int32_t D, int32_t max_len);
int vsp_attn_decode(const vsp_tensor* q, const vsp_kv_cache* cache, const int32_t* seq_lens, int32_t max_len,
                    vsp_tensor* out, float scale, void* workspace, size_t workspace_bytes, void* stream);

/* The decode step for a few tokens per sequence at once (the last T tokens of each context, already appended:
 * speculative-decoding verification, multi-token prediction): what GroupedQueryAttention::forward(x, cache,
 * start_pos) would compute for T > 1 and start_pos > 0 if its mask broadcast (src/nn/gqa_attention.cpp:128-148; the
 * reference throws there), i.e. the rows vsp_attn_prefill_cached returns, at the decode kernels' rate.  q, out
 * [B,Hq,T,D]: token t of sequence b sits at position L_b - T + t and attends keys [0, L_b - T + t].  The T tokens and the
 * Hq/Hkv query heads of a kv head share the 16 columns of the matrix instructions, so K and V are still read once per kv
 * head: T * Hq/Hkv <= 16 and D in {64, 128}, else VSP_ERR_UNSUPPORTED (use vsp_attn_prefill_cached).  T == 1 is
 * vsp_attn_decode, bit for bit.  Everything else as vsp_attn_decode; workspace >=
 * vsp_attn_decode_workspace_bytes(B * T, Hq, D, max_len).  A token placed before the start of its context
 * (L_b < T - t) gets zeros. */
int vsp_attn_decode_multi(const vsp_tensor* q, const vsp_kv_cache* cache, const int32_t* seq_lens, int32_t max_len,
                          vsp_tensor* out, float scale, void* workspace, size_t workspace_bytes, void* stream);

/* vsp_attn_decode for callers that cannot allocate device memory (code under HIP graph capture, tight
 * serving loops, harnesses that forbid hipMalloc).  No counterpart in the reference.  Same arguments,
 * validation, kernels and results (bit for bit) as vsp_attn_decode, minus the workspace: the split-K
 * partials go to a fixed 32 MiB array that is part of the library's code object (one copy per GPU, held
 * until the process ends), located on the first call on each device.  The call allocates and frees nothing.
 * The first call on a device looks the array's address up (a lock and two runtime queries, no launch of its own):
 * make that call outside any stream capture; every later call on that device may be captured.
 * Calls whose partials need more than that -- B * Hq * ceil(max_len / chunk) * (D + 2) * 4 bytes, chunk being
 * the split length the library picks (>= 256 tokens) -- return VSP_ERR_WORKSPACE: config 4 (B 32, 32 heads,
 * D 128, max_len 32768) needs 17 MiB.  Every call on one GPU shares that GPU's array: calls that overlap in
 * time on one GPU (different streams, different threads) race; serialise them or use vsp_attn_decode. */
int vsp_attn_decode_noalloc(const vsp_tensor* q, const vsp_kv_cache* cache, const int32_t* seq_lens, int32_t max_len,
                            vsp_tensor* out, float scale, void* stream);

/* Decode step plus the attention module's output projection in one call: replaces, for T == 1, the chain above
 * together with what follows it in GroupedQueryAttention::forward and MultiHeadAttention::forward -- the heads
 * merged by transpose(1,2).reshape({B,T,C}) and wo_ / out_proj applied (src/nn/gqa_attention.cpp:151-152,
 * src/nn/transformer.cpp:207-215; Linear::forward, src/nn/linear.cpp:41-49: y = x W^T + bias).
 * q, cache, seq_lens, max_len, scale: as vsp_attn_decode.  wo: [N, Hq*D], row pitch and base 16-byte aligned;
 * bias: [N] or NULL; y: [B, 1, N]; all of q's dtype (bf16 over VSP_KV_BF16 / VSP_KV_Q8_0 caches, fp32 over
 * VSP_KV_F32).  The merged heads never become a caller tensor: the combine kernel leaves them, rounded to q's dtype
 * exactly as vsp_attn_decode's `out` would hold them, at the head of `workspace`, and a projection kernel streams
 * W over them once (bf16: 16x16x32 MFMA with fp32 accumulation; up to 16 batch rows in one launch, K split over the
 * eight wavefronts of a workgroup; more rows with K split over up to eight workgroups whose partial tiles a second
 * kernel adds in index order before the bias and the rounding; bitwise run-to-run deterministic either way).
 * workspace >= vsp_attn_decode_proj_workspace_bytes(B, Hq, D, max_len, N), 16-byte aligned. */
size_t vsp_attn_decode_proj_workspace_bytes(int32_t B, int32_t Hq, int32_t D, int32_t max_len, int32_t N);
int vsp_attn_decode_proj(const vsp_tensor* q, const vsp_kv_cache* cache, const int32_t* seq_lens, int32_t max_len,
                         const vsp_tensor* wo, const vsp_tensor* bias, vsp_tensor* y, float scale, void* workspace,
                         size_t workspace_bytes, void* stream);

/* ---- host-side, bit-exact format helpers (pure CPU; exported for tests and callers) ---- */
uint16_t vsp_f32_to_bf16(float f);   /* include/vesper/core/half.h:162-173 */
float vsp_bf16_to_f32(uint16_t b);   /* include/vesper/core/half.h:175-181 */
uint16_t vsp_f32_to_f16(float f);    /* IEEE RNE */
float vsp_f16_to_f32(uint16_t h);
void vsp_q8_0_quantize_row(const float* x, int64_t n, uint16_t* scale, int8_t* qs);
void vsp_q8_0_dequantize_row(const uint16_t* scale, const int8_t* qs, int64_t n, float* x);
/* Host-side RoPE table: table[m][i] = {cosf(a), sinf(a)}, a = (float)(start_pos + m) * powf(theta,
 * -2.0f * i / D), m < count, i < D/2 -- the angles of functional::compute_rope_frequencies
 * (src/nn/functional.cpp:424-443) through ops::cos / ops::sin (std::cos / std::sin on float,
 * src/ops/elementwise.cpp:1039-1045).  The caller uploads it once per (D, theta). */
void vsp_rope_fill_table(float* table, int32_t start_pos, int32_t count, int32_t D, float theta);
/* The reference's slice clamping for one dimension (src/ops/view_ops.cpp:270-316, step 1). */
void vsp_slice_bounds(int64_t dim_size, int64_t start, int64_t stop, int64_t* out_start, int64_t* out_len);
/* GroupedQueryAttention constructor arithmetic and checks (src/nn/gqa_attention.cpp:38-57). */
int vsp_gqa_config(int64_t embed_dim, int64_t num_heads, int64_t num_kv_heads, int64_t* head_dim, int64_t* num_rep);

const char* vsp_status_str(int status);
const char* vsp_last_hip_error(void); /* text of the last HIP error seen by this thread ("" if none) */
int vsp_attn_abi_version(void);

#ifdef __cplusplus
}
#endif
#endif /* VSP_ATTN_H */
