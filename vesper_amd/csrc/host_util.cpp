// Host-side pieces of the C ABI: status text, bit-exact number-format helpers, the reference's
// slice and GQA-constructor arithmetic, per-thread HIP error text.
#include <math.h>

#include <string>

#include "kv_layout.hpp"
#include "vsp_common.hpp"

namespace vsp {
namespace {
thread_local std::string g_hip_error;
}
void set_hip_error(hipError_t e) { g_hip_error = hipGetErrorString(e); }
int check_launch() {
    hipError_t e = hipGetLastError();
    if (e != hipSuccess) {
        set_hip_error(e);
        return VSP_ERR_LAUNCH;
    }
    return VSP_OK;
}
int device_cu_count() {
    static const int cus = [] {
        int dev = 0, n = 0;
        if (hipGetDevice(&dev) == hipSuccess &&
            hipDeviceGetAttribute(&n, hipDeviceAttributeMultiprocessorCount, dev) == hipSuccess && n > 0)
            return n;
        return 256;
    }();
    return cus;
}
}  // namespace vsp

extern "C" {

const char* vsp_status_str(int status) {
    switch (status) {
        case VSP_OK: return "ok";
        case VSP_ERR_NDIM: return "flash_attention: inputs must be 4D [B, H, N, D]";
        case VSP_ERR_SHAPE: return "flash_attention: Q, K, V must have same shape";
        case VSP_ERR_DTYPE: return "flash_attention: Q, K, V must have same dtype";
        case VSP_ERR_DROPOUT: return "flash_attention: dropout_p must be in [0, 1)";
        case VSP_ERR_NUMEL: return "copy_from: element count mismatch.";
        case VSP_ERR_COPY_DTYPE: return "copy_from: dtype mismatch.";
        case VSP_ERR_REPEAT_NDIM: return "repeat_kv: input must be 4D [Batch, KV_Heads, SeqLen, HeadDim]";
        case VSP_ERR_GQA_HEADS: return "GroupedQueryAttention: num_heads must be divisible by num_kv_heads";
        case VSP_ERR_GQA_EMBED: return "GroupedQueryAttention: embed_dim must be divisible by num_heads";
        case VSP_ERR_BROADCAST: return "causal mask [T, T] cannot be broadcast onto scores [T, L]";
        case VSP_ERR_NULL: return "vsp_attn: required pointer is NULL";
        case VSP_ERR_UNSUPPORTED: return "vsp_attn: unsupported dtype / cache format / head_dim combination";
        case VSP_ERR_STRIDE: return "vsp_attn: unsupported stride (innermost stride must be 1)";
        case VSP_ERR_ALIGN: return "vsp_attn: pointer or row pitch not 16-byte aligned";
        case VSP_ERR_WORKSPACE: return "vsp_attn: workspace missing or too small";
        case VSP_ERR_ARG: return "vsp_attn: argument out of range";
        case VSP_ERR_LAUNCH: return "vsp_attn: HIP launch failed";
    }
    return "vsp_attn: unknown status";
}

const char* vsp_last_hip_error(void) { return vsp::g_hip_error.c_str(); }
int vsp_attn_abi_version(void) { return VSP_ATTN_ABI_VERSION; }

uint16_t vsp_f32_to_bf16(float f) { return vsp::f32_to_bf16_bits(f); }
float vsp_bf16_to_f32(uint16_t b) { return vsp::bf16_bits_to_f32(b); }

// IEEE binary32 -> binary16, round-to-nearest-even, via exact integer arithmetic on the significand.
uint16_t vsp_f32_to_f16(float f) {
    uint32_t x;
    memcpy(&x, &f, 4);
    const uint32_t sign = (x >> 16) & 0x8000u;
    const uint32_t a = x & 0x7FFFFFFFu;
    if (a >= 0x7F800000u) return (uint16_t)(sign | 0x7C00u | (a > 0x7F800000u ? 0x200u | ((a >> 13) & 0x3FFu) : 0u));
    if (a >= 0x47800000u) return (uint16_t)(sign | 0x7C00u);  // >= 65536 -> inf (65520..65535.99 handled by carry below)
    if (a < 0x33000000u) return (uint16_t)sign;                // < 2^-25 -> 0 (2^-25 itself ties to even = 0)
    uint32_t mant, shift;
    if (a < 0x38800000u) {  // result is subnormal: value = mant24 * 2^(e-150); target unit 2^-24
        mant = (a & 0x7FFFFFu) | 0x800000u;
        shift = 126u - (a >> 23);  // 14..24
        uint32_t q = mant >> shift, rem = mant & ((1u << shift) - 1u), half = 1u << (shift - 1);
        if (rem > half || (rem == half && (q & 1u))) ++q;
        return (uint16_t)(sign | q);
    }
    uint32_t q = ((a >> 23) - 112u) << 10 | ((a >> 13) & 0x3FFu);
    uint32_t rem = a & 0x1FFFu;
    if (rem > 0x1000u || (rem == 0x1000u && (q & 1u))) ++q;  // carries into the exponent, up to inf
    return (uint16_t)(sign | q);
}

float vsp_f16_to_f32(uint16_t h) {
    const uint32_t sign = ((uint32_t)h & 0x8000u) << 16;
    const uint32_t e = (h >> 10) & 0x1Fu, m = h & 0x3FFu;
    float r;
    if (e == 0) {
        r = ldexpf((float)m, -24);
    } else if (e == 31) {
        uint32_t x = 0x7F800000u | (m << 13);
        memcpy(&r, &x, 4);
    } else {
        uint32_t x = ((e + 112u) << 23) | (m << 13);
        memcpy(&r, &x, 4);
    }
    uint32_t x;
    memcpy(&x, &r, 4);
    x |= sign;
    memcpy(&r, &x, 4);
    return r;
}

// ggml block_q8_0 arithmetic per 32 elements.
void vsp_q8_0_quantize_row(const float* x, int64_t n, uint16_t* scale, int8_t* qs) {
    for (int64_t blk = 0; blk < n / vsp::kQBlock; ++blk) {
        const float* xb = x + blk * vsp::kQBlock;
        float amax = 0.0f;
        for (int i = 0; i < vsp::kQBlock; ++i) amax = fmaxf(amax, fabsf(xb[i]));
        const float d = amax / 127.0f;
        const float id = d != 0.0f ? 1.0f / d : 0.0f;
        scale[blk] = vsp_f32_to_f16(d);
        for (int i = 0; i < vsp::kQBlock; ++i) qs[blk * vsp::kQBlock + i] = (int8_t)roundf(xb[i] * id);
    }
}
void vsp_q8_0_dequantize_row(const uint16_t* scale, const int8_t* qs, int64_t n, float* x) {
    for (int64_t blk = 0; blk < n / vsp::kQBlock; ++blk) {
        const float d = vsp_f16_to_f32(scale[blk]);
        for (int i = 0; i < vsp::kQBlock; ++i) x[blk * vsp::kQBlock + i] = (float)qs[blk * vsp::kQBlock + i] * d;
    }
}

// compute_rope_frequencies (src/nn/functional.cpp:424-443) followed by ops::cos / ops::sin: float
// arithmetic throughout, `-2.0f * i / dim` evaluated left to right, the int position converted to float.
void vsp_rope_fill_table(float* table, int32_t start_pos, int32_t count, int32_t D, float theta) {
    const int32_t half = D / 2;
    for (int32_t m = 0; m < count; ++m) {
        const int32_t pos = start_pos + m;
        for (int32_t i = 0; i < half; ++i) {
            const float freq = powf(theta, -2.0f * (float)i / (float)D);
            const float angle = (float)pos * freq;
            float* e = table + ((int64_t)m * half + i) * 2;
            e[0] = cosf(angle);
            e[1] = sinf(angle);
        }
    }
}

void vsp_slice_bounds(int64_t dim_size, int64_t start, int64_t stop, int64_t* out_start, int64_t* out_len) {
    vsp::slice_bounds(dim_size, start, stop, out_start, out_len);
}

int vsp_gqa_config(int64_t embed_dim, int64_t num_heads, int64_t num_kv_heads, int64_t* head_dim, int64_t* num_rep) {
    if (num_heads <= 0 || num_kv_heads <= 0) return VSP_ERR_ARG;
    if (num_heads % num_kv_heads != 0) return VSP_ERR_GQA_HEADS;
    if (embed_dim % num_heads != 0) return VSP_ERR_GQA_EMBED;
    if (head_dim) *head_dim = embed_dim / num_heads;
    if (num_rep) *num_rep = num_heads / num_kv_heads;
    return VSP_OK;
}

size_t vsp_kv_plane_bytes(int32_t format, int32_t B, int32_t Hkv, int32_t S_max, int32_t D, int32_t plane) {
    return vsp::kv_plane_bytes(format, B, Hkv, S_max, D, plane);
}

}  // extern "C"
