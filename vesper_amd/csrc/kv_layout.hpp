// Physical layouts of the KV-cache planes: one place for the index arithmetic, shared by the
// host (sizes, validation) and every kernel that touches a plane.
//
// Logical content is the reference's: K, V of shape [B, Hkv, S_max, D]
// (src/nn/transformer.cpp:32-43).  S_pad = S_max rounded up to 64 for BF16/Q8_0 so that a decode
// wave may load whole 64-token groups without leaving the allocation.
#pragma once

#include <stdint.h>

#include "../../include/vsp_attn.h"

namespace vsp {

constexpr int kTokPad = 64;    // S_pad granularity
constexpr int kVBlkBf16 = 8;   // tokens per V block, bf16 (8 x 2 B = one 16-byte operand)
constexpr int kVBlkQ8 = 16;    // tokens per V block, int8 (16 x 1 B)
constexpr int kQBlock = 32;    // Q8_0 block length along D

__host__ __device__ inline int64_t kv_s_pad(int format, int64_t S_max) {
    return format == VSP_KV_F32 ? S_max : (S_max + kTokPad - 1) / kTokPad * kTokPad;
}

// Paged caches: logical (sequence b, token s) -> (page, token within the page).  The planes of a paged cache are
// laid out like a contiguous cache with batch = n_pages and token capacity = page_tokens, so after this
// translation every offset function below applies unchanged.  table == nullptr: contiguous, identity.
__host__ __device__ inline void kv_locate(const int32_t* table, int32_t page_tokens, int32_t pages_per_seq, int64_t& b, int64_t& s) {
    if (table) {
        const int64_t pg = s / page_tokens;
        s -= pg * page_tokens;
        b = table[b * pages_per_seq + pg];
    }
}

// ---- element offsets (in elements of the plane's type) ----
// row-major [B][H][S][D]: the reference layout (K of every format, V of F32)
__host__ __device__ inline int64_t kv_off_rowmajor(int64_t H, int64_t S, int64_t D, int64_t b, int64_t h, int64_t s,
                                                    int64_t d) {
    return ((b * H + h) * S + s) * D + d;
}
// token-blocked transposed [B][H][S/BLK][D][BLK]
__host__ __device__ inline int64_t kv_off_vblocked(int64_t H, int64_t S, int64_t D, int64_t BLK, int64_t b, int64_t h,
                                                    int64_t s, int64_t d) {
    return (((b * H + h) * (S / BLK) + s / BLK) * D + d) * BLK + s % BLK;
}
// K scales [B][H][S][D/32]
__host__ __device__ inline int64_t kv_off_kscale(int64_t H, int64_t S, int64_t D, int64_t b, int64_t h, int64_t s,
                                                  int64_t blk) {
    return ((b * H + h) * S + s) * (D / kQBlock) + blk;
}
// V scales [B][H][S/16][D/32][16]
__host__ __device__ inline int64_t kv_off_vscale(int64_t H, int64_t S, int64_t D, int64_t b, int64_t h, int64_t s,
                                                  int64_t blk) {
    return (((b * H + h) * (S / kVBlkQ8) + s / kVBlkQ8) * (D / kQBlock) + blk) * kVBlkQ8 + s % kVBlkQ8;
}

inline size_t kv_plane_bytes(int format, int64_t B, int64_t H, int64_t S_max, int64_t D, int plane) {
    if (B < 0 || H < 0 || S_max < 0 || D < 0) return 0;
    int64_t S = kv_s_pad(format, S_max);
    int64_t n = B * H * S * D;
    switch (format) {
        case VSP_KV_F32:
            return (plane == VSP_KV_PLANE_K || plane == VSP_KV_PLANE_V) ? (size_t)n * 4 : 0;
        case VSP_KV_BF16:
            return (plane == VSP_KV_PLANE_K || plane == VSP_KV_PLANE_V) ? (size_t)n * 2 : 0;
        case VSP_KV_Q8_0:
            if (plane == VSP_KV_PLANE_K || plane == VSP_KV_PLANE_V) return (size_t)n;
            return (size_t)(n / kQBlock) * 2;
    }
    return 0;
}

}  // namespace vsp
