// Shared declarations of libvsp_attn.so: device helpers, argument checks, launch plumbing.
#pragma once

#include <hip/hip_runtime.h>
#include <stdint.h>
#include <string.h>

#include "../../include/vsp_attn.h"

namespace vsp {

typedef __bf16 bf16x8_t __attribute__((ext_vector_type(8)));
typedef __bf16 bf16x4_t __attribute__((ext_vector_type(4)));
typedef _Float16 f16x8_t __attribute__((ext_vector_type(8)));
typedef _Float16 f16x2_t __attribute__((ext_vector_type(2)));
typedef float f32x4_t __attribute__((ext_vector_type(4)));
typedef float f32x16_t __attribute__((ext_vector_type(16)));
typedef uint32_t u32x4_t __attribute__((ext_vector_type(4)));
typedef uint32_t u32x2_t __attribute__((ext_vector_type(2)));

constexpr float kLog2e = 1.4426950408889634f;

// fp32 -> bf16 bits, the reference's round-to-nearest-even
// (include/vesper/core/half.h:162-173; src/ops/hip/cast.hip:28-34): no NaN special case.
__host__ __device__ inline uint16_t f32_to_bf16_bits(float f) {
    uint32_t bits;
#if defined(__HIP_DEVICE_COMPILE__)
    bits = __builtin_bit_cast(uint32_t, f);
#else
    memcpy(&bits, &f, sizeof bits);
#endif
    bits += 0x7FFFu + ((bits >> 16) & 1u);
    return (uint16_t)(bits >> 16);
}
__host__ __device__ inline float bf16_bits_to_f32(uint16_t b) {
    uint32_t bits = (uint32_t)b << 16;
#if defined(__HIP_DEVICE_COMPILE__)
    return __builtin_bit_cast(float, bits);
#else
    float f;
    memcpy(&f, &bits, sizeof f);
    return f;
#endif
}
// two fp32 -> packed bf16x2 (lo = a, hi = b), same rounding
__device__ inline uint32_t pack_bf16x2(float a, float b) {
    return (uint32_t)f32_to_bf16_bits(a) | ((uint32_t)f32_to_bf16_bits(b) << 16);
}

// Workgroup ids are dealt round-robin to the 8 XCDs (id % 8), each with an L2 of its own.  Position `pos` of a row of
// B * Hq workgroups is mapped to (batch, query head) = bh so that, when the number of (batch, kv head) groups is a
// multiple of 8, the n_rep query heads of one kv group all get positions of the same residue mod 8: the group's K/V
// tiles are then fetched into one XCD's L2 instead of up to n_rep of them.  Groups are numbered b * Hkv + kvh, so
// grp * n_rep + r == b * Hq + hq.  The map is a permutation of [0, B * Hq).
__device__ inline int xcd_grouped_head(int pos, int n_groups, int n_rep) {
    if ((n_groups & 7) != 0) return pos;
    const int xcd = pos & 7, slot = pos >> 3;
    return (xcd + 8 * (slot / n_rep)) * n_rep + slot % n_rep;
}

// per-thread last HIP error text (vsp_last_hip_error)
void set_hip_error(hipError_t e);
int check_launch();  // VSP_OK or VSP_ERR_LAUNCH after a kernel launch
int device_cu_count();  // compute units of the device that was current at the first call (256 if the query fails)
// decode.hip: the split-K combine (decode step; context-split prefill over a cache).  What the latter adds to the
// decode step's merge: the lower clamp of a row's length (a chunk is part of its context) and the LSE.
struct CombineExtra {
    const int32_t* chunk_lens = nullptr;  // per-row number of valid query rows (device), clamped to [0, len_floor]
    int32_t len_floor = 0;                // a row's length is at least this (its chunk length when chunk_lens is null)
    float* lse = nullptr;                 // lse[b][hq][t] = ln sum_j exp(score_j), or null
    int64_t sl[3] = {0, 0, 0};            // its strides (elements)
};
int launch_split_combine(const float* ws_o, const float* ws_ml, const int32_t* seq_lens, int32_t len, int32_t chunk, int32_t max_splits,
                         int64_t B, int64_t Hq, int64_t T, int64_t D, int32_t L_cap, vsp_tensor* out, hipStream_t st,
                         const CombineExtra& extra = CombineExtra{});

inline bool is_aligned16(const void* p) { return (reinterpret_cast<uintptr_t>(p) & 15u) == 0; }

inline int64_t round_up(int64_t x, int64_t m) { return (x + m - 1) / m * m; }
inline int64_t ceil_div(int64_t x, int64_t m) { return (x + m - 1) / m; }

// reference slice clamping for Slice(start, stop), step 1: src/ops/view_ops.cpp:270-316
inline void slice_bounds(int64_t dim_size, int64_t start, int64_t stop, int64_t* out_start, int64_t* out_len) {
    if (start < 0) start += dim_size;
    if (stop < 0) stop += dim_size;
    start = start < 0 ? 0 : (start > dim_size ? dim_size : start);
    stop = stop < 0 ? 0 : (stop > dim_size ? dim_size : stop);
    *out_start = start;
    *out_len = start >= stop ? 0 : stop - start;
}

}  // namespace vsp
