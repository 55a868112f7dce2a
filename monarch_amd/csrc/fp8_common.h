// Pieces shared by the fp8 codec kernels (flat-buffer and tensor-bucket forms).
#pragma once
#include <cfloat>

#include "mhip_device.h"

namespace mhip {

constexpr uint32_t kBlock = 1024;         // elements per scale
constexpr float kFp8Max = 448.0f;
constexpr float kAbsmaxFloor = 0x1p-40f;  // keeps 448/absmax finite for all-zero / denormal blocks

// all-reduce max over the 64 lanes of a wavefront, for unsigned 32-bit values
__device__ __forceinline__ uint32_t wave_max_u32(uint32_t v) {
    // DPP butterfly within each row of 16 lanes
    uint32_t o;
    o = (uint32_t)__builtin_amdgcn_update_dpp(0, (int)v, 0xB1, 0xF, 0xF, true);   // quad_perm [1,0,3,2]
    v = v > o ? v : o;
    o = (uint32_t)__builtin_amdgcn_update_dpp(0, (int)v, 0x4E, 0xF, 0xF, true);   // quad_perm [2,3,0,1]
    v = v > o ? v : o;
    o = (uint32_t)__builtin_amdgcn_update_dpp(0, (int)v, 0x141, 0xF, 0xF, true);  // row_half_mirror
    v = v > o ? v : o;
    o = (uint32_t)__builtin_amdgcn_update_dpp(0, (int)v, 0x140, 0xF, 0xF, true);  // row_mirror
    v = v > o ? v : o;
    // one value per row, combined on the scalar unit
    const uint32_t r0 = (uint32_t)__builtin_amdgcn_readlane((int)v, 0);
    const uint32_t r1 = (uint32_t)__builtin_amdgcn_readlane((int)v, 16);
    const uint32_t r2 = (uint32_t)__builtin_amdgcn_readlane((int)v, 32);
    const uint32_t r3 = (uint32_t)__builtin_amdgcn_readlane((int)v, 48);
    const uint32_t a = r0 > r1 ? r0 : r1, b = r2 > r3 ? r2 : r3;
    return a > b ? a : b;
}

__device__ __forceinline__ void block_factors(uint32_t absmax_bf16_bits, float* scale, float* inv) {
    float absmax = __uint_as_float(absmax_bf16_bits << 16);
    absmax = absmax < kAbsmaxFloor ? kAbsmaxFloor : absmax;
    absmax = absmax > FLT_MAX ? FLT_MAX : absmax;
    *scale = absmax / kFp8Max;
    *inv = kFp8Max / absmax;
}

// two bf16 values (one 32-bit word) -> two fp8 codes in the low or high half of `old`
template <bool HIGH>
__device__ __forceinline__ int quant_pair(uint32_t w, float inv, int old) {
    return __builtin_amdgcn_cvt_pk_fp8_f32(bf16_lo(w) * inv, bf16_hi(w) * inv, old, HIGH);
}

__device__ __forceinline__ uint8_t quant_one_careful(uint32_t h, float inv) {
    // NaN -> the fp8 NaN code with the input's sign, whatever its payload.  Taken from the bits: the multiply
    // below quiets a signalling NaN, and the sign of what the conversion then produces is not the input's.
    if ((h & 0x7fffu) > 0x7f80u) return (uint8_t)(((h >> 8) & 0x80u) | 0x7fu);
    float y = __uint_as_float(h << 16) * inv;
    y = y > kFp8Max ? kFp8Max : y;    // comparisons are false for NaN: it passes through
    y = y < -kFp8Max ? -kFp8Max : y;
    return (uint8_t)(__builtin_amdgcn_cvt_pk_fp8_f32(y, y, 0, false) & 0xff);
}

// largest t in [lo, hi) with offsets[t] * upe <= unit (offsets: element offsets of a bucket)
__device__ __forceinline__ uint32_t find_tensor(const uint64_t* __restrict__ offsets, uint32_t upe, uint32_t lo,
                                                uint32_t hi, uint64_t unit) {
    while (hi - lo > 1) {
        const uint32_t mid = lo + ((hi - lo) >> 1);
        if (offsets[mid] * upe <= unit) lo = mid; else hi = mid;
    }
    return lo;
}

// The same search done by a whole wavefront for one (wave-uniform) position: every step
// probes 64 entries at once and keeps the sixty-fifth of the range that holds the answer,
// so a table of up to 4225 tensors resolves in two dependent loads instead of twelve.
// All 64 lanes must call it with the same arguments.
__device__ __forceinline__ uint32_t wave_find_tensor(const uint64_t* __restrict__ offsets, uint32_t upe, uint32_t lo,
                                                     uint32_t hi, uint64_t unit) {
    const uint32_t lane = threadIdx.x & 63;
    while (hi - lo > 1) {
        const uint32_t span = hi - lo;
        if (span <= 65) {
            const uint32_t pos = lo + 1 + lane;
            const bool le = pos < hi && offsets[pos] * upe <= unit;
            return lo + (uint32_t)__popcll(__ballot(le));
        }
        const uint32_t pos = lo + (uint32_t)(((uint64_t)(lane + 1) * span) / 65);  // in (lo, hi), non-decreasing in lane
        const bool le = offsets[pos] * upe <= unit;
        const uint32_t c = (uint32_t)__popcll(__ballot(le));  // lanes 0..c-1 are <= unit (offsets are sorted)
        const uint32_t new_lo = c ? lo + (uint32_t)(((uint64_t)c * span) / 65) : lo;
        const uint32_t new_hi = c < 64 ? lo + (uint32_t)(((uint64_t)(c + 1) * span) / 65) : hi;
        lo = new_lo;
        hi = new_hi;
    }
    return lo;
}

// Two positions u1 <= u2 in one descent: the probes of a step are loaded once and compared with
// both, and the searches only part ways (rarely: the positions are a few thousand elements
// apart) when they fall into different sub-ranges.
__device__ __forceinline__ void wave_find_tensor_pair(const uint64_t* __restrict__ offsets, uint32_t upe, uint32_t lo,
                                                      uint32_t hi, uint64_t u1, uint64_t u2, uint32_t* t1,
                                                      uint32_t* t2) {
    const uint32_t lane = threadIdx.x & 63;
    while (hi - lo > 1) {
        const uint32_t span = hi - lo;
        if (span <= 65) {
            const uint32_t pos = lo + 1 + lane;
            const uint64_t off = pos < hi ? offsets[pos] * upe : ~0ull;
            *t1 = lo + (uint32_t)__popcll(__ballot(pos < hi && off <= u1));
            *t2 = lo + (uint32_t)__popcll(__ballot(pos < hi && off <= u2));
            return;
        }
        const uint32_t pos = lo + (uint32_t)(((uint64_t)(lane + 1) * span) / 65);
        const uint64_t off = offsets[pos] * upe;
        const uint32_t c1 = (uint32_t)__popcll(__ballot(off <= u1));
        const uint32_t c2 = (uint32_t)__popcll(__ballot(off <= u2));
        const uint32_t lo1 = c1 ? lo + (uint32_t)(((uint64_t)c1 * span) / 65) : lo;
        const uint32_t hi1 = c1 < 64 ? lo + (uint32_t)(((uint64_t)(c1 + 1) * span) / 65) : hi;
        if (c1 != c2) {
            const uint32_t lo2 = lo + (uint32_t)(((uint64_t)c2 * span) / 65);
            const uint32_t hi2 = c2 < 64 ? lo + (uint32_t)(((uint64_t)(c2 + 1) * span) / 65) : hi;
            *t1 = wave_find_tensor(offsets, upe, lo1, hi1, u1);
            *t2 = wave_find_tensor(offsets, upe, lo2, hi2, u2);
            return;
        }
        lo = lo1;
        hi = hi1;
    }
    *t1 = lo;
    *t2 = lo;
}

}  // namespace mhip
