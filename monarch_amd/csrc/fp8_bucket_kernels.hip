// Fused forms of the fp8 transfer codec that work on a tensor bucket directly, skipping
// the flat bf16 / fp32 staging buffers:
//
//   quantize_bucket          == flat_pack (bf16)  followed by  fp8_quantize
//                               3 bytes per element instead of 4 + 3
//   dequant_accumulate_bucket== fp8_dequant_accumulate into per-tensor fp32 accumulators
//                               (no flat accumulator, no flat_unpack): 9 bytes instead of 9 + 8
//
// Blocks of 1024 are still counted over the flat index space of the bucket, so codes and
// scales are bit-identical to the two-step pipeline.  A wavefront finds the tensors that
// hold the first and the last element of its span with two cooperative 65-ary searches over
// the offsets table; a span inside one tensor (the common case: tensors are >= 1K
// elements) then costs nothing extra, a block that straddles tensors resolves each
// 8-element (resp. 4-element) group on its own and falls back to single elements only
// where a group itself straddles.
#include "fp8_common.h"

namespace mhip {

struct BucketArgs {
    char* const* tensors;     // device table of ntensors pointers
    const uint64_t* offsets;  // device table of ntensors + 1 element offsets
    uint64_t total;           // elements in the bucket
    uint64_t nblocks;
    uint32_t ntensors;
};

__device__ __forceinline__ uint16_t bucket_elem_bf16(const BucketArgs& a, uint32_t t_lo, uint32_t t_hi, uint64_t e) {
    const uint32_t ti = find_tensor(a.offsets, 1, t_lo, t_hi + 1, e);
    return reinterpret_cast<const uint16_t*>(a.tensors[ti])[e - a.offsets[ti]];
}

// 8 consecutive bf16 elements of the bucket starting at flat element e
__device__ __forceinline__ uint4 bucket_load8_bf16(const BucketArgs& a, uint32_t t_lo, uint32_t t_hi, uint64_t e) {
    const uint32_t ti = find_tensor(a.offsets, 1, t_lo, t_hi + 1, e);
    const uint64_t begin = a.offsets[ti], end = a.offsets[ti + 1];
    if (e + 8 <= end) return load16_unaligned(a.tensors[ti] + (e - begin) * 2);
    uint32_t w[4];
#pragma unroll
    for (int k = 0; k < 4; ++k) {
        const uint32_t lo = bucket_elem_bf16(a, ti, t_hi, e + 2 * k);
        const uint32_t hi = bucket_elem_bf16(a, ti, t_hi, e + 2 * k + 1);
        w[k] = lo | (hi << 16);
    }
    return make_uint4(w[0], w[1], w[2], w[3]);
}

__device__ __noinline__ void quantize_bucket_block_careful(uint8_t* __restrict__ q, float* __restrict__ scales,
                                                           const BucketArgs& a, uint32_t t_lo, uint32_t t_hi,
                                                           uint64_t begin, uint32_t count, uint64_t b, int lane) {
    uint32_t m = 0;
    for (uint32_t i = lane; i < count; i += 64) {
        const uint32_t v = bucket_elem_bf16(a, t_lo, t_hi, begin + i) & 0x7fffu;
        if (v <= 0x7f80u && v > m) m = v;
    }
    m = wave_max_u32(m);
    float scale, inv;
    block_factors(m, &scale, &inv);
    if (lane == 0) scales[b] = scale;
    for (uint32_t i = lane; i < count; i += 64)
        q[begin + i] = quant_one_careful(bucket_elem_bf16(a, t_lo, t_hi, begin + i), inv);
}

// A wavefront handles kBucketBlocks consecutive blocks per step (8 KiB of input): one
// cooperative search pair locates the tensors of the first and the last element of the
// whole span; when they coincide (the common case) all 2 * kBucketBlocks loads of a lane
// are issued back to back from one base pointer.
constexpr int kBucketBlocks = 4;

__global__ __launch_bounds__(kThreads) void fp8_quantize_bucket_kernel(uint8_t* __restrict__ q, float* __restrict__ scales,
                                                                       BucketArgs a) {
    const int lane = threadIdx.x & 63;
    const uint64_t wave = (uint64_t)blockIdx.x * (kThreads / 64) + (threadIdx.x >> 6);
    const uint64_t nwaves = (uint64_t)gridDim.x * (kThreads / 64);
    for (uint64_t b0 = wave * kBucketBlocks; b0 < a.nblocks; b0 += nwaves * kBucketBlocks) {
        const uint64_t span_begin = b0 * kBlock;
        const uint64_t span_end = span_begin + (uint64_t)kBucketBlocks * kBlock < a.total
                                      ? span_begin + (uint64_t)kBucketBlocks * kBlock : a.total;
        uint32_t t_first, t_last;
        wave_find_tensor_pair(a.offsets, 1, 0, a.ntensors, span_begin, span_end - 1, &t_first, &t_last);
        uint4 lo[kBucketBlocks], hi[kBucketBlocks];
        const bool one_tensor = t_first == t_last && span_end - span_begin == (uint64_t)kBucketBlocks * kBlock;
        if (one_tensor) {  // wave-uniform
            const char* src = a.tensors[t_first] + (span_begin - a.offsets[t_first]) * 2;
#pragma unroll
            for (int j = 0; j < kBucketBlocks; ++j) {
                lo[j] = load16_unaligned(src + j * 2048 + lane * 16);
                hi[j] = load16_unaligned(src + j * 2048 + 1024 + lane * 16);
            }
        }
#pragma unroll
        for (int j = 0; j < kBucketBlocks; ++j) {
            const uint64_t b = b0 + j;
            if (b >= a.nblocks) break;
            const uint64_t begin = b * kBlock;
            const uint64_t end = begin + kBlock < a.total ? begin + kBlock : a.total;
            if (end - begin < kBlock) {  // short final block
                quantize_bucket_block_careful(q, scales, a, t_first, t_last, begin, (uint32_t)(end - begin), b, lane);
                continue;
            }
            if (!one_tensor) {
                lo[j] = bucket_load8_bf16(a, t_first, t_last, begin + lane * 8);
                hi[j] = bucket_load8_bf16(a, t_first, t_last, begin + 512 + lane * 8);
            }
            const uint32_t w[8] = {lo[j].x, lo[j].y, lo[j].z, lo[j].w, hi[j].x, hi[j].y, hi[j].z, hi[j].w};
            uint32_t m = 0;
#pragma unroll
            for (int k = 0; k < 8; ++k) {
                const uint32_t v = w[k] & 0x7fff7fffu;
                const uint32_t v0 = v & 0xffffu, v1 = v >> 16;
                m = v0 > m ? v0 : m;
                m = v1 > m ? v1 : m;
            }
            m = wave_max_u32(m);
            if (m >= 0x7f80u) {  // Inf or NaN in the block
                quantize_bucket_block_careful(q, scales, a, t_first, t_last, begin, kBlock, b, lane);
                continue;
            }
            float scale, inv;
            block_factors(m, &scale, &inv);
            if (lane == 0) scales[b] = scale;
            int c0 = 0, c1 = 0, c2 = 0, c3 = 0;
            c0 = quant_pair<false>(w[0], inv, c0); c0 = quant_pair<true>(w[1], inv, c0);
            c1 = quant_pair<false>(w[2], inv, c1); c1 = quant_pair<true>(w[3], inv, c1);
            c2 = quant_pair<false>(w[4], inv, c2); c2 = quant_pair<true>(w[5], inv, c2);
            c3 = quant_pair<false>(w[6], inv, c3); c3 = quant_pair<true>(w[7], inv, c3);
            uint8_t* dst = q + begin;
            store8_unaligned(dst + lane * 8, (uint32_t)c0, (uint32_t)c1);
            store8_unaligned(dst + 512 + lane * 8, (uint32_t)c2, (uint32_t)c3);
        }
    }
}

// out_t[j] += float(q[off_t + j]) * scale[(off_t + j) / 1024], accumulators are the bucket's
// own fp32 tensors.  One wavefront per 1024-element block, 4 lanes-groups of 4 elements each.
__global__ __launch_bounds__(kThreads) void fp8_dequant_accumulate_bucket_kernel(const uint8_t* __restrict__ q,
                                                                                 const float* __restrict__ scales,
                                                                                 BucketArgs a) {
    const int lane = threadIdx.x & 63;
    const uint64_t wave = (uint64_t)blockIdx.x * (kThreads / 64) + (threadIdx.x >> 6);
    const uint64_t nwaves = (uint64_t)gridDim.x * (kThreads / 64);
    for (uint64_t b = wave; b < a.nblocks; b += nwaves) {
        const uint64_t begin = b * kBlock;
        const uint64_t end = begin + kBlock < a.total ? begin + kBlock : a.total;
        uint32_t t_lo, t_hi;
        wave_find_tensor_pair(a.offsets, 1, 0, a.ntensors, begin, end - 1, &t_lo, &t_hi);
        const float s = scales[b];
        if (t_lo == t_hi && end - begin == kBlock) {
            // the whole block lies in one tensor: 4 steps of 256 elements, all loads first
            float* dst = reinterpret_cast<float*>(a.tensors[t_lo]) + (begin - a.offsets[t_lo]);
            uint32_t codes[4];
            uint4 acc[4];
#pragma unroll
            for (int j = 0; j < 4; ++j) {
                codes[j] = load4_unaligned(q + begin + j * 256 + lane * 4);
                acc[j] = load16_unaligned(dst + j * 256 + lane * 4);
            }
#pragma unroll
            for (int j = 0; j < 4; ++j) {
                const auto p01 = __builtin_amdgcn_cvt_pk_f32_fp8((int)codes[j], false);
                const auto p23 = __builtin_amdgcn_cvt_pk_f32_fp8((int)codes[j], true);
                uint4 r;
                r.x = __float_as_uint(__uint_as_float(acc[j].x) + p01[0] * s);
                r.y = __float_as_uint(__uint_as_float(acc[j].y) + p01[1] * s);
                r.z = __float_as_uint(__uint_as_float(acc[j].z) + p23[0] * s);
                r.w = __float_as_uint(__uint_as_float(acc[j].w) + p23[1] * s);
                store16_unaligned(dst + j * 256 + lane * 4, r);
            }
            continue;
        }
        // straddling or short block: element by element, 16 per lane at most
        for (uint64_t e = begin + lane; e < end; e += 64) {
            const uint32_t t = find_tensor(a.offsets, 1, t_lo, t_hi + 1, e);
            float* p = reinterpret_cast<float*>(a.tensors[t]) + (e - a.offsets[t]);
            const auto v = __builtin_amdgcn_cvt_pk_f32_fp8((int)q[e], false);
            *p = *p + v[0] * s;
        }
    }
}

// The same with n peers' payloads in one pass: every accumulator element crosses HBM once
// (n + 8 bytes per element instead of 9n).  Peers are added in order, product rounded before
// each add, so the result has the bits of n single-peer passes.
constexpr int kMaxBucketPeers = 64;

struct BucketPeersArgs {
    BucketArgs b;
    const uint8_t* q[kMaxBucketPeers];
    const float* scales[kMaxBucketPeers];
    uint32_t n;
};

__global__ __launch_bounds__(kThreads) void fp8_dequant_accumulate_bucket_many_kernel(BucketPeersArgs p) {
    const BucketArgs& a = p.b;
    const int lane = threadIdx.x & 63;
    const uint64_t wave = (uint64_t)blockIdx.x * (kThreads / 64) + (threadIdx.x >> 6);
    const uint64_t nwaves = (uint64_t)gridDim.x * (kThreads / 64);
    for (uint64_t b = wave; b < a.nblocks; b += nwaves) {
        const uint64_t begin = b * kBlock;
        const uint64_t end = begin + kBlock < a.total ? begin + kBlock : a.total;
        uint32_t t_lo, t_hi;
        wave_find_tensor_pair(a.offsets, 1, 0, a.ntensors, begin, end - 1, &t_lo, &t_hi);
        if (t_lo == t_hi && end - begin == kBlock) {
            float* dst = reinterpret_cast<float*>(a.tensors[t_lo]) + (begin - a.offsets[t_lo]);
            float v[4][4];
#pragma unroll
            for (int j = 0; j < 4; ++j) {
                const uint4 r = load16_unaligned(dst + j * 256 + lane * 4);
                v[j][0] = __uint_as_float(r.x); v[j][1] = __uint_as_float(r.y);
                v[j][2] = __uint_as_float(r.z); v[j][3] = __uint_as_float(r.w);
            }
            for (uint32_t r0 = 0; r0 < p.n; r0 += 4) {
                uint32_t codes[4][4];
                float s[4];
#pragma unroll
                for (int g = 0; g < 4; ++g) {
                    const uint32_t r = r0 + g < p.n ? r0 + g : p.n - 1;  // clamped: surplus loads are unused
                    s[g] = p.scales[r][b];
#pragma unroll
                    for (int j = 0; j < 4; ++j) codes[g][j] = load4_unaligned(p.q[r] + begin + j * 256 + lane * 4);
                }
#pragma unroll
                for (int g = 0; g < 4; ++g) {
                    if (r0 + g < p.n) {
#pragma unroll
                        for (int j = 0; j < 4; ++j) {
                            const auto p01 = __builtin_amdgcn_cvt_pk_f32_fp8((int)codes[g][j], false);
                            const auto p23 = __builtin_amdgcn_cvt_pk_f32_fp8((int)codes[g][j], true);
                            v[j][0] = v[j][0] + p01[0] * s[g];
                            v[j][1] = v[j][1] + p01[1] * s[g];
                            v[j][2] = v[j][2] + p23[0] * s[g];
                            v[j][3] = v[j][3] + p23[1] * s[g];
                        }
                    }
                }
            }
#pragma unroll
            for (int j = 0; j < 4; ++j)
                store16_unaligned(dst + j * 256 + lane * 4, make_uint4(__float_as_uint(v[j][0]), __float_as_uint(v[j][1]),
                                                                      __float_as_uint(v[j][2]), __float_as_uint(v[j][3])));
            continue;
        }
        for (uint64_t e = begin + lane; e < end; e += 64) {
            const uint32_t t = find_tensor(a.offsets, 1, t_lo, t_hi + 1, e);
            float* ptr = reinterpret_cast<float*>(a.tensors[t]) + (e - a.offsets[t]);
            float x = *ptr;
            for (uint32_t r = 0; r < p.n; ++r) {
                const auto c = __builtin_amdgcn_cvt_pk_f32_fp8((int)p.q[r][e], false);
                x = x + c[0] * p.scales[r][b];
            }
            *ptr = x;
        }
    }
}

}  // namespace mhip

using namespace mhip;

extern "C" {

int mhip_fp8_quantize_bucket(uint8_t* q, float* scales, const void* const* d_tensors, const uint64_t* d_offsets,
                             uint32_t ntensors, uint64_t total, uint32_t block, mhip_stream_t stream) {
    if (block != kBlock) return MHIP_ERR_UNSUPPORTED_BLOCK;
    if (ntensors == 0 || total == 0) return MHIP_SUCCESS;
    if (!q || !scales || !d_tensors || !d_offsets) return MHIP_ERR_UNDEFINED_TENSOR;
    if ((uintptr_t)scales & 3u) return MHIP_ERR_INVALID_ARGUMENT;
    BucketArgs a{};
    a.tensors = reinterpret_cast<char* const*>(const_cast<void* const*>(reinterpret_cast<const void* const*>(d_tensors)));
    a.offsets = d_offsets;
    a.total = total;
    a.nblocks = (total + kBlock - 1) / kBlock;
    a.ntensors = ntensors;
    const uint64_t per_wg = (kThreads / 64) * kBucketBlocks;
    const uint64_t wgs = (a.nblocks + per_wg - 1) / per_wg;
    const uint64_t cap = 0x7fffffffull;
    hipStream_t hs = static_cast<hipStream_t>(stream);
    DeviceGuard guard(hs);
    hipLaunchKernelGGL(fp8_quantize_bucket_kernel, dim3((uint32_t)(wgs > cap ? cap : wgs)), dim3(kThreads), 0, hs, q,
                       scales, a);
    return launch_status();
}

int mhip_fp8_dequant_accumulate_bucket(void* const* d_acc_tensors, const uint8_t* q, const float* scales,
                                       const uint64_t* d_offsets, uint32_t ntensors, uint64_t total, uint32_t block,
                                       mhip_stream_t stream) {
    if (block != kBlock) return MHIP_ERR_UNSUPPORTED_BLOCK;
    if (ntensors == 0 || total == 0) return MHIP_SUCCESS;
    if (!q || !scales || !d_acc_tensors || !d_offsets) return MHIP_ERR_UNDEFINED_TENSOR;
    if ((uintptr_t)scales & 3u) return MHIP_ERR_INVALID_ARGUMENT;
    BucketArgs a{};
    a.tensors = reinterpret_cast<char* const*>(d_acc_tensors);
    a.offsets = d_offsets;
    a.total = total;
    a.nblocks = (total + kBlock - 1) / kBlock;
    a.ntensors = ntensors;
    const uint64_t wgs = (a.nblocks + 3) / 4;
    const uint64_t cap = 0x7fffffffull;
    hipStream_t hs = static_cast<hipStream_t>(stream);
    DeviceGuard guard(hs);
    hipLaunchKernelGGL(fp8_dequant_accumulate_bucket_kernel, dim3((uint32_t)(wgs > cap ? cap : wgs)), dim3(kThreads), 0,
                       hs, q, scales, a);
    return launch_status();
}

int mhip_fp8_dequant_accumulate_bucket_many(void* const* d_acc_tensors, const uint8_t* const* q,
                                            const float* const* scales, uint32_t n, const uint64_t* d_offsets,
                                            uint32_t ntensors, uint64_t total, uint32_t block, mhip_stream_t stream) {
    if (block != kBlock) return MHIP_ERR_UNSUPPORTED_BLOCK;
    if (!q || !scales || n == 0) return MHIP_ERR_INVALID_ARGUMENT;
    if (n > (uint32_t)kMaxBucketPeers) return MHIP_ERR_TOO_MANY_INPUTS;
    if (ntensors == 0 || total == 0) return MHIP_SUCCESS;
    if (!d_acc_tensors || !d_offsets) return MHIP_ERR_UNDEFINED_TENSOR;
    BucketPeersArgs p{};
    for (uint32_t r = 0; r < n; ++r) {
        if (!q[r] || !scales[r]) return MHIP_ERR_UNDEFINED_TENSOR;
        if ((uintptr_t)scales[r] & 3u) return MHIP_ERR_INVALID_ARGUMENT;
        p.q[r] = q[r];
        p.scales[r] = scales[r];
    }
    p.n = n;
    p.b.tensors = reinterpret_cast<char* const*>(d_acc_tensors);
    p.b.offsets = d_offsets;
    p.b.total = total;
    p.b.nblocks = (total + kBlock - 1) / kBlock;
    p.b.ntensors = ntensors;
    const uint64_t wgs = (p.b.nblocks + 3) / 4;
    const uint64_t cap = 0x7fffffffull;
    hipStream_t hs = static_cast<hipStream_t>(stream);
    DeviceGuard guard(hs);
    hipLaunchKernelGGL(fp8_dequant_accumulate_bucket_many_kernel, dim3((uint32_t)(wgs > cap ? cap : wgs)), dim3(kThreads),
                       0, hs, p);
    return launch_status();
}

}  // extern "C"
