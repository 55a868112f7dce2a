// Block-scaled fp8 (OCP e4m3fn) codec for flat bf16 transfer buffers, gfx950.
//
// quantize: 3 bytes of HBM traffic per element (2 in, 1 out) + 4 per 1024-element block.
//   One wavefront owns one 1024-element block: each lane holds 16 elements in registers
//   (two 128-bit loads, each a fully coalesced 1 KiB wavefront access), the block absmax
//   is a lane-local max over packed 16-bit magnitudes followed by a DPP butterfly inside
//   each row of 16 lanes and four readlanes across rows - no LDS, no second pass over
//   memory - and the 16 codes leave as two 64-bit stores.
// dequant_accumulate: 9 bytes per element (1 code in, fp32 accumulator in and out).
//   A 256-thread workgroup step covers exactly one block, so the scale is uniform.
#include "fp8_common.h"

namespace mhip {

// Careful path for one block, whole wavefront: handles a short final block and blocks
// holding NaN or Inf (NaN is ignored by the absmax and encodes to an fp8 NaN; Inf
// saturates to +-448).
__device__ __noinline__ void quantize_block_careful(uint8_t* __restrict__ q, float* __restrict__ scales,
                                                    const uint16_t* __restrict__ x, uint64_t begin, uint32_t count,
                                                    uint64_t b, int lane) {
    // lane l owns elements l, 64 + l, ... of the block; all of its loads are issued before the first use
    constexpr int kSlots = kBlock / 64;
    uint16_t v[kSlots];
#pragma unroll
    for (int j = 0; j < kSlots; ++j) {
        const uint32_t i = j * 64 + lane;
        const uint16_t e = x[begin + (i < count ? i : count - 1)];  // no load is predicated
        v[j] = i < count ? e : (uint16_t)0;                          // elements past a short block's end count as zeros
    }
    uint32_t m = 0;
#pragma unroll
    for (int j = 0; j < kSlots; ++j) {
        const uint32_t a = v[j] & 0x7fffu;
        if (a <= 0x7f80u && a > m) m = a;
    }
    m = wave_max_u32(m);
    float scale, inv;
    block_factors(m, &scale, &inv);
    if (lane == 0) scales[b] = scale;
#pragma unroll
    for (int j = 0; j < kSlots; ++j) {
        const uint32_t i = j * 64 + lane;
        if (i < count) q[begin + i] = quant_one_careful(v[j], inv);
    }
}

// Blocks a wavefront quantises per step (all their loads are issued before the first max).  Measured on
// the 756 M-element bucket: 1 block 0.81 of peak, 2 blocks 0.79, 4 blocks 0.78 - more, smaller wavefront
// steps stream better than deeper ones here, as in the copy and reduce kernels.
constexpr int kQuantBlocks = 1;
constexpr int kQuantThreads = 64;  // single-wavefront workgroups: 0.825 of peak against 0.81 with 256 lanes

__global__ __launch_bounds__(kQuantThreads) void fp8_quantize_kernel(uint8_t* __restrict__ q, float* __restrict__ scales,
                                                                const uint16_t* __restrict__ x, uint64_t numel,
                                                                uint64_t nblocks) {
    const int lane = threadIdx.x & 63;
    const uint64_t wave = (uint64_t)blockIdx.x * (kQuantThreads / 64) + (threadIdx.x >> 6);
    const uint64_t nwaves = (uint64_t)gridDim.x * (kQuantThreads / 64);
    for (uint64_t b0 = wave * kQuantBlocks; b0 < nblocks; b0 += nwaves * kQuantBlocks) {
        uint4 lo[kQuantBlocks], hi[kQuantBlocks];
        bool full[kQuantBlocks];
#pragma unroll
        for (int j = 0; j < kQuantBlocks; ++j) {
            const uint64_t begin = (b0 + j) * kBlock;
            full[j] = b0 + j < nblocks && numel - begin >= kBlock;  // wave-uniform
            if (full[j]) {
                const char* src = reinterpret_cast<const char*>(x + begin);
                lo[j] = load16_unaligned(src + lane * 16);         // elements [8*lane, 8*lane+8)
                hi[j] = load16_unaligned(src + 1024 + lane * 16);  // elements [512+8*lane, ...)
            }
        }
#pragma unroll
        for (int j = 0; j < kQuantBlocks; ++j) {
            const uint64_t b = b0 + j;
            if (b >= nblocks) break;
            const uint64_t begin = b * kBlock;
            if (!full[j]) {  // short final block
                quantize_block_careful(q, scales, x, begin, (uint32_t)(numel - begin), b, lane);
                continue;
            }
            // magnitudes as 16-bit integers: bf16 order == integer order for |x|
            const uint32_t w[8] = {lo[j].x, lo[j].y, lo[j].z, lo[j].w, hi[j].x, hi[j].y, hi[j].z, hi[j].w};
            uint32_t m = 0;
#pragma unroll
            for (int k = 0; k < 8; ++k) {
                const uint32_t a = w[k] & 0x7fff7fffu;
                const uint32_t a0 = a & 0xffffu, a1 = a >> 16;
                m = a0 > m ? a0 : m;
                m = a1 > m ? a1 : m;
            }
            m = wave_max_u32(m);
            if (m >= 0x7f80u) {  // Inf or NaN somewhere in the block (wave-uniform, rare)
                quantize_block_careful(q, scales, x, begin, kBlock, b, lane);
                continue;
            }
            float scale, inv;
            block_factors(m, &scale, &inv);
            if (lane == 0) scales[b] = scale;
            // |x * inv| <= 448 * (1 + 2^-22) for every finite x of the block, which rounds to
            // at most 448, so no clamp is needed on this path.
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

// acc[i] += float(q[i]) * scale[i / 1024].  A workgroup covers kDeqThreads * 4 consecutive
// elements (a whole fraction of one block), four per lane: one 32-bit load of codes and one
// 128-bit load / store of the accumulator.
constexpr int kDeqThreads = 64;
constexpr int kDeqTile = kDeqThreads * 4;  // elements per workgroup
static_assert(kBlock % kDeqTile == 0, "a tile lies inside one block");

__global__ __launch_bounds__(kDeqThreads) void fp8_dequant_accumulate_kernel(float* __restrict__ acc,
                                                                             const uint8_t* __restrict__ q,
                                                                             const float* __restrict__ scales,
                                                                             uint64_t numel, uint64_t ntiles) {
    for (uint64_t tile = blockIdx.x; tile < ntiles; tile += gridDim.x) {
        const uint64_t i0 = tile * kDeqTile + threadIdx.x * 4;
        if ((tile + 1) * kDeqTile <= numel) {  // interior tile (workgroup-uniform)
            const uint32_t c = load4_unaligned(q + i0);
            const uint4 v = load16_unaligned(acc + i0);
            const float sc = scales[tile * kDeqTile / kBlock];
            const auto p01 = __builtin_amdgcn_cvt_pk_f32_fp8((int)c, false);
            const auto p23 = __builtin_amdgcn_cvt_pk_f32_fp8((int)c, true);
            // product rounded to fp32, then added: two roundings (contraction is off)
            uint4 r;
            r.x = __float_as_uint(__uint_as_float(v.x) + p01[0] * sc);
            r.y = __float_as_uint(__uint_as_float(v.y) + p01[1] * sc);
            r.z = __float_as_uint(__uint_as_float(v.z) + p23[0] * sc);
            r.w = __float_as_uint(__uint_as_float(v.w) + p23[1] * sc);
            store16_unaligned(acc + i0, r);
            continue;
        }
        // last tile: single elements at the ragged end
        for (uint64_t e = i0; e < numel && e < i0 + 4; ++e) {
            const auto p = __builtin_amdgcn_cvt_pk_f32_fp8((int)q[e], false);
            acc[e] = acc[e] + p[0] * scales[e / kBlock];
        }
    }
}

// acc[i] (+)= sum over r of float(q_r[i]) * scales_r[i / 1024], peers in order, every product
// rounded before its add: the same bits as n calls of the kernel above, but the fp32
// accumulator crosses HBM once instead of n times (n + 8 bytes per element instead of 9n;
// n + 4 when `overwrite` starts from zero instead of reading acc).
constexpr int kMaxPeers = 64;
struct DequantManyArgs {
    float* acc;
    const uint8_t* q[kMaxPeers];
    const float* scales[kMaxPeers];
    uint64_t numel;
    uint64_t ntiles;
    uint32_t n;
    uint32_t overwrite;
    uint32_t rotate;  // workgroup i takes tile i + i / 8 of its group of 8 tiles (see the entry point)
};

// N > 0: peers known at compile time; N == 0: a.n peers, eight at a time.  THREADS lanes cover THREADS * 4
// elements: single wavefronts are best when the accumulator is read (8 peers: 0.805 of peak against 0.80),
// 256 lanes when it is only written (0.82 against 0.78).
template <int N, int THREADS>
__global__ __launch_bounds__(THREADS) void fp8_dequant_accumulate_many_kernel(DequantManyArgs a) {
    constexpr int TILE = THREADS * 4;
    static_assert(kBlock % TILE == 0, "a tile lies inside one block");
    float* __restrict__ acc = a.acc;
    const uint32_t n = N > 0 ? N : a.n;
    uint32_t first = blockIdx.x;
    if (a.rotate && first < (gridDim.x & ~7u)) first = (first & ~7u) | ((first + (first >> 3)) & 7u);
    for (uint64_t tile = first; tile < a.ntiles; tile += gridDim.x) {
        const uint64_t i0 = tile * TILE + threadIdx.x * 4;
        if ((tile + 1) * TILE <= a.numel) {  // interior tile, workgroup-uniform
            const uint64_t b = tile * TILE / kBlock;
            float v[4] = {0.0f, 0.0f, 0.0f, 0.0f};
            if (!a.overwrite) {
                const uint4 r = load16_unaligned(acc + i0);
                v[0] = __uint_as_float(r.x); v[1] = __uint_as_float(r.y);
                v[2] = __uint_as_float(r.z); v[3] = __uint_as_float(r.w);
            }
            for (uint32_t r0 = 0; r0 < n; r0 += 8) {
                constexpr int G = N > 0 && N < 8 ? N : 8;
                uint32_t codes[G];
                float s[G];
#pragma unroll
                for (int g = 0; g < G; ++g) {
                    const uint32_t r = r0 + g < n ? r0 + g : n - 1;  // clamped: the extra loads of a short last group are unused
                    codes[g] = load4_unaligned(a.q[r] + i0);
                    s[g] = a.scales[r][b];
                }
#pragma unroll
                for (int g = 0; g < G; ++g) {
                    if (r0 + g < n) {
                        const auto p01 = __builtin_amdgcn_cvt_pk_f32_fp8((int)codes[g], false);
                        const auto p23 = __builtin_amdgcn_cvt_pk_f32_fp8((int)codes[g], true);
                        v[0] = v[0] + p01[0] * s[g];
                        v[1] = v[1] + p01[1] * s[g];
                        v[2] = v[2] + p23[0] * s[g];
                        v[3] = v[3] + p23[1] * s[g];
                    }
                }
            }
            store16_unaligned(acc + i0, make_uint4(__float_as_uint(v[0]), __float_as_uint(v[1]),
                                                   __float_as_uint(v[2]), __float_as_uint(v[3])));
            continue;
        }
        // last tile: element by element, eight peers' codes in flight at a time
        for (uint64_t e = i0; e < a.numel && e < i0 + 4; ++e) {
            float x = a.overwrite ? 0.0f : acc[e];
            for (uint32_t r0 = 0; r0 < n; r0 += 8) {
                uint8_t c[8];
                float s[8];
#pragma unroll
                for (int g = 0; g < 8; ++g) {
                    const uint32_t r = r0 + g < n ? r0 + g : n - 1;  // clamped: surplus loads are unused
                    c[g] = a.q[r][e];
                    s[g] = a.scales[r][e / kBlock];
                }
#pragma unroll
                for (int g = 0; g < 8; ++g) {
                    if (r0 + g < n) {
                        const auto p = __builtin_amdgcn_cvt_pk_f32_fp8((int)c[g], false);
                        x = x + p[0] * s[g];
                    }
                }
            }
            acc[e] = x;
        }
    }
}

template <int THREADS>
static void launch_dequant_many(DequantManyArgs& a, hipStream_t hs) {
    a.ntiles = (a.numel + THREADS * 4 - 1) / (THREADS * 4);
    const uint64_t cap = max_workgroups(THREADS);
    const dim3 grid((uint32_t)(a.ntiles > cap ? cap : a.ntiles)), blockdim(THREADS);
    switch (a.n) {
        case 2: MHIP_LAUNCH((fp8_dequant_accumulate_many_kernel<2, THREADS>), grid, blockdim, 0, hs, a); break;
        case 4: MHIP_LAUNCH((fp8_dequant_accumulate_many_kernel<4, THREADS>), grid, blockdim, 0, hs, a); break;
        case 8: MHIP_LAUNCH((fp8_dequant_accumulate_many_kernel<8, THREADS>), grid, blockdim, 0, hs, a); break;
        default: MHIP_LAUNCH((fp8_dequant_accumulate_many_kernel<0, THREADS>), grid, blockdim, 0, hs, a); break;
    }
}

}  // namespace mhip

using namespace mhip;

extern "C" {

int mhip_fp8_quantize(uint8_t* q, float* scales, const void* x_bf16, uint64_t numel, uint32_t block,
                      mhip_stream_t stream) {
    if (block != kBlock) return MHIP_ERR_UNSUPPORTED_BLOCK;
    if (numel == 0) return MHIP_SUCCESS;
    if (!q || !scales || !x_bf16) return MHIP_ERR_UNDEFINED_TENSOR;
    if (((uintptr_t)x_bf16 & 1u) || ((uintptr_t)scales & 3u)) return MHIP_ERR_INVALID_ARGUMENT;
    const uint64_t nblocks = (numel + kBlock - 1) / kBlock;
    const uint64_t per_wg = (kQuantThreads / 64) * kQuantBlocks;
    const uint64_t wgs = (nblocks + per_wg - 1) / per_wg;
    const uint64_t cap = max_workgroups(kQuantThreads);
    hipStream_t hs = static_cast<hipStream_t>(stream);
    DeviceGuard guard(hs);
    MHIP_LAUNCH(fp8_quantize_kernel, dim3((uint32_t)(wgs > cap ? cap : wgs)), dim3(kQuantThreads), 0, hs, q, scales,
                       static_cast<const uint16_t*>(x_bf16), numel, nblocks);
    return launch_status();
}

int mhip_fp8_dequant_accumulate(float* acc, const uint8_t* q, const float* scales, uint64_t numel, uint32_t block,
                                mhip_stream_t stream) {
    if (block != kBlock) return MHIP_ERR_UNSUPPORTED_BLOCK;
    if (numel == 0) return MHIP_SUCCESS;
    if (!acc || !q || !scales) return MHIP_ERR_UNDEFINED_TENSOR;
    if (((uintptr_t)acc & 3u) || ((uintptr_t)scales & 3u)) return MHIP_ERR_INVALID_ARGUMENT;
    const uint64_t ntiles = (numel + kDeqTile - 1) / kDeqTile;
    const uint64_t cap = max_workgroups(kDeqThreads);
    hipStream_t hs = static_cast<hipStream_t>(stream);
    DeviceGuard guard(hs);
    MHIP_LAUNCH(fp8_dequant_accumulate_kernel, dim3((uint32_t)(ntiles > cap ? cap : ntiles)), dim3(kDeqThreads), 0,
                       hs, acc, q, scales, numel, ntiles);
    return launch_status();
}

int mhip_fp8_dequant_accumulate_many(float* acc, const uint8_t* const* q, const float* const* scales, uint32_t n,
                                     uint64_t numel, uint32_t block, int overwrite, mhip_stream_t stream) {
    if (block != kBlock) return MHIP_ERR_UNSUPPORTED_BLOCK;
    if (!q || !scales || n == 0) return MHIP_ERR_INVALID_ARGUMENT;
    if (n > (uint32_t)kMaxPeers) return MHIP_ERR_TOO_MANY_INPUTS;
    if (numel == 0) return MHIP_SUCCESS;
    if (!acc) return MHIP_ERR_UNDEFINED_TENSOR;
    if ((uintptr_t)acc & 3u) return MHIP_ERR_INVALID_ARGUMENT;
    DequantManyArgs a{};
    for (uint32_t r = 0; r < n; ++r) {
        if (!q[r] || !scales[r]) return MHIP_ERR_UNDEFINED_TENSOR;
        if ((uintptr_t)scales[r] & 3u) return MHIP_ERR_INVALID_ARGUMENT;
        a.q[r] = q[r];
        a.scales[r] = scales[r];
    }
    a.acc = acc;
    a.numel = numel;
    a.n = n;
    a.overwrite = overwrite ? 1u : 0u;
    // Workgroup i runs on XCD i mod 8 and reads the same 256 bytes of every peer's codes, so with peers' buffers that
    // start at the same place in 2 KiB (separate allocations do) an XCD only ever sees one eighth of the address
    // phases, n times over.  Rotating the tile a workgroup takes inside its group of 8 by one per group spreads them:
    // 8 peers 0.778 -> 0.793 of peak.  The one-peer kernels lose 0.03 with it and keep the plain order.
    if (n >= 4) {
        uint32_t count[8] = {0, 0, 0, 0, 0, 0, 0, 0}, most = 0;
        for (uint32_t r = 0; r < n; ++r) ++count[((uintptr_t)q[r] >> 8) & 7u];
        for (uint32_t c : count) most = c > most ? c : most;
        a.rotate = most * 2 > n ? 1u : 0u;
    }
    hipStream_t hs = static_cast<hipStream_t>(stream);
    DeviceGuard guard(hs);
    if (a.overwrite) launch_dequant_many<256>(a, hs);
    else launch_dequant_many<kDeqThreads>(a, hs);
    return launch_status();
}

}  // extern "C"
