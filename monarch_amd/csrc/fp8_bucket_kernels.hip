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
// hold the first and the last element of its span from the bucket's block index (or with two
// cooperative 65-ary searches over the offsets table); a span inside one tensor (the common
// case: tensors are >= 1K elements) then costs nothing extra; a span or block that one
// boundary between two tensors cuts is loaded in one go as well, each lane's vector from the
// tensor it lies in; what is left (more boundaries, the short last block, blocks with Inf or
// NaN) is walked tensor by tensor, the lanes taking consecutive elements of each segment.
#include <mutex>

#include "fp8_common.h"

namespace mhip {

struct BucketArgs {
    char* const* tensors;     // device table of ntensors pointers
    const uint64_t* offsets;  // device table of ntensors + 1 element offsets
    const uint32_t* index;    // block index (see bucket_index_kernel), or null: search the offsets table
    uint64_t total;           // elements in the bucket
    uint64_t nblocks;
    uint32_t ntensors;
};

// Block index of a bucket: index[b] = the tensor that holds flat element b * 1024 for b < nblocks, and
// index[nblocks] = ntensors - 1.  Built once per bucket (the offsets do not change between steps), it replaces the
// table search every wavefront otherwise does per span: one load instead of two dependent probe rounds.
__global__ __launch_bounds__(kThreads) void bucket_index_kernel(uint32_t* __restrict__ index, const uint64_t* __restrict__ offsets,
                                                                uint32_t ntensors, uint64_t nblocks) {
    const uint64_t stride = (uint64_t)gridDim.x * kThreads;
    for (uint64_t b = (uint64_t)blockIdx.x * kThreads + threadIdx.x; b <= nblocks; b += stride)
        index[b] = b < nblocks ? find_tensor(offsets, 1, 0, ntensors, b * kBlock) : ntensors - 1;
}

// Tensors of the first and the last element of [begin, end), begin a block start.  With an index, *t_hi is exact
// when it equals *t_lo and an upper bound otherwise (the tensor-by-tensor walks skip the empty segments).
// All 64 lanes call it with the same arguments.
__device__ __forceinline__ void span_tensors(const BucketArgs& a, uint64_t begin, uint64_t end, uint32_t* t_lo, uint32_t* t_hi) {
    if (a.index != nullptr) {
        // clamped: an index that was built for another bucket, or that another call on this GPU is rewriting (the
        // library's static index is shared), must not send the table reads out of bounds
        const uint32_t last = a.ntensors - 1;
        uint32_t lo = a.index[begin / kBlock];
        lo = lo < last ? lo : last;
        uint32_t hi = a.offsets[lo + 1] >= end ? lo : a.index[(end + kBlock - 1) / kBlock];
        *t_lo = lo;
        *t_hi = hi < last ? hi : last;
    } else {
        wave_find_tensor_pair(a.offsets, 1, 0, a.ntensors, begin, end - 1, t_lo, t_hi);
    }
}

// Careful path for one block that straddles tensors, holds NaN / Inf, or is the short last block of
// the bucket, whole wavefront.  [t_lo, t_hi] are the tensors of its first and last element (t_hi may be an
// upper bound).  Lane l owns elements l, 64 + l, ... of the block, sixteen at most.  The block is walked tensor by
// tensor (a wave-uniform loop whose table reads are scalar loads): inside a segment the lanes read consecutive
// elements from one base pointer, no lane searches the table, and all loads of a segment are issued before any
// value is used, so the block costs a few memory latencies.  (Sixteen dependent 64-element steps per pass, as
// this path was first written, made a straddling span cost its wavefront about 10 us: invisible behind a 1.5 GB
// bucket, but most of the run time of a bucket of 4 M elements.)
constexpr int kCarefulSlots = kBlock / 64;

__device__ __forceinline__ void quantize_bucket_block_careful(uint8_t* __restrict__ q, float* __restrict__ scales,
                                                           char* const* tensors, const uint64_t* offsets, uint32_t t_lo,
                                                           uint32_t t_hi, uint64_t begin, uint32_t count, uint64_t b,
                                                           int lane) {
    const uint64_t end = begin + count;
    uint16_t x[kCarefulSlots];
#pragma unroll
    for (int j = 0; j < kCarefulSlots; ++j) x[j] = 0;  // elements past a short block's end count as zeros
    for (uint32_t t = t_lo; t <= t_hi; ++t) {
        const uint64_t off = offsets[t], next = offsets[t + 1];
        const uint64_t seg_b = begin > off ? begin : off, seg_e = end < next ? end : next;
        if (seg_b >= seg_e) continue;  // an empty tensor, or one past the block
        // The segment is elements [lo, hi) of the block, read from p.  No load is predicated (a lane outside the
        // segment reads the segment's nearest element and drops it), so all of them are in flight together.
        const uint16_t* __restrict__ p = reinterpret_cast<const uint16_t*>(tensors[t]) + (begin - off);
        const uint32_t lo = (uint32_t)(seg_b - begin), hi = (uint32_t)(seg_e - begin);
        uint16_t v[kCarefulSlots];
#pragma unroll
        for (int j = 0; j < kCarefulSlots; ++j) {
            const uint32_t i = j * 64 + lane;
            v[j] = p[i < lo ? lo : i >= hi ? hi - 1 : i];
        }
#pragma unroll
        for (int j = 0; j < kCarefulSlots; ++j) {
            const uint32_t i = j * 64 + lane;
            if (i >= lo && i < hi) x[j] = v[j];
        }
    }
    uint32_t m = 0;
#pragma unroll
    for (int j = 0; j < kCarefulSlots; ++j) {
        const uint32_t v = x[j] & 0x7fffu;
        if (v <= 0x7f80u && v > m) m = v;
    }
    m = wave_max_u32(m);
    float scale, inv;
    block_factors(m, &scale, &inv);
    if (lane == 0) scales[b] = scale;
#pragma unroll
    for (int j = 0; j < kCarefulSlots; ++j) {
        const uint64_t e = begin + j * 64 + lane;
        if (e < end) q[e] = quant_one_careful(x[j], inv);
    }
}

// A wavefront handles kBucketBlocks consecutive blocks per step (8 KiB of input): one
// cooperative search pair locates the tensors of the first and the last element of the
// whole span; when they coincide (the common case) all 2 * kBucketBlocks loads of a lane
// are issued back to back from one base pointer.
constexpr uint64_t kSmallBucketBlocks = 32768;  // buckets of up to 33.5 M elements take one block per wavefront step (see quantize_bucket)
constexpr int kBucketBlocks = 4;       // blocks per wavefront step of the quantiser on large buckets (template parameter NB)
// Lanes per workgroup.  Unlike the plain copy and the tensor-less quantiser, which stream best as single
// wavefronts, the bucket kernels want 4 wavefronts: quantise / dequantise / dequantise 8 peers reach
// 0.75 / 0.735 / 0.72 of peak with 256 lanes, 0.74 / 0.66 / 0.68 with 64 and 0.72 / 0.715 / 0.71 with 512.
constexpr int kBucketThreads = 256;

// One full block whose 16 elements per lane are already in registers.  Returns false (and does
// nothing) when the block holds Inf or NaN and has to take the careful path.
__device__ __forceinline__ bool quantize_loaded_block(uint8_t* __restrict__ q, float* __restrict__ scales, uint4 lo, uint4 hi,
                                                      uint64_t begin, uint64_t b, int lane) {
    const uint32_t w[8] = {lo.x, lo.y, lo.z, lo.w, hi.x, hi.y, hi.z, hi.w};
    uint32_t m = 0;
#pragma unroll
    for (int k = 0; k < 8; ++k) {
        const uint32_t v = w[k] & 0x7fff7fffu;
        const uint32_t v0 = v & 0xffffu, v1 = v >> 16;
        m = v0 > m ? v0 : m;
        m = v1 > m ? v1 : m;
    }
    m = wave_max_u32(m);
    if (m >= 0x7f80u) return false;  // wave-uniform
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
    return true;
}

// R rows of 1 KiB (512 elements each) that two tensors share: elements [0, cut) are the last ones of the first tensor,
// starting at `head`, the others the first ones of the second tensor, which starts at `next`; 0 < cut < 512 R.  A lane's
// vector comes from one of the two with the same unaligned load as in a span inside one tensor; the one vector that the
// cut goes through is fetched element by element - by every lane for its own vector of that row, which needs no
// branch - and all loads are in flight together.  (Through the careful path below a straddling block takes several
// round trips one after the other: a span of three tensors cost its wavefront about 10 us, invisible behind a 1.5 GB
// bucket and twice the rest of the run time of a bucket of 4 M elements.)
template <int R>
struct Rows {
    uint4 row[R];
};

template <int R>
__device__ __forceinline__ Rows<R> load_rows_of_two_tensors(const char* head, const char* next, uint32_t cut, int lane) {
    Rows<R> out;
    uint4 (&row)[R] = out.row;
    const char* rest = reinterpret_cast<const char*>(reinterpret_cast<uintptr_t>(next) - (uintptr_t)cut * 2);  // element e >= cut at rest + 2 e
#pragma unroll
    for (int k = 0; k < R; ++k) {
        uint32_t v0 = k * 512 + lane * 8;
        if (v0 < cut && v0 + 8 > cut) v0 = v0 >= 8 ? v0 - 8 : 8;  // the cut vector: a valid neighbour instead, replaced below
        if (v0 < cut) row[k] = load16_unaligned(head + v0 * 2);
        else row[k] = load16_unaligned(rest + v0 * 2);
    }
    if (cut % 8 != 0) {
        const uint32_t cut_row = cut / 512;
        uint32_t w[4];
#pragma unroll
        for (int i = 0; i < 8; ++i) {
            const uint32_t e = cut_row * 512 + lane * 8 + i;
            uint32_t x;
            if (e < cut) x = *reinterpret_cast<const uint16_t*>(head + e * 2);
            else x = *reinterpret_cast<const uint16_t*>(rest + e * 2);
            w[i / 2] = i % 2 ? w[i / 2] | (x << 16) : x;
        }
#pragma unroll
        for (int k = 0; k < R; ++k)
            if (k == (int)cut_row) row[k] = make_uint4(w[0], w[1], w[2], w[3]);  // wave-uniform
    }
    return out;
}

// The rare span that touches more than two tensors or holds the short last block: block by block, each block
// narrowed to its own tensors by a wave-uniform walk over the table; full blocks inside one tensor or shared by two
// are loaded first, all of them, and quantised then.  Returns the blocks (bit j: block b0 + j) that are left for the
// careful path.
template <int NB>
__device__ __forceinline__ uint32_t quantize_bucket_span_slow(uint8_t* __restrict__ q, float* __restrict__ scales,
                                                              char* const* tensors, const uint64_t* offsets, uint64_t total,
                                                              uint64_t nblocks, uint32_t ntensors, uint32_t t_first, uint32_t t_last,
                                                              uint64_t b0, int lane) {
    uint32_t redo = 0, loaded = 0;
    uint32_t tb = t_first;
    uint4 row[2 * NB];
#pragma unroll
    for (int j = 0; j < NB; ++j) {
        const uint64_t b = b0 + j;
        if (b < nblocks) {
            const uint64_t begin = b * kBlock;
            const uint64_t end = begin + kBlock < total ? begin + kBlock : total;
            while (tb < t_last && offsets[tb + 1] <= begin) ++tb;
            bool ok = false;
            if (end - begin == kBlock) {
                const uint64_t next = offsets[tb + 1];
                const char* src = tensors[tb] + (begin - offsets[tb]) * 2;
                if (next >= end) {  // a full block inside one tensor
                    row[2 * j] = load16_unaligned(src + lane * 16);
                    row[2 * j + 1] = load16_unaligned(src + 1024 + lane * 16);
                    ok = true;
                } else if (tb + 2 <= ntensors && offsets[tb + 2] >= end) {  // a full block that two tensors share
                    const Rows<2> both = load_rows_of_two_tensors<2>(src, tensors[tb + 1], (uint32_t)(next - begin), lane);
                    row[2 * j] = both.row[0];
                    row[2 * j + 1] = both.row[1];
                    ok = true;
                }
            }
            if (ok) loaded |= 1u << j;
            else redo |= 1u << j;
        }
    }
#pragma unroll
    for (int j = 0; j < NB; ++j) {
        const uint64_t b = b0 + j;
        if ((loaded >> j) & 1u)
            if (!quantize_loaded_block(q, scales, row[2 * j], row[2 * j + 1], b * kBlock, b, lane)) redo |= 1u << j;
    }
    return redo;
}
// The NB blocks of a span whose elements are in registers, row[2j] and row[2j + 1] holding block j.
// Returns the blocks (bit j: block b0 + j) that hold Inf or NaN and are left for the careful path.
template <int NB>
__device__ __forceinline__ uint32_t quantize_loaded_span(uint8_t* __restrict__ q, float* __restrict__ scales,
                                                         const uint4 (&row)[2 * NB], uint64_t b0, int lane) {
    uint32_t redo = 0;
#pragma unroll
    for (int j = 0; j < NB; ++j) {
        const uint64_t b = b0 + j;
        if (!quantize_loaded_block(q, scales, row[2 * j], row[2 * j + 1], b * kBlock, b, lane)) redo |= 1u << j;
    }
    return redo;
}

template <int NB>
__global__ __launch_bounds__(kBucketThreads) __attribute__((amdgpu_waves_per_eu(4))) void fp8_quantize_bucket_kernel(uint8_t* __restrict__ q, float* __restrict__ scales,
                                                                       BucketArgs a) {
    const int lane = threadIdx.x & 63;
    // The wavefront's number goes through a scalar register: what is derived from it (span, block index entry, offsets and
    // pointers of the span's tensors) is then wave-uniform for the compiler too.  In the quantiser, whose only stores go to
    // its restrict-qualified outputs, the table reads on the way to the first data load become scalar loads (fused
    // quantiser on the 756 M-element bucket 0.73 -> 0.79 of peak; 0.87 -> 0.94 of the flat quantiser on the same GPU).
    // The dequantisers store through pointers they loaded from a table, so the compiler keeps vector loads for their table
    // reads; forcing scalar loads there (reads through the constant address space) was measured and loses: single-peer
    // 0.746 -> 0.703, eight peers 0.716 -> 0.703, although buckets of a few MB gain 0.8 us.
    const uint64_t wave = (uint64_t)blockIdx.x * (kBucketThreads / 64) + (uint32_t)__builtin_amdgcn_readfirstlane((int)(threadIdx.x >> 6));
    const uint64_t nwaves = (uint64_t)gridDim.x * (kBucketThreads / 64);
    for (uint64_t b0 = wave * NB; b0 < a.nblocks; b0 += nwaves * NB) {
        const uint64_t span_begin = b0 * kBlock;
        const uint64_t span_end = span_begin + (uint64_t)NB * kBlock < a.total
                                      ? span_begin + (uint64_t)NB * kBlock : a.total;
        uint32_t t_first, t_last;
        span_tensors(a, span_begin, span_end, &t_first, &t_last);
        const bool full = span_end - span_begin == (uint64_t)NB * kBlock;
        // Blocks that need the careful path are only noted (bit j: block b0 + j; wave-uniform) and worked off in one
        // place at the end of the step, where the span's registers are free: inlined where the rows are live, that
        // path costs the whole kernel a quarter of its wavefronts; as a function that is not inlined, its table reads
        // become vector loads with a round trip each (6 us for one short block).
        uint32_t redo = 0;
        uint32_t t_redo = t_first;     // last tensor those blocks can touch
        uint4 row[2 * NB];  // row[2j] = first, row[2j + 1] = second 1 KiB of block j
        if (t_first == t_last && full) {
            // the whole span lies in one tensor (the common case): all loads of the lane back to back from one base pointer
            const uint64_t t_begin = a.offsets[t_first], t_end = a.offsets[t_first + 1];
            const char* src = a.tensors[t_first] + (span_begin - t_begin) * 2;
            const uint32_t shift = (uint32_t)((uintptr_t)src & 15u);
            if (shift != 0 && (span_begin - t_begin) * 2 >= shift && (t_end - span_end) * 2 >= 16 - shift) {
                const char* base = src - shift;  // 16-byte aligned, and [base, base + 8 KiB + 16) lies inside the tensor
#pragma unroll
                for (int k = 0; k < 2 * NB; ++k) row[k] = load16_aligned(base + k * 1024 + lane * 16);
                const uint4 tail = load16_aligned(base + 2 * NB * 1024);
                shift_rows_into_place<2 * NB>(row, tail, shift);
            } else {
#pragma unroll
                for (int k = 0; k < 2 * NB; ++k) row[k] = load16_unaligned(src + k * 1024 + lane * 16);
            }
            redo = quantize_loaded_span<NB>(q, scales, row, b0, lane);
        } else if (full && t_first + 2 <= a.ntensors && a.offsets[t_first + 2] >= span_end) {
            // one tensor ends inside the span and the next one holds the rest (every span that straddles tensors of
            // 4096 elements and more)
            const uint32_t cut = (uint32_t)(a.offsets[t_first + 1] - span_begin);  // 0 < cut < span length
            const char* head = a.tensors[t_first] + (span_begin - a.offsets[t_first]) * 2;
            const char* rest = reinterpret_cast<const char*>(reinterpret_cast<uintptr_t>(a.tensors[t_first + 1]) - (uintptr_t)cut * 2);
            // as in load_rows_of_two_tensors, on the span's own registers
#pragma unroll
            for (int k = 0; k < 2 * NB; ++k) {
                uint32_t v0 = k * 512 + lane * 8;
                if (v0 < cut && v0 + 8 > cut) v0 = v0 >= 8 ? v0 - 8 : 8;
                if (v0 < cut) row[k] = load16_unaligned(head + v0 * 2);
                else row[k] = load16_unaligned(rest + v0 * 2);
            }
            if (cut % 8 != 0) {
                const uint32_t cut_row = cut / 512;
                uint32_t w[4];
#pragma unroll
                for (int i = 0; i < 8; ++i) {
                    const uint32_t e = cut_row * 512 + lane * 8 + i;
                    uint32_t x;
                    if (e < cut) x = *reinterpret_cast<const uint16_t*>(head + e * 2);
                    else x = *reinterpret_cast<const uint16_t*>(rest + e * 2);
                    w[i / 2] = i % 2 ? w[i / 2] | (x << 16) : x;
                }
#pragma unroll
                for (int k = 0; k < 2 * NB; ++k)
                    if (k == (int)cut_row) row[k] = make_uint4(w[0], w[1], w[2], w[3]);  // wave-uniform
            }
            redo = quantize_loaded_span<NB>(q, scales, row, b0, lane);
            t_redo = t_first + 1;
        } else {  // more than two tensors, or the short last span of the bucket
            redo = quantize_bucket_span_slow<NB>(q, scales, a.tensors, a.offsets, a.total, a.nblocks, a.ntensors, t_first, t_last, b0, lane);
            t_redo = t_last;
        }
        for (uint64_t b = b0; redo != 0; ++b, redo >>= 1) {
            if (redo & 1u) {
                const uint64_t begin = b * kBlock;
                const uint32_t count = a.total - begin < kBlock ? (uint32_t)(a.total - begin) : (uint32_t)kBlock;
                quantize_bucket_block_careful(q, scales, a.tensors, a.offsets, t_first, t_redo, begin, count, b, lane);
            }
        }
    }
}

// The dequantisers' path for a block that straddles tensors or is the short last block of the bucket, whole
// wavefront: the accumulator elements of the block are read tensor by tensor with all loads of a segment in
// flight together (lane l owns elements l, 64 + l, ...), the n peers' codes are added in order, each peer's
// loads issued together (codes(r) is peer r's code buffer, scale(r) its scale for this block), and the sums are
// written back tensor by tensor.  [t_lo, t_hi] as in the quantiser's careful path.
template <typename Codes, typename Scale>
__device__ __forceinline__ void dequant_bucket_block_careful(const BucketArgs& a, uint32_t t_lo, uint32_t t_hi, uint64_t begin,
                                                             uint64_t end, int lane, uint32_t n, Codes&& codes, Scale&& scale) {
    // in two halves of 512 elements, which keeps the registers of this rare path under those of the common one
    constexpr int H = kCarefulSlots / 2;
    const uint32_t count = (uint32_t)(end - begin);
#pragma unroll 1
    for (uint32_t first = 0; first < count; first += H * 64) {
        float x[H];
#pragma unroll
        for (int j = 0; j < H; ++j) x[j] = 0.0f;
        for (uint32_t t = t_lo; t <= t_hi; ++t) {
            const uint64_t off = a.offsets[t], next = a.offsets[t + 1];
            const uint64_t seg_b = begin > off ? begin : off, seg_e = end < next ? end : next;
            if (seg_b >= seg_e) continue;  // an empty tensor, or one past the block
            // the segment is elements [lo, hi) of the block, read from p; no load is predicated
            const float* __restrict__ p = reinterpret_cast<const float*>(a.tensors[t]) + (begin - off);
            const uint32_t lo = (uint32_t)(seg_b - begin), hi = (uint32_t)(seg_e - begin);
            float v[H];
#pragma unroll
            for (int j = 0; j < H; ++j) {
                const uint32_t i = first + j * 64 + lane;
                v[j] = p[i < lo ? lo : i >= hi ? hi - 1 : i];
            }
#pragma unroll
            for (int j = 0; j < H; ++j) {
                const uint32_t i = first + j * 64 + lane;
                if (i >= lo && i < hi) x[j] = v[j];
            }
        }
        for (uint32_t r = 0; r < n; ++r) {
            const uint8_t* __restrict__ q = codes(r) + begin;
            const float s = scale(r);
            uint8_t c[H];
#pragma unroll
            for (int j = 0; j < H; ++j) {
                const uint32_t i = first + j * 64 + lane;
                c[j] = q[i < count ? i : count - 1];
            }
#pragma unroll
            for (int j = 0; j < H; ++j) {
                const auto v = __builtin_amdgcn_cvt_pk_f32_fp8((int)c[j], false);
                x[j] = x[j] + v[0] * s;  // product rounded, then added
            }
        }
        for (uint32_t t = t_lo; t <= t_hi; ++t) {
            const uint64_t off = a.offsets[t], next = a.offsets[t + 1];
            const uint64_t seg_b = begin > off ? begin : off, seg_e = end < next ? end : next;
            if (seg_b >= seg_e) continue;
            float* __restrict__ p = reinterpret_cast<float*>(a.tensors[t]) + (begin - off);
            const uint32_t lo = (uint32_t)(seg_b - begin), hi = (uint32_t)(seg_e - begin);
#pragma unroll
            for (int j = 0; j < H; ++j) {
                const uint32_t i = first + j * 64 + lane;
                if (i >= lo && i < hi) p[i] = x[j];
            }
        }
    }
}

// Accumulator elements of a full block that one tensor boundary cuts (every block that straddles tensors of 1024
// elements and more): element i of the block is head[i] for i < cut and rest[i] from there on.  Step j of a lane is
// elements j * 256 + lane * 4 .. + 3: a 128-bit access to one of the two tensors, except in the step that holds the
// vector the cut goes through, which every lane moves element by element (a wave-uniform choice, no lane branches).
// All loads of the block are then in flight together as in a block inside one tensor; through the careful path
// above such a block takes several round trips, which shows in buckets of a few million elements.
struct CutBlock {
    float* head;
    float* rest;
    uint32_t cut;  // 0 < cut < kBlock
    __device__ __forceinline__ CutBlock(const BucketArgs& a, uint32_t t, uint64_t begin) {
        cut = (uint32_t)(a.offsets[t + 1] - begin);
        head = reinterpret_cast<float*>(a.tensors[t]) + (begin - a.offsets[t]);
        rest = reinterpret_cast<float*>(reinterpret_cast<uintptr_t>(a.tensors[t + 1]) - (uintptr_t)cut * 4);
    }
    __device__ __forceinline__ bool by_elements(int j) const { return cut % 4 != 0 && cut / 256 == (uint32_t)j; }
    __device__ __forceinline__ float* at(uint32_t i) const { return (i < cut ? head : rest) + i; }
    __device__ __forceinline__ uint4 load(int j, int lane) const {
        const uint32_t v0 = j * 256 + lane * 4;
        if (by_elements(j))
            return make_uint4(__float_as_uint(*at(v0)), __float_as_uint(*at(v0 + 1)), __float_as_uint(*at(v0 + 2)),
                              __float_as_uint(*at(v0 + 3)));
        return load16_unaligned(at(v0));
    }
    __device__ __forceinline__ void store(int j, int lane, const uint4& r) const {
        const uint32_t v0 = j * 256 + lane * 4;
        if (by_elements(j)) {
            *at(v0) = __uint_as_float(r.x);
            *at(v0 + 1) = __uint_as_float(r.y);
            *at(v0 + 2) = __uint_as_float(r.z);
            *at(v0 + 3) = __uint_as_float(r.w);
        } else {
            store16_unaligned(at(v0), r);
        }
    }
};

// whether the full block [begin, begin + kBlock), whose first element tensor t holds, ends in tensor t + 1
__device__ __forceinline__ bool block_cut_once(const BucketArgs& a, uint32_t t, uint64_t begin) {
    return t + 2 <= a.ntensors && a.offsets[t + 1] < begin + kBlock && a.offsets[t + 2] >= begin + kBlock;
}

// One block of one peer: codes at q + begin, accumulator vectors through load(j) / store(j, r), 4 steps of 256
// elements, all loads first.
template <typename Load, typename Store>
__device__ __forceinline__ void dequant_accumulate_block(const uint8_t* __restrict__ q, float s, uint64_t begin, int lane, Load&& load,
                                                         Store&& store) {
    uint32_t codes[4];
    uint4 acc[4];
#pragma unroll
    for (int j = 0; j < 4; ++j) {
        codes[j] = load4_unaligned(q + begin + j * 256 + lane * 4);
        acc[j] = load(j);
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
        store(j, r);
    }
}

// out_t[j] += float(q[off_t + j]) * scale[(off_t + j) / 1024], accumulators are the bucket's
// own fp32 tensors.  One wavefront per 1024-element block, 4 lanes-groups of 4 elements each.
__global__ __launch_bounds__(kBucketThreads) __attribute__((amdgpu_waves_per_eu(7))) void fp8_dequant_accumulate_bucket_kernel(const uint8_t* __restrict__ q,
                                                                                 const float* __restrict__ scales,
                                                                                 BucketArgs a) {
    const int lane = threadIdx.x & 63;
    const uint64_t wave = (uint64_t)blockIdx.x * (kBucketThreads / 64) + (uint32_t)__builtin_amdgcn_readfirstlane((int)(threadIdx.x >> 6));  // see fp8_quantize_bucket_kernel
    const uint64_t nwaves = (uint64_t)gridDim.x * (kBucketThreads / 64);
    for (uint64_t b = wave; b < a.nblocks; b += nwaves) {
        const uint64_t begin = b * kBlock;
        const uint64_t end = begin + kBlock < a.total ? begin + kBlock : a.total;
        uint32_t t_lo, t_hi;
        span_tensors(a, begin, end, &t_lo, &t_hi);
        const float s = scales[b];
        if (t_lo == t_hi && end - begin == kBlock) {
            // the whole block lies in one tensor
            float* dst = reinterpret_cast<float*>(a.tensors[t_lo]) + (begin - a.offsets[t_lo]);
            dequant_accumulate_block(q, s, begin, lane, [&](int j) { return load16_unaligned(dst + j * 256 + lane * 4); },
                                     [&](int j, const uint4& r) { store16_unaligned(dst + j * 256 + lane * 4, r); });
            continue;
        }
        if (end - begin == kBlock && block_cut_once(a, t_lo, begin)) {
            const CutBlock c(a, t_lo, begin);
            dequant_accumulate_block(q, s, begin, lane, [&](int j) { return c.load(j, lane); },
                                     [&](int j, const uint4& r) { c.store(j, lane, r); });
            continue;
        }
        // more than two tensors, or the short last block
        dequant_bucket_block_careful(a, t_lo, t_hi, begin, end, lane, 1, [&](uint32_t) { return q; }, [&](uint32_t) { return s; });
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

// One full block of all peers: accumulator vectors through load(j) / store(j, r), peers four at a time with all
// their codes loaded before the first add.
template <typename Load, typename Store>
__device__ __forceinline__ void dequant_accumulate_block_peers(const BucketPeersArgs& p, uint64_t b, int lane, Load&& load, Store&& store) {
    const uint64_t begin = b * kBlock;
    float v[4][4];
#pragma unroll
    for (int j = 0; j < 4; ++j) {
        const uint4 r = load(j);
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
        store(j, make_uint4(__float_as_uint(v[j][0]), __float_as_uint(v[j][1]), __float_as_uint(v[j][2]), __float_as_uint(v[j][3])));
}

__global__ __launch_bounds__(kBucketThreads) __attribute__((amdgpu_waves_per_eu(7))) void fp8_dequant_accumulate_bucket_many_kernel(BucketPeersArgs p) {
    const BucketArgs& a = p.b;
    const int lane = threadIdx.x & 63;
    const uint64_t wave = (uint64_t)blockIdx.x * (kBucketThreads / 64) + (uint32_t)__builtin_amdgcn_readfirstlane((int)(threadIdx.x >> 6));  // see fp8_quantize_bucket_kernel
    const uint64_t nwaves = (uint64_t)gridDim.x * (kBucketThreads / 64);
    for (uint64_t b = wave; b < a.nblocks; b += nwaves) {
        const uint64_t begin = b * kBlock;
        const uint64_t end = begin + kBlock < a.total ? begin + kBlock : a.total;
        uint32_t t_lo, t_hi;
        span_tensors(a, begin, end, &t_lo, &t_hi);
        if (t_lo == t_hi && end - begin == kBlock) {
            float* dst = reinterpret_cast<float*>(a.tensors[t_lo]) + (begin - a.offsets[t_lo]);
            dequant_accumulate_block_peers(p, b, lane, [&](int j) { return load16_unaligned(dst + j * 256 + lane * 4); },
                                           [&](int j, const uint4& r) { store16_unaligned(dst + j * 256 + lane * 4, r); });
            continue;
        }
        if (end - begin == kBlock && block_cut_once(a, t_lo, begin)) {
            const CutBlock c(a, t_lo, begin);
            dequant_accumulate_block_peers(p, b, lane, [&](int j) { return c.load(j, lane); },
                                           [&](int j, const uint4& r) { c.store(j, lane, r); });
            continue;
        }
        // more than two tensors, or the short last block
        dequant_bucket_block_careful(a, t_lo, t_hi, begin, end, lane, p.n, [&](uint32_t r) { return p.q[r]; },
                                     [&](uint32_t r) { return p.scales[r][b]; });
    }
}

// shared by the entry points that quantise a bucket: `index` is a device pointer or null
static int quantize_bucket(uint8_t* q, float* scales, const void* const* d_tensors, const uint64_t* d_offsets,
                           uint32_t ntensors, uint64_t total, const uint32_t* index, hipStream_t hs) {
    BucketArgs a{};
    a.tensors = reinterpret_cast<char* const*>(const_cast<void* const*>(reinterpret_cast<const void* const*>(d_tensors)));
    a.offsets = d_offsets;
    a.index = index;
    a.total = total;
    a.nblocks = (total + kBlock - 1) / kBlock;
    a.ntensors = ntensors;
    // Buckets of up to kSmallBucketBlocks blocks run one block per wavefront step: a launch of a few MB is bound by how long its
    // wavefronts live (three dependent table reads, then the data), not by bandwidth, and four times as many wavefronts hide
    // that better; large buckets amortise the look-ups over four blocks.  One / four blocks per step, both in turn on one GPU:
    // 4.5 M elements 6.0 / 7.9 us (the flat quantiser alone: 5.1), 14 M 10.6 / 12.3 (8.6), 34 M 21.5 / 21.7, 68 M 38.8 / 36.8,
    // 134 M 73.3 / 66.0, 756 M 0.68 / 0.78 of peak.  With the tuning aids on, MONARCH_HIP_BUCKET_BLOCKS=1 / 4 overrides the
    // choice at every call (the parity tests run both forms on the same buckets).
    int nb = a.nblocks <= kSmallBucketBlocks ? 1 : kBucketBlocks;
    if (const char* e = tuning_env("MONARCH_HIP_BUCKET_BLOCKS")) nb = std::atoi(e) == 1 ? 1 : kBucketBlocks;
    const uint64_t per_wg = (uint64_t)(kBucketThreads / 64) * nb;
    const uint64_t wgs = (a.nblocks + per_wg - 1) / per_wg;
    const uint64_t cap = max_workgroups(kBucketThreads);
    const dim3 grid((uint32_t)(wgs > cap ? cap : wgs));
    if (nb == 1) MHIP_LAUNCH(fp8_quantize_bucket_kernel<1>, grid, dim3(kBucketThreads), 0, hs, q, scales, a);
    else MHIP_LAUNCH(fp8_quantize_bucket_kernel<kBucketBlocks>, grid, dim3(kBucketThreads), 0, hs, q, scales, a);
    return launch_status();
}

static int build_bucket_index(uint32_t* index, const uint64_t* d_offsets, uint32_t ntensors, uint64_t total, hipStream_t hs) {
    const uint64_t nblocks = (total + kBlock - 1) / kBlock;
    const uint64_t wgs = (nblocks + 1 + kThreads - 1) / kThreads;
    const uint64_t cap = max_workgroups(kThreads);
    MHIP_LAUNCH(bucket_index_kernel, dim3((uint32_t)(wgs > cap ? cap : wgs)), dim3(kThreads), 0, hs, index, d_offsets, ntensors,
                nblocks);
    return launch_status();
}

static int check_quantize_bucket_args(const void* q, const float* scales, const void* d_tensors, const void* d_offsets,
                                      uint32_t block) {
    if (block != kBlock) return MHIP_ERR_UNSUPPORTED_BLOCK;
    if (!q || !scales || !d_tensors || !d_offsets) return MHIP_ERR_UNDEFINED_TENSOR;
    if ((uintptr_t)scales & 3u) return MHIP_ERR_INVALID_ARGUMENT;
    return MHIP_SUCCESS;
}

// ---- block index kept by the library, for callers that cannot allocate the workspace ----
// mhip_fp8_quantize_bucket_static builds the bucket's block index into this array instead of into caller memory.
// Every GPU the library runs on holds its own copy (4 MiB) until the process ends.  In host code the array's name
// is only a handle for hipGetSymbolAddress: the device address is looked up once per device, with that device
// current, and kernels are given that address.
constexpr uint64_t kStaticIndexEntries = 1ull << 20;  // blocks of 1024 elements, plus the closing entry
static __device__ __align__(256) uint32_t scratch[kStaticIndexEntries];

constexpr int kMaxDevices = 64;
static std::mutex g_scratch_mutex;
static uint32_t* g_scratch_ptr[kMaxDevices];  // device address of `scratch` on each device, null until looked up

// Address of the current device's copy of `scratch`; the caller has made the launch device current.  The look-up
// happens once per device: from mhip_set_device / mhip_stream_create (the set-up calls of a process that uses this
// library), or else from the first call of the entry point on that device.  `capturing`: the look-up is not a stream
// operation and loads the device's code object the first time, so it must not fall inside a stream capture; a first
// call under capture is refused instead.
static int static_index_for_current_device(uint32_t** out, bool capturing) {
    int dev = -1;
    if (hipError_t e = hipGetDevice(&dev); e != hipSuccess) return (int)e;
    if (dev < 0 || dev >= kMaxDevices) return MHIP_ERR_INVALID_DEVICE;
    std::lock_guard<std::mutex> lock(g_scratch_mutex);
    if (g_scratch_ptr[dev] == nullptr) {
        if (capturing) return (int)hipErrorStreamCaptureUnsupported;
        uint32_t* ptr = nullptr;
        if (hipError_t e = hipGetSymbolAddress(reinterpret_cast<void**>(&ptr), HIP_SYMBOL(scratch)); e != hipSuccess) return (int)e;
        if (ptr == nullptr) return MHIP_ERR_INVALID_DEVICE;
        g_scratch_ptr[dev] = ptr;
    }
    if (out) *out = g_scratch_ptr[dev];
    return MHIP_SUCCESS;
}

int prepare_static_scratch() { return static_index_for_current_device(nullptr, false); }

}  // namespace mhip

using namespace mhip;

extern "C" {

int mhip_bucket_index_bytes(uint64_t total, uint32_t block, size_t* bytes) {
    if (!bytes) return MHIP_ERR_INVALID_ARGUMENT;
    if (block != kBlock) return MHIP_ERR_UNSUPPORTED_BLOCK;
    if (total > (1ull << 62)) return MHIP_ERR_INVALID_ARGUMENT;
    *bytes = (size_t)(((total + kBlock - 1) / kBlock + 1) * sizeof(uint32_t));
    return MHIP_SUCCESS;
}

int mhip_bucket_index_build(uint32_t* d_index, const uint64_t* d_offsets, uint32_t ntensors, uint64_t total, uint32_t block,
                            mhip_stream_t stream) {
    if (block != kBlock) return MHIP_ERR_UNSUPPORTED_BLOCK;
    if (ntensors == 0) return MHIP_ERR_INVALID_ARGUMENT;
    if (!d_index || !d_offsets) return MHIP_ERR_UNDEFINED_TENSOR;
    if ((uintptr_t)d_index & 3u) return MHIP_ERR_INVALID_ARGUMENT;
    hipStream_t hs = static_cast<hipStream_t>(stream);
    DeviceGuard guard(hs);
    return build_bucket_index(d_index, d_offsets, ntensors, total, hs);
}

int mhip_fp8_quantize_bucket(uint8_t* q, float* scales, const void* const* d_tensors, const uint64_t* d_offsets,
                             uint32_t ntensors, uint64_t total, uint32_t block, const uint32_t* d_index, mhip_stream_t stream) {
    if (block != kBlock) return MHIP_ERR_UNSUPPORTED_BLOCK;
    if (ntensors == 0 || total == 0) return MHIP_SUCCESS;
    if (int rc = check_quantize_bucket_args(q, scales, d_tensors, d_offsets, block)) return rc;
    if ((uintptr_t)d_index & 3u) return MHIP_ERR_INVALID_ARGUMENT;
    hipStream_t hs = static_cast<hipStream_t>(stream);
    DeviceGuard guard(hs);
    return quantize_bucket(q, scales, d_tensors, d_offsets, ntensors, total, d_index, hs);
}

int mhip_fp8_quantize_bucket_static(uint8_t* q, float* scales, const void* const* d_tensors, const uint64_t* d_offsets,
                                    uint32_t ntensors, uint64_t total, uint32_t block, mhip_stream_t stream) {
    if (block != kBlock) return MHIP_ERR_UNSUPPORTED_BLOCK;
    // the index needs ceil(total / 1024) + 1 entries
    if (total > (kStaticIndexEntries - 1) * kBlock) return MHIP_ERR_SCRATCH_TOO_SMALL;
    if (ntensors == 0 || total == 0) return MHIP_SUCCESS;
    if (int rc = check_quantize_bucket_args(q, scales, d_tensors, d_offsets, block)) return rc;
    hipStream_t hs = static_cast<hipStream_t>(stream);
    DeviceGuard guard(hs);
    uint32_t* index = nullptr;
    hipStreamCaptureStatus capture = hipStreamCaptureStatusNone;
    if (hs != nullptr && hipStreamIsCapturing(hs, &capture) != hipSuccess) capture = hipStreamCaptureStatusNone;
    if (int rc = static_index_for_current_device(&index, capture != hipStreamCaptureStatusNone)) return rc;
    // every entry the quantiser reads is rewritten by this build, so nothing of an earlier call has to be cleared
    if (int rc = build_bucket_index(index, d_offsets, ntensors, total, hs)) return rc;
    return quantize_bucket(q, scales, d_tensors, d_offsets, ntensors, total, index, hs);
}

int mhip_fp8_dequant_accumulate_bucket(void* const* d_acc_tensors, const uint8_t* q, const float* scales,
                                       const uint64_t* d_offsets, uint32_t ntensors, uint64_t total, uint32_t block,
                                       const uint32_t* d_index, mhip_stream_t stream) {
    if (block != kBlock) return MHIP_ERR_UNSUPPORTED_BLOCK;
    if (ntensors == 0 || total == 0) return MHIP_SUCCESS;
    if (!q || !scales || !d_acc_tensors || !d_offsets) return MHIP_ERR_UNDEFINED_TENSOR;
    if ((uintptr_t)scales & 3u) return MHIP_ERR_INVALID_ARGUMENT;
    BucketArgs a{};
    if ((uintptr_t)d_index & 3u) return MHIP_ERR_INVALID_ARGUMENT;
    a.tensors = reinterpret_cast<char* const*>(d_acc_tensors);
    a.offsets = d_offsets;
    a.index = d_index;
    a.total = total;
    a.nblocks = (total + kBlock - 1) / kBlock;
    a.ntensors = ntensors;
    const uint64_t wgs = (a.nblocks + 3) / 4;
    const uint64_t cap = max_workgroups(kBucketThreads);
    hipStream_t hs = static_cast<hipStream_t>(stream);
    DeviceGuard guard(hs);
    MHIP_LAUNCH(fp8_dequant_accumulate_bucket_kernel, dim3((uint32_t)(wgs > cap ? cap : wgs)), dim3(kBucketThreads), 0,
                       hs, q, scales, a);
    return launch_status();
}

int mhip_fp8_dequant_accumulate_bucket_many(void* const* d_acc_tensors, const uint8_t* const* q,
                                            const float* const* scales, uint32_t n, const uint64_t* d_offsets,
                                            uint32_t ntensors, uint64_t total, uint32_t block, const uint32_t* d_index,
                                            mhip_stream_t stream) {
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
    if ((uintptr_t)d_index & 3u) return MHIP_ERR_INVALID_ARGUMENT;
    p.b.tensors = reinterpret_cast<char* const*>(d_acc_tensors);
    p.b.offsets = d_offsets;
    p.b.index = d_index;
    p.b.total = total;
    p.b.nblocks = (total + kBlock - 1) / kBlock;
    p.b.ntensors = ntensors;
    const uint64_t wgs = (p.b.nblocks + 3) / 4;
    const uint64_t cap = max_workgroups(kBucketThreads);
    hipStream_t hs = static_cast<hipStream_t>(stream);
    DeviceGuard guard(hs);
    MHIP_LAUNCH(fp8_dequant_accumulate_bucket_many_kernel, dim3((uint32_t)(wgs > cap ? cap : wgs)), dim3(kBucketThreads),
                       0, hs, p);
    return launch_status();
}

}  // extern "C"
