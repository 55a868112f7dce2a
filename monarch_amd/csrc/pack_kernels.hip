// Slice pack/unpack and flat-bucket pack/unpack kernels for gfx950.
//
// Every copy is HBM-bound byte movement.  The packed (staging) side is contiguous, so
// work is cut into 16-byte chunks aligned on the packed address, consecutive lanes take
// consecutive chunks, and each wavefront instruction touches 1 KiB of contiguous staging
// memory.  What happens on the strided side depends on the view's contiguous runs:
//   slice_copy_kernel         rows are whole chunks: one 128-bit access per chunk and side
//   slice_copy_ragged_kernel  rows of at least a chunk that are not whole chunks: a chunk
//                             straddling a row boundary moves as two overlapping vectors
//   slice_unpack_lines_kernel unpacks of such rows from 256 bytes on: whole cache lines of the written side
//   slice_gather_kernel       runs shorter than (a few) chunks: the chunk's units are
//                             gathered / scattered one by one
//   contiguous_copy_kernel    one run of any alignment: rows on the destination's 1 KiB boundaries
// (views whose memory-contiguous dimension is not the innermost one go to the LDS-tiled
// transposing kernels instead).  The host picks the form per launch from the canonical slice.
#include "mhip_device.h"
#include "fp8_common.h"
#include "pack_internal.h"

namespace mhip {

constexpr int kMaxViews = 16;
// Lanes per workgroup of the slice copy kernels: single wavefronts stream best (column-block pack 0.767 -> 0.775 of
// peak, unpack 0.757 -> 0.792 against 256 lanes; ragged and short-run forms equal or better).
constexpr int kPackThreads = 64;
// Chunks per lane of slice_copy_kernel, all loads issued before the first store.  Large copies stream
// fastest with one chunk per lane and many workgroups (8 column blocks of 14 MiB: 0.76 of peak against
// 0.73 with eight chunks); copies of a few MiB finish sooner with fewer, fatter workgroups.
constexpr int kUnrollSmall = 4, kUnrollLarge = 1;
constexpr uint64_t kLargeCopyChunks = 1ull << 19;  // 8 MiB

struct PackArgs {
    char* base;                  // strided tensor
    char* packed[kMaxViews];     // staging buffers, one per view
    uint64_t offset[kMaxViews];  // view offsets, units
    uint64_t total;              // units per view
    uint64_t nchunks;            // 16-byte chunks per view, including a ragged first one
    uint32_t shift;              // units missing from chunk 0 so that chunk c starts 16-byte aligned
    uint32_t nviews;             // views handled by this launch
    uint64_t wg0;                // workgroups of this copy launched before this grid
    uint32_t pieces;             // slice_unpack_lines_kernel: cache lines a row can overlap
    FastDiv32 pieces_div;        //   division by it, valid in 32-bit mode
    uint64_t nrows;              //   rows per view
    uint64_t per_xcd;            // copies whose pieces share cache lines: workgroups in each XCD's contiguous
    uint64_t nwg;                //   share of the nwg workgroups (0: workgroup i takes tile i)
    uint32_t stream_stores;      // slice_copy_kernel unpacking 16-byte units, slice_unpack_lines_kernel: non-temporal
                                 //   instead of write-through stores
    DimsArg dims;
};

template <int U, bool PACK>
__device__ __forceinline__ void move_unit(char* strided, char* packed) {
    using T = typename UnitType<U>::type;
    using M = typename UnitType<U>::mem;  // the strided side may be less aligned than the unit
    if constexpr (PACK)
        *reinterpret_cast<T*>(packed) = *reinterpret_cast<const M*>(strided);
    else
        *reinterpret_cast<M*>(strided) = *reinterpret_cast<const T*>(packed);
}

// One chunk moved unit by unit, with every unit tested against the view's extent: the ragged first
// and last chunk of a view, and chunks that no vector form applies to.
template <int U, bool PACK, bool WIDE, int NDIM>
__device__ __forceinline__ void move_chunk_by_units(const PackArgs& a, char* strided, char* packed, uint64_t chunk) {
    constexpr int VU = 16 / U;
    const uint64_t tb = chunk * VU;
    for (int j = 0; j < VU; ++j) {
        const uint64_t t = tb + j - a.shift;
        if (tb + j >= a.shift && t < a.total) {
            uint64_t col;
            const uint64_t l = decode<WIDE, NDIM>(a.dims, t, &col);
            move_unit<U, PACK>(strided + l * U, packed + t * U);
        }
    }
}

template <int U, bool PACK, bool WIDE, int NDIM, int kUnroll>
__global__ __launch_bounds__(kPackThreads) void slice_copy_kernel(PackArgs a) {
    constexpr int VU = 16 / U;  // units per chunk
    // The view index is the fastest-varying part of the workgroup id, so that workgroups
    // running side by side work on the same rows of neighbouring views (for column blocks
    // of one tensor: neighbouring segments of the same rows).
    uint64_t wg = a.wg0 + blockIdx.x;
    if (a.per_xcd != 0) {  // each XCD on a contiguous share: see the note above copy_views
        wg = (wg & 7) * a.per_xcd + (wg >> 3);
        if (wg >= a.nwg) return;
    }
    const uint64_t tile = wg / a.nviews;
    const uint32_t v = (uint32_t)(wg % a.nviews);
    char* __restrict__ packed = a.packed[v];
    char* __restrict__ strided = a.base + a.offset[v] * U;
    const uint64_t c0 = tile * (kPackThreads * kUnroll) + threadIdx.x;

    if constexpr (NDIM == 0) {
        // Contiguous view: when the whole tile of this workgroup lies inside the
        // buffer (decided on the scalar unit), no per-chunk tests are needed at all.
        const uint64_t tile_first = tile * (kPackThreads * kUnroll) * VU;
        const uint64_t tile_end = tile_first + (uint64_t)(kPackThreads * kUnroll) * VU;
        if (tile_first >= a.shift && tile_end - a.shift <= a.total) {
            char* __restrict__ p = packed + (c0 * VU - a.shift) * U;
            char* __restrict__ s = strided + (c0 * VU - a.shift) * U;
            uint4 d[kUnroll];
#pragma unroll
            for (int i = 0; i < kUnroll; ++i) {
                if constexpr (PACK) d[i] = load16_unaligned(s + (size_t)i * kPackThreads * 16);
                else d[i] = load16_aligned(p + (size_t)i * kPackThreads * 16);
            }
#pragma unroll
            for (int i = 0; i < kUnroll; ++i) {
                if constexpr (PACK) store16_writethrough(p + (size_t)i * kPackThreads * 16, d[i]);
                else store16_unaligned(s + (size_t)i * kPackThreads * 16, d[i]);
            }
            return;
        }
    }

    uint64_t loc[kUnroll];
    uint64_t first[kUnroll];  // first packed unit of the chunk (may be "negative": see below)
    bool vec[kUnroll];
    bool live[kUnroll];
#pragma unroll
    for (int i = 0; i < kUnroll; ++i) {
        const uint64_t c = c0 + (uint64_t)i * kPackThreads;
        live[i] = c < a.nchunks;
        const uint64_t tb = c * VU;  // position counted from the aligned-down start
        vec[i] = false;
        first[i] = tb - a.shift;     // wraps for a ragged chunk 0; only used when tb >= shift
        if (live[i] && tb >= a.shift && first[i] + VU <= a.total) {
            uint64_t col;
            loc[i] = decode<WIDE, NDIM>(a.dims, first[i], &col);
            vec[i] = col + VU <= a.dims.run;
        }
    }
    bool all_vec = true;
#pragma unroll
    for (int i = 0; i < kUnroll; ++i) all_vec = all_vec && vec[i];
    uint4 data[kUnroll];
    if (all_vec) {
        // The common case, free of per-chunk predicates: all loads in flight, then all stores.  Stores to
        // 16-byte aligned addresses go out write-through (column blocks of 3584-byte runs: pack 0.77 -> 0.79 of
        // peak; 128-byte runs of a [B,H,S,D] -> [B,S,H,D] permute: 0.69 -> 0.77); unaligned ones do not
        // (a row pitch that is only 2-byte aligned: unpack 0.74 -> 0.71), nor do the gathering form, the
        // flat bucket pack and the fp8 accumulate, which all lose 1-2 points with it.
#pragma unroll
        for (int i = 0; i < kUnroll; ++i) {
            if constexpr (PACK)
                data[i] = load16_unaligned(strided + loc[i] * U);
            else
                data[i] = load16_aligned(packed + first[i] * U);
        }
#pragma unroll
        for (int i = 0; i < kUnroll; ++i) {
            if constexpr (PACK)
                store16_writethrough(packed + first[i] * U, data[i]);
            else if constexpr (U == 16) {
                if (a.stream_stores) store16_unaligned(strided + loc[i] * U, data[i]);  // wave-uniform
                else store16_writethrough(strided + loc[i] * U, data[i]);
            } else
                store16_unaligned(strided + loc[i] * U, data[i]);
        }
        return;
    }
#pragma unroll
    for (int i = 0; i < kUnroll; ++i) {
        if (vec[i]) {
            if constexpr (PACK)
                data[i] = load16_unaligned(strided + loc[i] * U);
            else
                data[i] = load16_aligned(packed + first[i] * U);
        }
    }
#pragma unroll
    for (int i = 0; i < kUnroll; ++i) {
        if (vec[i]) {
            if constexpr (PACK)
                store16_aligned(packed + first[i] * U, data[i]);
            else
                store16_unaligned(strided + loc[i] * U, data[i]);
        }
    }
    if constexpr (VU > 1) {
#pragma unroll
        for (int i = 0; i < kUnroll; ++i) {
            if (live[i] && !vec[i]) move_chunk_by_units<U, PACK, WIDE, NDIM>(a, strided, packed, c0 + (uint64_t)i * kPackThreads);
        }
    }
}

// The same copy for views whose rows are not whole chunks (row length not a multiple of 16
// bytes, or a staging address that is not 16-byte aligned): then about one chunk per row
// straddles a row boundary, and with several rows per wavefront step nearly every wavefront would
// fall off the predicate-free path above.  A straddling chunk is moved as two whole
// 16-byte vectors instead, each inside one row on both sides: "A" ends where the row ends,
// "B" starts where the next row starts.  They overlap the neighbouring chunks, which write
// the same bytes there.  Every lane issues its loads without per-lane predicates, so they stay
// in flight together; only the stores are predicated.  Lanes with nothing to load read the 16-byte
// aligned vector that holds the first byte of the side that is read: one address for the whole
// wavefront, and an ALIGNED one - a wavefront whose lanes all read the same vector at an address
// that is not 4-byte aligned (a bf16 view that starts at an odd column) takes far longer over it
// than over 64 consecutive ones.  The "B" loads are skipped by wavefronts without a straddling
// chunk (decided for the whole wavefront): bf16 rows of 7166 starting at column 1 0.57 -> 0.72 of
// peak, rows of 3580 0.54 -> 0.68, rows of 1790 0.50 -> 0.60; views on 4-byte boundaries unchanged.
// Needs rows of at least one chunk; the ragged first and last chunk of a view still go unit by unit.
constexpr int kRaggedUnroll = 1;  // measured: 1 chunk per lane 0.75, 2 0.73, 4 0.72, 8 0.72 of peak (fp32 rows of 1791)

template <int U, bool PACK, bool WIDE, int NDIM>
__global__ __launch_bounds__(kPackThreads) void slice_copy_ragged_kernel(PackArgs a) {
    constexpr int VU = 16 / U;
    constexpr int UN = kRaggedUnroll;
    uint64_t wg = a.wg0 + blockIdx.x;
    if (a.per_xcd != 0) {  // each XCD on a contiguous share: see the note above copy_views
        wg = (wg & 7) * a.per_xcd + (wg >> 3);
        if (wg >= a.nwg) return;
    }
    const uint64_t tile = wg / a.nviews;
    const uint32_t v = (uint32_t)(wg % a.nviews);
    char* __restrict__ packed = a.packed[v];
    char* __restrict__ strided = a.base + a.offset[v] * U;
    const uint64_t c0 = tile * (kPackThreads * UN) + threadIdx.x;
    // what idle lanes load: the aligned vector that holds the first byte of the side that is read
    const char* const idle = reinterpret_cast<const char*>((uintptr_t)(PACK ? strided : packed) & ~(uintptr_t)15);
    uint64_t pa[UN], sa[UN], pb[UN], sb[UN];  // packed / strided unit index of vector A and vector B
    bool do_a[UN], do_b[UN], edge[UN];
    bool any_b = false;
#pragma unroll
    for (int i = 0; i < UN; ++i) {
        const uint64_t c = c0 + (uint64_t)i * kPackThreads;
        const uint64_t tb = c * VU;
        const uint64_t first = tb - a.shift;
        pa[i] = sa[i] = pb[i] = sb[i] = 0;
        do_a[i] = do_b[i] = edge[i] = false;
        if (c < a.nchunks) {
            if (tb >= a.shift && first + VU <= a.total) {
                uint64_t col;
                const uint64_t loc = decode<WIDE, NDIM>(a.dims, first, &col);
                const uint64_t rem = a.dims.run - col;  // units of this row from `first` on
                do_a[i] = true;
                if (rem >= VU) {
                    pa[i] = first;
                    sa[i] = loc;
                } else {
                    pa[i] = first + rem - VU;
                    sa[i] = loc + rem - VU;
                    pb[i] = first + rem;
                    sb[i] = decode<WIDE, NDIM>(a.dims, first + rem, &col);
                    do_b[i] = any_b = true;
                }
            } else {
                edge[i] = true;
            }
        }
    }
    uint4 da[UN], db[UN] = {};
#pragma unroll
    for (int i = 0; i < UN; ++i) {
        const char* from = PACK ? strided + sa[i] * U : packed + pa[i] * U;
        da[i] = load16_unaligned(do_a[i] ? from : idle);
    }
    if (__builtin_amdgcn_ballot_w64(any_b) != 0) {  // one branch for the whole wavefront
#pragma unroll
        for (int i = 0; i < UN; ++i) {
            const char* from = PACK ? strided + sb[i] * U : packed + pb[i] * U;
            db[i] = load16_unaligned(do_b[i] ? from : idle);
        }
    }
#pragma unroll
    for (int i = 0; i < UN; ++i) {
        if (do_a[i]) {
            if constexpr (PACK) store16_unaligned(packed + pa[i] * U, da[i]);
            else store16_unaligned(strided + sa[i] * U, da[i]);
        }
    }
#pragma unroll
    for (int i = 0; i < UN; ++i) {
        if (do_b[i]) {
            if constexpr (PACK) store16_unaligned(packed + pb[i] * U, db[i]);
            else store16_unaligned(strided + sb[i] * U, db[i]);
        }
    }
#pragma unroll
    for (int i = 0; i < UN; ++i) {
        if (edge[i]) move_chunk_by_units<U, PACK, WIDE, NDIM>(a, strided, packed, c0 + (uint64_t)i * kPackThreads);
    }
}

// Unpacking rows that are not whole 16-byte chunks, laid out on the CACHE LINES of the side that is written.  The
// two-vector form above cuts the work on the packed side's 16-byte grid, so on the strided side every 1 KiB a
// wavefront writes starts and ends inside a cache line that the neighbouring wavefronts (on other XCDs) write as well,
// and such a line goes to HBM as two partial writes.  Here a row of R bytes overlaps at most `pieces` lines, and eight
// consecutive lanes take the eight 16-byte vectors of one line of one row: a wavefront writes eight whole lines, and no
// line is written by two wavefronts, whatever the rows' length and alignment.  Vectors inside the row are aligned on
// the written side (unaligned loads from the packed image, whose lines are only read); a vector that the row's start
// or end cuts is replaced by the row's first or last 16 bytes, an unaligned vector that overlaps its neighbour with the
// same bytes; lanes past the row's last line idle (they load the row's last vector and store nothing), so no load is
// predicated.  Against the two-vector form, [16384 rows at a 28 KiB pitch]: bf16 rows of 894 0.36 -> 0.43 of peak, of
// 1790 0.58 -> 0.62, of 3580 0.66 -> 0.70; u8 rows of 3581 0.51 -> 0.60, of 14333 0.645 -> 0.75; fp32 rows of 447
// 0.36 -> 0.42, of 1791 0.67 -> 0.71.  (A form with one 1 KiB-aligned piece of one row per wavefront, which this one
// replaces, gave 0.59 / 0.66 on bf16 rows of 1790 / 3580 and lost on rows around 1 KiB, whose pieces are half empty.)
// Launches that write less than 96 MiB store write-through, cut vectors included, as the whole-chunk form does at those
// sizes (u8 rows of 1788 0.41-0.44 -> 0.54-0.58, of 3580 0.59-0.63 -> 0.66-0.80, 82 MB 0.64 -> 0.76; eight bf16 column
// blocks of 1790 in one launch, 59 MB together, 0.70 -> 0.76); larger ones stream (117 MB in eight views 0.72 against
// 0.70 write-through, one view of 117 MB 0.71 against 0.66, of 235 MB 0.76 against 0.66).
template <int U, bool WIDE, int NDIM>
__global__ __launch_bounds__(kPackThreads) void slice_unpack_lines_kernel(PackArgs a) {
    uint64_t wg = a.wg0 + blockIdx.x;
    if (a.per_xcd != 0) {  // each XCD on a contiguous share: see the note above copy_views
        wg = (wg & 7) * a.per_xcd + (wg >> 3);
        if (wg >= a.nwg) return;
    }
    const uint64_t tile = wg / a.nviews;
    const uint32_t v = (uint32_t)(wg % a.nviews);
    const uint64_t task = tile * (kPackThreads / 8) + (threadIdx.x >> 3);  // one line of one row
    uint64_t r;                                                             // row of the view, in iteration order
    uint32_t line;
    if constexpr (WIDE) {
        r = task / a.pieces;
        line = (uint32_t)(task - r * a.pieces);
    } else {
        uint32_t q, m;
        a.pieces_div.divmod((uint32_t)task, q, m);
        r = q;
        line = m;
    }
    const bool live = r < a.nrows;
    if (!live) r = 0;
    uint64_t col;
    const uint64_t loc = decode<WIDE, NDIM>(a.dims, r * a.dims.run, &col);  // first unit of the row; col == 0
    char* __restrict__ row = a.base + (a.offset[v] + loc) * U;
    const char* __restrict__ prow = a.packed[v] + r * a.dims.run * U;       // the row in the packed image
    const int64_t run_bytes = (int64_t)(a.dims.run * U);                    // at least 16
    const int64_t lead = (int64_t)((uintptr_t)row & 127u);                  // the row starts `lead` bytes into its first line
    const int64_t at = (int64_t)line * 128 + (int64_t)(threadIdx.x & 7u) * 16 - lead;  // this lane's vector, relative to the row
    const bool active = live && at + 16 > 0 && at < run_bytes;
    int64_t o = at < 0 ? 0 : at;
    if (o > run_bytes - 16) o = run_bytes - 16;
    const uint4 d = load16_unaligned(prow + o);
    if (active) {
        if (a.stream_stores) store16_unaligned(row + o, d);  // wave-uniform
        else store16_writethrough(row + o, d);
    }
}

// Views whose contiguous runs are shorter than a chunk (element-strided selections such as
// x[:, ::2], rows of a few bytes): a lane still owns whole 16-byte chunks of the packed side,
// which it moves with one aligned 128-bit access, and gathers (pack) or scatters (unpack) the
// chunk's units one by one on the strided side.  All unit loads of a lane are issued before
// the first use and none is predicated.  Unit addresses come from one full decode per chunk
// followed by an odometer over the run and the innermost dimension outside it; a full decode
// is repeated only when that dimension wraps.  Strided-side accesses are NOT non-temporal:
// the lanes of a wavefront return to the same cache lines for every unit of their chunks.
constexpr int kGatherUnroll = 1;

template <int U, bool PACK, bool WIDE, int NDIM>
__global__ __launch_bounds__(kPackThreads) void slice_gather_kernel(PackArgs a) {
    using T = typename UnitType<U>::type;
    constexpr int VU = 16 / U;
    constexpr int UN = kGatherUnroll;
    const uint64_t wg = a.wg0 + blockIdx.x;
    const uint64_t tile = wg / a.nviews;
    const uint32_t v = (uint32_t)(wg % a.nviews);
    char* __restrict__ packed = a.packed[v];
    using M = typename UnitType<U>::mem;  // the strided side may be less aligned than the unit
    M* __restrict__ strided = reinterpret_cast<M*>(a.base) + a.offset[v];
    const uint64_t c0 = tile * (kPackThreads * UN) + threadIdx.x;
    const int nd = NDIM >= 0 ? NDIM : a.dims.ndim;
    const uint64_t run = a.dims.run;
    const uint64_t size_last = a.dims.size[nd - 1];
    const uint64_t step_last = a.dims.stride[nd - 1] - run;  // from one past a run's end to the start of the next run
    const uint64_t safe_first = a.shift ? VU - a.shift : 0;  // first unit of the view's first whole chunk (the host checks there is one)

    uint64_t off[UN][VU];
    bool full[UN], edge[UN];
#pragma unroll
    for (int i = 0; i < UN; ++i) {
        const uint64_t c = c0 + (uint64_t)i * kPackThreads;
        const uint64_t tb = c * VU;
        const uint64_t first = tb - a.shift;
        full[i] = c < a.nchunks && tb >= a.shift && first + VU <= a.total;
        edge[i] = c < a.nchunks && !full[i];
        if (full[i]) {
            uint64_t col;
            uint64_t loc = decode<WIDE, NDIM>(a.dims, first, &col);
            uint64_t ilast;  // index along the innermost dimension outside the run
            if constexpr (WIDE) {
                ilast = ((first - col) / run) % size_last;
            } else {
                uint32_t r32, c32, q32, i32;
                a.dims.run_div.divmod((uint32_t)first, r32, c32);
                a.dims.size_div[nd - 1].divmod(r32, q32, i32);
                ilast = i32;
            }
            off[i][0] = loc;
#pragma unroll
            for (int j = 1; j < VU; ++j) {
                ++col;
                ++loc;
                if (col == run) {
                    col = 0;
                    ++ilast;
                    loc += step_last;
                    if (ilast == size_last) {
                        loc = decode<WIDE, NDIM>(a.dims, first + j, &col);
                        ilast = 0;
                    }
                }
                off[i][j] = loc;
            }
        } else {
#pragma unroll
            for (int j = 0; j < VU; ++j) off[i][j] = 0;  // a valid unit: the view is not empty
        }
    }
    union Chunk {
        uint4 v;
        T e[VU];
    };
    Chunk d[UN];
    if constexpr (PACK) {
#pragma unroll
        for (int i = 0; i < UN; ++i)
#pragma unroll
            for (int j = 0; j < VU; ++j) d[i].e[j] = strided[off[i][j]];
#pragma unroll
        for (int i = 0; i < UN; ++i)
            if (full[i]) store16_aligned(packed + ((c0 + (uint64_t)i * kPackThreads) * VU - a.shift) * U, d[i].v);
    } else {
#pragma unroll
        for (int i = 0; i < UN; ++i) {
            const uint64_t first = (c0 + (uint64_t)i * kPackThreads) * VU - a.shift;
            d[i].v = load16_aligned(packed + (full[i] ? first : safe_first) * U);
        }
#pragma unroll
        for (int i = 0; i < UN; ++i)
            if (full[i]) {
#pragma unroll
                for (int j = 0; j < VU; ++j) strided[off[i][j]] = d[i].e[j];
            }
    }
    // ragged first and last chunk of the view: unit by unit
#pragma unroll
    for (int i = 0; i < UN; ++i) {
        if (edge[i]) move_chunk_by_units<U, PACK, WIDE, NDIM>(a, reinterpret_cast<char*>(strided), packed, c0 + (uint64_t)i * kPackThreads);
    }
}

// Contiguous copy between byte ranges of any alignment (a contiguous view, the "transfer" of a staging buffer):
// single-wavefront workgroups, one 16-byte vector per lane, non-temporal load, write-through store.  For a 50/50
// read/write stream this shape beats the 8-deep tile above by ~5% (16.6 vs 17.4 us for 48 MiB), and single-wavefront
// workgroups beat larger ones (48 MiB: 64 lanes 15.9-16.4 us, 128 lanes 16.7-17.1, 256 lanes 16.6-16.9, 1024 lanes
// 16.5; at 3 GiB 0.85 of peak against 0.75 with 256 lanes x 2 vectors).
//
// What a wavefront writes must be whole cache lines: a 1 KiB row that starts 16 bytes past a line boundary shares its
// first and last line with its neighbours, which run on other XCDs (workgroup i runs on XCD i mod 8) and write the
// line back as two partial lines (3 GiB with both ends 4 bytes past a 16-byte boundary: 0.60-0.65 of peak against
// 0.85).  So the rows are laid on the destination's 1 KiB boundaries - the first row starts with `pad` idle lanes -
// after a head of fewer than 16 bytes, which the first workgroup moves one by one together with the tail.
// The source is read with unaligned 128-bit loads where it is not aligned like the destination; its rows then share
// lines on the read side only, and each XCD takes a contiguous eighth of the rows (per_xcd != 0) so that the shared
// lines meet in one L2 (3 GiB, source 2 bytes off: 0.65 -> 0.70; reading the enclosing aligned vectors and shifting
// them into place instead measured the same with this shape, 0.71 / 0.70, and lower without the XCD shares).
struct ContigArgs {
    char* dst;
    const char* src;
    uint64_t nbytes;
    uint64_t head;     // bytes before the first 16-byte boundary of dst
    uint64_t nvec;     // whole 16-byte destination vectors after the head
    uint64_t per_xcd;  // rows in each XCD's contiguous share; 0: row i is workgroup i
    uint64_t wg0;      // workgroups of this copy launched before this grid
    uint32_t pad;      // idle lanes at the start of row 0
};
constexpr int kCopyThreads = 64;

__global__ __launch_bounds__(kCopyThreads) void contiguous_copy_kernel(ContigArgs a) {
    const uint64_t wg = a.wg0 + blockIdx.x;
    const uint64_t row = a.per_xcd != 0 ? (wg & 7) * a.per_xcd + (wg >> 3) : wg;
    const uint64_t c = row * kCopyThreads + threadIdx.x;  // position in the padded vector grid
    if (c >= a.pad && c - a.pad < a.nvec) {
        const uint64_t at = a.head + (c - a.pad) * 16;
        store16_writethrough(a.dst + at, load16_unaligned(a.src + at));
    }
    if (wg == 0) {
        for (uint64_t i = threadIdx.x; i < a.head; i += kCopyThreads) a.dst[i] = a.src[i];
        for (uint64_t i = a.head + a.nvec * 16 + threadIdx.x; i < a.nbytes; i += kCopyThreads) a.dst[i] = a.src[i];
    }
}

static int launch_contiguous_copy(char* dst, const char* src, uint64_t nbytes, hipStream_t stream) {
    ContigArgs a{};
    a.dst = dst;
    a.src = src;
    a.nbytes = nbytes;
    a.head = (16 - ((uintptr_t)dst & 15u)) & 15u;
    if (a.head > nbytes) a.head = nbytes;
    a.nvec = (nbytes - a.head) / 16;
    a.pad = (uint32_t)(((uintptr_t)(dst + a.head) & 1023u) / 16);
    uint64_t rows = (a.nvec + a.pad + kCopyThreads - 1) / kCopyThreads;
    if (rows == 0) rows = 1;  // the byte loops of the first workgroup
    if ((((uintptr_t)src - (uintptr_t)dst) & 127u) != 0) {
        a.per_xcd = (rows + 7) / 8;
        rows = a.per_xcd * 8;
    }
    return launch_in_pieces(rows, kCopyThreads, 8, [&](uint64_t wg0, uint32_t count) {
        a.wg0 = wg0;
        MHIP_LAUNCH(contiguous_copy_kernel, dim3(count), dim3(kCopyThreads), 0, stream, a);
    });
}

// ---------------- flat bucket <-> ragged tensors ----------------

struct FlatArgs {
    char* flat;
    char* const* tensors;     // device table of ntensors pointers
    const uint64_t* offsets;  // device table of ntensors+1 element offsets
    uint64_t total;           // units
    uint64_t nchunks;
    uint32_t ntensors;
    uint32_t shift;           // units
    uint32_t units_per_elem;
    uint64_t wg0;             // workgroups of this copy launched before this grid
    const uint32_t* index;    // block index of the bucket (tensor of element b * 1024), or null
    uint64_t per_xcd;         // indexed form: tiles in each XCD's contiguous share of the flat buffer
};

// Chunks per lane: 4 when gathering tensors into the flat buffer (0.74 of peak; 8 -> 0.71, 2 -> 0.69),
// 2 when scattering the flat buffer back (0.72; 8 -> 0.66, 1 -> 0.58).
// Lanes per workgroup: 256 (0.765 / 0.725 of peak gathering / scattering a bucket; 128 -> 0.744 / 0.708, 64 -> 0.755 / 0.715).
constexpr int kFlatThreads = kThreads;
template <bool PACK> struct FlatUnroll { static constexpr int value = PACK ? 4 : 2; };

// With a block index (FlatArgs::index, the one mhip_bucket_index_build writes) a wavefront finds the tensor of its
// first unit with one load instead of a table search, which makes single-wavefront workgroups of THREADS = 64 lanes
// with one 1 KiB row each affordable: the shape in which plain copies stream best on this part (a bucket of three
// 1 GiB tensors: 0.73-0.79 of peak with the search form, 0.85 indexed; 2 rows per wavefront 0.80, 4 rows 0.77).
// A tile is a 1 KiB row of the flat buffer, so on the tensor side a row starts wherever the tensor's offset puts it
// and shares its first and last cache line with the neighbouring rows.  Under the plain mapping (workgroup i runs
// on XCD i mod 8) neighbours sit on different XCDs, every shared line is fetched into two L2s and - scattering - is
// written back as two partial lines: 1500 ragged fp32 tensors in separate allocations unpack at 0.72 and pack at
// 0.77, against 0.83 when every tensor is a whole number of 512 B.  The indexed form therefore gives each XCD a
// contiguous eighth of the rows (tile = (wg mod 8) * per_xcd + wg / 8), so that neighbours meet in one L2:
// 0.80 / 0.78 on the ragged bucket, 0.83 / 0.82 on the aligned one (plain mapping: 0.83 / 0.83).  Blocks of 2 to
// 256 rows per XCD instead of one share each measured lower than both (0.72-0.78).
template <int U, bool PACK, int THREADS, int UNROLL, bool INDEXED>
__global__ __launch_bounds__(THREADS) void flat_copy_kernel(FlatArgs a) {
    constexpr int VU = 16 / U;
    constexpr int kFlatThreads = THREADS;
    constexpr int kUnroll = UNROLL;
    static_assert(!INDEXED || THREADS == 64, "the indexed form is one wavefront per workgroup");
    __shared__ uint32_t s_range[2];
    uint32_t r_lo = 0, r_hi = 0;  // tensors of the first and the last unit of this workgroup's tile
    uint64_t tile_id = a.wg0 + blockIdx.x;
    if constexpr (INDEXED) tile_id = (tile_id & 7) * a.per_xcd + (tile_id >> 3);
    const uint64_t block_c0 = tile_id * (kFlatThreads * kUnroll);
    if (block_c0 >= a.nchunks) return;  // padding of the last XCD shares (workgroup-uniform)
    if constexpr (INDEXED) {
        uint64_t c_last = block_c0 + kFlatThreads * kUnroll - 1;
        if (c_last >= a.nchunks) c_last = a.nchunks - 1;
        const uint64_t tb_first = block_c0 * VU, tb_last = c_last * VU + VU - 1;
        uint64_t u_first = tb_first >= a.shift ? tb_first - a.shift : 0;
        uint64_t u_last = tb_last >= a.shift ? tb_last - a.shift : 0;
        if (u_first >= a.total) u_first = a.total - 1;
        if (u_last >= a.total) u_last = a.total - 1;
        // index[b] holds the tensor of element b * 1024, which is at or before the tensor of this tile's first unit
        uint32_t lo = a.index[(u_first / a.units_per_elem) >> 10];
        if (lo >= a.ntensors) lo = a.ntensors - 1;  // an index built for another bucket must not send loads out of the tables
        while (lo + 1 < a.ntensors && a.offsets[lo + 1] * a.units_per_elem <= u_first) ++lo;
        uint32_t hi = lo;
        if (lo + 1 < a.ntensors && a.offsets[lo + 1] * a.units_per_elem <= u_last)
            hi = wave_find_tensor(a.offsets, a.units_per_elem, lo, a.ntensors, u_last);
        r_lo = lo;
        r_hi = hi;
    } else if (threadIdx.x < 64) {
        // wavefront 0 finds the tensors holding the first and the last unit this block touches
        uint64_t c_last = block_c0 + kFlatThreads * kUnroll - 1;
        if (c_last >= a.nchunks) c_last = a.nchunks - 1;
        const uint64_t tb_first = block_c0 * VU, tb_last = c_last * VU + VU - 1;
        uint64_t u_first = tb_first >= a.shift ? tb_first - a.shift : 0;
        uint64_t u_last = tb_last >= a.shift ? tb_last - a.shift : 0;
        if (u_first >= a.total) u_first = a.total - 1;
        if (u_last >= a.total) u_last = a.total - 1;
        const uint32_t lo = wave_find_tensor(a.offsets, a.units_per_elem, 0, a.ntensors, u_first);
        const uint32_t hi = wave_find_tensor(a.offsets, a.units_per_elem, lo, a.ntensors, u_last);
        if (threadIdx.x == 0) {
            s_range[0] = lo;
            s_range[1] = hi;
        }
    }
    if constexpr (!INDEXED) {
        __syncthreads();
        r_lo = s_range[0];
        r_hi = s_range[1];
    }
    const uint32_t t_lo = r_lo, t_hi = r_hi + 1;
    const uint32_t upe = a.units_per_elem;

    {
        // Workgroup-uniform fast path: the whole tile (8 or 16 KiB) lies inside one tensor (most of a
        // bucket's bytes are in tensors much larger than a tile) and inside the flat buffer.
        const uint64_t tile_first = block_c0 * VU;
        const uint64_t tile_end = tile_first + (uint64_t)(kFlatThreads * kUnroll) * VU;
        if (r_lo == r_hi && tile_first >= a.shift && tile_end - a.shift <= a.total) {
            if constexpr (PACK) {
                // Gathering: the tensor side is the one that is read.  Each wavefront takes kUnroll consecutive
                // 1 KiB rows, and when the tensor extends far enough around them it reads the enclosing
                // aligned vectors and shifts them into place instead of issuing unaligned 128-bit loads
                // (0.74 -> 0.77 of peak on a bucket of ragged bf16 tensors).  With one row per wavefront the
                // extra vector per row costs more than it saves (0.78 against 0.82 with unaligned loads).
                const int lane = threadIdx.x & 63;
                const uint64_t row0 = (block_c0 + (uint64_t)(threadIdx.x >> 6) * (kUnroll * 64)) * VU - a.shift;  // units
                const uint64_t t_begin = a.offsets[t_lo] * upe, t_end = a.offsets[t_lo + 1] * upe;
                char* __restrict__ f = a.flat + row0 * U + lane * 16;
                const char* t = a.tensors[t_lo] + (row0 - t_begin) * U;
                const uint32_t shift = (uint32_t)((uintptr_t)t & 15u);
                uint4 d[kUnroll];
                if (kUnroll > 1 && shift != 0 && (row0 - t_begin) * U >= shift && (t_end - row0) * U >= (uint64_t)kUnroll * 1024 + 16 - shift) {
                    const char* base = t - shift;
#pragma unroll
                    for (int i = 0; i < kUnroll; ++i) d[i] = load16_aligned(base + i * 1024 + lane * 16);
                    const uint4 tail = load16_aligned(base + kUnroll * 1024);
                    shift_rows_into_place<kUnroll>(d, tail, shift);
                } else {
#pragma unroll
                    for (int i = 0; i < kUnroll; ++i) d[i] = load16_unaligned(t + i * 1024 + lane * 16);
                }
#pragma unroll
                for (int i = 0; i < kUnroll; ++i) store16_aligned(f + i * 1024, d[i]);
                return;
            }
            const uint64_t first = (block_c0 + threadIdx.x) * VU - a.shift;
            char* __restrict__ f = a.flat + first * U;
            char* __restrict__ t = a.tensors[t_lo] + (first - a.offsets[t_lo] * upe) * U;
            uint4 d[kUnroll];
#pragma unroll
            for (int i = 0; i < kUnroll; ++i) {
                if constexpr (PACK) d[i] = load16_unaligned(t + (size_t)i * kFlatThreads * 16);
                else d[i] = load16_aligned(f + (size_t)i * kFlatThreads * 16);
            }
#pragma unroll
            for (int i = 0; i < kUnroll; ++i) {
                if constexpr (PACK) store16_aligned(f + (size_t)i * kFlatThreads * 16, d[i]);
                else store16_unaligned(t + (size_t)i * kFlatThreads * 16, d[i]);
            }
            return;
        }
    }

    // phase 1: resolve every chunk of this lane to (tensor address, flat address)
    char* tptr[kUnroll];
    char* fptr[kUnroll];
    bool vec[kUnroll];
    bool all_vec = true;
#pragma unroll
    for (int i = 0; i < kUnroll; ++i) {
        const uint64_t c = block_c0 + (uint64_t)i * kFlatThreads + threadIdx.x;
        const uint64_t tb = c * VU;
        const uint64_t first = tb - a.shift;
        vec[i] = false;
        if (c < a.nchunks && tb >= a.shift && first + VU <= a.total) {
            const uint32_t ti = find_tensor(a.offsets, upe, t_lo, t_hi, first);
            const uint64_t begin = a.offsets[ti] * upe, end = a.offsets[ti + 1] * upe;
            if (first + VU <= end) {
                tptr[i] = a.tensors[ti] + (first - begin) * U;
                fptr[i] = a.flat + first * U;
                vec[i] = true;
            }
        }
        all_vec = all_vec && vec[i];
    }
    // phase 2: move them; without predicates when every chunk is a plain 16-byte move
    uint4 data[kUnroll];
    if (all_vec) {
#pragma unroll
        for (int i = 0; i < kUnroll; ++i) data[i] = PACK ? load16_unaligned(tptr[i]) : load16_aligned(fptr[i]);
#pragma unroll
        for (int i = 0; i < kUnroll; ++i) {
            if constexpr (PACK) store16_aligned(fptr[i], data[i]); else store16_unaligned(tptr[i], data[i]);
        }
        return;
    }
#pragma unroll
    for (int i = 0; i < kUnroll; ++i) {
        const uint64_t c = block_c0 + (uint64_t)i * kFlatThreads + threadIdx.x;
        if (c >= a.nchunks) continue;
        if (vec[i]) {
            if constexpr (PACK) store16_aligned(fptr[i], load16_unaligned(tptr[i]));
            else store16_unaligned(tptr[i], load16_aligned(fptr[i]));
            continue;
        }
        if constexpr (VU > 1) {
            const uint64_t tb = c * VU;
            for (int j = 0; j < VU; ++j) {
                const uint64_t unit = tb + j - a.shift;
                if (tb + j >= a.shift && unit < a.total) {
                    const uint32_t ti = find_tensor(a.offsets, upe, t_lo, t_hi, unit);
                    char* t = a.tensors[ti] + (unit - a.offsets[ti] * upe) * U;
                    move_unit<U, PACK>(t, a.flat + unit * U);
                }
            }
        }
    }
}

// ---------------- host side ----------------

enum CopyForm { kWholeChunks, kRaggedRows, kShortRuns, kUnpackLines };

template <int U, bool PACK, int UNROLL>
static void launch_whole_chunks_u(bool wide, int ndim, dim3 grid, hipStream_t stream, const PackArgs& a) {
    const dim3 block(kPackThreads);
    if (wide) {
        MHIP_LAUNCH((slice_copy_kernel<U, PACK, true, -1, UNROLL>), grid, block, 0, stream, a);
        return;
    }
    switch (ndim) {  // the common shapes get a decode without loops
        case 0: MHIP_LAUNCH((slice_copy_kernel<U, PACK, false, 0, UNROLL>), grid, block, 0, stream, a); break;
        case 1: MHIP_LAUNCH((slice_copy_kernel<U, PACK, false, 1, UNROLL>), grid, block, 0, stream, a); break;
        case 2: MHIP_LAUNCH((slice_copy_kernel<U, PACK, false, 2, UNROLL>), grid, block, 0, stream, a); break;
        default: MHIP_LAUNCH((slice_copy_kernel<U, PACK, false, -1, UNROLL>), grid, block, 0, stream, a); break;
    }
}

template <int U, bool PACK>
static void launch_whole_chunks(bool wide, bool large, int ndim, dim3 grid, hipStream_t stream, const PackArgs& a) {
    if (large) launch_whole_chunks_u<U, PACK, kUnrollLarge>(wide, ndim, grid, stream, a);
    else launch_whole_chunks_u<U, PACK, kUnrollSmall>(wide, ndim, grid, stream, a);
}

template <int U, bool PACK>
static void launch_slice_copy_u(bool wide, bool large, CopyForm form, int ndim, dim3 grid, hipStream_t stream, const PackArgs& a) {
    const dim3 block(kPackThreads);
    if (form == kUnpackLines) {
        if constexpr (!PACK) {
            if (wide) {
                MHIP_LAUNCH((slice_unpack_lines_kernel<U, true, -1>), grid, block, 0, stream, a);
                return;
            }
            switch (ndim) {
                case 1: MHIP_LAUNCH((slice_unpack_lines_kernel<U, false, 1>), grid, block, 0, stream, a); break;
                case 2: MHIP_LAUNCH((slice_unpack_lines_kernel<U, false, 2>), grid, block, 0, stream, a); break;
                default: MHIP_LAUNCH((slice_unpack_lines_kernel<U, false, -1>), grid, block, 0, stream, a); break;
            }
        }
        return;
    }
    if constexpr (U < 16) {
        if (form == kShortRuns) {
            if (wide) {
                MHIP_LAUNCH((slice_gather_kernel<U, PACK, true, -1>), grid, block, 0, stream, a);
                return;
            }
            switch (ndim) {
                case 1: MHIP_LAUNCH((slice_gather_kernel<U, PACK, false, 1>), grid, block, 0, stream, a); break;
                case 2: MHIP_LAUNCH((slice_gather_kernel<U, PACK, false, 2>), grid, block, 0, stream, a); break;
                default: MHIP_LAUNCH((slice_gather_kernel<U, PACK, false, -1>), grid, block, 0, stream, a); break;
            }
            return;
        }
        if (form == kRaggedRows) {
            if (wide) {
                MHIP_LAUNCH((slice_copy_ragged_kernel<U, PACK, true, -1>), grid, block, 0, stream, a);
                return;
            }
            switch (ndim) {
                case 1: MHIP_LAUNCH((slice_copy_ragged_kernel<U, PACK, false, 1>), grid, block, 0, stream, a); break;
                case 2: MHIP_LAUNCH((slice_copy_ragged_kernel<U, PACK, false, 2>), grid, block, 0, stream, a); break;
                default: MHIP_LAUNCH((slice_copy_ragged_kernel<U, PACK, false, -1>), grid, block, 0, stream, a); break;
            }
            return;
        }
    }
    launch_whole_chunks<U, PACK>(wide, large, ndim, grid, stream, a);
}

template <bool PACK>
static void launch_slice_copy(uint32_t unit, bool wide, bool large, CopyForm form, dim3 grid, hipStream_t stream, const PackArgs& a) {
    switch (unit) {
        case 1: launch_slice_copy_u<1, PACK>(wide, large, form, a.dims.ndim, grid, stream, a); break;
        case 2: launch_slice_copy_u<2, PACK>(wide, large, form, a.dims.ndim, grid, stream, a); break;
        case 4: launch_slice_copy_u<4, PACK>(wide, large, form, a.dims.ndim, grid, stream, a); break;
        case 8: launch_slice_copy_u<8, PACK>(wide, large, form, a.dims.ndim, grid, stream, a); break;
        default: launch_slice_copy_u<16, PACK>(wide, large, form == kUnpackLines ? kUnpackLines : kWholeChunks, a.dims.ndim, grid, stream, a); break;
    }
}

// One view whose canonical form has more dimensions than the kernel decodes: peel the
// outermost dimension on the host.
template <bool PACK>
static int copy_views(char* base, char* const* packed, const mhip_slice_t* views, uint32_t nviews,
                      uint32_t elem_size, hipStream_t stream);

template <bool PACK>
static int copy_deep_view(char* base, char* packed, const mhip_slice_t& s, uint32_t elem_size, hipStream_t stream) {
    // s.ndim > 0 here; split along dimension 0 into sizes[0] views of one dimension fewer
    uint64_t inner = 1;
    for (uint32_t k = 1; k < s.ndim; ++k) inner *= s.sizes[k];
    for (uint64_t i = 0; i < s.sizes[0]; ++i) {
        mhip_slice_t sub{s.offset + i * s.strides[0], s.ndim - 1, s.sizes + 1, s.strides + 1};
        char* p = packed + i * inner * elem_size;
        if (int rc = copy_views<PACK>(base, &p, &sub, 1, elem_size, stream)) return rc;
    }
    return MHIP_SUCCESS;
}

// A pack of one view reads rows of the strided side in 1 KiB pieces cut on the packed side's grid.  When the rows are
// not whole cache lines (a column block that starts 16 bytes into a line, a pitch that is not a multiple of 128 bytes),
// nearly every piece starts and ends inside a line that the neighbouring pieces read as well - on other XCDs under the
// plain mapping (workgroup i runs on XCD i mod 8), so the line crosses HBM twice.  Giving each XCD a contiguous eighth
// of the pieces lets the neighbours meet in one L2: bf16 [16384, 14336] columns 8:1800 0.68 -> 0.72 of peak, columns
// 0:1784 0.69 -> 0.73, pitch 14335 0.68 -> 0.73, fp32 rows of 1024 at pitch 8191 0.70 -> 0.75.  Rows of whole lines
// measure the same either way or better (64 of 256 fp32 columns 0.57 -> 0.63; bf16 columns 0:1792 0.746 both ways), so
// every single-view pack of whole chunks takes the shares (the eight column blocks of one tensor in one launch, where
// the view index already pins each view to one XCD, lose with them: 0.78 -> 0.68).  The gathering form does not (bf16 rows of 1790: 0.69 -> 0.59,
// though fp32 rows of 255 gain 0.03).  The two-vector form and the line-by-line unpack take them for rows of 6 KiB and
// more (bf16 [16384, 14336], columns c:c+7166, packing 0.75 -> 0.78, unpacking 0.72 -> 0.755; rows of 7160 bytes +0.02 /
// +0.03 to +0.10; rows of 3580 bytes -0.02 either way, so shorter rows keep the plain mapping).
//
// Unpacks of whole chunks write the strided side in 1 KiB pieces cut on the packed side's grid.  With units under 16
// bytes (a view that starts 2-8 bytes past a 16-byte boundary, a pitch that is not a multiple of 16) every piece
// starts and ends inside a line its neighbours write as well, and the shares let those partial lines meet in one L2
// before they go to HBM: bf16 columns 1:7169 0.66 -> 0.73, 1:3585 0.60 -> 0.68, 1:1793 0.53 -> 0.59.  16-byte units
// store write-through while the copy is small enough to stay in the Infinity Cache (58 MB views: 0.87-0.89 in a
// rotation of 350 MB, 0.54-0.68 with non-temporal stores); from 96 MiB on they stream with non-temporal stores
// (one column block of 235 MB: 0.70 -> 0.81; 117 MB: 0.70 -> 0.755); when their rows do not start and end on cache
// lines they are unpacked line by line instead (rows of 256 bytes and more; columns 8:7176 0.59 -> 0.76), or take the
// shares (shorter rows).  Several views in one launch keep write-through stores at any size (the eight column blocks
// of a 117 MB tensor: 0.794 against 0.777).
constexpr uint64_t kSharesFromRowBytes = 6144;
constexpr uint64_t kStreamUnpackFromBytes = 96ull << 20;
template <bool PACK>
static int copy_views(char* base, char* const* packed, const mhip_slice_t* views, uint32_t nviews,
                      uint32_t elem_size, hipStream_t stream) {
    uint32_t k = 0;
    while (k < nviews) {
        CanonSlice first;
        uint32_t unit = 0;
        const uint64_t mask0 = (uint64_t)(uintptr_t)base | (uint64_t)(uintptr_t)packed[k];
        if (!canonicalize(views[k], elem_size, mask0, 16, &first, &unit)) {  // empty view: nothing to move
            ++k;
            continue;
        }
        if (first.ndim == 0) {  // one run, of any alignment
            char* strided = base + first.offset * unit;
            if (int rc = launch_contiguous_copy(PACK ? packed[k] : strided, PACK ? strided : packed[k], first.total * unit, stream))
                return rc;
            ++k;
            continue;
        }
        {
            int trc = MHIP_SUCCESS;
            if (try_transpose_copy<PACK>(base, packed[k], first, unit, stream, &trc)) {
                if (trc) return trc;
                ++k;
                continue;
            }
        }
        // The direct forms reach the strided side with accesses that tolerate any address (see UnitType), so the
        // address at which a view starts need not limit the unit: a bf16 view of even row length and pitch that
        // starts at an odd column is moved in 4-byte units from a base that is 2 bytes off.  On bf16 [16384, 14336]:
        // columns 1:895 pack 0.46 -> 0.66 of peak (the 4-byte gathering form instead of the 2-byte two-vector form),
        // 1:1791 0.61 -> 0.67, columns 1:897 unpack 0.41 -> 0.60, 1:1793 0.59 -> 0.70; never slower.
        uint64_t skew = 0;  // bytes from `base` to the address the unit offsets count from
        if (unit < 16) {
            CanonSlice relaxed;
            uint32_t unit_r = 0;
            uint64_t skew_r = 0;
            canonicalize(views[k], elem_size, (uint64_t)(uintptr_t)packed[k], 16, &relaxed, &unit_r, &skew_r);
            if (unit_r > unit) {
                first = relaxed;
                unit = unit_r;
                skew = skew_r;
            }
        }
        const bool any_base = skew != 0 || ((uintptr_t)base & (unit - 1)) != 0;  // the unit was chosen without the strided address
        PackArgs a{};
        bool fits32 = false;
        if (!make_dims_arg(first, &a.dims, &fits32)) {
            if (int rc = copy_deep_view<PACK>(base, packed[k], views[k], elem_size, stream)) return rc;
            ++k;
            continue;
        }
        const uint32_t shift_bytes = (uint32_t)((uintptr_t)packed[k] & 15u);
        a.base = base + skew;
        a.total = first.total;
        a.shift = shift_bytes / unit;
        const uint32_t vu = 16 / unit;
        a.nchunks = (first.total + a.shift + vu - 1) / vu;
        a.packed[0] = packed[k];
        a.offset[0] = first.offset;
        uint32_t nbatch = 1;
        // batch following views that differ only in offset and staging pointer
        while (k + nbatch < nviews && nbatch < (uint32_t)kMaxViews) {
            CanonSlice next;
            uint32_t unit2 = 0;
            uint64_t skew2 = 0;
            const uint64_t mask = (any_base ? 0 : (uint64_t)(uintptr_t)base) | (uint64_t)(uintptr_t)packed[k + nbatch];
            if (!canonicalize(views[k + nbatch], elem_size, mask, 16, &next, &unit2, any_base ? &skew2 : nullptr)) break;
            if (unit2 != unit || skew2 != skew || !same_shape(first, next)) break;
            if (((uintptr_t)packed[k + nbatch] & 15u) != shift_bytes) break;
            a.packed[nbatch] = packed[k + nbatch];
            a.offset[nbatch] = next.offset;
            ++nbatch;
        }
        CopyForm form = kWholeChunks;
        if (unit < 16 && first.ndim >= 1 && (first.run % vu != 0 || a.shift != 0)) {
            // Rows that are not whole chunks.  Measured on 8192^2 matrices with rows of r-1 of r elements:
            // gathering 4-byte units into a chunk streams at 0.77 of peak whatever the row length (the
            // two-vector form reaches 0.64-0.75), gathering 2-byte units at 0.50 (two-vector form: 0.50 at
            // 254-byte rows, 0.58 at 510, 0.69 at 2046); scattering units is slower than either beyond
            // 256-byte rows (fp32: 0.46-0.49 against 0.61-0.73).
            uint64_t gather_below = 16 * vu;                 // row length in units
            if (unit == 1) gather_below = 4 * vu;
            if (PACK && unit >= 4) gather_below = 256 * vu;  // rows under 4 KiB; longer ones: 0.72-0.75 two-vector vs 0.69-0.74
            if (first.run < gather_below && first.total >= 2 * vu) form = kShortRuns;
            else if (first.run >= vu) form = kRaggedRows;
        }
        // Unpacking ragged rows of 256 bytes and more line by line of the written side (see slice_unpack_lines_kernel).
        // Shorter rows keep the two-vector form: their two or three lines would leave half the lanes idle.  Rows of
        // whole chunks that do not start and end on cache lines go the same way once a single view is too large to
        // stay in the Infinity Cache (bf16 columns 8:7176 of [16384, 14336]: 0.73 with the chunk grid, streamed stores
        // and XCD shares, 0.76 line by line; below that size write-through stores on the chunk grid win, 0.85 against 0.58).
        uint64_t line_blocks = 0;
        bool wide = !fits32;
        bool lines_of_whole_chunks = false;
        if (!PACK && form == kWholeChunks && nbatch == 1 && first.total * unit >= kStreamUnpackFromBytes) {
            uint64_t mask = (uint64_t)(uintptr_t)(a.base + first.offset * unit) | (first.run * unit);
            for (int d = 0; d < first.ndim; ++d) mask |= first.dims[d].stride * unit;
            lines_of_whole_chunks = (mask & 127u) != 0;
        }
        if (!PACK && (form == kRaggedRows || lines_of_whole_chunks) && first.run * unit >= 256) {
            const uint64_t run_bytes = first.run * unit;
            uint64_t pitch_mask = 0;
            for (int d = 0; d < first.ndim; ++d) pitch_mask |= first.dims[d].stride * unit;
            // lines a row overlaps: all rows of a view start at the same place in their lines when all pitches are
            // whole lines (the views of one launch each at their own)
            const uint64_t row_align = any_base ? 1 : unit;  // what every row's address is a multiple of
            uint64_t lines = (run_bytes + 128 - row_align + 127) / 128;
            if ((pitch_mask & 127u) == 0) {
                uint64_t lead = 0;
                for (uint32_t v = 0; v < nbatch; ++v) {
                    const uint64_t l = (uintptr_t)(a.base + a.offset[v] * unit) & 127u;
                    lead = l > lead ? l : lead;
                }
                lines = (lead + run_bytes + 127) / 128;
            }
            const uint64_t nrows = first.total / first.run;
            if (lines < kFastDivLimit && nrows <= UINT64_MAX / 8 / lines) {
                form = kUnpackLines;
                a.pieces = (uint32_t)lines;
                a.pieces_div = FastDiv32((uint32_t)lines);
                a.nrows = nrows;
                if (nrows * lines + kPackThreads >= kFastDivLimit) wide = true;
                line_blocks = (nrows * lines + kPackThreads / 8 - 1) / (kPackThreads / 8);
                a.stream_stores = nbatch * first.total * unit >= kStreamUnpackFromBytes;  // by the bytes the launch writes
            }
        }
        const bool large = a.nchunks >= kLargeCopyChunks;
        const uint64_t per_block = (uint64_t)kPackThreads * (form == kRaggedRows ? kRaggedUnroll : form == kShortRuns ? kGatherUnroll : large ? kUnrollLarge : kUnrollSmall);
        uint64_t blocks = (a.nchunks + per_block - 1) / per_block;
        if (form == kUnpackLines) blocks = line_blocks;  // eight lanes per line of every row
        a.nviews = nbatch;
        uint64_t nwg = blocks * nbatch;
        // which single-view copies take XCD-contiguous shares, and how an unpack of 16-byte units stores: see the
        // note above copy_views
        bool shares = false;
        if (nbatch == 1) {
            const uint64_t run_bytes = first.run * unit;
            if (PACK) {
                shares = form == kWholeChunks || (form == kRaggedRows && run_bytes >= kSharesFromRowBytes);
            } else if (form == kUnpackLines) {
                shares = run_bytes >= kSharesFromRowBytes;
            } else if (form == kWholeChunks) {
                if (unit < 16) {
                    shares = true;
                } else if (first.total * unit >= kStreamUnpackFromBytes) {
                    a.stream_stores = 1;
                    uint64_t mask = (uint64_t)(uintptr_t)(a.base + first.offset * unit) | run_bytes;
                    for (int d = 0; d < first.ndim; ++d) mask |= first.dims[d].stride * unit;
                    shares = (mask & 127u) != 0;  // the 1 KiB pieces a wavefront writes are not whole cache lines
                }
            }
        }
        if (shares) {
            a.nwg = nwg;
            a.per_xcd = (nwg + 7) / 8;
            nwg = a.per_xcd * 8;
        }
        if (int rc = launch_in_pieces(nwg, kPackThreads, 8, [&](uint64_t wg0, uint32_t count) {
                a.wg0 = wg0;
                launch_slice_copy<PACK>(unit, wide, large, form, dim3(count), stream, a);
            }))
            return rc;
        k += nbatch;
    }
    return MHIP_SUCCESS;
}

template <bool PACK>
static int slice_copy_entry(char* base, char* const* packed, const mhip_slice_t* views, uint32_t nviews,
                            uint32_t elem_size, mhip_stream_t stream) {
    if (elem_size == 0 || (nviews && (!views || !packed))) return MHIP_ERR_INVALID_ARGUMENT;
    for (uint32_t k = 0; k < nviews; ++k) {
        const mhip_slice_t& s = views[k];
        if (s.ndim > MHIP_MAX_DIMS || (s.ndim && (!s.sizes || !s.strides))) return MHIP_ERR_INVALID_ARGUMENT;
        if (int rc = validate_slice(s.sizes, s.ndim, s.strides, s.ndim)) return rc;
        if (!slice_fits_address_space(s, elem_size)) return MHIP_ERR_INVALID_ARGUMENT;
        if (slice_len(s) != 0 && (!base || !packed[k])) return MHIP_ERR_UNDEFINED_TENSOR;
    }
    hipStream_t hs = static_cast<hipStream_t>(stream);
    DeviceGuard guard(hs);
    return copy_views<PACK>(base, packed, views, nviews, elem_size, hs);
}

template <bool PACK>
static int flat_copy_entry(char* flat, char* const* d_tensors, const uint64_t* d_offsets, uint32_t ntensors,
                           uint64_t total, uint32_t elem_size, const uint32_t* d_index, mhip_stream_t stream) {
    if (elem_size == 0) return MHIP_ERR_INVALID_ARGUMENT;
    if (ntensors == 0 || total == 0) return MHIP_SUCCESS;
    if (!flat || !d_tensors || !d_offsets) return MHIP_ERR_UNDEFINED_TENSOR;
    if ((uintptr_t)d_index & 3u) return MHIP_ERR_INVALID_ARGUMENT;
    // unit: the power-of-two part of the element size, limited by the flat buffer's alignment
    uint32_t unit = 16;
    while (unit > 1 && ((elem_size | (uintptr_t)flat) & (unit - 1))) unit >>= 1;
    // tensors are only guaranteed element-aligned, so the unit must divide the element size
    FlatArgs a{};
    a.flat = flat;
    a.tensors = d_tensors;
    a.offsets = d_offsets;
    a.units_per_elem = elem_size / unit;
    a.total = total * a.units_per_elem;
    a.ntensors = ntensors;
    a.shift = (uint32_t)(((uintptr_t)flat & 15u) / unit);
    const uint32_t vu = 16 / unit;
    a.nchunks = (a.total + a.shift + vu - 1) / vu;
    hipStream_t hs = static_cast<hipStream_t>(stream);
    DeviceGuard guard(hs);
    if (d_index != nullptr) {
        a.index = d_index;
        a.per_xcd = ((a.nchunks + 63) / 64 + 7) / 8;  // one 64-chunk row per workgroup, eight equal shares
        return launch_in_pieces(a.per_xcd * 8, 64, 8, [&](uint64_t wg0, uint32_t count) {
            a.wg0 = wg0;
            const dim3 grid(count), block(64);
            switch (unit) {
                case 1: MHIP_LAUNCH((flat_copy_kernel<1, PACK, 64, 1, true>), grid, block, 0, hs, a); break;
                case 2: MHIP_LAUNCH((flat_copy_kernel<2, PACK, 64, 1, true>), grid, block, 0, hs, a); break;
                case 4: MHIP_LAUNCH((flat_copy_kernel<4, PACK, 64, 1, true>), grid, block, 0, hs, a); break;
                case 8: MHIP_LAUNCH((flat_copy_kernel<8, PACK, 64, 1, true>), grid, block, 0, hs, a); break;
                default: MHIP_LAUNCH((flat_copy_kernel<16, PACK, 64, 1, true>), grid, block, 0, hs, a); break;
            }
        });
    }
    constexpr int kUnroll = FlatUnroll<PACK>::value;
    const uint64_t per_block = (uint64_t)kFlatThreads * kUnroll;
    const uint64_t blocks = (a.nchunks + per_block - 1) / per_block;
    return launch_in_pieces(blocks, kFlatThreads, 1, [&](uint64_t wg0, uint32_t count) {
        a.wg0 = wg0;
        const dim3 grid(count), block(kFlatThreads);
        switch (unit) {
            case 1: MHIP_LAUNCH((flat_copy_kernel<1, PACK, kFlatThreads, kUnroll, false>), grid, block, 0, hs, a); break;
            case 2: MHIP_LAUNCH((flat_copy_kernel<2, PACK, kFlatThreads, kUnroll, false>), grid, block, 0, hs, a); break;
            case 4: MHIP_LAUNCH((flat_copy_kernel<4, PACK, kFlatThreads, kUnroll, false>), grid, block, 0, hs, a); break;
            case 8: MHIP_LAUNCH((flat_copy_kernel<8, PACK, kFlatThreads, kUnroll, false>), grid, block, 0, hs, a); break;
            default: MHIP_LAUNCH((flat_copy_kernel<16, PACK, kFlatThreads, kUnroll, false>), grid, block, 0, hs, a); break;
        }
    });
}

}  // namespace mhip

using namespace mhip;

extern "C" {

int mhip_slice_pack(void* dst, const void* src_base, const mhip_slice_t* s, uint32_t elem_size,
                    mhip_stream_t stream) {
    if (!s) return MHIP_ERR_INVALID_ARGUMENT;
    char* p = static_cast<char*>(dst);
    return slice_copy_entry<true>(const_cast<char*>(static_cast<const char*>(src_base)), &p, s, 1, elem_size, stream);
}

int mhip_slice_unpack(void* dst_base, const void* src, const mhip_slice_t* s, uint32_t elem_size,
                      mhip_stream_t stream) {
    if (!s) return MHIP_ERR_INVALID_ARGUMENT;
    char* p = const_cast<char*>(static_cast<const char*>(src));
    return slice_copy_entry<false>(static_cast<char*>(dst_base), &p, s, 1, elem_size, stream);
}

int mhip_slice_pack_many(void* const* dsts, const void* src_base, const mhip_slice_t* views, uint32_t nviews,
                         uint32_t elem_size, mhip_stream_t stream) {
    return slice_copy_entry<true>(const_cast<char*>(static_cast<const char*>(src_base)),
                                  reinterpret_cast<char* const*>(dsts), views, nviews, elem_size, stream);
}

int mhip_slice_unpack_many(void* dst_base, const void* const* srcs, const mhip_slice_t* views, uint32_t nviews,
                           uint32_t elem_size, mhip_stream_t stream) {
    return slice_copy_entry<false>(static_cast<char*>(dst_base),
                                   reinterpret_cast<char* const*>(const_cast<void* const*>(
                                       reinterpret_cast<const void* const*>(srcs))),
                                   views, nviews, elem_size, stream);
}

int mhip_flat_pack(void* flat, const void* const* d_tensors, const uint64_t* d_offsets, uint32_t ntensors,
                   uint64_t total, uint32_t elem_size, const uint32_t* d_index, mhip_stream_t stream) {
    return flat_copy_entry<true>(static_cast<char*>(flat),
                                 reinterpret_cast<char* const*>(const_cast<void* const*>(
                                     reinterpret_cast<const void* const*>(d_tensors))),
                                 d_offsets, ntensors, total, elem_size, d_index, stream);
}

int mhip_flat_unpack(void* const* d_tensors, const void* flat, const uint64_t* d_offsets, uint32_t ntensors,
                     uint64_t total, uint32_t elem_size, const uint32_t* d_index, mhip_stream_t stream) {
    return flat_copy_entry<false>(const_cast<char*>(static_cast<const char*>(flat)),
                                  reinterpret_cast<char* const*>(d_tensors), d_offsets, ntensors, total,
                                  elem_size, d_index, stream);
}

}  // extern "C"
