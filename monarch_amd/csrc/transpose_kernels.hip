// LDS-tiled transposing pack / unpack for Slices whose innermost iteration dimension is
// NOT the memory-contiguous one (column-major views, permuted dims).
//
// Let c be the (unique) dimension with unit stride, and let q enumerate, row-major, all
// dimensions that come after c in iteration order (Q = product of their sizes).  In the
// packed image, q is the fast index; in memory, c is.  A workgroup moves a TILE x TILE
// tile: it reads rows that are contiguous along c, parks them in LDS, and writes rows
// that are contiguous along q, so that both HBM sides see coalesced wavefront accesses
// (the direct gather would fetch a whole 64-byte sector per element on one side).
// Elements of 1, 2, 4 and 8 bytes use slice_transpose_vec_kernel (256- or 512-byte tile rows, 16 bytes per lane
// on both HBM sides, LDS rows XOR-permuted in 16-byte groups); only the 16-byte-element variant,
// slice_transpose_kernel, uses a 32 x 32 tile padded by one element per row.
#include <cstdio>

#include "mhip_device.h"
#include "pack_internal.h"

namespace mhip {

// Orders in which the workgroups of the vector kernel take tiles.
enum : uint32_t { kWalkBlocked = 0, kWalkPackedFastest = 1, kWalkMemoryFastest = 2, kWalkDiagonal = 3 };

struct TransArgs {
    char* base;
    char* packed;
    uint64_t offset;   // units (elements), start of the view in memory
    uint64_t ntiles;   // nbatch * qtiles * ctiles
    uint32_t Sc, Q;    // extent along c and along q
    uint32_t ctiles, qtiles;
    uint64_t wg0;      // workgroups of this copy launched before this grid (a multiple of 8)
    uint32_t walk;      // kWalk*: the order in which workgroups take tiles (chosen on the host, see choose_walk)
    uint32_t xcd_ranges;  // 1: each XCD (workgroup index mod 8) owns a contiguous eighth of the walk; 0: workgroup i takes tile i
    uint32_t rotate;    // rotate the c-groups of each eighth of the walk against the previous one (see the host side)
    uint32_t qgroups;   // ceil(qtiles / group)
    uint64_t rows_per_eighth;  // ceil(nbatch * qgroups / 8)
    uint32_t aligned_stores;  // kStore*: how tile rows are written (write-through / streaming need 16-byte aligned rows)
    uint32_t seg_len, nseg, nstrips;  // strip kernel: positions of a written row per workgroup, segments per row, strips of written rows
    uint32_t group;    // tiles are walked in group x group blocks so that concurrently running workgroups
    uint32_t cgroups;  // touch neighbouring segments on BOTH sides (DRAM row locality); cgroups = ceil(ctiles/group)
    int n_inner;       // dimensions after c (decode q -> memory offset), outermost first
    int n_outer;       // dimensions before c (decode batch -> memory offset), outermost first
    uint32_t inner_size[kMaxCanonDims];
    FastDiv32 inner_div[kMaxCanonDims];
    uint64_t inner_stride[kMaxCanonDims];
    uint32_t outer_size[kMaxCanonDims];
    FastDiv32 outer_div[kMaxCanonDims];
    uint64_t outer_stride[kMaxCanonDims];
};

// Loads and stores of the 16-byte-element kernel (one element per lane, 512-byte runs).  It unpacks with streaming (nt) loads and stores - sixteen shapes of complex128,
// every one +0.01 to +0.07 of peak (8192^2 0.54 -> 0.59, 8200^2 0.64 -> 0.71) - and packs through the cache: there
// streaming stores cost up to 0.10 on power-of-two pitches (8192^2 0.54 -> 0.44) and gain 0.02 at most elsewhere.
template <bool STREAM, typename T> __device__ __forceinline__ T ldg(const T* p) {
    if constexpr (STREAM && sizeof(T) == 16) {
        const uint4 v = load16_aligned(p);
        return *reinterpret_cast<const T*>(&v);
    } else {
        return *p;
    }
}
template <bool STREAM, typename T> __device__ __forceinline__ void stg(T* p, T v) {
    if constexpr (STREAM && sizeof(T) == 16) store16_aligned(p, *reinterpret_cast<const uint4*>(&v));
    else *p = v;
}
// A tile row stored to HBM: through the cache, write-through or streaming (see choose_cache_policy).
enum : uint32_t { kStoreCached = 0, kStoreWriteThrough = 1, kStoreStreaming = 2 };
__device__ __forceinline__ void tstore(void* p, const u32x4& v, uint32_t policy) {
    if (policy == kStoreWriteThrough) store16_writethrough_raw(p, v);
    else if (policy == kStoreStreaming) __builtin_nontemporal_store(v, static_cast<u32x4_unaligned*>(p));
    else *static_cast<u32x4_unaligned*>(p) = v;
}
// A tile row loaded from HBM; STREAM marks the lines as not worth keeping (the nt bit).
template <bool STREAM> __device__ __forceinline__ u32x4 tload(const void* p) {
    if constexpr (STREAM) return __builtin_nontemporal_load(static_cast<const u32x4_unaligned*>(p));
    else return *static_cast<const u32x4_unaligned*>(p);
}

template <typename T, int TILE, bool PACK>
__global__ __launch_bounds__(kThreads) void slice_transpose_kernel(TransArgs a) {
    __shared__ T tile[TILE][TILE + 1];  // [q][c]
    __shared__ uint64_t s_off[TILE];
    constexpr int ROWS_PER_PASS = kThreads / TILE;
    const int lane_x = threadIdx.x % TILE;  // position along the contiguous side of a pass
    const int lane_y = threadIdx.x / TILE;
    T* __restrict__ mem = reinterpret_cast<T*>(a.base) + a.offset;
    T* __restrict__ packed = reinterpret_cast<T*>(a.packed);
    const uint64_t per_batch = (uint64_t)a.cgroups * ((a.qtiles + a.group - 1) / a.group) * a.group * a.group;

    for (uint64_t tile_id = blockIdx.x; tile_id < a.ntiles; tile_id += gridDim.x) {
        const uint64_t b = tile_id / per_batch;
        const uint32_t in_batch = (uint32_t)(tile_id - b * per_batch);
        const uint32_t gsz = a.group * a.group;
        const uint32_t grp = in_batch / gsz, within = in_batch - grp * gsz;
        const uint32_t gq = grp / a.cgroups, gc = grp - gq * a.cgroups;
        const uint32_t qt = gq * a.group + within / a.group, ct = gc * a.group + within % a.group;
        if (qt >= a.qtiles || ct >= a.ctiles) continue;  // padding of the blocked walk (uniform per workgroup)
        const uint32_t q0 = qt * TILE, c0 = ct * TILE;
        // memory offset of the batch: decode b over the dimensions before c
        uint64_t batch_off = 0;
        {
            uint64_t rem = b;
            for (int k = a.n_outer - 1; k >= 0; --k) {
                const uint64_t qd = rem / a.outer_size[k];
                batch_off += (rem - qd * a.outer_size[k]) * a.outer_stride[k];
                rem = qd;
            }
        }
        if (threadIdx.x < TILE) {
            uint32_t q = q0 + threadIdx.x;
            uint64_t off = 0;
            if (q < a.Q) {
                for (int k = a.n_inner - 1; k > 0; --k) {
                    uint32_t qd, r;
                    a.inner_div[k].divmod(q, qd, r);
                    off += (uint64_t)r * a.inner_stride[k];
                    q = qd;
                }
                off += (uint64_t)q * a.inner_stride[0];
            }
            s_off[threadIdx.x] = off;
        }
        __syncthreads();
        const uint64_t packed_row0 = (b * a.Sc + c0) * (uint64_t)a.Q + q0;  // packed index of tile element (c0, q0)
        // Interior tiles take loops without bounds tests, so that all 16 loads of a lane are in
        // flight before the first LDS write; edge tiles take the predicated form.
        const bool full = q0 + TILE <= a.Q && c0 + TILE <= a.Sc;
        const T* mem_tile = mem + batch_off + c0 + lane_x;              // + s_off[r] per row
        T* mem_tile_w = mem + batch_off + c0 + lane_x;
        T* packed_tile = packed + packed_row0 + lane_x;                 // + cc * Q per column
        if constexpr (PACK) {
            // memory -> LDS: lanes run along c
            if (full) {
                T v[TILE / ROWS_PER_PASS];
#pragma unroll
                for (int i = 0; i < TILE / ROWS_PER_PASS; ++i) v[i] = ldg<!PACK>(mem_tile + s_off[lane_y + i * ROWS_PER_PASS]);
#pragma unroll
                for (int i = 0; i < TILE / ROWS_PER_PASS; ++i) tile[lane_y + i * ROWS_PER_PASS][lane_x] = v[i];
            } else {
                for (int r = lane_y; r < TILE; r += ROWS_PER_PASS)
                    if (q0 + r < a.Q && c0 + lane_x < a.Sc) tile[r][lane_x] = ldg<!PACK>(mem_tile + s_off[r]);
            }
            __syncthreads();
            // LDS -> packed: lanes run along q
            if (full) {
#pragma unroll
                for (int i = 0; i < TILE / ROWS_PER_PASS; ++i) {
                    const int cc = lane_y + i * ROWS_PER_PASS;
                    stg<!PACK>(packed_tile + (uint64_t)cc * a.Q, tile[lane_x][cc]);
                }
            } else {
                for (int cc = lane_y; cc < TILE; cc += ROWS_PER_PASS)
                    if (c0 + cc < a.Sc && q0 + lane_x < a.Q) stg<!PACK>(packed_tile + (uint64_t)cc * a.Q, tile[lane_x][cc]);
            }
        } else {
            if (full) {
                T v[TILE / ROWS_PER_PASS];
#pragma unroll
                for (int i = 0; i < TILE / ROWS_PER_PASS; ++i)
                    v[i] = ldg<!PACK>(packed_tile + (uint64_t)(lane_y + i * ROWS_PER_PASS) * a.Q);
#pragma unroll
                for (int i = 0; i < TILE / ROWS_PER_PASS; ++i) tile[lane_x][lane_y + i * ROWS_PER_PASS] = v[i];
            } else {
                for (int cc = lane_y; cc < TILE; cc += ROWS_PER_PASS)
                    if (c0 + cc < a.Sc && q0 + lane_x < a.Q) tile[lane_x][cc] = ldg<!PACK>(packed_tile + (uint64_t)cc * a.Q);
            }
            __syncthreads();
            if (full) {
#pragma unroll
                for (int i = 0; i < TILE / ROWS_PER_PASS; ++i) {
                    const int r = lane_y + i * ROWS_PER_PASS;
                    stg<!PACK>(mem_tile_w + s_off[r], tile[r][lane_x]);
                }
            } else {
                for (int r = lane_y; r < TILE; r += ROWS_PER_PASS)
                    if (q0 + r < a.Q && c0 + lane_x < a.Sc) stg<!PACK>(mem_tile_w + s_off[r], tile[r][lane_x]);
            }
        }
        __syncthreads();  // the tile and s_off are reused by the next iteration
    }
}

// The tile (batch b, q-tile qt, c-tile ct) this workgroup takes, in the order the host chose (see choose_walk); false when
// the workgroup is padding of the walk.  Uniform over the workgroup.
__device__ __forceinline__ bool walk_tile(const TransArgs& a, uint64_t* b_out, uint32_t* qt_out, uint32_t* ct_out) {
    const uint64_t per_batch = (uint64_t)a.cgroups * ((a.qtiles + a.group - 1) / a.group) * a.group * a.group;

    // workgroup w runs on XCD w % 8
    const uint64_t per_xcd = (a.ntiles + 7) / 8;
    const uint64_t wg = a.wg0 + blockIdx.x;
    const uint64_t tile_id = a.xcd_ranges ? (wg % 8) * per_xcd + wg / 8 : wg;
    if (tile_id >= a.ntiles) return false;

    uint64_t b;
    uint32_t qt, ct;
    if (a.walk == kWalkBlocked) {
        b = tile_id / per_batch;
        const uint32_t in_batch = (uint32_t)(tile_id - b * per_batch);
        const uint32_t gsz = a.group * a.group;
        const uint32_t grp = in_batch / gsz, within = in_batch - grp * gsz;
        const uint32_t gq = grp / a.cgroups;
        uint32_t gc = grp - gq * a.cgroups;
        if (a.rotate) {
            // a function of the row of groups alone, so that every row still visits each of its c-groups once
            const uint32_t eighth = (uint32_t)((b * a.qgroups + gq) / a.rows_per_eighth);  // 0..7: the XCD, when ranges hold whole rows
            gc = (gc + eighth * a.cgroups / 8) % a.cgroups;
        }
        qt = gq * a.group + within / a.group;
        ct = gc * a.group + within % a.group;
        if (qt >= a.qtiles || ct >= a.ctiles) return false;  // padding of the blocked walk (uniform per workgroup)
    } else {
        const uint64_t plain = (uint64_t)a.qtiles * a.ctiles;
        b = tile_id / plain;
        const uint32_t t = (uint32_t)(tile_id - b * plain);
        if (a.walk == kWalkPackedFastest) {          // neighbours write neighbouring pieces of the same packed rows
            ct = t / a.qtiles;
            qt = t - ct * a.qtiles;
        } else if (a.walk == kWalkMemoryFastest) {   // neighbours read neighbouring pieces of the same memory rows
            qt = t / a.ctiles;
            ct = t - qt * a.ctiles;
        } else {                                     // kWalkDiagonal: neighbours differ in both coordinates
            const uint32_t d = t / a.qtiles;
            qt = t - d * a.qtiles;
            ct = (d + qt) % a.ctiles;
        }
    }
    *b_out = b;
    *qt_out = qt;
    *ct_out = ct;
    return true;
}

// ---- 16-byte-per-lane variant for elements of 1, 2, 4 and 8 bytes ----
// A tile is TQ x TC elements with TQ * sizeof(T) == TC * sizeof(T) == 256 bytes, so that every
// row of the tile is a 256-byte run on BOTH HBM sides and every lane moves 16 bytes
// (E = 16 / sizeof(T) elements) per global access.  The tile sits in LDS as [q][c] with the
// 16-byte groups of a row permuted by XOR with (q / E) % 16:
//   * the side whose vectors run along c moves whole groups (ds_read/write_b128); the 16 lanes
//     that share a row cover its 16 groups, i.e. all banks, whatever the permutation;
//   * the side whose vectors run along q gathers / scatters E scalars per lane.  The 16 lanes
//     that share a column c touch rows q = E*qv + j, whose groups are displaced by qv: 16
//     different displacements, so together with the 4 neighbouring columns of a wavefront the
//     64 lanes fall into 64 different banks (4-byte elements; narrower ones share words in
//     pairs, which is a broadcast, not a conflict).
// Tiles are handed to workgroups so that each XCD (workgroup index mod 8) owns a contiguous
// range of the blocked walk: tiles whose 256-byte rows share a cache line when rows are not
// 256-byte aligned are then combined in one L2 instead of being written as partial lines from
// eight of them.
template <typename T, int THREADS, bool PACK, int ROWB = 256, bool STREAM = false>
__global__ __launch_bounds__(THREADS) void slice_transpose_vec_kernel(TransArgs a) {
    constexpr int E = 16 / sizeof(T);
    constexpr int TQ = ROWB / sizeof(T), TC = TQ;
    constexpr int G = TC / E;  // groups of 16 bytes per LDS row (16 for 256-byte rows)
    static_assert(G == ROWB / 16 && (G == 16 || G == 32), "a tile row is 256 or 512 bytes");
    __shared__ __attribute__((aligned(16))) T tile[TQ * TC];
    __shared__ uint64_t s_off[TQ];
    union Vec {
        u32x4 v;
        T e[E];
    };
    // LDS position of element (q, c)
    auto at = [](int q, int c) { return q * TC + (c ^ (E * ((q / E) % G))); };

    T* __restrict__ mem = reinterpret_cast<T*>(a.base) + a.offset;
    T* __restrict__ packed = reinterpret_cast<T*>(a.packed);
    uint64_t b;
    uint32_t qt, ct;
    if (!walk_tile(a, &b, &qt, &ct)) return;
    // A tile that would hang over the edge is moved back inside when the extent allows it: it
    // then overlaps its neighbour, and both write the same bytes to the overlap.
    uint32_t q0 = qt * TQ, c0 = ct * TC;
    if (q0 + TQ > a.Q && a.Q >= (uint32_t)TQ) q0 = a.Q - TQ;
    if (c0 + TC > a.Sc && a.Sc >= (uint32_t)TC) c0 = a.Sc - TC;
    uint64_t batch_off = 0;
    {
        uint64_t rem = b;
        for (int k = a.n_outer - 1; k >= 0; --k) {
            const uint64_t qd = rem / a.outer_size[k];
            batch_off += (rem - qd * a.outer_size[k]) * a.outer_stride[k];
            rem = qd;
        }
    }
    if (threadIdx.x < TQ) {
        uint32_t q = q0 + threadIdx.x;
        uint64_t off = 0;
        if (q < a.Q) {
            for (int k = a.n_inner - 1; k > 0; --k) {
                uint32_t qd, r;
                a.inner_div[k].divmod(q, qd, r);
                off += (uint64_t)r * a.inner_stride[k];
                q = qd;
            }
            off += (uint64_t)q * a.inner_stride[0];
        }
        s_off[threadIdx.x] = off;
    }
    __syncthreads();
    T* mem_tile = mem + batch_off + c0;                                        // + s_off[q] + c
    T* packed_tile = packed + (b * a.Sc + c0) * (uint64_t)a.Q + q0;            // + c * Q + q
    const bool full = q0 + TQ <= a.Q && c0 + TC <= a.Sc;
    const int v16 = threadIdx.x % G;  // which 16-byte vector of a row
    const int r16 = threadIdx.x / G;  // which row of a pass of ROWS rows
    constexpr int ROWS = THREADS / G;
    // The side whose vectors run along q: lane -> (vector qv of the column, column cc of pass p).  With 16
    // vectors per column a wavefront takes 16 vectors of 4 neighbouring columns, which is what makes its 64
    // scalar LDS accesses fall into 64 banks.  With 32 vectors per column (512-byte rows) the same shape is
    // kept - 16 vectors x 4 columns per wavefront, the two halves of a column going to neighbouring
    // wavefronts - instead of 32 vectors x 2 columns, which would fold onto half of the banks.
    const int qv = G == 16 ? v16 : (threadIdx.x % 16) + 16 * ((threadIdx.x / 64) % 2);
    const int cc0 = G == 16 ? r16 : 4 * (threadIdx.x / 128) + (threadIdx.x % 64) / 16;
    constexpr int CSTEP = G == 16 ? ROWS : 4 * (THREADS / 128);  // columns per pass
    if (full) {
        constexpr int PASSES = TQ / ROWS;
        Vec d[PASSES];
        if constexpr (PACK) {
#pragma unroll
            for (int p = 0; p < PASSES; ++p) {
                const int q = r16 + ROWS * p;
                d[p].v = tload<STREAM>(mem_tile + s_off[q] + v16 * E);
            }
#pragma unroll
            for (int p = 0; p < PASSES; ++p) {
                const int q = r16 + ROWS * p;
                *reinterpret_cast<u32x4*>(&tile[at(q, v16 * E)]) = d[p].v;
            }
            __syncthreads();
            if constexpr (sizeof(T) == 2) {
                // Two neighbouring columns at once: eight 32-bit LDS reads fetch (q, c) and (q, c+1) for
                // eight rows, and a 2x2 transpose in registers turns them into the two output vectors.
                // Half the LDS instructions of the element-wise form, and no sub-dword accesses.
#pragma unroll
                for (int p = 0; p < PASSES / 2; ++p) {
                    const int c = 2 * (cc0 + CSTEP * p);
                    uint32_t w[E];
#pragma unroll
                    for (int j = 0; j < E; ++j) w[j] = *reinterpret_cast<const uint32_t*>(&tile[at(qv * E + j, c)]);
                    u32x4 lo, hi;
#pragma unroll
                    for (int k = 0; k < 4; ++k) {
                        lo[k] = (w[2 * k] & 0xffffu) | (w[2 * k + 1] << 16);
                        hi[k] = (w[2 * k] >> 16) | (w[2 * k + 1] & 0xffff0000u);
                    }
                    tstore(packed_tile + (uint64_t)c * a.Q + qv * E, lo, a.aligned_stores);
                    tstore(packed_tile + (uint64_t)(c + 1) * a.Q + qv * E, hi, a.aligned_stores);
                }
            } else {
#pragma unroll
                for (int p = 0; p < PASSES; ++p) {
                    const int cc = cc0 + CSTEP * p;
                    Vec o;
#pragma unroll
                    for (int j = 0; j < E; ++j) o.e[j] = tile[at(qv * E + j, cc)];
                    tstore(packed_tile + (uint64_t)cc * a.Q + qv * E, o.v, a.aligned_stores);
                }
            }
        } else {
            if constexpr (sizeof(T) == 2) {
                // the mirror image: rows c and c+1 of the packed side are loaded together and their
                // halves interleaved into eight 32-bit LDS writes
#pragma unroll
                for (int p = 0; p < PASSES / 2; ++p) {
                    const int c = 2 * (cc0 + CSTEP * p);
                    d[2 * p].v = tload<STREAM>(packed_tile + (uint64_t)c * a.Q + qv * E);
                    d[2 * p + 1].v = tload<STREAM>(packed_tile + (uint64_t)(c + 1) * a.Q + qv * E);
                }
#pragma unroll
                for (int p = 0; p < PASSES / 2; ++p) {
                    const int c = 2 * (cc0 + CSTEP * p);
                    const u32x4 lo = d[2 * p].v, hi = d[2 * p + 1].v;
#pragma unroll
                    for (int k = 0; k < 4; ++k) {
                        const uint32_t w0 = (lo[k] & 0xffffu) | (hi[k] << 16);
                        const uint32_t w1 = (lo[k] >> 16) | (hi[k] & 0xffff0000u);
                        *reinterpret_cast<uint32_t*>(&tile[at(qv * E + 2 * k, c)]) = w0;
                        *reinterpret_cast<uint32_t*>(&tile[at(qv * E + 2 * k + 1, c)]) = w1;
                    }
                }
            } else {
#pragma unroll
                for (int p = 0; p < PASSES; ++p) {
                    const int cc = cc0 + CSTEP * p;
                    d[p].v = tload<STREAM>(packed_tile + (uint64_t)cc * a.Q + qv * E);
                }
#pragma unroll
                for (int p = 0; p < PASSES; ++p) {
                    const int cc = cc0 + CSTEP * p;
#pragma unroll
                    for (int j = 0; j < E; ++j) tile[at(qv * E + j, cc)] = d[p].e[j];
                }
            }
            __syncthreads();
#pragma unroll
            for (int p = 0; p < PASSES; ++p) {
                const int q = r16 + ROWS * p;
                const u32x4 o = *reinterpret_cast<const u32x4*>(&tile[at(q, v16 * E)]);
                tstore(mem_tile + s_off[q] + v16 * E, o, a.aligned_stores);
            }
        }
        return;
    }
    // Narrow extent (fewer than a tile's worth of q or of c): element by element through the same
    // LDS layout.  Loads are unconditional, from a clamped address, so that a batch of them is
    // in flight at once; only the stores are predicated.
    constexpr int BATCH = TQ * TC / THREADS < 8 ? TQ * TC / THREADS : 8;
    static_assert((TQ * TC) % (THREADS * BATCH) == 0, "whole batches");
    if constexpr (PACK) {
        for (int i0 = threadIdx.x; i0 < TQ * TC; i0 += THREADS * BATCH) {
            T v[BATCH];
#pragma unroll
            for (int k = 0; k < BATCH; ++k) {
                const int i = i0 + k * THREADS, q = i / TC, c = i % TC;
                const bool ok = q0 + q < a.Q && c0 + c < a.Sc;
                v[k] = mem_tile[ok ? s_off[q] + c : s_off[0]];
            }
#pragma unroll
            for (int k = 0; k < BATCH; ++k) {
                const int i = i0 + k * THREADS;
                tile[at(i / TC, i % TC)] = v[k];
            }
        }
        __syncthreads();
        for (int i = threadIdx.x; i < TQ * TC; i += THREADS) {
            const int c = i / TQ, q = i % TQ;
            if (q0 + q < a.Q && c0 + c < a.Sc) packed_tile[(uint64_t)c * a.Q + q] = tile[at(q, c)];
        }
    } else {
        for (int i0 = threadIdx.x; i0 < TQ * TC; i0 += THREADS * BATCH) {
            T v[BATCH];
#pragma unroll
            for (int k = 0; k < BATCH; ++k) {
                const int i = i0 + k * THREADS, c = i / TQ, q = i % TQ;
                const bool ok = q0 + q < a.Q && c0 + c < a.Sc;
                v[k] = packed_tile[ok ? (uint64_t)c * a.Q + q : 0];
            }
#pragma unroll
            for (int k = 0; k < BATCH; ++k) {
                const int i = i0 + k * THREADS;
                tile[at(i % TQ, i / TQ)] = v[k];
            }
        }
        __syncthreads();
        for (int i = threadIdx.x; i < TQ * TC; i += THREADS) {
            const int q = i / TC, c = i % TC;
            if (q0 + q < a.Q && c0 + c < a.Sc) mem_tile[s_off[q] + c] = tile[at(q, c)];
        }
    }
}

// ---- the same tile when the rows of the side that is WRITTEN do not start on cache lines ----
// With 256-byte tile rows cut at fixed element positions, a written row piece that starts inside a 128-byte line shares
// its first and last line with the neighbouring tiles, and such a line reaches HBM as two partial writes (bf16 8200^2:
// 0.42 of peak against 0.68 at 8064^2, whose rows are whole lines).  Here every written row gets its own window of the
// tile's TX positions, moved back by d_w < 128 / sizeof(T) elements so that it starts on a line: the windows of one row
// still tile the row (256 bytes are two lines, so d_w is the same in every tile), every vector store is aligned and
// every line is written whole by one workgroup, except at the two ends of a row.  The windows of a tile's rows start
// at different places, so the tile reads up to D more rows of the other side than it writes positions: TX + D rows go
// through LDS (the same XOR-permuted layout), the surplus coming out of L2, where the neighbouring tile has just put it.
// Both kernels in turn on one GPU, pack / unpack: bf16 8200^2 0.42 / 0.42 -> 0.58 / 0.585 of peak, 5000 x 7000
// 0.53 / 0.55 -> 0.69 / 0.70; fp32 0.53 / 0.54 -> 0.65 / 0.645 and 0.46 / 0.46 -> 0.61 / 0.60; f64 0.64 / 0.63 ->
// 0.67 / 0.67 and 0.60 / 0.58 -> 0.63 / 0.62.  Rows that do start on lines keep the kernel above.  Loads go through
// the cache at every size: streaming (nt) loads lose what the neighbouring tile left in L2 (bf16 5000 x 7000 0.70 -> 0.49).
// W is the index of a written row (c when packing, q when unpacking), X the position along it.
template <typename T, int THREADS, bool PACK>
__global__ __launch_bounds__(THREADS) void slice_transpose_lines_kernel(TransArgs a) {
    constexpr int ES = sizeof(T), E = 16 / ES;
    constexpr int TW = 256 / ES, TX = 256 / ES, D = 128 / ES, XR = TX + D;
    constexpr int ROWS = THREADS / 16;
    static_assert(XR <= THREADS && TW <= THREADS, "one lane per decoded row");
    __shared__ __attribute__((aligned(16))) T tile[XR * TW];  // [read row][written row]
    __shared__ uint64_t s_off[PACK ? XR : TW];
    union Vec {
        u32x4 v;
        T e[E];
    };
    // LDS position of (read row xr, written row wc): xr * TW + (wc ^ (E * ((xr / E) % 16)))

    uint64_t b;
    uint32_t qt, ct;
    if (!walk_tile(a, &b, &qt, &ct)) return;
    const uint32_t Wn = PACK ? a.Sc : a.Q, Xn = PACK ? a.Q : a.Sc;
    uint32_t w0 = (PACK ? ct : qt) * TW;
    if (w0 + TW > Wn) w0 = Wn - TW;  // the host sends extents of at least a tile; the overlap is written twice, same bytes
    const int64_t x0 = (int64_t)(PACK ? qt : ct) * TX;

    T* __restrict__ mem = reinterpret_cast<T*>(a.base) + a.offset;
    T* __restrict__ packed = reinterpret_cast<T*>(a.packed);
    uint64_t batch_off = 0;
    {
        uint64_t rem = b;
        for (int k = a.n_outer - 1; k >= 0; --k) {
            const uint64_t qd = rem / a.outer_size[k];
            batch_off += (rem - qd * a.outer_size[k]) * a.outer_stride[k];
            rem = qd;
        }
    }
    // memory offsets of the q rows this tile touches: the read rows when packing (clamped into the extent: what a
    // clamped row holds is never written), the written rows when unpacking
    if (threadIdx.x < (PACK ? XR : TW)) {
        int64_t qi = PACK ? x0 - D + (int64_t)threadIdx.x : (int64_t)w0 + threadIdx.x;
        if (qi < 0) qi = 0;
        if (qi > (int64_t)a.Q - 1) qi = (int64_t)a.Q - 1;
        uint32_t q = (uint32_t)qi;
        uint64_t off = 0;
        for (int k = a.n_inner - 1; k > 0; --k) {
            uint32_t qd, r;
            a.inner_div[k].divmod(q, qd, r);
            off += (uint64_t)r * a.inner_stride[k];
            q = qd;
        }
        off += (uint64_t)q * a.inner_stride[0];
        s_off[threadIdx.x] = off;
    }
    __syncthreads();

    // ---- read side -> LDS: rows x0 - D .. x0 + TX - 1, TW consecutive written-row indices of each ----
    const int v16 = threadIdx.x % 16, r16 = threadIdx.x / 16;
    constexpr int LPASSES = (XR + ROWS - 1) / ROWS;
    Vec d[LPASSES];
#pragma unroll
    for (int p = 0; p < LPASSES; ++p) {
        int xr = r16 + ROWS * p;
        if (xr > XR - 1) xr = XR - 1;  // surplus lanes of the last pass repeat its last row
        const T* src;
        if constexpr (PACK) {
            src = mem + batch_off + s_off[xr] + w0 + v16 * E;
        } else {
            int64_t c = x0 - D + xr;
            if (c < 0) c = 0;
            if (c > (int64_t)a.Sc - 1) c = (int64_t)a.Sc - 1;
            src = packed + (b * a.Sc + (uint64_t)c) * (uint64_t)a.Q + w0 + v16 * E;
        }
        d[p].v = tload<false>(src);
    }
#pragma unroll
    for (int p = 0; p < LPASSES; ++p) {
        const int xr = r16 + ROWS * p;
        if (xr < XR) *reinterpret_cast<u32x4*>(&tile[xr * TW + E * (v16 ^ ((xr / E) % 16))]) = d[p].v;
    }
    __syncthreads();

    // ---- LDS -> written side: row w takes positions x0 - d_w .. x0 - d_w + TX - 1, a window that starts on a line ----
    constexpr int WPASSES = TW / ROWS;
    static_assert(TW % ROWS == 0, "whole passes");
#pragma unroll
    for (int p = 0; p < WPASSES; ++p) {
        // The four written rows of a wavefront take elements that sit in four different 32-bit words of one 16-byte
        // group: each row reads its own LDS rows (its window starts at its own place), so rows whose elements share
        // a word would meet in one bank at different addresses.
        constexpr int S = ES >= 4 ? 1 : 4 / ES;
        const int logical = r16 + ROWS * p;
        const int in_block = logical % (4 * S);
        const int wr = logical - in_block + (in_block % 4) * S + in_block / 4;
        T* row;  // position 0 of the written row
        if constexpr (PACK) row = packed + (b * a.Sc + w0 + wr) * (uint64_t)a.Q;
        else row = mem + batch_off + s_off[wr];
        const int dw = (int)((((uintptr_t)row + (uint64_t)x0 * ES) & 127u) / ES);
        const int64_t xs = x0 - dw + v16 * E;  // first position of this lane's vector
        const int xr0 = D - dw + v16 * E;      // and the LDS row that holds it
        // The E rows xr0 .. xr0 + E - 1 lie in at most two groups of E rows, i.e. see two XOR permutations: one base
        // address for each, and a compare per element instead of the permutation's arithmetic (which is what made the
        // kernel ALU-bound for narrow elements: 8 or 16 elements per vector).
        const int first = E - xr0 % E;         // elements in the first group
        const int k0 = (xr0 / E) % 16, k1 = (xr0 / E + 1) % 16;
        const T* __restrict__ p0 = tile + xr0 * TW + (wr ^ (E * k0));
        const T* __restrict__ p1 = tile + xr0 * TW + (wr ^ (E * k1));
        Vec o;
#pragma unroll
        for (int j = 0; j < E; ++j) o.e[j] = (j < first ? p0 : p1)[j * TW];
        if (xs >= 0 && xs + E <= (int64_t)Xn) {
            tstore(row + xs, o.v, kStoreStreaming);
        } else {
#pragma unroll
            for (int j = 0; j < E; ++j)
                if (xs + j >= 0 && xs + j < (int64_t)Xn) row[xs + j] = o.e[j];
        }
    }
}

// ---- written rows that do not start on cache lines, narrow elements: a workgroup walks ALONG the written rows ----
// The windows of the kernel above start up to a line early, so a tile reads D = 128 / sizeof(T) more rows of the other side
// than it writes positions; for 1-byte elements that is 384 rows of 256 bytes per tile (96 KiB of LDS, half again the
// reads), and the kernel loses to the fixed tiles.  Here a workgroup owns a strip of TW written rows and a segment
// [xs, xe) of their positions and moves along it in chunks of CH = D positions: chunk k (CH rows of the read side, 256
// bytes of each) goes into one half of a two-chunk ring in LDS while the other half still holds chunk k - 1, and
// written row w takes positions xs + k CH - d_w .. + CH - 1 of it, one whole 128-byte line, d_w < D being what its
// address needs to start on a line.  The rows a window starts early by are the tail of the chunk before, which the
// ring still holds: the read side crosses L2 once per segment (plus D rows where a segment starts), every line of
// the written side is stored whole by one instruction, and the ring is 64 KiB for 1-byte elements.  The next chunk's
// loads are issued before the current chunk's windows are stored.  u8 8200^2, pack / unpack, both kernels in turn on one
// GPU: 0.44 / 0.46 of peak (fixed tiles) -> 0.50 / 0.50 rotating over 800 MB of buffers, 0.464 / 0.472 -> 0.589 / 0.566
// rotating over 400 MB (partly out of the 256 MB Infinity Cache, as when the neighbouring stage of a pipeline has just
// written or is about to read them).  2-byte elements gain 0.02 over the kernel above, 4- and 8-byte elements lose 0.03 to
// 0.05, so only 1-byte elements take it.  (What bounds all of these is the access pattern itself: with rows that are not
// whole lines, bare 256-byte reads run at 4.9 TB/s and line-by-line writes of rows a pitch apart at 5.4 TB/s, against
// 6.4 and 5.6 for aligned rows.)
// W is the index of a written row (c when packing, q when unpacking), X the position along it.
template <typename T, int THREADS, bool PACK>
__global__ __launch_bounds__(THREADS) void slice_transpose_strip_kernel(TransArgs a) {
    constexpr int ES = sizeof(T), E = 16 / ES;
    constexpr int TW = 256 / ES, CH = 128 / ES, RING = 2 * CH;
    constexpr int LP = CH * 16 / THREADS;  // load passes: CH rows x 16 vectors
    constexpr int SP = TW * 8 / THREADS;   // store passes: TW rows x 8 vectors (one line of each row)
    static_assert(LP >= 1 && SP >= 1 && (CH * 16) % THREADS == 0 && (TW * 8) % THREADS == 0, "whole passes");
    constexpr int LROWS = THREADS / 16, SROWS = THREADS / 8;
    __shared__ __attribute__((aligned(16))) T tile[RING * TW];  // [read row, modulo the ring][written row]
    union Vec {
        u32x4 v;
        T e[E];
    };

    // workgroup i runs on XCD i % 8: each XCD takes a contiguous eighth of the (batch, segment, strip) list, strips
    // fastest, so that the strips that read neighbouring pieces of the same rows run side by side in one L2
    const uint64_t wg = a.wg0 + blockIdx.x;
    const uint64_t id = (wg % 8) * ((a.ntiles + 7) / 8) + wg / 8;
    if (id >= a.ntiles) return;
    const uint64_t per_batch = (uint64_t)a.nseg * a.nstrips;
    const uint64_t b = id / per_batch;
    const uint32_t in_batch = (uint32_t)(id - b * per_batch);
    const uint32_t seg = in_batch / a.nstrips, sw = in_batch - seg * a.nstrips;
    const uint32_t Wn = PACK ? a.Sc : a.Q, Xn = PACK ? a.Q : a.Sc;
    uint32_t w0 = sw * TW;
    if (w0 + TW > Wn) w0 = Wn - TW;  // the host sends extents of at least a strip; the overlap is written twice, same bytes
    const uint32_t xs = seg * a.seg_len;
    const uint32_t xe = xs + a.seg_len < Xn ? xs + a.seg_len : Xn;
    const int K = (int)((xe - xs + CH - 1) / CH);
    // the last segment of a row also stores what lies behind its last whole window: the row's last d_w positions
    const int iters = K + (seg + 1 == a.nseg ? 1 : 0);

    T* __restrict__ mem = reinterpret_cast<T*>(a.base) + a.offset;
    T* __restrict__ packed = reinterpret_cast<T*>(a.packed);
    uint64_t batch_off = 0;
    {
        uint64_t rem = b;
        for (int k = a.n_outer - 1; k >= 0; --k) {
            const uint64_t qd = rem / a.outer_size[k];
            batch_off += (rem - qd * a.outer_size[k]) * a.outer_stride[k];
            rem = qd;
        }
    }
    auto q_offset = [&](uint32_t q) {  // memory offset of row q of the batch
        uint64_t off = 0;
        for (int k = a.n_inner - 1; k > 0; --k) {
            uint32_t qd, r;
            a.inner_div[k].divmod(q, qd, r);
            off += (uint64_t)r * a.inner_stride[k];
            q = qd;
        }
        return off + (uint64_t)q * a.inner_stride[0];
    };

    const int v16 = threadIdx.x % 16, r16 = threadIdx.x / 16;
    const int v8 = threadIdx.x % 8, r8 = threadIdx.x / 8;
    // chunk c = read rows xs + c CH .. + CH - 1, clamped into the extent (what a clamped row holds is never stored)
    auto load_chunk = [&](int c, Vec* d) {
#pragma unroll
        for (int p = 0; p < LP; ++p) {
            int64_t x = (int64_t)xs + (int64_t)c * CH + r16 + LROWS * p;
            x = x < 0 ? 0 : (x > (int64_t)Xn - 1 ? (int64_t)Xn - 1 : x);
            const T* src;
            if constexpr (PACK) src = mem + batch_off + q_offset((uint32_t)x) + w0 + v16 * E;
            else src = packed + (b * a.Sc + (uint64_t)x) * (uint64_t)a.Q + w0 + v16 * E;
            d[p].v = tload<false>(src);
        }
    };
    auto put_chunk = [&](int c, const Vec* d) {
#pragma unroll
        for (int p = 0; p < LP; ++p) {
            const int rr = ((c + 1) * CH + r16 + LROWS * p) & (RING - 1);
            *reinterpret_cast<u32x4*>(&tile[rr * TW + E * (v16 ^ ((rr / E) % 16))]) = d[p].v;
        }
    };

    // The written rows of this lane.  The eight rows of a wavefront take elements that sit in eight different 32-bit words:
    // each row reads its own LDS rows (its window starts at its own place), so rows whose elements share a word would meet
    // in one bank at different addresses.
    constexpr int S = ES >= 4 ? 1 : 4 / ES;
    int wr[SP], dws[SP];
    T* rowp[SP];
#pragma unroll
    for (int p = 0; p < SP; ++p) {
        const int logical = r8 + SROWS * p;
        const int in_block = logical % (8 * S);
        wr[p] = logical - in_block + (in_block % 8) * S + in_block / 8;
        if constexpr (PACK) rowp[p] = packed + (b * a.Sc + w0 + wr[p]) * (uint64_t)a.Q;
        else rowp[p] = mem + batch_off + q_offset(w0 + wr[p]);
        dws[p] = (int)(((uintptr_t)rowp[p] & 127u) / ES);  // xs is a multiple of CH, i.e. of a line
    }

    Vec d[LP];
    if (xs > 0) {
        load_chunk(-1, d);
        put_chunk(-1, d);
    }
    load_chunk(0, d);
    put_chunk(0, d);
    __syncthreads();
    for (int k = 0; k < iters; ++k) {
        const bool more = k + 1 < K;
        if (more) load_chunk(k + 1, d);
#pragma unroll
        for (int p = 0; p < SP; ++p) {
            const int t0 = (k + 1) * CH - dws[p] + v8 * E;  // the vector's first element, counted from the first row of chunk -1
            const int64_t xw = (int64_t)xs + (int64_t)k * CH - dws[p] + v8 * E;
            // its E rows lie in at most two groups of E ring rows, i.e. see two XOR permutations
            const int r0 = t0 & (RING - 1);
            const int g0 = r0 / E, g1 = (g0 + 1) % (RING / E);
            const int first = E - r0 % E;
            const T* __restrict__ p0 = tile + r0 * TW + (wr[p] ^ (E * (g0 % 16)));
            const T* __restrict__ p1 = tile + (g1 * E - first) * TW + (wr[p] ^ (E * (g1 % 16)));
            Vec o;
#pragma unroll
            for (int j = 0; j < E; ++j) o.e[j] = (j < first ? p0 : p1)[j * TW];
            if (xw >= 0 && xw + E <= (int64_t)Xn) {
                tstore(rowp[p] + xw, o.v, kStoreStreaming);
            } else {
#pragma unroll
                for (int j = 0; j < E; ++j)
                    if (xw + j >= 0 && xw + j < (int64_t)Xn) rowp[p][xw + j] = o.e[j];
            }
        }
        __syncthreads();  // every window of this step has been read: the older half of the ring is free
        if (more) put_chunk(k + 1, d);
        __syncthreads();
    }
}

// Cache policy of a launch, from an A/B over sixteen shapes, both directions and four element sizes (fractions of the
// HBM peak; "cached" = plain loads, write-through stores on aligned rows; the table is
// profiles/transpose_cache_policy_ab.md):
//   * stores of whole aligned 16-byte vectors stream (nt) at every element size: 1/2-byte elements 0.66 / 0.67 on
//     average against 0.61 / 0.61 cached, up to 0.2 higher (u8 8192^2 0.58 -> 0.77 / 0.81, bf16 6144^2 0.59 -> 0.80);
//   * loads stream as well once source and destination together no longer fit the 256 MiB Infinity Cache (packed
//     bytes >= 120 MiB): +0.01 to +0.03 there for every element size (bf16 8192^2 0.66 -> 0.68, fp32 8192^2 0.75 ->
//     0.78), while below that size streaming loads cost up to 0.17 (bf16 6144^2 0.80 -> 0.63, fp32 4096^2 0.81 ->
//     0.69, u8 8192^2 0.77 -> 0.66).
// Streaming stores of rows that are not 16-byte aligned write partial lines (u8 5000 x 7000: 0.57 -> 0.42), so rows like
// that keep going through the cache, which combines what neighbouring tiles share; streaming loads need both sides
// aligned for the same reason.
// With the tuning aids on (MONARCH_HIP_TUNING=1 when the library was loaded), MONARCH_HIP_TRANSPOSE_POLICY overrides the choice at every call: 0 cached loads + write-through /
// cached stores, 1 streaming loads + streaming stores, 2 streaming loads only, 3 streaming stores only.
static void choose_cache_policy(TransArgs* a, bool* stream_loads, uint64_t packed_bytes, bool stores_aligned, bool both_sides_aligned) {
    if (stores_aligned) a->aligned_stores = kStoreStreaming;
    if (both_sides_aligned && packed_bytes >= (120ull << 20)) *stream_loads = true;
    if (const char* e = tuning_env("MONARCH_HIP_TRANSPOSE_POLICY")) {
        const int p = std::atoi(e);
        *stream_loads = p == 1 || p == 2;
        a->aligned_stores = (p == 1 || p == 3) ? kStoreStreaming : stores_aligned ? kStoreWriteThrough : kStoreCached;
    }
}

// Which walk a launch takes.  Measured on MI355X over sixteen shapes, both directions and four element sizes, every
// variant switched in turn inside one process (the table is profiles/transpose_walk_ab.md):
//   * when every row pitch of both sides is a multiple of 4 KiB (power-of-two matrices and the like), the rows of a
//     tile all fall on the same few positions of HBM's address interleave, and so do the tiles of a block of the
//     blocked walk.  The diagonal walk - consecutive workgroups step one tile along q AND along c, no XCD ranges -
//     keeps the workgroups in flight spread over all positions on both sides: 1/2/4-byte elements +0.025 to +0.037
//     of peak on average over the shapes of that class (-0.05 to +0.12 on single shapes); 8-byte elements lose
//     0.03 with it and keep the blocked walk;
//   * at every other pitch the rows of a tile spread by themselves, neighbouring tiles share partial cache lines, and
//     the blocked XCD-contiguous walk wins (the diagonal one loses 0.02 to 0.10 there).
// With the tuning aids on, MONARCH_HIP_TRANSPOSE_WALK overrides the choice at every call (so that variants can be
// switched in turn inside one process): "<walk>[,<xcd_ranges>[,<group>[,<rotate>]]]" with walk 0 blocked,
// 1 packed side fastest, 2 memory side fastest, 3 diagonal.
static void choose_walk(TransArgs* a, uint32_t unit, uint64_t nbatch) {
    bool interleave_aligned = unit <= 4 && ((uint64_t)a->Q * unit) % 4096 == 0;
    for (int k = 0; interleave_aligned && k < a->n_inner; ++k)
        if ((a->inner_stride[k] * unit) % 4096 != 0) interleave_aligned = false;
    if (interleave_aligned) {
        a->walk = kWalkDiagonal;
        a->xcd_ranges = 0;
        a->rotate = 0;
    }
    if (const char* e = tuning_env("MONARCH_HIP_TRANSPOSE_WALK")) {
        unsigned walk = 0, ranges = 1, group = a->group, rotate = 0;
        const int n = std::sscanf(e, "%u,%u,%u,%u", &walk, &ranges, &group, &rotate);
        if (n >= 1 && walk <= kWalkDiagonal) {
            a->walk = walk;
            a->xcd_ranges = n >= 2 ? (ranges ? 1 : 0) : 1;
            a->rotate = n >= 4 ? (rotate ? 1 : 0) : 0;
        }
        if (n >= 3 && group >= 1 && group <= 64) {
            a->group = group;
            a->cgroups = (a->ctiles + group - 1) / group;
            a->qgroups = (a->qtiles + group - 1) / group;
            a->rows_per_eighth = (nbatch * a->qgroups + 7) / 8;
        }
    }
}

template <bool PACK>
bool try_transpose_copy(char* base, char* packed, const CanonSlice& c, uint32_t unit, hipStream_t stream, int* rc) {
    if (c.run != 1 || c.ndim < 2 || c.ndim > kMaxCanonDims) return false;
    int cd = -1;
    for (int k = 0; k < c.ndim; ++k)
        if (c.dims[k].stride == 1) cd = k;
    if (cd < 0 || cd == c.ndim - 1) return false;
    TransArgs a{};
    uint64_t Q = 1, nbatch = 1;
    for (int k = cd + 1; k < c.ndim; ++k) {
        if (c.dims[k].size >= kFastDivLimit) return false;
        Q *= c.dims[k].size;
        if (Q >= kFastDivLimit) return false;
        const int j = a.n_inner++;
        a.inner_size[j] = (uint32_t)c.dims[k].size;
        a.inner_div[j] = FastDiv32((uint32_t)c.dims[k].size);
        a.inner_stride[j] = c.dims[k].stride;
    }
    for (int k = 0; k < cd; ++k) {
        if (c.dims[k].size >= kFastDivLimit) return false;
        nbatch *= c.dims[k].size;
        const int j = a.n_outer++;
        a.outer_size[j] = (uint32_t)c.dims[k].size;
        a.outer_div[j] = FastDiv32((uint32_t)c.dims[k].size);
        a.outer_stride[j] = c.dims[k].stride;
    }
    const uint64_t Sc = c.dims[cd].size;
    // worth it only when both sides have something to coalesce
    if (Sc < 8 || Q < 8 || Sc >= kFastDivLimit) return false;
    const bool vec = unit <= 8;  // 16-byte elements already move 16 bytes per lane in the scalar kernel
    // 4-byte elements whose rows are 512-byte aligned on both sides and whose extents are whole tiles get 128 x 128
    // tiles (512-byte runs, 64 KiB of LDS, 1024 lanes): 8192^2 fp32 0.65 -> 0.70 of peak.  Rows that are not aligned
    // that way do better with the 64 x 64 tile (8200^2: 0.61 against 0.57).
    bool big = unit == 4 && Sc % 128 == 0 && Q % 128 == 0 && c.offset % 128 == 0 && nbatch * Sc * Q >= (1ull << 25) &&
               (((uintptr_t)base | (uintptr_t)packed) & 511u) == 0;
    for (int k = 0; big && k < c.ndim; ++k)
        if (k != cd && c.dims[k].stride % 128 != 0) big = false;
    // 2-byte elements get the 512-byte-row tile too (256 x 256 elements, 128 KiB of LDS, one workgroup per CU) where
    // 256-byte runs do worst: matrices of 120 MiB and more whose rows are multiples of 16 KiB apart on both sides
    // (every row of a tile then falls on the same position of HBM's address interleave, and a 512-byte run halves
    // the number of pieces that meet there).  bf16, same GPU, both tiles in turn: 8192^2 pack / unpack 0.68 / 0.68 ->
    // 0.71 / 0.735 of peak, 16384 x 8192 0.67 / 0.67 -> 0.70 / 0.745, 8192 x 16384 0.69 / 0.67 -> 0.75 / 0.77,
    // 8 x 2048 x 8192 0.70 / 0.69 -> 0.73 / 0.74.  Smaller matrices lose with it (6144^2 0.80 -> 0.73, 4096 x 8192
    // unpack 0.79 -> 0.70), other pitches gain or lose 0.01 (12288^2), so they keep the 128 x 128 tile.
    if (unit == 2) {
        big = Sc % 256 == 0 && Q % 8192 == 0 && c.offset % 256 == 0 && nbatch * Sc * Q * 2 >= (120ull << 20) &&
              (((uintptr_t)base | (uintptr_t)packed) & 511u) == 0;
        for (int k = 0; big && k < c.ndim; ++k)
            if (k != cd && c.dims[k].stride % 8192 != 0) big = false;
    }
    // 8-byte elements: 64 x 64 tiles (512-byte runs, 32 KiB of LDS) on aligned matrices of 2^24 elements and more, with
    // 512 lanes while the shorter of the two row lengths is at most 4096 elements and 1024 lanes beyond.  f64, sixteen
    // shapes, the three forms in turn on one GPU: 4096^2 pack / unpack 0.65 / 0.61 -> 0.73 / 0.69, four of them
    // 0.70 / 0.65 -> 0.785 / 0.78, 8192 x 4096 0.68 / 0.64 -> 0.74 / 0.71, 8192^2 0.73 / 0.69 -> 0.74 / 0.70,
    // 12288^2 0.69 / 0.645 -> 0.69 / 0.69; within 0.015 either way on the rest.
    uint32_t big8_lanes = 0;
    if (unit == 8) {
        big = Sc % 64 == 0 && Q % 64 == 0 && c.offset % 64 == 0 && nbatch * Sc * Q >= (1ull << 24) &&
              (((uintptr_t)base | (uintptr_t)packed) & 511u) == 0;
        for (int k = 0; big && k < c.ndim; ++k)
            if (k != cd && c.dims[k].stride % 64 != 0) big = false;
        if (big) {
            const uint64_t mem_row = a.inner_stride[a.n_inner - 1];  // elements between consecutive q
            big8_lanes = (Q < mem_row ? Q : mem_row) <= 4096 ? 512 : 1024;
        }
    }
    const uint32_t tile = vec ? (big ? 512 : 256) / unit : 32;
    // Written rows that do not start on cache lines take a kernel whose windows do: 2-, 4- and 8-byte elements the one
    // with a window per row of a tile (slice_transpose_lines_kernel; the extent along the written rows grows by the
    // most a window can start early), 1-byte elements the one that walks along the written rows
    // (slice_transpose_strip_kernel; with per-tile windows they lose, 8200^2 0.475 -> 0.36: 96 KiB of LDS, byte-wise LDS reads).
    // With the tuning aids on, MONARCH_HIP_TRANSPOSE_LINES overrides the choice at every call: 0 fixed tiles, 1 windows per
    // tile, 2 strips (1- and 2-byte elements).
    bool lines = false, strips = false;
    uint32_t seg_chunks = 2;
    if (vec && !big && (PACK ? Sc : Q) >= tile) {
        uint64_t written = PACK ? ((uint64_t)(uintptr_t)packed | Q * unit) : ((uint64_t)(uintptr_t)base + c.offset * unit);
        if (!PACK)
            for (int k = 0; k < c.ndim; ++k)
                if (k != cd) written |= c.dims[k].stride * unit;
        const bool inside_lines = (written & 127u) != 0;
        lines = inside_lines && unit >= 2;
        // strips need enough of them to fill the part: 1024 workgroups of segments of 2 chunks (u8 7000 x 5000, 560
        // workgroups: 0.44 / 0.40 of peak against 0.57 / 0.58 with the fixed tiles; 8200^2, 1089 workgroups, wins)
        const uint64_t Wn = PACK ? Sc : Q, Xn = PACK ? Q : Sc;
        strips = inside_lines && unit == 1 && nbatch * ((Wn + 255) / 256) * ((Xn + 255) / 256) >= 1024;
        if (const char* e = tuning_env("MONARCH_HIP_TRANSPOSE_LINES")) {
            int v = 0, chunks = 0;
            const int n = std::sscanf(e, "%d,%d", &v, &chunks);
            lines = n >= 1 && v == 1;
            strips = n >= 1 && v == 2 && unit <= 2;
            if (n >= 2 && chunks >= 1 && chunks <= 64) seg_chunks = (uint32_t)chunks;  // "2,<chunks per segment>"
        }
    }
    if (strips) {
        // Segments of 2 chunks (256 bytes of every written row).  1-byte elements 8200^2, pack, chunks per segment 1 / 2 / 3 / 4 /
        // 8 / 16: rotating over 800 MB of buffers 0.456 / 0.504 / 0.484 / 0.456 / 0.414 / 0.380 of peak (fixed tiles 0.44), over
        // 400 MB (partly out of the Infinity Cache) 0.545 / 0.589 / 0.609 / 0.552 (fixed tiles 0.464).  A segment re-reads the
        // D rows before its start, but the segment before it runs at the same time on the same XCD, so most of them come out
        // of L2: FETCH_SIZE reads 1.12 x the bytes read with 2 chunks, 1.25 x with 4; the fixed tiles read 1.08 x and write
        // 1.09 x (partial lines stored twice), the strips write 1.03 x (the two ends of every row).
        const uint32_t chunk = 128 / unit, rows_per_strip = 256 / unit;
        const uint64_t Wn = PACK ? Sc : Q, Xn = PACK ? Q : Sc;
        a.base = base;
        a.packed = packed;
        a.offset = c.offset;
        a.Sc = (uint32_t)Sc;
        a.Q = (uint32_t)Q;
        a.seg_len = seg_chunks * chunk;
        a.nseg = (uint32_t)((Xn + a.seg_len - 1) / a.seg_len);
        a.nstrips = (uint32_t)((Wn + rows_per_strip - 1) / rows_per_strip);
        a.ntiles = nbatch * a.nseg * a.nstrips;
        const uint64_t nblocks = 8 * ((a.ntiles + 7) / 8);
        *rc = launch_in_pieces(nblocks, 512, 8, [&](uint64_t wg0, uint32_t count) {
            a.wg0 = wg0;
            if (unit == 1) MHIP_LAUNCH((slice_transpose_strip_kernel<uint8_t, 512, PACK>), dim3(count), dim3(512), 0, stream, a);
            else MHIP_LAUNCH((slice_transpose_strip_kernel<uint16_t, 512, PACK>), dim3(count), dim3(512), 0, stream, a);
        });
        return true;
    }
    const uint32_t early = lines ? 128 / unit - 1 : 0;
    a.base = base;
    a.packed = packed;
    a.offset = c.offset;
    a.Sc = (uint32_t)Sc;
    a.Q = (uint32_t)Q;
    a.ctiles = (uint32_t)((Sc + (PACK ? 0 : early) + tile - 1) / tile);
    a.qtiles = (uint32_t)((Q + (PACK ? early : 0) + tile - 1) / tile);
    // Tiles are walked in group x group blocks, and a block is about what one XCD runs at a time
    // (8 workgroups per CU of 4-byte tiles, 4 of 2-byte tiles), so that the eight XCDs each stream
    // runs of group * 256 bytes on both sides.  Measured at 8192^2 fp32 pack: group 1 0.47, 4 0.52,
    // 16 0.65 of peak; 2-byte elements do best at 8.
    // 1-byte elements (256 x 256 tiles, two workgroups per CU) do best at 4: 8200^2 0.40 -> 0.47, 5000 x 7000 0.51 -> 0.57,
    // never lower than 8 on the shapes of the walk table.
    a.group = big ? (unit == 2 ? 4 : 8) : (unit == 4 || unit == 8) ? 16 : unit == 2 ? 8 : 4;
    // the kernel with line-aligned windows re-reads rows of the tile before it along the written rows, and finds them
    // in L2 sooner with smaller blocks: 4-byte elements 8200^2 0.66 / 0.65 -> 0.68 / 0.67, 8-byte 0.67 -> 0.69
    if (lines && unit >= 4) a.group = 4;
    a.cgroups = (a.ctiles + a.group - 1) / a.group;
    bool stream_loads = false;
    if (vec) {
        // 16-byte accesses land on 16-byte boundaries when the rows of that side do
        const uint64_t e16 = 16 / unit;  // elements per vector
        const bool packed_aligned = ((uintptr_t)packed & 15u) == 0 && Q % e16 == 0;
        bool memory_aligned = ((uintptr_t)base & 15u) == 0 && c.offset % e16 == 0 && Sc % e16 == 0;
        for (int k = 0; memory_aligned && k < c.ndim; ++k)
            if (k != cd && c.dims[k].stride % e16 != 0) memory_aligned = false;
        const bool stores_aligned = PACK ? packed_aligned : memory_aligned;
        a.aligned_stores = stores_aligned ? kStoreWriteThrough : kStoreCached;
        choose_cache_policy(&a, &stream_loads, nbatch * Sc * Q * unit, stores_aligned, packed_aligned && memory_aligned);
    }
    {
        // Rows that are a multiple of 8 KiB apart share at most two of the 64 positions at which HBM interleaves
        // 256-byte pieces (a bare walk down such rows reads 4.0 TB/s at a 16 KiB pitch against 6.4 TB/s at
        // 16 KiB + 256 B), and all rows of a tile are such rows.  The eight XCDs walk the same c-groups at the
        // same time, so together they would lean on an eighth of the memory; rotating the c-groups of each eighth
        // of the walk (= each XCD's share) by an eighth of their number spreads them out.  Measured over ten
        // power-of-two shapes from 4096^2 to 16384^2, both directions, switched on and off in turn on one GPU:
        // 2-byte elements +0.023 of peak on average (-0.01 to +0.09; four 4096^2 matrices 0.45 -> 0.54), 4-byte
        // elements +0.005 (-0.03 to +0.05), which is why only the narrow elements use it.  At other pitches the rows of a tile spread by themselves and a rotation
        // costs up to 0.08.  (When the packed side's rows are 4 KiB multiples as well, choose_walk replaces the blocked
        // walk by the diagonal one and this rotation does not apply.)
        bool camped = unit <= 2;
        for (int k = 0; camped && k < a.n_inner; ++k)
            if ((a.inner_stride[k] * unit) % 8192 != 0) camped = false;
        a.rotate = camped ? 1 : 0;
    }
    const uint64_t qgroups = (a.qtiles + a.group - 1) / a.group;
    a.qgroups = (uint32_t)qgroups;
    a.rows_per_eighth = (nbatch * qgroups + 7) / 8;
    a.walk = kWalkBlocked;
    a.xcd_ranges = 1;
    if (vec) choose_walk(&a, unit, nbatch);
    a.ntiles = a.walk == kWalkBlocked ? nbatch * a.cgroups * a.qgroups * a.group * a.group : nbatch * (uint64_t)a.qtiles * a.ctiles;
    if (vec) {
        const uint64_t nblocks = 8 * ((a.ntiles + 7) / 8);  // one tile per workgroup, eight XCD ranges
        const uint32_t lanes = unit == 8 ? (big ? big8_lanes : 256) : big ? 1024 : 512;
        *rc = launch_in_pieces(nblocks, lanes, 8, [&](uint64_t wg0, uint32_t count) {
            a.wg0 = wg0;
            const dim3 grid(count);
            if (lines) {
                switch (unit) {
                    case 1: MHIP_LAUNCH((slice_transpose_lines_kernel<uint8_t, 512, PACK>), grid, dim3(512), 0, stream, a); break;
                    case 2: MHIP_LAUNCH((slice_transpose_lines_kernel<uint16_t, 512, PACK>), grid, dim3(512), 0, stream, a); break;
                    case 4: MHIP_LAUNCH((slice_transpose_lines_kernel<uint32_t, 512, PACK>), grid, dim3(512), 0, stream, a); break;
                    default: MHIP_LAUNCH((slice_transpose_lines_kernel<uint64_t, 256, PACK>), grid, dim3(256), 0, stream, a); break;
                }
                return;
            }
            if (stream_loads) {
                switch (unit) {
                    case 1: MHIP_LAUNCH((slice_transpose_vec_kernel<uint8_t, 512, PACK, 256, true>), grid, dim3(512), 0, stream, a); break;
                    case 2:
                        if (big) MHIP_LAUNCH((slice_transpose_vec_kernel<uint16_t, 1024, PACK, 512, true>), grid, dim3(1024), 0, stream, a);
                        else MHIP_LAUNCH((slice_transpose_vec_kernel<uint16_t, 512, PACK, 256, true>), grid, dim3(512), 0, stream, a);
                        break;
                    case 4:
                        if (big) MHIP_LAUNCH((slice_transpose_vec_kernel<uint32_t, 1024, PACK, 512, true>), grid, dim3(1024), 0, stream, a);
                        else MHIP_LAUNCH((slice_transpose_vec_kernel<uint32_t, 512, PACK, 256, true>), grid, dim3(512), 0, stream, a);
                        break;
                    default:
                        if (big8_lanes == 1024) MHIP_LAUNCH((slice_transpose_vec_kernel<uint64_t, 1024, PACK, 512, true>), grid, dim3(1024), 0, stream, a);
                        else if (big8_lanes == 512) MHIP_LAUNCH((slice_transpose_vec_kernel<uint64_t, 512, PACK, 512, true>), grid, dim3(512), 0, stream, a);
                        else MHIP_LAUNCH((slice_transpose_vec_kernel<uint64_t, 256, PACK, 256, true>), grid, dim3(256), 0, stream, a);
                        break;
                }
                return;
            }
            switch (unit) {
                case 1: MHIP_LAUNCH((slice_transpose_vec_kernel<uint8_t, 512, PACK>), grid, dim3(512), 0, stream, a); break;
                case 2:
                    if (big) MHIP_LAUNCH((slice_transpose_vec_kernel<uint16_t, 1024, PACK, 512>), grid, dim3(1024), 0, stream, a);
                    else MHIP_LAUNCH((slice_transpose_vec_kernel<uint16_t, 512, PACK>), grid, dim3(512), 0, stream, a);
                    break;
                case 4:
                    if (big) MHIP_LAUNCH((slice_transpose_vec_kernel<uint32_t, 1024, PACK, 512>), grid, dim3(1024), 0, stream, a);
                    else MHIP_LAUNCH((slice_transpose_vec_kernel<uint32_t, 512, PACK>), grid, dim3(512), 0, stream, a);
                    break;
                default:
                    if (big8_lanes == 1024) MHIP_LAUNCH((slice_transpose_vec_kernel<uint64_t, 1024, PACK, 512>), grid, dim3(1024), 0, stream, a);
                    else if (big8_lanes == 512) MHIP_LAUNCH((slice_transpose_vec_kernel<uint64_t, 512, PACK, 512>), grid, dim3(512), 0, stream, a);
                    else MHIP_LAUNCH((slice_transpose_vec_kernel<uint64_t, 256, PACK>), grid, dim3(256), 0, stream, a);
                    break;
            }
        });
        return true;
    }
    if (unit != 16) return false;
    const uint64_t cap = max_workgroups(kThreads);  // grid-stride kernel
    MHIP_LAUNCH((slice_transpose_kernel<uint4, 32, PACK>), dim3((uint32_t)(a.ntiles < cap ? a.ntiles : cap)), dim3(kThreads), 0,
                       stream, a);
    *rc = launch_status();
    return true;
}

template bool try_transpose_copy<true>(char*, char*, const CanonSlice&, uint32_t, hipStream_t, int*);
template bool try_transpose_copy<false>(char*, char*, const CanonSlice&, uint32_t, hipStream_t, int*);

}  // namespace mhip
