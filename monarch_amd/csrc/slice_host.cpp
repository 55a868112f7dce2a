// Host-side Slice algebra, DeviceMesh membership and SendTensor routing behind the C ABI.
// Mirrors ndslice::Slice (ndslice/src/slice.rs), DeviceMesh (monarch_tensor_worker/src/device_mesh.rs),
// WorkerActor::send_tensor's rank pairing (monarch_tensor_worker/src/lib.rs:722-731) and Tensor.to_mesh's
// checks (python/monarch/common/tensor.py:417-438); pure integer work, no GPU calls.
#include <algorithm>
#include <cstring>
#include <numeric>
#include <utility>
#include <vector>

#include "mhip_internal.h"

namespace mhip {

// Slice::new, slice.rs:99-139.
int validate_slice(const uint64_t* sizes, uint32_t nsizes, const uint64_t* strides, uint32_t nstrides) {
    if (nsizes != nstrides) return MHIP_ERR_INVALID_DIMS;
    if (nsizes > MHIP_MAX_DIMS) return MHIP_ERR_INVALID_ARGUMENT;
    std::vector<std::pair<uint64_t, uint64_t>> dims(nsizes);  // (stride, size)
    for (uint32_t k = 0; k < nsizes; ++k) dims[k] = {strides[k], sizes[k]};
    std::sort(dims.begin(), dims.end());
    uint64_t space = 1;  // stride * size of the previous (smaller-stride) dimension
    for (size_t k = 0; k < dims.size(); ++k) {
        const auto [stride, size] = dims[k];
        if (k > 0) {
            const auto [pstride, psize] = dims[k - 1];
            if (stride % pstride != 0) return MHIP_ERR_NONRECTANGULAR_SHAPE;
            if (stride == pstride && size != 1 && psize != 1) return MHIP_ERR_NONUNIQUE_STRIDES;
        }
        if (space > stride) return MHIP_ERR_STRIDE_TOO_SMALL;
        // The reference computes stride * size in usize (wrapping in release builds, panicking in
        // debug builds); a product that does not fit cannot describe addressable memory, so it is
        // refused here.
        if (__builtin_mul_overflow(stride, size, &space)) return MHIP_ERR_INVALID_ARGUMENT;
    }
    return MHIP_SUCCESS;
}

// True when offset + sum((size-1)*stride) + 1, times elem_size, fits in 63 bits: every byte
// address the slice can produce is then representable.
bool slice_fits_address_space(const mhip_slice_t& s, uint32_t elem_size) {
    uint64_t hi = s.offset;
    for (uint32_t k = 0; k < s.ndim; ++k) {
        if (s.sizes[k] == 0) return true;  // empty: nothing is addressed
        uint64_t ext;
        if (__builtin_mul_overflow(s.sizes[k] - 1, s.strides[k], &ext)) return false;
        if (__builtin_add_overflow(hi, ext, &hi)) return false;
    }
    uint64_t bytes;
    if (__builtin_add_overflow(hi, (uint64_t)1, &hi)) return false;
    if (__builtin_mul_overflow(hi, (uint64_t)elem_size, &bytes)) return false;
    uint64_t len = 1;
    for (uint32_t k = 0; k < s.ndim; ++k)
        if (__builtin_mul_overflow(len, s.sizes[k], &len)) return false;
    uint64_t packed;
    if (__builtin_mul_overflow(len, (uint64_t)elem_size, &packed)) return false;
    return bytes < (1ull << 63) && packed < (1ull << 63);
}

static inline bool bad(const mhip_slice_t* s) {
    return s == nullptr || s->ndim > MHIP_MAX_DIMS || (s->ndim > 0 && (!s->sizes || !s->strides));
}

uint64_t slice_len(const mhip_slice_t& s) {
    uint64_t n = 1;
    for (uint32_t k = 0; k < s.ndim; ++k) n *= s.sizes[k];
    return n;
}

// Row-major rank -> coordinates (CartesianIterator::next, slice.rs:764-781).
static void unravel(const uint64_t* sizes, uint32_t ndim, uint64_t index, uint64_t* coord) {
    for (uint32_t k = ndim; k-- > 0;) {
        coord[k] = index % sizes[k];
        index /= sizes[k];
    }
}

static uint64_t dot(const uint64_t* a, const uint64_t* b, uint32_t n) {
    uint64_t acc = 0;
    for (uint32_t k = 0; k < n; ++k) acc += a[k] * b[k];
    return acc;
}

// Slice::coordinates, slice.rs:347-374.
static int coordinates(const mhip_slice_t& s, uint64_t value, uint64_t* out) {
    if (value < s.offset) return MHIP_ERR_VALUE_NOT_IN_SLICE;
    uint64_t pos = value - s.offset;
    uint32_t order[MHIP_MAX_DIMS];
    std::iota(order, order + s.ndim, 0u);
    std::stable_sort(order, order + s.ndim,
                     [&](uint32_t a, uint32_t b) { return s.strides[a] < s.strides[b]; });
    for (uint32_t r = s.ndim; r-- > 0;) {
        const uint32_t d = order[r];
        uint64_t c = 0;
        if (s.sizes[d] > 1) {
            // Slice::new never yields a zero stride on a dimension longer than 1; a caller-built struct can
            if (s.strides[d] == 0) return MHIP_ERR_INVALID_ARGUMENT;
            c = pos / s.strides[d];
            pos %= s.strides[d];
        }
        if (c >= s.sizes[d]) return MHIP_ERR_VALUE_NOT_IN_SLICE;
        out[d] = c;
    }
    return pos == 0 ? MHIP_SUCCESS : MHIP_ERR_VALUE_NOT_IN_SLICE;
}

}  // namespace mhip

using namespace mhip;

extern "C" {

int mhip_slice_validate(uint64_t, const uint64_t* sizes, uint32_t nsizes, const uint64_t* strides,
                        uint32_t nstrides) {
    if ((nsizes && !sizes) || (nstrides && !strides)) return MHIP_ERR_INVALID_ARGUMENT;
    return validate_slice(sizes, nsizes, strides, nstrides);
}

int mhip_slice_len(const mhip_slice_t* s, uint64_t* len) {
    if (bad(s) || !len) return MHIP_ERR_INVALID_ARGUMENT;
    *len = slice_len(*s);
    return MHIP_SUCCESS;
}

int mhip_slice_is_contiguous(const mhip_slice_t* s, int* result) {
    if (bad(s) || !result) return MHIP_ERR_INVALID_ARGUMENT;
    uint64_t expect = 1;
    *result = 1;
    for (uint32_t k = s->ndim; k-- > 0;) {
        if (s->strides[k] != expect) {
            *result = 0;
            break;
        }
        expect *= s->sizes[k];
    }
    return MHIP_SUCCESS;
}

int mhip_slice_get(const mhip_slice_t* s, uint64_t index, uint64_t* loc) {
    if (bad(s) || !loc) return MHIP_ERR_INVALID_ARGUMENT;
    // slice.rs:523-537; an empty slice has no valid index (the reference would divide by zero).
    if (index >= slice_len(*s)) return MHIP_ERR_INDEX_OUT_OF_RANGE;
    uint64_t coord[MHIP_MAX_DIMS];
    unravel(s->sizes, s->ndim, index, coord);
    *loc = s->offset + dot(coord, s->strides, s->ndim);
    return MHIP_SUCCESS;
}

int mhip_slice_location(const mhip_slice_t* s, const uint64_t* coord, uint32_t ncoord, uint64_t* loc) {
    if (bad(s) || !loc || (ncoord && !coord)) return MHIP_ERR_INVALID_ARGUMENT;
    if (ncoord != s->ndim) return MHIP_ERR_INVALID_DIMS;
    *loc = s->offset + dot(coord, s->strides, s->ndim);
    return MHIP_SUCCESS;
}

int mhip_slice_coordinates(const mhip_slice_t* s, uint64_t value, uint64_t* coords) {
    if (bad(s) || (s->ndim && !coords)) return MHIP_ERR_INVALID_ARGUMENT;
    return coordinates(*s, value, coords);
}

int mhip_slice_index(const mhip_slice_t* s, uint64_t value, uint64_t* index) {
    if (bad(s) || !index) return MHIP_ERR_INVALID_ARGUMENT;
    uint64_t coord[MHIP_MAX_DIMS];
    if (int rc = coordinates(*s, value, coord)) return rc;
    uint64_t rank = 0;
    for (uint32_t k = 0; k < s->ndim; ++k) rank = rank * s->sizes[k] + coord[k];  // slice.rs:460-471
    *index = rank;
    return MHIP_SUCCESS;
}

int mhip_slice_iter(const mhip_slice_t* s, uint64_t start, uint64_t count, uint64_t* locs,
                    uint64_t* written) {
    if (bad(s) || !written || (count && !locs)) return MHIP_ERR_INVALID_ARGUMENT;
    const uint64_t len = slice_len(*s);
    uint64_t n = 0;
    if (start < len) {
        // odometer walk: same order as CartesianIterator, without a div/mod per item
        uint64_t coord[MHIP_MAX_DIMS];
        unravel(s->sizes, s->ndim, start, coord);
        uint64_t loc = s->offset + dot(coord, s->strides, s->ndim);
        const uint64_t stop = start + std::min(count, len - start);  // start + count may not fit 64 bits
        for (uint64_t i = start; i < stop; ++i) {
            locs[n++] = loc;
            for (uint32_t k = s->ndim; k-- > 0;) {
                if (++coord[k] < s->sizes[k]) {
                    loc += s->strides[k];
                    break;
                }
                loc -= (s->sizes[k] - 1) * s->strides[k];
                coord[k] = 0;
            }
        }
    }
    *written = n;
    return MHIP_SUCCESS;
}

int mhip_slice_select(const mhip_slice_t* s, uint32_t dim, uint64_t begin, uint64_t end, uint64_t step,
                      uint64_t* out_offset, uint64_t* out_sizes, uint64_t* out_strides) {
    if (bad(s) || !out_offset || !out_sizes || !out_strides || step == 0) return MHIP_ERR_INVALID_ARGUMENT;
    if (dim >= s->ndim) return MHIP_ERR_INDEX_OUT_OF_RANGE;           // slice.rs:298-303
    if (begin >= s->sizes[dim]) return MHIP_ERR_INDEX_OUT_OF_RANGE;   // :304-309
    if (end <= begin) return MHIP_ERR_EMPTY_RANGE;                    // :310-312
    std::copy(s->sizes, s->sizes + s->ndim, out_sizes);
    std::copy(s->strides, s->strides + s->ndim, out_strides);
    *out_offset = s->offset + begin * s->strides[dim];
    const uint64_t span = end - begin;
    out_sizes[dim] = span / step + (span % step != 0);
    out_strides[dim] = s->strides[dim] * step;
    return validate_slice(out_sizes, s->ndim, out_strides, s->ndim);  // :325
}

int mhip_slice_at(const mhip_slice_t* s, uint32_t dim, uint64_t index, uint64_t* out_offset,
                  uint64_t* out_sizes, uint64_t* out_strides) {
    if (bad(s) || !out_offset) return MHIP_ERR_INVALID_ARGUMENT;
    if (dim >= s->ndim) return MHIP_ERR_DIMENSION_OUT_OF_RANGE;       // slice.rs:244-249
    if (index >= s->sizes[dim]) return MHIP_ERR_INDEX_OUT_OF_RANGE;   // :250-255
    if (s->ndim > 1 && (!out_sizes || !out_strides)) return MHIP_ERR_INVALID_ARGUMENT;
    *out_offset = s->offset + index * s->strides[dim];
    for (uint32_t k = 0, j = 0; k < s->ndim; ++k) {
        if (k == dim) continue;
        out_sizes[j] = s->sizes[k];
        out_strides[j++] = s->strides[k];
    }
    return validate_slice(out_sizes, s->ndim - 1, out_strides, s->ndim - 1);  // :262
}

int mhip_slice_subview(const mhip_slice_t* s, const uint64_t* starts, uint32_t nstarts,
                       const uint64_t* lens, uint32_t nlens, uint64_t* out_offset) {
    if (bad(s) || !out_offset || (nstarts && !starts) || (nlens && !lens)) return MHIP_ERR_INVALID_ARGUMENT;
    if (nstarts != s->ndim || nlens != s->ndim) return MHIP_ERR_INVALID_DIMS;
    for (uint32_t d = 0; d < s->ndim; ++d)
        if (starts[d] > s->sizes[d] || lens[d] > s->sizes[d] - starts[d]) return MHIP_ERR_INDEX_OUT_OF_RANGE;  // no wrap
    *out_offset = s->offset + dot(starts, s->strides, s->ndim);
    return MHIP_SUCCESS;
}

int mhip_slice_view(const mhip_slice_t* s, const uint64_t* new_sizes, uint32_t nnew, uint64_t* out_strides) {
    if (bad(s) || nnew > MHIP_MAX_DIMS || (nnew && (!new_sizes || !out_strides))) return MHIP_ERR_INVALID_ARGUMENT;
    uint64_t want = 1;
    for (uint32_t k = 0; k < nnew; ++k)
        if (__builtin_mul_overflow(want, new_sizes[k], &want)) return MHIP_ERR_INCOMPATIBLE_VIEW;  // no slice holds 2^64 elements
    if (want != slice_len(*s) || s->offset != 0) return MHIP_ERR_INCOMPATIBLE_VIEW;  // slice.rs:594-606
    uint64_t acc = 1;
    for (uint32_t k = nnew; k-- > 0;) {
        out_strides[k] = acc;
        acc *= new_sizes[k];
    }
    // The new view is dense row-major from 0, so it addresses exactly [0, want); each of
    // those offsets has to be a member of the base (slice.rs:613-628).
    uint64_t scratch[MHIP_MAX_DIMS];
    for (uint64_t off = 0; off < want; ++off)
        if (coordinates(*s, off, scratch) != MHIP_SUCCESS) return MHIP_ERR_INCOMPATIBLE_VIEW;
    return MHIP_SUCCESS;
}

int mhip_slice_enforce_embedding(const mhip_slice_t* s, const mhip_slice_t* other) {
    if (bad(s) || bad(other)) return MHIP_ERR_INVALID_ARGUMENT;
    const uint64_t len = slice_len(*s);
    uint64_t scratch[MHIP_MAX_DIMS];
    const uint64_t chunk = 1024;
    std::vector<uint64_t> locs(chunk);
    for (uint64_t start = 0; start < len; start += chunk) {
        uint64_t n = 0;
        mhip_slice_iter(s, start, chunk, locs.data(), &n);
        for (uint64_t i = 0; i < n; ++i)
            if (int rc = coordinates(*other, locs[i], scratch)) return rc;
    }
    return MHIP_SUCCESS;
}

int mhip_slice_bounds(const mhip_slice_t* s, uint64_t* min_loc, uint64_t* max_loc) {
    if (bad(s) || !min_loc || !max_loc) return MHIP_ERR_INVALID_ARGUMENT;
    if (slice_len(*s) == 0) return MHIP_ERR_INVALID_ARGUMENT;
    uint64_t hi = s->offset;
    for (uint32_t k = 0; k < s->ndim; ++k) hi += (s->sizes[k] - 1) * s->strides[k];
    *min_loc = s->offset;
    *max_loc = hi;
    return MHIP_SUCCESS;
}

int mhip_mesh_dim_members(const mhip_slice_t* ranks, uint64_t rank, uint32_t dim, uint64_t* members,
                          uint64_t* dim_rank) {
    if (bad(ranks) || !members || !dim_rank) return MHIP_ERR_INVALID_ARGUMENT;
    if (dim >= ranks->ndim) return MHIP_ERR_DIMENSION_OUT_OF_RANGE;
    uint64_t coord[MHIP_MAX_DIMS];
    if (int rc = coordinates(*ranks, rank, coord)) return rc;
    // device_mesh.rs:84-85: walk the dimension from the member with coordinate 0
    const uint64_t stride = ranks->strides[dim];
    uint64_t m = rank - stride * coord[dim];
    for (uint64_t i = 0; i < ranks->sizes[dim]; ++i, m += stride) members[i] = m;
    *dim_rank = coord[dim];
    return MHIP_SUCCESS;
}

int mhip_mesh_ranks_for_dims(const mhip_slice_t* ranks, uint64_t rank, const uint32_t* dims,
                             uint32_t ndims, uint64_t* out, uint64_t cap, uint64_t* count) {
    if (bad(ranks) || !count || (ndims && !dims) || ndims > MHIP_MAX_DIMS) return MHIP_ERR_INVALID_ARGUMENT;
    *count = 0;
    if (ndims == 0) return MHIP_SUCCESS;  // device_mesh.rs:122-124
    uint64_t coord[MHIP_MAX_DIMS];
    if (int rc = coordinates(*ranks, rank, coord)) return rc;
    uint64_t sub_sizes[MHIP_MAX_DIMS], sub_strides[MHIP_MAX_DIMS];
    uint64_t total = 1, origin = rank;
    for (uint32_t d = 0; d < ndims; ++d) {
        if (dims[d] >= ranks->ndim) return MHIP_ERR_DIMENSION_OUT_OF_RANGE;
        sub_sizes[d] = ranks->sizes[dims[d]];
        // a one-member dimension contributes stride 0 (device_mesh.rs:148-154)
        sub_strides[d] = sub_sizes[d] > 1 ? ranks->strides[dims[d]] : 0;
        origin -= sub_strides[d] * coord[dims[d]];
        // a dimension named twice can make the product wrap: such a group fits no buffer
        if (__builtin_mul_overflow(total, sub_sizes[d], &total)) return MHIP_ERR_INVALID_ARGUMENT;
    }
    if (total > cap || (total && !out)) return MHIP_ERR_INVALID_ARGUMENT;
    const mhip_slice_t group{origin, ndims, sub_sizes, sub_strides};
    uint64_t n = 0;
    mhip_slice_iter(&group, 0, total, out, &n);
    *count = n;
    return MHIP_SUCCESS;
}

int mhip_send_tensor_route(const mhip_slice_t* from_ranks, const mhip_slice_t* to_ranks, uint64_t rank,
                           uint64_t* from_rank, uint64_t* to_rank) {
    if (bad(from_ranks) || bad(to_ranks) || !from_rank || !to_rank) return MHIP_ERR_INVALID_ARGUMENT;
    // lib.rs:722-731: the i-th sender pairs with the i-th receiver; a rank outside a slice, or an index
    // past the other slice's length, leaves that side empty
    auto pair = [rank](const mhip_slice_t* mine, const mhip_slice_t* other) -> uint64_t {
        uint64_t index = 0, peer = 0;
        if (mhip_slice_index(mine, rank, &index) != MHIP_SUCCESS) return MHIP_NO_RANK;
        if (mhip_slice_get(other, index, &peer) != MHIP_SUCCESS) return MHIP_NO_RANK;
        return peer;
    };
    *to_rank = pair(from_ranks, to_ranks);
    *from_rank = pair(to_ranks, from_ranks);
    return MHIP_SUCCESS;
}

int mhip_to_mesh_from_ranks(const char* const* slicing_names, const mhip_slice_t* slicing,
                            const char* const* mesh_names, const uint64_t* mesh_sizes, uint32_t mesh_ndim,
                            uint64_t* out_sizes, uint64_t* out_strides, uint32_t* out_ndim,
                            uint32_t* broadcast_dims, uint32_t* n_broadcast, uint32_t* culprit) {
    if (bad(slicing) || !out_ndim || !n_broadcast || mesh_ndim > MHIP_MAX_DIMS) return MHIP_ERR_INVALID_ARGUMENT;
    if ((slicing->ndim && (!slicing_names || !out_sizes || !out_strides)) ||
        (mesh_ndim && (!mesh_names || !mesh_sizes || !broadcast_dims)))
        return MHIP_ERR_INVALID_ARGUMENT;
    uint32_t kept = 0, bcast = 0;
    // tensor.py:417-433: walk the destination mesh's dimensions in its order
    for (uint32_t m = 0; m < mesh_ndim; ++m) {
        uint32_t index = slicing->ndim;
        for (uint32_t k = 0; k < slicing->ndim; ++k)
            if (std::strcmp(slicing_names[k], mesh_names[m]) == 0) { index = k; break; }  // list.index: first match
        if (index == slicing->ndim) {
            broadcast_dims[bcast++] = m;
            continue;
        }
        if (slicing->sizes[index] != mesh_sizes[m]) {
            if (culprit) *culprit = m;
            return MHIP_ERR_MESH_DIM_LENGTH_MISMATCH;
        }
        if (kept == slicing->ndim) return MHIP_ERR_INVALID_ARGUMENT;  // a name repeated in the destination mesh
        out_sizes[kept] = mesh_sizes[m];
        out_strides[kept++] = slicing->strides[index];
    }
    if (kept != slicing->ndim) {  // tensor.py:435-437
        if (culprit) {
            for (uint32_t k = 0; k < slicing->ndim; ++k) {
                bool found = false;
                for (uint32_t m = 0; m < mesh_ndim; ++m) found = found || std::strcmp(slicing_names[k], mesh_names[m]) == 0;
                if (!found) { *culprit = k; break; }
            }
        }
        return MHIP_ERR_MESH_DIM_MISSING;
    }
    *out_ndim = kept;
    *n_broadcast = bcast;
    return MHIP_SUCCESS;
}

}  // extern "C"
