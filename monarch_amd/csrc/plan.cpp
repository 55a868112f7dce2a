// Host-side planning: turn a Slice into the few numbers a copy kernel needs.
#include <vector>

#include "mhip_internal.h"

namespace mhip {

static inline uint32_t pow2_factor(uint64_t v, uint32_t cap) {
    // largest power of two <= cap dividing v (v == 0 divides by everything)
    uint32_t u = cap;
    while (u > 1 && (v & (u - 1))) u >>= 1;
    return u;
}

bool canonicalize(const mhip_slice_t& s, uint32_t elem_size, uint64_t align_mask, uint32_t max_unit,
                  CanonSlice* out, uint32_t* unit, uint64_t* skew) {
    uint64_t len = 1;
    for (uint32_t k = 0; k < s.ndim; ++k) len *= s.sizes[k];
    if (len == 0 || elem_size == 0) return false;

    // (size, byte stride), outermost first; the element itself is the innermost dimension.
    std::vector<CanonDim> dims;
    dims.reserve(s.ndim + 1);
    for (uint32_t k = 0; k < s.ndim; ++k)
        if (s.sizes[k] > 1) dims.push_back({s.sizes[k], s.strides[k] * elem_size});
    if (elem_size > 1) dims.push_back({elem_size, 1});

    // Merge neighbours (outer, inner) that walk one linear run.
    std::vector<CanonDim> merged;
    for (const CanonDim& d : dims) {
        if (!merged.empty() && merged.back().stride == d.stride * d.size) {
            // previous (outer) dimension steps by exactly the extent of this one
            merged.back().size *= d.size;
            merged.back().stride = d.stride;
        } else {
            merged.push_back(d);
        }
    }

    uint64_t run_bytes = 1;
    if (!merged.empty() && merged.back().stride == 1) {
        run_bytes = merged.back().size;
        merged.pop_back();
    }

    uint64_t mask = align_mask | run_bytes | (skew ? 0 : s.offset * elem_size);
    for (const CanonDim& d : merged) mask |= d.stride;
    const uint32_t u = pow2_factor(mask, max_unit);

    out->offset = s.offset * elem_size / u;
    if (skew) *skew = s.offset * elem_size % u;
    out->total = len * elem_size / u;
    out->run = run_bytes / u;
    out->ndim = (int)merged.size();
    for (size_t k = 0; k < merged.size(); ++k) out->dims[k] = {merged[k].size, merged[k].stride / u};
    *unit = u;
    return true;
}

bool same_shape(const CanonSlice& a, const CanonSlice& b) {
    if (a.ndim != b.ndim || a.run != b.run || a.total != b.total) return false;
    for (int k = 0; k < a.ndim; ++k)
        if (a.dims[k].size != b.dims[k].size || a.dims[k].stride != b.dims[k].stride) return false;
    return true;
}

}  // namespace mhip
