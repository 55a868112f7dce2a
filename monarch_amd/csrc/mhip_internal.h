// Internal declarations shared by the host-side sources of libmonarch_hip.so.
#pragma once
#include <cstdint>

#include "../../include/monarch_hip.h"
#include "fastdiv.h"

namespace mhip {

int validate_slice(const uint64_t* sizes, uint32_t nsizes, const uint64_t* strides, uint32_t nstrides);
uint64_t slice_len(const mhip_slice_t& s);
bool slice_fits_address_space(const mhip_slice_t& s, uint32_t elem_size);

// A Slice reduced to what a copy kernel needs.  Units are `unit` bytes.  Dimensions
// are in iteration order (outermost first); size-1 dimensions are dropped and
// neighbours that form one linear run are merged.  When `run` > 0 the innermost
// `run` units of every row are contiguous in the strided tensor as well, and dims[]
// holds only the dimensions OUTSIDE that run.
constexpr int kMaxCanonDims = 8;

struct CanonDim {
    uint64_t size;
    uint64_t stride;  // in units
};

struct CanonSlice {
    uint64_t offset = 0;  // units, relative to the base pointer
    uint64_t total = 0;   // units in the packed image
    uint64_t run = 1;     // contiguous units per row (>= 1)
    int ndim = 0;         // dimensions outside the run
    CanonDim dims[MHIP_MAX_DIMS + 1];
};

// Canonicalise `s` (elements of elem_size bytes) into unit-sized pieces.  `unit` is
// chosen as the largest power of two <= max_unit that divides the element size, every
// byte stride, the byte offset, and the alignments passed in `align_mask` (OR of the
// addresses involved).  Returns false for an empty slice.
// With `skew` the view's own byte offset does not limit the unit (for kernels whose accesses to the strided side
// tolerate any address): out->offset is rounded down to whole units and *skew receives the bytes left over, which the
// caller adds to the base pointer.
bool canonicalize(const mhip_slice_t& s, uint32_t elem_size, uint64_t align_mask, uint32_t max_unit,
                  CanonSlice* out, uint32_t* unit, uint64_t* skew = nullptr);

// Same dimension list for two canonical slices (offsets may differ).
bool same_shape(const CanonSlice& a, const CanonSlice& b);

// n <= kCopyManyMax contiguous copies of nbytes[g] bytes from src[g] to dst[g] in one launch on `stream` (a
// hipStream_t); src[g] may equal dst[g], other overlaps are not allowed.  Copies of no bytes are skipped.
constexpr int kCopyManyMax = 64;
int copy_many(void* const* dst, const void* const* src, const uint64_t* nbytes, uint32_t n, void* stream);

// Argument checks shared by the kernel-launching and the host forms of the mhip_rdmaxcel_* entry points
// (rdmaxcel_host.cpp): null and misaligned queue memory, queue sizes that are not powers of two, entry sizes.
int check_wqe(const mhip_wqe_params_t* p, bool send);
int check_cqe(const int32_t* result, const mhip_cqe_poll_params_t* p);
int check_ring(const void* dst, const void* src);

// Looks up, once per device, the address of the library's static scratch array on the CURRENT device (the block index
// of mhip_fp8_quantize_bucket_static).  Called from the set-up entry points so that the data path never does it.
int prepare_static_scratch();

}  // namespace mhip
