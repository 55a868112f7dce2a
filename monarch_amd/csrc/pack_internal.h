// Declarations shared between the copy kernels' host code.
#pragma once
#include <hip/hip_runtime.h>

#include "mhip_internal.h"

namespace mhip {

// Launches the LDS-tiled transposing copy when the canonical slice calls for it (the
// memory-contiguous dimension is not the innermost iteration dimension).  Returns false
// when the direct chunk copy should be used instead; otherwise *rc holds the launch status.
template <bool PACK>
bool try_transpose_copy(char* base, char* packed, const CanonSlice& c, uint32_t unit, hipStream_t stream, int* rc);

}  // namespace mhip
