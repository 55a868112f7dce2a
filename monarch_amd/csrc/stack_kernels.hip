// Reduction::Stack on the chunks one GPU holds: the data movement of all_gather_into_tensor
// (monarch_tensor_worker/src/stream.rs:1408-1417) and of all_to_all_single (stream.rs:1381-1399,
// torch-sys-cuda/src/nccl.rs:760-812) as one launch over all members.
//
// HBM-bound, 2 bytes of traffic per byte stacked.  Every member contributes one contiguous chunk that
// lands at chunk index g of the output, so the launch is n contiguous copies side by side: single-wavefront
// workgroups, one 16-byte vector per lane, non-temporal loads, like the contiguous copy of the pack path.
#include "mhip_device.h"

namespace mhip {

constexpr int kStackInputs = 64;
constexpr int kStackThreads = 64;

struct StackArgs {
    char* out;
    const char* in[kStackInputs];  // start of the chunk member g contributes
    uint64_t chunk_bytes;
    uint64_t tiles;                // workgroups per chunk
    uint64_t wg0;                  // workgroups of this call launched before this grid
    uint32_t aligned;              // every vector of every chunk is 16-byte aligned on both sides
};

__global__ __launch_bounds__(kStackThreads) void stack_copy_kernel(StackArgs a) {
    const uint64_t wg = a.wg0 + blockIdx.x;
    const uint64_t g = wg / a.tiles;           // chunks are the slow index: neighbours write neighbouring memory
    const uint64_t tile = wg - g * a.tiles;
    const char* src = a.in[g];   // may be the output itself (in-place all_to_all): no restrict
    char* dst = a.out + g * a.chunk_bytes;
    const uint64_t nvec = a.chunk_bytes / 16;
    const uint64_t v = tile * kStackThreads + threadIdx.x;
    if (v < nvec) {
        if (a.aligned) store16_writethrough(dst + v * 16, load16_aligned(src + v * 16));
        else store16_unaligned(dst + v * 16, load16_unaligned(src + v * 16));
    }
    if (tile == 0) {  // the chunk's last bytes, fewer than 16
        const uint64_t i = nvec * 16 + threadIdx.x;
        if (i < a.chunk_bytes) dst[i] = src[i];
    }
}

static int stack_entry(void* out, const void* const* in, uint32_t n, uint64_t src_offset_bytes, uint64_t chunk_bytes,
                       uint32_t elem_size, mhip_stream_t stream) {
    if (chunk_bytes == 0) return MHIP_SUCCESS;
    if (!out) return MHIP_ERR_UNDEFINED_TENSOR;
    StackArgs a{};
    a.out = static_cast<char*>(out);
    a.chunk_bytes = chunk_bytes;
    uintptr_t mask = (uintptr_t)out | chunk_bytes;
    for (uint32_t g = 0; g < n; ++g) {
        if (!in[g]) return MHIP_ERR_UNDEFINED_TENSOR;
        a.in[g] = static_cast<const char*>(in[g]) + src_offset_bytes;
        mask |= (uintptr_t)a.in[g];
    }
    const uint32_t pow2 = elem_size & (0u - elem_size);  // largest power of two dividing the element size
    if (mask & ((pow2 < 16 ? pow2 : 16u) - 1)) return MHIP_ERR_INVALID_ARGUMENT;  // not even element-aligned
    a.aligned = (mask & 15u) == 0;
    const uint64_t nvec = chunk_bytes / 16;
    a.tiles = nvec ? (nvec + kStackThreads - 1) / kStackThreads : 1;
    hipStream_t hs = static_cast<hipStream_t>(stream);
    DeviceGuard guard(hs);
    return launch_in_pieces(a.tiles * n, kStackThreads, 1, [&](uint64_t wg0, uint32_t count) {
        a.wg0 = wg0;
        MHIP_LAUNCH(stack_copy_kernel, dim3(count), dim3(kStackThreads), 0, hs, a);
    });
}

static int check_stack_args(const void* const* in, uint32_t n, uint32_t elem_size) {
    if (!in || n == 0 || elem_size == 0) return MHIP_ERR_INVALID_ARGUMENT;
    if (n > (uint32_t)kStackInputs) return MHIP_ERR_TOO_MANY_INPUTS;
    return MHIP_SUCCESS;
}

}  // namespace mhip

using namespace mhip;

extern "C" {

int mhip_stack(void* out, const void* const* in, uint32_t n, uint64_t numel, uint32_t elem_size, mhip_stream_t stream) {
    if (int rc = check_stack_args(in, n, elem_size)) return rc;
    uint64_t bytes;
    if (__builtin_mul_overflow(numel, (uint64_t)elem_size, &bytes) || bytes >= (1ull << 56)) return MHIP_ERR_INVALID_ARGUMENT;
    return stack_entry(out, in, n, 0, bytes, elem_size, stream);
}

int mhip_stack_scatter(void* out, const void* const* in, uint32_t n, uint32_t rank, uint64_t numel, uint32_t elem_size,
                       mhip_stream_t stream) {
    if (int rc = check_stack_args(in, n, elem_size)) return rc;
    if (rank >= n) return MHIP_ERR_INDEX_OUT_OF_RANGE;
    // all_to_all_single cuts each tensor into world_size chunks of numel / world_size elements (nccl.rs:780-781)
    if (numel % n != 0) return MHIP_ERR_INPUT_SIZE_MISMATCH;
    uint64_t chunk;
    if (__builtin_mul_overflow(numel / n, (uint64_t)elem_size, &chunk) || chunk >= (1ull << 56)) return MHIP_ERR_INVALID_ARGUMENT;
    // out may be in[rank]: the only bytes read and written through the same address are chunk `rank` of that tensor,
    // and each lane reads its vector before it writes it.  Chunks g != rank of in[rank] are overwritten by this call.
    return stack_entry(out, in, n, (uint64_t)rank * chunk, chunk, elem_size, stream);
}

}  // extern "C"
