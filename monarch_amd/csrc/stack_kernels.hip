// Reduction::Stack on the chunks one GPU holds: the data movement of all_gather_into_tensor
// (monarch_tensor_worker/src/stream.rs:1408-1417) and of all_to_all_single (stream.rs:1381-1399,
// torch-sys-cuda/src/nccl.rs:760-812) as one launch over all members.
//
// HBM-bound, 2 bytes of traffic per byte stacked.  Every member contributes one contiguous chunk that
// lands at chunk index g of the output, so the launch is n contiguous copies side by side.  The same kernel
// serves a message that moves several staging buffers at once (mhip_buffer_transfer_many).
#include "mhip_device.h"
#include "mhip_internal.h"

namespace mhip {

constexpr int kStackInputs = 64;

// n independent contiguous copies in one launch, each laid out like the contiguous copy of the pack path:
// single-wavefront workgroups, one 16-byte vector per lane, non-temporal load, write-through store, the rows
// a wavefront writes on the destination's 1 KiB boundaries (a row that starts inside a cache line shares its first
// and last line with rows on other XCDs, and the line goes to HBM as two partial writes), the fewer than 16
// bytes before the first and after the last whole vector one by one.  Copies are the slow index: neighbouring
// workgroups write neighbouring memory.
struct CopyManyArgs {
    char* dst[kCopyManyMax];
    const char* src[kCopyManyMax];   // may equal dst (in-place all_to_all): no restrict
    uint64_t nbytes[kCopyManyMax];
    uint64_t row0[kCopyManyMax + 1]; // first workgroup of each copy; row0[n] = workgroups in all
    uint64_t wg0;                    // workgroups of this call launched before this grid
    uint32_t n;
};
constexpr int kCopyManyThreads = 64;

__device__ __forceinline__ uint64_t copy_head(const char* dst, uint64_t nbytes) {
    const uint64_t head = (16 - ((uintptr_t)dst & 15u)) & 15u;
    return head < nbytes ? head : nbytes;
}

// UNIFORM: every copy has the same number of rows (the chunks of a Stack, the blocks of a reshard), the grid is
// rows x copies and a workgroup reads its copy from blockIdx.y; otherwise the grid is flat and a workgroup finds its
// copy by walking row0[] (8 x 48 MiB: 0.855 of peak against 0.834 with the walk).
template <bool UNIFORM>
__global__ __launch_bounds__(kCopyManyThreads) void copy_many_kernel(CopyManyArgs a) {
    uint32_t g = 0;
    uint64_t row;
    if constexpr (UNIFORM) {
        g = blockIdx.y;
        row = blockIdx.x;
    } else {
        const uint64_t wg = a.wg0 + blockIdx.x;
        while (g + 1 < a.n && wg >= a.row0[g + 1]) ++g;  // wave-uniform, at most n - 1 steps
        row = wg - a.row0[g];
    }
    char* dst = a.dst[g];
    const char* src = a.src[g];
    const uint64_t nbytes = a.nbytes[g];
    const uint64_t head = copy_head(dst, nbytes);
    const uint64_t nvec = (nbytes - head) / 16;
    const uint64_t pad = ((uintptr_t)(dst + head) & 1023u) / 16;  // idle lanes at the start of row 0
    const uint64_t c = row * kCopyManyThreads + threadIdx.x;       // position in the padded vector grid
    if (c >= pad && c - pad < nvec) {
        const uint64_t at = head + (c - pad) * 16;
        store16_writethrough(dst + at, load16_unaligned(src + at));
    }
    if (row == 0) {
        for (uint64_t i = threadIdx.x; i < head; i += kCopyManyThreads) dst[i] = src[i];
        for (uint64_t i = head + nvec * 16 + threadIdx.x; i < nbytes; i += kCopyManyThreads) dst[i] = src[i];
    }
}

int copy_many(void* const* dst, const void* const* src, const uint64_t* nbytes, uint32_t n, void* stream) {
    if (n == 0) return MHIP_SUCCESS;
    if (n > (uint32_t)kCopyManyMax) return MHIP_ERR_TOO_MANY_INPUTS;
    CopyManyArgs a{};
    uint32_t m = 0;
    uint64_t rows = 0, first_rows = 0;
    bool uniform = true;
    for (uint32_t g = 0; g < n; ++g) {
        if (nbytes[g] == 0) continue;
        if (!dst[g] || !src[g]) return MHIP_ERR_UNDEFINED_TENSOR;
        a.dst[m] = static_cast<char*>(dst[g]);
        a.src[m] = static_cast<const char*>(src[g]);
        a.nbytes[m] = nbytes[g];
        a.row0[m] = rows;
        const uint64_t head = (16 - ((uintptr_t)dst[g] & 15u)) & 15u;
        const uint64_t nvec = nbytes[g] > head ? (nbytes[g] - head) / 16 : 0;
        const uint64_t pad = (((uintptr_t)dst[g] + head) & 1023u) / 16;
        uint64_t r = (nvec + pad + kCopyManyThreads - 1) / kCopyManyThreads;
        if (r == 0) r = 1;  // at least the byte loops of row 0
        if (m == 0) first_rows = r;
        uniform = uniform && r == first_rows;
        rows += r;
        ++m;
    }
    if (m == 0) return MHIP_SUCCESS;
    a.row0[m] = rows;
    a.n = m;
    hipStream_t hs = static_cast<hipStream_t>(stream);
    DeviceGuard guard(hs);
    if (uniform && rows <= max_workgroups(kCopyManyThreads) && first_rows < (1ull << 31)) {
        MHIP_LAUNCH(copy_many_kernel<true>, dim3((uint32_t)first_rows, m), dim3(kCopyManyThreads), 0, hs, a);
        return launch_status();
    }
    return launch_in_pieces(rows, kCopyManyThreads, 1, [&](uint64_t wg0, uint32_t count) {
        a.wg0 = wg0;
        MHIP_LAUNCH(copy_many_kernel<false>, dim3(count), dim3(kCopyManyThreads), 0, hs, a);
    });
}

static int stack_entry(void* out, const void* const* in, uint32_t n, uint64_t src_offset_bytes, uint64_t chunk_bytes,
                       uint32_t elem_size, mhip_stream_t stream) {
    if (chunk_bytes == 0) return MHIP_SUCCESS;
    if (!out) return MHIP_ERR_UNDEFINED_TENSOR;
    void* dst[kStackInputs];
    const void* src[kStackInputs];
    uint64_t nbytes[kStackInputs];
    uintptr_t mask = (uintptr_t)out | chunk_bytes;
    for (uint32_t g = 0; g < n; ++g) {
        if (!in[g]) return MHIP_ERR_UNDEFINED_TENSOR;
        src[g] = static_cast<const char*>(in[g]) + src_offset_bytes;
        dst[g] = static_cast<char*>(out) + g * chunk_bytes;
        nbytes[g] = chunk_bytes;
        mask |= (uintptr_t)src[g];
    }
    const uint32_t pow2 = elem_size & (0u - elem_size);  // largest power of two dividing the element size
    if (mask & ((pow2 < 16 ? pow2 : 16u) - 1)) return MHIP_ERR_INVALID_ARGUMENT;  // not even element-aligned
    return copy_many(dst, src, nbytes, n, stream);
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
