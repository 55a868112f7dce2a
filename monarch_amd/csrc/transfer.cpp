// RdmaBuffer transfers and SendTensor's data movement on one GPU: the host logic that the reference keeps in
// Rust (monarch_rdma/src/rdma_components.rs, monarch_tensor_worker/src/stream.rs) behind the C ABI.  The bytes
// themselves are moved by the library's copy kernels; routing and the to_mesh checks are in slice_host.cpp.
#include "mhip_internal.h"

namespace mhip {

// One RDMA work request carries its length in the 32-bit field of a scatter/gather entry
// (rdma_components.rs:1041,1063 cast the buffer size with `as u32`, which truncates transfers of 4 GiB and
// more); a transfer is therefore cut into requests of at most this many bytes (a multiple of 16, so that
// every request after the first keeps the alignment of the first).
constexpr uint64_t kMaxSegmentBytes = (1ull << 32) - 16;

static int transfer(void* dst, const void* src, uint64_t bytes, uint64_t max_segment, mhip_stream_t stream,
                    uint32_t* segments) {
    if (segments) *segments = 0;
    if (max_segment == 0 || max_segment > kMaxSegmentBytes) max_segment = kMaxSegmentBytes;
    if (bytes == 0) return MHIP_SUCCESS;
    if (!dst || !src) return MHIP_ERR_UNDEFINED_TENSOR;
    const uint64_t unit_stride = 1;
    uint32_t posted = 0;
    for (uint64_t done = 0; done < bytes;) {
        const uint64_t len = bytes - done < max_segment ? bytes - done : max_segment;
        const mhip_slice_t run{0, 1, &len, &unit_stride};  // one contiguous run of `len` bytes
        if (int rc = mhip_slice_pack(static_cast<char*>(dst) + done, static_cast<const char*>(src) + done, &run, 1, stream))
            return rc;
        done += len;
        ++posted;
    }
    if (segments) *segments = posted;
    return MHIP_SUCCESS;
}

// The same walk for n buffers at once: every request of every buffer becomes one entry of a many-copy launch
// (kCopyManyMax entries per launch).
static int transfer_many(void* const* dsts, const void* const* srcs, const size_t* bytes, uint32_t n, uint64_t max_segment,
                         mhip_stream_t stream, uint32_t* segments) {
    if (segments) *segments = 0;
    if (n == 0) return MHIP_SUCCESS;
    if (!dsts || !srcs || !bytes) return MHIP_ERR_INVALID_ARGUMENT;
    if (max_segment == 0 || max_segment > kMaxSegmentBytes) max_segment = kMaxSegmentBytes;
    for (uint32_t g = 0; g < n; ++g)
        if (bytes[g] != 0 && (!dsts[g] || !srcs[g])) return MHIP_ERR_UNDEFINED_TENSOR;
    void* d[kCopyManyMax];
    const void* s[kCopyManyMax];
    uint64_t len[kCopyManyMax];
    uint32_t pending = 0, posted = 0;
    for (uint32_t g = 0; g < n; ++g) {
        for (uint64_t done = 0; done < bytes[g];) {
            const uint64_t l = bytes[g] - done < max_segment ? bytes[g] - done : max_segment;
            d[pending] = static_cast<char*>(dsts[g]) + done;
            s[pending] = static_cast<const char*>(srcs[g]) + done;
            len[pending] = l;
            done += l;
            ++posted;
            if (++pending == (uint32_t)kCopyManyMax) {
                if (int rc = copy_many(d, s, len, pending, stream)) return rc;
                pending = 0;
            }
        }
    }
    if (pending != 0)
        if (int rc = copy_many(d, s, len, pending, stream)) return rc;
    if (segments) *segments = posted;
    return MHIP_SUCCESS;
}

static inline bool bad_slice(const mhip_slice_t* s) {
    return s == nullptr || s->ndim > MHIP_MAX_DIMS || (s->ndim > 0 && (!s->sizes || !s->strides));
}

}  // namespace mhip

using namespace mhip;

extern "C" {

int mhip_buffer_transfer(void* dst, const void* src, size_t bytes, size_t max_segment_bytes, mhip_stream_t stream,
                         uint32_t* segments) {
    return transfer(dst, src, bytes, max_segment_bytes, stream, segments);
}

int mhip_buffer_transfer_many(void* const* dsts, const void* const* srcs, const size_t* bytes, uint32_t n,
                              size_t max_segment_bytes, mhip_stream_t stream, uint32_t* segments) {
    return transfer_many(dsts, srcs, bytes, n, max_segment_bytes, stream, segments);
}

int mhip_buffer_read_into(const mhip_rdma_buffer_t* local, const mhip_rdma_buffer_t* remote, mhip_stream_t stream) {
    if (!local || !remote) return MHIP_ERR_INVALID_ARGUMENT;
    // put(): local.size bytes, local.addr -> remote.addr (rdma_components.rs:842-858); a NIC refuses a write
    // past the end of the remote memory region
    if (local->size > remote->size) return MHIP_ERR_BUFFER_TOO_SMALL;
    return transfer(remote->addr, local->addr, local->size, 0, stream, nullptr);
}

int mhip_buffer_write_from(const mhip_rdma_buffer_t* local, const mhip_rdma_buffer_t* remote, mhip_stream_t stream) {
    if (!local || !remote) return MHIP_ERR_INVALID_ARGUMENT;
    // get(): local.size bytes, remote.addr -> local.addr (rdma_components.rs:986-1002)
    if (local->size > remote->size) return MHIP_ERR_BUFFER_TOO_SMALL;
    return transfer(local->addr, remote->addr, local->size, 0, stream, nullptr);
}

int mhip_send_tensor(void* result, size_t result_bytes, const void* src_base, const mhip_slice_t* src_view,
                     uint32_t elem_size, void* staging, mhip_stream_t stream) {
    if (bad_slice(src_view) || elem_size == 0) return MHIP_ERR_INVALID_ARGUMENT;
    if (int rc = validate_slice(src_view->sizes, src_view->ndim, src_view->strides, src_view->ndim)) return rc;
    if (!slice_fits_address_space(*src_view, elem_size)) return MHIP_ERR_INVALID_ARGUMENT;
    const uint64_t bytes = slice_len(*src_view) * elem_size;
    // the receiver allocates factory.size elements (stream.rs:1533-1538); a sender whose tensor has another size
    // would make ncclRecv wait for bytes that never come
    if (bytes != result_bytes) return MHIP_ERR_OUTPUT_SIZE_MISMATCH;
    if (bytes == 0) return MHIP_SUCCESS;
    if (!result || !src_base) return MHIP_ERR_UNDEFINED_TENSOR;
    if (!staging)  // from_rank == to_rank: the defensive copy of stream.rs:1497-1516
        return mhip_slice_pack(result, src_base, src_view, elem_size, stream);
    if (int rc = mhip_slice_pack(staging, src_base, src_view, elem_size, stream)) return rc;
    return transfer(result, staging, bytes, 0, stream, nullptr);
}

}  // extern "C"
