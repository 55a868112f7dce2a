// Device-initiated RDMA, the part that needs no NIC: building send / receive work-queue entries, ringing a
// doorbell and the single-shot completion-queue poll of rdmaxcel-sys/src/rdmaxcel.cu:82-93,139-160,201-245,
// 292-326, as kernels on the caller's stream (launch_* of rdmaxcel.cu:122-124,184-190,269-275,358-395) and as
// host functions (rdmaxcel_host.cpp: the reference's functions are __host__ __device__, and
// monarch_rdma/src/rdma_components.rs:88,880,1159-1163 calls the host side).
//
// Nothing here is bandwidth: an entry is 16 to 64 bytes and a call is one launch.  What the reference's launchers
// cost is a device-wide synchronisation per posted entry and, per poll, a managed allocation, a synchronisation and
// a free (rdmaxcel.cu:274,364-393); these entry points enqueue and return, and a poll writes to a device word the
// caller owns.  The functions themselves live in include/monarch_hip_rdmaxcel_device.h so that callers' own
// kernels can post from the device; every segment leaves as one aligned 16-byte store.
#include "mhip_device.h"
#include "mhip_internal.h"
#include "../../include/monarch_hip_rdmaxcel_device.h"

namespace mhip {

constexpr int kWqeThreads = 64;         // one wavefront; lane 0 works
constexpr int kPostThreads = 1024;      // one workgroup posts a whole chain: its barrier orders the entries before the record
constexpr uint64_t kMaxWqeSegment = (1ull << 31) - 16;

__global__ __launch_bounds__(kWqeThreads) void send_wqe_kernel(mhip_wqe_params_t p) {
    if (threadIdx.x == 0) mhip_rdmaxcel::send_wqe(p);
}

__global__ __launch_bounds__(kWqeThreads) void recv_wqe_kernel(mhip_wqe_params_t p) {
    if (threadIdx.x == 0) mhip_rdmaxcel::recv_wqe(p);
}

// count rings in order by one lane: each ring's 64 bytes must reach the register whole and before the next ring's.
__global__ __launch_bounds__(kWqeThreads) void db_ring_kernel(void* dst, const char* sq_buf, uint32_t stride, uint32_t wqe_cnt,
                                                              uint32_t first, uint32_t count) {
    if (threadIdx.x == 0) {
        for (uint32_t i = 0; i < count; ++i) {
            const uint32_t k = first + i;
            mhip_rdmaxcel::db_ring(dst, sq_buf + (uint64_t)(k % wqe_cnt) * stride);
            mhip_rdmaxcel::release_to_system();
        }
    }
}

__global__ __launch_bounds__(kWqeThreads) void cqe_poll_kernel(int32_t* result, mhip_cqe_poll_params_t p) {
    if (threadIdx.x == 0) {
        mhip_rdmaxcel::cqe_poll(result, p);
        mhip_rdmaxcel::release_to_system();
    }
}

// n entries of one transfer, one lane per entry: entry i moves [i * seg, min((i + 1) * seg, length)) of the local
// buffer to the same range of the remote one.  Slots are distinct (n <= wqe_cnt), so the entries can be written in
// any order; the doorbell record follows the workgroup's barrier.
__global__ __launch_bounds__(kPostThreads) void post_transfer_kernel(mhip_wqe_params_t p, uint64_t seg, uint32_t n) {
    const uint32_t idx0 = (uint32_t)p.wr_id;
    const uint64_t length = p.length;
    for (uint32_t i = threadIdx.x; i < n; i += kPostThreads) {
        mhip_wqe_params_t q = p;
        const uint64_t at = (uint64_t)i * seg;
        q.laddr = p.laddr + at;
        q.raddr = p.raddr + at;
        q.length = length - at < seg ? length - at : seg;
        const uint32_t idx = idx0 + i;
        mhip_rdmaxcel::Segment ctrl, raddr, data;
        mhip_rdmaxcel::build_send_wqe(q, idx, &ctrl, &raddr, &data);
        uint8_t* slot = p.buf + ((uint64_t)(idx & (p.wqe_cnt - 1u)) << mhip_rdmaxcel::kSendWqeShift);
        mhip_rdmaxcel::store_segment(slot, ctrl);
        mhip_rdmaxcel::store_segment(slot + 16, raddr);
        mhip_rdmaxcel::store_segment(slot + 32, data);
    }
    mhip_rdmaxcel::release_to_system();
    __syncthreads();
    if (threadIdx.x == 0) {
        mhip_rdmaxcel::store_word(p.dbrec + mhip_rdmaxcel::kSndDbr, mhip_rdmaxcel::be32((idx0 + n) & 0xFFFFFFu));
    }
}

}  // namespace mhip

using namespace mhip;

extern "C" {

int mhip_rdmaxcel_send_wqe(const mhip_wqe_params_t* params, mhip_stream_t stream) {
    if (int rc = check_wqe(params, true)) return rc;
    hipStream_t hs = static_cast<hipStream_t>(stream);
    DeviceGuard guard(hs);
    MHIP_LAUNCH(send_wqe_kernel, dim3(1), dim3(kWqeThreads), 0, hs, *params);
    return launch_status();
}

int mhip_rdmaxcel_recv_wqe(const mhip_wqe_params_t* params, mhip_stream_t stream) {
    if (int rc = check_wqe(params, false)) return rc;
    hipStream_t hs = static_cast<hipStream_t>(stream);
    DeviceGuard guard(hs);
    MHIP_LAUNCH(recv_wqe_kernel, dim3(1), dim3(kWqeThreads), 0, hs, *params);
    return launch_status();
}

int mhip_rdmaxcel_db_ring(void* dst, const void* src, mhip_stream_t stream) {
    if (int rc = check_ring(dst, src)) return rc;
    hipStream_t hs = static_cast<hipStream_t>(stream);
    DeviceGuard guard(hs);
    MHIP_LAUNCH(db_ring_kernel, dim3(1), dim3(kWqeThreads), 0, hs, dst, static_cast<const char*>(src), 0u, 1u, 0u, 1u);
    return launch_status();
}

int mhip_rdmaxcel_ring_doorbells(void* dst, const void* sq_buf, uint32_t stride, uint32_t wqe_cnt, uint32_t first_db_idx,
                                 uint32_t count, mhip_stream_t stream) {
    if (int rc = check_ring(dst, sq_buf)) return rc;
    if (stride < 64 || (stride & 7u) || wqe_cnt == 0) return MHIP_ERR_INVALID_ARGUMENT;
    if (count > wqe_cnt) return MHIP_ERR_WQE_OVERFLOW;
    if (count == 0) return MHIP_SUCCESS;
    hipStream_t hs = static_cast<hipStream_t>(stream);
    DeviceGuard guard(hs);
    MHIP_LAUNCH(db_ring_kernel, dim3(1), dim3(kWqeThreads), 0, hs, dst, static_cast<const char*>(sq_buf), stride, wqe_cnt,
                first_db_idx, count);
    return launch_status();
}

int mhip_rdmaxcel_cqe_poll(int32_t* d_result, const mhip_cqe_poll_params_t* params, mhip_stream_t stream) {
    if (int rc = check_cqe(d_result, params)) return rc;
    hipStream_t hs = static_cast<hipStream_t>(stream);
    DeviceGuard guard(hs);
    MHIP_LAUNCH(cqe_poll_kernel, dim3(1), dim3(kWqeThreads), 0, hs, d_result, *params);
    return launch_status();
}

int mhip_rdmaxcel_post_transfer(const mhip_wqe_params_t* params, size_t max_segment_bytes, uint32_t* n_wqes,
                                mhip_stream_t stream) {
    if (int rc = check_wqe(params, true)) return rc;
    uint64_t seg = max_segment_bytes;
    if (seg == 0 || seg > kMaxWqeSegment) seg = kMaxWqeSegment;
    const uint64_t length = params->length;
    const uint64_t n = length == 0 ? 1 : (length - 1) / seg + 1;
    if (n > params->wqe_cnt) return MHIP_ERR_WQE_OVERFLOW;
    if (n_wqes) *n_wqes = (uint32_t)n;
    hipStream_t hs = static_cast<hipStream_t>(stream);
    DeviceGuard guard(hs);
    MHIP_LAUNCH(post_transfer_kernel, dim3(1), dim3(kPostThreads), 0, hs, *params, seg, (uint32_t)n);
    return launch_status();
}

}  // extern "C"
