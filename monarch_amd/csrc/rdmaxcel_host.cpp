// Device-initiated RDMA, host side: the argument checks of the mhip_rdmaxcel_* entry points and the forms that build the
// entries on the calling thread (rdmaxcel-sys/src/rdmaxcel.cu:82-93,139-160,201-245,292-326 are __host__ __device__, and
// monarch_rdma/src/rdma_components.rs:88,880,1159-1163 calls the host side from Rust).  Plain C++ with no HIP in it, so
// that it also builds with the host compiler under the sanitizers (tests/c_abi/host_fuzz.cpp).
#include "mhip_internal.h"
#include "../../include/monarch_hip_rdmaxcel_device.h"

namespace mhip {

static bool power_of_two(uint32_t v) { return v != 0 && (v & (v - 1)) == 0; }

int check_wqe(const mhip_wqe_params_t* p, bool send) {
    if (!p || !p->buf || !p->dbrec) return MHIP_ERR_INVALID_ARGUMENT;
    if (((uintptr_t)p->buf & 15u) || ((uintptr_t)p->dbrec & 3u)) return MHIP_ERR_INVALID_ARGUMENT;
    if (send && !power_of_two(p->wqe_cnt)) return MHIP_ERR_INVALID_ARGUMENT;
    return MHIP_SUCCESS;
}

int check_cqe(const int32_t* result, const mhip_cqe_poll_params_t* p) {
    if (!result || !p || !p->cqe_buf || !p->dbrec) return MHIP_ERR_INVALID_ARGUMENT;
    if (p->cqe_size != 64 && p->cqe_size != 128) return MHIP_ERR_INVALID_ARGUMENT;
    if (!power_of_two(p->cqe_cnt)) return MHIP_ERR_INVALID_ARGUMENT;
    if (((uintptr_t)p->cqe_buf & 3u) || ((uintptr_t)p->dbrec & 3u) || ((uintptr_t)result & 3u)) return MHIP_ERR_INVALID_ARGUMENT;
    return MHIP_SUCCESS;
}

int check_ring(const void* dst, const void* src) {
    if (!dst || !src || ((uintptr_t)dst & 7u) || ((uintptr_t)src & 7u)) return MHIP_ERR_INVALID_ARGUMENT;
    return MHIP_SUCCESS;
}

}  // namespace mhip

using namespace mhip;

extern "C" {

int mhip_rdmaxcel_send_wqe_host(const mhip_wqe_params_t* params) {
    if (int rc = check_wqe(params, true)) return rc;
    mhip_rdmaxcel::send_wqe(*params);
    return MHIP_SUCCESS;
}

int mhip_rdmaxcel_recv_wqe_host(const mhip_wqe_params_t* params) {
    if (int rc = check_wqe(params, false)) return rc;
    mhip_rdmaxcel::recv_wqe(*params);
    return MHIP_SUCCESS;
}

int mhip_rdmaxcel_db_ring_host(void* dst, const void* src) {
    if (int rc = check_ring(dst, src)) return rc;
    mhip_rdmaxcel::db_ring(dst, src);
    mhip_rdmaxcel::release_to_system();
    return MHIP_SUCCESS;
}

int mhip_rdmaxcel_cqe_poll_host(int32_t* result, const mhip_cqe_poll_params_t* params) {
    if (int rc = check_cqe(result, params)) return rc;
    mhip_rdmaxcel::cqe_poll(result, *params);
    return MHIP_SUCCESS;
}

}  // extern "C"
