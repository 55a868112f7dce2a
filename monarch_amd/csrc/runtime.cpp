// Runtime pass-through and error text: the small part of the HIP runtime that the
// data path's callers reach through this library instead of through cuda-sys/nccl-sys.
#include <cstdint>
#include <cstdlib>
#include <hip/hip_runtime.h>

#include "mhip_device.h"
#include "mhip_internal.h"

#define MHIP_VERSION 100

namespace mhip {

// The only two reads of the environment in the library; both run while the library is loaded.
const bool g_tuning = [] {
    const char* e = std::getenv("MONARCH_HIP_TUNING");
    return e != nullptr && e[0] == '1' && e[1] == '\0';
}();
const uint64_t g_max_launch_lanes = [] {
    uint64_t v = 0xffffffffull;
    if (const char* e = std::getenv("MONARCH_HIP_TUNING"); e != nullptr && e[0] == '1' && e[1] == '\0') {
        if (const char* m = std::getenv("MONARCH_HIP_MAX_LAUNCH_LANES")) {
            const unsigned long long x = std::strtoull(m, nullptr, 10);
            if (x >= 8192 && x < v) v = x;
        }
    }
    return v;
}();

// Byte fill as a kernel rather than hipMemsetAsync: memset nodes recorded into a HIP graph have produced wrong
// results on replays after the first on this platform, kernel nodes have not, and callers may capture this call
// (clearing a staging chunk after it has been summed, parameter_server.rs:200-205).  16-byte vectors over the
// aligned middle of the range, single bytes at its ends.
constexpr int kFillThreads = 256;

__global__ __launch_bounds__(kFillThreads) void fill_kernel(unsigned char* dst, uint32_t word, uint64_t bytes, uint64_t head,
                                                            uint64_t nvec, uint64_t wg0) {
    const uint64_t wg = wg0 + blockIdx.x;
    const uint64_t v = wg * kFillThreads + threadIdx.x;
    if (v < nvec) store16_aligned(dst + head + v * 16, make_uint4(word, word, word, word));
    if (wg == 0) {
        for (uint64_t i = threadIdx.x; i < head; i += kFillThreads) dst[i] = (unsigned char)word;
        for (uint64_t i = head + nvec * 16 + threadIdx.x; i < bytes; i += kFillThreads) dst[i] = (unsigned char)word;
    }
}

}  // namespace mhip

using namespace mhip;

extern "C" {

const char* mhip_error_string(int status) {
    switch (status) {
        case MHIP_SUCCESS: return "success";
        case MHIP_ERR_INVALID_DIMS: return "invalid dims: sizes and strides differ in length";
        case MHIP_ERR_NONRECTANGULAR_SHAPE: return "nonrectangular shape";
        case MHIP_ERR_NONUNIQUE_STRIDES: return "nonunique strides";
        case MHIP_ERR_STRIDE_TOO_SMALL: return "stride must be larger than size of previous space";
        case MHIP_ERR_INDEX_OUT_OF_RANGE: return "index out of range";
        case MHIP_ERR_VALUE_NOT_IN_SLICE: return "value not in slice";
        case MHIP_ERR_INCOMPATIBLE_VIEW: return "incompatible view";
        case MHIP_ERR_NONCONTIGUOUS: return "noncontiguous shape";
        case MHIP_ERR_EMPTY_RANGE: return "empty range";
        case MHIP_ERR_DIMENSION_OUT_OF_RANGE: return "dimension out of range";
        case MHIP_ERR_INVALID_DATA_TYPE: return "invalid data type for a reduction";
        case MHIP_ERR_NONCONTIGUOUS_TENSOR: return "tensor used in collective must be contiguous";
        case MHIP_ERR_INVALID_DEVICE: return "tensor must be on a GPU device";
        case MHIP_ERR_FLOAT8_REDUCTION: return "float8 dtypes are not currently supported for reductions";
        case MHIP_ERR_TYPE_MISMATCH: return "output tensor must have the same type as input tensor";
        case MHIP_ERR_OUTPUT_SIZE_MISMATCH: return "output tensor size must be equal to world size times input tensor size";
        case MHIP_ERR_INPUT_SIZE_MISMATCH: return "input tensor must be the same size as output size times world size";
        case MHIP_ERR_UNDEFINED_TENSOR: return "undefined tensor (null pointer) used for operation";
        case MHIP_ERR_INVALID_ARGUMENT: return "an argument has an invalid value";
        case MHIP_ERR_UNSUPPORTED_OP: return "reduction op not supported for this dtype (Sum, Prod, Max, Min; Avg on floating types)";
        case MHIP_ERR_TOO_MANY_INPUTS: return "too many inputs for one reduce (at most 64)";
        case MHIP_ERR_UNSUPPORTED_BLOCK: return "unsupported fp8 scale block (must be 1024)";
        case MHIP_ERR_BUFFER_TOO_SMALL: return "remote buffer is smaller than the transfer";
        case MHIP_ERR_SCRATCH_TOO_SMALL: return "input exceeds what the library's static scratch holds (2^20 - 1 blocks of 1024 elements)";
        case MHIP_ERR_WQE_OVERFLOW: return "Overflow of WQE, possible data loss: more work requests than the queue has slots";
        case MHIP_ERR_MESH_DIM_LENGTH_MISMATCH: return "dimension of destination device_mesh has a different length than the source tensor";
        case MHIP_ERR_MESH_DIM_MISSING: return "destination mesh does not have a dimension of the source tensor";
        default: break;
    }
    if (status > 0 && status < 10000) return hipGetErrorString(static_cast<hipError_t>(status));
    return "unknown status";
}

int mhip_version(void) { return MHIP_VERSION; }

int mhip_device_count(int* count) { return count ? (int)hipGetDeviceCount(count) : MHIP_ERR_INVALID_ARGUMENT; }
int mhip_set_device(int device) {
    if (hipError_t e = hipSetDevice(device); e != hipSuccess) return (int)e;
    return prepare_static_scratch();  // so that no data-path call, possibly under stream capture, has to look it up
}
int mhip_device_synchronize(void) { return (int)hipDeviceSynchronize(); }

int mhip_stream_create(mhip_stream_t* stream) {
    if (!stream) return MHIP_ERR_INVALID_ARGUMENT;
    hipStream_t s = nullptr;
    hipError_t e = hipStreamCreateWithFlags(&s, hipStreamNonBlocking);  // default priority
    *stream = s;
    if (e != hipSuccess) return (int)e;
    return prepare_static_scratch();  // the stream's device is the current one
}
int mhip_stream_destroy(mhip_stream_t stream) { return (int)hipStreamDestroy(static_cast<hipStream_t>(stream)); }
int mhip_stream_synchronize(mhip_stream_t stream) { return (int)hipStreamSynchronize(static_cast<hipStream_t>(stream)); }

int mhip_event_create(mhip_event_t* event) {
    if (!event) return MHIP_ERR_INVALID_ARGUMENT;
    hipEvent_t e = nullptr;
    hipError_t rc = hipEventCreate(&e);
    *event = e;
    return (int)rc;
}
int mhip_event_destroy(mhip_event_t event) { return (int)hipEventDestroy(static_cast<hipEvent_t>(event)); }
int mhip_event_record(mhip_event_t event, mhip_stream_t stream) {
    return (int)hipEventRecord(static_cast<hipEvent_t>(event), static_cast<hipStream_t>(stream));
}
int mhip_event_synchronize(mhip_event_t event) { return (int)hipEventSynchronize(static_cast<hipEvent_t>(event)); }
int mhip_event_elapsed_ms(float* ms, mhip_event_t start, mhip_event_t stop) {
    if (!ms) return MHIP_ERR_INVALID_ARGUMENT;
    return (int)hipEventElapsedTime(ms, static_cast<hipEvent_t>(start), static_cast<hipEvent_t>(stop));
}
int mhip_stream_wait_event(mhip_stream_t stream, mhip_event_t event) {
    return (int)hipStreamWaitEvent(static_cast<hipStream_t>(stream), static_cast<hipEvent_t>(event), 0);
}

int mhip_malloc(void** ptr, size_t bytes) { return ptr ? (int)hipMalloc(ptr, bytes) : MHIP_ERR_INVALID_ARGUMENT; }
int mhip_free(void* ptr) { return (int)hipFree(ptr); }
int mhip_memcpy_htod(void* dst, const void* src, size_t bytes, mhip_stream_t stream) {
    return (int)hipMemcpyAsync(dst, src, bytes, hipMemcpyHostToDevice, static_cast<hipStream_t>(stream));
}
int mhip_memcpy_dtoh(void* dst, const void* src, size_t bytes, mhip_stream_t stream) {
    return (int)hipMemcpyAsync(dst, src, bytes, hipMemcpyDeviceToHost, static_cast<hipStream_t>(stream));
}
int mhip_memset(void* dst, int value, size_t bytes, mhip_stream_t stream) {
    if (bytes == 0) return MHIP_SUCCESS;
    if (!dst) return MHIP_ERR_UNDEFINED_TENSOR;
    const uint32_t b = (uint32_t)value & 0xffu, word = b * 0x01010101u;
    uint64_t head = (16 - ((uintptr_t)dst & 15u)) & 15u;
    if (head > bytes) head = bytes;
    const uint64_t nvec = (bytes - head) / 16;
    const uint64_t wgs = nvec ? (nvec + kFillThreads - 1) / kFillThreads : 1;  // workgroup 0 also writes the ends
    hipStream_t hs = static_cast<hipStream_t>(stream);
    DeviceGuard guard(hs);
    return launch_in_pieces(wgs, kFillThreads, 1, [&](uint64_t wg0, uint32_t count) {
        MHIP_LAUNCH(fill_kernel, dim3(count), dim3(kFillThreads), 0, hs, static_cast<unsigned char*>(dst), word,
                           (uint64_t)bytes, head, nvec, wg0);
    });
}

// ---- staging-buffer lifecycle -------------------------------------------------------
// The recipe of the reference's RDMA test environment (monarch_rdma/src/test_utils.rs:370-444)
// and of RdmaDomain::register_mr (monarch_rdma/src/rdma_components.rs:364-419) on the HIP
// virtual-memory API: a physical allocation pinned on the device, mapped at a reserved
// address with read/write access, exportable as a dma-buf for ibv_reg_dmabuf_mr.

int mhip_staging_slot_pitch(size_t slot_bytes, size_t* pitch_bytes) {
    if (!pitch_bytes || slot_bytes == 0) return MHIP_ERR_INVALID_ARGUMENT;
    constexpr size_t kPeriod = 16384, kSkew = 8192;
    if (slot_bytes > SIZE_MAX - kPeriod - kSkew) return MHIP_ERR_INVALID_ARGUMENT;
    *pitch_bytes = (slot_bytes + kPeriod - 1) / kPeriod * kPeriod + kSkew;
    return MHIP_SUCCESS;
}

int mhip_staging_alloc(void** ptr, size_t* padded_bytes, size_t bytes, int device) {
    if (!ptr || !padded_bytes || bytes == 0) return MHIP_ERR_INVALID_ARGUMENT;
    hipMemAllocationProp prop = {};
    prop.type = hipMemAllocationTypePinned;
    prop.location.type = hipMemLocationTypeDevice;
    prop.location.id = device;
    prop.requestedHandleTypes = hipMemHandleTypePosixFileDescriptor;
    size_t granularity = 0;
    hipError_t e = hipMemGetAllocationGranularity(&granularity, &prop, hipMemAllocationGranularityMinimum);
    if (e != hipSuccess) return (int)e;
    if (granularity == 0) return MHIP_ERR_INVALID_ARGUMENT;
    const size_t padded = ((bytes - 1) / granularity + 1) * granularity;
    hipMemGenericAllocationHandle_t handle;
    e = hipMemCreate(&handle, padded, &prop, 0);
    if (e != hipSuccess) return (int)e;
    void* va = nullptr;
    e = hipMemAddressReserve(&va, padded, granularity, nullptr, 0);
    if (e != hipSuccess) {
        (void)hipMemRelease(handle);
        return (int)e;
    }
    e = hipMemMap(va, padded, 0, handle, 0);
    if (e != hipSuccess) {
        (void)hipMemAddressFree(va, padded);
        (void)hipMemRelease(handle);
        return (int)e;
    }
    // the mapping keeps the physical memory alive; the creation reference can go now
    (void)hipMemRelease(handle);
    hipMemAccessDesc access = {};
    access.location.type = hipMemLocationTypeDevice;
    access.location.id = device;
    access.flags = hipMemAccessFlagsProtReadWrite;
    e = hipMemSetAccess(va, padded, &access, 1);
    if (e != hipSuccess) {
        (void)hipMemUnmap(va, padded);
        (void)hipMemAddressFree(va, padded);
        return (int)e;
    }
    *ptr = va;
    *padded_bytes = padded;
    return MHIP_SUCCESS;
}

int mhip_staging_free(void* ptr, size_t padded_bytes) {
    if (!ptr || padded_bytes == 0) return MHIP_ERR_INVALID_ARGUMENT;
    hipError_t e = hipMemUnmap(ptr, padded_bytes);
    if (e != hipSuccess) return (int)e;
    return (int)hipMemAddressFree(ptr, padded_bytes);
}

int mhip_pointer_is_device(const void* ptr, int* is_device) {
    if (!is_device) return MHIP_ERR_INVALID_ARGUMENT;
    // register_mr's test: the attribute query succeeds only for device memory the runtime knows
    hipPointerAttribute_t attr = {};
    const hipError_t e = hipPointerGetAttributes(&attr, ptr);
    if (e != hipSuccess) {
        (void)hipGetLastError();  // an unknown host pointer is an answer, not a sticky error
        *is_device = 0;
        return MHIP_SUCCESS;
    }
    *is_device = attr.type == hipMemoryTypeDevice ? 1 : 0;
    return MHIP_SUCCESS;
}

int mhip_export_dmabuf(int* fd, const void* ptr, size_t bytes) {
    if (!fd || !ptr || bytes == 0) return MHIP_ERR_INVALID_ARGUMENT;
    int out = -1;
    const hipError_t e = hipMemGetHandleForAddressRange(&out, const_cast<void*>(ptr), bytes, hipMemRangeHandleTypeDmaBufFd, 0);
    if (e != hipSuccess) return (int)e;
    *fd = out;
    return MHIP_SUCCESS;
}

}  // extern "C"
