"""GPU staging memory an RdmaBuffer could register: VMM allocation, device-pointer test, dma-buf export.
Follows the reference's RDMA test environment: two 2 MiB device buffers, the first filled with i % 256,
one transfer, byte-compare (monarch_rdma/src/test_utils.rs:370-467,529-569)."""
import ctypes as C
import os

import numpy as np
import pytest
import torch

from monarch_amd import Slice, _lib
from monarch_amd._lib import check, lib

pytestmark = pytest.mark.gpu
MiB = 1 << 20


def _alloc(nbytes):
    ptr, padded = C.c_void_p(), C.c_size_t()
    check(lib().mhip_staging_alloc(C.byref(ptr), C.byref(padded), nbytes, 0))
    return ptr.value, padded.value


def test_vmm_buffers_transfer_and_compare():
    torch.cuda.init()
    L = lib()
    size = 2 * MiB
    a, pa = _alloc(size)
    b, pb = _alloc(size)
    assert pa >= size and pb >= size and a % 4096 == 0 and b % 4096 == 0 and a != b
    pattern = (np.arange(size) % 256).astype(np.uint8)
    check(L.mhip_memcpy_htod(a, pattern.ctypes.data, size, None))
    check(L.mhip_memset(b, 0, size, None))
    check(L.mhip_device_synchronize())
    flat = Slice.new_row_major([size])
    check(L.mhip_slice_pack(b, a, C.byref(flat.c), 1, None))           # the "transfer": staging a -> staging b
    back = np.empty(size, dtype=np.uint8)
    check(L.mhip_memcpy_dtoh(back.ctypes.data, b, size, None))
    check(L.mhip_device_synchronize())
    assert np.array_equal(back, pattern)
    # a strided view of buffer a packed into buffer b and scattered back
    view = Slice(offset=3, sizes=[1000, 300], strides=[1024, 2])
    check(L.mhip_slice_pack(b, a, C.byref(view.c), 2, None))
    check(L.mhip_memset(a, 0, size, None))
    check(L.mhip_slice_unpack(a, b, C.byref(view.c), 2, None))
    check(L.mhip_memcpy_dtoh(back.ctypes.data, a, size, None))
    check(L.mhip_device_synchronize())
    want = np.zeros(size // 2, dtype=np.uint16)
    idx = view.locations().astype(np.int64)
    want[idx] = pattern.view(np.uint16)[idx]
    assert np.array_equal(back.view(np.uint16), want)
    is_dev = C.c_int(-1)
    check(L.mhip_pointer_is_device(a, C.byref(is_dev)))
    assert is_dev.value == 1
    t = torch.zeros(16, device="cuda:0")
    check(L.mhip_pointer_is_device(t.data_ptr(), C.byref(is_dev)))
    assert is_dev.value == 1
    check(L.mhip_pointer_is_device(pattern.ctypes.data, C.byref(is_dev)))
    assert is_dev.value == 0
    check(L.mhip_staging_free(a, pa))
    check(L.mhip_staging_free(b, pb))
    c, pc = _alloc(64 * MiB)      # the address space and memory are reusable afterwards
    check(L.mhip_memset(c, 7, 64 * MiB, None))
    check(L.mhip_device_synchronize())
    check(L.mhip_staging_free(c, pc))
    assert L.mhip_staging_alloc(None, None, 0, 0) == _lib.ERR_INVALID_ARGUMENT


def test_dmabuf_export_of_staging_memory():
    torch.cuda.init()
    L = lib()
    a, pa = _alloc(2 * MiB)
    fd = C.c_int(-1)
    rc = L.mhip_export_dmabuf(C.byref(fd), a, pa)
    try:
        if rc != 0:
            pytest.skip(f"this kernel/driver does not export dma-bufs for device memory: {L.mhip_error_string(rc).decode()}")
        assert fd.value >= 0
        assert os.fstat(fd.value) is not None
        os.close(fd.value)
    finally:
        check(L.mhip_staging_free(a, pa))
    assert L.mhip_export_dmabuf(None, a, 16) == _lib.ERR_INVALID_ARGUMENT
