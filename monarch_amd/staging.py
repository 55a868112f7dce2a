"""Staging transfers: Slice views <-> contiguous ``RDMABuffer`` bytes on one GPU.

``RDMABuffer`` keeps the reference's contract (python/monarch/_src/tensor_engine/rdma.py:80-207):
it only accepts 1-D contiguous ``uint8`` memory and moves flat byte ranges
(monarch_rdma/src/rdma_components.rs:94-171).  ``TensorBuffer`` is the API that file
leaves as a TODO (rdma.py:91-97): a non-contiguous, multi-byte-per-element tensor view is
gathered into such a buffer in ``Slice::iter`` order before ``read_into`` and scattered
back after ``write_from``.  All data movement happens in the library's HIP kernels.
"""
from __future__ import annotations

import ctypes as C
from typing import List, Optional, Sequence

import torch

from . import _torch
from ._lib import RdmaBufferC, check, lib, ptr_array
from .ndslice import Slice, slice_array


def _assert_tensor_is_1d_contiguous_uint8(t: torch.Tensor) -> None:
    # rdma.py:80-86, same messages
    if t.ndim != 1:
        raise ValueError(f"Tensor must be 1D, got {t.ndim}D")
    if t.dtype != torch.uint8:
        raise ValueError(f"Tensor must be uint8, got {t.dtype}")
    if not t.is_contiguous():
        raise ValueError("Tensor must be contiguous")


def _check_view_fits(base: torch.Tensor, s: Slice) -> None:
    if len(s) == 0:
        return
    _, hi = s.bounds()
    storage_elems = base.untyped_storage().nbytes() // base.element_size()
    if hi >= storage_elems:
        raise ValueError(f"slice reaches element {hi} but the storage holds {storage_elems}")


def _check_staging(buf: torch.Tensor, nbytes: int, device: torch.device) -> None:
    """A caller-supplied staging buffer: on the device of the tensor, contiguous, exactly ``nbytes`` long."""
    _torch.require_device(buf)
    if buf.device != device:
        raise ValueError(f"staging buffer is on {buf.device}, the tensor on {device}")
    if not buf.is_contiguous() or buf.numel() * buf.element_size() != nbytes:
        raise ValueError("staging buffer must be contiguous and hold exactly len(slice) elements")


def pack(base: torch.Tensor, s: Slice, out: Optional[torch.Tensor] = None, stream=None) -> torch.Tensor:
    """``out[i] = storage(base)[s.get(i)]``; returns a 1-D tensor of ``base.dtype``."""
    _torch.require_device(base)
    _check_view_fits(base, s)
    n = len(s)
    if out is None:
        out = torch.empty(n, dtype=base.dtype, device=base.device)
    else:
        _check_staging(out, n * base.element_size(), base.device)
    check(lib().mhip_slice_pack(out.data_ptr(), _torch.storage_ptr(base), C.byref(s.c), base.element_size(),
                                _torch.stream_handle(stream)))
    return out


def unpack(base: torch.Tensor, s: Slice, src: torch.Tensor, stream=None) -> None:
    """``storage(base)[s.get(i)] = src[i]``; elements outside the view keep their values."""
    _torch.require_device(base)
    _check_view_fits(base, s)
    _check_staging(src, len(s) * base.element_size(), base.device)
    check(lib().mhip_slice_unpack(_torch.storage_ptr(base), src.data_ptr(), C.byref(s.c), base.element_size(),
                                  _torch.stream_handle(stream)))


def pack_many(base: torch.Tensor, views: Sequence[Slice], outs: Optional[List[torch.Tensor]] = None,
              stream=None) -> List[torch.Tensor]:
    """Packs several views of one tensor (a reshard's column blocks) in as few launches as possible."""
    _torch.require_device(base)
    for s in views:
        _check_view_fits(base, s)
    if outs is None:
        outs = [torch.empty(len(s), dtype=base.dtype, device=base.device) for s in views]
    elif len(outs) != len(views):
        raise ValueError(f"{len(views)} views need {len(views)} staging buffers, got {len(outs)}")
    for s, o in zip(views, outs):
        _check_staging(o, len(s) * base.element_size(), base.device)
    arr = slice_array(views)
    check(lib().mhip_slice_pack_many(ptr_array([o.data_ptr() for o in outs]), _torch.storage_ptr(base), arr,
                                     len(views), base.element_size(), _torch.stream_handle(stream)))
    return outs


def unpack_many(base: torch.Tensor, views: Sequence[Slice], srcs: Sequence[torch.Tensor], stream=None) -> None:
    _torch.require_device(base)
    if len(srcs) != len(views):
        raise ValueError(f"{len(views)} views need {len(views)} staging buffers, got {len(srcs)}")
    for s, src in zip(views, srcs):
        _check_view_fits(base, s)
        _check_staging(src, len(s) * base.element_size(), base.device)
    arr = slice_array(views)
    check(lib().mhip_slice_unpack_many(_torch.storage_ptr(base), ptr_array([t.data_ptr() for t in srcs]), arr,
                                       len(views), base.element_size(), _torch.stream_handle(stream)))


# One RDMA work request carries its length in a 32-bit field of the scatter/gather entry
# (monarch_rdma/src/rdma_components.rs:1041,1063 cast the size with ``as u32``), so the library cuts a
# transfer of 4 GiB or more into several requests (``mhip_buffer_transfer``).  Segments are multiples of 16 bytes.
MAX_SEGMENT_BYTES = (1 << 32) - 16


def transfer(dst_ptr: int, src_ptr: int, nbytes: int, max_segment_bytes: int = 0, stream=None) -> int:
    """Moves ``nbytes`` bytes as one device copy per work request; returns the number of requests posted."""
    posted = C.c_uint32()
    check(lib().mhip_buffer_transfer(dst_ptr, src_ptr, nbytes, max_segment_bytes, _torch.stream_handle(stream),
                                     C.byref(posted)))
    return posted.value


def transfer_many(dst_ptrs, src_ptrs, nbytes, max_segment_bytes: int = 0, stream=None) -> int:
    """The same for several buffers at once, the requests of all of them in one launch (64 per launch); returns
    the number of requests posted."""
    n = len(nbytes)
    if len(dst_ptrs) != n or len(src_ptrs) != n:
        raise ValueError("transfer_many needs one destination, one source and one length per buffer")
    posted = C.c_uint32()
    check(lib().mhip_buffer_transfer_many((C.c_void_p * n)(*dst_ptrs), (C.c_void_p * n)(*src_ptrs),
                                          (C.c_size_t * n)(*nbytes), n, max_segment_bytes,
                                          _torch.stream_handle(stream), C.byref(posted)))
    return posted.value


class RDMABuffer:
    """A registered contiguous byte range ``{addr, size}`` (rdma_components.rs:94-102).

    On one GPU the transport is a flat device copy; the names keep the reference's
    direction: ``buf.read_into(dst)`` copies the buffer's bytes into ``dst`` and
    ``buf.write_from(src)`` copies ``src`` into the buffer.  As in the reference's binding
    (monarch_rdma/extension/lib.rs:135-190) the tensor becomes a local ``RdmaBuffer`` and the library's
    ``write_from`` / ``read_into`` run on it with this buffer as the remote side.
    """

    def __init__(self, data: torch.Tensor) -> None:
        _assert_tensor_is_1d_contiguous_uint8(data)
        _torch.require_device(data)
        self._data = data
        self.addr = data.data_ptr()
        self.size = data.numel()

    @property
    def data(self) -> torch.Tensor:
        return self._data

    def _remote(self, offset: int) -> RdmaBufferC:
        return RdmaBufferC(self.addr + offset, self.size - offset)

    def read_into(self, dst: torch.Tensor, offset: int = 0, stream=None) -> int:
        """Copies ``dst.numel()`` bytes of the buffer, from byte ``offset`` of it, into ``dst``.  (In the reference
        ``offset`` is added to the local address and then checked against ``dst.numel()``
        (python/monarch/_src/tensor_engine/rdma.py:160-165), which only ``offset == 0`` passes; every call that succeeds
        there means the same here, and a non-zero offset addresses the registered range instead of raising.)"""
        _assert_tensor_is_1d_contiguous_uint8(dst)
        _torch.require_device(dst)
        size = dst.numel()
        if offset < 0 or offset + size > self.size:
            raise ValueError(f"offset + size ({offset + size}) must be <= buffer size ({self.size})")
        local = RdmaBufferC(dst.data_ptr(), size)
        check(lib().mhip_buffer_write_from(C.byref(local), C.byref(self._remote(offset)), _torch.stream_handle(stream)))
        return size

    def write_from(self, src: torch.Tensor, offset: int = 0, stream=None) -> None:
        """Copies ``src`` into the buffer at byte ``offset`` of it (rdma.py:187-214; ``offset`` as in ``read_into``)."""
        _assert_tensor_is_1d_contiguous_uint8(src)
        _torch.require_device(src)
        size = src.numel()
        if offset < 0 or size + offset > self.size:
            raise ValueError(f"size + offset ({size + offset}) must be <= buffer size ({self.size})")
        local = RdmaBufferC(src.data_ptr(), size)
        check(lib().mhip_buffer_read_into(C.byref(local), C.byref(self._remote(offset)), _torch.stream_handle(stream)))


class TensorBuffer:
    """A tensor view staged through an ``RDMABuffer``: pack before the transfer out,
    unpack after the transfer in."""

    def __init__(self, view: torch.Tensor, staging: Optional[torch.Tensor] = None) -> None:
        _torch.require_device(view)
        self.view = view
        self.slice = Slice.of_tensor(view)
        nbytes = len(self.slice) * view.element_size()
        if staging is None:
            staging = torch.empty(nbytes, dtype=torch.uint8, device=view.device)
        self.buffer = RDMABuffer(staging)
        if self.buffer.size != nbytes:
            raise ValueError(f"staging buffer holds {self.buffer.size} bytes, the view needs {nbytes}")

    def stage(self, stream=None) -> RDMABuffer:
        """Gather the view into the staging bytes (call before ``buffer.read_into``)."""
        pack(self.view, self.slice, out=self.buffer.data, stream=stream)
        return self.buffer

    def commit(self, stream=None) -> None:
        """Scatter the staging bytes back into the view (call after ``buffer.write_from``)."""
        unpack(self.view, self.slice, self.buffer.data, stream=stream)


def slot_pitch(slot_bytes: int) -> int:
    """Byte distance between consecutive slots of a staging area (``mhip_staging_slot_pitch``)."""
    pitch = C.c_size_t()
    check(lib().mhip_staging_slot_pitch(slot_bytes, C.byref(pitch)))
    return pitch.value


class StagingArea:
    """``n_slots`` equally sized staging buffers carved from one allocation: slot *r* is where
    peer *r*'s chunk lands before the local combine, the per-worker chunks of the reference's
    parameter server (monarch_rdma/examples/parameter_server/parameter_server.rs:193-210).
    Slots are ``slot_pitch(slot_bytes)`` apart rather than back to back: reduce kernels read all
    slots side by side, and streams that start a multiple of 16 KiB apart collide in HBM."""

    def __init__(self, n_slots: int, slot_bytes: int, device="cuda:0") -> None:
        if n_slots <= 0 or slot_bytes <= 0:
            raise ValueError("a staging area needs at least one slot of at least one byte")
        self.n_slots, self.slot_bytes = n_slots, slot_bytes
        self.pitch = slot_pitch(slot_bytes)
        self.storage = torch.empty((n_slots - 1) * self.pitch + slot_bytes, dtype=torch.uint8, device=device)
        _torch.require_device(self.storage)

    def slot(self, r: int, dtype: torch.dtype = torch.uint8) -> torch.Tensor:
        """Slot ``r`` as a 1-D tensor of ``dtype`` (a view: no copy)."""
        if not 0 <= r < self.n_slots:
            raise IndexError(f"slot {r} of {self.n_slots}")
        return self.storage[r * self.pitch: r * self.pitch + self.slot_bytes].view(dtype)

    def slots(self, dtype: torch.dtype = torch.uint8) -> List[torch.Tensor]:
        return [self.slot(r, dtype) for r in range(self.n_slots)]

    def buffer(self, r: int) -> RDMABuffer:
        """Slot ``r`` as the 1-D uint8 buffer an RDMA transfer targets."""
        return RDMABuffer(self.slot(r))
