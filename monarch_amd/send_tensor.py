"""Point-to-point reshard (``Tensor.to_mesh`` / ``SendTensor``) on top of pack -> transfer -> unpack.

Mirrors, for the ranks whose data sits on this GPU:

* ``check_to_mesh``: the client-side validation of ``Tensor.to_mesh``
  (python/monarch/common/tensor.py:417-438), same messages;
* ``route``: which rank a worker sends to / receives from, from the ``from_ranks`` and
  ``to_ranks`` Slices of the message (monarch_tensor_worker/src/lib.rs:722-731);
  both are thin callers of the library's host code (``mhip_to_mesh_from_ranks``,
  ``mhip_send_tensor_route``), as ``DeviceMesh`` is of ``mhip_mesh_*``;
* ``stream_send_tensor``: what ``StreamActor::send_tensor`` leaves in ``result``
  (monarch_tensor_worker/src/stream.rs:1470-1560).  NCCL send/recv tolerates non-contiguous
  tensors (``is_p2p`` in torch-sys-cuda/src/nccl.rs:300-316); here the sender's view is
  gathered in ``Slice::iter`` order into contiguous staging bytes, which is what an
  ``RdmaBuffer`` moves, and the receiver's fresh tensor of ``factory.size`` is those bytes.
"""
from __future__ import annotations

import ctypes as C
from typing import Dict, Optional, Sequence, Tuple

import torch

from . import _lib, _torch
from ._lib import MhipError, check, lib, u64_array
from .ndslice import Slice
from .reduce import Factory


def _names(names: Sequence[str]):
    return (C.c_char_p * max(1, len(names)))(*[n.encode() for n in names])


def check_to_mesh(slicing_names: Sequence[str], slicing: Slice, mesh_names: Sequence[str], mesh_sizes: Sequence[int]):
    """Returns ``(from_ranks, broadcast_dims)`` or raises like ``Tensor.to_mesh``
    (``mhip_to_mesh_from_ranks``; the messages are those of python/monarch/common/tensor.py:426-437)."""
    slicing_names, mesh_names = list(slicing_names), list(mesh_names)
    nd = len(slicing_names)
    out_sizes, out_strides = u64_array([0] * nd), u64_array([0] * nd)
    out_ndim, n_bcast, culprit = C.c_uint32(), C.c_uint32(), C.c_uint32()
    bcast = (C.c_uint32 * max(1, len(mesh_names)))()
    rc = lib().mhip_to_mesh_from_ranks(_names(slicing_names), C.byref(slicing.c), _names(mesh_names),
                                       u64_array(list(mesh_sizes)), len(mesh_names), out_sizes, out_strides,
                                       C.byref(out_ndim), bcast, C.byref(n_bcast), C.byref(culprit))
    if rc == _lib.ERR_MESH_DIM_LENGTH_MISMATCH:
        raise ValueError(f"dimension {mesh_names[culprit.value]} of destination device_mesh has a different length "
                         "than the source tensor")
    if rc == _lib.ERR_MESH_DIM_MISSING:
        missing = set(slicing_names) - set(mesh_names)
        raise ValueError(f"destination mesh does not have dimensions {missing}")
    check(rc)
    n = out_ndim.value
    from_ranks = Slice(offset=slicing.offset, sizes=list(out_sizes)[:n], strides=list(out_strides)[:n])
    return from_ranks, [mesh_names[bcast[i]] for i in range(n_bcast.value)]


def route(from_ranks: Slice, to_ranks: Slice, rank: int) -> Tuple[Optional[int], Optional[int]]:
    """``(from_rank, to_rank)`` of ``rank``: the i-th sender pairs with the i-th receiver
    (``mhip_send_tensor_route``)."""
    fr, to = C.c_uint64(), C.c_uint64()
    check(lib().mhip_send_tensor_route(C.byref(from_ranks.c), C.byref(to_ranks.c), rank, C.byref(fr), C.byref(to)))
    return (None if fr.value == _lib.NO_RANK else fr.value, None if to.value == _lib.NO_RANK else to.value)


def stream_send_tensor(world: Dict[int, Optional[torch.Tensor]], rank: int, from_rank: Optional[int],
                       to_rank: Optional[int], factory: Factory, staging_bytes: Optional[torch.Tensor] = None,
                       stream=None) -> Optional[torch.Tensor]:
    """The tensor bound to ``result`` on ``rank`` (``None`` for a pure sender).  ``staging_bytes`` is the
    sender's registered staging buffer; without one a fresh buffer is used for the remote case."""
    if to_rank is None and from_rank is None:
        raise ValueError("tried to send tensor without a to/from rank")
    local = from_rank == to_rank
    if local:
        src = world[rank]  # local value: a defensive copy, stream.rs:1497-1516
    elif from_rank is not None:
        src = world[from_rank]
    else:
        return None
    if src is None:  # errored upstream: zeros of the factory still go over the wire, stream.rs:976-989
        return factory.zeros()
    _torch.require_device(src)
    out = torch.empty(factory.size, dtype=factory.dtype, device=src.device)
    view = Slice.of_tensor(src)
    nbytes = out.numel() * out.element_size()
    if out.numel() != src.numel():
        raise ValueError(f"factory size {tuple(factory.size)} does not match the sent tensor {tuple(src.shape)}")
    staging_ptr = None
    if not local:
        if staging_bytes is None:
            staging_bytes = torch.empty(nbytes, dtype=torch.uint8, device=src.device)
        elif staging_bytes.numel() * staging_bytes.element_size() != nbytes or not staging_bytes.is_contiguous():
            raise ValueError(f"staging buffer must hold exactly {nbytes} bytes")
        _torch.require_device(staging_bytes)
        staging_ptr = staging_bytes.data_ptr()
    try:
        check(lib().mhip_send_tensor(out.data_ptr(), nbytes, _torch.storage_ptr(src), C.byref(view.c),
                                     src.element_size(), staging_ptr, _torch.stream_handle(stream)))
    except MhipError as e:
        if e.status == _lib.ERR_OUTPUT_SIZE_MISMATCH:
            raise ValueError(f"factory size {tuple(factory.size)} does not match the sent tensor {tuple(src.shape)}")
        raise
    if staging_bytes is not None and stream is not None:
        staging_bytes.record_stream(stream)  # the copies queued on `stream` still read it
    return out
