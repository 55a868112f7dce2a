"""Point-to-point reshard (``Tensor.to_mesh`` / ``SendTensor``) on top of pack -> transfer -> unpack.

Mirrors, for the ranks whose data sits on this GPU:

* ``check_to_mesh``: the client-side validation of ``Tensor.to_mesh``
  (python/monarch/common/tensor.py:417-438), same messages;
* ``route``: which rank a worker sends to / receives from, from the ``from_ranks`` and
  ``to_ranks`` Slices of the message (monarch_tensor_worker/src/lib.rs:722-731);
* ``stream_send_tensor``: what ``StreamActor::send_tensor`` leaves in ``result``
  (monarch_tensor_worker/src/stream.rs:1470-1560).  NCCL send/recv tolerates non-contiguous
  tensors (``is_p2p`` in torch-sys-cuda/src/nccl.rs:300-316); here the sender's view is
  gathered in ``Slice::iter`` order into contiguous staging bytes, which is what an
  ``RdmaBuffer`` moves, and the receiver's fresh tensor of ``factory.size`` is those bytes.
"""
from __future__ import annotations

from typing import Dict, Optional, Sequence, Tuple

import torch

from . import _torch, staging
from .ndslice import Slice
from .reduce import Factory


def check_to_mesh(slicing_names: Sequence[str], slicing: Slice, mesh_names: Sequence[str], mesh_sizes: Sequence[int]):
    """Returns ``(from_ranks, broadcast_dims)`` or raises like ``Tensor.to_mesh``."""
    sizes, strides, broadcast_dims = [], [], []
    for name, size in zip(mesh_names, mesh_sizes):
        if name not in slicing_names:
            broadcast_dims.append(name)
            continue
        index = list(slicing_names).index(name)
        if slicing.sizes[index] != size:
            raise ValueError(f"dimension {name} of destination device_mesh has a different length than the source tensor")
        sizes.append(size)
        strides.append(slicing.strides[index])
    if len(sizes) != len(slicing_names):
        missing = set(slicing_names) - set(mesh_names)
        raise ValueError(f"destination mesh does not have dimensions {missing}")
    return Slice(offset=slicing.offset, sizes=sizes, strides=strides), broadcast_dims


def route(from_ranks: Slice, to_ranks: Slice, rank: int) -> Tuple[Optional[int], Optional[int]]:
    """``(from_rank, to_rank)`` of ``rank``: the i-th sender pairs with the i-th receiver."""
    def pair(mine: Slice, other: Slice) -> Optional[int]:
        try:
            return other[mine.index(rank)]
        except (ValueError, IndexError):
            return None
    return pair(to_ranks, from_ranks), pair(from_ranks, to_ranks)


def stream_send_tensor(world: Dict[int, Optional[torch.Tensor]], rank: int, from_rank: Optional[int],
                       to_rank: Optional[int], factory: Factory, stream=None) -> Optional[torch.Tensor]:
    """The tensor bound to ``result`` on ``rank`` (``None`` for a pure sender)."""
    if to_rank is None and from_rank is None:
        raise ValueError("tried to send tensor without a to/from rank")
    if from_rank == to_rank:
        src = world[rank]  # local value: a defensive copy, stream.rs:1497-1516
    elif from_rank is not None:
        src = world[from_rank]
    else:
        return None
    if src is None:  # errored upstream: zeros of the factory still go over the wire, stream.rs:976-989
        return factory.zeros()
    _torch.require_device(src)
    out = torch.empty(factory.size, dtype=factory.dtype, device=src.device)
    if out.numel() != src.numel():
        raise ValueError(f"factory size {tuple(factory.size)} does not match the sent tensor {tuple(src.shape)}")
    staging.pack(src, Slice.of_tensor(src), out=out.view(-1), stream=stream)
    return out
