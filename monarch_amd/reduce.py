"""Reduce over a device-mesh dimension, applied to the chunks one GPU holds.

Keeps the reference's API surface for this path:

* ``Reduction`` / ``Factory`` / ``Reduce``: field-for-field the worker message
  (monarch_messages/src/worker.rs:425-447,726-754).
* ``check_reduce_args``: the client-side validation of ``Tensor.reduce``
  (python/monarch/common/tensor.py:287-333) and the shape rule of ``_fake_reduce``
  (tensor.py:491-512), with the same exception types and messages.
* ``stream_reduce``: output placement and collective choice of ``StreamActor::reduce``
  (monarch_tensor_worker/src/stream.rs:1351-1468; python/monarch/worker/worker.py:200-255).

One GPU stands in for the whole group: ``group`` is the list of the members' local tensors
as they sit in this GPU's staging memory after the exchange, in member order.  The
arithmetic (fp32 accumulate in member order, one rounding) runs in ``mhip_reduce`` /
``mhip_reduce_scatter``; nothing is computed by torch.
"""
from __future__ import annotations

import ctypes as C
from dataclasses import dataclass, field
from enum import IntEnum
from typing import Dict, List, Optional, Sequence, Tuple, Union

import torch

from . import _lib, _torch
from ._lib import MhipError, check, lib, ptr_array
from .device_mesh import DeviceMesh
from .ndslice import Slice, slice_array

_valid_reduce = ("stack", "sum", "avg", "product", "min", "max", "band", "bor", "bxor")  # tensor.py:53-55


class ReduceOp(IntEnum):  # torch-sys-cuda/src/nccl.rs:285-292
    Sum = 0
    Prod = 1
    Max = 2
    Min = 3
    Avg = 4


@dataclass(frozen=True)
class Reduction:
    """``Reduction::Stack`` or ``Reduction::ReduceOp(op)``."""
    op: Optional[ReduceOp] = None  # None means Stack

    @property
    def is_stack(self) -> bool:
        return self.op is None

    @staticmethod
    def from_str(name: str) -> "Reduction":
        # python/monarch/common/messages.py:483-490: "stack" or an upper-cased ReduceOp name
        if name == "stack":
            return Reduction(None)
        table = {"sum": ReduceOp.Sum, "prod": ReduceOp.Prod, "max": ReduceOp.Max, "min": ReduceOp.Min,
                 "avg": ReduceOp.Avg}
        if name not in table:
            raise ValueError(f"unsupported reduction {name}")
        return Reduction(table[name])


@dataclass(frozen=True)
class Factory:
    size: Tuple[int, ...]
    dtype: torch.dtype
    layout: torch.layout = torch.strided
    device: torch.device = field(default_factory=lambda: torch.device("cuda", 0))

    @staticmethod
    def of(t: torch.Tensor) -> "Factory":
        return Factory(tuple(t.shape), t.dtype, t.layout, t.device)

    def zeros(self) -> torch.Tensor:
        return torch.zeros(self.size, dtype=self.dtype, layout=self.layout, device=self.device)


@dataclass
class Reduce:
    """``WorkerMessage::Reduce`` (monarch_messages/src/worker.rs:726-754)."""
    result: int
    tensor: int
    factory: Factory
    mesh: int
    stream: int
    dims: List[str]
    reduction: Reduction
    scatter: bool
    in_place: bool
    out: Optional[int]


def check_reduce_args(mesh_names: Sequence[str], mesh_sizes: Dict[str, int], shape: Sequence[int],
                      dims: Union[str, Sequence[str]], reduction: str = "sum", scatter: bool = False,
                      inplace: bool = False, out_shape: Optional[Sequence[int]] = None):
    """Validates like ``Tensor.reduce`` and returns ``(dims, result_shape)``."""
    if isinstance(dims, str):
        dims = (dims,)
    dims = tuple(dims)
    for d in dims:
        if d not in mesh_names:
            raise KeyError(f"dim {d} not found in {list(mesh_names)}")
    if len(dims) == 0:
        dims = tuple(mesh_names)
    if len(set(dims)) != len(dims):
        raise ValueError(f"reducing the same dimension twice: {dims}")
    if len(dims) > 1:
        if reduction == "stack" or scatter:
            raise ValueError(f"reduction {reduction} or scatter = {scatter} is not valid for multiple dimensions")
    if reduction not in _valid_reduce:
        raise ValueError(f"reduction {reduction} not supported, reductions are {_valid_reduce}")
    shape = tuple(shape)
    if inplace:
        if out_shape is not None:
            raise ValueError("`out` cannot be used with inplace reduce.")
        inplace_valid = (reduction == "gather" and scatter) or not scatter
        if not inplace_valid:
            raise ValueError(f"reduction {reduction} is not valid for in-place operation because "
                             "the output size will not match the input size.")
        return dims, shape
    n = mesh_sizes[dims[0]] if (reduction == "stack" or scatter) else -1
    if scatter:
        if len(shape) == 0 or shape[0] != n:
            raise TypeError(f"When scattering results the outer most dimension of tensor with sizes ({list(shape)} "
                            f"must match the size ({n})")
        result = shape if reduction == "stack" else shape[1:]
    else:
        result = (n, *shape) if reduction == "stack" else shape
    if out_shape is not None and tuple(out_shape) != tuple(result):
        raise ValueError(f"The given output shape, {torch.Size(out_shape)}, is incorrect. "
                         f"Reduce expects the shape to be {torch.Size(result)}.")
    return dims, tuple(result)


def all_reduce(out: torch.Tensor, group: Sequence[torch.Tensor], op: ReduceOp, stream=None) -> None:
    """Local combine of ``Communicator::all_reduce`` (torch-sys-cuda/src/nccl.rs:464-489):
    ``out = op(group)``; ``out`` may be one of the group's tensors (the in-place form)."""
    for t in (out, *group):
        _torch.require_contiguous(t)
    code = _torch.dtype_code(out.dtype)
    for t in group:
        if t.dtype != out.dtype:
            raise MhipError(_lib.ERR_TYPE_MISMATCH, "output tensor must have the same type as input tensor")
        if t.numel() != out.numel():
            raise MhipError(_lib.ERR_INPUT_SIZE_MISMATCH, "all group members must hold the same number of elements")
    check(lib().mhip_reduce(out.data_ptr(), ptr_array([t.data_ptr() for t in group]), len(group), out.numel(),
                            code, int(op), _torch.stream_handle(stream)))


def reduce_scatter_tensor(out: torch.Tensor, group: Sequence[torch.Tensor], rank: int, op: ReduceOp,
                          stream=None) -> None:
    """Local combine of ``Communicator::reduce_scatter_tensor`` (nccl.rs:661-703) for member
    ``rank``: ``out = op_g group[g].flat[rank*c : (rank+1)*c]`` with ``c = out.numel()``."""
    _torch.require_contiguous(out)
    for t in group:
        _torch.require_contiguous(t)
    n = len(group)
    for t in group:
        if t.dtype != out.dtype:
            raise MhipError(_lib.ERR_TYPE_MISMATCH, "output tensor must have the same type as input tensor")
        if t.numel() != out.numel() * n:
            raise MhipError(_lib.ERR_INPUT_SIZE_MISMATCH,
                            "input tensor must be the same size as output size times world size")
    code = _torch.dtype_code(out.dtype)
    c = out.numel()
    view = Slice(offset=rank * c, sizes=[c], strides=[1])
    check(lib().mhip_reduce_scatter(ptr_array([out.data_ptr()]), slice_array([view]), 1,
                                    ptr_array([t.data_ptr() for t in group]), None, c * n, n, code, int(op),
                                    _torch.stream_handle(stream)))


def reduce_scatter_views(outs: Sequence[torch.Tensor], out_views: Sequence[Slice], group: Sequence[torch.Tensor],
                         in_view: Optional[Slice], op: ReduceOp, stream=None) -> None:
    """Reduce ``group`` (each read through ``in_view``) and scatter the result through
    ``out_views`` (Slices of the reduced tensor) into contiguous ``outs`` in one pass."""
    for t in outs:
        _torch.require_contiguous(t)
    for t in group:
        _torch.require_device(t)
    code = _torch.dtype_code(outs[0].dtype)
    for t, v in zip(outs, out_views):
        if t.numel() != len(v):
            raise MhipError(_lib.ERR_OUTPUT_SIZE_MISMATCH, "output tensor does not match its view")
    in_numel = group[0].numel() if in_view is None else 0
    check(lib().mhip_reduce_scatter(ptr_array([t.data_ptr() for t in outs]), slice_array(out_views), len(outs),
                                    ptr_array([t.data_ptr() for t in group]),
                                    C.byref(in_view.c) if in_view is not None else None, in_numel, len(group), code,
                                    int(op), _torch.stream_handle(stream)))


def stream_reduce(group: Sequence[Optional[torch.Tensor]], rank: int, factory: Factory, reduction: Reduction,
                  scatter: bool, in_place: bool, out: Optional[torch.Tensor] = None, stream=None) -> torch.Tensor:
    """What ``StreamActor::reduce`` leaves in ``result`` on member ``rank`` of the group.

    ``group[g]`` is member g's local tensor; ``None`` stands for an input that errored
    upstream and is replaced by zeros of ``factory`` (stream.rs:976-989).
    """
    n = len(group)
    group = [factory.zeros() if t is None else t for t in group]
    local = group[rank]
    if reduction.is_stack:
        for t in group:
            _torch.require_contiguous(t)
            if t.dtype != local.dtype or t.numel() != local.numel():
                raise MhipError(_lib.ERR_TYPE_MISMATCH, "all group members must share dtype and size")
        ptrs = ptr_array([t.data_ptr() for t in group])
        if scatter:  # all_to_all_single, stream.rs:1381-1399
            output = local if in_place else (out if out is not None else torch.empty_like(local))
            _torch.require_contiguous(output)
            if output.numel() != local.numel() or output.dtype != local.dtype:
                raise MhipError(_lib.ERR_OUTPUT_SIZE_MISMATCH, "output tensor must match the input tensor")
            check(lib().mhip_stack_scatter(output.data_ptr(), ptrs, n, rank, local.numel(), local.element_size(),
                                           _torch.stream_handle(stream)))
            return output
        if in_place:
            raise ValueError("in-place, non-scatter not supported for stack reduce")
        output = out if out is not None else torch.empty((n, *factory.size), dtype=factory.dtype, device=local.device)
        _torch.require_contiguous(output)
        if output.numel() != n * local.numel() or output.dtype != local.dtype:
            raise MhipError(_lib.ERR_OUTPUT_SIZE_MISMATCH,
                            "output tensor size must be equal to world size times input tensor size")
        # all_gather_into_tensor, stream.rs:1408-1417
        check(lib().mhip_stack(output.data_ptr(), ptrs, n, local.numel(), local.element_size(),
                               _torch.stream_handle(stream)))
        return output
    op = reduction.op
    if scatter:
        if in_place:
            raise ValueError("in-place, scatter not supported for reduce")
        output = out if out is not None else torch.empty(factory.size[1:], dtype=factory.dtype, device=local.device)
        reduce_scatter_tensor(output, group, rank, op, stream)
        return output
    if in_place:
        output = local
    elif out is not None:
        output = out  # the reference first does out.copy_(in); the fused combine overwrites it anyway
    else:
        output = torch.empty_like(local)  # deep_clone in the reference
    members = list(group)
    members[rank] = local
    all_reduce(output, members, op, stream)
    return output


def reduce(world: Dict[int, Optional[torch.Tensor]], mesh: DeviceMesh, dims: Union[str, Sequence[str]],
           reduction: str = "sum", scatter: bool = False, inplace: bool = False,
           out: Optional[torch.Tensor] = None, stream=None) -> torch.Tensor:
    """``Tensor.reduce`` for the mesh's owning rank, with every rank's local tensor resident
    on this GPU (``world[rank]``)."""
    local = world[mesh.rank]
    shape = tuple(local.shape)
    dims, _ = check_reduce_args(mesh.names, mesh.sizes(), shape, dims, reduction, scatter, inplace,
                                None if out is None else tuple(out.shape))
    dims = sorted(dims)  # WorkerActor::reduce sorts for stable lookup, monarch_tensor_worker/src/lib.rs:621
    members = mesh.get_ranks_for_dim_slice(dims)
    group = [world[r] for r in members]
    name = {"product": "prod"}.get(reduction, reduction)
    return stream_reduce(group, members.index(mesh.rank), Factory.of(local), Reduction.from_str(name), scatter,
                         inplace, out, stream)
