"""PyTorch plumbing: device pointers, dtypes and the current HIP stream.  Nothing here computes."""
from __future__ import annotations

import torch

from . import _lib

_DTYPES = {
    torch.uint8: _lib.DTYPE_U8, torch.int8: _lib.DTYPE_I8, torch.int32: _lib.DTYPE_I32,
    torch.int64: _lib.DTYPE_I64, torch.float16: _lib.DTYPE_F16, torch.float32: _lib.DTYPE_F32,
    torch.float64: _lib.DTYPE_F64, torch.bfloat16: _lib.DTYPE_BF16, torch.bool: _lib.DTYPE_U8,
    torch.float8_e5m2: _lib.DTYPE_F8E5M2, torch.float8_e4m3fn: _lib.DTYPE_F8E4M3FN,
    torch.float8_e5m2fnuz: _lib.DTYPE_F8E5M2FNUZ, torch.float8_e4m3fnuz: _lib.DTYPE_F8E4M3FNUZ,
}


def dtype_code(dtype: torch.dtype) -> int:
    if dtype not in _DTYPES:
        raise _lib.MhipError(_lib.ERR_INVALID_DATA_TYPE, f"invalid data type: {dtype}")
    return _DTYPES[dtype]


def stream_handle(stream=None) -> int:
    """hipStream_t of ``stream`` (a torch.cuda.Stream) or of torch's current stream."""
    if stream is None:
        stream = torch.cuda.current_stream()
    return int(stream.cuda_stream)


def storage_ptr(t: torch.Tensor) -> int:
    """Address of element 0 of the tensor's storage (the base a Slice offset counts from)."""
    return t.untyped_storage().data_ptr()


def require_device(t: torch.Tensor) -> None:
    # check order of torch-sys-cuda/src/nccl.rs:300-316: defined -> on device -> dense
    if t is None:
        raise _lib.MhipError(_lib.ERR_UNDEFINED_TENSOR, "undefined tensor used for operation")
    if not t.is_cuda:
        raise _lib.MhipError(_lib.ERR_INVALID_DEVICE, f"tensor must be on a GPU device, got: {t.device.type}")
    if t.is_sparse:
        raise _lib.MhipError(_lib.ERR_INVALID_ARGUMENT, "got sparse tensor, only dense tensors allowed")


def require_contiguous(t: torch.Tensor) -> None:
    require_device(t)
    if not t.is_contiguous():
        raise _lib.MhipError(_lib.ERR_NONCONTIGUOUS_TENSOR, "tensor used in collective must be contiguous")
