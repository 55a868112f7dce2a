"""ctypes binding of ``libmonarch_hip.so`` (the C ABI in ``include/monarch_hip.h``).

This is the Python counterpart of the Rust ``hip-sys`` extern block: every symbol the
header declares is bound here with explicit argument types.  There is no fallback: if
the shared library is missing, importing a symbol raises ``MonarchHipNotBuilt``.
"""
from __future__ import annotations

import ctypes as C
import os
from typing import Sequence

_HERE = os.path.dirname(os.path.abspath(__file__))
LIB_PATH = os.path.join(_HERE, "libmonarch_hip.so")

MHIP_MAX_DIMS = 32

# status codes (include/monarch_hip.h)
SUCCESS = 0
ERR_INVALID_DIMS = 10001
ERR_NONRECTANGULAR_SHAPE = 10002
ERR_NONUNIQUE_STRIDES = 10003
ERR_STRIDE_TOO_SMALL = 10004
ERR_INDEX_OUT_OF_RANGE = 10005
ERR_VALUE_NOT_IN_SLICE = 10006
ERR_INCOMPATIBLE_VIEW = 10007
ERR_NONCONTIGUOUS = 10008
ERR_EMPTY_RANGE = 10009
ERR_DIMENSION_OUT_OF_RANGE = 10010
ERR_INVALID_DATA_TYPE = 10101
ERR_NONCONTIGUOUS_TENSOR = 10102
ERR_INVALID_DEVICE = 10103
ERR_FLOAT8_REDUCTION = 10104
ERR_TYPE_MISMATCH = 10105
ERR_OUTPUT_SIZE_MISMATCH = 10106
ERR_INPUT_SIZE_MISMATCH = 10107
ERR_UNDEFINED_TENSOR = 10108
ERR_INVALID_ARGUMENT = 10201
ERR_UNSUPPORTED_OP = 10202
ERR_TOO_MANY_INPUTS = 10203
ERR_UNSUPPORTED_BLOCK = 10204
ERR_BUFFER_TOO_SMALL = 10205
ERR_SCRATCH_TOO_SMALL = 10206
ERR_WQE_OVERFLOW = 10207
ERR_MESH_DIM_LENGTH_MISMATCH = 10301
ERR_MESH_DIM_MISSING = 10302
NO_RANK = (1 << 64) - 1

STATUS_NAMES = {
    ERR_INVALID_DIMS: "InvalidDims", ERR_NONRECTANGULAR_SHAPE: "NonrectangularShape",
    ERR_NONUNIQUE_STRIDES: "NonuniqueStrides", ERR_STRIDE_TOO_SMALL: "StrideTooSmall",
    ERR_INDEX_OUT_OF_RANGE: "IndexOutOfRange", ERR_VALUE_NOT_IN_SLICE: "ValueNotInSlice",
    ERR_INCOMPATIBLE_VIEW: "IncompatibleView", ERR_NONCONTIGUOUS: "NonContiguous",
    ERR_EMPTY_RANGE: "EmptyRange", ERR_DIMENSION_OUT_OF_RANGE: "DimensionOutOfRange",
    ERR_INVALID_DATA_TYPE: "InvalidDataType", ERR_NONCONTIGUOUS_TENSOR: "NoncontiguousTensor",
    ERR_INVALID_DEVICE: "InvalidDevice", ERR_FLOAT8_REDUCTION: "Float8Reduction",
    ERR_TYPE_MISMATCH: "TypeMismatch", ERR_OUTPUT_SIZE_MISMATCH: "OutputSizeMismatch",
    ERR_INPUT_SIZE_MISMATCH: "InputSizeMismatch", ERR_UNDEFINED_TENSOR: "UndefinedTensor",
    ERR_INVALID_ARGUMENT: "InvalidArgument", ERR_UNSUPPORTED_OP: "UnsupportedOp",
    ERR_TOO_MANY_INPUTS: "TooManyInputs", ERR_UNSUPPORTED_BLOCK: "UnsupportedBlock",
    ERR_BUFFER_TOO_SMALL: "BufferTooSmall", ERR_SCRATCH_TOO_SMALL: "ScratchTooSmall", ERR_WQE_OVERFLOW: "WqeOverflow",
    ERR_MESH_DIM_LENGTH_MISMATCH: "MeshDimLengthMismatch",
    ERR_MESH_DIM_MISSING: "MeshDimMissing",
}

# dtype codes (c10::ScalarType numbering)
DTYPE_U8, DTYPE_I8, DTYPE_I32, DTYPE_I64 = 0, 1, 3, 4
DTYPE_F16, DTYPE_F32, DTYPE_F64, DTYPE_BF16 = 5, 6, 7, 15
DTYPE_F8E5M2, DTYPE_F8E4M3FN, DTYPE_F8E5M2FNUZ, DTYPE_F8E4M3FNUZ = 23, 24, 25, 26
OP_SUM, OP_PROD, OP_MAX, OP_MIN, OP_AVG = 0, 1, 2, 3, 4


class MonarchHipNotBuilt(ImportError):
    pass


class MhipError(RuntimeError):
    """A non-zero status from the C ABI.  ``name`` is the class (``StrideTooSmall``,
    ``Float8Reduction`` ...) or ``HipError`` for a passed-through hipError_t."""

    def __init__(self, status: int, text: str):
        self.status = status
        self.name = STATUS_NAMES.get(status, "HipError" if 0 < status < 10000 else "Unknown")
        super().__init__(f"{self.name} ({status}): {text}")


class RdmaBufferC(C.Structure):
    _fields_ = [("addr", C.c_void_p), ("size", C.c_size_t)]


class WqeParamsC(C.Structure):
    """``mhip_wqe_params_t`` == ``wqe_params_t`` (rdmaxcel-sys/src/rdmaxcel.h:26-39)."""
    _fields_ = [("laddr", C.c_size_t), ("lkey", C.c_uint32), ("length", C.c_size_t), ("wr_id", C.c_uint64),
                ("signaled", C.c_uint8), ("op_type", C.c_uint32), ("raddr", C.c_size_t), ("rkey", C.c_uint32),
                ("qp_num", C.c_uint32), ("buf", C.c_void_p), ("dbrec", C.c_void_p), ("wqe_cnt", C.c_uint32)]


class CqePollParamsC(C.Structure):
    """``mhip_cqe_poll_params_t`` == ``cqe_poll_params_t`` (rdmaxcel.h:42-48)."""
    _fields_ = [("cqe_buf", C.c_void_p), ("cqe_size", C.c_uint32), ("consumer_index", C.c_uint32),
                ("cqe_cnt", C.c_uint32), ("dbrec", C.c_void_p)]


class SliceC(C.Structure):
    _fields_ = [("offset", C.c_uint64), ("ndim", C.c_uint32),
                ("sizes", C.POINTER(C.c_uint64)), ("strides", C.POINTER(C.c_uint64))]


_u64p = C.POINTER(C.c_uint64)
_u32p = C.POINTER(C.c_uint32)
_slicep = C.POINTER(SliceC)
_vp = C.c_void_p
_vpp = C.POINTER(C.c_void_p)
_bufp = C.POINTER(RdmaBufferC)
_cpp = C.POINTER(C.c_char_p)
_wqep = C.POINTER(WqeParamsC)
_cqep = C.POINTER(CqePollParamsC)

# name -> (restype, argtypes); mirrors include/monarch_hip.h declaration by declaration
SIGNATURES = {
    "mhip_error_string": (C.c_char_p, [C.c_int]),
    "mhip_version": (C.c_int, []),
    "mhip_dtype_size": (C.c_uint32, [C.c_int]),
    "mhip_slice_validate": (C.c_int, [C.c_uint64, _u64p, C.c_uint32, _u64p, C.c_uint32]),
    "mhip_slice_len": (C.c_int, [_slicep, _u64p]),
    "mhip_slice_is_contiguous": (C.c_int, [_slicep, C.POINTER(C.c_int)]),
    "mhip_slice_get": (C.c_int, [_slicep, C.c_uint64, _u64p]),
    "mhip_slice_location": (C.c_int, [_slicep, _u64p, C.c_uint32, _u64p]),
    "mhip_slice_coordinates": (C.c_int, [_slicep, C.c_uint64, _u64p]),
    "mhip_slice_index": (C.c_int, [_slicep, C.c_uint64, _u64p]),
    "mhip_slice_iter": (C.c_int, [_slicep, C.c_uint64, C.c_uint64, _vp, _u64p]),
    "mhip_slice_select": (C.c_int, [_slicep, C.c_uint32, C.c_uint64, C.c_uint64, C.c_uint64, _u64p, _u64p, _u64p]),
    "mhip_slice_at": (C.c_int, [_slicep, C.c_uint32, C.c_uint64, _u64p, _u64p, _u64p]),
    "mhip_slice_subview": (C.c_int, [_slicep, _u64p, C.c_uint32, _u64p, C.c_uint32, _u64p]),
    "mhip_slice_view": (C.c_int, [_slicep, _u64p, C.c_uint32, _u64p]),
    "mhip_slice_enforce_embedding": (C.c_int, [_slicep, _slicep]),
    "mhip_slice_bounds": (C.c_int, [_slicep, _u64p, _u64p]),
    "mhip_mesh_dim_members": (C.c_int, [_slicep, C.c_uint64, C.c_uint32, _u64p, _u64p]),
    "mhip_mesh_ranks_for_dims": (C.c_int, [_slicep, C.c_uint64, _u32p, C.c_uint32, _u64p, C.c_uint64, _u64p]),
    "mhip_slice_pack": (C.c_int, [_vp, _vp, _slicep, C.c_uint32, _vp]),
    "mhip_slice_unpack": (C.c_int, [_vp, _vp, _slicep, C.c_uint32, _vp]),
    "mhip_slice_pack_many": (C.c_int, [_vpp, _vp, _slicep, C.c_uint32, C.c_uint32, _vp]),
    "mhip_slice_unpack_many": (C.c_int, [_vp, _vpp, _slicep, C.c_uint32, C.c_uint32, _vp]),
    "mhip_flat_pack": (C.c_int, [_vp, _vp, _vp, C.c_uint32, C.c_uint64, C.c_uint32, _vp, _vp]),
    "mhip_flat_unpack": (C.c_int, [_vp, _vp, _vp, C.c_uint32, C.c_uint64, C.c_uint32, _vp, _vp]),
    "mhip_reduce": (C.c_int, [_vp, _vpp, C.c_uint32, C.c_uint64, C.c_int, C.c_int, _vp]),
    "mhip_reduce_scatter": (C.c_int, [_vpp, _slicep, C.c_uint32, _vpp, _slicep, C.c_uint64, C.c_uint32,
                                      C.c_int, C.c_int, _vp]),
    "mhip_stack": (C.c_int, [_vp, _vpp, C.c_uint32, C.c_uint64, C.c_uint32, _vp]),
    "mhip_stack_scatter": (C.c_int, [_vp, _vpp, C.c_uint32, C.c_uint32, C.c_uint64, C.c_uint32, _vp]),
    "mhip_buffer_read_into": (C.c_int, [_bufp, _bufp, _vp]),
    "mhip_buffer_write_from": (C.c_int, [_bufp, _bufp, _vp]),
    "mhip_buffer_transfer": (C.c_int, [_vp, _vp, C.c_size_t, C.c_size_t, _vp, _u32p]),
    "mhip_buffer_transfer_many": (C.c_int, [_vp, _vp, _vp, C.c_uint32, C.c_size_t, _vp, _vp]),
    "mhip_send_tensor_route": (C.c_int, [_slicep, _slicep, C.c_uint64, _u64p, _u64p]),
    "mhip_to_mesh_from_ranks": (C.c_int, [_cpp, _slicep, _cpp, _u64p, C.c_uint32, _u64p, _u64p, _u32p, _u32p, _u32p, _u32p]),
    "mhip_send_tensor": (C.c_int, [_vp, C.c_size_t, _vp, _slicep, C.c_uint32, _vp, _vp]),
    "mhip_rdmaxcel_send_wqe": (C.c_int, [_wqep, _vp]),
    "mhip_rdmaxcel_recv_wqe": (C.c_int, [_wqep, _vp]),
    "mhip_rdmaxcel_db_ring": (C.c_int, [_vp, _vp, _vp]),
    "mhip_rdmaxcel_ring_doorbells": (C.c_int, [_vp, _vp, C.c_uint32, C.c_uint32, C.c_uint32, C.c_uint32, _vp]),
    "mhip_rdmaxcel_cqe_poll": (C.c_int, [_vp, _cqep, _vp]),
    "mhip_rdmaxcel_post_transfer": (C.c_int, [_wqep, C.c_size_t, _u32p, _vp]),
    "mhip_rdmaxcel_send_wqe_host": (C.c_int, [_wqep]),
    "mhip_rdmaxcel_recv_wqe_host": (C.c_int, [_wqep]),
    "mhip_rdmaxcel_db_ring_host": (C.c_int, [_vp, _vp]),
    "mhip_rdmaxcel_cqe_poll_host": (C.c_int, [C.POINTER(C.c_int32), _cqep]),
    "mhip_fp8_quantize": (C.c_int, [_vp, _vp, _vp, C.c_uint64, C.c_uint32, _vp]),
    "mhip_fp8_dequant_accumulate": (C.c_int, [_vp, _vp, _vp, C.c_uint64, C.c_uint32, _vp]),
    "mhip_fp8_dequant_accumulate_many": (C.c_int, [_vp, _vpp, _vpp, C.c_uint32, C.c_uint64, C.c_uint32, C.c_int, _vp]),
    "mhip_fp8_quantize_bucket": (C.c_int, [_vp, _vp, _vp, _vp, C.c_uint32, C.c_uint64, C.c_uint32, _vp, _vp]),
    "mhip_fp8_dequant_accumulate_bucket": (C.c_int, [_vp, _vp, _vp, _vp, C.c_uint32, C.c_uint64, C.c_uint32, _vp, _vp]),
    "mhip_fp8_dequant_accumulate_bucket_many": (C.c_int, [_vp, _vpp, _vpp, C.c_uint32, _vp, C.c_uint32, C.c_uint64, C.c_uint32, _vp, _vp]),
    "mhip_fp8_quantize_bucket_static": (C.c_int, [_vp, _vp, _vp, _vp, C.c_uint32, C.c_uint64, C.c_uint32, _vp]),
    "mhip_bucket_index_bytes": (C.c_int, [C.c_uint64, C.c_uint32, C.POINTER(C.c_size_t)]),
    "mhip_bucket_index_build": (C.c_int, [_vp, _vp, C.c_uint32, C.c_uint64, C.c_uint32, _vp]),
    "mhip_device_count": (C.c_int, [C.POINTER(C.c_int)]),
    "mhip_set_device": (C.c_int, [C.c_int]),
    "mhip_device_synchronize": (C.c_int, []),
    "mhip_stream_create": (C.c_int, [_vpp]),
    "mhip_stream_destroy": (C.c_int, [_vp]),
    "mhip_stream_synchronize": (C.c_int, [_vp]),
    "mhip_event_create": (C.c_int, [_vpp]),
    "mhip_event_destroy": (C.c_int, [_vp]),
    "mhip_event_record": (C.c_int, [_vp, _vp]),
    "mhip_event_synchronize": (C.c_int, [_vp]),
    "mhip_event_elapsed_ms": (C.c_int, [C.POINTER(C.c_float), _vp, _vp]),
    "mhip_stream_wait_event": (C.c_int, [_vp, _vp]),
    "mhip_malloc": (C.c_int, [_vpp, C.c_size_t]),
    "mhip_free": (C.c_int, [_vp]),
    "mhip_memcpy_htod": (C.c_int, [_vp, _vp, C.c_size_t, _vp]),
    "mhip_memcpy_dtoh": (C.c_int, [_vp, _vp, C.c_size_t, _vp]),
    "mhip_memset": (C.c_int, [_vp, C.c_int, C.c_size_t, _vp]),
    "mhip_staging_alloc": (C.c_int, [_vpp, C.POINTER(C.c_size_t), C.c_size_t, C.c_int]),
    "mhip_staging_free": (C.c_int, [_vp, C.c_size_t]),
    "mhip_staging_slot_pitch": (C.c_int, [C.c_size_t, C.POINTER(C.c_size_t)]),
    "mhip_pointer_is_device": (C.c_int, [_vp, C.POINTER(C.c_int)]),
    "mhip_export_dmabuf": (C.c_int, [C.POINTER(C.c_int), _vp, C.c_size_t]),
}

_lib = None


def lib() -> C.CDLL:
    """The loaded library.  Raises ``MonarchHipNotBuilt`` when it has not been built
    (``python -c 'import __graft_entry__ as g; g.build()'`` or ``make -C monarch_amd/csrc``)."""
    global _lib
    if _lib is None:
        if not os.path.exists(LIB_PATH):
            raise MonarchHipNotBuilt(
                f"{LIB_PATH} is missing: build it with `make -C {os.path.join(_HERE, 'csrc')}`; "
                "there is no CPU fallback for the device path")
        handle = C.CDLL(LIB_PATH)
        for name, (res, args) in SIGNATURES.items():
            fn = getattr(handle, name)  # AttributeError if the header and the library drift apart
            fn.restype = res
            fn.argtypes = args
        _lib = handle
    return _lib


def check(status: int) -> None:
    if status != SUCCESS:
        raise MhipError(status, lib().mhip_error_string(status).decode())


def u64_array(values: Sequence[int]):
    return (C.c_uint64 * max(1, len(values)))(*values)


def ptr_array(values: Sequence[int]):
    return (C.c_void_p * max(1, len(values)))(*values)
