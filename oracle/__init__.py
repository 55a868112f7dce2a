"""ctypes front-end of the CPU oracle (``monarch_oracle.c``).

TEST INFRASTRUCTURE ONLY: imported by ``tests/``, ``__graft_entry__.smoke()`` and the
``cpu_baseline`` leg of ``bench.py``.  The product package never imports this module.
All arrays are numpy arrays on the host.
"""
from __future__ import annotations

import ctypes as C
import os
import subprocess
from typing import List, Sequence, Tuple

import numpy as np

_HERE = os.path.dirname(os.path.abspath(__file__))
_SO = os.path.join(_HERE, "libmonarch_oracle.so")

ERR_NAMES = {
    0: "Ok",
    1: "InvalidDims",
    2: "NonrectangularShape",
    3: "NonuniqueStrides",
    4: "StrideTooSmall",
    5: "IndexOutOfRange",
    6: "ValueNotInSlice",
    7: "IncompatibleView",
    8: "NonContiguous",
    9: "EmptyRange",
    10: "DimensionOutOfRange",
}


def build(force: bool = False) -> str:
    src = os.path.join(_HERE, "monarch_oracle.c")
    if force or not os.path.exists(_SO) or os.path.getmtime(_SO) < os.path.getmtime(src):
        subprocess.check_call(["make", "-C", _HERE, "-B", "libmonarch_oracle.so"],
                              stdout=subprocess.DEVNULL)
    return _SO


class OracleError(Exception):
    def __init__(self, code: int):
        super().__init__(ERR_NAMES.get(code, str(code)))
        self.code = code
        self.name = ERR_NAMES.get(code, str(code))


class _CSlice(C.Structure):
    _fields_ = [("offset", C.c_uint64), ("ndim", C.c_uint32),
                ("sizes", C.POINTER(C.c_uint64)), ("strides", C.POINTER(C.c_uint64))]


_lib = None


def load(path: str):
    """A handle on an oracle build at ``path`` with the non-int return types declared."""
    h = C.CDLL(path)
    h.o_slice_len.restype = C.c_uint64
    h.o_slice_iter.restype = C.c_uint64
    h.o_mesh_ranks_for_dims.restype = C.c_int64
    h.o_e4m3fn_encode.restype = C.c_uint8
    h.o_e4m3fn_encode.argtypes = [C.c_float, C.c_int]
    h.o_e4m3fn_decode.restype = C.c_float
    h.o_e4m3fn_decode.argtypes = [C.c_uint8]
    return h


def lib():
    global _lib
    if _lib is None:
        build()
        _lib = load(_SO)
    return _lib


def _u64(xs: Sequence[int]):
    return (C.c_uint64 * max(1, len(xs)))(*xs)


class OSlice:
    """Restatement of ``ndslice::Slice``; ``OSlice(...)`` validates like ``Slice::new``,
    ``OSlice.unchecked(...)`` constructs like ``new_row_major``/``subview`` do."""

    def __init__(self, offset: int, sizes: Sequence[int], strides: Sequence[int], _validate=True):
        self.offset, self.sizes, self.strides = int(offset), list(sizes), list(strides)
        if _validate:
            rc = lib().o_slice_new(C.c_uint64(self.offset), _u64(self.sizes), C.c_uint32(len(self.sizes)),
                                   _u64(self.strides), C.c_uint32(len(self.strides)))
            if rc:
                raise OracleError(rc)
        self._keep = (_u64(self.sizes), _u64(self.strides))
        self.c = _CSlice(self.offset, len(self.sizes), self._keep[0], self._keep[1])

    @classmethod
    def unchecked(cls, offset, sizes, strides):
        return cls(offset, sizes, strides, _validate=False)

    @classmethod
    def row_major(cls, sizes):
        strides, acc = [], 1
        for n in reversed(list(sizes)):
            strides.append(acc)
            acc *= n
        return cls.unchecked(0, sizes, list(reversed(strides)))

    def __repr__(self):
        return f"OSlice(offset={self.offset}, sizes={self.sizes}, strides={self.strides})"

    @property
    def ndim(self):
        return len(self.sizes)

    def __len__(self):
        return int(lib().o_slice_len(C.byref(self.c)))

    def is_contiguous(self) -> bool:
        return bool(lib().o_slice_is_contiguous(C.byref(self.c)))

    def get(self, i: int) -> int:
        out = C.c_uint64()
        rc = lib().o_slice_get(C.byref(self.c), C.c_uint64(i), C.byref(out))
        if rc:
            raise OracleError(rc)
        return out.value

    def location(self, coord: Sequence[int]) -> int:
        out = C.c_uint64()
        rc = lib().o_slice_location(C.byref(self.c), _u64(coord), C.c_uint32(len(coord)), C.byref(out))
        if rc:
            raise OracleError(rc)
        return out.value

    def iter(self) -> np.ndarray:
        n = len(self)
        out = np.empty(max(n, 1), dtype=np.uint64)
        lib().o_slice_iter(C.byref(self.c), out.ctypes.data_as(C.c_void_p), C.c_uint64(n))
        return out[:n]

    def coordinates(self, value: int) -> List[int]:
        out = _u64([0] * self.ndim)
        rc = lib().o_slice_coordinates(C.byref(self.c), C.c_uint64(value), out)
        if rc:
            raise OracleError(rc)
        return list(out)[: self.ndim]

    def index(self, value: int) -> int:
        out = C.c_uint64()
        rc = lib().o_slice_index(C.byref(self.c), C.c_uint64(value), C.byref(out))
        if rc:
            raise OracleError(rc)
        return out.value

    def contains(self, value: int) -> bool:
        try:
            self.coordinates(value)
            return True
        except OracleError:
            return False

    def select(self, dim, begin, end, step) -> "OSlice":
        off = C.c_uint64()
        sz, st = _u64([0] * self.ndim), _u64([0] * self.ndim)
        rc = lib().o_slice_select(C.byref(self.c), C.c_uint32(dim), C.c_uint64(begin), C.c_uint64(end),
                                  C.c_uint64(step), C.byref(off), sz, st)
        if rc:
            raise OracleError(rc)
        return OSlice.unchecked(off.value, list(sz)[: self.ndim], list(st)[: self.ndim])

    def at(self, dim, index) -> "OSlice":
        off = C.c_uint64()
        sz, st = _u64([0] * self.ndim), _u64([0] * self.ndim)
        rc = lib().o_slice_at(C.byref(self.c), C.c_uint32(dim), C.c_uint64(index), C.byref(off), sz, st)
        if rc:
            raise OracleError(rc)
        return OSlice.unchecked(off.value, list(sz)[: self.ndim - 1], list(st)[: self.ndim - 1])

    def subview(self, starts, lens) -> "OSlice":
        off = C.c_uint64()
        rc = lib().o_slice_subview(C.byref(self.c), _u64(starts), C.c_uint32(len(starts)), _u64(lens),
                                   C.c_uint32(len(lens)), C.byref(off))
        if rc:
            raise OracleError(rc)
        return OSlice.unchecked(off.value, list(lens), list(self.strides))

    def view(self, new_sizes) -> "OSlice":
        st = _u64([0] * len(new_sizes))
        rc = lib().o_slice_view(C.byref(self.c), _u64(new_sizes), C.c_uint32(len(new_sizes)), st)
        if rc:
            raise OracleError(rc)
        return OSlice.unchecked(0, list(new_sizes), list(st)[: len(new_sizes)])

    def enforce_embedding(self, other: "OSlice") -> "OSlice":
        rc = lib().o_slice_enforce_embedding(C.byref(self.c), C.byref(other.c))
        if rc:
            raise OracleError(rc)
        return self


def _ptr(a: np.ndarray):
    return a.ctypes.data_as(C.c_void_p)


def pack(src_base: np.ndarray, s: OSlice, runs: bool = False, threads: bool = False) -> np.ndarray:
    """dst[i] = src_base.flat[s.get(i)]; ``src_base`` is the flat storage.  ``runs`` copies one
    contiguous run per memcpy; ``threads`` also spreads the runs over every host core."""
    src_base = np.ascontiguousarray(src_base).reshape(-1)
    dst = np.empty(len(s), dtype=src_base.dtype)
    fn = lib().o_pack_runs_mt if threads else lib().o_pack_runs if runs else lib().o_slice_pack
    fn(_ptr(dst), _ptr(src_base), C.byref(s.c), C.c_uint32(src_base.itemsize))
    return dst


def unpack(dst_base: np.ndarray, src: np.ndarray, s: OSlice) -> None:
    """dst_base.flat[s.get(i)] = src[i], in place on the flat storage ``dst_base``."""
    assert dst_base.flags.c_contiguous and src.flags.c_contiguous and dst_base.dtype == src.dtype
    lib().o_slice_unpack(_ptr(dst_base), _ptr(src), C.byref(s.c), C.c_uint32(src.itemsize))


_REDUCE = {"float32": "o_reduce_f32", "float64": "o_reduce_f64", "uint16": "o_reduce_bf16",
           "uint8": "o_reduce_u8", "int32": "o_reduce_i32", "int64": "o_reduce_i64"}

SUM, AVG = 0, 4


def num_threads() -> int:
    """Host threads the ``threads=True`` variants use."""
    return int(lib().o_num_threads())


def reduce(ins: Sequence[np.ndarray], op: int = SUM, out: np.ndarray | None = None, half: bool = False,
           threads: bool = False) -> np.ndarray:
    """Elementwise Sum/Avg over ``ins``.  bf16 data is passed as uint16 bit patterns
    (``half=True``: the uint16 patterns are IEEE binary16 instead).  ``threads`` runs the same
    loop on every host core (fp32 and bf16 only)."""
    ins = [np.ascontiguousarray(x).reshape(-1) for x in ins]
    dt = ins[0].dtype
    if half:
        assert dt == np.uint16
        if out is None:
            out = np.empty_like(ins[0])
        ptrs = (C.c_void_p * len(ins))(*[x.ctypes.data for x in ins])
        lib().o_reduce_f16(_ptr(out), ptrs, C.c_uint32(len(ins)), C.c_uint64(ins[0].size), C.c_int(op))
        return out
    if out is None:
        out = np.empty_like(ins[0])
    ptrs = (C.c_void_p * len(ins))(*[x.ctypes.data for x in ins])
    name = _REDUCE[dt.name]
    if threads:
        assert dt.name in ("float32", "uint16")
        name += "_mt"
    args = [_ptr(out), ptrs, C.c_uint32(len(ins)), C.c_uint64(ins[0].size)]
    if dt.name in ("float32", "float64", "uint16"):
        args.append(C.c_int(op))
    else:
        assert op == SUM
    getattr(lib(), name)(*args)
    return out


PROD, MAX, MIN = 1, 2, 3
_DTYPE_CODES = {"uint8": 0, "int8": 1, "int32": 3, "int64": 4, "float32": 6, "float64": 7}


def reduce_op(ins: Sequence[np.ndarray], op: int, kind: str | None = None) -> np.ndarray:
    """Any ReduceOp (SUM, PROD, MAX, MIN, AVG) over ``ins``.  uint16 arrays are bit patterns: ``kind`` says
    whether of bf16 (default) or of IEEE half ("f16")."""
    ins = [np.ascontiguousarray(x).reshape(-1) for x in ins]
    dt = ins[0].dtype
    code = (5 if kind == "f16" else 15) if dt == np.uint16 else _DTYPE_CODES[dt.name]
    out = np.empty_like(ins[0])
    ptrs = (C.c_void_p * len(ins))(*[x.ctypes.data for x in ins])
    rc = lib().o_reduce_op(_ptr(out), ptrs, C.c_uint32(len(ins)), C.c_uint64(ins[0].size), C.c_int(code), C.c_int(op))
    assert rc == 0
    return out


def stack(ins: Sequence[np.ndarray]) -> np.ndarray:
    """Reduction::Stack without scatter: ``out[g] = ins[g]``, shape ``[n, numel]``."""
    ins = [np.ascontiguousarray(x).reshape(-1) for x in ins]
    out = np.empty((len(ins), ins[0].size), dtype=ins[0].dtype)
    ptrs = (C.c_void_p * len(ins))(*[x.ctypes.data for x in ins])
    lib().o_stack(_ptr(out), ptrs, C.c_uint32(len(ins)), C.c_uint64(ins[0].size), C.c_uint32(ins[0].itemsize))
    return out


def stack_scatter(ins: Sequence[np.ndarray], rank: int, out: np.ndarray | None = None) -> np.ndarray:
    """Reduction::Stack with scatter (all_to_all_single) as member ``rank`` sees it; ``out`` may be ``ins[rank]``."""
    assert all(x.flags.c_contiguous for x in ins)
    if out is None:
        out = np.empty_like(ins[0].reshape(-1))
    ptrs = (C.c_void_p * len(ins))(*[x.ctypes.data for x in ins])
    rc = lib().o_stack_scatter(_ptr(out), ptrs, C.c_uint32(len(ins)), C.c_uint32(rank), C.c_uint64(ins[0].size),
                               C.c_uint32(ins[0].itemsize))
    if rc:
        raise ValueError("numel must be a multiple of the group size and rank inside the group")
    return out


NO_RANK = (1 << 64) - 1


def send_tensor_route(from_ranks: OSlice, to_ranks: OSlice, rank: int):
    """``(from_rank, to_rank)`` of ``rank``, ``None`` where the reference has ``Option::None``."""
    fr, to = C.c_uint64(), C.c_uint64()
    lib().o_send_tensor_route(C.byref(from_ranks.c), C.byref(to_ranks.c), C.c_uint64(rank), C.byref(fr), C.byref(to))
    return (None if fr.value == NO_RANK else fr.value, None if to.value == NO_RANK else to.value)


def send_tensor(src_base: np.ndarray, view: OSlice) -> np.ndarray:
    """The receiver's contiguous result for a sender holding ``view`` of the flat storage ``src_base``."""
    src_base = np.ascontiguousarray(src_base).reshape(-1)
    out = np.empty(len(view), dtype=src_base.dtype)
    lib().o_send_tensor(_ptr(out), _ptr(src_base), C.byref(view.c), C.c_uint32(src_base.itemsize))
    return out


def reduce_scatter(ins: Sequence[np.ndarray], in_view: OSlice, out_views: Sequence[OSlice],
                   op: int = SUM) -> List[np.ndarray]:
    ins = [np.ascontiguousarray(x).reshape(-1) for x in ins]
    dt = ins[0].dtype
    outs = [np.empty(len(v), dtype=dt) for v in out_views]
    views = (_CSlice * len(out_views))(*[v.c for v in out_views])
    inp = (C.c_void_p * len(ins))(*[x.ctypes.data for x in ins])
    outp = (C.c_void_p * len(outs))(*[x.ctypes.data for x in outs])
    fn = {"float32": lib().o_reduce_scatter_f32, "uint16": lib().o_reduce_scatter_bf16}[dt.name]
    fn(outp, views, C.c_uint32(len(outs)), inp, C.byref(in_view.c), C.c_uint32(len(ins)), C.c_int(op))
    return outs


def bf16_to_f32(x: np.ndarray) -> np.ndarray:
    x = np.ascontiguousarray(x, dtype=np.uint16)
    out = np.empty(x.shape, dtype=np.float32)
    lib().o_bf16_to_f32(_ptr(out), _ptr(x), C.c_uint64(x.size))
    return out


def f32_to_bf16(x: np.ndarray) -> np.ndarray:
    x = np.ascontiguousarray(x, dtype=np.float32)
    out = np.empty(x.shape, dtype=np.uint16)
    lib().o_f32_to_bf16(_ptr(out), _ptr(x), C.c_uint64(x.size))
    return out


def f16_to_f32(x: np.ndarray) -> np.ndarray:
    x = np.ascontiguousarray(x, dtype=np.uint16)
    out = np.empty(x.shape, dtype=np.float32)
    lib().o_f16_to_f32(_ptr(out), _ptr(x), C.c_uint64(x.size))
    return out


def f32_to_f16(x: np.ndarray) -> np.ndarray:
    x = np.ascontiguousarray(x, dtype=np.float32)
    out = np.empty(x.shape, dtype=np.uint16)
    lib().o_f32_to_f16(_ptr(out), _ptr(x), C.c_uint64(x.size))
    return out


def mesh_dim_members(ranks: OSlice, rank: int, dim: int) -> Tuple[List[int], int]:
    out = _u64([0] * ranks.sizes[dim])
    dr = C.c_uint64()
    rc = lib().o_mesh_dim_members(C.byref(ranks.c), C.c_uint64(rank), C.c_uint32(dim), out, C.byref(dr))
    if rc:
        raise OracleError(rc)
    return list(out)[: ranks.sizes[dim]], dr.value


def mesh_ranks_for_dims(ranks: OSlice, rank: int, dims: Sequence[int]) -> List[int]:
    total = 1
    for d in dims:
        total *= ranks.sizes[d]
    out = _u64([0] * total)
    n = lib().o_mesh_ranks_for_dims(C.byref(ranks.c), C.c_uint64(rank), (C.c_uint32 * max(1, len(dims)))(*dims),
                                    C.c_uint32(len(dims)), out)
    if n < 0:
        raise OracleError(6)
    return list(out)[:n]


def e4m3fn_encode(f: float, saturate: bool = False) -> int:
    return int(lib().o_e4m3fn_encode(C.c_float(f), C.c_int(int(saturate))))


def e4m3fn_decode(c: int) -> float:
    return float(lib().o_e4m3fn_decode(C.c_uint8(c)))


def fp8_quantize(x_bf16: np.ndarray, block: int = 1024) -> Tuple[np.ndarray, np.ndarray]:
    x = np.ascontiguousarray(x_bf16, dtype=np.uint16).reshape(-1)
    nb = (x.size + block - 1) // block
    q = np.empty(x.size, dtype=np.uint8)
    scales = np.empty(nb, dtype=np.float32)
    lib().o_fp8_quantize(_ptr(q), _ptr(scales), _ptr(x), C.c_uint64(x.size), C.c_uint32(block))
    return q, scales


def fp8_dequant_accumulate(acc: np.ndarray, q: np.ndarray, scales: np.ndarray, block: int = 1024) -> None:
    assert acc.dtype == np.float32 and q.dtype == np.uint8 and scales.dtype == np.float32
    assert acc.flags.c_contiguous and q.flags.c_contiguous and scales.flags.c_contiguous
    lib().o_fp8_dequant_accumulate(_ptr(acc), _ptr(q), _ptr(scales), C.c_uint64(q.size), C.c_uint32(block))


def fp8_dequantize(q: np.ndarray, scales: np.ndarray, block: int = 1024) -> np.ndarray:
    out = np.empty(q.size, dtype=np.float32)
    lib().o_fp8_dequantize(_ptr(out), _ptr(q), _ptr(scales), C.c_uint64(q.size), C.c_uint32(block))
    return out


def flat_pack(tensors: Sequence[np.ndarray], offsets: Sequence[int]) -> np.ndarray:
    tensors = [np.ascontiguousarray(t).reshape(-1) for t in tensors]
    dt = tensors[0].dtype
    flat = np.zeros(offsets[-1], dtype=dt)
    ptrs = (C.c_void_p * len(tensors))(*[t.ctypes.data for t in tensors])
    lib().o_flat_pack(_ptr(flat), ptrs, _u64(offsets), C.c_uint32(len(tensors)), C.c_uint32(dt.itemsize))
    return flat


def flat_unpack(flat: np.ndarray, offsets: Sequence[int]) -> List[np.ndarray]:
    outs = [np.empty(offsets[i + 1] - offsets[i], dtype=flat.dtype) for i in range(len(offsets) - 1)]
    ptrs = (C.c_void_p * len(outs))(*[t.ctypes.data for t in outs])
    lib().o_flat_unpack(ptrs, _ptr(flat), _u64(offsets), C.c_uint32(len(outs)), C.c_uint32(flat.itemsize))
    return outs


# ---- device-initiated RDMA: WQE / CQE byte images (rdmaxcel-sys/src/rdmaxcel.cu) ----
class _CWqeParams(C.Structure):  # o_wqe_params_t
    _fields_ = [("laddr", C.c_uint64), ("lkey", C.c_uint32), ("length", C.c_uint64), ("wr_id", C.c_uint64),
                ("signaled", C.c_uint8), ("op_type", C.c_uint32), ("raddr", C.c_uint64), ("rkey", C.c_uint32),
                ("qp_num", C.c_uint32), ("buf", C.c_void_p), ("dbrec", C.c_void_p), ("wqe_cnt", C.c_uint32)]


class _CCqePollParams(C.Structure):  # o_cqe_poll_params_t
    _fields_ = [("cqe_buf", C.c_void_p), ("cqe_size", C.c_uint32), ("consumer_index", C.c_uint32),
                ("cqe_cnt", C.c_uint32), ("dbrec", C.c_void_p)]


def _wqe_params(buf: np.ndarray, dbrec: np.ndarray, wqe_cnt: int, *, laddr=0, lkey=0, length=0, wr_id=0, signaled=True,
                op_type=0, raddr=0, rkey=0, qp_num=0, buf_offset=0) -> _CWqeParams:
    assert buf.dtype == np.uint8 and dbrec.dtype == np.uint32 and buf.flags.c_contiguous
    return _CWqeParams(laddr, lkey, length, wr_id, 1 if signaled else 0, op_type, raddr, rkey, qp_num,
                       buf.ctypes.data + buf_offset, dbrec.ctypes.data, wqe_cnt)


def send_wqe(sq: np.ndarray, dbrec: np.ndarray, wqe_cnt: int, **fields) -> None:
    """rdmaxcel.cu:201-245 on host arrays: ``sq`` (uint8, wqe_cnt * 64 bytes) and ``dbrec`` (2 x uint32)."""
    p = _wqe_params(sq, dbrec, wqe_cnt, **fields)
    lib().o_send_wqe(C.byref(p))


def recv_wqe(rq_slot: np.ndarray, dbrec: np.ndarray, wqe_cnt: int, **fields) -> None:
    """rdmaxcel.cu:139-160: the data segment goes to the first 16 bytes of ``rq_slot`` (+ ``buf_offset``)."""
    p = _wqe_params(rq_slot, dbrec, wqe_cnt, **fields)
    lib().o_recv_wqe(C.byref(p))


def db_ring(dst: np.ndarray, src: np.ndarray) -> None:
    """rdmaxcel.cu:82-93: 64 bytes from ``src`` to ``dst``."""
    assert dst.dtype == np.uint8 and src.dtype == np.uint8 and dst.size >= 64 and src.size >= 64
    lib().o_db_ring(C.c_void_p(dst.ctypes.data), C.c_void_p(src.ctypes.data))


def cqe_poll(cq: np.ndarray, dbrec: np.ndarray, cqe_size: int, cqe_cnt: int, consumer_index: int, result: int = -1) -> int:
    """rdmaxcel.cu:292-326: one look at the CQ; returns the byte count, -2 (bad opcode) or ``result`` untouched."""
    assert cq.dtype == np.uint8 and dbrec.dtype == np.uint32
    p = _CCqePollParams(cq.ctypes.data, cqe_size, consumer_index, cqe_cnt, dbrec.ctypes.data)
    out = C.c_int32(result)
    lib().o_cqe_poll(C.byref(out), C.byref(p))
    return out.value
