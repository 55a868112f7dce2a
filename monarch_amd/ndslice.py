"""``Slice``: the Python face of ``ndslice::Slice`` over the C ABI.

Same surface as the reference's Python binding of Slice
(monarch_hyperactor/src/ndslice.rs:38-205): keyword constructor that validates like
``Slice::new`` (ndslice/src/slice.rs:99-139) and raises ``ValueError``; ``s[i]`` raises
``IndexError``; ``index``/``coordinates`` raise ``ValueError``; ``nditem`` raises
``IndexError``.  All index arithmetic runs in the library's host code.
"""
from __future__ import annotations

import ctypes as C
from typing import Iterator, List, Sequence

import numpy as np

from . import _lib
from ._lib import MhipError, SliceC, check, lib, u64_array

_ITER_CHUNK = 1 << 16


class Slice:
    __slots__ = ("_offset", "_sizes", "_strides", "_c", "_keep")

    def __init__(self, *, offset: int, sizes: Sequence[int], strides: Sequence[int], _validate: bool = True):
        sizes, strides = [int(x) for x in sizes], [int(x) for x in strides]
        if offset < 0 or any(x < 0 for x in sizes) or any(x < 0 for x in strides):
            raise ValueError("offset, sizes and strides must be non-negative")
        if _validate:
            rc = lib().mhip_slice_validate(offset, u64_array(sizes), len(sizes), u64_array(strides), len(strides))
            if rc:
                raise ValueError(str(MhipError(rc, lib().mhip_error_string(rc).decode())))
        self._offset, self._sizes, self._strides = int(offset), sizes, strides
        self._keep = (u64_array(sizes), u64_array(strides))
        self._c = SliceC(self._offset, len(sizes), self._keep[0], self._keep[1])

    # ---- constructors that skip validation, as the reference's do (slice.rs:152-175,630-660) ----
    @staticmethod
    def new_row_major(sizes: Sequence[int]) -> "Slice":
        strides, acc = [], 1
        for n in reversed(list(sizes)):
            strides.append(acc)
            acc *= n
        return Slice(offset=0, sizes=sizes, strides=list(reversed(strides)), _validate=False)

    @staticmethod
    def _unchecked(offset, sizes, strides) -> "Slice":
        return Slice(offset=offset, sizes=sizes, strides=strides, _validate=False)

    @staticmethod
    def from_list(ranks: Sequence[int]) -> List["Slice"]:
        """1-d slices covering ``ranks`` (monarch_hyperactor/src/ndslice.rs:167-194)."""
        if not ranks:
            return []
        ranks = sorted(ranks)
        result = []
        offset, size, stride = ranks[0], 1, 1
        for rank in ranks[1:]:
            if size == 1 and rank > offset:
                stride = rank - offset
                size += 1
            elif offset + size * stride == rank:
                size += 1
            else:
                result.append(Slice(offset=offset, sizes=[size], strides=[stride]))
                offset, size, stride = rank, 1, 1
        result.append(Slice(offset=offset, sizes=[size], strides=[stride]))
        return result

    @staticmethod
    def of_tensor(t) -> "Slice":
        """The Slice of a torch tensor view over its storage: ``(storage_offset, size, stride)``,
        the triple the reference rebuilds views from (python/monarch/common/function_caching.py:50-63)."""
        return Slice(offset=t.storage_offset(), sizes=list(t.shape), strides=list(t.stride()))

    # ---- accessors ----
    @property
    def ndim(self) -> int:
        return len(self._sizes)

    @property
    def offset(self) -> int:
        return self._offset

    @property
    def sizes(self) -> List[int]:
        return list(self._sizes)

    @property
    def strides(self) -> List[int]:
        return list(self._strides)

    @property
    def c(self) -> SliceC:
        return self._c

    def __len__(self) -> int:
        out = C.c_uint64()
        check(lib().mhip_slice_len(C.byref(self._c), C.byref(out)))
        return out.value

    def is_contiguous(self) -> bool:
        out = C.c_int()
        check(lib().mhip_slice_is_contiguous(C.byref(self._c), C.byref(out)))
        return bool(out.value)

    def get(self, index: int) -> int:
        out = C.c_uint64()
        check(lib().mhip_slice_get(C.byref(self._c), index, C.byref(out)))
        return out.value

    def __getitem__(self, key):
        if isinstance(key, slice):
            start, stop, step = key.indices(len(self))
            if start < 0 or stop < 0:
                raise IndexError("Only positive indices are support")
            try:
                return tuple(self.get(i) for i in range(start, stop, step))
            except MhipError as e:
                raise IndexError(str(e)) from None
        if not isinstance(key, int) or key < 0:
            raise TypeError("index must be a non-negative int")
        try:
            return self.get(key)
        except MhipError as e:
            raise IndexError(str(e)) from None

    def locations(self, start: int = 0, count: int | None = None) -> np.ndarray:
        """Locations of items ``[start, start+count)`` of the iteration, as uint64."""
        n = len(self)
        count = max(0, n - start) if count is None else min(count, max(0, n - start))
        out = np.empty(max(count, 1), dtype=np.uint64)
        written = C.c_uint64()
        check(lib().mhip_slice_iter(C.byref(self._c), start, count, out.ctypes.data, C.byref(written)))
        return out[: written.value]

    def __iter__(self) -> Iterator[int]:
        start = 0
        while True:
            chunk = self.locations(start, _ITER_CHUNK)
            if chunk.size == 0:
                return
            yield from chunk.tolist()
            start += chunk.size

    def __contains__(self, value: int) -> bool:
        try:
            self.coordinates(value)
            return True
        except ValueError:
            return False

    def nditem(self, coordinates: Sequence[int]) -> int:
        out = C.c_uint64()
        rc = lib().mhip_slice_location(C.byref(self._c), u64_array(list(coordinates)), len(coordinates), C.byref(out))
        if rc:
            raise IndexError(lib().mhip_error_string(rc).decode())
        return out.value

    location = nditem

    def coordinates(self, value: int) -> List[int]:
        out = u64_array([0] * self.ndim)
        rc = lib().mhip_slice_coordinates(C.byref(self._c), value, out)
        if rc:
            raise ValueError(f"value {value} not in slice")
        return list(out)[: self.ndim]

    def index(self, value: int) -> int:
        out = C.c_uint64()
        rc = lib().mhip_slice_index(C.byref(self._c), value, C.byref(out))
        if rc:
            raise ValueError(f"value {value} not in slice")
        return out.value

    # ---- view algebra ----
    def select(self, dim: int, begin: int, end: int, step: int = 1) -> "Slice":
        off = C.c_uint64()
        sz, st = u64_array([0] * self.ndim), u64_array([0] * self.ndim)
        rc = lib().mhip_slice_select(C.byref(self._c), dim, begin, end, step, C.byref(off), sz, st)
        if rc:
            raise ValueError(str(MhipError(rc, lib().mhip_error_string(rc).decode())))
        return Slice._unchecked(off.value, list(sz)[: self.ndim], list(st)[: self.ndim])

    def at(self, dim: int, index: int) -> "Slice":
        off = C.c_uint64()
        sz, st = u64_array([0] * self.ndim), u64_array([0] * self.ndim)
        rc = lib().mhip_slice_at(C.byref(self._c), dim, index, C.byref(off), sz, st)
        if rc:
            raise ValueError(str(MhipError(rc, lib().mhip_error_string(rc).decode())))
        n = self.ndim - 1
        return Slice._unchecked(off.value, list(sz)[:n], list(st)[:n])

    def subview(self, starts: Sequence[int], lens: Sequence[int]) -> "Slice":
        off = C.c_uint64()
        rc = lib().mhip_slice_subview(C.byref(self._c), u64_array(list(starts)), len(starts),
                                      u64_array(list(lens)), len(lens), C.byref(off))
        if rc:
            raise ValueError(str(MhipError(rc, lib().mhip_error_string(rc).decode())))
        return Slice._unchecked(off.value, list(lens), self._strides)

    def view(self, new_sizes: Sequence[int]) -> "Slice":
        st = u64_array([0] * len(new_sizes))
        rc = lib().mhip_slice_view(C.byref(self._c), u64_array(list(new_sizes)), len(new_sizes), st)
        if rc:
            raise ValueError(str(MhipError(rc, lib().mhip_error_string(rc).decode())))
        return Slice._unchecked(0, list(new_sizes), list(st)[: len(new_sizes)])

    def enforce_embedding(self, other: "Slice") -> "Slice":
        rc = lib().mhip_slice_enforce_embedding(C.byref(self._c), C.byref(other._c))
        if rc:
            raise ValueError(str(MhipError(rc, lib().mhip_error_string(rc).decode())))
        return self

    def bounds(self):
        lo, hi = C.c_uint64(), C.c_uint64()
        check(lib().mhip_slice_bounds(C.byref(self._c), C.byref(lo), C.byref(hi)))
        return lo.value, hi.value

    # ---- value semantics ----
    def __eq__(self, other) -> bool:
        return (isinstance(other, Slice) and self._offset == other._offset
                and self._sizes == other._sizes and self._strides == other._strides)

    def __hash__(self) -> int:
        return hash((self._offset, tuple(self._sizes), tuple(self._strides)))

    def __repr__(self) -> str:
        return f"Slice {{ offset: {self._offset}, sizes: {self._sizes}, strides: {self._strides} }}"

    def __getnewargs_ex__(self):
        return (), {"offset": self._offset, "sizes": self._sizes, "strides": self._strides}

    def __reduce__(self):
        return (_rebuild, (self._offset, self._sizes, self._strides))


def _rebuild(offset, sizes, strides):
    return Slice(offset=offset, sizes=sizes, strides=strides)


def slice_array(slices: Sequence[Slice]):
    """A C array of mhip_slice_t for the *_many entry points (keeps the Slices alive)."""
    arr = (SliceC * max(1, len(slices)))(*[s.c for s in slices])
    arr._keep = list(slices)
    return arr
