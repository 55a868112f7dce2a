"""Block-scaled fp8 (e4m3fn, one fp32 absmax scale per 1024 elements) transfer codec and the
flat bucket it runs on.

The reference ships fp8 tensors as raw bytes and refuses to reduce them
(torch-sys-cuda/src/nccl.rs:275-278,474-476); this codec is what makes a compressed
gradient exchange possible on that path: pack ragged tensors into one flat bf16 buffer
(the torch.cat / split idiom of python/tests/simulator/test_simulator.py:190-203),
quantise, move 1 byte per element plus 4 bytes per block, dequantise-and-accumulate
into an fp32 buffer, unpack.
"""
from __future__ import annotations

from typing import List, Sequence

import torch

from . import _torch
from ._lib import check, lib, ptr_array

BLOCK = 1024
FP8_MAX = 448.0


def _nblocks(n: int) -> int:
    return (n + BLOCK - 1) // BLOCK


def _check_payload(q: torch.Tensor, scales: torch.Tensor, n: int, device: torch.device) -> None:
    """Caller-supplied code and scale buffers: on ``device``, contiguous, one byte per element for ``n`` elements
    and one fp32 scale per 1024-element block.  A short buffer would be an out-of-bounds device write."""
    for t in (q, scales):
        _torch.require_contiguous(t)
        if t.device != device:
            raise ValueError(f"buffer is on {t.device}, the data on {device}")
    if q.element_size() != 1 or q.numel() != n:
        raise ValueError(f"q must hold {n} one-byte codes, got {q.numel()} elements of {q.element_size()} bytes")
    if scales.dtype != torch.float32 or scales.numel() != _nblocks(n):
        raise ValueError(f"scales must hold {_nblocks(n)} fp32 values, got {scales.numel()} of {scales.dtype}")


class FlatBucket:
    """Offsets table and device pointer table for a list of ragged tensors."""

    def __init__(self, tensors: Sequence[torch.Tensor]):
        if not tensors:
            raise ValueError("a bucket needs at least one tensor")
        self.dtype = tensors[0].dtype
        self.device = tensors[0].device
        for t in tensors:
            _torch.require_contiguous(t)
            if t.dtype != self.dtype:
                raise ValueError("all tensors of a bucket must share a dtype")
        self.tensors = list(tensors)  # the pointer table below is only valid while these are alive
        self.sizes = [t.numel() for t in tensors]
        self.offsets = [0]
        for n in self.sizes:
            self.offsets.append(self.offsets[-1] + n)
        self.total = self.offsets[-1]
        # device-resident tables, uploaded once and reused by every pack / unpack
        self.d_offsets = torch.tensor(self.offsets, dtype=torch.int64, device=self.device)
        self._tables = {}
        self._index = None
        self.d_ptrs = self.pointer_table(tensors)

    # Launches read a pointer table asynchronously, possibly on a stream torch's allocator does not know about, so a
    # table must not go back to the allocator while a launch may still be queued.  Tables are kept per set of
    # tensors (uploading is a host-synchronous copy, so a cached table is complete before any launch uses it);
    # the cache holds the tensors too, so a cached address cannot be handed to another tensor meanwhile.
    _MAX_TABLES = 8

    def pointer_table(self, tensors: Sequence[torch.Tensor]) -> torch.Tensor:
        if [t.numel() for t in tensors] != self.sizes:
            raise ValueError("tensor sizes do not match the bucket")
        key = tuple(t.data_ptr() for t in tensors)
        hit = self._tables.get(key)
        if hit is None:
            if len(self._tables) >= self._MAX_TABLES:   # retire the oldest once everything queued so far has run
                torch.cuda.synchronize(self.device)
                self._tables.pop(next(iter(self._tables)))
            hit = (torch.tensor(key, dtype=torch.int64, device=self.device), list(tensors))
            self._tables[key] = hit
        return hit[0]

    def block_index(self, stream=None) -> torch.Tensor:
        """The bucket's block index (``mhip_bucket_index_build``): which tensor holds the first element of every
        1024-element block.  Built on first use, then reused by the fused quantise / dequantise calls."""
        if self._index is None:
            import ctypes as C
            nbytes = C.c_size_t()
            check(lib().mhip_bucket_index_bytes(self.total, BLOCK, C.byref(nbytes)))
            index = torch.empty(nbytes.value // 4, dtype=torch.int32, device=self.device)
            check(lib().mhip_bucket_index_build(index.data_ptr(), self.d_offsets.data_ptr(), len(self.sizes), self.total,
                                                BLOCK, _torch.stream_handle(stream)))
            if stream is not None:  # later calls may come on another stream: the index must be complete by then
                stream.synchronize()
            else:
                torch.cuda.current_stream(self.device).synchronize()
            self._index = index
        return self._index

    def _index_ptr(self, indexed, stream):
        """``indexed`` None: use the index if ``block_index()`` has built it (nothing is allocated or synchronised
        inside a data-path call, so such calls stay capturable into HIP graphs); True: build it now if needed."""
        if indexed is None:
            return None if self._index is None else self._index.data_ptr()
        return self.block_index(stream).data_ptr() if indexed else None

    def pack(self, flat: torch.Tensor = None, d_ptrs: torch.Tensor = None, stream=None, indexed: bool = None) -> torch.Tensor:
        """flat[offsets[t] + j] = tensors[t][j]; ``indexed`` as in ``_index_ptr``."""
        if flat is None:
            flat = torch.empty(self.total, dtype=self.dtype, device=self.device)
        else:
            self._check_flat(flat, self.dtype)
        ptrs = self.d_ptrs if d_ptrs is None else d_ptrs
        if ptrs.dtype != torch.int64 or ptrs.numel() != len(self.sizes) or ptrs.device != self.device:
            raise ValueError("the pointer table must hold one int64 device pointer per tensor of the bucket")
        check(lib().mhip_flat_pack(flat.data_ptr(), ptrs.data_ptr(), self.d_offsets.data_ptr(), len(self.sizes),
                                   self.total, self.tensors[0].element_size(), self._index_ptr(indexed, stream),
                                   _torch.stream_handle(stream)))
        return flat

    def _check_flat(self, flat: torch.Tensor, dtype: torch.dtype) -> None:
        _torch.require_contiguous(flat)
        if flat.device != self.device:
            raise ValueError(f"flat buffer is on {flat.device}, the bucket on {self.device}")
        if flat.dtype != dtype or flat.numel() != self.total:
            raise ValueError(f"flat buffer must hold {self.total} elements of {dtype}, got {flat.numel()} of {flat.dtype}")

    def unpack(self, flat: torch.Tensor, outs: Sequence[torch.Tensor], stream=None, indexed: bool = None) -> None:
        """outs[t][j] = flat[offsets[t] + j]; ``flat`` may have any dtype of the outs' element size;
        ``indexed`` as in ``_index_ptr``."""
        _torch.require_contiguous(flat)
        if flat.numel() != self.total or flat.device != self.device:
            raise ValueError(f"flat buffer must hold {self.total} elements on {self.device}")
        for t in outs:
            _torch.require_contiguous(t)
            if t.element_size() != flat.element_size():
                raise ValueError("element size mismatch")
            if t.device != self.device:
                raise ValueError(f"output is on {t.device}, the bucket on {self.device}")
        ptrs = self.pointer_table(outs)
        check(lib().mhip_flat_unpack(ptrs.data_ptr(), flat.data_ptr(), self.d_offsets.data_ptr(), len(self.sizes),
                                     self.total, flat.element_size(), self._index_ptr(indexed, stream),
                                     _torch.stream_handle(stream)))


def quantize_bucket(bucket: FlatBucket, q: torch.Tensor = None, scales: torch.Tensor = None, stream=None,
                    indexed: bool = None):
    """Same codes and scales as ``quantize(bucket.pack())`` without the flat bf16 buffer.  With the bucket's block
    index (``bucket.block_index()`` called once beforehand, or ``indexed=True``) a wavefront loads the tensor of its
    span instead of searching the offsets table: same bits, faster."""
    if bucket.dtype != torch.bfloat16:
        raise ValueError("quantize_bucket expects a bf16 bucket")
    n = bucket.total
    if q is None:
        q = torch.empty(n, dtype=torch.uint8, device=bucket.device)
    if scales is None:
        scales = torch.empty(_nblocks(n), dtype=torch.float32, device=bucket.device)
    _check_payload(q, scales, n, bucket.device)
    check(lib().mhip_fp8_quantize_bucket(q.data_ptr(), scales.data_ptr(), bucket.d_ptrs.data_ptr(),
                                         bucket.d_offsets.data_ptr(), len(bucket.sizes), n, BLOCK,
                                         bucket._index_ptr(indexed, stream), _torch.stream_handle(stream)))
    return q, scales


def dequant_accumulate_bucket(bucket: FlatBucket, q: torch.Tensor, scales: torch.Tensor, stream=None,
                              indexed: bool = None) -> None:
    """``tensor_t[j] += float(q[off_t + j]) * scale`` on the bucket's own fp32 tensors."""
    if bucket.dtype != torch.float32:
        raise ValueError("dequant_accumulate_bucket expects a bucket of fp32 accumulators")
    _check_payload(q, scales, bucket.total, bucket.device)
    check(lib().mhip_fp8_dequant_accumulate_bucket(bucket.d_ptrs.data_ptr(), q.data_ptr(), scales.data_ptr(),
                                                   bucket.d_offsets.data_ptr(), len(bucket.sizes), bucket.total, BLOCK,
                                                   bucket._index_ptr(indexed, stream), _torch.stream_handle(stream)))


def quantize(flat_bf16: torch.Tensor, q: torch.Tensor = None, scales: torch.Tensor = None, stream=None):
    """Returns ``(q uint8[numel], scales f32[ceil(numel/1024)])``."""
    _torch.require_contiguous(flat_bf16)
    if flat_bf16.dtype != torch.bfloat16:
        raise ValueError("quantize expects a bf16 buffer")
    n = flat_bf16.numel()
    if q is None:
        q = torch.empty(n, dtype=torch.uint8, device=flat_bf16.device)
    if scales is None:
        scales = torch.empty(_nblocks(n), dtype=torch.float32, device=flat_bf16.device)
    _check_payload(q, scales, n, flat_bf16.device)
    check(lib().mhip_fp8_quantize(q.data_ptr(), scales.data_ptr(), flat_bf16.data_ptr(), n, BLOCK,
                                  _torch.stream_handle(stream)))
    return q, scales


def dequant_accumulate(acc: torch.Tensor, q: torch.Tensor, scales: torch.Tensor, stream=None) -> None:
    """acc[i] += float(q[i]) * scales[i // 1024] (fp32, product rounded before the add)."""
    _torch.require_contiguous(acc)
    if acc.dtype != torch.float32:
        raise ValueError("acc must be fp32")
    _check_payload(q, scales, acc.numel(), acc.device)
    check(lib().mhip_fp8_dequant_accumulate(acc.data_ptr(), q.data_ptr(), scales.data_ptr(), q.numel(), BLOCK,
                                            _torch.stream_handle(stream)))


def dequant_accumulate_many(acc: torch.Tensor, qs: Sequence[torch.Tensor], scales: Sequence[torch.Tensor],
                            overwrite: bool = False, stream=None) -> None:
    """The receive side of an exchange with ``len(qs)`` peers in one pass:
    ``acc = (0 if overwrite else acc) + sum_r float(qs[r]) * scales[r][i // 1024]``, peers in order,
    bit-identical to calling ``dequant_accumulate`` once per peer."""
    if len(qs) == 0 or len(qs) != len(scales):
        raise ValueError("one scales tensor per code tensor, at least one peer")
    _torch.require_contiguous(acc)
    if acc.dtype != torch.float32:
        raise ValueError("acc must be fp32")
    n = acc.numel()
    for q, s in zip(qs, scales):
        _check_payload(q, s, n, acc.device)
    check(lib().mhip_fp8_dequant_accumulate_many(acc.data_ptr(), ptr_array([q.data_ptr() for q in qs]),
                                                 ptr_array([s.data_ptr() for s in scales]), len(qs), n, BLOCK,
                                                 1 if overwrite else 0, _torch.stream_handle(stream)))


def dequant_accumulate_bucket_many(bucket: FlatBucket, qs: Sequence[torch.Tensor], scales: Sequence[torch.Tensor],
                                   stream=None, indexed: bool = None) -> None:
    """``dequant_accumulate_bucket`` for all peers' payloads in one pass (peers added in order)."""
    if bucket.dtype != torch.float32:
        raise ValueError("dequant_accumulate_bucket_many expects a bucket of fp32 accumulators")
    if len(qs) == 0 or len(qs) != len(scales):
        raise ValueError("one scales tensor per code tensor, at least one peer")
    for q, s in zip(qs, scales):
        _check_payload(q, s, bucket.total, bucket.device)
    check(lib().mhip_fp8_dequant_accumulate_bucket_many(
        bucket.d_ptrs.data_ptr(), ptr_array([q.data_ptr() for q in qs]), ptr_array([s.data_ptr() for s in scales]),
        len(qs), bucket.d_offsets.data_ptr(), len(bucket.sizes), bucket.total, BLOCK, bucket._index_ptr(indexed, stream),
        _torch.stream_handle(stream)))
