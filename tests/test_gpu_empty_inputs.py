"""Empty inputs (no elements, no bytes, no views, empty views among full ones) are accepted by every data-path entry point,
launch nothing that writes, and leave every buffer as it was.  The reference's Slice allows empty dimensions
(ndslice/src/slice.rs:382-384: len is the product of the sizes), and a gradient bucket may hold empty tensors."""
import ctypes as C

import pytest
import torch

from monarch_amd import Slice
from monarch_amd._lib import lib, ptr_array
from monarch_amd.ndslice import slice_array
from util import sync

pytestmark = pytest.mark.gpu
DEV = "cuda:0"
F32, BF16 = 6, 15   # c10::ScalarType numbers


def test_every_entry_point_takes_empty_inputs_and_writes_nothing():
    L = lib()
    s = torch.cuda.current_stream().cuda_stream
    canary = torch.full((4096,), 0x5A, dtype=torch.uint8, device=DEV)
    other = torch.full((4096,), 0x33, dtype=torch.uint8, device=DEV)
    p, o = canary.data_ptr(), other.data_ptr()
    empty = Slice(offset=5, sizes=[3, 0], strides=[1, 3])
    empty1 = Slice(offset=0, sizes=[0], strides=[1])
    ins = ptr_array([o, o + 1024])
    assert L.mhip_slice_pack(p, o, C.byref(empty.c), 4, s) == 0
    assert L.mhip_slice_unpack(p, o, C.byref(empty.c), 4, s) == 0
    views = slice_array([empty, empty1])
    assert L.mhip_slice_pack_many(ptr_array([p, p + 64]), o, views, 2, 2, s) == 0
    assert L.mhip_slice_unpack_many(p, ptr_array([o, o + 64]), views, 2, 2, s) == 0
    assert L.mhip_slice_pack_many(ptr_array([]), o, views, 0, 2, s) == 0
    for op in (0, 1, 2, 3, 4):
        assert L.mhip_reduce(p, ins, 2, 0, F32, op, s) == 0
    assert L.mhip_reduce_scatter(ptr_array([p, p + 64]), views, 2, ins, None, 0, 2, BF16, 0, s) == 0
    assert L.mhip_reduce_scatter(ptr_array([]), views, 0, ins, None, 16, 2, BF16, 0, s) == 0
    assert L.mhip_stack(p, ins, 2, 0, 4, s) == 0
    assert L.mhip_stack_scatter(p, ins, 2, 1, 0, 4, s) == 0
    assert L.mhip_buffer_transfer(p, o, 0, 0, s, None) == 0
    assert L.mhip_buffer_transfer_many(ptr_array([p]), ptr_array([o]), (C.c_size_t * 1)(0), 1, 0, s, None) == 0
    assert L.mhip_buffer_transfer_many(ptr_array([]), ptr_array([]), (C.c_size_t * 1)(0), 0, 0, s, None) == 0
    assert L.mhip_send_tensor(p, 0, o, C.byref(empty.c), 4, p + 512, s) == 0
    assert L.mhip_fp8_quantize(p, p + 1024, o, 0, 1024, s) == 0
    assert L.mhip_fp8_dequant_accumulate(p, o, o + 1024, 0, 1024, s) == 0
    offsets = torch.zeros(3, dtype=torch.int64, device=DEV)        # two tensors, both empty
    table = torch.tensor([o, o + 64], dtype=torch.int64, device=DEV)
    assert L.mhip_flat_pack(p, table.data_ptr(), offsets.data_ptr(), 2, 0, 2, None, s) == 0
    assert L.mhip_flat_unpack(table.data_ptr(), p, offsets.data_ptr(), 2, 0, 2, None, s) == 0
    assert L.mhip_fp8_quantize_bucket(p, p + 1024, table.data_ptr(), offsets.data_ptr(), 2, 0, 1024, None, s) == 0
    assert L.mhip_fp8_dequant_accumulate_bucket(table.data_ptr(), p, p + 1024, offsets.data_ptr(), 2, 0, 1024, None, s) == 0
    sync()
    assert bool((canary == 0x5A).all()) and bool((other == 0x33).all())


def test_empty_tensors_among_full_ones():
    # a bucket whose first, middle and last tensors are empty; a group of views with empty ones in between
    from monarch_amd import fp8, staging
    g = torch.Generator().manual_seed(4)
    sizes = [0, 1500, 0, 0, 2048, 7, 0]
    tensors = [torch.randn(k, generator=g).bfloat16().to(DEV) for k in sizes]
    bucket = fp8.FlatBucket(tensors)
    flat = bucket.pack()
    q1, s1 = fp8.quantize_bucket(bucket, indexed=True)
    q2, s2 = fp8.quantize(flat)
    sync()
    assert torch.equal(flat.view(torch.int16), torch.cat(tensors).view(torch.int16))
    assert torch.equal(q1, q2) and torch.equal(s1.view(torch.int32), s2.view(torch.int32))
    x = torch.arange(64 * 96, dtype=torch.int32, device=DEV).reshape(64, 96)
    views = [Slice(offset=0, sizes=[0], strides=[1]), Slice(offset=3, sizes=[64, 5], strides=[96, 1]),
             Slice(offset=9, sizes=[0, 4], strides=[96, 1]), Slice(offset=40, sizes=[64, 7], strides=[96, 1])]
    outs = staging.pack_many(x, views)
    sync()
    assert outs[0].numel() == 0 and outs[2].numel() == 0
    assert torch.equal(outs[1], x[:, 3:8].reshape(-1)) and torch.equal(outs[3], x[:, 40:47].reshape(-1))
