"""Stream-to-stream ordering the way the reference does it: the producer records an event after its call,
the consumer's stream waits for that event (monarch_tensor_worker/src/comm.rs:139-161,
torch-sys-cuda/src/cuda.rs:74-84,164-172).  The packs run on one stream, the reduce on another, both
created through the C ABI; nothing synchronises the host until the very end."""
import ctypes as C

import numpy as np
import pytest
import torch

import oracle
from monarch_amd import Slice, _lib
from monarch_amd._lib import check, lib, ptr_array
from util import oslice

pytestmark = pytest.mark.gpu
DEV = "cuda:0"


def test_pack_on_one_stream_reduce_on_another():
    L = lib()
    torch.cuda.init()
    s1, s2 = C.c_void_p(), C.c_void_p()
    check(L.mhip_stream_create(C.byref(s1)))
    check(L.mhip_stream_create(C.byref(s2)))
    packed_done, reduce_done = C.c_void_p(), C.c_void_p()
    check(L.mhip_event_create(C.byref(packed_done)))
    check(L.mhip_event_create(C.byref(reduce_done)))
    view = Slice(offset=3, sizes=[300, 1791], strides=[2047, 1])
    n, span_elems = 8, 3 + 299 * 2047 + 1791
    hosts = [np.random.default_rng(50 + k).uniform(-1, 1, size=span_elems).astype(np.float32) for k in range(n)]
    xs = [torch.from_numpy(h).to(DEV) for h in hosts]
    chunks = [torch.empty(len(view), device=DEV) for _ in range(n)]
    out = torch.empty(len(view), device=DEV)
    torch.cuda.synchronize()  # the uploads ran on torch's stream
    for rep in range(3):
        for x, c in zip(xs, chunks):
            check(L.mhip_slice_pack(c.data_ptr(), x.data_ptr(), C.byref(view.c), 4, s1))
        check(L.mhip_event_record(packed_done, s1))
        check(L.mhip_stream_wait_event(s2, packed_done))
        check(L.mhip_reduce(out.data_ptr(), ptr_array([c.data_ptr() for c in chunks]), n, len(view), _lib.DTYPE_F32,
                            _lib.OP_SUM, s2))
        check(L.mhip_event_record(reduce_done, s2))
        # the next round's packs overwrite the chunks: they must wait for this round's reduce
        check(L.mhip_stream_wait_event(s1, reduce_done))
    check(L.mhip_event_synchronize(reduce_done))
    want = oracle.reduce([oracle.pack(h, oslice(view)) for h in hosts], oracle.SUM)
    assert np.array_equal(out.cpu().numpy(), want)
    ms = C.c_float()
    check(L.mhip_event_elapsed_ms(C.byref(ms), packed_done, reduce_done))
    assert ms.value >= 0.0
    for e in (packed_done, reduce_done):
        check(L.mhip_event_destroy(e))
    for s in (s1, s2):
        check(L.mhip_stream_synchronize(s))
        check(L.mhip_stream_destroy(s))


def test_bucket_unpacks_on_a_side_stream_keep_their_pointer_tables():
    # FlatBucket uploads a table of output pointers per set of outputs; launches on a stream that torch's allocator
    # does not track read it asynchronously.  Several unpacks into different output sets are queued on a side stream
    # behind a long-running kernel, more tensors are allocated and freed meanwhile, and every result must still land
    # in its own outputs.
    from monarch_amd import fp8
    sizes = [4096, 1, 70000, 333, 2048, 9]
    total = sum(sizes)
    side = torch.cuda.Stream()
    src = [torch.zeros(n, dtype=torch.float32, device=DEV) for n in sizes]
    bucket = fp8.FlatBucket(src)
    flats = [torch.full((total,), float(k + 1), device=DEV) for k in range(6)]
    torch.cuda.synchronize()
    out_sets = []
    with torch.cuda.stream(side):
        big = torch.empty(1 << 28, dtype=torch.float32, device=DEV)
        big.normal_()                                       # keeps the side stream busy while the calls below queue up
    for k, flat in enumerate(flats):
        outs = [torch.empty(n, dtype=torch.float32, device=DEV) for n in sizes]
        bucket.unpack(flat, outs, stream=side)
        out_sets.append(outs)
        junk = [torch.full((len(sizes),), -1, dtype=torch.int64, device=DEV) for _ in range(8)]   # table-sized allocations
        del junk
    side.synchronize()
    torch.cuda.synchronize()
    for k, outs in enumerate(out_sets):
        for o in outs:
            assert torch.all(o == float(k + 1)), k
