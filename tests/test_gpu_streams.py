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


def test_calls_from_several_threads_each_on_its_own_stream():
    # Every StreamActor of the reference runs on an OS thread of its own and creates its stream lazily on that thread
    # (monarch_tensor_worker/src/stream.rs:447-452,538-563,613-624), so the entry points are called from several threads
    # at once, each with its own stream.  Four threads each loop over pack x4 -> reduce (avg) -> unpack -> fp8 quantise
    # on different shapes and element types; ctypes drops the interpreter lock for the duration of a foreign call, so
    # the calls overlap inside the library.  The host synchronises each thread's stream once, at the end.
    import threading

    L = lib()
    torch.cuda.init()
    nthreads, n, reps = 4, 4, 25
    jobs = []
    for t in range(nthreads):
        rows, cols, pitch = 200 + 37 * t, 509 + 256 * t, 1031 + 300 * t
        view = Slice(offset=1 + t, sizes=[rows, cols], strides=[pitch, 1])
        span_elems = view.offset + (rows - 1) * pitch + cols
        rng = np.random.default_rng(900 + t)
        hosts = [rng.uniform(-1, 1, size=span_elems).astype(np.float32) for _ in range(n)]
        packed = [oracle.pack(h, oslice(view)) for h in hosts]
        want_out = oracle.reduce(packed, oracle.AVG)
        want_dst = np.full(span_elems, -7.0, dtype=np.float32)
        oracle.unpack(want_dst, want_out, oslice(view))
        xq = torch.from_numpy(rng.standard_normal(5000 + 1024 * t).astype(np.float32)).bfloat16()
        want_q, want_s = oracle.fp8_quantize(xq.view(torch.uint16).numpy(), 1024)
        jobs.append(dict(
            view=view, want_out=want_out, want_dst=want_dst, want_q=want_q, want_s=want_s,
            xs=[torch.from_numpy(h).to(DEV) for h in hosts],
            chunks=[torch.empty(len(view), device=DEV) for _ in range(n)],
            out=torch.empty(len(view), device=DEV),
            dst=torch.full((span_elems,), -7.0, device=DEV),
            xq=xq.to(DEV), q=torch.empty(xq.numel(), dtype=torch.uint8, device=DEV),
            s=torch.empty((xq.numel() + 1023) // 1024, dtype=torch.float32, device=DEV)))
    torch.cuda.synchronize()
    failures = []
    start = threading.Barrier(nthreads)

    def work(job):
        try:
            stream = C.c_void_p()
            check(L.mhip_stream_create(C.byref(stream)))
            view, ins = job["view"], ptr_array([c.data_ptr() for c in job["chunks"]])
            start.wait()
            for _ in range(reps):
                for x, c in zip(job["xs"], job["chunks"]):
                    check(L.mhip_slice_pack(c.data_ptr(), x.data_ptr(), C.byref(view.c), 4, stream))
                check(L.mhip_reduce(job["out"].data_ptr(), ins, n, len(view), _lib.DTYPE_F32, _lib.OP_AVG, stream))
                check(L.mhip_slice_unpack(job["dst"].data_ptr(), job["out"].data_ptr(), C.byref(view.c), 4, stream))
                check(L.mhip_fp8_quantize(job["q"].data_ptr(), job["s"].data_ptr(), job["xq"].data_ptr(), job["xq"].numel(),
                                          1024, stream))
            check(L.mhip_stream_synchronize(stream))
            check(L.mhip_stream_destroy(stream))
        except Exception as e:  # reported by the main thread
            failures.append(repr(e))

    threads = [threading.Thread(target=work, args=(job,)) for job in jobs]
    for th in threads:
        th.start()
    for th in threads:
        th.join(timeout=100)
    assert not any(th.is_alive() for th in threads)
    assert not failures, failures
    for t, job in enumerate(jobs):
        assert np.array_equal(job["out"].cpu().numpy(), job["want_out"]), t
        assert np.array_equal(job["dst"].cpu().numpy(), job["want_dst"]), t
        assert np.array_equal(job["q"].cpu().numpy(), job["want_q"]), t
        assert np.array_equal(job["s"].cpu().numpy(), job["want_s"]), t
