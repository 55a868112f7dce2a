"""The device entry points only enqueue kernels on the caller's stream (no allocation, no
synchronisation, no memset node: mhip_memset itself is a fill kernel), so a caller can record them into a HIP graph.  A captured
pack -> reduce -> unpack pipeline and a captured fp8 round trip are replayed several times with
new input data and eager work in between, and every replay is compared with the eager result."""
import numpy as np
import pytest
import torch

import oracle
from monarch_amd import Slice, fp8, staging
from monarch_amd import reduce as R
from util import oslice, sync

pytestmark = pytest.mark.gpu
DEV = "cuda:0"


def test_pack_reduce_unpack_pipeline_replays():
    s = Slice(offset=0, sizes=[4, 128, 256], strides=[65536, 512, 1])  # every other row
    n = 8
    xs = [torch.zeros(4, 256, 256, device=DEV) for _ in range(n)]
    chunks = [torch.empty(len(s), device=DEV) for _ in range(n)]
    total = torch.empty(len(s), device=DEV)
    back = torch.zeros(4, 256, 256, device=DEV)

    def pipeline():
        for x, c in zip(xs, chunks):
            staging.pack(x, s, out=c)
        R.all_reduce(total, chunks, R.ReduceOp.Sum)
        staging.unpack(back, s, total)

    def fill(seed):
        hosts = [np.random.default_rng(seed + k).uniform(-1, 1, size=(4, 256, 256)).astype(np.float32) for k in range(n)]
        for x, h in zip(xs, hosts):
            x.copy_(torch.from_numpy(h))
        return hosts

    def expect(hosts):
        packed = [oracle.pack(h.reshape(-1), oslice(s)) for h in hosts]
        want = np.zeros(4 * 256 * 256, dtype=np.float32)
        oracle.unpack(want, oracle.reduce(packed, oracle.SUM), oslice(s))
        return want

    hosts = fill(100)
    pipeline()  # eager
    sync()
    assert np.array_equal(back.cpu().numpy().reshape(-1), expect(hosts))

    graph = torch.cuda.CUDAGraph()
    side = torch.cuda.Stream()
    side.wait_stream(torch.cuda.current_stream())
    with torch.cuda.stream(side):
        pipeline()  # warm the stream before capture
    torch.cuda.current_stream().wait_stream(side)
    sync()
    with torch.cuda.graph(graph, stream=side):
        pipeline()
    for rep in range(4):
        hosts = fill(200 + 10 * rep)
        back.zero_()
        scratch = torch.randn(1 << 20, device=DEV).sum()  # unrelated eager work between replays
        graph.replay()
        sync()
        assert np.array_equal(back.cpu().numpy().reshape(-1), expect(hosts)), rep
        assert torch.isfinite(scratch)


def test_fp8_bucket_round_trip_replays():
    g = torch.Generator().manual_seed(5)
    sizes = [1024, 3000, 1, 7777, 2048, 513]
    tensors = [torch.zeros(k, dtype=torch.bfloat16, device=DEV) for k in sizes]
    accs = [torch.zeros(k, dtype=torch.float32, device=DEV) for k in sizes]
    src, dst = fp8.FlatBucket(tensors), fp8.FlatBucket(accs)
    total = sum(sizes)
    q = torch.empty(total, dtype=torch.uint8, device=DEV)
    scales = torch.empty((total + 1023) // 1024, dtype=torch.float32, device=DEV)

    src.block_index()   # built before the capture: the captured calls then use the indexed kernels and allocate nothing
    dst.block_index()

    def pipeline():
        fp8.quantize_bucket(src, q, scales)
        fp8.dequant_accumulate_bucket(dst, q, scales)

    pipeline()
    sync()
    graph = torch.cuda.CUDAGraph()
    with torch.cuda.graph(graph):
        pipeline()
    for rep in range(3):
        hosts = [(torch.randn(k, generator=g) * (rep + 1)).bfloat16() for k in sizes]
        for t, h in zip(tensors, hosts):
            t.copy_(h)
        for a in accs:
            a.fill_(float(rep))
        graph.replay()
        sync()
        flat = torch.cat(hosts).view(torch.uint16).numpy()
        hq, hs = oracle.fp8_quantize(flat, 1024)
        want = np.full(total, float(rep), dtype=np.float32)
        oracle.fp8_dequant_accumulate(want, hq, hs, 1024)
        assert np.array_equal(q.cpu().numpy(), hq) and np.array_equal(scales.cpu().numpy(), hs)
        assert np.array_equal(torch.cat(accs).cpu().numpy(), want), rep


def test_memset_every_alignment_and_in_a_graph():
    # the byte fill is a kernel: exact at every start alignment and length, nothing written outside the
    # range, and it can be recorded into a graph (clear a staging chunk, then accumulate into it)
    import ctypes as C
    from monarch_amd._lib import check, lib
    stream = torch.cuda.current_stream().cuda_stream
    buf = torch.empty(4096, dtype=torch.uint8, device=DEV)
    for start in list(range(0, 19)) + [31, 33]:
        for nbytes in [0, 1, 2, 15, 16, 17, 31, 32, 33, 100, 1000, 4000]:
            buf.fill_(0xEE)
            check(lib().mhip_memset(buf.data_ptr() + start, 0x1A5, nbytes, stream))  # only the low byte counts
            sync()
            got = buf.cpu().numpy()
            assert (got[start:start + nbytes] == 0xA5).all() and (got[:start] == 0xEE).all() \
                and (got[start + nbytes:] == 0xEE).all(), (start, nbytes)
    big = torch.empty((3 << 20) + 5, dtype=torch.uint8, device=DEV)
    check(lib().mhip_memset(big.data_ptr() + 3, 7, big.numel() - 5, stream))
    sync()
    assert bool((big[3:-2] == 7).all())

    n = 5000
    acc = torch.empty(n, dtype=torch.float32, device=DEV)
    x = [torch.zeros(n, dtype=torch.float32, device=DEV) for _ in range(3)]

    def pipeline():
        check(lib().mhip_memset(acc.data_ptr(), 0, n * 4, torch.cuda.current_stream().cuda_stream))
        R.all_reduce(acc, [acc, *x], R.ReduceOp.Sum)  # in place: acc = 0 + sum of x

    pipeline()
    sync()
    graph = torch.cuda.CUDAGraph()
    with torch.cuda.graph(graph):
        pipeline()
    g = torch.Generator().manual_seed(9)
    for rep in range(4):
        hosts = [torch.randn(n, generator=g) for _ in x]
        for t, h in zip(x, hosts):
            t.copy_(h)
        acc.fill_(float("nan"))  # must be cleared by the replayed fill, every time
        junk = torch.randn(1 << 18, device=DEV).sum()
        graph.replay()
        sync()
        want = ((torch.zeros(n) + hosts[0]) + hosts[1]) + hosts[2]
        assert torch.equal(acc.cpu(), want), rep
        assert torch.isfinite(junk)


def test_strided_copy_forms_replay():
    # the forms whose launch geometry the host derives from addresses (XCD shares, line-by-line unpack, units on a
    # skewed base, line-aligned transposing windows) recorded once and replayed on new data
    g = torch.Generator(device=DEV).manual_seed(9)
    cases = [(torch.int16, (300, 4096), lambda x: x[:, 1:3581]),          # ragged rows of 7160 bytes at an odd column
             (torch.int16, (300, 4096), lambda x: x[:, 1:3585]),          # whole chunks from a skewed base
             (torch.int32, (257, 1031), lambda x: x[:, 3:].t()),          # transposing, written rows off the cache lines
             (torch.uint8, (600, 1000), lambda x: x[5:, 7:900])]          # one-byte units
    views, outs, backs, xs = [], [], [], []
    for dt, shape, view_of in cases:
        x = torch.zeros(shape, dtype=dt, device=DEV)
        v = view_of(x)
        xs.append(x)
        views.append((v, Slice.of_tensor(v), view_of))
        outs.append(torch.empty(v.numel(), dtype=dt, device=DEV))
        backs.append(torch.zeros_like(x))

    def pipeline():
        for (v, s, _), o, b in zip(views, outs, backs):
            staging.pack(v, s, out=o)
            staging.unpack(b, s, o)

    def fill():
        for x in xs:
            info = torch.iinfo(x.dtype)
            x.copy_(torch.randint(info.min, info.max, x.shape, dtype=x.dtype, generator=g, device=DEV))

    def check(tag):
        for (v, s, view_of), o, b, x in zip(views, outs, backs, xs):
            assert torch.equal(o.view(v.shape), v.contiguous()), tag
            want = torch.zeros_like(x)
            view_of(want).copy_(v)
            assert torch.equal(b, want), tag

    fill()
    pipeline()
    sync()
    check("eager")
    graph = torch.cuda.CUDAGraph()
    side = torch.cuda.Stream()
    side.wait_stream(torch.cuda.current_stream())
    with torch.cuda.stream(side):
        pipeline()
    torch.cuda.current_stream().wait_stream(side)
    sync()
    with torch.cuda.graph(graph, stream=side):
        pipeline()
    for rep in range(3):
        fill()
        for b in backs:
            b.zero_()
        scratch = torch.randn(1 << 20, device=DEV).sum()  # unrelated eager work between replays
        graph.replay()
        sync()
        check(rep)
        assert torch.isfinite(scratch)
