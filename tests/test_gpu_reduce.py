"""GPU parity: mhip_reduce / mhip_reduce_scatter and the Reduce host semantics."""
import itertools
import json
import os

import numpy as np
import pytest
import torch

import oracle
from monarch_amd import DeviceMesh, Slice, _lib
from monarch_amd import reduce as R
from monarch_amd._lib import MhipError
from oracle import AVG, SUM
from util import bits, oslice, sync

pytestmark = pytest.mark.gpu
DEV = "cuda:0"


@pytest.fixture(scope="module")
def vec(golden_dir):
    with open(os.path.join(golden_dir, "ndslice_vectors.json")) as f:
        return json.load(f)


def _rand(dtype, n, seed):
    g = torch.Generator().manual_seed(seed)
    if dtype in (torch.float32, torch.float64):
        return (torch.rand(n, generator=g, dtype=dtype) * 2 - 1)
    if dtype in (torch.bfloat16, torch.float16):
        return (torch.randn(n, generator=g) * 0.02).to(dtype)
    if dtype == torch.uint8:
        return torch.randint(0, 256, (n,), dtype=dtype, generator=g)
    info = torch.iinfo(dtype)
    return torch.randint(info.min, info.max, (n,), dtype=dtype, generator=g)


def _oracle_reduce(hosts, op, dtype):
    return oracle.reduce([bits(h) for h in hosts], op, half=dtype == torch.float16)


def test_golden_vectors(vec):
    for case in vec["reduce"]:
        ins = [torch.tensor(x, dtype=torch.float32, device=DEV) for x in case["inputs"]]
        if case["kind"] == "sum":
            out = torch.empty_like(ins[0])
            R.all_reduce(out, ins, R.ReduceOp.Sum)
            sync()
            assert out.cpu().tolist() == case["expected"], case["src"]
        else:
            for r, want in enumerate(case["expected_per_rank"]):
                out = torch.full((len(want),), 1.0, device=DEV)
                R.reduce_scatter_tensor(out, ins, r, R.ReduceOp.Sum)
                sync()
                assert out.cpu().tolist() == want, case["src"]


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16, torch.float16, torch.float64])
@pytest.mark.parametrize("n", [1, 2, 3, 4, 5, 8, 9, 16, 17, 64])
def test_reduce_float_bit_exact(dtype, n):
    for numel in (1, 7, 8, 1000, 4099, (1 << 18) + 3):
        hosts = [_rand(dtype, numel, 100 * n + r) for r in range(n)]
        devs = [h.to(DEV) for h in hosts]
        for op, code in ((R.ReduceOp.Sum, SUM), (R.ReduceOp.Avg, AVG)):
            out = torch.empty_like(devs[0])
            R.all_reduce(out, devs, op)
            sync()
            want = _oracle_reduce(hosts, code, dtype)
            assert np.array_equal(bits(out), want), (dtype, n, numel, op)


@pytest.mark.parametrize("dtype", [torch.uint8, torch.int8, torch.int32, torch.int64])
def test_reduce_integer_sum_wraps(dtype):
    for n, numel in ((2, 5), (3, 4099), (8, 65536 + 1)):
        hosts = [_rand(dtype, numel, 7 * n + r) for r in range(n)]
        devs = [h.to(DEV) for h in hosts]
        out = torch.empty_like(devs[0])
        R.all_reduce(out, devs, R.ReduceOp.Sum)
        sync()
        hs = [h.view(torch.uint8) if dtype == torch.int8 else h for h in hosts]
        want = oracle.reduce([bits(h) for h in hs], SUM)
        got = bits(out.view(torch.uint8) if dtype == torch.int8 else out)
        assert np.array_equal(got, want)
    with pytest.raises(MhipError) as e:
        R.all_reduce(out, devs, R.ReduceOp.Avg)
    assert e.value.name == "UnsupportedOp"


def test_reduce_in_place_and_misaligned():
    n, numel = 8, 10007
    hosts = [_rand(torch.bfloat16, numel + 3, r) for r in range(n)]
    # element-aligned only: every pointer 2 bytes off a 16-byte boundary
    devs = [h.to(DEV)[1: 1 + numel] for h in hosts]
    want = oracle.reduce([bits(h)[1: 1 + numel] for h in hosts], AVG)
    for alias in (0, 5):  # in place on the first member, and on another one
        work = [d.clone() for d in devs]
        keep = [torch.cat([torch.zeros(1, dtype=torch.bfloat16, device=DEV), w, torch.zeros(2, dtype=torch.bfloat16, device=DEV)])
                for w in work]
        views = [k[1: 1 + numel] for k in keep]
        R.all_reduce(views[alias], views, R.ReduceOp.Avg)
        sync()
        assert np.array_equal(bits(views[alias]), want)
        for r in range(n):
            if r != alias:
                assert torch.equal(views[r].view(torch.int16), devs[r].view(torch.int16))  # inputs untouched
            assert keep[r][0].item() == 0 and keep[r][-1].item() == 0


def test_reduce_nan_inf_bf16():
    x = torch.tensor([float("nan"), float("inf"), -float("inf"), 1.0, 3.3895314e38, 0.0, -0.0, 1e-40],
                     dtype=torch.float32).bfloat16()
    y = torch.tensor([1.0, 1.0, float("inf"), float("nan"), 3.3895314e38, -0.0, -0.0, 1e-40],
                     dtype=torch.float32).bfloat16()
    out = torch.empty(8, dtype=torch.bfloat16, device=DEV)
    for op, code in ((R.ReduceOp.Sum, SUM), (R.ReduceOp.Avg, AVG)):
        R.all_reduce(out, [x.to(DEV), y.to(DEV)], op)
        sync()
        assert np.array_equal(bits(out), oracle.reduce([bits(x), bits(y)], code))


def test_reduce_argument_errors():
    x = torch.zeros(16, device=DEV)
    out = torch.empty_like(x)
    with pytest.raises(MhipError) as e:  # nccl.rs:474-476
        R.all_reduce(out.to(torch.float8_e4m3fn), [x.to(torch.float8_e4m3fn)], R.ReduceOp.Sum)
    assert e.value.name == "Float8Reduction"
    with pytest.raises(MhipError) as e:
        R.all_reduce(out, [x] * 65, R.ReduceOp.Sum)
    assert e.value.name == "TooManyInputs"
    rc = _lib.lib().mhip_reduce(out.data_ptr(), _lib.ptr_array([x.data_ptr()]), 1, 16, _lib.DTYPE_F32, 5, None)
    assert rc == _lib.ERR_UNSUPPORTED_OP          # outside ncclRedOp_t, nccl.rs:285-292
    with pytest.raises(MhipError) as e:
        R.all_reduce(out, [x.double()], R.ReduceOp.Sum)
    assert e.value.name == "TypeMismatch"
    with pytest.raises(MhipError) as e:  # check order of nccl.rs:300-316: device before contiguity
        R.all_reduce(out, [torch.zeros(16)], R.ReduceOp.Sum)
    assert e.value.name == "InvalidDevice"
    with pytest.raises(MhipError) as e:
        R.all_reduce(out, [torch.zeros(16, 2, device=DEV)[:, 0]], R.ReduceOp.Sum)
    assert e.value.name == "NoncontiguousTensor"
    with pytest.raises(MhipError) as e:  # nccl.rs:683
        R.reduce_scatter_tensor(torch.empty(5, device=DEV), [x, x], 0, R.ReduceOp.Sum)
    assert e.value.name == "InputSizeMismatch"
    import ctypes as C
    from monarch_amd._lib import lib, ptr_array
    rc = lib().mhip_reduce(out.data_ptr(), ptr_array([x.data_ptr(), 0]), 2, 16, _lib.DTYPE_F32, 0, None)
    assert rc == _lib.ERR_UNDEFINED_TENSOR
    rc = lib().mhip_reduce(out.data_ptr(), ptr_array([x.data_ptr()]), 1, 16, 2, 0, None)  # Short: no NCCL type
    assert rc == _lib.ERR_INVALID_DATA_TYPE


def test_config2_bf16_bucket_full_size():
    n, numel = 8, 25_165_824
    g = torch.Generator(device=DEV).manual_seed(2000)
    devs = [(torch.randn(numel, generator=g, device=DEV) * 0.02).bfloat16() for _ in range(n)]
    hosts = [bits(d) for d in devs]
    want = oracle.reduce(hosts, AVG)
    out = torch.empty_like(devs[0])
    R.all_reduce(out, devs, R.ReduceOp.Avg)  # out of place
    sync()
    assert np.array_equal(bits(out), want)
    # library cross-check: within 1 bf16 ulp of torch's fp32 path
    ref = (torch.stack([d.float() for d in devs]).sum(0) / n).bfloat16()
    diff = (out.view(torch.int16).int() - ref.view(torch.int16).int()).abs().max().item()
    assert diff <= 1
    first = devs[0].clone()
    R.all_reduce(devs[0], devs, R.ReduceOp.Avg)  # in place on input 0
    sync()
    assert np.array_equal(bits(devs[0]), want)
    # linearity on exact data: sum of 8 copies == 8 * x in bf16 (exact scaling by a power of two)
    R.all_reduce(out, [first] * 8, R.ReduceOp.Sum)
    sync()
    assert torch.equal(out.view(torch.int16), (first.float() * 8).bfloat16().view(torch.int16))


def test_reduce_over_staging_area_slots():
    # the chunks of peers sit in the slots of one staging area (skewed pitch); slot 0 doubles as the output
    from monarch_amd import staging
    n, numel = 8, 300_001
    area = staging.StagingArea(n, numel * 2)
    assert area.pitch % 16384 == 8192 and area.pitch >= numel * 2
    hosts = [_rand(torch.bfloat16, numel, 700 + r) for r in range(n)]
    area.storage.fill_(0x5a)
    for r, h in enumerate(hosts):
        area.slot(r, torch.bfloat16).copy_(h)
        assert area.buffer(r).size == numel * 2
    want = _oracle_reduce(hosts, AVG, torch.bfloat16)
    out = torch.empty(numel, dtype=torch.bfloat16, device=DEV)
    R.all_reduce(out, area.slots(torch.bfloat16), R.ReduceOp.Avg)
    sync()
    assert np.array_equal(bits(out.cpu()), want)
    R.all_reduce(area.slot(0, torch.bfloat16), area.slots(torch.bfloat16), R.ReduceOp.Avg)   # in place on slot 0
    sync()
    assert np.array_equal(bits(area.slot(0, torch.bfloat16).cpu()), want)
    # the gaps between slots are never written
    gap = area.storage[numel * 2: area.pitch].cpu()
    assert bool((gap == 0x5a).all())
    with pytest.raises(IndexError):
        area.slot(n)


@pytest.mark.parametrize("numel", [1, 1023, 128 * 8 * 8 * 3, 128 * 8 * 61 + 777, 1_000_003])
def test_reduce_both_block_mappings(numel):
    # inputs that share a 16 KiB phase take the rotated block mapping (workgroup i takes chunk i + i / 8 of its
    # group of 8), inputs at different phases the plain one; both must cover every element exactly once, for
    # grids that are and are not a multiple of 8 workgroups
    n = 8
    hosts = [_rand(torch.float32, numel, 900 + r) for r in range(n)]
    want = oracle.reduce([h.numpy() for h in hosts], SUM)
    for pitch_bytes in (((numel * 4 + 16383) // 16384) * 16384, ((numel * 4 + 16383) // 16384) * 16384 + 4096):
        store = torch.zeros((n - 1) * pitch_bytes + numel * 4, dtype=torch.uint8, device=DEV)
        ins = [store[r * pitch_bytes: r * pitch_bytes + numel * 4].view(torch.float32) for r in range(n)]
        assert len({(t.data_ptr() >> 12) & 3 for t in ins}) == (1 if pitch_bytes % 16384 == 0 else 4)
        for t, h in zip(ins, hosts):
            t.copy_(h)
        out = torch.full((numel + 2,), 7.0, device=DEV)
        R.all_reduce(out[1:-1], ins, R.ReduceOp.Sum)
        sync()
        assert np.array_equal(out[1:-1].cpu().numpy(), want)
        assert out[0].item() == 7.0 and out[-1].item() == 7.0


def test_config1_sum_of_8_packed_chunks():
    from monarch_amd import staging
    s = Slice(offset=0, sizes=[4, 128, 256], strides=[65536, 512, 1])
    chunks, hosts, devs = [], [], []
    for k in range(8):
        rng = np.random.default_rng(1000 + k)
        x = rng.uniform(-1, 1, size=(4, 256, 256)).astype(np.float32)
        devs.append(torch.from_numpy(x).to(DEV))
        chunks.append(staging.pack(devs[-1], s))
        hosts.append(oracle.pack(x.reshape(-1), oslice(s)))
    out = torch.empty_like(chunks[0])
    R.all_reduce(out, chunks, R.ReduceOp.Sum)
    sync()
    assert np.array_equal(out.cpu().numpy(), oracle.reduce(hosts, SUM))
    np.testing.assert_allclose(out.cpu().numpy(), np.sum(np.stack(hosts).astype(np.float64), 0), rtol=1e-6, atol=1e-6)
    # the fused form reads the eight strided views directly: same bits, no staging chunks
    fused = torch.empty_like(out)
    R.reduce_scatter_views([fused], [Slice.new_row_major([len(s)])], devs, s, R.ReduceOp.Sum)
    sync()
    assert torch.equal(fused, out)


def _c4(H, G, Rr, Cc, K, seed, dtype=torch.float32):
    g = torch.Generator(device=DEV).manual_seed(seed)
    x = (torch.rand(H, G, Rr, Cc, generator=g, device=DEV) * 2 - 1).to(dtype)
    slab = Rr * Cc
    flat = x.view(-1)
    group = [flat[gi * slab:] for gi in range(G)]
    in_view = Slice(offset=0, sizes=[H, Rr, Cc], strides=[G * slab, Cc, 1])
    w = Cc // K
    out_views = [Slice(offset=k * w, sizes=[H, Rr, w], strides=[Rr * Cc, Cc, 1]) for k in range(K)]
    return x, group, in_view, out_views, w


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
@pytest.mark.parametrize("shape", [(2, 8, 16, 64, 8), (2, 3, 5, 40, 5), (1, 2, 7, 9, 3), (2, 8, 4, 56, 7)])
def test_reduce_scatter_mesh_dim_small(dtype, shape):
    H, G, Rr, Cc, K = shape
    x, group, in_view, out_views, w = _c4(H, G, Rr, Cc, K, seed=sum(shape), dtype=dtype)
    for op, code in ((R.ReduceOp.Sum, SUM), (R.ReduceOp.Avg, AVG)):
        outs = [torch.empty(H * Rr * w, dtype=dtype, device=DEV) for _ in range(K)]
        R.reduce_scatter_views(outs, out_views, group, in_view, op)
        sync()
        hx = bits(x).reshape(-1)
        slab = Rr * Cc
        want = oracle.reduce_scatter([hx[g * slab:] for g in range(G)], oslice(in_view),
                                     [oslice(v) for v in out_views], code)
        for k in range(K):
            assert np.array_equal(bits(outs[k]), want[k]), (shape, k, op)


@pytest.mark.parametrize("pad", [0, 1024])
def test_reduce_scatter_both_block_mappings(pad):
    # slabs of 3 x 16 KiB: back to back they share a 16 KiB phase (XCD-contiguous block mapping),
    # 4 KiB further apart they do not (plain mapping); 2*24*8 = 384 + ... workgroups, and a second
    # shape whose workgroup count is not a multiple of 8
    for H, G, Rr, Cc, K in ((2, 8, 24, 512, 8), (1, 8, 37, 512, 4)):
        slab = Rr * Cc
        pitch = slab + pad + (0 if (slab * 4) % 16384 == 0 else (16384 - (slab * 4) % 16384) // 4)
        g = torch.Generator(device=DEV).manual_seed(77 + pad)
        x = torch.rand(H * G * pitch, generator=g, device=DEV) * 2 - 1
        group = [x[gi * pitch:] for gi in range(G)]
        assert len({(t.data_ptr() >> 12) & 3 for t in group}) == (1 if pad == 0 else 4)
        in_view = Slice(offset=0, sizes=[H, Rr, Cc], strides=[G * pitch, Cc, 1])
        w = Cc // K
        out_views = [Slice(offset=k * w, sizes=[H, Rr, w], strides=[Rr * Cc, Cc, 1]) for k in range(K)]
        outs = [torch.empty(H * Rr * w, device=DEV) for _ in range(K)]
        R.reduce_scatter_views(outs, out_views, group, in_view, R.ReduceOp.Sum)
        sync()
        hx = x.cpu().numpy()
        want = oracle.reduce_scatter([hx[gi * pitch:] for gi in range(G)], oslice(in_view),
                                     [oslice(v) for v in out_views], SUM)
        for k in range(K):
            assert np.array_equal(outs[k].cpu().numpy(), want[k]), (H, G, Rr, Cc, K, k)


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16, torch.float64, torch.int32])
def test_reduce_scatter_rows_that_are_not_whole_vectors(dtype):
    # rows of at least one 16-byte vector whose length or offset is not a multiple of one: chunks that
    # straddle an output row are computed as two overlapping vectors
    for shape in [(2, 4, 9, 77, 7), (1, 3, 50, 1022, 2), (2, 8, 5, 129, 3), (1, 2, 300, 45, 1)]:
        H, G, Rr, Cc, K = shape
        x, group, in_view, out_views, w = _c4(H, G, Rr, Cc, K, seed=sum(shape), dtype=torch.float32)
        if dtype == torch.int32:
            x = (x * 1e6).to(torch.int32)
        else:
            x = x.to(dtype)
        slab = Rr * Cc
        group = [x.view(-1)[gi * slab:] for gi in range(G)]
        ops = ((R.ReduceOp.Sum, SUM),) if dtype == torch.int32 else ((R.ReduceOp.Sum, SUM), (R.ReduceOp.Avg, AVG))
        for op, code in ops:
            store = torch.full((K, H * Rr * w + 8), 7, dtype=dtype, device=DEV)
            outs = [store[k, 3: 3 + H * Rr * w] for k in range(K)]          # element-aligned only
            R.reduce_scatter_views(outs, out_views, group, in_view, op)
            sync()
            hx = bits(x).reshape(-1)
            want = oracle.reduce_scatter([hx[g * slab:] for g in range(G)], oslice(in_view),
                                         [oslice(v) for v in out_views], code) if dtype in (torch.float32, torch.bfloat16) else None
            for k in range(K):
                if want is not None:
                    assert np.array_equal(bits(outs[k]), want[k]), (shape, k, op)
                else:  # f64 / i32: torch on the host, same order
                    hv = x.cpu().view(H, G, Rr, Cc)
                    acc = hv[:, 0].clone()
                    for g in range(1, G):
                        acc = acc + hv[:, g]
                    if code == AVG:
                        acc = acc / G
                    assert torch.equal(outs[k].cpu().view(H, Rr, w), acc[:, :, k * w:(k + 1) * w]), (shape, k, op)
                assert bool((store[k, :3] == 7).all()) and bool((store[k, 3 + H * Rr * w:] == 7).all())


def test_reduce_scatter_vectors_crossing_input_rows():
    # outputs are flat chunks of the reduced tensor while the inputs are read through a view with padded
    # rows: output vectors that cross an input row fall back to single elements
    Rr, Cc, G, K = 40, 45, 3, 4
    pitch = Cc + 3
    g = torch.Generator(device=DEV).manual_seed(31)
    xs = [torch.rand(Rr * pitch, generator=g, device=DEV) * 2 - 1 for _ in range(G)]
    in_view = Slice(offset=0, sizes=[Rr, Cc], strides=[pitch, 1])
    c = Rr * Cc // K
    out_views = [Slice(offset=k * c, sizes=[c], strides=[1]) for k in range(K)]
    outs = [torch.empty(c, device=DEV) for _ in range(K)]
    R.reduce_scatter_views(outs, out_views, xs, in_view, R.ReduceOp.Sum)
    sync()
    want = oracle.reduce_scatter([t.cpu().numpy() for t in xs], oslice(in_view), [oslice(v) for v in out_views], SUM)
    for k in range(K):
        assert np.array_equal(outs[k].cpu().numpy(), want[k]), k


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
def test_reduce_scatter_fuzz(dtype):
    # random input views and random strided
    # selections of the reduced index space as outputs
    import random
    from util import span, valid_slices
    gen = random.Random(5)
    views = [v for v in valid_slices(120, seed=17, max_size=24, max_len=60_000) if len(v) >= 64][:40]
    assert len(views) >= 25
    for i, in_view in enumerate(views):
        L, G = len(in_view), gen.choice([1, 2, 3, 5, 8])
        n_store = span(in_view) + 4
        hosts = [_rand(dtype, n_store, 1000 * i + g) for g in range(G)]
        group = [h.to(DEV) for h in hosts]
        out_views = []
        for _ in range(gen.choice([1, 2, 4])):
            st = gen.choice([1, 1, 1, 2, 3])
            n = gen.randrange(1, max(2, (L - 1) // st))
            o = gen.randrange(0, L - (n - 1) * st)
            out_views.append(Slice(offset=o, sizes=[n], strides=[st]))
        if L % 4 == 0:   # and a two-dimensional one: column blocks of the index space seen as [L/4, 4]
            out_views.append(Slice(offset=1, sizes=[L // 4, 3], strides=[4, 1]))
        op, code = gen.choice([(R.ReduceOp.Sum, SUM), (R.ReduceOp.Avg, AVG)])
        outs = [torch.empty(len(v), dtype=dtype, device=DEV) for v in out_views]
        R.reduce_scatter_views(outs, out_views, group, in_view, op)
        sync()
        want = oracle.reduce_scatter([bits(h).reshape(-1) for h in hosts], oslice(in_view), [oslice(v) for v in out_views], code)
        for k in range(len(out_views)):
            assert np.array_equal(bits(outs[k]), want[k]), (i, in_view, out_views[k], G, op)


@pytest.mark.parametrize("sizes,strides", [([32776, 65535], [65537, 1]),    # rows of at least one vector: chunk form
                                           ([716_000_000, 3], [5, 1])])   # runs of 3: element form
def test_reduce_scatter_wide_index(sizes, strides):
    # an output of more than 2^31 elements: 64-bit decode of both the output view and the input layout.
    # int8 sums wrap, so torch's own add on the GPU is the expected value.
    view = Slice(offset=1, sizes=sizes, strides=strides)
    _, hi = view.bounds()
    group = []
    for g in range(2):
        t = torch.empty(hi + 1, dtype=torch.int8, device=DEV)
        step = 1 << 28
        for i in range(0, t.numel(), step):
            k = torch.arange(i, min(i + step, t.numel()), device=DEV, dtype=torch.int64)
            t[i:i + step] = ((k * (2654435761 + 2 * g)) >> (11 + g)).to(torch.int8)
            del k
        group.append(t)
    out = torch.empty(len(view), dtype=torch.int8, device=DEV)
    assert out.numel() >= 2**31
    R.reduce_scatter_views([out], [view], group, None, R.ReduceOp.Sum)
    sync()
    total = group[0] + group[1]
    want = torch.as_strided(total, sizes, strides, 1).contiguous().reshape(-1)
    assert torch.equal(out, want)


def test_config4_mesh_dim_reduce_scatter_full_size():
    H, G, Rr, Cc, K = 2, 8, 2048, 4096, 8
    x, group, in_view, out_views, w = _c4(H, G, Rr, Cc, K, seed=4000)
    outs = [torch.empty(H * Rr * w, dtype=torch.float32, device=DEV) for _ in range(K)]
    R.reduce_scatter_views(outs, out_views, group, in_view, R.ReduceOp.Sum)
    sync()
    # exact: fp32 adds in gpu order, which torch reproduces with explicit adds
    acc = x[:, 0].clone()
    for g in range(1, G):
        acc = acc + x[:, g]
    for k in range(K):
        assert torch.equal(outs[k].view(H, Rr, w), acc[:, :, k * w:(k + 1) * w])
    # oracle on two of the outputs (the div/mod walk is slow at full size)
    hx = x.cpu().numpy().reshape(-1)
    slab = Rr * Cc
    for k in (0, 7):
        want = oracle.reduce_scatter([hx[g * slab:] for g in range(G)], oslice(in_view), [oslice(out_views[k])], SUM)[0]
        assert np.array_equal(outs[k].cpu().numpy(), want)
    np.testing.assert_allclose(torch.cat([o.view(H, Rr, w) for o in outs], dim=2).cpu().numpy(),
                               x.sum(1).cpu().numpy(), rtol=1e-6, atol=1e-6)


def test_reduce_scatter_dim0_rule_all_ranks():
    # ncclReduceScatter: rank r receives the reduced flat chunk r (nccl.rs:683,693-701)
    n, c = 4, 1031
    hosts = [_rand(torch.float32, n * c, 40 + r) for r in range(n)]
    devs = [h.to(DEV) for h in hosts]
    total = oracle.reduce([h.numpy() for h in hosts], SUM)
    for r in range(n):
        out = torch.empty(c, device=DEV)
        R.reduce_scatter_tensor(out, devs, r, R.ReduceOp.Sum)
        sync()
        assert np.array_equal(out.cpu().numpy(), total[r * c:(r + 1) * c])


def test_stream_reduce_placement_and_errors():
    # test_controller.py:188-254 on a [2 hosts, 2 gpus] mesh: x[h,g] = 24h + 12g + arange(12)
    mesh_slice = Slice(offset=0, sizes=[2, 2], strides=[2, 1])
    xs = {(h, g): (24 * h + 12 * g + torch.arange(12, device=DEV).reshape(3, 4)).float()
          for h, g in itertools.product(range(2), range(2))}
    world = {2 * h + g: t for (h, g), t in xs.items()}
    mesh = DeviceMesh(["host", "gpu"], mesh_slice, 0)
    y = R.reduce(world, mesh, "gpu", "sum")
    g = R.reduce(world, mesh, "gpu", "stack")
    sync()
    assert torch.equal(y, xs[(0, 0)] + xs[(0, 1)])
    assert torch.equal(g, torch.stack([xs[(0, 0)], xs[(0, 1)]]))
    with pytest.raises(TypeError, match="When scattering"):
        R.reduce(world, mesh, "gpu", "sum", scatter=True)
    w2 = {r: t.reshape(2, 6) for r, t in world.items()}
    rs = R.reduce(w2, mesh, "gpu", "sum", scatter=True)
    atoa = R.reduce(w2, mesh, "gpu", "stack", scatter=True)
    rad = R.reduce(w2, mesh, (), "sum")
    rade = R.reduce(w2, mesh, ("gpu", "host"), "sum")
    sync()
    total = sum(xs.values()).reshape(2, 6)
    assert torch.equal(rs, (w2[0] + w2[1])[0]) and rs.shape == (6,)
    assert torch.equal(atoa, torch.stack([w2[0][0], w2[1][0]]))
    assert torch.equal(rad, total) and torch.equal(rade, total)
    for kw in (dict(scatter=True), dict(reduction="stack"), dict(reduction="stack", scatter=True)):
        with pytest.raises(ValueError, match="is not valid for multiple dimensions"):
            R.reduce(w2, mesh, (), **{"reduction": "sum", **kw})
    with pytest.raises(KeyError):
        R.reduce(w2, mesh, "nope")
    with pytest.raises(ValueError, match="reducing the same dimension twice"):
        R.reduce(w2, mesh, ("gpu", "gpu"))
    # test_reduce_out (test_controller.py:256-270): wrong out shape is refused
    with pytest.raises(ValueError, match="Reduce expects the shape to be torch.Size"):
        R.reduce(w2, mesh, "host", "sum", scatter=True, out=torch.empty(2, 4, device=DEV))
    # placement (stream.rs:1437-1458): in place aliases the input; out= is returned; default is a fresh tensor
    mine = w2[0].clone()
    w3 = dict(w2)
    w3[0] = mine
    r1 = R.reduce(w3, mesh, "gpu", "sum", inplace=True)
    assert r1.data_ptr() == mine.data_ptr()
    o = torch.empty(2, 6, device=DEV)
    r2 = R.reduce(w2, mesh, "gpu", "avg", out=o)
    r3 = R.reduce(w2, mesh, "gpu", "sum")
    sync()
    assert r2.data_ptr() == o.data_ptr() and r3.data_ptr() not in (w2[0].data_ptr(), o.data_ptr())
    assert torch.equal(r1, w2[0] + w2[1]) and torch.equal(r2, (w2[0] + w2[1]) / 2) and torch.equal(r3, r1)
    with pytest.raises(ValueError, match="cannot be used with inplace"):
        R.reduce(w2, mesh, "gpu", "sum", inplace=True, out=o)
    with pytest.raises(ValueError, match="not valid for in-place"):
        R.reduce(w2, mesh, "gpu", "sum", scatter=True, inplace=True)
    # an input that errored upstream is replaced by zeros of the factory (stream.rs:976-989)
    group = [None, w2[1]]
    r4 = R.stream_reduce(group, 1, R.Factory.of(w2[1]), R.Reduction.from_str("sum"), False, False)
    sync()
    assert torch.equal(r4, w2[1])
    # worker_reduce (comm.rs:1258-1431): ones(2,3) over a [2,2] mesh -> 2.0 over "x", 4.0 over "x","y"
    ones = {r: torch.ones(2, 3, device=DEV) for r in range(4)}
    m2 = DeviceMesh(["x", "y"], Slice(offset=0, sizes=[2, 2], strides=[2, 1]), 3)
    a = R.reduce(ones, m2, "x", "sum")
    b = R.reduce(ones, m2, ("x", "y"), "sum")
    sync()
    assert torch.all(a == 2.0) and torch.all(b == 4.0)


# ---------------- Prod / Max / Min, Reduction::Stack ----------------

_OTHER = ((R.ReduceOp.Prod, oracle.PROD), (R.ReduceOp.Max, oracle.MAX), (R.ReduceOp.Min, oracle.MIN))


def _obits(t):
    """Host array as the oracle's reduce_op wants it: signed integers keep their sign, bf16 / f16 become bits."""
    return bits(t)


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16, torch.float16, torch.float64, torch.uint8, torch.int8,
                                   torch.int32, torch.int64])
@pytest.mark.parametrize("n", [1, 2, 3, 8, 9, 17])
def test_reduce_prod_max_min_bit_exact(dtype, n):
    for numel in (1, 7, 1000, 4099, (1 << 17) + 5):
        hosts = [_rand(dtype, numel, 900 * n + r) for r in range(n)]
        if dtype in (torch.bfloat16, torch.float16):
            hosts = [h * 60 for h in hosts]      # products of values around 1, not around 0.02^n
        devs = [h.to(DEV) for h in hosts]
        for op, code in _OTHER:
            out = torch.empty_like(devs[0])
            R.all_reduce(out, devs, op)
            sync()
            want = oracle.reduce_op([_obits(h) for h in hosts], code, kind="f16" if dtype == torch.float16 else None)
            assert np.array_equal(_obits(out), want), (dtype, n, numel, op)


def test_reduce_max_min_nan_zero_rule_and_in_place():
    nan, inf = float("nan"), float("inf")
    a = torch.tensor([1.0, nan, nan, 3.0, nan, -0.0, 0.0, -inf, 5.0])
    b = torch.tensor([nan, 2.0, nan, nan, -5.0, 0.0, -0.0, inf, 5.0])
    c = torch.tensor([0.5, nan, nan, 4.0, nan, -0.0, -0.0, 0.0, -5.0])
    for dtype in (torch.float32, torch.bfloat16, torch.float16, torch.float64):
        hs = [t.to(dtype) for t in (a, b, c)]
        for op, code in _OTHER[1:]:
            work = [h.to(DEV) for h in hs]
            R.all_reduce(work[1], work, op)          # in place on member 1
            sync()
            want = oracle.reduce_op([_obits(h) for h in hs], code, kind="f16" if dtype == torch.float16 else None)
            got = _obits(work[1])
            if dtype in (torch.float32, torch.float64):
                assert np.array_equal(np.isnan(got), np.isnan(want))
                ok = ~np.isnan(want)
                assert np.array_equal(got[ok], want[ok]) and np.array_equal(np.signbit(got[ok]), np.signbit(want[ok]))
            else:
                assert np.array_equal(got, want)     # bit patterns, NaN canonical on both sides


def test_reduce_scatter_other_ops():
    rng = np.random.default_rng(12)
    hosts = [rng.uniform(-2, 2, size=(6, 40)).astype(np.float32) for _ in range(3)]
    devs = [torch.from_numpy(h).to(DEV) for h in hosts]
    in_view = Slice(offset=0, sizes=[6, 40], strides=[40, 1])
    for views in ([Slice(offset=10 * k, sizes=[6, 10], strides=[40, 1]) for k in range(4)],      # vector form
                  [Slice(offset=k, sizes=[6, 13], strides=[40, 2]) for k in range(2)]):           # element form
        for op, code in _OTHER:
            outs = [torch.empty(len(v), device=DEV) for v in views]
            R.reduce_scatter_views(outs, views, devs, in_view, op)
            sync()
            want = oracle.reduce_scatter([h.reshape(-1) for h in hosts], oslice(in_view), [oslice(v) for v in views], code)
            for o, w in zip(outs, want):
                assert np.array_equal(o.cpu().numpy(), w), op
    hb = [torch.from_numpy(h).bfloat16() for h in hosts]
    db = [h.to(DEV) for h in hb]
    views = [Slice(offset=k * 7, sizes=[6, 7], strides=[40, 1]) for k in range(5)]                # ragged rows
    for op, code in _OTHER:
        outs = [torch.empty(len(v), dtype=torch.bfloat16, device=DEV) for v in views]
        R.reduce_scatter_views(outs, views, db, in_view, op)
        sync()
        want = oracle.reduce_scatter([bits(h).reshape(-1) for h in hb], oslice(in_view), [oslice(v) for v in views], code)
        for o, w in zip(outs, want):
            assert np.array_equal(bits(o), w), op


def test_stack_reference_vectors():
    # all_gather_into_tensor, torch-sys-cuda/src/nccl.rs:927-959
    group = [torch.full((2, 2), float(i), device=DEV) for i in range(2)]
    for rank in range(2):
        out = R.stream_reduce(group, rank, R.Factory.of(group[0]), R.Reduction.from_str("stack"), False, False)
        sync()
        assert out.shape == (2, 2, 2) and torch.equal(out, torch.stack(group))
    # all_to_all_single, nccl.rs:996-1031
    group = [torch.tensor([0.0, 1.0], device=DEV), torch.tensor([2.0, 3.0], device=DEV)]
    want = [[0.0, 2.0], [1.0, 3.0]]
    for rank in range(2):
        out = R.stream_reduce(group, rank, R.Factory.of(group[0]), R.Reduction.from_str("stack"), True, False)
        sync()
        assert out.cpu().tolist() == want[rank]
    with pytest.raises(ValueError, match="in-place, non-scatter not supported for stack reduce"):   # stream.rs:1403-1406
        R.stream_reduce(group, 0, R.Factory.of(group[0]), R.Reduction.from_str("stack"), False, True)


@pytest.mark.parametrize("dtype", [torch.uint8, torch.bfloat16, torch.float32, torch.float64])
@pytest.mark.parametrize("n", [1, 2, 5, 8, 64])
def test_stack_and_stack_scatter_against_oracle(dtype, n):
    import ctypes as C
    lib = _lib.lib()
    es = torch.empty(0, dtype=dtype).element_size()
    for per in (1, 3, 8, 1000, 4099, 65536 + 24):
        numel = per * n
        hosts = [_rand(dtype, numel + 3, 31 * n + r) for r in range(n)]
        for skew in (0, 1):                                # element-aligned only when skewed
            devs = [h.to(DEV)[skew: skew + numel] for h in hosts]
            hs = [bits(h)[skew: skew + numel] for h in hosts]
            out = torch.zeros(n * numel + 2, dtype=dtype, device=DEV)
            ov = out[skew: skew + n * numel]
            rc = lib.mhip_stack(ov.data_ptr(), _lib.ptr_array([d.data_ptr() for d in devs]), n, numel, es, None)
            assert rc == 0
            sync()
            assert np.array_equal(bits(ov), oracle.stack(hs).reshape(-1)), (dtype, n, per, skew)
            assert bits(out)[-1] == 0 and (skew == 0 or bits(out)[0] == 0)
            for rank in sorted({0, n // 2, n - 1}):
                o2 = torch.zeros(numel + 2, dtype=dtype, device=DEV)
                rc = lib.mhip_stack_scatter(o2[1: 1 + numel].data_ptr(), _lib.ptr_array([d.data_ptr() for d in devs]), n,
                                            rank, numel, es, None)
                assert rc == 0
                sync()
                assert np.array_equal(bits(o2)[1: 1 + numel], oracle.stack_scatter(hs, rank)), (dtype, n, per, rank)
                assert bits(o2)[0] == 0 and bits(o2)[-1] == 0
    # in place on the member's own tensor (stream.rs:1383-1384)
    per = 517
    hosts = [_rand(dtype, per * n, 77 + r) for r in range(n)]
    devs = [h.to(DEV) for h in hosts]
    rank = n - 1
    out = R.stream_reduce(devs, rank, R.Factory.of(devs[0]), R.Reduction.from_str("stack"), True, True)
    sync()
    assert out.data_ptr() == devs[rank].data_ptr()
    assert np.array_equal(bits(out), oracle.stack_scatter([bits(h) for h in hosts], rank))
    for g in range(n):
        if g != rank:
            assert np.array_equal(bits(devs[g]), bits(hosts[g]))       # peers untouched
