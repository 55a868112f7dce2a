"""Random cases for the differential tests of the GPU entry points (tests/test_gpu_fuzz.py): Slice pack / unpack against
numpy indexing, reduces and fp8 buckets against the CPU oracle.  Shapes are drawn around the sizes at which the library
switches kernels (tile, chunk, block and vector widths and their neighbours), buffers start at odd alignments, and guard
zones either side of every buffer catch stray writes.  Each `*_case` function runs one case and raises AssertionError
naming it; run as a program it repeats them for a number of seconds: python tests/fuzz_cases.py SECONDS SEED [pack|many|reduce|scatter|fp8 ...]."""
import ctypes as C
import math
import os
import random
import sys
import time

import numpy as np
import torch

sys.path.insert(0, os.path.dirname(os.path.dirname(os.path.abspath(__file__))))
import oracle  # noqa: E402
from monarch_amd import Slice, fp8  # noqa: E402
from monarch_amd import reduce as R  # noqa: E402
from monarch_amd._lib import check, lib, ptr_array  # noqa: E402
from monarch_amd.ndslice import slice_array  # noqa: E402

DEV = "cuda:0"
GUARD = 1 << 16
EXTENTS = [1, 2, 3, 7, 8, 15, 16, 17, 31, 32, 33, 63, 64, 65, 100, 127, 128, 129, 191, 192, 255, 256, 257, 300, 383, 384, 511, 512,
           513, 640, 1000, 1023, 1024, 1025, 2047, 2048, 2050, 4100]
LENGTHS = [1, 2, 7, 8, 9, 15, 16, 17, 63, 64, 65, 255, 256, 257, 1000, 1023, 1024, 1025, 2047, 2048, 2049, 4095, 4096, 4099, 8191,
           8192, 8193, 16384, 65535, 65536, 65537, 262144 + 3, 1048576, 1048577]
OPS = [(R.ReduceOp.Sum, oracle.SUM), (R.ReduceOp.Avg, oracle.AVG), (R.ReduceOp.Prod, oracle.PROD), (R.ReduceOp.Max, oracle.MAX),
       (R.ReduceOp.Min, oracle.MIN)]
GROW = 0.0   # log2 of FUZZ_SCALE: stretches the log-uniform size draws of a long run
FLOATS = [torch.float32, torch.bfloat16, torch.float16, torch.float64]
INTS = [torch.uint8, torch.int8, torch.int32, torch.int64]


def _raw(t):
    """Host bytes of a tensor."""
    return t.detach().cpu().contiguous().view(torch.uint8).numpy()


def _obits(t):
    """Host array in the form the oracle takes: 16-bit floats as their bit patterns."""
    t = t.detach().cpu().contiguous()
    return t.view(torch.uint16).numpy() if t.dtype in (torch.bfloat16, torch.float16) else t.numpy()


# ---- Slice pack / unpack ----

def random_slice(gen, max_elems, max_span):
    """A Slice that is valid by construction (each stride a multiple of the one below and at least its extent), with gaps,
    non-unit innermost strides and every order of dimensions; extents from EXTENTS or log-uniform."""
    while True:
        ndim = gen.choice([1, 2, 2, 2, 3, 3, 4])
        sizes, total = [], 1
        for _ in range(ndim):
            z = gen.choice(EXTENTS) if gen.random() < 0.5 else int(2 ** gen.uniform(0, 12.5 + GROW / 2))
            z = max(1, min(z, max(1, max_elems // total)))
            sizes.append(z)
            total *= z
        stride = gen.choice([1, 1, 1, 1, 2, 3])
        strides = []
        for z in sizes:
            strides.append(stride)
            kind = gen.random()
            gap = 0 if kind < 0.45 else gen.choice([1, 2, 3, 4, 8, 13, 64]) if kind < 0.8 else gen.randrange(0, 4 * z + 2)
            stride = stride * (z + gap) if z > 1 else stride * gen.choice([1, 1, 2, 5])
        order = list(range(ndim))
        r = gen.random()
        if r < 0.4:
            order.reverse()          # row-major
        elif r < 0.7:
            gen.shuffle(order)       # else column-major as built: a full transposition
        sizes = [sizes[o] for o in order]
        strides = [strides[o] for o in order]
        offset = gen.choice([0, 0, gen.randrange(0, 1000)])
        span = offset + sum((z - 1) * s for z, s in zip(sizes, strides)) + 1
        if span <= max_span:
            return Slice(offset=offset, sizes=sizes, strides=strides), span, total


def locations(s):
    """Slice::iter as an index array (row-major over sizes)."""
    loc = np.array([s.offset], dtype=np.int64)
    for z, st in zip(s.sizes, s.strides):
        loc = (loc[:, None] + (np.arange(z, dtype=np.int64) * st)[None, :]).reshape(-1)
    return loc


def pack_case(gen, tag, max_bytes=6 << 20, max_span_bytes=96 << 20):
    es = gen.choice([1, 1, 2, 2, 2, 3, 4, 4, 4, 6, 8, 8, 12, 16])
    s, span, total = random_slice(gen, max_bytes // es, max_span_bytes // es)
    mis = gen.choice([0, 0, 0, es, 2 * es, 16, 64, 1, 3, 128 - es]) if gen.random() < 0.6 else 0
    dmis = gen.choice([0, 0, 0, es, 16, 1, 5, 64, 256]) if gen.random() < 0.5 else 0
    desc = f"{tag} es={es} offset={s.offset} sizes={list(s.sizes)} strides={list(s.strides)} mis={mis} dmis={dmis}"
    stream = torch.cuda.current_stream().cuda_stream
    nbytes = span * es
    store = torch.randint(0, 256, (GUARD + mis + nbytes + GUARD,), dtype=torch.uint8, device=DEV)
    host = store.cpu().numpy()
    base = store[GUARD + mis: GUARD + mis + nbytes]
    out_store = torch.full((GUARD + dmis + total * es + GUARD,), 0xAB, dtype=torch.uint8, device=DEV)
    out = out_store[GUARD + dmis: GUARD + dmis + total * es]
    check(lib().mhip_slice_pack(out.data_ptr(), base.data_ptr(), C.byref(s.c), es, stream))
    torch.cuda.synchronize()
    loc = locations(s)
    want = host[GUARD + mis: GUARD + mis + nbytes].reshape(span, es)[loc].reshape(-1)
    got = out_store.cpu().numpy()
    a, b = GUARD + dmis, GUARD + dmis + total * es
    assert np.array_equal(got[a:b], want), f"pack differs: {desc}"
    assert np.all(got[:a] == 0xAB) and np.all(got[b:] == 0xAB), f"pack wrote outside its output: {desc}"
    assert np.array_equal(store.cpu().numpy(), host), f"pack wrote its source: {desc}"
    canvas = torch.full_like(store, 0x5C)
    cbase = canvas[GUARD + mis: GUARD + mis + nbytes]
    check(lib().mhip_slice_unpack(cbase.data_ptr(), out.data_ptr(), C.byref(s.c), es, stream))
    torch.cuda.synchronize()
    hc = np.full(host.size, 0x5C, dtype=np.uint8)
    hc[GUARD + mis: GUARD + mis + nbytes].reshape(span, es)[loc] = want.reshape(total, es)
    assert np.array_equal(canvas.cpu().numpy(), hc), f"unpack differs or wrote outside the view: {desc}"
    return total * es


def many_case(gen, tag, max_bytes=2 << 20, max_span_bytes=24 << 20):
    """Several views of one base through mhip_slice_pack_many / _unpack_many, staging buffers at staggered alignments."""
    es = gen.choice([1, 2, 2, 4, 4, 8, 16, 6])
    k = gen.choice([1, 2, 3, 5, 8, 8, 13])
    views, span = [], 1
    family = gen.random() < 0.5
    if family:   # column blocks of one matrix, as a reshard makes them (unequal widths, the last one ragged)
        rows, cols = gen.choice(EXTENTS[8:]), gen.choice(EXTENTS[10:])
        pitch = cols + gen.choice([0, 0, 1, 3, 8])
        cuts = sorted(gen.sample(range(1, cols), min(k - 1, cols - 1))) if cols > 1 else []
        for lo, hi in zip([0] + cuts, cuts + [cols]):
            views.append(Slice(offset=lo, sizes=[rows, hi - lo], strides=[pitch, 1]))
        span = rows * pitch
    else:
        for _ in range(k):
            v, sp, _ = random_slice(gen, max_bytes // es // k, max_span_bytes // es)
            views.append(v)
            span = max(span, sp)
    if gen.random() < 0.3:
        views.insert(gen.randrange(len(views) + 1), Slice(offset=0, sizes=[0], strides=[1]))   # an empty view among them
    mis = gen.choice([0, 0, es, 16, 1, 64])
    desc = f"{tag} many es={es} mis={mis} views={[(v.offset, list(v.sizes), list(v.strides)) for v in views]}"
    stream = torch.cuda.current_stream().cuda_stream
    nbytes = span * es
    store = torch.randint(0, 256, (GUARD + mis + nbytes + GUARD,), dtype=torch.uint8, device=DEV)
    host = store.cpu().numpy()
    hb = host[GUARD + mis: GUARD + mis + nbytes].reshape(span, es)
    base_ptr = store.data_ptr() + GUARD + mis
    lens = [len(v) * es for v in views]
    starts, pos = [], GUARD
    for i, n in enumerate(lens):
        pos += gen.choice([0, 1, es, 16, 3, 128])
        starts.append(pos)
        pos += n
    out_store = torch.full((pos + GUARD,), 0xAB, dtype=torch.uint8, device=DEV)
    outs = ptr_array([out_store.data_ptr() + st for st in starts])
    arr = slice_array(views)
    check(lib().mhip_slice_pack_many(outs, base_ptr, arr, len(views), es, stream))
    torch.cuda.synchronize()
    got = out_store.cpu().numpy()
    want = np.full(got.size, 0xAB, dtype=np.uint8)
    locs = [locations(v) for v in views]
    for st, n, loc in zip(starts, lens, locs):
        want[st: st + n] = hb[loc].reshape(-1)
    assert np.array_equal(got, want), f"pack_many differs or wrote outside its outputs: {desc}"
    canvas = torch.full_like(store, 0x5C)
    check(lib().mhip_slice_unpack_many(canvas.data_ptr() + GUARD + mis, outs, arr, len(views), es, stream))
    torch.cuda.synchronize()
    hc = np.full(host.size, 0x5C, dtype=np.uint8)
    for loc in locs:   # views may overlap: they carry the same bytes where they do
        hc[GUARD + mis: GUARD + mis + nbytes].reshape(span, es)[loc] = hb[loc]
    assert np.array_equal(canvas.cpu().numpy(), hc), f"unpack_many differs or wrote outside the views: {desc}"
    return sum(lens)


# ---- reduce ----

def _rand_host(gen, dtype, n, seed, scale):
    g = torch.Generator().manual_seed(seed)
    if dtype in FLOATS:
        x = (torch.randn(n, generator=g, dtype=torch.float64 if dtype == torch.float64 else torch.float32) * scale).to(dtype)
        if gen.random() < 0.2:
            for _ in range(3):
                x[gen.randrange(n)] = gen.choice([float("nan"), float("inf"), -float("inf"), 0.0, -0.0])
        return x
    if dtype == torch.uint8:
        return torch.randint(0, 256, (n,), dtype=dtype, generator=g)
    info = torch.iinfo(dtype)
    return torch.randint(info.min, info.max, (n,), dtype=dtype, generator=g)


def _same(got, want, dtype):
    if dtype in (torch.float32, torch.float64):   # NaN payloads are not part of the contract; positions, values and zero signs are
        ok = ~np.isnan(want)
        return (np.array_equal(np.isnan(got), ~ok) and np.array_equal(got[ok], want[ok])
                and np.array_equal(np.signbit(got[ok]), np.signbit(want[ok])))
    return np.array_equal(got, want)


def reduce_case(gen, tag, max_numel=1 << 21):
    dtype = gen.choice(FLOATS + FLOATS + INTS)
    n = gen.choice([1, 2, 2, 3, 4, 5, 7, 8, 8, 8, 9, 12, 16, 17, 24])
    numel = min(max_numel, gen.choice(LENGTHS) if gen.random() < 0.6 else int(2 ** gen.uniform(0, 21 + GROW)))
    op, code = gen.choice(OPS)
    if dtype in INTS and op == R.ReduceOp.Avg:
        op, code = OPS[0]
    scale = 1.0 if op == R.ReduceOp.Prod else gen.choice([0.02, 1.0, 1e3])
    pads = [gen.choice([0, 0, 1, 2, 3, 5, 8]) for _ in range(n)]
    alias = gen.choice([None, None, gen.randrange(n)])
    opad = gen.choice([0, 1, 3, 4])
    desc = f"{tag} reduce {dtype} n={n} numel={numel} op={op.name} pads={pads} alias={alias} opad={opad}"
    hosts = [_rand_host(gen, dtype, numel, gen.randrange(1 << 30), scale) for _ in range(n)]
    stores = [torch.zeros(numel + p + 4, dtype=dtype, device=DEV) for p in pads]
    views = []
    for st, p, h in zip(stores, pads, hosts):
        v = st[p: p + numel]
        v.copy_(h)
        views.append(v)
    if alias is None:
        ostore = torch.zeros(numel + opad + 4, dtype=dtype, device=DEV)
        out = ostore[opad: opad + numel]
    else:
        ostore, out, opad = stores[alias], views[alias], pads[alias]
    R.all_reduce(out, views, op)
    torch.cuda.synchronize()
    if code in (oracle.SUM, oracle.AVG) and dtype in FLOATS:
        want = oracle.reduce([_obits(h) for h in hosts], code, half=dtype == torch.float16)
    else:
        want = oracle.reduce_op([_obits(h) for h in hosts], code, kind="f16" if dtype == torch.float16 else None)
    assert _same(_obits(out), want, dtype), f"reduce differs: {desc}"
    full = _raw(ostore).reshape(-1, ostore.element_size())
    assert not full[:opad].any() and not full[opad + numel:].any(), f"reduce wrote outside its output: {desc}"
    for r in range(n):
        assert r == alias or np.array_equal(_raw(views[r]), _raw(hosts[r])), f"reduce wrote input {r}: {desc}"
    return numel * n


def scatter_case(gen, tag, max_len=1 << 18):
    """mhip_reduce_scatter: members read through a random view (or contiguous), the reduced index space cut into contiguous
    chunks (the dim-0 rule), column blocks (the fused last-dim form) or strided selections.  Checked against the oracle's
    plain reduce of the gathered inputs, indexed with numpy."""
    dtype = gen.choice([torch.float32, torch.float32, torch.bfloat16, torch.bfloat16, torch.float16, torch.float64, torch.int32])
    G = gen.choice([1, 2, 3, 5, 8, 8, 16])
    op, code = gen.choice(OPS)
    if dtype == torch.int32 and op == R.ReduceOp.Avg:
        op, code = OPS[0]
    es = torch.empty(0, dtype=dtype).element_size()
    if gen.random() < 0.5:
        in_view, L = None, min(max_len, gen.choice(LENGTHS) if gen.random() < 0.5 else int(2 ** gen.uniform(3, 18 + GROW)))
        span, loc_in = L, None
    else:
        in_view, span, L = random_slice(gen, max_len, (16 << 20) // es)
        loc_in = locations(in_view)
    form = gen.choice(["chunks", "columns", "strided"]) if L >= 8 else "strided"
    out_views = []
    if form == "chunks":
        parts = gen.choice([p for p in (1, 2, 4, 8) if L % p == 0])
        c = L // parts
        out_views = [Slice(offset=r * c, sizes=[c], strides=[1]) for r in gen.sample(range(parts), gen.randrange(1, parts + 1))]
    elif form == "columns":
        cols = gen.choice([d for d in (2, 3, 4, 8, 16, 24, 64, 100, 128, 512, 1000, 4096) if L % d == 0] or [1])
        rows = L // cols
        cuts = sorted(gen.sample(range(1, cols), min(gen.choice([0, 1, 3, 7]), cols - 1))) if cols > 1 else []
        out_views = [Slice(offset=lo, sizes=[rows, hi - lo], strides=[cols, 1]) for lo, hi in zip([0] + cuts, cuts + [cols])]
    else:
        for _ in range(gen.choice([1, 2, 4])):
            st = gen.choice([1, 1, 2, 3, 7])
            n = gen.randrange(1, max(2, (L - 1) // st + 1))
            out_views.append(Slice(offset=gen.randrange(0, L - (n - 1) * st), sizes=[n], strides=[st]))
    desc = (f"{tag} scatter {dtype} G={G} op={op.name} L={L} in_view="
            f"{None if in_view is None else (in_view.offset, list(in_view.sizes), list(in_view.strides))} "
            f"outs={[(v.offset, list(v.sizes), list(v.strides)) for v in out_views[:8]]}")
    scale = 1.0 if op == R.ReduceOp.Prod else gen.choice([0.02, 1.0])
    hosts = [_rand_host(gen, dtype, span, gen.randrange(1 << 30), scale) for _ in range(G)]
    group = [h.to(DEV) for h in hosts]
    pads = [gen.choice([0, 0, 1, 3, 4]) for _ in out_views]
    ostores = [torch.zeros(len(v) + p + 4, dtype=dtype, device=DEV) for v, p in zip(out_views, pads)]
    outs = [st[p: p + len(v)] for st, p, v in zip(ostores, pads, out_views)]
    R.reduce_scatter_views(outs, out_views, group, in_view, op)
    torch.cuda.synchronize()
    gathered = [_obits(h) if loc_in is None else _obits(h)[loc_in] for h in hosts]
    if code in (oracle.SUM, oracle.AVG) and dtype in FLOATS:
        red = oracle.reduce(gathered, code, half=dtype == torch.float16)
    else:
        red = oracle.reduce_op(gathered, code, kind="f16" if dtype == torch.float16 else None)
    for k, (o, v, st, p) in enumerate(zip(outs, out_views, ostores, pads)):
        assert _same(_obits(o), red[locations(v)], dtype), f"output {k} differs: {desc}"
        full = _raw(st).reshape(-1, es)
        assert not full[:p].any() and not full[p + len(v):].any(), f"wrote beside output {k}: {desc}"
    for h, d in zip(hosts, group):
        assert np.array_equal(_raw(d), _raw(h)), f"reduce_scatter wrote an input: {desc}"
    return L * G


# ---- fp8 buckets ----

def _gradient_like(gen, total, seed):
    g = torch.Generator().manual_seed(seed)
    x = torch.randn(total, generator=g)
    x = torch.where(torch.rand(total, generator=g) < 0.001, x * 50, x)
    if gen.random() < 0.3:
        x = x * gen.choice([1e-30, 1e-3, 1e4, 1e30])
    return x.bfloat16()


def fp8_case(gen, tag, max_tensor=300000):
    ntens = gen.choice([1, 2, 3, 5, 17, 40, 64, 65, 130, 300])
    kinds = [(0, 1), (1, 9), (9, 600), (600, 1500), (1500, 5000), (5000, 40000), (40000, max(40001, max_tensor))]
    sizes = []
    for _ in range(ntens):
        lo, hi = gen.choice(kinds)
        nn = gen.randrange(lo, hi)
        sizes.append(nn // 8 * 8 if gen.random() < 0.3 else nn)
    if sum(sizes) == 0:
        sizes[0] = 5
    if gen.random() < 0.4:
        sizes[-1] += (-sum(sizes)) % 1024      # no short last block
    total = sum(sizes)
    indexed = gen.choice([True, False])
    npeers = gen.choice([1, 1, 2, 3, 8])
    desc = f"{tag} fp8 ntens={ntens} total={total} indexed={indexed} npeers={npeers} sizes={sizes if ntens <= 40 else sizes[:40]}"
    offs = np.concatenate([[0], np.cumsum(sizes)]).astype(np.int64)
    flat_h = _gradient_like(gen, total, gen.randrange(1 << 30))
    for _ in range(gen.choice([0, 0, 3, 8])):
        flat_h[gen.randrange(total)] = gen.choice([float("nan"), float("inf"), -float("inf")])
    store = [torch.zeros(nn + 6, dtype=torch.bfloat16, device=DEV) for nn in sizes]
    dev = []
    for i, (st, nn) in enumerate(zip(store, sizes)):
        sh = gen.randrange(0, 5)
        v = st[sh: sh + nn]
        v.copy_(flat_h[offs[i]: offs[i + 1]])
        dev.append(v)
    bucket = fp8.FlatBucket(dev)
    q1, s1 = fp8.quantize_bucket(bucket, indexed=indexed)
    flat = bucket.pack(indexed=indexed)
    q2, s2 = fp8.quantize(flat)
    torch.cuda.synchronize()
    wq, ws = oracle.fp8_quantize(_obits(flat_h), 1024)
    assert np.array_equal(_obits(flat), _obits(flat_h)), f"flat pack differs: {desc}"
    for name, q, s in (("fused", q1, s1), ("flat", q2, s2)):
        assert np.array_equal(q.cpu().numpy(), wq), f"{name} quantiser codes differ: {desc}"
        assert np.array_equal(s.cpu().numpy().view(np.uint32), ws.view(np.uint32)), f"{name} quantiser scales differ: {desc}"
    # receive side: peers' payloads derived from the codes, kept free of NaN codes and non-finite scales
    qf = q1.clone()
    qf[(qf & 0x7F) == 0x7F] = 0x23
    peers_q = [torch.where(((qf ^ (k * 0x11)) & 0x7F) == 0x7F, torch.full_like(qf, 0x31), qf ^ (k * 0x11)) for k in range(npeers)]
    peers_s = [torch.where(torch.isfinite(s1), s1, torch.ones_like(s1)) * (1.0 + 0.25 * k) for k in range(npeers)]
    acc_h = np.random.default_rng(gen.randrange(1 << 30)).normal(size=total).astype(np.float32)
    astore = [torch.zeros(nn + 3, dtype=torch.float32, device=DEV) for nn in sizes]
    accs = []
    for i, (st, nn) in enumerate(zip(astore, sizes)):
        sh = gen.randrange(0, 3)
        a = st[sh: sh + nn]
        a.copy_(torch.from_numpy(acc_h[offs[i]: offs[i + 1]]))
        accs.append((a, sh))
    abucket = fp8.FlatBucket([a for a, _ in accs])
    acc_flat = torch.from_numpy(acc_h.copy()).to(DEV)
    if npeers == 1:
        fp8.dequant_accumulate_bucket(abucket, peers_q[0], peers_s[0], indexed=indexed)
        fp8.dequant_accumulate(acc_flat, peers_q[0], peers_s[0])
    else:
        fp8.dequant_accumulate_bucket_many(abucket, peers_q, peers_s, indexed=indexed)
        fp8.dequant_accumulate_many(acc_flat, peers_q, peers_s)
    for pq, ps in zip(peers_q, peers_s):
        oracle.fp8_dequant_accumulate(acc_h, pq.cpu().numpy(), ps.cpu().numpy(), 1024)
    torch.cuda.synchronize()
    assert np.array_equal(acc_flat.cpu().numpy().view(np.uint32), acc_h.view(np.uint32)), f"flat dequantiser differs: {desc}"
    for i, ((a, sh), st, nn) in enumerate(zip(accs, astore, sizes)):
        assert np.array_equal(a.cpu().numpy().view(np.uint32), acc_h[offs[i]: offs[i + 1]].view(np.uint32)), \
            f"fused dequantiser differs in tensor {i}: {desc}"
        assert st[:sh].abs().sum() == 0 and st[sh + nn:].abs().sum() == 0, f"fused dequantiser wrote beside tensor {i}: {desc}"
    outs = [torch.empty(nn, dtype=torch.float32, device=DEV) for nn in sizes]
    fp8.FlatBucket(outs).unpack(acc_flat, outs, indexed=indexed)
    torch.cuda.synchronize()
    for i, o in enumerate(outs):
        assert np.array_equal(o.cpu().numpy().view(np.uint32), acc_h[offs[i]: offs[i + 1]].view(np.uint32)), \
            f"flat unpack differs in tensor {i}: {desc}"
    return total


CASES = {"pack": pack_case, "many": many_case, "reduce": reduce_case, "scatter": scatter_case, "fp8": fp8_case}


def long_run(seconds, seed, kinds):
    gen = random.Random(seed)
    t0, n = time.time(), {k: 0 for k in kinds}
    global GROW
    scale = int(os.environ.get("FUZZ_SCALE", "1"))   # FUZZ_SCALE=8: cases up to eight times as large (fewer of them per second)
    GROW = math.log2(scale)
    bounds = {"pack": dict(max_bytes=(6 << 20) * scale, max_span_bytes=(96 << 20) * scale),
              "many": dict(max_bytes=(2 << 20) * scale, max_span_bytes=(24 << 20) * scale),
              "reduce": dict(max_numel=(1 << 21) * scale), "scatter": dict(max_len=(1 << 18) * scale),
              "fp8": dict(max_tensor=300000 * scale)}
    while time.time() - t0 < seconds:
        k = gen.choice(kinds)
        tag = f"seed {seed} case {sum(n.values())}"
        print(tag, k, flush=True)  # names the case before anything of it runs on the GPU
        CASES[k](gen, tag, **bounds[k])
        n[k] += 1
    print("ok:", ", ".join(f"{v} {k}" for k, v in n.items()), f"in {time.time() - t0:.0f} s, seed {seed}", flush=True)


if __name__ == "__main__":
    long_run(float(sys.argv[1]) if len(sys.argv) > 1 else 60.0, int(sys.argv[2]) if len(sys.argv) > 2 else 1,
             sys.argv[3:] or list(CASES))
