"""GPU parity: block-scaled fp8 codec and flat bucket pack/unpack against the CPU oracle."""
import numpy as np
import pytest
import torch

import oracle
from monarch_amd import fp8
from util import bits, sync

pytestmark = pytest.mark.gpu
DEV = "cuda:0"


def _c5_like(n, seed, device="cpu"):
    g = torch.Generator(device=device).manual_seed(seed)
    x = torch.randn(n, generator=g, device=device)
    out = torch.rand(n, generator=g, device=device) < 1e-3
    return torch.where(out, x * 50, x).bfloat16()


def _check_quant(x: torch.Tensor):
    q, s = fp8.quantize(x.to(DEV))
    sync()
    wq, ws = oracle.fp8_quantize(bits(x), 1024)
    gq = q.cpu().numpy()
    assert np.array_equal(gq, wq)                      # every code, the sign bit of NaN codes included
    assert np.array_equal(s.cpu().numpy().view(np.uint32), ws.view(np.uint32))
    return q, s


def test_every_bf16_pattern_at_unit_scale():
    # blocks whose absmax is exactly 448 have inv == 1: the codes are the bare e4m3fn RNE conversion of
    # every finite bf16 value up to 448 (pinned against the format via the oracle's torch-checked encoder)
    h = torch.arange(65536, dtype=torch.int32).to(torch.uint16).view(torch.bfloat16)
    vals = h[(h.float().abs() <= 448) & ~h.float().isnan()]
    per = 1023
    nblk = (vals.numel() + per - 1) // per
    x = torch.zeros(nblk * 1024, dtype=torch.bfloat16)
    xv = x.view(nblk, 1024)
    xv[:, 0] = 448.0
    pad = torch.zeros(nblk * per, dtype=torch.bfloat16)
    pad[: vals.numel()] = vals
    xv[:, 1:] = pad.view(nblk, per)
    q, s = _check_quant(x)
    assert torch.all(s == 1.0)
    direct = np.array([oracle.e4m3fn_encode(float(v), True) for v in x.float().numpy()], dtype=np.uint8)
    assert np.array_equal(q.cpu().numpy(), direct)


def test_every_bf16_pattern_mixed_scales():
    h = torch.arange(65536, dtype=torch.int32).to(torch.uint16).view(torch.bfloat16)
    g = torch.Generator().manual_seed(0)
    perm = torch.randperm(65536, generator=g)
    _check_quant(h[perm])            # NaN / Inf blocks take the careful path
    finite = h[~h.float().isnan() & ~h.float().isinf()]
    _check_quant(finite[torch.randperm(finite.numel(), generator=g)])
    _check_quant(finite.sort().values)  # blocks of similar magnitude, including all-denormal ones


def test_edge_blocks():
    z = torch.zeros(2048, dtype=torch.bfloat16)
    z[1024:] = -0.0
    q, s = _check_quant(z)
    assert torch.all(q[:1024] == 0) and torch.all(q[1024:] == 0x80)
    x = torch.ones(4096, dtype=torch.bfloat16)
    x[3] = float("nan")
    x[5] = -2.0
    x[1024 + 7] = float("inf")
    x[1024 + 8] = float("-inf")
    x[2048 + 10] = 50.0
    x[3072:] = 1e-30
    q, s = _check_quant(x)
    qc = q.cpu()
    assert (qc[3] & 0x7F) == 0x7F and qc[5] == 0xFE and qc[1024 + 7] == 0x7E and qc[1024 + 8] == 0xFE
    for n in (1, 5, 1023, 1025, 2047, 4097):  # short tails
        _check_quant(_c5_like(n, seed=n))


def test_quantize_dequant_accumulate_ragged():
    g = torch.Generator().manual_seed(5000)
    sizes = torch.exp(torch.rand(40, generator=g) * (np.log(2**17) - np.log(2**10)) + np.log(2**10)).round().long().tolist()
    sizes += [1, 2, 1024, 1023, 1025]
    tensors = [_c5_like(n, seed=5000 + i) for i, n in enumerate(sizes)]
    dev = [t.to(DEV) for t in tensors]
    bucket = fp8.FlatBucket(dev)
    flat = bucket.pack()
    sync()
    hflat = oracle.flat_pack([bits(t) for t in tensors], bucket.offsets)
    assert np.array_equal(bits(flat), hflat)
    q, s = fp8.quantize(flat)
    sync()
    wq, ws = oracle.fp8_quantize(hflat, 1024)
    assert np.array_equal(q.cpu().numpy(), wq) and np.array_equal(s.cpu().numpy(), ws)
    rng = np.random.default_rng(1)
    acc_h = rng.normal(size=bucket.total).astype(np.float32)
    acc = torch.from_numpy(acc_h.copy()).to(DEV)
    for _ in range(3):  # accumulate the same payload three times
        fp8.dequant_accumulate(acc, q, s)
        oracle.fp8_dequant_accumulate(acc_h, wq, ws, 1024)
    sync()
    assert np.array_equal(acc.cpu().numpy().view(np.uint32), acc_h.view(np.uint32))
    outs = [torch.empty(n, dtype=torch.float32, device=DEV) for n in sizes]
    bucket.unpack(acc, outs)
    sync()
    want = oracle.flat_unpack(acc_h, bucket.offsets)
    for o, w in zip(outs, want):
        assert np.array_equal(o.cpu().numpy(), w)


@pytest.mark.parametrize("npeers", [1, 2, 3, 4, 8, 9, 17])
def test_dequant_accumulate_from_many_peers(npeers):
    # one pass over n peers' payloads == n single-peer passes, bit for bit, also when starting from zero
    for numel in (1, 1023, 2048, 2 * 1024 * 7 + 5, 300_000):
        payloads = []
        for r in range(npeers):
            x = _c5_like(numel, seed=31 * npeers + r) * float(1 + r % 3)
            wq, ws = oracle.fp8_quantize(bits(x), 1024)
            payloads.append((wq, ws))
        rng = np.random.default_rng(numel)
        acc_h = rng.normal(size=numel).astype(np.float32)
        qs = [torch.from_numpy(wq).to(DEV) for wq, _ in payloads]
        ss = [torch.from_numpy(ws).to(DEV) for _, ws in payloads]
        for overwrite in (False, True):
            want = np.zeros(numel, dtype=np.float32) if overwrite else acc_h.copy()
            for wq, ws in payloads:
                oracle.fp8_dequant_accumulate(want, wq, ws, 1024)
            store = torch.full((numel + 2,), 7.0, device=DEV)
            acc = store[1:-1]
            acc.copy_(torch.from_numpy(acc_h))
            fp8.dequant_accumulate_many(acc, qs, ss, overwrite=overwrite)
            sync()
            assert np.array_equal(acc.cpu().numpy().view(np.uint32), want.view(np.uint32)), (npeers, numel, overwrite)
            assert store[0].item() == 7.0 and store[-1].item() == 7.0
            if not overwrite:   # and the same as the single-peer entry point called n times
                seq = torch.from_numpy(acc_h.copy()).to(DEV)
                for q, s_ in zip(qs, ss):
                    fp8.dequant_accumulate(seq, q, s_)
                sync()
                assert torch.equal(seq, acc)


@pytest.mark.parametrize("npeers", [1, 3, 4, 8, 9])
def test_dequant_accumulate_bucket_from_many_peers(npeers):
    sizes = [1024, 3000, 1, 7777, 2048, 513, 40_000, 5]
    total = sum(sizes)
    payloads = []
    for r in range(npeers):
        x = _c5_like(total, seed=77 * npeers + r) * float(1 + r % 4)
        payloads.append(oracle.fp8_quantize(bits(x), 1024))
    qs = [torch.from_numpy(wq).to(DEV) for wq, _ in payloads]
    ss = [torch.from_numpy(ws).to(DEV) for _, ws in payloads]
    rng = np.random.default_rng(npeers)
    acc_h = rng.normal(size=total).astype(np.float32)
    offs = np.concatenate([[0], np.cumsum(sizes)])
    accs = [torch.from_numpy(acc_h[offs[i]: offs[i + 1]].copy()).to(DEV) for i in range(len(sizes))]
    bucket = fp8.FlatBucket(accs)
    fp8.dequant_accumulate_bucket_many(bucket, qs, ss)
    sync()
    want = acc_h.copy()
    for wq, ws in payloads:
        oracle.fp8_dequant_accumulate(want, wq, ws, 1024)
    got = torch.cat(accs).cpu().numpy()
    assert np.array_equal(got.view(np.uint32), want.view(np.uint32)), npeers


def test_fused_bucket_forms_equal_two_step_pipeline():
    # ragged sizes around block boundaries, empty tensors, odd element alignment, NaN/Inf blocks
    g = torch.Generator().manual_seed(77)
    sizes = [1500, 0, 1024, 7, 3, 2048, 1, 1023, 1025, 4096 + 5, 0, 9, 8 * 1024, 333]
    tensors = []
    for i, n in enumerate(sizes):
        t = _c5_like(n, seed=700 + i)
        if i == 5:
            t[100] = float("nan"); t[1500] = float("inf")
        tensors.append(t)
    store = [torch.zeros(n + 6, dtype=torch.bfloat16, device=DEV) for n in sizes]
    dev = []
    for i, (t, st) in enumerate(zip(tensors, store)):
        v = st[i % 4: i % 4 + t.numel()]  # 2-byte aligned only
        v.copy_(t)
        dev.append(v)
    bucket = fp8.FlatBucket(dev)
    q2, s2 = fp8.quantize(bucket.pack())
    q1, s1 = fp8.quantize_bucket(bucket)
    sync()
    assert torch.equal(q1, q2) and torch.equal(s1.view(torch.int32), s2.view(torch.int32))
    wq, ws = oracle.fp8_quantize(oracle.flat_pack([bits(t) for t in tensors], bucket.offsets), 1024)
    nan = (wq & 0x7F) == 0x7F
    assert np.array_equal(q1.cpu().numpy()[~nan], wq[~nan]) and np.array_equal(s1.cpu().numpy(), ws)
    # receive side: accumulate twice into per-tensor fp32 buffers vs flat accumulate + unpack
    rng = np.random.default_rng(3)
    acc_h = rng.normal(size=bucket.total).astype(np.float32)
    outs_store = [torch.zeros(n + 3, dtype=torch.float32, device=DEV) for n in sizes]
    outs = [st[i % 3: i % 3 + n] for i, (st, n) in enumerate(zip(outs_store, sizes))]
    offs = bucket.offsets
    for o, lo, hi in zip(outs, offs[:-1], offs[1:]):
        o.copy_(torch.from_numpy(acc_h[lo:hi]))
    abucket = fp8.FlatBucket(outs)
    qf = q1.clone()
    qf[(qf & 0x7F) == 0x7F] = 0x11  # keep the comparison free of NaN
    wq2 = qf.cpu().numpy()
    for _ in range(2):
        fp8.dequant_accumulate_bucket(abucket, qf, s1)
        oracle.fp8_dequant_accumulate(acc_h, wq2, ws, 1024)
    sync()
    want = oracle.flat_unpack(acc_h, offs)
    for o, w, st, i, n in zip(outs, want, outs_store, range(len(sizes)), sizes):
        assert np.array_equal(o.cpu().numpy().view(np.uint32), w.view(np.uint32))
        assert st[: i % 3].abs().sum() == 0 and st[i % 3 + n:].abs().sum() == 0  # neighbours untouched


@pytest.mark.parametrize("seed", [1, 2, 3, 4, 5, 6])
@pytest.mark.parametrize("indexed", [True, False])
def test_spans_and_blocks_shared_by_tensors(seed, indexed):
    # The fused forms load a span (4 blocks) or a block that one boundary between tensors cuts in one go, take the
    # careful path for more boundaries and for the short last block, and put off blocks with Inf / NaN until the rest
    # of their span is done.  Random mixes of tensor sizes put boundaries everywhere: on and off multiples of 8
    # elements, in the first and last vector of a span, several in one block, empty tensors between them; Inf and
    # NaN land in blocks of every kind; tensors start on 2-byte (4-byte for the accumulators) boundaries only.
    rng = np.random.default_rng(9000 + seed)
    kinds = [(1, 9), (9, 600), (600, 1500), (1500, 5000), (5000, 40000)]
    sizes = []
    for _ in range(int(rng.integers(12, 40))):
        lo, hi = kinds[int(rng.integers(0, len(kinds)))]
        n = int(rng.integers(lo, hi))
        if rng.random() < 0.3:
            n = n // 8 * 8                      # cuts on whole vectors too
        sizes.append(0 if rng.random() < 0.05 else n)
    if seed % 2:
        sizes[-1] += (-sum(sizes)) % 1024       # odd seeds: no short last block
    total = sum(sizes)
    offs = np.concatenate([[0], np.cumsum(sizes)]).astype(np.int64)
    flat_h = _c5_like(total, seed=seed)
    for pos in rng.integers(0, total, size=6):  # Inf / NaN in six blocks
        flat_h[int(pos)] = float("nan") if pos % 2 else float("-inf")
    store = [torch.zeros(n + 6, dtype=torch.bfloat16, device=DEV) for n in sizes]
    dev = []
    for i, (st, n) in enumerate(zip(store, sizes)):
        v = st[i % 4: i % 4 + n]
        v.copy_(flat_h[offs[i]: offs[i + 1]])
        dev.append(v)
    bucket = fp8.FlatBucket(dev)
    q1, s1 = fp8.quantize_bucket(bucket, indexed=indexed)
    sync()
    wq, ws = oracle.fp8_quantize(bits(flat_h), 1024)
    assert np.array_equal(q1.cpu().numpy(), wq), (seed, sizes)
    assert np.array_equal(s1.cpu().numpy().view(np.uint32), ws.view(np.uint32)), (seed, sizes)
    # receive side: one peer, then three peers in one pass, into staggered fp32 accumulators
    qf = q1.clone()
    qf[(qf & 0x7F) == 0x7F] = 0x23              # keep the sums free of NaN
    peers_q = [qf, qf ^ 0x05, qf ^ 0x40]
    peers_q = [torch.where((p & 0x7F) == 0x7F, torch.full_like(p, 0x31), p) for p in peers_q]
    peers_s = [s1, s1 * 0.5, s1 * 1.25]
    acc_h = rng.normal(size=total).astype(np.float32)
    astore = [torch.zeros(n + 3, dtype=torch.float32, device=DEV) for n in sizes]
    accs = [st[i % 3: i % 3 + n] for i, (st, n) in enumerate(zip(astore, sizes))]
    for a, lo, hi in zip(accs, offs[:-1], offs[1:]):
        a.copy_(torch.from_numpy(acc_h[lo:hi]))
    abucket = fp8.FlatBucket(accs)
    fp8.dequant_accumulate_bucket(abucket, peers_q[0], peers_s[0], indexed=indexed)
    oracle.fp8_dequant_accumulate(acc_h, peers_q[0].cpu().numpy(), peers_s[0].cpu().numpy(), 1024)
    fp8.dequant_accumulate_bucket_many(abucket, peers_q, peers_s, indexed=indexed)
    for pq, ps in zip(peers_q, peers_s):
        oracle.fp8_dequant_accumulate(acc_h, pq.cpu().numpy(), ps.cpu().numpy(), 1024)
    sync()
    for i, (a, st, n) in enumerate(zip(accs, astore, sizes)):
        assert np.array_equal(a.cpu().numpy().view(np.uint32), acc_h[offs[i]: offs[i + 1]].view(np.uint32)), (seed, i, sizes)
        assert st[: i % 3].abs().sum() == 0 and st[i % 3 + n:].abs().sum() == 0  # neighbours untouched
    for i, (st, n) in enumerate(zip(store, sizes)):                              # the quantiser only reads
        assert st[: i % 4].abs().sum() == 0 and st[i % 4 + n:].abs().sum() == 0


@pytest.mark.parametrize("ntensors", [1, 2, 64, 65, 66, 67, 130, 4225, 4226, 9000])
def test_many_small_tensors_table_search(ntensors):
    # exercises the cooperative table search at its range boundaries (65-ary steps) with empty tensors mixed in
    g = torch.Generator().manual_seed(ntensors)
    sizes = torch.randint(0, 4, (ntensors,), generator=g).tolist()
    sizes[ntensors // 2] = 3000
    if sum(sizes) == 0:
        sizes[0] = 5
    total = sum(sizes)
    big = _c5_like(total, seed=ntensors)
    offs = np.concatenate([[0], np.cumsum(sizes)]).tolist()
    dbig = big.to(DEV)
    dev = [dbig[offs[i]: offs[i + 1]].clone() if sizes[i] else dbig[:0] for i in range(ntensors)]
    bucket = fp8.FlatBucket(dev)
    flat = bucket.pack()
    sync()
    assert torch.equal(flat.view(torch.int16), dbig.view(torch.int16))
    q1, s1 = fp8.quantize_bucket(bucket)
    q2, s2 = fp8.quantize(flat)
    sync()
    assert torch.equal(q1, q2) and torch.equal(s1, s2)
    accs = [torch.zeros(n, dtype=torch.float32, device=DEV) for n in sizes]
    fp8.dequant_accumulate_bucket(fp8.FlatBucket(accs), q1, s1)
    acc = torch.zeros(total, dtype=torch.float32, device=DEV)
    fp8.dequant_accumulate(acc, q1, s1)
    outs = [torch.empty(n, dtype=torch.float32, device=DEV) for n in sizes]
    bucket.unpack(acc, outs)
    sync()
    assert torch.equal(torch.cat(accs), acc) and torch.equal(torch.cat(outs), acc)


def test_flat_pack_alignment_and_empty_tensors():
    g = torch.Generator().manual_seed(3)
    for dtype, sizes in ((torch.uint8, [3, 0, 17, 1, 4096, 0, 5]), (torch.bfloat16, [1, 3, 0, 8, 1025, 7]),
                         (torch.float32, [5, 1, 0, 2049]), (torch.float64, [3, 1, 1000])):
        tensors = [torch.randint(0, 255, (n,), generator=g).to(dtype) for n in sizes]
        store = [torch.zeros(n + 4, dtype=dtype, device=DEV) for n in sizes]
        dev = []
        for i, (t, st) in enumerate(zip(tensors, store)):
            v = st[i % 3: i % 3 + t.numel()]  # staggered, only element-aligned
            v.copy_(t)
            dev.append(v)
        bucket = fp8.FlatBucket(dev)
        for shift, indexed in ((0, False), (1, False), (3, False), (0, True), (1, True), (3, True)):  # flat buffer alignment
            fstore = torch.zeros(bucket.total + 8, dtype=dtype, device=DEV)
            flat = fstore[shift: shift + bucket.total]
            bucket.pack(flat, indexed=indexed)
            sync()
            want = oracle.flat_pack([bits(t) for t in tensors], bucket.offsets)
            assert np.array_equal(bits(flat), want)
            assert fstore[:shift].abs().sum() == 0 and fstore[shift + bucket.total:].abs().sum() == 0
            outs = [torch.zeros(n + 2, dtype=dtype, device=DEV)[1: 1 + n] for n in sizes]
            bucket.unpack(flat, outs, indexed=indexed)
            sync()
            for o, t in zip(outs, tensors):
                assert torch.equal(o.cpu(), t)


@pytest.mark.parametrize("dtype", [torch.uint8, torch.bfloat16, torch.float32, torch.float64, torch.complex128])
def test_flat_copies_with_block_index_match_table_search(dtype):
    """The indexed form (one wavefront per 1 KiB row of the flat buffer, tensor found through the block index, each XCD
    on a contiguous share of the rows) and the table-search form move the same bytes: rows inside one tensor, rows that
    straddle many small or empty tensors, a bucket shorter than a row, guard elements around every destination."""
    rng = np.random.default_rng(77)
    es = torch.empty(0, dtype=dtype).element_size()
    row = 1024 // es  # elements per 1 KiB row
    for trial, sizes in enumerate((
            [3],
            [row - 1, 1, row, row + 1, 0, 0, 5 * row + 3],
            rng.integers(0, 12, size=300).tolist() + [7 * row + 1] + rng.integers(0, 3 * row, size=90).tolist(),
            np.round(np.exp(rng.uniform(np.log(2**4), np.log(2**17), size=120))).astype(np.int64).tolist() + [0, 1])):
        host = [torch.from_numpy(rng.integers(0, 256, size=n * es, dtype=np.uint8)) for n in sizes]
        store = [torch.zeros(n * es + 64, dtype=torch.uint8, device=DEV) for n in sizes]
        dev = []
        for i, (h, st) in enumerate(zip(host, store)):
            v = st[(i % 4) * es: (i % 4) * es + h.numel()]  # staggered, only element-aligned
            v.copy_(h)
            dev.append(v.view(dtype))
        bucket = fp8.FlatBucket(dev)
        want = np.concatenate([h.numpy() for h in host])
        for shift in (0, 1):
            flats = []
            for indexed in (False, True):
                fstore = torch.full(((bucket.total + 8) * es,), 0xA5, dtype=torch.uint8, device=DEV)
                flat = fstore[shift * es: (shift + bucket.total) * es].view(dtype)
                bucket.pack(flat, indexed=indexed)
                sync()
                got = fstore.cpu().numpy()
                assert np.array_equal(got[shift * es: (shift + bucket.total) * es], want), (trial, shift, indexed)
                assert (got[:shift * es] == 0xA5).all() and (got[(shift + bucket.total) * es:] == 0xA5).all()
                flats.append(flat)
                ostore = [torch.full((n * es + 64,), 0x5A, dtype=torch.uint8, device=DEV) for n in sizes]
                outs = [st[(1 + i % 3) * es: (1 + i % 3) * es + n * es].view(dtype) for i, (st, n) in enumerate(zip(ostore, sizes))]
                bucket.unpack(flat, outs, indexed=indexed)
                sync()
                for i, (st, h, n) in enumerate(zip(ostore, host, sizes)):
                    o = st.cpu().numpy()
                    lo = (1 + i % 3) * es
                    assert np.array_equal(o[lo: lo + n * es], h.numpy()), (trial, shift, indexed, i)
                    assert (o[:lo] == 0x5A).all() and (o[lo + n * es:] == 0x5A).all(), (trial, shift, indexed, i)


def test_config5_full_size_properties():
    # 1500 tensors, log-uniform sizes in [2^10, 2^22]; checked through size-independent properties on the
    # GPU plus the oracle on a sample of blocks
    rng = np.random.default_rng(5000)
    sizes = np.round(np.exp(rng.uniform(np.log(2**10), np.log(2**22), size=1500))).astype(np.int64).tolist()
    total = sum(sizes)
    big = _c5_like(total, seed=5001, device=DEV)  # one draw, carved into the 1500 tensors
    offs = np.concatenate([[0], np.cumsum(sizes)])
    tensors = [big[offs[i]: offs[i + 1]].clone() for i in range(1500)]
    bucket = fp8.FlatBucket(tensors)
    flat = bucket.pack()
    sync()
    assert torch.equal(flat.view(torch.int16), big.view(torch.int16))
    q, s = fp8.quantize(flat)
    sync()
    nb = s.numel()
    pad = nb * 1024 - total
    xf = torch.cat([flat.float(), torch.zeros(pad, device=DEV)]).view(nb, 1024)
    amax = xf.abs().amax(1)
    assert np.array_equal(s.cpu().numpy(), amax.cpu().numpy() / np.float32(448.0))  # IEEE division
    qp = torch.cat([q, torch.zeros(pad, dtype=torch.uint8, device=DEV)]).view(nb, 1024)
    assert torch.all((qp & 0x7F).amax(1) == 0x7E)  # every block's largest magnitude maps to +-448
    xhat = qp.view(torch.float8_e4m3fn).float() * s[:, None]
    code_e = ((qp & 0x7F) >> 3).float()
    spacing = torch.where(code_e == 0, torch.tensor(2.0**-9, device=DEV), torch.exp2(code_e - 10))
    assert torch.all((xf - xhat).abs() <= 0.5 * spacing * s[:, None] * 1.001)
    acc = torch.zeros(total, dtype=torch.float32, device=DEV)
    fp8.dequant_accumulate(acc, q, s)
    fp8.dequant_accumulate(acc, q, s)
    sync()
    assert torch.equal(acc, (xhat.view(-1)[:total] + xhat.view(-1)[:total]))  # x + x is exact
    # oracle on sampled blocks (first, last, and every 997th)
    hflat, hq, hs = bits(flat), q.cpu().numpy(), s.cpu().numpy()
    for b in sorted(set([0, nb - 1, nb - 2] + list(range(0, nb, 997)))):
        lo, hi = b * 1024, min((b + 1) * 1024, total)
        wq, ws = oracle.fp8_quantize(hflat[lo:hi], 1024)
        assert np.array_equal(hq[lo:hi], wq) and hs[b] == ws[0]
    outs = [torch.empty(n, dtype=torch.float32, device=DEV) for n in sizes]
    bucket.unpack(acc, outs)
    sync()
    for i in (0, 1, 749, 1498, 1499):
        assert torch.equal(outs[i], acc[offs[i]: offs[i + 1]])
    assert torch.equal(torch.cat(outs), acc)
    # fused forms give the same bits as the staged pipeline at full size
    qb, sb = fp8.quantize_bucket(bucket)
    sync()
    assert torch.equal(qb, q) and torch.equal(sb, s)
    accs = [torch.zeros(n, dtype=torch.float32, device=DEV) for n in sizes]
    ab = fp8.FlatBucket(accs)
    fp8.dequant_accumulate_bucket(ab, q, s)
    fp8.dequant_accumulate_bucket(ab, q, s)
    sync()
    assert torch.equal(torch.cat(accs), acc)


@pytest.mark.parametrize("ntensors", [1, 2, 7, 66, 700, 4226])
def test_block_index_forms_match_table_search(ntensors):
    # the bucket's block index against its definition, and the fused forms with and without it, bit for bit
    g = torch.Generator().manual_seed(1000 + ntensors)
    if ntensors <= 7:
        sizes = torch.randint(1, 9000, (ntensors,), generator=g).tolist()
    else:
        sizes = torch.randint(0, 3000 if ntensors < 1000 else 40, (ntensors,), generator=g).tolist()
        sizes[ntensors // 3] = 5000       # whole blocks inside one tensor next to blocks that span dozens
        sizes[0] = 0
    total = sum(sizes)
    offs = np.concatenate([[0], np.cumsum(sizes)])
    big = _c5_like(total, seed=ntensors)
    big[total // 2] = float("nan")
    dbig = big.to(DEV)
    dev = [dbig[offs[i]: offs[i + 1]].clone() for i in range(ntensors)]
    bucket = fp8.FlatBucket(dev)
    q0, s0 = fp8.quantize_bucket(bucket, indexed=False)
    index = bucket.block_index()
    sync()
    nblocks = (total + 1023) // 1024
    starts = np.arange(nblocks, dtype=np.int64) * 1024
    want = np.searchsorted(offs, starts, side="right") - 1        # the last tensor whose offset is <= the block start
    got = index.cpu().numpy()
    assert got.size == nblocks + 1 and np.array_equal(got[:nblocks], want) and got[nblocks] == ntensors - 1
    q1, s1 = fp8.quantize_bucket(bucket)                          # picks the index up now that it exists
    sync()
    assert torch.equal(q0, q1) and torch.equal(s0.view(torch.int32), s1.view(torch.int32))
    wq, ws = oracle.fp8_quantize(bits(big), 1024)
    assert np.array_equal(q1.cpu().numpy(), wq) and np.array_equal(s1.cpu().numpy(), ws)
    qf = q1.clone()
    qf[(qf & 0x7F) == 0x7F] = 0x11
    rng = np.random.default_rng(ntensors)
    init = torch.from_numpy(rng.normal(size=total).astype(np.float32)).to(DEV)
    results = []
    for indexed in (False, True):
        accs = [init[offs[i]: offs[i + 1]].clone() for i in range(ntensors)]
        ab = fp8.FlatBucket(accs)
        fp8.dequant_accumulate_bucket(ab, qf, s1, indexed=indexed)
        fp8.dequant_accumulate_bucket_many(ab, [qf, qf & 0xF7, qf], [s1, s1 * 0.5, s1], indexed=indexed)
        sync()
        results.append(torch.cat(accs))
    assert torch.equal(results[0].view(torch.int32), results[1].view(torch.int32))
    acc_h = init.cpu().numpy().copy()
    hq = qf.cpu().numpy()
    for hq_r, hs_r in ((hq, ws), (hq, ws), (hq & 0xF7, ws * np.float32(0.5)), (hq, ws)):  # clearing a bit never makes a NaN code
        oracle.fp8_dequant_accumulate(acc_h, hq_r, hs_r, 1024)
    assert np.array_equal(results[1].cpu().numpy().view(np.uint32), acc_h.view(np.uint32))
