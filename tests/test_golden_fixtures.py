"""The committed binary fixtures of tests/golden (written by tests/golden/make_fixtures.py from torch's CPU casts
and ``torch.as_strided``, without the oracle or the product) against the oracle, the library's host code and
the device kernels."""
import ctypes as C
import json
import os
import random

import numpy as np
import pytest
import torch

import oracle
from oracle import OSlice


@pytest.fixture(scope="module")
def table(golden_dir):
    t = np.fromfile(os.path.join(golden_dir, "e4m3fn_from_bf16_scale1.bin"), dtype=np.uint8)
    assert t.size == 65536
    return t


@pytest.fixture(scope="module")
def fuzz(golden_dir):
    with open(os.path.join(golden_dir, "ndslice_fuzz_slices.json")) as f:
        meta = json.load(f)
    locs = np.fromfile(os.path.join(golden_dir, "ndslice_fuzz_locations.bin"), dtype="<u4")
    assert len(meta["slices"]) == 1000 and locs.size == meta["total_locations"]
    return meta["slices"], locs


def _patterns():
    return np.arange(65536, dtype=np.uint32).astype(np.uint16)


def _unit_scale_blocks(table):
    """All bf16 patterns that a block of absmax 448 can hold (|x| <= 448, and NaN, which the block maximum
    ignores), laid out in 1024-element blocks that start with 448.0, and the codes the table gives them."""
    h = _patterns()
    mag = h & 0x7FFF
    keep = (mag <= 0x43E0) | (mag > 0x7F80)          # 0x43E0 is 448.0
    vals = h[keep]
    per = 1023
    nblk = (vals.size + per - 1) // per
    x = np.zeros((nblk, 1024), dtype=np.uint16)
    x[:, 0] = 0x43E0
    body = np.zeros(nblk * per, dtype=np.uint16)
    body[: vals.size] = vals
    x[:, 1:] = body.reshape(nblk, per)
    return x.reshape(-1), table[x.reshape(-1)]


# ---------------- CPU: the oracle and the library's host code ----------------

def test_table_sanity(table):
    # spot values fixed by the format itself: 448 -> 0x7E, 1.0 -> 0x38, 2^-9 -> 0x01, -0.0 -> 0x80, +Inf clamps to 448
    assert table[0x43E0] == 0x7E and table[0x3F80] == 0x38 and table[0x3B00] == 0x01
    assert table[0x8000] == 0x80 and table[0x0000] == 0 and table[0x7F80] == 0x7E and table[0xFF80] == 0xFE
    assert table[0x7FC0] == 0x7F and table[0xFFC0] == 0xFF
    # odd symmetry and monotonicity over the finite positive half
    assert np.array_equal(table[:0x8000] | 0x80, table[0x8000:])
    fin = table[:0x7F81].astype(np.int32)
    assert np.all(np.diff(fin) >= 0) and fin[-1] == 0x7E


def test_oracle_encoder_matches_table(table):
    x = oracle.bf16_to_f32(_patterns())
    got = np.array([oracle.e4m3fn_encode(float(v), True) for v in x], dtype=np.uint8)
    nan = np.isnan(x)
    assert np.array_equal(got[~nan], table[~nan])
    # float() of a NaN keeps its sign on this platform; the block quantiser below is checked on the bits
    assert np.all((got[nan] & 0x7F) == 0x7F)


def test_oracle_quantizer_matches_table_at_unit_scale(table):
    x, want = _unit_scale_blocks(table)
    q, s = oracle.fp8_quantize(x, 1024)
    assert np.all(s == np.float32(1.0))
    assert np.array_equal(q, want)                     # NaN codes included, sign and all


def test_oracle_iteration_matches_fuzz_fixture(fuzz):
    slices, locs = fuzz
    for e in slices:
        s = OSlice(e["offset"], e["sizes"], e["strides"])          # Slice::new must accept every one
        want = locs[e["first"]: e["first"] + e["count"]]
        assert len(s) == e["count"]
        assert np.array_equal(s.iter().astype(np.uint32), want), e
        for i in (0, e["count"] // 2, e["count"] - 1):
            assert s.get(i) == want[i]
    # packing an arange storage yields the locations themselves
    e = max(slices, key=lambda e: e["count"])
    s = OSlice(e["offset"], e["sizes"], e["strides"])
    span = int(locs[e["first"]: e["first"] + e["count"]].max()) + 1
    assert np.array_equal(oracle.pack(np.arange(span, dtype=np.uint32), s), locs[e["first"]: e["first"] + e["count"]])


def test_fuzz_generator_with_oracle_validation_reproduces_fixture(fuzz):
    # the generator of python/tests/_monarch/test_ndslice.py:143-167 driven by the oracle's Slice::new:
    # the same 1000 slices come out, so accept / reject agrees on every candidate drawn on the way
    slices, _ = fuzz
    gen = random.Random(0)
    for e in slices:
        while True:
            ndim = gen.choices([1, 2, 3, 4], [1, 2, 3, 4])[0]
            sizes = [gen.randrange(1, 10) for _ in range(ndim)]
            strides, run = [], 1
            for j in range(ndim):
                run *= gen.randrange(1 if j == 0 else 2, 4)
                strides.append(run)
            order = list(range(ndim))
            gen.shuffle(order)
            offset = gen.randrange(10000)
            try:
                s = OSlice(offset, [sizes[o] for o in order], [strides[o] for o in order])
                break
            except oracle.OracleError:
                continue
        assert (s.offset, s.sizes, s.strides) == (e["offset"], e["sizes"], e["strides"])


def test_host_library_matches_fuzz_fixture(fuzz):
    from monarch_amd import Slice
    from util import fuzz_slices

    slices, locs = fuzz
    mine = fuzz_slices(1000, seed=0)                   # same generator, validated by the library's Slice
    for e, s in zip(slices, mine):
        assert (s.offset, list(s.sizes), list(s.strides)) == (e["offset"], e["sizes"], e["strides"])
        want = locs[e["first"]: e["first"] + e["count"]]
        assert len(s) == e["count"]
        assert np.array_equal(np.asarray(list(s), dtype=np.uint32), want)


# ---------------- GPU: the kernels ----------------

@pytest.mark.gpu
def test_device_quantize_matches_table_at_unit_scale(table):
    from monarch_amd import fp8

    x, want = _unit_scale_blocks(table)
    xd = torch.from_numpy(x.view(np.int16).copy()).view(torch.bfloat16).to("cuda:0")
    q, s = fp8.quantize(xd)
    torch.cuda.synchronize()
    assert torch.all(s == 1.0)
    got = q.cpu().numpy()
    bad = np.flatnonzero(got != want)                  # every code, NaN sign bits included
    assert bad.size == 0, [(hex(int(x[i])), hex(int(got[i])), hex(int(want[i]))) for i in bad[:8]]


@pytest.mark.gpu
def test_device_pack_matches_fuzz_fixture(fuzz):
    from monarch_amd import Slice, staging

    slices, locs = fuzz
    span = int(locs.max()) + 1
    base = torch.arange(span, dtype=torch.int32, device="cuda:0")
    views = [Slice(offset=e["offset"], sizes=e["sizes"], strides=e["strides"]) for e in slices]
    outs = [staging.pack(base, v) for v in views]
    torch.cuda.synchronize()
    for e, o in zip(slices, outs):
        want = locs[e["first"]: e["first"] + e["count"]]
        assert np.array_equal(o.view(torch.int32).cpu().numpy().astype(np.uint32), want), e
    # and back: unpacking the locations into zeros puts each location at its own index
    for e, v, o in list(zip(slices, views, outs))[::7]:
        back = torch.zeros(span, dtype=torch.int32, device="cuda:0")
        staging.unpack(back, v, o)
        want = np.zeros(span, dtype=np.int32)
        idx = locs[e["first"]: e["first"] + e["count"]]
        want[idx] = idx
        torch.cuda.synchronize()
        assert np.array_equal(back.cpu().numpy(), want)
