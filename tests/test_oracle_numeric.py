"""Pins the numeric half of the CPU oracle: Reduce sum/avg, bf16 rounding, the
reduce-scatter rule and the fp8 e4m3fn block-scaled codec.

Sources of truth: the reference's small known-answer tests (golden JSON), closed forms
from python/tests/test_controller.py:188-254, and library routines (torch CPU casts and
sums) for what the reference leaves open (bf16, avg, fp8)."""
import itertools
import json
import os

import numpy as np
import pytest
import torch

import oracle
from oracle import AVG, SUM, OSlice


@pytest.fixture(scope="module")
def vec(golden_dir):
    with open(os.path.join(golden_dir, "ndslice_vectors.json")) as f:
        return json.load(f)


def bits(t: torch.Tensor) -> np.ndarray:
    return t.view(torch.uint16).numpy() if t.dtype == torch.bfloat16 else t.numpy()


def test_bf16_round_matches_torch():
    rng = np.random.default_rng(0)
    # random bit patterns cover normals, subnormals, inf, nan and every tie case
    u = rng.integers(0, 2**32, size=2_000_000, dtype=np.uint64).astype(np.uint32)
    ties = (rng.integers(0, 2**16, size=70000, dtype=np.uint64).astype(np.uint32) << 16) | 0x8000
    u = np.concatenate([u, ties, ties + 1, ties - 1])
    f = u.view(np.float32)
    got = oracle.f32_to_bf16(f)
    want = torch.from_numpy(f).to(torch.bfloat16).view(torch.uint16).numpy()
    nan = np.isnan(f)
    assert np.array_equal(got[~nan], want[~nan])
    assert np.all((got[nan] & 0x7FFF) > 0x7F80)
    # widening is exact
    h = np.arange(65536, dtype=np.uint16)
    back = oracle.bf16_to_f32(h)
    assert np.array_equal(back.view(np.uint32), h.astype(np.uint32) << 16)


def test_f16_round_matches_torch():
    h = np.arange(65536, dtype=np.uint16)
    want = torch.from_numpy(h.view(np.int16).copy()).view(torch.float16).float().numpy()
    got = oracle.f16_to_f32(h)
    nan = np.isnan(want)
    assert np.array_equal(np.isnan(got), nan) and np.array_equal(got[~nan].view(np.uint32), want[~nan].view(np.uint32))
    rng = np.random.default_rng(1)
    u = rng.integers(0, 2**32, size=1_000_000, dtype=np.uint64).astype(np.uint32)
    small = rng.normal(0, 1e-4, size=300_000).astype(np.float32).view(np.uint32)   # subnormal halves and ties
    edge = np.array([65504.0, 65519.9, 65520.0, 65536.0, 1e9, 2.0**-24, 2.0**-25, 1.5 * 2.0**-25, 2.0**-14, 0.0, -0.0],
                    dtype=np.float32).view(np.uint32)
    ties = ((rng.integers(0, 2**19, size=100_000, dtype=np.uint64).astype(np.uint32) << 13) | 0x1000) + 0x38000000
    u = np.concatenate([u, small, edge, ties, ties + 1, ties - 1])
    f = u.view(np.float32)
    got = oracle.f32_to_f16(f)
    want = torch.from_numpy(f).to(torch.float16).view(torch.int16).numpy().view(np.uint16)
    nan = np.isnan(f)
    assert np.array_equal(got[~nan], want[~nan])
    assert np.all((got[nan] & 0x7FFF) > 0x7C00)
    a = torch.randn(5000).half()
    b = torch.randn(5000).half()
    got = oracle.reduce([a.view(torch.int16).numpy().view(np.uint16), b.view(torch.int16).numpy().view(np.uint16)], AVG, half=True)
    want = ((a.float() + b.float()) / 2).half().view(torch.int16).numpy().view(np.uint16)
    assert np.array_equal(got, want)


def test_reduce_golden(vec):
    for case in vec["reduce"]:
        ins = [np.array(x, dtype=np.float32) for x in case["inputs"]]
        if case["kind"] == "sum":
            assert oracle.reduce(ins, SUM).tolist() == case["expected"], case["src"]
        else:
            n = len(ins)
            c = ins[0].size // n
            in_view = OSlice(0, [ins[0].size], [1])
            for r, want in enumerate(case["expected_per_rank"]):
                outs = oracle.reduce_scatter(ins, in_view, [OSlice(r * c, [c], [1])], SUM)
                assert outs[0].tolist() == want, case["src"]


def test_reduce_closed_form_test_controller():
    # python/tests/test_controller.py:188-242: x[h,g] = 24h + 12g + arange(12)
    xs = {(h, g): (24 * h + 12 * g + np.arange(12)).astype(np.float32)
          for h, g in itertools.product(range(2), range(2))}
    y = oracle.reduce([xs[(0, 0)], xs[(0, 1)]], SUM)
    assert np.array_equal(y, xs[(0, 0)] + xs[(0, 1)])
    rad = oracle.reduce([xs[k] for k in sorted(xs)], SUM)
    assert np.array_equal(rad, sum(xs.values()))
    # worker_reduce, monarch_tensor_worker/src/comm.rs:1258-1431: ones over 2 / 4 ranks
    ones = np.ones(6, dtype=np.float32)
    assert np.all(oracle.reduce([ones, ones], SUM) == 2.0)
    assert np.all(oracle.reduce([ones] * 4, SUM) == 4.0)
    # scatter of x.reshape(2, 6) over "gpu" (N=2): rank r gets row r of the sum, shape rule
    # tensor.py:494-503 (sum over dim 0 of [N, ...])
    a, b = xs[(0, 0)], xs[(0, 1)]
    for r in range(2):
        out = oracle.reduce_scatter([a, b], OSlice(0, [12], [1]), [OSlice(6 * r, [6], [1])], SUM)[0]
        assert np.array_equal(out, (a + b).reshape(2, 6)[r])


@pytest.mark.parametrize("n", [1, 2, 3, 8, 16])
def test_reduce_f32_vs_torch(n):
    rng = np.random.default_rng(n)
    ins = [rng.uniform(-1, 1, size=4099).astype(np.float32) for _ in range(n)]
    want = torch.stack([torch.from_numpy(x) for x in ins]).double().sum(0)
    got = oracle.reduce(ins, SUM)
    np.testing.assert_allclose(got, want.numpy(), rtol=1e-6, atol=1e-6)
    got = oracle.reduce(ins, AVG)
    np.testing.assert_allclose(got, (want / n).numpy(), rtol=1e-6, atol=1e-6)
    # left-to-right fp32 order, stated exactly
    acc = ins[0].copy()
    for x in ins[1:]:
        acc = acc + x
    assert np.array_equal(oracle.reduce(ins, SUM), acc)
    assert np.array_equal(oracle.reduce(ins, AVG), acc / np.float32(n))
    assert np.array_equal(oracle.reduce(ins, AVG, threads=True), acc / np.float32(n))
    # in place on input 0
    first = ins[0].copy()
    oracle.reduce([first] + ins[1:], SUM, out=first)
    assert np.array_equal(first, acc)


@pytest.mark.parametrize("n", [2, 8])
def test_reduce_bf16_vs_torch(n):
    g = torch.Generator().manual_seed(n)
    ts = [(torch.randn(100003, generator=g) * 0.02).bfloat16() for _ in range(n)]
    ins = [bits(t) for t in ts]
    for op, div in ((SUM, 1), (AVG, n)):
        got = oracle.reduce(ins, op)
        ref32 = torch.stack(ts).float().sum(0) / div  # fp32 accumulate, then round once
        want = ref32.bfloat16()
        gotf = torch.from_numpy(oracle.bf16_to_f32(got))
        # within 1 bf16 ulp of torch's CPU result (torch may sum in another order)
        ulp = torch.maximum(want.float().abs(), torch.tensor(2.0**-126)) * 2.0**-7
        assert torch.all((gotf - want.float()).abs() <= ulp)
        # and exactly the rounding of the left-to-right fp32 sum
        acc = ts[0].float()
        for t in ts[1:]:
            acc = acc + t.float()
        assert np.array_equal(got, bits((acc / div).bfloat16()))
        assert np.array_equal(oracle.reduce(ins, op, threads=True), got)  # the all-cores loop is the same loop


def test_reduce_integer_wraps():
    # parameter_server.rs:200-205: u8 wrapping_add over the per-worker chunks
    a = np.array([250, 1, 128], dtype=np.uint8)
    b = np.array([10, 2, 128], dtype=np.uint8)
    assert oracle.reduce([a, b], SUM).tolist() == [4, 3, 0]
    x = np.array([2**31 - 1, -5], dtype=np.int32)
    assert oracle.reduce([x, np.array([1, 2], dtype=np.int32)], SUM).tolist() == [-(2**31), -3]
    y = np.array([2**62, -1], dtype=np.int64)
    assert oracle.reduce([y, y], SUM).tolist() == [-(2**63), -2]


def test_reduce_scatter_c4_shape_small():
    # C4 at reduced size: x[h, g, r, c]; sum over g; last dim scattered into 8 column blocks
    H, G, R, Cc, K = 2, 8, 16, 64, 8
    rng = np.random.default_rng(4)
    x = rng.uniform(-1, 1, size=(H, G, R, Cc)).astype(np.float32)
    flat = x.reshape(-1)
    slab = R * Cc
    ins = [flat[g * slab:] for g in range(G)]
    in_view = OSlice(0, [H, R, Cc], [G * slab, Cc, 1])
    w = Cc // K
    out_views = [OSlice(k * w, [H, R, w], [R * Cc, Cc, 1]) for k in range(K)]
    outs = oracle.reduce_scatter(ins, in_view, out_views, SUM)
    red = torch.from_numpy(x).sum(1)
    for k in range(K):
        want = red[:, :, k * w:(k + 1) * w].contiguous().flatten().numpy()
        np.testing.assert_allclose(outs[k], want, rtol=1e-6, atol=1e-6)
    # exact left-to-right order
    acc = x[:, 0].copy()
    for g in range(1, G):
        acc = acc + x[:, g]
    for k in range(K):
        assert np.array_equal(outs[k], acc[:, :, k * w:(k + 1) * w].reshape(-1))


# ---------------- fp8 e4m3fn ----------------

def test_e4m3fn_decode_all_codes_vs_torch():
    codes = torch.arange(256, dtype=torch.uint8)
    want = codes.view(torch.float8_e4m3fn).float().numpy()
    got = np.array([oracle.e4m3fn_decode(int(c)) for c in range(256)], dtype=np.float32)
    nan = np.isnan(want)
    assert nan.sum() == 2 and np.array_equal(np.isnan(got), nan)
    assert np.array_equal(got[~nan], want[~nan])
    assert oracle.e4m3fn_decode(0x7E) == 448.0 and oracle.e4m3fn_decode(0x01) == 2.0**-9
    assert oracle.e4m3fn_decode(0x08) == 2.0**-6


def test_e4m3fn_encode_all_bf16_patterns_vs_torch():
    h = torch.arange(65536, dtype=torch.int32).to(torch.uint16)
    x = h.view(torch.bfloat16).float()
    want = x.to(torch.float8_e4m3fn).view(torch.uint8).numpy()  # non-saturating cast
    got = np.array([oracle.e4m3fn_encode(float(v), False) if not np.isnan(v) else 0x7F
                    for v in x.numpy()], dtype=np.uint8)
    xn = x.numpy()
    nan_in = np.isnan(xn)
    nan_out = (want & 0x7F) == 0x7F
    assert np.array_equal((got & 0x7F) == 0x7F, nan_out)
    ok = ~nan_out
    assert np.array_equal(got[ok], want[ok])
    # with the codec's clamp, every finite input lands on a finite code
    sat = np.array([oracle.e4m3fn_encode(float(v), True) for v in xn[~nan_in]], dtype=np.uint8)
    clamped = torch.from_numpy(xn[~nan_in]).clamp(-448, 448).to(torch.float8_e4m3fn).view(torch.uint8).numpy()
    assert np.array_equal(sat, clamped)


def test_e4m3fn_encode_fp32_ties_and_midpoints():
    # every midpoint between adjacent codes rounds to the even mantissa; just above/below go up/down
    vals = np.array([oracle.e4m3fn_decode(c) for c in range(0x7F)], dtype=np.float64)
    for c in range(0x7E):
        mid = np.float32((vals[c] + vals[c + 1]) / 2)
        want = c if c % 2 == 0 else c + 1
        assert oracle.e4m3fn_encode(float(mid)) == want
        assert oracle.e4m3fn_encode(float(np.nextafter(mid, np.float32(1e9)))) == c + 1
        assert oracle.e4m3fn_encode(float(np.nextafter(mid, np.float32(-1e9)))) == c
        assert oracle.e4m3fn_encode(-float(mid)) == want | 0x80
    rng = np.random.default_rng(5)
    f = np.concatenate([rng.uniform(-500, 500, 200000), rng.normal(0, 0.01, 200000)]).astype(np.float32)
    want = torch.from_numpy(f).to(torch.float8_e4m3fn).view(torch.uint8).numpy()
    got = np.array([oracle.e4m3fn_encode(float(v)) for v in f], dtype=np.uint8)
    assert np.array_equal(got, want)


def _c5_like(n, seed):
    g = torch.Generator().manual_seed(seed)
    x = torch.randn(n, generator=g)
    out = torch.rand(n, generator=g) < 1e-3
    x = torch.where(out, x * 50, x)
    return x.bfloat16()


def test_fp8_quantize_invariants():
    x = _c5_like(1024 * 37 + 333, seed=1)
    q, scales = oracle.fp8_quantize(bits(x), 1024)
    xf = x.float().numpy()
    nb = scales.size
    assert nb == 38
    xhat = oracle.fp8_dequantize(q, scales, 1024)
    for b in range(nb):
        blk = slice(b * 1024, min((b + 1) * 1024, xf.size))
        amax = np.abs(xf[blk]).max()
        assert scales[b] == np.float32(amax) / np.float32(448.0)
        # the largest-magnitude element maps to code 0x7E (448)
        assert (q[blk] & 0x7F).max() == 0x7E
        # dequantised value: |x - xhat| <= half the code spacing at that magnitude, times scale
        codes = q[blk] & 0x7F
        e = (codes >> 3).astype(np.int32)
        spacing = np.where(e == 0, 2.0**-9, 2.0 ** (e - 7 - 3))
        # one extra code spacing covers the fp32 roundings of 448/absmax and of x*inv
        err = np.abs(xf[blk] - xhat[blk])
        assert np.all(err <= (0.5 * spacing) * scales[b] * 1.001 + 1e-30)
    # codec equals torch's clamp+cast applied to the same scaled values
    inv = (np.float32(448.0) / (scales * np.float32(448.0)))  # not bit-identical to 448/absmax: recompute
    amax = np.array([np.abs(xf[b * 1024:(b + 1) * 1024]).max() for b in range(nb)], dtype=np.float32)
    inv = np.float32(448.0) / amax
    y = xf * np.repeat(inv, 1024)[: xf.size]
    want = torch.from_numpy(y.astype(np.float32)).clamp(-448, 448).to(torch.float8_e4m3fn).view(torch.uint8).numpy()
    assert np.array_equal(q, want)
    # decode is the product float(q) * scale, rounded once
    dec = torch.from_numpy(q).view(torch.float8_e4m3fn).float().numpy() * np.repeat(scales, 1024)[: xf.size]
    assert np.array_equal(xhat, dec.astype(np.float32))


def test_fp8_edge_blocks():
    block = 1024
    z = np.zeros(block, dtype=np.uint16)
    q, s = oracle.fp8_quantize(z, block)
    assert np.all(q == 0) and s[0] == np.float32(2.0**-40) / np.float32(448)
    assert np.all(oracle.fp8_dequantize(q, s, block) == 0)
    # negative zero keeps its sign bit, decodes to -0.0
    nz = np.full(block, 0x8000, dtype=np.uint16)
    q, s = oracle.fp8_quantize(nz, block)
    assert np.all(q == 0x80)
    # NaN propagates as an fp8 NaN and does not poison the block scale
    x = torch.ones(block).bfloat16()
    x[3] = float("nan")
    x[5] = -2.0
    q, s = oracle.fp8_quantize(bits(x), block)
    assert (q[3] & 0x7F) == 0x7F and s[0] == np.float32(2.0) / np.float32(448)
    assert q[5] == 0xFE and q[0] == oracle.e4m3fn_encode(224.0)
    # Inf saturates to +-448 and pins the scale at FLT_MAX/448
    x = torch.ones(block).bfloat16()
    x[7] = float("inf")
    x[8] = float("-inf")
    q, s = oracle.fp8_quantize(bits(x), block)
    assert q[7] == 0x7E and q[8] == 0xFE and np.isfinite(s[0])
    # a 50x outlier crushes the rest of its block towards the subnormal grid but not others
    x = torch.full((2 * block,), 0.01).bfloat16()
    x[10] = 50.0
    q, s = oracle.fp8_quantize(bits(x), block)
    xhat = oracle.fp8_dequantize(q, s, block)
    assert abs(xhat[10] - 50.0) == 0 and abs(xhat[block + 1] - 0.01) < 0.01 * 2**-4
    # short tail block
    x = _c5_like(block + 5, seed=2)
    q, s = oracle.fp8_quantize(bits(x), block)
    assert s.size == 2 and (q[block:] & 0x7F).max() == 0x7E


def test_fp8_dequant_accumulate_and_flat():
    rng = np.random.default_rng(9)
    sizes = [1024, 1, 4097, 2048, 333]
    offsets = np.concatenate([[0], np.cumsum(sizes)]).tolist()
    tensors = [bits(_c5_like(n, seed=10 + i)) for i, n in enumerate(sizes)]
    flat = oracle.flat_pack(tensors, offsets)
    assert np.array_equal(flat, np.concatenate(tensors))
    q, s = oracle.fp8_quantize(flat, 1024)
    acc = rng.normal(size=flat.size).astype(np.float32)
    acc0 = acc.copy()
    oracle.fp8_dequant_accumulate(acc, q, s, 1024)
    xhat = oracle.fp8_dequantize(q, s, 1024)
    assert np.array_equal(acc, acc0 + xhat)  # two roundings: product, then sum
    outs = oracle.flat_unpack(acc, offsets)
    assert [o.size for o in outs] == sizes
    assert np.array_equal(np.concatenate(outs), acc)


# ---------------- pins for f64 reduce and for bf16 / Avg reduce-scatter ----------------
# Reference semantics: ncclReduceScatter's flat-chunk rule, torch-sys-cuda/src/nccl.rs:683,693-701
# (output r = chunk r of the elementwise reduction over the group), Avg = sum / group size
# (nccl.rs:285-292).  The expected values below are built from explicit member-order adds in
# torch / numpy, never from the oracle's own formula, with n_in != n_out so that dividing by the
# number of outputs instead of the number of group members fails, and with values whose partial
# sums are not representable in bf16 so that rounding after every add fails.

@pytest.mark.parametrize("n", [1, 2, 3, 7])
def test_reduce_f64_left_to_right(n):
    rng = np.random.default_rng(640 + n)
    # magnitudes spread over 30 binades: the order of the adds changes the low bits
    ins = [(rng.uniform(-1, 1, size=2053) * 10.0 ** rng.integers(-15, 15, size=2053)).astype(np.float64)
           for _ in range(n)]
    acc = ins[0].copy()
    for x in ins[1:]:
        acc = acc + x                      # IEEE double adds in member order
    got = oracle.reduce(ins, SUM)
    assert got.dtype == np.float64 and np.array_equal(got.view(np.uint64), acc.view(np.uint64))
    got = oracle.reduce(ins, AVG)
    assert np.array_equal(got.view(np.uint64), (acc / np.float64(n)).view(np.uint64))
    # the sum is a double sum, not a float one: it keeps bits an fp32 accumulator would drop
    if n > 1:
        a = np.array([1.0, 2.0**-40], dtype=np.float64)
        assert oracle.reduce([a, a[::-1].copy()], SUM).tolist() == [1.0 + 2.0**-40] * 2
    # in place on member 0
    first = ins[0].copy()
    oracle.reduce([first] + ins[1:], AVG, out=first)
    assert np.array_equal(first, acc / np.float64(n))


def _strided_inputs(n_in, rows, cols, pitch, slab, seed, bf16):
    """n_in flat storages holding a [rows, cols] tensor at row pitch `pitch` starting at `slab`."""
    g = torch.Generator().manual_seed(seed)
    ts = []
    for _ in range(n_in):
        t = torch.randn(slab + rows * pitch + 5, generator=g)
        ts.append(t.bfloat16() if bf16 else t)
    return ts


@pytest.mark.parametrize("op", [SUM, AVG])
@pytest.mark.parametrize("n_in,n_out", [(3, 2), (5, 4), (2, 6)])
def test_reduce_scatter_bf16_member_order(op, n_in, n_out):
    rows, cols, pitch, slab = 12, 24, 40, 7
    ts = _strided_inputs(n_in, rows, cols, pitch, slab, 900 + 10 * n_in + n_out, bf16=True)
    in_view = OSlice(slab, [rows, cols], [pitch, 1])
    w = cols // n_out
    out_views = [OSlice(k * w, [rows, w], [cols, 1]) for k in range(n_out)]
    outs = oracle.reduce_scatter([bits(t) for t in ts], in_view, out_views, op)
    # explicit adds in member order on the strided views, fp32 accumulate, one rounding at the end
    views = [torch.as_strided(t, (rows, cols), (pitch, 1), slab).float() for t in ts]
    acc = views[0].clone()
    for v in views[1:]:
        acc = acc + v
    if op == AVG:
        acc = acc / n_in
    want = acc.bfloat16()
    for k in range(n_out):
        assert np.array_equal(outs[k], bits(want[:, k * w:(k + 1) * w].contiguous().flatten())), (k, op)
    if n_in > 2:
        # rounding to bf16 after every add gives another answer on these inputs: the pin can tell
        per_add = views[0].bfloat16()
        for v in views[1:]:
            per_add = (per_add.float() + v).bfloat16()
        assert not torch.equal(per_add, acc.bfloat16() if op == SUM else (acc * n_in).bfloat16())


@pytest.mark.parametrize("n_in,n_out", [(3, 2), (5, 4), (2, 6)])
def test_reduce_scatter_f32_avg_member_order(n_in, n_out):
    rows, cols, pitch, slab = 12, 24, 40, 7
    ts = _strided_inputs(n_in, rows, cols, pitch, slab, 700 + 10 * n_in + n_out, bf16=False)
    in_view = OSlice(slab, [rows, cols], [pitch, 1])
    # the flat-chunk rule of nccl.rs:683,693-701 on the reduced tensor: output r = elements [r*c, (r+1)*c)
    c = rows * cols // n_out
    out_views = [OSlice(r * c, [c], [1]) for r in range(n_out)]
    outs = oracle.reduce_scatter([t.numpy() for t in ts], in_view, out_views, AVG)
    views = [torch.as_strided(t, (rows, cols), (pitch, 1), slab) for t in ts]
    acc = views[0].clone()
    for v in views[1:]:
        acc = acc + v
    want = (acc / n_in).flatten()
    for r in range(n_out):
        assert np.array_equal(outs[r], want[r * c:(r + 1) * c].numpy()), r
    assert not torch.equal(acc / n_out, acc / n_in)
    # and a column-block scatter of the same average
    w = cols // n_out
    outs = oracle.reduce_scatter([t.numpy() for t in ts], in_view,
                                 [OSlice(k * w, [rows, w], [cols, 1]) for k in range(n_out)], AVG)
    for k in range(n_out):
        assert np.array_equal(outs[k], (acc / n_in)[:, k * w:(k + 1) * w].contiguous().flatten().numpy())
