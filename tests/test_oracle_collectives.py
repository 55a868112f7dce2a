"""Pins the oracle's Prod / Max / Min reduces, Reduction::Stack (all_gather / all_to_all) and SendTensor result
against the reference's own test vectors where it holds any, and against numpy / torch routines elsewhere.
Expected values are built from library calls and explicit member-order chains, never from the oracle's formula."""
import numpy as np
import pytest
import torch

import oracle
from oracle import MAX, MIN, PROD, SUM, OSlice


def _bf16_bits(t):
    return t.view(torch.uint16).numpy()


# ---------------- Prod / Max / Min (torch-sys-cuda/src/nccl.rs:285-292) ----------------

@pytest.mark.parametrize("dtype", [np.float32, np.float64])
@pytest.mark.parametrize("n", [1, 2, 5])
def test_float_prod_max_min_member_order(dtype, n):
    rng = np.random.default_rng(100 + n)
    ins = [rng.uniform(-2, 2, size=1031).astype(dtype) for _ in range(n)]
    prod = ins[0].copy()
    for x in ins[1:]:
        prod = prod * x                                  # IEEE multiplies in member order, in the tensor's type
    assert np.array_equal(oracle.reduce_op(ins, PROD), prod)
    assert np.array_equal(oracle.reduce_op(ins, MAX), np.maximum.reduce(ins))
    assert np.array_equal(oracle.reduce_op(ins, MIN), np.minimum.reduce(ins))
    assert np.array_equal(oracle.reduce_op(ins, SUM), oracle.reduce(ins, SUM))


def test_max_min_nan_and_signed_zero_rule():
    nan = np.float32("nan")
    a = np.array([1.0, nan, nan, 3.0, nan, -0.0, 0.0, -np.inf], dtype=np.float32)
    b = np.array([nan, 2.0, nan, nan, -5.0, 0.0, -0.0, np.inf], dtype=np.float32)
    c = np.array([0.5, nan, nan, 4.0, nan, -0.0, -0.0, 0.0], dtype=np.float32)
    # a NaN operand is skipped unless all operands are NaN: numpy's fmax / fmin have exactly that rule
    got = oracle.reduce_op([a, b, c], MAX)
    want = np.fmax(np.fmax(a, b), c)
    assert np.array_equal(np.isnan(got), np.isnan(want)) and np.array_equal(got[~np.isnan(want)], want[~np.isnan(want)])
    got_min = oracle.reduce_op([a, b, c], MIN)
    want_min = np.fmin(np.fmin(a, b), c)
    assert np.array_equal(np.isnan(got_min), np.isnan(want_min))
    assert np.array_equal(got_min[~np.isnan(want_min)], want_min[~np.isnan(want_min)])
    assert got.tolist()[:2] == [1.0, 2.0] and np.isnan(got[2]) and got[3] == 4.0 and got[4] == -5.0 and got[7] == np.inf
    # ties keep the accumulator: the first of +0 / -0 in member order decides the sign bit
    assert np.signbit(got[5]) and not np.signbit(got[6])
    assert np.signbit(got_min[5]) and not np.signbit(got_min[6])


@pytest.mark.parametrize("op", [PROD, MAX, MIN])
def test_bf16_and_f16_other_ops_accumulate_in_fp32_and_round_once(op):
    g = torch.Generator().manual_seed(17 + op)
    ts = [(torch.randn(4099, generator=g) * 1.3).bfloat16() for _ in range(4)]
    acc = ts[0].float()
    for t in ts[1:]:
        f = t.float()
        acc = acc * f if op == PROD else torch.maximum(acc, f) if op == MAX else torch.minimum(acc, f)
    want = acc.bfloat16()
    assert np.array_equal(oracle.reduce_op([_bf16_bits(t) for t in ts], op), _bf16_bits(want))
    if op == PROD:  # rounding after every multiply gives another answer: the pin can tell
        per = ts[0]
        for t in ts[1:]:
            per = (per.float() * t.float()).bfloat16()
        assert not torch.equal(per, want)
    hs = [(torch.randn(4099, generator=g) * 1.3).half() for _ in range(4)]
    acc = hs[0].float()
    for t in hs[1:]:
        f = t.float()
        acc = acc * f if op == PROD else torch.maximum(acc, f) if op == MAX else torch.minimum(acc, f)
    got = oracle.reduce_op([t.view(torch.int16).numpy().view(np.uint16) for t in hs], op, kind="f16")
    assert np.array_equal(got, acc.half().view(torch.int16).numpy().view(np.uint16))


@pytest.mark.parametrize("dtype", [np.uint8, np.int8, np.int32, np.int64])
def test_integer_prod_wraps_and_max_min_follow_the_sign(dtype):
    info = np.iinfo(dtype)
    rng = np.random.default_rng(int(info.bits))
    ins = [rng.integers(info.min, info.max, size=2050, dtype=dtype, endpoint=True) for _ in range(3)]
    for x in ins:
        x[:4] = [info.min, info.max, 0, info.max]
    with np.errstate(over="ignore"):
        prod = ins[0] * ins[1] * ins[2]                  # numpy integer multiply wraps modulo 2^bits
    assert np.array_equal(oracle.reduce_op(ins, PROD), prod)
    assert np.array_equal(oracle.reduce_op(ins, MAX), np.maximum.reduce(ins))
    assert np.array_equal(oracle.reduce_op(ins, MIN), np.minimum.reduce(ins))
    # the sign matters: -1 is the smallest int8 but the largest uint8
    if dtype == np.int8:
        a, b = np.array([-1], dtype=np.int8), np.array([1], dtype=np.int8)
        assert oracle.reduce_op([a, b], MAX).tolist() == [1]
        assert oracle.reduce_op([a.view(np.uint8), b.view(np.uint8)], MAX).tolist() == [255]


def test_reduce_scatter_other_ops():
    rng = np.random.default_rng(3)
    ins = [rng.uniform(-2, 2, size=48).astype(np.float32) for _ in range(3)]
    view = OSlice(0, [48], [1])
    for op, fn in ((MAX, np.maximum), (MIN, np.minimum), (PROD, np.multiply)):
        red = fn(fn(ins[0], ins[1]), ins[2])
        outs = oracle.reduce_scatter(ins, view, [OSlice(r * 12, [12], [1]) for r in range(4)], op)
        for r in range(4):
            assert np.array_equal(outs[r], red[r * 12:(r + 1) * 12]), (op, r)


# ---------------- Reduction::Stack ----------------

def test_stack_matches_reference_all_gather_vector():
    # torch-sys-cuda/src/nccl.rs:927-959: rank i holds full([2,2], i); every rank ends with stack of both
    ins = [np.full((2, 2), float(i), dtype=np.float32) for i in range(2)]
    got = oracle.stack(ins).reshape(2, 2, 2)
    assert got.tolist() == [[[0.0, 0.0], [0.0, 0.0]], [[1.0, 1.0], [1.0, 1.0]]]
    g = torch.Generator().manual_seed(1)
    for dtype in (torch.uint8, torch.int16, torch.float32, torch.float64):
        ts = [torch.randint(0, 200, (3, 5), generator=g).to(dtype) for _ in range(5)]
        assert np.array_equal(oracle.stack([t.numpy() for t in ts]).reshape(5, 3, 5), torch.stack(ts).numpy())


def test_stack_scatter_matches_reference_all_to_all_vector():
    # torch-sys-cuda/src/nccl.rs:996-1031: rank 0 holds [0,1], rank 1 holds [2,3]; rank 0 ends with [0,2], rank 1 with [1,3]
    ins = [np.array([0.0, 1.0], dtype=np.float32), np.array([2.0, 3.0], dtype=np.float32)]
    assert oracle.stack_scatter(ins, 0).tolist() == [0.0, 2.0]
    assert oracle.stack_scatter(ins, 1).tolist() == [1.0, 3.0]
    # torch.distributed.all_to_all_single semantics spelled with chunk / cat
    g = torch.Generator().manual_seed(2)
    n = 4
    ts = [torch.randn(n * 7, generator=g) for _ in range(n)]
    for rank in range(n):
        want = torch.cat([t.chunk(n)[rank] for t in ts])
        assert np.array_equal(oracle.stack_scatter([t.numpy() for t in ts], rank), want.numpy())
    # in place on the member's own tensor (stream.rs:1383-1384): peers' chunks are read before anything is overwritten
    arrs = [t.numpy().copy() for t in ts]
    want = torch.cat([t.chunk(n)[2] for t in ts]).numpy()
    oracle.stack_scatter(arrs, 2, out=arrs[2])
    assert np.array_equal(arrs[2], want)
    with pytest.raises(ValueError):
        oracle.stack_scatter([np.zeros(7, dtype=np.float32)] * 2, 0)


# ---------------- SendTensor ----------------

def test_send_tensor_result_is_the_contiguous_view():
    # monarch_tensor_worker/src/comm.rs:1434-1584: full([2,3], 2.0) sent from rank 0 arrives unchanged on rank 1
    x = np.full((2, 3), 2.0, dtype=np.float32)
    assert oracle.send_tensor(x, OSlice.row_major([2, 3])).reshape(2, 3).tolist() == x.tolist()
    assert oracle.send_tensor_route(OSlice(0, [1], [1]), OSlice(1, [1], [1]), 0) == (None, 1)
    assert oracle.send_tensor_route(OSlice(0, [1], [1]), OSlice(1, [1], [1]), 1) == (0, None)
    assert oracle.send_tensor_route(OSlice(0, [1], [1]), OSlice(0, [1], [1]), 0) == (0, 0)   # comm.rs:1602-1712
    assert oracle.send_tensor_route(OSlice(0, [1], [1]), OSlice(1, [1], [1]), 5) == (None, None)
    # a non-contiguous sender: the receiver holds torch's .contiguous() of the view
    g = torch.Generator().manual_seed(5)
    base = torch.randn(6, 10, generator=g)
    view = base.t()[1:9:2]
    s = OSlice(view.storage_offset(), list(view.shape), list(view.stride()))
    got = oracle.send_tensor(base.numpy().reshape(-1), s)
    assert np.array_equal(got.reshape(view.shape), view.contiguous().numpy())
    # a column block of a weight (the reshard of config 3 at small size)
    w = torch.arange(8 * 16, dtype=torch.int16).reshape(8, 16)
    for k in range(4):
        got = oracle.send_tensor(w.numpy().reshape(-1), OSlice(4 * k, [8, 4], [16, 1]))
        assert np.array_equal(got.reshape(8, 4), w[:, 4 * k:4 * k + 4].numpy())
