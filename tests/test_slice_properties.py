"""Property tests (hypothesis) of the library's host-side Slice against the CPU oracle, modelled on the
reference's proptest strategies (ndslice/src/strategy.rs:76-195): row-major bases, rectangular subviews,
chains of select / at, and the theorems checked there."""
import pytest

hypothesis = pytest.importorskip("hypothesis")
from hypothesis import given, settings, strategies as st  # noqa: E402

from monarch_amd import Slice  # noqa: E402
from oracle import OracleError, OSlice  # noqa: E402

SET = dict(max_examples=150, deadline=None)


@st.composite
def base_and_subview(draw, max_dims=4, max_len=8):
    sizes = draw(st.lists(st.integers(1, max_len), min_size=1, max_size=max_dims))
    starts, lens = [], []
    for n in sizes:
        s0 = draw(st.integers(0, n - 1))
        starts.append(s0)
        lens.append(draw(st.integers(1, n - s0)))
    return sizes, starts, lens


@settings(**SET)
@given(base_and_subview())
def test_subview_coordinate_inclusion(args):
    # strategy.rs:626-642
    sizes, starts, lens = args
    base = Slice.new_row_major(sizes)
    sub = base.subview(starts, lens)
    osub = OSlice.row_major(sizes).subview(starts, lens)
    assert (sub.offset, sub.sizes, sub.strides) == (osub.offset, osub.sizes, osub.strides)
    assert sub.locations().tolist() == osub.iter().tolist()
    off = base.coordinates(sub.offset)
    for loc in sub:
        v = sub.coordinates(loc)
        assert base.nditem([a + b for a, b in zip(v, off)]) == loc
    assert sub.enforce_embedding(base) is sub


@st.composite
def select_chain(draw):
    sizes = draw(st.lists(st.integers(1, 9), min_size=1, max_size=4))
    ops = []
    cur = list(sizes)
    for _ in range(draw(st.integers(0, 4))):
        dim = draw(st.integers(0, len(cur) - 1))
        if draw(st.booleans()) and len(cur) > 1:
            idx = draw(st.integers(0, cur[dim] - 1))
            ops.append(("at", dim, idx))
            cur.pop(dim)
        else:
            b = draw(st.integers(0, cur[dim] - 1))
            e = draw(st.integers(b + 1, cur[dim] + 2))   # may exceed the size: callers clamp (shape.rs:335-340)
            e = min(e, cur[dim])
            step = draw(st.integers(1, 4))
            ops.append(("select", dim, b, e, step))
            cur[dim] = (e - b + step - 1) // step
    return sizes, ops


@settings(**SET)
@given(select_chain())
def test_select_at_chains_agree_with_oracle(args):
    sizes, ops = args
    s, o = Slice.new_row_major(sizes), OSlice.row_major(sizes)
    for op in ops:
        try:
            o2 = o.at(op[1], op[2]) if op[0] == "at" else o.select(*op[1:])
            err = None
        except OracleError as e:
            o2, err = None, e.name
        if err is None:
            s = s.at(op[1], op[2]) if op[0] == "at" else s.select(*op[1:])
            o = o2
            assert (s.offset, s.sizes, s.strides) == (o.offset, o.sizes, o.strides)
        else:
            with pytest.raises(ValueError, match=err):
                s.at(op[1], op[2]) if op[0] == "at" else s.select(*op[1:])
            break
    locs = s.locations().tolist()
    assert locs == o.iter().tolist()
    assert len(set(locs)) == len(locs)                      # validated slices are injective
    for i, loc in enumerate(locs[:64]):
        assert s[i] == loc and s.index(loc) == i            # get and index are inverse (slice.rs:1073-1108)


@settings(**SET)
@given(st.lists(st.integers(1, 7), min_size=0, max_size=4), st.data())
def test_view_reshape_of_dense_slices(sizes, data):
    # slice.rs:966-1028: a dense row-major base reshapes to any factorisation of its length
    base = Slice.new_row_major(sizes)
    n = len(base)
    factors, rest = [], n
    while rest > 1 and len(factors) < 3:
        divs = [d for d in range(1, rest + 1) if rest % d == 0]
        d = data.draw(st.sampled_from(divs))
        factors.append(d)
        rest //= d
    factors.append(rest)
    v = base.view(factors)
    assert v.offset == 0 and len(v) == n and v.is_contiguous()
    assert v.locations().tolist() == list(range(n))
    with pytest.raises(ValueError, match="IncompatibleView"):
        base.view(factors + [2])
