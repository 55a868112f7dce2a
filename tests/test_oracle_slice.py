"""Pins the CPU oracle's Slice restatement against the reference's own test vectors
(tests/golden/ndslice_vectors.json), the seeded fuzz of
python/tests/_monarch/test_ndslice.py:143-167, and numpy's as_strided (a library
routine) on small shapes."""
import json
import math
import os
import random

import numpy as np
import pytest

from oracle import OracleError, OSlice, mesh_dim_members, mesh_ranks_for_dims
import oracle


@pytest.fixture(scope="module")
def vec(golden_dir):
    with open(os.path.join(golden_dir, "ndslice_vectors.json")) as f:
        return json.load(f)


def mk(t):
    return OSlice(t[0], t[1], t[2])


def test_get_vectors(vec):
    for case in vec["get"]:
        s = mk(case["slice"])
        assert [s.get(i) for i in case["index"]] == case["loc"], case["src"]


def test_iter_vectors(vec):
    for case in vec["iter"]:
        s = mk(case["slice"])
        want = case["locs"] if "locs" in case else list(range(*case["locs_range"]))
        assert s.iter().tolist() == want, case["src"]
        # slice.rs:900-901: iteration corresponds with get
        assert s.iter().tolist() == [s.get(i) for i in range(len(s))]


def test_coordinates_index_vectors(vec):
    for case in vec["coordinates"]:
        s = mk(case["slice"])
        for v, c in case["ok"]:
            assert s.coordinates(v) == c, case["src"]
        for v in case["err"]:
            with pytest.raises(OracleError) as e:
                s.coordinates(v)
            assert e.value.name == "ValueNotInSlice"
    for case in vec["index"]:
        s = mk(case["slice"])
        for v, i in case["ok"]:
            assert s.index(v) == i, case["src"]
        for v in case["err"]:
            with pytest.raises(OracleError):
                s.index(v)


def test_select_at_view_embedding_vectors(vec):
    for case in vec["select"]:
        s = mk(case["slice"])
        for dim, b, e, step in case["ops"]:
            s = s.select(dim, b, e, step)
        if "locs" in case:
            assert s.iter().tolist() == case["locs"], case["src"]
        if "result" in case:
            assert [s.offset, s.sizes, s.strides] == case["result"], case["src"]
    for case in vec["at"] + vec["at_more"]:
        r = mk(case["slice"]).at(case["dim"], case["index"])
        assert [r.offset, r.sizes, r.strides] == case["result"], case["src"]
    for case in vec["view"]:
        s = mk(case["slice"])
        if "error" in case:
            with pytest.raises(OracleError) as e:
                s.view(case["new_sizes"])
            assert e.value.name == case["error"], case["src"]
        else:
            v = s.view(case["new_sizes"])
            assert v.strides == case["strides"] and v.offset == 0, case["src"]
    # slice.rs:601-606: a base that does not start at 0 is refused even when it is empty (every other such base already
    # fails the membership test of offset 0)
    with pytest.raises(OracleError) as e:
        OSlice(3, [0], [1]).view([0])
    assert e.value.name == "IncompatibleView"
    for case in vec["embedding"]:
        base, view = mk(case["base"]), mk(case["view"])
        if case["ok"]:
            view.enforce_embedding(base)
        else:
            with pytest.raises(OracleError):
                view.enforce_embedding(base)


def test_select_errors():
    # slice.rs:298-312 and shape.rs:506-524 (1..1 is empty, 8 is out of range for gpu=8)
    s = OSlice(0, [2, 8], [8, 1])
    with pytest.raises(OracleError) as e:
        s.select(1, 1, 1, 1)
    assert e.value.name == "EmptyRange"
    with pytest.raises(OracleError) as e:
        s.select(1, 8, 9, 1)
    assert e.value.name == "IndexOutOfRange"
    with pytest.raises(OracleError) as e:
        s.select(2, 0, 1, 1)
    assert e.value.name == "IndexOutOfRange"
    with pytest.raises(OracleError) as e:
        s.at(2, 0)
    assert e.value.name == "DimensionOutOfRange"
    with pytest.raises(OracleError) as e:
        s.at(0, 2)
    assert e.value.name == "IndexOutOfRange"


def test_validation_rules():
    # Each rule of Slice::new (slice.rs:99-139) with a witness that trips only it.
    with pytest.raises(OracleError) as e:
        OSlice(0, [2, 3], [3])
    assert e.value.name == "InvalidDims"
    with pytest.raises(OracleError) as e:
        OSlice(0, [2, 2], [3, 2])  # 3 % 2 != 0
    assert e.value.name == "NonrectangularShape"
    with pytest.raises(OracleError) as e:
        OSlice(0, [2, 2], [2, 2])
    assert e.value.name == "NonuniqueStrides"
    with pytest.raises(OracleError) as e:
        OSlice(0, [2, 3], [2, 1])  # stride 2 < 1*3
    assert e.value.name == "StrideTooSmall"
    with pytest.raises(OracleError) as e:
        OSlice(0, [2], [0])
    assert e.value.name == "StrideTooSmall"
    # repeated strides are fine when a size is 1 (slice.rs:118-121, :929)
    OSlice(0, [2, 1, 1], [1, 1, 1])
    OSlice(0, [1, 1], [1, 1])
    # strides need not be monotone in dim order (slice.rs:875)
    OSlice(0, [2, 2, 2], [4, 32, 1])
    # gaps are fine
    OSlice(10, [10, 2], [10, 5])
    # empty dims: len 0, nothing iterated
    s = OSlice(0, [3, 0], [1, 3])
    assert len(s) == 0 and s.iter().tolist() == []


def test_len_contiguous_rowmajor():
    s = OSlice.row_major([4, 4, 4])  # slice.rs:959-964
    assert (s.offset, s.sizes, s.strides) == (0, [4, 4, 4], [16, 4, 1])
    assert s.is_contiguous()
    assert s.iter().tolist() == list(range(64))  # slice.rs:62-63
    assert not OSlice(0, [4, 128, 256], [65536, 512, 1]).is_contiguous()
    assert len(OSlice(37, [], [])) == 1
    assert OSlice(5, [], []).is_contiguous()
    # doc example slice.rs:72-80
    s = OSlice(0, [2, 4, 2], [8, 2, 1])
    sub = OSlice(6, [2, 2], [8, 1])
    for x in range(2):
        for y in range(2):
            assert sub.location([x, y]) == s.location([x, 3, y])
    # test_at_1d_to_0d, slice.rs:1031-1043
    zero_d = OSlice.row_major([5]).at(0, 3)
    assert (zero_d.offset, zero_d.sizes, zero_d.strides) == (3, [], []) and zero_d.location([]) == 3


def test_subview_inclusion():
    # strategy.rs:626-642
    rng = random.Random(1)
    for _ in range(200):
        ndim = rng.randrange(1, 5)
        base = OSlice.row_major([rng.randrange(1, 9) for _ in range(ndim)])
        starts = [rng.randrange(0, n) for n in base.sizes]
        lens = [rng.randrange(1, n - st + 1) for n, st in zip(base.sizes, starts)]
        sub = base.subview(starts, lens)
        off_in_base = base.coordinates(sub.offset)
        for loc in sub.iter().tolist():
            v = sub.coordinates(loc)
            b = [a + c for a, c in zip(v, off_in_base)]
            assert base.location(b) == loc
    with pytest.raises(OracleError):
        OSlice.row_major([2, 3]).subview([1, 1], [2, 2])


def _check(s: OSlice):
    """The check() of python/tests/_monarch/test_ndslice.py:99-133."""
    elems = s.iter().tolist()
    all_ = set(elems)
    assert len(all_) == len(elems), "wrong checks for valid strides"
    for i, e in enumerate(elems):
        assert s.get(i) == e, "index broken"
        assert s.index(e) == i, "inverse broken"
    n = math.prod(s.sizes)
    with pytest.raises(OracleError):
        s.get(n)
    if not all_:
        return
    for i in range(min(all_), max(all_) + 1):
        if i not in all_:
            assert not s.contains(i), "index broken, extra elements"
        else:
            assert s.contains(i)


def fuzz_slices(n=1000, seed=0):
    """The seeded generator of python/tests/_monarch/test_ndslice.py:143-167
    (rejection sampling included), re-expressed with the oracle as validator."""
    gen = random.Random(seed)

    def fuzz():
        while True:
            ndim = gen.choices([1, 2, 3, 4], [1, 2, 3, 4])[0]
            sizes = [gen.randrange(1, 10) for _ in range(ndim)]
            strides, run = [], 1
            for j in range(ndim):
                run *= gen.randrange(1 if j == 0 else 2, 4)
                strides.append(run)
            order = list(range(ndim))
            gen.shuffle(order)
            try:
                return OSlice(gen.randrange(10000), [sizes[o] for o in order], [strides[o] for o in order])
            except OracleError:
                continue

    return [fuzz() for _ in range(n)]


def test_named_and_fuzz_check(vec):
    for t in vec["check_named"]["slices"]:
        _check(mk(t))
    for s in fuzz_slices():
        _check(s)


def test_get_closed_form_and_as_strided():
    # get(i) == offset + sum(((i // prod(sizes[k+1:])) % sizes[k]) * strides[k]), and the
    # whole iteration equals numpy's as_strided view flattened in C order.
    for s in fuzz_slices(200, seed=7):
        n = len(s)
        span = s.offset + sum((z - 1) * st for z, st in zip(s.sizes, s.strides)) + 1
        base = np.arange(span, dtype=np.int64)
        view = np.lib.stride_tricks.as_strided(base[s.offset:], shape=s.sizes,
                                               strides=[st * 8 for st in s.strides])
        assert view.reshape(-1).tolist() == s.iter().tolist()
        for i in range(0, n, max(1, n // 17)):
            loc, rest = s.offset, i
            for k in reversed(range(s.ndim)):
                loc += (rest % s.sizes[k]) * s.strides[k]
                rest //= s.sizes[k]
            assert s.get(i) == loc


def test_device_mesh_vectors(vec):
    for case in vec["device_mesh"]:
        ranks = mk(case["ranks"])
        for d, want in case["dims"].items():
            members, dr = mesh_dim_members(ranks, case["rank"], int(d))
            assert members == want["members"] and dr == want["rank"], case["src"]
            assert members[dr] == case["rank"]  # device_mesh.rs:86
        for dims, want in case["for_dims"]:
            assert mesh_ranks_for_dims(ranks, case["rank"], dims) == want, case["src"]
    # C4: mesh [2 hosts, 8 gpus], dim "gpu" => 8 members 8h..8h+7
    ranks = OSlice(0, [2, 8], [8, 1])
    for r in range(16):
        members, dr = mesh_dim_members(ranks, r, 1)
        assert members == list(range(8 * (r // 8), 8 * (r // 8) + 8)) and dr == r % 8


def test_pack_unpack_against_as_strided():
    import torch
    rng = np.random.default_rng(3)
    for s in fuzz_slices(150, seed=11) + [OSlice(0, [4, 128, 256], [65536, 512, 1]), OSlice(37, [], [])]:
        span = s.offset + sum((z - 1) * st for z, st in zip(s.sizes, s.strides)) + 1
        for dt in (np.uint8, np.uint16, np.float32, np.float64):
            base = rng.integers(0, 255, size=span + 3).astype(dt)
            got = oracle.pack(base, s)
            want = torch.as_strided(torch.from_numpy(base), s.sizes, s.strides, s.offset).contiguous().flatten().numpy()
            assert np.array_equal(got, want)
            assert np.array_equal(oracle.pack(base, s, runs=True), want)
            assert np.array_equal(oracle.pack(base, s, threads=True), want)
            # unpack: round trip on the view, untouched elsewhere
            dst = np.full_like(base, 7)
            oracle.unpack(dst, got, s)
            mask = np.zeros(base.size, dtype=bool)
            mask[s.iter().astype(np.int64)] = True
            assert np.array_equal(dst[mask], base[mask])
            assert np.all(dst[~mask] == 7)
