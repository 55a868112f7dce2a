"""Host-side product logic (the library's C++ Slice / DeviceMesh behind the C ABI, and its
Python face) against the reference's test vectors and against the CPU oracle.  No GPU."""
import json
import math
import os
import pickle
import random

import pytest

from monarch_amd import DeviceMesh, Slice
from oracle import OracleError, OSlice
from util import fuzz_slices


@pytest.fixture(scope="module")
def vec(golden_dir):
    with open(os.path.join(golden_dir, "ndslice_vectors.json")) as f:
        return json.load(f)


def mk(t):
    return Slice(offset=t[0], sizes=t[1], strides=t[2])


def test_reference_python_cases():
    # python/tests/_monarch/test_ndslice.py:19-61, verbatim behaviour
    s = Slice(offset=0, sizes=[2, 3], strides=[3, 1])
    for i in range(4):
        assert s[i] == i
    assert list(s) == list(range(6))
    s = Slice(offset=0, sizes=[3, 4, 5], strides=[20, 5, 1])
    assert s[3 * 4 + 1] == 13
    s = Slice(offset=0, sizes=[2, 2, 2], strides=[4, 32, 1])
    assert s[2] == 32 and s[1] == 1
    s = Slice(offset=10, sizes=[10, 2], strides=[10, 5])
    assert list(s) == list(range(10, 106, 5))
    assert list(s) == [s[i] for i in range(len(s))]
    s = Slice(offset=0, sizes=[2, 3], strides=[3, 1])
    assert s.coordinates(0) == [0, 0] and s.coordinates(3) == [1, 0]
    with pytest.raises(ValueError):
        s.coordinates(6)
    s = Slice(offset=10, sizes=[2, 3], strides=[3, 1])
    with pytest.raises(ValueError):
        s.coordinates(6)
    assert s.coordinates(10) == [0, 0] and s.coordinates(13) == [1, 0]
    s = Slice(offset=0, sizes=[2, 3], strides=[3, 1])
    assert s.index(3) == 3
    with pytest.raises(ValueError):
        s.index(14)
    assert Slice(offset=0, sizes=[2, 2], strides=[4, 2]).index(2) == 1
    assert s[1:5:2] == (1, 3)
    assert s.nditem([1, 2]) == 5
    with pytest.raises(IndexError):
        s.nditem([1])


def test_from_list_repr_pickle_eq():
    # test_ndslice.py:63-96,169-181
    assert Slice.from_list([]) == []
    sl = Slice.from_list([1, 2, 3])
    assert len(sl) == 1 and (sl[0].offset, sl[0].sizes, sl[0].strides) == (1, [3], [1])
    sl = Slice.from_list([1, 3, 5])
    assert len(sl) == 1 and (sl[0].offset, sl[0].sizes, sl[0].strides) == (1, [3], [2])
    sl = Slice.from_list([1, 2, 4, 5, 6])
    assert [(x.offset, x.sizes, x.strides) for x in sl] == [(1, [2], [1]), (4, [3], [1])]
    sl = Slice.from_list(list(range(100)))
    assert [(x.offset, x.sizes, x.strides) for x in sl] == [(0, [100], [1])]
    sl = Slice.from_list([1, 2, 3, 10, 11, 12])
    assert [(x.offset, x.sizes, x.strides) for x in sl] == [(1, [3], [1]), (10, [3], [1])]
    s = Slice(offset=10, sizes=[2, 3], strides=[3, 1])
    assert pickle.loads(pickle.dumps(s)) == s and hash(pickle.loads(pickle.dumps(s))) == hash(s)
    s = Slice(offset=0, sizes=[2, 3], strides=[3, 1])
    assert str(s) == "Slice { offset: 0, sizes: [2, 3], strides: [3, 1] }" == repr(s)
    assert s != Slice(offset=1, sizes=[2, 3], strides=[3, 1]) and s != "x"


def test_golden_vectors(vec):
    for case in vec["get"]:
        s = mk(case["slice"])
        assert [s[i] for i in case["index"]] == case["loc"], case["src"]
    for case in vec["iter"]:
        s = mk(case["slice"])
        want = case["locs"] if "locs" in case else list(range(*case["locs_range"]))
        assert list(s) == want and s.locations().tolist() == want, case["src"]
    for case in vec["coordinates"]:
        s = mk(case["slice"])
        for v, c in case["ok"]:
            assert s.coordinates(v) == c
        for v in case["err"]:
            with pytest.raises(ValueError):
                s.coordinates(v)
    for case in vec["index"]:
        s = mk(case["slice"])
        for v, i in case["ok"]:
            assert s.index(v) == i
        for v in case["err"]:
            with pytest.raises(ValueError):
                s.index(v)
    for case in vec["select"]:
        s = mk(case["slice"])
        for dim, b, e, step in case["ops"]:
            s = s.select(dim, b, e, step)
        if "locs" in case:
            assert list(s) == case["locs"], case["src"]
        if "result" in case:
            assert [s.offset, s.sizes, s.strides] == case["result"], case["src"]
    for case in vec["at"] + vec["at_more"]:
        r = mk(case["slice"]).at(case["dim"], case["index"])
        assert [r.offset, r.sizes, r.strides] == case["result"], case["src"]
    for case in vec["view"]:
        s = mk(case["slice"])
        if "error" in case:
            with pytest.raises(ValueError, match=case["error"]):
                s.view(case["new_sizes"])
        else:
            assert s.view(case["new_sizes"]).strides == case["strides"]
    for case in vec["embedding"]:
        base, view = mk(case["base"]), mk(case["view"])
        if case["ok"]:
            assert view.enforce_embedding(base) is view
        else:
            with pytest.raises(ValueError):
                view.enforce_embedding(base)


def test_validation_classes_match_oracle():
    # same accept/reject decision and same error class as the oracle on random candidates,
    # including invalid ones (overlapping, non-rectangular, repeated strides, zero sizes)
    gen = random.Random(5)
    seen = set()
    for _ in range(4000):
        ndim = gen.randrange(0, 5)
        sizes = [gen.choice([0, 1, 1, 2, 3, 4, 7]) for _ in range(ndim)]
        strides = [gen.choice([0, 1, 1, 2, 3, 4, 6, 8, 12, 16, 24]) for _ in range(ndim)]
        try:
            OSlice(3, sizes, strides)
            want = None
        except OracleError as e:
            want = e.name
        try:
            Slice(offset=3, sizes=sizes, strides=strides)
            got = None
        except ValueError as e:
            got = str(e).split(" ")[0]
        assert got == want, (sizes, strides)
        seen.add(want)
    assert {None, "NonrectangularShape", "NonuniqueStrides", "StrideTooSmall"} <= seen
    with pytest.raises(ValueError, match="InvalidDims"):
        Slice(offset=0, sizes=[2, 3], strides=[3])


def test_error_classes_of_select_at_subview():
    s = Slice(offset=0, sizes=[2, 8], strides=[8, 1])
    with pytest.raises(ValueError, match="EmptyRange"):
        s.select(1, 1, 1, 1)
    with pytest.raises(ValueError, match="IndexOutOfRange"):
        s.select(1, 8, 9, 1)
    with pytest.raises(ValueError, match="IndexOutOfRange"):
        s.select(2, 0, 1, 1)
    with pytest.raises(ValueError, match="DimensionOutOfRange"):
        s.at(2, 0)
    with pytest.raises(ValueError, match="IndexOutOfRange"):
        s.at(0, 2)
    with pytest.raises(ValueError, match="InvalidDims"):
        s.subview([0], [1])
    with pytest.raises(ValueError, match="IndexOutOfRange"):
        s.subview([1, 1], [2, 2])
    assert s.subview([1, 2], [1, 3]) == Slice(offset=10, sizes=[1, 3], strides=[8, 1])
    # select re-validates its result (slice.rs:325): stepping the inner dim of [2,4]/[4,1] by 3
    # gives strides [4,3], which no longer nest
    t = Slice(offset=0, sizes=[2, 4], strides=[4, 1])
    with pytest.raises(ValueError, match="NonrectangularShape"):
        t.select(1, 0, 4, 3)
    with pytest.raises(OracleError) as e:
        OSlice(0, [2, 4], [4, 1]).select(1, 0, 4, 3)
    assert e.value.name == "NonrectangularShape"


def _check(s: Slice):
    """check() of python/tests/_monarch/test_ndslice.py:99-133."""
    elems = list(s)
    all_ = set(elems)
    assert len(all_) == len(elems), "wrong checks for valid strides"
    for i, e in enumerate(s):
        assert s[i] == e, "index broken"
        assert s.index(e) == i, "inverse broken"
    n = math.prod(s.sizes)
    with pytest.raises(IndexError):
        s[n]
    with pytest.raises(TypeError):
        s[-1]
    if not all_:
        return
    for i in range(min(all_), max(all_) + 1):
        if i not in all_:
            assert i not in s
            with pytest.raises(ValueError):
                s.index(i)


def test_named_and_fuzz_check(vec):
    for t in vec["check_named"]["slices"]:
        _check(mk(t))
    for s in fuzz_slices(1000, seed=0):
        _check(s)


def test_product_equals_oracle_on_fuzz():
    for s in fuzz_slices(300, seed=21):
        o = OSlice.unchecked(s.offset, s.sizes, s.strides)
        assert s.locations().tolist() == o.iter().tolist()
        assert len(s) == len(o) and s.is_contiguous() == o.is_contiguous()
        lo, hi = s.bounds()
        locs = o.iter()
        assert (lo, hi) == (int(locs.min()), int(locs.max()))
        for v in range(lo, min(hi, lo + 40) + 1):
            try:
                want = o.coordinates(v)
            except OracleError:
                want = None
            got = s.coordinates(v) if v in s else None
            assert got == want
        # partial iteration windows agree with the full walk
        n = len(s)
        assert s.locations(n // 3, 5).tolist() == locs[n // 3: n // 3 + 5].tolist()


def test_of_tensor_is_as_strided_triple():
    import torch
    x = torch.arange(4 * 256 * 256, dtype=torch.float32).reshape(4, 256, 256)
    v = x[:, ::2, :]
    s = Slice.of_tensor(v)
    assert (s.offset, s.sizes, s.strides) == (0, [4, 128, 256], [65536, 512, 1])
    assert torch.equal(x.reshape(-1)[torch.from_numpy(s.locations().astype("int64"))], v.reshape(-1))
    assert Slice.new_row_major([4, 4, 4]).strides == [16, 4, 1]
    assert Slice.new_row_major([3, 0, 2]).is_contiguous() and len(Slice.new_row_major([3, 0, 2])) == 0


def test_device_mesh(vec):
    for case in vec["device_mesh"]:
        names = [f"d{i}" for i in range(len(case["ranks"][1]))]
        mesh = DeviceMesh(names, mk(case["ranks"]), case["rank"])
        for d, want in case["dims"].items():
            dim = mesh.dims[names[int(d)]]
            assert dim.members == want["members"] and dim.rank == want["rank"], case["src"]
            assert dim.members[dim.rank] == case["rank"]
        for dims, want in case["for_dims"]:
            assert mesh.get_ranks_for_dim_slice([names[i] for i in dims]) == want, case["src"]
    mesh = DeviceMesh(["host", "gpu"], Slice(offset=0, sizes=[2, 8], strides=[8, 1]), 11)
    assert mesh.group_size(["gpu"]) == 8 and mesh.get_ranks_for_dim_slice(["gpu"]) == list(range(8, 16))
    assert mesh.all_ranks == list(range(16)) and mesh.sizes() == {"host": 2, "gpu": 8}
    with pytest.raises(KeyError):
        mesh.get_ranks_for_dim_slice(["nope"])
    with pytest.raises(ValueError):
        DeviceMesh(["host", "gpu"], Slice(offset=0, sizes=[2, 8], strides=[8, 1]), 16)
    with pytest.raises(ValueError):
        DeviceMesh(["host"], Slice(offset=0, sizes=[2, 8], strides=[8, 1]), 0)


def test_reduce_argument_validation_messages():
    # python/monarch/common/tensor.py:287-333 and _fake_reduce (:491-512); messages quoted in
    # python/tests/test_controller.py:197,204-215,262-265
    from monarch_amd.reduce import Reduction, ReduceOp, check_reduce_args
    names, sizes = ["host", "gpu"], {"host": 2, "gpu": 2}
    assert check_reduce_args(names, sizes, (3, 4), "gpu", "sum") == (("gpu",), (3, 4))
    assert check_reduce_args(names, sizes, (3, 4), "gpu", "stack") == (("gpu",), (2, 3, 4))
    assert check_reduce_args(names, sizes, (2, 6), "gpu", "sum", scatter=True) == (("gpu",), (6,))
    assert check_reduce_args(names, sizes, (2, 6), "gpu", "stack", scatter=True) == (("gpu",), (2, 6))
    assert check_reduce_args(names, sizes, (2, 6), (), "sum") == (("host", "gpu"), (2, 6))
    with pytest.raises(TypeError, match="When scattering results the outer most dimension"):
        check_reduce_args(names, sizes, (3, 4), "gpu", "sum", scatter=True)
    with pytest.raises(TypeError, match="When scattering"):
        check_reduce_args(names, sizes, (), "gpu", "sum", scatter=True)
    for kw in (dict(scatter=True), dict(reduction="stack"), dict(reduction="stack", scatter=True)):
        with pytest.raises(ValueError, match="is not valid for multiple dimensions"):
            check_reduce_args(names, sizes, (2, 6), (), **kw)
    with pytest.raises(KeyError, match="dim x not found"):
        check_reduce_args(names, sizes, (2, 6), "x")
    with pytest.raises(ValueError, match="reducing the same dimension twice"):
        check_reduce_args(names, sizes, (2, 6), ("gpu", "gpu"))
    with pytest.raises(ValueError, match="not supported, reductions are"):
        check_reduce_args(names, sizes, (2, 6), "gpu", "median")
    with pytest.raises(ValueError, match="`out` cannot be used with inplace reduce"):
        check_reduce_args(names, sizes, (2, 6), "gpu", "sum", inplace=True, out_shape=(2, 6))
    with pytest.raises(ValueError, match="is not valid for in-place operation"):
        check_reduce_args(names, sizes, (2, 6), "gpu", "sum", scatter=True, inplace=True)
    with pytest.raises(ValueError, match=r"Reduce expects the shape to be torch.Size\(\[6\]\)"):
        check_reduce_args(names, sizes, (2, 6), "host", "sum", scatter=True, out_shape=(2, 4))
    assert Reduction.from_str("stack").is_stack and Reduction.from_str("avg").op == ReduceOp.Avg
    assert int(ReduceOp.Sum) == 0 and int(ReduceOp.Avg) == 4  # nccl.rs:285-292


def test_send_tensor_routing_and_to_mesh_checks():
    # monarch_tensor_worker/src/lib.rs:722-731: the i-th rank of from_ranks sends to the i-th of to_ranks
    from monarch_amd.send_tensor import check_to_mesh, route
    from_ranks = Slice(offset=0, sizes=[2, 2], strides=[4, 1])   # ranks 0, 1, 4, 5
    to_ranks = Slice(offset=2, sizes=[2, 2], strides=[4, 1])     # ranks 2, 3, 6, 7
    assert route(from_ranks, to_ranks, 0) == (None, 2)
    assert route(from_ranks, to_ranks, 5) == (None, 7)
    assert route(from_ranks, to_ranks, 6) == (4, None)
    assert route(from_ranks, to_ranks, 8) == (None, None)
    same = Slice(offset=0, sizes=[4], strides=[1])
    assert route(same, same, 3) == (3, 3)                         # local: from == to
    shifted = Slice(offset=1, sizes=[3], strides=[1])
    assert route(Slice(offset=0, sizes=[3], strides=[1]), shifted, 1) == (0, 2)   # both sender and receiver
    # python/monarch/common/tensor.py:417-438
    slicing = Slice(offset=0, sizes=[2, 8], strides=[8, 1])
    fr, bc = check_to_mesh(["host", "gpu"], slicing, ["host", "gpu"], [2, 8])
    assert fr == slicing and bc == []
    fr, bc = check_to_mesh(["gpu"], Slice(offset=8, sizes=[8], strides=[1]), ["replica", "gpu"], [3, 8])
    assert fr == Slice(offset=8, sizes=[8], strides=[1]) and bc == ["replica"]
    with pytest.raises(ValueError, match="dimension gpu of destination device_mesh has a different length"):
        check_to_mesh(["host", "gpu"], slicing, ["host", "gpu"], [2, 4])
    with pytest.raises(ValueError, match="destination mesh does not have dimensions"):
        check_to_mesh(["host", "gpu"], slicing, ["gpu"], [8])


def test_transfer_and_stack_argument_checks_without_a_gpu():
    # everything that is refused before a launch: lengths fit the 32-bit field of a scatter/gather entry
    # (rdma_components.rs:1041,1063), buffers must be large enough, stack chunks must divide evenly
    import ctypes as C
    from monarch_amd import _lib
    from monarch_amd._lib import RdmaBufferC
    from monarch_amd.staging import MAX_SEGMENT_BYTES
    lib = _lib.lib()
    assert MAX_SEGMENT_BYTES < 2**32 and MAX_SEGMENT_BYTES % 16 == 0
    posted = C.c_uint32(7)
    assert lib.mhip_buffer_transfer(None, None, 0, 0, None, C.byref(posted)) == 0 and posted.value == 0
    assert lib.mhip_buffer_transfer(None, 16, 32, 0, None, None) == _lib.ERR_UNDEFINED_TENSOR
    small, big = RdmaBufferC(4096, 100), RdmaBufferC(8192, 101)
    assert lib.mhip_buffer_read_into(C.byref(big), C.byref(small), None) == _lib.ERR_BUFFER_TOO_SMALL
    assert lib.mhip_buffer_write_from(C.byref(big), C.byref(small), None) == _lib.ERR_BUFFER_TOO_SMALL
    assert lib.mhip_buffer_read_into(None, C.byref(small), None) == _lib.ERR_INVALID_ARGUMENT
    empty = RdmaBufferC(None, 0)
    assert lib.mhip_buffer_read_into(C.byref(empty), C.byref(small), None) == 0     # nothing to move
    one = (C.c_void_p * 2)(4096, 8192)
    assert lib.mhip_stack_scatter(4096, one, 2, 0, 7, 4, None) == _lib.ERR_INPUT_SIZE_MISMATCH   # 7 elements, 2 members
    assert lib.mhip_stack_scatter(4096, one, 2, 2, 8, 4, None) == _lib.ERR_INDEX_OUT_OF_RANGE
    assert lib.mhip_stack(4096, one, 0, 8, 4, None) == _lib.ERR_INVALID_ARGUMENT
    assert lib.mhip_stack(None, one, 2, 8, 4, None) == _lib.ERR_UNDEFINED_TENSOR
    assert lib.mhip_stack(4096, one, 2, 0, 4, None) == 0
    many = (C.c_void_p * 65)(*([4096] * 65))
    assert lib.mhip_stack(4096, many, 65, 8, 4, None) == _lib.ERR_TOO_MANY_INPUTS
    assert lib.mhip_stack(4098, one, 2, 8, 4, None) == _lib.ERR_INVALID_ARGUMENT     # not element-aligned
    s = Slice(offset=0, sizes=[4, 6], strides=[6, 1])
    assert lib.mhip_send_tensor(4096, 95, 8192, C.byref(s.c), 4, None, None) == _lib.ERR_OUTPUT_SIZE_MISMATCH
    assert lib.mhip_send_tensor(None, 96, 8192, C.byref(s.c), 4, None, None) == _lib.ERR_UNDEFINED_TENSOR
    bad = Slice(offset=0, sizes=[2, 2], strides=[2, 2], _validate=False)
    assert lib.mhip_send_tensor(4096, 16, 8192, C.byref(bad.c), 4, None, None) == _lib.ERR_NONUNIQUE_STRIDES


def test_send_tensor_routing_matches_reference_cases_and_oracle():
    import random
    import oracle
    from monarch_amd.send_tensor import check_to_mesh, route
    # monarch_tensor_worker/src/comm.rs:1493-1537: from_ranks {0,[1],[1]}, to_ranks {1,[1],[1]} on ranks 0 and 1;
    # comm.rs:1662 (send_tensor_local): both slices {0,[1],[1]}
    one = lambda off: Slice(offset=off, sizes=[1], strides=[1])
    assert route(one(0), one(1), 0) == (None, 1) and route(one(0), one(1), 1) == (0, None)
    assert route(one(0), one(0), 0) == (0, 0)
    # python/tests/test_controller.py:311-323 (test_movement) on a 2 x 2 mesh {0,[2,2],[2,1]}: host 0 -> host 1
    sm0, sm1 = Slice(offset=0, sizes=[2], strides=[1]), Slice(offset=2, sizes=[2], strides=[1])
    fr, bc = check_to_mesh(["gpu"], sm0, ["gpu"], [2])
    assert fr == sm0 and bc == []
    assert [route(fr, sm1, r) for r in range(4)] == [(None, 2), (None, 3), (0, None), (1, None)]
    # test_controller.py:325-338 (test_broadcast_one): host=1 submesh to the whole mesh broadcasts along host
    fr, bc = check_to_mesh(["gpu"], sm1, ["host", "gpu"], [2, 2])
    assert fr == sm1 and bc == ["host"]
    # test_controller.py:340-352 (test_broadcast_two): a single device (no named dims left) to the whole mesh
    fr, bc = check_to_mesh([], Slice(offset=3, sizes=[], strides=[]), ["host", "gpu"], [2, 2])
    assert fr == Slice(offset=3, sizes=[], strides=[]) and bc == ["host", "gpu"]
    assert route(fr, one(0), 3) == (None, 0) and route(fr, one(0), 0) == (3, None)
    # random rank slices: the library's routing and the oracle's agree on every rank, senders and receivers pair up
    gen = random.Random(7)
    for _ in range(200):
        nd = gen.randrange(1, 4)
        sizes = [gen.randrange(1, 4) for _ in range(nd)]
        strides, acc = [], 1
        for z in reversed(sizes):
            strides.insert(0, acc)
            acc *= z * gen.randrange(1, 3)
        a = Slice(offset=gen.randrange(5), sizes=sizes, strides=strides)
        kind = gen.randrange(3)
        if kind == 0:      # same shape elsewhere
            b = Slice(offset=gen.randrange(40), sizes=sizes, strides=strides)
        elif kind == 1:    # same number of ranks, another shape
            rm = Slice.new_row_major(sizes[::-1])
            b = Slice(offset=gen.randrange(40), sizes=rm.sizes, strides=rm.strides)
        else:              # fewer or more receivers than senders
            b = Slice(offset=gen.randrange(40), sizes=[gen.randrange(1, 7)], strides=[gen.randrange(1, 3)])
        oa, ob = oracle.OSlice.unchecked(a.offset, a.sizes, a.strides), oracle.OSlice.unchecked(b.offset, b.sizes, b.strides)
        senders, receivers = list(a), list(b)
        for rank in range(0, 80):
            got = route(a, b, rank)
            assert got == oracle.send_tensor_route(oa, ob, rank), (a, b, rank)
            want_to = receivers[senders.index(rank)] if rank in senders and senders.index(rank) < len(receivers) else None
            want_from = senders[receivers.index(rank)] if rank in receivers and receivers.index(rank) < len(senders) else None
            assert got == (want_from, want_to)
