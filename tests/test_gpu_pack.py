"""GPU parity: mhip_slice_pack / unpack (+ _many) against the CPU oracle, bit-exact."""
import numpy as np
import pytest
import torch

import oracle
from monarch_amd import Slice, staging
from monarch_amd._lib import MhipError
from util import valid_slices, bits, fuzz_slices, oslice, span, sync

pytestmark = pytest.mark.gpu
DEV = "cuda:0"


def _storage(nbytes, seed):
    g = torch.Generator().manual_seed(seed)
    return torch.randint(0, 256, (nbytes,), dtype=torch.uint8, generator=g)


def _roundtrip(s: Slice, elem_size: int, seed: int, misalign: int = 0, dst_misalign: int = 0):
    """pack and unpack one slice of `elem_size`-byte elements; compare with the oracle bytes."""
    n_elems = span(s)
    host = _storage((n_elems + 2) * elem_size + misalign, seed)
    dev = host.to(DEV)
    base = dev[misalign: misalign + n_elems * elem_size]
    hbase = host.numpy()[misalign: misalign + n_elems * elem_size]
    n = len(s)
    # oracle works on structured elements of elem_size bytes
    dt = np.dtype((np.void, elem_size))
    want = oracle.pack(hbase.view(dt), oslice(s)).view(np.uint8)
    out_store = torch.full((n * elem_size + dst_misalign + 32,), 0xAB, dtype=torch.uint8, device=DEV)
    out = out_store[dst_misalign: dst_misalign + n * elem_size]
    from monarch_amd._lib import check, lib
    import ctypes as C
    check(lib().mhip_slice_pack(out.data_ptr(), base.data_ptr(), C.byref(s.c), elem_size,
                                torch.cuda.current_stream().cuda_stream))
    sync()
    got = out_store.cpu().numpy()
    assert np.array_equal(got[dst_misalign: dst_misalign + n * elem_size], want), (s, elem_size, misalign)
    assert np.all(got[:dst_misalign] == 0xAB) and np.all(got[dst_misalign + n * elem_size:] == 0xAB)
    # unpack into a canvas of 0x5C: view positions get the packed bytes, the rest stays
    canvas = torch.full_like(dev, 0x5C)
    cbase = canvas[misalign: misalign + n_elems * elem_size]
    check(lib().mhip_slice_unpack(cbase.data_ptr(), out.data_ptr(), C.byref(s.c), elem_size,
                                  torch.cuda.current_stream().cuda_stream))
    sync()
    hcanvas = np.full(host.numel(), 0x5C, dtype=np.uint8)
    oracle.unpack(hcanvas[misalign: misalign + n_elems * elem_size].view(dt), want.view(dt), oslice(s))
    assert np.array_equal(canvas.cpu().numpy(), hcanvas), (s, elem_size, misalign)


NAMED = [
    dict(offset=0, sizes=[3, 4], strides=[4, 1]),
    dict(offset=0, sizes=[3, 4], strides=[1, 4]),        # column-major: a transpose
    dict(offset=1, sizes=[3], strides=[2]),
    dict(offset=1, sizes=[3, 3], strides=[12, 2]),
    dict(offset=0, sizes=[4, 3, 8], strides=[48, 16, 2]),
    dict(offset=24, sizes=[4, 3, 8], strides=[96, 16, 2]),
    dict(offset=37, sizes=[], strides=[]),               # 0-d: one element
    dict(offset=0, sizes=[2, 2, 2], strides=[4, 32, 1]),
    dict(offset=10, sizes=[10, 2], strides=[10, 5]),
    dict(offset=5, sizes=[3, 0], strides=[1, 3]),        # empty: nothing moves
    dict(offset=3, sizes=[1, 1, 7], strides=[1, 1, 1]),
    dict(offset=0, sizes=[64, 100], strides=[128, 1]),   # runs of 100 elements, not a multiple of 16 bytes
    dict(offset=7, sizes=[33, 50], strides=[64, 1]),
]


@pytest.mark.parametrize("elem_size", [1, 2, 4, 8, 16, 3, 6, 12])
def test_named_slices(elem_size):
    for i, kw in enumerate(NAMED):
        _roundtrip(Slice(**kw), elem_size, seed=i)


@pytest.mark.parametrize("elem_size", [1, 2, 4, 8])
def test_fuzz_slices(elem_size):
    for i, s in enumerate(fuzz_slices(120, seed=elem_size)):
        _roundtrip(s, elem_size, seed=i, misalign=(i % 4) * elem_size, dst_misalign=(i % 3) * elem_size)


@pytest.mark.parametrize("elem_size", [1, 2, 4])
def test_fuzz_slices_with_longer_rows(elem_size):
    # valid-by-construction slices with sizes up to 39 in up to four dimensions: rows long enough for the
    # two-vector and whole-chunk forms, short-run and transposing views, at every alignment of both sides
    picked = valid_slices(80, seed=100 + elem_size)
    assert sum(len(s) > 1000 for s in picked) >= 12
    for i, s in enumerate(picked):
        _roundtrip(s, elem_size, seed=i, misalign=(i % 5) * elem_size, dst_misalign=(i % 7) * elem_size)


def test_contiguous_copy_at_every_alignment():
    # one run of bytes, every combination of source and destination alignment within a 16-byte vector, and
    # destinations anywhere inside a 1 KiB row (the copy lays its rows on the destination's 1 KiB boundaries and
    # gives each XCD an eighth of them when the source is aligned differently); lengths around a vector, a row
    # and eight rows, plus ragged ends
    import ctypes as C
    from monarch_amd._lib import check, lib
    g = torch.Generator().manual_seed(9)
    host = torch.randint(0, 256, (80_000,), dtype=torch.uint8, generator=g)
    src_store = host.to(DEV)
    stream = torch.cuda.current_stream().cuda_stream
    cases = [(n, so, do) for n in (1, 15, 95, 96, 97, 111, 128, 1000, 4097, 70_001) for so in (0, 1, 2, 5, 8, 15)
             for do in (0, 1, 3, 8, 14)]
    cases += [(n, so, do) for n in (1, 17, 1023, 1024, 1025, 8191, 8192, 8193, 9000, 66_000) for so in (0, 3, 128, 1000)
              for do in (112, 496, 1000, 1007)]
    for n, so, do in cases:
        s = Slice.new_row_major([n])
        dst_store = torch.full((n + 1100,), 0xEE, dtype=torch.uint8, device=DEV)
        check(lib().mhip_slice_pack(dst_store.data_ptr() + 16 + do, src_store.data_ptr() + so, C.byref(s.c), 1, stream))
        back = torch.full((n + 1100,), 0x11, dtype=torch.uint8, device=DEV)
        check(lib().mhip_slice_unpack(back.data_ptr() + 16 + so, dst_store.data_ptr() + 16 + do, C.byref(s.c), 1, stream))
        sync()
        got = dst_store.cpu()
        assert torch.equal(got[16 + do: 16 + do + n], host[so: so + n]), (n, so, do)
        assert bool((got[:16 + do] == 0xEE).all()) and bool((got[16 + do + n:] == 0xEE).all()), (n, so, do)
        gb = back.cpu()
        assert torch.equal(gb[16 + so: 16 + so + n], host[so: so + n]), (n, so, do)
        assert bool((gb[:16 + so] == 0x11).all()) and bool((gb[16 + so + n:] == 0x11).all()), (n, so, do)


def test_odd_byte_alignment():
    for i, s in enumerate(fuzz_slices(40, seed=99)):
        _roundtrip(s, 1, seed=i, misalign=1 + (i % 15), dst_misalign=(i * 7) % 16)
    _roundtrip(Slice(offset=3, sizes=[5000], strides=[1]), 1, seed=1, misalign=5, dst_misalign=9)
    _roundtrip(Slice(offset=3, sizes=[40, 300], strides=[301, 1]), 2, seed=2, misalign=2, dst_misalign=6)


@pytest.mark.parametrize("elem_size", [1, 2, 4, 8, 3, 6])
def test_rows_that_are_not_whole_chunks(elem_size):
    # rows at least 16 bytes long whose length is not a multiple of 16 bytes, and staging addresses
    # that are not 16-byte aligned: chunks straddling a row boundary move as two overlapping vectors
    cases = [Slice(offset=1, sizes=[300, 1791], strides=[2047, 1]), Slice(offset=0, sizes=[1200, 17], strides=[19, 1]),
             Slice(offset=5, sizes=[7, 50, 129], strides=[52 * 131, 131, 1]), Slice(offset=0, sizes=[2500, 33], strides=[40, 1]),
             Slice(offset=2, sizes=[3, 2, 40, 100], strides=[2 * 40 * 128 * 2, 40 * 128, 128, 1]),
             Slice(offset=0, sizes=[1000, 128], strides=[136, 1])]   # whole chunks, but the staging address is shifted
    for i, s in enumerate(cases):
        for dst_misalign in (0, elem_size, 5 * elem_size):
            _roundtrip(s, elem_size, seed=i, misalign=(i % 3) * elem_size, dst_misalign=dst_misalign)


@pytest.mark.parametrize("elem_size", [1, 2, 4])
def test_views_that_start_off_the_unit_of_their_shape(elem_size):
    # row length and pitch allow a wider unit than the address the view starts at (a bf16 view of even shape at an odd
    # column, a base pointer that is only element-aligned): the copy runs in the wider unit from a skewed base
    e = elem_size
    cases = [Slice(offset=1, sizes=[300, 8 // e * 447], strides=[8 // e * 1024, 1]),     # rows of 3576 bytes: 8-byte units
             Slice(offset=3, sizes=[100, 16 // e * 224], strides=[16 // e * 512, 1]),    # whole 16-byte chunks, 16-byte units
             Slice(offset=1, sizes=[64, 16 // e * 500], strides=[16 // e * 512, 1]),     # rows of 8000 bytes
             Slice(offset=5, sizes=[9, 40, 4 // e * 33], strides=[40 * 4 // e * 64, 4 // e * 64, 1]),  # rows of 132 bytes: gathered
             Slice(offset=7, sizes=[2000, 4 // e * 3], strides=[4 // e * 5, 1]),          # runs of 12 bytes
             Slice(offset=2, sizes=[70, 16 // e * 70], strides=[16 // e * 71, 1])]
    for i, s in enumerate(cases):
        for misalign in (0, e, 3 * e):
            for dst_misalign in (0, 16):
                _roundtrip(s, e, seed=40 + i, misalign=misalign, dst_misalign=dst_misalign)
    # rows of 8-byte-granular shape from a base that is 2 bytes off: some rows start 122 bytes into a cache line, deeper
    # than any address that is a multiple of the unit, and overlap one line more
    _roundtrip(Slice(offset=0, sizes=[56, 776 // e], strides=[792 // e, 1]), e, seed=47, misalign=2 if e <= 2 else e, dst_misalign=0)
    # several views in one launch: equal skews batch, different ones do not
    g = torch.Generator().manual_seed(41)
    x = torch.randint(0, 256, (64, 8192 * e), dtype=torch.uint8, generator=g)
    dev = x.to(DEV)
    n = 16 // e * 100
    offsets = [1, 1 + n, 1 + 2 * n, 2 + 3 * n, 5 + 4 * n]
    views = [Slice(offset=o, sizes=[64, n], strides=[8192, 1]) for o in offsets]
    outs = [torch.empty(64 * n * e, dtype=torch.uint8, device=DEV) for _ in views]
    import ctypes as C
    from monarch_amd._lib import check, lib, ptr_array
    from monarch_amd.ndslice import slice_array
    arr = slice_array(views)
    stream = torch.cuda.current_stream().cuda_stream
    check(lib().mhip_slice_pack_many(ptr_array([o.data_ptr() for o in outs]), dev.data_ptr(), arr, len(views), e, stream))
    back = torch.full_like(dev, 0x3C)
    check(lib().mhip_slice_unpack_many(back.data_ptr(), ptr_array([o.data_ptr() for o in outs]), arr, len(views), e, stream))
    sync()
    want = torch.full_like(x, 0x3C)
    for o, out in zip(offsets, outs):
        assert torch.equal(out.cpu().view(64, n * e), x[:, o * e: (o + n) * e]), o
        want[:, o * e: (o + n) * e] = x[:, o * e: (o + n) * e]
    assert torch.equal(back.cpu(), want)


@pytest.mark.parametrize("elem_size", [2, 4, 8, 6])
def test_unpack_of_ragged_rows_by_cache_lines_of_the_written_side(elem_size):
    # rows of 256 bytes and more that are not whole 16-byte chunks are unpacked line by line of the strided side:
    # rows that start anywhere inside a line, rows of exactly 2 KiB, three and four dimensions, shifted staging,
    # rows just above and below 256 bytes, rows that end one element into a line
    cases = [Slice(offset=3, sizes=[5, 40, 1027], strides=[46200, 1100, 1]), Slice(offset=0, sizes=[64, 1025], strides=[1031, 1]),
             Slice(offset=509, sizes=[31, 2049], strides=[2051, 1]), Slice(offset=1, sizes=[2, 3, 5, 1301], strides=[33600, 8400, 1400, 1]),
             Slice(offset=7, sizes=[3, 9001], strides=[9002, 1]),
             Slice(offset=0, sizes=[700, 129], strides=[192, 1]), Slice(offset=5, sizes=[900, 127], strides=[131, 1]),
             Slice(offset=0, sizes=[333, 65], strides=[64 * 3, 1]), Slice(offset=63, sizes=[50, 7, 257], strides=[7 * 320, 320, 1])]
    for i, s in enumerate(cases):
        for dst_misalign in (0, elem_size, 7 * elem_size):
            _roundtrip(s, elem_size, seed=20 + i, misalign=(i % 4) * elem_size, dst_misalign=dst_misalign)
    # several views of one tensor in one launch
    g = torch.Generator().manual_seed(21)
    nbytes = elem_size
    x = torch.randint(0, 256, (40, 5000 * nbytes), dtype=torch.uint8, generator=g)
    dev = x.to(DEV)
    views = [Slice(offset=k * 1203 + 1, sizes=[40, 1201], strides=[5000, 1]) for k in range(4)]
    outs = [torch.empty(40 * 1201 * nbytes + 3, dtype=torch.uint8, device=DEV)[3:] for _ in views]
    import ctypes as C
    from monarch_amd._lib import check, lib, ptr_array
    from monarch_amd.ndslice import slice_array
    arr = slice_array(views)
    stream = torch.cuda.current_stream().cuda_stream
    check(lib().mhip_slice_pack_many(ptr_array([o.data_ptr() for o in outs]), dev.data_ptr(), arr, len(views), nbytes, stream))
    back = torch.full_like(dev, 0x3C)
    check(lib().mhip_slice_unpack_many(back.data_ptr(), ptr_array([o.data_ptr() for o in outs]), arr, len(views), nbytes, stream))
    sync()
    want = torch.full_like(x, 0x3C)
    for v in views:
        want[:, (v.offset) * nbytes: (v.offset + 1201) * nbytes] = x[:, v.offset * nbytes: (v.offset + 1201) * nbytes]
    assert torch.equal(back.cpu(), want)
    # the same with a pitch of whole cache lines: every view's rows then sit at one place in their lines, each view
    # at its own, and the number of lines a row overlaps differs between the views of the launch
    x = torch.randint(0, 256, (40, 4096 * nbytes), dtype=torch.uint8, generator=g)
    dev = x.to(DEV)
    views = [Slice(offset=k * 1201, sizes=[40, 1201], strides=[4096, 1]) for k in range(3)]
    arr = slice_array(views)
    check(lib().mhip_slice_pack_many(ptr_array([o.data_ptr() for o in outs]), dev.data_ptr(), arr, len(views), nbytes, stream))
    back = torch.full_like(dev, 0x3C)
    check(lib().mhip_slice_unpack_many(back.data_ptr(), ptr_array([o.data_ptr() for o in outs]), arr, len(views), nbytes, stream))
    sync()
    want = torch.full_like(x, 0x3C)
    want[:, :3 * 1201 * nbytes] = x[:, :3 * 1201 * nbytes]
    assert torch.equal(back.cpu(), want)


def test_wide_index_unpack_of_long_ragged_rows():
    # more than 2^31 two-byte units in rows of 32767 at a pitch of 32769: 64-bit decode in the piecewise unpack
    _check_large_view(torch.int16, [65600, 32767], [32769, 1], offset=1)


@pytest.mark.parametrize("elem_size", [1, 2, 4, 8, 6])
def test_runs_shorter_than_a_chunk(elem_size):
    # element-strided selections and rows of a few bytes: packed chunks are gathered / scattered unit by
    # unit, with the unit addresses stepped by an odometer that re-decodes when the inner dimension wraps
    cases = [Slice(offset=0, sizes=[500, 333], strides=[700, 2]),              # x[:, ::2]
             Slice(offset=3, sizes=[5, 7, 9], strides=[7 * 9 * 4 * 2, 9 * 4, 4]),
             Slice(offset=1, sizes=[4000, 3], strides=[5, 1]),                  # rows of 3 elements
             Slice(offset=0, sizes=[3, 2, 50, 2], strides=[2 * 50 * 8 * 2, 50 * 8, 8, 4]),
             Slice(offset=2, sizes=[20000], strides=[3]),
             Slice(offset=0, sizes=[9, 100, 5], strides=[5, 45 * 2, 1])]          # non-monotone strides, short runs
    for i, s in enumerate(cases):
        for dst_misalign in (0, 3 * elem_size):
            _roundtrip(s, elem_size, seed=40 + i, misalign=(i % 2) * elem_size, dst_misalign=dst_misalign)


def test_maximum_number_of_dimensions():
    # 32 dimensions (the library's limit): fourteen of size 2 that cannot merge, the rest of size 1
    sizes, strides, acc = [], [], 1
    for k in range(32):
        if k % 2 == 0 and len([z for z in sizes if z == 2]) < 14:
            sizes.append(2)
            strides.append(acc)
            acc *= 3
        else:
            sizes.append(1)
            strides.append(acc)
    s = Slice(offset=2, sizes=list(reversed(sizes)), strides=list(reversed(strides)))
    assert s.ndim == 32 and len(s) == 2**14
    _roundtrip(s, 2, seed=8)
    _roundtrip(s, 16, seed=9)
    with pytest.raises(ValueError, match="InvalidArgument"):
        Slice(offset=0, sizes=[1] * 33, strides=[1] * 33)


def test_many_dims_peels_on_host():
    # 10 dims that cannot merge (every stride leaves a gap): more than the kernel decodes at once
    sizes = [2] * 10
    strides, acc = [], 1
    for _ in sizes:
        strides.append(acc)
        acc *= 3
    s = Slice(offset=1, sizes=sizes, strides=list(reversed(strides)))
    _roundtrip(s, 4, seed=5)
    # and the same with the dims in scrambled (non-monotone stride) order
    perm = [3, 0, 7, 1, 9, 2, 8, 4, 6, 5]
    s = Slice(offset=0, sizes=[sizes[p] for p in perm], strides=[list(reversed(strides))[p] for p in perm])
    _roundtrip(s, 2, seed=6)


def test_config1_f32_every_other_row():
    # fp32 [4,256,256], view {0,[4,128,256],[65536,512,1]}: pack, unpack back
    rng = np.random.default_rng(1000)
    x = rng.uniform(-1, 1, size=(4, 256, 256)).astype(np.float32)
    s = Slice(offset=0, sizes=[4, 128, 256], strides=[65536, 512, 1])
    dev = torch.from_numpy(x).to(DEV)
    packed = staging.pack(dev, s)
    sync()
    want = oracle.pack(x.reshape(-1), oslice(s))
    assert np.array_equal(packed.cpu().numpy(), want)
    assert np.array_equal(want.reshape(4, 128, 256), x[:, ::2, :])  # the view itself
    back = torch.zeros_like(dev)
    staging.unpack(back, s, packed)
    sync()
    ref = np.zeros_like(x)
    ref[:, ::2, :] = x[:, ::2, :]
    assert np.array_equal(back.cpu().numpy(), ref)


def test_config3_column_blocks_full_size():
    # bf16 [4096,14336]; 8 views {k*1792,[4096,1792],[14336,1]} -> 8 send buffers -> zeroed tensor
    g = torch.Generator(device=DEV).manual_seed(3000)
    w = (torch.randn(4096, 14336, generator=g, device=DEV) * 0.02).bfloat16()
    views = [Slice(offset=k * 1792, sizes=[4096, 1792], strides=[14336, 1]) for k in range(8)]
    bufs = staging.pack_many(w, views)
    sync()
    hw = bits(w).reshape(-1)
    for k in (0, 3, 7):
        want = oracle.pack(hw, oslice(views[k]), runs=True)
        assert np.array_equal(bits(bufs[k]), want)
    for k in range(8):  # every buffer equals the column block
        assert torch.equal(bufs[k].view(4096, 1792), w[:, k * 1792:(k + 1) * 1792])
    back = torch.zeros_like(w)
    staging.unpack_many(back, views, bufs)
    sync()
    assert torch.equal(back.view(torch.int16), w.view(torch.int16))  # the 8 views tile the tensor
    # single-view entry point gives the same bytes
    one = staging.pack(w, views[5])
    sync()
    assert torch.equal(one.view(torch.int16), bufs[5].view(torch.int16))


def test_contiguous_pack_is_memcmp():
    g = torch.Generator(device=DEV).manual_seed(2001)
    x = (torch.randn(25_165_824, generator=g, device=DEV) * 0.02).bfloat16()
    s = Slice.new_row_major([x.numel()])
    out = staging.pack(x, s)
    sync()
    assert torch.equal(out.view(torch.int16), x.view(torch.int16))
    back = torch.empty_like(x)
    staging.unpack(back, s, out)
    sync()
    assert torch.equal(back.view(torch.int16), x.view(torch.int16))


def test_transposed_matrix():
    g = torch.Generator().manual_seed(7)
    x = torch.randint(-2**31, 2**31 - 1, (257, 515), dtype=torch.int32, generator=g)
    dev = x.to(DEV)
    s = Slice(offset=0, sizes=[515, 257], strides=[1, 515])  # iterate columns: packs x.T
    out = staging.pack(dev, s)
    sync()
    assert np.array_equal(out.cpu().numpy(), x.numpy().T.reshape(-1))
    assert np.array_equal(out.cpu().numpy(), oracle.pack(x.numpy().reshape(-1), oslice(s)))


def test_pack_many_mixed_views_and_alignment():
    g = torch.Generator().manual_seed(8)
    x = torch.randint(0, 2**15, (64, 96), dtype=torch.int16, generator=g)
    dev = x.to(DEV)
    views = [Slice(offset=0, sizes=[64, 32], strides=[96, 1]), Slice(offset=32, sizes=[64, 32], strides=[96, 1]),
             Slice(offset=64, sizes=[64, 31], strides=[96, 1]), Slice(offset=95, sizes=[64], strides=[96]),
             Slice(offset=0, sizes=[0], strides=[1])]
    store = torch.zeros(64 * 96 + 64, dtype=torch.int16, device=DEV)
    outs, pos = [], 0
    for i, v in enumerate(views):
        pos += i  # staggers the staging alignment
        outs.append(store[pos: pos + len(v)])
        pos += len(v)
    staging.pack_many(dev, views, outs)
    sync()
    for v, o in zip(views, outs):
        assert np.array_equal(o.cpu().numpy(), oracle.pack(x.numpy().reshape(-1), oslice(v)))
    back = torch.zeros_like(dev)
    staging.unpack_many(back, views, outs)
    sync()
    assert torch.equal(back, dev)


def test_wide_index_path_over_2g_units():
    # more than 2^31 one-byte units (odd addresses force unit = 1): exercises 64-bit decode
    n = 2**31 + 4096 + 2
    src = torch.empty(n + 2, dtype=torch.uint8, device=DEV)
    src.view(torch.int16)[:] = torch.arange((n + 2) // 2, device=DEV, dtype=torch.int32).to(torch.int16)
    dst = torch.zeros(n + 2, dtype=torch.uint8, device=DEV)
    s = Slice(offset=0, sizes=[n], strides=[1])
    import ctypes as C
    from monarch_amd._lib import check, lib
    check(lib().mhip_slice_pack(dst.data_ptr() + 1, src.data_ptr() + 1, C.byref(s.c), 1,
                                torch.cuda.current_stream().cuda_stream))
    sync()
    assert dst[0].item() == 0 and dst[n + 1].item() == 0
    assert torch.equal(dst[1: n + 1], src[1: n + 1])


def _check_large_view(dtype, sizes, strides, offset=0, min_bytes=2**31):
    """pack against torch's own strided gather on the GPU (the CPU walk would take minutes at this size),
    then unpack into zeros: the view comes back and nothing else is written."""
    s = Slice(offset=offset, sizes=sizes, strides=strides)
    _, hi = s.bounds()
    es = torch.empty(0, dtype=dtype).element_size()
    src = torch.empty(hi + 1, dtype=dtype, device=DEV)
    raw = src.view(torch.uint8)
    step = 1 << 28
    for i in range(0, raw.numel(), step):  # a pattern with no short period
        k = torch.arange(i, min(i + step, raw.numel()), device=DEV, dtype=torch.int64)
        raw[i:i + step] = ((k * 2654435761) >> 13).to(torch.uint8)
        del k
    want = torch.as_strided(src, sizes, strides, offset).contiguous().reshape(-1)
    got = staging.pack(src, s)
    sync()
    assert got.numel() * es >= min_bytes
    assert torch.equal(got.view(torch.uint8), want.view(torch.uint8))
    del want
    back = torch.zeros_like(src)
    staging.unpack(back, s, got)
    sync()
    view = torch.as_strided(back, sizes, strides, offset)
    assert torch.equal(view.contiguous().reshape(-1).view(torch.uint8), got.view(torch.uint8))
    # every byte outside the view is still zero: the non-zero count of the whole equals that of the view
    assert int(torch.count_nonzero(back.view(torch.uint8))) == int(torch.count_nonzero(got.view(torch.uint8)))


def test_wide_index_rows_that_are_not_whole_chunks():
    # 2^31 + 2^19 one-byte units in rows of 65535 at a pitch of 65537: 64-bit decode in the two-vector form
    _check_large_view(torch.uint8, [32776, 65535], [65537, 1], offset=3)


def test_wide_index_short_runs():
    # more than 2^31 one-byte units in runs of 3 of 5: 64-bit decode in the gathering form
    _check_large_view(torch.uint8, [716_000_000, 3], [5, 1], offset=1)


def test_wide_index_whole_chunks():
    # more than 2^31 two-byte units in rows of 4096 bf16 at an odd pitch: 64-bit decode in the whole-chunk form
    _check_large_view(torch.bfloat16, [524_296, 4096], [4097, 1])


@pytest.mark.parametrize("c0,cols", [(0, 7168), (8, 7168), (0, 7160), (1, 7168), (3, 7163)])
def test_single_view_unpacks_of_96_mib_and_more(c0, cols):
    # from 96 MiB on, an unpack of one view streams its stores and, where its rows do not start and end on cache
    # lines, gives each XCD a contiguous share of the pieces: whole-line rows, rows 16 bytes into a line, rows of
    # 14320 bytes, rows at a 2-byte offset (whole chunks) and ragged rows
    _check_large_view(torch.bfloat16, [8192, cols], [14336, 1], offset=c0, min_bytes=96 << 20)


def test_tensor_buffer_round_trip():
    # the RDMABuffer contract: 1-D contiguous uint8 only; TensorBuffer stages a strided view through it
    g = torch.Generator().manual_seed(9)
    x = torch.randn(10, 10, generator=g).to(DEV)
    view = x[2:8, 1:9:2]
    tb = staging.TensorBuffer(view)
    buf = tb.stage()
    remote = torch.zeros(buf.size, dtype=torch.uint8, device=DEV)
    buf.read_into(remote)
    y = torch.zeros(10, 10, device=DEV)
    tb2 = staging.TensorBuffer(y[2:8, 1:9:2])
    tb2.buffer.write_from(remote)
    tb2.commit()
    sync()
    ref = torch.zeros(10, 10)
    ref[2:8, 1:9:2] = x.cpu()[2:8, 1:9:2]
    assert torch.equal(y.cpu(), ref)
    with pytest.raises(ValueError, match="Tensor must be 1D"):
        staging.RDMABuffer(x)
    with pytest.raises(ValueError, match="Tensor must be uint8"):
        staging.RDMABuffer(x.flatten())
    with pytest.raises(ValueError, match="must be <="):
        buf.read_into(torch.zeros(buf.size + 1, dtype=torch.uint8, device=DEV))


def test_rdma_buffer_transfer_in_segments():
    # a transfer longer than one work request can carry goes out as several requests (the length field of a
    # scatter/gather entry is 32 bits, rdma_components.rs:1041,1063); here with the request size lowered
    g = torch.Generator().manual_seed(3)
    host = torch.randint(0, 256, (5003,), dtype=torch.uint8, generator=g)
    src = host.to(DEV)
    for limit, nbytes, so, do in ((1008, 4000, 1001, 0), (16, 100, 3, 5), (4096, 4096, 0, 0), (0, 5003, 0, 0), (1, 37, 11, 2)):
        dst = torch.zeros(nbytes + 16, dtype=torch.uint8, device=DEV)
        posted = staging.transfer(dst.data_ptr() + do, src.data_ptr() + so, nbytes, limit)
        sync()
        assert posted == (1 if limit == 0 else -(-nbytes // limit))
        want = torch.zeros(nbytes + 16, dtype=torch.uint8)
        want[do: do + nbytes] = host[so: so + nbytes]
        assert torch.equal(dst.cpu(), want)
    buf = staging.RDMABuffer(src)
    dst = torch.zeros(4000, dtype=torch.uint8, device=DEV)
    assert buf.read_into(dst, offset=1001) == 4000
    sync()
    assert torch.equal(dst.cpu(), host[1001:5001])
    buf.write_from(torch.full((3000,), 9, dtype=torch.uint8, device=DEV), offset=7)
    sync()
    want = host.clone()
    want[7:3007] = 9
    assert torch.equal(buf.data.cpu(), want)
    # the library's own RdmaBuffer calls: local.size bytes, in the direction the name says
    import ctypes as C
    from monarch_amd._lib import RdmaBufferC, lib
    a = torch.arange(64, dtype=torch.uint8, device=DEV)
    b = torch.zeros(100, dtype=torch.uint8, device=DEV)
    la, rb = RdmaBufferC(a.data_ptr(), 64), RdmaBufferC(b.data_ptr(), 100)
    assert lib().mhip_buffer_read_into(C.byref(la), C.byref(rb), None) == 0        # a -> b (put)
    sync()
    assert torch.equal(b[:64].cpu(), a.cpu()) and torch.count_nonzero(b[64:]) == 0
    b[:64] = 7
    assert lib().mhip_buffer_write_from(C.byref(la), C.byref(rb), None) == 0       # b -> a (get)
    sync()
    assert torch.all(a == 7)


def test_transfer_of_many_buffers_in_one_launch():
    # the requests of several buffers in one launch: ragged lengths, every alignment of source and destination,
    # empty buffers, more requests than one launch holds (64), guard bytes around every destination
    import ctypes as C
    from monarch_amd._lib import lib
    g = torch.Generator().manual_seed(12)
    host = torch.randint(0, 256, (400_000,), dtype=torch.uint8, generator=g)
    src = host.to(DEV)
    for limit, lens in ((0, [1, 0, 15, 16, 17, 1023, 1024, 1025, 70_001, 33]), (4096, [100_000, 5, 0, 40_000, 4096, 4097]),
                        (1000, [60_000, 30_000, 7]), (0, list(range(90, 190)))):
        n = len(lens)
        so = [(7 * j) % 19 + 1000 * j for j in range(n)]
        do = [(5 * j) % 1031 for j in range(n)]
        dsts = [torch.full((l + 1100,), 0xEE, dtype=torch.uint8, device=DEV) for l in lens]
        posted = staging.transfer_many([d.data_ptr() + o for d, o in zip(dsts, do)], [src.data_ptr() + o for o in so], lens, limit)
        sync()
        assert posted == sum((1 if limit == 0 else -(-l // limit)) if l else 0 for l in lens)
        for j, (d, l) in enumerate(zip(dsts, lens)):
            got = d.cpu()
            assert torch.equal(got[do[j]: do[j] + l], host[so[j]: so[j] + l]), (limit, j)
            assert bool((got[:do[j]] == 0xEE).all()) and bool((got[do[j] + l:] == 0xEE).all()), (limit, j)
    assert lib().mhip_buffer_transfer_many(None, None, None, 0, 0, None, None) == 0
    one = (C.c_void_p * 1)(src.data_ptr())
    null = (C.c_void_p * 1)(None)
    assert lib().mhip_buffer_transfer_many(null, one, (C.c_size_t * 1)(8), 1, 0, None, None) == 10108  # UndefinedTensor
    assert lib().mhip_buffer_transfer_many(null, one, (C.c_size_t * 1)(0), 1, 0, None, None) == 0


def test_staging_buffers_are_validated_before_launch():
    x = torch.zeros(8, 8, device=DEV)
    s = Slice(offset=0, sizes=[8, 4], strides=[8, 1])
    with pytest.raises(ValueError, match="exactly len"):
        staging.pack(x, s, out=torch.empty(31, device=DEV))
    with pytest.raises(MhipError):
        staging.pack(x, s, out=torch.empty(32))                      # host memory
    with pytest.raises(ValueError, match="exactly len"):
        staging.pack_many(x, [s, s], outs=[torch.empty(32, device=DEV), torch.empty(16, device=DEV)])
    with pytest.raises(ValueError, match="staging buffers"):
        staging.pack_many(x, [s, s], outs=[torch.empty(32, device=DEV)])
    with pytest.raises(ValueError, match="contiguous"):
        staging.unpack(x, s, torch.empty(32, 2, device=DEV)[:, 0])


def test_config3_reshard_end_to_end():
    # to_mesh of a column-sharded weight: [4096, 14336] bf16 -> 8 column-block views -> 8 staging buffers ->
    # buffer transfer (several requests each) -> 8 receiver tensors [4096, 1792]; and back into a zeroed weight
    from monarch_amd.reduce import Factory
    from monarch_amd.send_tensor import route, stream_send_tensor
    rows, cols, k = 4096, 14336, 8
    w = cols // k
    g = torch.Generator(device=DEV).manual_seed(3000)
    x = (torch.randn(rows, cols, generator=g, device=DEV) * 0.02).bfloat16()
    views = [Slice(offset=j * w, sizes=[rows, w], strides=[cols, 1]) for j in range(k)]
    area = staging.StagingArea(k, rows * w * 2, DEV)
    bufs = [area.slot(j) for j in range(k)]
    staging.pack_many(x, views, outs=[b.view(torch.bfloat16) for b in bufs])
    recv = [torch.empty(rows, w, dtype=torch.bfloat16, device=DEV) for _ in range(k)]
    for j in range(k):
        posted = staging.transfer(recv[j].data_ptr(), bufs[j].data_ptr(), rows * w * 2, 4 << 20)
        assert posted == 4                                    # 14 MiB in requests of 4 MiB
    sync()
    hx = bits(x).reshape(-1)
    for j in (0, 3, 7):
        want = oracle.send_tensor(hx, oslice(views[j]))
        assert np.array_equal(bits(recv[j]).reshape(-1), want), j
    for j in range(k):
        assert torch.equal(recv[j], x[:, j * w:(j + 1) * w])
    # the same transfers as one launch
    recv2 = [torch.empty(rows, w, dtype=torch.bfloat16, device=DEV) for _ in range(k)]
    assert staging.transfer_many([r.data_ptr() for r in recv2], [b.data_ptr() for b in bufs], [rows * w * 2] * k) == k
    sync()
    for j in range(k):
        assert torch.equal(recv2[j], recv[j])
    back = torch.zeros_like(x)
    staging.unpack_many(back, views, [r.view(-1) for r in recv])
    sync()
    assert torch.equal(back.view(torch.int16), x.view(torch.int16))
    # the same through the SendTensor entry point, one message per destination rank
    from_ranks, to_ranks = Slice(offset=0, sizes=[1], strides=[1]), Slice(offset=5, sizes=[1], strides=[1])
    assert route(from_ranks, to_ranks, 5) == (0, None) and route(from_ranks, to_ranks, 0) == (None, 5)
    col = x[:, 5 * w: 6 * w]                                   # the sender's (non-contiguous) tensor
    got = stream_send_tensor({0: col}, 5, 0, None, Factory.of(col), staging_bytes=bufs[5])
    sync()
    assert got.is_contiguous() and np.array_equal(bits(got).reshape(-1), oracle.send_tensor(hx, oslice(views[5])))


@pytest.mark.parametrize("dtype", [torch.uint8, torch.int16, torch.int32, torch.int64, torch.complex128])
def test_transposing_views_lds_path(dtype):
    # permuted views: the memory-contiguous dimension is not the innermost iteration dimension
    g = torch.Generator().manual_seed(11)
    cases = [((70, 130), (1, 0)), ((64, 64), (1, 0)), ((5, 67, 33), (0, 2, 1)), ((5, 67, 33), (2, 1, 0)),
             ((3, 4, 40, 50), (1, 3, 0, 2)), ((9, 200), (1, 0)), ((200, 9), (1, 0)), ((2, 3, 129, 65), (3, 0, 2, 1)),
             ((33, 8, 8), (2, 1, 0))]
    for shape, perm in cases:
        n = int(np.prod(shape))
        if dtype == torch.complex128:
            host = torch.view_as_complex(torch.randn(n, 2, generator=g, dtype=torch.float64)).reshape(shape)
        else:
            info = torch.iinfo(dtype)
            host = torch.randint(info.min, info.max, shape, dtype=dtype, generator=g)
        dev = host.to(DEV)
        view = dev.permute(perm)[..., 1:] if len(shape) > 2 else dev.permute(perm)
        hview = host.permute(perm)[..., 1:] if len(shape) > 2 else host.permute(perm)
        s = Slice.of_tensor(view)
        out = staging.pack(view, s)
        sync()
        assert torch.equal(out.cpu(), hview.contiguous().flatten()), (shape, perm, dtype)
        back = torch.zeros_like(dev)
        staging.unpack(back, s, out)
        sync()
        ref = torch.zeros_like(host)
        (ref.permute(perm)[..., 1:] if len(shape) > 2 else ref.permute(perm)).copy_(hview)
        assert torch.equal(back.cpu(), ref), (shape, perm, dtype)
        if dtype in (torch.int16, torch.int32):
            hb = host.numpy().reshape(-1)
            assert np.array_equal(out.cpu().numpy(), oracle.pack(hb, oslice(s)))


@pytest.mark.parametrize("dtype", [torch.uint8, torch.int16, torch.int32, torch.int64])
def test_transposing_views_interior_and_edge_tiles(dtype):
    # large enough for whole 256-byte x 256-byte tiles at every element size, with rows that are
    # not 16-byte aligned (odd pitch, odd offset), ragged edges on both sides, and a packed-side
    # index that spans two iteration dimensions
    g = torch.Generator().manual_seed(13)
    info = torch.iinfo(dtype)
    for shape, view_of in [((523, 777), lambda t: t[3:, 5:].t()),
                           ((4, 300, 261), lambda t: t.permute(2, 0, 1)),
                           ((2, 270, 2, 259), lambda t: t.permute(0, 3, 2, 1)[:, 1:])]:
        host = torch.randint(info.min, info.max, shape, dtype=dtype, generator=g)
        dev = host.to(DEV)
        view, hview = view_of(dev), view_of(host)
        s = Slice.of_tensor(view)
        out = staging.pack(view, s)
        sync()
        assert torch.equal(out.cpu(), hview.contiguous().flatten()), (shape, dtype)
        back = torch.full_like(dev, 7)
        staging.unpack(back, s, out)
        sync()
        ref = torch.full_like(host, 7)
        view_of(ref).copy_(hview)
        assert torch.equal(back.cpu(), ref), (shape, dtype)


@pytest.mark.parametrize("dtype", [torch.uint8, torch.int16, torch.int32, torch.int64])
def test_transposes_whose_written_rows_start_inside_cache_lines(dtype):
    # written rows that start anywhere in a cache line, with the kernel the library picks for them (both kernels, forced
    # in turn, run in tests/tuning_variants.py): extents of exactly one tile, of a tile and a bit, shorter than the early start of a
    # window, batches, offsets, a packed side spanning two dimensions
    g = torch.Generator().manual_seed(18)
    info = torch.iinfo(dtype)
    t = 256 // torch.empty(0, dtype=dtype).element_size()
    cases = [((t, t + 1), lambda x: x.t()), ((t + 3, t), lambda x: x.t()), ((2 * t + 5, 3 * t + 7), lambda x: x[1:, 2:].t()),
             ((7, t + 9), lambda x: x.t()), ((t + 9, 7), lambda x: x.t()), ((3, t + 2, t + 1), lambda x: x.transpose(1, 2)),
             ((2, t + 1, 2, 300 // (t // 32 + 1) + t), lambda x: x.permute(0, 3, 2, 1)[:, 1:]), ((1100, 1031), lambda x: x[:, 5:].t())]
    for shape, view_of in cases:
        host = torch.randint(info.min, info.max, shape, dtype=dtype, generator=g)
        dev = host.to(DEV)
        view, hview = view_of(dev), view_of(host)
        s = Slice.of_tensor(view)
        out = staging.pack(view, s)
        sync()
        assert torch.equal(out.cpu(), hview.contiguous().flatten()), (shape, dtype)
        back = torch.full_like(dev, 7)
        staging.unpack(back, s, out)
        sync()
        ref = torch.full_like(host, 7)
        view_of(ref).copy_(hview)
        assert torch.equal(back.cpu(), ref), (shape, dtype)


def test_transpose_large_square():
    g = torch.Generator(device=DEV).manual_seed(12)
    x = (torch.randn(4096, 4096, generator=g, device=DEV)).bfloat16()
    s = Slice(offset=0, sizes=[4096, 4096], strides=[1, 4096])
    out = staging.pack(x, s)
    sync()
    assert torch.equal(out.view(4096, 4096).view(torch.int16), x.t().contiguous().view(torch.int16))
    back = torch.zeros_like(x)
    staging.unpack(back, s, out)
    sync()
    assert torch.equal(back.view(torch.int16), x.view(torch.int16))


def test_transpose_large_aligned_fp32_tiles():
    # 2^25 four-byte elements with 512-byte aligned rows on both sides: the 128 x 128 tile form, with a batch dimension
    g = torch.Generator(device=DEV).manual_seed(14)
    x = torch.randn(2, 4096, 4096, generator=g, device=DEV)
    view = x.transpose(1, 2)
    s = Slice.of_tensor(view)
    out = staging.pack(view, s)
    sync()
    assert torch.equal(out.view(2, 4096, 4096), view.contiguous())
    back = torch.zeros_like(x)
    staging.unpack(back, s, out)
    sync()
    assert torch.equal(back, x)


def test_transpose_large_aligned_bf16_tiles():
    # 2^25 and more two-byte elements with 512-byte aligned rows: the 256 x 128 tile form, with a batch
    # dimension and with tile counts that are not multiples of the walk's block size
    g = torch.Generator(device=DEV).manual_seed(15)
    for shape in [(2, 4096, 4096), (1, 4224, 8192 + 256), (3, 2944, 3840)]:
        x = torch.randn(*shape, generator=g, device=DEV).bfloat16()
        view = x.transpose(1, 2)
        s = Slice.of_tensor(view)
        out = staging.pack(view, s)
        sync()
        assert torch.equal(out.view(view.shape).view(torch.int16), view.contiguous().view(torch.int16)), shape
        back = torch.zeros_like(x)
        staging.unpack(back, s, out)
        sync()
        assert torch.equal(back.view(torch.int16), x.view(torch.int16)), shape


def test_transpose_large_aligned_f64_tiles():
    # 2^24 and more eight-byte elements with 512-byte aligned rows: the 64 x 64 tile form with 512 lanes (a row
    # length of 4096 or less) and with 1024 lanes, with a batch dimension
    g = torch.Generator(device=DEV).manual_seed(17)
    for shape in [(1, 4096, 4096), (2, 4096, 2048), (1, 4160, 8192 + 64)]:
        x = torch.randint(-2**62, 2**62, shape, dtype=torch.int64, generator=g, device=DEV)
        view = x.transpose(1, 2)
        s = Slice.of_tensor(view)
        out = staging.pack(view, s)
        sync()
        assert torch.equal(out.view(view.shape), view.contiguous()), shape
        back = torch.zeros_like(x)
        staging.unpack(back, s, out)
        sync()
        assert torch.equal(back, x), shape
        del x, view, out, back


def test_transpose_bf16_matrices_of_120_mib_and_more_with_rows_16_kib_apart():
    # the 256 x 256 tile form of two-byte elements, with and without a batch dimension and with more rows than columns
    g = torch.Generator(device=DEV).manual_seed(16)
    for shape in [(1, 8192, 8192), (2, 8192, 8192), (1, 16384, 8192)]:
        x = torch.randint(-32768, 32767, shape, dtype=torch.int16, generator=g, device=DEV)
        view = x.transpose(1, 2)
        s = Slice.of_tensor(view)
        out = staging.pack(view, s)
        sync()
        assert torch.equal(out.view(view.shape), view.contiguous()), shape
        back = torch.zeros_like(x)
        staging.unpack(back, s, out)
        sync()
        assert torch.equal(back, x), shape
        del x, view, out, back


@pytest.mark.parametrize("dtype", [torch.uint8, torch.int16, torch.float32, torch.float64])
def test_transposes_whose_rows_are_a_multiple_of_8k_apart(dtype):
    # at these pitches the tile walk is rotated per eighth of the tiles; shapes with ragged edges, batches,
    # fewer and more c-groups than eight, and eighths that end in the middle of a row of groups
    es = torch.empty(0, dtype=dtype).element_size()
    g = torch.Generator(device=DEV).manual_seed(16)
    for batch, rows, pitch_bytes in [(1, 1000, 8192), (3, 700, 8192), (1, 2100, 16384), (5, 300, 24576), (2, 515, 32768),
                                     (1, 4100, 8192), (7, 129, 16384)]:
        cols = pitch_bytes // es
        x = torch.randint(0, 255, (batch, rows, cols), dtype=torch.uint8, generator=g, device=DEV).to(dtype) \
            if dtype != torch.uint8 else torch.randint(0, 255, (batch, rows, cols), dtype=torch.uint8, generator=g, device=DEV)
        if dtype.is_floating_point:
            x = x * 1.5 - 100
        for view in (x.transpose(1, 2), x.transpose(1, 2)[:, 3:, 1:]):
            s = Slice.of_tensor(view)
            out = staging.pack(view, s)
            sync()
            assert torch.equal(out.view(view.shape), view.contiguous()), (dtype, batch, rows, pitch_bytes)
            back = torch.zeros_like(x)
            staging.unpack(back, s, out)
            sync()
            want = torch.zeros_like(x)
            want.transpose(1, 2)[:, view.shape[1] * -1:, view.shape[2] * -1:] = view
            assert torch.equal(back, want), (dtype, batch, rows, pitch_bytes)


def test_stream_send_tensor_semantics():
    from monarch_amd.reduce import Factory
    from monarch_amd.send_tensor import route, stream_send_tensor
    g = torch.Generator().manual_seed(21)
    base = torch.randn(6, 10, generator=g).to(DEV)
    view = base.t()[1:9:2]                      # non-contiguous sender tensor, shape [4, 6]
    world = {0: view, 1: None, 2: torch.ones(4, 6, device=DEV)}
    f = Factory.of(view)
    got = stream_send_tensor(world, 3, from_rank=0, to_rank=None, factory=f)    # receiver
    sync()
    assert got.is_contiguous() and torch.equal(got, view) and got.data_ptr() != base.data_ptr()
    assert stream_send_tensor(world, 0, from_rank=None, to_rank=3, factory=f) is None   # pure sender
    local = stream_send_tensor(world, 2, from_rank=2, to_rank=2, factory=f)     # defensive copy
    sync()
    assert torch.equal(local, world[2]) and local.data_ptr() != world[2].data_ptr()
    zeros = stream_send_tensor(world, 3, from_rank=1, to_rank=None, factory=f)  # errored input -> zeros
    assert torch.count_nonzero(zeros) == 0 and zeros.shape == (4, 6)
    with pytest.raises(ValueError, match="without a to/from rank"):
        stream_send_tensor(world, 0, None, None, f)
    fr, to = Slice(offset=0, sizes=[2], strides=[1]), Slice(offset=2, sizes=[2], strides=[1])
    assert route(fr, to, 3) == (1, None)
