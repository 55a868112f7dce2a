"""The transposing kernel's variants, each forced in turn: tile walks, cache policies, line-aligned windows on and off.

The library picks one variant per shape by itself and reads no environment variable after it has been loaded unless
MONARCH_HIP_TUNING=1 was set at load time.  This file therefore runs in a child process that sets the switch
(tests/test_gpu_tuning_variants.py starts it); pytest does not collect it by name.  Every variant must move the same bytes.
"""
import os

import pytest
import torch

from monarch_amd import Slice, staging
from util import sync

pytestmark = pytest.mark.gpu
DEV = "cuda:0"


def test_the_switch_is_on():
    assert os.environ.get("MONARCH_HIP_TUNING") == "1", "run through tests/test_gpu_tuning_variants.py"


@pytest.mark.parametrize("lines", ["0", "1", "2"])
@pytest.mark.parametrize("dtype", [torch.uint8, torch.int16, torch.int32, torch.int64])
def test_transposes_with_line_aligned_windows_and_without(dtype, lines, monkeypatch):
    # written rows that start anywhere in a cache line, through the kernel whose windows start on lines and through
    # the fixed-position tiles: extents of exactly one tile, of a tile and a bit, shorter than the early start of a
    # window, batches, offsets, a packed side spanning two dimensions
    monkeypatch.setenv("MONARCH_HIP_TRANSPOSE_LINES", lines)
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


@pytest.mark.parametrize("walk", ["0,1,4,0", "0,1,4,1", "0,1,16,1", "0,0,8,0", "1,0", "1,1", "2,0", "2,1", "3,0", "3,1"])
def test_every_tile_walk_of_the_transposing_kernel_moves_the_same_bytes(walk, monkeypatch):
    # the library picks one walk per shape; every walk it can pick (and the variants the A/B sweep forces) must give the
    # same bytes: whole and partial tiles, batches, a tile count that is no multiple of 8, pitches that are and are not
    # multiples of 4 KiB
    monkeypatch.setenv("MONARCH_HIP_TRANSPOSE_WALK", walk)
    g = torch.Generator().manual_seed(sum(walk.encode()))
    cases = [(torch.int16, (1, 256, 384, 384)), (torch.int16, (3, 200, 333, 340)), (torch.int32, (1, 192, 64, 64)),
             (torch.int32, (2, 130, 257, 300)), (torch.uint8, (1, 512, 768, 768)), (torch.uint8, (2, 300, 515, 600)),
             (torch.int64, (1, 96, 160, 160)), (torch.int32, (1, 1024, 2048, 2048)), (torch.int16, (1, 2048, 1024, 2048))]
    for dtype, (b, r, c, pitch) in cases:
        info = torch.iinfo(dtype)
        host = torch.randint(info.min, info.max, (b, r, pitch), dtype=dtype, generator=g)
        dev = host.to(DEV)
        view, hview = dev[:, :, :c].transpose(1, 2), host[:, :, :c].transpose(1, 2)
        s = Slice.of_tensor(view)
        out = staging.pack(view, s)
        sync()
        assert torch.equal(out.cpu(), hview.contiguous().flatten()), (walk, dtype, b, r, c, pitch)
        back = torch.zeros_like(dev)
        staging.unpack(back, s, out)
        sync()
        ref = torch.zeros_like(host)
        ref[:, :, :c] = host[:, :, :c]
        assert torch.equal(back.cpu(), ref), (walk, dtype, b, r, c, pitch)


@pytest.mark.parametrize("policy", ["0", "1", "2", "3"])
def test_every_cache_policy_of_the_transposing_kernel_moves_the_same_bytes(policy, monkeypatch):
    # cached / write-through / streaming loads and stores, forced on aligned and unaligned rows alike (the library only
    # streams aligned rows; correctness must not depend on that)
    monkeypatch.setenv("MONARCH_HIP_TRANSPOSE_POLICY", policy)
    g = torch.Generator().manual_seed(40 + int(policy))
    cases = [(torch.int32, (1, 523, 772, 777)), (torch.int16, (2, 300, 515, 600)), (torch.uint8, (1, 512, 768, 768)),
             (torch.int64, (1, 96, 160, 160)), (torch.int32, (1, 1024, 2048, 2048)), (torch.int16, (1, 515, 260, 261))]
    for dtype, (b, r, c, pitch) in cases:
        info = torch.iinfo(dtype)
        host = torch.randint(info.min, info.max, (b, r, pitch), dtype=dtype, generator=g)
        dev = host.to(DEV)
        view, hview = dev[:, :, :c].transpose(1, 2), host[:, :, :c].transpose(1, 2)
        s = Slice.of_tensor(view)
        for rep in range(3):
            out = staging.pack(view, s)
            sync()
            assert torch.equal(out.cpu(), hview.contiguous().flatten()), (policy, dtype, b, r, c, pitch, rep)
        back = torch.zeros_like(dev)
        staging.unpack(back, s, out)
        sync()
        ref = torch.zeros_like(host)
        ref[:, :, :c] = host[:, :, :c]
        assert torch.equal(back.cpu(), ref), (policy, dtype, b, r, c, pitch)


@pytest.mark.parametrize("blocks", ["1", "4"])
def test_fused_quantiser_with_one_and_four_blocks_per_wavefront_step(blocks, monkeypatch):
    # the library runs one block per step on buckets of up to 32768 blocks and four beyond; both forms, forced in turn
    # on ragged buckets whose spans straddle one and several tensors, must equal flat pack + quantise bit for bit
    import numpy as np
    from monarch_amd import fp8
    monkeypatch.setenv("MONARCH_HIP_BUCKET_BLOCKS", blocks)
    g = torch.Generator().manual_seed(90 + int(blocks))
    for sizes in ([5000, 1, 1024, 777, 30000, 2049, 0, 4096, 4097, 13], [200000], [3] * 700, [1023, 1025, 4095, 4097, 8191, 16385]):
        tensors = [torch.randn(k, generator=g).bfloat16().to(DEV) for k in sizes]
        if tensors[0].numel() > 10:
            tensors[0][7] = float("inf")
            tensors[0][9] = float("nan")
        bucket = fp8.FlatBucket(tensors)
        q_ref, s_ref = fp8.quantize(bucket.pack())
        for indexed in (True, False):
            q, s = fp8.quantize_bucket(bucket, indexed=indexed)
            sync()
            assert torch.equal(q, q_ref) and torch.equal(s.view(torch.int32), s_ref.view(torch.int32)), (blocks, sizes[:4], indexed)


def test_random_transposing_views_through_every_form_of_the_kernels():
    # seeded random shapes around the tile sizes (extents of a tile minus one, a tile, a tile and a bit, halves, tiny ones,
    # batches, views that start inside the matrix, pitches that put no written row on a cache line), each through a
    # form drawn at random: the library's choice, fixed tiles, per-tile windows, strips with segments of 1, 2 and 4 chunks
    import ctypes as C
    import random
    libc = C.CDLL(None)
    gen = random.Random(2718)
    forms = [None, "0", "1", "2", "2,1", "2,4"]
    try:
        for n in range(600):
            dtype = gen.choice([torch.uint8, torch.uint8, torch.int16, torch.int16, torch.int32, torch.int64])
            t = 256 // torch.empty(0, dtype=dtype).element_size()

            def extent():
                if gen.random() < 0.4:
                    return gen.choice([t - 1, t, t + 1, 2 * t - 1, 2 * t, 2 * t + 1, 3 * t + 5, t // 2, t // 2 + 1, 7, 1])
                return int(2 ** gen.uniform(0, 10.5))
            b, rows, cols = gen.choice([1, 1, 1, 2, 3]), extent(), extent()
            pitch = cols + gen.choice([0, 0, 1, 3, 8, 64, 65])
            r0, c0 = gen.choice([0, 0, 1, 5]), gen.choice([0, 0, 1, 2, 7])
            if rows <= r0 or cols <= c0:
                continue
            form = gen.choice(forms)
            if form is None:
                libc.unsetenv(b"MONARCH_HIP_TRANSPOSE_LINES")
            else:
                libc.setenv(b"MONARCH_HIP_TRANSPOSE_LINES", form.encode(), 1)
            info = torch.iinfo(dtype)
            host = torch.randint(info.min, info.max, (b, rows, pitch), dtype=dtype)
            dev = host.to(DEV)
            view, hview = dev[:, r0:, c0:cols].transpose(1, 2), host[:, r0:, c0:cols].transpose(1, 2)
            s = Slice.of_tensor(view)
            out = staging.pack(view, s)
            sync()
            assert torch.equal(out.cpu(), hview.contiguous().flatten()), (n, dtype, b, rows, cols, pitch, r0, c0, form)
            back = torch.full_like(dev, 7)
            staging.unpack(back, s, out)
            sync()
            ref = torch.full_like(host, 7)
            ref[:, r0:, c0:cols] = host[:, r0:, c0:cols]
            assert torch.equal(back.cpu(), ref), (n, dtype, b, rows, cols, pitch, r0, c0, form)
    finally:
        libc.unsetenv(b"MONARCH_HIP_TRANSPOSE_LINES")
