"""Writes the binary golden fixtures of this directory.  Run in the build container:

    python tests/golden/make_fixtures.py

Needs only the standard library, numpy and torch's CPU casts; it imports neither the
oracle nor the product, so the files it writes are an independent statement of the answers.

e4m3fn_from_bf16_scale1.bin
    65 536 bytes: entry h is the e4m3fn code of the bf16 value with bit pattern h under the
    block codec at scale 1 (absmax 448): clamp to [-448, 448], then round to nearest even.
    NaN inputs give the NaN code with the input's sign (0x7F / 0xFF).  Finite values and
    clamping come from ``torch.clamp`` + torch's ``float8_e4m3fn`` CPU cast.

ndslice_fuzz_slices.json, ndslice_fuzz_locations.bin
    The 1000 slices that the fuzz generator of python/tests/_monarch/test_ndslice.py:143-167
    yields from ``random.Random(0)`` (rejection sampling on ``Slice::new``'s rules,
    ndslice/src/slice.rs:99-139), and for each the memory locations in iteration order
    (little-endian uint32, concatenated; ``first`` and ``count`` in the JSON index into it).
    Locations come from ``torch.as_strided`` over an ``arange`` storage, the
    (size, stride, storage_offset) model of python/monarch/common/function_caching.py:50-63.
"""
import json
import os
import random

import numpy as np
import torch

HERE = os.path.dirname(os.path.abspath(__file__))


def e4m3fn_table() -> np.ndarray:
    h = torch.arange(65536, dtype=torch.int32).to(torch.uint16)
    x = h.view(torch.bfloat16).float()
    codes = x.clamp(-448.0, 448.0).to(torch.float8_e4m3fn).view(torch.uint8).numpy().copy()
    nan = torch.isnan(x).numpy()
    sign = ((h.numpy().astype(np.uint16) >> 8) & 0x80).astype(np.uint8)
    codes[nan] = sign[nan] | 0x7F
    return codes


def slice_is_valid(sizes, strides) -> bool:
    """Slice::new's acceptance rule: sort the (stride, size) pairs; every stride must be a multiple of the one
    before it, equal strides need a size of 1 among the two, and a stride must cover the extent
    (stride * size) of the dimension before it."""
    pairs = sorted(zip(strides, sizes))
    prev_stride, prev_size = 1, 1
    for stride, size in pairs:
        if stride % prev_stride != 0:
            return False
        if stride == prev_stride and size != 1 and prev_size != 1:
            return False
        if stride < prev_stride * prev_size:
            return False
        prev_stride, prev_size = stride, size
    return True


def fuzz(gen: random.Random):
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
        sizes, strides = [sizes[o] for o in order], [strides[o] for o in order]
        if slice_is_valid(sizes, strides):
            return offset, sizes, strides


def main() -> None:
    table = e4m3fn_table()
    assert table.size == 65536 and table.dtype == np.uint8
    table.tofile(os.path.join(HERE, "e4m3fn_from_bf16_scale1.bin"))

    gen = random.Random(0)
    entries, chunks, first = [], [], 0
    for _ in range(1000):
        offset, sizes, strides = fuzz(gen)
        span = offset + sum((z - 1) * st for z, st in zip(sizes, strides)) + 1
        locs = torch.as_strided(torch.arange(span, dtype=torch.int64), sizes, strides, offset).reshape(-1)
        locs = locs.numpy().astype("<u4")
        entries.append({"offset": offset, "sizes": sizes, "strides": strides, "first": first, "count": int(locs.size)})
        chunks.append(locs)
        first += int(locs.size)
    np.concatenate(chunks).tofile(os.path.join(HERE, "ndslice_fuzz_locations.bin"))
    with open(os.path.join(HERE, "ndslice_fuzz_slices.json"), "w") as f:
        json.dump({"src": "python/tests/_monarch/test_ndslice.py:143-167, random.Random(0), 1000 draws",
                   "total_locations": first, "slices": entries}, f, separators=(",", ":"))
        f.write("\n")
    print(f"wrote e4m3fn table (65536 codes), {len(entries)} slices, {first} locations")


if __name__ == "__main__":
    main()
