"""Helpers shared by the GPU parity tests."""
import random

import numpy as np
import torch

from monarch_amd import Slice
from oracle import OSlice


def bits(t: torch.Tensor) -> np.ndarray:
    """Host numpy array with the tensor's raw element bits (bf16 -> uint16)."""
    t = t.detach().cpu().contiguous()
    if t.dtype == torch.bfloat16:
        return t.view(torch.uint16).numpy()
    if t.dtype == torch.float16:
        return t.view(torch.uint16).numpy()
    return t.numpy()


def oslice(s: Slice) -> OSlice:
    return OSlice.unchecked(s.offset, s.sizes, s.strides)


def span(s) -> int:
    """Number of storage elements a slice needs."""
    if any(z == 0 for z in s.sizes):
        return s.offset + 1
    return s.offset + sum((z - 1) * st for z, st in zip(s.sizes, s.strides)) + 1


def fuzz_slices(n, seed, max_size=10, max_offset=10000):
    """The generator of python/tests/_monarch/test_ndslice.py:143-167 (rejection sampling)."""
    gen = random.Random(seed)
    out = []
    while len(out) < n:
        ndim = gen.choices([1, 2, 3, 4], [1, 2, 3, 4])[0]
        sizes = [gen.randrange(1, max_size) for _ in range(ndim)]
        strides, run = [], 1
        for j in range(ndim):
            run *= gen.randrange(1 if j == 0 else 2, 4)
            strides.append(run)
        order = list(range(ndim))
        gen.shuffle(order)
        try:
            out.append(Slice(offset=gen.randrange(max_offset), sizes=[sizes[o] for o in order],
                             strides=[strides[o] for o in order]))
        except ValueError:
            continue
    return out


def valid_slices(n, seed, max_size=40, max_len=150_000, max_offset=1000):
    """Random slices that are valid by construction: each stride is the extent of the dimension below it
    times a random gap factor, a unit innermost stride two times out of three, dimensions in random order.
    (The reference's rejection sampler above rarely accepts anything beyond one short dimension.)"""
    gen = random.Random(seed)
    out = []
    while len(out) < n:
        ndim = gen.choice([1, 2, 2, 3, 3, 4])
        sizes = [gen.randrange(1, max_size) for _ in range(ndim)]
        total = 1
        for z in sizes:
            total *= z
        if total > max_len:
            continue
        strides, stride = [], gen.choice([1, 1, 2, 3])
        for z in sizes:
            strides.append(stride)
            stride = stride * z * gen.choice([1, 1, 2]) if z > 1 else stride * gen.choice([1, 2])
        order = list(range(ndim))
        if gen.random() < 0.5:
            gen.shuffle(order)
        else:
            order.reverse()  # row-major: innermost stride last
        out.append(Slice(offset=gen.randrange(max_offset), sizes=[sizes[o] for o in order],
                         strides=[strides[o] for o in order]))
    return out


def sync():
    torch.cuda.synchronize()
