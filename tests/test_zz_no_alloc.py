"""The allocation-free entry point mhip_fp8_quantize_bucket_static against mhip_fp8_quantize_bucket, through the
C ABI: same codes and scales bit for bit, on two calls in a row of which the second has the smaller input (the
static index then still holds entries of the first call beyond what the second one rewrites)."""
import ctypes as C

import numpy as np
import pytest
import torch

from monarch_amd import _lib

pytestmark = pytest.mark.gpu
DEV = "cuda:0"


def _bucket(sizes, seed):
    g = torch.Generator().manual_seed(seed)
    total = sum(sizes)
    x = torch.randn(total, generator=g)
    x = torch.where(torch.rand(total, generator=g) < 1e-3, x * 50, x).bfloat16()
    x[total // 3] = float("nan")
    offs = np.concatenate([[0], np.cumsum(sizes)]).astype(np.int64)
    dx = x.to(DEV)
    tensors = [dx[offs[i]: offs[i + 1]].clone() for i in range(len(sizes))]
    d_ptrs = torch.tensor([t.data_ptr() for t in tensors], dtype=torch.int64, device=DEV)
    d_offs = torch.from_numpy(offs).to(DEV)
    return tensors, d_ptrs, d_offs, total


def _both(lib, sizes, seed):
    tensors, d_ptrs, d_offs, total = _bucket(sizes, seed)
    nblk = (total + 1023) // 1024
    out = []
    for name in ("mhip_fp8_quantize_bucket", "mhip_fp8_quantize_bucket_static"):
        q = torch.full((total + 64,), 0xAB, dtype=torch.uint8, device=DEV)        # guard bytes behind the payload
        s = torch.full((nblk + 4,), -1.0, dtype=torch.float32, device=DEV)
        stream = torch.cuda.current_stream().cuda_stream
        if name.endswith("_static"):
            rc = lib.mhip_fp8_quantize_bucket_static(q.data_ptr(), s.data_ptr(), d_ptrs.data_ptr(), d_offs.data_ptr(),
                                                     len(sizes), total, 1024, stream)
        else:
            rc = lib.mhip_fp8_quantize_bucket(q.data_ptr(), s.data_ptr(), d_ptrs.data_ptr(), d_offs.data_ptr(), len(sizes),
                                              total, 1024, None, stream)
        assert rc == 0, (name, rc)
        torch.cuda.synchronize()
        out.append((q.cpu().numpy(), s.cpu().numpy().view(np.uint32)))
    (q0, s0), (q1, s1) = out
    assert np.array_equal(q0, q1) and np.array_equal(s0, s1)
    assert np.all(q1[total:] == 0xAB) and np.all(s1[nblk:] == np.float32(-1.0).view(np.uint32))
    return total


def test_static_index_entry_point_matches_on_two_calls_in_a_row():
    lib = _lib.lib()
    g = torch.Generator().manual_seed(7)
    large = torch.randint(1, 40000, (300,), generator=g).tolist() + [0, 5, 1024, 3]
    small = [700, 1, 2048, 333, 0, 9000]
    t1 = _both(lib, large, 1)
    t2 = _both(lib, small, 2)          # fewer blocks than the call before: the index is rebuilt, not reused
    assert t2 < t1
    _both(lib, large[:50], 3)


def test_static_index_entry_point_refuses_what_does_not_fit():
    lib = _lib.lib()
    limit = ((1 << 20) - 1) * 1024
    # refused before anything is launched or dereferenced
    assert lib.mhip_fp8_quantize_bucket_static(16, 16, 16, 16, 1, limit + 1, 1024, None) == _lib.ERR_SCRATCH_TOO_SMALL
    assert lib.mhip_fp8_quantize_bucket_static(16, 16, 16, 16, 1, 1 << 40, 1024, None) == _lib.ERR_SCRATCH_TOO_SMALL
    assert b"scratch" in lib.mhip_error_string(_lib.ERR_SCRATCH_TOO_SMALL)
    assert lib.mhip_fp8_quantize_bucket_static(16, 16, 16, 16, 1, 100, 512, None) == _lib.ERR_UNSUPPORTED_BLOCK
    assert lib.mhip_fp8_quantize_bucket_static(None, 16, 16, 16, 1, 100, 1024, None) == _lib.ERR_UNDEFINED_TENSOR
    assert lib.mhip_fp8_quantize_bucket_static(None, None, None, None, 0, 0, 1024, None) == 0


def test_static_index_entry_point_records_into_a_graph_and_allocates_nothing():
    # the callers it exists for: code under stream capture.  The scratch address is resolved at set-up
    # (mhip_set_device / mhip_stream_create, or an earlier call), so the captured call only launches kernels; every
    # replay, with new tensor contents and eager work in between, equals the eager mhip_fp8_quantize_bucket.
    lib = _lib.lib()
    assert lib.mhip_set_device(0) == 0
    sizes = [5000, 1, 1024, 777, 30000, 2049]
    tensors, d_ptrs, d_offs, total = _bucket(sizes, 11)
    nblk = (total + 1023) // 1024
    q = torch.zeros(total, dtype=torch.uint8, device=DEV)
    s = torch.zeros(nblk, dtype=torch.float32, device=DEV)
    q_ref, s_ref = torch.zeros_like(q), torch.zeros_like(s)
    side = torch.cuda.Stream()
    torch.cuda.synchronize()
    free_before = torch.cuda.mem_get_info()[0]
    graph = torch.cuda.CUDAGraph()
    with torch.cuda.graph(graph, stream=side):
        rc = lib.mhip_fp8_quantize_bucket_static(q.data_ptr(), s.data_ptr(), d_ptrs.data_ptr(), d_offs.data_ptr(), len(sizes), total,
                                                 1024, torch.cuda.current_stream().cuda_stream)
    assert rc == 0
    assert torch.cuda.mem_get_info()[0] >= free_before - (2 << 20)   # the call took no device memory (the graph itself: a little)
    for rep in range(3):
        g = torch.Generator().manual_seed(100 + rep)
        for t in tensors:
            t.copy_(torch.randn(t.numel(), generator=g).bfloat16())
        other = torch.randn(1 << 18, device=DEV).sum()                # unrelated eager work between replays
        graph.replay()
        assert lib.mhip_fp8_quantize_bucket(q_ref.data_ptr(), s_ref.data_ptr(), d_ptrs.data_ptr(), d_offs.data_ptr(), len(sizes), total,
                                            1024, None, torch.cuda.current_stream().cuda_stream) == 0
        torch.cuda.synchronize()
        assert torch.equal(q, q_ref) and torch.equal(s.view(torch.int32), s_ref.view(torch.int32)), rep
        assert torch.isfinite(other)
