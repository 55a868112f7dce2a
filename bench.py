#!/usr/bin/env python3
"""Benchmark of the mesh data-movement / reduce hot path on one MI355X.

    python bench.py [--gpus 1] [--steps K] [--warmup W] [--workload NAME] [--all]

A step is one pass of the hot path over one batch of synthetic, seeded input that is
already resident in HBM.  The default workload is the bf16 gradient-bucket reduce
(8 x 25,165,824 bf16 -> fp32 sum -> /8 -> bf16).  Prints ONE JSON line; ``value`` is
algorithmic GB/s (every input element read once, every output element written once)
over wall-clock time; ``roofline.achieved`` is the same bytes over the average kernel
duration measured with HIP events on the launch stream.
"""
from __future__ import annotations

import argparse
import ctypes as C
import json
import os
import sys
import time

ROOT = os.path.dirname(os.path.abspath(__file__))
if ROOT not in sys.path:
    sys.path.insert(0, ROOT)

HBM_PEAK_GBS = 8000.0
METRIC = "pack/unpack + reduce GB/s on 1 MI355X, % of HBM peak, vs host-CPU path"

# HBM bytes per launch come from the committed rocprofv3 counter summary (FETCH_SIZE / WRITE_SIZE runs, scaled by what the
# same counters read for a plain copy of known size): the table is read from the file, so a figure here is always the
# one the profile states.  A workload without a row reports null.
TRAFFIC_SOURCE = os.path.join("profiles", "bench_workloads_all_kernels.md")


def measured_traffic(path: str = None) -> dict:
    """workload -> {"traffic": scaled HBM bytes per launch, "algorithmic": bytes per launch} from the summary's table."""
    path = path or os.path.join(ROOT, TRAFFIC_SOURCE)
    table = {}
    if not os.path.exists(path):
        return table
    header = None
    for line in open(path):
        cells = [c.strip() for c in line.strip().strip("|").split("|")]
        if "scaled traffic B" in cells and "workload" in cells:
            header = cells
            continue
        if header and len(cells) == len(header) and not set(cells[0]) <= set("-: "):
            row = dict(zip(header, cells))
            try:
                table[row["workload"]] = {"traffic": int(row["scaled traffic B"]), "algorithmic": int(row["algorithmic B"])}
            except ValueError:
                continue
        elif header and not line.strip().startswith("|"):
            header = None
    return table


def _load():
    import torch
    import monarch_amd
    from monarch_amd import _lib

    lib = monarch_amd.lib()  # raises if the HIP library was not built: no fallback
    return torch, lib, _lib


def STREAM() -> int:
    import torch
    return torch.cuda.current_stream().cuda_stream


def prepared(symbol, *args):
    """A launch with its ctypes arguments built once: the timed loop then costs one foreign call per step."""
    import monarch_amd
    fn = getattr(monarch_amd.lib(), symbol)
    keep = args  # keeps pointer tables and Slice structs alive

    def call(_i=0):
        return fn(*keep)

    return call


class Events:
    """HIP event pair on an explicit stream, through the C ABI."""

    def __init__(self, lib, stream):
        self.lib, self.stream = lib, stream
        self.a, self.b = C.c_void_p(), C.c_void_p()
        assert lib.mhip_event_create(C.byref(self.a)) == 0 and lib.mhip_event_create(C.byref(self.b)) == 0

    def start(self):
        assert self.lib.mhip_event_record(self.a, self.stream) == 0

    def stop_ms(self) -> float:
        assert self.lib.mhip_event_record(self.b, self.stream) == 0
        assert self.lib.mhip_event_synchronize(self.b) == 0
        ms = C.c_float()
        assert self.lib.mhip_event_elapsed_ms(C.byref(ms), self.a, self.b) == 0
        return ms.value


# ---------------------------------------------------------------------------
# workloads: each returns (name, algorithmic_bytes_per_step, launch(i), cpu_baseline(), kernel_name)
# ---------------------------------------------------------------------------

def wl_c1(torch, stage="pack"):
    """Config 1, the reference's CPU-runnable shape: launch-latency-bound on a GPU (reported, not a target)."""
    import numpy as np
    from monarch_amd import Slice, _lib, staging
    from monarch_amd._lib import ptr_array
    s = Slice(offset=0, sizes=[4, 128, 256], strides=[65536, 512, 1])
    xs = [torch.from_numpy(np.random.default_rng(1000 + k).uniform(-1, 1, size=(4, 256, 256)).astype(np.float32)).to("cuda:0")
          for k in range(8)]
    chunks = [staging.pack(x, s) for x in xs]
    out = torch.empty_like(chunks[0])
    back = torch.zeros_like(xs[0])
    n = chunks[0].numel()
    if stage == "pack":
        nbytes, kern = 2 * n * 4, "slice_copy_kernel<16>"
        launch = prepared("mhip_slice_pack", chunks[0].data_ptr(), xs[0].data_ptr(), C.byref(s.c), 4, STREAM())
    elif stage == "unpack":
        nbytes, kern = 2 * n * 4, "slice_copy_kernel<16>"
        launch = prepared("mhip_slice_unpack", back.data_ptr(), chunks[0].data_ptr(), C.byref(s.c), 4, STREAM())
    else:
        nbytes, kern = 9 * n * 4, "reduce_kernel<f32,8,sum>"
        launch = prepared("mhip_reduce", out.data_ptr(), ptr_array([c.data_ptr() for c in chunks]), 8, n, _lib.DTYPE_F32,
                          _lib.OP_SUM, STREAM())
    launch.keep = (xs, chunks, out, back, s)

    def cpu():
        import oracle
        os_ = oracle.OSlice(s.offset, s.sizes, s.strides)
        hx = xs[0].cpu().numpy().reshape(-1)
        hc = [c.cpu().numpy() for c in chunks]
        reps, t0 = 0, time.perf_counter()
        while reps < 20 or time.perf_counter() - t0 < 2.0:
            if stage == "pack":
                oracle.pack(hx, os_)
            elif stage == "unpack":
                oracle.unpack(hx, hc[0], os_)
            else:
                oracle.reduce(hc, oracle.SUM)
            reps += 1
        dt = (time.perf_counter() - t0) / reps
        return {"value": nbytes / dt / 1e9, "unit": "GB/s", "cores": 1, "kind": "port",
                "sample": f"full workload, {reps} passes of the oracle"}

    return f"c1_f32_every_other_row_{stage}", nbytes, launch, cpu, kern, "f32" if stage == "reduce" else "u8"


def wl_c1_pipeline(torch, mode="eager"):
    """Config 1 end to end: 8 every-other-row views -> their elementwise sum -> unpacked into a view.
    eager: 8 packs + reduce + unpack (10 launches); graph: the same 10 kernels replayed as one HIP graph;
    fused: mhip_reduce_scatter reads the 8 strided views directly (2 launches); fused_graph: those two as a graph.
    GB/s counts the fused pipeline's bytes for every mode, so the modes compare by time."""
    import numpy as np
    from monarch_amd import Slice, staging
    from monarch_amd import reduce as R
    s = Slice(offset=0, sizes=[4, 128, 256], strides=[65536, 512, 1])
    n = 8
    xs = [torch.from_numpy(np.random.default_rng(1000 + k).uniform(-1, 1, size=(4, 256, 256)).astype(np.float32)).to("cuda:0")
          for k in range(n)]
    chunks = [torch.empty(len(s), device="cuda:0") for _ in range(n)]
    total = torch.empty(len(s), device="cuda:0")
    back = torch.zeros(4, 256, 256, device="cuda:0")
    whole = Slice.new_row_major([len(s)])
    nbytes = (n + 1) * len(s) * 4 + 2 * len(s) * 4

    from monarch_amd import _lib
    from monarch_amd._lib import ptr_array
    from monarch_amd.ndslice import slice_array

    def calls(stream):  # prepared C-ABI calls on `stream`: the timed loop pays no Python wrapper cost
        packs = [prepared("mhip_slice_pack", c.data_ptr(), x.data_ptr(), C.byref(s.c), 4, stream) for x, c in zip(xs, chunks)]
        red = prepared("mhip_reduce", total.data_ptr(), ptr_array([c.data_ptr() for c in chunks]), n, len(s),
                       _lib.DTYPE_F32, _lib.OP_SUM, stream)
        unp = prepared("mhip_slice_unpack", back.data_ptr(), total.data_ptr(), C.byref(s.c), 4, stream)
        fus = prepared("mhip_reduce_scatter", ptr_array([total.data_ptr()]), slice_array([whole]), 1,
                       ptr_array([x.data_ptr() for x in xs]), C.byref(s.c), 0, n, _lib.DTYPE_F32, _lib.OP_SUM, stream)
        return packs + [red, unp], [fus, unp]

    def run(seq):
        rc = 0
        for f in seq:
            rc |= f()
        return rc

    def eager():
        for x, c in zip(xs, chunks):
            staging.pack(x, s, out=c)
        R.all_reduce(total, chunks, R.ReduceOp.Sum)
        staging.unpack(back, s, total)

    def fused():
        R.reduce_scatter_views([total], [whole], xs, s, R.ReduceOp.Sum)
        staging.unpack(back, s, total)

    body = eager if mode in ("eager", "graph") else fused
    body()  # once through the checked host API
    torch.cuda.synchronize()
    if mode.endswith("graph"):
        graph = torch.cuda.CUDAGraph()
        with torch.cuda.graph(graph):
            seq_e, seq_f = calls(STREAM())  # the capture stream is current here
            assert run(seq_e if mode == "graph" else seq_f) == 0

        def launch(_i=0):
            graph.replay()
            return 0
    else:
        seq_e, seq_f = calls(STREAM())
        seq = seq_e if mode == "eager" else seq_f

        def launch(_i=0):
            return run(seq)
    launch.keep = (xs, chunks, total, back)

    def cpu():
        import oracle
        os_ = oracle.OSlice(s.offset, s.sizes, s.strides)
        hx = [x.cpu().numpy().reshape(-1) for x in xs]
        hb = np.zeros(4 * 256 * 256, dtype=np.float32)
        reps, t0 = 0, time.perf_counter()
        while reps < 5 or time.perf_counter() - t0 < 2.0:
            oracle.unpack(hb, oracle.reduce([oracle.pack(h, os_) for h in hx], oracle.SUM), os_)
            reps += 1
        dt = (time.perf_counter() - t0) / reps
        return {"value": nbytes / dt / 1e9, "unit": "GB/s", "cores": 1, "kind": "port",
                "sample": f"full pipeline, {reps} passes of the oracle (per-element Slice::get walk, scalar sum)"}

    kern = {"eager": "10 launches", "graph": "10 kernels, one graph launch", "fused": "reduce_scatter_kernel + slice_copy_kernel",
            "fused_graph": "2 kernels, one graph launch"}[mode]
    return f"c1_pipeline_{mode}", nbytes, launch, cpu, kern, "f32"


def wl_c2(torch, in_place=False, sets=3, separate=False):
    """8 bf16 chunks of one gradient bucket -> their average.  By default the chunks are the slots of
    one staging area laid out by the library (`mhip_staging_slot_pitch`); `separate` allocates them
    as eight independent torch tensors instead (which end up a multiple of 16 KiB apart)."""
    from monarch_amd import _lib, staging
    from monarch_amd import reduce as R
    from monarch_amd._lib import ptr_array
    n, numel = 8, 25_165_824
    g = torch.Generator(device="cuda:0").manual_seed(2000)
    bufs = []
    for _ in range(sets):  # rotate buffer sets so that no pass is served from the 256 MB Infinity Cache
        if separate:
            ins = [(torch.randn(numel, generator=g, device="cuda:0") * 0.02).bfloat16() for _ in range(n)]
        else:
            area = staging.StagingArea(n, numel * 2)
            ins = area.slots(torch.bfloat16)
            for t in ins:
                t.copy_((torch.randn(numel, generator=g, device="cuda:0") * 0.02).bfloat16())
        out = ins[0] if in_place else torch.empty_like(ins[0])
        bufs.append((ins, out))
    nbytes = (n + 1) * numel * 2

    for ins, out in bufs:  # one checked call through the host API, then raw prepared calls in the timed loop
        R.all_reduce(out, ins, R.ReduceOp.Avg)
    calls = [prepared("mhip_reduce", out.data_ptr(), ptr_array([t.data_ptr() for t in ins]), n, numel,
                      _lib.DTYPE_BF16, _lib.OP_AVG, STREAM()) for ins, out in bufs]

    def launch(i):
        return calls[i % sets]()

    def cpu():
        import numpy as np
        import oracle
        g2 = torch.Generator(device="cuda:0").manual_seed(2000)
        hosts = [(torch.randn(numel, generator=g2, device="cuda:0") * 0.02).bfloat16().cpu().view(torch.uint16).numpy()
                 for _ in range(n)]
        out = np.empty_like(hosts[0])
        reps, t0 = 0, time.perf_counter()
        while reps < 3 or time.perf_counter() - t0 < 10.0:
            oracle.reduce(hosts, oracle.AVG, out=out)
            reps += 1
        dt = (time.perf_counter() - t0) / reps
        # the same loop spread over every host core
        oracle.reduce(hosts, oracle.AVG, out=out, threads=True)
        t1 = time.perf_counter()
        for _ in range(3):
            oracle.reduce(hosts, oracle.AVG, out=out, threads=True)
        dt_mt = (time.perf_counter() - t1) / 3
        # the same reduction through torch's CPU kernels on all host threads (a library path, for scale)
        hts = [torch.from_numpy(h.view(np.int16)).view(torch.bfloat16) for h in hosts]
        t1 = time.perf_counter()
        (torch.stack(hts).float().sum(0) / n).bfloat16()
        dt_torch = time.perf_counter() - t1
        return {"value": nbytes / dt / 1e9, "unit": "GB/s", "cores": 1, "kind": "port",
                "sample": f"full workload, {reps} passes of the oracle's scalar fp32-accumulate loop",
                "all_cores": {"value": nbytes / dt_mt / 1e9, "unit": "GB/s", "cores": oracle.num_threads(),
                              "sample": "3 passes of the same loop under OpenMP"},
                "torch_cpu": {"value": nbytes / dt_torch / 1e9, "unit": "GB/s", "cores": torch.get_num_threads(),
                              "sample": "one pass of torch.stack(xs).float().sum(0)/8 -> bf16"}}

    name = ("c2_bf16_bucket_reduce_avg8" + ("_inplace" if in_place else "") + ("_separate_allocations" if separate else "")
            + (f"_{sets}_buffer_sets" if sets != 3 else ""))
    return name, nbytes, launch, cpu, "reduce_kernel<bf16,8,avg>", "bf16"


def wl_c2p(torch, unpack=False, sets=6):
    from monarch_amd import Slice, staging
    numel = 25_165_824
    g = torch.Generator(device="cuda:0").manual_seed(2001)
    s = Slice.new_row_major([numel])
    bufs = [((torch.randn(numel, generator=g, device="cuda:0") * 0.02).bfloat16(),
             torch.empty(numel, dtype=torch.bfloat16, device="cuda:0")) for _ in range(sets)]
    nbytes = 2 * numel * 2

    for x, st in bufs:
        staging.pack(x, s, out=st)
    if unpack:
        calls = [prepared("mhip_slice_unpack", x.data_ptr(), st.data_ptr(), C.byref(s.c), 2, STREAM()) for x, st in bufs]
    else:
        calls = [prepared("mhip_slice_pack", st.data_ptr(), x.data_ptr(), C.byref(s.c), 2, STREAM()) for x, st in bufs]

    def launch(i):
        return calls[i % sets]()

    def cpu():
        import numpy as np
        import oracle
        h = bufs[0][0].cpu().view(torch.uint16).numpy()
        os_ = oracle.OSlice(0, [numel], [1])
        t0 = time.perf_counter()
        oracle.pack(h, os_)
        dt = time.perf_counter() - t0
        oracle.pack(h, os_, threads=True)
        t1 = time.perf_counter()
        for _ in range(5):
            oracle.pack(h, os_, threads=True)
        dt_mt = (time.perf_counter() - t1) / 5
        return {"value": nbytes / dt / 1e9, "unit": "GB/s", "cores": 1, "kind": "port",
                "sample": "full workload, 1 pass of the per-element Slice::get walk",
                "all_cores": {"value": nbytes / dt_mt / 1e9, "unit": "GB/s", "cores": oracle.num_threads(),
                              "sample": "5 passes of one memcpy per contiguous run (here: the whole buffer)"}}

    return ("c2p_contiguous_unpack" if unpack else "c2p_contiguous_pack"), nbytes, launch, cpu, "contiguous_copy_kernel", "u8"


def wl_ref_copy(torch, how="hip", sets=6):
    """Not this library: the platform's own device-to-device copy of the c2p buffers (48 MiB in, 48 MiB out, same rotation),
    as context for the fractions the library's copies reach.  how = "hip": hipMemcpyAsync; "torch": Tensor.copy_."""
    numel = 25_165_824
    g = torch.Generator(device="cuda:0").manual_seed(2001)
    bufs = [((torch.randn(numel, generator=g, device="cuda:0") * 0.02).bfloat16(),
             torch.empty(numel, dtype=torch.bfloat16, device="cuda:0")) for _ in range(sets)]
    nbytes = 2 * numel * 2
    if how == "hip":
        hip = C.CDLL("libamdhip64.so")
        hip.hipMemcpyAsync.argtypes = [C.c_void_p, C.c_void_p, C.c_size_t, C.c_int, C.c_void_p]
        hip.hipMemcpyAsync.restype = C.c_int
        stream = STREAM()
        args = [(st.data_ptr(), x.data_ptr()) for x, st in bufs]

        def launch(i):
            d, s_ = args[i % sets]
            return hip.hipMemcpyAsync(d, s_, numel * 2, 3, stream)  # 3 = hipMemcpyDeviceToDevice
    else:
        def launch(i):
            x, st = bufs[i % sets]
            st.copy_(x)
            return 0

    def cpu():
        import numpy as np
        h = bufs[0][0].cpu().view(torch.uint16).numpy()
        out = np.empty_like(h)
        t0 = time.perf_counter()
        for _ in range(5):
            np.copyto(out, h)
        dt = (time.perf_counter() - t0) / 5
        return {"value": nbytes / dt / 1e9, "unit": "GB/s", "cores": 1, "kind": "port", "sample": "5 passes of numpy.copyto (memcpy)"}

    return (f"ref_copy_{how}_48mib", nbytes, launch, cpu,
            "hipMemcpyAsync, device to device (the runtime's kernel)" if how == "hip" else "torch Tensor.copy_ (PyTorch's kernel)", "u8")


def wl_c3(torch, unpack=False, sets=3):
    from monarch_amd import Slice, staging
    from monarch_amd._lib import ptr_array
    from monarch_amd.ndslice import slice_array
    g = torch.Generator(device="cuda:0").manual_seed(3000)
    views = [Slice(offset=k * 1792, sizes=[4096, 1792], strides=[14336, 1]) for k in range(8)]
    bufs = []
    for _ in range(sets):
        w = (torch.randn(4096, 14336, generator=g, device="cuda:0") * 0.02).bfloat16()
        outs = [torch.empty(4096 * 1792, dtype=torch.bfloat16, device="cuda:0") for _ in range(8)]
        staging.pack_many(w, views, outs)
        bufs.append((w, outs))
    nbytes = 2 * 4096 * 14336 * 2

    arr = slice_array(views)
    if unpack:
        calls = [prepared("mhip_slice_unpack_many", w.data_ptr(), ptr_array([o.data_ptr() for o in outs]), arr, 8, 2,
                          STREAM()) for w, outs in bufs]
    else:
        calls = [prepared("mhip_slice_pack_many", ptr_array([o.data_ptr() for o in outs]), w.data_ptr(), arr, 8, 2,
                          STREAM()) for w, outs in bufs]

    def launch(i):
        return calls[i % sets]()

    def cpu():
        import oracle
        h = bufs[0][0].cpu().view(torch.uint16).numpy().reshape(-1)
        ov = [oracle.OSlice(v.offset, v.sizes, v.strides) for v in views]
        t0 = time.perf_counter()
        for v in ov[:2]:
            oracle.pack(h, v)
        dt = (time.perf_counter() - t0) * 4
        for v in ov:
            oracle.pack(h, v, threads=True)
        t1 = time.perf_counter()
        for _ in range(3):
            for v in ov:
                oracle.pack(h, v, threads=True)
        dt_mt = (time.perf_counter() - t1) / 3
        return {"value": nbytes / dt / 1e9, "unit": "GB/s", "cores": 1, "kind": "port",
                "sample": "2 of the 8 column blocks through the per-element Slice::get walk, scaled x4",
                "all_cores": {"value": nbytes / dt_mt / 1e9, "unit": "GB/s", "cores": oracle.num_threads(),
                              "sample": "3 passes over all 8 blocks, one memcpy per 3584-byte row, rows under OpenMP"}}

    return ("c3_column_block_unpack" if unpack else "c3_column_block_pack"), nbytes, launch, cpu, "slice_copy_kernel<16>", "u8"


def wl_ragged(torch, unpack=False, sets=3):
    """A column block that fits no 16-byte grid: columns 1:7167 of a bf16 [16384, 14336] matrix (rows of 14332 bytes that
    start 2 bytes into a 16-byte vector), packed to / unpacked from one contiguous buffer.  The view is moved in 4-byte
    units from a base that is 2 bytes off: the two-vector form packing, the line-by-line form unpacking."""
    from monarch_amd import Slice
    g = torch.Generator(device="cuda:0").manual_seed(3100)
    rows, pitch, c0, cols = 16384, 14336, 1, 7166
    view = Slice(offset=c0, sizes=[rows, cols], strides=[pitch, 1])
    bufs = []
    for _ in range(sets):
        w = (torch.randn(rows, pitch, generator=g, device="cuda:0") * 0.02).bfloat16()
        out = w[:, c0:c0 + cols].contiguous().reshape(-1)
        bufs.append((w, out))
    nbytes = 2 * rows * cols * 2
    if unpack:
        calls = [prepared("mhip_slice_unpack", w.data_ptr(), o.data_ptr(), C.byref(view.c), 2, STREAM()) for w, o in bufs]
    else:
        calls = [prepared("mhip_slice_pack", o.data_ptr(), w.data_ptr(), C.byref(view.c), 2, STREAM()) for w, o in bufs]

    def launch(i):
        return calls[i % sets]()

    def cpu():
        import oracle
        h = bufs[0][0][:2048].cpu().view(torch.uint16).numpy().reshape(-1)
        ov = oracle.OSlice(c0, [2048, cols], [pitch, 1])
        t0 = time.perf_counter()
        oracle.pack(h, ov)
        dt = time.perf_counter() - t0
        return {"value": nbytes / 8 / dt / 1e9, "unit": "GB/s", "cores": 1, "kind": "port",
                "sample": "2048 of the 16384 rows through the per-element Slice::get walk"}

    kernel = "slice_unpack_lines_kernel<4>" if unpack else "slice_copy_ragged_kernel<4>"
    return ("ragged_column_block_unpack" if unpack else "ragged_column_block_pack"), nbytes, launch, cpu, kernel, "u8"


def wl_c3_reshard(torch, sets=3, one_by_one=False):
    """Configuration 3 end to end (SendTensor / to_mesh of a column-sharded weight): the 8 column blocks are packed
    into 8 staging buffers in one launch, and the buffers are transferred into their receivers' contiguous tensors
    in a second one (``one_by_one``: one launch per buffer, as the reference posts its work requests).
    Bytes per step: pack reads and writes 117 MB, the transfers read and write them again."""
    from monarch_amd import Slice, staging
    from monarch_amd._lib import ptr_array
    from monarch_amd.ndslice import slice_array
    g = torch.Generator(device="cuda:0").manual_seed(3000)
    rows, cols, k = 4096, 14336, 8
    w = cols // k
    views = [Slice(offset=j * w, sizes=[rows, w], strides=[cols, 1]) for j in range(k)]
    arr = slice_array(views)
    bufs = []
    for _ in range(sets):
        x = (torch.randn(rows, cols, generator=g, device="cuda:0") * 0.02).bfloat16()
        area = staging.StagingArea(k, rows * w * 2)
        recv = [torch.empty(rows, w, dtype=torch.bfloat16, device="cuda:0") for _ in range(k)]
        staging.pack_many(x, views, [area.slot(j, torch.bfloat16) for j in range(k)])
        bufs.append((x, area, recv))
    nbytes = 4 * rows * cols * 2
    seqs = []
    for x, area, recv in bufs:
        seq = [prepared("mhip_slice_pack_many", ptr_array([area.slot(j).data_ptr() for j in range(k)]), x.data_ptr(), arr, k, 2,
                        STREAM())]
        if one_by_one:
            seq += [prepared("mhip_buffer_transfer", recv[j].data_ptr(), area.slot(j).data_ptr(), rows * w * 2, 0, STREAM(), None)
                    for j in range(k)]
        else:
            seq.append(prepared("mhip_buffer_transfer_many", ptr_array([t.data_ptr() for t in recv]),
                                ptr_array([area.slot(j).data_ptr() for j in range(k)]), (C.c_size_t * k)(*[rows * w * 2] * k), k, 0,
                                STREAM(), None))
        seqs.append(seq)

    def launch(i):
        rc = 0
        for f in seqs[i % sets]:
            rc |= f()
        return rc

    def cpu():
        import oracle
        h = bufs[0][0].cpu().view(torch.uint16).numpy().reshape(-1)
        v = oracle.OSlice(views[0].offset, views[0].sizes, views[0].strides)
        t0 = time.perf_counter()
        oracle.send_tensor(h, v)
        dt = (time.perf_counter() - t0) * k
        return {"value": nbytes / dt / 1e9, "unit": "GB/s", "cores": 1, "kind": "port",
                "sample": "1 of the 8 column blocks through the oracle's send_tensor (Slice::get walk + byte copy), scaled x8"}

    if one_by_one:
        return "c3_reshard_end_to_end_one_transfer_per_buffer", nbytes, launch, cpu, "slice_copy_kernel<16> + 8 x contiguous_copy_kernel", "u8"
    return "c3_reshard_end_to_end", nbytes, launch, cpu, "slice_copy_kernel<16> + copy_many_kernel", "u8"


def wl_stack(torch, scatter=False, sets=None):
    """Reduction::Stack of the C2 bucket's 8 chunks in one launch: all_gather_into_tensor (out[g] = in[g]) or, with
    scatter, all_to_all_single as member 3 sees it (out chunk g = chunk 3 of member g).  The all_to_all touches
    96 MiB per launch, so it rotates over 12 buffer sets (1.1 GB touched); the all_gather moves 1.6 GB per set."""
    sets = sets or (12 if scatter else 2)
    from monarch_amd import staging
    from monarch_amd._lib import ptr_array
    n, numel = 8, 25_165_824
    g = torch.Generator(device="cuda:0").manual_seed(2002)
    bufs = []
    for _ in range(sets):
        area = staging.StagingArea(n, numel * 2)
        ins = area.slots(torch.bfloat16)
        for t in ins:
            t.copy_((torch.randn(numel, generator=g, device="cuda:0") * 0.02).bfloat16())
        out = torch.empty((1 if scatter else n) * numel, dtype=torch.bfloat16, device="cuda:0")
        bufs.append((area, ins, out))
    nbytes = 2 * (1 if scatter else n) * numel * 2
    if scatter:
        calls = [prepared("mhip_stack_scatter", out.data_ptr(), ptr_array([t.data_ptr() for t in ins]), n, 3, numel, 2, STREAM())
                 for _, ins, out in bufs]
    else:
        calls = [prepared("mhip_stack", out.data_ptr(), ptr_array([t.data_ptr() for t in ins]), n, numel, 2, STREAM())
                 for _, ins, out in bufs]

    def launch(i):
        return calls[i % sets]()

    def cpu():
        import oracle
        hs = [t.cpu().view(torch.uint16).numpy() for t in bufs[0][1]]
        t0 = time.perf_counter()
        if scatter:
            oracle.stack_scatter(hs, 3)
        else:
            oracle.stack(hs)
        dt = time.perf_counter() - t0
        return {"value": nbytes / dt / 1e9, "unit": "GB/s", "cores": 1, "kind": "port",
                "sample": "full workload, 1 pass of the oracle's byte loops"}

    return ("stack_scatter_bf16_8" if scatter else "stack_bf16_8"), nbytes, launch, cpu, "copy_many_kernel", "u8"


def wl_transpose(torch, dtype_name="f32", unpack=False, sets=3, n=None):
    from monarch_amd import Slice, staging
    n = n or int(os.environ.get("MONARCH_BENCH_TRANSPOSE_N", "8192"))
    dt = {"f32": torch.float32, "bf16": torch.bfloat16, "u8": torch.uint8}[dtype_name]
    g = torch.Generator(device="cuda:0").manual_seed(6000)
    s = Slice(offset=0, sizes=[n, n], strides=[1, n])  # iterate columns first: packs x.T

    def values():
        if dt == torch.uint8:
            return torch.randint(0, 256, (n, n), generator=g, device="cuda:0", dtype=torch.uint8)
        return torch.randn(n, n, generator=g, device="cuda:0").to(dt)

    bufs = [(values(), torch.empty(n * n, dtype=dt, device="cuda:0")) for _ in range(sets)]
    es = bufs[0][0].element_size()
    nbytes = 2 * n * n * es
    for x, st in bufs:
        staging.pack(x, s, out=st)
    if unpack:
        calls = [prepared("mhip_slice_unpack", x.data_ptr(), st.data_ptr(), C.byref(s.c), es, STREAM()) for x, st in bufs]
    else:
        calls = [prepared("mhip_slice_pack", st.data_ptr(), x.data_ptr(), C.byref(s.c), es, STREAM()) for x, st in bufs]

    def launch(i):
        return calls[i % sets]()

    def cpu():
        import oracle
        m = 2048
        h = bufs[0][0][:m, :m].contiguous().cpu().view({1: torch.uint8, 2: torch.uint16, 4: torch.int32}[es]).numpy().reshape(-1)
        t0 = time.perf_counter()
        oracle.pack(h, oracle.OSlice(0, [m, m], [1, m]))
        dt_ = (time.perf_counter() - t0) * (n * n / (m * m))
        return {"value": nbytes / dt_ / 1e9, "unit": "GB/s", "cores": 1, "kind": "port",
                "sample": f"{m}x{m} corner through the per-element Slice::get walk, scaled to {n}x{n}"}

    name = f"transpose_{dtype_name}_{n}x{n}_" + ("unpack" if unpack else "pack")
    kernel = ("slice_transpose_vec_kernel" if n * es % 128 == 0 else
              "slice_transpose_strip_kernel" if es == 1 else "slice_transpose_lines_kernel")
    return name, nbytes, launch, cpu, kernel, "u8"


def wl_c4(torch, sets=2, slots=False):
    """Mesh [2 hosts, 8 gpus] x [2048, 4096] fp32, summed over gpus, last dim scattered 8 ways.  By default
    the 16 slabs are one dense tensor, as the configuration states it; `slots` places them in the slots of a
    staging area instead (pitch 32 MiB + 8 KiB), which is where peers' slabs would land on a real mesh."""
    from monarch_amd import Slice, _lib, staging
    from monarch_amd._lib import ptr_array
    from monarch_amd.ndslice import slice_array
    H, G, Rr, Cc, K = 2, 8, 2048, 4096, 8
    g = torch.Generator(device="cuda:0").manual_seed(4000)
    slab, w = Rr * Cc, Cc // K
    pitch = staging.slot_pitch(slab * 4) // 4 if slots else slab
    in_view = Slice(offset=0, sizes=[H, Rr, Cc], strides=[G * pitch, Cc, 1])
    out_views = [Slice(offset=k * w, sizes=[H, Rr, w], strides=[Rr * Cc, Cc, 1]) for k in range(K)]
    bufs = []
    for _ in range(sets):
        if slots:
            area = staging.StagingArea(H * G, slab * 4)
            x = area.storage.view(torch.float32)
            for t in area.slots(torch.float32):
                t.copy_(torch.rand(slab, generator=g, device="cuda:0") * 2 - 1)
        else:
            x = (torch.rand(H, G, Rr, Cc, generator=g, device="cuda:0") * 2 - 1).view(-1)
        group = [x[gi * pitch:] for gi in range(G)]
        outs = [torch.empty(H * Rr * w, device="cuda:0") for _ in range(K)]
        bufs.append((x, group, outs))
    nbytes = H * G * slab * 4 + H * slab * 4

    arr = slice_array(out_views)
    calls = [prepared("mhip_reduce_scatter", ptr_array([o.data_ptr() for o in outs]), arr, K,
                      ptr_array([t.data_ptr() for t in group]), C.byref(in_view.c), 0, G, _lib.DTYPE_F32, _lib.OP_SUM,
                      STREAM()) for _, group, outs in bufs]

    def launch(i):
        return calls[i % sets]()

    def cpu():
        import oracle
        hx = bufs[0][0].cpu().numpy().reshape(-1)
        ov = oracle.OSlice(in_view.offset, in_view.sizes, in_view.strides)
        o0 = oracle.OSlice(out_views[0].offset, out_views[0].sizes, out_views[0].strides)
        t0 = time.perf_counter()
        oracle.reduce_scatter([hx[gi * pitch:] for gi in range(G)], ov, [o0], oracle.SUM)
        dt = (time.perf_counter() - t0) * K
        # the library path of the same work on the host: sum over the gpu axis, then 8 contiguous column slices
        # (the shape rule of python/monarch/common/tensor.py:494-503 followed by the column-block scatter)
        if slots:
            ht = torch.stack([torch.from_numpy(hx[i * pitch: i * pitch + slab]) for i in range(H * G)]).view(H, G, Rr, Cc)
        else:
            ht = torch.from_numpy(hx).view(H, G, Rr, Cc)
        ht.sum(1)
        t1 = time.perf_counter()
        red = ht.sum(1)
        cols = [red[:, :, k * w:(k + 1) * w].contiguous() for k in range(K)]
        dt_torch = time.perf_counter() - t1
        del cols
        return {"value": nbytes / dt / 1e9, "unit": "GB/s", "cores": 1, "kind": "port",
                "sample": "1 of the 8 scatter outputs through the oracle, scaled x8",
                "torch_cpu": {"value": nbytes / dt_torch / 1e9, "unit": "GB/s", "cores": torch.get_num_threads(),
                              "sample": "one pass of x.sum(1) and 8 .contiguous() column slices on the full tensor"}}

    name = "c4_mesh_dim_reduce_scatter_f32" + ("_staging_slots" if slots else "") + (f"_{sets}_buffer_sets" if sets != 2 else "")
    return name, nbytes, launch, cpu, "reduce_scatter_kernel<f32,vec>", "f32"


_C5 = {}


def _c5_setup(torch):
    """The bucket of configuration 5, built once per process: its stages share the tensors, the flat buffer and the payload."""
    if not _C5:
        import numpy as np
        from monarch_amd import fp8
        rng = np.random.default_rng(5000)
        sizes = np.round(np.exp(rng.uniform(np.log(2**10), np.log(2**22), size=1500))).astype(np.int64).tolist()
        total = sum(sizes)
        g = torch.Generator(device="cuda:0").manual_seed(5001)
        x = torch.randn(total, generator=g, device="cuda:0")
        x = torch.where(torch.rand(total, generator=g, device="cuda:0") < 1e-3, x * 50, x).bfloat16()
        offs = np.concatenate([[0], np.cumsum(sizes)])
        tensors = [x[offs[i]: offs[i + 1]].clone() for i in range(1500)]
        del x
        bucket = fp8.FlatBucket(tensors)
        flat = bucket.pack()
        q, s = fp8.quantize(flat)
        _C5.update(fp8=fp8, bucket=bucket, tensors=tensors, sizes=sizes, total=total, flat=flat, q=q, s=s)
    c = _C5
    return c["fp8"], c["bucket"], c["tensors"], c["sizes"], c["total"], c["flat"], c["q"], c["s"]


def release_shared():
    _C5.clear()


def wl_c5(torch, stage="quantize"):
    fp8, bucket, tensors, sizes, total, flat, q, s = _c5_setup(torch)
    nblk = (total + 1023) // 1024
    # the fused bucket forms run with the bucket's block index unless the stage name ends in "_search"
    index = None if stage.endswith("_search") else bucket.block_index().data_ptr()
    stage = stage[: -len("_search")] if stage.endswith("_search") else stage
    acc = torch.zeros(total, device="cuda:0") if "dequant" in stage or stage == "flat_unpack" else None
    if stage in ("flat_pack", "quantize", "quantize_bucket"):   # these write the shared buffers: give them their own
        flat = torch.empty_like(flat) if stage == "flat_pack" else flat
        q, s = (torch.empty_like(q), torch.empty_like(s)) if stage != "flat_pack" else (q, s)
    outs = [torch.empty(n, device="cuda:0") for n in sizes] if stage == "flat_unpack" else None
    if stage == "flat_pack":
        nbytes, kern = 4 * total, "flat_copy_kernel<pack>"
        launch = prepared("mhip_flat_pack", flat.data_ptr(), bucket.d_ptrs.data_ptr(), bucket.d_offsets.data_ptr(),
                          len(sizes), total, 2, index, STREAM())
    elif stage == "quantize":
        nbytes, kern = 3 * total + 4 * nblk, "fp8_quantize_kernel"
        launch = prepared("mhip_fp8_quantize", q.data_ptr(), s.data_ptr(), flat.data_ptr(), total, 1024, STREAM())
    elif stage == "quantize_bucket":
        nbytes, kern = 3 * total + 4 * nblk, "fp8_quantize_bucket_kernel"
        launch = prepared("mhip_fp8_quantize_bucket", q.data_ptr(), s.data_ptr(), bucket.d_ptrs.data_ptr(),
                          bucket.d_offsets.data_ptr(), len(sizes), total, 1024, index, STREAM())
    elif stage in ("dequant_bucket", "dequant_bucket_arena"):
        nbytes, kern = 9 * total + 4 * nblk, "fp8_dequant_accumulate_bucket_kernel"
        if stage.endswith("arena"):
            # the same accumulators carved out of one allocation, each starting on a 256-byte boundary (so not the flat
            # layout): what the kernel does when 1500 separate allocations are not in the way
            starts, at = [], 0
            for n in sizes:
                starts.append(at)
                at += (n + 63) // 64 * 64
            arena = torch.zeros(at, device="cuda:0")
            accs = [arena[st: st + n] for st, n in zip(starts, sizes)]
        else:
            accs = [torch.zeros(n, device="cuda:0") for n in sizes]
        aptrs = bucket.pointer_table(accs)
        launch = prepared("mhip_fp8_dequant_accumulate_bucket", aptrs.data_ptr(), q.data_ptr(), s.data_ptr(),
                          bucket.d_offsets.data_ptr(), len(sizes), total, 1024, index, STREAM())
        launch.keep = accs
    elif stage == "dequant_bucket_many8":
        qs = [q] + [(q ^ (r + 1)).contiguous() for r in range(1, 8)]
        ss = [s] + [(s * (1.0 + 0.125 * r)).contiguous() for r in range(1, 8)]
        nbytes, kern = (8 + 8) * total + 8 * 4 * nblk, "fp8_dequant_accumulate_bucket_many_kernel"
        accs = [torch.zeros(n, device="cuda:0") for n in sizes]
        aptrs = bucket.pointer_table(accs)
        from monarch_amd._lib import ptr_array
        launch = prepared("mhip_fp8_dequant_accumulate_bucket_many", aptrs.data_ptr(), ptr_array([t.data_ptr() for t in qs]),
                          ptr_array([t.data_ptr() for t in ss]), 8, bucket.d_offsets.data_ptr(), len(sizes), total, 1024,
                          index, STREAM())
        launch.keep = (accs, qs, ss)
    elif stage in ("dequant_many8", "dequant_many8_overwrite"):
        # 8 peers' payloads (the same codes perturbed per peer) into one accumulator in one pass
        over = stage.endswith("overwrite")
        qs = [q] + [(q ^ (r + 1)).contiguous() for r in range(1, 8)]
        ss = [s] + [(s * (1.0 + 0.125 * r)).contiguous() for r in range(1, 8)]
        nbytes, kern = (8 + (4 if over else 8)) * total + 8 * 4 * nblk, "fp8_dequant_accumulate_many_kernel<8>"
        from monarch_amd._lib import ptr_array
        launch = prepared("mhip_fp8_dequant_accumulate_many", acc.data_ptr(), ptr_array([t.data_ptr() for t in qs]),
                          ptr_array([t.data_ptr() for t in ss]), 8, total, 1024, 1 if over else 0, STREAM())
        launch.keep = (qs, ss)
    elif stage == "dequant_accumulate":
        nbytes, kern = 9 * total + 4 * nblk, "fp8_dequant_accumulate_kernel"
        launch = prepared("mhip_fp8_dequant_accumulate", acc.data_ptr(), q.data_ptr(), s.data_ptr(), total, 1024,
                          STREAM())
    else:
        nbytes, kern = 8 * total, "flat_copy_kernel<unpack>"
        ptrs = bucket.pointer_table(outs)

        launch = prepared("mhip_flat_unpack", ptrs.data_ptr(), acc.data_ptr(), bucket.d_offsets.data_ptr(), len(sizes),
                          total, 4, index, STREAM())

    def cpu():
        import numpy as np
        import oracle
        sample = min(total, 64 * 1024 * 1024)
        h = flat[:sample].cpu().view(torch.uint16).numpy()
        t0 = time.perf_counter()
        if stage in ("quantize", "quantize_bucket"):
            oracle.fp8_quantize(h, 1024)
        elif stage.startswith("dequant"):
            hq, hs = q[:sample].cpu().numpy(), s[: (sample + 1023) // 1024].cpu().numpy()
            ha = np.zeros(sample, dtype=np.float32)
            t0 = time.perf_counter()
            for _ in range(8 if "many8" in stage else 1):  # one oracle pass per peer
                oracle.fp8_dequant_accumulate(ha, hq, hs, 1024)
        else:
            # the oracle's flat pack / unpack (one memcpy per tensor) over the leading tensors of the bucket
            k = max(1, int(np.searchsorted(np.cumsum(sizes), sample)))
            sample = int(np.sum(sizes[:k]))
            es = 2 if stage == "flat_pack" else 4
            hts = [np.zeros(n, dtype=np.uint16 if es == 2 else np.float32) for n in sizes[:k]]
            offs = np.concatenate([[0], np.cumsum(sizes[:k])]).tolist()
            t0 = time.perf_counter()
            if stage == "flat_pack":
                oracle.flat_pack(hts, offs)
            else:
                oracle.flat_unpack(np.zeros(sample, dtype=np.float32), offs)
        dt = (time.perf_counter() - t0) * (total / sample)
        rec = {"value": nbytes / dt / 1e9, "unit": "GB/s", "cores": 1, "kind": "port",
               "sample": f"first {sample} elements of the flat buffer through the oracle, scaled to {total}"}
        if stage in ("quantize", "quantize_bucket"):
            # the library path of the same codec on the host: per-block absmax, scale, clamp to +-448, torch's e4m3fn cast
            ht = torch.from_numpy(h[: sample // 1024 * 1024].view(np.int16)).view(torch.bfloat16)
            t1 = time.perf_counter()
            xf = ht.float().view(-1, 1024)
            amax = xf.abs().amax(1, keepdim=True).clamp_min(2.0**-40)
            (xf * (448.0 / amax)).clamp(-448.0, 448.0).to(torch.float8_e4m3fn)
            dt_torch = (time.perf_counter() - t1) * (total / ht.numel())
            rec["torch_cpu"] = {"value": nbytes / dt_torch / 1e9, "unit": "GB/s", "cores": torch.get_num_threads(),
                                "sample": f"absmax / scale / clamp / to(float8_e4m3fn) over the first {ht.numel()} elements, scaled"}
        return rec

    return f"c5_fp8_{stage}" + ("_table_search" if index is None and "bucket" in stage else ""), nbytes, launch, cpu, kern, \
        "bf16->f8e4m3fn"


LAYOUT = {  # where a workload's inputs live, when that is the library's choice
    "c2": "8 slots of one staging area, pitch mhip_staging_slot_pitch(48 MiB) = 48 MiB + 8 KiB",
    "c2_inplace": "8 slots of one staging area, pitch 48 MiB + 8 KiB; output = slot 0",
    "c2_separate": "8 separate torch allocations",
    "c2_cold": "as c2, rotating over 8 buffer sets (3.6 GB)",
    "c4_cold": "as c4, rotating over 5 buffer sets (3 GB)",
    "c2_inplace_separate": "8 separate torch allocations; output = input 0",
    "c4": "one dense [2,8,2048,4096] tensor (slab pitch 32 MiB)",
    "c4_slots": "16 slots of one staging area, pitch 32 MiB + 8 KiB",
}

WORKLOADS = {
    "c1_pack": lambda t: wl_c1(t, "pack"),
    "c1_unpack": lambda t: wl_c1(t, "unpack"),
    "c1_reduce": lambda t: wl_c1(t, "reduce"),
    "c1_pipeline": lambda t: wl_c1_pipeline(t, "eager"),
    "c1_pipeline_graph": lambda t: wl_c1_pipeline(t, "graph"),
    "c1_pipeline_fused": lambda t: wl_c1_pipeline(t, "fused"),
    "c1_pipeline_fused_graph": lambda t: wl_c1_pipeline(t, "fused_graph"),
    "c2": lambda t: wl_c2(t, False),
    "c2_inplace": lambda t: wl_c2(t, True),
    "c2_separate": lambda t: wl_c2(t, False, separate=True),
    # the same launches rotated over 3.6 GB (c2) and 3 GB (c4) instead of 1.4 / 1.2 GB: nothing of a buffer set is
    # left in the 256 MB Infinity Cache or the L2s when its turn comes again
    "c2_cold": lambda t: wl_c2(t, False, sets=8),
    "c4_cold": lambda t: wl_c4(t, sets=5),
    "c2_inplace_separate": lambda t: wl_c2(t, True, separate=True),
    "c2p_pack": lambda t: wl_c2p(t, False),
    "c2p_unpack": lambda t: wl_c2p(t, True),
    # the platform's own copies of the same buffers, for context
    "ref_copy_hip": lambda t: wl_ref_copy(t, "hip"),
    "ref_copy_torch": lambda t: wl_ref_copy(t, "torch"),
    "ragged_pack": lambda t: wl_ragged(t, False), "ragged_unpack": lambda t: wl_ragged(t, True),
    "c3_pack": lambda t: wl_c3(t, False),
    "c3_unpack": lambda t: wl_c3(t, True),
    "c3_reshard_e2e": wl_c3_reshard,
    "c3_reshard_e2e_one_by_one": lambda t: wl_c3_reshard(t, one_by_one=True),
    "stack8": lambda t: wl_stack(t, False),
    "stack_scatter8": lambda t: wl_stack(t, True),
    "c4": wl_c4,
    "c4_slots": lambda t: wl_c4(t, slots=True),
    "tr_f32_pack": lambda t: wl_transpose(t, "f32", False),
    "tr_f32_unpack": lambda t: wl_transpose(t, "f32", True),
    "tr_bf16_pack": lambda t: wl_transpose(t, "bf16", False),
    "tr_bf16_unpack": lambda t: wl_transpose(t, "bf16", True),
    # rows of 16400 bytes: no written row starts on a cache line
    "tr_bf16_8200_pack": lambda t: wl_transpose(t, "bf16", False, n=8200),
    "tr_bf16_8200_unpack": lambda t: wl_transpose(t, "bf16", True, n=8200),
    "tr_u8_8200_pack": lambda t: wl_transpose(t, "u8", False, n=8200, sets=6),
    "tr_u8_8200_unpack": lambda t: wl_transpose(t, "u8", True, n=8200, sets=6),
    "c5_flat_pack": lambda t: wl_c5(t, "flat_pack"),
    "c5_quantize": lambda t: wl_c5(t, "quantize"),
    "c5_dequant": lambda t: wl_c5(t, "dequant_accumulate"),
    "c5_quantize_bucket": lambda t: wl_c5(t, "quantize_bucket"),
    "c5_dequant_bucket": lambda t: wl_c5(t, "dequant_bucket"),
    "c5_dequant_bucket_arena": lambda t: wl_c5(t, "dequant_bucket_arena"),
    "c5_quantize_bucket_search": lambda t: wl_c5(t, "quantize_bucket_search"),
    "c5_dequant_bucket_search": lambda t: wl_c5(t, "dequant_bucket_search"),
    "c5_flat_unpack": lambda t: wl_c5(t, "flat_unpack"),
    "c5_flat_pack_search": lambda t: wl_c5(t, "flat_pack_search"),
    "c5_flat_unpack_search": lambda t: wl_c5(t, "flat_unpack_search"),
    "c5_dequant_many8": lambda t: wl_c5(t, "dequant_many8"),
    "c5_dequant_many8_overwrite": lambda t: wl_c5(t, "dequant_many8_overwrite"),
    "c5_dequant_bucket_many8": lambda t: wl_c5(t, "dequant_bucket_many8"),
}


SWEEPS = {
    # name -> (environment variable the library reads at every call when MONARCH_HIP_TUNING=1 was set at load time,
    #          {column: value or None for the library's choice})
    "transpose_walks": ("MONARCH_HIP_TRANSPOSE_WALK",
                        {"library": None, "blocked 4": "0,1,4,0", "blocked 4 rot": "0,1,4,1", "blocked 8": "0,1,8,0",
                         "blocked 8 rot": "0,1,8,1", "blocked 16": "0,1,16,0", "packed fastest": "1,0", "memory fastest": "2,0",
                         "diagonal, XCD ranges": "3,1", "diagonal": "3,0"}),
    "transpose_policies": ("MONARCH_HIP_TRANSPOSE_POLICY",
                           {"library": None, "cached loads, write-through stores": "0", "streaming loads and stores": "1",
                            "streaming loads only": "2", "streaming stores only": "3"}),
}


_SWEEP_COMMON = """\
Command (repository root, one GPU; under a minute):

    python bench.py --sweep {which} > profiles/{file}

Every cell is the fraction of the 8 TB/s HBM peak that `mhip_slice_pack` / `mhip_slice_unpack` reach on a transposing
view (`x[:, :, :cols].transpose(1, 2)` of a `[batch, rows, pitch]` tensor; algorithmic bytes = 2 x elements x element
size) with one variant forced through `{{envvar}}`; `library` is what the host code picks by itself.  All variants of a
row are switched in turn inside one process on one GPU: medians of {{reps}} alternations of {{launches}} launches, 3 rotating
buffer sets.  Matrices of 4096 x 4096 and smaller partly live in the 256 MB Infinity Cache across the three buffer sets.  Shapes whose written rows do not start on cache lines (8200 x 8200, 5000 x 7000) run the kernel with
line-aligned windows for 2-, 4- and 8-byte elements under every variant of this table; 1-byte elements of such shapes with at least 1024 strip
segments (8200 x 8200) run the strip kernel, which has one order of its own and ignores the walk: its columns differ by run-to-run noise only.
"""
SWEEP_HEADERS = {
    "transpose_walks": "# Transposing pack / unpack: A/B of the tile walks (MI355X)\n\n"
    + _SWEEP_COMMON.format(which="transpose_walks", file="transpose_walk_ab.md") + """\
`blocked g`: XCD-contiguous ranges of g x g tile blocks (`rot`: each XCD's share starts an eighth of the c-groups
further on); `packed fastest` / `memory fastest`: plain row-major walks; `diagonal`: consecutive workgroups step one
tile along both axes.  The selection rule (`choose_walk` in `monarch_amd/csrc/transpose_kernels.hip`): 1/2/4-byte
elements whose row pitches are multiples of 4 KiB on both sides take the diagonal walk, everything else the blocked
walk (block 4 for 1-byte, 8 for 2-byte, 16 for 4/8-byte elements; 8 with the 512-byte-row tiles of 4- and 8-byte elements, 4 with that of 2-byte elements).  Every walk
runs with the cache policy the library picks for the element size.""",
    "transpose_policies": "# Transposing pack / unpack: A/B of the cache policies of its loads and stores (MI355X)\n\n"
    + _SWEEP_COMMON.format(which="transpose_policies", file="transpose_cache_policy_ab.md") + """\
`cached loads, write-through stores`: plain 128-bit loads, `global_store_dwordx4 ... sc1`; `streaming`: the `nt`
policy bit on loads and/or stores.  The selection rule (`choose_cache_policy` in
`monarch_amd/csrc/transpose_kernels.hip`): stores of whole aligned 16-byte vectors stream; loads stream too when both
sides are aligned and the packed bytes reach 120 MiB (source and destination together no longer fit the 256 MiB
Infinity Cache); everything else keeps cached loads and write-through or cached stores.  Every policy runs with the tile walk the
library picks for the shape.""",
}


def sweep_transpose(which, dtypes, reps=5, launches=30):
    """A/B of the transposing kernel's tile walks (--sweep transpose_walks) or cache policies (--sweep
    transpose_policies): every variant is switched in turn inside one process through an environment variable the
    library reads at every call, medians of `reps` alternations of `launches` launches, three rotating buffer sets.
    Prints one Markdown table per element size: fraction of HBM peak per variant."""
    envvar, variants = SWEEPS[which]
    os.environ["MONARCH_HIP_TUNING"] = "1"  # the library looks at its tuning variables only when this is set while it loads
    torch, lib, _ = _load()
    from monarch_amd import Slice
    torch.cuda.set_device(0)
    stream = C.c_void_p(torch.cuda.current_stream().cuda_stream)
    libc = C.CDLL(None)

    def setenv(v):
        if v is None:
            libc.unsetenv(envvar.encode())
        else:
            libc.setenv(envvar.encode(), v.encode(), 1)

    types = {"u8": (torch.uint8, 1), "bf16": (torch.bfloat16, 2), "f32": (torch.float32, 4), "f64": (torch.float64, 8)}
    # (batch, rows, cols, pitch): of a [batch, rows, pitch] tensor the part [:, :, :cols] is packed transposed
    shapes = [(1, 8192, 8192, 8192), (1, 4096, 4096, 4096), (4, 4096, 4096, 4096), (1, 16384, 8192, 8192),
              (1, 8192, 16384, 16384), (1, 8192, 4096, 4096), (1, 4096, 8192, 8192), (8, 2048, 8192, 8192),
              (1, 8064, 8064, 8064), (1, 8200, 8200, 8200), (1, 8192, 8192, 8320), (1, 8192, 8192, 8256),
              (1, 6144, 6144, 6144), (1, 12288, 12288, 12288), (1, 5000, 7000, 7000), (1, 3072, 4096, 4096)]
    print(SWEEP_HEADERS[which].format(envvar=envvar, reps=reps, launches=launches))
    for name in dtypes:
        dt, es = types[name]
        print(f"\n### {name} ({es}-byte elements)\n")
        print("| batch, rows, cols, pitch | direction | " + " | ".join(variants) + " | best |")
        print("|---|---|" + "---:|" * len(variants) + "---|")
        for (b, r, c, pitch) in shapes:
            if b * r * pitch * es > (3 << 30):
                continue
            bufs = []
            for _ in range(3):
                x = torch.empty(b, r, pitch, dtype=dt, device="cuda:0")
                x.view(torch.uint8).random_(0, 255)
                bufs.append((x, torch.empty(b * r * c, dtype=dt, device="cuda:0")))
            s = Slice.of_tensor(bufs[0][0][:, :, :c].transpose(1, 2))
            for sym in ("mhip_slice_pack", "mhip_slice_unpack"):
                if sym.endswith("unpack"):
                    calls = [prepared(sym, x.data_ptr(), st.data_ptr(), C.byref(s.c), es, STREAM()) for x, st in bufs]
                else:
                    calls = [prepared(sym, st.data_ptr(), x.data_ptr(), C.byref(s.c), es, STREAM()) for x, st in bufs]
                res = {k: [] for k in variants}
                for _ in range(reps):
                    for k, v in variants.items():
                        setenv(v)
                        for i in range(4):
                            assert calls[i % 3]() == 0
                        torch.cuda.synchronize()
                        ev = Events(lib, stream)
                        ev.start()
                        for i in range(launches):
                            calls[i % 3]()
                        res[k].append(2 * b * r * c * es / (ev.stop_ms() / launches) / 1e6 / HBM_PEAK_GBS)
                setenv(None)
                med = {k: sorted(v)[len(v) // 2] for k, v in res.items()}
                best = max(med, key=med.get)
                print(f"| {b}, {r}, {c}, {pitch} | {sym[11:]} | " + " | ".join(f"{med[k]:.3f}" for k in variants) + f" | {best} |",
                      flush=True)
            del bufs, calls
            torch.cuda.empty_cache()


PLATFORM_HEADER = """\
# The library's kernels beside the platform's own on the same buffers (MI355X)

Command (repository root, one GPU; under a minute):

    python bench.py --sweep platform > profiles/platform_kernels_same_buffers.md

Context, not a target: the reference holds no device kernel for this path (its data movement is NCCL's, ibverbs' and
PyTorch's), so the nearest yardstick on this GPU is what the ROCm runtime and PyTorch do with the same bytes.  Every row
times both sides on the same buffers in one process: HIP events on the launch stream, median of 3 runs of {launches} launches,
rotating buffer sets; fraction of the 8 TB/s HBM peak over the same algorithmic bytes.  The PyTorch calls are the
single-kernel forms that compute the same result (checked once per row before timing; `same result` says whether the bytes
are identical: `torch.mean` adds the eight members in an order of its own, so an element here and there rounds the other way).
"""


def sweep_platform(launches=30):
    """The library's kernels beside hipMemcpyAsync and PyTorch's own kernels on the same buffers (--sweep platform)."""
    torch, lib, _ = _load()
    from monarch_amd import Slice, _torch
    from monarch_amd import reduce as R
    torch.cuda.set_device(0)
    stream = C.c_void_p(torch.cuda.current_stream().cuda_stream)
    hip = C.CDLL("libamdhip64.so")
    hip.hipMemcpyAsync.argtypes = [C.c_void_p, C.c_void_p, C.c_size_t, C.c_int, C.c_void_p]
    hip.hipMemcpyAsync.restype = C.c_int

    def frac(fn, nbytes, nsets):
        res = []
        for _ in range(3):
            for i in range(4):
                fn(i % nsets)
            torch.cuda.synchronize()
            ev = Events(lib, stream)
            ev.start()
            for i in range(launches):
                fn(i % nsets)
            res.append(nbytes / (ev.stop_ms() / launches) / 1e6 / HBM_PEAK_GBS)
        return sorted(res)[1]

    torch.manual_seed(7)
    print(PLATFORM_HEADER.format(launches=launches))
    print("| operation | algorithmic bytes | this library | platform | platform call | same result |")
    print("|---|---:|---:|---:|---|---|")

    def row(what, nbytes, ours, theirs, call, same):
        print(f"| {what} | {nbytes} | {ours:.3f} | {theirs:.3f} | {call} | {same} |", flush=True)

    # contiguous copy, 48 MiB in and out (workload c2p)
    numel, sets = 25_165_824, 6
    bufs = [(torch.empty(numel, dtype=torch.bfloat16, device="cuda:0").normal_(), torch.empty(numel, dtype=torch.bfloat16, device="cuda:0"))
            for _ in range(sets)]
    s = Slice.new_row_major([numel])
    calls = [prepared("mhip_slice_pack", st.data_ptr(), x.data_ptr(), C.byref(s.c), 2, STREAM()) for x, st in bufs]
    ours = frac(lambda i: calls[i](), 4 * numel, sets)
    ptrs = [(st.data_ptr(), x.data_ptr()) for x, st in bufs]
    th = frac(lambda i: hip.hipMemcpyAsync(ptrs[i][0], ptrs[i][1], 2 * numel, 3, stream), 4 * numel, sets)
    row("contiguous pack, 48 MiB", 4 * numel, ours, th, "`hipMemcpyAsync`, device to device", "yes")
    tt = frac(lambda i: bufs[i][1].copy_(bufs[i][0]), 4 * numel, sets)
    row("contiguous pack, 48 MiB", 4 * numel, ours, tt, "`dst.copy_(src)`", "yes")
    del bufs, calls
    torch.cuda.empty_cache()

    # bf16 bucket reduce, avg over 8 members of 48 MiB (workload c2), members as the rows of one [8, N] tensor
    sets = 3
    stacks = [(torch.empty(8, numel, dtype=torch.bfloat16, device="cuda:0").normal_(0, 0.02), torch.empty(numel, dtype=torch.bfloat16, device="cuda:0"),
               torch.empty(numel, dtype=torch.bfloat16, device="cuda:0")) for _ in range(sets)]
    nbytes = 18 * numel

    def ours_reduce(i):
        x, o, _ = stacks[i]
        R.all_reduce(o, [x[g] for g in range(8)], R.ReduceOp.Avg)

    def torch_reduce(i):
        x, _, o = stacks[i]
        torch.mean(x, dim=0, out=o)

    ours_reduce(0)
    torch_reduce(0)
    torch.cuda.synchronize()
    same = "yes" if torch.equal(stacks[0][1].view(torch.int16), stacks[0][2].view(torch.int16)) else \
        f"no ({(stacks[0][1].view(torch.int16) != stacks[0][2].view(torch.int16)).sum().item()} of {numel} elements differ)"
    calls = []
    for x, o, _ in stacks:
        ptrs_in = (C.c_void_p * 8)(*[x[g].data_ptr() for g in range(8)])
        calls.append(prepared("mhip_reduce", o.data_ptr(), ptrs_in, 8, numel, _torch.dtype_code(torch.bfloat16), int(R.ReduceOp.Avg), STREAM()))
    ours = frac(lambda i: calls[i](), nbytes, sets)
    tt = frac(torch_reduce, nbytes, sets)
    row("bf16 reduce, avg of 8 x 48 MiB", nbytes, ours, tt, "`torch.mean(x[8, N], dim=0, out=o)`", same)
    del stacks, calls
    torch.cuda.empty_cache()

    # column block of a [4096, 14336] bf16 matrix (one of workload c3's eight views), and all eight
    rows_, cols_, w = 4096, 14336, 1792
    sets = 3
    mats = [(torch.empty(rows_, cols_, dtype=torch.bfloat16, device="cuda:0").normal_(), torch.empty(8, rows_, w, dtype=torch.bfloat16, device="cuda:0"),
             torch.empty(8, rows_, w, dtype=torch.bfloat16, device="cuda:0")) for _ in range(sets)]
    views = [Slice(offset=k * w, sizes=[rows_, w], strides=[cols_, 1]) for k in range(8)]

    from monarch_amd._lib import ptr_array
    from monarch_amd.ndslice import slice_array
    varr = slice_array(views)
    c3calls = [prepared("mhip_slice_pack_many", ptr_array([o[k].data_ptr() for k in range(8)]), x.data_ptr(), varr, 8, 2, STREAM())
               for x, o, _ in mats]

    def ours_c3(i):
        return c3calls[i]()

    def torch_c3(i):
        x, _, o = mats[i]
        o.copy_(x.view(rows_, 8, w).transpose(0, 1))

    ours_c3(0)
    torch_c3(0)
    torch.cuda.synchronize()
    same = "yes" if torch.equal(mats[0][1].view(torch.int16), mats[0][2].view(torch.int16)) else "no"
    nbytes = 4 * rows_ * cols_
    row("8 column blocks of [4096, 14336] bf16", nbytes, frac(ours_c3, nbytes, sets), frac(torch_c3, nbytes, sets),
        "`o[8, R, w].copy_(x.view(R, 8, w).transpose(0, 1))`", same)
    del mats
    torch.cuda.empty_cache()

    # transposing packs
    for name, dt, es, n in (("bf16", torch.bfloat16, 2, 8192), ("f32", torch.float32, 4, 8192), ("u8", torch.uint8, 1, 8192),
                            ("bf16", torch.bfloat16, 2, 8200), ("u8", torch.uint8, 1, 8200)):
        sets = 3 if es > 1 else 6
        tb = []
        for _ in range(sets):
            x = torch.empty(n, n, dtype=dt, device="cuda:0")
            x.view(torch.uint8).random_(0, 255)
            tb.append((x, torch.empty(n * n, dtype=dt, device="cuda:0"), torch.empty(n, n, dtype=dt, device="cuda:0")))
        sl = Slice.of_tensor(tb[0][0].t())
        calls = [prepared("mhip_slice_pack", o.data_ptr(), x.data_ptr(), C.byref(sl.c), es, STREAM()) for x, o, _ in tb]

        def torch_tr(i):
            x, _, o = tb[i]
            o.copy_(x.t())

        calls[0]()
        torch_tr(0)
        torch.cuda.synchronize()
        same = "yes" if torch.equal(tb[0][1].view(torch.uint8), tb[0][2].view(-1).view(torch.uint8)) else "no"
        nbytes = 2 * n * n * es
        row(f"transposing pack {n} x {n} {name}", nbytes, frac(lambda i: calls[i](), nbytes, sets), frac(torch_tr, nbytes, sets),
            "`o.copy_(x.t())`", same)
        del tb, calls
        torch.cuda.empty_cache()


REDUCE_OPS_HEADER = """\
# mhip_reduce over element types, member counts and ops (MI355X)

Command (repository root, one GPU; about a minute):

    python bench.py --sweep reduce_ops > profiles/reduce_ops_dtypes.md

Every cell is the fraction of the 8 TB/s HBM peak that `mhip_reduce` reaches on n members of 48 MiB each into a separate
48 MiB output (algorithmic bytes = (n + 1) x 48 MiB), members and outputs in separate allocations, median of 3 runs of
{launches} launches, 2 to 4 rotating buffer sets (at most 3 GiB of them).  Sum and Avg are the ops of the path; Prod, Max and Min
share one kernel per type that tests the op once per 16-byte vector.
"""


def sweep_reduce_ops(launches=20):
    """Fraction of HBM peak of mhip_reduce over dtype x member count x op (--sweep reduce_ops)."""
    torch, lib, _ = _load()
    from monarch_amd import _torch
    from monarch_amd import reduce as R
    torch.cuda.set_device(0)
    stream = C.c_void_p(torch.cuda.current_stream().cuda_stream)
    ops = [R.ReduceOp.Sum, R.ReduceOp.Avg, R.ReduceOp.Prod, R.ReduceOp.Max, R.ReduceOp.Min]
    print(REDUCE_OPS_HEADER.format(launches=launches))
    print("| element type | members | " + " | ".join(o.name for o in ops) + " |")
    print("|---|---:|" + "---:|" * len(ops))
    for dt in (torch.bfloat16, torch.float16, torch.float32, torch.float64, torch.int32, torch.int64, torch.uint8, torch.int8):
        es = torch.empty(0, dtype=dt).element_size()
        numel = (48 << 20) // es
        for n in (2, 3, 4, 8, 16, 33):
            sets = max(2, min(4, (3 << 30) // ((n + 1) * (48 << 20))))
            bufs = []
            for _ in range(sets):
                xs = [torch.empty(numel, dtype=dt, device="cuda:0") for _ in range(n)]
                for x in xs:
                    x.view(torch.uint8).random_(0, 100)   # small positive values in every type: no NaN, no Inf
                bufs.append((xs, torch.empty(numel, dtype=dt, device="cuda:0")))
            cells = []
            for op in ops:
                if op == R.ReduceOp.Avg and not dt.is_floating_point:
                    cells.append("—")
                    continue
                calls = []
                for xs, o in bufs:
                    ptrs = (C.c_void_p * n)(*[x.data_ptr() for x in xs])
                    calls.append(prepared("mhip_reduce", o.data_ptr(), ptrs, n, numel, _torch.dtype_code(dt), int(op), STREAM()))
                res = []
                for _ in range(3):
                    for i in range(sets):
                        assert calls[i]() == 0
                    torch.cuda.synchronize()
                    ev = Events(lib, stream)
                    ev.start()
                    for i in range(launches):
                        calls[i % sets]()
                    res.append((n + 1) * numel * es / (ev.stop_ms() / launches) / 1e6 / HBM_PEAK_GBS)
                cells.append(f"{sorted(res)[1]:.3f}")
            print(f"| {str(dt)[6:]} | {n} | " + " | ".join(cells) + " |", flush=True)
            del bufs, calls
            torch.cuda.empty_cache()


STRIDED_VIEWS_HEADER = """\
# Strided pack / unpack of one column range: row length x alignment (MI355X)

Command (repository root, one GPU; under a minute):

    python bench.py --sweep strided_views > profiles/strided_views_map.md

Every cell is the fraction of the 8 TB/s HBM peak that `mhip_slice_pack` / `mhip_slice_unpack` reach on the view
`x[:, c0:c0 + cols]` of a `[16384, pitch]` matrix whose rows are 28 KiB apart (algorithmic bytes = 2 x elements x
element size); median of 3 runs of {launches} launches, 3 rotating buffer sets.  Rows of a multiple of 16 bytes take the
whole-chunk form (line by line when a view of 96 MiB and more does not start and end its rows on cache lines), other
rows the two-vector form when packed (the gathering form under 4 KiB where shape and pitch are 4-byte granular) and the
line-by-line form when unpacked; a view that starts off the unit of its shape (c0 = 1) is moved in that unit from a
skewed base.  Views of 59 MB and less (rows of 1792 bytes and less) partly live in the 256 MB Infinity Cache across the
three buffer sets; the larger ones do not.
"""


def sweep_strided_views(dtypes, launches=20):
    """Fraction of HBM peak of single-view strided packs and unpacks over row lengths and starting columns
    (--sweep strided_views): whole-chunk rows, ragged rows, views that start off the unit of their shape."""
    torch, lib, _ = _load()
    from monarch_amd import Slice
    torch.cuda.set_device(0)
    stream = C.c_void_p(torch.cuda.current_stream().cuda_stream)
    types = {"u8": (torch.uint8, 1), "bf16": (torch.bfloat16, 2), "f32": (torch.float32, 4), "f64": (torch.float64, 8)}
    rows, pitch_bytes = 16384, 28672
    print(STRIDED_VIEWS_HEADER.format(launches=launches))
    for name in dtypes:
        dt, es = types[name]
        pitch = pitch_bytes // es
        bufs = []
        for _ in range(3):
            x = torch.empty(rows, pitch, dtype=dt, device="cuda:0")
            x.view(torch.uint8).random_(0, 255)
            bufs.append((x, torch.empty(rows * pitch // 2, dtype=dt, device="cuda:0")))
        print(f"\n### {name} ({es}-byte elements), pitch {pitch}\n")
        print("| cols (row bytes) | c0 | pack | unpack |")
        print("|---|---:|---:|---:|")
        for row_bytes in (1788, 1792, 3580, 3584, 7160, 7168, 14332, 14336):
            cols = row_bytes // es
            for c0 in (0, 1, 16 // es):
                if c0 + cols > pitch:
                    continue
                s = Slice.of_tensor(bufs[0][0][:, c0:c0 + cols])
                cell = []
                for sym in ("mhip_slice_pack", "mhip_slice_unpack"):
                    if sym.endswith("unpack"):
                        calls = [prepared(sym, x.data_ptr(), st.data_ptr(), C.byref(s.c), es, STREAM()) for x, st in bufs]
                    else:
                        calls = [prepared(sym, st.data_ptr(), x.data_ptr(), C.byref(s.c), es, STREAM()) for x, st in bufs]
                    res = []
                    for _ in range(3):
                        for i in range(3):
                            assert calls[i % 3]() == 0
                        torch.cuda.synchronize()
                        ev = Events(lib, stream)
                        ev.start()
                        for i in range(launches):
                            calls[i % 3]()
                        res.append(2 * rows * cols * es / (ev.stop_ms() / launches) / 1e6 / HBM_PEAK_GBS)
                    cell.append(sorted(res)[1])
                print(f"| {cols} ({cols * es}) | {c0} | {cell[0]:.3f} | {cell[1]:.3f} |", flush=True)
        del bufs, calls
        torch.cuda.empty_cache()


BUCKET_SIZES_HEADER = """\
# The stages of configuration 5 on buckets of a few to a hundred million elements (MI355X)

Command (repository root, one GPU; under a minute):

    python bench.py --sweep bucket_sizes > profiles/fp8_bucket_sizes.md

Buckets of bf16 tensors with `round(exp(U(ln 2^10, ln 2^21)))` elements each (numpy `default_rng(total in M)`), drawn
until the bucket holds the stated number of elements, every tensor an allocation of its own; the flat buffers, codes,
scales and fp32 accumulators beside them.  Every cell is the time of one launch in microseconds and, in brackets, the
fraction of the 8 TB/s HBM peak its algorithmic bytes make of it (flat pack 4 T, quantise 3 T + 4 B, dequantise and
accumulate 9 T + 4 B, flat unpack of fp32 8 T; T elements, B blocks of 1024): median of 3 runs of {launches} launches,
3 rotating bucket sets, all forms with the bucket's block index.  A launch of a few MB is bound by its longest
wavefront, not by bandwidth: the rows show what the rare paths of the fused kernels (tensor boundaries inside a span,
the short last block) cost there.
"""


def sweep_bucket_sizes(launches=30):
    """Time per launch of the flat-bucket and fp8 stages against the bucket's size (--sweep bucket_sizes)."""
    import numpy as np
    torch, lib, _ = _load()
    from monarch_amd import fp8
    torch.cuda.set_device(0)
    stream = C.c_void_p(torch.cuda.current_stream().cuda_stream)
    stages = ("flat_pack", "quantize", "quantize_bucket", "dequant", "dequant_bucket", "flat_unpack")
    print(BUCKET_SIZES_HEADER.format(launches=launches))
    print("| elements | tensors | " + " | ".join(stages) + " |")
    print("|---:|---:|" + "---:|" * len(stages))
    for total_m in (4, 13, 32, 64, 128):
        rng = np.random.default_rng(total_m)
        sizes = []
        while sum(sizes) < total_m << 20:
            sizes.append(int(round(np.exp(rng.uniform(np.log(2 ** 10), np.log(2 ** 21))))))
        total, n = sum(sizes), len(sizes)
        nblk = (total + 1023) // 1024
        sets = []
        for _ in range(3):
            tensors = [torch.empty(k, dtype=torch.bfloat16, device="cuda:0").normal_() for k in sizes]
            bucket = fp8.FlatBucket(tensors)
            flat = bucket.pack()
            q, sc = fp8.quantize(flat)
            accs = [torch.zeros(k, device="cuda:0") for k in sizes]
            outs = [torch.empty(k, device="cuda:0") for k in sizes]
            sets.append(dict(bucket=bucket, tensors=tensors, flat=flat, q=q, s=sc, acc=torch.zeros(total, device="cuda:0"), accs=accs,
                             outs=outs, aptrs=bucket.pointer_table(accs), optrs=bucket.pointer_table(outs),
                             index=bucket.block_index().data_ptr()))
        torch.cuda.synchronize()
        cells = []
        for stage in stages:
            calls = []
            for d in sets:
                b = d["bucket"]
                tables = (b.d_offsets.data_ptr(), n, total)
                if stage == "flat_pack":
                    nbytes = 4 * total
                    calls.append(prepared("mhip_flat_pack", d["flat"].data_ptr(), b.d_ptrs.data_ptr(), *tables, 2, d["index"], STREAM()))
                elif stage == "quantize":
                    nbytes = 3 * total + 4 * nblk
                    calls.append(prepared("mhip_fp8_quantize", d["q"].data_ptr(), d["s"].data_ptr(), d["flat"].data_ptr(), total, 1024, STREAM()))
                elif stage == "quantize_bucket":
                    nbytes = 3 * total + 4 * nblk
                    calls.append(prepared("mhip_fp8_quantize_bucket", d["q"].data_ptr(), d["s"].data_ptr(), b.d_ptrs.data_ptr(), *tables, 1024,
                                          d["index"], STREAM()))
                elif stage == "dequant":
                    nbytes = 9 * total + 4 * nblk
                    calls.append(prepared("mhip_fp8_dequant_accumulate", d["acc"].data_ptr(), d["q"].data_ptr(), d["s"].data_ptr(), total, 1024,
                                          STREAM()))
                elif stage == "dequant_bucket":
                    nbytes = 9 * total + 4 * nblk
                    calls.append(prepared("mhip_fp8_dequant_accumulate_bucket", d["aptrs"].data_ptr(), d["q"].data_ptr(), d["s"].data_ptr(),
                                          *tables, 1024, d["index"], STREAM()))
                else:
                    nbytes = 8 * total
                    calls.append(prepared("mhip_flat_unpack", d["optrs"].data_ptr(), d["acc"].data_ptr(), *tables, 4, d["index"], STREAM()))
            res = []
            for _ in range(3):
                for c in calls:
                    assert c() == 0
                torch.cuda.synchronize()
                ev = Events(lib, stream)
                ev.start()
                for i in range(launches):
                    calls[i % 3]()
                res.append(ev.stop_ms() / launches * 1e3)
            us = sorted(res)[1]
            cells.append(f"{us:.1f} ({nbytes / us / 1e3 / HBM_PEAK_GBS:.2f})")
        print(f"| {total} | {n} | " + " | ".join(cells) + " |", flush=True)
        del sets, calls
        torch.cuda.empty_cache()


# The default run reports these beside the headline workload, measured in the same process:
# workload -> fraction of HBM peak that BASELINE.json's north star asks of its class (None: no target stated)
SUMMARY = {
    "c2": 0.75, "c2_inplace": 0.75, "c2_separate": 0.75, "c2_cold": 0.75, "c2p_pack": 0.75, "c2p_unpack": 0.75,
    "c3_pack": 0.60, "c3_unpack": 0.60, "c3_reshard_e2e": 0.60, "ragged_pack": 0.60, "ragged_unpack": 0.60,
    "c4": 0.60, "c4_slots": 0.60, "c4_cold": 0.60,
    "c5_flat_pack": 0.60, "c5_quantize": 0.60, "c5_dequant": 0.60, "c5_flat_unpack": 0.60,
    "c5_quantize_bucket": 0.60, "c5_dequant_bucket": 0.60, "c5_dequant_many8": 0.60,
    "stack8": None, "stack_scatter8": None,
    "c5_dequant_bucket_arena": None,   # c5_dequant_bucket with the 1500 accumulators inside one allocation
    "ref_copy_hip": None, "ref_copy_torch": None,   # not this library: hipMemcpyAsync and torch's copy_ on the c2p buffers
    "tr_f32_pack": None, "tr_f32_unpack": None, "tr_bf16_pack": None, "tr_bf16_unpack": None,
    "tr_bf16_8200_pack": None, "tr_bf16_8200_unpack": None, "tr_u8_8200_pack": None, "tr_u8_8200_unpack": None,
    # configuration 1 (1 MiB views): launch-bound, reported as time per call
    "c1_pack": None, "c1_unpack": None, "c1_reduce": None, "c1_pipeline": None, "c1_pipeline_fused": None,
}


def sig(x, digits=4):
    """x rounded to `digits` significant digits (the bench line has to stay short enough for the driver's tail)."""
    if x is None or x == 0 or x != x:
        return x
    from math import floor, log10
    return round(x, digits - 1 - floor(log10(abs(x))))


INFINITY_CACHE_BYTES = 256 << 20
# workloads that are pipelines of launches in which a kernel reads what the one before it has just written
PIPELINES = ("c3_reshard_e2e", "c3_reshard_e2e_one_by_one", "c1_pipeline", "c1_pipeline_fused")


def measure(torch, lib, workload: str, steps: int, warmup: int):
    torch.cuda.synchronize()
    held_before, free_before = torch.cuda.memory_allocated(), torch.cuda.mem_get_info()[0]
    name, nbytes, launch, cpu, kernel, dtype = WORKLOADS[workload](torch)
    torch.cuda.synchronize()
    # device memory of the workload's rotating buffer sets: what one rotation walks through.  Staging areas are mapped
    # by the library, not by torch, hence the device's own free-memory figure beside torch's.  (The C5 stages share one
    # set of buffers made by the first of them; each of their launches alone moves 3 GB and more.)
    rotation = max(torch.cuda.memory_allocated() - held_before, free_before - torch.cuda.mem_get_info()[0], nbytes)
    stream = C.c_void_p(torch.cuda.current_stream().cuda_stream)
    rc = 0
    for i in range(warmup):
        rc |= launch(i)
    torch.cuda.synchronize()
    ev = Events(lib, stream)
    t0 = time.perf_counter()
    ev.start()
    for i in range(steps):
        rc |= launch(i)
    kernel_ms = ev.stop_ms() / steps
    if rc != 0:
        sys.exit(f"a launch of {workload} returned status {rc}")
    torch.cuda.synchronize()
    wall_ms = (time.perf_counter() - t0) * 1e3 / steps
    # a figure quoted against the HBM peak is cache-assisted when a rotation is short enough for a good part of it to stay
    # in the 256 MB Infinity Cache, or when a kernel of the step reads what the previous one wrote
    assisted = rotation < 2 * INFINITY_CACHE_BYTES or workload in PIPELINES
    return dict(name=name, nbytes=nbytes, cpu=cpu, kernel=kernel, dtype=dtype, kernel_ms=kernel_ms, wall_ms=wall_ms,
                keep=launch, rotation=rotation, cache_assisted=assisted)


def short_cpu(cpu: dict) -> dict:
    """A workload's CPU legs as GB/s figures only: 1-core port of the reference loop, the same on all cores, torch CPU."""
    out = {"port": sig(cpu["value"], 3)}
    if "all_cores" in cpu:
        out["all_cores"] = sig(cpu["all_cores"]["value"], 3)
    if "torch_cpu" in cpu:
        out["torch"] = sig(cpu["torch_cpu"]["value"], 3)
    return out


def run(workload: str, steps: int, warmup: int, cpu_baseline: bool, summary: bool = False):
    torch, lib, _ = _load()
    torch.cuda.set_device(0)
    traffic = measured_traffic()
    m = measure(torch, lib, workload, steps, warmup)
    nbytes = m["nbytes"]
    achieved = nbytes / (m["kernel_ms"] * 1e-3) / 1e9
    rec = {
        "metric": METRIC, "value": sig(nbytes / (m["wall_ms"] * 1e-3) / 1e9, 6), "unit": "GB/s", "n_gpus": 1,
        "steps": steps, "warmup": warmup, "ms_per_step": sig(m["wall_ms"], 6), "higher_is_better": True,
        "scaling": "weak", "vs_baseline": None, "dtype": m["dtype"], "data": "synthetic",
        "config": {"workload": m["name"], "algorithmic_bytes_per_step": nbytes, "kernel": m["kernel"],
                   **({"layout": LAYOUT[workload]} if workload in LAYOUT else {})},
        "roofline": {"bound": "hbm", "achieved": sig(achieved, 6), "peak": HBM_PEAK_GBS, "unit": "GB/s",
                     "frac": sig(achieved, 6) / HBM_PEAK_GBS, "traffic": traffic.get(workload, {}).get("traffic"),
                     "traffic_source": TRAFFIC_SOURCE,
                     # what one rotation of the buffer sets walks through; under 2 x 256 MB part of it stays in the
                     # Infinity Cache.  frac_cold: the same kernel rotating over 8 sets (3.6 GB), filled in by the default run
                     "rotation_bytes": m["rotation"], "cache_assisted": m["cache_assisted"], "frac_cold": None},
    }
    if cpu_baseline:
        rec["cpu_baseline"] = m["cpu"]()
        rec["cpu_baseline"]["host_cpus"] = os.cpu_count()
    if summary:
        # every other class of the path, same process, same method (HIP events on the launch stream, rotating buffer
        # sets), fewer launches; short entries (`--all` prints every workload's full record); the CPU legs here are the
        # short ones (the headline's own leg runs above)
        import gc
        k_steps, k_warm = max(5, min(steps, 60)), max(2, min(warmup, 10))
        cpu_legs = ("c2p_pack", "c3_pack", "c3_reshard_e2e", "c4", "c5_quantize", "c5_dequant", "stack8", "c1_pack", "c1_reduce")

        def entry(w, mm, with_cpu):
            frac = mm["nbytes"] / (mm["kernel_ms"] * 1e-3) / 1e9 / HBM_PEAK_GBS
            t = traffic.get(w, {}).get("traffic")
            e = {"ms": sig(mm["kernel_ms"]), "frac": sig(frac), "target": SUMMARY[w], "bytes": mm["nbytes"],
                 "traffic_x": sig(t / mm["nbytes"]) if t else None, "rot_mb": int(mm["rotation"] >> 20)}
            if mm["cache_assisted"]:
                e["cache_assisted"] = True
            if with_cpu:
                e["cpu"] = short_cpu(mm["cpu"]())
            return e

        out = {}
        if workload in SUMMARY:
            out[workload] = entry(workload, m, False)
        m = None
        for w in SUMMARY:
            if w in out:
                continue
            gc.collect()
            torch.cuda.empty_cache()  # the previous workload's buffer sets go back before the next ones are made
            mm = measure(torch, lib, w, k_steps, k_warm)
            out[w] = entry(w, mm, cpu_baseline and w in cpu_legs)
            mm = None
        # rows without a target first, rows that carry one last: a reader that keeps only the end of the line keeps those
        order = [w for w in SUMMARY if SUMMARY[w] is None] + [w for w in SUMMARY if SUMMARY[w] is not None]
        rec["workloads"] = {w: out[w] for w in order}
        if workload == "c2" and "c2_cold" in out:
            rec["roofline"]["frac_cold"] = out["c2_cold"]["frac"]
        rec["config"]["workloads_note"] = (f"{k_steps} launches after {k_warm}, HIP events; frac = bytes / ms / 8 TB/s; traffic_x = counter "
                                           "bytes / bytes; rot_mb = MiB one buffer rotation walks; cache_assisted: rotation < 512 MiB, or "
                                           "a kernel reads what the one before wrote; cpu: GB/s")
    release_shared()
    return rec


def main():
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=200)
    ap.add_argument("--warmup", type=int, default=20)
    ap.add_argument("--workload", default=None, choices=sorted(WORKLOADS))
    ap.add_argument("--all", action="store_true", help="also run every other workload with its own CPU leg; their lines go to stderr")
    ap.add_argument("--no-summary", action="store_true", help="leave out the `workloads` object of the default run")
    ap.add_argument("--no-cpu-baseline", action="store_true")
    ap.add_argument("--sweep", choices=sorted(SWEEPS) + ["strided_views", "bucket_sizes", "platform", "reduce_ops"], help="print a table instead of the bench line")
    ap.add_argument("--dtypes", default="u8,bf16,f32,f64", help="element types of --sweep")
    args = ap.parse_args()
    if args.gpus != 1:
        sys.exit("bench.py measures one GPU: this build has no multi-GPU path (run with --gpus 1)")
    if args.sweep == "reduce_ops":
        sweep_reduce_ops()
        return
    if args.sweep == "platform":
        sweep_platform()
        return
    if args.sweep == "bucket_sizes":
        sweep_bucket_sizes()
        return
    if args.sweep == "strided_views":
        sweep_strided_views([d for d in args.dtypes.split(",") if d != "f64"])
        return
    if args.sweep:
        sweep_transpose(args.sweep, args.dtypes.split(","))
        return
    headline = args.workload or "c2"
    if args.all:
        for w in sorted(WORKLOADS):
            if w != headline:
                rec = run(w, args.steps, args.warmup, not args.no_cpu_baseline)
                print(json.dumps(rec), file=sys.stderr, flush=True)
    # a named workload is a single measurement (what the profiler runs); the default run adds the summary
    summary = args.workload is None and not args.no_summary
    print(json.dumps(run(headline, args.steps, args.warmup, not args.no_cpu_baseline, summary)), flush=True)


if __name__ == "__main__":
    main()
