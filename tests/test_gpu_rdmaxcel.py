"""Device-built work-queue / completion-queue entries against the oracle, byte for byte.

The queues are ordinary device memory standing in for the mlx5dv_qp / mlx5dv_cq buffers; the flow follows the
reference's GPU helpers (monarch_rdma/src/test_utils.rs:131-257: send_wqe_gpu, recv_wqe_gpu, ring_db_gpu,
wait_for_completion_gpu) and its wrap-around test (rdma_manager_actor_tests.rs:520-575: four sends fill the queue,
the fifth wraps).  The completion entries a NIC would write are written by the test.  Every kernel here looks at
its queue once and exits; nothing spins.
"""
import ctypes as C

import numpy as np
import pytest
import torch

import oracle
from monarch_amd import _lib
from monarch_amd._lib import CqePollParamsC, WqeParamsC, check, lib
from monarch_amd.rdmaxcel import (MLX5_OPCODE_RDMA_READ, MLX5_OPCODE_RDMA_WRITE, MLX5_OPCODE_RDMA_WRITE_IMM, CompletionQueue,
                                  PollTarget, QueuePair, RegisteredBuffer)

pytestmark = pytest.mark.gpu
FILL = 0xEE


def dev_bytes(n, fill=FILL):
    return torch.full((n,), fill, dtype=torch.uint8, device="cuda")


def host(t):
    torch.cuda.synchronize()
    return t.cpu().numpy().copy()


def stream():
    return int(torch.cuda.current_stream().cuda_stream)


def wqe(buf, dbrec, wqe_cnt, *, laddr=0, lkey=0, length=0, wr_id=0, signaled=True, op_type=0, raddr=0, rkey=0, qp_num=0, buf_offset=0):
    return WqeParamsC(laddr, lkey, length, wr_id, 1 if signaled else 0, op_type, raddr, rkey, qp_num, buf.data_ptr() + buf_offset,
                      dbrec.data_ptr(), wqe_cnt)


def random_fields(rng):
    return dict(laddr=int(rng.integers(0, 2**63)) * 2 + 1, lkey=int(rng.integers(0, 2**32)), length=int(rng.integers(0, 2**40)),
                wr_id=int(rng.integers(0, 2**34)), signaled=bool(rng.integers(0, 2)),
                op_type=int(rng.choice([MLX5_OPCODE_RDMA_WRITE, MLX5_OPCODE_RDMA_WRITE_IMM, MLX5_OPCODE_RDMA_READ, 0xFF])),
                raddr=int(rng.integers(0, 2**63)), rkey=int(rng.integers(0, 2**32)), qp_num=int(rng.integers(0, 2**32)))


def test_send_and_recv_wqe_bytes_match_oracle():
    rng = np.random.default_rng(77)
    L = lib()
    # the hand-derived case of tests/test_oracle_rdmaxcel.py first, then random ones; several posts into one queue
    cases = [(4, dict(laddr=0x00007F1234567890, lkey=0xAABBCCDD, length=0x00100000, wr_id=5, signaled=True, op_type=0x08,
                      raddr=0x00007E00DEADBEE0, rkey=0x11223344, qp_num=0x001234)),
             (8, dict(laddr=0xFFFFFFFFFFFFFFF0, lkey=1, length=0x100000010, wr_id=0x01FFFFFF, signaled=False, op_type=0x10,
                      raddr=0x0102030405060708, rkey=0x80000000, qp_num=0xFFFFFFFF))]
    cases += [(1 << int(rng.integers(0, 8)), random_fields(rng)) for _ in range(40)]
    for cnt, f in cases:
        sq, dbrec = dev_bytes(cnt * 64), torch.tensor([0x11111111, 0x22222222], dtype=torch.int64, device="cuda").to(torch.int32)
        want_sq, want_db = np.full(cnt * 64, FILL, dtype=np.uint8), np.array([0x11111111, 0x22222222], dtype=np.uint32)
        p = wqe(sq, dbrec, cnt, **f)
        check(L.mhip_rdmaxcel_send_wqe(C.byref(p), stream()))
        oracle.send_wqe(want_sq, want_db, cnt, **f)
        slot = int(rng.integers(0, cnt)) * 64 + 16 * int(rng.integers(0, 4))
        p = wqe(sq, dbrec, cnt, buf_offset=slot, **f)
        check(L.mhip_rdmaxcel_recv_wqe(C.byref(p), stream()))
        oracle.recv_wqe(want_sq, want_db, cnt, buf_offset=slot, **f)
        assert host(sq).tobytes() == want_sq.tobytes(), (cnt, f)
        assert host(dbrec).view(np.uint32).tobytes() == want_db.tobytes(), (cnt, f)
    # the first case's bytes, spelled out: a check that does not go through the oracle
    sq, dbrec = dev_bytes(4 * 64), torch.zeros(2, dtype=torch.int32, device="cuda")
    p = wqe(sq, dbrec, 4, **cases[0][1])
    check(L.mhip_rdmaxcel_send_wqe(C.byref(p), stream()))
    assert host(sq)[64:112].tobytes() == bytes.fromhex(
        "00000508" "00123403" "0000000A" "00000000" "00007E00DEADBEE0" "11223344" "00000000" "00100000" "AABBCCDD" "00007F1234567890")
    assert host(dbrec).view(np.uint8).tobytes() == bytes.fromhex("00000000" "00000006")


def test_wr_id_wraps_past_the_queue_like_the_reference_wraparound_test():
    # rdma_manager_actor_tests.rs:520-575: a queue of four, five posts; the fifth lands in slot 0 again
    L = lib()
    cnt = 4
    sq, dbrec = dev_bytes(cnt * 64), torch.zeros(2, dtype=torch.int32, device="cuda")
    want_sq, want_db = np.full(cnt * 64, FILL, dtype=np.uint8), np.zeros(2, dtype=np.uint32)
    for i in range(5):
        f = dict(laddr=0x7000_0000_0000 + i * 4096, lkey=17, length=(1 << 20) * (2 if i == 4 else 1), wr_id=i, signaled=True,
                 op_type=MLX5_OPCODE_RDMA_WRITE, raddr=0x6000_0000_0000, rkey=23, qp_num=0x4A)
        p = wqe(sq, dbrec, cnt, **f)
        check(L.mhip_rdmaxcel_send_wqe(C.byref(p), stream()))
        oracle.send_wqe(want_sq, want_db, cnt, **f)
    got = host(sq)
    assert got.tobytes() == want_sq.tobytes()
    assert got[0:4].tobytes() == bytes.fromhex("00000408") and got[32:36].tobytes() == bytes.fromhex("00200000")  # slot 0 holds post 4
    assert host(dbrec).view(np.uint8)[4:].tobytes() == bytes.fromhex("00000005")


def test_doorbell_rings():
    L = lib()
    src = torch.arange(256, dtype=torch.int32, device="cuda").to(torch.uint8)
    dst = dev_bytes(128)
    check(L.mhip_rdmaxcel_db_ring(dst.data_ptr() + 8, src.data_ptr() + 24, stream()))
    got = host(dst)
    want = np.full(128, FILL, dtype=np.uint8)
    oracle.db_ring(want[8:], host(src)[24:])
    assert got.tobytes() == want.tobytes() and got[8:72].tobytes() == bytes(range(24, 88))
    # the ring loop of RdmaQueuePair::ring_doorbell: what the register holds after rings k = 6, 7, 8 of a queue of 4
    # slots with stride 64 is the slot of the last one, (8 % 4) = 0
    reg = dev_bytes(64)
    check(L.mhip_rdmaxcel_ring_doorbells(reg.data_ptr(), src.data_ptr(), 64, 4, 6, 3, stream()))
    assert host(reg).tobytes() == bytes(range(0, 64))
    check(L.mhip_rdmaxcel_ring_doorbells(reg.data_ptr(), src.data_ptr(), 64, 4, 6, 2, stream()))
    assert host(reg).tobytes() == bytes(range(192, 256))            # k = 7 -> slot 3
    check(L.mhip_rdmaxcel_ring_doorbells(reg.data_ptr(), src.data_ptr(), 128, 2, 0xFFFFFFFF, 1, stream()))
    assert host(reg).tobytes() == bytes(range(128, 192))            # 0xFFFFFFFF % 2 = 1, stride 128


def write_cqe(cq_host, cqe_size, entry, op_own, byte_cnt):
    base = entry * cqe_size
    cq_host[base + 44:base + 48] = np.frombuffer(int(byte_cnt & 0xFFFFFFFF).to_bytes(4, "big"), dtype=np.uint8)
    cq_host[base + cqe_size - 1] = op_own


@pytest.mark.parametrize("cqe_size", [64, 128])
def test_cqe_poll_two_laps_against_oracle(cqe_size):
    # Two laps of a queue of four: the owner bit a NIC writes flips per lap; entries start as never written
    # (opcode 0xF), become good completions, one bad opcode, and the poll is a single look each time.
    L = lib()
    cnt = 4
    cq_host = np.zeros(cqe_size * cnt, dtype=np.uint8)
    cq_host[cqe_size - 1::cqe_size] = 0xF0                                  # invalid opcode: not owned by software
    cq = torch.from_numpy(cq_host.copy()).cuda()
    dbrec = torch.full((2,), 0x5A5A5A5A, dtype=torch.int32, device="cuda")
    want_db = np.full(2, 0x5A5A5A5A, dtype=np.uint32)
    result = torch.full((1,), -1, dtype=torch.int32, device="cuda")

    def poll(ci):
        result.fill_(-1)
        p = CqePollParamsC(cq.data_ptr(), cqe_size, ci, cnt, dbrec.data_ptr())
        check(L.mhip_rdmaxcel_cqe_poll(result.data_ptr(), C.byref(p), stream()))
        got = int(host(result)[0])
        want = oracle.cqe_poll(cq_host, want_db, cqe_size, cnt, ci)
        assert got == want, (ci, got, want)
        assert host(dbrec).view(np.uint32).tobytes() == want_db.tobytes(), ci
        return got

    assert poll(0) == -1                                                     # nothing written yet: left untouched
    for ci in range(8):
        lap, entry = ci // cnt, ci % cnt
        assert poll(ci) == -1                                                # the entry still belongs to the NIC (stale lap or 0xF)
        opcode = 0xD if ci == 6 else (0, 1, 2, 3)[ci % 4]                    # ci 6: a completion with error
        write_cqe(cq_host, cqe_size, entry, (opcode << 4) | (lap & 1), 4096 * (ci + 1))
        cq.copy_(torch.from_numpy(cq_host))
        assert poll(ci) == (-2 if ci == 6 else 4096 * (ci + 1))
        assert int.from_bytes(want_db[:1].tobytes(), "big") == ci + 1        # the record follows the consumer index
    assert poll(8) == -1                                                     # lap 2 wants owner bit 0; entry 0 still carries lap 1's bit


def test_cqe_poll_result_word_is_left_alone_when_not_owned():
    L = lib()
    cq = torch.zeros(64 * 2, dtype=torch.uint8, device="cuda")
    cq[63] = 0x01                                                            # lap 0 wants owner bit 0
    dbrec = torch.tensor([123, 456], dtype=torch.int32, device="cuda")
    result = torch.tensor([-1, 99], dtype=torch.int32, device="cuda")
    p = CqePollParamsC(cq.data_ptr(), 64, 0, 2, dbrec.data_ptr())
    check(L.mhip_rdmaxcel_cqe_poll(result.data_ptr(), C.byref(p), stream()))
    assert host(result).tolist() == [-1, 99] and host(dbrec).tolist() == [123, 456]
    result[0] = 77                                                           # whatever the caller left there stays, too
    check(L.mhip_rdmaxcel_cqe_poll(result.data_ptr(), C.byref(p), stream()))
    assert host(result).tolist() == [77, 99]


def test_post_transfer_equals_sequential_send_wqes():
    L = lib()
    rng = np.random.default_rng(5)
    for cnt, length, seg, wr_id in [(8, 5 * 4096 + 17, 4096, 0), (8, 8 * 4096, 4096, 6), (4, 0, 0, 3), (8, 1 << 33, 0, 0xFFFFFF),
                                    (2048, 1500 * 8192 - 5, 8192, 0x00FFFFF0), (16, 3 << 30, 1 << 30, 14), (4, 100, 1 << 40, 1)]:
        f = random_fields(rng)
        f.update(length=length, wr_id=wr_id)
        sq, dbrec = dev_bytes(cnt * 64), torch.tensor([9, 9], dtype=torch.int32, device="cuda")
        p = wqe(sq, dbrec, cnt, **f)
        n = C.c_uint32()
        check(L.mhip_rdmaxcel_post_transfer(C.byref(p), seg, C.byref(n), stream()))
        eff = seg if 0 < seg <= (1 << 31) - 16 else (1 << 31) - 16
        want_n = max(1, -(-length // eff))
        assert n.value == want_n
        want_sq, want_db = np.full(cnt * 64, FILL, dtype=np.uint8), np.array([9, 9], dtype=np.uint32)
        for i in range(want_n):
            g = dict(f)
            g.update(laddr=f["laddr"] + i * eff, raddr=f["raddr"] + i * eff, length=min(eff, length - i * eff), wr_id=wr_id + i)
            oracle.send_wqe(want_sq, want_db, cnt, **g)
        assert host(sq).tobytes() == want_sq.tobytes(), (cnt, length, seg)
        assert host(dbrec).view(np.uint32).tobytes() == want_db.tobytes(), (cnt, length, seg)


def test_queue_pair_flow_like_the_reference_gpu_helpers():
    # send_wqe_gpu -> ring_db_gpu -> (the NIC completes) -> wait_for_completion_gpu, with the reference's counters
    cnt = 4
    sq, rq = dev_bytes(cnt * 64, 0), dev_bytes(cnt * 16, 0)
    dbrec, reg = torch.zeros(2, dtype=torch.int32, device="cuda"), dev_bytes(64, 0)
    scq, rcq = torch.zeros(64 * cnt, dtype=torch.uint8, device="cuda"), torch.zeros(64 * cnt, dtype=torch.uint8, device="cuda")
    scq[63::64] = 0xF0
    rcq[63::64] = 0xF0
    cqdb = torch.zeros(4, dtype=torch.int32, device="cuda")
    result = torch.full((1,), -1, dtype=torch.int32, device="cuda")
    qp = QueuePair(qp_num=0x77, sq_buf=sq.data_ptr(), sq_wqe_cnt=cnt, rq_buf=rq.data_ptr(), rq_wqe_cnt=cnt, dbrec=dbrec.data_ptr(),
                   bf_reg=reg.data_ptr(), send_cq=CompletionQueue(scq.data_ptr(), 64, cnt, cqdb.data_ptr()),
                   recv_cq=CompletionQueue(rcq.data_ptr(), 64, cnt, cqdb.data_ptr() + 8), poll_result=result.data_ptr())
    local, remote = RegisteredBuffer(0x7000_0000, 1 << 20, lkey=5, rkey=6), RegisteredBuffer(0x9000_0000, 1 << 20, lkey=7, rkey=8)
    s = stream()
    for i in range(6):                                                    # six puts through a queue of four
        qp.enqueue_put(local, remote, s)
        assert qp.send_wqe_idx == i + 1 and qp.send_db_idx == i
        qp.ring_doorbell(s)
        assert qp.send_db_idx == i + 1
        got_reg, got_sq = host(reg), host(sq)
        assert got_reg.tobytes() == got_sq[(i % cnt) * 64:(i % cnt) * 64 + 64].tobytes()      # the register received this post's slot
        assert got_sq[(i % cnt) * 64:(i % cnt) * 64 + 4].tobytes() == bytes([0, 0, i, MLX5_OPCODE_RDMA_WRITE])
        qp.launch_cqe_poll(PollTarget.Send, s)
        assert not qp.completed(PollTarget.Send, int(host(result)[0]))    # not completed yet
        scq[(i % cnt) * 64 + 44:(i % cnt) * 64 + 48] = torch.tensor([0, 0x10, 0, 0], dtype=torch.uint8, device="cuda")
        scq[(i % cnt) * 64 + 63] = (i // cnt) & 1                         # the NIC's completion: opcode 0, this lap's owner bit
        qp.launch_cqe_poll(PollTarget.Send, s)
        assert qp.completed(PollTarget.Send, int(host(result)[0])) and int(host(result)[0]) == 1 << 20
        result.fill_(-1)
        assert qp.send_cq_idx == i + 1
    assert host(dbrec).view(np.uint8)[4:].tobytes() == bytes.fromhex("00000006")
    assert host(cqdb).view(np.uint8)[:4].tobytes() == bytes.fromhex("00000006")
    # a receive: zero-length segment at the receive queue's start, receive record = index + 1
    qp.recv(local, remote, s)
    assert host(rq)[:16].tobytes() == bytes.fromhex("00000000" "00000005" "0000000000000000")
    assert host(dbrec).view(np.uint8)[:4].tobytes() == bytes.fromhex("00000001")
    # posting more than the queue holds before ringing is the reference's overflow error
    for _ in range(5):
        qp.enqueue_get(local, remote, s)
    with pytest.raises(RuntimeError, match="Overflow of WQE"):
        qp.ring_doorbell(s)
    # a chained transfer takes several slots in one launch
    qp2 = QueuePair(qp_num=1, sq_buf=sq.data_ptr(), sq_wqe_cnt=cnt, rq_buf=rq.data_ptr(), rq_wqe_cnt=cnt, dbrec=dbrec.data_ptr(),
                    bf_reg=reg.data_ptr(), send_cq=qp.send_cq, recv_cq=qp.recv_cq, poll_result=result.data_ptr())
    assert qp2.enqueue_transfer(local, remote, max_segment_bytes=1 << 18, stream=s) == 4 and qp2.send_wqe_idx == 4
    with pytest.raises(RuntimeError, match="Overflow of WQE"):
        qp2.enqueue_transfer(local, remote, max_segment_bytes=1 << 18, stream=s)
    qp2.ring_doorbell(s)
    assert host(reg).tobytes() == host(sq)[192:256].tobytes()
    torch.cuda.synchronize()


def test_host_mode_queue_pair_on_host_memory_gives_the_same_bytes():
    # the host functions the reference's Rust calls directly, on pinned host memory the device forms can reach too
    cnt = 4
    sq_h = torch.zeros(cnt * 64, dtype=torch.uint8).pin_memory()
    db_h = torch.zeros(2, dtype=torch.int32).pin_memory()
    reg_h = torch.zeros(64, dtype=torch.uint8).pin_memory()
    cq_h = torch.zeros(64 * cnt, dtype=torch.uint8).pin_memory()
    cqdb_h = torch.zeros(2, dtype=torch.int32).pin_memory()
    res = (C.c_int32 * 1)(-1)
    host_qp = QueuePair(qp_num=9, sq_buf=sq_h.data_ptr(), sq_wqe_cnt=cnt, rq_buf=sq_h.data_ptr(), rq_wqe_cnt=cnt, dbrec=db_h.data_ptr(),
                        bf_reg=reg_h.data_ptr(), send_cq=CompletionQueue(cq_h.data_ptr(), 64, cnt, cqdb_h.data_ptr()),
                        recv_cq=CompletionQueue(cq_h.data_ptr(), 64, cnt, cqdb_h.data_ptr()), device=False,
                        poll_result=C.addressof(res))
    sq_d, db_d, reg_d = dev_bytes(cnt * 64, 0), torch.zeros(2, dtype=torch.int32, device="cuda"), dev_bytes(64, 0)
    dev_qp = QueuePair(qp_num=9, sq_buf=sq_d.data_ptr(), sq_wqe_cnt=cnt, rq_buf=sq_d.data_ptr(), rq_wqe_cnt=cnt, dbrec=db_d.data_ptr(),
                       bf_reg=reg_d.data_ptr(), send_cq=host_qp.send_cq, recv_cq=host_qp.recv_cq, poll_result=0)
    a, b = RegisteredBuffer(0x1234_5678_9AB0, 12345, lkey=1, rkey=2), RegisteredBuffer(0x0FED_CBA9_8760, 99999, lkey=3, rkey=4)
    for qp in (host_qp, dev_qp):
        qp.enqueue_put(a, b, stream())
        qp.enqueue_get(b, a, stream())
        qp.enqueue_put_with_recv(a, b, stream())
        qp.ring_doorbell(stream())
    torch.cuda.synchronize()
    assert sq_h.numpy().tobytes() == host(sq_d).tobytes()
    assert db_h.numpy().tobytes() == host(db_d).tobytes()
    assert reg_h.numpy().tobytes() == host(reg_d).tobytes()
    # a device-side poll of a completion queue that lives in pinned host memory (where a NIC's CQ is mapped from)
    cq_h[63::64] = 0xF0
    result = torch.full((1,), -1, dtype=torch.int32, device="cuda")
    dev_qp.poll_result = result.data_ptr()
    dev_qp.launch_cqe_poll(PollTarget.Send, stream())
    assert int(host(result)[0]) == -1
    cq_h[44:48] = torch.tensor([0, 0, 1, 0], dtype=torch.uint8)
    cq_h[63] = 0x00
    dev_qp.launch_cqe_poll(PollTarget.Send, stream())
    assert int(host(result)[0]) == 256 and cqdb_h.numpy().view(np.uint8)[:4].tobytes() == bytes.fromhex("00000001")
    host_qp.launch_cqe_poll(PollTarget.Send)
    assert res[0] == 256


def test_posting_ringing_and_polling_record_into_a_graph():
    # the entry points only enqueue kernels (no synchronisation, no allocation: the reference's launchers synchronise
    # the device per entry and allocate managed memory per poll), so a caller can record a post -> ring -> poll sequence
    # once and replay it; every replay, with a new completion written in between, must give the eager result
    L = lib()
    cnt = 4
    sq, dbrec, reg = dev_bytes(cnt * 64, 0), torch.zeros(2, dtype=torch.int32, device="cuda"), dev_bytes(64, 0)
    cq = torch.zeros(64 * cnt, dtype=torch.uint8, device="cuda")
    cq[63::64] = 0xF0
    cqdb = torch.zeros(2, dtype=torch.int32, device="cuda")
    result = torch.full((1,), -1, dtype=torch.int32, device="cuda")
    f = dict(laddr=0x7000_0000_1000, lkey=3, length=1 << 16, wr_id=2, signaled=True, op_type=MLX5_OPCODE_RDMA_WRITE_IMM,
             raddr=0x7100_0000_2000, rkey=4, qp_num=0x99)
    p = wqe(sq, dbrec, cnt, **f)
    c = CqePollParamsC(cq.data_ptr(), 64, 2, cnt, cqdb.data_ptr())
    side = torch.cuda.Stream()
    torch.cuda.synchronize()
    graph = torch.cuda.CUDAGraph()
    with torch.cuda.graph(graph, stream=side):
        s = stream()
        check(L.mhip_memset(result.data_ptr(), 0xFF, 4, s))
        check(L.mhip_rdmaxcel_send_wqe(C.byref(p), s))
        check(L.mhip_rdmaxcel_ring_doorbells(reg.data_ptr(), sq.data_ptr(), 64, cnt, 2, 1, s))
        check(L.mhip_rdmaxcel_cqe_poll(result.data_ptr(), C.byref(c), s))
    want_sq, want_db = np.zeros(cnt * 64, dtype=np.uint8), np.zeros(2, dtype=np.uint32)
    oracle.send_wqe(want_sq, want_db, cnt, **f)
    for rep, (op_own, count, want) in enumerate([(0xF0, 0, -1), (0x00, 4096, 4096), (0xD0, 0, -2), (0x01, 7, -1)]):
        sq.zero_(); dbrec.zero_(); reg.zero_(); cqdb.zero_()
        cq[2 * 64 + 44:2 * 64 + 48] = torch.tensor(list(int(count).to_bytes(4, "big")), dtype=torch.uint8, device="cuda")
        cq[2 * 64 + 63] = op_own
        other = torch.randn(1 << 16, device="cuda").sum()   # unrelated eager work between replays
        graph.replay()
        assert int(host(result)[0]) == want, rep
        assert host(sq).tobytes() == want_sq.tobytes() and host(dbrec).view(np.uint32).tobytes() == want_db.tobytes(), rep
        assert host(reg).tobytes() == want_sq[128:192].tobytes(), rep
        assert int(host(cqdb)[0]) == (int.from_bytes((3).to_bytes(4, "big"), "little") if want != -1 else 0), rep
        assert torch.isfinite(other)
