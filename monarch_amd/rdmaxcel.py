"""Device-initiated RDMA bookkeeping over caller-owned queue memory.

``QueuePair`` mirrors the counters and method names of the reference's ``RdmaQueuePair``
(monarch_rdma/src/rdma_components.rs:470-500, 795-1002, 1107-1172) and of its GPU test helpers
(monarch_rdma/src/test_utils.rs:131-257: ``send_wqe_gpu``, ``recv_wqe_gpu``, ``ring_db_gpu``,
``wait_for_completion_gpu``), with the queue memory passed in as addresses: the send queue, the
receive queue, the doorbell record, the doorbell register and the two completion queues are whatever
the caller mapped (``mlx5dv_qp`` / ``mlx5dv_cq`` buffers, or ordinary memory in tests).  Every entry is
built by the library (``mhip_rdmaxcel_*``); this module only keeps the indices.

``device=True`` posts through kernels on a stream (the ``launch_*`` forms); ``device=False`` calls the
host functions the reference's Rust calls directly (rdma_components.rs:88, 880, 1159-1163).
"""
from __future__ import annotations

import ctypes as C
from dataclasses import dataclass
from enum import Enum
from typing import Optional

from ._lib import CqePollParamsC, WqeParamsC, check, lib

# <infiniband/mlx5dv.h> opcodes RdmaQueuePair::send_wqe maps RdmaOperation to (rdma_components.rs:1119-1124)
MLX5_OPCODE_RDMA_WRITE = 0x08
MLX5_OPCODE_RDMA_WRITE_IMM = 0x09
MLX5_OPCODE_RDMA_READ = 0x10
SEND_WQE_BYTES = 64  # MLX5_SEND_WQE_BB


class RdmaOperation(Enum):  # monarch_rdma/src/ibverbs_primitives.rs RdmaOperation
    Write = "write"
    Read = "read"
    Recv = "recv"
    WriteWithImm = "write_with_imm"


class PollTarget(Enum):  # rdma_components.rs PollTarget
    Send = "send"
    Recv = "recv"


_OPCODES = {RdmaOperation.Write: MLX5_OPCODE_RDMA_WRITE, RdmaOperation.WriteWithImm: MLX5_OPCODE_RDMA_WRITE_IMM,
            RdmaOperation.Read: MLX5_OPCODE_RDMA_READ, RdmaOperation.Recv: 0}


@dataclass
class RegisteredBuffer:
    """The fields of ``RdmaBuffer`` a work request carries (rdma_components.rs:94-102)."""
    addr: int
    size: int
    lkey: int = 0
    rkey: int = 0


@dataclass
class CompletionQueue:
    """``mlx5dv_cq`` fields ``launch_cqe_poll`` reads (rdmaxcel-sys/src/rdmaxcel.cu:371-376)."""
    buf: int
    cqe_size: int
    cqe_cnt: int
    dbrec: int


class QueuePair:
    def __init__(self, *, qp_num: int, sq_buf: int, sq_wqe_cnt: int, rq_buf: int, rq_wqe_cnt: int, dbrec: int, bf_reg: int,
                 send_cq: CompletionQueue, recv_cq: CompletionQueue, sq_stride: int = SEND_WQE_BYTES, rq_stride: int = 16,
                 device: bool = True, poll_result: Optional[int] = None):
        self.qp_num, self.sq_buf, self.sq_wqe_cnt, self.sq_stride = qp_num, sq_buf, sq_wqe_cnt, sq_stride
        self.rq_buf, self.rq_wqe_cnt, self.rq_stride = rq_buf, rq_wqe_cnt, rq_stride
        self.dbrec, self.bf_reg, self.send_cq, self.recv_cq = dbrec, bf_reg, send_cq, recv_cq
        self.device = device
        # a device word (device=True) or host int32 (device=False) that polls write to; the caller owns it
        self.poll_result = poll_result
        # rdma_components.rs:490-500
        self.send_wqe_idx = self.send_db_idx = self.send_cq_idx = 0
        self.recv_wqe_idx = self.recv_db_idx = self.recv_cq_idx = 0

    # -- rdma_components.rs:1107-1172 ------------------------------------------------------
    def send_wqe(self, laddr: int, lkey: int, length: int, wr_id: int, signaled: bool, op_type: RdmaOperation, raddr: int,
                 rkey: int, stream: int = 0) -> None:
        recv = op_type == RdmaOperation.Recv
        # the reference addresses the receive queue's start for every receive (rdma_components.rs:1137-1141)
        p = WqeParamsC(laddr, lkey, length, wr_id, 1 if signaled else 0, _OPCODES[op_type], raddr, rkey, self.qp_num,
                       self.rq_buf if recv else self.sq_buf, self.dbrec, self.sq_wqe_cnt)
        L = lib()
        if self.device:
            check((L.mhip_rdmaxcel_recv_wqe if recv else L.mhip_rdmaxcel_send_wqe)(C.byref(p), stream))
        else:
            check((L.mhip_rdmaxcel_recv_wqe_host if recv else L.mhip_rdmaxcel_send_wqe_host)(C.byref(p)))

    def _enqueue(self, op: RdmaOperation, lhandle: RegisteredBuffer, rhandle: RegisteredBuffer, stream: int) -> None:
        idx = self.send_wqe_idx
        self.send_wqe_idx += 1
        self.send_wqe(lhandle.addr, lhandle.lkey, lhandle.size, idx, True, op, rhandle.addr, rhandle.rkey, stream)

    def enqueue_put(self, lhandle, rhandle, stream: int = 0) -> None:  # rdma_components.rs:900-919
        self._enqueue(RdmaOperation.Write, lhandle, rhandle, stream)

    def enqueue_put_with_recv(self, lhandle, rhandle, stream: int = 0) -> None:  # :933-952
        self._enqueue(RdmaOperation.WriteWithImm, lhandle, rhandle, stream)

    def enqueue_get(self, lhandle, rhandle, stream: int = 0) -> None:  # :966-985
        self._enqueue(RdmaOperation.Read, lhandle, rhandle, stream)

    def recv(self, lhandle, rhandle, stream: int = 0) -> None:  # :803-819: a zero-length receive
        idx = self.recv_wqe_idx
        self.recv_wqe_idx += 1
        self.send_wqe(0, lhandle.lkey, 0, idx, True, RdmaOperation.Recv, 0, rhandle.rkey, stream)

    def enqueue_transfer(self, lhandle, rhandle, max_segment_bytes: int = 0, op: RdmaOperation = RdmaOperation.Write,
                         stream: int = 0) -> int:
        """``lhandle.size`` bytes as a chain of work requests in one launch (``mhip_rdmaxcel_post_transfer``);
        returns how many were posted.  Device mode only."""
        if not self.device:
            raise ValueError("enqueue_transfer posts from the device")
        room = self.sq_wqe_cnt - (self.send_wqe_idx - self.send_db_idx)
        p = WqeParamsC(lhandle.addr, lhandle.lkey, lhandle.size, self.send_wqe_idx, 1, _OPCODES[op], rhandle.addr, rhandle.rkey,
                       self.qp_num, self.sq_buf, self.dbrec, self.sq_wqe_cnt)
        seg = max_segment_bytes if max_segment_bytes else (1 << 31) - 16
        if max(1, -(-lhandle.size // seg)) > room:  # slots not yet handed to the NIC must not be overwritten
            raise RuntimeError("Overflow of WQE, possible data loss")
        n = C.c_uint32()
        check(lib().mhip_rdmaxcel_post_transfer(C.byref(p), max_segment_bytes, C.byref(n), stream))
        self.send_wqe_idx += n.value
        return n.value

    # -- rdma_components.rs:868-885 / test_utils.rs:191-209 ---------------------------------
    def ring_doorbell(self, stream: int = 0) -> None:
        if self.sq_wqe_cnt < self.send_wqe_idx - self.send_db_idx:
            raise RuntimeError("Overflow of WQE, possible data loss")
        count = self.send_wqe_idx - self.send_db_idx
        L = lib()
        if self.device:
            check(L.mhip_rdmaxcel_ring_doorbells(self.bf_reg, self.sq_buf, self.sq_stride, self.sq_wqe_cnt,
                                                 self.send_db_idx & 0xFFFFFFFF, count, stream))
        else:
            for k in range(self.send_db_idx, self.send_wqe_idx):
                check(L.mhip_rdmaxcel_db_ring_host(self.bf_reg, self.sq_buf + (k % self.sq_wqe_cnt) * self.sq_stride))
        self.send_db_idx = self.send_wqe_idx

    # -- test_utils.rs:211-257 --------------------------------------------------------------
    def launch_cqe_poll(self, target: PollTarget, stream: int = 0) -> None:
        """One poll of the target queue at its current consumer index; the result lands in ``poll_result``."""
        cq, idx = (self.send_cq, self.send_cq_idx) if target == PollTarget.Send else (self.recv_cq, self.recv_cq_idx)
        p = CqePollParamsC(cq.buf, cq.cqe_size, idx & 0xFFFFFFFF, cq.cqe_cnt, cq.dbrec)
        if self.device:
            check(lib().mhip_rdmaxcel_cqe_poll(self.poll_result, C.byref(p), stream))
        else:
            check(lib().mhip_rdmaxcel_cqe_poll_host(C.cast(self.poll_result, C.POINTER(C.c_int32)), C.byref(p)))

    def completed(self, target: PollTarget, byte_cnt: int) -> bool:
        """What ``wait_for_completion_gpu`` does with a poll's result (test_utils.rs:238-252): ``byte_cnt >= 0``
        is CQE_POLL_TRUE and advances the consumer index (rdmaxcel.cu:392); -2 is an error; -1 means try again."""
        if byte_cnt == -2:
            raise RuntimeError(f"Error polling {'send' if target == PollTarget.Send else 'receive'} completion")
        if byte_cnt < 0:
            return False
        if target == PollTarget.Send:
            self.send_cq_idx += 1
        else:
            self.recv_cq_idx += 1
        return True
