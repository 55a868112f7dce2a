"""Work-queue / completion-queue entries: the oracle against hand-derived bytes, the library's host forms against
the oracle.  No GPU needed.

The reference holds no byte vector for these functions (its tests need two NICs,
monarch_rdma/src/rdma_manager_actor_tests.rs:396-600): parity unpinned in the reference.  The expected bytes below
were written out by hand from the published mlx5 layouts (rdma-core <infiniband/mlx5dv.h>):

  control segment : opmod_idx_opcode(4, BE) | qpn_ds(4, BE) | signature(1) | reserved(2) | fm_ce_se(1) | imm(4)
  remote address  : raddr(8, BE) | rkey(4, BE) | reserved(4)
  data segment    : byte_count(4, BE) | lkey(4, BE) | addr(8, BE)
  send slot = 64 bytes; doorbell record word 0 = receive counter, word 1 = send counter, both BE
  completion entry: byte_cnt(4, BE) at byte 44, op_own in the last byte (opcode << 4 | owner bit)
"""
import ctypes as C

import numpy as np
import pytest

import oracle
from monarch_amd import _lib

FILL = 0xEE


def hexbytes(s: str) -> np.ndarray:
    return np.frombuffer(bytes.fromhex(s.replace("|", " ")), dtype=np.uint8)


def fresh(nbytes):
    return np.full(nbytes, FILL, dtype=np.uint8)


def dbrec_bytes(dbrec):
    return dbrec.view(np.uint8)


# ---------------------------------------------------------------------------------------------
# the two implementations under one calling convention, so that every known answer checks both
# ---------------------------------------------------------------------------------------------
class OracleImpl:
    name = "oracle"
    send_wqe = staticmethod(oracle.send_wqe)
    recv_wqe = staticmethod(oracle.recv_wqe)
    db_ring = staticmethod(oracle.db_ring)
    cqe_poll = staticmethod(oracle.cqe_poll)


class HostImpl:
    """The product's host functions (mhip_rdmaxcel_*_host)."""
    name = "library-host"

    @staticmethod
    def _params(buf, dbrec, wqe_cnt, *, laddr=0, lkey=0, length=0, wr_id=0, signaled=True, op_type=0, raddr=0, rkey=0, qp_num=0,
                buf_offset=0):
        return _lib.WqeParamsC(laddr, lkey, length, wr_id, 1 if signaled else 0, op_type, raddr, rkey, qp_num,
                               buf.ctypes.data + buf_offset, dbrec.ctypes.data, wqe_cnt)

    @classmethod
    def send_wqe(cls, sq, dbrec, wqe_cnt, **f):
        p = cls._params(sq, dbrec, wqe_cnt, **f)
        _lib.check(_lib.lib().mhip_rdmaxcel_send_wqe_host(C.byref(p)))

    @classmethod
    def recv_wqe(cls, rq, dbrec, wqe_cnt, **f):
        p = cls._params(rq, dbrec, wqe_cnt, **f)
        _lib.check(_lib.lib().mhip_rdmaxcel_recv_wqe_host(C.byref(p)))

    @staticmethod
    def db_ring(dst, src):
        _lib.check(_lib.lib().mhip_rdmaxcel_db_ring_host(dst.ctypes.data, src.ctypes.data))

    @staticmethod
    def cqe_poll(cq, dbrec, cqe_size, cqe_cnt, consumer_index, result=-1):
        p = _lib.CqePollParamsC(cq.ctypes.data, cqe_size, consumer_index, cqe_cnt, dbrec.ctypes.data)
        out = C.c_int32(result)
        _lib.check(_lib.lib().mhip_rdmaxcel_cqe_poll_host(C.byref(out), C.byref(p)))
        return out.value


IMPLS = [OracleImpl, HostImpl]


def aligned(nbytes, align=64):
    raw = np.full(nbytes + align, FILL, dtype=np.uint8)
    off = (-raw.ctypes.data) % align
    return raw[off:off + nbytes]


# ---------------------------------------------------------------------------------------------
# known answers
# ---------------------------------------------------------------------------------------------
@pytest.mark.parametrize("impl", IMPLS, ids=lambda i: i.name)
def test_send_wqe_known_bytes_signaled_write(impl):
    sq, dbrec = aligned(4 * 64), np.array([0xAAAAAAAA, 0xBBBBBBBB], dtype=np.uint32)
    impl.send_wqe(sq, dbrec, 4, laddr=0x00007F1234567890, lkey=0xAABBCCDD, length=0x00100000, wr_id=5, signaled=True,
                  op_type=0x08, raddr=0x00007E00DEADBEE0, rkey=0x11223344, qp_num=0x001234)
    want = fresh(4 * 64)
    # wr_id 5 in a queue of 4 -> slot 1 (byte 64)
    want[64:112] = hexbytes(
        "00 00 05 08 | 00 12 34 03 | 00 00 00 0A | 00 00 00 00"    # index 5, opcode 0x08; qpn 0x001234, 3 units; CQ update + solicited
        "00 00 7E 00 DE AD BE E0 | 11 22 33 44 | 00 00 00 00"      # remote address, rkey
        "00 10 00 00 | AA BB CC DD | 00 00 7F 12 34 56 78 90")     # 1 MiB, lkey, local address
    assert sq.tobytes() == want.tobytes()                            # bytes 48-63 of the slot and the other slots untouched
    assert dbrec_bytes(dbrec).tobytes() == bytes.fromhex("AA AA AA AA 00 00 00 06")  # receive word untouched; send counter 6


@pytest.mark.parametrize("impl", IMPLS, ids=lambda i: i.name)
def test_send_wqe_known_bytes_truncations_and_24_bit_record(impl):
    sq, dbrec = aligned(8 * 64), np.array([7, 7], dtype=np.uint32)
    # wr_id 0x01FFFFFF: its top byte falls off the 32-bit shift, bits 16-23 land in the opmod byte, the record wraps at 24 bits;
    # qp_num's top byte falls off too; length is cut to 32 bits; unsignaled
    impl.send_wqe(sq, dbrec, 8, laddr=0xFFFFFFFFFFFFFFF0, lkey=1, length=0x100000010, wr_id=0x01FFFFFF, signaled=False, op_type=0x10,
                  raddr=0x0102030405060708, rkey=0x80000000, qp_num=0xFFFFFFFF)
    want = fresh(8 * 64)
    want[448:496] = hexbytes(
        "FF FF FF 10 | FF FF FF 03 | 00 00 00 00 | 00 00 00 00"
        "01 02 03 04 05 06 07 08 | 80 00 00 00 | 00 00 00 00"
        "00 00 00 10 | 00 00 00 01 | FF FF FF FF FF FF FF F0")
    assert sq.tobytes() == want.tobytes()
    assert dbrec_bytes(dbrec)[4:].tobytes() == bytes.fromhex("00 00 00 00")   # (0x01FFFFFF + 1) & 0xFFFFFF
    assert dbrec[0] == 7
    # a wr_id above 32 bits posts as its low word
    sq2, db2 = aligned(8 * 64), np.zeros(2, dtype=np.uint32)
    impl.send_wqe(sq2, db2, 8, wr_id=(1 << 32) + 3, op_type=0x09, qp_num=1)
    assert sq2[192:200].tobytes() == bytes.fromhex("00 00 03 09 00 00 01 03")
    assert dbrec_bytes(db2)[4:].tobytes() == bytes.fromhex("00 00 00 04")


@pytest.mark.parametrize("impl", IMPLS, ids=lambda i: i.name)
def test_recv_wqe_known_bytes(impl):
    rq, dbrec = aligned(64), np.array([0x55555555, 0x66666666], dtype=np.uint32)
    impl.recv_wqe(rq, dbrec, 4, laddr=0x1122334455667788, lkey=0x01020304, length=4096, wr_id=7, buf_offset=16)
    want = fresh(64)
    want[16:32] = hexbytes("00 00 10 00 | 01 02 03 04 | 11 22 33 44 55 66 77 88")
    assert rq.tobytes() == want.tobytes()
    assert dbrec_bytes(dbrec).tobytes() == bytes.fromhex("00 00 00 08 66 66 66 66")   # wr_id + 1; send word untouched
    # the receive counter is a full 32-bit word: no 24-bit mask, wraps at 2^32
    impl.recv_wqe(rq, dbrec, 4, wr_id=0x00FFFFFF)
    assert dbrec_bytes(dbrec)[:4].tobytes() == bytes.fromhex("01 00 00 00")
    impl.recv_wqe(rq, dbrec, 4, wr_id=0xFFFFFFFF)
    assert dbrec_bytes(dbrec)[:4].tobytes() == bytes.fromhex("00 00 00 00")
    assert rq[:16].tobytes() == bytes(16)                                               # an all-zero segment at the queue's start


@pytest.mark.parametrize("impl", IMPLS, ids=lambda i: i.name)
def test_db_ring_copies_exactly_64_bytes(impl):
    src = aligned(128)
    src[:] = np.arange(128, dtype=np.uint8)
    dst = aligned(128)
    impl.db_ring(dst, src[8:])
    assert dst[:64].tobytes() == bytes(range(8, 72)) and dst[64:].tobytes() == bytes([FILL] * 64)


def make_cq(cqe_size, cqe_cnt):
    cq = aligned(cqe_size * cqe_cnt)
    cq[:] = 0
    return cq


def set_cqe(cq, cqe_size, entry, op_own, byte_cnt_be: str):
    base = entry * cqe_size
    cq[base + 44:base + 48] = hexbytes(byte_cnt_be)
    cq[base + cqe_size - 1] = op_own


@pytest.mark.parametrize("impl", IMPLS, ids=lambda i: i.name)
def test_cqe_poll_known_answers(impl):
    cq, dbrec = make_cq(64, 4), np.array([0x77777777, 0x88888888], dtype=np.uint32)
    set_cqe(cq, 64, 0, 0x00, "00 10 00 00")     # opcode 0, owner bit 0: owned on lap 0
    assert impl.cqe_poll(cq, dbrec, 64, 4, 0) == 0x00100000
    assert dbrec_bytes(dbrec).tobytes() == bytes.fromhex("00 00 00 01 88 88 88 88")

    def untouched(op_own, consumer_index):
        d = np.array([0x77777777, 0x88888888], dtype=np.uint32)
        q = make_cq(64, 4)
        set_cqe(q, 64, consumer_index & 3, op_own, "00 00 00 40")
        assert impl.cqe_poll(q, d, 64, 4, consumer_index, result=-1) == -1
        assert d[0] == 0x77777777 and d[1] == 0x88888888

    untouched(0x01, 0)        # owner bit 1 on lap 0: still the NIC's
    untouched(0xF0, 0)        # opcode 0xF marks an entry that was never written, whatever the owner bit says
    untouched(0xF1, 4)        # ... on lap 1 as well
    untouched(0x20, 5)        # lap 1 wants owner bit 1

    for op_own in (0x40, 0x80, 0xD0, 0xE0):      # owned, but an opcode of 4 and above is not a good completion
        d = np.array([0, 0], dtype=np.uint32)
        q = make_cq(64, 4)
        set_cqe(q, 64, 2, op_own, "00 00 00 40")
        assert impl.cqe_poll(q, d, 64, 4, 2) == -2
        assert dbrec_bytes(d)[:4].tobytes() == bytes.fromhex("00 00 00 03")
    for op_own in (0x10, 0x20, 0x30):            # opcodes 1-3 are good
        q = make_cq(64, 4)
        set_cqe(q, 64, 3, op_own, "00 00 00 40")
        assert impl.cqe_poll(q, np.zeros(2, dtype=np.uint32), 64, 4, 3) == 64


@pytest.mark.parametrize("impl", IMPLS, ids=lambda i: i.name)
def test_cqe_poll_second_lap_large_entries_and_record_wrap(impl):
    # lap 1 of a queue of 4 entries of 128 bytes: consumer index 5 -> entry 1, owner bit must be 1
    cq, dbrec = make_cq(128, 4), np.zeros(2, dtype=np.uint32)
    set_cqe(cq, 128, 1, 0x21, "00 00 02 00")
    assert impl.cqe_poll(cq, dbrec, 128, 4, 5) == 512
    assert dbrec_bytes(dbrec)[:4].tobytes() == bytes.fromhex("00 00 00 06")
    # the record keeps 24 bits: consumer index 0x00FFFFFF -> entry 3, lap parity (0xFFFFFF / 4) & 1 = 1, record 0
    cq2, db2 = make_cq(64, 4), np.array([5, 5], dtype=np.uint32)
    set_cqe(cq2, 64, 3, 0x01, "80 00 00 00")
    assert impl.cqe_poll(cq2, db2, 64, 4, 0x00FFFFFF) == -(1 << 31)     # the byte count is returned as a signed word
    assert dbrec_bytes(db2).tobytes() == bytes.fromhex("00 00 00 00 05 00 00 00")
    # consumer index 0xFFFFFFFF: entry 3, parity (0xFFFFFFFF / 4) & 1 = 1, record (0) & 0xFFFFFF
    cq3, db3 = make_cq(64, 4), np.array([9, 9], dtype=np.uint32)
    set_cqe(cq3, 64, 3, 0x01, "00 00 00 01")
    assert impl.cqe_poll(cq3, db3, 64, 4, 0xFFFFFFFF) == 1
    assert db3[0] == 0


# ---------------------------------------------------------------------------------------------
# the library's host forms against the oracle on random parameters
# ---------------------------------------------------------------------------------------------
def test_host_forms_equal_oracle_on_random_parameters():
    rng = np.random.default_rng(4242)
    for _ in range(2000):
        cnt = 1 << int(rng.integers(0, 8))
        f = dict(laddr=int(rng.integers(0, 2**63)) * 2 + int(rng.integers(0, 2)), lkey=int(rng.integers(0, 2**32)),
                 length=int(rng.integers(0, 2**40)), wr_id=int(rng.integers(0, 2**34)), signaled=bool(rng.integers(0, 2)),
                 op_type=int(rng.choice([0x08, 0x09, 0x10, 0x0A, 0xFF])), raddr=int(rng.integers(0, 2**63)),
                 rkey=int(rng.integers(0, 2**32)), qp_num=int(rng.integers(0, 2**32)))
        a, b = aligned(cnt * 64), aligned(cnt * 64)
        da, db = np.array([1, 2], dtype=np.uint32), np.array([1, 2], dtype=np.uint32)
        oracle.send_wqe(a, da, cnt, **f)
        HostImpl.send_wqe(b, db, cnt, **f)
        assert a.tobytes() == b.tobytes() and da.tobytes() == db.tobytes()
        slot = int(rng.integers(0, cnt)) * 64
        oracle.recv_wqe(a, da, cnt, buf_offset=slot, **f)
        HostImpl.recv_wqe(b, db, cnt, buf_offset=slot, **f)
        assert a.tobytes() == b.tobytes() and da.tobytes() == db.tobytes()
    for _ in range(2000):
        size, cnt = int(rng.choice([64, 128])), 1 << int(rng.integers(0, 6))
        cq = aligned(size * cnt)
        cq[:] = rng.integers(0, 256, size * cnt, dtype=np.uint8)
        for e in range(cnt):  # mostly plausible op_own bytes, some arbitrary
            if rng.random() < 0.8:
                cq[e * size + size - 1] = int(rng.choice([0x00, 0x01, 0x10, 0x21, 0xD0, 0xD1, 0xF0, 0xF1, 0x40]))
        ci = int(rng.integers(0, 2**32))
        da, db = np.array([3, 4], dtype=np.uint32), np.array([3, 4], dtype=np.uint32)
        assert oracle.cqe_poll(cq, da, size, cnt, ci) == HostImpl.cqe_poll(cq, db, size, cnt, ci)
        assert da.tobytes() == db.tobytes()


def test_argument_checks_without_a_gpu():
    L = _lib.lib()
    sq, dbrec = aligned(256), np.zeros(2, dtype=np.uint32)
    bad = _lib.ERR_INVALID_ARGUMENT
    p = HostImpl._params(sq, dbrec, 4)
    for fn in (L.mhip_rdmaxcel_send_wqe_host, L.mhip_rdmaxcel_recv_wqe_host):
        assert fn(None) == bad
    assert L.mhip_rdmaxcel_send_wqe(None, None) == bad and L.mhip_rdmaxcel_recv_wqe(None, None) == bad
    for cnt in (0, 3, 6, 0xFFFFFFFF):                       # the slot is idx & (wqe_cnt - 1): powers of two only
        p.wqe_cnt = cnt
        assert L.mhip_rdmaxcel_send_wqe_host(C.byref(p)) == bad and L.mhip_rdmaxcel_send_wqe(C.byref(p), None) == bad
        assert L.mhip_rdmaxcel_post_transfer(C.byref(p), 0, None, None) == bad
    p = HostImpl._params(sq, dbrec, 4, buf_offset=8)         # a segment is one 16-byte store
    assert L.mhip_rdmaxcel_send_wqe_host(C.byref(p)) == bad and L.mhip_rdmaxcel_recv_wqe_host(C.byref(p)) == bad
    p = HostImpl._params(sq, dbrec, 4)
    p.dbrec = dbrec.ctypes.data + 2
    assert L.mhip_rdmaxcel_send_wqe_host(C.byref(p)) == bad
    p.dbrec = None
    assert L.mhip_rdmaxcel_recv_wqe_host(C.byref(p)) == bad
    assert sq.tobytes() == bytes([FILL] * 256)               # refused calls wrote nothing
    # a transfer that needs more work requests than the queue has slots
    p = HostImpl._params(sq, dbrec, 4, length=5 * 4096)
    n = C.c_uint32(77)
    assert L.mhip_rdmaxcel_post_transfer(C.byref(p), 4096, C.byref(n), None) == _lib.ERR_WQE_OVERFLOW and n.value == 77
    assert b"Overflow of WQE" in L.mhip_error_string(_lib.ERR_WQE_OVERFLOW)
    # completion queue
    cq, out = make_cq(64, 4), C.c_int32(-1)
    q = _lib.CqePollParamsC(cq.ctypes.data, 64, 0, 4, dbrec.ctypes.data)
    assert L.mhip_rdmaxcel_cqe_poll_host(None, C.byref(q)) == bad and L.mhip_rdmaxcel_cqe_poll_host(C.byref(out), None) == bad
    for size, cnt in ((48, 4), (96, 4), (64, 0), (64, 3), (0, 4)):
        q = _lib.CqePollParamsC(cq.ctypes.data, size, 0, cnt, dbrec.ctypes.data)
        assert L.mhip_rdmaxcel_cqe_poll_host(C.byref(out), C.byref(q)) == bad
        assert L.mhip_rdmaxcel_cqe_poll(16, C.byref(q), None) == bad
    q = _lib.CqePollParamsC(cq.ctypes.data + 1, 64, 0, 4, dbrec.ctypes.data)
    assert L.mhip_rdmaxcel_cqe_poll_host(C.byref(out), C.byref(q)) == bad
    assert out.value == -1
    # doorbells
    assert L.mhip_rdmaxcel_db_ring_host(None, sq.ctypes.data) == bad and L.mhip_rdmaxcel_db_ring_host(sq.ctypes.data + 4, sq.ctypes.data) == bad
    assert L.mhip_rdmaxcel_db_ring(None, None, None) == bad
    assert L.mhip_rdmaxcel_ring_doorbells(16, 16, 64, 4, 0, 5, None) == _lib.ERR_WQE_OVERFLOW
    assert L.mhip_rdmaxcel_ring_doorbells(16, 16, 32, 4, 0, 1, None) == bad and L.mhip_rdmaxcel_ring_doorbells(16, 16, 64, 0, 0, 0, None) == bad
    assert L.mhip_rdmaxcel_ring_doorbells(16, 16, 64, 4, 0, 0, None) == 0   # nothing to ring


def test_parameter_structs_have_the_reference_layout():
    # wqe_params_t / cqe_poll_params_t of rdmaxcel-sys/src/rdmaxcel.h:26-48 under the x86-64 SysV ABI
    W = _lib.WqeParamsC
    offsets = {n: getattr(W, n).offset for n, _ in W._fields_}
    assert offsets == dict(laddr=0, lkey=8, length=16, wr_id=24, signaled=32, op_type=36, raddr=40, rkey=48, qp_num=52, buf=56,
                           dbrec=64, wqe_cnt=72) and C.sizeof(W) == 80
    Q = _lib.CqePollParamsC
    assert {n: getattr(Q, n).offset for n, _ in Q._fields_} == dict(cqe_buf=0, cqe_size=8, consumer_index=12, cqe_cnt=16, dbrec=24)
    assert C.sizeof(Q) == 32


def test_header_structs_have_that_layout_in_c(tmp_path):
    import os
    import subprocess
    root = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
    src = r'''
#include <stddef.h>
#include "monarch_hip.h"
#define AT(T, f, o) _Static_assert(offsetof(T, f) == o, #f)
AT(mhip_wqe_params_t, laddr, 0); AT(mhip_wqe_params_t, lkey, 8); AT(mhip_wqe_params_t, length, 16); AT(mhip_wqe_params_t, wr_id, 24);
AT(mhip_wqe_params_t, signaled, 32); AT(mhip_wqe_params_t, op_type, 36); AT(mhip_wqe_params_t, raddr, 40); AT(mhip_wqe_params_t, rkey, 48);
AT(mhip_wqe_params_t, qp_num, 52); AT(mhip_wqe_params_t, buf, 56); AT(mhip_wqe_params_t, dbrec, 64); AT(mhip_wqe_params_t, wqe_cnt, 72);
_Static_assert(sizeof(mhip_wqe_params_t) == 80, "size");
AT(mhip_cqe_poll_params_t, cqe_buf, 0); AT(mhip_cqe_poll_params_t, cqe_size, 8); AT(mhip_cqe_poll_params_t, consumer_index, 12);
AT(mhip_cqe_poll_params_t, cqe_cnt, 16); AT(mhip_cqe_poll_params_t, dbrec, 24);
_Static_assert(sizeof(mhip_cqe_poll_params_t) == 32, "size");
int main(void) { return 0; }
'''
    r = subprocess.run(["gcc", "-std=c11", "-I", os.path.join(root, "include"), "-x", "c", "-", "-fsyntax-only"], input=src, text=True,
                       capture_output=True)
    assert r.returncode == 0, r.stderr


def test_device_header_compiles_as_plain_host_cxx(tmp_path):
    # the header callers' own kernels include is also plain C++ for host code: same bytes as the oracle
    import os
    import subprocess
    root = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
    src = r'''
#include <cstdio>
#include <cstring>
#include "monarch_hip_rdmaxcel_device.h"
int main() {
  alignas(64) unsigned char sq[128]; std::memset(sq, 0xEE, sizeof sq);
  uint32_t dbrec[2] = {0, 0};
  mhip_wqe_params_t p{}; p.laddr = 0x1000; p.lkey = 2; p.length = 64; p.wr_id = 1; p.signaled = 1; p.op_type = 8; p.raddr = 0x2000;
  p.rkey = 3; p.qp_num = 9; p.buf = sq; p.dbrec = dbrec; p.wqe_cnt = 2;
  mhip_rdmaxcel::send_wqe(p);
  for (int i = 64; i < 112; ++i) std::printf("%02x", sq[i]);
  std::printf(" %08x\n", dbrec[1]);
  // the other three functions once each, on the same memory
  mhip_rdmaxcel::recv_wqe(p);
  alignas(8) unsigned char reg[64];
  mhip_rdmaxcel::db_ring(reg, sq + 64);
  alignas(4) unsigned char cq[128]; std::memset(cq, 0, sizeof cq); cq[44] = 0x12; cq[63] = 0x00;
  uint32_t cqdb[1] = {0};
  mhip_cqe_poll_params_t q{cq, 64, 0, 2, cqdb};
  int32_t res = -1;
  mhip_rdmaxcel::cqe_poll(&res, q);
  std::printf("%02x%02x %08x %08x\n", sq[3], reg[3], (unsigned)res, cqdb[0]);
}
'''
    exe = tmp_path / "t"
    # under the host sanitizers: the 16-byte segment stores, the doorbell record and the byte swaps have no undefined behaviour
    r = subprocess.run(["g++", "-std=c++17", "-O1", "-g", "-Wall", "-Werror", "-fsanitize=address,undefined", "-fno-sanitize-recover=all",
                        "-I", os.path.join(root, "include"), "-x", "c++", "-", "-o", str(exe)], input=src, text=True, capture_output=True)
    assert r.returncode == 0, r.stderr
    run = subprocess.run([str(exe)], capture_output=True, text=True)
    assert run.returncode == 0, run.stderr[-2000:]
    out = run.stdout.split()
    assert out[0] == ("00000108" "00000903" "0000000a" "00000000" "0000000000002000" "00000003" "00000000"
                      "00000040" "00000002" "0000000000001000")
    assert out[1] == "02000000"   # big-endian 2 read back as a little-endian word
    # recv_wqe put byte_count 0x40 big-endian at the queue's start; the ring copied the posted slot; the poll read 0x12000000
    assert out[2:] == ["4008", "12000000", "01000000"]
