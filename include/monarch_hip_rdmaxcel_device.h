/*
 * monarch_hip_rdmaxcel_device.h - work-queue and completion-queue entry functions of the
 * device-initiated RDMA path, for HIP C++ callers that post work requests from inside their own
 * kernels (gfx950) or from host code.
 *
 * Counterpart of the `__host__ __device__` functions rdmaxcel-sys/src/rdmaxcel.h:80,87-90 declares
 * (db_ring, cqe_poll, send_wqe, recv_wqe; definitions rdmaxcel-sys/src/rdmaxcel.cu:82-93,139-160,
 * 201-245,292-326) and that monarch_rdma/examples/cuda_ping_pong/cuda_ping_pong.cu:60-110 calls from
 * its own kernel.  Device functions cannot cross a C ABI, so they are offered as a header; the
 * `mhip_rdmaxcel_*` entry points of monarch_hip.h are built from exactly these functions.
 *
 * Wire format (rdma-core <infiniband/mlx5dv.h>, every multi-byte field big-endian):
 *   control segment  (16 B): opmod_idx_opcode, qpn_ds, signature, 2 reserved bytes, fm_ce_se, imm
 *   remote-address   (16 B): raddr (8), rkey (4), reserved (4)
 *   data segment     (16 B): byte_count (4), lkey (4), addr (8)
 * A send WQE is control + remote-address + data = 48 bytes = 3 units of 16 bytes (the DS count) in a
 * 64-byte slot; a receive WQE is one data segment.  Each segment is built in registers and leaves as ONE
 * aligned 16-byte store, so a reader of the queue (the NIC) never sees a torn segment, and a
 * system-scope release fence orders the segments before the doorbell-record word.
 *
 * This header needs no InfiniBand headers.  It compiles as HIP (host + device) and as plain C++ (host only).
 */
#ifndef MONARCH_HIP_RDMAXCEL_DEVICE_H
#define MONARCH_HIP_RDMAXCEL_DEVICE_H

#include <stdint.h>

#include "monarch_hip.h"

#if defined(__HIPCC__)
#include <hip/hip_runtime.h>
#define MHIP_RDMAXCEL_FN __host__ __device__ inline
#else
#define MHIP_RDMAXCEL_FN inline
#endif

namespace mhip_rdmaxcel {

/* <infiniband/mlx5dv.h> */
constexpr uint32_t kSendWqeShift = 6;        /* MLX5_SEND_WQE_SHIFT: 64-byte send slots */
constexpr uint32_t kRcvDbr = 0;              /* MLX5_RCV_DBR */
constexpr uint32_t kSndDbr = 1;              /* MLX5_SND_DBR */
constexpr uint8_t kCtrlCqUpdate = 2 << 2;    /* MLX5_WQE_CTRL_CQ_UPDATE */
constexpr uint8_t kCtrlSolicited = 1 << 1;   /* MLX5_WQE_CTRL_SOLICITED */
constexpr uint32_t kCqeByteCntOffset = 44;   /* mlx5_cqe64.byte_cnt */

struct alignas(16) Segment {
    uint32_t w[4];
};

MHIP_RDMAXCEL_FN uint32_t be32(uint32_t v) { return __builtin_bswap32(v); }
MHIP_RDMAXCEL_FN uint32_t be64_hi(uint64_t v) { return __builtin_bswap32((uint32_t)(v >> 32)); }  /* first word in memory */
MHIP_RDMAXCEL_FN uint32_t be64_lo(uint64_t v) { return __builtin_bswap32((uint32_t)v); }          /* second word in memory */

/* Stores so far become visible to every agent of the system (the NIC included) before later ones. */
MHIP_RDMAXCEL_FN void release_to_system() {
#if defined(__HIP_DEVICE_COMPILE__)
    __threadfence_system();
#else
    __atomic_thread_fence(__ATOMIC_SEQ_CST);
#endif
}

MHIP_RDMAXCEL_FN void store_word(uint32_t* p, uint32_t v) { *(volatile uint32_t*)p = v; }
MHIP_RDMAXCEL_FN void store_segment(uint8_t* p, const Segment& s) { *reinterpret_cast<Segment*>(p) = s; }

MHIP_RDMAXCEL_FN Segment data_segment(const mhip_wqe_params_t& p) {
    return Segment{{be32((uint32_t)p.length), be32(p.lkey), be64_hi(p.laddr), be64_lo(p.laddr)}};
}

/* db_ring, rdmaxcel.cu:82-93: the first 64 bytes of a send WQE to the doorbell register, lowest address
 * first, as eight 64-bit stores (a register written through a write-combining mapping wants them in order
 * and whole). */
MHIP_RDMAXCEL_FN void db_ring(void* dst, const void* src) {
    volatile uint64_t* d = static_cast<volatile uint64_t*>(dst);
    const volatile uint64_t* s = static_cast<const volatile uint64_t*>(src);
    for (int i = 0; i < 8; ++i) d[i] = s[i];
}

/* recv_wqe, rdmaxcel.cu:139-160: one data segment at p.buf itself (the caller addresses the slot), then
 * the receive doorbell record = wr_id + 1 in 32 bits.  p.buf must be 16-byte aligned. */
MHIP_RDMAXCEL_FN void recv_wqe(const mhip_wqe_params_t& p) {
    store_segment(p.buf, data_segment(p));
    release_to_system();
    store_word(p.dbrec + kRcvDbr, be32((uint32_t)(p.wr_id + 1)));
}

/* The 48 bytes of send WQE number `idx` (the low 32 bits of wr_id), rdmaxcel.cu:206-230. */
MHIP_RDMAXCEL_FN void build_send_wqe(const mhip_wqe_params_t& p, uint32_t idx, Segment* ctrl, Segment* raddr, Segment* data) {
    const uint32_t fm_ce_se = p.signaled ? (uint32_t)(kCtrlCqUpdate | kCtrlSolicited) : 0u;
    /* word 2 in memory order: signature (0), two reserved bytes (0), fm_ce_se -> fm_ce_se is the word's last byte */
    *ctrl = Segment{{be32((idx << 8) | p.op_type), be32((p.qp_num << 8) | (48u / 16u)), fm_ce_se << 24, 0u}};
    *raddr = Segment{{be64_hi(p.raddr), be64_lo(p.raddr), be32(p.rkey), 0u}};
    *data = data_segment(p);
}

/* send_wqe, rdmaxcel.cu:201-245: control + remote-address + data segments into slot
 * idx & (wqe_cnt - 1) of the send queue, then the send doorbell record = (idx + 1) & 0xFFFFFF.
 * p.buf must be 16-byte aligned and p.wqe_cnt a power of two. */
MHIP_RDMAXCEL_FN void send_wqe(const mhip_wqe_params_t& p) {
    const uint32_t idx = (uint32_t)p.wr_id;
    Segment ctrl, raddr, data;
    build_send_wqe(p, idx, &ctrl, &raddr, &data);
    uint8_t* slot = p.buf + ((uint64_t)(idx & (p.wqe_cnt - 1u)) << kSendWqeShift);
    store_segment(slot, ctrl);
    store_segment(slot + 16, raddr);
    store_segment(slot + 32, data);
    release_to_system();
    store_word(p.dbrec + kSndDbr, be32((idx + 1u) & 0xFFFFFFu));
}

/* cqe_poll, rdmaxcel.cu:292-326: ONE look at completion-queue entry consumer_index & (cqe_cnt - 1); no
 * loop.  Software owns the entry when bit 0 of its last byte (op_own) equals the lap parity
 * (consumer_index / cqe_cnt) & 1 and its opcode (upper 4 bits) is not 0xF.  Owned with an opcode below 4:
 * *byte_cnt = the big-endian word at byte 44; owned with any other opcode: *byte_cnt = -2; both store
 * (consumer_index + 1) & 0xFFFFFF big-endian into the CQ's doorbell record.  Not owned: nothing is
 * written (the caller initialises *byte_cnt to -1, rdmaxcel.cu:293,368).  op_own is read before the byte
 * count with an acquire fence between the two: the NIC writes op_own last.  cqe_buf and cqe_size must be
 * multiples of 4 and p.cqe_cnt a power of two. */
MHIP_RDMAXCEL_FN void cqe_poll(int32_t* byte_cnt, const mhip_cqe_poll_params_t& p) {
    const uint32_t idx = p.consumer_index;
    const uint8_t* cqe = p.cqe_buf + (uint64_t)(idx & (p.cqe_cnt - 1u)) * p.cqe_size;
    const uint8_t op_own = *(const volatile uint8_t*)(cqe + p.cqe_size - 1);
    const uint32_t opcode = op_own >> 4;
    const bool owned = ((op_own & 1u) == ((idx / p.cqe_cnt) & 1u)) && opcode != 0xFu;
    if (!owned) return;
    release_to_system();  /* a full fence: also keeps the byte-count load behind the ownership load */
    if ((opcode & 0xCu) == 0) {
        *byte_cnt = (int32_t)be32(*(const volatile uint32_t*)(cqe + kCqeByteCntOffset));
    } else {
        *byte_cnt = -2;
    }
    store_word(p.dbrec, be32((idx + 1u) & 0xFFFFFFu));
}

}  // namespace mhip_rdmaxcel

#endif /* MONARCH_HIP_RDMAXCEL_DEVICE_H */
