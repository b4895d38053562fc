/* wqe.c -- scalar builder of the 64-byte send-queue entry (RC transport).
 * Test infrastructure only (see oracle.h).
 *
 * Restates, byte by byte, what the reference writes into a slot:
 *   library/src/gpu_ib/queue_pair.cpp:205-273  update_posted_wqe_generic
 *   library/src/gpu_ib/segment_builder.cpp:29-128 (control, remote-address,
 *     atomic, data and inline-data segments)
 *   library/src/gpu_ib/endian.cpp:27-77 (swap_endian_store)
 *   library/src/gpu_ib/queue_pair.cpp:67-78, thread_policy.cpp:170-216
 *     (completion flag at byte 11, doorbell record and doorbell value)
 *   library/src/gpu_ib/connection_policy.cpp:45-79 (RC: one slot per operation,
 *     no address-vector segment)
 *   library/src/gpu_ib/queue_pair.cpp:318-325,376-384 (the two entries that move
 *     no data: quiet's zero-byte read and fence's flush write)
 * The segment layouts belong to rdma-core's <infiniband/mlx5dv.h>
 * (mlx5_wqe_ctrl_seg, mlx5_wqe_raddr_seg, mlx5_wqe_data_seg,
 * mlx5_wqe_atomic_seg, mlx5_wqe_inl_data_seg), a dependency the reference does
 * not vendor and does not pin to a version (library/CMakeLists.txt:162); they
 * are restated here from that public format.
 *
 * PARITY UNPINNED: the reference holds no test, golden vector or fixture for
 * WQE bytes.  What the tests check instead is fixed by the format itself:
 * every multi-byte NIC field reads back big-endian, DS equals the number of
 * 16-byte segments, the slot index is counter % ring size, the inline flag is
 * bit 31 of the byte count, the completion byte is 8, and bytes the reference
 * never writes keep their previous content.
 */
#include <string.h>

#include "oracle.h"

uint16_t orc_bswap16(uint16_t v) { return (uint16_t)((v << 8) | (v >> 8)); }
uint32_t orc_bswap32(uint32_t v) {
  return (v << 24) | ((v & 0xff00u) << 8) | ((v >> 8) & 0xff00u) | (v >> 24);
}
uint64_t orc_bswap64(uint64_t v) {
  return ((uint64_t)orc_bswap32((uint32_t)v) << 32) | orc_bswap32((uint32_t)(v >> 32));
}

static void put_be16(uint8_t *p, uint16_t v) { p[0] = (uint8_t)(v >> 8); p[1] = (uint8_t)v; }
static void put_be32(uint8_t *p, uint32_t v) {
  p[0] = (uint8_t)(v >> 24); p[1] = (uint8_t)(v >> 16); p[2] = (uint8_t)(v >> 8); p[3] = (uint8_t)v;
}
static void put_be64(uint8_t *p, uint64_t v) {
  put_be32(p, (uint32_t)(v >> 32));
  put_be32(p + 4, (uint32_t)v);
}
/* A value the reference stores as a native (little-endian) word. */
static void put_le32(uint8_t *p, uint32_t v) {
  p[0] = (uint8_t)v; p[1] = (uint8_t)(v >> 8); p[2] = (uint8_t)(v >> 16); p[3] = (uint8_t)(v >> 24);
}

void orc_wqe_build(uint8_t slot[64], const orc_qp_t *qp, uint32_t sq_counter,
                   const orc_wqe_req_t *rq) {
  const int is_atomic = rq->opcode == 0x11 || rq->opcode == 0x12;
  const int is_write = rq->opcode == 0x08;

  /* Control segment (segment_builder.cpp:35-60).  opmod_idx_opcode is the
   * native word (opcode << 24) | (bswap16(index) << 8): byte 0 opmod = 0,
   * bytes 1-2 the 16-bit entry index big-endian, byte 3 the opcode. */
  slot[0] = 0;
  put_be16(slot + 1, (uint16_t)sq_counter);
  slot[3] = rq->opcode;
  /* qpn_ds is the native word (DS << 24) | ctrl_qp_sq: the three bytes
   * harvested from the template entry, then the segment count. */
  slot[4] = (uint8_t)(qp->ctrl_qp_sq);
  slot[5] = (uint8_t)(qp->ctrl_qp_sq >> 8);
  slot[6] = (uint8_t)(qp->ctrl_qp_sq >> 16);
  /* DS: control + remote address (+ data) (+ atomic); a zero-byte read counts two
   * (segment_builder.cpp:43-49). */
  slot[7] = (uint8_t)(rq->form == ORC_WQE_ZERO_BYTE_READ ? 2 : is_atomic ? 4 : 3);
  slot[8] = (uint8_t)qp->ctrl_sig;                 /* signature */
  /* bytes 9-10 reserved: never written */
  slot[11] = (uint8_t)(qp->ctrl_sig >> 24);        /* fm_ce_se */
  put_le32(slot + 12, (uint32_t)(qp->ctrl_sig >> 32)); /* imm */

  /* Remote-address segment (segment_builder.cpp:75-85). */
  put_be64(slot + 16, rq->raddr);
  put_le32(slot + 24, rq->rkey);                   /* key kept as harvested */
  /* bytes 28-31 reserved: never written */

  if (rq->form == ORC_WQE_ZERO_BYTE_READ) {
    /* zero_b_rd passes a null local address: update_data_seg returns before it
     * writes anything (segment_builder.cpp:89-91), the third segment keeps what
     * the slot held. */
  } else if (rq->form == ORC_WQE_FLUSH_WRITE) {
    /* size 0 became 4 (queue_pair.cpp:230-233); with a null local address the inline
     * segment gets one payload byte, 1 (segment_builder.cpp:110-116). */
    put_be32(slot + 32, 4u | 0x80000000u);
    slot[36] = 1;
  } else if (is_atomic) {
    /* Atomic segment (segment_builder.cpp:62-73) then a data segment that
     * names the 8-byte return slot (queue_pair.cpp:251-256). */
    put_be64(slot + 32, rq->atomic_data);
    put_be64(slot + 40, rq->atomic_cmp);
    put_be32(slot + 48, 8u);
    put_le32(slot + 52, qp->atomic_lkey);
    put_be64(slot + 56, qp->atomic_ret_base + 8ull * rq->atomic_pos);
  } else if (is_write && rq->size <= 8) {
    /* Inline data (segment_builder.cpp:105-121): flagged byte count, then
     * the payload bytes; the rest of the segment is left alone. */
    put_be32(slot + 32, (rq->size & 0x3ffu) | 0x80000000u);
    memcpy(slot + 36, rq->inline_bytes, rq->size);
  } else {
    /* Data pointer segment (segment_builder.cpp:87-103). */
    put_be32(slot + 32, rq->size & 0x7fffffffu);
    put_le32(slot + 36, qp->lkey);
    put_be64(slot + 40, rq->laddr);
  }

  /* set_completion_flag_on_wqe (queue_pair.cpp:74-78). */
  if (rq->request_cqe) slot[11] = 8;
}

uint16_t orc_wqe_index(const uint8_t slot[64]) { return (uint16_t)((slot[1] << 8) | slot[2]); }
uint8_t orc_wqe_opcode(const uint8_t slot[64]) { return slot[3]; }
uint64_t orc_wqe_raddr(const uint8_t slot[64]) {
  uint64_t v = 0;
  for (int i = 0; i < 8; ++i) v = (v << 8) | slot[16 + i];
  return v;
}

/* ring_doorbell (queue_pair.cpp:67-72): the doorbell record receives the
 * queue's counter big-endian, the doorbell register the first eight bytes of
 * the entry that closed the post (thread_policy.cpp:183-185). */
void orc_doorbell(const uint8_t last_slot[64], uint32_t sq_counter_after, uint64_t mailbox[2]) {
  uint8_t rec[8] = {0};
  put_be32(rec, sq_counter_after);
  memcpy(&mailbox[0], rec, 8);
  memcpy(&mailbox[1], last_slot, 8);
}
