/* consume.c -- scalar consumer of a send-queue ring: what the NIC does with the
 * entries in the reference, restated on the CPU.  Test infrastructure only
 * (see oracle.h).
 *
 * The reference has no software consumer: its rings are read by a ConnectX
 * NIC.  What is restated here is the documented execution of the four
 * opcodes the reference posts (library/src/gpu_ib/queue_pair.cpp:205-273:
 * RDMA WRITE with a data or inline segment, RDMA READ, atomic fetch-add and
 * compare-and-swap with the previous value returned to the address in the
 * fourth segment), in queue order as on an RC queue pair, and the tail of the
 * completion entry the reference's quiet reads back (queue_pair.cpp:118-191:
 * op_own at byte 63 with the owner bit = bit cq_log_size of the consumer's
 * running number, opcode nibble 0; wqe_counter at bytes 60-61).  The two
 * entries that move no data are taken off the ring and completed like the
 * others: quiet's zero-byte read (queue_pair.cpp:318-325: READ with DS = 2, the
 * third segment is not part of the entry) and fence's flush write
 * (queue_pair.cpp:376-384: a 4-byte inline write of the value 1 to the
 * destination's flush word under the flush key); on this path there is nothing
 * to flush, so executing them changes no memory.
 *
 * PARITY UNPINNED: the reference holds no vector for what a consumer does.
 * The tests pin this file by construction instead: entries built by
 * orc_wqe_build from known operations must replay to the memory image
 * orc_small_ops / memcpy produce for the same operations, and every field is
 * decoded byte-wise here, independently of the word-wise GPU decoder.
 */
#include <string.h>

#include "oracle.h"

static uint16_t get_be16(const uint8_t *p) { return (uint16_t)((p[0] << 8) | p[1]); }
static uint32_t get_be32(const uint8_t *p) {
  return ((uint32_t)p[0] << 24) | ((uint32_t)p[1] << 16) | ((uint32_t)p[2] << 8) | p[3];
}
static uint64_t get_be64(const uint8_t *p) {
  return ((uint64_t)get_be32(p) << 32) | get_be32(p + 4);
}
static uint32_t get_le32(const uint8_t *p) {
  return (uint32_t)p[0] | ((uint32_t)p[1] << 8) | ((uint32_t)p[2] << 16) | ((uint32_t)p[3] << 24);
}

/* Offset from slice 0 of [addr, addr+size) when it lies in one PE's heap. */
static int heap_offset(const orc_arena_t *a, uint64_t addr, uint64_t size, uint64_t *rel, int *pe) {
  if (addr < a->heap_base0) return 0;
  uint64_t r = addr - a->heap_base0;
  uint64_t p = r / a->slice_stride;
  uint64_t off = r % a->slice_stride;
  if (p >= (uint64_t)a->num_pes || off > a->heap_size || size > a->heap_size - off) return 0;
  *rel = r;
  *pe = (int)p;
  return 1;
}

void orc_sq_consume(const orc_qp_t *qp, const uint8_t *ring, uint32_t consumed, uint32_t published,
                    const orc_arena_t *arena, uint8_t *target, const uint8_t *sources,
                    uint64_t *atomic_ret, uint8_t *cq, uint32_t cq_size, uint32_t *cq_producer,
                    orc_consume_totals_t *t) {
  uint32_t c = consumed;
  if (published - c > qp->max_nwqe) {
    t->lost += published - c - qp->max_nwqe;
    c = published - qp->max_nwqe;
  }
  uint32_t cq_log = 0;
  while ((1u << cq_log) < cq_size) ++cq_log;

  for (; c != published; ++c) {
    const uint8_t *s = ring + 64ull * (c % qp->max_nwqe);
    t->retired++;
    uint8_t opcode = s[3];
    int is_atomic = opcode == 0x11 || opcode == 0x12;
    int is_write = opcode == 0x08, is_read = opcode == 0x10;
    int ok = s[0] == 0 && get_be16(s + 1) == (uint16_t)c &&
             (get_le32(s + 4) & 0xffffffu) == qp->ctrl_qp_sq && (is_atomic || is_write || is_read);
    const int zero_byte_read = is_read && s[7] == 2;
    ok = ok && (zero_byte_read || s[7] == (is_atomic ? 4 : 3));
    uint64_t raddr = get_be64(s + 16);
    uint32_t rkey = get_le32(s + 24);
    uint32_t size = 0;
    int inl = 0;
    uint64_t laddr = 0;
    if (is_atomic) {
      size = 8;
      laddr = get_be64(s + 56);
      ok = ok && (raddr & 7) == 0 && get_be32(s + 48) == 8 && get_le32(s + 52) == qp->atomic_lkey &&
           (laddr & 7) == 0 && laddr >= qp->atomic_ret_base &&
           laddr < qp->atomic_ret_base + 8ull * 4096;
    } else if (zero_byte_read) {
      size = 0;           /* nothing beyond the second segment belongs to the entry */
    } else {
      uint32_t count = get_be32(s + 32);
      inl = (count >> 31) & 1;
      size = inl ? (count & 0x3ffu) : count;
      if (inl) {
        ok = ok && is_write && size <= 12;
      } else {
        ok = ok && get_le32(s + 36) == qp->lkey;
        laddr = get_be64(s + 40);
      }
    }
    uint64_t roff = 0;
    int dest_pe = 0;
    int flush_write = 0;
    if (ok && is_write && inl && arena->flush_rkeys && raddr >= arena->flush_base &&
        raddr - arena->flush_base < 64ull * (uint64_t)arena->num_pes) {
      /* fence's entry: the flush word of one PE, its flush key, four bytes, the first one 1 */
      uint64_t p = (raddr - arena->flush_base) / 64;
      flush_write = 1;
      ok = (raddr - arena->flush_base) % 64 == 0 && size == 4 && s[36] == 1 &&
           rkey == arena->flush_rkeys[p];
    } else {
      ok = ok && heap_offset(arena, raddr, size, &roff, &dest_pe) && rkey == arena->rkeys[dest_pe];
    }

    if (!ok) {
      t->rejected++;
    } else {
      t->bytes += size;
      if (is_atomic) t->atomics++; else if (is_write) t->writes++; else t->reads++;
      if (target && !flush_write) {
        uint8_t *remote = target + roff;
        if (is_atomic) {
          uint64_t old, operand = get_be64(s + 32), compare = get_be64(s + 40);
          memcpy(&old, remote, 8);
          uint64_t next = old;
          if (opcode == 0x12) next = old + operand;
          else if (old == compare) next = operand;
          memcpy(remote, &next, 8);
          atomic_ret[(laddr - qp->atomic_ret_base) / 8] = old;
        } else if (inl) {
          memcpy(remote, s + 36, size);
        } else if (size) {
          uint64_t loff = 0;
          int local_pe = 0;
          if (!heap_offset(arena, laddr, size, &loff, &local_pe)) {
            t->local_skipped++;
          } else if (is_write) {
            memmove(remote, sources + loff, size);
          } else {
            memmove(target + loff, remote, size);
          }
        }
      }
    }
    if (s[11] == 8) {
      uint8_t *e = cq + 64ull * (*cq_producer % cq_size);
      memset(e, 0, 64);
      e[57] = s[4];
      e[58] = s[5];
      e[59] = s[6];
      e[60] = s[1];
      e[61] = s[2];
      e[63] = (uint8_t)((*cq_producer >> cq_log) & 1u);
      (*cq_producer)++;
      t->completions++;
    }
  }
}
