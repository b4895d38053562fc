/* ringcheck.c -- bulk comparison of send-queue ring images with the scalar WQE
 * builder, and bulk / threaded forms of the builder and of the small-operation
 * model for timing.  Test infrastructure only (see oracle.h).
 *
 * orc_ring_check walks the entries of a ring image in counter order.  Which
 * operation got which counter is decided by the GPU's scheduling, so each
 * entry is matched by what it says - opcode, remote address, operand(s) -
 * against the multiset of operations issued on that ring, rebuilt with
 * orc_wqe_build (wqe.c; reference: queue_pair.cpp:205-273,
 * segment_builder.cpp:29-128) at the entry's own counter, and compared over all
 * 64 bytes.  Two fields cannot be predicted and are taken from the entry after
 * a range check: the completion flag (byte 11: 8, or the template's fm_ce_se;
 * slot max_nwqe - 2 must carry 8, queue_pair.cpp:80-85) and the AMO return
 * position (bytes 56-63; counted per position so the caller can check that
 * positions are handed out densely, atomic_return.hpp:34-40).
 *
 * The two entries that move no data are known to the checker too: a READ with
 * DS = 2 is quiet's zero-byte read (expected as opcode 0x10, the remote address,
 * data 0, size 0) and an inline WRITE to a flush word is fence's flush write
 * (expected as opcode 0x08, the flush word's address, data 1, size 4); see wqe.c.
 *
 * full_slot != 0: the ring never wrapped, bytes the builder leaves alone must
 * be zero (the ring's initial content).  full_slot == 0: the ring wrapped;
 * bytes the builder leaves alone hold what an older entry left there and are
 * not compared.
 */
#include <pthread.h>
#include <stdlib.h>
#include <string.h>

#include "oracle.h"

static int expect_cmp(const orc_wqe_expect_t *a, uint32_t opcode, uint64_t raddr, uint64_t data,
                      uint64_t cmp) {
  if (a->opcode != opcode) return a->opcode < opcode ? -1 : 1;
  if (a->raddr != raddr) return a->raddr < raddr ? -1 : 1;
  if (a->data != data) return a->data < data ? -1 : 1;
  if (a->cmp != cmp) return a->cmp < cmp ? -1 : 1;
  return 0;
}

static uint64_t be_to_u64(const uint8_t *p, int n) {
  uint64_t v = 0;
  for (int i = 0; i < n; ++i) v = (v << 8) | p[i];
  return v;
}

long orc_ring_check(const uint8_t *image, const orc_qp_t *qp, uint32_t first_counter,
                    uint32_t count, const orc_wqe_expect_t *expect, size_t n_expect,
                    uint8_t *used, const orc_arena_t *arena, int full_slot, uint32_t *pos_count,
                    uint32_t *n_atomic, uint32_t *n_cqe, int *why) {
  const uint32_t mask = qp->max_nwqe - 1;
  const uint8_t plain_ce = (uint8_t)(qp->ctrl_sig >> 24);
  *n_atomic = 0;
  *n_cqe = 0;
  for (uint32_t k = 0; k < count; ++k) {
    const uint32_t c = first_counter + k;
    const uint8_t *slot = image + 64ull * (c & mask);
    *why = 1; /* index field */
    if (orc_wqe_index(slot) != (uint16_t)c) return 1 + (long)k;
    const uint8_t opcode = slot[3];
    const int is_atomic = opcode == 0x11 || opcode == 0x12;
    const uint64_t raddr = be_to_u64(slot + 16, 8);
    uint64_t data = 0, cmp = 0;
    uint32_t size = 8, pos = 0;
    int form = ORC_WQE_DATA;
    const int to_flush_word = arena->flush_rkeys && raddr >= arena->flush_base &&
                              raddr - arena->flush_base < 64ull * (uint64_t)arena->num_pes;
    *why = 2; /* an opcode the stream cannot have produced */
    if (opcode == 0x10 && slot[7] == 2) {
      form = ORC_WQE_ZERO_BYTE_READ;
      size = 0;
    } else if (opcode == 0x08 && to_flush_word) {
      const uint32_t bc = (uint32_t)be_to_u64(slot + 32, 4);
      *why = 4;
      if (bc != (0x80000000u | 4u) || (raddr - arena->flush_base) % 64) return 1 + (long)k;
      form = ORC_WQE_FLUSH_WRITE;
      size = 4;
      data = slot[36];
    } else if (is_atomic) {
      data = be_to_u64(slot + 32, 8);
      cmp = be_to_u64(slot + 40, 8);
      const uint64_t ret = be_to_u64(slot + 56, 8);
      *why = 3; /* return slot outside the ring's window */
      if (ret < qp->atomic_ret_base || ((ret - qp->atomic_ret_base) & 7u) ||
          (ret - qp->atomic_ret_base) / 8 >= 4096)
        return 1 + (long)k;
      pos = (uint32_t)((ret - qp->atomic_ret_base) / 8);
    } else if (opcode == 0x08) {
      const uint32_t bc = (uint32_t)be_to_u64(slot + 32, 4);
      *why = 4; /* the small-operation streams post inline writes of 1..8 bytes only */
      if (!(bc & 0x80000000u) || (bc & 0x3ffu) == 0 || (bc & 0x3ffu) > 8) return 1 + (long)k;
      size = bc & 0x3ffu;
      for (uint32_t i = 0; i < size; ++i) data |= (uint64_t)slot[36 + i] << (8 * i);
    } else {
      return 1 + (long)k;
    }
    *why = 5; /* completion flag */
    if (slot[11] != 8 && slot[11] != plain_ce) return 1 + (long)k;
    if ((c & mask) == qp->max_nwqe - 2 && slot[11] != 8) return 1 + (long)k;
    /* the operation this entry stands for: lower bound, then the first unused equal */
    size_t lo = 0, hi = n_expect;
    while (lo < hi) {
      const size_t mid = lo + (hi - lo) / 2;
      if (expect_cmp(&expect[mid], opcode, raddr, data, cmp) < 0) lo = mid + 1; else hi = mid;
    }
    while (lo < n_expect && used[lo] && expect_cmp(&expect[lo], opcode, raddr, data, cmp) == 0) ++lo;
    *why = 6; /* no operation of this ring explains the entry (or it appears twice) */
    if (lo >= n_expect || expect_cmp(&expect[lo], opcode, raddr, data, cmp) != 0 ||
        expect[lo].size != size)
      return 1 + (long)k;
    used[lo] = 1;
    /* destination slice (or flush word) -> the key the entry must carry */
    *why = 7;
    uint32_t key;
    if (form == ORC_WQE_FLUSH_WRITE) {
      key = arena->flush_rkeys[(raddr - arena->flush_base) / 64];
    } else {
      if (raddr < arena->heap_base0) return 1 + (long)k;
      const uint64_t pe = (raddr - arena->heap_base0) / arena->slice_stride;
      if (pe >= (uint64_t)arena->num_pes) return 1 + (long)k;
      key = arena->rkeys[pe];
    }
    orc_wqe_req_t rq;
    memset(&rq, 0, sizeof rq);
    rq.opcode = opcode;
    rq.size = form == ORC_WQE_DATA ? size : 0;
    rq.form = form;
    rq.raddr = raddr;
    rq.rkey = key;
    rq.atomic_data = data;
    rq.atomic_cmp = cmp;
    for (uint32_t i = 0; i < 8; ++i) rq.inline_bytes[i] = (uint8_t)(data >> (8 * i));
    rq.atomic_pos = pos;
    rq.request_cqe = slot[11] == 8;
    uint8_t want[64];
    if (full_slot) memset(want, 0, 64); else memcpy(want, slot, 64);
    orc_wqe_build(want, qp, c, &rq);
    *why = 8; /* bytes */
    if (memcmp(want, slot, 64) != 0) return 1 + (long)k;
    if (is_atomic) {
      ++*n_atomic;
      if (pos_count) ++pos_count[pos];
    }
    if (slot[11] == 8) ++*n_cqe;
  }
  *why = 0;
  return 0;
}

/* Builds n entries with running numbers first_counter, first_counter+1, ... into
 * the ring (slot = counter mod max_nwqe): the scalar builder as a stream. */
void orc_wqe_build_many(uint8_t *ring, const orc_qp_t *qp, uint32_t first_counter,
                        const orc_wqe_req_t *reqs, size_t n) {
  const uint32_t mask = qp->max_nwqe - 1;
  for (size_t i = 0; i < n; ++i) {
    const uint32_t c = first_counter + (uint32_t)i;
    orc_wqe_build(ring + 64ull * (c & mask), qp, c, &reqs[i]);
  }
}

/* The 8-byte put / 64-bit fetch-add subset of orc_small_ops spread over host
 * threads with real atomics: what the reference's host path does through
 * MPI_Put / MPI_Fetch_and_op(MPI_SUM) on one node (host_helpers.hpp:52-88,
 * host_templates.hpp:285-307), as a best-effort CPU figure.  Thread t takes
 * the t-th contiguous part of the stream.  Returns -1 for other kinds. */
typedef struct {
  char *heap;
  size_t stride;
  const orc_small_op_t *ops;
  size_t begin, end;
  int64_t *fetched;
  int bad;
} small_part_t;

static void *small_part(void *arg) {
  small_part_t *p = (small_part_t *)arg;
  for (size_t i = p->begin; i < p->end; ++i) {
    const orc_small_op_t *o = &p->ops[i];
    int64_t *target = (int64_t *)(p->heap + (size_t)o->pe * p->stride + o->offset);
    if (o->kind == 0) {            /* p: 8-byte put */
      __atomic_store_n(target, o->value, __ATOMIC_RELAXED);
    } else if (o->kind == 1) {     /* fetch_add */
      int64_t old = __atomic_fetch_add(target, o->value, __ATOMIC_RELAXED);
      if (p->fetched) p->fetched[i] = old;
    } else {
      p->bad = 1;
    }
  }
  return NULL;
}

int orc_small_ops_mt(char *heap, size_t stride, const orc_small_op_t *ops, size_t n,
                     int64_t *fetched, int threads) {
  if (threads < 1) threads = 1;
  if (threads > 256) threads = 256;
  pthread_t tid[256];
  small_part_t part[256];
  const size_t share = (n + (size_t)threads - 1) / (size_t)threads;
  for (int t = 0; t < threads; ++t) {
    size_t b = share * (size_t)t, e = b + share;
    if (b > n) b = n;
    if (e > n) e = n;
    part[t] = (small_part_t){heap, stride, ops, b, e, fetched, 0};
    if (t && pthread_create(&tid[t], NULL, small_part, &part[t]) != 0) return -2;
  }
  small_part(&part[0]);
  int bad = part[0].bad;
  for (int t = 1; t < threads; ++t) {
    pthread_join(tid[t], NULL);
    bad |= part[t].bad;
  }
  return bad ? -1 : 0;
}
