/* oracle.h -- CPU restatement of the reference's algorithms for the device
 * data path.  TEST INFRASTRUCTURE ONLY: it is the checker that tests, the
 * smoke run and the benchmark's CPU-baseline leg compare the GPU library
 * against; the library itself never calls it.
 *
 * All PEs are modelled in one address space: PE p's symmetric-heap slice is
 * `heap + p*stride`.  Symmetric objects are named by their byte offset in the
 * slice.  Each function cites the reference code it restates.
 *
 * Pinning status of each function (what independent evidence fixes it) is
 * listed next to its definition.
 */
#ifndef ROCSHMEM_ORACLE_H
#define ROCSHMEM_ORACLE_H

#include <stddef.h>
#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

enum orc_dtype { ORC_SHORT = 0, ORC_INT, ORC_LONG, ORC_LONGLONG, ORC_FLOAT, ORC_DOUBLE, ORC_BF16 };
enum orc_op { ORC_SUM = 0, ORC_MAX, ORC_MIN, ORC_PROD, ORC_AND, ORC_OR, ORC_XOR };

size_t orc_dtype_size(int dtype);

/* ---- reductions (reduce.c) ------------------------------------------------ */

/* In-type fold in ascending member order, result to every member's dest.
 * Returns 0, or -1 for an undefined (dtype, op) pair. */
int orc_to_all(int dtype, int op, char *heap, size_t stride, size_t dest_off, size_t src_off,
               size_t n, int pe_start, int log_stride, int pe_size);
/* Team form: members pe_start + k * pe_stride, any pe_stride >= 1. */
int orc_to_all_team(int dtype, int op, char *heap, size_t stride, size_t dest_off, size_t src_off,
                    size_t n, int pe_start, int pe_stride, int pe_size);
/* The GPU library's floating-point contract (float sum/prod folded in double, bfloat16 sum
 * in float, ascending members, one rounding); see reduce.c. */
int orc_to_all_rounded_once(int dtype, int op, char *heap, size_t stride, size_t dest_off,
                            size_t src_off, size_t n, int pe_start, int pe_stride, int pe_size);
/* Ground truth: the same reduction evaluated in long double on the exact
 * values of the inputs, returned as double.  out[n]. */
int orc_to_all_f64(int dtype, int op, const char *heap, size_t stride, size_t src_off, size_t n,
                   int pe_start, int log_stride, int pe_size, double *out);
/* Sum over members of |x| per element (the scale of the tolerance test). */
int orc_abs_sum_f64(int dtype, const char *heap, size_t stride, size_t src_off, size_t n,
                    int pe_start, int log_stride, int pe_size, double *out);
/* Multi-threaded orc_to_all over `threads` host threads (CPU baseline). */
int orc_to_all_mt(int dtype, int op, char *heap, size_t stride, size_t dest_off, size_t src_off,
                  size_t n, int pe_start, int log_stride, int pe_size, int threads);
uint16_t orc_float_to_bf16(float f);
float orc_bf16_to_float(uint16_t b);

/* ---- put / get / broadcast / alltoall / fcollect (rma.c) ------------------- */

void orc_put(char *heap, size_t stride, size_t dest_off, size_t src_off, size_t nbytes,
             int src_pe, int dest_pe);
void orc_get(char *heap, size_t stride, size_t dest_off, size_t src_off, size_t nbytes,
             int my_pe, int from_pe);
void orc_broadcast(char *heap, size_t stride, size_t dest_off, size_t src_off, size_t nbytes,
                   int root_idx, int pe_start, int log_stride, int pe_size);
void orc_alltoall(char *heap, size_t stride, size_t dest_off, size_t src_off, size_t block_bytes,
                  int pe_start, int log_stride, int pe_size);
void orc_fcollect(char *heap, size_t stride, size_t dest_off, size_t src_off, size_t block_bytes,
                  int pe_start, int log_stride, int pe_size);
/* Team forms of the three: members pe_start + k * pe_stride, any pe_stride >= 1. */
void orc_broadcast_team(char *heap, size_t stride, size_t dest_off, size_t src_off, size_t nbytes,
                        int root_idx, int pe_start, int pe_stride, int pe_size);
void orc_alltoall_team(char *heap, size_t stride, size_t dest_off, size_t src_off,
                       size_t block_bytes, int pe_start, int pe_stride, int pe_size);
void orc_fcollect_team(char *heap, size_t stride, size_t dest_off, size_t src_off,
                       size_t block_bytes, int pe_start, int pe_stride, int pe_size);
/* memcpy spread over `threads` host threads (CPU baseline for put/get). */
void orc_copy_mt(char *dst, const char *src, size_t nbytes, int threads);

/* ---- small operations (amo.c) ----------------------------------------------- */

typedef struct orc_small_op {
  uint32_t kind;   /* same codes as rsm_small_kind */
  uint32_t pe;
  uint64_t offset;
  int64_t value;
  int64_t aux;
} orc_small_op_t;

/* Applies ops[0..n) one after the other (a legal serialisation) with op i
 * issued by PE issuer_pe[i]; fetched[i] gets what a fetching op returns. */
int orc_small_ops(char *heap, size_t stride, const orc_small_op_t *ops, const uint32_t *issuer_pe,
                  size_t n, int64_t *fetched);

/* ---- 64-byte WQE builder (wqe.c) ---------------------------------------------- */

typedef struct orc_qp {
  uint32_t ctrl_qp_sq;
  uint64_t ctrl_sig;
  uint32_t lkey;
  uint32_t atomic_lkey;
  uint64_t atomic_ret_base;
  uint32_t max_nwqe;
} orc_qp_t;

typedef struct orc_wqe_req {
  uint8_t opcode;        /* 0x08 write, 0x10 read, 0x11 compare-swap, 0x12 fetch-add */
  uint32_t size;
  uint64_t raddr;
  uint32_t rkey;
  uint64_t laddr;
  uint64_t atomic_data;
  uint64_t atomic_cmp;
  uint8_t inline_bytes[8];
  uint32_t atomic_pos;   /* return-slot index, already reduced modulo 4096 */
  int request_cqe;       /* completion flag byte <- 8 */
  int form;              /* ORC_WQE_DATA, or one of the two entries that move no data */
} orc_wqe_req_t;
/* Forms of an entry.  ORC_WQE_ZERO_BYTE_READ: QueuePair::zero_b_rd (queue_pair.cpp:318-325),
 * posted by quiet before it polls (thread_policy.cpp:35-108): opcode READ, DS = 2, remote
 * address = base of the destination's heap, no data segment written.  ORC_WQE_FLUSH_WRITE:
 * QueuePair::fence (queue_pair.cpp:376-384): a WRITE of size 0 is turned into a 4-byte inline
 * write (queue_pair.cpp:230-233) whose first payload byte is 1 (segment_builder.cpp:110-116),
 * addressed to the destination's flush word under the flush key (`raddr`, `rkey` as given). */
enum { ORC_WQE_DATA = 0, ORC_WQE_ZERO_BYTE_READ = 1, ORC_WQE_FLUSH_WRITE = 2 };

/* Overwrites, inside the 64-byte slot, exactly the bytes the reference writes. */
void orc_wqe_build(uint8_t slot[64], const orc_qp_t *qp, uint32_t sq_counter,
                   const orc_wqe_req_t *rq);
/* ---- ring consumer (consume.c) ------------------------------------------------- */

typedef struct orc_arena {
  uint64_t heap_base0;   /* address of PE 0's heap as the entries name it */
  uint64_t slice_stride;
  uint64_t heap_size;
  int num_pes;
  const uint32_t *rkeys; /* per destination PE, as stored in the entries */
  /* Flush words (what the reference's hdp_address[] / hdp_rkey[] name, network_policy.cpp:114-180):
   * PE p's at flush_base + 64 p under flush_rkeys[p]; flush_rkeys NULL: no flush writes expected. */
  uint64_t flush_base;
  const uint32_t *flush_rkeys;
} orc_arena_t;

typedef struct orc_consume_totals {
  uint64_t retired, writes, reads, atomics, bytes, completions, lost, rejected, local_skipped;
} orc_consume_totals_t;

/* Retires entries [consumed, published) of one ring in order.  `target` (may be
 * NULL: check and complete only) and `sources` are host images laid out like
 * the arena: operations are executed on `target`, payloads of non-inline writes
 * are read from `sources`.  `atomic_ret` is the ring's 4096-word return window,
 * `cq` its completion queue of `cq_size` 64-byte entries. */
void orc_sq_consume(const orc_qp_t *qp, const uint8_t *ring, uint32_t consumed, uint32_t published,
                    const orc_arena_t *arena, uint8_t *target, const uint8_t *sources,
                    uint64_t *atomic_ret, uint8_t *cq, uint32_t cq_size, uint32_t *cq_producer,
                    orc_consume_totals_t *totals);

/* ---- bulk ring check, bulk / threaded forms for timing (ringcheck.c) ------------ */

/* One operation as its ring entry describes it.  `data`: the atomic operand, or
 * the inline payload as a little-endian integer; `cmp`: compare operand (0 unless
 * compare-and-swap); `size`: payload bytes (8 for atomics). */
typedef struct orc_wqe_expect {
  uint64_t raddr;
  uint64_t data;
  uint64_t cmp;
  uint32_t opcode;
  uint32_t size;
} orc_wqe_expect_t;

/* Entries first_counter .. first_counter+count-1 of a ring image against the
 * builder; `expect` sorted ascending by (opcode, raddr, data, cmp), `used`
 * n_expect zero bytes that come back 1 for every operation an entry stood for.
 * Returns 0 when all entries are right, else 1 + the position of the first
 * wrong entry with the reason in *why (see ringcheck.c). */
long orc_ring_check(const uint8_t *image, const orc_qp_t *qp, uint32_t first_counter,
                    uint32_t count, const orc_wqe_expect_t *expect, size_t n_expect,
                    uint8_t *used, const orc_arena_t *arena, int full_slot, uint32_t *pos_count,
                    uint32_t *n_atomic, uint32_t *n_cqe, int *why);
void orc_wqe_build_many(uint8_t *ring, const orc_qp_t *qp, uint32_t first_counter,
                        const orc_wqe_req_t *reqs, size_t n);
int orc_small_ops_mt(char *heap, size_t stride, const orc_small_op_t *ops, size_t n,
                     int64_t *fetched, int threads);

/* Parse helpers used by the ring checker. */
uint16_t orc_wqe_index(const uint8_t slot[64]);
uint8_t orc_wqe_opcode(const uint8_t slot[64]);
uint64_t orc_wqe_raddr(const uint8_t slot[64]);
/* Doorbell record / doorbell value after the entry with counter `last_counter`
 * closed a post that advanced the queue to `sq_counter_after`. */
void orc_doorbell(const uint8_t last_slot[64], uint32_t sq_counter_after, uint64_t mailbox[2]);
uint16_t orc_bswap16(uint16_t v);
uint32_t orc_bswap32(uint32_t v);
uint64_t orc_bswap64(uint64_t v);

/* ---- wave-level models (wave.c) -------------------------------------------------- */

/* WfCoalOn::coalesce for one 64-lane wave. */
void orc_coalesce(uint64_t lane_mask, const int32_t *pe, const uint64_t *src, const uint64_t *dst,
                  const uint64_t *size, uint8_t *must_send, uint64_t *out_size);
/* Block::fetch_incr for one wave: returns the values the active lanes get,
 * ~0 for inactive lanes; *counter advances by the number of active lanes. */
void orc_fetch_incr(uint64_t lane_mask, uint64_t *counter, uint64_t out[64]);

/* ---- symmetric allocator model (alloc.c) ------------------------------------------- */

typedef struct orc_alloc orc_alloc_t;
orc_alloc_t *orc_alloc_create(size_t heap_bytes);
void orc_alloc_destroy(orc_alloc_t *a);
size_t orc_alloc_alloc(orc_alloc_t *a, size_t request);   /* (size_t)-1 when nothing fits */
int orc_alloc_free(orc_alloc_t *a, size_t offset);
size_t orc_alloc_in_use(const orc_alloc_t *a);

#ifdef __cplusplus
}
#endif
#endif
