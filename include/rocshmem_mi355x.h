/* rocshmem_mi355x.h -- C ABI of librocshmem_mi355x.so.
 *
 * The reference (ROCm/ROC_SHMEM) exposes a C++ host/device interface that is
 * linked into the user's kernels; it has no foreign-function boundary of its
 * own.  This header is that boundary for the MI355X-native data path: plain C
 * entry points that (a) mirror the reference's host lifecycle calls and
 * (b) launch, for every PE of the job at once, a grid of workgroups in which
 * each workgroup issues the named roc_shmem_* device call on its share of the
 * data -- the role the reference's functional test kernels play
 * (clients/functional_tests/ in the reference).  All PEs live in one process
 * and one GPU; a symmetric address passed in is the address in PE 0's slice
 * unless stated otherwise.
 *
 * Return value: 0 on success, negative on error (rsm_last_error() has the
 * message).  No entry point takes or returns C++ or torch types.
 */
#ifndef ROCSHMEM_MI355X_C_ABI_H
#define ROCSHMEM_MI355X_C_ABI_H

#include <stddef.h>
#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

/* ---- codes -------------------------------------------------------------- */

/* Element types of the reductions (reference: library/include/roc_shmem.hpp:1190-1198;
 * RSM_BF16 is an extension). */
enum rsm_dtype {
  RSM_SHORT = 0,
  RSM_INT = 1,
  RSM_LONG = 2,
  RSM_LONGLONG = 3,
  RSM_FLOAT = 4,
  RSM_DOUBLE = 5,
  RSM_BF16 = 6
};

/* Reduction operators, numerically equal to ROC_SHMEM_OP (roc_shmem.hpp:52-61). */
enum rsm_op {
  RSM_SUM = 0,
  RSM_MAX = 1,
  RSM_MIN = 2,
  RSM_PROD = 3,
  RSM_AND = 4,
  RSM_OR = 5,
  RSM_XOR = 6
};

enum rsm_rma_kind { RSM_PUT = 0, RSM_GET = 1, RSM_PUT_NBI = 2, RSM_GET_NBI = 3 };
/* RSM_WG_SHARED: every message is moved by all workgroups of the PE together
 * (roc_shmemx_ctx_{put,get}mem_wg_shard, an extension); it is complete when the launch is
 * (stream order): the kernel issues no quiet of its own, since a message is complete only
 * when every workgroup that shares it has returned. */
enum rsm_granularity { RSM_THREAD = 0, RSM_WAVE = 1, RSM_WG = 2, RSM_WG_SHARED = 3 };

/* Kinds of the small-operation stream executed by rsm_small_ops(). */
enum rsm_small_kind {
  RSM_OP_P64 = 0,        /* roc_shmem_ctx_long_p            (8-byte inline put)        */
  RSM_OP_FADD64 = 1,     /* roc_shmem_ctx_int64_atomic_fetch_add                       */
  RSM_OP_ADD64 = 2,      /* roc_shmem_ctx_int64_atomic_add                             */
  RSM_OP_FINC64 = 3,     /* roc_shmem_ctx_int64_atomic_fetch_inc                       */
  RSM_OP_INC64 = 4,      /* roc_shmem_ctx_int64_atomic_inc                             */
  RSM_OP_CSWAP64 = 5,    /* roc_shmem_ctx_int64_atomic_compare_swap (cond in `aux`)    */
  RSM_OP_FETCH64 = 6,    /* roc_shmem_ctx_int64_atomic_fetch                           */
  RSM_OP_SET64 = 7,      /* roc_shmem_ctx_int64_atomic_set                             */
  RSM_OP_SWAP64 = 8,     /* roc_shmem_ctx_int64_atomic_swap                            */
  RSM_OP_P32 = 9,        /* roc_shmem_ctx_int_p             (4-byte inline put)        */
  RSM_OP_FADD32 = 10,    /* roc_shmem_ctx_int_atomic_fetch_add                         */
  RSM_OP_PUTMEM = 11,    /* roc_shmem_ctx_putmem_nbi of `aux` bytes from `value` (a symmetric offset) */
  RSM_OP_GETMEM = 12,    /* roc_shmem_ctx_getmem_nbi of `aux` bytes into `value` (a symmetric offset) */
  RSM_OP_FAND64 = 13,    /* roc_shmem_ctx_uint64_atomic_fetch_and                      */
  RSM_OP_FOR64 = 14,     /* roc_shmem_ctx_uint64_atomic_fetch_or                       */
  RSM_OP_FXOR64 = 15,    /* roc_shmem_ctx_uint64_atomic_fetch_xor                      */
  RSM_OP_NONE = 255      /* lane sits this round out (stays inactive)                  */
};

/* One small operation: issued by the thread that owns it, towards PE `pe`,
 * on the symmetric object at byte offset `offset` of the heap. */
typedef struct rsm_small_op {
  uint32_t kind;
  uint32_t pe;
  uint64_t offset;
  int64_t value;
  int64_t aux;
} rsm_small_op_t;

/* Host threads.  Entry points may be called from any host thread; the library
 * runs one of them at a time (one recursive lock around the whole interface).
 * Kernels they launch on different streams still run concurrently on the
 * device; two launches that use the same contexts (the same (PE, workgroup
 * index) pairs) at the same time share send queues and pSync slices and must
 * not overlap. */

/* Argument checks of the data-path entry points.  A symmetric operand must lie
 * inside a live allocation of rsm_malloc and the bytes the call touches
 * (elements x element size, team size x block, messages x stride, wgs_per_pe
 * pSync slices) must fit that allocation; otherwise the call returns non-zero
 * with a message in rsm_last_error() and launches nothing.  The reference
 * checks none of this; a kernel that runs past an allocation overwrites its
 * neighbours or faults the device. */

/* Launch shape shared by the data-path entry points. */
typedef struct rsm_launch {
  int wgs_per_pe;   /* workgroups acting for each PE (>= 1)                        */
  int wg_size;      /* threads per workgroup, multiple of 64, <= 1024              */
  size_t tile;      /* elements (or bytes) per device call; 0 = chosen by the entry point */
  void *stream;     /* hipStream_t, NULL = the default stream                      */
} rsm_launch_t;

/* ---- lifecycle (reference: roc_shmem_init/finalize/malloc/free/n_pes,
 *      library/src/roc_shmem.cpp:71-135) ------------------------------------- */

/* Arguments equal to 0 fall back to ROC_SHMEM_NUM_PES / ROC_SHMEM_HEAP_SIZE /
 * ROC_SHMEM_NUM_BLOCKS / ROC_SHMEM_SQ_SIZE and then to the defaults
 * (8 PEs, 1 GiB per PE, 64 contexts per PE, 1024-entry send queues). */
int rsm_init(int num_pes, size_t heap_bytes_per_pe, int num_blocks, unsigned sq_size);
int rsm_finalize(void);
int rsm_is_initialized(void);
const char *rsm_last_error(void);
int rsm_n_pes(void);
int rsm_num_blocks(void);
size_t rsm_heap_size(void);
size_t rsm_slice_stride(void);
void *rsm_malloc(size_t bytes);                 /* NULL on failure or bytes == 0 */
int rsm_free(void *ptr);
size_t rsm_heap_bytes_in_use(void);
void *rsm_ptr(const void *sym, int pe);         /* roc_shmem_ptr: address of `sym` in PE `pe`'s slice */
void *rsm_heap_base(int pe);                    /* first byte of PE `pe`'s slice (reference: base_heap[pe]) */
int rsm_state_units(void);                      /* translation units holding a copy of the device state */
int rsm_take_status(void);                      /* sticky device status word, cleared by the call */

/* Lockstep pacing of large sharded transfers and reductions (no counterpart in the
 * reference).  Rates are bytes of memory traffic per tick of the GPU's 100 MHz constant
 * clock; 0 switches pacing off.  Defaults: reductions 67000 (6.7 TB/s) when their passes are
 * 128 KiB per member (workgroups of 1024 lanes) and 63000 with shorter passes, copies 0; also
 * settable through ROC_SHMEM_PACE_REDUCE (both kinds of pass), ROC_SHMEM_PACE_REDUCE_SHORT and
 * ROC_SHMEM_PACE_COPY.  A reduce rate set through rsm_set_pacing holds for both kinds of pass
 * (setting the default for long passes again brings both defaults back); rsm_get_pacing
 * reports the rate for long passes.  With a rate set, the workgroups of large reductions -
 * sharded calls, and standard calls when the whole grid is inside calls like them - of
 * rsm_rma(..., RSM_WG_SHARED) transfers (roc_shmemx_ctx_{put,get}mem_wg_shard) of 64 passes
 * or more per workgroup and of large alltoalls that fill the chip issue their loads and stores
 * by a common schedule of time slots derived from the rate (a wave that is early waits for
 * its slot, one that is late goes at once) instead of drifting apart - in a reduction the
 * whole chip loads in one slot and stores in the next; results are the same, only the
 * timing changes.  The best rate is the one the card just sustains (fp32 sum over 8 x 2^26:
 * 6.00 TB/s free, 6.57 at 67000, 6.46 at 70000, 6.25 at 90000, 5.77 at 58000);
 * rsm_tune_reduce_pacing measures it for one reduction on this card. */
int rsm_set_pacing(unsigned copy_bytes_per_tick, unsigned reduce_bytes_per_tick);
int rsm_get_pacing(unsigned *copy_bytes_per_tick, unsigned *reduce_bytes_per_tick);
/* Measures, on this card and for this very reduction (same arguments as rsm_to_all, tile 0),
 * the rate at which sharded reductions are best paced: runs the reduction free and at rates
 * from 5.6 to 7.2 TB/s, nine launches each (about 0.25 s for 4 GiB of traffic), and sets the
 * reduce rate to the best one - or to 0 when pacing does not gain at least 1 % over
 * running free.  `dest` receives the reduction's ordinary result.  Outputs (may be
 * NULL): the rate set, milliseconds per launch free and as set.  Synchronous. */
int rsm_tune_reduce_pacing(int dtype, int op, void *dest, const void *source, size_t nreduce,
                           int pe_start, int log_pe_stride, int pe_size, long *pSync,
                           const rsm_launch_t *launch, unsigned *rate_out, float *free_ms_out,
                           float *paced_ms_out);

/* Plain streams over a symmetric buffer, to measure what the memory system of the card at
 * hand delivers (no counterpart in the reference): the grid's workgroups read
 * (RSM_STREAM_READ), write (RSM_STREAM_WRITE) or copy (RSM_STREAM_COPY: the first half onto
 * the second half) the `bytes_per_pe` bytes at `buf` of every PE's slice, one PE's after
 * the other, in passes dealt round-robin to the workgroups, all of them inside one compact
 * window at any moment, 16 bytes per lane per access, loads non-temporal, stores with the
 * policy of the collectives' results.  launch->tile is the size of a pass in bytes,
 * wg_size * 16 * {1, 2, 4, 8} (0 = 8 accesses, the 128 KiB passes of the library's large
 * collectives at 1024 lanes).  The shape of the launch matters more than the card: workgroups
 * that stay and take pass after pass, as a device-side collective's do, reach 6.3-6.9 TB/s
 * one way; a grid of as many small workgroups as passes (wgs_per_pe = passes per PE, 256
 * lanes, one access each), which the hardware hands out in address order, 7.1-7.6 TB/s;
 * copies stay at 6.1-6.7 TB/s either way.  The caller times the launches.
 * READ folds all 16-byte vectors of a PE's buffer with XOR into the four 32-bit words at
 * `checksum` (symmetric, 16 bytes, zeroed by the caller; NULL: the loads are performed and
 * nothing is folded, as a timed run of many small workgroups wants) of that PE's slice; WRITE stores
 * {i mod 2^32, i >> 32, pe, seed} into vector i.  `buf` and `bytes_per_pe` must be
 * multiples of 16 (32 for the copies).  For comparison, RSM_STREAM_RUNTIME_FILL and
 * RSM_STREAM_RUNTIME_COPY run the HIP runtime's own kernels over the same buffers, one call
 * per PE on the launch's stream (the launch's shape is not used): hipMemsetAsync of every
 * byte to `seed` & 0xff, and hipMemcpyAsync of each buffer's first half onto its second
 * half.  Those two are not for a stream under graph capture. */
enum rsm_stream_kind {
  RSM_STREAM_READ = 0,
  RSM_STREAM_WRITE = 1,
  RSM_STREAM_RUNTIME_FILL = 2,
  RSM_STREAM_RUNTIME_COPY = 3,
  RSM_STREAM_COPY = 4
};
int rsm_stream_probe(int kind, void *buf, size_t bytes_per_pe, void *checksum, unsigned seed,
                     const rsm_launch_t *launch);

/* ---- teams (reference: roc_shmem.cpp:188-313, team.cpp:47-107) ------------ */

uint64_t rsm_team_world(void);
int rsm_team_split_strided(uint64_t parent, int start, int stride, int size, uint64_t *new_team);
int rsm_team_destroy(uint64_t team);
int rsm_team_n_pes(uint64_t team);
int rsm_team_translate_pe(uint64_t src_team, int src_pe, uint64_t dst_team);

/* ---- plumbing: host<->device copies, streams, events ---------------------- */

int rsm_copy_to_device(void *dst, const void *host_src, size_t bytes);
int rsm_copy_to_host(void *host_dst, const void *src, size_t bytes);
int rsm_fill(void *dst, int byte_value, size_t bytes);
int rsm_synchronize(void);
int rsm_stream_synchronize(void *stream);       /* NULL = the default stream */
void *rsm_device_alloc(size_t bytes);           /* ordinary (non-symmetric) device memory */
int rsm_device_free(void *ptr);
void *rsm_stream_create(void);
int rsm_stream_destroy(void *stream);
void *rsm_event_create(void);
int rsm_event_destroy(void *event);
int rsm_event_record(void *event, void *stream);
int rsm_event_elapsed_ms(void *start, void *stop, float *ms);   /* synchronises on `stop` */

/* Graphs (no counterpart in the reference; for launch-bound sequences of small
 * operations).  The data-path entry points below (rsm_to_all*, rsm_broadcast*,
 * rsm_alltoall, rsm_fcollect, rsm_barrier_all, rsm_putmem/rsm_getmem, rsm_small_ops)
 * only launch kernels on launch->stream: between rsm_capture_begin(stream) and
 * rsm_capture_end(stream) they are recorded instead of run.  rsm_capture_end returns
 * an executable graph (NULL on error); rsm_graph_launch replays it on any stream.
 * `stream` must come from rsm_stream_create.  Symmetric objects named by the
 * recorded calls must stay allocated while the graph is in use; calls that copy,
 * allocate or synchronise (lifecycle, memory, inspection) must stay outside. */
int rsm_capture_begin(void *stream);
void *rsm_capture_end(void *stream);
int rsm_graph_launch(void *graph, void *stream);
int rsm_graph_destroy(void *graph);

/* ---- reductions ------------------------------------------------------------
 * roc_shmem_ctx_<T>_<op>_wg_to_all, active-set form (roc_shmem.hpp:837-851;
 * GPUIBContext::to_all, gpu_ib/context_ib_tmpl_device.hpp:262-307).  With
 * `launch->tile` > 0, workgroup w of every member PE makes one standard call
 * per tile w, w+wgs_per_pe, ... of `launch->tile` elements.  With tile == 0 the
 * PE's workgroups share a single reduction through the sharded extension
 * (roc_shmemx_ctx_<T>_<op>_wg_to_all_shard: passes of the whole range dealt
 * round-robin to members and workgroups).  Either way workgroup w uses its own
 * pSync slice pSync + w*256: `pSync` holds wgs_per_pe*256 longs, all
 * ROC_SHMEM_SYNC_VALUE on entry and on return; `pWrk` may be NULL (unused). */
int rsm_to_all(int dtype, int op, void *dest, const void *source, size_t nreduce, int pe_start,
               int log_pe_stride, int pe_size, void *pWrk, long *pSync,
               const rsm_launch_t *launch);
/* rsm_to_all for callers that cannot allocate device memory (code recorded into a HIP
 * graph, serving loops, harnesses that forbid hipMalloc).  No counterpart in the
 * reference, whose active-set reductions always take the caller's pSync.  Same result
 * as rsm_to_all with launch->tile == 0 (the sharded form); the synchronisation flags live
 * in an array of the library's own (4 MiB of device memory per GPU, held until the process
 * ends) instead of a caller-allocated pSync, and the call allocates and frees nothing.
 * Limit: num_pes * launch->wgs_per_pe <= 2048 workgroups and launch->tile == 0, otherwise the
 * call fails with a message and launches nothing.  All calls on one GPU share the array:
 * calls that overlap in time on one GPU (different streams, different host threads) race;
 * calls that follow each other on one stream are safe. */
int rsm_to_all_noalloc(int dtype, int op, void *dest, const void *source, size_t nreduce,
                       int pe_start, int log_pe_stride, int pe_size, const rsm_launch_t *launch);
/* Team form (roc_shmem.hpp:848-851; context_ib_tmpl_device.hpp:238-260). */
int rsm_to_all_team(int dtype, int op, uint64_t team, void *dest, const void *source,
                    size_t nreduce, const rsm_launch_t *launch);

/* ---- workgroup / wavefront / thread RMA -------------------------------------
 * roc_shmemx_ctx_{put,get}mem[_nbi]_{wg,wave} and roc_shmem_ctx_{put,get}mem[_nbi]
 * (roc_shmem.hpp:907-977,2029-2566; context_ib_device.cpp:84-321).  PE p
 * moves messages m = 0..n_msgs-1 of `msg_bytes` each between its own
 * `source + m*src_stride` / `dest + m*dst_stride` and PE (p+pe_shift)%n_pes,
 * the messages being dealt round-robin to its workgroups, waves or threads
 * according to `granularity`.  Every workgroup ends with a quiet; with the non-blocking
 * kinds a workgroup (wave, thread) also issues one after every 64 of its calls, the window
 * of the reference's message-rate kernel (clients/functional_tests/primitive_mr_tester.cpp:
 * 44-49). */
int rsm_rma(int kind, int granularity, void *dest, const void *source, size_t msg_bytes,
            size_t n_msgs, size_t dst_stride, size_t src_stride, int pe_shift,
            const rsm_launch_t *launch);

/* ---- broadcast / alltoall / fcollect / barrier -------------------------------
 * roc_shmem_ctx_<T>_wg_broadcast (roc_shmem.hpp:873-887; context_ib_tmpl_device.hpp:
 * 455-519): `pe_root` is the root's ordinal in the active set; the root's
 * dest is not written.  Tiled like rsm_to_all (pSync: wgs_per_pe*256 longs). */
int rsm_broadcast(size_t elem_size, void *dest, const void *source, size_t nelem, int pe_root,
                  int pe_start, int log_pe_stride, int pe_size, long *pSync,
                  const rsm_launch_t *launch);
int rsm_broadcast_team(size_t elem_size, uint64_t team, void *dest, const void *source,
                       size_t nelem, int pe_root, const rsm_launch_t *launch);
/* roc_shmem_ctx_<T>_wg_alltoall (roc_shmem.hpp:892-895; context_ib_tmpl_device.hpp:
 * 521-558) and _wg_fcollect (:899-902; :845-876).  With wgs_per_pe > 1 the
 * workgroups of a PE call the sharded extension, one shard each. */
int rsm_alltoall(size_t elem_size, uint64_t team, void *dest, const void *source, size_t nelem,
                 const rsm_launch_t *launch);
int rsm_fcollect(size_t elem_size, uint64_t team, void *dest, const void *source, size_t nelem,
                 const rsm_launch_t *launch);
/* roc_shmem_ctx_wg_barrier_all repeated `iterations` times by every workgroup
 * (context_ib_device_coll.cpp:105-120). */
int rsm_barrier_all(int iterations, const rsm_launch_t *launch);

/* ---- small puts and AMOs ------------------------------------------------------
 * Thread t of the grid issues ops[t], ops[t+T], ... (T = total threads) through
 * the thread-level API (roc_shmem.hpp:907-1147; context_ib_device.cpp:84-184,
 * context_ib_tmpl_device.hpp:365-453), every op also leaving its 64-byte WQE
 * in the issuing workgroup's send queue (queue_pair.cpp:205-273).  `ops` is
 * device memory.  `fetched` (device, n_ops int64, may be NULL) receives the
 * value returned by fetching operations.  An operation that names a PE that
 * does not exist or bytes outside the heap is skipped and raises the status
 * word (rsm_take_status() == 2) instead of faulting the device. */
int rsm_small_ops(const rsm_small_op_t *ops, size_t n_ops, int64_t *fetched,
                  const rsm_launch_t *launch);

/* ---- send-queue inspection (reference: debug_print_sq, include/debug.hpp,
 *      gpu_ib/qe_dumper.cpp:51-76) ---------------------------------------------- */

int rsm_sq_reset(void);                                        /* zero all rings and indices */
int rsm_sq_read(int pe, int block, unsigned index, uint64_t out_words[8]);
int rsm_sq_image(int pe, int block, void *host_out, size_t bytes);
int rsm_sq_state(int pe, int block, uint32_t *sq_counter, uint32_t *published,
                 uint32_t *atomic_counter, uint64_t mailbox[2]);
/* Per-queue constants a CPU WQE builder needs. */
int rsm_sq_constants(int pe, int block, uint32_t *ctrl_qp_sq, uint64_t *ctrl_sig, uint32_t *lkey,
                     uint32_t *atomic_lkey, uint64_t *atomic_ret_base, uint32_t *max_nwqe);
int rsm_sq_rkey(int dest_pe, uint32_t *rkey);
/* What a fence's entry on a live queue is addressed to: PE `pe`'s flush word and the key it
 * is named under (reference: hdp_address[] / hdp_rkey[], network_policy.cpp:114-180;
 * QueuePair::fence, queue_pair.cpp:376-384). */
int rsm_sq_flush_target(int pe, uint64_t *addr, uint32_t *rkey);

/* ---- consumer pass, completion queues, queue mode -----------------------------------
 * What a NIC does with the rings in the reference: take published entries off
 * a ring in order, complete them (reference reader: QueuePair::quiet_internal,
 * gpu_ib/queue_pair.cpp:118-191) and free their slots (waitSQSpace,
 * queue_pair.cpp:400-415).  Here a kernel does it, between producer kernels. */
typedef struct rsm_consume_totals {
  uint64_t retired;        /* entries taken off the rings                          */
  uint64_t writes;         /* RDMA WRITE entries, inline or not                    */
  uint64_t reads;          /* RDMA READ entries                                    */
  uint64_t atomics;        /* fetch-add and compare-and-swap entries               */
  uint64_t bytes;          /* payload bytes the entries describe                   */
  uint64_t completions;    /* completion entries written                           */
  uint64_t lost;           /* entries overwritten before the pass saw them         */
  uint64_t rejected;       /* malformed entries: retired, never executed           */
  uint64_t local_skipped;  /* local buffer outside the symmetric heap: not executed */
} rsm_consume_totals_t;
/* Retire what the rings of PE `pe`, block `block` (-1: all) have published.
 * `target_arena` NULL: check every entry and write completions only.  Otherwise
 * a device buffer laid out like the arena (rsm_arena): every well-formed entry
 * is also executed against it, ring by ring in index order - replaying the
 * rings onto a copy of the arena taken before the producers ran reproduces
 * what they did (swap / set, recorded as compare-and-swap with compare operand
 * 0, only where the target held 0).  Payloads of non-inline writes are read
 * where the producer left them.  Synchronous. */
int rsm_sq_consume(int pe, int block, void *target_arena, rsm_consume_totals_t *totals);
/* 0 (default, or ROC_SHMEM_SQ_MODE unset): rings are logs, a slot is reused once
 * its previous entry is published.  1 (ROC_SHMEM_SQ_MODE=queue): rings are queues,
 * a slot is reused only after rsm_sq_consume retired it; a producer that finds
 * its ring full waits (bounded) and raises the status word. */
int rsm_sq_set_mode(int queue_mode);
/* A consumer that runs at the same time as the producers (what the NIC is to the
 * reference's queues: entries are retired while kernels post, QueuePair::quiet_internal
 * reads the completions, queue_pair.cpp:118-191, waitSQSpace blocks on retirement,
 * :400-415).  rsm_sq_consumer_start switches the rings to queue mode, launches a
 * persistent kernel on a stream of the library's own that checks and retires what the
 * rings publish (completion entries, `consumed`), and returns when all its waves are
 * resident.  Until rsm_sq_consumer_stop, producers (rsm_small_ops and any kernel that
 * posts) block in their post when their ring is full and go on when the consumer has freed
 * slots; roc_shmem_ctx_quiet posts a zero-byte read (READ, DS = 2; QueuePair::zero_b_rd,
 * queue_pair.cpp:318-325, as the reference's quiet does, thread_policy.cpp:35-108) and collects
 * the completions its queue has asked for, that entry's included (bounded waits, status word
 * on timeout); roc_shmem_ctx_fence posts the flush write of QueuePair::fence
 * (queue_pair.cpp:376-384).  Without a live consumer neither posts anything: both are memory
 * fences, and nothing would complete the entries.  Entries and completions are written
 * through to memory meanwhile, and the pacing of large reductions and copies rests (rates 0;
 * restored by rsm_sq_consumer_stop): a paced grid counts on all its workgroups being
 * resident, which the consumer's waves may prevent.  rsm_sq_consumer_stop: call it when the producers' streams have been
 * synchronised (it synchronises the default stream itself); it lets the consumer drain the
 * rings, waits for it, restores the previous mode and returns what was retired.  Between
 * the two calls synchronise streams, not the device: entry points that synchronise the
 * device (rsm_synchronize, rsm_take_status, rsm_sq_reset, rsm_sq_consume) refuse to run,
 * and a consumer wave whose rings stay silent for ROC_SHMEM_CONSUMER_IDLE_S seconds
 * (default 5) leaves by itself, which rsm_sq_consumer_stop reports as an error. */
int rsm_sq_consumer_start(void);
int rsm_sq_consumer_stop(rsm_consume_totals_t *totals);
int rsm_sq_consumer_running(void);
/* Reader side of a completion queue (reference: cq_consumer_counter, quiet_counter,
 * dbrec_cq, queue_pair.hpp:340-396): completions taken by quiet, completions asked for
 * and not yet taken, and the completion queue's doorbell record. */
int rsm_cq_reader_state(int pe, int block, uint32_t *cq_consumer, uint32_t *quiet_counter,
                        uint32_t *cq_doorbell_record);
int rsm_sq_consumer_state(int pe, int block, uint32_t *consumed, uint32_t *cq_producer);
int rsm_cq_image(int pe, int block, void *host_out, size_t bytes);        /* sq_size x 64 B */
int rsm_atomic_ret_image(int pe, int block, void *host_out, size_t bytes); /* 4096 x 8 B     */
/* The arena holding every PE slice: PE p's heap starts at base + p*slice_stride. */
int rsm_arena(void **base, size_t *bytes, size_t *slice_stride);

/* ---- wave-level known-answer drivers ----------------------------------------------
 * Block::fetch_incr contract (containers/share_strategy.hpp:70-83): lanes named
 * by `lane_mask` of every wave of an n_wgs x wg_size grid call the
 * wave-aggregated fetch-and-add on one zeroed counter.  `per_thread` (host,
 * n_wgs*wg_size uint64, ~0 for inactive lanes) gets each lane's value,
 * `*counter_out` the final counter. */
int rsm_kat_fetch_incr(uint64_t lane_mask, int n_wgs, int wg_size, uint64_t *per_thread,
                       uint64_t *counter_out);
/* WfCoalOn::coalesce contract (wf_coal_policy.cpp:57-172) for one wave: inputs
 * are 64-entry host arrays; outputs must_send[64] (0/1) and out_size[64]. */
int rsm_kat_coalesce(uint64_t lane_mask, const int32_t *pe, const uint64_t *src,
                     const uint64_t *dst, const uint64_t *size, uint8_t *must_send,
                     uint64_t *out_size);

/* ---- host-logic hooks (no GPU needed) ------------------------------------------------
 * A free-standing instance of the symmetric-heap allocator that rsm_malloc uses
 * (reference behaviour: library/src/memory/pow2_bins.hpp:90-125,264-287): offsets
 * inside a heap of `heap_bytes`; rsm_host_alloc_alloc returns (size_t)-1 when
 * nothing fits or the request is 0. */
void *rsm_host_alloc_create(size_t heap_bytes);
void rsm_host_alloc_destroy(void *allocator);
size_t rsm_host_alloc_alloc(void *allocator, size_t request);
int rsm_host_alloc_free(void *allocator, size_t offset);
size_t rsm_host_alloc_in_use(void *allocator);
/* The range check rsm_to_all and rsm_broadcast apply to an active set before they launch
 * (members pe_start + k * 2^log_pe_stride, k < pe_size, must all be PEs below num_pes;
 * reference: the PE_start / logPE_stride / PE_size triple of roc_shmem.hpp:837-847).
 * 1 when the set is acceptable, 0 otherwise. */
int rsm_host_active_set_in_range(int pe_start, int log_pe_stride, int pe_size, int num_pes);

#ifdef __cplusplus
}
#endif

#endif
