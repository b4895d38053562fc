/* rma.c -- put / get / broadcast / alltoall / fcollect as byte moves between
 * slices.  Test infrastructure only (see oracle.h).
 *
 * put/get: library/src/gpu_ib/context_ib_device.cpp:84-119,148-321 -- the target
 *   address is base_heap[pe] + (ptr - base_heap[my_pe]); the intended effect
 *   of the copy helpers in library/src/util.hpp:248-325 is memcpy(dst, src, n).
 *   Host-centric equivalent: MPI_Put / MPI_Get of MPI_CHAR,
 *   library/src/host/host_helpers.hpp:52-88.
 * broadcast: context_ib_tmpl_device.hpp:455-519 -- every member except the root
 *   receives the root's source; the root's dest is untouched.
 * alltoall: context_ib_tmpl_device.hpp:528-558 -- member i's block j lands in
 *   member j's block i, self block included.
 * fcollect: context_ib_tmpl_device.hpp:845-876 -- member i's block lands in
 *   block i of every member.
 *
 * Pinned by: clients/functional_tests/primitive_tester.cpp:97-129 and
 * extended_primitives.cpp:87-119 ('0' fill arrives over a '1' fill),
 * clients/sos_tests/put1.cpp, bigput.cpp:202-263 (Source[i] = i+1),
 * tester.cpp:236-271 and sos_tests/broadcast_active_set.cpp:84-128 (root's dest
 * keeps its old value), tester.cpp:310-334 ((src_pe << 16) + dst_pe pattern),
 * tester.cpp:336-355 (fcollect value = source rank).  The team forms with a
 * stride that is not a power of two have no test in the reference; they are
 * pinned by moving the blocks by hand in numpy and by agreement with the
 * active-set forms for powers of two (tests/test_oracle_team_strides.py).
 */
#include <pthread.h>
#include <string.h>

#include "oracle.h"

/* Member k of the set {pe_start + k * pe_stride}: 1 << logPE_stride for an active set, any stride
 * for a team (roc_shmem_team_split_strided, library/src/roc_shmem.cpp:236-250). */
static int member_pe(int k, int pe_start, int pe_stride) { return pe_start + k * pe_stride; }

void orc_put(char *heap, size_t stride, size_t dest_off, size_t src_off, size_t nbytes,
             int src_pe, int dest_pe) {
  if (!nbytes) return;  /* zero-length RMA is a no-op, context_device.cpp:80-82 */
  memmove(heap + (size_t)dest_pe * stride + dest_off, heap + (size_t)src_pe * stride + src_off,
          nbytes);
}

void orc_get(char *heap, size_t stride, size_t dest_off, size_t src_off, size_t nbytes,
             int my_pe, int from_pe) {
  if (!nbytes) return;
  memmove(heap + (size_t)my_pe * stride + dest_off, heap + (size_t)from_pe * stride + src_off,
          nbytes);
}

void orc_broadcast_team(char *heap, size_t stride, size_t dest_off, size_t src_off, size_t nbytes,
                   int root_idx, int pe_start, int pe_stride, int pe_size) {
  if (!nbytes) return;
  const char *src = heap + (size_t)member_pe(root_idx, pe_start, pe_stride) * stride + src_off;
  for (int m = 0; m < pe_size; ++m) {
    if (m == root_idx) continue;
    memmove(heap + (size_t)member_pe(m, pe_start, pe_stride) * stride + dest_off, src, nbytes);
  }
}

void orc_alltoall_team(char *heap, size_t stride, size_t dest_off, size_t src_off, size_t block_bytes,
                  int pe_start, int pe_stride, int pe_size) {
  if (!block_bytes) return;
  for (int i = 0; i < pe_size; ++i)
    for (int j = 0; j < pe_size; ++j)
      memmove(heap + (size_t)member_pe(j, pe_start, pe_stride) * stride + dest_off + (size_t)i * block_bytes,
              heap + (size_t)member_pe(i, pe_start, pe_stride) * stride + src_off + (size_t)j * block_bytes,
              block_bytes);
}

void orc_fcollect_team(char *heap, size_t stride, size_t dest_off, size_t src_off, size_t block_bytes,
                  int pe_start, int pe_stride, int pe_size) {
  if (!block_bytes) return;
  for (int i = 0; i < pe_size; ++i)
    for (int j = 0; j < pe_size; ++j)
      memmove(heap + (size_t)member_pe(j, pe_start, pe_stride) * stride + dest_off + (size_t)i * block_bytes,
              heap + (size_t)member_pe(i, pe_start, pe_stride) * stride + src_off, block_bytes);
}

/* Active-set forms: the members are pe_start + (k << log_stride). */
void orc_broadcast(char *heap, size_t stride, size_t dest_off, size_t src_off, size_t nbytes,
                   int root_idx, int pe_start, int log_stride, int pe_size) {
  orc_broadcast_team(heap, stride, dest_off, src_off, nbytes, root_idx, pe_start, 1 << log_stride, pe_size);
}

void orc_alltoall(char *heap, size_t stride, size_t dest_off, size_t src_off, size_t block_bytes,
                  int pe_start, int log_stride, int pe_size) {
  orc_alltoall_team(heap, stride, dest_off, src_off, block_bytes, pe_start, 1 << log_stride, pe_size);
}

void orc_fcollect(char *heap, size_t stride, size_t dest_off, size_t src_off, size_t block_bytes,
                  int pe_start, int log_stride, int pe_size) {
  orc_fcollect_team(heap, stride, dest_off, src_off, block_bytes, pe_start, 1 << log_stride, pe_size);
}

struct copy_job { char *dst; const char *src; size_t n; };
static void *copy_worker(void *arg) {
  struct copy_job *j = (struct copy_job *)arg;
  memcpy(j->dst, j->src, j->n);
  return NULL;
}

void orc_copy_mt(char *dst, const char *src, size_t nbytes, int threads) {
  if (threads < 1) threads = 1;
  if (threads > 256) threads = 256;
  pthread_t tid[256];
  struct copy_job jobs[256];
  size_t share = (nbytes + threads - 1) / threads;
  share = (share + 63) & ~(size_t)63;
  for (int t = 0; t < threads; ++t) {
    size_t b = share * t, e = b + share;
    if (b > nbytes) b = nbytes;
    if (e > nbytes) e = nbytes;
    jobs[t] = (struct copy_job){dst + b, src + b, e - b};
    pthread_create(&tid[t], NULL, copy_worker, &jobs[t]);
  }
  for (int t = 0; t < threads; ++t) pthread_join(tid[t], NULL);
}
