/* amo.c -- sequential model of small puts and atomic memory operations.
 * Test infrastructure only (see oracle.h).
 *
 * Restates the meaning of the thread-level calls
 * (library/src/roc_shmem_gpu.cpp:298-330,555-640; GPUIBContext::p / amo_*,
 * library/src/gpu_ib/context_ib_tmpl_device.hpp:115-118,365-453) and of the
 * host-centric equivalents MPI_Fetch_and_op(MPI_SUM) / MPI_Compare_and_swap
 * (library/src/host/host_templates.hpp:285-331): fetch_inc = fetch_add(1),
 * inc = add(1), fetch = fetch_add(0); compare_swap(dest, cond, value) stores
 * `value` iff *dest == cond and returns the old value; set/swap exchange
 * unconditionally.  Operands have the width of their type (the reference's
 * NIC path always moves 64 bits, queue_pair.cpp:251-254,346, which clobbers
 * the neighbour of a 32-bit operand; that defect is not restated).
 *
 * Applying the operations one after the other is one legal serialisation of
 * any concurrent execution.  The final heap does not depend on the order as
 * long as the stream obeys the usual rules: put targets are distinct and
 * disjoint from AMO targets, and the AMOs on one word commute (adds with
 * adds, bitwise ops of one kind).  Fetched values of concurrent executions
 * are a permutation of this model's along each word only for equal addends.
 *
 * Pinned by: clients/functional_tests/amo_standard_tester.cpp:76-117 closed forms
 * (fetch_add -> 2*(n-1) last fetched, fetch_inc -> n-1, add -> 2*n, inc -> n),
 * clients/sos_tests/cxx_test_shmem_atomic_add.cpp:85-144 (npes*(npes+1)/2),
 * lfinc.cpp:90-111 (fetch_inc returns 0..n-1 in issue order),
 * cxx_test_shmem_atomic_cswap.cpp, amo_bitwise_tester.cpp:74-121.
 */
#include <string.h>

#include "oracle.h"

enum {
  K_P64 = 0, K_FADD64, K_ADD64, K_FINC64, K_INC64, K_CSWAP64, K_FETCH64, K_SET64, K_SWAP64,
  K_P32, K_FADD32, K_PUTMEM, K_GETMEM, K_FAND64, K_FOR64, K_FXOR64
};

int orc_small_ops(char *heap, size_t stride, const orc_small_op_t *ops, const uint32_t *issuer_pe,
                  size_t n, int64_t *fetched) {
  for (size_t i = 0; i < n; ++i) {
    const orc_small_op_t *o = &ops[i];
    if (o->kind == 255) continue;
    char *target = heap + (size_t)o->pe * stride + o->offset;
    char *mine = heap + (size_t)issuer_pe[i] * stride;
    int64_t old64 = 0;
    int fetches = 0;
    switch (o->kind) {
      case K_P64: memcpy(target, &o->value, 8); break;
      case K_P32: { int32_t v = (int32_t)o->value; memcpy(target, &v, 4); } break;
      case K_FADD64: case K_ADD64: case K_FINC64: case K_INC64: case K_FETCH64: {
        int64_t add = (o->kind == K_FINC64 || o->kind == K_INC64) ? 1
                      : (o->kind == K_FETCH64) ? 0 : o->value;
        memcpy(&old64, target, 8);
        uint64_t nv = (uint64_t)old64 + (uint64_t)add;
        memcpy(target, &nv, 8);
        fetches = (o->kind == K_FADD64 || o->kind == K_FINC64 || o->kind == K_FETCH64);
      } break;
      case K_CSWAP64:
        memcpy(&old64, target, 8);
        if (old64 == o->aux) memcpy(target, &o->value, 8);
        fetches = 1;
        break;
      case K_SET64: memcpy(target, &o->value, 8); break;
      case K_SWAP64:
        memcpy(&old64, target, 8);
        memcpy(target, &o->value, 8);
        fetches = 1;
        break;
      case K_FADD32: {
        int32_t old32;
        memcpy(&old32, target, 4);
        uint32_t nv = (uint32_t)old32 + (uint32_t)(int32_t)o->value;
        memcpy(target, &nv, 4);
        old64 = old32;
        fetches = 1;
      } break;
      case K_PUTMEM: memmove(target, mine + o->value, (size_t)o->aux); break;
      case K_GETMEM: memmove(mine + o->value, target, (size_t)o->aux); break;
      case K_FAND64: case K_FOR64: case K_FXOR64: {
        uint64_t cur, v = (uint64_t)o->value;
        memcpy(&cur, target, 8);
        old64 = (int64_t)cur;
        cur = o->kind == K_FAND64 ? (cur & v) : o->kind == K_FOR64 ? (cur | v) : (cur ^ v);
        memcpy(target, &cur, 8);
        fetches = 1;
      } break;
      default: return -1;
    }
    if (fetches && fetched) fetched[i] = old64;
  }
  return 0;
}
