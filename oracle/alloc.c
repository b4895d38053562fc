/* alloc.c -- model of the symmetric-heap allocator.  Test infrastructure only
 * (see oracle.h).
 *
 * Restates the observable behaviour of the reference's Pow2Bins strategy:
 * library/src/memory/pow2_bins.hpp:90-125 (alloc: exact bin, refilled from the
 * next larger non-empty bin), :264-287 (split: the record is halved, the upper
 * half is pushed first so the lower half is handed out first), :149-152 (free:
 * the block returns to the bin of its size, blocks are never merged);
 * library/src/memory/binner.hpp:109-134,190-231 (bins are the powers of two from
 * 128 bytes up, the heap is assigned as its binary decomposition);
 * library/src/memory/bin.hpp (a bin is a LIFO stack).
 * Pinned by: clients/unit_tests/single_heap_gtest.cpp:26-142 and
 * pow2_bins_gtest.cpp:26-157 (alloc(1) takes 128 bytes, alloc(4097) takes 8192,
 * alloc(0) yields nothing, a fresh 1 GiB heap satisfies one 1 GiB request), and
 * offset for offset by the reference's own Pow2Bins compiled from its sources
 * (build_ref.sh, ref_alloc_wrapper.cpp) on fresh heaps and random alloc/free
 * sequences (tests/test_host_allocator.py).
 */
#include <stdlib.h>
#include <string.h>

#include "oracle.h"

#define ORC_BINS 56
#define ORC_MIN_SHIFT 7

struct orc_alloc {
  size_t heap_bytes;
  size_t *stack[ORC_BINS];
  size_t depth[ORC_BINS], cap[ORC_BINS];
  size_t *live_off, *live_size;
  size_t n_live, cap_live;
};

static void bin_push(orc_alloc_t *a, int b, size_t off) {
  if (a->depth[b] == a->cap[b]) {
    a->cap[b] = a->cap[b] ? a->cap[b] * 2 : 8;
    a->stack[b] = (size_t *)realloc(a->stack[b], a->cap[b] * sizeof(size_t));
  }
  a->stack[b][a->depth[b]++] = off;
}

orc_alloc_t *orc_alloc_create(size_t heap_bytes) {
  orc_alloc_t *a = (orc_alloc_t *)calloc(1, sizeof(*a));
  a->heap_bytes = heap_bytes;
  size_t off = 0;
  for (int b = ORC_BINS - 1; b >= 0; --b) {
    size_t s = (size_t)1 << (b + ORC_MIN_SHIFT);
    if (heap_bytes - off >= s) {
      bin_push(a, b, off);
      off += s;
    }
  }
  return a;
}

void orc_alloc_destroy(orc_alloc_t *a) {
  if (!a) return;
  for (int b = 0; b < ORC_BINS; ++b) free(a->stack[b]);
  free(a->live_off);
  free(a->live_size);
  free(a);
}

static int refill(orc_alloc_t *a, int b) {
  if (b + 1 >= ORC_BINS) return 0;
  if (a->depth[b + 1] == 0 && !refill(a, b + 1)) return 0;
  size_t block = a->stack[b + 1][--a->depth[b + 1]];
  bin_push(a, b, block + ((size_t)1 << (b + ORC_MIN_SHIFT)));
  bin_push(a, b, block);
  return 1;
}

size_t orc_alloc_alloc(orc_alloc_t *a, size_t request) {
  if (!request) return (size_t)-1;
  int b = 0;
  while (b < ORC_BINS && ((size_t)1 << (b + ORC_MIN_SHIFT)) < request) ++b;
  if (b >= ORC_BINS || ((size_t)1 << (b + ORC_MIN_SHIFT)) > a->heap_bytes) return (size_t)-1;
  if (a->depth[b] == 0 && !refill(a, b)) return (size_t)-1;
  size_t off = a->stack[b][--a->depth[b]];
  if (a->n_live == a->cap_live) {
    a->cap_live = a->cap_live ? a->cap_live * 2 : 16;
    a->live_off = (size_t *)realloc(a->live_off, a->cap_live * sizeof(size_t));
    a->live_size = (size_t *)realloc(a->live_size, a->cap_live * sizeof(size_t));
  }
  a->live_off[a->n_live] = off;
  a->live_size[a->n_live] = (size_t)1 << (b + ORC_MIN_SHIFT);
  ++a->n_live;
  return off;
}

int orc_alloc_free(orc_alloc_t *a, size_t offset) {
  for (size_t i = 0; i < a->n_live; ++i) {
    if (a->live_off[i] == offset) {
      int b = 0;
      while (((size_t)1 << (b + ORC_MIN_SHIFT)) < a->live_size[i]) ++b;
      bin_push(a, b, offset);
      a->live_off[i] = a->live_off[a->n_live - 1];
      a->live_size[i] = a->live_size[a->n_live - 1];
      --a->n_live;
      return 0;
    }
  }
  return -1;
}

size_t orc_alloc_in_use(const orc_alloc_t *a) {
  size_t t = 0;
  for (size_t i = 0; i < a->n_live; ++i) t += a->live_size[i];
  return t;
}
