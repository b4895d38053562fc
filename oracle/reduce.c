/* reduce.c -- reductions.  Test infrastructure only (see oracle.h).
 *
 * Restates library/src/gpu_ib/context_ib_tmpl_device.hpp:50-113 (OpWrap<Op>::Calc
 * and compute_reduce: `dst[i] = dst[i] (op) src[i]` in the element type) as
 * used by internal_direct_allreduce (:184-236): the destination starts as a
 * copy of one member's source and every other member's source is folded in.
 * Integer and/or/xor/max/min and wrapping sum/prod do not depend on the fold
 * order; for floating point the order here is ascending member index.  The
 * host-centric path gives the same answers through MPI_Allreduce
 * (library/src/host/host_templates.hpp:333-357).
 *
 * Pinned by: closed forms of clients/sos_tests/to_all.cpp:123-153,213-251,
 * 310-346,407-428,471-503,632-652,696-701; big_reduction.cpp:76-107;
 * reduce_in_place.cpp:58-69; reduce_active_set.cpp:78-113;
 * shmem_team_reduce.cpp:88-101; clients/functional_tests/tester.cpp:149-164;
 * a brute-force scalar fold on small random inputs; and, for floating
 * point, agreement of the in-type fold with the long-double ground truth on
 * exactly representable inputs.  The team form with a stride that is not a
 * power of two has no test in the reference (its collectives address members
 * by a truncated log2 of the stride, library/src/team.cpp:68); it is pinned by
 * brute-force folds over the members and by agreement with the active-set form
 * for strides that are powers of two (tests/test_oracle_team_strides.py).
 */
#include <math.h>
#include <pthread.h>
#include <stdlib.h>
#include <string.h>

#include "oracle.h"

size_t orc_dtype_size(int dtype) {
  switch (dtype) {
    case ORC_SHORT: case ORC_BF16: return 2;
    case ORC_INT: case ORC_FLOAT: return 4;
    case ORC_LONG: case ORC_LONGLONG: case ORC_DOUBLE: return 8;
    default: return 0;
  }
}

float orc_bf16_to_float(uint16_t b) {
  uint32_t u = (uint32_t)b << 16;
  float f;
  memcpy(&f, &u, 4);
  return f;
}

/* Round to nearest, ties to even; NaN stays NaN. */
uint16_t orc_float_to_bf16(float f) {
  uint32_t u;
  memcpy(&u, &f, 4);
  if ((u & 0x7fffffffu) > 0x7f800000u) return (uint16_t)((u >> 16) | 0x0040u);
  u += 0x7fffu + ((u >> 16) & 1u);
  return (uint16_t)(u >> 16);
}

/* Member k of the set {pe_start + k * pe_stride}.  The active-set calls pass 1 << logPE_stride; a
 * team may have any stride (roc_shmem_team_split_strided, library/src/roc_shmem.cpp:236-250). */
static int member_pe(int k, int pe_start, int pe_stride) { return pe_start + k * pe_stride; }

/* Integer fold on an unsigned carrier of the element's width: two's-complement
 * wrap for sum and prod, signed comparison for max and min. */
#define DEF_INT_FOLD(NAME, S, U)                                  \
  static S NAME(int op, S a, S b) {                               \
    switch (op) {                                                 \
      case ORC_SUM: return (S)(U)((U)a + (U)b);                   \
      case ORC_PROD: return (S)(U)((uint64_t)(U)a * (uint64_t)(U)b); \
      case ORC_AND: return (S)(a & b);                            \
      case ORC_OR: return (S)(a | b);                             \
      case ORC_XOR: return (S)(a ^ b);                            \
      case ORC_MAX: return a > b ? a : b;                         \
      default: return a < b ? a : b;                              \
    }                                                             \
  }
DEF_INT_FOLD(fold_i16, int16_t, uint16_t)
DEF_INT_FOLD(fold_i32, int32_t, uint32_t)
DEF_INT_FOLD(fold_i64, int64_t, uint64_t)

/* max/min ignore a NaN operand, as the device max()/min() overloads
 * (fmaxf/fminf) that OpWrap<ROC_SHMEM_MAX/MIN>::Calc calls do. */
static float fold_f32(int op, float a, float b) {
  switch (op) {
    case ORC_SUM: return a + b;
    case ORC_PROD: return a * b;
    case ORC_MAX: return (a >= b || b != b) ? a : b;
    default: return (a <= b || b != b) ? a : b;
  }
}
static double fold_f64(int op, double a, double b) {
  switch (op) {
    case ORC_SUM: return a + b;
    case ORC_PROD: return a * b;
    case ORC_MAX: return (a >= b || b != b) ? a : b;
    default: return (a <= b || b != b) ? a : b;
  }
}

static int op_defined(int dtype, int op) {
  if (op < ORC_SUM || op > ORC_XOR) return 0;
  if (dtype == ORC_FLOAT || dtype == ORC_DOUBLE) return op <= ORC_PROD;
  if (dtype == ORC_BF16) return op <= ORC_MIN;
  return dtype >= ORC_SHORT && dtype <= ORC_LONGLONG;
}

/* dst[i] = dst[i] (op) src[i] over [0, n): the shape of compute_reduce
 * (context_ib_tmpl_device.hpp:106-113), one typed loop per operator so the
 * compiler can vectorise it. */
#define DEF_COMBINE(NAME, T, FOLD)                                              \
  static void NAME(int op, T *restrict dst, const T *restrict src, size_t n) {  \
    switch (op) {                                                               \
      case ORC_SUM: for (size_t i = 0; i < n; ++i) dst[i] = FOLD(ORC_SUM, dst[i], src[i]); break;   \
      case ORC_PROD: for (size_t i = 0; i < n; ++i) dst[i] = FOLD(ORC_PROD, dst[i], src[i]); break; \
      case ORC_AND: for (size_t i = 0; i < n; ++i) dst[i] = FOLD(ORC_AND, dst[i], src[i]); break;   \
      case ORC_OR: for (size_t i = 0; i < n; ++i) dst[i] = FOLD(ORC_OR, dst[i], src[i]); break;     \
      case ORC_XOR: for (size_t i = 0; i < n; ++i) dst[i] = FOLD(ORC_XOR, dst[i], src[i]); break;   \
      case ORC_MAX: for (size_t i = 0; i < n; ++i) dst[i] = FOLD(ORC_MAX, dst[i], src[i]); break;   \
      default: for (size_t i = 0; i < n; ++i) dst[i] = FOLD(ORC_MIN, dst[i], src[i]); break;        \
    }                                                                           \
  }
DEF_COMBINE(combine_i16, int16_t, fold_i16)
DEF_COMBINE(combine_i32, int32_t, fold_i32)
DEF_COMBINE(combine_i64, int64_t, fold_i64)
DEF_COMBINE(combine_f32, float, fold_f32)
DEF_COMBINE(combine_f64, double, fold_f64)

/* bfloat16 has no arithmetic of its own.  A sum step is done in float and
 * rounded back to the element type, which is what an in-type
 * `dst[i] += src[i]` amounts to; max/min keep the selected operand's bits. */
static void combine_bf16(int op, uint16_t *restrict dst, const uint16_t *restrict src, size_t n) {
  for (size_t i = 0; i < n; ++i) {
    float fa = orc_bf16_to_float(dst[i]), fx = orc_bf16_to_float(src[i]);
    if (op == ORC_SUM) dst[i] = orc_float_to_bf16(fa + fx);
    else if (op == ORC_MAX) dst[i] = (fa >= fx || fx != fx) ? dst[i] : src[i];
    else dst[i] = (fa <= fx || fx != fx) ? dst[i] : src[i];
  }
}

/* Elements [e0, e1): the first member's destination starts as a copy of its
 * source, every other member's source is folded in ascending order, and the
 * result is copied to the remaining members' destinations.  The fold runs in
 * a bounded scratch block so that dest == source (in place) and misaligned
 * offsets are handled the same way. */
static void reduce_range(int dtype, int op, char *heap, size_t stride, size_t dest_off,
                         size_t src_off, size_t e0, size_t e1, int pe_start, int pe_stride,
                         int pe_size) {
  enum { BLOCK = 4096 };
  const size_t es = orc_dtype_size(dtype);
  union { int64_t i64[BLOCK]; double f64[BLOCK]; char bytes[BLOCK * 8]; } acc, in;
  for (size_t b = e0; b < e1; b += BLOCK) {
    const size_t n = (e1 - b < BLOCK) ? e1 - b : BLOCK;
    memcpy(acc.bytes, heap + (size_t)member_pe(0, pe_start, pe_stride) * stride + src_off + b * es, n * es);
    for (int k = 1; k < pe_size; ++k) {
      memcpy(in.bytes, heap + (size_t)member_pe(k, pe_start, pe_stride) * stride + src_off + b * es, n * es);
      switch (dtype) {
        case ORC_SHORT: combine_i16(op, (int16_t *)acc.bytes, (const int16_t *)in.bytes, n); break;
        case ORC_INT: combine_i32(op, (int32_t *)acc.bytes, (const int32_t *)in.bytes, n); break;
        case ORC_LONG: case ORC_LONGLONG: combine_i64(op, acc.i64, in.i64, n); break;
        case ORC_FLOAT: combine_f32(op, (float *)acc.bytes, (const float *)in.bytes, n); break;
        case ORC_DOUBLE: combine_f64(op, acc.f64, in.f64, n); break;
        default: combine_bf16(op, (uint16_t *)acc.bytes, (const uint16_t *)in.bytes, n); break;
      }
    }
    for (int m = 0; m < pe_size; ++m)
      memcpy(heap + (size_t)member_pe(m, pe_start, pe_stride) * stride + dest_off + b * es, acc.bytes, n * es);
  }
}

int orc_to_all(int dtype, int op, char *heap, size_t stride, size_t dest_off, size_t src_off,
               size_t n, int pe_start, int log_stride, int pe_size) {
  if (!op_defined(dtype, op)) return -1;
  reduce_range(dtype, op, heap, stride, dest_off, src_off, 0, n, pe_start, 1 << log_stride, pe_size);
  return 0;
}

/* The team form (GPUIBContext::to_all(team, ...), context_ib_tmpl_device.hpp:238-260): the members
 * are the team's, pe_start + k * pe_stride in world ranks. */
int orc_to_all_team(int dtype, int op, char *heap, size_t stride, size_t dest_off, size_t src_off,
                    size_t n, int pe_start, int pe_stride, int pe_size) {
  if (!op_defined(dtype, op) || pe_stride < 1) return -1;
  reduce_range(dtype, op, heap, stride, dest_off, src_off, 0, n, pe_start, pe_stride, pe_size);
  return 0;
}

/* The arithmetic the GPU library documents for its floating-point reductions,
 * restated so that its results can be compared bit for bit instead of by
 * tolerance: float sum and prod are folded in double in ascending member order
 * and rounded to float once; bfloat16 sum is folded in float and rounded to
 * bfloat16 once (nearest, ties to even); everything else is the in-type fold of
 * orc_to_all_team.  This is the library's contract, not the reference's: the
 * reference folds in the element type in an order that differs per PE and per
 * algorithm (context_ib_tmpl_device.hpp:120-236) and through MPI_Allreduce on
 * the host path, so its floating-point bits are not fixed by anything.  Pinned
 * by the ground truth: wherever the wide fold is exact (eight float terms
 * within 2^26 of each other, eight bfloat16 terms within 2^13), the result must
 * be the correctly rounded true sum, i.e. the long-double result of
 * orc_to_all_f64 rounded to the element type (tests/test_oracle_reduce.py). */
int orc_to_all_rounded_once(int dtype, int op, char *heap, size_t stride, size_t dest_off,
                            size_t src_off, size_t n, int pe_start, int pe_stride, int pe_size) {
  if (!op_defined(dtype, op) || pe_stride < 1) return -1;
  const int wide_float = dtype == ORC_FLOAT && (op == ORC_SUM || op == ORC_PROD);
  const int wide_bf16 = dtype == ORC_BF16 && op == ORC_SUM;
  if (!wide_float && !wide_bf16) {
    reduce_range(dtype, op, heap, stride, dest_off, src_off, 0, n, pe_start, pe_stride, pe_size);
    return 0;
  }
  const size_t es = orc_dtype_size(dtype);
  for (size_t i = 0; i < n; ++i) {
    char out[4];
    if (wide_float) {
      double acc = 0;
      for (int k = 0; k < pe_size; ++k) {
        float x;
        memcpy(&x, heap + (size_t)member_pe(k, pe_start, pe_stride) * stride + src_off + i * es, 4);
        acc = k == 0 ? (double)x : (op == ORC_SUM ? acc + (double)x : acc * (double)x);
      }
      float r = (float)acc;
      memcpy(out, &r, 4);
    } else {
      float acc = 0;
      for (int k = 0; k < pe_size; ++k) {
        uint16_t b;
        memcpy(&b, heap + (size_t)member_pe(k, pe_start, pe_stride) * stride + src_off + i * es, 2);
        acc = k == 0 ? orc_bf16_to_float(b) : acc + orc_bf16_to_float(b);
      }
      uint16_t r = orc_float_to_bf16(acc);
      memcpy(out, &r, 2);
    }
    for (int m = 0; m < pe_size; ++m)
      memcpy(heap + (size_t)member_pe(m, pe_start, pe_stride) * stride + dest_off + i * es, out, es);
  }
  return 0;
}

static long double load_ld(int dtype, const char *p) {
  switch (dtype) {
    case ORC_SHORT: { int16_t v; memcpy(&v, p, 2); return v; }
    case ORC_INT: { int32_t v; memcpy(&v, p, 4); return v; }
    case ORC_LONG: case ORC_LONGLONG: { int64_t v; memcpy(&v, p, 8); return (long double)v; }
    case ORC_FLOAT: { float v; memcpy(&v, p, 4); return v; }
    case ORC_DOUBLE: { double v; memcpy(&v, p, 8); return v; }
    default: { uint16_t v; memcpy(&v, p, 2); return orc_bf16_to_float(v); }
  }
}

int orc_to_all_f64(int dtype, int op, const char *heap, size_t stride, size_t src_off, size_t n,
                   int pe_start, int log_stride, int pe_size, double *out) {
  if (op != ORC_SUM && op != ORC_MAX && op != ORC_MIN && op != ORC_PROD) return -1;
  const size_t es = orc_dtype_size(dtype);
  if (!es) return -1;
  for (size_t i = 0; i < n; ++i) {
    long double acc = load_ld(dtype, heap + (size_t)member_pe(0, pe_start, 1 << log_stride) * stride + src_off + i * es);
    for (int k = 1; k < pe_size; ++k) {
      long double x = load_ld(dtype, heap + (size_t)member_pe(k, pe_start, 1 << log_stride) * stride + src_off + i * es);
      switch (op) {
        case ORC_SUM: acc += x; break;
        case ORC_PROD: acc *= x; break;
        case ORC_MAX: acc = (acc >= x || x != x) ? acc : x; break;
        default: acc = (acc <= x || x != x) ? acc : x; break;
      }
    }
    out[i] = (double)acc;
  }
  return 0;
}

int orc_abs_sum_f64(int dtype, const char *heap, size_t stride, size_t src_off, size_t n,
                    int pe_start, int log_stride, int pe_size, double *out) {
  const size_t es = orc_dtype_size(dtype);
  if (!es) return -1;
  for (size_t i = 0; i < n; ++i) {
    long double acc = 0;
    for (int k = 0; k < pe_size; ++k)
      acc += fabsl(load_ld(dtype, heap + (size_t)member_pe(k, pe_start, 1 << log_stride) * stride + src_off + i * es));
    out[i] = (double)acc;
  }
  return 0;
}

struct mt_job {
  int dtype, op;
  char *heap;
  size_t stride, dest_off, src_off, e0, e1;
  int pe_start, log_stride, pe_size;
};

static void *mt_worker(void *arg) {
  struct mt_job *j = (struct mt_job *)arg;
  reduce_range(j->dtype, j->op, j->heap, j->stride, j->dest_off, j->src_off, j->e0, j->e1,
               j->pe_start, 1 << j->log_stride, j->pe_size);
  return NULL;
}

int orc_to_all_mt(int dtype, int op, char *heap, size_t stride, size_t dest_off, size_t src_off,
                  size_t n, int pe_start, int log_stride, int pe_size, int threads) {
  if (!op_defined(dtype, op)) return -1;
  if (threads < 1) threads = 1;
  if (threads > 256) threads = 256;
  pthread_t tid[256];
  struct mt_job jobs[256];
  size_t share = (n + threads - 1) / threads;
  for (int t = 0; t < threads; ++t) {
    size_t e0 = share * t, e1 = e0 + share;
    if (e0 > n) e0 = n;
    if (e1 > n) e1 = n;
    jobs[t] = (struct mt_job){dtype, op, heap, stride, dest_off, src_off, e0, e1, pe_start, log_stride, pe_size};
    pthread_create(&tid[t], NULL, mt_worker, &jobs[t]);
  }
  for (int t = 0; t < threads; ++t) pthread_join(tid[t], NULL);
  return 0;
}
