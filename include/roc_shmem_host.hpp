// roc_shmem_host.hpp -- host-initiated data path of the roc_shmem_* interface.
//
// The reference forwards these calls to MPI one-sided operations and
// collectives (library/src/host/host_templates.hpp:151-357, host_helpers.hpp:
// 52-88; declared in library/include/roc_shmem.hpp:907-1147).  Here one process
// hosts every PE, so
//   * put/get/p/g and the AMOs act for the host's current PE
//     (roc_shmemx_set_pe) on PE `pe`'s slice: a device copy, or a
//     read-modify-write that is atomic with respect to other host calls;
//   * to_all and broadcast are collective in the reference (every PE's
//     process makes the call); here a single call performs the whole
//     collective for all member PEs by launching the device path and waiting
//     for it.  pWrk / pSync arguments are accepted and not used.
// Included from roc_shmem.hpp.
#ifndef ROCSHMEM_MI355X_ROC_SHMEM_HOST_HPP
#define ROCSHMEM_MI355X_ROC_SHMEM_HOST_HPP

#include <chrono>
#include <cstdio>
#include <cstdlib>
#include <cstring>

namespace rocshmem {

__host__ inline void roc_shmem_ctx_putmem(roc_shmem_ctx_t, void *dest, const void *source,
                                          size_t nelems, int pe) {
  hostx::putmem(dest, source, nelems, pe, true);
}
__host__ inline void roc_shmem_ctx_putmem_nbi(roc_shmem_ctx_t, void *dest, const void *source,
                                              size_t nelems, int pe) {
  hostx::putmem(dest, source, nelems, pe, false);
}
__host__ inline void roc_shmem_ctx_getmem(roc_shmem_ctx_t, void *dest, const void *source,
                                          size_t nelems, int pe) {
  hostx::getmem(dest, source, nelems, pe, true);
}
__host__ inline void roc_shmem_ctx_getmem_nbi(roc_shmem_ctx_t, void *dest, const void *source,
                                              size_t nelems, int pe) {
  hostx::getmem(dest, source, nelems, pe, false);
}
__host__ inline void roc_shmem_putmem(void *dest, const void *source, size_t nelems, int pe) {
  hostx::putmem(dest, source, nelems, pe, true);
}
__host__ inline void roc_shmem_putmem_nbi(void *dest, const void *source, size_t nelems, int pe) {
  hostx::putmem(dest, source, nelems, pe, false);
}
__host__ inline void roc_shmem_getmem(void *dest, const void *source, size_t nelems, int pe) {
  hostx::getmem(dest, source, nelems, pe, true);
}
__host__ inline void roc_shmem_getmem_nbi(void *dest, const void *source, size_t nelems, int pe) {
  hostx::getmem(dest, source, nelems, pe, false);
}
__host__ inline void roc_shmem_ctx_quiet(roc_shmem_ctx_t) { roc_shmem_quiet(); }
__host__ inline void roc_shmem_ctx_fence(roc_shmem_ctx_t) { roc_shmem_fence(); }

#define ROCSHMEM_HOST_STANDARD_TYPES(X) \
  X(float, float)                       \
  X(double, double)                     \
  X(char, char)                         \
  X(signed char, schar)                 \
  X(short, short)                       \
  X(int, int)                           \
  X(long, long)                         \
  X(long long, longlong)                \
  X(unsigned char, uchar)               \
  X(unsigned short, ushort)             \
  X(unsigned int, uint)                 \
  X(unsigned long, ulong)               \
  X(unsigned long long, ulonglong)

#define ROCSHMEM_HOST_RMA(T, TNAME)                                                            \
  __host__ inline void roc_shmem_ctx_##TNAME##_put(roc_shmem_ctx_t, T *dest, const T *source,  \
                                                   size_t nelems, int pe) {                    \
    hostx::putmem(dest, source, nelems * sizeof(T), pe, true);                                 \
  }                                                                                            \
  __host__ inline void roc_shmem_##TNAME##_put(T *dest, const T *source, size_t nelems,        \
                                               int pe) {                                       \
    hostx::putmem(dest, source, nelems * sizeof(T), pe, true);                                 \
  }                                                                                            \
  __host__ inline void roc_shmem_ctx_##TNAME##_put_nbi(roc_shmem_ctx_t, T *dest,               \
                                                       const T *source, size_t nelems,         \
                                                       int pe) {                               \
    hostx::putmem(dest, source, nelems * sizeof(T), pe, false);                                \
  }                                                                                            \
  __host__ inline void roc_shmem_##TNAME##_put_nbi(T *dest, const T *source, size_t nelems,    \
                                                   int pe) {                                   \
    hostx::putmem(dest, source, nelems * sizeof(T), pe, false);                                \
  }                                                                                            \
  __host__ inline void roc_shmem_ctx_##TNAME##_get(roc_shmem_ctx_t, T *dest, const T *source,  \
                                                   size_t nelems, int pe) {                    \
    hostx::getmem(dest, source, nelems * sizeof(T), pe, true);                                 \
  }                                                                                            \
  __host__ inline void roc_shmem_##TNAME##_get(T *dest, const T *source, size_t nelems,        \
                                               int pe) {                                       \
    hostx::getmem(dest, source, nelems * sizeof(T), pe, true);                                 \
  }                                                                                            \
  __host__ inline void roc_shmem_ctx_##TNAME##_get_nbi(roc_shmem_ctx_t, T *dest,               \
                                                       const T *source, size_t nelems,         \
                                                       int pe) {                               \
    hostx::getmem(dest, source, nelems * sizeof(T), pe, false);                                \
  }                                                                                            \
  __host__ inline void roc_shmem_##TNAME##_get_nbi(T *dest, const T *source, size_t nelems,    \
                                                   int pe) {                                   \
    hostx::getmem(dest, source, nelems * sizeof(T), pe, false);                                \
  }                                                                                            \
  __host__ inline void roc_shmem_ctx_##TNAME##_p(roc_shmem_ctx_t, T *dest, T value, int pe) {  \
    hostx::putmem(dest, &value, sizeof(T), pe, true);                                          \
  }                                                                                            \
  __host__ inline void roc_shmem_##TNAME##_p(T *dest, T value, int pe) {                       \
    hostx::putmem(dest, &value, sizeof(T), pe, true);                                          \
  }                                                                                            \
  __host__ inline T roc_shmem_ctx_##TNAME##_g(roc_shmem_ctx_t, const T *source, int pe) {      \
    T v;                                                                                       \
    hostx::getmem(&v, source, sizeof(T), pe, true);                                            \
    return v;                                                                                  \
  }                                                                                            \
  __host__ inline T roc_shmem_##TNAME##_g(const T *source, int pe) {                           \
    T v;                                                                                       \
    hostx::getmem(&v, source, sizeof(T), pe, true);                                            \
    return v;                                                                                  \
  }                                                                                            \
  __host__ inline void roc_shmem_ctx_##TNAME##_broadcast(                                      \
      roc_shmem_ctx_t, T *dest, const T *source, int nelem, int pe_root, int pe_start,         \
      int log_pe_stride, int pe_size, long *) {                                                \
    hostx::broadcast(sizeof(T), dest, source, nelem, pe_root, pe_start, log_pe_stride,         \
                     pe_size);                                                                 \
  }                                                                                            \
  __host__ inline void roc_shmem_ctx_##TNAME##_broadcast(roc_shmem_ctx_t, roc_shmem_team_t team, \
                                                         T *dest, const T *source, int nelem,  \
                                                         int pe_root) {                        \
    hostx::broadcast_team(sizeof(T), team, dest, source, nelem, pe_root);                      \
  }
ROCSHMEM_HOST_STANDARD_TYPES(ROCSHMEM_HOST_RMA)
#undef ROCSHMEM_HOST_RMA

// ---- reductions -------------------------------------------------------------

#define ROCSHMEM_HOST_REDUCTION(T, TNAME, DT, OPNAME, OP)                                      \
  __host__ inline void roc_shmem_ctx_##TNAME##_##OPNAME##_to_all(                              \
      roc_shmem_ctx_t, T *dest, const T *source, int nreduce, int PE_start, int logPE_stride,  \
      int PE_size, T *, long *) {                                                              \
    hostx::to_all(DT, OP, dest, source, nreduce, PE_start, logPE_stride, PE_size);             \
  }                                                                                            \
  __host__ inline void roc_shmem_ctx_##TNAME##_##OPNAME##_to_all(                              \
      roc_shmem_ctx_t, roc_shmem_team_t team, T *dest, const T *source, int nreduce) {         \
    hostx::to_all_team(DT, OP, team, dest, source, nreduce);                                   \
  }
#define ROCSHMEM_HOST_ARITH(T, TNAME, DT)           \
  ROCSHMEM_HOST_REDUCTION(T, TNAME, DT, sum, 0)     \
  ROCSHMEM_HOST_REDUCTION(T, TNAME, DT, max, 1)     \
  ROCSHMEM_HOST_REDUCTION(T, TNAME, DT, min, 2)     \
  ROCSHMEM_HOST_REDUCTION(T, TNAME, DT, prod, 3)
#define ROCSHMEM_HOST_BITS(T, TNAME, DT)            \
  ROCSHMEM_HOST_REDUCTION(T, TNAME, DT, and, 4)     \
  ROCSHMEM_HOST_REDUCTION(T, TNAME, DT, or, 5)      \
  ROCSHMEM_HOST_REDUCTION(T, TNAME, DT, xor, 6)
ROCSHMEM_HOST_ARITH(short, short, 0)
ROCSHMEM_HOST_BITS(short, short, 0)
ROCSHMEM_HOST_ARITH(int, int, 1)
ROCSHMEM_HOST_BITS(int, int, 1)
ROCSHMEM_HOST_ARITH(long, long, 2)
ROCSHMEM_HOST_BITS(long, long, 2)
ROCSHMEM_HOST_ARITH(long long, longlong, 3)
ROCSHMEM_HOST_BITS(long long, longlong, 3)
ROCSHMEM_HOST_ARITH(float, float, 4)
ROCSHMEM_HOST_ARITH(double, double, 5)
#undef ROCSHMEM_HOST_BITS
#undef ROCSHMEM_HOST_ARITH
#undef ROCSHMEM_HOST_REDUCTION

// ---- atomic memory operations ---------------------------------------------------

namespace hostx {
template <typename T>
inline uint64_t to_bits(T v) {
  uint64_t b = 0;
  std::memcpy(&b, &v, sizeof(T));
  return b;
}
template <typename T>
inline T from_bits(uint64_t b) {
  T v;
  std::memcpy(&v, &b, sizeof(T));
  return v;
}
}  // namespace hostx

// ---- wait_until / test ------------------------------------------------------------------
// Reference: HostInterface::wait_until / test / test_and_compare, library/src/host/
// host_templates.hpp:426-487 (an atomic fetch of the calling PE's own copy of the word, compared
// on the host; wait_until repeats it until the comparison holds); declared for the 13 standard
// types at library/include/roc_shmem.hpp:1152-1163,1973-2019.  The calling PE is the host's
// current PE.  The reference spins for ever; so does this wait with ROC_SHMEM_WAIT_LIMIT_S=0.
// With a positive limit (the default is 2 s) it gives up after that many seconds, prints a
// message and exits like the library's other fatal errors.
namespace hostx {
template <typename T>
inline T own_value(const T *ptr) {
  const uint64_t bits = fetch_own(ptr, static_cast<int>(sizeof(T)));
  T v;
  std::memcpy(&v, &bits, sizeof(T));  // little-endian host: the low bytes hold the word
  return v;
}
template <typename T>
inline bool compare(roc_shmem_cmps cmp, T have, T want) {
  switch (cmp) {
    case ROC_SHMEM_CMP_EQ: return have == want;
    case ROC_SHMEM_CMP_NE: return have != want;
    case ROC_SHMEM_CMP_GT: return have > want;
    case ROC_SHMEM_CMP_GE: return have >= want;
    case ROC_SHMEM_CMP_LT: return have < want;
    default: return have <= want;
  }
}
template <typename T>
inline void wait_until(const T *ptr, roc_shmem_cmps cmp, T val) {
  const auto start = std::chrono::steady_clock::now();
  const double limit = wait_limit_seconds();
  while (!compare(cmp, own_value(ptr), val)) {
    if (limit > 0 &&
        std::chrono::duration<double>(std::chrono::steady_clock::now() - start).count() > limit) {
      fprintf(stderr, "rocshmem: roc_shmem_wait_until: condition not met after %.1f s\n", limit);
      exit(EXIT_FAILURE);
    }
  }
}
}  // namespace hostx

#define ROCSHMEM_HOST_WAIT(T, TNAME)                                                           \
  __host__ inline void roc_shmem_##TNAME##_wait_until(T *ptr, roc_shmem_cmps cmp, T val) {     \
    hostx::wait_until<T>(ptr, cmp, val);                                                       \
  }                                                                                            \
  __host__ inline int roc_shmem_##TNAME##_test(T *ptr, roc_shmem_cmps cmp, T val) {            \
    return hostx::compare<T>(cmp, hostx::own_value<T>(ptr), val) ? 1 : 0;                      \
  }
ROCSHMEM_HOST_STANDARD_TYPES(ROCSHMEM_HOST_WAIT)
#undef ROCSHMEM_HOST_WAIT

#define ROCSHMEM_HOST_AMO_TYPES(X) \
  X(int, int)                      \
  X(long, long)                    \
  X(long long, longlong)           \
  X(unsigned int, uint)            \
  X(unsigned long, ulong)          \
  X(unsigned long long, ulonglong) \
  X(int32_t, int32)                \
  X(int64_t, int64)                \
  X(uint32_t, uint32)              \
  X(uint64_t, uint64)              \
  X(size_t, size)                  \
  X(ptrdiff_t, ptrdiff)

#define ROCSHMEM_HOST_AMO(T, TNAME)                                                            \
  __host__ inline T roc_shmem_ctx_##TNAME##_atomic_fetch_add(roc_shmem_ctx_t, T *dest, T value, \
                                                             int pe) {                         \
    return hostx::from_bits<T>(hostx::amo(0, dest, hostx::to_bits(value), 0, pe, sizeof(T)));  \
  }                                                                                            \
  __host__ inline T roc_shmem_##TNAME##_atomic_fetch_add(T *dest, T value, int pe) {           \
    return hostx::from_bits<T>(hostx::amo(0, dest, hostx::to_bits(value), 0, pe, sizeof(T)));  \
  }                                                                                            \
  __host__ inline void roc_shmem_ctx_##TNAME##_atomic_add(roc_shmem_ctx_t, T *dest, T value,   \
                                                          int pe) {                            \
    (void)hostx::amo(0, dest, hostx::to_bits(value), 0, pe, sizeof(T));                        \
  }                                                                                            \
  __host__ inline void roc_shmem_##TNAME##_atomic_add(T *dest, T value, int pe) {              \
    (void)hostx::amo(0, dest, hostx::to_bits(value), 0, pe, sizeof(T));                        \
  }                                                                                            \
  __host__ inline T roc_shmem_ctx_##TNAME##_atomic_fetch_inc(roc_shmem_ctx_t, T *dest,         \
                                                             int pe) {                         \
    return hostx::from_bits<T>(hostx::amo(0, dest, 1, 0, pe, sizeof(T)));                      \
  }                                                                                            \
  __host__ inline T roc_shmem_##TNAME##_atomic_fetch_inc(T *dest, int pe) {                    \
    return hostx::from_bits<T>(hostx::amo(0, dest, 1, 0, pe, sizeof(T)));                      \
  }                                                                                            \
  __host__ inline void roc_shmem_ctx_##TNAME##_atomic_inc(roc_shmem_ctx_t, T *dest, int pe) {  \
    (void)hostx::amo(0, dest, 1, 0, pe, sizeof(T));                                            \
  }                                                                                            \
  __host__ inline void roc_shmem_##TNAME##_atomic_inc(T *dest, int pe) {                       \
    (void)hostx::amo(0, dest, 1, 0, pe, sizeof(T));                                            \
  }                                                                                            \
  __host__ inline T roc_shmem_ctx_##TNAME##_atomic_fetch(roc_shmem_ctx_t, T *dest, int pe) {   \
    return hostx::from_bits<T>(hostx::amo(0, dest, 0, 0, pe, sizeof(T)));                      \
  }                                                                                            \
  __host__ inline T roc_shmem_##TNAME##_atomic_fetch(T *dest, int pe) {                        \
    return hostx::from_bits<T>(hostx::amo(0, dest, 0, 0, pe, sizeof(T)));                      \
  }                                                                                            \
  __host__ inline T roc_shmem_ctx_##TNAME##_atomic_compare_swap(roc_shmem_ctx_t, T *dest,      \
                                                                T cond, T value, int pe) {     \
    return hostx::from_bits<T>(                                                                \
        hostx::amo(1, dest, hostx::to_bits(value), hostx::to_bits(cond), pe, sizeof(T)));      \
  }                                                                                            \
  __host__ inline T roc_shmem_##TNAME##_atomic_compare_swap(T *dest, T cond, T value,          \
                                                            int pe) {                          \
    return hostx::from_bits<T>(                                                                \
        hostx::amo(1, dest, hostx::to_bits(value), hostx::to_bits(cond), pe, sizeof(T)));      \
  }                                                                                            \
  __host__ inline T roc_shmem_ctx_##TNAME##_atomic_swap(roc_shmem_ctx_t, T *dest, T value,     \
                                                        int pe) {                              \
    return hostx::from_bits<T>(hostx::amo(2, dest, hostx::to_bits(value), 0, pe, sizeof(T)));  \
  }                                                                                            \
  __host__ inline T roc_shmem_##TNAME##_atomic_swap(T *dest, T value, int pe) {                \
    return hostx::from_bits<T>(hostx::amo(2, dest, hostx::to_bits(value), 0, pe, sizeof(T)));  \
  }                                                                                            \
  __host__ inline void roc_shmem_ctx_##TNAME##_atomic_set(roc_shmem_ctx_t, T *dest, T value,   \
                                                          int pe) {                            \
    (void)hostx::amo(2, dest, hostx::to_bits(value), 0, pe, sizeof(T));                        \
  }                                                                                            \
  __host__ inline void roc_shmem_##TNAME##_atomic_set(T *dest, T value, int pe) {              \
    (void)hostx::amo(2, dest, hostx::to_bits(value), 0, pe, sizeof(T));                        \
  }
ROCSHMEM_HOST_AMO_TYPES(ROCSHMEM_HOST_AMO)
#undef ROCSHMEM_HOST_AMO

// fetch / set / swap also exist for float and double (reference: roc_shmem.hpp:1647-1648,
// 1713-1714,1747-1748): the word is moved as its bit pattern.
#define ROCSHMEM_HOST_AMO_FLOATING(T, TNAME)                                                   \
  __host__ inline T roc_shmem_ctx_##TNAME##_atomic_fetch(roc_shmem_ctx_t, T *dest, int pe) {   \
    return hostx::from_bits<T>(hostx::amo(0, dest, 0, 0, pe, sizeof(T)));                      \
  }                                                                                            \
  __host__ inline T roc_shmem_##TNAME##_atomic_fetch(T *dest, int pe) {                        \
    return hostx::from_bits<T>(hostx::amo(0, dest, 0, 0, pe, sizeof(T)));                      \
  }                                                                                            \
  __host__ inline T roc_shmem_ctx_##TNAME##_atomic_swap(roc_shmem_ctx_t, T *dest, T value,     \
                                                        int pe) {                              \
    return hostx::from_bits<T>(hostx::amo(2, dest, hostx::to_bits(value), 0, pe, sizeof(T)));  \
  }                                                                                            \
  __host__ inline T roc_shmem_##TNAME##_atomic_swap(T *dest, T value, int pe) {                \
    return hostx::from_bits<T>(hostx::amo(2, dest, hostx::to_bits(value), 0, pe, sizeof(T)));  \
  }                                                                                            \
  __host__ inline void roc_shmem_ctx_##TNAME##_atomic_set(roc_shmem_ctx_t, T *dest, T value,   \
                                                          int pe) {                            \
    (void)hostx::amo(2, dest, hostx::to_bits(value), 0, pe, sizeof(T));                        \
  }                                                                                            \
  __host__ inline void roc_shmem_##TNAME##_atomic_set(T *dest, T value, int pe) {              \
    (void)hostx::amo(2, dest, hostx::to_bits(value), 0, pe, sizeof(T));                        \
  }
ROCSHMEM_HOST_AMO_FLOATING(float, float)
ROCSHMEM_HOST_AMO_FLOATING(double, double)
#undef ROCSHMEM_HOST_AMO_FLOATING

// Bitwise operations (reference: roc_shmem.hpp:1068-1147,1781-1953): seven types.
#define ROCSHMEM_HOST_AMO_BITWISE_TYPES(X) \
  X(unsigned int, uint)                    \
  X(unsigned long, ulong)                  \
  X(unsigned long long, ulonglong)         \
  X(int32_t, int32)                        \
  X(int64_t, int64)                        \
  X(uint32_t, uint32)                      \
  X(uint64_t, uint64)

#define ROCSHMEM_HOST_AMO_BITWISE_ONE(T, TNAME, OP, KIND)                                      \
  __host__ inline T roc_shmem_ctx_##TNAME##_atomic_fetch_##OP(roc_shmem_ctx_t, T *dest,        \
                                                              T value, int pe) {               \
    return hostx::from_bits<T>(hostx::amo(KIND, dest, hostx::to_bits(value), 0, pe, sizeof(T))); \
  }                                                                                            \
  __host__ inline T roc_shmem_##TNAME##_atomic_fetch_##OP(T *dest, T value, int pe) {          \
    return hostx::from_bits<T>(hostx::amo(KIND, dest, hostx::to_bits(value), 0, pe, sizeof(T))); \
  }                                                                                            \
  __host__ inline void roc_shmem_ctx_##TNAME##_atomic_##OP(roc_shmem_ctx_t, T *dest, T value,  \
                                                           int pe) {                           \
    (void)hostx::amo(KIND, dest, hostx::to_bits(value), 0, pe, sizeof(T));                     \
  }                                                                                            \
  __host__ inline void roc_shmem_##TNAME##_atomic_##OP(T *dest, T value, int pe) {             \
    (void)hostx::amo(KIND, dest, hostx::to_bits(value), 0, pe, sizeof(T));                     \
  }
#define ROCSHMEM_HOST_AMO_BITWISE(T, TNAME)          \
  ROCSHMEM_HOST_AMO_BITWISE_ONE(T, TNAME, and, 3)    \
  ROCSHMEM_HOST_AMO_BITWISE_ONE(T, TNAME, or, 4)     \
  ROCSHMEM_HOST_AMO_BITWISE_ONE(T, TNAME, xor, 5)
ROCSHMEM_HOST_AMO_BITWISE_TYPES(ROCSHMEM_HOST_AMO_BITWISE)
#undef ROCSHMEM_HOST_AMO_BITWISE
#undef ROCSHMEM_HOST_AMO_BITWISE_ONE

}  // namespace rocshmem

#endif
