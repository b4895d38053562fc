// Element-wise reduction of the source slices of an active set.
//
// The reference folds `dst[i] = dst[i] (op) src[i]` with a thread-strided
// scalar loop per peer (compute_reduce / OpWrap<Op>::Calc,
// library/src/gpu_ib/context_ib_tmpl_device.hpp:50-113), after staging every
// peer's data through pWrk.  All slices are directly addressable here, so a
// workgroup streams its share of the element range once: 16-byte
// non-temporal loads from each member's source, a fold in ascending member
// order, 16-byte stores into each member's destination.
//
// Arithmetic contract
//   integers  : two's-complement wrap for sum/prod, exact and/or/xor/max/min
//               (any fold order gives the same bits);
//   float     : sum and prod are folded in double and rounded once;
//   double    : folded in double, ascending member order;
//   bfloat16  : sum is folded in float and rounded once (nearest-even);
//   max / min : exact selection; a NaN operand is ignored, as fmax/fmin do.
#ifndef ROCSHMEM_MI355X_DEVICE_REDUCE_HPP
#define ROCSHMEM_MI355X_DEVICE_REDUCE_HPP

#include <hip/hip_bf16.h>

#include <type_traits>

#include "copy.hpp"
#include "sync.hpp"

namespace rocshmem {
namespace detail {

// ---- accumulator traits ----------------------------------------------------

template <typename T, ROC_SHMEM_OP Op>
struct AccOf {
  using type = T;
};
template <>
struct AccOf<float, ROC_SHMEM_SUM> {
  using type = double;
};
template <>
struct AccOf<float, ROC_SHMEM_PROD> {
  using type = double;
};
template <ROC_SHMEM_OP Op>
struct AccOf<__hip_bfloat16, Op> {
  using type = float;
};

__device__ __forceinline__ float bf16_bits_to_float(uint16_t b) {
  return __uint_as_float(static_cast<uint32_t>(b) << 16);
}

// Round-to-nearest-even float -> bfloat16 bits; NaN stays a quiet NaN.
__device__ __forceinline__ uint16_t float_to_bf16_bits(float f) {
  uint32_t u = __float_as_uint(f);
  if ((u & 0x7fffffffu) > 0x7f800000u) return static_cast<uint16_t>((u >> 16) | 0x0040u);
  u += 0x7fffu + ((u >> 16) & 1u);
  return static_cast<uint16_t>(u >> 16);
}

// Storage element <-> accumulator conversions.  Elem is the in-memory type
// (bfloat16 is handled as its 16-bit pattern).
template <typename T>
struct Storage {
  using elem = T;
};
template <>
struct Storage<__hip_bfloat16> {
  using elem = uint16_t;
};

template <typename T, typename Acc>
__device__ __forceinline__ Acc to_acc(typename Storage<T>::elem e) {
  if constexpr (std::is_same<T, __hip_bfloat16>::value) {
    return bf16_bits_to_float(e);
  } else {
    return static_cast<Acc>(e);
  }
}

template <typename T, typename Acc>
__device__ __forceinline__ typename Storage<T>::elem from_acc(Acc a) {
  if constexpr (std::is_same<T, __hip_bfloat16>::value) {
    return float_to_bf16_bits(a);
  } else {
    return static_cast<T>(a);
  }
}

// ---- the fold --------------------------------------------------------------

template <ROC_SHMEM_OP Op, typename A>
__device__ __forceinline__ A fold(A a, A b) {
  if constexpr (std::is_integral<A>::value) {
    using U = typename std::make_unsigned<A>::type;
    if constexpr (Op == ROC_SHMEM_SUM) return static_cast<A>(static_cast<U>(a) + static_cast<U>(b));
    if constexpr (Op == ROC_SHMEM_PROD) {
      // Multiply in a type at least as wide as unsigned int so that a 16-bit
      // product cannot overflow a promoted signed int.
      using W = typename std::conditional<(sizeof(U) < 4), uint32_t, U>::type;
      return static_cast<A>(static_cast<U>(static_cast<W>(static_cast<U>(a)) *
                                           static_cast<W>(static_cast<U>(b))));
    }
    if constexpr (Op == ROC_SHMEM_AND) return static_cast<A>(a & b);
    if constexpr (Op == ROC_SHMEM_OR) return static_cast<A>(a | b);
    if constexpr (Op == ROC_SHMEM_XOR) return static_cast<A>(a ^ b);
    if constexpr (Op == ROC_SHMEM_MAX) return a >= b ? a : b;
    if constexpr (Op == ROC_SHMEM_MIN) return a <= b ? a : b;
  } else {
    if constexpr (Op == ROC_SHMEM_SUM) return a + b;
    if constexpr (Op == ROC_SHMEM_PROD) return a * b;
    if constexpr (Op == ROC_SHMEM_MAX) return (a >= b || b != b) ? a : b;
    if constexpr (Op == ROC_SHMEM_MIN) return (a <= b || b != b) ? a : b;
  }
  return a;
}

// ---- vector path -----------------------------------------------------------

template <typename T>
struct VecOf {
  using elem = typename Storage<T>::elem;
  static constexpr int kElems = 16 / sizeof(elem);
  union Pack {
    u32x4 raw;
    elem e[kElems];
  };
};

constexpr int kReduceUnroll = 2;   // vectors per lane per pass
constexpr int kReducePeChunk = 4;  // members whose loads are issued together

struct ActiveSet {
  int pe_start;
  int log_stride;
  int size;
  __device__ __forceinline__ int pe_at(int k) const { return pe_start + (k << log_stride); }
};

// Reduce vectors [v_begin, v_end) of the symmetric arrays `src`/`dst` (given
// as this PE's addresses, both 16-byte aligned) over all members and write
// the result into every member's destination.
template <typename T, ROC_SHMEM_OP Op>
__device__ __forceinline__ void reduce_vectors(T *dst, const T *src, size_t v_begin,
                                               size_t v_end, const ActiveSet &as, int my_pe,
                                               uint32_t tid, uint32_t nthr) {
  using Acc = typename AccOf<T, Op>::type;
  using V = VecOf<T>;
  constexpr int E = V::kElems;
  constexpr int U = kReduceUnroll;
  constexpr int C = kReducePeChunk;

  const int64_t stride = static_cast<int64_t>(g_state.slice_stride);
  const char *src0 = reinterpret_cast<const char *>(src) +
                     (static_cast<int64_t>(as.pe_start) - my_pe) * stride;
  char *dst0 =
      reinterpret_cast<char *>(dst) + (static_cast<int64_t>(as.pe_start) - my_pe) * stride;
  const int64_t member_step = stride << as.log_stride;

  auto src_vec = [&](int k) {
    return reinterpret_cast<const u32x4 *>(src0 + k * member_step);
  };
  auto dst_vec = [&](int k) { return reinterpret_cast<u32x4 *>(dst0 + k * member_step); };

  size_t i = v_begin + tid;
  const size_t step = nthr;

  // Full passes: U vectors per lane.
  for (; i + (U - 1) * step < v_end; i += U * step) {
    Acc acc[U][E];
    {
      const u32x4 *s = src_vec(0);
#pragma unroll
      for (int u = 0; u < U; ++u) {
        typename V::Pack p;
        p.raw = __builtin_nontemporal_load(&s[i + u * step]);
#pragma unroll
        for (int e = 0; e < E; ++e) acc[u][e] = to_acc<T, Acc>(p.e[e]);
      }
    }
    int k = 1;
    for (; k + C <= as.size; k += C) {
      typename V::Pack p[C][U];
#pragma unroll
      for (int c = 0; c < C; ++c) {
        const u32x4 *s = src_vec(k + c);
#pragma unroll
        for (int u = 0; u < U; ++u) p[c][u].raw = __builtin_nontemporal_load(&s[i + u * step]);
      }
#pragma unroll
      for (int c = 0; c < C; ++c)
#pragma unroll
        for (int u = 0; u < U; ++u)
#pragma unroll
          for (int e = 0; e < E; ++e)
            acc[u][e] = fold<Op, Acc>(acc[u][e], to_acc<T, Acc>(p[c][u].e[e]));
    }
    for (; k < as.size; ++k) {
      const u32x4 *s = src_vec(k);
      typename V::Pack p[U];
#pragma unroll
      for (int u = 0; u < U; ++u) p[u].raw = __builtin_nontemporal_load(&s[i + u * step]);
#pragma unroll
      for (int u = 0; u < U; ++u)
#pragma unroll
        for (int e = 0; e < E; ++e) acc[u][e] = fold<Op, Acc>(acc[u][e], to_acc<T, Acc>(p[u].e[e]));
    }
    typename V::Pack out[U];
#pragma unroll
    for (int u = 0; u < U; ++u)
#pragma unroll
      for (int e = 0; e < E; ++e) out[u].e[e] = from_acc<T, Acc>(acc[u][e]);
    for (int m = 0; m < as.size; ++m) {
      u32x4 *d = dst_vec(m);
#pragma unroll
      for (int u = 0; u < U; ++u) __builtin_nontemporal_store(out[u].raw, &d[i + u * step]);
    }
  }
  // Remainder: one vector per lane.
  for (; i < v_end; i += step) {
    Acc acc[E];
    {
      typename V::Pack p;
      p.raw = __builtin_nontemporal_load(&src_vec(0)[i]);
#pragma unroll
      for (int e = 0; e < E; ++e) acc[e] = to_acc<T, Acc>(p.e[e]);
    }
    for (int k = 1; k < as.size; ++k) {
      typename V::Pack p;
      p.raw = __builtin_nontemporal_load(&src_vec(k)[i]);
#pragma unroll
      for (int e = 0; e < E; ++e) acc[e] = fold<Op, Acc>(acc[e], to_acc<T, Acc>(p.e[e]));
    }
    typename V::Pack out;
#pragma unroll
    for (int e = 0; e < E; ++e) out.e[e] = from_acc<T, Acc>(acc[e]);
    for (int m = 0; m < as.size; ++m) __builtin_nontemporal_store(out.raw, &dst_vec(m)[i]);
  }
}

// Scalar path for element range [e_begin, e_end): unaligned arrays and tails.
template <typename T, ROC_SHMEM_OP Op>
__device__ __forceinline__ void reduce_elements(T *dst, const T *src, size_t e_begin,
                                                size_t e_end, const ActiveSet &as, int my_pe,
                                                uint32_t tid, uint32_t nthr) {
  using Acc = typename AccOf<T, Op>::type;
  using Elem = typename Storage<T>::elem;
  const int64_t stride = static_cast<int64_t>(g_state.slice_stride);
  const char *src0 = reinterpret_cast<const char *>(src) +
                     (static_cast<int64_t>(as.pe_start) - my_pe) * stride;
  char *dst0 =
      reinterpret_cast<char *>(dst) + (static_cast<int64_t>(as.pe_start) - my_pe) * stride;
  const int64_t member_step = stride << as.log_stride;
  for (size_t i = e_begin + tid; i < e_end; i += nthr) {
    Acc acc = to_acc<T, Acc>(reinterpret_cast<const Elem *>(src0)[i]);
    for (int k = 1; k < as.size; ++k) {
      acc = fold<Op, Acc>(
          acc, to_acc<T, Acc>(reinterpret_cast<const Elem *>(src0 + k * member_step)[i]));
    }
    Elem out = from_acc<T, Acc>(acc);
    for (int m = 0; m < as.size; ++m) reinterpret_cast<Elem *>(dst0 + m * member_step)[i] = out;
  }
}

// Workgroup-collective all-reduce over an active set.  Called by one
// workgroup per member with identical arguments (reference contract:
// GPUIBContext::to_all, context_ib_tmpl_device.hpp:262-307).  Member k of the
// set reduces the k-th share of the element range and writes it to all
// members; the two flag barriers order "every source is ready" before the
// loads and "every destination is complete" before the return.  pWrk is not
// needed.  dest == source (in place) is allowed: a share is read and then
// overwritten by the same lanes.
template <typename T, ROC_SHMEM_OP Op>
__device__ __forceinline__ void wg_all_reduce(int my_pe, T *dest, const T *source, int nreduce,
                                              int pe_start, int log_stride, int pe_size,
                                              long *psync) {
  if (nreduce <= 0) return;  // reference: Context::to_all early-out, context_tmpl_device.hpp:68-70
  if (pe_size > kMaxPes || pe_size <= 0) {
    status_raise(kStatusBadArgument);
    return;
  }
  const ActiveSet as{pe_start, log_stride, pe_size};
  const int my_idx = (my_pe - pe_start) >> log_stride;
  const uint32_t tid = flat_thread_id();
  const uint32_t nthr = flat_block_size();
  const size_t n = static_cast<size_t>(nreduce);

  wg_flag_barrier(psync, 0, my_pe, my_idx, pe_start, log_stride, pe_size);

  constexpr size_t E = VecOf<T>::kElems;
  const bool aligned =
      ((reinterpret_cast<uintptr_t>(dest) | reinterpret_cast<uintptr_t>(source)) & 15u) == 0;
  if (aligned) {
    const size_t nvec = n / E;
    const size_t share = (nvec + pe_size - 1) / pe_size;
    size_t v0 = share * my_idx;
    size_t v1 = v0 + share;
    if (v0 > nvec) v0 = nvec;
    if (v1 > nvec) v1 = nvec;
    reduce_vectors<T, Op>(dest, source, v0, v1, as, my_pe, tid, nthr);
    if (my_idx == pe_size - 1 && nvec * E < n) {
      reduce_elements<T, Op>(dest, source, nvec * E, n, as, my_pe, tid, nthr);
    }
  } else {
    const size_t share = (n + pe_size - 1) / pe_size;
    size_t e0 = share * my_idx;
    size_t e1 = e0 + share;
    if (e0 > n) e0 = n;
    if (e1 > n) e1 = n;
    reduce_elements<T, Op>(dest, source, e0, e1, as, my_pe, tid, nthr);
  }

  wg_flag_barrier(psync, 1, my_pe, my_idx, pe_start, log_stride, pe_size);
}

}  // namespace detail
}  // namespace rocshmem

#endif
