// Thread-level RMA and atomic memory operations.
//
// Every lane may issue (ROC_SHMEM_THREAD_MULTIPLE).  A put/get moves its
// bytes with direct loads and stores into the destination slice and records
// the message as a WQE in the context's send queue, after merging
// lane-contiguous messages of the wave (reference: GPUIBContext::putmem /
// putmem_nbi / getmem / getmem_nbi, library/src/gpu_ib/context_ib_device.cpp:
// 84-119,148-184).  An AMO is one native device-scope atomic of the operand's
// own width plus its WQE record (reference: amo_* -> QueuePair::atomic_fetch,
// context_ib_tmpl_device.hpp:365-453, queue_pair.cpp:327-374, where every AMO
// is a 64-bit NIC round trip regardless of the operand type).
#ifndef ROCSHMEM_MI355X_DEVICE_SMALL_OPS_HPP
#define ROCSHMEM_MI355X_DEVICE_SMALL_OPS_HPP

#include "wqe.hpp"

namespace rocshmem {
namespace detail {

// Up to 8 payload bytes starting at `src`, packed little-endian.
__device__ __forceinline__ uint64_t gather_inline(const void *src, uint32_t size) {
  uintptr_t a = reinterpret_cast<uintptr_t>(src);
  if (size == 8 && (a & 7u) == 0) return *static_cast<const uint64_t *>(src);
  if (size == 4 && (a & 3u) == 0) return *static_cast<const uint32_t *>(src);
  uint64_t v = 0;
  const uint8_t *b = static_cast<const uint8_t *>(src);
  for (uint32_t i = 0; i < size && i < 8; ++i) v |= static_cast<uint64_t>(b[i]) << (8 * i);
  return v;
}

__device__ __forceinline__ void thread_put(DeviceCtx *ctx, void *dest, const void *source,
                                           size_t nbytes, int pe) {
  if (nbytes == 0) return;  // reference: Context::putmem early-out, context_device.cpp:80-82
  char *remote = translate(static_cast<char *>(dest), ctx->my_pe, pe);
  // The operation itself goes first: its latency is what a waiting PE sees,
  // and it overlaps with the chain of queue atomics behind the post.
  lane_copy(remote, source, nbytes);
  CoalesceResult c = wave_coalesce(pe, reinterpret_cast<uint64_t>(source),
                                   reinterpret_cast<uint64_t>(dest), nbytes);
  WqeRequest rq;
  rq.opcode = kOpcodeRdmaWrite;
  rq.size = static_cast<uint32_t>(c.size);
  rq.raddr = reinterpret_cast<uint64_t>(remote);
  rq.laddr = reinterpret_cast<uint64_t>(source);
  rq.atomic_data = 0;
  rq.atomic_cmp = 0;
  rq.inline_data = 0;
  rq.pe = pe;
  if (c.must_send && c.size <= kInlineThreshold) {
    rq.inline_data = gather_inline(source, static_cast<uint32_t>(c.size));
  }
  wave_post(ctx, c.must_send, rq);
}

__device__ __forceinline__ void thread_get(DeviceCtx *ctx, void *dest, const void *source,
                                           size_t nbytes, int pe) {
  if (nbytes == 0) return;
  const char *remote = translate(static_cast<const char *>(source), ctx->my_pe, pe);
  lane_copy(dest, remote, nbytes);
  CoalesceResult c = wave_coalesce(pe, reinterpret_cast<uint64_t>(source),
                                   reinterpret_cast<uint64_t>(dest), nbytes);
  WqeRequest rq;
  rq.opcode = kOpcodeRdmaRead;
  rq.size = static_cast<uint32_t>(c.size);
  rq.raddr = reinterpret_cast<uint64_t>(remote);
  rq.laddr = reinterpret_cast<uint64_t>(dest);
  rq.atomic_data = 0;
  rq.atomic_cmp = 0;
  rq.inline_data = 0;
  rq.pe = pe;
  wave_post(ctx, c.must_send, rq);
}

// Single-element put of a register value (reference: GPUIBContext::p,
// context_ib_tmpl_device.hpp:115-118).  The reference passes the address of a
// stack copy, which never satisfies the coalescer's contiguity test, so every
// lane posts its own inline entry; the same holds here without touching
// scratch memory.
// One element of a standard type through device-coherent accesses (see
// coherent_store in copy.hpp).
template <typename T>
__device__ __forceinline__ void element_store(T *p, T value) {
  static_assert(sizeof(T) == 1 || sizeof(T) == 2 || sizeof(T) == 4 || sizeof(T) == 8, "element size");
  using W = typename std::conditional<
      sizeof(T) == 8, uint64_t,
      typename std::conditional<sizeof(T) == 4, uint32_t,
                                typename std::conditional<sizeof(T) == 2, uint16_t, uint8_t>::type>::type>::type;
  W bits;
  __builtin_memcpy(&bits, &value, sizeof(T));
  coherent_store<W>(p, bits);
}
template <typename T>
__device__ __forceinline__ T element_load(const T *p) {
  static_assert(sizeof(T) == 1 || sizeof(T) == 2 || sizeof(T) == 4 || sizeof(T) == 8, "element size");
  using W = typename std::conditional<
      sizeof(T) == 8, uint64_t,
      typename std::conditional<sizeof(T) == 4, uint32_t,
                                typename std::conditional<sizeof(T) == 2, uint16_t, uint8_t>::type>::type>::type;
  W bits = coherent_load<W>(p);
  T value;
  __builtin_memcpy(&value, &bits, sizeof(T));
  return value;
}

template <typename T>
__device__ __forceinline__ void thread_p(DeviceCtx *ctx, T *dest, T value, int pe) {
  T *remote = translate(own(dest, ctx), ctx->my_pe, pe);
  element_store(remote, value);
  uint64_t bits = 0;
  __builtin_memcpy(&bits, &value, sizeof(T));
  WqeRequest rq;
  rq.opcode = kOpcodeRdmaWrite;
  rq.size = sizeof(T);
  rq.raddr = reinterpret_cast<uint64_t>(remote);
  rq.laddr = 0;
  rq.atomic_data = 0;
  rq.atomic_cmp = 0;
  rq.inline_data = bits;
  rq.pe = pe;
  wave_post(ctx, true, rq);
}

template <typename T>
__device__ __forceinline__ T thread_g(DeviceCtx *ctx, const T *source, int pe) {
  const T *remote = translate(source, ctx->my_pe, pe);
  const T value = element_load(remote);
  WqeRequest rq;
  rq.opcode = kOpcodeRdmaRead;
  rq.size = sizeof(T);
  rq.raddr = reinterpret_cast<uint64_t>(remote);
  rq.laddr = 0;
  rq.atomic_data = 0;
  rq.atomic_cmp = 0;
  rq.inline_data = 0;
  rq.pe = pe;
  wave_post(ctx, true, rq);
  return value;
}

// ---- atomics ---------------------------------------------------------------

template <typename T>
struct AtomicWord {
  static_assert(sizeof(T) == 4 || sizeof(T) == 8, "AMO operands are 32 or 64 bits wide");
  using type = typename std::conditional<sizeof(T) == 8, uint64_t, uint32_t>::type;
};

template <typename T>
__device__ __forceinline__ uint64_t amo_bits(T v) {
  typename AtomicWord<T>::type w;
  __builtin_memcpy(&w, &v, sizeof(T));
  return static_cast<uint64_t>(w);
}

template <typename T>
__device__ __forceinline__ void amo_record(DeviceCtx *ctx, uint8_t opcode, T *remote, T data,
                                           T cmp, int pe) {
  WqeRequest rq;
  rq.opcode = opcode;
  rq.size = 8;
  rq.raddr = reinterpret_cast<uint64_t>(remote);
  rq.laddr = 0;
  // The reference widens the operand to int64_t before it reaches the WQE
  // (QueuePair::atomic_fetch takes int64_t value, queue_pair.cpp:327-329).
  if constexpr (std::is_integral<T>::value && std::is_signed<T>::value) {
    rq.atomic_data = static_cast<uint64_t>(static_cast<int64_t>(data));
    rq.atomic_cmp = static_cast<uint64_t>(static_cast<int64_t>(cmp));
  } else if constexpr (std::is_integral<T>::value) {
    rq.atomic_data = static_cast<uint64_t>(data);
    rq.atomic_cmp = static_cast<uint64_t>(cmp);
  } else {
    rq.atomic_data = amo_bits(data);
    rq.atomic_cmp = amo_bits(cmp);
  }
  rq.inline_data = 0;
  rq.pe = pe;
  wave_post(ctx, true, rq);
}

__device__ __forceinline__ uint32_t first_lane_word(uint32_t v) { return first_lane_u32(v); }
__device__ __forceinline__ uint64_t first_lane_word(uint64_t v) { return first_lane_u64(v); }
__device__ __forceinline__ uint32_t lane_word(uint32_t v, int lane) {
  return __builtin_amdgcn_readlane(v, lane);
}
__device__ __forceinline__ uint64_t lane_word(uint64_t v, int lane) {
  const uint32_t lo = __builtin_amdgcn_readlane(static_cast<uint32_t>(v), lane);
  const uint32_t hi = __builtin_amdgcn_readlane(static_cast<uint32_t>(v >> 32), lane);
  return (static_cast<uint64_t>(hi) << 32) | lo;
}

// fetch_add on `remote` by every active lane.  Atomics on one word are
// carried out one after the other where the word lives (12 ns each at agent
// scope: 83 M/s however many lanes ask), so lanes of the wave that name the
// same word add the sum of their operands with one atomic, and each gets what
// it would have fetched had they gone in lane order: the word's previous value
// plus the operands of the group's lanes below it.  Any serialisation is a
// valid outcome of concurrent AMOs; this is one.
//
// Groups are looked for leader by leader (the lowest lane not yet served and
// every lane with its address).  The search stops at the first leader without
// a partner, so a wave whose lanes all name different words (the usual case,
// uniformly random targets) pays one round of a dozen instructions; at most
// kCombineRounds groups are formed.  Lanes left over issue their own atomic.
constexpr int kCombineRounds = 16;
template <typename T>
__device__ __forceinline__ T wave_fetch_add(T *remote, T value) {
  using W = typename AtomicWord<T>::type;
  const uint64_t active = __ballot(1);
  const uint64_t addr = reinterpret_cast<uint64_t>(remote);
  const uint32_t me = lane_id();
  W v;
  __builtin_memcpy(&v, &value, sizeof(T));
  W fetched = 0;
  uint64_t todo = active;
  for (int round = 0; round < kCombineRounds && todo; ++round) {
    const int leader = __builtin_ctzll(todo);
    const uint64_t group = __ballot(addr == lane_word(addr, leader)) & todo;
    const uint32_t members = __popcll(group);
    if (members == 1) break;
    W below = 0, total = 0;
    if ((__ballot(v == lane_word(v, leader)) & group) == group) {
      // one operand for the whole group (increments, a common addend): closed form
      below = static_cast<W>(rank_in_mask(group)) * v;
      total = static_cast<W>(members) * lane_word(v, leader);
    } else {
      for (uint64_t g = group; g; g &= g - 1) {
        const int lane = __builtin_ctzll(g);
        if (me == static_cast<uint32_t>(lane)) below = total;
        total += lane_word(v, lane);
      }
    }
    W base = 0;
    if (me == static_cast<uint32_t>(leader)) {
      base = __hip_atomic_fetch_add(reinterpret_cast<W *>(remote), total, __ATOMIC_RELAXED,
                                    __HIP_MEMORY_SCOPE_AGENT);
    }
    base = lane_word(base, leader);
    if ((group >> me) & 1u) fetched = base + below;
    todo &= ~group;
  }
  if ((todo >> me) & 1u) {
    fetched = __hip_atomic_fetch_add(reinterpret_cast<W *>(remote), v, __ATOMIC_RELAXED,
                                     __HIP_MEMORY_SCOPE_AGENT);
  }
  T old;
  __builtin_memcpy(&old, &fetched, sizeof(T));
  return old;
}

template <typename T>
__device__ __forceinline__ T amo_fetch_add(DeviceCtx *ctx, T *dest, T value, int pe) {
  T *remote = translate(own(dest, ctx), ctx->my_pe, pe);
  const T old = wave_fetch_add(remote, value);
  amo_record<T>(ctx, kOpcodeAtomicFa, remote, value, T(0), pe);
  return old;
}

template <typename T>
__device__ __forceinline__ void amo_add(DeviceCtx *ctx, T *dest, T value, int pe) {
  T *remote = translate(own(dest, ctx), ctx->my_pe, pe);
  (void)wave_fetch_add(remote, value);
  amo_record<T>(ctx, kOpcodeAtomicFa, remote, value, T(0), pe);
}

// compare_swap(dest, cond, value): store `value` iff *dest == cond; returns the old value.
template <typename T>
__device__ __forceinline__ T amo_fetch_cas(DeviceCtx *ctx, T *dest, T value, T cond, int pe) {
  T *remote = translate(own(dest, ctx), ctx->my_pe, pe);
  using W = typename AtomicWord<T>::type;
  W expected, desired;
  __builtin_memcpy(&expected, &cond, sizeof(T));
  __builtin_memcpy(&desired, &value, sizeof(T));
  __hip_atomic_compare_exchange_strong(reinterpret_cast<W *>(remote), &expected, desired,
                                       __ATOMIC_RELAXED, __ATOMIC_RELAXED,
                                       __HIP_MEMORY_SCOPE_AGENT);
  amo_record<T>(ctx, kOpcodeAtomicCs, remote, value, cond, pe);
  T old;
  __builtin_memcpy(&old, &expected, sizeof(T));
  return old;
}

// Unconditional exchange.  The reference approximates amo_set with a
// compare-and-swap loop whose first guess for the old value is zero
// (context_ib_tmpl_device.hpp:389-406) and asserts on amo_swap (:408-412).
// Here both are one native exchange, recorded as the first entry that loop
// would post: a compare-and-swap with compare operand 0.
template <typename T>
__device__ __forceinline__ T amo_swap(DeviceCtx *ctx, T *dest, T value, int pe) {
  T *remote = translate(own(dest, ctx), ctx->my_pe, pe);
  using W = typename AtomicWord<T>::type;
  W desired;
  __builtin_memcpy(&desired, &value, sizeof(T));
  W prev = __hip_atomic_exchange(reinterpret_cast<W *>(remote), desired, __ATOMIC_RELAXED,
                                 __HIP_MEMORY_SCOPE_AGENT);
  amo_record<T>(ctx, kOpcodeAtomicCs, remote, value, T(0), pe);
  T old;
  __builtin_memcpy(&old, &prev, sizeof(T));
  return old;
}

template <typename T>
__device__ __forceinline__ T amo_fetch(DeviceCtx *ctx, T *dest, int pe) {
  // reference: fetch == fetch_add(0), roc_shmem_gpu.cpp:589-598
  T *remote = translate(own(dest, ctx), ctx->my_pe, pe);
  using W = typename AtomicWord<T>::type;
  W raw = __hip_atomic_load(reinterpret_cast<W *>(remote), __ATOMIC_RELAXED,
                            __HIP_MEMORY_SCOPE_AGENT);
  amo_record<T>(ctx, kOpcodeAtomicFa, remote, T(0), T(0), pe);
  T old;
  __builtin_memcpy(&old, &raw, sizeof(T));
  return old;
}

enum BitOp { kBitAnd, kBitOr, kBitXor };

// Bitwise AMOs have no mlx5 opcode (the reference asserts,
// context_ib_tmpl_device.hpp:408-445); they run natively and leave no WQE.
template <typename T, int Op>
__device__ __forceinline__ T amo_fetch_bitwise(DeviceCtx *ctx, T *dest, T value, int pe) {
  T *remote = translate(own(dest, ctx), ctx->my_pe, pe);
  if constexpr (Op == kBitAnd)
    return __hip_atomic_fetch_and(remote, value, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
  else if constexpr (Op == kBitOr)
    return __hip_atomic_fetch_or(remote, value, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
  else
    return __hip_atomic_fetch_xor(remote, value, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
}

}  // namespace detail
}  // namespace rocshmem

#endif
