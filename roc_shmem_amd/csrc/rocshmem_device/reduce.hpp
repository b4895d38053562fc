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

constexpr int kReduceUnroll = 8;   // vectors per lane per pass
constexpr uint32_t kMinStandardSlotTicks = 1500;   // 15 us: the shortest slots standard calls are paced with
constexpr int kReducePeChunk = 1;  // members whose loads are issued together

// Members of a collective: world PEs pe_start + k * pe_stride, k < size.  The
// active-set calls name powers of two (1 << logPE_stride); a team may have any
// stride (roc_shmem_team_split_strided, library/src/roc_shmem.cpp:236-250).
struct ActiveSet {
  int pe_start;
  int pe_stride;
  int size;
  __device__ __forceinline__ int pe_at(int k) const { return pe_start + k * pe_stride; }
};

// Ordinal of the PE `rel` places after pe_start in a set of stride pe_stride.
__device__ __forceinline__ int member_index(int rel, int pe_stride) {
  if ((pe_stride & (pe_stride - 1)) == 0) return rel >> __builtin_ctz(pe_stride);
  return rel / pe_stride;
}

// Reduce vectors [v_begin, v_end) of the symmetric arrays `src`/`dst` (given
// as this PE's addresses, both 16-byte aligned) over all members and write
// the result into every member's destination.
//
// One pass of the workgroup covers U*nthr consecutive vectors of every
// member: access u of lane t is vector u*nthr + t of the pass, so each
// load/store instruction of the workgroup sweeps nthr*16 consecutive bytes
// and the U accesses of one member follow each other through U*nthr*16
// consecutive bytes (128 KiB for 1024 lanes and U = 8).  Measured on MI355X
// (8 slices x 256 MiB): 32 KiB per member per pass reaches 5.2 TB/s, 128 KiB
// 5.8 TB/s; dealing the same bytes to waves as private 8 KiB chunks instead
// (every instruction of the workgroup then touches sixteen separate 1 KiB
// pieces) drops to 4.9 TB/s.
//
// Memory is addressed through raw buffer descriptors: the pass base of each
// member is workgroup-uniform and lives in scalar registers (descriptor +
// scalar offset), the only per-lane address part is the 32-bit `tid*16`.
// Besides freeing some thirty vector registers of 64-bit addresses, the
// descriptor's size field makes the last, partial pass safe without a
// separate loop: accesses past `valid` bytes load zeros and store nothing.
template <typename T, ROC_SHMEM_OP Op, int U = kReduceUnroll, int C = kReducePeChunk>
__device__ __forceinline__ void reduce_vectors(T *dst, const T *src, size_t v_begin,
                                               size_t v_end, const ActiveSet &as, int my_pe,
                                               uint32_t tid, uint32_t nthr, size_t first_pass = 0,
                                               size_t pass_step = 1, Pacer pacer = Pacer{0u, 0u},
                                               uint32_t start_at = 0) {
  using Acc = typename AccOf<T, Op>::type;
  using V = VecOf<T>;
  constexpr int E = V::kElems;
  constexpr int kNt = 2;                       // cache policy: non-temporal
  // Results are written through to memory (kWriteThrough), so that the barrier
  // that ends the collective need not write this XCD's L2 back (wg_flag_barrier).
  // (-DROCSHMEM_AB_PLAIN_STORES: an A/B build for measurements, whose stores stay in the L2
  // and whose closing barrier writes it back.)
#ifdef ROCSHMEM_AB_PLAIN_STORES
  constexpr int kStore = kNt;
#else
  constexpr int kStore = kNt | kWriteThrough;
#endif

  const int64_t stride = static_cast<int64_t>(g_state.slice_stride);
  char *src0 = const_cast<char *>(reinterpret_cast<const char *>(src)) +
               (static_cast<int64_t>(as.pe_start) - my_pe) * stride;
  char *dst0 =
      reinterpret_cast<char *>(dst) + (static_cast<int64_t>(as.pe_start) - my_pe) * stride;
  const int64_t member_step = stride * as.pe_stride;

  const uint32_t lane_off = tid * 16u;
  const uint32_t access_bytes = nthr * 16u;       // bytes one instruction of the workgroup sweeps
  const uint32_t pass_bytes = access_bytes * U;   // at most 128 KiB
  // The range and the deal are the same in every lane.  Saying so keeps the loop's bookkeeping
  // in scalar registers: the callers derive them through 64-bit compares and divisions, which
  // the compiler carries out on the vector unit, and whatever is computed from a vector value
  // stays one (twenty vector registers and as many spills in the streaming kernels).
  v_begin = uniform(v_begin);
  v_end = uniform(v_end);
  first_pass = uniform(first_pass);
  pass_step = uniform(pass_step);
  start_at = uniform(start_at);
  const size_t byte_end = v_end * 16;

  // This workgroup takes passes first_pass, first_pass + pass_step, ... of the range: `mine` of
  // them, visited in the order start_at, start_at + 1, ..., mine - 1, 0, ..., start_at - 1.
  const size_t step_bytes = pass_step * pass_bytes;
  const size_t byte_begin = v_begin * 16 + first_pass * pass_bytes;
  if (byte_begin >= byte_end) return;
  // A short first pass is the only one, and a wave whose every lane lies past
  // its end has nothing to do in it.  Its accesses would be clipped, but a
  // clipped access still costs its issue slots: a 4 KiB reduction by one
  // workgroup of 1024 lanes took 10.4 us against 7.1 us by one of 256, now 8.0.
  if (byte_end - byte_begin < pass_bytes && uniform((tid & ~63u) * 16u) >= byte_end - byte_begin)
    return;
  const uint32_t mine = uniform(static_cast<uint32_t>((byte_end - byte_begin + step_bytes - 1) / step_bytes));
  if (start_at >= mine) start_at = uniform(start_at % mine);
  for (uint32_t turn = 0; turn < mine; ++turn) {
    uint32_t p = turn + start_at;
    if (p >= mine) p -= mine;
    const size_t b = byte_begin + p * step_bytes;
    const size_t left = byte_end - b;
    const int valid = static_cast<int>(left < pass_bytes ? left : pass_bytes);
    Acc acc[U][E];
    pacer.wait_slot();
    {
      __amdgpu_buffer_rsrc_t rs = uniform_rsrc(src0 + b, valid);
#pragma unroll
      for (int u = 0; u < U; ++u) {
        typename V::Pack p;
        p.raw = __builtin_amdgcn_raw_buffer_load_b128(rs, lane_off, u * access_bytes, kNt);
#pragma unroll
        for (int e = 0; e < E; ++e) acc[u][e] = to_acc<T, Acc>(p.e[e]);
      }
    }
    int k = 1;
    for (; k + C <= as.size; k += C) {
      typename V::Pack p[C][U];
#pragma unroll
      for (int c = 0; c < C; ++c) {
        __amdgpu_buffer_rsrc_t rs = uniform_rsrc(src0 + (k + c) * member_step + b, valid);
#pragma unroll
        for (int u = 0; u < U; ++u)
          p[c][u].raw = __builtin_amdgcn_raw_buffer_load_b128(rs, lane_off, u * access_bytes, kNt);
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
      __amdgpu_buffer_rsrc_t rs = uniform_rsrc(src0 + k * member_step + b, valid);
      typename V::Pack p[U];
#pragma unroll
      for (int u = 0; u < U; ++u)
        p[u].raw = __builtin_amdgcn_raw_buffer_load_b128(rs, lane_off, u * access_bytes, kNt);
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
    // (load and store slots of equal length: a load slot of 0.8, 0.9, 1.1 or 1.2 of the store
    // slot's length measured 6397, 6483, 6557 and 6463 GB/s at the best rate of each against 6565)
    pacer.wait_slot();
    for (int m = 0; m < as.size; ++m) {
      __amdgpu_buffer_rsrc_t rd = uniform_rsrc(dst0 + m * member_step + b, valid);
#pragma unroll
      for (int u = 0; u < U; ++u)
        __builtin_amdgcn_raw_buffer_store_b128(out[u].raw, rd, lane_off, u * access_bytes, kStore);
    }
    if (turn == 0) timeline_mark(2);            // stores of the first burst issued
    if (turn + 1 == mine) timeline_mark(3);     // stores of the last pass issued
  }
  // every wave has its own stores in memory before it meets the others
  __builtin_amdgcn_s_waitcnt(0);
  timeline_mark(4);
  timeline_mark(6, (__builtin_amdgcn_s_getreg((3 << 11) | (0 << 6) | 20) & 15u) |
                       (static_cast<uint64_t>(pacer.period) << 16));
}

// The same reduction with the loads staged through LDS: every lane's 16-byte
// loads go straight from memory into the workgroup's LDS (global_load_lds,
// no vector registers in between), `chunk` members' worth at a time, and the
// fold reads them back from LDS.  Each lane reads only what it loaded itself,
// so the waves need no barrier among themselves.  `stage` holds `stage_bytes`
// of dynamic LDS; only whole passes are handled here (the caller gives the
// remainder to reduce_vectors).  Kept as a measured alternative: with eight
// members it frees some sixty vector registers per lane and lets all members'
// loads of a pass be in flight together, and on MI355X it is slower all the
// same (the stream is bound by the memory system, not by registers or by
// loads in flight), so the register path above is the one every call takes
// unless the caller asks for this one.
template <typename T, ROC_SHMEM_OP Op, int U>
__device__ __forceinline__ void reduce_vectors_lds(T *dst, const T *src, size_t n_passes,
                                                   const ActiveSet &as, int my_pe, uint32_t tid,
                                                   uint32_t nthr, size_t first_pass, size_t pass_step,
                                                   char *stage, uint32_t stage_bytes) {
  using Acc = typename AccOf<T, Op>::type;
  using V = VecOf<T>;
  constexpr int E = V::kElems;
  constexpr int kNt = 2;
  constexpr int kStore = kNt | kWriteThrough;   // as in reduce_vectors
  const int64_t stride = static_cast<int64_t>(g_state.slice_stride);
  char *src0 = const_cast<char *>(reinterpret_cast<const char *>(src)) +
               (static_cast<int64_t>(as.pe_start) - my_pe) * stride;
  char *dst0 =
      reinterpret_cast<char *>(dst) + (static_cast<int64_t>(as.pe_start) - my_pe) * stride;
  const int64_t member_step = stride * as.pe_stride;
  const uint32_t lane_off = tid * 16u;
  const uint32_t wave_off = (tid & ~63u) * 16u;     // where this wave's 64 slots start
  const uint32_t access_bytes = nthr * 16u;
  const uint32_t pass_bytes = access_bytes * U;
  int chunk = static_cast<int>(stage_bytes / pass_bytes);   // members staged together
  if (chunk > as.size) chunk = as.size;
  if (chunk < 1) return;
  typedef __attribute__((address_space(3))) void *LdsPtr;
  typedef const __attribute__((address_space(1))) void *GlobalPtr;
  for (size_t pass = first_pass; pass < n_passes; pass += pass_step) {
    const size_t b = pass * pass_bytes;
    Acc acc[U][E];
    for (int k0 = 0; k0 < as.size; k0 += chunk) {
      const int members = as.size - k0 < chunk ? as.size - k0 : chunk;
      for (int c = 0; c < members; ++c) {
        const char *from = src0 + (k0 + c) * member_step + b + lane_off;
#pragma unroll
        for (int u = 0; u < U; ++u)
          __builtin_amdgcn_global_load_lds(
              (GlobalPtr)(from + u * access_bytes),   // address-space casts: C style only
              (LdsPtr)(stage + (c * U + u) * access_bytes + wave_off), 16, 0, kNt);
      }
      __builtin_amdgcn_s_waitcnt(0);
      for (int c = 0; c < members; ++c) {
#pragma unroll
        for (int u = 0; u < U; ++u) {
          typename V::Pack p;
          p.raw = *reinterpret_cast<const u32x4 *>(stage + (c * U + u) * access_bytes + lane_off);
#pragma unroll
          for (int e = 0; e < E; ++e) {
            const Acc x = to_acc<T, Acc>(p.e[e]);
            acc[u][e] = (k0 + c == 0) ? x : fold<Op, Acc>(acc[u][e], x);
          }
        }
      }
    }
    typename V::Pack out[U];
#pragma unroll
    for (int u = 0; u < U; ++u)
#pragma unroll
      for (int e = 0; e < E; ++e) out[u].e[e] = from_acc<T, Acc>(acc[u][e]);
    for (int m = 0; m < as.size; ++m) {
      __amdgpu_buffer_rsrc_t rd = uniform_rsrc(dst0 + m * member_step + b, static_cast<int>(pass_bytes));
#pragma unroll
      for (int u = 0; u < U; ++u)
        __builtin_amdgcn_raw_buffer_store_b128(out[u].raw, rd, lane_off, u * access_bytes, kStore);
    }
  }
  __builtin_amdgcn_s_waitcnt(0);
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
  const int64_t member_step = stride * as.pe_stride;
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
__device__ __forceinline__ void wg_all_reduce(int my_pe, T *dest, const T *source, size_t nreduce,
                                              int pe_start, int pe_stride, int pe_size,
                                              long *psync, int shard = 0, int nshards = 1,
                                              int64_t psync_pe_step = 0, char *lds_stage = nullptr,
                                              uint32_t lds_stage_bytes = 0) {
  // Workgroup-collective: every lane holds the same arguments.
  my_pe = uniform(my_pe);
  dest = own(uniform(dest), my_pe);       // symmetric arguments: the caller's own copies
  source = own(uniform(source), my_pe);
  nreduce = uniform(nreduce);
  pe_start = uniform(pe_start);
  pe_stride = uniform(pe_stride);
  pe_size = uniform(pe_size);
  psync = own(uniform(psync), my_pe);
  shard = uniform(shard);
  nshards = uniform(nshards);
  psync_pe_step = static_cast<int64_t>(uniform(static_cast<unsigned long>(psync_pe_step)));
  if (nreduce == 0) return;  // reference: Context::to_all early-out, context_tmpl_device.hpp:68-70
  if (pe_size > kMaxPes || pe_size <= 0 || nshards <= 0 || shard < 0 || shard >= nshards) {
    status_raise(kStatusBadArgument);
    return;
  }
  const ActiveSet as{pe_start, pe_stride, pe_size};
  const int my_idx = member_index(my_pe - pe_start, pe_stride);
  const uint32_t tid = flat_thread_id();
  const uint32_t nthr = flat_block_size();
  const size_t n = nreduce;
  // The range is dealt to pe_size * nshards workgroups: member k's workgroup
  // of shard s is part s * pe_size + k.
  const size_t parts = static_cast<size_t>(pe_size) * nshards;
  // (-DROCSHMEM_AB_SWAP_DEAL: an A/B build for measurements in which neighbouring members swap
  // their passes.  With 8 PEs every PE's workgroups run on one XCD, and the odd XCDs end a
  // large reduction 10-13 us after the even ones (6-8 % later when the workgroups run free);
  // with the passes swapped it is still the odd XCDs, so it is the XCD and not the address.)
#ifdef ROCSHMEM_AB_SWAP_DEAL
  const size_t part = static_cast<size_t>(shard) * pe_size + (my_idx ^ 1);
#else
  const size_t part = static_cast<size_t>(shard) * pe_size + my_idx;
#endif

  constexpr size_t E = VecOf<T>::kElems;
  // The vector path stores 16-byte aligned and loads at any 4-byte alignment,
  // so it takes every pair of arrays that agree modulo 4 (all pairs of 4- and
  // 8-byte elements; 2-byte elements an even number of elements apart): the
  // elements in front of the destination's next boundary and behind the last
  // whole vector go one by one, the rest in vectors.  The boundary is the one
  // copies use (stream_head): 1 KiB for large arrays, so that the 1 KiB a wave
  // stores with one instruction never straddles two.  8 x 2^26 fp32 shifted by
  // one element used to take the element path at 2.5 TB/s and now run at the
  // aligned arrays' 5.9 TB/s.
  const uintptr_t dest_at = reinterpret_cast<uintptr_t>(dest);
  const uintptr_t differ = dest_at ^ reinterpret_cast<uintptr_t>(source);
  const bool coaligned = (differ & 3u) == 0 && dest_at % sizeof(typename Storage<T>::elem) == 0;
  size_t lead = 0, nvec = 0;
  if (coaligned) {
    const size_t bytes = n * sizeof(typename Storage<T>::elem);
    const uintptr_t boundary = bytes >= 65536 ? kStoreChunkBytes : bytes >= 4096 ? 128u : 16u;
    lead = ((boundary - (dest_at & (boundary - 1))) & (boundary - 1)) / sizeof(typename Storage<T>::elem);
    if (lead > n) lead = n;
    nvec = (n - lead) / E;
  }
  const size_t full_pass_vecs = static_cast<size_t>(kReduceUnroll) * nthr;
  // A stream: every workgroup of the call has two full passes or more.  Its passes are dealt
  // round-robin over the call's workgroups, and it may follow the schedule (Pacer).
  const bool stream = nvec >= 2 * parts * full_pass_vecs;
  // A standard (unsharded) call knows its own members only, and the schedule is sized for all
  // the workgroups that stream at the same time.  Such a call therefore counts itself in while
  // it runs and follows the schedule only when (nearly) every workgroup of the grid is inside
  // a call like it - a grid that tiles one large reduction over its workgroups; a lone large
  // call in a grid that does other things runs free.
  // (And only when its slots would be long enough, see below: a call that would run free
  // whatever the count says does not pay for the count.)
  const uint64_t pass_bytes_full = static_cast<uint64_t>(full_pass_vecs) * 16u;
  const uint32_t pace_rate = pass_bytes_full >= (128u << 10) ? g_state.pace_reduce_bytes_per_tick
                                                             : g_state.pace_reduce_short_bytes_per_tick;
  const bool counted = stream && nshards == 1 && pace_rate != 0 && grid_is_resident() &&
                       grid_workgroups() * pass_bytes_full * static_cast<uint64_t>(pe_size) >=
                           static_cast<uint64_t>(kMinStandardSlotTicks) * pace_rate;
  if (counted && tid == 0)
    __hip_atomic_fetch_add(streaming_workgroups(), 1u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);

  timeline_mark(0);
  wg_flag_barrier(psync, 0, my_pe, my_idx, pe_start, pe_stride, pe_size, psync_pe_step);
  timeline_mark(1);
  // How many workgroups stream right now, read once for the whole workgroup: one look at the
  // word instead of one per wave, and the workgroup's waves then agree on whether they follow
  // the schedule (the count may cross the line between two waves' looks).
  __shared__ uint32_t streaming_now;
  if (counted) {
    if (tid == 0)
      streaming_now = __hip_atomic_load(streaming_workgroups(), __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
    __syncthreads();
  }

  // Whether this workgroup stores anything that is not written through (the
  // element path's plain stores): decides how the closing barrier releases.
  bool plain_stores = false;
  if (coaligned) {
    T *const vec_dest = dest + lead;
    const T *const vec_source = source + lead;
    // Vectors [v0, v1) in passes first_pass, first_pass + pass_step, ... of this workgroup.
    size_t v0 = 0, v1 = nvec, first_pass = part, pass_step = parts;
    bool short_passes = nvec < parts * full_pass_vecs;
    Pacer pacer{0u, 0u};
    uint32_t start_at = 0;
    if (nshards == 1 && !stream) {
      // One workgroup per member and less than two full passes each: member k takes the k-th
      // contiguous share (dealing a single pass or two would leave members without work).
      const size_t share = (nvec + pe_size - 1) / pe_size;
      v0 = share * my_idx;
      v1 = v0 + share;
      if (v0 > nvec) v0 = nvec;
      if (v1 > nvec) v1 = nvec;
      first_pass = 0;
      pass_step = 1;
      short_passes = v1 - v0 < full_pass_vecs;
    }
    if (stream) {
      // Passes are dealt round-robin over all workgroups of the call, so that the workgroups
      // running at one moment sweep one compact window of every array.  Measured on MI355X
      // (8 -> 8 fp32 reduction, no barriers): 6.06 TB/s against 5.86 TB/s when every
      // workgroup walks a region of its own; giving each member a contiguous share and
      // striding only within it was no better and less even across launch shapes.
      // Paced (see Pacer) when the library holds a rate and the grid fills the chip (8 PEs,
      // fp32, paced against free at the default rate: with two passes per workgroup +1 % at
      // 32 x 1024 lanes per PE, +5 % at 32 x 512, +8 % at 64 x 512; with four +2 to +6 %;
      // with eight +6 %).
      const uint64_t pass_bytes = static_cast<uint64_t>(full_pass_vecs) * 16u;
      const uint64_t wgs = grid_workgroups();
      // A grid that tiles one large array over standard calls: each call deals its own tile,
      // so the workgroups of different calls move through their tiles in step, and when every
      // one of them starts at its tile's first passes, all windows in flight agree in the
      // address bits that count passes within a tile and differ only in the bits that number
      // the tiles; the memory system serves that badly (8 PEs, 32 x 1024 lanes per PE, one
      // call per workgroup over a tile of 2^21 floats: 4600 GB/s, against 5800 when every
      // member walks a contiguous share of the tile).  A call therefore starts its round-robin
      // at a turn taken from its address: 5 g / W for a tile that begins g passes into the
      // slice, in a grid of W workgroups.  g / W alone - how many grids' worth of passes lie in
      // front of the tile - already differs between the tiles that would collide, so that the
      // windows in flight differ in every address bit between a pass and a grid's worth of
      // passes, as those of one sharded call do; but with it the rate depended on the slice
      // stride, the members' arrays lying at distances that bring some windows back onto each
      // other, and the finer turns of 5 g / W do not show that (1 GiB per PE: 6373-6400 GB/s
      // either way, the sharded form 6381; 576 MiB: 5970 against 6404; 1100 MiB: 6040 against
      // 6276; five other strides within 1 % of each other).
      // The address is taken relative to the caller's slice, so that all members of a call
      // agree on the turn whatever the slice stride is.  (32-bit arithmetic in KiB: the offset
      // and a pass are multiples of it.)
      if (nshards == 1 && nvec / full_pass_vecs < wgs) {
        const uint64_t into_slice = reinterpret_cast<uintptr_t>(vec_dest) -
                                    reinterpret_cast<uintptr_t>(g_state.heap_base0) -
                                    static_cast<uint64_t>(my_pe) * g_state.slice_stride;
        start_at = 5u * (static_cast<uint32_t>(into_slice >> 10) / static_cast<uint32_t>(pass_bytes >> 10)) /
                   static_cast<uint32_t>(wgs);
      }
      const uint32_t rate = pace_rate;
      if (nshards > 1) {
        if (rate != 0 && grid_is_resident())
          pacer = make_anchored_pacer(rate, parts * pass_bytes * static_cast<uint64_t>(pe_size));
      } else if (counted) {
        // Standard calls follow the schedule when (nearly) the whole grid is inside calls like
        // them, and when the slots are long enough: with few members a pass is few rounds of
        // loads, the slots are short, and what the change of direction costs is no longer paid
        // for (tiled standard calls, paced against free at the default rate: 16 and 8 members,
        // slots of 80 and 40 us, +6 to +9 %; 4 members, 20 us, -2 to +3 %; 2 members, 10 us,
        // -7.5 to +4 %, mostly losses.  The sharded form gains down to 2 members).
        const uint32_t inside = uniform(streaming_now);
        if (static_cast<uint64_t>(inside) * 4u >= wgs * 3u)
          pacer = make_anchored_pacer(rate, wgs * pass_bytes * static_cast<uint64_t>(pe_size));
      }
    }
    if (lds_stage != nullptr && stream && nshards > 1) {
      // whole passes through LDS, two vectors per lane per member; what is left of the
      // range goes the usual way, to whoever's turn it would have been
      const size_t lds_pass_vecs = 2u * nthr;
      const size_t whole = nvec / lds_pass_vecs;
      reduce_vectors_lds<T, Op, 2>(vec_dest, vec_source, whole, as, my_pe, tid, nthr, part, parts, lds_stage,
                                   uniform(lds_stage_bytes));
      if (whole * lds_pass_vecs < nvec && whole % parts == part)
        reduce_vectors<T, Op, 2, 1>(vec_dest, vec_source, whole * lds_pass_vecs, nvec, as, my_pe, tid, nthr);
    } else if (short_passes) {
      // Less than one full pass per workgroup costs the chain of load latencies, and full
      // passes would leave most workgroups idle while a few walk eight members' loads one
      // after the other: passes of two vectors per lane with four members' loads issued
      // together (a 4096-element int64 reduction among 4 PEs: 9.1 -> 6.1 us per call; fp32
      // sum among 8 PEs, 1 MiB per PE with 16 workgroups of 512 lanes each 16.5 -> 13.0 us,
      // 256 KiB with 4 workgroups of 1024 lanes 21.9 -> 11.3 us).
      reduce_vectors<T, Op, 2, 4>(vec_dest, vec_source, v0, v1, as, my_pe, tid, nthr, first_pass, pass_step);
    } else {
      reduce_vectors<T, Op>(vec_dest, vec_source, v0, v1, as, my_pe, tid, nthr, first_pass, pass_step, pacer,
                            start_at);
    }
    if (part == parts - 1) {
      if (lead) reduce_elements<T, Op>(dest, source, 0, lead, as, my_pe, tid, nthr);
      if (lead + nvec * E < n)
        reduce_elements<T, Op>(dest, source, lead + nvec * E, n, as, my_pe, tid, nthr);
      plain_stores = lead != 0 || lead + nvec * E < n;
    }
  } else {
    plain_stores = true;
    const size_t share = (n + parts - 1) / parts;
    size_t e0 = share * part;
    size_t e1 = e0 + share;
    if (e0 > n) e0 = n;
    if (e1 > n) e1 = n;
    reduce_elements<T, Op>(dest, source, e0, e1, as, my_pe, tid, nthr);
  }

#ifdef ROCSHMEM_AB_PLAIN_STORES
  plain_stores = true;
#endif
  wg_flag_barrier(psync, 1, my_pe, my_idx, pe_start, pe_stride, pe_size, psync_pe_step,
                  !plain_stores);
  timeline_mark(5);
  if (counted && tid == 0)
    __hip_atomic_fetch_sub(streaming_workgroups(), 1u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
}

}  // namespace detail
}  // namespace rocshmem

#endif
