// Agent-scope synchronisation between the workgroups that stand for the PEs
// of one collective: bounded flag waits and an all-to-all flag barrier on
// the caller's (or the team's) pSync array.
//
// Every wait is bounded by DeviceState::wait_limit_ticks of the 100 MHz
// constant clock; a wait that gives up records kStatusWaitTimeout in the
// sticky status word, after which every later wait returns at once, so a
// mis-launched grid drains instead of hanging the device.
#ifndef ROCSHMEM_MI355X_DEVICE_SYNC_HPP
#define ROCSHMEM_MI355X_DEVICE_SYNC_HPP

#include "state.hpp"
#include "wave.hpp"

namespace rocshmem {
namespace detail {

// Per translation unit copy of the runtime state; the host library uploads it
// into every registered translation unit during roc_shmem_init().
static __constant__ DeviceState g_state;

__device__ __forceinline__ void fence_release_agent() {
  __builtin_amdgcn_fence(__ATOMIC_RELEASE, "agent");
}
__device__ __forceinline__ void fence_acquire_agent() {
  __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "agent");
}
__device__ __forceinline__ void fence_acq_rel_agent() {
  __builtin_amdgcn_fence(__ATOMIC_SEQ_CST, "agent");
}

__device__ __forceinline__ bool status_failed() {
  return __hip_atomic_load(g_state.status, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT) !=
         kStatusOk;
}

__device__ __forceinline__ void status_raise(uint32_t code) {
  uint32_t expected = kStatusOk;
  __hip_atomic_compare_exchange_strong(g_state.status, &expected, code, __ATOMIC_RELAXED,
                                       __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
}

// How many workgroups are inside a large standard (unsharded) reduction at this moment: a word
// of its own cache line in the status block, counted up and down by those calls themselves
// (wg_all_reduce), which is how a call that knows only its own members learns whether the
// whole grid streams with it.
constexpr int kStreamingWorkgroupsWord = 16;
__device__ __forceinline__ uint32_t *streaming_workgroups() {
  return g_state.status + kStreamingWorkgroupsWord;
}

// Clock reading number `mark` of the calling wave, in builds with -DROCSHMEM_TIMELINE (and when
// the host has put a buffer in place: ROC_SHMEM_TIMELINE_FILE); nothing otherwise.
#ifdef ROCSHMEM_TIMELINE
__device__ __forceinline__ void timeline_mark(int mark, uint64_t value = ~0ull) {
  uint64_t *buf = *reinterpret_cast<uint64_t *const *>(g_state.status + kTimelinePointerWord);
  const uint32_t wave = blockIdx.x * 16u + flat_thread_id() / 64u;
  if (buf && wave < static_cast<uint32_t>(kTimelineWaves) && lane_id() == 0)
    buf[wave * kTimelineMarks + mark] = value == ~0ull ? wall_clock64() : value;
}
#else
__device__ __forceinline__ void timeline_mark(int, uint64_t = 0) {}
#endif

// Translate a symmetric address of PE `from_pe` into the slice of PE `to_pe`.
template <typename T>
__device__ __forceinline__ T *translate(T *ptr, int from_pe, int to_pe) {
  int64_t delta = (static_cast<int64_t>(to_pe) - from_pe) *
                  static_cast<int64_t>(g_state.slice_stride);
  return reinterpret_cast<T *>(
      reinterpret_cast<uintptr_t>(ptr) + static_cast<uintptr_t>(delta));
}

// The calling PE's own copy of the symmetric object that `ptr` names by its symmetric address;
// every other pointer (and every pointer when DeviceState::rebase_args is off) comes back
// unchanged.  All PEs live in one process, so a kernel argument holds one value for the
// workgroups of every PE: the address roc_shmem_malloc returned, which is the object's
// address in PE 0's slice - that address is what stands for "my copy" in a call.  The
// roc_shmem_* calls pass their symmetric and local buffer arguments through this, which lets a
// kernel written for the reference (one process per PE, every process passing its own address:
// reduction_tester.cpp:74-104, primitive_tester.cpp:32-82) run unchanged.  A pointer into
// another PE's slice - what roc_shmem_ptr returns, say, handed on as the local side of a put or
// a get or as the word to wait on - is an address like any other and is used as it is, as the
// reference uses it (context_ib_device.cpp:128-137).  One case cannot be told apart: PE 0's
// copy, named on purpose by a workgroup of another PE, has the symmetric address itself and is
// taken for the caller's own copy (roc_shmemx_my_addr and roc_shmem_ptr give explicit control).
template <typename T>
__device__ __forceinline__ T *own(T *ptr, int my_pe) {
  const uint64_t rel =
      reinterpret_cast<uint64_t>(ptr) - reinterpret_cast<uint64_t>(g_state.heap_base0);
  if (!g_state.rebase_args || rel >= g_state.slice_stride) return ptr;   // below the arena: rel wraps
  return reinterpret_cast<T *>(const_cast<char *>(g_state.heap_base0) +
                               static_cast<uint64_t>(my_pe) * g_state.slice_stride + rel);
}
template <typename T>
__device__ __forceinline__ T *own(T *ptr, const DeviceCtx *c) {
  return own(ptr, c->my_pe);
}


enum WaitCmp { kWaitEq, kWaitNe, kWaitGt, kWaitGe, kWaitLt, kWaitLe };

template <typename T>
__device__ __forceinline__ bool compare_for_wait(T have, int cmp, T want) {
  switch (cmp) {
    case kWaitEq: return have == want;
    case kWaitNe: return have != want;
    case kWaitGt: return have > want;
    case kWaitGe: return have >= want;
    case kWaitLt: return have < want;
    default: return have <= want;
  }
}

// Spin until `*ptr cmp want` holds, reading through agent-scope atomic loads
// (the reference polls with uncached loads, context_tmpl_device.hpp:199-246).
// Returns false on timeout or when the status word is already raised.
template <typename T>
struct WaitWord {
  static_assert(sizeof(T) == 1 || sizeof(T) == 2 || sizeof(T) == 4 || sizeof(T) == 8,
                "wait on naturally aligned words of 1, 2, 4 or 8 bytes");
  using type = typename std::conditional<
      sizeof(T) == 8, uint64_t,
      typename std::conditional<sizeof(T) == 4, uint32_t,
                                typename std::conditional<sizeof(T) == 2, uint16_t,
                                                          uint8_t>::type>::type>::type;
};

template <typename T>
__device__ __forceinline__ bool bounded_wait(const T *ptr, int cmp, T want) {
  using Word = typename WaitWord<T>::type;
  const Word *wptr = reinterpret_cast<const Word *>(ptr);
  uint64_t start = wall_clock64();
  uint32_t spins = 0;
  for (;;) {
    Word raw = __hip_atomic_load(wptr, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
    T have;
    __builtin_memcpy(&have, &raw, sizeof(T));
    if (compare_for_wait(have, cmp, want)) return true;
    __builtin_amdgcn_s_sleep(1);
    if ((++spins & 63u) == 0) {
      if (status_failed()) return false;
      if (wall_clock64() - start > g_state.wait_limit_ticks) {
        status_raise(kStatusWaitTimeout);
        return false;
      }
    }
  }
}

// All-to-all flag barrier among the `n_pes` workgroups (one per PE of the
// active set) that share one collective call.  `psync` is this PE's copy of
// the symmetric pSync slice, `set` selects slots [set*n_pes, (set+1)*n_pes).
//
// Arrival: thread t < n_pes publishes everything this workgroup wrote and
// sets slot `my_idx` in the copy owned by member t.  Completion: thread t
// waits for slot t of the own copy, then clears it, so the array is all
// ROC_SHMEM_SYNC_VALUE again on return (the reference restores it the same
// way, context_ib_tmpl_device.hpp:178-180,231-233).  Two consecutive barriers
// must use different sets; the same set may be reused once a barrier on the
// other set has completed in between.
//
// Must be called by every thread of the workgroup.
//
// Fences are issued by the few lanes that handle flags, not by every wave:
// the workgroup barrier in front guarantees that all the workgroup's stores
// have left for L2 (s_waitcnt before s_barrier), so one L2 write-back covers
// them, and one invalidate of this CU's L1 and this XCD's L2 before the
// closing workgroup barrier covers every wave that resumes after it.  With a
// fence per wave, 256 workgroups of 16 waves spent 31 us in one barrier
// (each fence walks a whole L2); the flag lanes alone need a fraction of it.
//
// `pe_step` is the distance in bytes between two PEs' copies of the flag array:
// 0 stands for the slice stride of the symmetric heap (pSync is a symmetric
// object); a flag array that lives outside the heap names its own.
//
// `written_through`: the caller vouches that everything this workgroup has
// stored since its last release went to memory past the L2 (stores with the
// sc1 policy bit, kWriteThrough) and that every wave has waited for its own
// such stores (s_waitcnt vmcnt(0)) before it came here.  Then there is nothing
// in this XCD's L2 to write back for the other members, and the flag lanes
// skip the write-back: at the end of a large reduction, where the 32
// workgroups of an XCD arrive together and each write-back walks the whole L2,
// that took 9 us of 690 (8 x 2^26 fp32: 6215 -> 6285 GB/s).  The same protocol
// as the send queues' (wqe.hpp): data written through, the writer waits for
// it, then an agent-scope atomic hands over.
__device__ __forceinline__ void wg_flag_barrier(long *psync, int set, int my_pe, int my_idx,
                                                int pe_start, int pe_stride, int n_pes,
                                                int64_t pe_step = 0, bool written_through = false) {
  __syncthreads();
  const uint32_t tid = flat_thread_id();
  const uint32_t nthr = flat_block_size();
  if (pe_step == 0) pe_step = static_cast<int64_t>(g_state.slice_stride);
  if (tid < static_cast<uint32_t>(n_pes)) {
    if (written_through) {
      __builtin_amdgcn_fence(__ATOMIC_RELEASE, "workgroup");
    } else {
      fence_release_agent();
    }
    for (uint32_t t = tid; t < static_cast<uint32_t>(n_pes); t += nthr) {
      int peer = pe_start + static_cast<int>(t) * pe_stride;
      unsigned long long *slot = reinterpret_cast<unsigned long long *>(
          reinterpret_cast<char *>(psync) + (static_cast<int64_t>(peer) - my_pe) * pe_step) +
          set * n_pes + my_idx;
      __hip_atomic_store(slot, 1ull, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
    }
    for (uint32_t t = tid; t < static_cast<uint32_t>(n_pes); t += nthr) {
      unsigned long long *mine =
          reinterpret_cast<unsigned long long *>(psync + set * n_pes + static_cast<int>(t));
      bounded_wait<unsigned long long>(mine, kWaitEq, 1ull);
      __hip_atomic_store(mine, 0ull, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
    }
    fence_acquire_agent();
  }
  __syncthreads();
}

// Barrier on a pSync slice that the library owns (a team's barrier pool): no
// resets and one round instead of two.  Call number e of a slice writes e into
// slot `my_idx` of every member's copy and waits until each slot of its own
// copy has reached e; the count of calls made so far sits in slot kEpochSlot
// of the own copy.  Slots only grow, so a member that is already in call e+1
// can only satisfy, never spoil, the wait of one still in call e, and nothing
// has to be cleared between calls.  Every member must call it the same number
// of times on a slice, which a collective guarantees; the host zeroes the pool
// when the team is made.  Two flag barriers in a row took 1.7-2.4 us for 4
// PEs (the figure differs from card to card), this one call 1.1-1.5 us.
constexpr int kEpochSlot = kSyncSlots - 1;   // kMaxPes arrival slots fit below it

__device__ __forceinline__ void wg_epoch_barrier(long *psync, int my_pe, int my_idx,
                                                 int pe_start, int pe_stride, int n_pes) {
  __syncthreads();
  const uint32_t tid = flat_thread_id();
  const uint32_t nthr = flat_block_size();
  unsigned long long *own = reinterpret_cast<unsigned long long *>(psync);
  unsigned long long epoch = 0;
  if (tid < static_cast<uint32_t>(n_pes)) {
    fence_release_agent();
    epoch = __hip_atomic_load(own + kEpochSlot, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT) + 1;
    for (uint32_t t = tid; t < static_cast<uint32_t>(n_pes); t += nthr) {
      int peer = pe_start + static_cast<int>(t) * pe_stride;
      unsigned long long *slot =
          reinterpret_cast<unsigned long long *>(translate(psync, my_pe, peer)) + my_idx;
      __hip_atomic_store(slot, epoch, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
    }
    for (uint32_t t = tid; t < static_cast<uint32_t>(n_pes); t += nthr)
      bounded_wait<unsigned long long>(own + t, kWaitGe, epoch);
    fence_acquire_agent();
  }
  __syncthreads();
  // Behind the workgroup barrier every lane that reads the count has read it,
  // so lane 0 may advance it; the next call starts with a workgroup barrier,
  // behind which all lanes see the new count.
  if (tid == 0)
    __hip_atomic_store(own + kEpochSlot, epoch, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
}

}  // namespace detail
}  // namespace rocshmem

#endif
