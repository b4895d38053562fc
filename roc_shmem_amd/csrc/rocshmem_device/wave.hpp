// Wavefront-level building blocks for gfx950 (64 lanes): lane bookkeeping,
// wave-aggregated fetch-add and the neighbour-run message coalescer.
#ifndef ROCSHMEM_MI355X_DEVICE_WAVE_HPP
#define ROCSHMEM_MI355X_DEVICE_WAVE_HPP

#include "state.hpp"

namespace rocshmem {
namespace detail {

__device__ __forceinline__ uint32_t lane_id() {
  return __builtin_amdgcn_mbcnt_hi(~0u, __builtin_amdgcn_mbcnt_lo(~0u, 0u));
}

// Number of set bits of `mask` strictly below this lane (v_mbcnt pair).
__device__ __forceinline__ uint32_t rank_in_mask(uint64_t mask) {
  return __builtin_amdgcn_mbcnt_hi(static_cast<uint32_t>(mask >> 32),
                                   __builtin_amdgcn_mbcnt_lo(static_cast<uint32_t>(mask), 0u));
}

__device__ __forceinline__ uint64_t active_lanes() { return __ballot(1); }

__device__ __forceinline__ uint32_t flat_thread_id() {
  return threadIdx.x + blockDim.x * (threadIdx.y + blockDim.y * threadIdx.z);
}

__device__ __forceinline__ uint32_t flat_block_size() {
  return blockDim.x * blockDim.y * blockDim.z;
}

__device__ __forceinline__ uint32_t first_lane_u32(uint32_t v) {
  return __builtin_amdgcn_readfirstlane(v);
}

__device__ __forceinline__ uint64_t first_lane_u64(uint64_t v) {
  uint32_t lo = __builtin_amdgcn_readfirstlane(static_cast<uint32_t>(v));
  uint32_t hi = __builtin_amdgcn_readfirstlane(static_cast<uint32_t>(v >> 32));
  return (static_cast<uint64_t>(hi) << 32) | lo;
}

// Workgroup- and wave-collective calls receive the same arguments in every
// lane.  Passing such a value through v_readfirstlane tells the compiler so:
// address arithmetic built on it stays in scalar registers and memory
// instructions can take a scalar base, instead of every lane carrying a
// 64-bit address (a context handle read back from LDS, for one, is a vector
// value to the compiler even though all lanes hold the same pointer).
__device__ __forceinline__ uint32_t uniform(uint32_t v) { return first_lane_u32(v); }
__device__ __forceinline__ int uniform(int v) {
  return static_cast<int>(first_lane_u32(static_cast<uint32_t>(v)));
}
__device__ __forceinline__ unsigned long uniform(unsigned long v) {
  return static_cast<unsigned long>(first_lane_u64(static_cast<uint64_t>(v)));
}
__device__ __forceinline__ unsigned long long uniform(unsigned long long v) {
  return static_cast<unsigned long long>(first_lane_u64(static_cast<uint64_t>(v)));
}
template <typename T>
__device__ __forceinline__ T *uniform(T *p) {
  return reinterpret_cast<T *>(first_lane_u64(reinterpret_cast<uint64_t>(p)));
}

// Workgroup barrier without the memory fence of __syncthreads(): the lanes
// meet, their outstanding stores keep draining.  For points where the lanes
// only need to know that all of them got here (every lane has consumed what
// it loaded), not that anybody's stores have landed.  Every lane of the
// workgroup must reach it.
__device__ __forceinline__ void wg_rendezvous() { __asm__ volatile("s_barrier" ::: "memory"); }

// Value of `v` in lane-1 through DPP wave_shr:1.  A lane whose lower
// neighbour is inactive (or lane 0) keeps its own value.
__device__ __forceinline__ uint32_t from_lower_lane(uint32_t v) {
  return __builtin_amdgcn_update_dpp(v, v, 0x138 /* wave_shr:1 */, 0xf, 0xf, false);
}

__device__ __forceinline__ uint64_t from_lower_lane(uint64_t v) {
  uint32_t lo = from_lower_lane(static_cast<uint32_t>(v));
  uint32_t hi = from_lower_lane(static_cast<uint32_t>(v >> 32));
  return (static_cast<uint64_t>(hi) << 32) | lo;
}

// Wave-aggregated fetch-and-add: the lowest active lane performs one atomic
// for the whole wave, every active lane receives a distinct consecutive
// value in ascending lane order.  Same contract as the reference's
// Block::fetch_incr (library/src/containers/share_strategy.hpp:70-83) without
// its 64-step broadcast_up loop: the base travels through v_readfirstlane
// and the per-lane offset is one v_mbcnt pair.
template <typename U>
__device__ __forceinline__ U wave_fetch_incr(U *counter, uint64_t *mask_out = nullptr) {
  uint64_t mask = active_lanes();
  uint32_t n = __popcll(mask);
  uint32_t rank = rank_in_mask(mask);
  U base = 0;
  if (rank == 0) {
    base = __hip_atomic_fetch_add(counter, static_cast<U>(n), __ATOMIC_RELAXED,
                                  __HIP_MEMORY_SCOPE_AGENT);
  }
  if constexpr (sizeof(U) == 8) {
    base = static_cast<U>(first_lane_u64(static_cast<uint64_t>(base)));
  } else {
    base = static_cast<U>(first_lane_u32(static_cast<uint32_t>(base)));
  }
  if (mask_out) *mask_out = mask;
  return base + static_cast<U>(rank);
}

// Result of the coalescer for one lane.
struct CoalesceResult {
  bool must_send;   // this lane posts a message (it is the head of a run)
  uint64_t size;    // bytes the posted message covers (own size * run length)
};

// Merge lane-contiguous messages.  Lane l is absorbed by lane l-1 iff lane
// l-1 is active, both carry the same size and PE, and both source and
// destination of l start exactly where those of l-1 end; lane 0 is never
// absorbed.  A sending lane's size grows by one `size` per absorbed lane in
// the unbroken run directly above it.  (Reference: WfCoalOn::coalesce,
// library/src/wf_coal_policy.cpp:57-172; like the reference, the size is
// compared as a 32-bit quantity.)
__device__ __forceinline__ CoalesceResult wave_coalesce(int pe, uint64_t src, uint64_t dst,
                                                        uint64_t size) {
  uint64_t lower_src = from_lower_lane(src);
  uint64_t lower_dst = from_lower_lane(dst);
  uint32_t lower_pe = from_lower_lane(static_cast<uint32_t>(pe));
  uint32_t lower_size = from_lower_lane(static_cast<uint32_t>(size));

  uint64_t mask = active_lanes();
  uint32_t lane = lane_id();
  bool lower_active = lane != 0 && ((mask >> (lane - 1)) & 1ull);

  bool absorbed = lower_active && lower_size == static_cast<uint32_t>(size) &&
                  lower_src + size == src && lower_dst + size == dst &&
                  lower_pe == static_cast<uint32_t>(pe);

  uint64_t absorbed_mask = __ballot(absorbed);

  CoalesceResult r;
  r.must_send = !absorbed;
  r.size = size;
  if (!absorbed) {
    // Count the unbroken run of absorbed lanes directly above this one.
    uint64_t above = (lane == 63) ? 0ull : (absorbed_mask >> (lane + 1));
    uint32_t run = __builtin_ctzll(~above);  // `above` has at most 63 bits, so ~above != 0
    r.size = size * (1ull + run);
  }
  return r;
}

}  // namespace detail
}  // namespace rocshmem

#endif
