// Workgroup-collective data movement between the slices of an active set:
// broadcast, alltoall, fcollect, and the barrier/sync family.
//
// Each collective is entered by one workgroup per member PE with identical
// arguments (reference: GPUIBContext::broadcast / alltoall_broadcast /
// fcollect_broadcast, library/src/gpu_ib/context_ib_tmpl_device.hpp:455-558,
// 845-876; internal_sync, context_ib_device_coll.cpp:30-89).  Because every
// slice is addressable, the work of one call is split over its member
// workgroups by byte range rather than by peer: member k moves the k-th share
// of the payload for all peers, reading each source byte once.  Every call is
// bracketed by two flag barriers on distinct halves of the pSync slice, which
// also makes back-to-back calls on the same pSync safe.
//
// A `shard`/`nshards` pair restricts a call to one equal part of every block,
// so that several workgroups of a PE (each with its own pSync slice) can
// share one large collective.
#ifndef ROCSHMEM_MI355X_DEVICE_COLL_HPP
#define ROCSHMEM_MI355X_DEVICE_COLL_HPP

#include "copy.hpp"
#include "reduce.hpp"
#include "sync.hpp"

namespace rocshmem {
namespace detail {

// Split [0, n) into `parts` contiguous shares whose interior boundaries are
// multiples of `quantum`; returns share `idx`.
__device__ __forceinline__ void split_range(size_t n, int parts, int idx, size_t quantum,
                                            size_t &begin, size_t &end) {
  size_t share = (n + parts - 1) / parts;
  share = (share + quantum - 1) / quantum * quantum;
  begin = share * static_cast<size_t>(idx);
  end = begin + share;
  if (begin > n) begin = n;
  if (end > n) end = n;
}

// Vector body of wg_copy_to_members: passes first_pass, first_pass +
// pass_step, ... of `body` bytes (a multiple of 16) from `src` to the `ndst`
// destinations dst0 + m * member_step, m counting past `skip_at`.  `dst0` is
// 16-byte aligned.  kBufferLoads: `src` is 4-byte aligned and read through a
// buffer descriptor; otherwise it is read with per-lane unaligned vector loads.
template <bool kBufferLoads, int U = kStreamUnroll>
__device__ __forceinline__ void copy_passes_to_members(char *dst0, const char *src, size_t body,
                                                       int64_t member_step, int ndst, int skip_at,
                                                       uint32_t tid, uint32_t nthr,
                                                       size_t first_pass, size_t pass_step) {
  constexpr int kNt = 2;
  // written through to memory, and waited for below, so that the collective's closing
  // barrier need not write this XCD's L2 back (wg_flag_barrier, written_through)
  constexpr int kStore = kNt | kWriteThrough;
  const uint32_t lane_off = tid * 16u;
  const uint32_t access_bytes = nthr * 16u;
  const uint32_t pass_bytes = access_bytes * U;
  const size_t step_bytes = pass_step * pass_bytes;
  const size_t first_byte = first_pass * pass_bytes;
  // A short first pass is the only one; a wave whose every lane lies past its
  // end leaves (its clipped accesses would still cost their issue slots: a
  // 4 KiB broadcast by one workgroup of 1024 lanes took 13.4 us, now 7.1).
  if (first_byte < body && body - first_byte < pass_bytes &&
      uniform((tid & ~63u) * 16u) >= body - first_byte)
    return;
  for (size_t b = first_byte; b < body; b += step_bytes) {
    const size_t left = body - b;
    const int valid = static_cast<int>(left < pass_bytes ? left : pass_bytes);
    u32x4 v[U];
    if constexpr (kBufferLoads) {
      __amdgpu_buffer_rsrc_t rs = uniform_rsrc(src + b, valid);
#pragma unroll
      for (int u = 0; u < U; ++u)
        v[u] = __builtin_amdgcn_raw_buffer_load_b128(rs, lane_off, u * access_bytes, kNt);
    } else if (static_cast<uint32_t>(valid) == pass_bytes) {
#pragma unroll
      for (int u = 0; u < U; ++u)
        v[u] = __builtin_nontemporal_load(
            reinterpret_cast<const u32x4_a1 *>(src + b + u * access_bytes + lane_off));
    } else {
#pragma unroll
      for (int u = 0; u < U; ++u) {
        const uint32_t off = u * access_bytes + lane_off;  // valid is a multiple of 16
        v[u] = u32x4{0, 0, 0, 0};
        if (off < static_cast<uint32_t>(valid))
          v[u] = __builtin_nontemporal_load(reinterpret_cast<const u32x4_a1 *>(src + b + off));
      }
    }
    // Destination i of the ndst that are written, without a branch around the
    // skipped member: a conditional `continue` in this loop cost a sixth of
    // the broadcast's bandwidth.
    for (int i = 0; i < ndst; ++i) {
      const int m = i + (i >= skip_at ? 1 : 0);
      __amdgpu_buffer_rsrc_t rd = uniform_rsrc(dst0 + m * member_step + b, valid);
#pragma unroll
      for (int u = 0; u < U; ++u)
        __builtin_amdgcn_raw_buffer_store_b128(v[u], rd, lane_off, u * access_bytes, kStore);
    }
  }
  __builtin_amdgcn_s_waitcnt(0);
}

// Copy `n` bytes from `src` into the same symmetric address `dst_mine` of
// every member for which `skip_idx != member index`.  Every source vector is
// loaded once and stored to each destination (raw-buffer addressing as in
// stream_copy_uniform); payloads under 256 bytes are copied per destination.
// Arguments are workgroup-uniform.
//
// `first_pass` / `pass_step` (vector path only; the caller checks alignment
// and size first) restrict the call to passes first_pass, first_pass +
// pass_step, ... of the vector body, and `edges` says whether this caller
// moves the unaligned head and tail bytes.  Returns whether everything this
// caller stored was written through to memory and waited for (the vector
// body is; head, tail and payloads under 256 bytes are plain stores).
__device__ __forceinline__ bool wg_copy_to_members(char *dst_mine, const char *src, size_t n,
                                                   const ActiveSet &as, int my_pe, int skip_idx,
                                                   uint32_t tid, uint32_t nthr,
                                                   size_t first_pass = 0, size_t pass_step = 1,
                                                   bool edges = true) {
  if (n == 0) return true;
  const int64_t stride = static_cast<int64_t>(g_state.slice_stride);
  char *dst0 = dst_mine + (static_cast<int64_t>(as.pe_start) - my_pe) * stride;
  const int64_t member_step = stride * as.pe_stride;
  // The vector path stores 16-byte aligned; it loads through a buffer
  // descriptor when the source then sits at a 4-byte boundary and with
  // per-lane unaligned vector loads otherwise.
  const bool coaligned =
      ((reinterpret_cast<uintptr_t>(dst_mine) ^ reinterpret_cast<uintptr_t>(src)) & 3u) == 0;
  if (n < 256) {
    for (int m = 0; m < as.size; ++m) {
      if (m == skip_idx) continue;
      group_copy_uniform(dst0 + m * member_step, src, n, tid, nthr);
    }
    return false;
  }
  const size_t head = stream_head(dst_mine, n);
  const size_t body = (n - head) & ~static_cast<size_t>(15);
  const size_t tail = n - head - body;
  for (size_t t = tid; edges && t < head + tail; t += nthr) {
    size_t off = t < head ? t : body + t;  // head bytes, then the bytes after the vectors
    char b = src[off];
    for (int m = 0; m < as.size; ++m)
      if (m != skip_idx) dst0[m * member_step + off] = b;
  }
  const bool skips = skip_idx >= 0 && skip_idx < as.size;
  const int ndst = as.size - (skips ? 1 : 0);
  const int skip_at = skips ? skip_idx : as.size;
  // One loop per way of loading, so that neither carries the other's registers and branches.
  if (coaligned && body <= 2 * static_cast<size_t>(nthr) * 16u) {
    // What two accesses of the group cover does not issue eight per destination.
    copy_passes_to_members<true, 2>(dst0 + head, src + head, body, member_step, ndst, skip_at, tid,
                                    nthr, first_pass, pass_step);
  } else if (coaligned) {
    copy_passes_to_members<true>(dst0 + head, src + head, body, member_step, ndst, skip_at, tid, nthr,
                                 first_pass, pass_step);
  } else {
    copy_passes_to_members<false>(dst0 + head, src + head, body, member_step, ndst, skip_at, tid, nthr,
                                  first_pass, pass_step);
  }
  return !(edges && head + tail != 0);
}

// Broadcast `nbytes` from the root member's `source` to every other member's
// `dest`; the root's `dest` is not written (reference: internal_put_broadcast
// / internal_get_broadcast, context_ib_tmpl_device.hpp:455-478).  `root_idx`
// is the root's ordinal within the active set.
//
// `shard` / `nshards`: several workgroups of every member share the call.  A
// large payload is dealt to them pass by pass (the
// workgroups running at one moment then write one compact window of every
// destination: 1 -> 15 broadcast of 64 MiB on MI355X, 5.8 TB/s with 8
// workgroups of 1024 lanes per PE against 5.6 TB/s with a contiguous range
// per workgroup); anything else is cut into contiguous ranges.
__device__ __forceinline__ void wg_broadcast_bytes(int my_pe, void *dest, const void *source,
                                                   size_t nbytes, int root_idx, int pe_start,
                                                   int pe_stride, int pe_size, long *psync,
                                                   int shard = 0, int nshards = 1) {
  my_pe = uniform(my_pe);
  shard = uniform(shard);
  nshards = uniform(nshards);
  dest = own(uniform(dest), my_pe);       // symmetric arguments: the caller's own copies
  source = own(uniform(source), my_pe);
  nbytes = uniform(nbytes);
  root_idx = uniform(root_idx);
  pe_start = uniform(pe_start);
  pe_stride = uniform(pe_stride);
  pe_size = uniform(pe_size);
  psync = own(uniform(psync), my_pe);
  if (nbytes == 0) return;
  if (pe_size > kMaxPes || pe_size <= 0 || root_idx < 0 || root_idx >= pe_size || nshards <= 0 ||
      shard < 0 || shard >= nshards) {
    status_raise(kStatusBadArgument);
    return;
  }
  const ActiveSet as{pe_start, pe_stride, pe_size};
  const int my_idx = member_index(my_pe - pe_start, pe_stride);
  const uint32_t tid = flat_thread_id();
  const uint32_t nthr = flat_block_size();
  const size_t parts = static_cast<size_t>(pe_size) * nshards;
  const size_t part = static_cast<size_t>(shard) * pe_size + my_idx;

  wg_flag_barrier(psync, 0, my_pe, my_idx, pe_start, pe_stride, pe_size);

  const char *root_src = translate(static_cast<const char *>(source), my_pe, as.pe_at(root_idx));
  const size_t pass_bytes = static_cast<size_t>(nthr) * 16u * kStreamUnroll;
  bool through;
  if (nbytes >= 2 * parts * pass_bytes) {
    through = wg_copy_to_members(static_cast<char *>(dest), root_src, nbytes, as, my_pe, root_idx, tid,
                                 nthr, part, parts, part == 0);
  } else {
    size_t b, e;
    split_range(nbytes, static_cast<int>(parts), static_cast<int>(part), 256, b, e);
    through = wg_copy_to_members(static_cast<char *>(dest) + b, root_src + b, e - b, as, my_pe,
                                 root_idx, tid, nthr);
  }

  wg_flag_barrier(psync, 1, my_pe, my_idx, pe_start, pe_stride, pe_size, 0, through);
}

// Alltoall block exchange: member i's block j goes to member j's block i,
// self block included (reference: alltoall_broadcast,
// context_ib_tmpl_device.hpp:528-558).  `block_bytes` is the size of one
// block; `nshards` workgroups of every member share the call, each moving
// one contiguous range of every block (dealing the blocks pass by pass was
// measured slower here: 5.9 against 6.1 TB/s for 16 x 16 blocks of 4 MiB).
__device__ __forceinline__ void wg_alltoall_bytes(int my_pe, void *dest, const void *source,
                                                  size_t block_bytes, int shard, int nshards,
                                                  int pe_start, int pe_stride, int pe_size,
                                                  long *psync) {
  my_pe = uniform(my_pe);
  dest = own(uniform(dest), my_pe);       // symmetric arguments: the caller's own copies
  source = own(uniform(source), my_pe);
  block_bytes = uniform(block_bytes);
  shard = uniform(shard);
  nshards = uniform(nshards);
  pe_start = uniform(pe_start);
  pe_stride = uniform(pe_stride);
  pe_size = uniform(pe_size);
  psync = own(uniform(psync), my_pe);
  if (block_bytes == 0) return;
  if (pe_size > kMaxPes || pe_size <= 0 || nshards <= 0 || shard < 0 || shard >= nshards) {
    status_raise(kStatusBadArgument);
    return;
  }
  const ActiveSet as{pe_start, pe_stride, pe_size};
  const int my_idx = member_index(my_pe - pe_start, pe_stride);
  const uint32_t tid = flat_thread_id();
  const uint32_t nthr = flat_block_size();

  wg_flag_barrier(psync, 0, my_pe, my_idx, pe_start, pe_stride, pe_size);

  char *dst_mine = static_cast<char *>(dest) + static_cast<size_t>(my_idx) * block_bytes;
  const char *src = static_cast<const char *>(source);
  size_t b, e;
  split_range(block_bytes, nshards, shard, 256, b, e);
  const size_t len = e - b;
  const uintptr_t alike = reinterpret_cast<uintptr_t>(dst_mine + b) |
                          reinterpret_cast<uintptr_t>(src + b) | block_bytes | len;
  bool through = false;
  if (len >= kNonTemporalBytes && (alike & 15u) == 0 && stream_head(dst_mine + b, len) == 0) {
    // Large ranges between aligned blocks: the streaming loop itself, its stores written
    // through and waited for, so that the closing barrier skips the L2 write-back.
    // One schedule across the blocks (Pacer), when the caller has set a rate for copies (off by
    // default), the grid fills the chip and every workgroup has passes enough for the slots'
    // start to vanish.  16 PEs x 64 MiB at 67000: 6243-6289 -> 6440-6455 GB/s; other shapes lose
    // (8 PEs x 128 MiB by 32 x 1024 lanes per PE: 6218 -> 5653), hence the caller's choice.
    Pacer pacer{0u, 0u};
    const size_t pass_bytes = static_cast<size_t>(nthr) * 16u * kStreamUnroll;
    if (g_state.pace_copy_bytes_per_tick != 0 && len * pe_size >= 16 * pass_bytes && grid_is_resident())
      pacer = make_pacer(g_state.pace_copy_bytes_per_tick, grid_workgroups() * pass_bytes);
    for (int jj = 0; jj < pe_size; ++jj) {
      int j = my_idx + jj;      // start at the own index: concurrent members hit different slices
      if (j >= pe_size) j -= pe_size;
      stream_copy_paced<2 /* nt */ | kWriteThrough, kStreamUnroll>(
          translate(dst_mine, my_pe, as.pe_at(j)) + b, src + static_cast<size_t>(j) * block_bytes + b,
          len, tid, nthr, 0, 1, pacer);
    }
    __builtin_amdgcn_s_waitcnt(0);
    through = true;
  } else if (len != 0 && len <= static_cast<size_t>(nthr) * 16u && (alike & 15u) == 0) {
    // Blocks that one access of the workgroup covers: one copy after the other
    // would be a chain of pe_size load latencies; here eight blocks' loads are in
    // flight before the first store (4 KiB or 32 KiB among 8 PEs: 9.2 -> 6.8 us per call).
    constexpr int kBlocks = 8;
    const uint32_t lane_off = tid * 16u;
    if (uniform((tid & ~63u) * 16u) < len) {
      for (int j0 = 0; j0 < pe_size; j0 += kBlocks) {
        u32x4 v[kBlocks];
#pragma unroll
        for (int c = 0; c < kBlocks; ++c) {
          if (j0 + c < pe_size) {
            int j = my_idx + j0 + c;
            if (j >= pe_size) j -= pe_size;
            __amdgpu_buffer_rsrc_t rs =
                uniform_rsrc(src + static_cast<size_t>(j) * block_bytes + b, static_cast<int>(len));
            v[c] = __builtin_amdgcn_raw_buffer_load_b128(rs, lane_off, 0, 0);
          }
        }
#pragma unroll
        for (int c = 0; c < kBlocks; ++c) {
          if (j0 + c < pe_size) {
            int j = my_idx + j0 + c;
            if (j >= pe_size) j -= pe_size;
            __amdgpu_buffer_rsrc_t rd =
                uniform_rsrc(translate(dst_mine, my_pe, as.pe_at(j)) + b, static_cast<int>(len));
            __builtin_amdgcn_raw_buffer_store_b128(v[c], rd, lane_off, 0, 0);
          }
        }
      }
    }
  } else {
    for (int jj = 0; jj < pe_size; ++jj) {
      // Start at the own index so that concurrent members hit different slices.
      int j = my_idx + jj;
      if (j >= pe_size) j -= pe_size;
      group_copy_uniform(translate(dst_mine, my_pe, as.pe_at(j)) + b,
                         src + static_cast<size_t>(j) * block_bytes + b, len, tid, nthr);
    }
  }

  wg_flag_barrier(psync, 1, my_pe, my_idx, pe_start, pe_stride, pe_size, 0, through);
}

// Fcollect: member i's `block_bytes` land in block i of every member's dest
// (reference: fcollect_broadcast, context_ib_tmpl_device.hpp:845-876).
__device__ __forceinline__ void wg_fcollect_bytes(int my_pe, void *dest, const void *source,
                                                  size_t block_bytes, int shard, int nshards,
                                                  int pe_start, int pe_stride, int pe_size,
                                                  long *psync) {
  my_pe = uniform(my_pe);
  dest = own(uniform(dest), my_pe);       // symmetric arguments: the caller's own copies
  source = own(uniform(source), my_pe);
  block_bytes = uniform(block_bytes);
  shard = uniform(shard);
  nshards = uniform(nshards);
  pe_start = uniform(pe_start);
  pe_stride = uniform(pe_stride);
  pe_size = uniform(pe_size);
  psync = own(uniform(psync), my_pe);
  if (block_bytes == 0) return;
  if (pe_size > kMaxPes || pe_size <= 0 || nshards <= 0 || shard < 0 || shard >= nshards) {
    status_raise(kStatusBadArgument);
    return;
  }
  const ActiveSet as{pe_start, pe_stride, pe_size};
  const int my_idx = member_index(my_pe - pe_start, pe_stride);
  const uint32_t tid = flat_thread_id();
  const uint32_t nthr = flat_block_size();

  wg_flag_barrier(psync, 0, my_pe, my_idx, pe_start, pe_stride, pe_size);

  // The member's own block goes to block my_idx of everybody; the member's
  // workgroups take one contiguous range of it each (dealing a 4 MiB block
  // pass by pass was measured slower: 5.4 against 5.9 TB/s).
  char *dst_mine = static_cast<char *>(dest) + static_cast<size_t>(my_idx) * block_bytes;
  const char *src = static_cast<const char *>(source);
  size_t b, e;
  split_range(block_bytes, nshards, shard, 256, b, e);
  const bool through = wg_copy_to_members(dst_mine + b, src + b, e - b, as, my_pe, -1, tid, nthr);

  wg_flag_barrier(psync, 1, my_pe, my_idx, pe_start, pe_stride, pe_size, 0, through);
}

// Barrier among the member workgroups (reference: internal_sync,
// context_ib_device_coll.cpp:67-89).  `psync` is a slice of the team's barrier
// pool, which only this routine uses.
__device__ __forceinline__ void wg_sync_members(int my_pe, int pe_start, int pe_stride,
                                                int pe_size, long *psync) {
  my_pe = uniform(my_pe);
  pe_start = uniform(pe_start);
  pe_stride = uniform(pe_stride);
  pe_size = uniform(pe_size);
  psync = own(uniform(psync), my_pe);
  if (pe_size > kMaxPes || pe_size <= 0) {
    status_raise(kStatusBadArgument);
    return;
  }
  const int my_idx = member_index(my_pe - pe_start, pe_stride);
  wg_epoch_barrier(psync, my_pe, my_idx, pe_start, pe_stride, pe_size);
}

}  // namespace detail
}  // namespace rocshmem

#endif
