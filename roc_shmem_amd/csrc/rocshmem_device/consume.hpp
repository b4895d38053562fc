// Consumer pass over the send-queue rings: the part a NIC plays in the
// reference.
//
// Producers (wqe.hpp) execute every operation themselves and leave a 64-byte
// work-queue entry behind.  The consumer pass reads the entries a ring has
// published and not yet retired, in index order, with a decoder written
// independently of the producer's encoder (field positions from the layout
// table at the top of wqe.hpp; reference: SegmentBuilder,
// library/src/gpu_ib/segment_builder.cpp:29-128), and for each entry
//   * checks that it is well-formed: the index field equals the slot's
//     position in the stream, the queue number is the ring's, the remote
//     address lies in a PE slice whose key the entry carries, atomics are
//     8-byte aligned and name a return slot inside the ring's own window; the
//     two entries that move no data (quiet's zero-byte read: READ with DS = 2;
//     fence's flush write: 4 inline bytes, the first one 1, to a PE's flush
//     word under its flush key) are recognised, completed and change nothing;
//   * optionally executes it against a *target arena* laid out like the
//     symmetric heap (RDMA WRITE, inline WRITE, RDMA READ, fetch-add,
//     compare-and-swap, with the old value of an atomic stored to the return
//     slot the entry names), so that replaying the rings onto a copy of the
//     heap taken before the producers ran reproduces what they did;
//   * writes a completion entry for every WQE that requests one (the
//     reference polls these in quiet_internal, queue_pair.cpp:118-191) and
//     retires the entry (SqCounters::consumed), which is what frees the slot
//     when rings run in queue mode.
// One wave owns one ring, so a ring's entries take effect in order, as on a
// reliable-connection queue pair; nothing orders different rings.
//
// Completion entry (64 bytes, the tail of rdma-core's mlx5_cqe64 as the
// reference reads it): bytes 56-59 BE32 queue number, 60-61 BE16 index of the
// completed WQE, 62 signature (0), 63 op_own = opcode 0 (requester
// completion) << 4 | owner bit, the owner bit being bit cq_log_size of the
// completion's own running number.  Bytes 0-55 are zero.  Entries a reader
// has not been given yet hold op_own 0xF0 (invalid opcode).
#ifndef ROCSHMEM_MI355X_DEVICE_CONSUME_HPP
#define ROCSHMEM_MI355X_DEVICE_CONSUME_HPP

#include "copy.hpp"
#include "sync.hpp"
#include "wqe.hpp"

namespace rocshmem {
namespace detail {

struct ConsumeTotals {
  unsigned long long retired;        // entries taken off the rings
  unsigned long long writes;         // RDMA WRITE entries (inline or not)
  unsigned long long reads;          // RDMA READ entries
  unsigned long long atomics;        // fetch-add and compare-and-swap entries
  unsigned long long bytes;          // payload bytes the entries describe
  unsigned long long completions;    // completion entries written
  unsigned long long lost;           // entries overwritten before the pass saw them
  unsigned long long rejected;       // malformed entries (retired, never executed)
  unsigned long long local_skipped;  // well-formed, but the local buffer is outside the heap
};

__device__ __forceinline__ uint64_t lane_u64(uint64_t v, int lane) {
  uint32_t lo = __builtin_amdgcn_readlane(static_cast<uint32_t>(v), lane);
  uint32_t hi = __builtin_amdgcn_readlane(static_cast<uint32_t>(v >> 32), lane);
  return (static_cast<uint64_t>(hi) << 32) | lo;
}

// Offset of [addr, addr+size) from the first slice when the range lies inside
// one PE's heap; ~0 otherwise.  *pe receives the slice.
__device__ __forceinline__ uint64_t heap_offset(uint64_t addr, uint64_t size, int *pe) {
  const uint64_t base = reinterpret_cast<uint64_t>(g_state.heap_base0);
  if (addr < base) return ~0ull;
  const uint64_t rel = addr - base;
  const uint64_t p = rel / g_state.slice_stride;
  const uint64_t off = rel - p * g_state.slice_stride;
  if (p >= static_cast<uint64_t>(g_state.num_pes) || off > g_state.heap_size ||
      size > g_state.heap_size - off)
    return ~0ull;
  *pe = static_cast<int>(p);
  return rel;
}

// What one 64-byte entry says, and whether it is well formed.  `c` is the
// entry's running number in its ring; w0..w7 are its eight 64-bit words.
struct DecodedEntry {
  bool ok, is_atomic, is_write, is_read, inl, wants_completion, no_data;
  uint32_t head, opcode, size;
  uint64_t laddr, roff;
};

__device__ __forceinline__ DecodedEntry decode_entry(const SqRing &ring, uint32_t c,
                                                     uint64_t ret_lo, uint64_t ret_hi, uint64_t w0,
                                                     uint64_t w1, uint64_t w2, uint64_t w3,
                                                     uint64_t w4, uint64_t w5, uint64_t w6,
                                                     uint64_t w7) {
  const uint32_t head = static_cast<uint32_t>(w0);            // bytes 0..3
  const uint32_t opcode = head >> 24;
  const uint32_t index = __builtin_bswap16(static_cast<uint16_t>(head >> 8));
  const uint32_t qpn_ds = static_cast<uint32_t>(w0 >> 32);    // bytes 4..7
  const uint32_t ds = qpn_ds >> 24;
  const uint32_t fm_ce_se = static_cast<uint32_t>(w1 >> 24) & 0xffu;  // byte 11
  const uint64_t raddr = __builtin_bswap64(w2);
  const uint32_t rkey = static_cast<uint32_t>(w3);

  const bool is_atomic = opcode == kOpcodeAtomicFa || opcode == kOpcodeAtomicCs;
  const bool is_write = opcode == kOpcodeRdmaWrite;
  const bool is_read = opcode == kOpcodeRdmaRead;
  const bool zero_byte_read = is_read && ds == 2u;
  bool ok = (head & 0xffu) == 0 && index == (c & 0xffffu) &&
            (qpn_ds & 0xffffffu) == ring.ctrl_qp_sq && (is_atomic || is_write || is_read) &&
            (zero_byte_read || ds == (is_atomic ? 4u : 3u));

  uint32_t size = 0;
  bool inl = false;
  uint64_t laddr = 0;
  if (is_atomic) {
    size = 8;
    ok = ok && (raddr & 7u) == 0 && __builtin_bswap32(static_cast<uint32_t>(w6)) == 8u &&
         static_cast<uint32_t>(w6 >> 32) == ring.atomic_lkey;
    laddr = __builtin_bswap64(w7);
    ok = ok && (laddr & 7u) == 0 && laddr >= ret_lo && laddr < ret_hi;
  } else if (zero_byte_read) {
    size = 0;   // nothing beyond the second segment belongs to the entry
  } else {
    const uint32_t count = __builtin_bswap32(static_cast<uint32_t>(w4));
    inl = (count & 0x80000000u) != 0;
    size = inl ? (count & 0x3ffu) : count;
    if (inl) {
      ok = ok && is_write && size <= 12u;   // what fits the third segment
    } else {
      ok = ok && static_cast<uint32_t>(w4 >> 32) == ring.lkey;
      laddr = __builtin_bswap64(w5);
    }
  }
  int dest_pe = 0;
  uint64_t roff = ~0ull;
  bool flush_write = false;
  if (ok && is_write && inl && raddr >= ring.flush_base &&
      raddr - ring.flush_base < 64ull * static_cast<uint64_t>(g_state.num_pes)) {
    const uint64_t p = (raddr - ring.flush_base) / 64u;
    flush_write = true;
    ok = (raddr - ring.flush_base) % 64u == 0 && size == 4u &&
         (static_cast<uint32_t>(w4 >> 32) & 0xffu) == 1u && rkey == ring.flush_rkey_by_pe[p];
    roff = 0;
  } else {
    roff = ok ? heap_offset(raddr, size, &dest_pe) : ~0ull;
    ok = ok && roff != ~0ull && rkey == ring.rkey_by_pe[dest_pe];
  }
  DecodedEntry d;
  d.no_data = flush_write || zero_byte_read;
  d.ok = ok;
  d.is_atomic = is_atomic;
  d.is_write = is_write;
  d.is_read = is_read;
  d.inl = inl;
  d.wants_completion = fm_ce_se == kCqUpdate;
  d.head = head;
  d.opcode = opcode;
  d.size = size;
  d.laddr = laddr;
  d.roff = roff;
  return d;
}

// Check and complete entries [c, c + todo) of a ring without executing them:
// nothing takes effect, so the order of the entries does not matter and every
// lane takes one of its own, 64 per round (one entry at a time, a pass over
// 1 Mi entries in 1024 rings took 1.45 ms, this way 0.22 ms).  kCoherent: the
// producers' kernel may still be running, possibly on another XCD, so entries
// are read and completions written with agent-scope accesses that bypass this
// XCD's L2; otherwise plain cached accesses.  Adds to `t` (lane-uniform counts;
// t.bytes is left to the caller, who sums `lane_bytes` over the wave).
template <bool kCoherent>
__device__ __forceinline__ void check_range(const SqRing &ring, uint32_t c, uint32_t todo,
                                            uint32_t &cq_producer, ConsumeTotals &t,
                                            unsigned long long &lane_bytes) {
  constexpr int kAux = kCoherent ? 16 /* sc1 */ : 0;
  const uint32_t lane = lane_id();
  const uint32_t mask = ring.max_nwqe - 1;
  const uint64_t ret_lo = ring.atomic_ret_base;
  const uint64_t ret_hi = ring.atomic_ret_base + 8ull * kAtomicRetSlots;
  __amdgpu_buffer_rsrc_t sq_mem = __builtin_amdgcn_make_buffer_rsrc(
      uniform(ring.sq), 0, static_cast<int>(uniform(ring.max_nwqe)) * 64, kRawBufferFlags);
  __amdgpu_buffer_rsrc_t cq_mem = __builtin_amdgcn_make_buffer_rsrc(
      uniform(ring.cq), 0, static_cast<int>(uniform(ring.cq_size)) * 64, kRawBufferFlags);
  for (uint32_t done = 0; done < todo; done += 64) {
    const uint32_t ci = c + done + lane;
    const bool active = done + lane < todo;
    uint64_t w[8] = {0, 0, 0, 0, 0, 0, 0, 0};
    if (active) {
      const uint32_t at = (ci & mask) * 64u;
#pragma unroll
      for (int q = 0; q < 4; ++q) {
        const u32x4 v = __builtin_amdgcn_raw_buffer_load_b128(sq_mem, at + 16u * q, 0, kAux);
        w[2 * q] = (static_cast<uint64_t>(v.y) << 32) | v.x;
        w[2 * q + 1] = (static_cast<uint64_t>(v.w) << 32) | v.z;
      }
    }
    const DecodedEntry d =
        decode_entry(ring, ci, ret_lo, ret_hi, w[0], w[1], w[2], w[3], w[4], w[5], w[6], w[7]);
    const bool good = active && d.ok;
    t.retired += __popcll(__ballot(active));
    t.rejected += __popcll(__ballot(active && !d.ok));
    t.atomics += __popcll(__ballot(good && d.is_atomic));
    t.writes += __popcll(__ballot(good && !d.is_atomic && d.is_write));
    t.reads += __popcll(__ballot(good && !d.is_atomic && !d.is_write));
    if (good) lane_bytes += d.size;
    const bool wants = active && d.wants_completion;
    const uint64_t wanting = __ballot(wants);
    if (wants) {
      const uint32_t number = cq_producer + rank_in_mask(wanting);
      const uint32_t at = (number & (ring.cq_size - 1)) * 64u;
      const uint32_t owner = (number >> ring.cq_log_size) & 1u;
      const u32x4 zero = {0, 0, 0, 0};
      // bytes 56-59 queue number, 60-61 index of the completed entry, 62 signature, 63 op_own
      const u32x4 tail = {0, 0, (ring.ctrl_qp_sq & 0xffffffu) << 8,
                          ((d.head >> 8) & 0xffffu) | (owner << 24)};
      __builtin_amdgcn_raw_buffer_store_b128(zero, cq_mem, at, 0, kAux);
      __builtin_amdgcn_raw_buffer_store_b128(zero, cq_mem, at + 16u, 0, kAux);
      __builtin_amdgcn_raw_buffer_store_b128(zero, cq_mem, at + 32u, 0, kAux);
      __builtin_amdgcn_raw_buffer_store_b128(tail, cq_mem, at + 48u, 0, kAux);
    }
    cq_producer += __popcll(wanting);
    t.completions += __popcll(wanting);
  }
}

__device__ __forceinline__ void add_totals(ConsumeTotals *totals, const ConsumeTotals &t) {
  atomicAdd(&totals->retired, t.retired);
  atomicAdd(&totals->writes, t.writes);
  atomicAdd(&totals->reads, t.reads);
  atomicAdd(&totals->atomics, t.atomics);
  atomicAdd(&totals->bytes, t.bytes);
  atomicAdd(&totals->completions, t.completions);
  atomicAdd(&totals->lost, t.lost);
  atomicAdd(&totals->rejected, t.rejected);
  atomicAdd(&totals->local_skipped, t.local_skipped);
}

__device__ __forceinline__ unsigned long long wave_sum(unsigned long long v) {
#pragma unroll
  for (int off = 32; off > 0; off >>= 1) v += __shfl_xor(v, off);
  return v;
}

// Retire everything ring `ctx` has published.  Called by all 64 lanes of one
// wave, after the producers' kernel has ended.  `target` is the arena
// operations are executed against (nullptr: check and complete only).
__device__ __forceinline__ void consume_ring(const DeviceCtx *ctx, char *target,
                                             ConsumeTotals *totals) {
  const SqRing &ring = ctx->ring;
  SqCounters *cnt = ctx->counters;
  const uint32_t lane = lane_id();
  const uint32_t published =
      uniform(__hip_atomic_load(&cnt->published, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT));
  uint32_t c = uniform(__hip_atomic_load(&cnt->consumed, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT));
  uint32_t cq_producer =
      uniform(__hip_atomic_load(&cnt->cq_producer, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT));
  const uint32_t mask = ring.max_nwqe - 1;
  const uint64_t ret_lo = ring.atomic_ret_base;
  const uint64_t ret_hi = ring.atomic_ret_base + 8ull * kAtomicRetSlots;

  ConsumeTotals t = {};
  if (published - c > ring.max_nwqe) {
    t.lost = published - c - ring.max_nwqe;
    c = published - ring.max_nwqe;
  }

  if (target == nullptr) {
    unsigned long long lane_bytes = 0;
    check_range<false>(ring, c, published - c, cq_producer, t, lane_bytes);
    t.bytes = wave_sum(lane_bytes);
    c = published;
  }

  for (; c != published; ++c) {
    // Eight lanes fetch the entry, everybody gets the words.
    const uint64_t *slot = ring.sq + 8ull * (c & mask);
    uint64_t mine = lane < 8 ? slot[lane] : 0;
    const uint64_t w0 = lane_u64(mine, 0), w1 = lane_u64(mine, 1), w2 = lane_u64(mine, 2),
                   w3 = lane_u64(mine, 3), w4 = lane_u64(mine, 4), w5 = lane_u64(mine, 5),
                   w6 = lane_u64(mine, 6), w7 = lane_u64(mine, 7);
    ++t.retired;

    const DecodedEntry d = decode_entry(ring, c, ret_lo, ret_hi, w0, w1, w2, w3, w4, w5, w6, w7);
    const bool ok = d.ok, is_atomic = d.is_atomic, is_write = d.is_write, inl = d.inl;
    const uint32_t head = d.head, opcode = d.opcode, size = d.size;
    const uint64_t laddr = d.laddr, roff = d.roff;

    if (!ok) {
      ++t.rejected;
    } else {
      t.bytes += size;
      if (is_atomic) {
        ++t.atomics;
      } else if (is_write) {
        ++t.writes;
      } else {
        ++t.reads;
      }
      if (target != nullptr && !d.no_data) {
        char *remote = target + roff;
        if (is_atomic) {
          if (lane == 0) {
            unsigned long long *word = reinterpret_cast<unsigned long long *>(remote);
            const unsigned long long operand = __builtin_bswap64(w4);
            unsigned long long old;
            if (opcode == kOpcodeAtomicFa) {
              old = __hip_atomic_fetch_add(word, operand, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
            } else {
              old = __builtin_bswap64(w5);
              __hip_atomic_compare_exchange_strong(word, &old, operand, __ATOMIC_RELAXED,
                                                   __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
            }
            *reinterpret_cast<unsigned long long *>(laddr) = old;
          }
          // The atomic ran in the L2; drop what this CU's vector cache holds
          // so that a later entry of this ring reads the new value.
          __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "agent");
        } else if (inl) {
          if (lane < size) {
            const uint64_t bits = lane < 4 ? (w4 >> (32 + 8 * lane)) : (w5 >> (8 * (lane - 4)));
            remote[lane] = static_cast<char>(bits);
          }
        } else if (size != 0) {
          int local_pe = 0;
          const uint64_t loff = heap_offset(laddr, size, &local_pe);
          if (loff == ~0ull) {
            ++t.local_skipped;
          } else if (is_write) {
            // The payload is read where the producer left it.
            wave_copy(remote, reinterpret_cast<const void *>(laddr), size);
          } else {
            wave_copy(target + loff, remote, size);
          }
        }
        // Entries of one ring take effect in order: this wave's stores are
        // complete before it touches the next entry.
        __builtin_amdgcn_fence(__ATOMIC_RELEASE, "workgroup");
      }
    }

    if (d.wants_completion) {
      uint64_t *cqe = ring.cq + 8ull * (cq_producer & (ring.cq_size - 1));
      if (lane < 8) {
        uint64_t word = 0;
        if (lane == 7) {
          const uint64_t owner = (cq_producer >> ring.cq_log_size) & 1u;
          word = (static_cast<uint64_t>(ring.ctrl_qp_sq & 0xffffffu) << 8) |
                 (static_cast<uint64_t>((head >> 8) & 0xffffu) << 32) | (owner << 56);
        }
        cqe[lane] = word;
      }
      ++cq_producer;
      ++t.completions;
    }
  }

  if (lane == 0) {
    __builtin_amdgcn_fence(__ATOMIC_RELEASE, "workgroup");
    __hip_atomic_store(&cnt->cq_producer, cq_producer, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
    __hip_atomic_store(&cnt->consumed, c, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
    if (t.retired | t.lost) add_totals(totals, t);
  }
}

// What the host and a live consumer kernel share (host memory the device can
// address).  `stop` is written by the host, the rest by the device.
struct LiveControl {
  uint32_t stop;      // host: every producer has finished, drain and leave
  uint32_t running;   // device: every consumer wave is resident and polling
  uint32_t expired;   // device: a wave left because nothing happened for the idle limit
  uint32_t pad_;
};

// Device-memory words of a live consumer kernel, zeroed before it starts.
struct LiveRelay {
  uint32_t arrived;   // consumer waves that have started
  uint32_t stop;      // the host's stop request, handed on by the wave that reads host memory
};

// A consumer that runs at the same time as the producers: one wave serves
// rings first_ring, first_ring + ring_step, ... and keeps retiring what they
// publish (check, completion entry, `consumed`), which frees the slots the
// producers are waiting for (queue mode).  It leaves when the host has set
// `stop` and one more scan of its rings found nothing new - the host sets the
// flag after the producers' kernels have ended - or when none of its rings
// has moved for `idle_limit_ticks`, so that every wave reaches an exit whatever
// the host does.  Check and complete only: the producers execute their own
// operations.
__device__ __forceinline__ void consume_live(const DeviceCtx *table, uint32_t first_ring,
                                             uint32_t ring_step, uint32_t n_rings,
                                             ConsumeTotals *totals, LiveControl *control,
                                             LiveRelay *relay, uint32_t n_waves,
                                             uint64_t idle_limit_ticks) {
  const uint32_t lane = lane_id();
  // One wave talks to the host; host memory is a bus round trip away.
  const bool liaison = first_ring == 0;
  if (lane == 0) {
    // the last wave to arrive tells the host that all of them are resident
    const uint32_t before =
        __hip_atomic_fetch_add(&relay->arrived, 1u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
    if (before + 1 == n_waves)
      __hip_atomic_store(&control->running, 1u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_SYSTEM);
  }
  ConsumeTotals t = {};
  unsigned long long lane_bytes = 0;
  uint64_t last_progress = wall_clock64();
  bool stop_seen = false;
  uint32_t idle_polls = 0;
  for (;;) {
    bool progress = false;
    for (uint32_t r = first_ring; r < n_rings; r += ring_step) {
      const DeviceCtx *ctx = table + r;
      const SqRing &ring = ctx->ring;
      SqCounters *cnt = ctx->counters;
      const uint32_t published =
          uniform(__hip_atomic_load(&cnt->published, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT));
      uint32_t c =
          uniform(__hip_atomic_load(&cnt->consumed, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT));
      if (published == c) continue;
      progress = true;
      uint32_t cq_producer = uniform(
          __hip_atomic_load(&cnt->cq_producer, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT));
      if (published - c > ring.max_nwqe) {
        // producers whose wait for space gave up overwrote entries nobody had seen
        t.lost += published - c - ring.max_nwqe;
        c = published - ring.max_nwqe;
      }
      check_range<true>(ring, c, published - c, cq_producer, t, lane_bytes);
      // the completion entries are in memory before the indices that announce them move
      __builtin_amdgcn_fence(__ATOMIC_RELEASE, "workgroup");
      if (lane == 0) {
        __hip_atomic_store(&cnt->cq_producer, cq_producer, __ATOMIC_RELAXED,
                           __HIP_MEMORY_SCOPE_AGENT);
        __hip_atomic_store(&cnt->consumed, published, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
      }
    }
    if (progress) {
      last_progress = wall_clock64();
      idle_polls = 0;
      continue;
    }
    if (stop_seen) break;   // a whole scan after the stop request found nothing new
    __builtin_amdgcn_s_sleep(8);
    ++idle_polls;
    uint32_t stop = 0;
    if (lane == 0) {
      // The host's flag is read by the liaison wave only, on every 16th idle
      // scan, and handed on through device memory.
      if (liaison && (idle_polls & 15u) == 0 &&
          __hip_atomic_load(&control->stop, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_SYSTEM) != 0)
        __hip_atomic_store(&relay->stop, 1u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
      stop = __hip_atomic_load(&relay->stop, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
    }
    stop_seen = uniform(stop) != 0;
    if (!stop_seen && (idle_polls & 15u) == 0 &&
        wall_clock64() - last_progress > idle_limit_ticks) {
      if (lane == 0)
        __hip_atomic_store(&control->expired, 1u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_SYSTEM);
      break;
    }
  }
  t.bytes = wave_sum(lane_bytes);
  if (lane == 0 && (t.retired | t.lost)) add_totals(totals, t);
}

}  // namespace detail
}  // namespace rocshmem

#endif
