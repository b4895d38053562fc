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
//     8-byte aligned and name a return slot inside the ring's own window;
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

// Retire everything ring `ctx` has published.  Called by all 64 lanes of one
// wave.  `target` is the arena operations are executed against (nullptr: check
// and complete only).
// What one 64-byte entry says, and whether it is well formed.  `c` is the
// entry's running number in its ring; w0..w7 are its eight 64-bit words.
struct DecodedEntry {
  bool ok, is_atomic, is_write, is_read, inl, wants_completion;
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
  bool ok = (head & 0xffu) == 0 && index == (c & 0xffffu) &&
            (qpn_ds & 0xffffffu) == ring.ctrl_qp_sq && (is_atomic || is_write || is_read) &&
            ds == (is_atomic ? 4u : 3u);

  uint32_t size = 0;
  bool inl = false;
  uint64_t laddr = 0;
  if (is_atomic) {
    size = 8;
    ok = ok && (raddr & 7u) == 0 && __builtin_bswap32(static_cast<uint32_t>(w6)) == 8u &&
         static_cast<uint32_t>(w6 >> 32) == ring.atomic_lkey;
    laddr = __builtin_bswap64(w7);
    ok = ok && (laddr & 7u) == 0 && laddr >= ret_lo && laddr < ret_hi;
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
  const uint64_t roff = ok ? heap_offset(raddr, size, &dest_pe) : ~0ull;
  ok = ok && roff != ~0ull && rkey == ring.rkey_by_pe[dest_pe];
  DecodedEntry d;
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
    // Check and complete only: nothing takes effect, so the order of the entries
    // does not matter and every lane takes one of its own, 64 per round (one
    // entry at a time, a pass over 1 Mi entries in 1024 rings took 1.45 ms).
    typedef uint64_t u64x2 __attribute__((ext_vector_type(2)));
    const uint32_t todo = published - c;
    unsigned long long lane_bytes = 0;
    for (uint32_t done = 0; done < todo; done += 64) {
      const uint32_t ci = c + done + lane;
      const bool active = done + lane < todo;
      uint64_t w[8] = {0, 0, 0, 0, 0, 0, 0, 0};
      if (active) {
        const u64x2 *slot = reinterpret_cast<const u64x2 *>(ring.sq + 8ull * (ci & mask));
#pragma unroll
        for (int q = 0; q < 4; ++q) {
          const u64x2 v = slot[q];
          w[2 * q] = v.x;
          w[2 * q + 1] = v.y;
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
        u64x2 *cqe = reinterpret_cast<u64x2 *>(ring.cq + 8ull * (number & (ring.cq_size - 1)));
        const uint64_t owner = (number >> ring.cq_log_size) & 1u;
        const uint64_t last = (static_cast<uint64_t>(ring.ctrl_qp_sq & 0xffffffu) << 8) |
                              (static_cast<uint64_t>((d.head >> 8) & 0xffffu) << 32) | (owner << 56);
        cqe[0] = u64x2{0, 0};
        cqe[1] = u64x2{0, 0};
        cqe[2] = u64x2{0, 0};
        cqe[3] = u64x2{0, last};
      }
      cq_producer += __popcll(wanting);
      t.completions += __popcll(wanting);
    }
#pragma unroll
    for (int off = 32; off > 0; off >>= 1) lane_bytes += __shfl_xor(lane_bytes, off);
    t.bytes = lane_bytes;
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
      if (target != nullptr) {
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
    if (t.retired | t.lost) {
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
  }
}

}  // namespace detail
}  // namespace rocshmem

#endif
