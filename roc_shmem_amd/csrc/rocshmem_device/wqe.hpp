// GPU-built 64-byte work-queue entries in a send-queue ring.
//
// Byte layout, opcodes and field encodings follow what the reference writes
// for the RC transport: SegmentBuilder (library/src/gpu_ib/segment_builder.cpp:
// 29-128), QueuePair::update_posted_wqe_generic (queue_pair.cpp:205-273), the
// completion flag and doorbell of the multi-thread post policy
// (thread_policy.cpp:170-216, queue_pair.cpp:67-78) and the byte swaps of
// endian.cpp:27-77.  A WQE is four 16-byte segments:
//   0 control   : 00 | idx_hi idx_lo | opcode | qpn[3] | DS | sig | 00 00 | fm_ce_se | imm[4]
//   1 remote    : BE64 raddr | rkey | 00000000
//   2 data      : BE32 byte_count | lkey | BE64 laddr          (size > 8, or READ)
//     inline    : BE32 (size | 0x80000000) | payload[size]      (WRITE, size <= 8)
//     atomic    : BE64 swap_add | BE64 compare
//   3 atomic only: BE32 8 | atomic_lkey | BE64 &atomic_ret[pos]
// Bytes the reference never writes (inline padding, segment 3 of non-atomic
// entries) are left as the ring holds them.  Two entries move no data: the
// zero-byte read that quiet posts before it polls (QueuePair::zero_b_rd,
// queue_pair.cpp:318-325; thread_policy.cpp:35-108): opcode READ, DS = 2, remote
// address = the destination's heap base, third segment not written; and the
// flush write that fence posts (QueuePair::fence, queue_pair.cpp:376-384): a
// WRITE of size 0 becomes a 4-byte inline write (queue_pair.cpp:230-233) whose
// first payload byte is 1 (segment_builder.cpp:110-116), addressed to the
// destination's flush word under the flush key.
//
// What differs from the reference is how lanes get their slots.  The
// reference serialises waves with a per-queue spin lock and lets every lane
// call atomicAdd (thread_policy.cpp:218-323).  Here one wave reserves all the
// slots its posting lanes need with a single atomic (ballot + v_mbcnt +
// v_readlane), every posting lane assembles its entry in registers and
// writes it with 16-byte stores, and completed ranges are published in index
// order through SqCounters::published before the doorbell record moves.  A
// slot is reused only after its previous occupant has been published
// (the reference's waitSQSpace, queue_pair.cpp:400-415, plays this role).
//
// No device-wide release fence sits on this path.  An agent-scope release on a
// part with one L2 per XCD writes a whole L2 back; two of them per post held
// 10 M eight-byte puts at 1.0 G ops/s, against 12.9 G ops/s with the ordering
// used here: a wave waits for its own stores (s_waitcnt) and hands the queue
// on through agent-scope atomics on `published` and the mailbox words.  That
// orders everything producers need among themselves.  Ring bytes are complete
// in memory when the kernel ends or after roc_shmem_ctx_quiet; see wave_post
// at the end of this file for rings that several workgroups share.
#ifndef ROCSHMEM_MI355X_DEVICE_WQE_HPP
#define ROCSHMEM_MI355X_DEVICE_WQE_HPP

#include "copy.hpp"
#include "sync.hpp"
#include "wave.hpp"

namespace rocshmem {
namespace detail {

constexpr uint8_t kOpcodeRdmaWrite = 0x08;
constexpr uint8_t kOpcodeRdmaRead = 0x10;
constexpr uint8_t kOpcodeAtomicCs = 0x11;
constexpr uint8_t kOpcodeAtomicFa = 0x12;
constexpr uint32_t kInlineThreshold = 8;  // reference: queue_pair.hpp:324
constexpr uint8_t kCqUpdate = 8;          // fm_ce_se value that requests a CQE

__device__ __forceinline__ uint32_t be32(uint32_t v) { return __builtin_bswap32(v); }

// A 64-bit value stored big-endian occupies two little-endian 32-bit words:
// first the swapped high half, then the swapped low half.
__device__ __forceinline__ uint32_t be64_first(uint64_t v) {
  return __builtin_bswap32(static_cast<uint32_t>(v >> 32));
}
__device__ __forceinline__ uint32_t be64_second(uint64_t v) {
  return __builtin_bswap32(static_cast<uint32_t>(v));
}

enum WqeForm : uint8_t { kWqeData = 0, kWqeZeroByteRead = 1, kWqeFlushWrite = 2 };

struct WqeRequest {
  uint8_t opcode;
  uint32_t size;         // bytes the entry covers (already merged by the coalescer)
  uint64_t raddr;        // target address in the destination slice
  uint64_t laddr;        // local buffer address (ignored for atomics)
  uint64_t atomic_data;  // add / swap operand
  uint64_t atomic_cmp;   // compare operand (0 for fetch-add)
  uint64_t inline_data;  // payload bytes, little-endian packed, when size <= 8 and WRITE
  int pe;
  WqeForm form = kWqeData;
};

// The completion reader's two counters as the one 64-bit word they share (SqCounters).
__device__ __forceinline__ unsigned long long *reader_word(SqCounters *cnt) {
  return reinterpret_cast<unsigned long long *>(&cnt->cq_consumer);
}

// Post one entry per lane that passes `sends == true`.  Called by every lane
// that is active at the call site (senders and absorbed lanes alike).
template <int kRingPolicy>
__device__ __forceinline__ void wave_post_with(DeviceCtx *ctx, bool sends, const WqeRequest &rq) {
  const uint64_t send_mask = __ballot(sends);
  if (send_mask == 0) return;
  const uint32_t n = __popcll(send_mask);
  const uint32_t rank = rank_in_mask(send_mask);
  const uint32_t first = __builtin_ctzll(send_mask);
  const bool is_atomic = rq.opcode == kOpcodeAtomicFa || rq.opcode == kOpcodeAtomicCs;
  const uint64_t atomic_mask = __ballot(sends && is_atomic);

  SqCounters *cnt = ctx->counters;
  const uint32_t ring_size = ctx->ring.max_nwqe;
  uint32_t base = 0, abase = 0;
  if (sends && rank == 0) {
    // Issued together so their latencies overlap: the index that frees slots
    // (only ever grows, so an early read is conservative) and the reservation.
    // Slots are freed by publication when the ring is a log and by the
    // consumer pass when it is a queue.
    uint32_t *freed = g_state.sq_queue_mode ? &cnt->consumed : &cnt->published;
    uint32_t seen = __hip_atomic_load(freed, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
    base = __hip_atomic_fetch_add(&cnt->sq_counter, n, __ATOMIC_RELAXED,
                                  __HIP_MEMORY_SCOPE_AGENT);
    if (atomic_mask) {
      abase = __hip_atomic_fetch_add(&cnt->atomic_counter,
                                     static_cast<uint32_t>(__popcll(atomic_mask)),
                                     __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
    }
    // Queue space: entry c may be written once entry c - ring_size is freed.
    if (static_cast<int32_t>(base + n - seen - ring_size) > 0) {
      const uint32_t need = base + n - ring_size;
      uint64_t start = wall_clock64();
      uint32_t spins = 0;
      while (static_cast<int32_t>(
                 need - __hip_atomic_load(freed, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT)) >
             0) {
        __builtin_amdgcn_s_sleep(1);
        if ((++spins & 63u) == 0 &&
            (status_failed() || wall_clock64() - start > g_state.wait_limit_ticks)) {
          status_raise(kStatusWaitTimeout);
          break;
        }
      }
    }
  }
  base = __builtin_amdgcn_readlane(base, first);
  abase = __builtin_amdgcn_readlane(abase, first);

  const SqRing &ring = ctx->ring;
  const uint32_t my_counter = base + rank;
  const bool last = sends && rank == n - 1;

  constexpr int kThrough = kRingPolicy;
  __amdgpu_buffer_rsrc_t ring_mem = __builtin_amdgcn_make_buffer_rsrc(
      uniform(ring.sq), 0, static_cast<int>(uniform(ring.max_nwqe)) * 64, kRawBufferFlags);

  // A completion is requested by the entry that closes the wave's post (the
  // multi-thread policy, thread_policy.cpp:170-216) and by the entry in slot
  // max_nwqe - 2 of every lap (queue_pair.cpp:80-101: the completion queue
  // must not starve however the posts fall).
  const uint32_t slot = my_counter & (ring.max_nwqe - 1);
  const bool wants_cqe = sends && (last || slot == ring.max_nwqe - 2u);
  const uint32_t n_cqe = __popcll(__ballot(wants_cqe));

  uint32_t first8_lo = 0, first8_hi = 0;
  if (sends) {
    const uint32_t at = slot * 64u;   // byte offset of the entry in the ring
    const uint16_t idx16 = static_cast<uint16_t>(my_counter);
    const bool inl = rq.opcode == kOpcodeRdmaWrite && rq.size <= kInlineThreshold;

    // Segment 0: control.
    const uint32_t ds = rq.form == kWqeZeroByteRead ? 2u : is_atomic ? 4u : 3u;
    u32x4 c;
    c.x = (static_cast<uint32_t>(rq.opcode) << 24) |
          (static_cast<uint32_t>(__builtin_bswap16(idx16)) << 8);
    c.y = (ds << 24) | ring.ctrl_qp_sq;
    const uint32_t fm_ce_se =
        wants_cqe ? kCqUpdate : static_cast<uint32_t>((ring.ctrl_sig >> 24) & 0xffu);
    c.z = static_cast<uint32_t>(ring.ctrl_sig & 0xffu) | (fm_ce_se << 24);
    c.w = static_cast<uint32_t>(ring.ctrl_sig >> 32);
    __builtin_amdgcn_raw_buffer_store_b128(c, ring_mem, at, 0, kThrough);
    first8_lo = c.x;
    first8_hi = c.y;

    // Segment 1: remote address and key.
    u32x4 r;
    r.x = be64_first(rq.raddr);
      r.y = be64_second(rq.raddr);
    r.z = rq.form == kWqeFlushWrite ? ring.flush_rkey_by_pe[rq.pe] : ring.rkey_by_pe[rq.pe];
    r.w = 0;
    __builtin_amdgcn_raw_buffer_store_b128(r, ring_mem, at + 16u, 0, kThrough);

    if (rq.form == kWqeZeroByteRead) {
      // no third segment
    } else if (rq.form == kWqeFlushWrite) {
      __builtin_amdgcn_raw_buffer_store_b32(be32(4u | 0x80000000u), ring_mem, at + 32u, 0, kThrough);
      __builtin_amdgcn_raw_buffer_store_b8(static_cast<uint8_t>(1), ring_mem, at + 36u, 0, kThrough);
    } else if (is_atomic) {
      u32x4 a;
      a.x = be64_first(rq.atomic_data);
      a.y = be64_second(rq.atomic_data);
      a.z = be64_first(rq.atomic_cmp);
      a.w = be64_second(rq.atomic_cmp);
      __builtin_amdgcn_raw_buffer_store_b128(a, ring_mem, at + 32u, 0, kThrough);
      const uint32_t pos = (abase + rank_in_mask(atomic_mask)) % kAtomicRetSlots;
      u32x4 d;
      d.x = be32(8u);
      d.y = ring.atomic_lkey;
      d.z = be64_first(ring.atomic_ret_base + 8ull * pos);
      d.w = be64_second(ring.atomic_ret_base + 8ull * pos);
      __builtin_amdgcn_raw_buffer_store_b128(d, ring_mem, at + 48u, 0, kThrough);
    } else if (inl) {
      // Only the bytes the entry defines are written: byte count, payload.
      __builtin_amdgcn_raw_buffer_store_b32(be32((rq.size & 0x3ffu) | 0x80000000u), ring_mem,
                                            at + 32u, 0, kThrough);
      if (rq.size == 8) {
        __builtin_amdgcn_raw_buffer_store_b32(static_cast<uint32_t>(rq.inline_data), ring_mem,
                                              at + 36u, 0, kThrough);
        __builtin_amdgcn_raw_buffer_store_b32(static_cast<uint32_t>(rq.inline_data >> 32),
                                              ring_mem, at + 40u, 0, kThrough);
      } else if (rq.size == 4) {
        __builtin_amdgcn_raw_buffer_store_b32(static_cast<uint32_t>(rq.inline_data), ring_mem,
                                              at + 36u, 0, kThrough);
      } else {
        for (uint32_t i = 0; i < rq.size; ++i)
          __builtin_amdgcn_raw_buffer_store_b8(static_cast<uint8_t>(rq.inline_data >> (8 * i)),
                                               ring_mem, at + 36u + i, 0, kThrough);
      }
    } else {
      u32x4 d;
      d.x = be32(rq.size & 0x7fffffffu);
      d.y = ring.lkey;
      d.z = be64_first(rq.laddr);
      d.w = be64_second(rq.laddr);
      __builtin_amdgcn_raw_buffer_store_b128(d, ring_mem, at + 32u, 0, kThrough);
    }
  }

  // Publish in index order.  The last posting lane waits until every earlier
  // range is published, moves the doorbell record and writes the doorbell
  // value (first 8 bytes of the wave's last entry, as the reference's
  // finishPost does), then hands the queue on.  s_waitcnt (what a
  // workgroup-scope release amounts to) makes the wave's own stores complete
  // before each hand-over.
  __builtin_amdgcn_fence(__ATOMIC_RELEASE, "workgroup");
  if (last) {
    // quiet_counter (queue_pair.cpp:80-101): completions asked of a live
    // consumer that roc_shmem_ctx_quiet has yet to collect.
    if (g_state.sq_queue_mode == kSqLive)
      __hip_atomic_fetch_add(reader_word(cnt), static_cast<unsigned long long>(n_cqe) << 32, __ATOMIC_RELAXED,
                             __HIP_MEMORY_SCOPE_AGENT);
    bounded_wait<uint32_t>(&cnt->published, kWaitEq, base);
    __hip_atomic_store(reinterpret_cast<unsigned long long *>(&ring.mailbox[0]),
                       static_cast<unsigned long long>(be32(base + n)), __ATOMIC_RELAXED,
                       __HIP_MEMORY_SCOPE_AGENT);
    __hip_atomic_store(reinterpret_cast<unsigned long long *>(&ring.mailbox[1]),
                       (static_cast<unsigned long long>(first8_hi) << 32) | first8_lo,
                       __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
    __builtin_amdgcn_fence(__ATOMIC_RELEASE, "workgroup");
    __hip_atomic_store(&cnt->published, base + n, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
  }
}

// quiet on a queue with a live consumer (reference: QueuePair::quiet_internal,
// queue_pair.cpp:118-191).  Completions arrive in order, so the reader looks at what has been
// requested and not yet taken (quiet_counter), polls only the entry of the last of them until
// the consumer has written it - valid when its owner bit equals the lap parity of its running
// number and its opcode is not "invalid" - and only then takes them: it moves the completion
// queue's consumer index, lowers quiet_counter by what it took and writes the completion
// queue's doorbell record (mailbox word 2).  As in the reference the counters change after the
// poll, so several waves may quiet one queue at the same time and each returns only when every
// completion that was requested before it looked has been written: one that finds nothing
// requested can rely on whoever took the completions having seen them first.  Both counters
// sit in one 64-bit word (reader_word) that is changed by compare-and-swap; a wave whose swap
// fails (another reader took completions, or more were requested meanwhile) looks again.  The
// wait is bounded like every other.
__device__ __forceinline__ void quiet_live(DeviceCtx *ctx) {
  SqCounters *cnt = ctx->counters;
  const SqRing &ring = ctx->ring;
  uint64_t start = wall_clock64();
  uint32_t spins = 0;
  for (;;) {
    unsigned long long seen = __hip_atomic_load(reader_word(cnt), __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
    const uint32_t requested = static_cast<uint32_t>(seen >> 32);
    const uint32_t taken = static_cast<uint32_t>(seen);
    if (requested == 0) return;
    const uint32_t number = taken + requested - 1;
    // last 8 bytes of the completion entry: ... | BE32 qpn | BE16 wqe index | signature | op_own
    const unsigned long long *tail = reinterpret_cast<const unsigned long long *>(
        ring.cq + 8ull * (number & (ring.cq_size - 1)) + 7);
    const uint32_t parity = (number >> ring.cq_log_size) & 1u;
    bool gave_up = false;
    for (;;) {
      const unsigned long long word =
          __hip_atomic_load(tail, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
      const uint32_t op_own = static_cast<uint32_t>(word >> 56);
      if ((op_own & 1u) == parity && (op_own >> 4) != 0xFu) {
        // a requester completion of this queue (opcode 0, the queue's number)
        if ((op_own >> 4) != 0u ||
            static_cast<uint32_t>(word) != ((ring.ctrl_qp_sq & 0xffffffu) << 8))
          status_raise(kStatusBadCompletion);
        break;
      }
      __builtin_amdgcn_s_sleep(1);
      if ((++spins & 63u) == 0 &&
          (status_failed() || wall_clock64() - start > g_state.wait_limit_ticks)) {
        status_raise(kStatusWaitTimeout);
        gave_up = true;
        break;
      }
    }
    // (requested, taken) -> (requested - what this reader saw, taken + the same); a reader
    // that gave up takes them all the same, so that the counters stay in step with the entries
    const unsigned long long next = static_cast<unsigned long long>(taken + requested);
    if (__hip_atomic_compare_exchange_strong(reader_word(cnt), &seen, next, __ATOMIC_RELAXED, __ATOMIC_RELAXED,
                                             __HIP_MEMORY_SCOPE_AGENT)) {
      __hip_atomic_store(reinterpret_cast<unsigned long long *>(&ring.mailbox[2]),
                         static_cast<unsigned long long>(be32(number + 1)), __ATOMIC_RELAXED,
                         __HIP_MEMORY_SCOPE_AGENT);
      return;
    }
    if (gave_up) return;
  }
}

__device__ __forceinline__ void wave_post(DeviceCtx *ctx, bool sends, const WqeRequest &rq);

// The entries quiet and fence leave on a queue with a live consumer, posted by
// the lowest active lane of the calling wave (the reference's multi-thread
// policy picks one lane per wave the same way, thread_policy.cpp:40-71).  The
// reference posts one per destination queue pair; a context here has one queue
// for all destinations, so it posts one, addressed to the calling PE.
__device__ __forceinline__ void post_no_data_entry(DeviceCtx *ctx, WqeForm form) {
  const uint64_t active = __ballot(true);
  WqeRequest rq;
  rq.opcode = form == kWqeZeroByteRead ? kOpcodeRdmaRead : kOpcodeRdmaWrite;
  rq.size = 0;
  rq.raddr = form == kWqeZeroByteRead
                 ? reinterpret_cast<uint64_t>(g_state.heap_base0) +
                       static_cast<uint64_t>(ctx->my_pe) * g_state.slice_stride
                 : ctx->ring.flush_base + 64ull * static_cast<uint64_t>(ctx->my_pe);
  rq.laddr = 0;
  rq.atomic_data = 0;
  rq.atomic_cmp = 0;
  rq.inline_data = 0;
  rq.pe = ctx->my_pe;
  rq.form = form;
  wave_post(ctx, lane_id() == static_cast<uint32_t>(__builtin_ctzll(active)), rq);
}

// A ring that only one workgroup feeds (at most ROC_SHMEM_NUM_BLOCKS
// workgroups per PE in the grid) is written with ordinary cached stores.  A
// ring that several workgroups share may be fed from different XCDs, each
// with its own write-back L2: there the entries are written through to memory
// (agent-scope stores, sc1), so that a slot two workgroups write one after
// the other holds the later entry whatever order the L2s are written back
// in.  Writing through costs a fifth of the small-put rate (10.5 against
// 13.2 G ops/s for 10 M eight-byte puts), hence the switch.  A ring whose
// consumer runs at the same time as its producers (kSqLive) is written through
// too: the consumer may sit on another XCD and reads the entries while the
// producers' kernel is still running.
__device__ __forceinline__ void wave_post(DeviceCtx *ctx, bool sends, const WqeRequest &rq) {
  const bool shared_ring =
      gridDim.x > static_cast<unsigned>(g_state.num_pes) * static_cast<unsigned>(g_state.num_blocks) ||
      gridDim.y * gridDim.z > 1;
  if (shared_ring || g_state.sq_queue_mode == kSqLive) {
    wave_post_with<16 /* sc1: write through */>(ctx, sends, rq);
  } else {
    wave_post_with<0>(ctx, sends, rq);
  }
}

}  // namespace detail
}  // namespace rocshmem

#endif
