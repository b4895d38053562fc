// Device-visible runtime state of the MI355X data path.
//
// One process hosts every PE.  PE p owns the symmetric-heap slice
//   [heap_base0 + p*slice_stride, heap_base0 + p*slice_stride + heap_size)
// of a single HBM arena, so the reference's address translation
//   base_heap[pe] + (ptr - base_heap[my_pe])
// (library/src/gpu_ib/context_ib_device.cpp:86,99,222) becomes one multiply-add.
#ifndef ROCSHMEM_MI355X_DEVICE_STATE_HPP
#define ROCSHMEM_MI355X_DEVICE_STATE_HPP

#include <hip/hip_runtime.h>
#include <stddef.h>
#include <stdint.h>

namespace rocshmem {
namespace detail {

constexpr int kWaveSize = 64;      // reference: WF_SIZE, library/src/constants.hpp:56
constexpr int kMaxPes = 128;       // two flag sets of kMaxPes fit ROC_SHMEM_*_SYNC_SIZE (256)
constexpr int kSyncSlots = 256;    // longs per pSync slice
constexpr int kAtomicRetSlots = 4096;  // reference: atomic_return.hpp:34-40

enum : uint32_t { kSqLog = 0, kSqQueue = 1, kSqLive = 2 };

// Sticky status codes written to DeviceState::status[0].
enum : uint32_t {
  kStatusOk = 0,
  kStatusWaitTimeout = 1,   // a bounded flag wait gave up
  kStatusBadArgument = 2,   // e.g. active set larger than kMaxPes
  kStatusBadCompletion = 3, // quiet found a completion entry that does not belong to its queue
};

// Active-set description relative to the world (reference: TeamInfo,
// library/src/team.hpp:38-75; log_stride is kept integral here).
struct TeamInfo {
  int pe_start;
  int stride;
  int log_stride;
  int size;
};

// Device-side team object (reference: GPUIBTeam, library/src/gpu_ib/gpu_ib_team.hpp).
// The pSync pools are symmetric-heap offsets valid in every slice; each
// context block owns a private kSyncSlots-long slice of each pool so that
// several workgroups of one PE can run team collectives concurrently.
struct Team {
  TeamInfo wrt_world;
  int valid;
  int pad_;
  uint64_t barrier_psync_off;
  uint64_t reduce_psync_off;
  uint64_t bcast_psync_off;
  uint64_t alltoall_psync_off;
};

// Send-queue ring of one context (reference: QueuePair, queue_pair.hpp:337-418).
struct SqRing {
  uint64_t *sq;             // max_nwqe slots of 8 x u64 (64 B each)
  uint64_t *mailbox;        // [0] doorbell record (BE32 in the low word), [1] doorbell value
  const uint32_t *rkey_by_pe;  // remote key per destination PE, stored as the NIC would read it
  uint64_t atomic_ret_base; // address AMO results would be DMA'd to (never written here)
  uint64_t ctrl_sig;
  uint32_t ctrl_qp_sq;
  uint32_t lkey;
  uint32_t atomic_lkey;
  uint32_t max_nwqe;
  // Completion queue filled by the consumer pass (reference: current_cq_q,
  // cq_size, cq_log_size, queue_pair.hpp:340-396): cq_size 64-byte entries.
  uint64_t *cq;
  uint32_t cq_size;
  uint32_t cq_log_size;
  // Flush words (reference: hdp_address[] / hdp_rkey[], network_policy.cpp:114-180; what a
  // fence's entry is addressed to, queue_pair.cpp:376-384): PE p's at flush_base + 64 p
  // under flush_rkey_by_pe[p].  Named by entries, never written.
  const uint32_t *flush_rkey_by_pe;
  uint64_t flush_base;
};

// Mutable producer indices of a ring, on their own cache line.
struct alignas(64) SqCounters {
  uint32_t sq_counter;      // free-running WQE index (reference: queue_pair.hpp:378)
  uint32_t published;       // every WQE below this index is complete in memory
  uint32_t atomic_counter;  // free-running AMO return-slot index
  uint32_t consumed;        // every WQE below this index has been retired by the consumer pass
  uint32_t cq_producer;     // free-running count of completion entries written
  uint32_t pad0_;
  // The reader's pair, one naturally aligned 64-bit word (quiet_counter in the upper half) that
  // posts and quiets change with single 64-bit atomics, so that concurrent quiets on one queue
  // always see a consistent (taken, still requested) pair:
  uint32_t cq_consumer;     // completion entries a reader (quiet) has taken (reference: cq_consumer_counter)
  uint32_t quiet_counter;   // completions requested from a live consumer and not yet taken by quiet
  uint32_t pad_[8];
};
static_assert(offsetof(SqCounters, cq_consumer) % 8 == 0 &&
                  offsetof(SqCounters, quiet_counter) == offsetof(SqCounters, cq_consumer) + 4,
              "cq_consumer and quiet_counter form one aligned 64-bit word");

// One context = one (PE, block) pair (reference: GPUIBContext members,
// context_ib_device.hpp:278-299, minus all NIC state).
struct DeviceCtx {
  int my_pe;
  int num_pes;
  int block_id;
  int options;
  SqRing ring;
  SqCounters *counters;
};

struct DeviceState {
  char *heap_base0;
  uint64_t slice_stride;
  uint64_t heap_size;
  int num_pes;
  int num_blocks;
  DeviceCtx *ctx_table;        // [num_pes * num_blocks]
  char *const *base_heap;      // slice base per PE (reference: base_heap[])
  Team *team_world;
  uint32_t *status;
  uint64_t wait_limit_ticks;   // wall_clock64() ticks a flag wait may take
  // kSqLog: a ring is a log, a slot may be rewritten once its previous entry
  // is published.  kSqQueue: a ring is a queue, a slot may be rewritten only
  // after the consumer pass (run between producer kernels) has retired its
  // previous entry.  kSqLive: a queue whose consumer runs at the same time as
  // the producers: entries and completions are written through to memory, and
  // quiet waits until the ring's entries are retired.
  uint32_t sq_queue_mode;
  // 1: roc_shmem_* calls move symmetric-heap arguments into the calling PE's
  // slice before they use them (one kernel argument then serves the workgroups
  // of every PE); 0: arguments are used as given.
  uint32_t rebase_args;
  uint64_t arena_bytes;        // num_pes * slice_stride
  // Lockstep pacing of large streaming copies / reductions (see Pacer in copy.hpp): bytes of
  // traffic the memory system takes per tick of the 100 MHz clock when all workgroups issue in
  // step; 0 = workgroups run free.
  uint32_t pace_copy_bytes_per_tick;
  uint32_t pace_reduce_bytes_per_tick;
  // The rate for reductions whose passes are shorter than 128 KiB per member (workgroups of
  // fewer than 1024 lanes): their slots are half as long, they sustain a little less, and a
  // schedule ahead of what the card sustains costs them more (32 x 512 lanes per PE: 6208 GB/s
  // at 63000, 5814-6196 from launch shape to launch shape and rate to rate beyond it).
  uint32_t pace_reduce_short_bytes_per_tick;
  // Grids that are paced: at most pace_max_grid_lanes lanes (compute units x 1024, what is
  // resident together of the streaming kernels, which need 65-128 vector registers: the slots
  // are sized for all workgroups of the grid running at once) and at least
  // pace_min_grid_workgroups workgroups (one per compute unit: on half a chip the schedule
  // measured 1-3 % slower than none).
  uint32_t pace_max_grid_lanes;
  uint32_t pace_min_grid_workgroups;
};

// Timeline builds (-DROCSHMEM_TIMELINE): words 32-33 of the status block hold the device
// address of kTimelineBytes of clock readings, kTimelineMarks 64-bit readings for each of the
// first kTimelineWaves waves of a grid (wave = workgroup * 16 + wave of the workgroup), or 0.
constexpr int kTimelinePointerWord = 32;
constexpr int kTimelineMarks = 8;
constexpr int kTimelineWaves = 2048 * 16;
constexpr size_t kTimelineBytes = static_cast<size_t>(kTimelineWaves) * kTimelineMarks * 8;

// Fingerprint of the structures device code and the host library share.  Device
// code is compiled into every user program (the interface is header-only); a
// program built against other headers than the library it loads would index
// ctx_table with the wrong stride and follow wild pointers, so every unit hands
// its fingerprint to the library, which refuses to initialise on a mismatch.
// Bump kStateRevision when a layout changes without changing a size, or when
// units must agree on how they use shared memory (3: the barrier pool holds
// call counts, not flags that are reset; 4: live queues, cq_consumer;
// 5: arguments rebased into the caller's slice; 6: pacing; 7: paced bursts follow a
// schedule of start times; 8: quiet and fence post on live queues; 9: word 16 of the status block
// counts the workgroups inside large standard reductions, the completion reader's counters are
// one 64-bit word).
constexpr uint32_t kStateRevision = 9;
constexpr uint32_t kStateLayout =
    (kStateRevision * 0x01000193u) ^
    static_cast<uint32_t>(sizeof(DeviceState) | (sizeof(DeviceCtx) << 8) | (sizeof(Team) << 16) |
                          (sizeof(SqCounters) << 24));

}  // namespace detail
}  // namespace rocshmem

#endif
