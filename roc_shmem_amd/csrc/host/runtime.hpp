// Host-side runtime of the MI355X data path: the HBM arena that holds every
// PE's symmetric-heap slice, the symmetric allocator, context and send-queue
// tables, and teams.  Plain C++ over the HIP runtime, nothing else.
#ifndef ROCSHMEM_MI355X_HOST_RUNTIME_HPP
#define ROCSHMEM_MI355X_HOST_RUNTIME_HPP

#include <hip/hip_runtime.h>

#include <cstddef>
#include <cstdint>
#include <map>
#include <mutex>
#include <string>
#include <vector>

#include "rocshmem_device/state.hpp"

namespace rocshmem {
namespace host {

// Symmetric-heap allocator handing out slice-relative offsets.  Observable
// behaviour follows the reference's Pow2Bins strategy
// (library/src/memory/pow2_bins.hpp:90-125,264-287, binner.hpp:109-134):
// requests round up to a power of two with a 128-byte floor; an empty bin is
// refilled by halving a block of the next non-empty larger bin, lower half
// handed out first; freed blocks go back on top of their bin and are never
// merged; a zero-byte request yields nothing.
class Pow2Allocator {
 public:
  static constexpr size_t kMinBlock = 128;  // reference: ALIGNMENT, constants.hpp:39
  static constexpr size_t kNoOffset = ~size_t(0);

  Pow2Allocator() = default;
  explicit Pow2Allocator(size_t heap_bytes);

  size_t alloc(size_t request);  // kNoOffset when nothing fits (or request == 0)
  bool free(size_t offset);      // false when `offset` is not an outstanding allocation
  size_t bytes_in_use() const;
  // End offset of the outstanding block that contains `offset`, kNoOffset when there is none.
  size_t block_end(size_t offset) const;
  size_t heap_bytes() const { return heap_bytes_; }

 private:
  bool refill(std::map<size_t, std::vector<size_t>>::iterator it);
  size_t heap_bytes_ = 0;
  std::map<size_t, std::vector<size_t>> bins_;  // block size -> LIFO stack of offsets
  std::map<size_t, size_t> outstanding_;        // offset -> block size
};

struct Options {
  int num_pes = 8;                 // ROC_SHMEM_NUM_PES
  size_t heap_size = 1ull << 30;   // ROC_SHMEM_HEAP_SIZE, per PE (reference: heap_memory.hpp:114)
  int num_blocks = 64;             // ROC_SHMEM_NUM_BLOCKS, contexts per PE
  uint32_t sq_size = 1024;         // ROC_SHMEM_SQ_SIZE (reference: connection.hpp:225)
  size_t slice_pad = 0;            // ROC_SHMEM_SLICE_PAD, extra bytes between slices
  double wait_limit_s = 2.0;       // ROC_SHMEM_WAIT_LIMIT_S, bound of a flag wait; 0 = no limit
  bool sq_queue_mode = false;      // ROC_SHMEM_SQ_MODE=queue: slots are freed by the consumer pass
  double consumer_idle_s = 5.0;    // ROC_SHMEM_CONSUMER_IDLE_S: a live consumer wave leaves when
                                   // nothing was published on its rings for this long
  // ROC_SHMEM_HEAP_HOST_VISIBLE (default 1): the arena is fine-grained device memory, which host
  // code can dereference like the reference's heap (hipExtMallocWithFlags, heap_type.hpp:50) and
  // which kernels stream as fast as ordinary device memory; 0: plain hipMalloc.
  bool heap_host_visible = true;
  // ROC_SHMEM_REBASE_ARGS (default 1): device calls move symmetric-heap arguments into the
  // calling PE's slice, so a kernel may pass roc_shmem_malloc's pointer straight through.
  bool rebase_args = true;
  // ROC_SHMEM_PACE_COPY / ROC_SHMEM_PACE_REDUCE / ROC_SHMEM_PACE_REDUCE_SHORT: bytes per tick
  // of the 100 MHz clock for the lockstep pacing of large sharded copies / reductions (device
  // Pacer); 0 = off.  Reductions are paced by default at the rate where the schedule gained
  // most on the cards seen, one rate for passes of 128 KiB per member (workgroups of 1024
  // lanes) and one for shorter passes (fp32 sum over 8 x 2^26, GB/s at 63000 / 64000 / 65000 /
  // 66000 / 67000 / 68000 / 70000 and running free; 32 x 1024 lanes per PE: 6236 6321 6411 6503
  // 6571 6546 6456 | 6001; 32 x 512, whose shorter slots leave less room: 6208 5972 6144 5869
  // 6196 5814 5819 | 5860, steady up to 63000 and uneven beyond).  A rate the caller sets
  // (rsm_set_pacing, the tuner) holds for both kinds of pass; setting the default long rate
  // again brings both defaults back.
  // Copies run free by default.  With a rate, sharded puts and gets that keep a workgroup busy
  // for 64 passes or more and alltoalls whose blocks stream follow a schedule of their own; it
  // pays in some shapes and costs in others (alltoall at 67000 against free: 16 PEs x 64 MiB
  // +1.4 to +2.9 %, 8 PEs x 128 MiB by 32 x 1024 lanes per PE -9 %), so it is the caller's choice.
  uint32_t pace_copy = 0;
  uint32_t pace_reduce = 67000;
  uint32_t pace_reduce_short = 63000;
  // ROC_SHMEM_REDUCE_LDS=1: rsm_to_all runs float / long / bfloat16 sums through the LDS-staged
  // form of the sharded reduction (a measured alternative, slower on MI355X; default 0).
  bool reduce_lds = false;
  static Options from_env();
};

struct TeamRecord {
  detail::Team image;      // host copy of the device object
  detail::Team *device;    // the handle a roc_shmem_team_t points at
  size_t pool_offset;      // symmetric offset of the pSync pools
};

class Runtime {
 public:
  // Returns an empty string on success, an error message otherwise.
  static std::string create(const Options &opt);
  static void destroy();
  static Runtime *get() { return instance_; }

  const Options &options() const { return opt_; }
  int num_pes() const { return opt_.num_pes; }
  size_t slice_stride() const { return stride_; }
  char *slice_base(int pe) const { return arena_ + stride_ * static_cast<size_t>(pe); }
  bool owns(const void *p) const;
  int pe_of(const void *p) const;

  int current_pe() const { return current_pe_; }
  void set_current_pe(int pe) { current_pe_ = pe; }

  void *sym_malloc(size_t bytes);   // the object's symmetric address (in PE 0's slice), nullptr on failure
  bool sym_free(void *ptr);
  void *translate(const void *ptr, int pe) const;
  size_t bytes_in_use() const {
    std::lock_guard<std::mutex> lk(alloc_mu_);
    return alloc_.bytes_in_use();
  }

  detail::Team *team_world() const { return world_->device; }
  // 0 on success (handle in *out, nullptr if arguments describe no team), -1 on bad arguments.
  int team_split(detail::Team *parent, int start, int stride, int size, detail::Team **out);
  void team_destroy(detail::Team *team);
  const TeamRecord *team_record(const detail::Team *team) const;
  int live_teams() const { return static_cast<int>(teams_.size()); }

  detail::DeviceCtx *ctx_device(int pe, int block) const {
    return ctx_table_dev_ + static_cast<size_t>(pe) * opt_.num_blocks + block;
  }
  const detail::DeviceCtx &ctx_image(int pe, int block) const {
    return ctx_images_[static_cast<size_t>(pe) * opt_.num_blocks + block];
  }
  // Zero every ring, mailbox, producer and consumer index; completion entries
  // go back to "owned by hardware, invalid".
  void reset_queues(hipStream_t stream);
  // false: rings are logs that wrap freely; true: rings are queues whose
  // slots are freed only by the consumer pass.  Returns false when the state
  // could not be re-uploaded.
  bool set_sq_queue_mode(bool queue);
  // The same with the mode given as detail::kSqLog / kSqQueue / kSqLive.
  bool set_sq_mode(uint32_t mode);
  // Rates of the lockstep pacing (0 = off); false when the state could not be re-uploaded.
  bool set_pacing(uint32_t copy_bytes_per_tick, uint32_t reduce_bytes_per_tick);
  // The one place the library waits for the whole device.  A kernel that runs until it is told
  // to stop (the live send-queue consumer) makes such a wait last until that kernel gives up by
  // itself and leaves the queues without a consumer, so whoever starts one registers it here
  // with the routine that stops it: while it is registered, wait_for_device() returns false
  // without waiting (callers refuse, or wait for their own streams), state changes that need an
  // idle device (set_pacing, set_sq_mode) fail, and teardown stops the kernel first.
  bool wait_for_device();
  void persistent_kernel_started(void (*stop)());
  void persistent_kernel_stopped();
  bool persistent_kernel_running() const { return persistent_stop_ != nullptr; }
  bool sq_queue_mode() const { return state_.sq_queue_mode != 0; }
  const detail::DeviceState &device_state() const { return state_; }
  char *arena() const { return arena_; }
  char *flush_words() const { return flush_words_dev_; }
  // End (as a heap offset) of the live symmetric allocation that contains heap offset `offset`,
  // Pow2Allocator::kNoOffset when no allocation does.
  size_t allocation_end(size_t offset) const {
    std::lock_guard<std::mutex> lk(alloc_mu_);
    return alloc_.block_end(offset);
  }
  size_t arena_bytes() const { return stride_ * static_cast<size_t>(opt_.num_pes); }

  // Reads and clears the sticky device status word.  When it was raised, the team pSync pools
  // and the host collectives' pSync are zeroed in every PE slice (reset_sync_pools), so that
  // the collectives and barriers that follow start from a consistent state.
  uint32_t take_status();
  void reset_sync_pools();

  // pSync slices (num_blocks x 256 longs, zeroed, in every PE's heap) that the
  // host-initiated active-set collectives use; allocated on first use,
  // nullptr when the heap has no room.
  long *host_psync();
  // 256 bytes of device memory for small results of library kernels.
  void *result_scratch() const { return status_dev_ ? reinterpret_cast<char *>(status_dev_) + 256 : nullptr; }

  static constexpr int kMaxTeams = 40;  // reference: team_tracker.hpp:125

 private:
  Runtime() = default;
  std::string init(const Options &opt);
  void teardown();
  TeamRecord *make_team(const detail::TeamInfo &info);

  static Runtime *instance_;
  Options opt_;
  size_t stride_ = 0;
  char *arena_ = nullptr;
  Pow2Allocator alloc_;
  mutable std::mutex alloc_mu_;  // guards alloc_: entry points look allocations up while other threads allocate
  int current_pe_ = 0;

  char **base_heap_dev_ = nullptr;
  detail::DeviceCtx *ctx_table_dev_ = nullptr;
  std::vector<detail::DeviceCtx> ctx_images_;
  char *queue_mem_ = nullptr;   // rings + mailboxes + atomic-return windows
  size_t queue_mem_bytes_ = 0;
  char *cq_mem_ = nullptr;      // completion queues, sq_size 64-byte entries per ring
  size_t cq_mem_bytes_ = 0;
  detail::SqCounters *counters_dev_ = nullptr;
  uint32_t *rkeys_dev_ = nullptr;
  char *flush_words_dev_ = nullptr;
  uint32_t *status_dev_ = nullptr;
  void (*persistent_stop_)() = nullptr;   // stops the registered persistent kernel; null = none runs
  uint64_t *timeline_dev_ = nullptr;   // ROC_SHMEM_TIMELINE_FILE: clock readings of a timeline build
  detail::Team *teams_dev_ = nullptr;   // kMaxTeams objects
  std::vector<int> free_team_slots_;
  std::map<const detail::Team *, TeamRecord> teams_;
  TeamRecord *world_ = nullptr;
  long *host_psync_ = nullptr;
  detail::DeviceState state_{};
};

// Every translation unit that contains kernels registers a function that
// copies the device state into its own __constant__ instance.
// Returns false when any unit could not be updated and verified.
bool upload_state_everywhere(const detail::DeviceState &state);
// False when a registered unit was compiled against different state structures.
bool state_layouts_agree();
// Number of distinct translation units registered for state uploads.
int registered_state_units();

}  // namespace host
}  // namespace rocshmem

#endif
