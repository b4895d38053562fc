#include "runtime.hpp"

#include <algorithm>
#include <cstdio>
#include <cstdlib>
#include <cstring>
#include <functional>
#include <sstream>

namespace rocshmem {
namespace host {

// ---------------------------------------------------------------------------
// Pow2Allocator
// ---------------------------------------------------------------------------

static size_t round_up_pow2(size_t v) {
  size_t p = Pow2Allocator::kMinBlock;
  while (p < v) p <<= 1;
  return p;
}

Pow2Allocator::Pow2Allocator(size_t heap_bytes) : heap_bytes_(heap_bytes) {
  // One bin per power of two from the floor up to the largest power of two
  // that fits; the heap is handed to the bins as its binary decomposition,
  // largest block at the lowest address.
  size_t top = kMinBlock;
  while ((top << 1) <= heap_bytes && (top << 1) != 0) top <<= 1;
  for (size_t s = kMinBlock; s <= top; s <<= 1) bins_[s];
  size_t offset = 0;
  for (size_t s = top; s >= kMinBlock; s >>= 1) {
    if (heap_bytes - offset >= s) {
      bins_[s].push_back(offset);
      offset += s;
    }
  }
}

bool Pow2Allocator::refill(std::map<size_t, std::vector<size_t>>::iterator it) {
  auto next = std::next(it);
  if (next == bins_.end()) return false;
  if (next->second.empty() && !refill(next)) return false;
  size_t block = next->second.back();
  next->second.pop_back();
  // Upper half goes in first so that the lower half is handed out first.
  it->second.push_back(block + it->first);
  it->second.push_back(block);
  return true;
}

size_t Pow2Allocator::alloc(size_t request) {
  if (request == 0) return kNoOffset;
  size_t want = round_up_pow2(request);
  auto it = bins_.find(want);
  if (it == bins_.end()) return kNoOffset;
  if (it->second.empty() && !refill(it)) return kNoOffset;
  size_t off = it->second.back();
  it->second.pop_back();
  outstanding_[off] = want;
  return off;
}

bool Pow2Allocator::free(size_t offset) {
  auto it = outstanding_.find(offset);
  if (it == outstanding_.end()) return false;
  bins_[it->second].push_back(offset);
  outstanding_.erase(it);
  return true;
}

size_t Pow2Allocator::block_end(size_t offset) const {
  auto it = outstanding_.upper_bound(offset);
  if (it == outstanding_.begin()) return kNoOffset;
  --it;
  return offset < it->first + it->second ? it->first + it->second : kNoOffset;
}

size_t Pow2Allocator::bytes_in_use() const {
  size_t total = 0;
  for (const auto &kv : outstanding_) total += kv.second;
  return total;
}

// ---------------------------------------------------------------------------
// Options
// ---------------------------------------------------------------------------

static bool env_u64(const char *name, unsigned long long *out) {
  const char *s = getenv(name);
  if (!s || !*s) return false;
  char *end = nullptr;
  unsigned long long v = strtoull(s, &end, 0);
  if (end == s) return false;
  *out = v;
  return true;
}

Options Options::from_env() {
  Options o;
  unsigned long long v;
  if (env_u64("ROC_SHMEM_NUM_PES", &v)) o.num_pes = static_cast<int>(v);
  if (env_u64("ROC_SHMEM_HEAP_SIZE", &v)) o.heap_size = static_cast<size_t>(v);
  if (env_u64("ROC_SHMEM_NUM_BLOCKS", &v)) o.num_blocks = static_cast<int>(v);
  if (env_u64("ROC_SHMEM_SQ_SIZE", &v)) o.sq_size = static_cast<uint32_t>(v);
  if (env_u64("ROC_SHMEM_SLICE_PAD", &v)) o.slice_pad = static_cast<size_t>(v);
  if (const char *s = getenv("ROC_SHMEM_WAIT_LIMIT_S")) {
    char *end = nullptr;
    double d = strtod(s, &end);
    if (end != s && d >= 0) o.wait_limit_s = d;   // 0: waits never give up
  }
  if (const char *s = getenv("ROC_SHMEM_CONSUMER_IDLE_S")) {
    char *end = nullptr;
    double d = strtod(s, &end);
    if (end != s && d > 0 && d < 1e6) o.consumer_idle_s = d;
  }
  if (const char *s = getenv("ROC_SHMEM_SQ_MODE")) o.sq_queue_mode = strcmp(s, "queue") == 0;
  if (env_u64("ROC_SHMEM_HEAP_HOST_VISIBLE", &v)) o.heap_host_visible = v != 0;
  if (env_u64("ROC_SHMEM_REBASE_ARGS", &v)) o.rebase_args = v != 0;
  if (env_u64("ROC_SHMEM_REDUCE_LDS", &v)) o.reduce_lds = v != 0;
  if (env_u64("ROC_SHMEM_PACE_COPY", &v)) o.pace_copy = static_cast<uint32_t>(v);
  if (env_u64("ROC_SHMEM_PACE_REDUCE", &v)) o.pace_reduce = o.pace_reduce_short = static_cast<uint32_t>(v);
  if (env_u64("ROC_SHMEM_PACE_REDUCE_SHORT", &v)) o.pace_reduce_short = static_cast<uint32_t>(v);
  return o;
}

// ---------------------------------------------------------------------------
// Runtime
// ---------------------------------------------------------------------------

Runtime *Runtime::instance_ = nullptr;

#define RT_HIP(expr)                                                             \
  do {                                                                           \
    hipError_t e_ = (expr);                                                      \
    if (e_ != hipSuccess) {                                                      \
      std::ostringstream os_;                                                    \
      os_ << #expr << " failed: " << hipGetErrorString(e_);                      \
      return os_.str();                                                          \
    }                                                                            \
  } while (0)

std::string Runtime::create(const Options &opt) {
  if (instance_) return "runtime already initialised";
  Runtime *rt = new Runtime();
  std::string err = rt->init(opt);
  if (!err.empty()) {
    rt->teardown();
    delete rt;
    return err;
  }
  instance_ = rt;
  return "";
}

void Runtime::destroy() {
  if (!instance_) return;
  instance_->teardown();
  delete instance_;
  instance_ = nullptr;
}

static uint32_t bswap32(uint32_t v) { return __builtin_bswap32(v); }

std::string Runtime::init(const Options &opt) {
  opt_ = opt;
  if (opt_.num_pes < 1 || opt_.num_pes > detail::kMaxPes)
    return "ROC_SHMEM_NUM_PES must be in [1, 128]";
  if (opt_.num_blocks < 1) return "ROC_SHMEM_NUM_BLOCKS must be positive";
  // A wave posts up to 64 entries at once; they must fit the ring.
  if (opt_.sq_size < 64 || (opt_.sq_size & (opt_.sq_size - 1)))
    return "ROC_SHMEM_SQ_SIZE must be a power of two, at least 64";
  if (opt_.heap_size < (1u << 20) || (opt_.heap_size & 4095))
    return "ROC_SHMEM_HEAP_SIZE must be a multiple of 4096 and at least 1 MiB";
  if (opt_.slice_pad & 4095) return "ROC_SHMEM_SLICE_PAD must be a multiple of 4096";

  const int P = opt_.num_pes;
  const int B = opt_.num_blocks;
  stride_ = opt_.heap_size + opt_.slice_pad;
  if (opt_.heap_host_visible) {
    RT_HIP(hipExtMallocWithFlags(reinterpret_cast<void **>(&arena_), stride_ * P,
                                 hipDeviceMallocFinegrained));
  } else {
    RT_HIP(hipMalloc(reinterpret_cast<void **>(&arena_), stride_ * P));
  }
  alloc_ = Pow2Allocator(opt_.heap_size);

  // Slice base table (reference: RemoteHeapInfo's base_heap[], remote_heap_info.hpp:142-152).
  std::vector<char *> bases(P);
  for (int p = 0; p < P; ++p) bases[p] = slice_base(p);
  RT_HIP(hipMalloc(reinterpret_cast<void **>(&base_heap_dev_), sizeof(char *) * P));
  RT_HIP(hipMemcpy(base_heap_dev_, bases.data(), sizeof(char *) * P, hipMemcpyHostToDevice));

  // Send queues.  Per ring: sq_size 64-byte slots, a 64-byte mailbox
  // (doorbell record + doorbell value) and the AMO return window.
  const size_t ring_bytes = static_cast<size_t>(opt_.sq_size) * 64 + 64 +
                            static_cast<size_t>(detail::kAtomicRetSlots) * 8;
  const size_t rings = static_cast<size_t>(P) * B;
  queue_mem_bytes_ = ring_bytes * rings;
  RT_HIP(hipMalloc(reinterpret_cast<void **>(&queue_mem_), queue_mem_bytes_));
  RT_HIP(hipMemset(queue_mem_, 0, queue_mem_bytes_));
  RT_HIP(hipMalloc(reinterpret_cast<void **>(&counters_dev_), sizeof(detail::SqCounters) * rings));
  RT_HIP(hipMemset(counters_dev_, 0, sizeof(detail::SqCounters) * rings));
  // Completion queues: as many entries as the send queue has slots
  // (reference: cqe = max_send_wr, connection.cpp:200-206).
  const size_t cq_bytes = static_cast<size_t>(opt_.sq_size) * 64;
  cq_mem_bytes_ = cq_bytes * rings;
  RT_HIP(hipMalloc(reinterpret_cast<void **>(&cq_mem_), cq_mem_bytes_));

  // Synthetic queue-pair constants standing in for what the reference
  // harvests from a NIC-built template WQE (connection.cpp:379-391).
  // Heap keys, then the flush keys (reference: hdp_rkey[], network_policy.cpp:114-180).
  std::vector<uint32_t> rkeys(2 * static_cast<size_t>(P));
  for (int p = 0; p < P; ++p) {
    rkeys[p] = bswap32(0x1000u + p);
    rkeys[P + p] = bswap32(0x4000u + p);
  }
  RT_HIP(hipMalloc(reinterpret_cast<void **>(&rkeys_dev_), sizeof(uint32_t) * rkeys.size()));
  RT_HIP(hipMemcpy(rkeys_dev_, rkeys.data(), sizeof(uint32_t) * rkeys.size(), hipMemcpyHostToDevice));
  // One 64-byte flush word per PE: what fence's entries are addressed to (the reference's
  // hdp_address[]).  Nothing flushes through them on this path; they give the entries a target.
  RT_HIP(hipMalloc(reinterpret_cast<void **>(&flush_words_dev_), 64 * static_cast<size_t>(P)));
  RT_HIP(hipMemset(flush_words_dev_, 0, 64 * static_cast<size_t>(P)));

  ctx_images_.resize(rings);
  for (int p = 0; p < P; ++p) {
    for (int b = 0; b < B; ++b) {
      const size_t r = static_cast<size_t>(p) * B + b;
      detail::DeviceCtx &c = ctx_images_[r];
      c.my_pe = p;
      c.num_pes = P;
      c.block_id = b;
      c.options = 0;
      char *base = queue_mem_ + ring_bytes * r;
      c.ring.sq = reinterpret_cast<uint64_t *>(base);
      c.ring.mailbox = reinterpret_cast<uint64_t *>(base + static_cast<size_t>(opt_.sq_size) * 64);
      c.ring.atomic_ret_base =
          reinterpret_cast<uint64_t>(base + static_cast<size_t>(opt_.sq_size) * 64 + 64);
      c.ring.rkey_by_pe = rkeys_dev_;
      c.ring.flush_rkey_by_pe = rkeys_dev_ + P;
      c.ring.flush_base = reinterpret_cast<uint64_t>(flush_words_dev_);
      c.ring.ctrl_sig = 0;
      // Queue-pair number 0x000100 + ring index, laid out as the three
      // big-endian bytes that follow the opcode word of a WQE.
      c.ring.ctrl_qp_sq = bswap32((0x000100u + static_cast<uint32_t>(r)) << 8) & 0xffffffu;
      c.ring.lkey = bswap32(0x2000u);
      c.ring.atomic_lkey = bswap32(0x3000u);
      c.ring.max_nwqe = opt_.sq_size;
      c.ring.cq = reinterpret_cast<uint64_t *>(cq_mem_ + cq_bytes * r);
      c.ring.cq_size = opt_.sq_size;
      c.ring.cq_log_size = static_cast<uint32_t>(__builtin_ctz(opt_.sq_size));
      c.counters = counters_dev_ + r;
    }
  }
  RT_HIP(hipMalloc(reinterpret_cast<void **>(&ctx_table_dev_), sizeof(detail::DeviceCtx) * rings));
  RT_HIP(hipMemcpy(ctx_table_dev_, ctx_images_.data(), sizeof(detail::DeviceCtx) * rings,
                   hipMemcpyHostToDevice));

  // status word (first 64 bytes), the count of workgroups inside large standard reductions (next
  // 64 bytes) and, 256 bytes in, a scratch area for small kernel results
  RT_HIP(hipMalloc(reinterpret_cast<void **>(&status_dev_), 512));
  RT_HIP(hipMemset(status_dev_, 0, 512));
  // A timeline build of the device code (-DROCSHMEM_TIMELINE) writes clock readings of every
  // wave of a large reduction where the pointer at byte 128 of the status block points; the
  // readings of the last launch are written to ROC_SHMEM_TIMELINE_FILE when the runtime goes.
  if (getenv("ROC_SHMEM_TIMELINE_FILE")) {
    RT_HIP(hipMalloc(reinterpret_cast<void **>(&timeline_dev_), detail::kTimelineBytes));
    RT_HIP(hipMemset(timeline_dev_, 0, detail::kTimelineBytes));
    RT_HIP(hipMemcpy(status_dev_ + detail::kTimelinePointerWord, &timeline_dev_, sizeof(timeline_dev_),
                     hipMemcpyHostToDevice));
  }

  RT_HIP(hipMalloc(reinterpret_cast<void **>(&teams_dev_), sizeof(detail::Team) * kMaxTeams));
  RT_HIP(hipMemset(teams_dev_, 0, sizeof(detail::Team) * kMaxTeams));
  for (int i = kMaxTeams - 1; i >= 0; --i) free_team_slots_.push_back(i);

  detail::TeamInfo world_info{0, 1, 0, P};
  world_ = make_team(world_info);
  if (!world_) return "could not allocate the world team's pSync pools";

  state_.heap_base0 = arena_;
  state_.slice_stride = stride_;
  state_.heap_size = opt_.heap_size;
  state_.num_pes = P;
  state_.num_blocks = B;
  state_.ctx_table = ctx_table_dev_;
  state_.base_heap = base_heap_dev_;
  state_.team_world = world_->device;
  state_.status = status_dev_;
  // 100 MHz clock; a limit of 0 means "never give up" (the reference's behaviour)
  state_.wait_limit_ticks = opt_.wait_limit_s > 0 && opt_.wait_limit_s < 1e9
                                ? static_cast<uint64_t>(opt_.wait_limit_s * 100e6)
                                : ~0ull;
  state_.sq_queue_mode = opt_.sq_queue_mode ? 1u : 0u;
  state_.pace_copy_bytes_per_tick = opt_.pace_copy;
  state_.pace_reduce_bytes_per_tick = opt_.pace_reduce;
  state_.pace_reduce_short_bytes_per_tick = opt_.pace_reduce_short;
  {
    int dev = 0, cus = 0;
    RT_HIP(hipGetDevice(&dev));
    RT_HIP(hipDeviceGetAttribute(&cus, hipDeviceAttributeMultiprocessorCount, dev));
    state_.pace_max_grid_lanes = static_cast<uint32_t>(cus) * 1024u;
    state_.pace_min_grid_workgroups = static_cast<uint32_t>(cus);
  }
  state_.rebase_args = opt_.rebase_args ? 1u : 0u;
  state_.arena_bytes = stride_ * static_cast<uint64_t>(P);
  reset_queues(nullptr);
  if (!state_layouts_agree())
    return "a translation unit of this program was compiled against other device headers than "
           "this library (rebuild it against include/ and roc_shmem_amd/csrc of this library)";
  if (!upload_state_everywhere(state_))
    return "could not upload the device state into every translation unit";
  RT_HIP(hipDeviceSynchronize());
  return "";
}

bool Runtime::wait_for_device() {
  if (persistent_stop_) return false;
  return hipDeviceSynchronize() == hipSuccess;
}

void Runtime::persistent_kernel_started(void (*stop)()) { persistent_stop_ = stop; }
void Runtime::persistent_kernel_stopped() { persistent_stop_ = nullptr; }

void Runtime::teardown() {
  if (persistent_stop_) {
    void (*stop)() = persistent_stop_;
    stop();                       // unregisters itself (persistent_kernel_stopped)
    persistent_stop_ = nullptr;
  }
  (void)wait_for_device();
  if (timeline_dev_) {
    if (const char *path = getenv("ROC_SHMEM_TIMELINE_FILE")) {
      std::vector<char> host(detail::kTimelineBytes);
      if (hipMemcpy(host.data(), timeline_dev_, host.size(), hipMemcpyDeviceToHost) == hipSuccess) {
        if (FILE *f = fopen(path, "wb")) {
          (void)fwrite(host.data(), 1, host.size(), f);
          fclose(f);
        }
      }
    }
    (void)hipFree(timeline_dev_);
    timeline_dev_ = nullptr;
  }
  if (teams_dev_) (void)hipFree(teams_dev_);
  if (status_dev_) (void)hipFree(status_dev_);
  if (ctx_table_dev_) (void)hipFree(ctx_table_dev_);
  if (rkeys_dev_) (void)hipFree(rkeys_dev_);
  if (flush_words_dev_) (void)hipFree(flush_words_dev_);
  if (counters_dev_) (void)hipFree(counters_dev_);
  if (queue_mem_) (void)hipFree(queue_mem_);
  if (cq_mem_) (void)hipFree(cq_mem_);
  if (base_heap_dev_) (void)hipFree(base_heap_dev_);
  if (arena_) (void)hipFree(arena_);
  teams_dev_ = nullptr;
  status_dev_ = nullptr;
  ctx_table_dev_ = nullptr;
  rkeys_dev_ = nullptr;
  flush_words_dev_ = nullptr;
  counters_dev_ = nullptr;
  queue_mem_ = nullptr;
  cq_mem_ = nullptr;
  base_heap_dev_ = nullptr;
  arena_ = nullptr;
  teams_.clear();
  world_ = nullptr;
  host_psync_ = nullptr;
  detail::DeviceState cleared{};
  (void)upload_state_everywhere(cleared);
}

bool Runtime::owns(const void *p) const {
  const char *c = static_cast<const char *>(p);
  return c >= arena_ && c < arena_ + stride_ * static_cast<size_t>(opt_.num_pes);
}

int Runtime::pe_of(const void *p) const {
  if (!owns(p)) return -1;
  return static_cast<int>((static_cast<const char *>(p) - arena_) / stride_);
}

void *Runtime::sym_malloc(size_t bytes) {
  size_t off;
  {
    std::lock_guard<std::mutex> alloc_guard(alloc_mu_);
    off = alloc_.alloc(bytes);
  }
  if (off == Pow2Allocator::kNoOffset) return nullptr;
  // The symmetric address of an object is its address in PE 0's slice, whichever PE the host
  // thread stands for at the moment: it is what device calls take for "the caller's own copy".
  return slice_base(0) + off;
}

bool Runtime::sym_free(void *ptr) {
  if (!ptr || !owns(ptr)) return false;
  size_t off = (static_cast<char *>(ptr) - arena_) % stride_;
  std::lock_guard<std::mutex> alloc_guard(alloc_mu_);
  return alloc_.free(off);
}

void *Runtime::translate(const void *ptr, int pe) const {
  if (!owns(ptr) || pe < 0 || pe >= opt_.num_pes) return nullptr;
  size_t off = (static_cast<const char *>(ptr) - arena_) % stride_;
  return slice_base(pe) + off;
}

TeamRecord *Runtime::make_team(const detail::TeamInfo &info) {
  if (free_team_slots_.empty()) return nullptr;
  // Four pSync pools, one kSyncSlots-long slice per context block each
  // (reference: per-team pool slices, gpu_ib_team.cpp:30-52, backend_ib.cpp:335-381).
  const size_t pool_bytes = static_cast<size_t>(opt_.num_blocks) * detail::kSyncSlots * sizeof(long);
  std::unique_lock<std::mutex> alloc_guard(alloc_mu_);
  size_t off = alloc_.alloc(4 * pool_bytes);
  alloc_guard.unlock();
  if (off == Pow2Allocator::kNoOffset) return nullptr;
  for (int p = 0; p < opt_.num_pes; ++p) {
    if (hipMemset(slice_base(p) + off, 0, 4 * pool_bytes) != hipSuccess) return nullptr;
  }
  int slot = free_team_slots_.back();
  free_team_slots_.pop_back();
  TeamRecord rec;
  rec.image.wrt_world = info;
  rec.image.valid = 1;
  rec.image.pad_ = 0;
  rec.image.barrier_psync_off = off;
  rec.image.reduce_psync_off = off + pool_bytes;
  rec.image.bcast_psync_off = off + 2 * pool_bytes;
  rec.image.alltoall_psync_off = off + 3 * pool_bytes;
  rec.device = teams_dev_ + slot;
  rec.pool_offset = off;
  if (hipMemcpy(rec.device, &rec.image, sizeof(detail::Team), hipMemcpyHostToDevice) !=
      hipSuccess)
    return nullptr;
  auto ins = teams_.emplace(rec.device, rec);
  return &ins.first->second;
}

int Runtime::team_split(detail::Team *parent, int start, int stride, int size,
                        detail::Team **out) {
  *out = nullptr;
  if (!parent) return 0;  // reference: splitting an invalid team yields an invalid team, returns 0
  const TeamRecord *prec = team_record(parent);
  if (!prec) return -1;
  const detail::TeamInfo &pi = prec->image.wrt_world;
  // reference: sanity checks of roc_shmem_team_split_strided, roc_shmem.cpp:237-252
  if (start < 0 || start >= pi.size || size < 1 || size > pi.size || stride < 1) return -1;
  int start_world = pi.pe_start + pi.stride * start;
  int stride_world = stride * pi.stride;
  int end_world = start_world + stride_world * (size - 1);
  if (end_world >= opt_.num_pes) return -1;
  // Any stride makes a team, as in the reference; log_stride is its log2 rounded down
  // (library/src/team.cpp:68), exact for the powers of two the active-set calls can name.
  int log_stride = 0;
  while ((2 << log_stride) <= stride_world) ++log_stride;
  // teams_ holds the world team too; the reference counts user teams only
  // (num_user_teams >= max_num_teams - 1 aborts, roc_shmem.cpp:224-228).
  if (static_cast<int>(teams_.size()) - 1 >= kMaxTeams - 1) {
    fprintf(stderr, "rocshmem: too many teams (limit %d)\n", kMaxTeams);
    abort();  // reference: roc_shmem.cpp:224-228
  }
  detail::TeamInfo info{start_world, stride_world, log_stride, size};
  TeamRecord *rec = make_team(info);
  if (!rec) return -1;
  *out = rec->device;
  return 0;
}

void Runtime::team_destroy(detail::Team *team) {
  auto it = teams_.find(team);
  if (it == teams_.end() || &it->second == world_) return;
  std::unique_lock<std::mutex> alloc_guard(alloc_mu_);
  alloc_.free(it->second.pool_offset);
  alloc_guard.unlock();
  free_team_slots_.push_back(static_cast<int>(it->second.device - teams_dev_));
  teams_.erase(it);
}

const TeamRecord *Runtime::team_record(const detail::Team *team) const {
  auto it = teams_.find(team);
  return it == teams_.end() ? nullptr : &it->second;
}

bool Runtime::set_sq_queue_mode(bool queue) {
  return set_sq_mode(queue ? detail::kSqQueue : detail::kSqLog);
}

bool Runtime::set_pacing(uint32_t copy_bytes_per_tick, uint32_t reduce_bytes_per_tick) {
  if (!wait_for_device()) return false;
  state_.pace_copy_bytes_per_tick = copy_bytes_per_tick;
  state_.pace_reduce_bytes_per_tick = reduce_bytes_per_tick;
  // one rate named by the caller holds for every shape; naming the default brings both defaults back
  state_.pace_reduce_short_bytes_per_tick =
      reduce_bytes_per_tick == opt_.pace_reduce ? opt_.pace_reduce_short : reduce_bytes_per_tick;
  return upload_state_everywhere(state_);
}

bool Runtime::set_sq_mode(uint32_t mode) {
  if (!wait_for_device()) return false;
  state_.sq_queue_mode = mode;
  return upload_state_everywhere(state_);
}

void Runtime::reset_queues(hipStream_t stream) {
  (void)hipMemsetAsync(queue_mem_, 0, queue_mem_bytes_, stream);
  (void)hipMemsetAsync(cq_mem_, 0, cq_mem_bytes_, stream);
  // op_own (last byte of every completion entry) = invalid opcode, owner 0:
  // what a reader finds before the first completion lands in an entry.
  (void)hipMemset2DAsync(cq_mem_ + 63, 64, 0xF0, 1, cq_mem_bytes_ / 64, stream);
  (void)hipMemsetAsync(counters_dev_, 0,
                       sizeof(detail::SqCounters) * static_cast<size_t>(opt_.num_pes) *
                           opt_.num_blocks,
                       stream);
}

long *Runtime::host_psync() {
  if (!host_psync_) {
    const size_t bytes = static_cast<size_t>(opt_.num_blocks) * detail::kSyncSlots * sizeof(long);
    std::unique_lock<std::mutex> alloc_guard(alloc_mu_);
    size_t off = alloc_.alloc(bytes);
    alloc_guard.unlock();
    if (off == Pow2Allocator::kNoOffset) return nullptr;
    for (int p = 0; p < opt_.num_pes; ++p) {
      if (hipMemset(slice_base(p) + off, 0, bytes) != hipSuccess) return nullptr;
    }
    host_psync_ = reinterpret_cast<long *>(slice_base(0) + off);
  }
  return host_psync_;
}

uint32_t Runtime::take_status() {
  uint32_t v = 0;
  const bool idle = wait_for_device();
  (void)hipMemcpy(&v, status_dev_, sizeof(v), hipMemcpyDeviceToHost);
  // (with a persistent kernel running the word is read and left as it is: the pools below may
  // be in use)
  if (v && idle) {
    // A wait that gave up leaves synchronisation state behind that later calls would trip
    // over: flags that were set and never consumed, and barrier call counts that differ
    // between the members that got through and those that did not.  Nothing is running
    // (the device was synchronised above), so put every library-owned pool back to zero.
    reset_sync_pools();
    // (and the count of streaming workgroups, which calls that gave up may not have left)
    (void)hipMemset(status_dev_, 0, 128);
  }
  return v;
}

void Runtime::reset_sync_pools() {
  const size_t pool_bytes = static_cast<size_t>(opt_.num_blocks) * detail::kSyncSlots * sizeof(long);
  for (const auto &kv : teams_)
    for (int p = 0; p < opt_.num_pes; ++p)
      (void)hipMemset(slice_base(p) + kv.second.pool_offset, 0, 4 * pool_bytes);
  if (host_psync_) {
    const size_t off = reinterpret_cast<char *>(host_psync_) - slice_base(0);
    for (int p = 0; p < opt_.num_pes; ++p) (void)hipMemset(slice_base(p) + off, 0, pool_bytes);
  }
  (void)wait_for_device();
}

// ---------------------------------------------------------------------------
// State upload registry
// ---------------------------------------------------------------------------

typedef bool (*UploadFn)(const detail::DeviceState *);
struct Unit {
  UploadFn fn;
  uint32_t layout;
  bool operator<(const Unit &o) const { return std::less<UploadFn>()(fn, o.fn); }
  bool operator==(const Unit &o) const { return fn == o.fn; }
};
static std::vector<Unit> &registry() {
  static std::vector<Unit> units;
  return units;
}

bool state_layouts_agree() {
  for (const Unit &u : registry())
    if (u.layout != detail::kStateLayout) return false;
  return true;
}

bool upload_state_everywhere(const detail::DeviceState &state) {
  if (!state_layouts_agree()) return false;
  bool ok = true;
  for (const Unit &u : registry()) ok = u.fn(&state) && ok;
  return ok;
}

int registered_state_units() {
  std::vector<Unit> units = registry();
  std::sort(units.begin(), units.end());
  return static_cast<int>(std::unique(units.begin(), units.end()) - units.begin());
}

}  // namespace host

namespace detail {
typedef bool (*StateUploadFn)(const DeviceState *);
void register_state_upload(StateUploadFn fn, uint32_t layout) {
  host::registry().push_back(host::Unit{fn, layout});
}
}  // namespace detail

}  // namespace rocshmem
