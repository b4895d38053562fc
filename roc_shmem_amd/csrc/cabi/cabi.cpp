// C ABI: lifecycle, teams, plumbing and send-queue inspection.
#include <cstring>
#include <mutex>

#include "cabi_common.hpp"
#include "roc_shmem.hpp"

namespace rsm {

static std::string g_error;
static std::mutex g_error_mu;

int fail(const std::string &msg) {
  std::lock_guard<std::mutex> lk(g_error_mu);
  g_error = msg;
  return -1;
}
void clear_error() {
  std::lock_guard<std::mutex> lk(g_error_mu);
  g_error.clear();
}

bool resolve_launch(const rsm_launch_t *in, Launch *out) {
  using rocshmem::host::Runtime;
  Runtime *rt = Runtime::get();
  if (!rt) {
    fail("rsm_init has not been called");
    return false;
  }
  if (!in) {
    fail("launch description is NULL");
    return false;
  }
  if (in->wgs_per_pe < 1 || in->wg_size < 64 || in->wg_size > 1024 || (in->wg_size % 64)) {
    fail("launch: wgs_per_pe must be >= 1 and wg_size a multiple of 64 in [64, 1024]");
    return false;
  }
  unsigned long long grid = 1ull * in->wgs_per_pe * rt->num_pes();
  if (grid > 0x7fffffffull) {
    fail("launch: grid too large");
    return false;
  }
  out->wgs_per_pe = in->wgs_per_pe;
  out->wg_size = in->wg_size;
  out->tile = in->tile;
  out->stream = static_cast<hipStream_t>(in->stream);
  out->grid = static_cast<unsigned>(grid);
  return true;
}

std::recursive_mutex &abi_lock() {
  static std::recursive_mutex mu;
  return mu;
}

bool check_symmetric(const void *p, const char *what, bool allow_null) {
  using rocshmem::host::Runtime;
  Runtime *rt = Runtime::get();
  if (!p) {
    if (allow_null) return true;
    fail(std::string(what) + " is NULL");
    return false;
  }
  if (!rt || rt->pe_of(p) != 0) {
    fail(std::string(what) + " is not a symmetric address of PE 0");
    return false;
  }
  return true;
}

bool check_extent(const void *p, size_t bytes, const char *what) {
  using rocshmem::host::Pow2Allocator;
  using rocshmem::host::Runtime;
  Runtime *rt = Runtime::get();
  if (!rt || !p || !rt->owns(p)) return true;  // not symmetric: nothing to compare with
  const size_t offset = (static_cast<const char *>(p) - rt->arena()) % rt->slice_stride();
  const size_t end = rt->allocation_end(offset);
  if (end == Pow2Allocator::kNoOffset) {
    fail(std::string(what) + ": the address (heap offset " + std::to_string(offset) +
         ") is not inside a live symmetric allocation");
    return false;
  }
  if (bytes > end - offset) {
    fail(std::string(what) + ": " + std::to_string(bytes) + " bytes at heap offset " +
         std::to_string(offset) + " do not fit the symmetric allocation that holds them (it ends at offset " +
         std::to_string(end) + ")");
    return false;
  }
  return true;
}

bool active_set_in_range(int pe_start, int log_pe_stride, int pe_size, int num_pes) {
  if (num_pes < 1 || pe_start < 0 || pe_start >= num_pes || log_pe_stride < 0 ||
      log_pe_stride > 30 || pe_size < 1 || pe_size > rocshmem::detail::kMaxPes)
    return false;
  if (pe_size == 1) return true;
  const int64_t last = pe_start + (static_cast<int64_t>(pe_size - 1) << log_pe_stride);
  return last < num_pes;
}

bool device_idle(const char *who) {
  rocshmem::host::Runtime *rt = rocshmem::host::Runtime::get();
  if (rt && rt->persistent_kernel_running()) {
    fail(std::string(who) + ": a live send-queue consumer is running (rsm_sq_consumer_stop first; "
                            "rsm_stream_synchronize waits for one stream)");
    return false;
  }
  const bool idle = rt ? rt->wait_for_device() : hipStreamSynchronize(nullptr) == hipSuccess;
  if (!idle) {
    fail(std::string(who) + ": waiting for the device failed: " + hipGetErrorString(hipGetLastError()));
    return false;
  }
  return true;
}

int after_launch(const char *what) {
  hipError_t e = hipGetLastError();
  if (e != hipSuccess) return fail(std::string(what) + ": " + hipGetErrorString(e));
  return 0;
}

}  // namespace rsm

using rocshmem::host::Options;
using rocshmem::host::Runtime;
namespace detail = rocshmem::detail;

#define RSM_NEED_RT(rt)                                       \
  Runtime *rt = Runtime::get();                               \
  if (!rt) return rsm::fail("rsm_init has not been called")

#define RSM_HIP(expr)                                                              \
  do {                                                                             \
    hipError_t e_ = (expr);                                                        \
    if (e_ != hipSuccess)                                                          \
      return rsm::fail(std::string(#expr " failed: ") + hipGetErrorString(e_));    \
  } while (0)

extern "C" {

int rsm_init(int num_pes, size_t heap_bytes_per_pe, int num_blocks, unsigned sq_size) {
  RSM_ENTRY;
  rsm::clear_error();
  Options o = Options::from_env();
  if (num_pes) o.num_pes = num_pes;
  if (heap_bytes_per_pe) o.heap_size = heap_bytes_per_pe;
  if (num_blocks) o.num_blocks = num_blocks;
  if (sq_size) o.sq_size = sq_size;
  std::string err = Runtime::create(o);
  if (!err.empty()) return rsm::fail(err);
  if (!rsm::noalloc_flags()) {
    Runtime::destroy();
    return -1;
  }
  rocshmem::ROC_SHMEM_TEAM_WORLD =
      reinterpret_cast<rocshmem::roc_shmem_team_t>(Runtime::get()->team_world());
  return 0;
}

int rsm_finalize(void) {
  RSM_ENTRY;
  if (Runtime::get()) rsm::consumer_shutdown();
  Runtime::destroy();
  rocshmem::ROC_SHMEM_TEAM_WORLD = nullptr;
  return 0;
}

int rsm_is_initialized(void) { return Runtime::get() ? 1 : 0; }

const char *rsm_last_error(void) {
  RSM_ENTRY;
  static thread_local std::string copy;
  std::lock_guard<std::mutex> lk(rsm::g_error_mu);
  copy = rsm::g_error;
  return copy.c_str();
}

int rsm_n_pes(void) { return Runtime::get() ? Runtime::get()->num_pes() : -1; }
int rsm_num_blocks(void) { return Runtime::get() ? Runtime::get()->options().num_blocks : -1; }
size_t rsm_heap_size(void) { return Runtime::get() ? Runtime::get()->options().heap_size : 0; }
size_t rsm_slice_stride(void) { return Runtime::get() ? Runtime::get()->slice_stride() : 0; }

void *rsm_malloc(size_t bytes) {
  RSM_ENTRY;
  Runtime *rt = Runtime::get();
  if (!rt) {
    rsm::fail("rsm_init has not been called");
    return nullptr;
  }
  int keep = rt->current_pe();
  rt->set_current_pe(0);
  void *p = rt->sym_malloc(bytes);
  rt->set_current_pe(keep);
  if (!p && bytes) rsm::fail("symmetric heap exhausted");
  return p;
}

int rsm_free(void *ptr) {
  RSM_ENTRY;
  RSM_NEED_RT(rt);
  if (!rsm::device_idle("rsm_free")) return -1;
  return rt->sym_free(ptr) ? 0 : rsm::fail("rsm_free: not an outstanding symmetric allocation");
}

size_t rsm_heap_bytes_in_use(void) { return Runtime::get() ? Runtime::get()->bytes_in_use() : 0; }

void *rsm_ptr(const void *sym, int pe) {
  RSM_ENTRY;
  Runtime *rt = Runtime::get();
  return rt ? rt->translate(sym, pe) : nullptr;
}

void *rsm_heap_base(int pe) {
  RSM_ENTRY;
  Runtime *rt = Runtime::get();
  if (!rt || pe < 0 || pe >= rt->num_pes()) return nullptr;
  return rt->slice_base(pe);
}

int rsm_state_units(void) { return rocshmem::host::registered_state_units(); }

int rsm_take_status(void) {
  RSM_ENTRY;
  RSM_NEED_RT(rt);
  if (rsm::live_consumer_running())
    return rsm::fail("rsm_take_status: a live send-queue consumer is running (rsm_sq_consumer_stop first)");
  return static_cast<int>(rt->take_status());
}

int rsm_set_pacing(unsigned copy_bytes_per_tick, unsigned reduce_bytes_per_tick) {
  RSM_ENTRY;
  RSM_NEED_RT(rt);
  if (rsm::live_consumer_running()) return rsm::fail("rsm_set_pacing: a live send-queue consumer is running");
  if (!rt->set_pacing(copy_bytes_per_tick, reduce_bytes_per_tick))
    return rsm::fail("rsm_set_pacing: could not update the device state");
  return 0;
}

int rsm_get_pacing(unsigned *copy_bytes_per_tick, unsigned *reduce_bytes_per_tick) {
  RSM_ENTRY;
  RSM_NEED_RT(rt);
  if (copy_bytes_per_tick) *copy_bytes_per_tick = rt->device_state().pace_copy_bytes_per_tick;
  if (reduce_bytes_per_tick) *reduce_bytes_per_tick = rt->device_state().pace_reduce_bytes_per_tick;
  return 0;
}

uint64_t rsm_team_world(void) {
  RSM_ENTRY;
  Runtime *rt = Runtime::get();
  return rt ? reinterpret_cast<uint64_t>(rt->team_world()) : 0;
}

int rsm_team_split_strided(uint64_t parent, int start, int stride, int size, uint64_t *new_team) {
  RSM_ENTRY;
  RSM_NEED_RT(rt);
  if (!new_team) return rsm::fail("new_team is NULL");
  detail::Team *out = nullptr;
  int rc = rt->team_split(reinterpret_cast<detail::Team *>(parent), start, stride, size, &out);
  *new_team = reinterpret_cast<uint64_t>(out);
  if (rc != 0) return rsm::fail("team_split_strided: invalid arguments");
  return 0;
}

int rsm_team_destroy(uint64_t team) {
  RSM_ENTRY;
  RSM_NEED_RT(rt);
  if (!rsm::device_idle("rsm_team_destroy")) return -1;
  rt->team_destroy(reinterpret_cast<detail::Team *>(team));
  return 0;
}

int rsm_team_n_pes(uint64_t team) {
  RSM_ENTRY;
  return rocshmem::roc_shmem_team_n_pes(reinterpret_cast<rocshmem::roc_shmem_team_t>(team));
}

int rsm_team_translate_pe(uint64_t src_team, int src_pe, uint64_t dst_team) {
  RSM_ENTRY;
  if (!Runtime::get()) return -1;
  return rocshmem::roc_shmem_team_translate_pe(
      reinterpret_cast<rocshmem::roc_shmem_team_t>(src_team), src_pe,
      reinterpret_cast<rocshmem::roc_shmem_team_t>(dst_team));
}

int rsm_copy_to_device(void *dst, const void *host_src, size_t bytes) {
  RSM_ENTRY;
  RSM_HIP(hipMemcpy(dst, host_src, bytes, hipMemcpyHostToDevice));
  return 0;
}
int rsm_copy_to_host(void *host_dst, const void *src, size_t bytes) {
  RSM_ENTRY;
  RSM_HIP(hipMemcpy(host_dst, src, bytes, hipMemcpyDeviceToHost));
  return 0;
}
int rsm_fill(void *dst, int byte_value, size_t bytes) {
  RSM_ENTRY;
  RSM_HIP(hipMemset(dst, byte_value, bytes));
  return 0;
}
int rsm_synchronize(void) {
  RSM_ENTRY;
  return rsm::device_idle("rsm_synchronize") ? 0 : -1;
}
int rsm_stream_synchronize(void *stream) {
  RSM_ENTRY;
  RSM_HIP(hipStreamSynchronize(static_cast<hipStream_t>(stream)));
  return 0;
}
void *rsm_device_alloc(size_t bytes) {
  RSM_ENTRY;
  void *p = nullptr;
  if (hipMalloc(&p, bytes) != hipSuccess) {
    rsm::fail("hipMalloc failed");
    return nullptr;
  }
  return p;
}
int rsm_device_free(void *ptr) {
  RSM_ENTRY;
  RSM_HIP(hipFree(ptr));
  return 0;
}
void *rsm_stream_create(void) {
  RSM_ENTRY;
  hipStream_t s = nullptr;
  if (hipStreamCreate(&s) != hipSuccess) {
    rsm::fail("hipStreamCreate failed");
    return nullptr;
  }
  return s;
}
int rsm_stream_destroy(void *stream) {
  RSM_ENTRY;
  RSM_HIP(hipStreamDestroy(static_cast<hipStream_t>(stream)));
  return 0;
}
void *rsm_event_create(void) {
  RSM_ENTRY;
  hipEvent_t e = nullptr;
  if (hipEventCreate(&e) != hipSuccess) {
    rsm::fail("hipEventCreate failed");
    return nullptr;
  }
  return e;
}
int rsm_event_destroy(void *event) {
  RSM_ENTRY;
  RSM_HIP(hipEventDestroy(static_cast<hipEvent_t>(event)));
  return 0;
}
int rsm_event_record(void *event, void *stream) {
  RSM_ENTRY;
  RSM_HIP(hipEventRecord(static_cast<hipEvent_t>(event), static_cast<hipStream_t>(stream)));
  return 0;
}
int rsm_event_elapsed_ms(void *start, void *stop, float *ms) {
  RSM_ENTRY;
  RSM_HIP(hipEventSynchronize(static_cast<hipEvent_t>(stop)));
  RSM_HIP(hipEventElapsedTime(ms, static_cast<hipEvent_t>(start), static_cast<hipEvent_t>(stop)));
  return 0;
}

// ---- graphs --------------------------------------------------------------------
// The data-path entry points only launch kernels on launch->stream, so a run of
// them can be recorded once and replayed as one submission.

int rsm_capture_begin(void *stream) {
  RSM_ENTRY;
  if (!stream) return rsm::fail("rsm_capture_begin: capture needs a stream of its own, not the default stream");
  RSM_HIP(hipStreamBeginCapture(static_cast<hipStream_t>(stream), hipStreamCaptureModeThreadLocal));
  return 0;
}

void *rsm_capture_end(void *stream) {
  RSM_ENTRY;
  hipGraph_t graph = nullptr;
  hipError_t e = hipStreamEndCapture(static_cast<hipStream_t>(stream), &graph);
  if (e != hipSuccess || !graph) {
    rsm::fail(std::string("rsm_capture_end: ") + hipGetErrorString(e));
    return nullptr;
  }
  hipGraphExec_t exec = nullptr;
  e = hipGraphInstantiate(&exec, graph, nullptr, nullptr, 0);
  (void)hipGraphDestroy(graph);
  if (e != hipSuccess) {
    rsm::fail(std::string("rsm_capture_end: hipGraphInstantiate: ") + hipGetErrorString(e));
    return nullptr;
  }
  return exec;
}

int rsm_graph_launch(void *graph, void *stream) {
  RSM_ENTRY;
  RSM_HIP(hipGraphLaunch(static_cast<hipGraphExec_t>(graph), static_cast<hipStream_t>(stream)));
  return 0;
}

int rsm_graph_destroy(void *graph) {
  RSM_ENTRY;
  RSM_HIP(hipGraphExecDestroy(static_cast<hipGraphExec_t>(graph)));
  return 0;
}

// ---- send-queue inspection ---------------------------------------------------

static bool sq_args_ok(Runtime *rt, int pe, int block) {
  return pe >= 0 && pe < rt->num_pes() && block >= 0 && block < rt->options().num_blocks;
}

int rsm_sq_reset(void) {
  RSM_ENTRY;
  RSM_NEED_RT(rt);
  if (!rsm::device_idle("rsm_sq_reset")) return -1;
  rt->reset_queues(nullptr);
  return rsm::device_idle("rsm_sq_reset") ? 0 : -1;
}

int rsm_sq_read(int pe, int block, unsigned index, uint64_t out_words[8]) {
  RSM_ENTRY;
  RSM_NEED_RT(rt);
  if (!sq_args_ok(rt, pe, block) || index >= rt->options().sq_size)
    return rsm::fail("rsm_sq_read: arguments out of range");
  if (!rsm::device_idle("rsm_sq_read")) return -1;
  RSM_HIP(hipMemcpy(out_words, rt->ctx_image(pe, block).ring.sq + 8ull * index, 64,
                    hipMemcpyDeviceToHost));
  return 0;
}

int rsm_sq_image(int pe, int block, void *host_out, size_t bytes) {
  RSM_ENTRY;
  RSM_NEED_RT(rt);
  if (!sq_args_ok(rt, pe, block) || bytes > 64ull * rt->options().sq_size)
    return rsm::fail("rsm_sq_image: arguments out of range");
  if (!rsm::device_idle("rsm_sq_image")) return -1;
  RSM_HIP(hipMemcpy(host_out, rt->ctx_image(pe, block).ring.sq, bytes, hipMemcpyDeviceToHost));
  return 0;
}

int rsm_sq_state(int pe, int block, uint32_t *sq_counter, uint32_t *published,
                 uint32_t *atomic_counter, uint64_t mailbox[2]) {
  RSM_ENTRY;
  RSM_NEED_RT(rt);
  if (!sq_args_ok(rt, pe, block)) return rsm::fail("rsm_sq_state: arguments out of range");
  if (!rsm::device_idle("rsm_sq_state")) return -1;
  detail::SqCounters c;
  const detail::DeviceCtx &ctx = rt->ctx_image(pe, block);
  RSM_HIP(hipMemcpy(&c, ctx.counters, sizeof(c), hipMemcpyDeviceToHost));
  if (sq_counter) *sq_counter = c.sq_counter;
  if (published) *published = c.published;
  if (atomic_counter) *atomic_counter = c.atomic_counter;
  if (mailbox) RSM_HIP(hipMemcpy(mailbox, ctx.ring.mailbox, 16, hipMemcpyDeviceToHost));
  return 0;
}

int rsm_sq_constants(int pe, int block, uint32_t *ctrl_qp_sq, uint64_t *ctrl_sig, uint32_t *lkey,
                     uint32_t *atomic_lkey, uint64_t *atomic_ret_base, uint32_t *max_nwqe) {
  RSM_ENTRY;
  RSM_NEED_RT(rt);
  if (!sq_args_ok(rt, pe, block)) return rsm::fail("rsm_sq_constants: arguments out of range");
  const detail::SqRing &r = rt->ctx_image(pe, block).ring;
  if (ctrl_qp_sq) *ctrl_qp_sq = r.ctrl_qp_sq;
  if (ctrl_sig) *ctrl_sig = r.ctrl_sig;
  if (lkey) *lkey = r.lkey;
  if (atomic_lkey) *atomic_lkey = r.atomic_lkey;
  if (atomic_ret_base) *atomic_ret_base = r.atomic_ret_base;
  if (max_nwqe) *max_nwqe = r.max_nwqe;
  return 0;
}

int rsm_sq_rkey(int dest_pe, uint32_t *rkey) {
  RSM_ENTRY;
  RSM_NEED_RT(rt);
  if (dest_pe < 0 || dest_pe >= rt->num_pes() || !rkey)
    return rsm::fail("rsm_sq_rkey: arguments out of range");
  *rkey = __builtin_bswap32(0x1000u + dest_pe);
  return 0;
}

int rsm_sq_flush_target(int pe, uint64_t *addr, uint32_t *rkey) {
  RSM_ENTRY;
  RSM_NEED_RT(rt);
  if (pe < 0 || pe >= rt->num_pes() || !addr || !rkey)
    return rsm::fail("rsm_sq_flush_target: arguments out of range");
  *addr = reinterpret_cast<uint64_t>(rt->flush_words()) + 64ull * static_cast<uint64_t>(pe);
  *rkey = __builtin_bswap32(0x4000u + pe);
  return 0;
}

// ---- host-logic hooks ------------------------------------------------------------

int rsm_host_active_set_in_range(int pe_start, int log_pe_stride, int pe_size, int num_pes) {
  return rsm::active_set_in_range(pe_start, log_pe_stride, pe_size, num_pes) ? 1 : 0;
}

void *rsm_host_alloc_create(size_t heap_bytes) {
  RSM_ENTRY;
  return new rocshmem::host::Pow2Allocator(heap_bytes);
}
void rsm_host_alloc_destroy(void *allocator) {
  RSM_ENTRY;
  delete static_cast<rocshmem::host::Pow2Allocator *>(allocator);
}
size_t rsm_host_alloc_alloc(void *allocator, size_t request) {
  RSM_ENTRY;
  return static_cast<rocshmem::host::Pow2Allocator *>(allocator)->alloc(request);
}
int rsm_host_alloc_free(void *allocator, size_t offset) {
  RSM_ENTRY;
  return static_cast<rocshmem::host::Pow2Allocator *>(allocator)->free(offset) ? 0 : -1;
}
size_t rsm_host_alloc_in_use(void *allocator) {
  RSM_ENTRY;
  return static_cast<rocshmem::host::Pow2Allocator *>(allocator)->bytes_in_use();
}

}  // extern "C"
