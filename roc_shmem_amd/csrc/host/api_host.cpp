// Host half of the roc_shmem_* interface (reference: library/src/roc_shmem.cpp).
// Failures print to stderr and end the process, as the reference's CHECK_HIP /
// VERIFY_BACKEND do (library/src/util.hpp:89-97, roc_shmem.cpp:54-61).
#include <cstdio>
#include <cstdlib>
#include <mutex>

#include "roc_shmem.hpp"
#include "rocshmem_mi355x.h"
#include "runtime.hpp"

namespace rocshmem {

roc_shmem_team_t ROC_SHMEM_TEAM_WORLD = nullptr;

namespace {
// The host interface reports ROC_SHMEM_THREAD_MULTIPLE: calls that change
// library state (allocator, teams, read-modify-write emulation of the AMOs,
// the shared pSync of host collectives) are serialised here.
std::recursive_mutex g_host_lock;
#define HOST_LOCKED std::lock_guard<std::recursive_mutex> host_guard_(g_host_lock)

host::Runtime *runtime_or_die(const char *fn) {
  host::Runtime *rt = host::Runtime::get();
  if (!rt) {
    fprintf(stderr, "rocshmem: %s called before roc_shmem_init\n", fn);
    abort();
  }
  return rt;
}
}  // namespace

__host__ void roc_shmem_init(MPI_Comm) {
  std::string err = host::Runtime::create(host::Options::from_env());
  if (!err.empty()) {
    fprintf(stderr, "rocshmem: init failed: %s\n", err.c_str());
    exit(EXIT_FAILURE);
  }
  ROC_SHMEM_TEAM_WORLD = reinterpret_cast<roc_shmem_team_t>(host::Runtime::get()->team_world());
}

__host__ void roc_shmem_init_thread(int, int *provided, MPI_Comm comm) {
  roc_shmem_init(comm);
  roc_shmem_query_thread(provided);
}

__host__ void roc_shmem_query_thread(int *provided) { *provided = ROC_SHMEM_THREAD_MULTIPLE; }

__host__ void roc_shmem_finalize() {
  host::Runtime::destroy();
  ROC_SHMEM_TEAM_WORLD = nullptr;
}

// Counters are collected with rocprofv3, not by the library.
__host__ void roc_shmem_dump_stats() {}
__host__ void roc_shmem_reset_stats() {}

__host__ void roc_shmem_global_exit(int status) {
  host::Runtime::destroy();
  exit(status);
}

__host__ void *roc_shmem_malloc(size_t size) {
  HOST_LOCKED;
  host::Runtime *rt = runtime_or_die("roc_shmem_malloc");
  void *p = rt->sym_malloc(size);
  roc_shmem_barrier_all();  // reference: barrier after every allocation, roc_shmem.cpp:118-126
  return p;
}

__host__ void roc_shmem_free(void *ptr) {
  HOST_LOCKED;
  host::Runtime *rt = runtime_or_die("roc_shmem_free");
  roc_shmem_barrier_all();
  rt->sym_free(ptr);
}

__host__ int roc_shmem_n_pes() { return runtime_or_die("roc_shmem_n_pes")->num_pes(); }
__host__ int roc_shmem_my_pe() { return runtime_or_die("roc_shmem_my_pe")->current_pe(); }

__host__ int roc_shmem_ctx_create(int64_t, roc_shmem_ctx_t *ctx) {
  runtime_or_die("roc_shmem_ctx_create");
  ctx->ctx_opaque = nullptr;  // "the context of the calling PE"
  ctx->team_opaque = nullptr;
  return 0;
}
__host__ void roc_shmem_ctx_destroy(roc_shmem_ctx_t) {}

__host__ int roc_shmem_team_n_pes(roc_shmem_team_t team) {
  if (team == ROC_SHMEM_TEAM_INVALID) return -1;
  const host::TeamRecord *r =
      runtime_or_die("roc_shmem_team_n_pes")->team_record(reinterpret_cast<detail::Team *>(team));
  return r ? r->image.wrt_world.size : -1;
}

__host__ int roc_shmem_team_my_pe(roc_shmem_team_t team) {
  if (team == ROC_SHMEM_TEAM_INVALID) return -1;
  host::Runtime *rt = runtime_or_die("roc_shmem_team_my_pe");
  const host::TeamRecord *r = rt->team_record(reinterpret_cast<detail::Team *>(team));
  if (!r) return -1;
  const detail::TeamInfo &t = r->image.wrt_world;
  int pe = rt->current_pe();
  if (pe < t.pe_start || (pe - t.pe_start) % t.stride) return -1;
  int idx = (pe - t.pe_start) / t.stride;
  return idx < t.size ? idx : -1;
}

__host__ int roc_shmem_team_translate_pe(roc_shmem_team_t src_team, int src_pe,
                                         roc_shmem_team_t dest_team) {
  if (src_team == ROC_SHMEM_TEAM_INVALID || dest_team == ROC_SHMEM_TEAM_INVALID) return -1;
  host::Runtime *rt = runtime_or_die("roc_shmem_team_translate_pe");
  const host::TeamRecord *s = rt->team_record(reinterpret_cast<detail::Team *>(src_team));
  const host::TeamRecord *d = rt->team_record(reinterpret_cast<detail::Team *>(dest_team));
  if (!s || !d) return -1;
  const detail::TeamInfo &si = s->image.wrt_world;
  const detail::TeamInfo &di = d->image.wrt_world;
  int in_world = si.pe_start + si.stride * src_pe;
  if (in_world < di.pe_start || (in_world - di.pe_start) % di.stride) return -1;
  int idx = (in_world - di.pe_start) / di.stride;
  return idx < di.size ? idx : -1;
}

__host__ int roc_shmem_team_split_strided(roc_shmem_team_t parent_team, int start, int stride,
                                          int size, const roc_shmem_team_config_t *, long,
                                          roc_shmem_team_t *new_team) {
  HOST_LOCKED;
  host::Runtime *rt = runtime_or_die("roc_shmem_team_split_strided");
  *new_team = ROC_SHMEM_TEAM_INVALID;
  detail::Team *out = nullptr;
  int rc = rt->team_split(reinterpret_cast<detail::Team *>(parent_team), start, stride, size, &out);
  if (rc == 0) *new_team = reinterpret_cast<roc_shmem_team_t>(out);
  return rc;
}

__host__ void roc_shmem_team_destroy(roc_shmem_team_t team) {
  HOST_LOCKED;
  if (team == ROC_SHMEM_TEAM_INVALID || team == ROC_SHMEM_TEAM_WORLD) return;
  runtime_or_die("roc_shmem_team_destroy")->team_destroy(reinterpret_cast<detail::Team *>(team));
}

// Every PE is this process: the host-side barrier is "all device work has finished".
// (While a kernel runs that ends only when told to - the live send-queue consumer, started
// through the C interface - the wait covers the default stream, on which this interface
// launches; the whole device would not go idle.)
static void wait_for_work(host::Runtime *rt) {
  if (!rt->wait_for_device()) (void)hipStreamSynchronize(nullptr);
}
__host__ void roc_shmem_barrier_all() { wait_for_work(runtime_or_die("roc_shmem_barrier_all")); }
__host__ void roc_shmem_sync_all() { roc_shmem_barrier_all(); }
__host__ void roc_shmem_quiet() { roc_shmem_barrier_all(); }
__host__ void roc_shmem_fence() {}

__host__ void debug_print_sq(int dest_pe, int src_wg, int index_wqe) {
  host::Runtime *rt = runtime_or_die("debug_print_sq");
  if (dest_pe < 0 || dest_pe >= rt->num_pes() || src_wg < 0 ||
      src_wg >= rt->options().num_blocks || index_wqe < 0 ||
      static_cast<uint32_t>(index_wqe) >= rt->options().sq_size) {
    fprintf(stderr, "debug_print_sq: arguments out of range\n");
    return;
  }
  uint64_t words[8];
  const detail::DeviceCtx &c = rt->ctx_image(dest_pe, src_wg);
  wait_for_work(rt);
  (void)hipMemcpy(words, c.ring.sq + 8ull * index_wqe, sizeof(words), hipMemcpyDeviceToHost);
  printf("SQ pe %d block %d entry %d:", dest_pe, src_wg, index_wqe);
  for (int i = 0; i < 8; ++i) printf(" %016llx", static_cast<unsigned long long>(words[i]));
  printf("\n");
}

__host__ void debug_print_cq(int dest_pe, int src_wg, int cqe_num) {
  host::Runtime *rt = runtime_or_die("debug_print_cq");
  if (dest_pe < 0 || dest_pe >= rt->num_pes() || src_wg < 0 ||
      src_wg >= rt->options().num_blocks || cqe_num < 0 ||
      static_cast<uint32_t>(cqe_num) >= rt->options().sq_size) {
    fprintf(stderr, "debug_print_cq: arguments out of range\n");
    return;
  }
  // Completion entries are written by the consumer pass (rsm_sq_consume).
  uint64_t words[8];
  const detail::DeviceCtx &c = rt->ctx_image(dest_pe, src_wg);
  wait_for_work(rt);
  (void)hipMemcpy(words, c.ring.cq + 8ull * cqe_num, sizeof(words), hipMemcpyDeviceToHost);
  printf("CQ pe %d block %d entry %d:", dest_pe, src_wg, cqe_num);
  for (int i = 0; i < 8; ++i) printf(" %016llx", static_cast<unsigned long long>(words[i]));
  printf("\n");
}

__host__ void roc_shmemx_set_pe(int pe) {
  host::Runtime *rt = runtime_or_die("roc_shmemx_set_pe");
  if (pe < 0 || pe >= rt->num_pes()) {
    fprintf(stderr, "roc_shmemx_set_pe: PE %d out of range\n", pe);
    abort();
  }
  rt->set_current_pe(pe);
}

__host__ void *roc_shmemx_host_ptr(const void *ptr, int pe) {
  return runtime_or_die("roc_shmemx_host_ptr")->translate(ptr, pe);
}

__host__ int roc_shmemx_take_status() {
  return static_cast<int>(runtime_or_die("roc_shmemx_take_status")->take_status());
}

// ---------------------------------------------------------------------------
// Host-initiated data path (see include/roc_shmem_host.hpp)
// ---------------------------------------------------------------------------

namespace hostx {

namespace {
void die(const char *what) {
  fprintf(stderr, "rocshmem: %s: %s\n", what, rsm_last_error());
  exit(EXIT_FAILURE);
}
void check_hip(hipError_t e, const char *what) {
  if (e != hipSuccess) {
    fprintf(stderr, "rocshmem: %s: %s\n", what, hipGetErrorString(e));
    exit(EXIT_FAILURE);  // reference: CHECK_HIP, library/src/util.hpp:89-97
  }
}
// Address of a symmetric object in PE `pe`'s slice; aborts when `sym` is not symmetric.
void *remote_of(host::Runtime *rt, const void *sym, int pe, const char *fn) {
  void *p = rt->translate(sym, pe);
  if (!p) {
    fprintf(stderr, "rocshmem: %s: not a symmetric address / PE out of range\n", fn);
    abort();
  }
  return p;
}
// Launch shape of host-initiated collectives, from sweeps over 4, 8 and 16 PEs and 64 KiB to
// 256 MiB per PE.  Reductions read as much as they write and every workgroup walks all members:
// about 64 KiB of each member's array per workgroup, at least 4 workgroups from 128 KiB up, at
// most one per CU, 1024 lanes once the arrays stream (32 MiB).  A broadcast almost only writes:
// one workgroup below 512 KiB, 16 up to 8 MiB, then one of 1024 lanes per second CU.  Never
// more workgroups per PE than the library has contexts (pSync slices) for.  `members` PEs take
// part; the grid has workgroups for every PE, and those of the others return at once.
rsm_launch_t collective_launch(host::Runtime *rt, size_t bytes, bool broadcast, int members) {
  rsm_launch_t l;
  const int pes = members < 1 ? 1 : members;
  int per_pe, wg_size;
  if (broadcast) {
    if (bytes < (512u << 10)) {
      per_pe = 1, wg_size = 512;
    } else if (bytes < (8u << 20)) {
      per_pe = 16, wg_size = 512;
    } else {
      per_pe = 128 / pes, wg_size = 1024;
    }
  } else {
    const size_t want = bytes / (static_cast<size_t>(65536) * pes);
    per_pe = 1;
    while (static_cast<size_t>(per_pe) * 2 <= want && per_pe * 2 * pes <= 256) per_pe *= 2;
    if (per_pe < 4 && bytes >= (128u << 10)) per_pe = 4;
    wg_size = bytes < (32u << 20) ? 512 : 1024;
  }
  if (per_pe * rt->num_pes() > 2048) per_pe = 2048 / rt->num_pes();
  if (per_pe > rt->options().num_blocks) per_pe = rt->options().num_blocks;
  if (per_pe < 1) per_pe = 1;
  l.wgs_per_pe = per_pe;
  l.wg_size = wg_size;
  l.tile = 0;
  l.stream = nullptr;
  return l;
}
// A host-initiated collective returns only when its kernel has finished, and a kernel whose flag
// waits gave up has produced incomplete results: fail like the library's other fatal errors
// rather than hand them back with a normal return (take_status also puts the barrier pools
// back in order, which matters to a caller that catches the exit in a test harness only).
void finish_collective(host::Runtime *rt, const char *what) {
  wait_for_work(rt);
  check_hip(hipGetLastError(), what);
  const uint32_t status = rt->take_status();
  if (status != 0) {
    fprintf(stderr,
            "rocshmem: %s: the device raised status %u (%s); the results are incomplete\n", what,
            status,
            status == detail::kStatusWaitTimeout
                ? "a flag wait gave up after ROC_SHMEM_WAIT_LIMIT_S seconds"
                : "an argument was refused on the device");
    exit(EXIT_FAILURE);
  }
}
size_t reduce_elem_size(int dtype) {
  switch (dtype) {
    case RSM_SHORT: case RSM_BF16: return 2;
    case RSM_INT: case RSM_FLOAT: return 4;
    default: return 8;
  }
}
}  // namespace

void putmem(void *dest, const void *source, size_t nbytes, int pe, bool blocking) {
  if (!nbytes) return;
  host::Runtime *rt = runtime_or_die("roc_shmem_putmem");
  void *remote = remote_of(rt, dest, pe, "roc_shmem_putmem");
  if (blocking) {
    check_hip(hipMemcpy(remote, source, nbytes, hipMemcpyDefault), "roc_shmem_putmem");
  } else {
    check_hip(hipMemcpyAsync(remote, source, nbytes, hipMemcpyDefault, nullptr),
              "roc_shmem_putmem_nbi");
  }
}

void getmem(void *dest, const void *source, size_t nbytes, int pe, bool blocking) {
  if (!nbytes) return;
  host::Runtime *rt = runtime_or_die("roc_shmem_getmem");
  const void *remote = remote_of(rt, source, pe, "roc_shmem_getmem");
  if (blocking) {
    check_hip(hipMemcpy(dest, remote, nbytes, hipMemcpyDefault), "roc_shmem_getmem");
  } else {
    check_hip(hipMemcpyAsync(dest, remote, nbytes, hipMemcpyDefault, nullptr),
              "roc_shmem_getmem_nbi");
  }
}

uint64_t fetch_own(const void *ptr, int width) {
  host::Runtime *rt = runtime_or_die("roc_shmem_test");
  const void *mine = remote_of(rt, ptr, rt->current_pe(), "roc_shmem_test");
  if (reinterpret_cast<uintptr_t>(mine) & static_cast<uintptr_t>(width - 1)) {
    fprintf(stderr, "rocshmem: roc_shmem_test: the word is not naturally aligned\n");
    abort();
  }
  uint64_t bits = 0;
  if (rt->options().heap_host_visible) {
    // The arena is host-visible: one atomic load over the bus sees what a
    // kernel that is still running has stored with device or system scope.
    switch (width) {
      case 1: bits = __atomic_load_n(static_cast<const uint8_t *>(mine), __ATOMIC_ACQUIRE); break;
      case 2: bits = __atomic_load_n(static_cast<const uint16_t *>(mine), __ATOMIC_ACQUIRE); break;
      case 4: bits = __atomic_load_n(static_cast<const uint32_t *>(mine), __ATOMIC_ACQUIRE); break;
      default: bits = __atomic_load_n(static_cast<const uint64_t *>(mine), __ATOMIC_ACQUIRE); break;
    }
  } else {
    // Plain device memory: a copy on the null stream, which runs after the
    // kernels launched before it.
    check_hip(hipMemcpy(&bits, mine, width, hipMemcpyDeviceToHost), "roc_shmem_test");
  }
  return bits;
}

double wait_limit_seconds() { return runtime_or_die("roc_shmem_wait_until")->options().wait_limit_s; }

uint64_t amo(int kind, void *dest, uint64_t value, uint64_t cond, int pe, int width) {
  HOST_LOCKED;
  host::Runtime *rt = runtime_or_die("roc_shmem_atomic");
  void *remote = remote_of(rt, dest, pe, "roc_shmem_atomic");
  const uint64_t mask = width == 8 ? ~0ull : 0xffffffffull;
  uint64_t old = 0;
  wait_for_work(rt);
  check_hip(hipMemcpy(&old, remote, width, hipMemcpyDeviceToHost), "roc_shmem_atomic");
  uint64_t next = old;
  switch (kind) {
    case 0: next = (old + value) & mask; break;
    case 1: if (old == (cond & mask)) next = value & mask; break;
    case 2: next = value & mask; break;
    case 3: next = old & value; break;
    case 4: next = (old | value) & mask; break;
    default: next = (old ^ value) & mask; break;
  }
  if (next != old) check_hip(hipMemcpy(remote, &next, width, hipMemcpyHostToDevice), "roc_shmem_atomic");
  return old;
}

namespace {
// Library-owned pSync for host-initiated active-set collectives.
long *host_psync(host::Runtime *rt) {
  long *psync = rt->host_psync();
  if (!psync) {
    fprintf(stderr, "rocshmem: no room for the host collectives' pSync\n");
    abort();
  }
  return psync;
}
}  // namespace

void to_all(int dtype, int op, void *dest, const void *source, int nreduce, int pe_start,
            int log_pe_stride, int pe_size) {
  HOST_LOCKED;
  if (nreduce <= 0) return;
  host::Runtime *rt = runtime_or_die("roc_shmem_to_all");
  rsm_launch_t l = collective_launch(rt, static_cast<size_t>(nreduce) * reduce_elem_size(dtype),
                                     false, pe_size);
  if (rsm_to_all(dtype, op, remote_of(rt, dest, 0, "roc_shmem_to_all"),
                 remote_of(rt, source, 0, "roc_shmem_to_all"), static_cast<size_t>(nreduce),
                 pe_start, log_pe_stride, pe_size, nullptr, host_psync(rt), &l))
    die("roc_shmem_to_all");
  finish_collective(rt, "roc_shmem_to_all");
}

void to_all_team(int dtype, int op, roc_shmem_team_t team, void *dest, const void *source,
                 int nreduce) {
  if (nreduce <= 0 || team == ROC_SHMEM_TEAM_INVALID) return;
  host::Runtime *rt = runtime_or_die("roc_shmem_to_all");
  rsm_launch_t l = collective_launch(rt, static_cast<size_t>(nreduce) * reduce_elem_size(dtype),
                                     false, roc_shmem_team_n_pes(team));
  if (rsm_to_all_team(dtype, op, reinterpret_cast<uint64_t>(team),
                      remote_of(rt, dest, 0, "roc_shmem_to_all"),
                      remote_of(rt, source, 0, "roc_shmem_to_all"),
                      static_cast<size_t>(nreduce), &l))
    die("roc_shmem_to_all");
  finish_collective(rt, "roc_shmem_to_all");
}

void broadcast(size_t elem_size, void *dest, const void *source, int nelem, int pe_root,
               int pe_start, int log_pe_stride, int pe_size) {
  HOST_LOCKED;
  if (nelem <= 0) return;
  host::Runtime *rt = runtime_or_die("roc_shmem_broadcast");
  rsm_launch_t l = collective_launch(rt, static_cast<size_t>(nelem) * elem_size, true, pe_size);
  if (rsm_broadcast(elem_size, remote_of(rt, dest, 0, "roc_shmem_broadcast"),
                    remote_of(rt, source, 0, "roc_shmem_broadcast"), static_cast<size_t>(nelem),
                    pe_root, pe_start, log_pe_stride, pe_size, host_psync(rt), &l))
    die("roc_shmem_broadcast");
  finish_collective(rt, "roc_shmem_broadcast");
}

void broadcast_team(size_t elem_size, roc_shmem_team_t team, void *dest, const void *source,
                    int nelem, int pe_root) {
  if (nelem <= 0 || team == ROC_SHMEM_TEAM_INVALID) return;
  host::Runtime *rt = runtime_or_die("roc_shmem_broadcast");
  rsm_launch_t l = collective_launch(rt, static_cast<size_t>(nelem) * elem_size, true,
                                     roc_shmem_team_n_pes(team));
  if (rsm_broadcast_team(elem_size, reinterpret_cast<uint64_t>(team),
                         remote_of(rt, dest, 0, "roc_shmem_broadcast"),
                         remote_of(rt, source, 0, "roc_shmem_broadcast"),
                         static_cast<size_t>(nelem), pe_root, &l))
    die("roc_shmem_broadcast");
  finish_collective(rt, "roc_shmem_broadcast");
}

}  // namespace hostx

}  // namespace rocshmem
