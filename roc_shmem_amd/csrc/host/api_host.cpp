// Host half of the roc_shmem_* interface (reference: library/src/roc_shmem.cpp).
// Failures print to stderr and end the process, as the reference's CHECK_HIP /
// VERIFY_BACKEND do (library/src/util.hpp:89-97, roc_shmem.cpp:54-61).
#include <cstdio>
#include <cstdlib>

#include "roc_shmem.hpp"
#include "runtime.hpp"

namespace rocshmem {

roc_shmem_team_t ROC_SHMEM_TEAM_WORLD = nullptr;

namespace {
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
  host::Runtime *rt = runtime_or_die("roc_shmem_malloc");
  void *p = rt->sym_malloc(size);
  roc_shmem_barrier_all();  // reference: barrier after every allocation, roc_shmem.cpp:118-126
  return p;
}

__host__ void roc_shmem_free(void *ptr) {
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
  host::Runtime *rt = runtime_or_die("roc_shmem_team_split_strided");
  *new_team = ROC_SHMEM_TEAM_INVALID;
  detail::Team *out = nullptr;
  int rc = rt->team_split(reinterpret_cast<detail::Team *>(parent_team), start, stride, size, &out);
  if (rc == 0) *new_team = reinterpret_cast<roc_shmem_team_t>(out);
  return rc;
}

__host__ void roc_shmem_team_destroy(roc_shmem_team_t team) {
  if (team == ROC_SHMEM_TEAM_INVALID || team == ROC_SHMEM_TEAM_WORLD) return;
  runtime_or_die("roc_shmem_team_destroy")->team_destroy(reinterpret_cast<detail::Team *>(team));
}

// Every PE is this process: the host-side barrier is "all device work has finished".
__host__ void roc_shmem_barrier_all() {
  runtime_or_die("roc_shmem_barrier_all");
  (void)hipDeviceSynchronize();
}
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
  (void)hipDeviceSynchronize();
  (void)hipMemcpy(words, c.ring.sq + 8ull * index_wqe, sizeof(words), hipMemcpyDeviceToHost);
  printf("SQ pe %d block %d entry %d:", dest_pe, src_wg, index_wqe);
  for (int i = 0; i < 8; ++i) printf(" %016llx", static_cast<unsigned long long>(words[i]));
  printf("\n");
}

__host__ void debug_print_cq(int, int, int) {
  printf("CQ: this build has no completion queue (operations complete in program order)\n");
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

}  // namespace rocshmem
