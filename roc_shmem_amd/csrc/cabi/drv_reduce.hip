// C ABI: reductions.  The kernels below drive the device API the way the
// reference's ReductionTest kernel does (clients/functional_tests/
// reduction_tester.cpp:74-104), for every PE of the job in one grid.
#include "cabi_common.hpp"
#include "roc_shmem.hpp"

using namespace rocshmem;

namespace {

template <typename T, ROC_SHMEM_OP Op>
struct ToAll;

#define RSM_TO_ALL(T, TNAME, OPNAME, OP)                                                      \
  template <>                                                                                 \
  struct ToAll<T, OP> {                                                                       \
    static __device__ __forceinline__ void active_set(roc_shmem_ctx_t ctx, T *dest,           \
                                                      const T *source, int n, int pe_start,   \
                                                      int log_stride, int pe_size, T *pWrk,   \
                                                      long *pSync) {                          \
      roc_shmem_ctx_##TNAME##_##OPNAME##_wg_to_all(ctx, dest, source, n, pe_start,            \
                                                   log_stride, pe_size, pWrk, pSync);         \
    }                                                                                         \
    static __device__ __forceinline__ void team(roc_shmem_ctx_t ctx, roc_shmem_team_t team,   \
                                                T *dest, const T *source, int n) {            \
      roc_shmem_ctx_##TNAME##_##OPNAME##_wg_to_all(ctx, team, dest, source, n);               \
    }                                                                                         \
    static __device__ __forceinline__ void active_set_shard(                                  \
        roc_shmem_ctx_t ctx, T *dest, const T *source, size_t n, int pe_start, int log_stride, \
        int pe_size, T *pWrk, long *pSync, int shard, int nshards) {                          \
      roc_shmemx_ctx_##TNAME##_##OPNAME##_wg_to_all_shard(ctx, dest, source, n, pe_start,     \
                                                          log_stride, pe_size, pWrk, pSync,   \
                                                          shard, nshards);                    \
    }                                                                                         \
    static __device__ __forceinline__ void team_shard(roc_shmem_ctx_t ctx,                    \
                                                      roc_shmem_team_t team, T *dest,         \
                                                      const T *source, size_t n, int shard,   \
                                                      int nshards) {                          \
      roc_shmemx_ctx_##TNAME##_##OPNAME##_wg_to_all_shard(ctx, team, dest, source, n, shard,  \
                                                          nshards);                           \
    }                                                                                         \
  };
#define RSM_TO_ALL_ARITH(T, TNAME)            \
  RSM_TO_ALL(T, TNAME, sum, ROC_SHMEM_SUM)    \
  RSM_TO_ALL(T, TNAME, max, ROC_SHMEM_MAX)    \
  RSM_TO_ALL(T, TNAME, min, ROC_SHMEM_MIN)    \
  RSM_TO_ALL(T, TNAME, prod, ROC_SHMEM_PROD)
#define RSM_TO_ALL_BITS(T, TNAME)             \
  RSM_TO_ALL(T, TNAME, and, ROC_SHMEM_AND)    \
  RSM_TO_ALL(T, TNAME, or, ROC_SHMEM_OR)      \
  RSM_TO_ALL(T, TNAME, xor, ROC_SHMEM_XOR)
RSM_TO_ALL_ARITH(short, short)
RSM_TO_ALL_BITS(short, short)
RSM_TO_ALL_ARITH(int, int)
RSM_TO_ALL_BITS(int, int)
RSM_TO_ALL_ARITH(long, long)
RSM_TO_ALL_BITS(long, long)
RSM_TO_ALL_ARITH(long long, longlong)
RSM_TO_ALL_BITS(long long, longlong)
RSM_TO_ALL_ARITH(float, float)
RSM_TO_ALL_ARITH(double, double)
RSM_TO_ALL(__hip_bfloat16, bf16, sum, ROC_SHMEM_SUM)
RSM_TO_ALL(__hip_bfloat16, bf16, max, ROC_SHMEM_MAX)
RSM_TO_ALL(__hip_bfloat16, bf16, min, ROC_SHMEM_MIN)

// Flag scratch of rsm_to_all_noalloc: room for kNoAllocMaxWgs workgroups' flag
// slices (ROC_SHMEM_REDUCE_SYNC_SIZE longs each, 4 MiB in all), laid out PE-major
// ([pe][workgroup][256]) so that two PEs' copies of a workgroup's slice are a fixed
// number of bytes apart, as the copies of a symmetric pSync are.  Every device that
// loads the library holds its own copy until the process ends.  In host code this
// name is a stand-in, not a device address: host code uses the address that
// hipGetSymbolAddress returned (noalloc_flags()).
constexpr unsigned kNoAllocMaxWgs = 2048;
static __device__ __align__(256) long g_noalloc_flags[kNoAllocMaxWgs * ROC_SHMEM_REDUCE_SYNC_SIZE];

__global__ void __launch_bounds__(256) clear_flags_kernel(long *flags, size_t n) {
  const size_t i = static_cast<size_t>(blockIdx.x) * blockDim.x + threadIdx.x;
  if (i < n) flags[i] = ROC_SHMEM_SYNC_VALUE;
}

// Forms of the reduction kernel.  kTiled: one standard call per tile, tiles dealt
// round-robin to the PE's workgroups.  kSharded: the PE's workgroups share one reduction
// (sharded extension), pSync is the caller's symmetric array.  kShardedStaticFlags: the
// same with the flags in the library's own array (`pSync0` is its device address).  Separate
// kernels rather than branches: with more than one form inlined into one kernel the compiler
// ran out of scalar registers.
// kShardedLds: the sharded form with the loads staged through dynamic LDS (a measured
// alternative, built for the three benchmark reductions only; see reduce_vectors_lds).
enum ToAllForm { kTiled = 0, kSharded = 1, kShardedStaticFlags = 2, kShardedLds = 3 };

template <typename T, ROC_SHMEM_OP Op, int kForm>
__global__ void __launch_bounds__(1024)
    to_all_kernel(T *dest0, const T *source0, size_t n, size_t tile, int pe_start, int log_stride,
                  int pe_size, T *pWrk0, long *pSync0) {
  __shared__ roc_shmem_ctx_t ctx;
  roc_shmem_wg_init();
  roc_shmem_wg_ctx_create(ROC_SHMEM_CTX_WG_PRIVATE, &ctx);
  const int me = roc_shmem_ctx_my_pe(ctx);
  const int npes = roc_shmem_ctx_n_pes(ctx);
  // (the quotients are the same in every lane, but a division is carried out on the vector unit:
  // saying so keeps the tile loop's bookkeeping in scalar registers)
  const size_t w = detail::uniform(static_cast<size_t>(blockIdx.x / npes));
  const size_t nw = detail::uniform(static_cast<size_t>(gridDim.x / npes));
  const int rel = me - pe_start;
  const bool member = rel >= 0 && (rel & ((1 << log_stride) - 1)) == 0 &&
                      (rel >> log_stride) < pe_size;
  if (member) {
    T *dest = roc_shmemx_my_addr(dest0);
    const T *source = roc_shmemx_my_addr(source0);
    if constexpr (kForm == kShardedLds) {
      extern __shared__ __attribute__((aligned(16))) char lds_stage[];
      long *pSync = roc_shmemx_my_addr(pSync0) + w * ROC_SHMEM_REDUCE_SYNC_SIZE;
      detail::wg_all_reduce<T, Op>(me, dest, source, n, pe_start, 1 << log_stride, pe_size, pSync,
                                   static_cast<int>(w), static_cast<int>(nw), 0, lds_stage,
                                   static_cast<uint32_t>(tile));
    } else if constexpr (kForm == kShardedStaticFlags) {
      long *flags = pSync0 + (static_cast<size_t>(me) * nw + w) * ROC_SHMEM_REDUCE_SYNC_SIZE;
      const int64_t pe_step = static_cast<int64_t>(nw) * ROC_SHMEM_REDUCE_SYNC_SIZE * sizeof(long);
      detail::wg_all_reduce<T, Op>(me, dest, source, n, pe_start, 1 << log_stride, pe_size, flags,
                                   static_cast<int>(w), static_cast<int>(nw), pe_step);
    } else {
      T *pWrk = roc_shmemx_my_addr(pWrk0);
      long *pSync = roc_shmemx_my_addr(pSync0) + w * ROC_SHMEM_REDUCE_SYNC_SIZE;
      if constexpr (kForm == kSharded) {
        ToAll<T, Op>::active_set_shard(ctx, dest, source, n, pe_start, log_stride, pe_size, pWrk,
                                       pSync, static_cast<int>(w), static_cast<int>(nw));
      } else {
        for (size_t off = w * tile; off < n; off += nw * tile) {
          size_t cnt = n - off < tile ? n - off : tile;
          ToAll<T, Op>::active_set(ctx, dest + off, source + off, static_cast<int>(cnt), pe_start,
                                   log_stride, pe_size, pWrk, pSync);
        }
      }
    }
  }
  roc_shmem_wg_ctx_destroy(ctx);
  roc_shmem_wg_finalize();
}

template <typename T, ROC_SHMEM_OP Op, bool kShard>
__global__ void __launch_bounds__(1024)
    to_all_team_kernel(roc_shmem_team_t team, T *dest0, const T *source0, size_t n, size_t tile,
                       int pe_start, int stride, int pe_size) {
  __shared__ roc_shmem_ctx_t ctx;
  roc_shmem_wg_init();
  roc_shmem_wg_team_create_ctx(team, ROC_SHMEM_CTX_WG_PRIVATE, &ctx);
  const int me = roc_shmem_ctx_my_pe(ctx);
  const int npes = roc_shmem_ctx_n_pes(ctx);
  const size_t w = blockIdx.x / npes;
  const size_t nw = gridDim.x / npes;
  const int rel = me - pe_start;
  const bool member = rel >= 0 && rel % stride == 0 && rel / stride < pe_size;
  if (member) {
    T *dest = roc_shmemx_my_addr(dest0);
    const T *source = roc_shmemx_my_addr(source0);
    if constexpr (kShard) {
      ToAll<T, Op>::team_shard(ctx, team, dest, source, n, static_cast<int>(w),
                               static_cast<int>(nw));
    } else {
      for (size_t off = w * tile; off < n; off += nw * tile) {
        size_t cnt = n - off < tile ? n - off : tile;
        ToAll<T, Op>::team(ctx, team, dest + off, source + off, static_cast<int>(cnt));
      }
    }
  }
  roc_shmem_wg_ctx_destroy(ctx);
  roc_shmem_wg_finalize();
}

struct ReduceArgs {
  void *dest;
  const void *source;
  size_t n;
  size_t tile;
  int pe_start, log_stride, pe_size;
  void *pWrk;
  long *pSync;
  roc_shmem_team_t team;
  int stride;
  bool static_flags;   // pSync is the device address of the library's own flag array
  bool lds;            // loads staged through LDS (ROC_SHMEM_REDUCE_LDS=1)
};

template <typename T, ROC_SHMEM_OP Op, int kForm>
void launch_active_set(const rsm::Launch &l, const ReduceArgs &a) {
  hipLaunchKernelGGL((to_all_kernel<T, Op, kForm>), dim3(l.grid), dim3(l.wg_size), 0, l.stream,
                     static_cast<T *>(a.dest), static_cast<const T *>(a.source), a.n, a.tile,
                     a.pe_start, a.log_stride, a.pe_size, static_cast<T *>(a.pWrk), a.pSync);
}

template <typename T, ROC_SHMEM_OP Op, bool kShard>
void launch_team(const rsm::Launch &l, const ReduceArgs &a) {
  hipLaunchKernelGGL((to_all_team_kernel<T, Op, kShard>), dim3(l.grid), dim3(l.wg_size), 0,
                     l.stream, a.team, static_cast<T *>(a.dest), static_cast<const T *>(a.source),
                     a.n, a.tile, a.pe_start, a.stride, a.pe_size);
}

// Dynamic LDS of the LDS-staged form: room for all members at two vectors per lane, at most
// 128 KiB (the form then stages the members in several rounds).
constexpr size_t kLdsStageLimit = 128u << 10;

template <typename T, ROC_SHMEM_OP Op>
bool launch_lds(const rsm::Launch &l, const ReduceArgs &a) {
  const size_t per_member = static_cast<size_t>(l.wg_size) * 16u * 2u;
  size_t bytes = per_member * static_cast<size_t>(a.pe_size);
  if (bytes > kLdsStageLimit) bytes = kLdsStageLimit / per_member * per_member;
  const void *kernel = reinterpret_cast<const void *>(&to_all_kernel<T, Op, kShardedLds>);
  if (hipFuncSetAttribute(kernel, hipFuncAttributeMaxDynamicSharedMemorySize, static_cast<int>(bytes)) !=
      hipSuccess)
    return false;
  // `tile` carries the size of the stage to the kernel (the form has no tiles)
  hipLaunchKernelGGL((to_all_kernel<T, Op, kShardedLds>), dim3(l.grid), dim3(l.wg_size), bytes, l.stream,
                     static_cast<T *>(a.dest), static_cast<const T *>(a.source), a.n, bytes, a.pe_start,
                     a.log_stride, a.pe_size, static_cast<T *>(a.pWrk), a.pSync);
  return true;
}

template <typename T, ROC_SHMEM_OP Op>
void launch_one(const rsm::Launch &l, const ReduceArgs &a) {
  if constexpr ((std::is_same<T, float>::value || std::is_same<T, long>::value ||
                 std::is_same<T, __hip_bfloat16>::value) && Op == ROC_SHMEM_SUM) {
    if (a.lds && !a.team && !a.static_flags && a.tile == 0 && launch_lds<T, Op>(l, a)) return;
  }
  if (a.static_flags) {
    launch_active_set<T, Op, kShardedStaticFlags>(l, a);
  } else if (a.team) {
    a.tile == 0 ? launch_team<T, Op, true>(l, a) : launch_team<T, Op, false>(l, a);
  } else {
    a.tile == 0 ? launch_active_set<T, Op, kSharded>(l, a) : launch_active_set<T, Op, kTiled>(l, a);
  }
}

template <typename T>
bool launch_arith(int op, const rsm::Launch &l, const ReduceArgs &a) {
  switch (op) {
    case RSM_SUM: launch_one<T, ROC_SHMEM_SUM>(l, a); return true;
    case RSM_MAX: launch_one<T, ROC_SHMEM_MAX>(l, a); return true;
    case RSM_MIN: launch_one<T, ROC_SHMEM_MIN>(l, a); return true;
    case RSM_PROD: launch_one<T, ROC_SHMEM_PROD>(l, a); return true;
    default: return false;
  }
}

template <typename T>
bool launch_int(int op, const rsm::Launch &l, const ReduceArgs &a) {
  switch (op) {
    case RSM_AND: launch_one<T, ROC_SHMEM_AND>(l, a); return true;
    case RSM_OR: launch_one<T, ROC_SHMEM_OR>(l, a); return true;
    case RSM_XOR: launch_one<T, ROC_SHMEM_XOR>(l, a); return true;
    default: return launch_arith<T>(op, l, a);
  }
}

bool launch_bf16(int op, const rsm::Launch &l, const ReduceArgs &a) {
  switch (op) {
    case RSM_SUM: launch_one<__hip_bfloat16, ROC_SHMEM_SUM>(l, a); return true;
    case RSM_MAX: launch_one<__hip_bfloat16, ROC_SHMEM_MAX>(l, a); return true;
    case RSM_MIN: launch_one<__hip_bfloat16, ROC_SHMEM_MIN>(l, a); return true;
    default: return false;
  }
}

size_t dtype_size(int dtype) {
  switch (dtype) {
    case RSM_SHORT: case RSM_BF16: return 2;
    case RSM_INT: case RSM_FLOAT: return 4;
    case RSM_LONG: case RSM_LONGLONG: case RSM_DOUBLE: return 8;
    default: return 0;
  }
}

bool op_defined(int dtype, int op) {
  switch (dtype) {
    case RSM_SHORT: case RSM_INT: case RSM_LONG: case RSM_LONGLONG: return op >= RSM_SUM && op <= RSM_XOR;
    case RSM_FLOAT: case RSM_DOUBLE: return op == RSM_SUM || op == RSM_MAX || op == RSM_MIN || op == RSM_PROD;
    case RSM_BF16: return op == RSM_SUM || op == RSM_MAX || op == RSM_MIN;
    default: return false;
  }
}

// Everything that can be refused is refused here, before anything is launched.
int check_args(int dtype, int op, const rsm::Launch &l, const ReduceArgs &a) {
  const size_t es = dtype_size(dtype);
  if (!es) return rsm::fail("to_all: unknown dtype");
  if (!op_defined(dtype, op)) return rsm::fail("to_all: operator not defined for this dtype");
  if (a.n == 0) return 0;  // zero-element reductions are no-ops (context_tmpl_device.hpp:68-70)
  if (a.n > (~size_t{0} >> 4) || !rsm::check_extent(a.dest, a.n * es, "to_all: dest") ||
      !rsm::check_extent(a.source, a.n * es, "to_all: source") ||
      !rsm::check_extent(a.static_flags ? nullptr : a.pSync, static_cast<size_t>(l.wgs_per_pe) * ROC_SHMEM_REDUCE_SYNC_SIZE * sizeof(long),
                         "to_all: pSync (wgs_per_pe slices of ROC_SHMEM_REDUCE_SYNC_SIZE longs)"))
    return -1;
  // tile == 0: the PE's workgroups share one reduction through the sharded
  // extension; otherwise each standard call covers `tile` elements.
  if (a.tile > 0x7fffffffull) return rsm::fail("to_all: tile does not fit the API's int nreduce");
  return 0;
}

int run(int dtype, int op, const rsm::Launch &l, ReduceArgs a, bool checked = false) {
  if (!checked && check_args(dtype, op, l, a) != 0) return -1;
  if (a.n == 0) return 0;
  bool ok = false;
  switch (dtype) {
    case RSM_SHORT: ok = launch_int<short>(op, l, a); break;
    case RSM_INT: ok = launch_int<int>(op, l, a); break;
    case RSM_LONG: ok = launch_int<long>(op, l, a); break;
    case RSM_LONGLONG: ok = launch_int<long long>(op, l, a); break;
    case RSM_FLOAT: ok = launch_arith<float>(op, l, a); break;
    case RSM_DOUBLE: ok = launch_arith<double>(op, l, a); break;
    case RSM_BF16: ok = launch_bf16(op, l, a); break;
  }
  if (!ok) return rsm::fail("to_all: operator not defined for this dtype");
  return rsm::after_launch("to_all");
}

// Device address of g_noalloc_flags on each device, looked up once per device.
constexpr int kMaxDevices = 64;
long *g_noalloc_flags_at[kMaxDevices] = {};

}  // namespace

namespace rsm {

// Called by rsm_init (and, should a caller switch devices afterwards, by the entry point's
// first call on the new device), with the device current: asks the runtime where this
// device's copy of the flag array lives.  Allocates nothing.
long *noalloc_flags() {
  int dev = -1;
  if (hipGetDevice(&dev) != hipSuccess || dev < 0 || dev >= kMaxDevices) {
    fail("to_all_noalloc: cannot tell the current device");
    return nullptr;
  }
  if (!g_noalloc_flags_at[dev]) {
    long *at = nullptr;
    hipError_t e = hipGetSymbolAddress(reinterpret_cast<void **>(&at), HIP_SYMBOL(g_noalloc_flags));
    if (e != hipSuccess || !at) {
      fail(std::string("to_all_noalloc: hipGetSymbolAddress: ") + hipGetErrorString(e));
      return nullptr;
    }
    g_noalloc_flags_at[dev] = at;
  }
  return g_noalloc_flags_at[dev];
}

}  // namespace rsm

extern "C" {

int rsm_to_all_noalloc(int dtype, int op, void *dest, const void *source, size_t nreduce,
                       int pe_start, int log_pe_stride, int pe_size, const rsm_launch_t *launch) {
  RSM_ENTRY;
  rsm::Launch l;
  if (!rsm::resolve_launch(launch, &l)) return -1;
  host::Runtime *rt = host::Runtime::get();
  if (!rsm::check_symmetric(dest, "dest") || !rsm::check_symmetric(source, "source")) return -1;
  if (!rsm::active_set_in_range(pe_start, log_pe_stride, pe_size, rt->num_pes()))
    return rsm::fail("to_all_noalloc: active set out of range");
  if (l.tile != 0)
    return rsm::fail("to_all_noalloc: launch->tile must be 0 (the PE's workgroups share one reduction)");
  if (l.grid > kNoAllocMaxWgs)
    return rsm::fail("to_all_noalloc: " + std::to_string(l.grid) + " workgroups (PEs x wgs_per_pe) exceed the " +
                     std::to_string(kNoAllocMaxWgs) + " the library's flag array has room for");
  long *flags = rsm::noalloc_flags();
  if (!flags) return -1;
  ReduceArgs a{dest, source, nreduce, 0, pe_start, log_pe_stride, pe_size, nullptr, flags,
               nullptr, 1 << log_pe_stride, true, false};
  // a call that is going to be refused queues nothing, not even the clearing of the flags
  if (check_args(dtype, op, l, a) != 0) return -1;
  if (nreduce == 0) return 0;
  // The array is shared by every call on this device and keeps what the last call left: the
  // slices this grid uses start at zero whatever happened before (a call whose waits gave up
  // leaves flags set).  A kernel, not hipMemsetAsync, so that the call can be recorded in a graph.
  const size_t n_flags = static_cast<size_t>(l.grid) * ROC_SHMEM_REDUCE_SYNC_SIZE;
  hipLaunchKernelGGL(clear_flags_kernel, dim3(static_cast<unsigned>((n_flags + 255) / 256)), dim3(256),
                     0, l.stream, flags, n_flags);
  return run(dtype, op, l, a, true);
}

int rsm_tune_reduce_pacing(int dtype, int op, void *dest, const void *source, size_t nreduce,
                           int pe_start, int log_pe_stride, int pe_size, long *pSync,
                           const rsm_launch_t *launch, unsigned *rate_out, float *free_ms_out,
                           float *paced_ms_out) {
  RSM_ENTRY;
  host::Runtime *rt = host::Runtime::get();
  if (!rt) return rsm::fail("rsm_init has not been called");
  if (rsm::live_consumer_running()) return rsm::fail("rsm_tune_reduce_pacing: a live send-queue consumer is running");
  if (!launch) return rsm::fail("launch description is NULL");
  hipStream_t stream = static_cast<hipStream_t>(launch->stream);
  const unsigned copy_rate = rt->device_state().pace_copy_bytes_per_tick;
  // what is in force now comes back on every path that does not end with a measured choice
  const unsigned reduce_rate_before = rt->device_state().pace_reduce_bytes_per_tick;
  hipEvent_t t0 = nullptr, t1 = nullptr;
  if (hipEventCreate(&t0) != hipSuccess || hipEventCreate(&t1) != hipSuccess) {
    if (t0) (void)hipEventDestroy(t0);
    return rsm::fail("rsm_tune_reduce_pacing: hipEventCreate failed");
  }
  int rc = 0;
  // milliseconds per launch at `rate` (0 = free running): eight launches queued back to back
  // after a warm-up, the way a caller's loop issues them (launches timed one by one on an idle
  // device tolerate a rate about 2 % higher than a queue of them does)
  auto measure = [&](unsigned rate, float *ms_out) -> bool {
    constexpr int kLaunches = 8;
    if (!rt->set_pacing(copy_rate, rate)) return false;
    for (int i = 0; i <= kLaunches; ++i) {
      if (i == 1 && hipEventRecord(t0, stream) != hipSuccess) return false;
      if (rsm_to_all(dtype, op, dest, source, nreduce, pe_start, log_pe_stride, pe_size, nullptr, pSync,
                     launch) != 0)
        return false;
    }
    if (hipEventRecord(t1, stream) != hipSuccess || hipEventSynchronize(t1) != hipSuccess) return false;
    float ms = 0;
    if (hipEventElapsedTime(&ms, t0, t1) != hipSuccess) return false;
    *ms_out = ms / kLaunches;
    return true;
  };
  float free_ms = 0, best_ms = 0;
  unsigned best_rate = 0;
  if (!measure(0, &free_ms)) rc = -1;
  // Rates the memory system of an MI355X may sustain in lockstep: 5.6 .. 7.2 TB/s in 1 % steps.
  for (unsigned rate = 56000; rc == 0 && rate <= 72000; rate += 600) {
    float ms = 0;
    if (!measure(rate, &ms)) { rc = -1; break; }
    if (best_rate == 0 || ms < best_ms) { best_ms = ms; best_rate = rate; }
  }
  unsigned chosen = 0;
  float chosen_ms = free_ms;
  if (rc == 0 && best_rate != 0) {
    // The best rate and running free once more, so that one lucky sample decides nothing; the
    // schedule stays only if it still gains 1 %.  (No margin below the best rate is needed: a
    // rate beyond what the card sustains costs a little, not the cliff a gate on slots has.)
    float best_again = 0, again_free = 0;
    if (!measure(best_rate, &best_again) || !measure(0, &again_free)) {
      rc = -1;
    } else {
      if (again_free < free_ms) free_ms = again_free;
      if (best_again > best_ms) best_ms = best_again;
      chosen_ms = free_ms;
      if (best_ms < free_ms * 0.99f) { chosen = best_rate; chosen_ms = best_ms; }
    }
  }
  if (!rt->set_pacing(copy_rate, rc == 0 ? chosen : reduce_rate_before) && rc == 0) rc = -1;
  (void)hipEventDestroy(t0);
  (void)hipEventDestroy(t1);
  if (rc != 0) {
    if (rsm_last_error()[0] == 0) rsm::fail("rsm_tune_reduce_pacing: a launch or an event failed");
    return -1;
  }
  if (rate_out) *rate_out = chosen;
  if (free_ms_out) *free_ms_out = free_ms;
  if (paced_ms_out) *paced_ms_out = chosen_ms;
  return 0;
}

int rsm_to_all(int dtype, int op, void *dest, const void *source, size_t nreduce, int pe_start,
               int log_pe_stride, int pe_size, void *pWrk, long *pSync,
               const rsm_launch_t *launch) {
  RSM_ENTRY;
  rsm::Launch l;
  if (!rsm::resolve_launch(launch, &l)) return -1;
  host::Runtime *rt = host::Runtime::get();
  if (!rsm::check_symmetric(dest, "dest") || !rsm::check_symmetric(source, "source") ||
      !rsm::check_symmetric(pSync, "pSync") || !rsm::check_symmetric(pWrk, "pWrk", true))
    return -1;
  if (!rsm::active_set_in_range(pe_start, log_pe_stride, pe_size, rt->num_pes()))
    return rsm::fail("to_all: active set out of range");
  ReduceArgs a{dest, source, nreduce, l.tile, pe_start, log_pe_stride, pe_size, pWrk, pSync,
               nullptr, 1 << log_pe_stride, false, rt->options().reduce_lds};
  return run(dtype, op, l, a);
}

int rsm_to_all_team(int dtype, int op, uint64_t team, void *dest, const void *source,
                    size_t nreduce, const rsm_launch_t *launch) {
  RSM_ENTRY;
  rsm::Launch l;
  if (!rsm::resolve_launch(launch, &l)) return -1;
  host::Runtime *rt = host::Runtime::get();
  if (!rsm::check_symmetric(dest, "dest") || !rsm::check_symmetric(source, "source")) return -1;
  const host::TeamRecord *rec = rt->team_record(reinterpret_cast<detail::Team *>(team));
  if (!rec) return rsm::fail("to_all_team: invalid team");
  if (l.wgs_per_pe > rt->options().num_blocks)
    return rsm::fail("to_all_team: wgs_per_pe exceeds the contexts per PE (team pSync slices)");
  const detail::TeamInfo &ti = rec->image.wrt_world;
  ReduceArgs a{dest, source, nreduce, l.tile, ti.pe_start, 0, ti.size, nullptr,
               nullptr, reinterpret_cast<roc_shmem_team_t>(team), ti.stride, false, false};
  return run(dtype, op, l, a);
}

}  // extern "C"
