// C ABI: broadcast, alltoall, fcollect and barrier.  Kernels follow the shape
// of the reference's BroadcastTest / AlltoallTest / FcollectTest / BarrierAllTest
// kernels (clients/functional_tests/broadcast_tester.cpp, alltoall_tester.cpp,
// fcollect_tester.cpp, barrier_all_tester.cpp), for every PE in one grid.
#include "cabi_common.hpp"
#include "roc_shmem.hpp"

using namespace rocshmem;

namespace {

// Element-size tag -> the typed API name used for it.
template <int Bytes> struct ElemOf;
template <> struct ElemOf<1> { using type = char; };
template <> struct ElemOf<2> { using type = short; };
template <> struct ElemOf<4> { using type = int; };
template <> struct ElemOf<8> { using type = long; };

__device__ __forceinline__ void bcast_call(roc_shmem_ctx_t c, char *d, const char *s, int n, int root, int ps, int ls, int sz, long *p) { roc_shmem_ctx_char_wg_broadcast(c, d, s, n, root, ps, ls, sz, p); }
__device__ __forceinline__ void bcast_call(roc_shmem_ctx_t c, short *d, const short *s, int n, int root, int ps, int ls, int sz, long *p) { roc_shmem_ctx_short_wg_broadcast(c, d, s, n, root, ps, ls, sz, p); }
__device__ __forceinline__ void bcast_call(roc_shmem_ctx_t c, int *d, const int *s, int n, int root, int ps, int ls, int sz, long *p) { roc_shmem_ctx_int_wg_broadcast(c, d, s, n, root, ps, ls, sz, p); }
__device__ __forceinline__ void bcast_call(roc_shmem_ctx_t c, long *d, const long *s, int n, int root, int ps, int ls, int sz, long *p) { roc_shmem_ctx_long_wg_broadcast(c, d, s, n, root, ps, ls, sz, p); }

__device__ __forceinline__ void bcast_team_call(roc_shmem_ctx_t c, roc_shmem_team_t t, char *d, const char *s, int n, int root) { roc_shmem_ctx_char_wg_broadcast(c, t, d, s, n, root); }
__device__ __forceinline__ void bcast_team_call(roc_shmem_ctx_t c, roc_shmem_team_t t, short *d, const short *s, int n, int root) { roc_shmem_ctx_short_wg_broadcast(c, t, d, s, n, root); }
__device__ __forceinline__ void bcast_team_call(roc_shmem_ctx_t c, roc_shmem_team_t t, int *d, const int *s, int n, int root) { roc_shmem_ctx_int_wg_broadcast(c, t, d, s, n, root); }
__device__ __forceinline__ void bcast_team_call(roc_shmem_ctx_t c, roc_shmem_team_t t, long *d, const long *s, int n, int root) { roc_shmem_ctx_long_wg_broadcast(c, t, d, s, n, root); }

#define RSM_BCAST_SHARD(T, TNAME)                                                               \
  __device__ __forceinline__ void bcast_shard_call(roc_shmem_ctx_t c, T *d, const T *s, size_t n, \
                                                   int root, int ps, int ls, int sz, long *p,   \
                                                   int sh, int nsh) {                           \
    roc_shmemx_ctx_##TNAME##_wg_broadcast_shard(c, d, s, n, root, ps, ls, sz, p, sh, nsh);      \
  }                                                                                             \
  __device__ __forceinline__ void bcast_team_shard_call(roc_shmem_ctx_t c, roc_shmem_team_t t,  \
                                                        T *d, const T *s, size_t n, int root,   \
                                                        int sh, int nsh) {                      \
    roc_shmemx_ctx_##TNAME##_wg_broadcast_shard(c, t, d, s, n, root, sh, nsh);                  \
  }
RSM_BCAST_SHARD(char, char)
RSM_BCAST_SHARD(short, short)
RSM_BCAST_SHARD(int, int)
RSM_BCAST_SHARD(long, long)
#undef RSM_BCAST_SHARD

__device__ __forceinline__ void a2a_call(roc_shmem_ctx_t c, roc_shmem_team_t t, char *d, const char *s, int n, int sh, int nsh) { roc_shmemx_ctx_char_wg_alltoall_shard(c, t, d, s, n, sh, nsh); }
__device__ __forceinline__ void a2a_call(roc_shmem_ctx_t c, roc_shmem_team_t t, short *d, const short *s, int n, int sh, int nsh) { roc_shmemx_ctx_short_wg_alltoall_shard(c, t, d, s, n, sh, nsh); }
__device__ __forceinline__ void a2a_call(roc_shmem_ctx_t c, roc_shmem_team_t t, int *d, const int *s, int n, int sh, int nsh) { roc_shmemx_ctx_int_wg_alltoall_shard(c, t, d, s, n, sh, nsh); }
__device__ __forceinline__ void a2a_call(roc_shmem_ctx_t c, roc_shmem_team_t t, long *d, const long *s, int n, int sh, int nsh) { roc_shmemx_ctx_long_wg_alltoall_shard(c, t, d, s, n, sh, nsh); }

__device__ __forceinline__ void fcol_call(roc_shmem_ctx_t c, roc_shmem_team_t t, char *d, const char *s, int n, int sh, int nsh) { roc_shmemx_ctx_char_wg_fcollect_shard(c, t, d, s, n, sh, nsh); }
__device__ __forceinline__ void fcol_call(roc_shmem_ctx_t c, roc_shmem_team_t t, short *d, const short *s, int n, int sh, int nsh) { roc_shmemx_ctx_short_wg_fcollect_shard(c, t, d, s, n, sh, nsh); }
__device__ __forceinline__ void fcol_call(roc_shmem_ctx_t c, roc_shmem_team_t t, int *d, const int *s, int n, int sh, int nsh) { roc_shmemx_ctx_int_wg_fcollect_shard(c, t, d, s, n, sh, nsh); }
__device__ __forceinline__ void fcol_call(roc_shmem_ctx_t c, roc_shmem_team_t t, long *d, const long *s, int n, int sh, int nsh) { roc_shmemx_ctx_long_wg_fcollect_shard(c, t, d, s, n, sh, nsh); }

__device__ __forceinline__ bool in_set(int me, int pe_start, int stride, int pe_size) {
  int rel = me - pe_start;
  return rel >= 0 && rel % stride == 0 && rel / stride < pe_size;
}

// kTeam: the team form of the call; kShard: the PE's workgroups share one broadcast (sharded
// extension), otherwise one standard call per tile.  Four kernels rather than branches: with
// all four calls inlined into one kernel the compiler ran out of scalar registers and the
// store loop ran a sixth slower.
template <typename T, bool kTeam, bool kShard>
__global__ void __launch_bounds__(1024)
    broadcast_kernel(roc_shmem_team_t team, T *dest0, const T *source0, size_t n, size_t tile,
                     int pe_root, int pe_start, int log_stride, int pe_stride, int pe_size,
                     long *pSync0) {
  __shared__ roc_shmem_ctx_t ctx;
  roc_shmem_wg_init();
  roc_shmem_wg_ctx_create(ROC_SHMEM_CTX_WG_PRIVATE, &ctx);
  const int me = roc_shmem_ctx_my_pe(ctx);
  const int npes = roc_shmem_ctx_n_pes(ctx);
  const size_t w = blockIdx.x / npes;
  const size_t nw = gridDim.x / npes;
  if (in_set(me, pe_start, pe_stride, pe_size)) {
    T *dest = roc_shmemx_my_addr(dest0);
    const T *source = roc_shmemx_my_addr(source0);
    long *pSync = kTeam ? nullptr : roc_shmemx_my_addr(pSync0) + w * ROC_SHMEM_BCAST_SYNC_SIZE;
    if constexpr (kShard) {
      if constexpr (kTeam) {
        bcast_team_shard_call(ctx, team, dest, source, n, pe_root, static_cast<int>(w),
                              static_cast<int>(nw));
      } else {
        bcast_shard_call(ctx, dest, source, n, pe_root, pe_start, log_stride, pe_size, pSync,
                         static_cast<int>(w), static_cast<int>(nw));
      }
    } else {
      for (size_t off = w * tile; off < n; off += nw * tile) {
        size_t cnt = n - off < tile ? n - off : tile;
        if constexpr (kTeam) {
          bcast_team_call(ctx, team, dest + off, source + off, static_cast<int>(cnt), pe_root);
        } else {
          bcast_call(ctx, dest + off, source + off, static_cast<int>(cnt), pe_root, pe_start,
                     log_stride, pe_size, pSync);
        }
      }
    }
  }
  roc_shmem_wg_ctx_destroy(ctx);
  roc_shmem_wg_finalize();
}

template <typename T, bool kFcollect>
__global__ void __launch_bounds__(1024)
    exchange_kernel(roc_shmem_team_t team, T *dest0, const T *source0, int nelem, int pe_start,
                    int stride, int pe_size) {
  __shared__ roc_shmem_ctx_t ctx;
  roc_shmem_wg_init();
  roc_shmem_wg_team_create_ctx(team, ROC_SHMEM_CTX_WG_PRIVATE, &ctx);
  const int me = roc_shmem_ctx_my_pe(ctx);
  const int npes = roc_shmem_ctx_n_pes(ctx);
  const int w = blockIdx.x / npes;
  const int nw = gridDim.x / npes;
  if (in_set(me, pe_start, stride, pe_size)) {
    T *dest = roc_shmemx_my_addr(dest0);
    const T *source = roc_shmemx_my_addr(source0);
    if (kFcollect) {
      fcol_call(ctx, team, dest, source, nelem, w, nw);
    } else {
      a2a_call(ctx, team, dest, source, nelem, w, nw);
    }
  }
  roc_shmem_wg_ctx_destroy(ctx);
  roc_shmem_wg_finalize();
}

__global__ void __launch_bounds__(1024) barrier_kernel(int iterations) {
  __shared__ roc_shmem_ctx_t ctx;
  roc_shmem_wg_init();
  roc_shmem_wg_ctx_create(ROC_SHMEM_CTX_WG_PRIVATE, &ctx);
  for (int i = 0; i < iterations; ++i) roc_shmem_ctx_wg_barrier_all(ctx);
  roc_shmem_wg_ctx_destroy(ctx);
  roc_shmem_wg_finalize();
}

struct BcastArgs {
  roc_shmem_team_t team;
  void *dest;
  const void *source;
  size_t n, tile;
  int root, pe_start, log_stride, pe_stride, pe_size;  // log_stride: active-set form only
  long *pSync;
};

template <typename T, bool kTeam, bool kShard>
void launch_bcast_form(const rsm::Launch &l, const BcastArgs &a) {
  hipLaunchKernelGGL((broadcast_kernel<T, kTeam, kShard>), dim3(l.grid), dim3(l.wg_size), 0,
                     l.stream, a.team, static_cast<T *>(a.dest), static_cast<const T *>(a.source),
                     a.n, a.tile, a.root, a.pe_start, a.log_stride, a.pe_stride, a.pe_size,
                     a.pSync);
}

template <typename T>
void launch_bcast(const rsm::Launch &l, const BcastArgs &a) {
  const bool shard = a.tile == 0;
  if (a.team) {
    shard ? launch_bcast_form<T, true, true>(l, a) : launch_bcast_form<T, true, false>(l, a);
  } else {
    shard ? launch_bcast_form<T, false, true>(l, a) : launch_bcast_form<T, false, false>(l, a);
  }
}

int run_bcast(size_t elem_size, const rsm::Launch &l, BcastArgs a) {
  if (a.n == 0) return 0;
  if (elem_size == 0 || elem_size > 8 || a.n > (~size_t{0} >> 4) ||
      !rsm::check_extent(a.dest, a.n * elem_size, "broadcast: dest") ||
      !rsm::check_extent(a.source, a.n * elem_size, "broadcast: source") ||
      !rsm::check_extent(a.pSync, static_cast<size_t>(l.wgs_per_pe) * ROC_SHMEM_BCAST_SYNC_SIZE * sizeof(long),
                         "broadcast: pSync (wgs_per_pe slices of ROC_SHMEM_BCAST_SYNC_SIZE longs)"))
    return -1;
  // tile == 0: the PE's workgroups share one broadcast through the sharded extension.
  if (a.tile > 0x7fffffffull) return rsm::fail("broadcast: tile does not fit the API's int nelem");
  switch (elem_size) {
    case 1: launch_bcast<char>(l, a); break;
    case 2: launch_bcast<short>(l, a); break;
    case 4: launch_bcast<int>(l, a); break;
    case 8: launch_bcast<long>(l, a); break;
    default: return rsm::fail("broadcast: element size must be 1, 2, 4 or 8");
  }
  return rsm::after_launch("broadcast");
}

template <bool kFcollect>
int run_exchange(size_t elem_size, uint64_t team, void *dest, const void *source, size_t nelem,
                 const rsm_launch_t *launch) {
  rsm::Launch l;
  if (!rsm::resolve_launch(launch, &l)) return -1;
  host::Runtime *rt = host::Runtime::get();
  if (!rsm::check_symmetric(dest, "dest") || !rsm::check_symmetric(source, "source")) return -1;
  const host::TeamRecord *rec = rt->team_record(reinterpret_cast<detail::Team *>(team));
  if (!rec) return rsm::fail("alltoall/fcollect: invalid team");
  if (l.wgs_per_pe > rt->options().num_blocks)
    return rsm::fail("alltoall/fcollect: wgs_per_pe exceeds the contexts per PE");
  if (nelem == 0) return 0;
  if (nelem > 0x7fffffffull) return rsm::fail("alltoall/fcollect: nelem does not fit an int");
  const detail::TeamInfo &ti = rec->image.wrt_world;
  roc_shmem_team_t t = reinterpret_cast<roc_shmem_team_t>(team);
  const int n = static_cast<int>(nelem);
  if (elem_size == 0 || elem_size > 8) return rsm::fail("alltoall/fcollect: element size must be 1, 2, 4 or 8");
  const size_t block = nelem * elem_size, all_blocks = block * static_cast<size_t>(ti.size);
  if (!rsm::check_extent(dest, all_blocks, "alltoall/fcollect: dest (team size blocks)") ||
      !rsm::check_extent(source, kFcollect ? block : all_blocks, "alltoall/fcollect: source"))
    return -1;
#define RSM_EXCHANGE(T)                                                                        \
  hipLaunchKernelGGL((exchange_kernel<T, kFcollect>), dim3(l.grid), dim3(l.wg_size), 0,        \
                     l.stream, t, static_cast<T *>(dest), static_cast<const T *>(source), n,   \
                     ti.pe_start, ti.stride, ti.size)
  switch (elem_size) {
    case 1: RSM_EXCHANGE(char); break;
    case 2: RSM_EXCHANGE(short); break;
    case 4: RSM_EXCHANGE(int); break;
    case 8: RSM_EXCHANGE(long); break;
    default: return rsm::fail("alltoall/fcollect: element size must be 1, 2, 4 or 8");
  }
#undef RSM_EXCHANGE
  return rsm::after_launch(kFcollect ? "fcollect" : "alltoall");
}

}  // namespace

extern "C" {

int rsm_broadcast(size_t elem_size, void *dest, const void *source, size_t nelem, int pe_root,
                  int pe_start, int log_pe_stride, int pe_size, long *pSync,
                  const rsm_launch_t *launch) {
  RSM_ENTRY;
  rsm::Launch l;
  if (!rsm::resolve_launch(launch, &l)) return -1;
  host::Runtime *rt = host::Runtime::get();
  if (!rsm::check_symmetric(dest, "dest") || !rsm::check_symmetric(source, "source") ||
      !rsm::check_symmetric(pSync, "pSync"))
    return -1;
  if (!rsm::active_set_in_range(pe_start, log_pe_stride, pe_size, rt->num_pes()) || pe_root < 0 ||
      pe_root >= pe_size)
    return rsm::fail("broadcast: active set or root out of range");
  BcastArgs a{nullptr, dest, source, nelem, l.tile, pe_root, pe_start, log_pe_stride,
              1 << log_pe_stride, pe_size, pSync};
  return run_bcast(elem_size, l, a);
}

int rsm_broadcast_team(size_t elem_size, uint64_t team, void *dest, const void *source,
                       size_t nelem, int pe_root, const rsm_launch_t *launch) {
  RSM_ENTRY;
  rsm::Launch l;
  if (!rsm::resolve_launch(launch, &l)) return -1;
  host::Runtime *rt = host::Runtime::get();
  if (!rsm::check_symmetric(dest, "dest") || !rsm::check_symmetric(source, "source")) return -1;
  const host::TeamRecord *rec = rt->team_record(reinterpret_cast<detail::Team *>(team));
  if (!rec) return rsm::fail("broadcast_team: invalid team");
  if (l.wgs_per_pe > rt->options().num_blocks)
    return rsm::fail("broadcast_team: wgs_per_pe exceeds the contexts per PE");
  const detail::TeamInfo &ti = rec->image.wrt_world;
  if (pe_root < 0 || pe_root >= ti.size) return rsm::fail("broadcast_team: root out of range");
  BcastArgs a{reinterpret_cast<roc_shmem_team_t>(team), dest, source, nelem, l.tile, pe_root,
              ti.pe_start, 0, ti.stride, ti.size, nullptr};
  return run_bcast(elem_size, l, a);
}

int rsm_alltoall(size_t elem_size, uint64_t team, void *dest, const void *source, size_t nelem,
                 const rsm_launch_t *launch) {
  RSM_ENTRY;
  return run_exchange<false>(elem_size, team, dest, source, nelem, launch);
}

int rsm_fcollect(size_t elem_size, uint64_t team, void *dest, const void *source, size_t nelem,
                 const rsm_launch_t *launch) {
  RSM_ENTRY;
  return run_exchange<true>(elem_size, team, dest, source, nelem, launch);
}

int rsm_barrier_all(int iterations, const rsm_launch_t *launch) {
  RSM_ENTRY;
  rsm::Launch l;
  if (!rsm::resolve_launch(launch, &l)) return -1;
  if (l.wgs_per_pe > host::Runtime::get()->options().num_blocks)
    return rsm::fail("barrier_all: wgs_per_pe exceeds the contexts per PE");
  hipLaunchKernelGGL(barrier_kernel, dim3(l.grid), dim3(l.wg_size), 0, l.stream, iterations);
  return rsm::after_launch("barrier_all");
}

}  // extern "C"
