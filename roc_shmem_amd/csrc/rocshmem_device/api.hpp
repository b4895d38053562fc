// Device half of the roc_shmem_* interface: thin inline wrappers that resolve
// the context, apply the reference's PE-translation rules and call into the
// gfx950 data path.  Included from roc_shmem.hpp.
//
// Forwarding rules kept from the reference (library/src/roc_shmem_gpu.cpp):
//  * standard RMA (put/get/p/g and their mem/nbi forms) translate a
//    team-relative PE through the context's team (:240-247, :298-395);
//  * AMOs and the roc_shmemx_*_wg / *_wave forms pass the PE through
//    untranslated (:555-598, :667-795);
//  * zero-length RMA and zero-element collectives return at once
//    (context_device.cpp:80-82, context_tmpl_device.hpp:68-70).
#ifndef ROCSHMEM_MI355X_DEVICE_API_HPP
#define ROCSHMEM_MI355X_DEVICE_API_HPP

#include "coll.hpp"
#include "copy.hpp"
#include "reduce.hpp"
#include "small_ops.hpp"
#include "sync.hpp"
#include "wave.hpp"
#include "wqe.hpp"

namespace rocshmem {

namespace detail {

// Per translation unit hook.  Every unit that includes this header owns a
// private __constant__ copy of the runtime state; the hook below copies a new
// state into this unit's copy and reads it back.  Both the function and the
// registrar object have internal linkage on purpose: with external (inline)
// linkage the linker would keep a single instance that refers to one unit's
// copy only, and kernels of every other unit would run on a zeroed state.
namespace {
bool upload_state_to_this_unit(const DeviceState *s) {
  if (hipMemcpyToSymbol(HIP_SYMBOL(g_state), s, sizeof(DeviceState), 0,
                        hipMemcpyHostToDevice) != hipSuccess)
    return false;
  DeviceState check;
  if (hipMemcpyFromSymbol(&check, HIP_SYMBOL(g_state), sizeof(DeviceState), 0,
                          hipMemcpyDeviceToHost) != hipSuccess)
    return false;
  return __builtin_memcmp(&check, s, sizeof(DeviceState)) == 0;
}
struct StateRegistrar {
  StateRegistrar() { register_state_upload(&upload_state_to_this_unit, kStateLayout); }
};
StateRegistrar g_state_registrar;
}  // namespace

__device__ __forceinline__ int launch_pe() { return blockIdx.x % g_state.num_pes; }
__device__ __forceinline__ int launch_wg_rank() { return blockIdx.x / g_state.num_pes; }

__device__ __forceinline__ DeviceCtx *launch_ctx() {
  return g_state.ctx_table + launch_pe() * g_state.num_blocks +
         launch_wg_rank() % g_state.num_blocks;
}

__device__ __forceinline__ DeviceCtx *ctx_of(roc_shmem_ctx_t ctx) {
  return ctx.ctx_opaque ? static_cast<DeviceCtx *>(ctx.ctx_opaque) : launch_ctx();
}

// The PE a context handle acts for.  A handle names a context of the launching PE's table row
// (roc_shmem_wg_ctx_create, ROC_SHMEM_CTX_DEFAULT), so this is the grid position's PE and needs
// no look at the context: the calls that only move data (put, get, the collectives) never load
// from the context table, which used to put a chain of dependent memory reads - the handle from
// LDS, then the context's PE from memory - in front of a call's first payload load.
__device__ __forceinline__ int pe_of(roc_shmem_ctx_t) { return launch_pe(); }

// reference: translate_pe, roc_shmem_gpu.cpp:240-247
__device__ __forceinline__ int world_pe(roc_shmem_ctx_t ctx, int pe) {
  if (ctx.team_opaque) {
    const TeamInfo *t = static_cast<const TeamInfo *>(ctx.team_opaque);
    return t->pe_start + t->stride * pe;
  }
  return pe;
}

__device__ __forceinline__ Team *team_of(roc_shmem_team_t team) {
  return reinterpret_cast<Team *>(team);
}

// This PE's copy of a team-owned pSync slice for the calling context's block.  PE and block
// follow from the grid position (launch_ctx), so nothing is read from the context.
__device__ __forceinline__ long *team_psync(roc_shmem_ctx_t, uint64_t pool_off) {
  char *slice = g_state.heap_base0 + static_cast<uint64_t>(launch_pe()) * g_state.slice_stride;
  return reinterpret_cast<long *>(slice + pool_off) +
         static_cast<size_t>(launch_wg_rank() % g_state.num_blocks) * kSyncSlots;
}

}  // namespace detail

// ---------------------------------------------------------------------------
// Lifecycle, contexts, queries
// ---------------------------------------------------------------------------

__device__ inline void roc_shmem_query_thread(int *provided) {
  *provided = ROC_SHMEM_THREAD_MULTIPLE;
}
__device__ inline void roc_shmem_wg_init_thread(int, int *provided) {
  roc_shmem_query_thread(provided);
}
__device__ inline void roc_shmem_wg_init() {}
__device__ inline void roc_shmem_wg_finalize() {}

// Workgroup-collective.  `ctx` usually lives in LDS; thread 0 fills it in
// (reference: roc_shmem_wg_ctx_create, roc_shmem_gpu.cpp:259-267).
__device__ inline void roc_shmem_wg_ctx_create(int64_t options, roc_shmem_ctx_t *ctx) {
  if (detail::flat_thread_id() == 0) {
    ctx->ctx_opaque = detail::launch_ctx();
    ctx->team_opaque = nullptr;
  }
  (void)options;
  __syncthreads();
}

__device__ inline int roc_shmem_wg_team_create_ctx(roc_shmem_team_t team, long options,
                                                   roc_shmem_ctx_t *ctx) {
  if (team == ROC_SHMEM_TEAM_INVALID) return -1;
  if (detail::flat_thread_id() == 0) {
    ctx->ctx_opaque = detail::launch_ctx();
    ctx->team_opaque = &detail::team_of(team)->wrt_world;
  }
  (void)options;
  __syncthreads();
  return 0;
}

__device__ inline void roc_shmem_wg_ctx_destroy(roc_shmem_ctx_t) {}

__device__ inline int roc_shmem_ctx_n_pes(roc_shmem_ctx_t ctx) {
  (void)ctx;
  return detail::g_state.num_pes;
}
__device__ inline int roc_shmem_n_pes() { return detail::g_state.num_pes; }
__device__ inline int roc_shmem_ctx_my_pe(roc_shmem_ctx_t ctx) {
  return detail::pe_of(ctx);
}
__device__ inline int roc_shmem_my_pe() { return detail::launch_pe(); }

__device__ inline uint64_t roc_shmem_timer() { return wall_clock64(); }

// reference: team_translate_pe, team.cpp:47-60 and Team::get_pe_in_my_team, :89-107
__device__ inline int roc_shmem_team_translate_pe(roc_shmem_team_t src_team, int src_pe,
                                                  roc_shmem_team_t dest_team) {
  if (src_team == ROC_SHMEM_TEAM_INVALID || dest_team == ROC_SHMEM_TEAM_INVALID) return -1;
  const detail::TeamInfo &s = detail::team_of(src_team)->wrt_world;
  const detail::TeamInfo &d = detail::team_of(dest_team)->wrt_world;
  int in_world = s.pe_start + s.stride * src_pe;
  if (in_world < d.pe_start) return -1;
  if ((in_world - d.pe_start) % d.stride) return -1;
  int idx = (in_world - d.pe_start) / d.stride;
  return idx >= d.size ? -1 : idx;
}

// Every slice is directly addressable (reference: shmem_ptr returns nullptr
// when the target is not IPC-mapped, context_ib_device.cpp:128-137).
__device__ inline void *roc_shmem_ptr(const void *dest, int pe) {
  return detail::translate(detail::own(const_cast<void *>(dest), detail::launch_pe()),
                           detail::launch_pe(), pe);
}

// extension: the calling PE's address of the symmetric object that `ptr`
// names in any PE's slice; pointers outside the symmetric heap come back
// unchanged.  Lets one kernel argument serve the workgroups of every PE.
template <typename T>
__device__ inline T *roc_shmemx_my_addr(T *ptr) {
  const char *c = reinterpret_cast<const char *>(ptr);
  const char *base = detail::g_state.heap_base0;
  const uint64_t span = detail::g_state.slice_stride * static_cast<uint64_t>(detail::g_state.num_pes);
  if (c < base || static_cast<uint64_t>(c - base) >= span) return ptr;
  // (the usual argument is the symmetric address, in PE 0's slice: no division then)
  const uint64_t rel = static_cast<uint64_t>(c - base);
  const uint64_t off = rel < detail::g_state.slice_stride ? rel : rel % detail::g_state.slice_stride;
  return reinterpret_cast<T *>(const_cast<char *>(base) +
                               static_cast<uint64_t>(detail::launch_pe()) *
                                   detail::g_state.slice_stride +
                               off);
}

// ---------------------------------------------------------------------------
// Ordering
// ---------------------------------------------------------------------------

// fence: what the calling PE has issued is ordered before what it issues next.
// The operations are direct stores and atomics, which the memory fence orders.
// On a queue with a live consumer the call also leaves the entry the
// reference's fence posts (QueuePair::fence, queue_pair.cpp:376-384: an inline
// write to the flush word), one per call, since a context has one queue for
// all destinations.
__device__ inline void roc_shmem_ctx_fence(roc_shmem_ctx_t ctx) {
  detail::fence_acq_rel_agent();
  if (detail::g_state.sq_queue_mode == detail::kSqLive)
    detail::post_no_data_entry(detail::ctx_of(ctx), detail::kWqeFlushWrite);
}
__device__ inline void roc_shmem_ctx_fence(roc_shmem_ctx_t ctx, int) { roc_shmem_ctx_fence(ctx); }
__device__ inline void roc_shmem_fence() { roc_shmem_ctx_fence(ROC_SHMEM_CTX_DEFAULT); }
__device__ inline void roc_shmem_fence(int) { roc_shmem_ctx_fence(ROC_SHMEM_CTX_DEFAULT); }
// quiet: everything the calling PE has issued is complete and visible.  The
// operations themselves are direct stores and atomics, which the fence
// completes.  With a live consumer on the send queues the call also collects
// the completions its queue has asked for, as the reference's quiet does: a
// zero-byte read that asks for a completion (quiet_heavy, thread_policy.cpp:
// 35-108; QueuePair::zero_b_rd, queue_pair.cpp:318-325), then the poll
// (QueuePair::quiet_internal, queue_pair.cpp:118-191).
__device__ inline void roc_shmem_ctx_quiet(roc_shmem_ctx_t ctx) {
  detail::fence_acq_rel_agent();
  if (detail::g_state.sq_queue_mode == detail::kSqLive) {
    detail::post_no_data_entry(detail::ctx_of(ctx), detail::kWqeZeroByteRead);
    detail::quiet_live(detail::ctx_of(ctx));
  }
}
__device__ inline void roc_shmem_quiet() { roc_shmem_ctx_quiet(ROC_SHMEM_CTX_DEFAULT); }
__device__ inline void roc_shmem_ctx_threadfence_system(roc_shmem_ctx_t) {
  __threadfence_system();
}
__device__ inline void roc_shmem_threadfence_system() { __threadfence_system(); }

// ---------------------------------------------------------------------------
// Thread-level RMA
// ---------------------------------------------------------------------------

__device__ inline void roc_shmem_ctx_putmem(roc_shmem_ctx_t ctx, void *dest, const void *source,
                                            size_t nelems, int pe) {
  // The copy is synchronous in the calling lane, so `source` is reusable on
  // return (local completion, all OpenSHMEM asks of a blocking put).  Remote
  // visibility comes with quiet/fence/barrier; the reference adds a device-wide
  // __threadfence here (fence_.flush(), context_ib_device.cpp:164), which on a
  // multi-XCD part means writing back a whole L2 per call.
  detail::DeviceCtx *c = detail::ctx_of(ctx);
  detail::thread_put(c, detail::own(dest, c), detail::own(source, c), nelems, detail::world_pe(ctx, pe));
}
__device__ inline void roc_shmem_ctx_putmem_nbi(roc_shmem_ctx_t ctx, void *dest,
                                                const void *source, size_t nelems, int pe) {
  detail::DeviceCtx *c = detail::ctx_of(ctx);
  detail::thread_put(c, detail::own(dest, c), detail::own(source, c), nelems, detail::world_pe(ctx, pe));
}
__device__ inline void roc_shmem_ctx_getmem(roc_shmem_ctx_t ctx, void *dest, const void *source,
                                            size_t nelems, int pe) {
  detail::DeviceCtx *c = detail::ctx_of(ctx);
  detail::thread_get(c, detail::own(dest, c), detail::own(source, c), nelems, detail::world_pe(ctx, pe));
}
__device__ inline void roc_shmem_ctx_getmem_nbi(roc_shmem_ctx_t ctx, void *dest,
                                                const void *source, size_t nelems, int pe) {
  detail::DeviceCtx *c = detail::ctx_of(ctx);
  detail::thread_get(c, detail::own(dest, c), detail::own(source, c), nelems, detail::world_pe(ctx, pe));
}
__device__ inline void roc_shmem_putmem(void *dest, const void *source, size_t nelems, int pe) {
  roc_shmem_ctx_putmem(ROC_SHMEM_CTX_DEFAULT, dest, source, nelems, pe);
}
__device__ inline void roc_shmem_putmem_nbi(void *dest, const void *source, size_t nelems,
                                            int pe) {
  roc_shmem_ctx_putmem_nbi(ROC_SHMEM_CTX_DEFAULT, dest, source, nelems, pe);
}
__device__ inline void roc_shmem_getmem(void *dest, const void *source, size_t nelems, int pe) {
  roc_shmem_ctx_getmem(ROC_SHMEM_CTX_DEFAULT, dest, source, nelems, pe);
}
__device__ inline void roc_shmem_getmem_nbi(void *dest, const void *source, size_t nelems,
                                            int pe) {
  roc_shmem_ctx_getmem_nbi(ROC_SHMEM_CTX_DEFAULT, dest, source, nelems, pe);
}

// ---------------------------------------------------------------------------
// Workgroup- and wavefront-level RMA (reference: roc_shmem.hpp:2029-2566;
// GPUIBContext::putmem_wg ..., context_ib_device.cpp:189-321).  The PE is a
// world PE.  Blocking and non-blocking forms move the data the same way;
// roc_shmem_ctx_quiet / fence / a barrier make it visible to other PEs.
// ---------------------------------------------------------------------------

__device__ inline void roc_shmemx_ctx_putmem_nbi_wg(roc_shmem_ctx_t ctx, void *dest,
                                                    const void *source, size_t nelems, int pe) {
  if (nelems == 0) return;
  const int me = detail::pe_of(ctx);
  detail::wg_copy(detail::translate(detail::own(dest, me), me, pe), detail::own(source, me), nelems);
}
__device__ inline void roc_shmemx_ctx_putmem_wg(roc_shmem_ctx_t ctx, void *dest,
                                                const void *source, size_t nelems, int pe) {
  // On return the source is reusable, and every wave's stores are ordered before
  // whatever any lane of the workgroup issues next (a workgroup-scope release,
  // then the waves meet), so one lane's roc_shmem_ctx_quiet or fence afterwards -
  // an agent-scope release, which is cumulative - covers the whole workgroup's
  // put.  What is not done here is the L2 write-back that makes the bytes
  // visible to PEs on other XCDs: that is quiet's (the reference flushes in
  // the put itself, context_ib_device.cpp:148-165,219-236; with one L2 per XCD a
  // flush per call costs most of the bandwidth of small messages).
  roc_shmemx_ctx_putmem_nbi_wg(ctx, dest, source, nelems, pe);
  if (nelems != 0) {
    __builtin_amdgcn_fence(__ATOMIC_RELEASE, "workgroup");
    detail::wg_rendezvous();
  }
}
__device__ inline void roc_shmemx_ctx_getmem_nbi_wg(roc_shmem_ctx_t ctx, void *dest,
                                                    const void *source, size_t nelems, int pe) {
  if (nelems == 0) return;
  const int me = detail::pe_of(ctx);
  detail::wg_copy(detail::own(dest, me), detail::translate(detail::own(source, me), me, pe), nelems);
}
__device__ inline void roc_shmemx_ctx_getmem_wg(roc_shmem_ctx_t ctx, void *dest,
                                                const void *source, size_t nelems, int pe) {
  // Every lane of the workgroup may read any byte of `dest` on return.
  roc_shmemx_ctx_getmem_nbi_wg(ctx, dest, source, nelems, pe);
  if (nelems != 0) __syncthreads();
}
// extension: one transfer shared by `nshards` workgroups of the calling PE.
// (Always inlined: as a separate function the call takes its callee's register
// count, whatever the calling kernel was compiled for.)
// All of them pass the same dest / source / nelems / pe and their own shard
// number; a large transfer between mutually aligned buffers is dealt to them
// pass by pass.  Non-blocking in the sense of the _nbi forms: the source may
// be reused and the destination read when all shards have returned and
// roc_shmem_ctx_quiet (or the kernel's end) has passed.
__device__ __forceinline__ void roc_shmemx_ctx_putmem_wg_shard(roc_shmem_ctx_t ctx, void *dest,
                                                      const void *source, size_t nelems, int pe,
                                                      int shard, int nshards) {
  if (nelems == 0) return;
  const int me = detail::pe_of(ctx);
  detail::wg_copy_shard(detail::translate(detail::own(dest, me), me, pe), detail::own(source, me), nelems,
                        shard, nshards, detail::g_state.pace_copy_bytes_per_tick);
}
__device__ __forceinline__ void roc_shmemx_ctx_getmem_wg_shard(roc_shmem_ctx_t ctx, void *dest,
                                                      const void *source, size_t nelems, int pe,
                                                      int shard, int nshards) {
  if (nelems == 0) return;
  const int me = detail::pe_of(ctx);
  detail::wg_copy_shard(detail::own(dest, me), detail::translate(detail::own(source, me), me, pe), nelems,
                        shard, nshards, detail::g_state.pace_copy_bytes_per_tick);
}
__device__ inline void roc_shmemx_ctx_putmem_nbi_wave(roc_shmem_ctx_t ctx, void *dest,
                                                      const void *source, size_t nelems,
                                                      int pe) {
  if (nelems == 0) return;
  const int me = detail::pe_of(ctx);
  detail::wave_copy(detail::translate(detail::own(dest, me), me, pe), detail::own(source, me), nelems);
}
__device__ inline void roc_shmemx_ctx_putmem_wave(roc_shmem_ctx_t ctx, void *dest,
                                                  const void *source, size_t nelems, int pe) {
  // Same data movement as the non-blocking form: the lanes' own loads have
  // returned before their stores issue, so the source is reusable on return.
  roc_shmemx_ctx_putmem_nbi_wave(ctx, dest, source, nelems, pe);
}
__device__ inline void roc_shmemx_ctx_getmem_nbi_wave(roc_shmem_ctx_t ctx, void *dest,
                                                      const void *source, size_t nelems,
                                                      int pe) {
  if (nelems == 0) return;
  const int me = detail::pe_of(ctx);
  detail::wave_copy(detail::own(dest, me), detail::translate(detail::own(source, me), me, pe), nelems);
}
__device__ inline void roc_shmemx_ctx_getmem_wave(roc_shmem_ctx_t ctx, void *dest,
                                                  const void *source, size_t nelems, int pe) {
  // Same data movement as the non-blocking form: the wave's later loads of
  // `dest` follow its stores through the same vector memory pipeline.
  roc_shmemx_ctx_getmem_nbi_wave(ctx, dest, source, nelems, pe);
}

#define ROCSHMEM_X_DEFAULT_CTX_MEM(NAME)                                                  \
  __device__ inline void roc_shmemx_##NAME(void *dest, const void *source, size_t nelems, \
                                           int pe) {                                      \
    roc_shmemx_ctx_##NAME(ROC_SHMEM_CTX_DEFAULT, dest, source, nelems, pe);               \
  }
ROCSHMEM_X_DEFAULT_CTX_MEM(putmem_wg)
ROCSHMEM_X_DEFAULT_CTX_MEM(putmem_nbi_wg)
ROCSHMEM_X_DEFAULT_CTX_MEM(getmem_wg)
ROCSHMEM_X_DEFAULT_CTX_MEM(getmem_nbi_wg)
ROCSHMEM_X_DEFAULT_CTX_MEM(putmem_wave)
ROCSHMEM_X_DEFAULT_CTX_MEM(putmem_nbi_wave)
ROCSHMEM_X_DEFAULT_CTX_MEM(getmem_wave)
ROCSHMEM_X_DEFAULT_CTX_MEM(getmem_nbi_wave)
#undef ROCSHMEM_X_DEFAULT_CTX_MEM

// ---------------------------------------------------------------------------
// Typed RMA over the 13 standard types (reference: roc_shmem.hpp:1224-1237 and
// the PUT/GET/P/G generator macros :907-977, :2029-2110)
// ---------------------------------------------------------------------------

#define ROCSHMEM_STANDARD_TYPES(X)  \
  X(float, float)                   \
  X(double, double)                 \
  X(char, char)                     \
  X(signed char, schar)             \
  X(short, short)                   \
  X(int, int)                       \
  X(long, long)                     \
  X(long long, longlong)            \
  X(unsigned char, uchar)           \
  X(unsigned short, ushort)         \
  X(unsigned int, uint)             \
  X(unsigned long, ulong)           \
  X(unsigned long long, ulonglong)

#define ROCSHMEM_TYPED_RMA(T, TNAME)                                                          \
  __device__ inline void roc_shmem_ctx_##TNAME##_put(roc_shmem_ctx_t ctx, T *dest,            \
                                                     const T *source, size_t nelems, int pe) { \
    roc_shmem_ctx_putmem(ctx, dest, source, nelems * sizeof(T), pe);                           \
  }                                                                                            \
  __device__ inline void roc_shmem_##TNAME##_put(T *dest, const T *source, size_t nelems,      \
                                                 int pe) {                                     \
    roc_shmem_ctx_##TNAME##_put(ROC_SHMEM_CTX_DEFAULT, dest, source, nelems, pe);              \
  }                                                                                            \
  __device__ inline void roc_shmem_ctx_##TNAME##_put_nbi(                                      \
      roc_shmem_ctx_t ctx, T *dest, const T *source, size_t nelems, int pe) {                  \
    roc_shmem_ctx_putmem_nbi(ctx, dest, source, nelems * sizeof(T), pe);                       \
  }                                                                                            \
  __device__ inline void roc_shmem_##TNAME##_put_nbi(T *dest, const T *source, size_t nelems,  \
                                                     int pe) {                                 \
    roc_shmem_ctx_##TNAME##_put_nbi(ROC_SHMEM_CTX_DEFAULT, dest, source, nelems, pe);          \
  }                                                                                            \
  __device__ inline void roc_shmem_ctx_##TNAME##_get(roc_shmem_ctx_t ctx, T *dest,             \
                                                     const T *source, size_t nelems, int pe) { \
    roc_shmem_ctx_getmem(ctx, dest, source, nelems * sizeof(T), pe);                           \
  }                                                                                            \
  __device__ inline void roc_shmem_##TNAME##_get(T *dest, const T *source, size_t nelems,      \
                                                 int pe) {                                     \
    roc_shmem_ctx_##TNAME##_get(ROC_SHMEM_CTX_DEFAULT, dest, source, nelems, pe);              \
  }                                                                                            \
  __device__ inline void roc_shmem_ctx_##TNAME##_get_nbi(                                      \
      roc_shmem_ctx_t ctx, T *dest, const T *source, size_t nelems, int pe) {                  \
    roc_shmem_ctx_getmem_nbi(ctx, dest, source, nelems * sizeof(T), pe);                       \
  }                                                                                            \
  __device__ inline void roc_shmem_##TNAME##_get_nbi(T *dest, const T *source, size_t nelems,  \
                                                     int pe) {                                 \
    roc_shmem_ctx_##TNAME##_get_nbi(ROC_SHMEM_CTX_DEFAULT, dest, source, nelems, pe);          \
  }                                                                                            \
  __device__ inline void roc_shmem_ctx_##TNAME##_p(roc_shmem_ctx_t ctx, T *dest, T value,      \
                                                   int pe) {                                   \
    detail::DeviceCtx *c = detail::ctx_of(ctx);                                                \
    detail::thread_p<T>(c, detail::own(dest, c), value, detail::world_pe(ctx, pe));            \
  }                                                                                            \
  __device__ inline void roc_shmem_##TNAME##_p(T *dest, T value, int pe) {                     \
    roc_shmem_ctx_##TNAME##_p(ROC_SHMEM_CTX_DEFAULT, dest, value, pe);                         \
  }                                                                                            \
  __device__ inline T roc_shmem_ctx_##TNAME##_g(roc_shmem_ctx_t ctx, const T *source,          \
                                                int pe) {                                      \
    detail::DeviceCtx *c = detail::ctx_of(ctx);                                                \
    return detail::thread_g<T>(c, detail::own(source, c), detail::world_pe(ctx, pe));          \
  }                                                                                            \
  __device__ inline T roc_shmem_##TNAME##_g(const T *source, int pe) {                         \
    return roc_shmem_ctx_##TNAME##_g(ROC_SHMEM_CTX_DEFAULT, source, pe);                       \
  }
ROCSHMEM_STANDARD_TYPES(ROCSHMEM_TYPED_RMA)
#undef ROCSHMEM_TYPED_RMA

#define ROCSHMEM_TYPED_RMA_GRAN(T, TNAME, KIND, MEMKIND, GRAN, CONST_SRC)                     \
  __device__ inline void roc_shmemx_ctx_##TNAME##_##KIND##_##GRAN(                             \
      roc_shmem_ctx_t ctx, T *dest, const T *source, size_t nelems, int pe) {                  \
    roc_shmemx_ctx_##MEMKIND##_##GRAN(ctx, dest, source, nelems * sizeof(T), pe);              \
  }                                                                                            \
  __device__ inline void roc_shmemx_##TNAME##_##KIND##_##GRAN(T *dest, const T *source,        \
                                                              size_t nelems, int pe) {         \
    roc_shmemx_ctx_##MEMKIND##_##GRAN(ROC_SHMEM_CTX_DEFAULT, dest, source, nelems * sizeof(T), \
                                      pe);                                                     \
  }
#define ROCSHMEM_TYPED_RMA_GRAN_ALL(T, TNAME)                      \
  ROCSHMEM_TYPED_RMA_GRAN(T, TNAME, put, putmem, wg, )             \
  ROCSHMEM_TYPED_RMA_GRAN(T, TNAME, put, putmem, wave, )           \
  ROCSHMEM_TYPED_RMA_GRAN(T, TNAME, get, getmem, wg, )             \
  ROCSHMEM_TYPED_RMA_GRAN(T, TNAME, get, getmem, wave, )           \
  ROCSHMEM_TYPED_RMA_GRAN(T, TNAME, put_nbi, putmem_nbi, wg, )     \
  ROCSHMEM_TYPED_RMA_GRAN(T, TNAME, put_nbi, putmem_nbi, wave, )   \
  ROCSHMEM_TYPED_RMA_GRAN(T, TNAME, get_nbi, getmem_nbi, wg, )     \
  ROCSHMEM_TYPED_RMA_GRAN(T, TNAME, get_nbi, getmem_nbi, wave, )
ROCSHMEM_STANDARD_TYPES(ROCSHMEM_TYPED_RMA_GRAN_ALL)
#undef ROCSHMEM_TYPED_RMA_GRAN_ALL
#undef ROCSHMEM_TYPED_RMA_GRAN

// ---------------------------------------------------------------------------
// Reductions (reference: roc_shmem.hpp:837-868,1190-1198; both overloads)
// ---------------------------------------------------------------------------

namespace detail {
template <typename T, ROC_SHMEM_OP Op>
__device__ __forceinline__ void to_all_active_set(roc_shmem_ctx_t ctx, T *dest, const T *source,
                                                  size_t nreduce, int pe_start, int log_stride,
                                                  int pe_size, long *psync, int shard = 0,
                                                  int nshards = 1) {
  wg_all_reduce<T, Op>(pe_of(ctx), dest, source, nreduce, pe_start, 1 << log_stride,
                       pe_size, psync, shard, nshards);
}
// reference: GPUIBContext::to_all(team, ...), context_ib_tmpl_device.hpp:238-260
template <typename T, ROC_SHMEM_OP Op>
__device__ __forceinline__ void to_all_team(roc_shmem_ctx_t ctx, roc_shmem_team_t team, T *dest,
                                            const T *source, size_t nreduce, int shard = 0,
                                            int nshards = 1) {
  const Team *t = team_of(team);
  wg_all_reduce<T, Op>(pe_of(ctx), dest, source, nreduce, t->wrt_world.pe_start,
                       t->wrt_world.stride, t->wrt_world.size,
                       team_psync(ctx, t->reduce_psync_off), shard, nshards);
}
}  // namespace detail

// The _shard forms are an extension: `nshards` workgroups of every member PE
// share one reduction.  All of them pass the same dest / source / nreduce
// (a size_t here) and their own shard number; shard s uses its own pSync
// (active-set form) or the pSync slice of its context's block (team form).
// Every source must be complete before any workgroup of that PE calls, and a
// destination is complete only when all shards have returned (at the latest
// when the kernel ends).
#define ROCSHMEM_REDUCTION(T, TNAME, OPNAME, OP)                                              \
  __device__ inline void roc_shmem_ctx_##TNAME##_##OPNAME##_wg_to_all(                         \
      roc_shmem_ctx_t ctx, T *dest, const T *source, int nreduce, int PE_start,                \
      int logPE_stride, int PE_size, T *pWrk, long *pSync) {                                   \
    (void)pWrk;                                                                                \
    if (nreduce <= 0) return;                                                                  \
    detail::to_all_active_set<T, OP>(ctx, dest, source, static_cast<size_t>(nreduce),          \
                                     PE_start, logPE_stride, PE_size, pSync);                  \
  }                                                                                            \
  __device__ inline void roc_shmem_ctx_##TNAME##_##OPNAME##_wg_to_all(                         \
      roc_shmem_ctx_t ctx, roc_shmem_team_t team, T *dest, const T *source, int nreduce) {     \
    if (nreduce <= 0) return;                                                                  \
    detail::to_all_team<T, OP>(ctx, team, dest, source, static_cast<size_t>(nreduce));         \
  }                                                                                            \
  __device__ inline void roc_shmemx_ctx_##TNAME##_##OPNAME##_wg_to_all_shard(                  \
      roc_shmem_ctx_t ctx, T *dest, const T *source, size_t nreduce, int PE_start,             \
      int logPE_stride, int PE_size, T *pWrk, long *pSync, int shard, int nshards) {           \
    (void)pWrk;                                                                                \
    detail::to_all_active_set<T, OP>(ctx, dest, source, nreduce, PE_start, logPE_stride,       \
                                     PE_size, pSync, shard, nshards);                          \
  }                                                                                            \
  __device__ inline void roc_shmemx_ctx_##TNAME##_##OPNAME##_wg_to_all_shard(                  \
      roc_shmem_ctx_t ctx, roc_shmem_team_t team, T *dest, const T *source, size_t nreduce,    \
      int shard, int nshards) {                                                                \
    detail::to_all_team<T, OP>(ctx, team, dest, source, nreduce, shard, nshards);              \
  }
#define ROCSHMEM_ARITH_REDUCTIONS(T, TNAME)            \
  ROCSHMEM_REDUCTION(T, TNAME, sum, ROC_SHMEM_SUM)     \
  ROCSHMEM_REDUCTION(T, TNAME, min, ROC_SHMEM_MIN)     \
  ROCSHMEM_REDUCTION(T, TNAME, max, ROC_SHMEM_MAX)     \
  ROCSHMEM_REDUCTION(T, TNAME, prod, ROC_SHMEM_PROD)
#define ROCSHMEM_BITWISE_REDUCTIONS(T, TNAME)          \
  ROCSHMEM_REDUCTION(T, TNAME, or, ROC_SHMEM_OR)       \
  ROCSHMEM_REDUCTION(T, TNAME, and, ROC_SHMEM_AND)     \
  ROCSHMEM_REDUCTION(T, TNAME, xor, ROC_SHMEM_XOR)
ROCSHMEM_ARITH_REDUCTIONS(int, int)
ROCSHMEM_BITWISE_REDUCTIONS(int, int)
ROCSHMEM_ARITH_REDUCTIONS(short, short)
ROCSHMEM_BITWISE_REDUCTIONS(short, short)
ROCSHMEM_ARITH_REDUCTIONS(long, long)
ROCSHMEM_BITWISE_REDUCTIONS(long, long)
ROCSHMEM_ARITH_REDUCTIONS(long long, longlong)
ROCSHMEM_BITWISE_REDUCTIONS(long long, longlong)
ROCSHMEM_ARITH_REDUCTIONS(float, float)
ROCSHMEM_ARITH_REDUCTIONS(double, double)
// extension: bfloat16 sum/max/min (the reference has no 16-bit float type).
ROCSHMEM_REDUCTION(__hip_bfloat16, bf16, sum, ROC_SHMEM_SUM)
ROCSHMEM_REDUCTION(__hip_bfloat16, bf16, max, ROC_SHMEM_MAX)
ROCSHMEM_REDUCTION(__hip_bfloat16, bf16, min, ROC_SHMEM_MIN)
#undef ROCSHMEM_BITWISE_REDUCTIONS
#undef ROCSHMEM_ARITH_REDUCTIONS
#undef ROCSHMEM_REDUCTION

// ---------------------------------------------------------------------------
// Broadcast / alltoall / fcollect (reference: roc_shmem.hpp:873-902)
// ---------------------------------------------------------------------------

#define ROCSHMEM_COLLECTIVES(T, TNAME)                                                         \
  /* PE_root is the root's ordinal within the active set (OpenSHMEM 1.4; the */                \
  /* reference's host path passes it to MPI_Bcast the same way).             */                \
  __device__ inline void roc_shmem_ctx_##TNAME##_wg_broadcast(                                 \
      roc_shmem_ctx_t ctx, T *dest, const T *source, int nelem, int pe_root, int pe_start,     \
      int log_pe_stride, int pe_size, long *p_sync) {                                          \
    if (nelem <= 0) return;                                                                    \
    detail::wg_broadcast_bytes(detail::pe_of(ctx), dest, source,                       \
                               static_cast<size_t>(nelem) * sizeof(T), pe_root, pe_start,      \
                               1 << log_pe_stride, pe_size, p_sync);                           \
  }                                                                                            \
  __device__ inline void roc_shmem_ctx_##TNAME##_wg_broadcast(                                 \
      roc_shmem_ctx_t ctx, roc_shmem_team_t team, T *dest, const T *source, int nelem,         \
      int pe_root) {                                                                           \
    if (nelem <= 0) return;                                                                    \
    const detail::Team *t = detail::team_of(team);                                             \
    detail::wg_broadcast_bytes(detail::pe_of(ctx), dest, source, static_cast<size_t>(nelem) * sizeof(T), \
                               pe_root, t->wrt_world.pe_start, t->wrt_world.stride,            \
                               t->wrt_world.size, detail::team_psync(ctx, t->bcast_psync_off));  \
  }                                                                                            \
  /* extension: `nshards` workgroups of every member share one broadcast (same */              \
  /* arguments in all of them, nelem a size_t; complete when all have returned) */             \
  __device__ inline void roc_shmemx_ctx_##TNAME##_wg_broadcast_shard(                          \
      roc_shmem_ctx_t ctx, T *dest, const T *source, size_t nelem, int pe_root, int pe_start,  \
      int log_pe_stride, int pe_size, long *p_sync, int shard, int nshards) {                  \
    detail::wg_broadcast_bytes(detail::pe_of(ctx), dest, source, nelem * sizeof(T),    \
                               pe_root, pe_start, 1 << log_pe_stride, pe_size, p_sync, shard,  \
                               nshards);                                                       \
  }                                                                                            \
  __device__ inline void roc_shmemx_ctx_##TNAME##_wg_broadcast_shard(                          \
      roc_shmem_ctx_t ctx, roc_shmem_team_t team, T *dest, const T *source, size_t nelem,      \
      int pe_root, int shard, int nshards) {                                                   \
    const detail::Team *t = detail::team_of(team);                                             \
    detail::wg_broadcast_bytes(detail::pe_of(ctx), dest, source, nelem * sizeof(T), pe_root,             \
                               t->wrt_world.pe_start, t->wrt_world.stride,                     \
                               t->wrt_world.size, detail::team_psync(ctx, t->bcast_psync_off),   \
                               shard, nshards);                                                \
  }                                                                                            \
  /* extension: `nshards` workgroups of every member share the exchange */                        \
  __device__ inline void roc_shmemx_ctx_##TNAME##_wg_alltoall_shard(                           \
      roc_shmem_ctx_t ctx, roc_shmem_team_t team, T *dest, const T *source, int nelem,         \
      int shard, int nshards) {                                                                \
    if (nelem <= 0) return;                                                                    \
    const detail::Team *t = detail::team_of(team);                                             \
    detail::wg_alltoall_bytes(detail::pe_of(ctx), dest, source, static_cast<size_t>(nelem) * sizeof(T),  \
                              shard, nshards, t->wrt_world.pe_start, t->wrt_world.stride,      \
                              t->wrt_world.size, detail::team_psync(ctx, t->alltoall_psync_off)); \
  }                                                                                            \
  __device__ inline void roc_shmem_ctx_##TNAME##_wg_alltoall(                                  \
      roc_shmem_ctx_t ctx, roc_shmem_team_t team, T *dest, const T *source, int nelem) {       \
    roc_shmemx_ctx_##TNAME##_wg_alltoall_shard(ctx, team, dest, source, nelem, 0, 1);          \
  }                                                                                            \
  __device__ inline void roc_shmemx_ctx_##TNAME##_wg_fcollect_shard(                           \
      roc_shmem_ctx_t ctx, roc_shmem_team_t team, T *dest, const T *source, int nelem,         \
      int shard, int nshards) {                                                                \
    if (nelem <= 0) return;                                                                    \
    const detail::Team *t = detail::team_of(team);                                             \
    detail::wg_fcollect_bytes(detail::pe_of(ctx), dest, source, static_cast<size_t>(nelem) * sizeof(T),  \
                              shard, nshards, t->wrt_world.pe_start, t->wrt_world.stride,      \
                              t->wrt_world.size, detail::team_psync(ctx, t->alltoall_psync_off)); \
  }                                                                                            \
  __device__ inline void roc_shmem_ctx_##TNAME##_wg_fcollect(                                  \
      roc_shmem_ctx_t ctx, roc_shmem_team_t team, T *dest, const T *source, int nelem) {       \
    roc_shmemx_ctx_##TNAME##_wg_fcollect_shard(ctx, team, dest, source, nelem, 0, 1);          \
  }
ROCSHMEM_STANDARD_TYPES(ROCSHMEM_COLLECTIVES)
#undef ROCSHMEM_COLLECTIVES

// ---------------------------------------------------------------------------
// Barriers (reference: context_ib_device_coll.cpp:91-120)
// ---------------------------------------------------------------------------

__device__ inline void roc_shmem_ctx_wg_team_sync(roc_shmem_ctx_t ctx, roc_shmem_team_t team) {
  const detail::Team *t = detail::team_of(team);
  detail::wg_sync_members(detail::pe_of(ctx), t->wrt_world.pe_start, t->wrt_world.stride,
                          t->wrt_world.size, detail::team_psync(ctx, t->barrier_psync_off));
}
__device__ inline void roc_shmem_wg_team_sync(roc_shmem_team_t team) {
  roc_shmem_ctx_wg_team_sync(ROC_SHMEM_CTX_DEFAULT, team);
}
__device__ inline void roc_shmem_ctx_wg_sync_all(roc_shmem_ctx_t ctx) {
  const detail::Team *t = detail::g_state.team_world;
  detail::wg_sync_members(detail::pe_of(ctx), 0, 1, detail::g_state.num_pes,
                          detail::team_psync(ctx, t->barrier_psync_off));
}
__device__ inline void roc_shmem_wg_sync_all() { roc_shmem_ctx_wg_sync_all(ROC_SHMEM_CTX_DEFAULT); }
__device__ inline void roc_shmem_ctx_wg_barrier_all(roc_shmem_ctx_t ctx) {
  // quiet + sync_all; the barrier's arrival already publishes prior stores.
  roc_shmem_ctx_wg_sync_all(ctx);
}
__device__ inline void roc_shmem_wg_barrier_all() {
  roc_shmem_ctx_wg_barrier_all(ROC_SHMEM_CTX_DEFAULT);
}

// ---------------------------------------------------------------------------
// Atomic memory operations (reference: roc_shmem.hpp:982-1147,1548-1953)
// ---------------------------------------------------------------------------

#define ROCSHMEM_AMO_STANDARD_TYPES(X) \
  X(int, int)                          \
  X(long, long)                        \
  X(long long, longlong)               \
  X(unsigned int, uint)                \
  X(unsigned long, ulong)              \
  X(unsigned long long, ulonglong)     \
  X(int32_t, int32)                    \
  X(int64_t, int64)                    \
  X(uint32_t, uint32)                  \
  X(uint64_t, uint64)                  \
  X(size_t, size)                      \
  X(ptrdiff_t, ptrdiff)

#define ROCSHMEM_AMO_STANDARD(T, TNAME)                                                        \
  __device__ inline T roc_shmem_ctx_##TNAME##_atomic_fetch_add(roc_shmem_ctx_t ctx, T *dest,   \
                                                               T value, int pe) {              \
    return detail::amo_fetch_add<T>(detail::ctx_of(ctx), dest, value, pe);                     \
  }                                                                                            \
  __device__ inline T roc_shmem_##TNAME##_atomic_fetch_add(T *dest, T value, int pe) {         \
    return roc_shmem_ctx_##TNAME##_atomic_fetch_add(ROC_SHMEM_CTX_DEFAULT, dest, value, pe);   \
  }                                                                                            \
  __device__ inline T roc_shmem_ctx_##TNAME##_atomic_compare_swap(                             \
      roc_shmem_ctx_t ctx, T *dest, T cond, T value, int pe) {                                 \
    return detail::amo_fetch_cas<T>(detail::ctx_of(ctx), dest, value, cond, pe);               \
  }                                                                                            \
  __device__ inline T roc_shmem_##TNAME##_atomic_compare_swap(T *dest, T cond, T value,        \
                                                              int pe) {                        \
    return roc_shmem_ctx_##TNAME##_atomic_compare_swap(ROC_SHMEM_CTX_DEFAULT, dest, cond,      \
                                                       value, pe);                             \
  }                                                                                            \
  __device__ inline T roc_shmem_ctx_##TNAME##_atomic_fetch_inc(roc_shmem_ctx_t ctx, T *dest,   \
                                                               int pe) {                       \
    return detail::amo_fetch_add<T>(detail::ctx_of(ctx), dest, static_cast<T>(1), pe);                      \
  }                                                                                            \
  __device__ inline T roc_shmem_##TNAME##_atomic_fetch_inc(T *dest, int pe) {                  \
    return roc_shmem_ctx_##TNAME##_atomic_fetch_inc(ROC_SHMEM_CTX_DEFAULT, dest, pe);          \
  }                                                                                            \
  __device__ inline void roc_shmem_ctx_##TNAME##_atomic_add(roc_shmem_ctx_t ctx, T *dest,      \
                                                            T value, int pe) {                 \
    detail::amo_add<T>(detail::ctx_of(ctx), dest, value, pe);                                  \
  }                                                                                            \
  __device__ inline void roc_shmem_##TNAME##_atomic_add(T *dest, T value, int pe) {            \
    roc_shmem_ctx_##TNAME##_atomic_add(ROC_SHMEM_CTX_DEFAULT, dest, value, pe);                \
  }                                                                                            \
  __device__ inline void roc_shmem_ctx_##TNAME##_atomic_inc(roc_shmem_ctx_t ctx, T *dest,      \
                                                            int pe) {                          \
    detail::amo_add<T>(detail::ctx_of(ctx), dest, static_cast<T>(1), pe);                                   \
  }                                                                                            \
  __device__ inline void roc_shmem_##TNAME##_atomic_inc(T *dest, int pe) {                     \
    roc_shmem_ctx_##TNAME##_atomic_inc(ROC_SHMEM_CTX_DEFAULT, dest, pe);                       \
  }
ROCSHMEM_AMO_STANDARD_TYPES(ROCSHMEM_AMO_STANDARD)
#undef ROCSHMEM_AMO_STANDARD

// fetch / set / swap also exist for float and double (reference: :1647-1760).
#define ROCSHMEM_AMO_EXTENDED(T, TNAME)                                                        \
  __device__ inline T roc_shmem_ctx_##TNAME##_atomic_fetch(roc_shmem_ctx_t ctx, T *dest,       \
                                                           int pe) {                           \
    return detail::amo_fetch<T>(detail::ctx_of(ctx), dest, pe);                                \
  }                                                                                            \
  __device__ inline T roc_shmem_##TNAME##_atomic_fetch(T *dest, int pe) {                      \
    return roc_shmem_ctx_##TNAME##_atomic_fetch(ROC_SHMEM_CTX_DEFAULT, dest, pe);              \
  }                                                                                            \
  __device__ inline void roc_shmem_ctx_##TNAME##_atomic_set(roc_shmem_ctx_t ctx, T *dest,      \
                                                            T value, int pe) {                 \
    (void)detail::amo_swap<T>(detail::ctx_of(ctx), dest, value, pe);                           \
  }                                                                                            \
  __device__ inline void roc_shmem_##TNAME##_atomic_set(T *dest, T value, int pe) {            \
    roc_shmem_ctx_##TNAME##_atomic_set(ROC_SHMEM_CTX_DEFAULT, dest, value, pe);                \
  }                                                                                            \
  __device__ inline T roc_shmem_ctx_##TNAME##_atomic_swap(roc_shmem_ctx_t ctx, T *dest,        \
                                                          T value, int pe) {                   \
    return detail::amo_swap<T>(detail::ctx_of(ctx), dest, value, pe);                          \
  }                                                                                            \
  __device__ inline T roc_shmem_##TNAME##_atomic_swap(T *dest, T value, int pe) {              \
    return roc_shmem_ctx_##TNAME##_atomic_swap(ROC_SHMEM_CTX_DEFAULT, dest, value, pe);        \
  }
ROCSHMEM_AMO_STANDARD_TYPES(ROCSHMEM_AMO_EXTENDED)
ROCSHMEM_AMO_EXTENDED(float, float)
ROCSHMEM_AMO_EXTENDED(double, double)
#undef ROCSHMEM_AMO_EXTENDED

#define ROCSHMEM_AMO_BITWISE_TYPES(X) \
  X(unsigned int, uint)               \
  X(unsigned long, ulong)             \
  X(unsigned long long, ulonglong)    \
  X(int32_t, int32)                   \
  X(int64_t, int64)                   \
  X(uint32_t, uint32)                 \
  X(uint64_t, uint64)

#define ROCSHMEM_AMO_BITWISE_ONE(T, TNAME, OPNAME, OP)                                         \
  __device__ inline T roc_shmem_ctx_##TNAME##_atomic_fetch_##OPNAME(                           \
      roc_shmem_ctx_t ctx, T *dest, T value, int pe) {                                         \
    return detail::amo_fetch_bitwise<T, OP>(detail::ctx_of(ctx), dest, value, pe);             \
  }                                                                                            \
  __device__ inline T roc_shmem_##TNAME##_atomic_fetch_##OPNAME(T *dest, T value, int pe) {    \
    return roc_shmem_ctx_##TNAME##_atomic_fetch_##OPNAME(ROC_SHMEM_CTX_DEFAULT, dest, value,   \
                                                         pe);                                  \
  }                                                                                            \
  __device__ inline void roc_shmem_ctx_##TNAME##_atomic_##OPNAME(roc_shmem_ctx_t ctx, T *dest, \
                                                                 T value, int pe) {            \
    (void)detail::amo_fetch_bitwise<T, OP>(detail::ctx_of(ctx), dest, value, pe);              \
  }                                                                                            \
  __device__ inline void roc_shmem_##TNAME##_atomic_##OPNAME(T *dest, T value, int pe) {       \
    roc_shmem_ctx_##TNAME##_atomic_##OPNAME(ROC_SHMEM_CTX_DEFAULT, dest, value, pe);           \
  }
#define ROCSHMEM_AMO_BITWISE(T, TNAME)                          \
  ROCSHMEM_AMO_BITWISE_ONE(T, TNAME, and, detail::kBitAnd)      \
  ROCSHMEM_AMO_BITWISE_ONE(T, TNAME, or, detail::kBitOr)        \
  ROCSHMEM_AMO_BITWISE_ONE(T, TNAME, xor, detail::kBitXor)
ROCSHMEM_AMO_BITWISE_TYPES(ROCSHMEM_AMO_BITWISE)
#undef ROCSHMEM_AMO_BITWISE
#undef ROCSHMEM_AMO_BITWISE_ONE

// ---------------------------------------------------------------------------
// Point-to-point synchronisation (reference: roc_shmem.hpp:1152-1163;
// Context::wait_until / test, context_tmpl_device.hpp:199-246).  Waits are
// bounded; see sync.hpp.
// ---------------------------------------------------------------------------

#define ROCSHMEM_WAIT_TYPES(X) \
  X(float, float)              \
  X(double, double)            \
  X(char, char)                \
  X(signed char, schar)        \
  X(short, short)              \
  X(unsigned char, uchar)      \
  X(unsigned short, ushort)    \
  X(int, int)                  \
  X(long, long)                \
  X(long long, longlong)       \
  X(unsigned int, uint)        \
  X(unsigned long, ulong)      \
  X(unsigned long long, ulonglong)

#define ROCSHMEM_WAIT(T, TNAME)                                                                \
  __device__ inline void roc_shmem_##TNAME##_wait_until(T *ptr, roc_shmem_cmps cmp, T val) {   \
    detail::bounded_wait<T>(detail::own(ptr, detail::launch_pe()), static_cast<int>(cmp), val); \
    detail::fence_acquire_agent();                                                             \
  }                                                                                            \
  __device__ inline int roc_shmem_##TNAME##_test(T *ptr, roc_shmem_cmps cmp, T val) {          \
    using W = typename detail::WaitWord<T>::type;                                              \
    W raw = __hip_atomic_load(reinterpret_cast<W *>(detail::own(ptr, detail::launch_pe())),    \
                              __ATOMIC_RELAXED,                                                \
                              __HIP_MEMORY_SCOPE_AGENT);                                       \
    T have;                                                                                    \
    __builtin_memcpy(&have, &raw, sizeof(T));                                                  \
    int ok = detail::compare_for_wait(have, static_cast<int>(cmp), val) ? 1 : 0;               \
    if (ok) detail::fence_acquire_agent();                                                     \
    return ok;                                                                                 \
  }
ROCSHMEM_WAIT_TYPES(ROCSHMEM_WAIT)
#undef ROCSHMEM_WAIT

}  // namespace rocshmem

#endif
