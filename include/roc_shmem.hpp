// roc_shmem.hpp -- OpenSHMEM-style host/device API of the MI355X-native data path.
//
// Same names, argument order and meaning as ROC_SHMEM's public interface
// (library/include/roc_shmem.hpp in the reference), so kernels written against
// that header compile against this one.  The implementation behind it is
// different in kind: one process hosts every PE, each PE's symmetric-heap
// slice lives in the same GPU's HBM, and a workgroup acts for the PE that the
// launch grid assigns to it:
//
//     pe      = blockIdx.x % roc_shmem_n_pes()
//     wg_rank = blockIdx.x / roc_shmem_n_pes()      (index among that PE's workgroups)
//
// Device functions are defined inline (no relocatable device code needed);
// host functions live in librocshmem_mi355x.so.
//
// Extensions over the reference interface are marked "extension" where they are
// defined: bfloat16 reductions (roc_shmem_ctx_bf16_{sum,max,min}_wg_to_all);
// the _shard forms, which let several workgroups of every member PE share one
// operation (roc_shmemx_ctx_<T>_<op>_wg_to_all_shard, ..._wg_broadcast_shard,
// ..._wg_alltoall_shard, ..._wg_fcollect_shard, roc_shmemx_ctx_{put,get}mem_wg_shard);
// roc_shmemx_my_addr; swap / set / bitwise atomics; and the host helpers
// roc_shmemx_set_pe, roc_shmemx_host_ptr, roc_shmemx_take_status.
#ifndef ROCSHMEM_MI355X_ROC_SHMEM_HPP
#define ROCSHMEM_MI355X_ROC_SHMEM_HPP

#include <hip/hip_runtime.h>
#include <stddef.h>
#include <stdint.h>

#if defined(__has_include)
#if __has_include(<mpi.h>) && !defined(ROCSHMEM_NO_MPI)
#include <mpi.h>
#else
#include "compat/mpi.h"
#endif
#else
#include "compat/mpi.h"
#endif

namespace rocshmem {

// ---------------------------------------------------------------------------
// Enumerations, constants and handle types (reference: roc_shmem.hpp:52-131)
// ---------------------------------------------------------------------------

enum ROC_SHMEM_OP {
  ROC_SHMEM_SUM,
  ROC_SHMEM_MAX,
  ROC_SHMEM_MIN,
  ROC_SHMEM_PROD,
  ROC_SHMEM_AND,
  ROC_SHMEM_OR,
  ROC_SHMEM_XOR,
  ROC_SHMEM_REPLACE
};

enum roc_shmem_cmps {
  ROC_SHMEM_CMP_EQ,
  ROC_SHMEM_CMP_NE,
  ROC_SHMEM_CMP_GT,
  ROC_SHMEM_CMP_GE,
  ROC_SHMEM_CMP_LT,
  ROC_SHMEM_CMP_LE,
};

enum roc_shmem_thread_ops {
  ROC_SHMEM_THREAD_SINGLE,
  ROC_SHMEM_THREAD_FUNNELED,
  ROC_SHMEM_THREAD_WG_FUNNELED,
  ROC_SHMEM_THREAD_SERIALIZED,
  ROC_SHMEM_THREAD_MULTIPLE
};

enum roc_shmem_team_configs { ROC_SHMEM_TEAM_DEFAULT_CONFIGS, ROC_SHMEM_TEAM_NUM_CONTEXTS };

typedef struct {
  int num_contexts;
} roc_shmem_team_config_t;

constexpr size_t ROC_SHMEM_REDUCE_MIN_WRKDATA_SIZE = 1024;
constexpr size_t ROC_SHMEM_ATA_MAX_WRKDATA_SIZE = 4 * 1024 * 1024;
constexpr size_t ROC_SHMEM_BARRIER_SYNC_SIZE = 256;
constexpr size_t ROC_SHMEM_REDUCE_SYNC_SIZE = 256;
constexpr size_t ROC_SHMEM_BCAST_SYNC_SIZE = ROC_SHMEM_BARRIER_SYNC_SIZE;
constexpr size_t ROC_SHMEM_ALLTOALL_SYNC_SIZE = ROC_SHMEM_BARRIER_SYNC_SIZE + 1;
constexpr size_t ROC_SHMEM_FCOLLECT_SYNC_SIZE = ROC_SHMEM_ALLTOALL_SYNC_SIZE;
constexpr size_t ROC_SHMEM_SYNC_VALUE = 0;

const int ROC_SHMEM_CTX_ZERO = 0;
const int ROC_SHMEM_CTX_NOSTORE = 1;
const int ROC_SHMEM_CTX_SERIALIZED = 2;
const int ROC_SHMEM_CTX_WG_PRIVATE = 4;
const int ROC_SHMEM_CTX_SHARED = 8;

typedef struct {
  void *ctx_opaque;
  void *team_opaque;
} roc_shmem_ctx_t;

// The default context.  A null ctx_opaque names "the context of the calling
// workgroup's PE and block", on the device and on the host alike.
static __constant__ roc_shmem_ctx_t ROC_SHMEM_CTX_DEFAULT = {nullptr, nullptr};

typedef uint64_t *roc_shmem_team_t;
extern roc_shmem_team_t ROC_SHMEM_TEAM_WORLD;
const roc_shmem_team_t ROC_SHMEM_TEAM_INVALID = nullptr;

}  // namespace rocshmem

#include "rocshmem_device/state.hpp"

namespace rocshmem {

// ---------------------------------------------------------------------------
// Host interface (reference: roc_shmem.hpp:144-330, roc_shmem.cpp:71-313)
// ---------------------------------------------------------------------------

// Bring the runtime up: ROC_SHMEM_NUM_PES slices of ROC_SHMEM_HEAP_SIZE bytes
// in one HBM arena, ROC_SHMEM_NUM_BLOCKS contexts per PE each with a
// ROC_SHMEM_SQ_SIZE-entry send queue.  `comm` is accepted for source
// compatibility and ignored (there is a single process).
__host__ void roc_shmem_init(MPI_Comm comm = MPI_COMM_WORLD);
__host__ void roc_shmem_init_thread(int requested, int *provided, MPI_Comm comm = MPI_COMM_WORLD);
__host__ void roc_shmem_query_thread(int *provided);
__host__ void roc_shmem_finalize();
__host__ void roc_shmem_dump_stats();
__host__ void roc_shmem_reset_stats();
__host__ void roc_shmem_global_exit(int status);

// Symmetric allocation: the returned address belongs to the host's current
// PE (see roc_shmemx_set_pe); the same offset is reserved in every slice.
__host__ void *roc_shmem_malloc(size_t size);
__host__ void roc_shmem_free(void *ptr);
__host__ int roc_shmem_n_pes();
__host__ int roc_shmem_my_pe();

__host__ int roc_shmem_ctx_create(int64_t options, roc_shmem_ctx_t *ctx);
__host__ void roc_shmem_ctx_destroy(roc_shmem_ctx_t ctx);

__host__ int roc_shmem_team_translate_pe(roc_shmem_team_t src_team, int src_pe,
                                         roc_shmem_team_t dest_team);
__host__ int roc_shmem_team_n_pes(roc_shmem_team_t team);
__host__ int roc_shmem_team_my_pe(roc_shmem_team_t team);
__host__ int roc_shmem_team_split_strided(roc_shmem_team_t parent_team, int start, int stride,
                                          int size, const roc_shmem_team_config_t *config,
                                          long config_mask, roc_shmem_team_t *new_team);
__host__ void roc_shmem_team_destroy(roc_shmem_team_t team);

__host__ void roc_shmem_barrier_all();
__host__ void roc_shmem_sync_all();
__host__ void roc_shmem_quiet();
__host__ void roc_shmem_fence();

// Dump the eight 64-bit words of one send-queue entry / report the queue's
// producer state (reference: library/include/debug.hpp, qe_dumper.cpp:51-76).
__host__ void debug_print_sq(int dest_pe, int src_wg, int index_wqe);
__host__ void debug_print_cq(int dest_pe, int src_wg, int cqe_index);

// extension: the PE on whose behalf subsequent host calls act (one process
// stands for every PE, so "my PE" on the host is a setting, not an identity).
__host__ void roc_shmemx_set_pe(int pe);
// extension: address of symmetric object `ptr` (given for the current PE) in PE `pe`'s slice.
__host__ void *roc_shmemx_host_ptr(const void *ptr, int pe);
// extension: first non-zero status raised by device code since the last call (0 = none).
__host__ int roc_shmemx_take_status();

// Non-template workers behind the typed host data-path functions of
// roc_shmem_host.hpp.  `dest`/`source` naming a symmetric object are the
// current PE's addresses (roc_shmemx_set_pe); the other side may be any host
// or device pointer.
namespace hostx {
void putmem(void *dest, const void *source, size_t nbytes, int pe, bool blocking);
void getmem(void *dest, const void *source, size_t nbytes, int pe, bool blocking);
// kind: 0 fetch_add, 1 compare_swap, 2 swap, 3 fetch_and, 4 fetch_or, 5 fetch_xor; width 4 or 8.
// Returns the previous value of the word, zero-extended.
uint64_t amo(int kind, void *dest, uint64_t value, uint64_t cond, int pe, int width);
// The current PE's copy of the naturally aligned word of `width` (1, 2, 4 or 8) bytes at the
// symmetric address `ptr`, zero-extended, as a kernel that is still running has left it.
uint64_t fetch_own(const void *ptr, int width);
double wait_limit_seconds();  // bound of a host-side wait (ROC_SHMEM_WAIT_LIMIT_S)
// dtype / op use the codes of rsm_dtype / rsm_op (rocshmem_mi355x.h).
void to_all(int dtype, int op, void *dest, const void *source, int nreduce, int pe_start,
            int log_pe_stride, int pe_size);
void to_all_team(int dtype, int op, roc_shmem_team_t team, void *dest, const void *source,
                 int nreduce);
void broadcast(size_t elem_size, void *dest, const void *source, int nelem, int pe_root,
               int pe_start, int log_pe_stride, int pe_size);
void broadcast_team(size_t elem_size, roc_shmem_team_t team, void *dest, const void *source,
                    int nelem, int pe_root);
}  // namespace hostx

namespace detail {
// Registration of one translation unit's copy of the device state.
typedef bool (*StateUploadFn)(const DeviceState *);
// `layout` is the unit's detail::kStateLayout; roc_shmem_init fails when it is
// not the library's own.
void register_state_upload(StateUploadFn fn, uint32_t layout);
}  // namespace detail

}  // namespace rocshmem

// ---------------------------------------------------------------------------
// Device interface
// ---------------------------------------------------------------------------
#if defined(__HIPCC__)
#include "rocshmem_device/api.hpp"
#endif

// Typed host data-path functions (put/get/p/g, AMOs, to_all, broadcast).
#include "roc_shmem_host.hpp"

#endif  // ROCSHMEM_MI355X_ROC_SHMEM_HPP
