// Shared helpers of the C-ABI translation units.
#ifndef ROCSHMEM_MI355X_CABI_COMMON_HPP
#define ROCSHMEM_MI355X_CABI_COMMON_HPP

#include <hip/hip_runtime.h>

#include <mutex>
#include <string>

#include "host/runtime.hpp"
#include "rocshmem_mi355x.h"

namespace rsm {

int fail(const std::string &msg);   // records the message, returns -1
void clear_error();

struct Launch {
  int wgs_per_pe;
  int wg_size;
  size_t tile;
  hipStream_t stream;
  unsigned grid;   // wgs_per_pe * num_pes
};

// Validates the runtime and the launch shape; false (with the error set) on failure.
bool resolve_launch(const rsm_launch_t *in, Launch *out);

// True when `p` is a symmetric address in PE 0's slice (or NULL when allowed).
// One lock for the whole C ABI: entry points may be called from any host thread, one runs at a
// time (they share the allocator, the team table and the last-error text).  Recursive because
// entry points call each other.
std::recursive_mutex &abi_lock();
#define RSM_ENTRY std::lock_guard<std::recursive_mutex> rsm_entry_guard_(rsm::abi_lock())

bool check_symmetric(const void *p, const char *what, bool allow_null = false);
// `bytes` starting at the symmetric address `p` stay inside the live symmetric allocation that
// contains `p` (a kernel that ran past it would overwrite its neighbours or fault the device);
// true for addresses outside the arena, which cannot be judged here.
bool check_extent(const void *p, size_t bytes, const char *what);

// Members pe_start + k * 2^log_pe_stride, k < pe_size, of an active set all exist among
// `num_pes` PEs and the set has at most kMaxPes members.  Pure host arithmetic in 64 bits:
// a 32-bit shift by a large log_pe_stride wraps and would let a set through whose members
// lie far outside the arena.
bool active_set_in_range(int pe_start, int log_pe_stride, int pe_size, int num_pes);

// Device address, on the current device, of the flag array that rsm_to_all_noalloc uses
// (defined beside the array in drv_reduce.hip); looked up on a device's first call, which
// rsm_init makes.  nullptr, with the error set, when the runtime cannot resolve it.
long *noalloc_flags();

// Stops a live send-queue consumer, if one is running, and releases its stream and control
// block (drv_consume.hip); rsm_finalize calls it before the runtime is destroyed.
void consumer_shutdown();
void consumer_stop_for_teardown();   // the same stop, in the form the runtime's teardown calls
// True between rsm_sq_consumer_start and rsm_sq_consumer_stop.  A device-wide synchronisation
// would then wait for the consumer kernel, which runs until it is told to stop: entry points
// that synchronise the device refuse to run meanwhile (use rsm_stream_synchronize).
bool live_consumer_running();

// Waits until the device is idle, for entry points that read or change what kernels use.  With
// a live consumer running the wait would only end when the consumer gave up by itself (and the
// queues would be left without one): the call is refused instead, false with the error set.
bool device_idle(const char *who);

// hipGetLastError() after a launch, folded into the error convention.
int after_launch(const char *what);

}  // namespace rsm

#endif
