// C ABI: the consumer pass over the send queues, completion-queue inspection
// and the log/queue switch of the rings.
#include <chrono>

#include "cabi_common.hpp"
#include "roc_shmem.hpp"
#include "rocshmem_device/consume.hpp"

using namespace rocshmem;
using rocshmem::host::Runtime;

namespace {

// One wave per ring; rings outside the selection leave at once.
__global__ void __launch_bounds__(64)
    consume_kernel(int pe_sel, int block_sel, char *target, detail::ConsumeTotals *totals) {
  const int ring = blockIdx.x;
  const int pe = ring / detail::g_state.num_blocks;
  const int block = ring % detail::g_state.num_blocks;
  if ((pe_sel >= 0 && pe != pe_sel) || (block_sel >= 0 && block != block_sel)) return;
  detail::consume_ring(&detail::g_state.ctx_table[ring], target, totals);
}

// The consumer that runs beside the producers: wave w serves rings w, w + gridDim.x, ...
__global__ void __launch_bounds__(64)
    consume_live_kernel(detail::ConsumeTotals *totals, detail::LiveControl *control,
                        detail::LiveRelay *relay, uint64_t idle_limit_ticks) {
  const uint32_t n_rings =
      static_cast<uint32_t>(detail::g_state.num_pes) * static_cast<uint32_t>(detail::g_state.num_blocks);
  detail::consume_live(detail::g_state.ctx_table, blockIdx.x, gridDim.x, n_rings, totals, control,
                       relay, gridDim.x, idle_limit_ticks);
}

__global__ void clear_words_kernel(uint32_t *words, int n) {
  if (static_cast<int>(threadIdx.x) < n) words[threadIdx.x] = 0;
}

// State of the live consumer, one per process (the library drives one device).
struct LiveConsumer {
  hipStream_t stream = nullptr;             // non-blocking: work on the null stream does not wait for it
  detail::LiveControl *control = nullptr;   // host memory the device can address
  bool running = false;
  uint32_t mode_before = detail::kSqLog;
  // pacing rates that were set when the consumer started: a paced grid assumes that all of its
  // workgroups are resident, which the consumer's waves may prevent, so pacing rests meanwhile
  uint32_t pace_copy_before = 0, pace_reduce_before = 0;
};
LiveConsumer g_live;

constexpr unsigned kLiveMaxWaves = 1024;

bool ring_args_ok(Runtime *rt, int pe, int block) {
  return pe >= 0 && pe < rt->num_pes() && block >= 0 && block < rt->options().num_blocks;
}

}  // namespace

namespace rsm {
bool live_consumer_running() { return g_live.running; }

// What the runtime calls when it is torn down with the consumer still up (a finalize through
// the host interface, which knows nothing of this file).
void consumer_stop_for_teardown() {
  if (g_live.running) {
    rsm_consume_totals_t ignored;
    (void)rsm_sq_consumer_stop(&ignored);
  }
}

// Called by rsm_finalize before the runtime goes away: a consumer that is still running is
// told to stop and waited for, and what start allocated is released.
void consumer_shutdown() {
  if (g_live.running) {
    rsm_consume_totals_t ignored;
    (void)rsm_sq_consumer_stop(&ignored);
  }
  if (g_live.stream) (void)hipStreamDestroy(g_live.stream);
  if (g_live.control) (void)hipHostFree(g_live.control);
  g_live = LiveConsumer{};
}
}  // namespace rsm

#define CONSUME_HIP(expr)                                                          \
  do {                                                                             \
    hipError_t e_ = (expr);                                                        \
    if (e_ != hipSuccess)                                                          \
      return rsm::fail(std::string(#expr " failed: ") + hipGetErrorString(e_));    \
  } while (0)

extern "C" {

int rsm_sq_consume(int pe, int block, void *target_arena, rsm_consume_totals_t *totals) {
  RSM_ENTRY;
  Runtime *rt = Runtime::get();
  if (!rt) return rsm::fail("rsm_init has not been called");
  if (!rsm::device_idle("rsm_sq_consume")) return -1;
  if ((pe != -1 && (pe < 0 || pe >= rt->num_pes())) ||
      (block != -1 && (block < 0 || block >= rt->options().num_blocks)))
    return rsm::fail("rsm_sq_consume: pe / block out of range (-1 selects all)");
  static_assert(sizeof(rsm_consume_totals_t) == sizeof(detail::ConsumeTotals), "totals layout");
  static_assert(sizeof(detail::ConsumeTotals) <= 256, "totals fit the runtime's result scratch");
  detail::ConsumeTotals *dev = static_cast<detail::ConsumeTotals *>(rt->result_scratch());
  CONSUME_HIP(hipMemset(dev, 0, sizeof(*dev)));
  const unsigned rings = static_cast<unsigned>(rt->num_pes()) * rt->options().num_blocks;
  hipLaunchKernelGGL(consume_kernel, dim3(rings), dim3(64), 0, nullptr, pe, block,
                     static_cast<char *>(target_arena), dev);
  CONSUME_HIP(hipGetLastError());
  if (!rsm::device_idle("rsm_sq_consume")) return -1;
  rsm_consume_totals_t host = {};
  CONSUME_HIP(hipMemcpy(&host, dev, sizeof(host), hipMemcpyDeviceToHost));
  if (totals) *totals = host;
  return 0;
}

int rsm_sq_consumer_start(void) {
  RSM_ENTRY;
  Runtime *rt = Runtime::get();
  if (!rt) return rsm::fail("rsm_init has not been called");
  if (g_live.running) return rsm::fail("rsm_sq_consumer_start: a consumer is already running");
  if (!g_live.stream)
    CONSUME_HIP(hipStreamCreateWithFlags(&g_live.stream, hipStreamNonBlocking));
  if (!g_live.control)
    CONSUME_HIP(hipHostMalloc(reinterpret_cast<void **>(&g_live.control), sizeof(detail::LiveControl),
                              hipHostMallocDefault));
  // Everything launched so far has finished before the rings change hands.
  if (!rsm::device_idle("rsm_sq_consumer_start")) return -1;
  g_live.mode_before = rt->device_state().sq_queue_mode;
  g_live.pace_copy_before = rt->device_state().pace_copy_bytes_per_tick;
  g_live.pace_reduce_before = rt->device_state().pace_reduce_bytes_per_tick;
  if (!rt->set_sq_mode(detail::kSqLive))
    return rsm::fail("rsm_sq_consumer_start: could not update the device state");
  if (!rt->set_pacing(0, 0)) {
    // live rings without a consumer would block their producers: back to the mode before
    (void)rt->set_sq_mode(g_live.mode_before);
    (void)rt->set_pacing(g_live.pace_copy_before, g_live.pace_reduce_before);
    return rsm::fail("rsm_sq_consumer_start: could not update the device state");
  }
  *g_live.control = detail::LiveControl{};
  detail::ConsumeTotals *totals = static_cast<detail::ConsumeTotals *>(rt->result_scratch());
  static_assert(sizeof(detail::ConsumeTotals) + sizeof(detail::LiveRelay) <= 256, "result scratch");
  detail::LiveRelay *relay = reinterpret_cast<detail::LiveRelay *>(totals + 1);
  hipLaunchKernelGGL(clear_words_kernel, dim3(1), dim3(64), 0, g_live.stream,
                     reinterpret_cast<uint32_t *>(totals),
                     static_cast<int>((sizeof(detail::ConsumeTotals) + sizeof(detail::LiveRelay)) / 4));
  const unsigned rings = static_cast<unsigned>(rt->num_pes()) * rt->options().num_blocks;
  const unsigned waves = rings < kLiveMaxWaves ? rings : kLiveMaxWaves;
  const uint64_t idle_ticks = static_cast<uint64_t>(rt->options().consumer_idle_s * 100e6);
  hipLaunchKernelGGL(consume_live_kernel, dim3(waves), dim3(64), 0, g_live.stream, totals,
                     g_live.control, relay, idle_ticks);
  hipError_t launched = hipGetLastError();
  if (launched != hipSuccess) {
    (void)rt->set_sq_mode(g_live.mode_before);
    (void)rt->set_pacing(g_live.pace_copy_before, g_live.pace_reduce_before);
    return rsm::fail(std::string("rsm_sq_consumer_start: ") + hipGetErrorString(launched));
  }
  g_live.running = true;
  rt->persistent_kernel_started(&rsm::consumer_stop_for_teardown);
  // Producers are launched only when every consumer wave is resident: a grid
  // that filled the device first would wait for a consumer that cannot start.
  const auto t0 = std::chrono::steady_clock::now();
  while (__atomic_load_n(&g_live.control->running, __ATOMIC_ACQUIRE) == 0) {
    if (std::chrono::duration<double>(std::chrono::steady_clock::now() - t0).count() > 5.0) {
      rsm_consume_totals_t ignored;
      (void)rsm_sq_consumer_stop(&ignored);
      return rsm::fail("rsm_sq_consumer_start: the consumer kernel did not become resident within 5 s");
    }
  }
  return 0;
}

int rsm_sq_consumer_stop(rsm_consume_totals_t *totals) {
  RSM_ENTRY;
  Runtime *rt = Runtime::get();
  if (!rt) return rsm::fail("rsm_init has not been called");
  if (!g_live.running) return rsm::fail("rsm_sq_consumer_stop: no consumer is running");
  // Producers on the null stream have finished; callers synchronise their own streams first.
  CONSUME_HIP(hipStreamSynchronize(nullptr));
  __atomic_store_n(&g_live.control->stop, 1u, __ATOMIC_RELEASE);
  hipError_t waited = hipStreamSynchronize(g_live.stream);
  g_live.running = false;
  rt->persistent_kernel_stopped();
  const bool expired = __atomic_load_n(&g_live.control->expired, __ATOMIC_ACQUIRE) != 0;
  const bool mode_ok = rt->set_sq_mode(g_live.mode_before) &&
                       rt->set_pacing(g_live.pace_copy_before, g_live.pace_reduce_before);
  if (waited != hipSuccess)
    return rsm::fail(std::string("rsm_sq_consumer_stop: ") + hipGetErrorString(waited));
  rsm_consume_totals_t host = {};
  CONSUME_HIP(hipMemcpy(&host, rt->result_scratch(), sizeof(host), hipMemcpyDeviceToHost));
  if (totals) *totals = host;
  if (!mode_ok) return rsm::fail("rsm_sq_consumer_stop: could not restore the queue mode");
  if (expired)
    return rsm::fail("rsm_sq_consumer_stop: consumer waves had left before the stop request (nothing "
                     "was published for ROC_SHMEM_CONSUMER_IDLE_S seconds); the totals are what they retired");
  return 0;
}

int rsm_sq_consumer_running(void) {
  RSM_ENTRY;
  return g_live.running ? 1 : 0;
}

int rsm_cq_reader_state(int pe, int block, uint32_t *cq_consumer, uint32_t *quiet_counter,
                        uint32_t *cq_doorbell_record) {
  RSM_ENTRY;
  Runtime *rt = Runtime::get();
  if (!rt) return rsm::fail("rsm_init has not been called");
  if (!ring_args_ok(rt, pe, block)) return rsm::fail("rsm_cq_reader_state: arguments out of range");
  if (!rsm::device_idle("rsm_cq_reader_state")) return -1;
  detail::SqCounters c;
  const detail::DeviceCtx &ctx = rt->ctx_image(pe, block);
  CONSUME_HIP(hipMemcpy(&c, ctx.counters, sizeof(c), hipMemcpyDeviceToHost));
  uint64_t record = 0;
  CONSUME_HIP(hipMemcpy(&record, ctx.ring.mailbox + 2, 8, hipMemcpyDeviceToHost));
  if (cq_consumer) *cq_consumer = c.cq_consumer;
  if (quiet_counter) *quiet_counter = c.quiet_counter;
  if (cq_doorbell_record) *cq_doorbell_record = __builtin_bswap32(static_cast<uint32_t>(record));
  return 0;
}

int rsm_sq_set_mode(int queue_mode) {
  RSM_ENTRY;
  Runtime *rt = Runtime::get();
  if (!rt) return rsm::fail("rsm_init has not been called");
  if (g_live.running) return rsm::fail("rsm_sq_set_mode: a live consumer is running");
  if (!rt->set_sq_queue_mode(queue_mode != 0))
    return rsm::fail("rsm_sq_set_mode: could not update the device state");
  return 0;
}

int rsm_sq_consumer_state(int pe, int block, uint32_t *consumed, uint32_t *cq_producer) {
  RSM_ENTRY;
  Runtime *rt = Runtime::get();
  if (!rt) return rsm::fail("rsm_init has not been called");
  if (!ring_args_ok(rt, pe, block)) return rsm::fail("rsm_sq_consumer_state: arguments out of range");
  if (!rsm::device_idle("rsm_sq_consumer_state")) return -1;
  detail::SqCounters c;
  CONSUME_HIP(hipMemcpy(&c, rt->ctx_image(pe, block).counters, sizeof(c), hipMemcpyDeviceToHost));
  if (consumed) *consumed = c.consumed;
  if (cq_producer) *cq_producer = c.cq_producer;
  return 0;
}

int rsm_cq_image(int pe, int block, void *host_out, size_t bytes) {
  RSM_ENTRY;
  Runtime *rt = Runtime::get();
  if (!rt) return rsm::fail("rsm_init has not been called");
  if (!ring_args_ok(rt, pe, block) || bytes > 64ull * rt->options().sq_size)
    return rsm::fail("rsm_cq_image: arguments out of range");
  if (!rsm::device_idle("rsm_cq_image")) return -1;
  CONSUME_HIP(hipMemcpy(host_out, rt->ctx_image(pe, block).ring.cq, bytes, hipMemcpyDeviceToHost));
  return 0;
}

int rsm_atomic_ret_image(int pe, int block, void *host_out, size_t bytes) {
  RSM_ENTRY;
  Runtime *rt = Runtime::get();
  if (!rt) return rsm::fail("rsm_init has not been called");
  if (!ring_args_ok(rt, pe, block) || bytes > 8ull * detail::kAtomicRetSlots)
    return rsm::fail("rsm_atomic_ret_image: arguments out of range");
  if (!rsm::device_idle("rsm_atomic_ret_image")) return -1;
  CONSUME_HIP(hipMemcpy(host_out,
                        reinterpret_cast<const void *>(rt->ctx_image(pe, block).ring.atomic_ret_base),
                        bytes, hipMemcpyDeviceToHost));
  return 0;
}

int rsm_arena(void **base, size_t *bytes, size_t *slice_stride) {
  RSM_ENTRY;
  Runtime *rt = Runtime::get();
  if (!rt) return rsm::fail("rsm_init has not been called");
  if (base) *base = rt->arena();
  if (bytes) *bytes = rt->arena_bytes();
  if (slice_stride) *slice_stride = rt->slice_stride();
  return 0;
}

}  // extern "C"
