// C ABI: the consumer pass over the send queues, completion-queue inspection
// and the log/queue switch of the rings.
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

bool ring_args_ok(Runtime *rt, int pe, int block) {
  return pe >= 0 && pe < rt->num_pes() && block >= 0 && block < rt->options().num_blocks;
}

}  // namespace

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
  CONSUME_HIP(hipDeviceSynchronize());
  rsm_consume_totals_t host = {};
  CONSUME_HIP(hipMemcpy(&host, dev, sizeof(host), hipMemcpyDeviceToHost));
  if (totals) *totals = host;
  return 0;
}

int rsm_sq_set_mode(int queue_mode) {
  RSM_ENTRY;
  Runtime *rt = Runtime::get();
  if (!rt) return rsm::fail("rsm_init has not been called");
  if (!rt->set_sq_queue_mode(queue_mode != 0))
    return rsm::fail("rsm_sq_set_mode: could not update the device state");
  return 0;
}

int rsm_sq_consumer_state(int pe, int block, uint32_t *consumed, uint32_t *cq_producer) {
  RSM_ENTRY;
  Runtime *rt = Runtime::get();
  if (!rt) return rsm::fail("rsm_init has not been called");
  if (!ring_args_ok(rt, pe, block)) return rsm::fail("rsm_sq_consumer_state: arguments out of range");
  CONSUME_HIP(hipDeviceSynchronize());
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
  CONSUME_HIP(hipDeviceSynchronize());
  CONSUME_HIP(hipMemcpy(host_out, rt->ctx_image(pe, block).ring.cq, bytes, hipMemcpyDeviceToHost));
  return 0;
}

int rsm_atomic_ret_image(int pe, int block, void *host_out, size_t bytes) {
  RSM_ENTRY;
  Runtime *rt = Runtime::get();
  if (!rt) return rsm::fail("rsm_init has not been called");
  if (!ring_args_ok(rt, pe, block) || bytes > 8ull * detail::kAtomicRetSlots)
    return rsm::fail("rsm_atomic_ret_image: arguments out of range");
  CONSUME_HIP(hipDeviceSynchronize());
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
