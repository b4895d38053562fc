// C ABI: streams of small puts and atomic memory operations issued through
// the thread-level API by every lane of the grid (the workload of the
// reference's random-access and AMO testers,
// clients/functional_tests/random_access_tester.cpp:97-122,
// amo_standard_tester.cpp:32-74), and the wave-level known-answer drivers.
#include "cabi_common.hpp"
#include "roc_shmem.hpp"

using namespace rocshmem;

namespace {

__global__ void __launch_bounds__(1024)
    small_ops_kernel(const rsm_small_op_t *__restrict__ ops, size_t n_ops,
                     int64_t *__restrict__ fetched, char *heap0) {
  __shared__ roc_shmem_ctx_t ctx;
  roc_shmem_wg_init();
  roc_shmem_wg_ctx_create(ROC_SHMEM_CTX_WG_PRIVATE, &ctx);
  char *heap = roc_shmemx_my_addr(heap0);  // base of the calling PE's slice
  const size_t total = static_cast<size_t>(gridDim.x) * blockDim.x;
  for (size_t i = static_cast<size_t>(blockIdx.x) * blockDim.x + threadIdx.x; i < n_ops;
       i += total) {
    const rsm_small_op_t op = ops[i];
    const int pe = static_cast<int>(op.pe);
    // An operation that names a PE or bytes outside the heap is skipped and reported through
    // the status word; issued, it would fault the device.
    const uint64_t heap_bytes = detail::g_state.heap_size;
    const bool bulk = op.kind == RSM_OP_PUTMEM || op.kind == RSM_OP_GETMEM;
    const uint64_t width = bulk ? static_cast<uint64_t>(op.aux)
                                : (op.kind == RSM_OP_P32 || op.kind == RSM_OP_FADD32 ? 4u : 8u);
    const uint64_t local = bulk ? static_cast<uint64_t>(op.value) : 0u;
    if (op.pe >= static_cast<uint32_t>(detail::g_state.num_pes) || width > heap_bytes ||
        op.offset > heap_bytes - width || local > heap_bytes - width) {
      detail::status_raise(detail::kStatusBadArgument);
      continue;
    }
    char *sym = heap + op.offset;
    int64_t got = 0;
    bool fetches = false;
    switch (op.kind) {
      case RSM_OP_P64:
        roc_shmem_ctx_long_p(ctx, reinterpret_cast<long *>(sym), static_cast<long>(op.value), pe);
        break;
      case RSM_OP_FADD64:
        got = roc_shmem_ctx_int64_atomic_fetch_add(ctx, reinterpret_cast<int64_t *>(sym),
                                                   op.value, pe);
        fetches = true;
        break;
      case RSM_OP_ADD64:
        roc_shmem_ctx_int64_atomic_add(ctx, reinterpret_cast<int64_t *>(sym), op.value, pe);
        break;
      case RSM_OP_FINC64:
        got = roc_shmem_ctx_int64_atomic_fetch_inc(ctx, reinterpret_cast<int64_t *>(sym), pe);
        fetches = true;
        break;
      case RSM_OP_INC64:
        roc_shmem_ctx_int64_atomic_inc(ctx, reinterpret_cast<int64_t *>(sym), pe);
        break;
      case RSM_OP_CSWAP64:
        got = roc_shmem_ctx_int64_atomic_compare_swap(ctx, reinterpret_cast<int64_t *>(sym),
                                                      op.aux, op.value, pe);
        fetches = true;
        break;
      case RSM_OP_FETCH64:
        got = roc_shmem_ctx_int64_atomic_fetch(ctx, reinterpret_cast<int64_t *>(sym), pe);
        fetches = true;
        break;
      case RSM_OP_SET64:
        roc_shmem_ctx_int64_atomic_set(ctx, reinterpret_cast<int64_t *>(sym), op.value, pe);
        break;
      case RSM_OP_SWAP64:
        got = roc_shmem_ctx_int64_atomic_swap(ctx, reinterpret_cast<int64_t *>(sym), op.value, pe);
        fetches = true;
        break;
      case RSM_OP_P32:
        roc_shmem_ctx_int_p(ctx, reinterpret_cast<int *>(sym), static_cast<int>(op.value), pe);
        break;
      case RSM_OP_FADD32:
        got = roc_shmem_ctx_int_atomic_fetch_add(ctx, reinterpret_cast<int *>(sym),
                                                 static_cast<int>(op.value), pe);
        fetches = true;
        break;
      case RSM_OP_PUTMEM:
        roc_shmem_ctx_putmem_nbi(ctx, sym, heap + op.value, static_cast<size_t>(op.aux), pe);
        break;
      case RSM_OP_GETMEM:
        roc_shmem_ctx_getmem_nbi(ctx, heap + op.value, sym, static_cast<size_t>(op.aux), pe);
        break;
      case RSM_OP_FAND64:
        got = static_cast<int64_t>(roc_shmem_ctx_uint64_atomic_fetch_and(
            ctx, reinterpret_cast<uint64_t *>(sym), static_cast<uint64_t>(op.value), pe));
        fetches = true;
        break;
      case RSM_OP_FOR64:
        got = static_cast<int64_t>(roc_shmem_ctx_uint64_atomic_fetch_or(
            ctx, reinterpret_cast<uint64_t *>(sym), static_cast<uint64_t>(op.value), pe));
        fetches = true;
        break;
      case RSM_OP_FXOR64:
        got = static_cast<int64_t>(roc_shmem_ctx_uint64_atomic_fetch_xor(
            ctx, reinterpret_cast<uint64_t *>(sym), static_cast<uint64_t>(op.value), pe));
        fetches = true;
        break;
      default:
        break;
    }
    if (fetches && fetched) fetched[i] = got;
  }
  // One quiet for the workgroup, once all its lanes have issued their operations.
  __syncthreads();
  if (threadIdx.x == 0) roc_shmem_ctx_quiet(ctx);
  roc_shmem_wg_ctx_destroy(ctx);
  roc_shmem_wg_finalize();
}

__global__ void fetch_incr_kernel(uint64_t lane_mask, unsigned long long *counter,
                                  uint64_t *per_thread) {
  const size_t t = static_cast<size_t>(blockIdx.x) * blockDim.x + threadIdx.x;
  const uint32_t lane = threadIdx.x % 64;
  uint64_t got = ~0ull;
  if ((lane_mask >> lane) & 1ull) {
    got = detail::wave_fetch_incr<unsigned long long>(counter);
  }
  per_thread[t] = got;
}

__global__ void coalesce_kernel(uint64_t lane_mask, const int32_t *pe, const uint64_t *src,
                                const uint64_t *dst, const uint64_t *size, uint8_t *must_send,
                                uint64_t *out_size) {
  const uint32_t lane = threadIdx.x;
  if ((lane_mask >> lane) & 1ull) {
    detail::CoalesceResult r = detail::wave_coalesce(pe[lane], src[lane], dst[lane], size[lane]);
    must_send[lane] = r.must_send ? 1 : 0;
    out_size[lane] = r.size;
  }
}

}  // namespace

#define RSM_HIP(expr)                                                              \
  do {                                                                             \
    hipError_t e_ = (expr);                                                        \
    if (e_ != hipSuccess)                                                          \
      return rsm::fail(std::string(#expr " failed: ") + hipGetErrorString(e_));    \
  } while (0)

extern "C" {

int rsm_small_ops(const rsm_small_op_t *ops, size_t n_ops, int64_t *fetched,
                  const rsm_launch_t *launch) {
  RSM_ENTRY;
  rsm::Launch l;
  if (!rsm::resolve_launch(launch, &l)) return -1;
  if (!ops) return rsm::fail("small_ops: ops is NULL");
  if (n_ops == 0) return 0;
  hipLaunchKernelGGL(small_ops_kernel, dim3(l.grid), dim3(l.wg_size), 0, l.stream, ops, n_ops,
                     fetched, host::Runtime::get()->slice_base(0));
  return rsm::after_launch("small_ops");
}

int rsm_kat_fetch_incr(uint64_t lane_mask, int n_wgs, int wg_size, uint64_t *per_thread,
                       uint64_t *counter_out) {
  RSM_ENTRY;
  if (n_wgs < 1 || wg_size < 64 || wg_size > 1024 || wg_size % 64)
    return rsm::fail("kat_fetch_incr: bad grid");
  const size_t n = static_cast<size_t>(n_wgs) * wg_size;
  unsigned long long *counter = nullptr;
  uint64_t *out = nullptr;
  RSM_HIP(hipMalloc(reinterpret_cast<void **>(&counter), 8));
  RSM_HIP(hipMalloc(reinterpret_cast<void **>(&out), n * 8));
  RSM_HIP(hipMemset(counter, 0, 8));
  hipLaunchKernelGGL(fetch_incr_kernel, dim3(n_wgs), dim3(wg_size), 0, nullptr, lane_mask, counter,
                     out);
  int rc = rsm::after_launch("kat_fetch_incr");
  if (rc == 0 && !rsm::device_idle("kat_fetch_incr")) rc = -1;
  if (rc == 0) {
    RSM_HIP(hipMemcpy(per_thread, out, n * 8, hipMemcpyDeviceToHost));
    RSM_HIP(hipMemcpy(counter_out, counter, 8, hipMemcpyDeviceToHost));
  }
  (void)hipFree(counter);
  (void)hipFree(out);
  return rc;
}

int rsm_kat_coalesce(uint64_t lane_mask, const int32_t *pe, const uint64_t *src,
                     const uint64_t *dst, const uint64_t *size, uint8_t *must_send,
                     uint64_t *out_size) {
  RSM_ENTRY;
  char *buf = nullptr;
  const size_t bytes = 64 * (4 + 8 + 8 + 8 + 1 + 8) + 64;
  RSM_HIP(hipMalloc(reinterpret_cast<void **>(&buf), bytes));
  RSM_HIP(hipMemset(buf, 0, bytes));
  uint64_t *d_src = reinterpret_cast<uint64_t *>(buf);
  uint64_t *d_dst = d_src + 64;
  uint64_t *d_size = d_dst + 64;
  uint64_t *d_out = d_size + 64;
  int32_t *d_pe = reinterpret_cast<int32_t *>(d_out + 64);
  uint8_t *d_send = reinterpret_cast<uint8_t *>(d_pe + 64);
  RSM_HIP(hipMemcpy(d_src, src, 64 * 8, hipMemcpyHostToDevice));
  RSM_HIP(hipMemcpy(d_dst, dst, 64 * 8, hipMemcpyHostToDevice));
  RSM_HIP(hipMemcpy(d_size, size, 64 * 8, hipMemcpyHostToDevice));
  RSM_HIP(hipMemcpy(d_pe, pe, 64 * 4, hipMemcpyHostToDevice));
  hipLaunchKernelGGL(coalesce_kernel, dim3(1), dim3(64), 0, nullptr, lane_mask, d_pe, d_src, d_dst,
                     d_size, d_send, d_out);
  int rc = rsm::after_launch("kat_coalesce");
  if (rc == 0 && !rsm::device_idle("kat_coalesce")) rc = -1;
  if (rc == 0) {
    RSM_HIP(hipMemcpy(must_send, d_send, 64, hipMemcpyDeviceToHost));
    RSM_HIP(hipMemcpy(out_size, d_out, 64 * 8, hipMemcpyDeviceToHost));
  }
  (void)hipFree(buf);
  return rc;
}

}  // extern "C"
