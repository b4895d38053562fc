// C ABI: workgroup-, wavefront- and thread-level put/get.  The kernel mirrors
// the reference's ExtendedPrimitiveTest / PrimitiveTest kernels
// (clients/functional_tests/extended_primitives.cpp:33-76,
// primitive_tester.cpp:32-82), with every PE of the job in one grid.
#include "cabi_common.hpp"
#include "roc_shmem.hpp"

using namespace rocshmem;

namespace {

constexpr unsigned kWindowCalls = 64;   // non-blocking calls between two quiets

__global__ void __launch_bounds__(1024)
    rma_kernel(int kind, int granularity, char *dest0, const char *source0, size_t msg_bytes,
               size_t n_msgs, size_t dst_stride, size_t src_stride, int pe_shift) {
  __shared__ roc_shmem_ctx_t ctx;
  roc_shmem_wg_init();
  roc_shmem_wg_ctx_create(ROC_SHMEM_CTX_WG_PRIVATE, &ctx);
  const int me = roc_shmem_ctx_my_pe(ctx);
  const int npes = roc_shmem_ctx_n_pes(ctx);
  const int target = (me + pe_shift) % npes;
  const size_t w = blockIdx.x / npes;
  const size_t nw = gridDim.x / npes;
  char *dest = roc_shmemx_my_addr(dest0);
  const char *source = roc_shmemx_my_addr(source0);

  // The non-blocking kinds follow the reference's message-rate kernel (primitive_mr_tester.cpp:
  // 44-49): windows of 64 calls, a quiet after each window.
  const bool windows = kind == RSM_PUT_NBI || kind == RSM_GET_NBI;
  // (a unit - workgroup, wave or lane - issues `span` message numbers' worth between two quiets;
  // the last window's quiet is the kernel's)
  if (granularity == RSM_WG) {
    const size_t span = windows ? kWindowCalls * nw : n_msgs;
    for (size_t m0 = w; m0 < n_msgs; m0 += span) {
      const size_t m_end = n_msgs - m0 > span ? m0 + span : n_msgs;
      for (size_t m = m0; m < m_end; m += nw) {
        char *d = dest + m * dst_stride;
        const char *s = source + m * src_stride;
        switch (kind) {
          case RSM_PUT: roc_shmemx_ctx_putmem_wg(ctx, d, s, msg_bytes, target); break;
          case RSM_GET: roc_shmemx_ctx_getmem_wg(ctx, d, s, msg_bytes, target); break;
          case RSM_PUT_NBI: roc_shmemx_ctx_putmem_nbi_wg(ctx, d, s, msg_bytes, target); break;
          default: roc_shmemx_ctx_getmem_nbi_wg(ctx, d, s, msg_bytes, target); break;
        }
      }
      if (windows && n_msgs - m0 > span) {     // every lane of the workgroup counts alike
        __syncthreads();
        if (threadIdx.x == 0) roc_shmem_ctx_quiet(ctx);
      }
    }
  } else if (granularity == RSM_WG_SHARED) {
    for (size_t m = 0; m < n_msgs; ++m) {
      char *d = dest + m * dst_stride;
      const char *s = source + m * src_stride;
      if (kind == RSM_PUT || kind == RSM_PUT_NBI) {
        roc_shmemx_ctx_putmem_wg_shard(ctx, d, s, msg_bytes, target, static_cast<int>(w),
                                       static_cast<int>(nw));
      } else {
        roc_shmemx_ctx_getmem_wg_shard(ctx, d, s, msg_bytes, target, static_cast<int>(w),
                                       static_cast<int>(nw));
      }
    }
  } else if (granularity == RSM_WAVE) {
    const size_t waves_per_wg = blockDim.x / 64;
    const size_t wave = w * waves_per_wg + threadIdx.x / 64;
    const size_t n_waves = nw * waves_per_wg;
    const size_t span = windows ? kWindowCalls * n_waves : n_msgs;
    for (size_t m0 = wave; m0 < n_msgs; m0 += span) {
      const size_t m_end = n_msgs - m0 > span ? m0 + span : n_msgs;
      for (size_t m = m0; m < m_end; m += n_waves) {
        char *d = dest + m * dst_stride;
        const char *s = source + m * src_stride;
        switch (kind) {
          case RSM_PUT: roc_shmemx_ctx_putmem_wave(ctx, d, s, msg_bytes, target); break;
          case RSM_GET: roc_shmemx_ctx_getmem_wave(ctx, d, s, msg_bytes, target); break;
          case RSM_PUT_NBI: roc_shmemx_ctx_putmem_nbi_wave(ctx, d, s, msg_bytes, target); break;
          default: roc_shmemx_ctx_getmem_nbi_wave(ctx, d, s, msg_bytes, target); break;
        }
      }
      // (a wave's own window: its first lane's quiet covers what the wave has issued)
      if (windows && n_msgs - m0 > span && threadIdx.x % 64 == 0) roc_shmem_ctx_quiet(ctx);
    }
  } else {
    const size_t thread = w * blockDim.x + threadIdx.x;
    const size_t n_threads = nw * blockDim.x;
    const size_t span = windows ? kWindowCalls * n_threads : n_msgs;
    for (size_t m0 = thread; m0 < n_msgs; m0 += span) {
      const size_t m_end = n_msgs - m0 > span ? m0 + span : n_msgs;
      for (size_t m = m0; m < m_end; m += n_threads) {
        char *d = dest + m * dst_stride;
        const char *s = source + m * src_stride;
        switch (kind) {
          case RSM_PUT: roc_shmem_ctx_putmem(ctx, d, s, msg_bytes, target); break;
          case RSM_GET: roc_shmem_ctx_getmem(ctx, d, s, msg_bytes, target); break;
          case RSM_PUT_NBI: roc_shmem_ctx_putmem_nbi(ctx, d, s, msg_bytes, target); break;
          default: roc_shmem_ctx_getmem_nbi(ctx, d, s, msg_bytes, target); break;
        }
      }
      if (windows && n_msgs - m0 > span) roc_shmem_ctx_quiet(ctx);
    }
  }
  // The reference's tester kernels end with a quiet.  A message that the PE's workgroups share
  // is complete when all of them have returned, which no single workgroup can know: there the
  // end of the kernel is the completion point and a quiet per workgroup would only cost (every
  // quiet writes the XCD's whole L2 back: 6.26 -> 6.43 TB/s for 64 MiB messages without it).
  // The waves meet first (__syncthreads: a workgroup-scope release and acquire around the
  // barrier), so that the one lane's quiet, an agent-scope release after it, covers what every
  // wave of the workgroup has issued - the non-blocking forms return without the waves having met.
  if (granularity != RSM_WG_SHARED) {
    __syncthreads();
    if (threadIdx.x == 0) roc_shmem_ctx_quiet(ctx);
  }
  roc_shmem_wg_ctx_destroy(ctx);
  roc_shmem_wg_finalize();
}

// RSM_WG_SHARED alone, for grids of many short-lived workgroups (one workgroup per share of a few
// KiB is the launch shape of the fastest plain copy): nothing in front of the call but the
// kernel's arguments - no context handle in LDS, no workgroup barrier - so that the first payload
// load is a dozen scalar instructions away from the workgroup's start.
// (A build of the same kernel for eight waves per SIMD, 57 vector registers against 71, was no
// better for workgroups of 128 or 256 lanes: +4 % with 4 KiB shares by 256 lanes, -3 to -5 % with
// 8 KiB shares and with 128-lane workgroups.)
__global__ void __launch_bounds__(1024)
    rma_shared_kernel(int is_put, char *dest, const char *source, size_t msg_bytes, size_t n_msgs,
                      size_t dst_stride, size_t src_stride, int pe_shift) {
  const int npes = roc_shmem_n_pes();
  const int target = (roc_shmem_my_pe() + pe_shift) % npes;
  const int w = static_cast<int>(blockIdx.x / npes);
  const int nw = static_cast<int>(gridDim.x / npes);
  for (size_t m = 0; m < n_msgs; ++m) {
    char *d = dest + m * dst_stride;
    const char *s = source + m * src_stride;
    if (is_put) {
      roc_shmemx_ctx_putmem_wg_shard(ROC_SHMEM_CTX_DEFAULT, d, s, msg_bytes, target, w, nw);
    } else {
      roc_shmemx_ctx_getmem_wg_shard(ROC_SHMEM_CTX_DEFAULT, d, s, msg_bytes, target, w, nw);
    }
  }
}


}  // namespace

extern "C" int rsm_rma(int kind, int granularity, void *dest, const void *source,
                       size_t msg_bytes, size_t n_msgs, size_t dst_stride, size_t src_stride,
                       int pe_shift, const rsm_launch_t *launch) {
  RSM_ENTRY;
  rsm::Launch l;
  if (!rsm::resolve_launch(launch, &l)) return -1;
  if (kind < RSM_PUT || kind > RSM_GET_NBI) return rsm::fail("rma: unknown kind");
  if (granularity < RSM_THREAD || granularity > RSM_WG_SHARED)
    return rsm::fail("rma: unknown granularity");
  if (!dest || !source) return rsm::fail("rma: NULL buffer");
  host::Runtime *rt = host::Runtime::get();
  // The remote side of the transfer must be symmetric.
  const void *remote = (kind == RSM_PUT || kind == RSM_PUT_NBI) ? dest : source;
  if (rt->pe_of(remote) != 0) return rsm::fail("rma: the remote buffer is not a symmetric address of PE 0");
  if (pe_shift < 0) return rsm::fail("rma: pe_shift must be non-negative");
  if (n_msgs == 0) return 0;
  // Both sides of every message must stay inside the heap when they are symmetric.
  if (msg_bytes > (~size_t{0} >> 2) || n_msgs > (~size_t{0} >> 2) / (dst_stride | src_stride | 1))
    return rsm::fail("rma: sizes overflow");
  if (!rsm::check_extent(dest, (n_msgs - 1) * dst_stride + msg_bytes, "rma: dest") ||
      !rsm::check_extent(source, (n_msgs - 1) * src_stride + msg_bytes, "rma: source"))
    return -1;
  if (granularity == RSM_WG_SHARED) {
    hipLaunchKernelGGL(rma_shared_kernel, dim3(l.grid),
                       dim3(l.wg_size), 0, l.stream, (kind == RSM_PUT || kind == RSM_PUT_NBI) ? 1 : 0,
                       static_cast<char *>(dest), static_cast<const char *>(source), msg_bytes, n_msgs,
                       dst_stride, src_stride, pe_shift);
    return rsm::after_launch("rma");
  }
  hipLaunchKernelGGL(rma_kernel, dim3(l.grid), dim3(l.wg_size), 0, l.stream, kind, granularity,
                     static_cast<char *>(dest), static_cast<const char *>(source), msg_bytes,
                     n_msgs, dst_stride, src_stride, pe_shift);
  return rsm::after_launch("rma");
}
