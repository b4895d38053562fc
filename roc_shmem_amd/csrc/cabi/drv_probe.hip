// C ABI: plain read-only and write-only streams over a symmetric buffer.
//
// What a card's memory system delivers differs from card to card by several
// per cent (reads alone 6.8-7.1 TB/s, writes alone 6.3-6.65 TB/s on MI355X), and
// a stream that reads and writes as much cannot beat the harmonic mean of the
// two.  These two kernels measure that on the card at hand, with the access
// pattern the library's own streams use (128 KiB passes dealt round-robin to the
// workgroups, 16 bytes per lane per access, non-temporal), so that a rate can be
// judged against the card and not only against the datasheet.  No counterpart in
// the reference.
#include "cabi_common.hpp"
#include "roc_shmem.hpp"

using namespace rocshmem;

namespace {

constexpr int kProbeUnroll = 8;

// All workgroups of the grid sweep the PEs' buffers one after the other: pass g of
// the run is pass g % passes_per_pe of PE g / passes_per_pe, and workgroup b takes
// passes b, b + grid, ...  At any moment the whole grid is inside one compact
// window of one buffer, which is how the large reductions and broadcasts of this
// library meet memory (every workgroup on the same member at the same time) and
// what gives one-way streams their best rate (8 windows at once, one per PE,
// measured 2-5 % lower).

__device__ __forceinline__ char *slice_of(char *at_pe0, int pe) {
  return at_pe0 + static_cast<uint64_t>(pe) * detail::g_state.slice_stride;
}

__device__ __forceinline__ void fold_into(uint32_t *checksum_pe0, int pe, detail::u32x4 acc) {
  uint32_t *checksum = reinterpret_cast<uint32_t *>(slice_of(reinterpret_cast<char *>(checksum_pe0), pe));
#pragma unroll
  for (int e = 0; e < 4; ++e) {
    uint32_t v = acc[e];
    for (int d = 32; d >= 1; d >>= 1) v ^= __shfl_xor(v, d, 64);
    if ((threadIdx.x & 63u) == 0 && v != 0)
      __hip_atomic_fetch_xor(checksum + e, v, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
  }
}

// Folds every 16-byte vector of PE p's buffer with XOR into checksum[0..3] of PE
// p's slice (so the loads cannot be dropped, and a test can check them).
// `buf0` and `checksum0` are PE 0's addresses.
__global__ void __launch_bounds__(1024)
    stream_read_kernel(char *buf0, size_t bytes, uint32_t *checksum0) {
  const int npes = detail::g_state.num_pes;
  const uint32_t access = blockDim.x * 16u, pass = access * kProbeUnroll;
  const size_t per_pe = (bytes + pass - 1) / pass;
  detail::u32x4 acc = {0u, 0u, 0u, 0u};
  int acc_pe = -1;
  for (size_t g = blockIdx.x; g < per_pe * npes; g += gridDim.x) {
    const int pe = static_cast<int>(g / per_pe);
    const size_t b = (g % per_pe) * pass;
    if (pe != acc_pe) {
      if (acc_pe >= 0) fold_into(checksum0, acc_pe, acc);
      acc = detail::u32x4{0u, 0u, 0u, 0u};
      acc_pe = pe;
    }
    const size_t left = bytes - b;
    __amdgpu_buffer_rsrc_t rs =
        detail::uniform_rsrc(slice_of(buf0, pe) + b, static_cast<int>(left < pass ? left : pass));
#pragma unroll
    for (int u = 0; u < kProbeUnroll; ++u)
      acc ^= __builtin_amdgcn_raw_buffer_load_b128(rs, threadIdx.x * 16u, u * access, 2 /* nt */);
  }
  if (acc_pe >= 0) fold_into(checksum0, acc_pe, acc);
}

// Vector i of PE p's buffer becomes {i, i >> 32, p, seed}.
__global__ void __launch_bounds__(1024)
    stream_write_kernel(char *buf0, size_t bytes, uint32_t seed) {
  const int npes = detail::g_state.num_pes;
  const uint32_t access = blockDim.x * 16u, pass = access * kProbeUnroll;
  const size_t per_pe = (bytes + pass - 1) / pass;
  for (size_t g = blockIdx.x; g < per_pe * npes; g += gridDim.x) {
    const int pe = static_cast<int>(g / per_pe);
    const size_t b = (g % per_pe) * pass;
    const size_t left = bytes - b;
    __amdgpu_buffer_rsrc_t rd =
        detail::uniform_rsrc(slice_of(buf0, pe) + b, static_cast<int>(left < pass ? left : pass));
#pragma unroll
    for (int u = 0; u < kProbeUnroll; ++u) {
      const uint64_t i = (b + static_cast<uint64_t>(u) * access) / 16u + threadIdx.x;
      const detail::u32x4 v = {static_cast<uint32_t>(i), static_cast<uint32_t>(i >> 32),
                               static_cast<uint32_t>(pe), seed};
      __builtin_amdgcn_raw_buffer_store_b128(v, rd, threadIdx.x * 16u, u * access, 2 /* nt */);
    }
  }
}

}  // namespace

extern "C" int rsm_stream_probe(int kind, void *buf, size_t bytes_per_pe, void *checksum,
                                unsigned seed, const rsm_launch_t *launch) {
  RSM_ENTRY;
  rsm::Launch l;
  if (!rsm::resolve_launch(launch, &l)) return -1;
  if (kind != RSM_STREAM_READ && kind != RSM_STREAM_WRITE) return rsm::fail("stream_probe: unknown kind");
  if (!rsm::check_symmetric(buf, "buf")) return -1;
  if ((reinterpret_cast<uintptr_t>(buf) | bytes_per_pe) & 15u)
    return rsm::fail("stream_probe: buffer and size must be multiples of 16 bytes");
  if (!rsm::check_extent(buf, bytes_per_pe, "stream_probe: buf")) return -1;
  if (bytes_per_pe == 0) return 0;
  if (kind == RSM_STREAM_READ) {
    if (!rsm::check_symmetric(checksum, "checksum") ||
        !rsm::check_extent(checksum, 16, "stream_probe: checksum"))
      return -1;
    hipLaunchKernelGGL(stream_read_kernel, dim3(l.grid), dim3(l.wg_size), 0, l.stream,
                       static_cast<char *>(buf), bytes_per_pe, static_cast<uint32_t *>(checksum));
  } else {
    hipLaunchKernelGGL(stream_write_kernel, dim3(l.grid), dim3(l.wg_size), 0, l.stream,
                       static_cast<char *>(buf), bytes_per_pe, seed);
  }
  return rsm::after_launch("stream_probe");
}
