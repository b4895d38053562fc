// C ABI: plain read-only, write-only and copy streams over a symmetric buffer.
//
// What a card's memory system delivers differs from card to card by several
// per cent, and much more with the shape of the launch: workgroups that stay and
// take one pass after the other (the shape a device-side collective has) reach
// 6.3-6.9 TB/s one way on MI355X, a grid of one small workgroup per pass, handed
// out by the hardware in address order, 7.1-7.6 TB/s; a stream that reads and
// writes as much stays at 6.4-6.7 TB/s whatever hands out its passes.  These
// kernels measure that on the card at hand, so that a rate can be judged against
// the card and not only against the datasheet.  Two more kinds run the HIP
// runtime's own fill and device-to-device copy over the same buffers, for
// comparison.  No counterpart in the reference.
#include "cabi_common.hpp"
#include "roc_shmem.hpp"

using namespace rocshmem;

namespace {

constexpr int kNt = 2;
constexpr int kStore = kNt | detail::kWriteThrough;   // the policy of the collectives' streaming stores

// All workgroups of the grid sweep the PEs' buffers one after the other: pass g of
// the run is pass g % passes_per_pe of PE g / passes_per_pe, and workgroup b takes
// passes b, b + grid, ...  (a grid of as many workgroups as passes gives every
// workgroup one).  At any moment the whole grid is inside one compact window of one
// buffer, which is how the large reductions and broadcasts of this library meet
// memory (every workgroup on the same member at the same time) and what gives
// one-way streams their best rate (8 windows at once, one per PE, measured 2-5 %
// lower).  A pass is U accesses of the workgroup, each of blockDim.x * 16 bytes.

// Where a workgroup stands in that sweep.  The host passes the number of passes per
// PE; the one division a workgroup makes is a 32-bit one, and moving on costs
// additions only (a 64-bit division per pass, some 150 scalar instructions during
// which the workgroup issues no memory access, took a tenth of the write rate of
// workgroups that stay, and two of them a sixth of the rate of a grid of one small
// workgroup per pass).
struct PassWalk {
  uint32_t g, total, per_pe, pe, idx;
  __device__ __forceinline__ PassWalk(uint32_t passes_per_pe)
      : g(blockIdx.x), total(passes_per_pe * static_cast<uint32_t>(detail::g_state.num_pes)),
        per_pe(passes_per_pe), pe(blockIdx.x / passes_per_pe), idx(blockIdx.x - pe * passes_per_pe) {}
  __device__ __forceinline__ bool live() const { return g < total; }
  __device__ __forceinline__ void next() {
    g += gridDim.x;
    if (g >= total) return;
    idx += gridDim.x;
    while (idx >= per_pe) {   // g < total: ends with pe = g / per_pe < num_pes
      idx -= per_pe;
      ++pe;
    }
  }
};

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
// p's slice (so that a test can check the loads).  `buf0` and `checksum0` are PE
// 0's addresses.  Without a checksum the loads are only performed (the folds'
// atomics would dominate a grid of one small workgroup per pass).
template <int U>
__global__ void __launch_bounds__(1024)
    stream_read_kernel(char *buf0, size_t bytes, uint32_t passes_per_pe, uint32_t *checksum0) {
  const uint32_t access = blockDim.x * 16u, pass = access * U;
  detail::u32x4 acc = {0u, 0u, 0u, 0u};
  int acc_pe = -1;
  for (PassWalk w(passes_per_pe); w.live(); w.next()) {
    const int pe = static_cast<int>(w.pe);
    const size_t b = static_cast<size_t>(w.idx) * pass;
    if (pe != acc_pe) {
      if (acc_pe >= 0 && checksum0) fold_into(checksum0, acc_pe, acc);
      acc = detail::u32x4{0u, 0u, 0u, 0u};
      acc_pe = pe;
    }
    const size_t left = bytes - b;
    __amdgpu_buffer_rsrc_t rs =
        detail::uniform_rsrc(slice_of(buf0, pe) + b, static_cast<int>(left < pass ? left : pass));
#pragma unroll
    for (int u = 0; u < U; ++u)
      acc ^= __builtin_amdgcn_raw_buffer_load_b128(rs, threadIdx.x * 16u, u * access, kNt);
  }
  if (acc_pe >= 0 && checksum0) fold_into(checksum0, acc_pe, acc);
  asm volatile("" ::"v"(acc));   // the loads stay even when nothing is folded
}

// Vector i of PE p's buffer becomes {i, i >> 32, p, seed}.
//
// The stores' whole offset goes through the vector register, none through the
// scalar offset.  A 16-byte buffer store reads its data registers for a few
// cycles after it has issued; the compiler keeps a vector instruction that
// overwrites them away for two wait states, but only when the store's scalar
// offset is not a register.  With `u * access` in a scalar register and the next
// vector's index computed into the same registers right behind the store, 32 of
// 131073 vectors came out with their successor's index on gfx950 (the last four
// lanes of a row of sixteen).  Data that comes from loads, or that is not
// rewritten within a few instructions of its store (every other kernel of this
// library), is not exposed to this.
template <int U>
__global__ void __launch_bounds__(1024)
    stream_write_kernel(char *buf0, size_t bytes, uint32_t passes_per_pe, uint32_t seed) {
  const uint32_t access = blockDim.x * 16u, pass = access * U;
  for (PassWalk w(passes_per_pe); w.live(); w.next()) {
    const int pe = static_cast<int>(w.pe);
    const size_t b = static_cast<size_t>(w.idx) * pass;
    const size_t left = bytes - b;
    __amdgpu_buffer_rsrc_t rd =
        detail::uniform_rsrc(slice_of(buf0, pe) + b, static_cast<int>(left < pass ? left : pass));
    // All vectors of the pass first, then the stores back to back: workgroups that stay
    // lose a tenth of their write rate to a few index instructions between the stores.
    detail::u32x4 v[U];
#pragma unroll
    for (int u = 0; u < U; ++u) {
      const uint64_t i = (b + static_cast<uint64_t>(u) * access) / 16u + threadIdx.x;
      v[u] = detail::u32x4{static_cast<uint32_t>(i), static_cast<uint32_t>(i >> 32),
                           static_cast<uint32_t>(pe), seed};
    }
#pragma unroll
    for (int u = 0; u < U; ++u)
      __builtin_amdgcn_raw_buffer_store_b128(v[u], rd, threadIdx.x * 16u + u * access, 0, kStore);
  }
}

// The first `half` bytes of every PE's buffer are copied onto the `half` bytes behind them.
template <int U>
__global__ void __launch_bounds__(1024)
    stream_copy_kernel(char *buf0, size_t half, uint32_t passes_per_pe) {
  const uint32_t access = blockDim.x * 16u, pass = access * U;
  for (PassWalk w(passes_per_pe); w.live(); w.next()) {
    const int pe = static_cast<int>(w.pe);
    const size_t b = static_cast<size_t>(w.idx) * pass;
    const size_t left = half - b;
    const int valid = static_cast<int>(left < pass ? left : pass);
    char *from = slice_of(buf0, pe) + b;
    __amdgpu_buffer_rsrc_t rs = detail::uniform_rsrc(from, valid);
    __amdgpu_buffer_rsrc_t rd = detail::uniform_rsrc(from + half, valid);
    detail::u32x4 v[U];
#pragma unroll
    for (int u = 0; u < U; ++u)
      v[u] = __builtin_amdgcn_raw_buffer_load_b128(rs, threadIdx.x * 16u, u * access, kNt);
#pragma unroll
    for (int u = 0; u < U; ++u)
      __builtin_amdgcn_raw_buffer_store_b128(v[u], rd, threadIdx.x * 16u, u * access, kStore);
  }
}

template <int U>
int launch_stream(int kind, const rsm::Launch &l, char *buf, size_t bytes, uint32_t *checksum, unsigned seed) {
  const size_t span = kind == RSM_STREAM_COPY ? bytes / 2 : bytes;
  const size_t pass = static_cast<size_t>(l.wg_size) * 16u * U;
  const size_t per_pe = (span + pass - 1) / pass;
  // the kernels count passes in 32 bits
  if (per_pe * static_cast<size_t>(host::Runtime::get()->num_pes()) >= (size_t{1} << 31))
    return rsm::fail("stream_probe: too many passes (2^31 or more); use larger passes");
  const uint32_t n = static_cast<uint32_t>(per_pe);
  if (kind == RSM_STREAM_READ)
    hipLaunchKernelGGL(stream_read_kernel<U>, dim3(l.grid), dim3(l.wg_size), 0, l.stream, buf, bytes, n, checksum);
  else if (kind == RSM_STREAM_WRITE)
    hipLaunchKernelGGL(stream_write_kernel<U>, dim3(l.grid), dim3(l.wg_size), 0, l.stream, buf, bytes, n, seed);
  else
    hipLaunchKernelGGL(stream_copy_kernel<U>, dim3(l.grid), dim3(l.wg_size), 0, l.stream, buf, span, n);
  return rsm::after_launch("stream_probe");
}

}  // namespace

extern "C" int rsm_stream_probe(int kind, void *buf, size_t bytes_per_pe, void *checksum,
                                unsigned seed, const rsm_launch_t *launch) {
  RSM_ENTRY;
  rsm::Launch l;
  if (!rsm::resolve_launch(launch, &l)) return -1;
  if (kind < RSM_STREAM_READ || kind > RSM_STREAM_COPY) return rsm::fail("stream_probe: unknown kind");
  if (!rsm::check_symmetric(buf, "buf")) return -1;
  if ((reinterpret_cast<uintptr_t>(buf) | bytes_per_pe) & 15u)
    return rsm::fail("stream_probe: buffer and size must be multiples of 16 bytes");
  const bool halves = kind == RSM_STREAM_RUNTIME_COPY || kind == RSM_STREAM_COPY;
  if (halves && (bytes_per_pe & 31u))
    return rsm::fail("stream_probe: a copy needs a multiple of 32 bytes (two halves)");
  if (!rsm::check_extent(buf, bytes_per_pe, "stream_probe: buf")) return -1;
  if (bytes_per_pe == 0) return 0;
  if (kind == RSM_STREAM_RUNTIME_FILL || kind == RSM_STREAM_RUNTIME_COPY) {
    // The HIP runtime's own fill and device-to-device copy, one call per PE on the
    // launch's stream: what the vendor's kernels reach on the same buffers.
    host::Runtime *rt = host::Runtime::get();
    for (int pe = 0; pe < rt->num_pes(); ++pe) {
      char *at = static_cast<char *>(buf) + static_cast<size_t>(pe) * rt->slice_stride();
      const hipError_t e =
          kind == RSM_STREAM_RUNTIME_FILL
              ? hipMemsetAsync(at, static_cast<int>(seed & 0xffu), bytes_per_pe, l.stream)
              : hipMemcpyAsync(at + bytes_per_pe / 2, at, bytes_per_pe / 2, hipMemcpyDeviceToDevice, l.stream);
      if (e != hipSuccess) return rsm::fail(std::string("stream_probe: runtime call failed: ") + hipGetErrorString(e));
    }
    return 0;
  }
  if (kind == RSM_STREAM_READ && checksum &&
      (!rsm::check_symmetric(checksum, "checksum") || !rsm::check_extent(checksum, 16, "stream_probe: checksum")))
    return -1;
  // launch->tile: bytes of one workgroup pass, wg_size * 16 * {1, 2, 4, 8}; 0 = 8 accesses.
  const size_t access = static_cast<size_t>(l.wg_size) * 16u;
  const size_t tile = l.tile ? l.tile : access * 8u;
  char *b = static_cast<char *>(buf);
  uint32_t *c = static_cast<uint32_t *>(checksum);
  if (tile == access) return launch_stream<1>(kind, l, b, bytes_per_pe, c, seed);
  if (tile == access * 2u) return launch_stream<2>(kind, l, b, bytes_per_pe, c, seed);
  if (tile == access * 4u) return launch_stream<4>(kind, l, b, bytes_per_pe, c, seed);
  if (tile == access * 8u) return launch_stream<8>(kind, l, b, bytes_per_pe, c, seed);
  return rsm::fail("stream_probe: launch->tile must be wg_size * 16 * {1, 2, 4, 8} bytes, or 0");
}
