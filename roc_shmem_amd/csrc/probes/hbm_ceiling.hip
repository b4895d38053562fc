// Streaming ceilings of the card, measured with plain kernels that know nothing
// of the library: read only, write only, copy, and the reduction's traffic
// shape (P sources -> P destinations) without any synchronisation.  The
// benchmark prints them next to the library's figures, so that "fraction of
// the 8 TB/s pin rate" can be read against what a bare kernel reaches.
//
// Every kernel moves 16 bytes per lane per access, 8 accesses per lane per
// pass (128 KiB per pass for 1024 lanes), through raw buffer descriptors, and
// deals the passes round-robin to the workgroups, so that the workgroups
// running at one moment sweep one compact window of every array.
//
// Output: one JSON object on stdout; GB/s counts every byte read plus every
// byte written.
#include <hip/hip_runtime.h>
#include <stdint.h>
#include <stdio.h>

#include <algorithm>
#include <vector>

typedef uint32_t u32x4 __attribute__((ext_vector_type(4)));
typedef float f32x4 __attribute__((ext_vector_type(4)));
constexpr int kUnroll = 8;
constexpr int kFlags = 0x00020000;  // untyped 32-bit buffer data
constexpr int kNt = 2;              // non-temporal

#define CHECK(expr)                                                               \
  do {                                                                            \
    hipError_t e_ = (expr);                                                       \
    if (e_ != hipSuccess) {                                                       \
      fprintf(stderr, "%s: %s\n", #expr, hipGetErrorString(e_));                  \
      return 1;                                                                   \
    }                                                                             \
  } while (0)

__global__ void __launch_bounds__(1024) read_kernel(const char *src, size_t bytes, u32x4 *sink) {
  const uint32_t access = blockDim.x * 16u, pass = access * kUnroll;
  u32x4 acc = {0, 0, 0, 0};
  for (size_t b = (size_t)blockIdx.x * pass; b < bytes; b += (size_t)gridDim.x * pass) {
    const size_t left = bytes - b;
    __amdgpu_buffer_rsrc_t rs = __builtin_amdgcn_make_buffer_rsrc(
        const_cast<char *>(src) + b, 0, (int)(left < pass ? left : pass), kFlags);
#pragma unroll
    for (int u = 0; u < kUnroll; ++u)
      acc ^= __builtin_amdgcn_raw_buffer_load_b128(rs, threadIdx.x * 16u, u * access, kNt);
  }
  if (acc.x == 0x12345678u && acc.y == 0x9abcdef0u) sink[0] = acc;  // keeps the loads alive
}

__global__ void __launch_bounds__(1024) write_kernel(char *dst, size_t bytes) {
  const uint32_t access = blockDim.x * 16u, pass = access * kUnroll;
  const u32x4 v = {1, 2, 3, threadIdx.x};
  for (size_t b = (size_t)blockIdx.x * pass; b < bytes; b += (size_t)gridDim.x * pass) {
    const size_t left = bytes - b;
    __amdgpu_buffer_rsrc_t rd =
        __builtin_amdgcn_make_buffer_rsrc(dst + b, 0, (int)(left < pass ? left : pass), kFlags);
#pragma unroll
    for (int u = 0; u < kUnroll; ++u)
      __builtin_amdgcn_raw_buffer_store_b128(v, rd, threadIdx.x * 16u, u * access, kNt);
  }
}

// Slice k is copied into slice (k+1) % slices; blockIdx.x % slices picks the slice.
__global__ void __launch_bounds__(1024)
    copy_kernel(char *arena, size_t stride, size_t src_off, size_t dst_off, size_t bytes, int slices) {
  const uint32_t access = blockDim.x * 16u, pass = access * kUnroll;
  const int k = blockIdx.x % slices, j = blockIdx.x / slices, per_slice = gridDim.x / slices;
  const char *s = arena + k * stride + src_off;
  char *d = arena + ((k + 1) % slices) * stride + dst_off;
  for (size_t b = (size_t)j * pass; b < bytes; b += (size_t)per_slice * pass) {
    const size_t left = bytes - b;
    const int valid = (int)(left < pass ? left : pass);
    __amdgpu_buffer_rsrc_t rs = __builtin_amdgcn_make_buffer_rsrc(const_cast<char *>(s) + b, 0, valid, kFlags);
    __amdgpu_buffer_rsrc_t rd = __builtin_amdgcn_make_buffer_rsrc(d + b, 0, valid, kFlags);
    u32x4 v[kUnroll];
#pragma unroll
    for (int u = 0; u < kUnroll; ++u)
      v[u] = __builtin_amdgcn_raw_buffer_load_b128(rs, threadIdx.x * 16u, u * access, kNt);
#pragma unroll
    for (int u = 0; u < kUnroll; ++u)
      __builtin_amdgcn_raw_buffer_store_b128(v[u], rd, threadIdx.x * 16u, u * access, kNt);
  }
}

// fp32 sum of `slices` sources into `slices` destinations; every pass is
// reduced by one workgroup for everybody.
__global__ void __launch_bounds__(1024)
    reduce_kernel(char *arena, size_t stride, size_t src_off, size_t dst_off, size_t bytes, int slices) {
  const uint32_t access = blockDim.x * 16u, pass = access * kUnroll;
  for (size_t b = (size_t)blockIdx.x * pass; b < bytes; b += (size_t)gridDim.x * pass) {
    const size_t left = bytes - b;
    const int valid = (int)(left < pass ? left : pass);
    f32x4 acc[kUnroll];
#pragma unroll
    for (int u = 0; u < kUnroll; ++u) acc[u] = f32x4{0, 0, 0, 0};
    for (int m = 0; m < slices; ++m) {
      __amdgpu_buffer_rsrc_t rs =
          __builtin_amdgcn_make_buffer_rsrc(arena + m * stride + src_off + b, 0, valid, kFlags);
      f32x4 v[kUnroll];
#pragma unroll
      for (int u = 0; u < kUnroll; ++u)
        v[u] = __builtin_bit_cast(
            f32x4, __builtin_amdgcn_raw_buffer_load_b128(rs, threadIdx.x * 16u, u * access, kNt));
#pragma unroll
      for (int u = 0; u < kUnroll; ++u) acc[u] += v[u];
    }
    for (int m = 0; m < slices; ++m) {
      __amdgpu_buffer_rsrc_t rd =
          __builtin_amdgcn_make_buffer_rsrc(arena + m * stride + dst_off + b, 0, valid, kFlags);
#pragma unroll
      for (int u = 0; u < kUnroll; ++u)
        __builtin_amdgcn_raw_buffer_store_b128(__builtin_bit_cast(u32x4, acc[u]), rd,
                                               threadIdx.x * 16u, u * access, kNt);
    }
  }
}

template <typename F>
static float ms_per_launch(F launch, int iters) {
  hipEvent_t a, b;
  (void)hipEventCreate(&a);
  (void)hipEventCreate(&b);
  for (int i = 0; i < 3; ++i) launch();
  (void)hipDeviceSynchronize();
  (void)hipEventRecord(a, 0);
  for (int i = 0; i < iters; ++i) launch();
  (void)hipEventRecord(b, 0);
  (void)hipEventSynchronize(b);
  float ms = 0;
  (void)hipEventElapsedTime(&ms, a, b);
  (void)hipEventDestroy(a);
  (void)hipEventDestroy(b);
  return ms / iters;
}

int main() {
  const int slices = 8, iters = 10;
  const size_t stride = 1ull << 30, half = 256ull << 20;  // per slice: 256 MiB source, 256 MiB destination
  char *arena = nullptr;
  CHECK(hipMalloc(reinterpret_cast<void **>(&arena), stride * slices));
  CHECK(hipMemset(arena, 0, stride * slices));
  const size_t flat = 4ull << 30;  // read-only / write-only sweep the first 4 GiB
  struct Best { double gbps = 0; int grid = 0, block = 0; };
  Best rd, wr, cp, red;
  for (int block : {512, 1024}) {
    for (int grid : {256, 512, 1024, 2048}) {
      auto take = [&](Best &best, double bytes, float ms) {
        double g = bytes / ms / 1e6;
        if (g > best.gbps) best = Best{g, grid, block};
      };
      take(rd, (double)flat, ms_per_launch([&] {
             hipLaunchKernelGGL(read_kernel, dim3(grid), dim3(block), 0, 0, arena, flat,
                                reinterpret_cast<u32x4 *>(arena + flat));
           }, iters));
      take(wr, (double)flat, ms_per_launch([&] {
             hipLaunchKernelGGL(write_kernel, dim3(grid), dim3(block), 0, 0, arena, flat);
           }, iters));
      take(cp, 2.0 * slices * half, ms_per_launch([&] {
             hipLaunchKernelGGL(copy_kernel, dim3(grid), dim3(block), 0, 0, arena, stride, (size_t)0,
                                half, half, slices);
           }, iters));
      take(red, 2.0 * slices * half, ms_per_launch([&] {
             hipLaunchKernelGGL(reduce_kernel, dim3(grid), dim3(block), 0, 0, arena, stride, (size_t)0,
                                half, half, slices);
           }, iters));
    }
  }
  CHECK(hipGetLastError());
  CHECK(hipDeviceSynchronize());
  auto show = [](const char *name, const Best &b, bool last) {
    printf("\"%s\": {\"GBps\": %.1f, \"grid\": %d, \"block\": %d}%s", name, b.gbps, b.grid, b.block,
           last ? "" : ", ");
  };
  printf("{");
  show("read_only_4GiB", rd, false);
  show("write_only_4GiB", wr, false);
  show("copy_8x256MiB_to_neighbour", cp, false);
  show("reduce_fp32_8_to_8_x256MiB_no_barrier", red, true);
  printf("}\n");
  (void)hipFree(arena);
  return 0;
}
