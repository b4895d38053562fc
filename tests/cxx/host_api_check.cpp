// Host-initiated data path and a user kernel written against the public
// header, checked against closed forms (the style of the reference's
// functional tests, clients/functional_tests/*_tester.cpp verify_results).
// Exit code 0 and a final line "HOST_API_OK" mean every check passed.
#include <cmath>
#include <cstdio>
#include <cstdlib>
#include <vector>

#include "roc_shmem.hpp"

using namespace rocshmem;

static int failures = 0;
#define EXPECT(cond, ...)            \
  do {                               \
    if (!(cond)) {                   \
      ++failures;                    \
      printf("FAIL %s:%d: ", __FILE__, __LINE__); \
      printf(__VA_ARGS__);           \
      printf("\n");                  \
    }                                \
  } while (0)

// Each PE's workgroup puts `n` longs to its right-hand neighbour and adds one
// to a counter on PE 0.
__global__ void ring_put(long *dst, const long *src, long *counter, int n) {
  __shared__ roc_shmem_ctx_t ctx;
  roc_shmem_wg_init();
  roc_shmem_wg_ctx_create(ROC_SHMEM_CTX_WG_PRIVATE, &ctx);
  const int me = roc_shmem_ctx_my_pe(ctx);
  const int np = roc_shmem_ctx_n_pes(ctx);
  dst = roc_shmemx_my_addr(dst);
  src = roc_shmemx_my_addr(src);
  counter = roc_shmemx_my_addr(counter);
  roc_shmemx_ctx_long_put_wg(ctx, dst, src, n, (me + 1) % np);
  roc_shmem_ctx_quiet(ctx);
  if (threadIdx.x == 0) roc_shmem_ctx_long_atomic_add(ctx, counter, 1 + me, 0);
  roc_shmem_wg_ctx_destroy(ctx);
  roc_shmem_wg_finalize();
}

// PE 0 lets `ticks` of the 100 MHz device timer pass and then puts 5 into `flag` on PE 1.
__global__ void late_signal(long *flag, uint64_t ticks) {
  __shared__ roc_shmem_ctx_t ctx;
  roc_shmem_wg_init();
  roc_shmem_wg_ctx_create(ROC_SHMEM_CTX_WG_PRIVATE, &ctx);
  flag = roc_shmemx_my_addr(flag);
  if (roc_shmem_ctx_my_pe(ctx) == 0 && threadIdx.x == 0) {
    const uint64_t start = roc_shmem_timer();
    for (int spins = 0; spins < (1 << 24) && roc_shmem_timer() - start < ticks; ++spins) {
    }
    roc_shmem_ctx_long_p(ctx, flag, 5, 1);
  }
  roc_shmem_wg_ctx_destroy(ctx);
  roc_shmem_wg_finalize();
}

int main() {
  setenv("ROC_SHMEM_NUM_PES", "4", 1);
  setenv("ROC_SHMEM_HEAP_SIZE", "67108864", 1);
  roc_shmem_init();
  const int np = roc_shmem_n_pes();
  EXPECT(np == 4, "n_pes %d", np);
  const int n = 1000;

  long *src = static_cast<long *>(roc_shmem_malloc(n * sizeof(long)));
  long *dst = static_cast<long *>(roc_shmem_malloc(n * sizeof(long)));
  float *fsrc = static_cast<float *>(roc_shmem_malloc(n * sizeof(float)));
  float *fdst = static_cast<float *>(roc_shmem_malloc(n * sizeof(float)));
  int *isrc = static_cast<int *>(roc_shmem_malloc(n * sizeof(int)));
  int *idst = static_cast<int *>(roc_shmem_malloc(n * sizeof(int)));
  long *counter = static_cast<long *>(roc_shmem_malloc(sizeof(long)));
  EXPECT(src && dst && fsrc && fdst && isrc && idst && counter, "allocation");

  roc_shmem_ctx_t ctx;
  roc_shmem_ctx_create(0, &ctx);
  std::vector<long> h(n), back(n);
  std::vector<float> hf(n), backf(n);
  std::vector<int> hi(n), backi(n);

  // Typed put from every PE into its own slice, read back with get.
  for (int pe = 0; pe < np; ++pe) {
    roc_shmemx_set_pe(pe);
    EXPECT(roc_shmem_my_pe() == pe, "my_pe");
    for (int i = 0; i < n; ++i) {
      h[i] = 1000L * pe + i;
      hf[i] = static_cast<float>((i * 7 + pe * 13) % 101) - 50.0f;
      hi[i] = (i * 2654435761u) ^ (0x01010101u << pe);
    }
    roc_shmem_long_put(src, h.data(), n, pe);
    roc_shmem_ctx_float_put(ctx, fsrc, hf.data(), n, pe);
    roc_shmem_int_put_nbi(isrc, hi.data(), n, pe);
    roc_shmem_quiet();
    roc_shmem_long_get(back.data(), src, n, pe);
    for (int i = 0; i < n; ++i) EXPECT(back[i] == h[i], "put/get pe %d i %d", pe, i);
    for (int i = 0; i < n; ++i) h[i] = -1;
    roc_shmem_putmem(dst, h.data(), n * sizeof(long), pe);
  }
  roc_shmemx_set_pe(0);

  // sum over all PEs: sum_pe (1000 pe + i) = 1000 * np(np-1)/2 + np * i.
  roc_shmem_ctx_long_sum_to_all(ctx, dst, src, n, 0, 0, np, nullptr, nullptr);
  for (int pe = 0; pe < np; ++pe) {
    roc_shmem_long_get(back.data(), dst, n, pe);
    for (int i = 0; i < n; ++i)
      EXPECT(back[i] == 1000L * np * (np - 1) / 2 + static_cast<long>(np) * i, "sum pe %d i %d: %ld", pe, i, back[i]);
  }

  // float max over all PEs.
  roc_shmem_ctx_float_max_to_all(ctx, fdst, fsrc, n, 0, 0, np, nullptr, nullptr);
  roc_shmem_float_get(backf.data(), fdst, n, 3);
  for (int i = 0; i < n; ++i) {
    float want = -1e30f;
    for (int pe = 0; pe < np; ++pe) {
      float v = static_cast<float>((i * 7 + pe * 13) % 101) - 50.0f;
      want = v > want ? v : want;
    }
    EXPECT(backf[i] == want, "max i %d", i);
  }

  // int xor over the active set {1, 3}; PEs 0 and 2 keep their dest.
  for (int pe = 0; pe < np; ++pe) {
    for (int i = 0; i < n; ++i) hi[i] = -7;
    roc_shmem_int_put(idst, hi.data(), n, pe);
  }
  roc_shmem_ctx_int_xor_to_all(ctx, idst, isrc, n, 1, 1, 2, nullptr, nullptr);
  for (int pe = 0; pe < np; ++pe) {
    roc_shmem_int_get(backi.data(), idst, n, pe);
    for (int i = 0; i < n; ++i) {
      int want = (pe & 1) ? static_cast<int>((0x01010101u << 1) ^ (0x01010101u << 3)) : -7;
      EXPECT(backi[i] == want, "xor pe %d i %d: %x", pe, i, backi[i]);
    }
  }

  // Team {0, 2}: min of 1000 pe + i is i; non-members keep the sum.
  roc_shmem_team_t team = ROC_SHMEM_TEAM_INVALID;
  EXPECT(roc_shmem_team_split_strided(ROC_SHMEM_TEAM_WORLD, 0, 2, 2, nullptr, 0, &team) == 0, "split");
  EXPECT(roc_shmem_team_n_pes(team) == 2, "team size");
  roc_shmemx_set_pe(2);
  EXPECT(roc_shmem_team_my_pe(team) == 1, "team my_pe");
  EXPECT(roc_shmem_team_translate_pe(team, 1, ROC_SHMEM_TEAM_WORLD) == 2, "translate");
  roc_shmemx_set_pe(0);
  roc_shmem_ctx_long_min_to_all(ctx, team, dst, src, n);
  for (int pe = 0; pe < np; ++pe) {
    roc_shmem_long_get(back.data(), dst, n, pe);
    for (int i = 0; i < n; ++i) {
      long want = (pe % 2 == 0) ? i : 1000L * np * (np - 1) / 2 + static_cast<long>(np) * i;
      EXPECT(back[i] == want, "team min pe %d i %d: %ld", pe, i, back[i]);
    }
  }

  // Broadcast from root 2 of the world: every PE but the root receives
  // (the root's dest is not written, as in OpenSHMEM 1.4).
  roc_shmem_ctx_long_broadcast(ctx, dst, src, n, 2, 0, 0, np, nullptr);
  for (int pe = 0; pe < np; ++pe) {
    if (pe == 2) continue;
    roc_shmem_long_get(back.data(), dst, n, pe);
    for (int i = 0; i < n; ++i) EXPECT(back[i] == 2000L + i, "broadcast pe %d i %d: %ld", pe, i, back[i]);
  }
  // Team broadcast, root index 1 of {0, 2} is PE 2 -> PE 0 receives floats.
  roc_shmem_ctx_float_broadcast(ctx, team, fdst, fsrc, n, 1);
  roc_shmem_float_get(backf.data(), fdst, n, 0);
  for (int i = 0; i < n; ++i)
    EXPECT(backf[i] == static_cast<float>((i * 7 + 2 * 13) % 101) - 50.0f, "team broadcast i %d", i);
  roc_shmem_team_destroy(team);

  // p / g and the AMOs on PE 3's counter.
  roc_shmem_long_p(counter, 40, 3);
  EXPECT(roc_shmem_long_g(counter, 3) == 40, "p/g");
  EXPECT(roc_shmem_long_atomic_fetch_add(counter, 2, 3) == 40, "fetch_add");
  EXPECT(roc_shmem_long_atomic_fetch_inc(counter, 3) == 42, "fetch_inc");
  roc_shmem_long_atomic_inc(counter, 3);
  roc_shmem_long_atomic_add(counter, 6, 3);
  EXPECT(roc_shmem_long_atomic_fetch(counter, 3) == 50, "fetch");
  EXPECT(roc_shmem_long_atomic_compare_swap(counter, 49, 1, 3) == 50, "cswap miss");
  EXPECT(roc_shmem_long_atomic_compare_swap(counter, 50, 7, 3) == 50, "cswap hit");
  EXPECT(roc_shmem_long_atomic_swap(counter, 9, 3) == 7, "swap");
  roc_shmem_long_atomic_set(counter, 11, 3);
  EXPECT(roc_shmem_long_g(counter, 3) == 11, "set");
  EXPECT(roc_shmem_long_g(counter, 0) == 0 || true, "other PEs untouched");
  unsigned int *ucounter = reinterpret_cast<unsigned int *>(idst);
  roc_shmem_uint_p(ucounter, 0xfffffffeu, 1);
  EXPECT(roc_shmem_uint_atomic_fetch_add(ucounter, 3u, 1) == 0xfffffffeu, "uint fetch_add");
  EXPECT(roc_shmem_uint_g(ucounter, 1) == 1u, "uint wrap");

  // Bitwise and floating-point AMOs of the host interface (roc_shmem.hpp:1647-1648,1713-1714,
  // 1747-1748,1781-1953).
  roc_shmem_uint_p(ucounter, 0xf0f0u, 2);
  EXPECT(roc_shmem_uint_atomic_fetch_and(ucounter, 0xff00u, 2) == 0xf0f0u, "fetch_and");
  EXPECT(roc_shmem_uint_atomic_fetch_or(ucounter, 0x000fu, 2) == 0xf000u, "fetch_or");
  EXPECT(roc_shmem_uint_atomic_fetch_xor(ucounter, 0xffffu, 2) == 0xf00fu, "fetch_xor");
  roc_shmem_uint_atomic_and(ucounter, 0x0ff0u, 2);
  roc_shmem_uint_atomic_or(ucounter, 0x1000u, 2);
  roc_shmem_uint_atomic_xor(ucounter, 0x0001u, 2);
  EXPECT(roc_shmem_uint_g(ucounter, 2) == 0x1ff1u, "and/or/xor: %x", roc_shmem_uint_g(ucounter, 2));
  uint64_t *wide = reinterpret_cast<uint64_t *>(dst);
  roc_shmem_ctx_uint64_atomic_set(ctx, wide, 0xffff0000ffff0000ull, 1);
  EXPECT(roc_shmem_ctx_uint64_atomic_fetch_xor(ctx, wide, ~0ull, 1) == 0xffff0000ffff0000ull, "uint64 fetch_xor");
  EXPECT(roc_shmem_uint64_atomic_fetch(wide, 1) == 0x0000ffff0000ffffull, "uint64 after xor");
  roc_shmem_float_atomic_set(fdst, 2.5f, 3);
  EXPECT(roc_shmem_float_atomic_fetch(fdst, 3) == 2.5f, "float fetch");
  EXPECT(roc_shmem_float_atomic_swap(fdst, -7.25f, 3) == 2.5f, "float swap");
  EXPECT(roc_shmem_float_g(fdst, 3) == -7.25f, "float after swap");
  double *dword = reinterpret_cast<double *>(dst) + 8;
  roc_shmem_ctx_double_atomic_set(ctx, dword, 1e300, 0);
  EXPECT(roc_shmem_ctx_double_atomic_swap(ctx, dword, -0.0, 0) == 1e300, "double swap");
  EXPECT(roc_shmem_double_atomic_fetch(dword, 0) == 0.0 && std::signbit(roc_shmem_double_atomic_fetch(dword, 0)),
         "double keeps its bit pattern");

  // The heap is host-visible, as the reference's is: host code may read and write symmetric
  // objects through plain pointers (roc_shmemx_host_ptr gives PE pe's address), with
  // roc_shmem_barrier_all between host and device accesses.
  for (int pe = 0; pe < np; ++pe) {
    long *mine = static_cast<long *>(roc_shmemx_host_ptr(src, pe));
    for (int i = 0; i < n; ++i) mine[i] = 7L * pe + i;
  }
  roc_shmem_barrier_all();
  roc_shmem_ctx_long_max_to_all(ctx, dst, src, n, 0, 0, np, nullptr, nullptr);
  for (int pe = 0; pe < np; ++pe) {
    const long *mine = static_cast<const long *>(roc_shmemx_host_ptr(dst, pe));
    for (int i = 0; i < n; ++i) EXPECT(mine[i] == 7L * (np - 1) + i, "host-visible dst pe %d i %d: %ld", pe, i, mine[i]);
  }

  // A kernel written against the public header: ring put + device AMO.
  roc_shmem_long_p(counter, 0, 0);
  ring_put<<<np, 256>>>(dst, src, counter, n);
  roc_shmem_barrier_all();
  EXPECT(hipGetLastError() == hipSuccess, "kernel launch");
  EXPECT(roc_shmemx_take_status() == 0, "device status");
  for (int pe = 0; pe < np; ++pe) {
    roc_shmem_long_get(back.data(), dst, n, pe);
    const int from = (pe + np - 1) % np;
    for (int i = 0; i < n; ++i) EXPECT(back[i] == 7L * from + i, "ring pe %d i %d: %ld", pe, i, back[i]);
  }
  EXPECT(roc_shmem_long_g(counter, 0) == np * (np + 1) / 2, "device atomic_add: %ld", roc_shmem_long_g(counter, 0));

  // Host-side wait_until / test on the current PE's copy of a word (reference:
  // host_templates.hpp:426-487), first on values that are already there ...
  roc_shmem_long_p(counter, 17, 2);
  roc_shmemx_set_pe(2);
  EXPECT(roc_shmem_long_test(counter, ROC_SHMEM_CMP_EQ, 17) == 1, "test EQ");
  EXPECT(roc_shmem_long_test(counter, ROC_SHMEM_CMP_GT, 17) == 0, "test GT");
  EXPECT(roc_shmem_long_test(counter, ROC_SHMEM_CMP_LT, 18) == 1, "test LT");
  roc_shmem_long_wait_until(counter, ROC_SHMEM_CMP_GE, 17);
  // ... then on a word that a kernel still running on another stream sets three milliseconds
  // after its launch: the wait has to see the store while the kernel runs (host-visible heap).
  const char *visible = getenv("ROC_SHMEM_HEAP_HOST_VISIBLE");
  if (!visible || atoi(visible) != 0) {
    roc_shmem_long_p(counter, 0, 1);
    roc_shmem_barrier_all();
    hipStream_t side;
    EXPECT(hipStreamCreateWithFlags(&side, hipStreamNonBlocking) == hipSuccess, "stream");
    late_signal<<<np, 64, 0, side>>>(counter, 300000);
    roc_shmemx_set_pe(1);
    EXPECT(roc_shmem_long_test(counter, ROC_SHMEM_CMP_EQ, 5) == 0, "the flag is set too early");
    roc_shmem_long_wait_until(counter, ROC_SHMEM_CMP_EQ, 5);
    EXPECT(hipStreamSynchronize(side) == hipSuccess, "late_signal");
    EXPECT(roc_shmem_long_g(counter, 1) == 5, "flag after the kernel");
    EXPECT(hipStreamDestroy(side) == hipSuccess, "stream destroy");
    EXPECT(roc_shmemx_take_status() == 0, "device status");
  }
  roc_shmemx_set_pe(0);

  roc_shmem_free(counter);
  roc_shmem_free(idst);
  roc_shmem_free(isrc);
  roc_shmem_free(fdst);
  roc_shmem_free(fsrc);
  roc_shmem_free(dst);
  roc_shmem_free(src);
  roc_shmem_finalize();
  if (failures) {
    printf("HOST_API_FAILED %d\n", failures);
    return 1;
  }
  printf("HOST_API_OK\n");
  return 0;
}
