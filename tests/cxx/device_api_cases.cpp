// User kernels written the way the reference's functional testers are
// (clients/functional_tests/*_tester.cpp), compiled against the public header
// only, each citing the tester it follows.  Differences forced by "one process
// hosts every PE": the grid carries the workgroups of all PEs
// (blockIdx.x % n_pes is the PE, blockIdx.x / n_pes the workgroup's index within
// it, where the reference uses blockIdx.x), kernel arguments that name
// symmetric objects and are dereferenced by the kernel itself pass through
// roc_shmemx_my_addr (the library's calls find the caller's copy themselves, see
// reference_kernels_unchanged), and "only rank 0 launches" becomes "only PE 0's
// workgroups act".
// Exit code 0 and a final line "DEVICE_API_OK" mean every case passed.
#include <cstdio>
#include <cstdlib>
#include <cstring>
#include <vector>

#include "roc_shmem.hpp"
#include "rocshmem_mi355x.h"

using namespace rocshmem;

static int failures = 0;
static const char *current_case = "";
#define EXPECT(cond, ...)                                               \
  do {                                                                  \
    if (!(cond)) {                                                      \
      if (++failures <= 20) {                                           \
        printf("FAIL [%s] %s:%d: ", current_case, __FILE__, __LINE__);  \
        printf(__VA_ARGS__);                                            \
        printf("\n");                                                   \
      }                                                                 \
    }                                                                   \
  } while (0)

static int npes;

static void finish_kernel(const char *what) {
  roc_shmem_barrier_all();
  hipError_t e = hipGetLastError();
  EXPECT(e == hipSuccess, "%s: %s", what, hipGetErrorString(e));
  EXPECT(roc_shmemx_take_status() == 0, "%s: device status word raised", what);
}

template <typename T>
static std::vector<T> load(const T *sym, int n, int pe) {
  std::vector<T> v(n);
  roc_shmem_getmem(v.data(), sym, n * sizeof(T), pe);
  return v;
}
template <typename T>
static void fill(T *sym, int n, T value, int pe) {
  std::vector<T> v(n, value);
  roc_shmem_putmem(sym, v.data(), n * sizeof(T), pe);
}

__device__ inline int wg_index() { return blockIdx.x / roc_shmem_n_pes(); }

// ---- ping_pong_tester.cpp:32-62 ----------------------------------------------------------
__global__ void PingPongTest(int loop, int skip, uint64_t *timer, int *r_buf) {
  __shared__ roc_shmem_ctx_t ctx;
  roc_shmem_wg_init();
  roc_shmem_wg_ctx_create(ROC_SHMEM_CTX_WG_PRIVATE, &ctx);
  int pe = roc_shmem_ctx_my_pe(ctx);
  r_buf = roc_shmemx_my_addr(r_buf);
  const int w = wg_index();
  if (threadIdx.x == 0 && pe < 2) {
    uint64_t start = 0;
    for (int i = 0; i < loop + skip; i++) {
      if (i == skip) start = roc_shmem_timer();
      if (pe == 0) {
        roc_shmem_ctx_int_p(ctx, &r_buf[w], i + 1, 1);
        roc_shmem_int_wait_until(&r_buf[w], ROC_SHMEM_CMP_EQ, i + 1);
      } else {
        roc_shmem_int_wait_until(&r_buf[w], ROC_SHMEM_CMP_EQ, i + 1);
        roc_shmem_ctx_int_p(ctx, &r_buf[w], i + 1, 0);
      }
    }
    timer[blockIdx.x] = roc_shmem_timer() - start;
  }
  roc_shmem_wg_ctx_destroy(ctx);
  roc_shmem_wg_finalize();
}

static void ping_pong() {
  current_case = "ping_pong_tester.cpp";
  const int wgs = 4, loop = 200, skip = 20;
  int *r_buf = static_cast<int *>(roc_shmem_malloc(sizeof(int) * wgs));
  uint64_t *timer = nullptr;
  (void)hipMalloc(reinterpret_cast<void **>(&timer), sizeof(uint64_t) * wgs * npes);
  (void)hipMemset(timer, 0, sizeof(uint64_t) * wgs * npes);
  for (int pe = 0; pe < npes; ++pe) fill(r_buf, wgs, 0, pe);
  PingPongTest<<<wgs * npes, 64>>>(loop, skip, timer, r_buf);
  finish_kernel("PingPongTest");
  for (int pe = 0; pe < 2; ++pe)
    for (int v : load(r_buf, wgs, pe)) EXPECT(v == loop + skip, "PE %d r_buf = %d", pe, v);
  std::vector<uint64_t> t(wgs * npes);
  (void)hipMemcpy(t.data(), timer, sizeof(uint64_t) * t.size(), hipMemcpyDeviceToHost);
  // ticks of the 100 MHz constant clock; one iteration is a full round trip
  printf("  ping-pong round trip: %.2f us (p + wait_until, 4 pairs at once)\n",
         t[0] / 100.0 / loop);
  (void)hipFree(timer);
  roc_shmem_free(r_buf);
}

// ---- roc_shmem_<T>_wait_until / _test, all six comparisons (context_tmpl_device.hpp:199-246) ----
__global__ void CompareTest(long *word, float *fword, int *results) {
  roc_shmem_wg_init();
  word = roc_shmemx_my_addr(word);
  fword = roc_shmemx_my_addr(fword);
  if (threadIdx.x == 0 && roc_shmem_my_pe() == 0) {
    int k = 0;
    // *word == 5
    results[k++] = roc_shmem_long_test(word, ROC_SHMEM_CMP_EQ, 5);
    results[k++] = roc_shmem_long_test(word, ROC_SHMEM_CMP_EQ, 6);
    results[k++] = roc_shmem_long_test(word, ROC_SHMEM_CMP_NE, 6);
    results[k++] = roc_shmem_long_test(word, ROC_SHMEM_CMP_NE, 5);
    results[k++] = roc_shmem_long_test(word, ROC_SHMEM_CMP_GT, 4);
    results[k++] = roc_shmem_long_test(word, ROC_SHMEM_CMP_GT, 5);
    results[k++] = roc_shmem_long_test(word, ROC_SHMEM_CMP_GE, 5);
    results[k++] = roc_shmem_long_test(word, ROC_SHMEM_CMP_GE, 6);
    results[k++] = roc_shmem_long_test(word, ROC_SHMEM_CMP_LT, 6);
    results[k++] = roc_shmem_long_test(word, ROC_SHMEM_CMP_LT, 5);
    results[k++] = roc_shmem_long_test(word, ROC_SHMEM_CMP_LE, 5);
    results[k++] = roc_shmem_long_test(word, ROC_SHMEM_CMP_LE, 4);
    // satisfied waits return at once
    roc_shmem_long_wait_until(word, ROC_SHMEM_CMP_EQ, 5);
    roc_shmem_long_wait_until(word, ROC_SHMEM_CMP_NE, 0);
    roc_shmem_long_wait_until(word, ROC_SHMEM_CMP_GT, -1);
    roc_shmem_long_wait_until(word, ROC_SHMEM_CMP_GE, 5);
    roc_shmem_long_wait_until(word, ROC_SHMEM_CMP_LT, 100);
    roc_shmem_long_wait_until(word, ROC_SHMEM_CMP_LE, 5);
    // *fword == -1.5f
    results[k++] = roc_shmem_float_test(fword, ROC_SHMEM_CMP_LT, -1.0f);
    results[k++] = roc_shmem_float_test(fword, ROC_SHMEM_CMP_GT, -1.0f);
    roc_shmem_float_wait_until(fword, ROC_SHMEM_CMP_EQ, -1.5f);
    results[k++] = 77;
  }
  roc_shmem_wg_finalize();
}

static void compare_ops() {
  current_case = "wait_until / test comparisons";
  long *word = static_cast<long *>(roc_shmem_malloc(sizeof(long)));
  float *fword = static_cast<float *>(roc_shmem_malloc(sizeof(float)));
  int *results = nullptr;
  (void)hipMalloc(reinterpret_cast<void **>(&results), 32 * sizeof(int));
  (void)hipMemset(results, 0xff, 32 * sizeof(int));
  roc_shmem_long_p(word, 5, 0);
  roc_shmem_float_p(fword, -1.5f, 0);
  CompareTest<<<npes, 64>>>(word, fword, results);
  finish_kernel("CompareTest");
  int got[15];
  (void)hipMemcpy(got, results, sizeof(got), hipMemcpyDeviceToHost);
  const int want[15] = {1, 0, 1, 0, 1, 0, 1, 0, 1, 0, 1, 0, 1, 0, 77};
  for (int i = 0; i < 15; ++i) EXPECT(got[i] == want[i], "result %d = %d, expected %d", i, got[i], want[i]);
  (void)hipFree(results);
  roc_shmem_free(fword);
  roc_shmem_free(word);
}

// ---- the ping-pong of ping_pong_tester.cpp on 1- and 2-byte words (roc_shmem.hpp:1973-2019 declares
// wait_until / test for char, schar, short, uchar and ushort as well): neighbouring workgroups
// use neighbouring bytes, so four flags share one 32-bit word.
#define NARROW_PING_PONG(T, TNAME)                                                        \
  __global__ void PingPong_##TNAME(int loop, T *r_buf, int *bad) {                       \
    __shared__ roc_shmem_ctx_t ctx;                                                       \
    roc_shmem_wg_init();                                                                  \
    roc_shmem_wg_ctx_create(ROC_SHMEM_CTX_WG_PRIVATE, &ctx);                              \
    int pe = roc_shmem_ctx_my_pe(ctx);                                                    \
    r_buf = roc_shmemx_my_addr(r_buf);                                                    \
    const int w = wg_index();                                                             \
    if (threadIdx.x == 0 && pe < 2) {                                                     \
      for (int i = 0; i < loop; i++) {                                                    \
        const T v = static_cast<T>(i + 1);                                                \
        if (pe == 0) {                                                                    \
          roc_shmem_ctx_##TNAME##_p(ctx, &r_buf[w], v, 1);                                \
          roc_shmem_##TNAME##_wait_until(&r_buf[w], ROC_SHMEM_CMP_EQ, v);                 \
        } else {                                                                          \
          for (int spins = 0; spins < (1 << 22); ++spins) /* bounded: never hangs */      \
            if (roc_shmem_##TNAME##_test(&r_buf[w], ROC_SHMEM_CMP_GE, v)) break;          \
          if (r_buf[w] != v) atomicAdd(bad, 1);                                           \
          roc_shmem_ctx_##TNAME##_p(ctx, &r_buf[w], v, 0);                                \
        }                                                                                 \
      }                                                                                   \
    }                                                                                     \
    roc_shmem_wg_ctx_destroy(ctx);                                                        \
    roc_shmem_wg_finalize();                                                              \
  }                                                                                       \
  static void narrow_ping_pong_##TNAME() {                                                \
    const int wgs = 4, loop = 100;                                                        \
    T *r_buf = static_cast<T *>(roc_shmem_malloc(16));                                    \
    int *bad = nullptr;                                                                   \
    (void)hipMalloc(reinterpret_cast<void **>(&bad), sizeof(int));                        \
    (void)hipMemset(bad, 0, sizeof(int));                                                 \
    for (int pe = 0; pe < npes; ++pe) fill(r_buf, static_cast<int>(16 / sizeof(T)), static_cast<T>(0), pe); \
    PingPong_##TNAME<<<wgs * npes, 64>>>(loop, r_buf, bad);                               \
    finish_kernel("PingPong_" #TNAME);                                                    \
    int h = -1;                                                                           \
    (void)hipMemcpy(&h, bad, sizeof(int), hipMemcpyDeviceToHost);                         \
    EXPECT(h == 0, #TNAME ": %d rounds saw a value other than the one sent", h);          \
    for (int pe = 0; pe < 2; ++pe) {                                                      \
      std::vector<T> got = load(r_buf, static_cast<int>(16 / sizeof(T)), pe);             \
      for (int w = 0; w < wgs; ++w)                                                       \
        EXPECT(got[w] == static_cast<T>(loop), #TNAME ": PE %d flag %d ends at %d", pe, w, (int)got[w]); \
      EXPECT(got[wgs] == 0, #TNAME ": the word after the flags was written on PE %d", pe); \
    }                                                                                     \
    (void)hipFree(bad);                                                                   \
    roc_shmem_free(r_buf);                                                                \
  }
NARROW_PING_PONG(short, short)
NARROW_PING_PONG(unsigned char, uchar)
NARROW_PING_PONG(signed char, schar)
NARROW_PING_PONG(unsigned short, ushort)
NARROW_PING_PONG(char, char)
#undef NARROW_PING_PONG

static void narrow_ping_pong() {
  current_case = "wait_until / test on 1- and 2-byte words";
  narrow_ping_pong_short();
  narrow_ping_pong_uchar();
  narrow_ping_pong_schar();
  narrow_ping_pong_ushort();
  narrow_ping_pong_char();
}

// ---- shmem_ptr_tester.cpp:31-44 ------------------------------------------------------------------
__global__ void ShmemPtrTest(char *r_buf, int *available) {
  roc_shmem_wg_init();
  if (threadIdx.x == 0 && roc_shmem_my_pe() == 0) {
    char *local_addr = roc_shmemx_my_addr(r_buf) + 4;
    void *remote_addr = roc_shmem_ptr(local_addr, 1);
    if (remote_addr != NULL) {
      *available = 1;
      static_cast<char *>(remote_addr)[0] = '1';
    }
  }
  roc_shmem_wg_finalize();
}

static void shmem_ptr() {
  current_case = "shmem_ptr_tester.cpp";
  char *r_buf = static_cast<char *>(roc_shmem_malloc(64));
  int *available = nullptr;
  (void)hipMalloc(reinterpret_cast<void **>(&available), sizeof(int));
  (void)hipMemset(available, 0, sizeof(int));
  for (int pe = 0; pe < npes; ++pe) fill(r_buf, 64, '0', pe);
  ShmemPtrTest<<<npes, 64>>>(r_buf, available);
  finish_kernel("ShmemPtrTest");
  int avail = 0;
  (void)hipMemcpy(&avail, available, sizeof(int), hipMemcpyDeviceToHost);
  EXPECT(avail == 1, "every slice is directly addressable here");
  for (int pe = 0; pe < npes; ++pe) {
    std::vector<char> got = load(r_buf, 64, pe);
    for (int i = 0; i < 64; ++i)
      EXPECT(got[i] == ((pe == 1 && i == 4) ? '1' : '0'), "PE %d byte %d = %c", pe, i, got[i]);
  }
  (void)hipFree(available);
  roc_shmem_free(r_buf);
}

// ---- a roc_shmem_ptr result handed on as the local side of a call ------------------------------
// The reference hands back a plain address (context_ib_device.cpp:128-137) that a program may use
// like any other local address.  PE `me` copies from PE me+1's copy of `a` into PE me+2's copy of
// `b` (a put whose source is another PE's memory), fetches PE me+1's `a` into its own `c` through a
// get whose destination is its own roc_shmem_ptr address, and waits on a word of PE me+1 that PE
// me+1 sets itself.  Only pointers that name PE 0's copy from elsewhere cannot be told from the
// symmetric address, so PE 0's copies are named through roc_shmemx_my_addr by PE 0 alone here.
__global__ void ShmemPtrAsArgumentTest(long *a, long *b, long *c, long *flag, int n, int *errors) {
  __shared__ roc_shmem_ctx_t ctx;
  roc_shmem_wg_init();
  roc_shmem_wg_ctx_create(ROC_SHMEM_CTX_WG_PRIVATE, &ctx);
  const int me = roc_shmem_ctx_my_pe(ctx);
  const int np = roc_shmem_ctx_n_pes(ctx);
  const int next = (me + 1) % np, after = (me + 2) % np;
  // a source in PE next's slice (never PE 0's: see above)
  if (next != 0) {
    long *theirs = static_cast<long *>(roc_shmem_ptr(a, next));
    roc_shmemx_ctx_putmem_wg(ctx, b, theirs, n * sizeof(long), after);
  } else {
    roc_shmemx_ctx_putmem_wg(ctx, b, a, n * sizeof(long), after);   // keeps the pattern whole: own a
  }
  // a destination given as the caller's own roc_shmem_ptr address
  long *mine_c = static_cast<long *>(roc_shmem_ptr(c, me));
  roc_shmemx_ctx_getmem_wg(ctx, mine_c, a, n * sizeof(long), next);
  if (threadIdx.x == 0) {
    roc_shmem_ctx_quiet(ctx);
    // every PE raises its own flag; its left neighbour waits on it through a plain address
    roc_shmem_ctx_long_p(ctx, flag, 7 + me, me);
    if (next != 0) {
      long *their_flag = static_cast<long *>(roc_shmem_ptr(flag, next));
      roc_shmem_long_wait_until(their_flag, ROC_SHMEM_CMP_EQ, 7 + next);
      if (roc_shmem_long_test(their_flag, ROC_SHMEM_CMP_NE, 7 + next)) atomicAdd(errors, 1);
    }
  }
  roc_shmem_wg_ctx_destroy(ctx);
  roc_shmem_wg_finalize();
}

static void shmem_ptr_as_argument() {
  current_case = "roc_shmem_ptr results as local arguments";
  const int n = 512;
  long *a = static_cast<long *>(roc_shmem_malloc(n * sizeof(long)));
  long *b = static_cast<long *>(roc_shmem_malloc(n * sizeof(long)));
  long *c = static_cast<long *>(roc_shmem_malloc(n * sizeof(long)));
  long *flag = static_cast<long *>(roc_shmem_malloc(sizeof(long)));
  int *errors = nullptr;
  (void)hipMalloc(reinterpret_cast<void **>(&errors), sizeof(int));
  (void)hipMemset(errors, 0, sizeof(int));
  for (int pe = 0; pe < npes; ++pe) {
    std::vector<long> v(n);
    for (int i = 0; i < n; ++i) v[i] = 1000L * pe + i;
    roc_shmem_putmem(a, v.data(), n * sizeof(long), pe);
    fill(b, n, -1L, pe);
    fill(c, n, -2L, pe);
    fill(flag, 1, 0L, pe);
  }
  ShmemPtrAsArgumentTest<<<npes, 256>>>(a, b, c, flag, n, errors);
  finish_kernel("ShmemPtrAsArgumentTest");
  int bad = 0;
  (void)hipMemcpy(&bad, errors, sizeof(int), hipMemcpyDeviceToHost);
  EXPECT(bad == 0, "test() on another PE's word, named by a plain address, saw a stale value");
  for (int pe = 0; pe < npes; ++pe) {
    // b of PE pe was written by PE pe-2 with the a of PE pe-1 (or with its own a when pe-1 is PE 0)
    const int writer = (pe - 2 + 2 * npes) % npes, from = (writer + 1) % npes;
    const int expect_a_of = from != 0 ? from : writer;
    std::vector<long> got_b = load(b, n, pe), got_c = load(c, n, pe);
    for (int i = 0; i < n; ++i) {
      EXPECT(got_b[i] == 1000L * expect_a_of + i, "b of PE %d [%d] = %ld, expected a of PE %d", pe, i, got_b[i],
             expect_a_of);
      EXPECT(got_c[i] == 1000L * ((pe + 1) % npes) + i, "c of PE %d [%d] = %ld", pe, i, got_c[i]);
    }
  }
  (void)hipFree(errors);
  roc_shmem_free(flag);
  roc_shmem_free(c);
  roc_shmem_free(b);
  roc_shmem_free(a);
}

// ---- team_ctx_infra_tester.cpp:41-90 ---------------------------------------------------------------
#define NUM_TEAMS 39  // ROC_SHMEM_MAX_NUM_TEAMS - 1
__global__ void TeamCtxInfraTest(roc_shmem_team_t *team, int *errors) {
  __shared__ roc_shmem_ctx_t ctx1, ctx2, ctx3;
  __shared__ roc_shmem_ctx_t ctx[NUM_TEAMS];
  roc_shmem_wg_init();
  roc_shmem_wg_team_create_ctx(team[0], ROC_SHMEM_CTX_WG_PRIVATE, &ctx1);
  roc_shmem_wg_team_create_ctx(team[0], ROC_SHMEM_CTX_WG_PRIVATE, &ctx2);
  roc_shmem_wg_ctx_destroy(ctx1);
  roc_shmem_wg_team_create_ctx(team[0], ROC_SHMEM_CTX_WG_PRIVATE, &ctx3);
  __syncthreads();
  if (ctx3.team_opaque != ctx2.team_opaque) atomicAdd(errors, 1);
  roc_shmem_wg_ctx_destroy(ctx2);
  roc_shmem_wg_ctx_destroy(ctx3);
  __syncthreads();
  for (int team_i = 0; team_i < NUM_TEAMS; team_i++)
    roc_shmem_wg_team_create_ctx(team[team_i], ROC_SHMEM_CTX_WG_PRIVATE, &ctx[team_i]);
  if (ctx[0].team_opaque == ctx[NUM_TEAMS - 1].team_opaque) atomicAdd(errors, 1);
  for (int a = 0; a < NUM_TEAMS; a++)
    for (int b = a + 1; b < NUM_TEAMS; b++)
      if (threadIdx.x == 0 && ctx[a].team_opaque == ctx[b].team_opaque) atomicAdd(errors, 1);
  __syncthreads();
  for (int team_i = 0; team_i < NUM_TEAMS; team_i++) roc_shmem_wg_ctx_destroy(ctx[team_i]);
  // an invalid team is refused (roc_shmem_gpu.cpp:269-274)
  if (roc_shmem_wg_team_create_ctx(ROC_SHMEM_TEAM_INVALID, ROC_SHMEM_CTX_WG_PRIVATE, &ctx1) != -1)
    atomicAdd(errors, 1);
  roc_shmem_wg_finalize();
}

static void team_ctx_infra() {
  current_case = "team_ctx_infra_tester.cpp";
  roc_shmem_team_t dup[NUM_TEAMS];
  for (int i = 0; i < NUM_TEAMS; ++i) {
    dup[i] = ROC_SHMEM_TEAM_INVALID;
    roc_shmem_team_split_strided(ROC_SHMEM_TEAM_WORLD, 0, 1, npes, nullptr, 0, &dup[i]);
    EXPECT(dup[i] != ROC_SHMEM_TEAM_INVALID, "team %d is invalid", i);
  }
  roc_shmem_team_t *dev_teams = nullptr;
  int *errors = nullptr;
  (void)hipMalloc(reinterpret_cast<void **>(&dev_teams), sizeof(dup));
  (void)hipMemcpy(dev_teams, dup, sizeof(dup), hipMemcpyHostToDevice);
  (void)hipMalloc(reinterpret_cast<void **>(&errors), sizeof(int));
  (void)hipMemset(errors, 0, sizeof(int));
  TeamCtxInfraTest<<<npes * 2, 64>>>(dev_teams, errors);
  finish_kernel("TeamCtxInfraTest");
  int n = -1;
  (void)hipMemcpy(&n, errors, sizeof(int), hipMemcpyDeviceToHost);
  EXPECT(n == 0, "%d context/team identity errors", n);
  for (int i = 0; i < NUM_TEAMS; ++i) roc_shmem_team_destroy(dup[i]);
  (void)hipFree(errors);
  (void)hipFree(dev_teams);
}

// ---- team_ctx_primitive_tester.cpp:33-68: put / get through a team context; PE numbers are the
// team's.  The team here is {1, 3} of the world, so team PE 1 is world PE 3.
__global__ void TeamCtxPrimitiveTest(char *s_buf, char *r_buf, int size, int type,
                                     roc_shmem_team_t team) {
  __shared__ roc_shmem_ctx_t ctx;
  roc_shmem_wg_init();
  roc_shmem_wg_team_create_ctx(team, ROC_SHMEM_CTX_WG_PRIVATE, &ctx);
  s_buf = roc_shmemx_my_addr(s_buf);
  r_buf = roc_shmemx_my_addr(r_buf);
  if (type >= 4) {
    // The AMOs and the wg/wave calls take `pe` as a world PE even on a team
    // context (roc_shmem_gpu.cpp:556-561,667-795): 2 is not a member of {1, 3}.
    if (roc_shmem_my_pe() == 1) {
      if (type == 4) {
        roc_shmemx_ctx_putmem_wg(ctx, r_buf, s_buf, size, 2);
      } else if (threadIdx.x == 0) {
        roc_shmem_ctx_int_atomic_add(ctx, reinterpret_cast<int *>(r_buf), 0x01010101, 2);
      }
    }
  } else if (threadIdx.x == 0 && roc_shmem_my_pe() == 1) {   // team PE 0
    switch (type) {
      case 0: roc_shmem_ctx_getmem(ctx, r_buf, s_buf, size, 1); break;
      case 1: roc_shmem_ctx_getmem_nbi(ctx, r_buf, s_buf, size, 1); break;
      case 2: roc_shmem_ctx_putmem(ctx, r_buf, s_buf, size, 1); break;
      default: roc_shmem_ctx_putmem_nbi(ctx, r_buf, s_buf, size, 1); break;
    }
    roc_shmem_ctx_quiet(ctx);
  }
  roc_shmem_wg_ctx_destroy(ctx);
  roc_shmem_wg_finalize();
}

static void team_ctx_primitive() {
  current_case = "team_ctx_primitive_tester.cpp";
  if (npes < 4) return;
  const int size = 1000;
  char *s_buf = static_cast<char *>(roc_shmem_malloc(size));
  char *r_buf = static_cast<char *>(roc_shmem_malloc(size));
  roc_shmem_team_t team = ROC_SHMEM_TEAM_INVALID;
  roc_shmem_team_split_strided(ROC_SHMEM_TEAM_WORLD, 1, 2, 2, nullptr, 0, &team);
  EXPECT(team != ROC_SHMEM_TEAM_INVALID, "split {1, 3}");
  for (int type = 0; type < 6; ++type) {
    for (int pe = 0; pe < npes; ++pe) {
      fill(s_buf, size, static_cast<char>('a' + pe), pe);
      fill(r_buf, size, '1', pe);
    }
    TeamCtxPrimitiveTest<<<npes, 64>>>(s_buf, r_buf, size, type, team);
    finish_kernel("TeamCtxPrimitiveTest");
    for (int pe = 0; pe < npes; ++pe) {
      // get: world PE 1 receives PE 3's source; put: world PE 3 receives PE 1's source;
      // wg put / atomic add with pe = 2: world PE 2 is the target
      std::vector<char> got = load(r_buf, size, pe);
      for (int i = 0; i < size; ++i) {
        char want = '1';
        if (type < 2 && pe == 1) want = 'a' + 3;
        if ((type == 2 || type == 3) && pe == 3) want = 'a' + 1;
        if (type == 4 && pe == 2) want = 'a' + 1;
        if (type == 5 && pe == 2 && i < 4) want = '2';   // '1' + 1 in each byte of the first int
        EXPECT(got[i] == want, "type %d PE %d byte %d = %c", type, pe, i, got[i]);
      }
    }
  }
  roc_shmem_team_destroy(team);
  roc_shmem_free(r_buf);
  roc_shmem_free(s_buf);
}

// ---- sync_tester.cpp:33-63 and barrier_all_tester.cpp: loops of sync_all / team_sync / barrier_all,
// here with a hand-off in every round so that a barrier that lets a PE through early is seen.
__global__ void SyncTest(int loop, int type, long *slot, roc_shmem_team_t team, int *errors) {
  __shared__ roc_shmem_ctx_t ctx;
  roc_shmem_wg_init();
  roc_shmem_wg_ctx_create(ROC_SHMEM_CTX_WG_PRIVATE, &ctx);
  slot = roc_shmemx_my_addr(slot) + wg_index();
  const int me = roc_shmem_ctx_my_pe(ctx);
  const int n = roc_shmem_ctx_n_pes(ctx);
  for (int i = 1; i <= loop; i++) {
    if (threadIdx.x == 0) {
      roc_shmem_ctx_long_p(ctx, slot, 1000L * me + i, (me + 1) % n);
      roc_shmem_ctx_quiet(ctx);
    }
    switch (type) {
      case 0: roc_shmem_ctx_wg_sync_all(ctx); break;
      case 1: roc_shmem_ctx_wg_team_sync(ctx, team); break;
      default: roc_shmem_ctx_wg_barrier_all(ctx); break;
    }
    if (threadIdx.x == 0 && roc_shmem_ctx_long_g(ctx, slot, me) != 1000L * ((me + n - 1) % n) + i)
      atomicAdd(errors, 1);
    // nobody overwrites a slot before its owner has looked at it
    switch (type) {
      case 0: roc_shmem_ctx_wg_sync_all(ctx); break;
      case 1: roc_shmem_ctx_wg_team_sync(ctx, team); break;
      default: roc_shmem_ctx_wg_barrier_all(ctx); break;
    }
  }
  roc_shmem_wg_ctx_destroy(ctx);
  roc_shmem_wg_finalize();
}

static void sync_and_barrier() {
  current_case = "sync_tester.cpp / barrier_all_tester.cpp";
  const int wgs = 3, loop = 50;
  long *slot = static_cast<long *>(roc_shmem_malloc(sizeof(long) * wgs));
  int *errors = nullptr;
  (void)hipMalloc(reinterpret_cast<void **>(&errors), sizeof(int));
  roc_shmem_team_t dup = ROC_SHMEM_TEAM_INVALID;
  roc_shmem_team_split_strided(ROC_SHMEM_TEAM_WORLD, 0, 1, npes, nullptr, 0, &dup);
  for (int type = 0; type < 3; ++type) {
    (void)hipMemset(errors, 0, sizeof(int));
    for (int pe = 0; pe < npes; ++pe) fill(slot, wgs, -1L, pe);
    SyncTest<<<npes * wgs, 128>>>(loop, type, slot, dup, errors);
    finish_kernel("SyncTest");
    int n = -1;
    (void)hipMemcpy(&n, errors, sizeof(int), hipMemcpyDeviceToHost);
    EXPECT(n == 0, "type %d: %d hand-offs seen too early or too late", type, n);
  }
  roc_shmem_team_destroy(dup);
  (void)hipFree(errors);
  roc_shmem_free(slot);
}

// A team of stride 3 (world PEs 0 and 3; shmem_team_translate.cpp:46-47 splits the world this way):
// team_sync with a hand-off between the two members in every round, then a sum reduction over the
// team inside the same kernel.  PEs 1 and 2 run the kernel too and must be left alone.
__global__ void StridedTeamTest(int loop, long *slot, int *dst, const int *src, int n,
                                roc_shmem_team_t team, roc_shmem_team_t world, int *errors) {
  __shared__ roc_shmem_ctx_t ctx;
  roc_shmem_wg_init();
  roc_shmem_wg_ctx_create(ROC_SHMEM_CTX_WG_PRIVATE, &ctx);
  const int me = roc_shmem_ctx_my_pe(ctx);
  const int rank = roc_shmem_team_translate_pe(world, me, team);
  if (rank >= 0) {
    slot = roc_shmemx_my_addr(slot);
    const int other = roc_shmem_team_translate_pe(team, 1 - rank, world);
    for (int i = 1; i <= loop; i++) {
      if (threadIdx.x == 0) {
        roc_shmem_ctx_long_p(ctx, slot, 1000L * me + i, other);
        roc_shmem_ctx_quiet(ctx);
      }
      roc_shmem_ctx_wg_team_sync(ctx, team);
      if (threadIdx.x == 0 && roc_shmem_ctx_long_g(ctx, slot, me) != 1000L * other + i) atomicAdd(errors, 1);
      roc_shmem_ctx_wg_team_sync(ctx, team);
    }
    roc_shmem_ctx_int_sum_wg_to_all(ctx, team, roc_shmemx_my_addr(dst), roc_shmemx_my_addr(src), n);
  }
  roc_shmem_wg_ctx_destroy(ctx);
  roc_shmem_wg_finalize();
}

static void strided_team() {
  current_case = "team of stride 3";
  if (npes < 4) return;
  const int n = 3000, loop = 40;
  long *slot = static_cast<long *>(roc_shmem_malloc(sizeof(long)));
  int *src = static_cast<int *>(roc_shmem_malloc(n * sizeof(int)));
  int *dst = static_cast<int *>(roc_shmem_malloc(n * sizeof(int)));
  int *errors = nullptr;
  (void)hipMalloc(reinterpret_cast<void **>(&errors), sizeof(int));
  (void)hipMemset(errors, 0, sizeof(int));
  roc_shmem_team_t team = ROC_SHMEM_TEAM_INVALID;
  const int ret = roc_shmem_team_split_strided(ROC_SHMEM_TEAM_WORLD, 0, 3, 2, nullptr, 0, &team);
  EXPECT(ret == 0 && team != ROC_SHMEM_TEAM_INVALID, "split {0, 3} returned %d", ret);
  if (team != ROC_SHMEM_TEAM_INVALID) {
    for (int pe = 0; pe < npes; ++pe) {
      fill(slot, 1, -1L, pe);
      fill(src, n, 100 * (pe + 1), pe);
      fill(dst, n, -5, pe);
    }
    StridedTeamTest<<<npes, 256>>>(loop, slot, dst, src, n, team, ROC_SHMEM_TEAM_WORLD, errors);
    finish_kernel("StridedTeamTest");
    int bad = -1;
    (void)hipMemcpy(&bad, errors, sizeof(int), hipMemcpyDeviceToHost);
    EXPECT(bad == 0, "%d hand-offs seen too early or too late", bad);
    for (int pe = 0; pe < npes; ++pe) {
      std::vector<int> got = load(dst, n, pe);
      const int want = (pe == 0 || pe == 3) ? 100 * 1 + 100 * 4 : -5;
      for (int i = 0; i < n; ++i) EXPECT(got[i] == want, "PE %d [%d] = %d, expected %d", pe, i, got[i], want);
    }
    roc_shmem_team_destroy(team);
  }
  (void)hipFree(errors);
  roc_shmem_free(dst);
  roc_shmem_free(src);
  roc_shmem_free(slot);
}

// ---- swarm_tester.cpp:31-58: every thread of PE 0's workgroup gets its own chunk from PE 1 -------
__global__ void GetSwarmTest(int loop, char *s_buf, char *r_buf, int size) {
  __shared__ roc_shmem_ctx_t ctx;
  int provided;
  roc_shmem_wg_init_thread(ROC_SHMEM_THREAD_MULTIPLE, &provided);
  roc_shmem_wg_ctx_create(ROC_SHMEM_CTX_WG_PRIVATE, &ctx);
  __syncthreads();
  s_buf = roc_shmemx_my_addr(s_buf);
  r_buf = roc_shmemx_my_addr(r_buf);
  int index = threadIdx.x * size;
  if (roc_shmem_ctx_my_pe(ctx) == 0 && provided == ROC_SHMEM_THREAD_MULTIPLE) {
    for (int i = 0; i < loop; i++) {
      roc_shmem_ctx_getmem(ctx, &r_buf[index], &s_buf[index], size, 1);
      __syncthreads();
    }
  }
  roc_shmem_wg_ctx_destroy(ctx);
  roc_shmem_wg_finalize();
}

static void swarm() {
  current_case = "swarm_tester.cpp";
  const int wg_size = 256;
  for (int size : {1, 4, 8, 24, 100}) {
    char *s_buf = static_cast<char *>(roc_shmem_malloc(size * wg_size));
    char *r_buf = static_cast<char *>(roc_shmem_malloc(size * wg_size));
    for (int pe = 0; pe < npes; ++pe) {
      fill(s_buf, size * wg_size, pe == 1 ? '0' : 'x', pe);
      fill(r_buf, size * wg_size, '1', pe);
    }
    GetSwarmTest<<<npes, wg_size>>>(3, s_buf, r_buf, size);
    finish_kernel("GetSwarmTest");
    for (char c : load(r_buf, size * wg_size, 0)) EXPECT(c == '0', "size %d: got %c", size, c);
    for (char c : load(r_buf, size * wg_size, 1)) EXPECT(c == '1', "size %d: PE 1 was written", size);
    roc_shmem_free(r_buf);
    roc_shmem_free(s_buf);
  }
}

// ---- amo_standard_tester.cpp:117-163, amo_extended_tester.cpp:110-150, amo_bitwise_tester.cpp:125-170:
// thread 0 of every workgroup of PE 0 issues `iters` operations on one word of PE 1; the closed
// forms are the testers' verifyResults (num_msgs = iters * workgroups).
enum AmoOp { FAdd, FInc, Add, Inc, FCswap, Fetch, Set, Swap, FAnd, And, FOr, Or, FXor, Xor };

#define AMO_KERNEL_COMMON(T, TNAME, EXTRA)                                                        \
  __global__ void AMOTest_##TNAME(int iters, int type, T *r_buf, T *s_buf, T *ret_val) {         \
    __shared__ roc_shmem_ctx_t ctx;                                                               \
    roc_shmem_wg_init();                                                                          \
    roc_shmem_wg_ctx_create(ROC_SHMEM_CTX_WG_PRIVATE, &ctx);                                      \
    r_buf = roc_shmemx_my_addr(r_buf);                                                            \
    s_buf = roc_shmemx_my_addr(s_buf);                                                            \
    if (threadIdx.x == 0 && roc_shmem_ctx_my_pe(ctx) == 0) {                                      \
      T ret = 0;                                                                                  \
      T cond = 0;                                                                                 \
      for (int i = 0; i < iters; i++) {                                                           \
        switch (type) {                                                                           \
          case Fetch: ret = roc_shmem_ctx_##TNAME##_atomic_fetch(ctx, r_buf, 1); break;           \
          case Set: roc_shmem_ctx_##TNAME##_atomic_set(ctx, r_buf, 44, 1); break;                 \
          case Swap: ret = roc_shmem_ctx_##TNAME##_atomic_swap(ctx, r_buf, ret + 1, 1); break;    \
          EXTRA                                                                                   \
          default: break;                                                                         \
        }                                                                                         \
      }                                                                                           \
      roc_shmem_ctx_quiet(ctx);                                                                   \
      ret_val[wg_index()] = ret;                                                                  \
      roc_shmem_ctx_getmem(ctx, &s_buf[wg_index()], r_buf, sizeof(T), 1);                         \
    }                                                                                             \
    roc_shmem_wg_ctx_destroy(ctx);                                                                \
    roc_shmem_wg_finalize();                                                                      \
  }
#define AMO_STANDARD_OPS(TNAME)                                                                   \
  case FAdd: ret = roc_shmem_ctx_##TNAME##_atomic_fetch_add(ctx, r_buf, 2, 1); break;             \
  case FInc: ret = roc_shmem_ctx_##TNAME##_atomic_fetch_inc(ctx, r_buf, 1); break;                \
  case FCswap:                                                                                    \
    ret = roc_shmem_ctx_##TNAME##_atomic_compare_swap(ctx, r_buf, cond, i, 1);                    \
    cond = i;                                                                                     \
    break;                                                                                        \
  case Add: roc_shmem_ctx_##TNAME##_atomic_add(ctx, r_buf, 2, 1); break;                          \
  case Inc: roc_shmem_ctx_##TNAME##_atomic_inc(ctx, r_buf, 1); break;
#define AMO_BITWISE_OPS(TNAME)                                                                    \
  case FAnd: ret = roc_shmem_ctx_##TNAME##_atomic_fetch_and(ctx, r_buf, 0xFFFF, 1); break;        \
  case And: roc_shmem_ctx_##TNAME##_atomic_and(ctx, r_buf, 0xFFFF, 1); break;                     \
  case FOr: ret = roc_shmem_ctx_##TNAME##_atomic_fetch_or(ctx, r_buf, 0xFFFF, 1); break;          \
  case Or: roc_shmem_ctx_##TNAME##_atomic_or(ctx, r_buf, 0xFFFF, 1); break;                       \
  case FXor: ret = roc_shmem_ctx_##TNAME##_atomic_fetch_xor(ctx, r_buf, 0xFFFF, 1); break;        \
  case Xor: roc_shmem_ctx_##TNAME##_atomic_xor(ctx, r_buf, 0xFFFF, 1); break;

AMO_KERNEL_COMMON(float, float, )
AMO_KERNEL_COMMON(double, double, )
AMO_KERNEL_COMMON(int, int, AMO_STANDARD_OPS(int))
AMO_KERNEL_COMMON(long, long, AMO_STANDARD_OPS(long))
AMO_KERNEL_COMMON(long long, longlong, AMO_STANDARD_OPS(longlong))
AMO_KERNEL_COMMON(unsigned int, uint, AMO_STANDARD_OPS(uint) AMO_BITWISE_OPS(uint))
AMO_KERNEL_COMMON(unsigned long, ulong, AMO_STANDARD_OPS(ulong) AMO_BITWISE_OPS(ulong))
AMO_KERNEL_COMMON(unsigned long long, ulonglong, AMO_STANDARD_OPS(ulonglong) AMO_BITWISE_OPS(ulonglong))

template <typename T, typename Launch>
static void amo_case(const char *tname, Launch launch, bool standard, bool bitwise) {
  const int max_wgs = 8, iters = 25;
  T *r_buf = static_cast<T *>(roc_shmem_malloc(sizeof(T)));
  T *s_buf = static_cast<T *>(roc_shmem_malloc(sizeof(T) * max_wgs));
  T *ret_val = nullptr;
  (void)hipMalloc(reinterpret_cast<void **>(&ret_val), sizeof(T) * max_wgs);
  for (int type = FAdd; type <= Xor; ++type) {
    const bool is_standard = type <= FCswap, is_bitwise = type >= FAnd;
    if ((is_standard && !standard) || (is_bitwise && !bitwise)) continue;
    // compare-swap chains and swaps are only determined with one issuing workgroup
    const int wgs = (type == FCswap || type == Swap) ? 1 : max_wgs;
    const long num_msgs = static_cast<long>(iters) * wgs;
    for (int pe = 0; pe < npes; ++pe) {
      fill(r_buf, 1, static_cast<T>(0), pe);
      fill(s_buf, max_wgs, static_cast<T>(0), pe);
    }
    (void)hipMemset(ret_val, 0, sizeof(T) * max_wgs);
    launch(wgs * npes, iters, type, r_buf, s_buf, ret_val);
    finish_kernel("AMOTest");
    double expected = 0;
    bool fetch_op = false;
    switch (type) {
      case FAdd: expected = 2 * (num_msgs - 1); fetch_op = true; break;
      case FInc: expected = num_msgs - 1; fetch_op = true; break;
      case Add: expected = 2 * num_msgs; break;
      case Inc: expected = num_msgs; break;
      case FCswap: expected = (num_msgs - 2) / wgs; fetch_op = true; break;
      case Fetch: expected = 0; fetch_op = true; break;
      case Set: expected = 44; break;
      case Swap: expected = num_msgs / 2; fetch_op = true; break;
      case FAnd: case And: expected = 0; fetch_op = type == FAnd; break;
      case FOr: case Or: expected = 0xFFFF; fetch_op = type == FOr; break;
      case FXor: expected = 0xFFFF; fetch_op = true; break;
      case Xor: expected = (num_msgs % 2) ? 0xFFFF : 0; break;
    }
    std::vector<T> got(max_wgs);
    if (fetch_op) {
      (void)hipMemcpy(got.data(), ret_val, sizeof(T) * max_wgs, hipMemcpyDeviceToHost);
    } else {
      // The testers take the largest value the workgroups read back after their own operations;
      // that is the final value for add / inc / set / or, but not for xor, which toggles.  The
      // word itself, read after the kernel, is what every non-fetching operation is checked on.
      got.assign(max_wgs, load(r_buf, 1, 1)[0]);
      if (type != Xor && type != And) {
        std::vector<T> seen = load(s_buf, max_wgs, 0);
        T top = seen[0];
        for (T v : seen) top = v > top ? v : top;
        EXPECT(top == got[0], "%s op %d: largest value read back differs from the final one", tname, type);
      }
    }
    T best = got[0];
    for (T v : got) best = v > best ? v : best;
    EXPECT(static_cast<double>(best) == expected, "%s op %d: got %g, expected %g", tname, type,
           static_cast<double>(best), expected);
    for (int pe = 0; pe < npes; ++pe)
      if (pe != 1) EXPECT(load(r_buf, 1, pe)[0] == static_cast<T>(0), "%s op %d touched PE %d", tname, type, pe);
  }
  (void)hipFree(ret_val);
  roc_shmem_free(s_buf);
  roc_shmem_free(r_buf);
}

static void amo_testers() {
  current_case = "amo_standard / amo_extended / amo_bitwise testers";
#define RUN_AMO(T, TNAME, STD, BIT)                                                              \
  amo_case<T>(#TNAME,                                                                             \
              [](int grid, int iters, int type, T *r, T *s, T *rv) {                              \
                AMOTest_##TNAME<<<grid, 64>>>(iters, type, r, s, rv);                             \
              },                                                                                  \
              STD, BIT);
  RUN_AMO(float, float, false, false)
  RUN_AMO(double, double, false, false)
  RUN_AMO(int, int, true, false)
  RUN_AMO(long, long, true, false)
  RUN_AMO(long long, longlong, true, false)
  RUN_AMO(unsigned int, uint, true, true)
  RUN_AMO(unsigned long, ulong, true, true)
  RUN_AMO(unsigned long long, ulonglong, true, true)
#undef RUN_AMO
}

// ---- random_access_tester.cpp:32-93,103-126,178-221: every wave of PE 0's workgroup holds a few
// "bins" of coal_coef neighbouring lanes; the lanes of a bin put (or get) `size` bytes each to
// consecutive addresses of one randomly chosen PE, so the coalescer merges a bin into one message.
__device__ bool thread_passing(int num_bins, const uint32_t *bin_threads, const uint32_t *off_bins,
                               const uint32_t *pe_bins, int *offset, int *pe, int coal_coef, int size_ints) {
  bool pass = false;
  const int wave_id = threadIdx.x / 64;
  const int off = wave_id * num_bins;
  const uint32_t lane = threadIdx.x % 64;
  for (int i = 0; i < num_bins; i++) {
    if (lane >= bin_threads[i + off] && lane < bin_threads[i + off] + coal_coef) {
      pass = true;
      *offset = off_bins[i + off] + (lane - bin_threads[i + off]) * size_ints;
      *pe = pe_bins[i + off];
    }
  }
  return pass;
}

__global__ void RandomAccessTest(int loop, int *s_buf, int *r_buf, int size, int is_get, int coal_coef,
                                 int num_bins, const uint32_t *threads_bins, const uint32_t *off_bins,
                                 const uint32_t *pe_bins) {
  __shared__ roc_shmem_ctx_t ctx;
  roc_shmem_wg_init();
  roc_shmem_wg_ctx_create(ROC_SHMEM_CTX_WG_PRIVATE, &ctx);
  s_buf = roc_shmemx_my_addr(s_buf);
  r_buf = roc_shmemx_my_addr(r_buf);
  int offset = 0, pe = 0;
  if (roc_shmem_ctx_my_pe(ctx) == 0 &&
      thread_passing(num_bins, threads_bins, off_bins, pe_bins, &offset, &pe, coal_coef,
                     size / static_cast<int>(sizeof(int)))) {
    for (int i = 0; i < loop; i++) {
      if (is_get) {
        roc_shmem_ctx_getmem(ctx, r_buf + offset, s_buf + offset, size, pe);
      } else {
        roc_shmem_ctx_putmem(ctx, r_buf + offset, s_buf + offset, size, pe);
      }
    }
    roc_shmem_ctx_quiet(ctx);
  }
  roc_shmem_wg_ctx_destroy(ctx);
  roc_shmem_wg_finalize();
}

static void random_access() {
  current_case = "random_access_tester.cpp";
  const int wg_size = 256, num_waves = wg_size / 64, space = 8;
  uint32_t seed = 12345;
  auto next = [&seed]() { seed = seed * 1664525u + 1013904223u; return seed >> 8; };
  for (int size : {4, 8, 16, 64}) {
    for (int coal_coef : {1, 4, 8}) {
      const int thread_access = 16, num_bins = thread_access / coal_coef;   // bins per wave
      if (num_bins < 1 || 64 / num_bins - coal_coef - 1 < 0) continue;
      const int size_ints = size / static_cast<int>(sizeof(int));
      const int total_ints = space * size_ints * wg_size;
      std::vector<uint32_t> threads_bins(num_waves * num_bins), off_bins(num_waves * num_bins),
          pe_bins(num_waves * num_bins);
      for (int j = 0; j < num_waves; j++)
        for (int i = 0; i < num_bins; i++) {
          const int bin = j * num_bins + i;
          int quad = 64 / num_bins;
          const int range = quad - coal_coef - 1;
          threads_bins[bin] = (range ? next() % range : 0) + i * quad;
          quad = total_ints / (num_bins * num_waves);                 // one region of the buffer per bin
          off_bins[bin] = next() % (quad - (size_ints * coal_coef - 1)) + bin * quad;
          pe_bins[bin] = next() % npes;
        }
      uint32_t *d_threads = nullptr, *d_off = nullptr, *d_pe = nullptr;
      const size_t bin_bytes = sizeof(uint32_t) * threads_bins.size();
      (void)hipMalloc(reinterpret_cast<void **>(&d_threads), bin_bytes);
      (void)hipMalloc(reinterpret_cast<void **>(&d_off), bin_bytes);
      (void)hipMalloc(reinterpret_cast<void **>(&d_pe), bin_bytes);
      (void)hipMemcpy(d_threads, threads_bins.data(), bin_bytes, hipMemcpyHostToDevice);
      (void)hipMemcpy(d_off, off_bins.data(), bin_bytes, hipMemcpyHostToDevice);
      (void)hipMemcpy(d_pe, pe_bins.data(), bin_bytes, hipMemcpyHostToDevice);
      int *s_buf = static_cast<int *>(roc_shmem_malloc(total_ints * sizeof(int)));
      int *r_buf = static_cast<int *>(roc_shmem_malloc(total_ints * sizeof(int)));
      for (int is_get = 0; is_get < 2; ++is_get) {
        for (int pe = 0; pe < npes; ++pe) {
          fill(s_buf, total_ints, 1, pe);
          fill(r_buf, total_ints, 0, pe);
        }
        RandomAccessTest<<<npes, wg_size>>>(2, s_buf, r_buf, size, is_get, coal_coef, num_bins, d_threads,
                                            d_off, d_pe);
        finish_kernel("RandomAccessTest");
        for (int pe = 0; pe < npes; ++pe) {
          std::vector<int> want(total_ints, 0);
          for (size_t bin = 0; bin < off_bins.size(); ++bin) {
            const bool lands_here = is_get ? pe == 0 : static_cast<int>(pe_bins[bin]) == pe;
            if (!lands_here) continue;
            for (int j = 0; j < size_ints * coal_coef; j++) want[off_bins[bin] + j] = 1;
          }
          std::vector<int> got = load(r_buf, total_ints, pe);
          for (int i = 0; i < total_ints; ++i)
            EXPECT(got[i] == want[i], "size %d coal %d %s PE %d int %d: got %d", size, coal_coef,
                   is_get ? "get" : "put", pe, i, got[i]);
        }
      }
      roc_shmem_free(r_buf);
      roc_shmem_free(s_buf);
      (void)hipFree(d_pe);
      (void)hipFree(d_off);
      (void)hipFree(d_threads);
    }
  }
}

// ---- the context-less forms (ROC_SHMEM_CTX_DEFAULT; roc_shmem.hpp:907-1147) ------------------------
__global__ void DefaultCtxTest(long *data, long *counter, int n) {
  roc_shmem_wg_init();
  data = roc_shmemx_my_addr(data);
  counter = roc_shmemx_my_addr(counter);
  const int me = roc_shmem_my_pe();
  const int np = roc_shmem_n_pes();
  if (threadIdx.x == 0) {
    roc_shmem_long_p(&data[0], 10 + me, (me + 1) % np);
    roc_shmem_putmem(&data[1], &data[n], sizeof(long) * 2, (me + 1) % np);  // data[n..n+1] -> neighbour's data[1..2]
    roc_shmem_long_atomic_add(counter, me + 1, 0);
    (void)roc_shmem_long_atomic_fetch_inc(counter + 1, 0);
    roc_shmem_fence();
    roc_shmem_quiet();
  }
  roc_shmem_wg_barrier_all();
  if (threadIdx.x == 0) {
    data[3] = roc_shmem_long_g(&data[0], (me + 1) % np);   // what the neighbour received from me
    roc_shmem_getmem(&data[4], &data[1], sizeof(long) * 2, (me + 1) % np);
  }
  roc_shmem_wg_sync_all();
  roc_shmem_wg_finalize();
}

static void default_ctx() {
  current_case = "context-less device API";
  const int n = 8;
  long *data = static_cast<long *>(roc_shmem_malloc(sizeof(long) * (n + 2)));
  long *counter = static_cast<long *>(roc_shmem_malloc(sizeof(long) * 2));
  for (int pe = 0; pe < npes; ++pe) {
    std::vector<long> v(n + 2, -1);
    v[n] = 100 + pe;
    v[n + 1] = 200 + pe;
    roc_shmem_putmem(data, v.data(), sizeof(long) * (n + 2), pe);
    fill(counter, 2, 0L, pe);
  }
  DefaultCtxTest<<<npes, 64>>>(data, counter, n);
  finish_kernel("DefaultCtxTest");
  for (int pe = 0; pe < npes; ++pe) {
    const int left = (pe + npes - 1) % npes;
    std::vector<long> got = load(data, n + 2, pe);
    EXPECT(got[0] == 10 + left && got[1] == 100 + left && got[2] == 200 + left, "PE %d received %ld %ld %ld",
           pe, got[0], got[1], got[2]);
    EXPECT(got[3] == 10 + pe && got[4] == 100 + pe && got[5] == 200 + pe, "PE %d read back %ld %ld %ld", pe,
           got[3], got[4], got[5]);
  }
  std::vector<long> c = load(counter, 2, 0);
  EXPECT(c[0] == npes * (npes + 1) / 2 && c[1] == npes, "counters %ld %ld", c[0], c[1]);
  roc_shmem_free(counter);
  roc_shmem_free(data);
}

// ---- primitive_mr_tester.cpp:32-58,102-118: thread 0 of every workgroup of PE 0 issues 64 * loop
// windows of 64 putmem_nbi of `size` bytes to PE 1, with a quiet after every window; afterwards
// r_buf on PE 1 holds the source's '0' characters.  8192 posts per workgroup and launch, so the
// 1024-entry send queue wraps several times.
__global__ void PrimitiveMRTest(int loop, uint64_t *timer, char *s_buf, char *r_buf, int size) {
  __shared__ roc_shmem_ctx_t ctx;
  roc_shmem_wg_init();
  roc_shmem_wg_ctx_create(ROC_SHMEM_CTX_WG_PRIVATE, &ctx);
  s_buf = roc_shmemx_my_addr(s_buf);
  r_buf = roc_shmemx_my_addr(r_buf);
  if (threadIdx.x == 0 && roc_shmem_ctx_my_pe(ctx) == 0) {
    uint64_t start = roc_shmem_timer();
    for (int win_i = 0; win_i < 64 * loop; win_i++) {
      for (int i = 0; i < 64; i++) roc_shmem_ctx_putmem_nbi(ctx, r_buf, s_buf, size, 1);
      roc_shmem_ctx_quiet(ctx);
    }
    timer[wg_index()] = roc_shmem_timer() - start;
  }
  __syncthreads();
  roc_shmem_wg_ctx_destroy(ctx);
  roc_shmem_wg_finalize();
}

static void primitive_mr() {
  current_case = "primitive_mr_tester.cpp";
  const int wgs = 4, max_size = 1024;
  uint64_t *timer;
  EXPECT(hipMalloc(&timer, wgs * sizeof(uint64_t)) == hipSuccess, "hipMalloc");
  char *s_buf = static_cast<char *>(roc_shmem_malloc(max_size));
  char *r_buf = static_cast<char *>(roc_shmem_malloc(max_size));
  for (int size : {1, 8, 9, 64, 1000}) {
    for (int pe = 0; pe < npes; ++pe) {
      fill(s_buf, max_size, '0', pe);
      fill(r_buf, max_size, '1', pe);
    }
    for (int launch = 0; launch < 2; ++launch)  // warm-up and benchmark launch, as the tester does
      PrimitiveMRTest<<<wgs * npes, 64>>>(2, timer, s_buf, r_buf, size);
    finish_kernel("PrimitiveMRTest");
    std::vector<char> got = load(r_buf, max_size, 1);
    for (int i = 0; i < max_size; ++i)
      EXPECT(got[i] == (i < size ? '0' : '1'), "size %d: r_buf[%d] on PE 1 = %c", size, i, got[i]);
    for (int pe = 0; pe < npes; ++pe)
      if (pe != 1)
        for (char c : load(r_buf, max_size, pe)) EXPECT(c == '1', "size %d: PE %d was written", size, pe);
    uint64_t ticks[wgs];
    EXPECT(hipMemcpy(ticks, timer, sizeof(ticks), hipMemcpyDeviceToHost) == hipSuccess, "timer copy");
    printf("  putmem_nbi(%d B), quiet after every 64: %.0f ns per message issued by one lane\n", size,
           ticks[0] * 10.0 / (64 * 2 * 64));
  }
  roc_shmem_free(r_buf);
  roc_shmem_free(s_buf);
  EXPECT(hipFree(timer) == hipSuccess, "hipFree");
}

// ---- primitive_amo_tester.cpp:30-100,160-215: thread 0 of every workgroup of PE 0 issues
// loop + skip int64 operations on one word of PE 1, then quiet, and reads the word back with
// getmem; verifyResults' closed forms with num_msgs = (loop + skip) * workgroups.
enum PrimAmo { PFAdd, PFInc, PFetch, PFCswap, PAdd, PInc };
__global__ void PrimitiveAMOTest(int loop, int skip, char *r_buf, int64_t *s_buf, int64_t *ret_val, int type) {
  __shared__ roc_shmem_ctx_t ctx;
  roc_shmem_wg_init();
  roc_shmem_wg_ctx_create(ROC_SHMEM_CTX_WG_PRIVATE, &ctx);
  r_buf = roc_shmemx_my_addr(r_buf);
  s_buf = roc_shmemx_my_addr(s_buf);
  if (threadIdx.x == 0 && roc_shmem_ctx_my_pe(ctx) == 0) {
    int64_t ret = 0, cond = 0;
    for (int i = 0; i < loop + skip; i++) {
      switch (type) {
        case PFAdd: ret = roc_shmem_ctx_int64_atomic_fetch_add(ctx, (int64_t *)r_buf, 2, 1); break;
        case PFInc: ret = roc_shmem_ctx_int64_atomic_fetch_inc(ctx, (int64_t *)r_buf, 1); break;
        case PFetch: ret = roc_shmem_ctx_int64_atomic_fetch(ctx, (int64_t *)r_buf, 1); break;
        case PFCswap:
          ret = roc_shmem_ctx_int64_atomic_compare_swap(ctx, (int64_t *)r_buf, cond, (int64_t)i, 1);
          cond = i;
          break;
        case PAdd: roc_shmem_ctx_int64_atomic_add(ctx, (int64_t *)r_buf, 2, 1); break;
        case PInc: roc_shmem_ctx_int64_atomic_inc(ctx, (int64_t *)r_buf, 1); break;
        default: break;
      }
    }
    roc_shmem_ctx_quiet(ctx);
    ret_val[wg_index()] = ret;
    // a get to check the result of the ops that fetch nothing
    roc_shmem_ctx_getmem(ctx, &s_buf[wg_index()], r_buf, sizeof(int64_t), 1);
  }
  roc_shmem_wg_ctx_destroy(ctx);
  roc_shmem_wg_finalize();
}

static void primitive_amo() {
  current_case = "primitive_amo_tester.cpp";
  const int loop = 100, skip = 10, max_wgs = 8;
  int64_t *ret_val;
  EXPECT(hipMalloc(&ret_val, max_wgs * sizeof(int64_t)) == hipSuccess, "hipMalloc");
  char *r_buf = static_cast<char *>(roc_shmem_malloc(sizeof(int64_t)));
  int64_t *s_buf = static_cast<int64_t *>(roc_shmem_malloc(max_wgs * sizeof(int64_t)));
  for (int type = PFAdd; type <= PInc; ++type) {
    // the compare-and-swap chain (cond = previous i) has a closed form for one workgroup only
    for (int wgs : {1, max_wgs}) {
      if (type == PFCswap && wgs > 1) continue;
      for (int pe = 0; pe < npes; ++pe) {
        fill(reinterpret_cast<int64_t *>(r_buf), 1, int64_t{0}, pe);
        fill(s_buf, max_wgs, int64_t{0}, pe);
      }
      EXPECT(hipMemset(ret_val, 0, max_wgs * sizeof(int64_t)) == hipSuccess, "memset");
      PrimitiveAMOTest<<<wgs * npes, 64>>>(loop, skip, r_buf, s_buf, ret_val, type);
      finish_kernel("PrimitiveAMOTest");
      const int64_t num_msgs = static_cast<int64_t>(loop + skip) * wgs;
      int64_t expected = 0;
      switch (type) {
        case PFAdd: expected = 2 * (num_msgs - 1); break;
        case PFInc: expected = num_msgs - 1; break;
        case PAdd: expected = 2 * num_msgs; break;
        case PInc: expected = num_msgs; break;
        case PFCswap: expected = (num_msgs - 2) / wgs; break;
        default: break;
      }
      int64_t fetched[max_wgs];
      EXPECT(hipMemcpy(fetched, ret_val, sizeof(fetched), hipMemcpyDeviceToHost) == hipSuccess, "copy");
      std::vector<int64_t> read_back = load(s_buf, max_wgs, 0);
      int64_t best_ret = fetched[0], best_read = read_back[0];
      for (int w = 1; w < wgs; ++w) {
        best_ret = fetched[w] > best_ret ? fetched[w] : best_ret;
        best_read = read_back[w] > best_read ? read_back[w] : best_read;
      }
      if (type <= PFCswap) {
        EXPECT(best_ret == expected, "type %d, %d workgroups: fetched %ld, expected %ld", type, wgs,
               static_cast<long>(best_ret), static_cast<long>(expected));
      } else {
        EXPECT(best_read == expected, "type %d, %d workgroups: read back %ld, expected %ld", type, wgs,
               static_cast<long>(best_read), static_cast<long>(expected));
      }
    }
  }
  roc_shmem_free(s_buf);
  roc_shmem_free(r_buf);
  EXPECT(hipFree(ret_val) == hipSuccess, "hipFree");
}

// ---- many collectives inside one kernel (the shape of sos_tests/bcast_flood.cpp and
// shmem_team_b2b_collectives.cpp, on the device): `rounds` reductions back to back on one pSync,
// every PE changing its source between two of them; then as many broadcasts from a moving root.
__global__ void BackToBackCollectives(int rounds, long *src, long *dst, long *pWrk, long *pSync, int n,
                                      uint64_t *timer) {
  __shared__ roc_shmem_ctx_t ctx;
  roc_shmem_wg_init();
  roc_shmem_wg_ctx_create(ROC_SHMEM_CTX_WG_PRIVATE, &ctx);
  const int np = roc_shmem_ctx_n_pes(ctx);
  src = roc_shmemx_my_addr(src);
  dst = roc_shmemx_my_addr(dst);
  pWrk = roc_shmemx_my_addr(pWrk);
  pSync = roc_shmemx_my_addr(pSync);
  const uint64_t start = roc_shmem_timer();
  for (int r = 0; r < rounds; ++r) {
    roc_shmem_ctx_long_sum_wg_to_all(ctx, dst, src, n, 0, 0, np, pWrk, pSync);
    // the reduction has returned on this PE, so every PE has read this source
    for (int k = threadIdx.x; k < n; k += blockDim.x) src[k] += 1;
  }
  if (threadIdx.x == 0) timer[blockIdx.x] = roc_shmem_timer() - start;
  for (int r = 0; r < rounds; ++r)
    roc_shmem_ctx_long_wg_broadcast(ctx, src, dst, n, r % np, 0, 0, np, pSync);
  roc_shmem_wg_ctx_destroy(ctx);
  roc_shmem_wg_finalize();
}

static void back_to_back_collectives() {
  current_case = "collectives back to back inside one kernel";
  const int n = 4096, rounds = 100;
  long *src = static_cast<long *>(roc_shmem_malloc(n * sizeof(long)));
  long *dst = static_cast<long *>(roc_shmem_malloc(n * sizeof(long)));
  long *pWrk = static_cast<long *>(roc_shmem_malloc(ROC_SHMEM_REDUCE_MIN_WRKDATA_SIZE * sizeof(long)));
  long *pSync = static_cast<long *>(roc_shmem_malloc(ROC_SHMEM_REDUCE_SYNC_SIZE * sizeof(long)));
  uint64_t *timer;
  EXPECT(hipMalloc(&timer, npes * sizeof(uint64_t)) == hipSuccess, "hipMalloc");
  std::vector<long> v(n);
  for (int pe = 0; pe < npes; ++pe) {
    for (int k = 0; k < n; ++k) v[k] = pe + k;
    roc_shmem_putmem(src, v.data(), n * sizeof(long), pe);
    fill(dst, n, -1L, pe);
    fill(pSync, static_cast<int>(ROC_SHMEM_REDUCE_SYNC_SIZE), 0L, pe);
  }
  BackToBackCollectives<<<npes, 512>>>(rounds, src, dst, pWrk, pSync, n, timer);
  finish_kernel("BackToBackCollectives");
  // the last reduction saw src_p[k] = p + k + rounds - 1
  for (int pe = 0; pe < npes; ++pe) {
    std::vector<long> got = load(dst, n, pe);
    for (int k = 0; k < n; ++k) {
      const long want = static_cast<long>(npes) * (k + rounds - 1) + static_cast<long>(npes) * (npes - 1) / 2;
      if (got[k] != want) {
        EXPECT(false, "PE %d dst[%d] = %ld, expected %ld", pe, k, got[k], want);
        break;
      }
    }
    // every broadcast copied dst (the same everywhere) over src of all PEs but that round's root,
    // and every PE has been a receiver by then
    std::vector<long> s = load(src, n, pe);
    EXPECT(s == got, "PE %d: src differs from dst after the broadcasts (src[7] = %ld)", pe, s[7]);
    for (long x : load(pSync, static_cast<int>(ROC_SHMEM_REDUCE_SYNC_SIZE), pe)) EXPECT(x == 0, "pSync on PE %d", pe);
  }
  uint64_t ticks = 0;
  EXPECT(hipMemcpy(&ticks, timer, sizeof(ticks), hipMemcpyDeviceToHost) == hipSuccess, "timer copy");
  printf("  sum_to_all of %d longs inside one kernel: %.2f us per call (%d PEs, one workgroup each)\n", n,
         ticks * 0.01 / rounds, npes);
  EXPECT(hipFree(timer) == hipSuccess, "hipFree");
  roc_shmem_free(pSync);
  roc_shmem_free(pWrk);
  roc_shmem_free(dst);
  roc_shmem_free(src);
}

// ---- reduction_tester.cpp:74-104 and primitive_tester.cpp:32-82, kernels unchanged ---------
// The reference's tester kernels hand the pointers roc_shmem_malloc returned straight to the
// library: every process passes its own address.  Here one value serves the workgroups of
// every PE (it lies in PE 0's slice), and the roc_shmem_* calls move it into the caller's
// slice themselves, so the kernels below contain no roc_shmemx_my_addr.  Only the grid
// differs from the reference's launch (one workgroup per PE instead of one per process).
__global__ void ReductionTestUnchanged(int loop, int skip, uint64_t *timer, int *s_buf, int *r_buf,
                                       int *pWrk, long *pSync, int size) {
  __shared__ roc_shmem_ctx_t ctx;
  roc_shmem_wg_init();
  roc_shmem_wg_ctx_create(ROC_SHMEM_CTX_WG_PRIVATE, &ctx);
  int n_pes = roc_shmem_ctx_n_pes(ctx);
  __syncthreads();
  uint64_t start = 0;
  for (int i = 0; i < loop + skip; i++) {
    if (i == skip && hipThreadIdx_x == 0) start = roc_shmem_timer();
    roc_shmem_ctx_int_sum_wg_to_all(ctx, r_buf, s_buf, size, 0, 0, n_pes, pWrk, pSync);
    roc_shmem_ctx_wg_barrier_all(ctx);
  }
  __syncthreads();
  if (hipThreadIdx_x == 0) timer[hipBlockIdx_x] = roc_shmem_timer() - start;
  roc_shmem_wg_ctx_destroy(ctx);
  roc_shmem_wg_finalize();
}

__global__ void PrimitiveTestUnchanged(int loop, char *s_buf, char *r_buf, long *counter, long *flag,
                                       int size, int type) {
  __shared__ roc_shmem_ctx_t ctx;
  roc_shmem_wg_init();
  roc_shmem_wg_ctx_create(ROC_SHMEM_CTX_WG_PRIVATE, &ctx);
  const int me = roc_shmem_ctx_my_pe(ctx), np = roc_shmem_ctx_n_pes(ctx);
  if (hipThreadIdx_x == 0) {
    for (int i = 0; i < loop; i++) {
      switch (type) {
        case 0: roc_shmem_ctx_putmem(ctx, r_buf, s_buf, size, (me + 1) % np); break;
        case 1: roc_shmem_ctx_getmem(ctx, r_buf, s_buf, size, (me + 1) % np); break;
        case 2: roc_shmem_ctx_putmem_nbi(ctx, r_buf, s_buf, size, (me + 1) % np); break;
        default: roc_shmem_ctx_getmem_nbi(ctx, r_buf, s_buf, size, (me + 1) % np); break;
      }
    }
    roc_shmem_ctx_long_atomic_add(ctx, counter, me + 1, 0);
    roc_shmem_ctx_quiet(ctx);
    // tell the neighbour, wait for the other neighbour: p and wait_until on symmetric words
    roc_shmem_ctx_long_p(ctx, flag, me + 100, (me + 1) % np);
    roc_shmem_long_wait_until(flag, ROC_SHMEM_CMP_EQ, (me + np - 1) % np + 100);
  }
  __syncthreads();
  roc_shmemx_ctx_putmem_wg(ctx, r_buf + size, s_buf, size, (me + 1) % np);
  roc_shmem_ctx_quiet(ctx);
  roc_shmem_wg_ctx_destroy(ctx);
  roc_shmem_wg_finalize();
}

static void reference_kernels_unchanged() {
  current_case = "tester kernels without roc_shmemx_my_addr";
  const int size = 3000;
  int *s_buf = static_cast<int *>(roc_shmem_malloc(size * sizeof(int)));
  int *r_buf = static_cast<int *>(roc_shmem_malloc(size * sizeof(int)));
  int *pWrk = static_cast<int *>(roc_shmem_malloc(ROC_SHMEM_REDUCE_MIN_WRKDATA_SIZE * sizeof(int)));
  long *pSync = static_cast<long *>(roc_shmem_malloc(ROC_SHMEM_REDUCE_SYNC_SIZE * sizeof(long)));
  uint64_t *timer;
  EXPECT(hipMalloc(&timer, npes * sizeof(uint64_t)) == hipSuccess, "hipMalloc");
  std::vector<int> v(size);
  for (int pe = 0; pe < npes; ++pe) {
    for (int k = 0; k < size; ++k) v[k] = (pe + 1) * 1000 + k;
    roc_shmem_putmem(s_buf, v.data(), size * sizeof(int), pe);
    fill(r_buf, size, -1, pe);
    fill(pSync, static_cast<int>(ROC_SHMEM_REDUCE_SYNC_SIZE), 0L, pe);
  }
  ReductionTestUnchanged<<<npes, 256>>>(5, 2, timer, s_buf, r_buf, pWrk, pSync, size);
  finish_kernel("ReductionTestUnchanged");
  for (int pe = 0; pe < npes; ++pe) {
    std::vector<int> got = load(r_buf, size, pe);
    for (int k = 0; k < size; ++k) {
      const int want = 1000 * npes * (npes + 1) / 2 + npes * k;
      if (got[k] != want) {
        EXPECT(false, "PE %d r_buf[%d] = %d, expected %d", pe, k, got[k], want);
        break;
      }
    }
  }
  roc_shmem_free(pSync);
  roc_shmem_free(pWrk);
  roc_shmem_free(r_buf);
  roc_shmem_free(s_buf);
  EXPECT(hipFree(timer) == hipSuccess, "hipFree");

  const int bytes = 5000;
  char *cs = static_cast<char *>(roc_shmem_malloc(bytes));
  char *cr = static_cast<char *>(roc_shmem_malloc(2 * bytes));
  long *counter = static_cast<long *>(roc_shmem_malloc(sizeof(long)));
  long *flag = static_cast<long *>(roc_shmem_malloc(sizeof(long)));
  for (int type = 0; type < 4; ++type) {
    std::vector<char> c(bytes);
    for (int pe = 0; pe < npes; ++pe) {
      for (int k = 0; k < bytes; ++k) c[k] = static_cast<char>(pe * 31 + k * 7 + type);
      roc_shmem_putmem(cs, c.data(), bytes, pe);
      fill(cr, 2 * bytes, static_cast<char>(0x55), pe);
      fill(counter, 1, 0L, pe);
      fill(flag, 1, 0L, pe);
    }
    PrimitiveTestUnchanged<<<npes, 128>>>(2, cs, cr, counter, flag, bytes, type);
    finish_kernel("PrimitiveTestUnchanged");
    const bool is_put = type == 0 || type == 2;
    for (int pe = 0; pe < npes; ++pe) {
      // put: PE pe holds what its left neighbour sent; get: what its right neighbour owns
      const int from = is_put ? (pe + npes - 1) % npes : (pe + 1) % npes;
      const int from_wg = (pe + npes - 1) % npes;        // the workgroup put is always a put
      std::vector<char> got = load(cr, 2 * bytes, pe);
      for (int k = 0; k < bytes; ++k) {
        if (got[k] != static_cast<char>(from * 31 + k * 7 + type) ||
            got[bytes + k] != static_cast<char>(from_wg * 31 + k * 7 + type)) {
          EXPECT(false, "type %d PE %d byte %d", type, pe, k);
          break;
        }
      }
      EXPECT(load(flag, 1, pe)[0] == (pe + npes - 1) % npes + 100, "flag on PE %d", pe);
    }
    EXPECT(load(counter, 1, 0)[0] == static_cast<long>(npes) * (npes + 1) / 2, "counter on PE 0 = %ld",
           load(counter, 1, 0)[0]);
  }
  roc_shmem_free(flag);
  roc_shmem_free(counter);
  roc_shmem_free(cr);
  roc_shmem_free(cs);
}

// ---- blocking put, quiet, flag: the payload is there when the flag is ----------------------
// Reference: putmem_wg completes and flushes before it returns (context_ib_device.cpp:
// 148-165,219-236).  Here a blocking put gives local completion and quiet makes it visible:
// PE p puts 64 KiB into PE p+1 (another XCD, another L2), calls quiet, then sets a flag there
// with p; PE p+1 waits for the flag and must find every byte of the payload.
__global__ void PutQuietFlagTest(int rounds, char *s_buf, char *r_buf, long *flag, int size, int *errors) {
  __shared__ roc_shmem_ctx_t ctx;
  roc_shmem_wg_init();
  roc_shmem_wg_ctx_create(ROC_SHMEM_CTX_WG_PRIVATE, &ctx);
  const int me = roc_shmem_ctx_my_pe(ctx), np = roc_shmem_ctx_n_pes(ctx);
  const int right = (me + 1) % np, left = (me + np - 1) % np;
  s_buf = roc_shmemx_my_addr(s_buf);      // dereferenced below, not only passed to the library
  r_buf = roc_shmemx_my_addr(r_buf);
  int bad = 0;
  for (int r = 1; r <= rounds; ++r) {
    for (int k = threadIdx.x; k < size; k += blockDim.x) s_buf[k] = static_cast<char>(me * 17 + k + r);
    __syncthreads();
    roc_shmemx_ctx_putmem_wg(ctx, r_buf, s_buf, size, right);
    if (threadIdx.x == 0) {
      roc_shmem_ctx_quiet(ctx);
      roc_shmem_ctx_long_p(ctx, flag, r, right);
      roc_shmem_long_wait_until(flag, ROC_SHMEM_CMP_EQ, r);
    }
    __syncthreads();
    for (int k = threadIdx.x; k < size; k += blockDim.x)
      if (r_buf[k] != static_cast<char>(left * 17 + k + r)) ++bad;
    // nobody overwrites r_buf before its owner has checked it
    roc_shmem_ctx_wg_barrier_all(ctx);
  }
  if (bad) atomicAdd(errors, bad);
  roc_shmem_wg_ctx_destroy(ctx);
  roc_shmem_wg_finalize();
}

static void put_quiet_flag() {
  current_case = "blocking put + quiet, then a flag";
  const int size = 64 << 10, rounds = 20;
  char *s_buf = static_cast<char *>(roc_shmem_malloc(size));
  char *r_buf = static_cast<char *>(roc_shmem_malloc(size));
  long *flag = static_cast<long *>(roc_shmem_malloc(sizeof(long)));
  int *errors;
  EXPECT(hipMalloc(&errors, sizeof(int)) == hipSuccess, "hipMalloc");
  EXPECT(hipMemset(errors, 0, sizeof(int)) == hipSuccess, "hipMemset");
  for (int pe = 0; pe < npes; ++pe) fill(flag, 1, 0L, pe);
  PutQuietFlagTest<<<npes, 1024>>>(rounds, s_buf, r_buf, flag, size, errors);
  finish_kernel("PutQuietFlagTest");
  int bad = -1;
  EXPECT(hipMemcpy(&bad, errors, sizeof(int), hipMemcpyDeviceToHost) == hipSuccess, "copy");
  EXPECT(bad == 0, "%d payload bytes were not there when the flag was", bad);
  EXPECT(hipFree(errors) == hipSuccess, "hipFree");
  roc_shmem_free(flag);
  roc_shmem_free(r_buf);
  roc_shmem_free(s_buf);
}

// ---- a collective's result is there when the call returns ---------------------------------------
// Every workgroup reduces a tile of its own, round after round, writing new inputs before each
// call and reading its whole tile of the result right after it: what the other PEs' workgroups
// (on other XCDs) stored must be visible once the closing barrier has passed, with no help from
// the end of a kernel.  256 KiB tiles take the streaming path (results written through to
// memory, closing barrier without an L2 write-back); the ragged tiles take the element path for
// their ends (plain stores, closing barrier with the write-back).
__global__ void ResultVisibleTest(int rounds, int *src, int *dst, int *pWrk, long *pSync, int tile, int n_valid,
                                  int *errors) {
  __shared__ roc_shmem_ctx_t ctx;
  roc_shmem_wg_init();
  roc_shmem_wg_ctx_create(ROC_SHMEM_CTX_WG_PRIVATE, &ctx);
  const int me = roc_shmem_ctx_my_pe(ctx), np = roc_shmem_ctx_n_pes(ctx), w = wg_index();
  int *my_src = roc_shmemx_my_addr(src) + static_cast<size_t>(w) * tile;    // dereferenced below
  int *my_dst = roc_shmemx_my_addr(dst) + static_cast<size_t>(w) * tile;
  int bad = 0;
  for (int r = 0; r < rounds; ++r) {
    for (int k = threadIdx.x; k < n_valid; k += blockDim.x) my_src[k] = (me + 1) * (k % 1021 + r) + w;
    roc_shmem_ctx_int_sum_wg_to_all(ctx, dst + static_cast<size_t>(w) * tile, src + static_cast<size_t>(w) * tile,
                                    n_valid, 0, 0, np, pWrk, pSync + w * ROC_SHMEM_REDUCE_SYNC_SIZE);
    const int pes_sum = np * (np + 1) / 2;
    for (int k = threadIdx.x; k < n_valid; k += blockDim.x)
      if (my_dst[k] != pes_sum * (k % 1021 + r) + np * w) ++bad;
  }
  if (bad) atomicAdd(errors, bad);
  roc_shmem_wg_ctx_destroy(ctx);
  roc_shmem_wg_finalize();
}

static void result_visible_after_collective() {
  current_case = "collective result visible on return";
  const int wgs = 8, tile = 64 << 10, rounds = 60;
  int *src = static_cast<int *>(roc_shmem_malloc(sizeof(int) * wgs * tile));
  int *dst = static_cast<int *>(roc_shmem_malloc(sizeof(int) * wgs * tile));
  int *pWrk = static_cast<int *>(roc_shmem_malloc(sizeof(int) * ROC_SHMEM_REDUCE_MIN_WRKDATA_SIZE));
  long *pSync = static_cast<long *>(roc_shmem_malloc(sizeof(long) * wgs * ROC_SHMEM_REDUCE_SYNC_SIZE));
  int *errors;
  EXPECT(hipMalloc(&errors, sizeof(int)) == hipSuccess, "hipMalloc");
  for (int pe = 0; pe < npes; ++pe) fill(pSync, wgs * ROC_SHMEM_REDUCE_SYNC_SIZE, 0L, pe);
  for (int n_valid : {tile, tile - 3}) {          // aligned tiles; tiles with a ragged end
    EXPECT(hipMemset(errors, 0, sizeof(int)) == hipSuccess, "hipMemset");
    roc_shmem_barrier_all();
    ResultVisibleTest<<<npes * wgs, 512>>>(rounds, src, dst, pWrk, pSync, tile, n_valid, errors);
    finish_kernel("ResultVisibleTest");
    int bad = -1;
    EXPECT(hipMemcpy(&bad, errors, sizeof(int), hipMemcpyDeviceToHost) == hipSuccess, "copy");
    EXPECT(bad == 0, "%d elements of a result were not there when the call returned (n = %d)", bad, n_valid);
  }
  EXPECT(hipFree(errors) == hipSuccess, "hipFree");
  roc_shmem_free(pSync);
  roc_shmem_free(pWrk);
  roc_shmem_free(dst);
  roc_shmem_free(src);
}

// The same for the copying collectives: alltoall, fcollect and broadcast over the world team, each
// checked by every PE right after it returns, with new inputs every round.  Blocks of 64 KiB take
// the streaming path (written through, closing barrier without a write-back), blocks of 100
// bytes the plain-store path.
__global__ void CopiesVisibleTest(int rounds, roc_shmem_team_t team, int *src, int *dst, int nelem, int *errors) {
  __shared__ roc_shmem_ctx_t ctx;
  roc_shmem_wg_init();
  roc_shmem_wg_ctx_create(ROC_SHMEM_CTX_WG_PRIVATE, &ctx);
  const int me = roc_shmem_ctx_my_pe(ctx), np = roc_shmem_ctx_n_pes(ctx);
  int *my_src = roc_shmemx_my_addr(src), *my_dst = roc_shmemx_my_addr(dst);   // dereferenced below
  int bad = 0;
  for (int r = 0; r < rounds; ++r) {
    // alltoall: my block j goes to PE j's block `me`
    for (int k = threadIdx.x; k < np * nelem; k += blockDim.x) my_src[k] = (me << 20) + k * 7 + r;
    roc_shmem_ctx_int_wg_alltoall(ctx, team, dst, src, nelem);
    for (int k = threadIdx.x; k < np * nelem; k += blockDim.x) {
      const int from = k / nelem, at = me * nelem + k % nelem;
      if (my_dst[k] != (from << 20) + at * 7 + r) ++bad;
    }
    roc_shmem_ctx_wg_team_sync(ctx, team);      // everybody has checked before dst is written again
    // fcollect: my first block lands in block `me` of everybody
    for (int k = threadIdx.x; k < nelem; k += blockDim.x) my_src[k] = (me << 20) - k * 3 - r;
    roc_shmem_ctx_int_wg_fcollect(ctx, team, dst, src, nelem);
    for (int k = threadIdx.x; k < np * nelem; k += blockDim.x)
      if (my_dst[k] != ((k / nelem) << 20) - (k % nelem) * 3 - r) ++bad;
    roc_shmem_ctx_wg_team_sync(ctx, team);
    // broadcast from a moving root: everybody but the root receives its first block
    const int root = r % np;
    for (int k = threadIdx.x; k < nelem; k += blockDim.x) my_src[k] = (me << 20) ^ (k * 5 + r);
    roc_shmem_ctx_int_wg_broadcast(ctx, team, dst, src, nelem, root);
    if (me != root)
      for (int k = threadIdx.x; k < nelem; k += blockDim.x)
        if (my_dst[k] != ((root << 20) ^ (k * 5 + r))) ++bad;
    roc_shmem_ctx_wg_team_sync(ctx, team);
  }
  if (bad) atomicAdd(errors, bad);
  roc_shmem_wg_ctx_destroy(ctx);
  roc_shmem_wg_finalize();
}

static void copies_visible_after_collective() {
  current_case = "alltoall / fcollect / broadcast results visible on return";
  int *errors;
  EXPECT(hipMalloc(&errors, sizeof(int)) == hipSuccess, "hipMalloc");
  for (int nelem : {16 << 10, 25}) {
    int *src = static_cast<int *>(roc_shmem_malloc(sizeof(int) * npes * nelem));
    int *dst = static_cast<int *>(roc_shmem_malloc(sizeof(int) * npes * nelem));
    EXPECT(hipMemset(errors, 0, sizeof(int)) == hipSuccess, "hipMemset");
    roc_shmem_barrier_all();
    CopiesVisibleTest<<<npes, 512>>>(40, ROC_SHMEM_TEAM_WORLD, src, dst, nelem, errors);
    finish_kernel("CopiesVisibleTest");
    int bad = -1;
    EXPECT(hipMemcpy(&bad, errors, sizeof(int), hipMemcpyDeviceToHost) == hipSuccess, "copy");
    EXPECT(bad == 0, "%d elements were not there when a collective returned (blocks of %d ints)", bad, nelem);
    roc_shmem_free(dst);
    roc_shmem_free(src);
  }
  EXPECT(hipFree(errors) == hipSuccess, "hipFree");
}

// ---- fence and quiet on queues with a live consumer -----------------------------------------
// Reference: roc_shmem_ctx_fence posts an inline write to the destination's flush word
// (QueuePair::fence, queue_pair.cpp:376-384) and roc_shmem_ctx_quiet a zero-byte read before it
// polls for completions (quiet_heavy, thread_policy.cpp:35-108; zero_b_rd, queue_pair.cpp:318-325).
// With a consumer running beside the kernel the same entries appear on the context's queue, in
// program order between the puts, and quiet returns with every completion collected.
__global__ void FenceQuietLiveTest(long *word) {
  __shared__ roc_shmem_ctx_t ctx;
  roc_shmem_wg_init();
  roc_shmem_wg_ctx_create(ROC_SHMEM_CTX_WG_PRIVATE, &ctx);
  const int me = roc_shmem_ctx_my_pe(ctx), right = (me + 1) % roc_shmem_ctx_n_pes(ctx);
  if (threadIdx.x == 0) {
    roc_shmem_ctx_long_p(ctx, word, 100 + me, right);
    roc_shmem_ctx_fence(ctx);
    roc_shmem_ctx_long_p(ctx, word + 1, 200 + me, right);
    roc_shmem_ctx_quiet(ctx);
  }
  roc_shmem_wg_ctx_destroy(ctx);
  roc_shmem_wg_finalize();
}

static uint64_t be64_of(uint64_t le_word) { return __builtin_bswap64(le_word); }

static void fence_quiet_live() {
  current_case = "fence and quiet on live queues";
  long *word = static_cast<long *>(roc_shmem_malloc(2 * sizeof(long)));
  for (int pe = 0; pe < npes; ++pe) fill(word, 2, 0L, pe);
  roc_shmem_barrier_all();
  hipStream_t stream;
  EXPECT(hipStreamCreate(&stream) == hipSuccess, "hipStreamCreate");
  EXPECT(rsm_sq_reset() == 0, "rsm_sq_reset: %s", rsm_last_error());
  EXPECT(rsm_sq_consumer_start() == 0, "rsm_sq_consumer_start: %s", rsm_last_error());
  FenceQuietLiveTest<<<npes, 64, 0, stream>>>(word);
  EXPECT(hipStreamSynchronize(stream) == hipSuccess, "hipStreamSynchronize");
  rsm_consume_totals_t t;
  EXPECT(rsm_sq_consumer_stop(&t) == 0, "rsm_sq_consumer_stop: %s", rsm_last_error());
  finish_kernel("FenceQuietLiveTest");
  EXPECT(t.retired == 4ull * npes && t.writes == 3ull * npes && t.reads == 1ull * npes && t.atomics == 0 &&
             t.rejected == 0 && t.lost == 0 && t.bytes == (8ull + 4 + 8) * npes,
         "totals: retired %llu writes %llu reads %llu rejected %llu lost %llu bytes %llu",
         (unsigned long long)t.retired, (unsigned long long)t.writes, (unsigned long long)t.reads,
         (unsigned long long)t.rejected, (unsigned long long)t.lost, (unsigned long long)t.bytes);
  for (int pe = 0; pe < npes; ++pe) {
    const int left = (pe + npes - 1) % npes;
    auto got = load(word, 2, pe);
    EXPECT(got[0] == 100 + left && got[1] == 200 + left, "PE %d holds %ld %ld", pe, got[0], got[1]);
    uint32_t sq_counter = 0, published = 0, atomic_counter = 0, cq_consumer = 0, quiet_counter = 9, cq_db = 0;
    uint64_t mailbox[2];
    EXPECT(rsm_sq_state(pe, 0, &sq_counter, &published, &atomic_counter, mailbox) == 0, "rsm_sq_state");
    EXPECT(sq_counter == 4 && published == 4, "PE %d: %u entries posted, %u published", pe, sq_counter, published);
    EXPECT(rsm_cq_reader_state(pe, 0, &cq_consumer, &quiet_counter, &cq_db) == 0, "rsm_cq_reader_state");
    EXPECT(quiet_counter == 0 && cq_consumer == 4, "PE %d: quiet left %u completions, took %u", pe,
           quiet_counter, cq_consumer);
    uint64_t flush_addr = 0;
    uint32_t flush_key = 0, heap_key = 0;
    EXPECT(rsm_sq_flush_target(pe, &flush_addr, &flush_key) == 0 && rsm_sq_rkey(pe, &heap_key) == 0, "keys");
    uint64_t e[8];
    // entry 1: fence's flush write
    EXPECT(rsm_sq_read(pe, 0, 1, e) == 0, "rsm_sq_read");
    const uint8_t *b = reinterpret_cast<const uint8_t *>(e);
    EXPECT(b[3] == 0x08 && b[7] == 3 && b[1] == 0 && b[2] == 1 && b[11] == 8, "PE %d fence entry: control %02x ds %u",
           pe, b[3], b[7]);
    EXPECT(be64_of(e[2]) == flush_addr && static_cast<uint32_t>(e[3]) == flush_key,
           "PE %d fence entry: address %llx key %x", pe, (unsigned long long)be64_of(e[2]),
           static_cast<uint32_t>(e[3]));
    EXPECT(b[32] == 0x80 && b[33] == 0 && b[34] == 0 && b[35] == 4 && b[36] == 1, "PE %d fence entry: inline segment", pe);
    // entry 3: quiet's zero-byte read, addressed to the PE's own heap
    EXPECT(rsm_sq_read(pe, 0, 3, e) == 0, "rsm_sq_read");
    EXPECT(b[3] == 0x10 && b[7] == 2 && b[2] == 3 && b[11] == 8, "PE %d quiet entry: opcode %02x ds %u", pe, b[3], b[7]);
    EXPECT(be64_of(e[2]) == reinterpret_cast<uint64_t>(rsm_heap_base(pe)) && static_cast<uint32_t>(e[3]) == heap_key,
           "PE %d quiet entry: address %llx", pe, (unsigned long long)be64_of(e[2]));
    EXPECT(e[4] == 0 && e[5] == 0 && e[6] == 0 && e[7] == 0, "PE %d quiet entry wrote beyond its two segments", pe);
  }
  EXPECT(hipStreamDestroy(stream) == hipSuccess, "hipStreamDestroy");
  roc_shmem_free(word);
}

int main() {
  if (!getenv("ROC_SHMEM_NUM_PES")) setenv("ROC_SHMEM_NUM_PES", "4", 1);
  setenv("ROC_SHMEM_HEAP_SIZE", "67108864", 0);
  roc_shmem_init();
  npes = roc_shmem_n_pes();
  struct {
    const char *name;
    void (*run)();
  } cases[] = {{"ping_pong", ping_pong},       {"compare_ops", compare_ops},
               {"narrow_ping_pong", narrow_ping_pong},
               {"shmem_ptr", shmem_ptr},       {"shmem_ptr_as_argument", shmem_ptr_as_argument},
               {"team_ctx_infra", team_ctx_infra},
               {"team_ctx_primitive", team_ctx_primitive}, {"sync_and_barrier", sync_and_barrier},
               {"strided_team", strided_team},
               {"swarm", swarm},               {"amo_testers", amo_testers},
               {"random_access", random_access},
               {"default_ctx", default_ctx},   {"primitive_mr", primitive_mr},
               {"primitive_amo", primitive_amo},
               {"back_to_back_collectives", back_to_back_collectives},
               {"reference_kernels_unchanged", reference_kernels_unchanged},
               {"put_quiet_flag", put_quiet_flag},
               {"result_visible_after_collective", result_visible_after_collective},
               {"copies_visible_after_collective", copies_visible_after_collective},
               {"fence_quiet_live", fence_quiet_live}};
  for (auto &c : cases) {
    const int before = failures;
    c.run();
    printf("%-28s %s\n", c.name, failures == before ? "ok" : "FAILED");
    fflush(stdout);
  }
  roc_shmem_finalize();
  if (failures) {
    printf("DEVICE_API_FAILED %d\n", failures);
    return 1;
  }
  printf("DEVICE_API_OK\n");
  return 0;
}
