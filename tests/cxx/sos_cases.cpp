// The reference's host-program tests (clients/sos_tests/*.cpp), restated for a
// process that hosts every PE.  Each case keeps the reference's inputs and its
// closed-form expectation and cites the file it follows.  Where the
// reference's SPMD code says "every PE does X", the case loops over the PEs
// with roc_shmemx_set_pe; where it dereferences symmetric memory on the host,
// the case goes through roc_shmem_<T>_put / _get, which also works when the
// arena is not host-visible (ROC_SHMEM_HEAP_HOST_VISIBLE=0).  A collective is
// called once for all members.
// Exit code 0 and a final line "SOS_CASES_OK" mean every case passed.
#include <cstdio>
#include <cstdlib>
#include <cstring>
#include <vector>

#include "roc_shmem.hpp"

using namespace rocshmem;

static int failures = 0;
static const char *current_case = "";
#define EXPECT(cond, ...)                                        \
  do {                                                           \
    if (!(cond)) {                                               \
      if (++failures <= 20) {                                    \
        printf("FAIL [%s] %s:%d: ", current_case, __FILE__, __LINE__); \
        printf(__VA_ARGS__);                                     \
        printf("\n");                                            \
      }                                                          \
    }                                                            \
  } while (0)

// A symmetric array of n elements of T with host-side access per PE.
template <typename T>
struct Sym {
  T *ptr;
  int n;
  explicit Sym(int count) : ptr(static_cast<T *>(roc_shmem_malloc(count * sizeof(T)))), n(count) {
    if (!ptr) {
      printf("roc_shmem_malloc failed\n");
      exit(2);
    }
  }
  ~Sym() { roc_shmem_free(ptr); }
  void store(int pe, const std::vector<T> &v) const {
    roc_shmem_putmem(ptr, v.data(), static_cast<size_t>(n) * sizeof(T), pe);
  }
  void fill(int pe, T value) const { store(pe, std::vector<T>(n, value)); }
  std::vector<T> load(int pe) const {
    std::vector<T> v(n);
    roc_shmem_getmem(v.data(), ptr, static_cast<size_t>(n) * sizeof(T), pe);
    return v;
  }
};

static int npes;

// ---- reductions ---------------------------------------------------------------------

#define FOR_REDUCE_TYPES(X) X(short, short) X(int, int) X(long, long) X(float, float) X(double, double) X(long long, longlong)
#define FOR_BITWISE_TYPES(X) X(short, short) X(int, int) X(long, long) X(long long, longlong)

// clients/sos_tests/to_all.cpp:118-760, N = 128: max/min of me+i, sum of me, and of me,
// prod of me+1, or of (me+1)%4, xor of me%2, checked on every PE.
template <typename T, typename Call, typename Src, typename Want>
static void reduce_case(const char *name, Call call, Src src_of, Want want_of) {
  current_case = name;
  const int N = 128;
  Sym<T> src(N), dst(N);
  for (int me = 0; me < npes; ++me) {
    std::vector<T> v(N);
    for (int i = 0; i < N; ++i) v[i] = static_cast<T>(src_of(me, i));
    src.store(me, v);
    dst.fill(me, static_cast<T>(-9));
  }
  roc_shmem_barrier_all();
  call(dst.ptr, src.ptr, N);
  for (int me = 0; me < npes; ++me) {
    std::vector<T> got = dst.load(me);
    for (int i = 0; i < N; ++i)
      EXPECT(got[i] == static_cast<T>(want_of(i)), "PE %d element %d: %g, expected %g", me, i,
             static_cast<double>(got[i]), static_cast<double>(want_of(i)));
  }
}

static void to_all_cases() {
  long factorial = 1;
  for (int i = 1; i <= npes; ++i) factorial *= i;
#define MAXMIN_SUM_PROD(T, TNAME)                                                                  \
  reduce_case<T>("to_all.cpp max " #TNAME,                                                         \
                 [](T *d, const T *s, int n) {                                                     \
                   roc_shmem_ctx_##TNAME##_max_to_all(ROC_SHMEM_CTX_DEFAULT, d, s, n, 0, 0, npes,  \
                                                      nullptr, nullptr);                           \
                 },                                                                                \
                 [](int me, int i) { return me + i; }, [](int i) { return npes - 1 + i; });        \
  reduce_case<T>("to_all.cpp min " #TNAME,                                                         \
                 [](T *d, const T *s, int n) {                                                     \
                   roc_shmem_ctx_##TNAME##_min_to_all(ROC_SHMEM_CTX_DEFAULT, d, s, n, 0, 0, npes,  \
                                                      nullptr, nullptr);                           \
                 },                                                                                \
                 [](int me, int i) { return me + i; }, [](int i) { return i; });                   \
  reduce_case<T>("to_all.cpp sum " #TNAME,                                                         \
                 [](T *d, const T *s, int n) {                                                     \
                   roc_shmem_ctx_##TNAME##_sum_to_all(ROC_SHMEM_CTX_DEFAULT, d, s, n, 0, 0, npes,  \
                                                      nullptr, nullptr);                           \
                 },                                                                                \
                 [](int me, int) { return me; }, [](int) { return npes * (npes - 1) / 2; });       \
  reduce_case<T>("to_all.cpp prod " #TNAME,                                                        \
                 [](T *d, const T *s, int n) {                                                     \
                   roc_shmem_ctx_##TNAME##_prod_to_all(ROC_SHMEM_CTX_DEFAULT, d, s, n, 0, 0, npes, \
                                                       nullptr, nullptr);                          \
                 },                                                                                \
                 [](int me, int) { return me + 1; }, [factorial](int) { return factorial; });
  FOR_REDUCE_TYPES(MAXMIN_SUM_PROD)
#undef MAXMIN_SUM_PROD
#define BITWISE(T, TNAME)                                                                          \
  reduce_case<T>("to_all.cpp and " #TNAME,                                                         \
                 [](T *d, const T *s, int n) {                                                     \
                   roc_shmem_ctx_##TNAME##_and_to_all(ROC_SHMEM_CTX_DEFAULT, d, s, n, 0, 0, npes,  \
                                                      nullptr, nullptr);                           \
                 },                                                                                \
                 [](int me, int) { return me; }, [](int) { return 0; });                           \
  reduce_case<T>("to_all.cpp or " #TNAME,                                                          \
                 [](T *d, const T *s, int n) {                                                     \
                   roc_shmem_ctx_##TNAME##_or_to_all(ROC_SHMEM_CTX_DEFAULT, d, s, n, 0, 0, npes,   \
                                                     nullptr, nullptr);                            \
                 },                                                                                \
                 [](int me, int) { return (me + 1) % 4; }, [](int) { return npes == 1 ? 1 : 3; }); \
  reduce_case<T>("to_all.cpp xor " #TNAME,                                                         \
                 [](T *d, const T *s, int n) {                                                     \
                   roc_shmem_ctx_##TNAME##_xor_to_all(ROC_SHMEM_CTX_DEFAULT, d, s, n, 0, 0, npes,  \
                                                      nullptr, nullptr);                           \
                 },                                                                                \
                 [](int me, int) { return me % 2; }, [](int) { return (npes / 2) % 2; });
  FOR_BITWISE_TYPES(BITWISE)
#undef BITWISE
}

// clients/sos_tests/max_reduction.cpp:65-99: N = 3, src = me + i, long max -> npes - 1 + i.
static void max_reduction() {
  current_case = "max_reduction.cpp";
  const int N = 3;
  Sym<long> src(N), dst(N);
  for (int me = 0; me < npes; ++me) src.store(me, {me + 0L, me + 1L, me + 2L});
  roc_shmem_barrier_all();
  roc_shmem_ctx_long_max_to_all(ROC_SHMEM_CTX_DEFAULT, dst.ptr, src.ptr, N, 0, 0, npes, nullptr, nullptr);
  for (int me = 0; me < npes; ++me) {
    std::vector<long> got = dst.load(me);
    for (int i = 0; i < N; ++i) EXPECT(got[i] == npes - 1 + i, "PE %d dst[%d] = %ld", me, i, got[i]);
  }
}

// clients/sos_tests/big_reduction.cpp:76-107 (long max over N elements of me + i) and
// reduce_in_place.cpp:58-69 (dest == source).
static void big_and_in_place_reduction() {
  current_case = "big_reduction.cpp / reduce_in_place.cpp";
  const int N = 1 << 20;
  Sym<long> buf(N);
  std::vector<long> v(N);
  for (int me = 0; me < npes; ++me) {
    for (int i = 0; i < N; ++i) v[i] = me + i;
    buf.store(me, v);
  }
  roc_shmem_barrier_all();
  roc_shmem_ctx_long_max_to_all(ROC_SHMEM_CTX_DEFAULT, buf.ptr, buf.ptr, N, 0, 0, npes, nullptr, nullptr);
  for (int me = 0; me < npes; ++me) {
    std::vector<long> got = buf.load(me);
    for (int i = 0; i < N; ++i) EXPECT(got[i] == npes - 1 + i, "PE %d [%d] = %ld", me, i, got[i]);
  }
}

// clients/sos_tests/reduce_active_set.cpp:78-113: for i = 0..npes-1 the PEs i..npes-1 sum
// src = me (long long); members get sum_{p>=i} p, the others keep -1.
static void reduce_active_set() {
  current_case = "reduce_active_set.cpp";
  const int N = 4;
  Sym<long long> src(N), dst(N);
  for (int start = 0; start < npes; ++start) {
    for (int me = 0; me < npes; ++me) {
      src.fill(me, me);
      dst.fill(me, -1);
    }
    roc_shmem_barrier_all();
    roc_shmem_ctx_longlong_sum_to_all(ROC_SHMEM_CTX_DEFAULT, dst.ptr, src.ptr, N, start, 0, npes - start,
                                      nullptr, nullptr);
    long long want = 0;
    for (int p = start; p < npes; ++p) want += p;
    for (int me = 0; me < npes; ++me) {
      std::vector<long long> got = dst.load(me);
      for (int i = 0; i < N; ++i)
        EXPECT(got[i] == (me >= start ? want : -1), "start %d PE %d [%d] = %lld", start, me, i, got[i]);
    }
  }
}

// clients/sos_tests/shmem_team_reduce.cpp:88-101 on the world team: src = 1 -> and/or/max/min/prod
// give 1, sum gives npes, xor gives npes % 2.
static void team_reduce() {
  current_case = "shmem_team_reduce.cpp";
  const int N = 10;
  Sym<int> src(N), dst(N);
  for (int me = 0; me < npes; ++me) src.fill(me, 1);
  struct {
    void (*call)(roc_shmem_ctx_t, roc_shmem_team_t, int *, const int *, int);
    int want;
    const char *name;
  } ops[] = {
      {roc_shmem_ctx_int_and_to_all, 1, "and"},   {roc_shmem_ctx_int_or_to_all, 1, "or"},
      {roc_shmem_ctx_int_max_to_all, 1, "max"},   {roc_shmem_ctx_int_min_to_all, 1, "min"},
      {roc_shmem_ctx_int_prod_to_all, 1, "prod"}, {roc_shmem_ctx_int_sum_to_all, npes, "sum"},
      {roc_shmem_ctx_int_xor_to_all, npes % 2, "xor"},
  };
  for (auto &op : ops) {
    for (int me = 0; me < npes; ++me) dst.fill(me, -7);
    op.call(ROC_SHMEM_CTX_DEFAULT, ROC_SHMEM_TEAM_WORLD, dst.ptr, src.ptr, N);
    for (int me = 0; me < npes; ++me) {
      std::vector<int> got = dst.load(me);
      for (int i = 0; i < N; ++i) EXPECT(got[i] == op.want, "%s PE %d [%d] = %d", op.name, me, i, got[i]);
    }
  }
}

// ---- put / get -------------------------------------------------------------------------

// clients/sos_tests/put1.cpp:38-68: PE 0 puts ten longs 1..10 into PE 1.
static void put1() {
  current_case = "put1.cpp";
  long source[10] = {1, 2, 3, 4, 5, 6, 7, 8, 9, 10};
  Sym<long> target(10);
  for (int me = 0; me < npes; ++me) target.fill(me, 0);
  roc_shmemx_set_pe(0);
  roc_shmem_long_put(target.ptr, source, 10, 1);
  roc_shmem_barrier_all();
  std::vector<long> got = target.load(1);
  EXPECT(memcmp(got.data(), source, sizeof(source)) == 0, "target on PE 1 differs from the source");
  for (int me = 0; me < npes; ++me)
    if (me != 1) {
      std::vector<long> other = target.load(me);
      for (long x : other) EXPECT(x == 0, "PE %d was written", me);
    }
}

// clients/sos_tests/get_nbi.cpp:47-76 (PE 0 gets source = i + 1 from every PE, quiet, compare) and
// put_nbi.cpp (the mirror image with put_nbi + quiet).
static void get_nbi_put_nbi() {
  current_case = "get_nbi.cpp / put_nbi.cpp";
  Sym<long> source(10), target(10);
  std::vector<long> pattern(10);
  for (int i = 0; i < 10; ++i) pattern[i] = i + 1;
  for (int me = 0; me < npes; ++me) {
    source.store(me, pattern);
    target.fill(me, 0);
  }
  roc_shmem_barrier_all();
  roc_shmemx_set_pe(0);
  for (int j = 0; j < npes; ++j) {
    long local[10] = {0};
    roc_shmem_long_get_nbi(local, source.ptr, 10, j);
    roc_shmem_quiet();
    for (int i = 0; i < 10; ++i) EXPECT(local[i] == i + 1, "get_nbi from PE %d [%d] = %ld", j, i, local[i]);
  }
  for (int j = 0; j < npes; ++j) roc_shmem_long_put_nbi(target.ptr, pattern.data(), 10, j);
  roc_shmem_quiet();
  for (int j = 0; j < npes; ++j) {
    std::vector<long> got = target.load(j);
    for (int i = 0; i < 10; ++i) EXPECT(got[i] == i + 1, "put_nbi to PE %d [%d] = %ld", j, i, got[i]);
  }
}

// clients/sos_tests/bigput.cpp:202-263 and bigget.cpp: a large block of Source[i] = i + 1 moved
// to / from the next PE arrives unchanged.
static void bigput_bigget() {
  current_case = "bigput.cpp / bigget.cpp";
  const int N = 1 << 20;
  Sym<int> source(N), target(N);
  std::vector<int> pattern(N), back(N);
  for (int i = 0; i < N; ++i) pattern[i] = i + 1;
  for (int me = 0; me < npes; ++me) {
    source.store(me, pattern);
    target.fill(me, -90);
  }
  for (int me = 0; me < npes; ++me) {
    roc_shmemx_set_pe(me);
    // the host-side put takes any host or device pointer as its local buffer
    roc_shmem_int_put(target.ptr, pattern.data(), N, (me + 1) % npes);
  }
  roc_shmem_barrier_all();
  for (int me = 0; me < npes; ++me) {
    roc_shmemx_set_pe(me);
    roc_shmem_int_get(back.data(), target.ptr, N, (me + 1) % npes);
    EXPECT(back == pattern, "block fetched by PE %d differs", me);
  }
}

// clients/sos_tests/cxx_test_shmem_p.cpp:42-62 and cxx_test_shmem_g.cpp:42-64, all standard types,
// with and without a context: p of (TYPE)me to the right-hand neighbour; g from it.
template <typename T, typename P, typename G>
static void p_g_case(const char *name, P p, G g) {
  current_case = name;
  Sym<T> remote(1);
  for (int me = 0; me < npes; ++me) {
    roc_shmemx_set_pe(me);
    p(remote.ptr, static_cast<T>(me), (me + 1) % npes);
  }
  roc_shmem_barrier_all();
  for (int me = 0; me < npes; ++me)
    EXPECT(remote.load(me)[0] == static_cast<T>((me + npes - 1) % npes), "p: PE %d", me);
  for (int me = 0; me < npes; ++me) remote.fill(me, static_cast<T>(me));
  roc_shmem_barrier_all();
  for (int me = 0; me < npes; ++me) {
    roc_shmemx_set_pe(me);
    EXPECT(g(remote.ptr, (me + 1) % npes) == static_cast<T>((me + 1) % npes), "g: PE %d", me);
  }
}

static void p_and_g() {
#define PG(T, TNAME)                                                                              \
  p_g_case<T>("cxx_test_shmem_p/g " #TNAME,                                                       \
              [](T *d, T v, int pe) { roc_shmem_##TNAME##_p(d, v, pe); },                         \
              [](const T *s, int pe) { return roc_shmem_##TNAME##_g(s, pe); });                   \
  p_g_case<T>("cxx_test_shmem_p/g ctx " #TNAME,                                                   \
              [](T *d, T v, int pe) { roc_shmem_ctx_##TNAME##_p(ROC_SHMEM_CTX_DEFAULT, d, v, pe); }, \
              [](const T *s, int pe) { return roc_shmem_ctx_##TNAME##_g(ROC_SHMEM_CTX_DEFAULT, s, pe); });
  PG(float, float) PG(double, double) PG(char, char) PG(signed char, schar) PG(short, short) PG(int, int)
  PG(long, long) PG(long long, longlong) PG(unsigned char, uchar) PG(unsigned short, ushort)
  PG(unsigned int, uint) PG(unsigned long, ulong) PG(unsigned long long, ulonglong)
#undef PG
}

// ---- atomics ------------------------------------------------------------------------------

#define FOR_AMO_TYPES(X)                                                                            \
  X(int, int) X(long, long) X(long long, longlong) X(unsigned int, uint) X(unsigned long, ulong)    \
  X(unsigned long long, ulonglong) X(int32_t, int32) X(int64_t, int64) X(uint32_t, uint32)          \
  X(uint64_t, uint64) X(size_t, size) X(ptrdiff_t, ptrdiff)

template <typename T, typename Add, typename FetchAdd>
static void atomic_add_case(const char *name, Add add, FetchAdd fetch_add) {
  // cxx_test_shmem_atomic_add.cpp:85-144: every PE adds me + 1 to every PE -> npes(npes+1)/2;
  // the fetching form additionally returns something no larger than the final value.
  current_case = name;
  Sym<T> remote(1);
  for (int me = 0; me < npes; ++me) remote.fill(me, 0);
  roc_shmem_barrier_all();
  for (int me = 0; me < npes; ++me) {
    roc_shmemx_set_pe(me);
    for (int i = 0; i < npes; ++i) add(remote.ptr, static_cast<T>(me + 1), i);
  }
  roc_shmem_barrier_all();
  const T total = static_cast<T>(npes * (npes + 1) / 2);
  for (int me = 0; me < npes; ++me) EXPECT(remote.load(me)[0] == total, "add: PE %d", me);
  for (int me = 0; me < npes; ++me) remote.fill(me, 0);
  for (int me = 0; me < npes; ++me) {
    roc_shmemx_set_pe(me);
    for (int i = 0; i < npes; ++i) {
      T old = fetch_add(remote.ptr, static_cast<T>(me + 1), i);
      EXPECT(old <= total, "fetch_add: PE %d old too large", me);
    }
  }
  for (int me = 0; me < npes; ++me) EXPECT(remote.load(me)[0] == total, "fetch_add: PE %d", me);
}

template <typename T, typename Fetch, typename Inc, typename FetchInc, typename Cswap>
static void atomic_fetch_inc_cswap_case(const char *name, Fetch fetch, Inc inc, FetchInc fetch_inc,
                                        Cswap cswap) {
  current_case = name;
  Sym<T> remote(1);
  // cxx_test_shmem_atomic_fetch.cpp:66-107: *remote = me; fetch from the neighbour gives its rank.
  for (int me = 0; me < npes; ++me) remote.fill(me, static_cast<T>(me));
  roc_shmem_barrier_all();
  for (int me = 0; me < npes; ++me) {
    roc_shmemx_set_pe(me);
    EXPECT(fetch(remote.ptr, (me + 1) % npes) == static_cast<T>((me + 1) % npes), "fetch: PE %d", me);
  }
  // cxx_test_shmem_atomic_inc.cpp:85-147: every PE increments every PE once -> npes; a fetched
  // old value is never larger than npes.
  for (int me = 0; me < npes; ++me) remote.fill(me, 0);
  for (int me = 0; me < npes; ++me) {
    roc_shmemx_set_pe(me);
    for (int i = 0; i < npes; ++i) inc(remote.ptr, i);
  }
  for (int me = 0; me < npes; ++me) EXPECT(remote.load(me)[0] == static_cast<T>(npes), "inc: PE %d", me);
  for (int me = 0; me < npes; ++me) remote.fill(me, 0);
  for (int me = 0; me < npes; ++me) {
    roc_shmemx_set_pe(me);
    for (int i = 0; i < npes; ++i) EXPECT(fetch_inc(remote.ptr, i) <= static_cast<T>(npes), "fetch_inc old");
  }
  for (int me = 0; me < npes; ++me)
    EXPECT(remote.load(me)[0] == static_cast<T>(npes), "fetch_inc: PE %d", me);
  // cxx_test_shmem_atomic_cswap.cpp:73-111: *remote = npes; cswap(cond npes, value me) on the
  // neighbour returns npes and leaves the left-hand neighbour's rank.
  for (int me = 0; me < npes; ++me) remote.fill(me, static_cast<T>(npes));
  roc_shmem_barrier_all();
  for (int me = 0; me < npes; ++me) {
    roc_shmemx_set_pe(me);
    T old = cswap(remote.ptr, static_cast<T>(npes), static_cast<T>(me), (me + 1) % npes);
    EXPECT(old == static_cast<T>(npes), "cswap old: PE %d", me);
  }
  for (int me = 0; me < npes; ++me)
    EXPECT(remote.load(me)[0] == static_cast<T>((me + npes - 1) % npes), "cswap: PE %d", me);
}

static void atomics() {
#define AMO(T, TNAME)                                                                               \
  atomic_add_case<T>("cxx_test_shmem_atomic_add " #TNAME,                                           \
                     [](T *d, T v, int pe) { roc_shmem_##TNAME##_atomic_add(d, v, pe); },           \
                     [](T *d, T v, int pe) { return roc_shmem_##TNAME##_atomic_fetch_add(d, v, pe); }); \
  atomic_add_case<T>(                                                                               \
      "cxx_test_shmem_atomic_add ctx " #TNAME,                                                      \
      [](T *d, T v, int pe) { roc_shmem_ctx_##TNAME##_atomic_add(ROC_SHMEM_CTX_DEFAULT, d, v, pe); }, \
      [](T *d, T v, int pe) {                                                                       \
        return roc_shmem_ctx_##TNAME##_atomic_fetch_add(ROC_SHMEM_CTX_DEFAULT, d, v, pe);           \
      });                                                                                           \
  atomic_fetch_inc_cswap_case<T>(                                                                   \
      "cxx_test_shmem_atomic_fetch/inc/cswap " #TNAME,                                              \
      [](T *d, int pe) { return roc_shmem_##TNAME##_atomic_fetch(d, pe); },                         \
      [](T *d, int pe) { roc_shmem_##TNAME##_atomic_inc(d, pe); },                                  \
      [](T *d, int pe) { return roc_shmem_##TNAME##_atomic_fetch_inc(d, pe); },                     \
      [](T *d, T c, T v, int pe) { return roc_shmem_##TNAME##_atomic_compare_swap(d, c, v, pe); }); \
  atomic_fetch_inc_cswap_case<T>(                                                                   \
      "cxx_test_shmem_atomic_fetch/inc/cswap ctx " #TNAME,                                          \
      [](T *d, int pe) { return roc_shmem_ctx_##TNAME##_atomic_fetch(ROC_SHMEM_CTX_DEFAULT, d, pe); }, \
      [](T *d, int pe) { roc_shmem_ctx_##TNAME##_atomic_inc(ROC_SHMEM_CTX_DEFAULT, d, pe); },       \
      [](T *d, int pe) { return roc_shmem_ctx_##TNAME##_atomic_fetch_inc(ROC_SHMEM_CTX_DEFAULT, d, pe); }, \
      [](T *d, T c, T v, int pe) {                                                                  \
        return roc_shmem_ctx_##TNAME##_atomic_compare_swap(ROC_SHMEM_CTX_DEFAULT, d, c, v, pe);     \
      });
  FOR_AMO_TYPES(AMO)
#undef AMO
}

// clients/sos_tests/atomic_inc.cpp / lfinc.cpp:90-111: `loops` rounds in which every PE
// fetch-increments one counter on PE 0; the values handed out are 0 .. npes*loops-1, each once.
static void lfinc() {
  current_case = "lfinc.cpp / atomic_inc.cpp";
  const int loops = 10;
  Sym<long> counter(1);
  for (int me = 0; me < npes; ++me) counter.fill(me, 0);
  std::vector<int> seen(npes * loops, 0);
  for (int round = 0; round < loops; ++round)
    for (int me = 0; me < npes; ++me) {
      roc_shmemx_set_pe(me);
      long v = roc_shmem_long_atomic_fetch_inc(counter.ptr, 0);
      EXPECT(v >= 0 && v < npes * loops && seen[v]++ == 0, "value %ld handed out twice or out of range", v);
    }
  EXPECT(counter.load(0)[0] == npes * loops, "final count %ld", counter.load(0)[0]);
}

// clients/sos_tests/mt_a2a.cpp:50-118, one thread's view: every PE adds its rank to dest[tid] on
// every PE (sum (npes-1)npes/2), increments flag[tid] everywhere (npes), then puts -1 to its
// neighbour and reads -1 back from every PE.
static void mt_a2a() {
  current_case = "mt_a2a.cpp";
  const int T = 8;
  Sym<long> dest(T), flag(T);
  for (int me = 0; me < npes; ++me) {
    dest.fill(me, 0);
    flag.fill(me, 0);
  }
  for (int me = 0; me < npes; ++me) {
    roc_shmemx_set_pe(me);
    for (int tid = 0; tid < T; ++tid)
      for (int i = 1; i <= npes; ++i) roc_shmem_int64_atomic_add(reinterpret_cast<int64_t *>(&dest.ptr[tid]), me, (me + i) % npes);
  }
  roc_shmem_fence();
  for (int me = 0; me < npes; ++me) {
    roc_shmemx_set_pe(me);
    for (int tid = 0; tid < T; ++tid)
      for (int i = 1; i <= npes; ++i) roc_shmem_int64_atomic_inc(reinterpret_cast<int64_t *>(&flag.ptr[tid]), (me + i) % npes);
  }
  for (int me = 0; me < npes; ++me) {
    std::vector<long> d = dest.load(me), f = flag.load(me);
    for (int tid = 0; tid < T; ++tid)
      EXPECT(d[tid] == (npes - 1) * npes / 2 && f[tid] == npes, "PE %d tid %d: dest %ld flag %ld", me, tid,
             d[tid], f[tid]);
  }
  roc_shmem_barrier_all();
  for (int me = 0; me < npes; ++me) {
    roc_shmemx_set_pe(me);
    long val = -1;
    for (int tid = 0; tid < T; ++tid) roc_shmem_long_put(&dest.ptr[tid], &val, 1, (me + 1) % npes);
  }
  roc_shmem_barrier_all();
  for (int me = 0; me < npes; ++me) {
    roc_shmemx_set_pe(me);
    for (int tid = 0; tid < T; ++tid)
      for (int i = 1; i <= npes; ++i) {
        long val = 0;
        roc_shmem_long_get(&val, &dest.ptr[tid], 1, (me + i) % npes);
        EXPECT(val == -1, "PE %d tid %d from PE %d: %ld", me, tid, (me + i) % npes, val);
      }
  }
}

// ---- broadcast ---------------------------------------------------------------------------------

// clients/sos_tests/bcast.cpp:99-133: ten rounds, 16 bytes growing by 1 KiB each; root 1 of the
// world; src[i] = i + 1 (src[0] stays 0); every PE but the root receives, the root's dst stays 0.
static void bcast() {
  current_case = "bcast.cpp";
  int n_bytes = 16;
  for (int loop = 1; loop <= 10; ++loop) {
    const int n = n_bytes / static_cast<int>(sizeof(long));
    Sym<long> buf(2 * n);
    long *dst = buf.ptr, *src = buf.ptr + n;
    std::vector<long> init(2 * n, 0);
    for (int i = 1; i < n; ++i) init[n + i] = i + 1;
    for (int me = 0; me < npes; ++me) buf.store(me, init);
    roc_shmem_barrier_all();
    roc_shmem_ctx_long_broadcast(ROC_SHMEM_CTX_DEFAULT, dst, src, n, 1, 0, 0, npes, nullptr);
    for (int me = 0; me < npes; ++me) {
      std::vector<long> got = buf.load(me);
      for (int i = 0; i < n; ++i)
        EXPECT(got[i] == (me == 1 ? 0 : init[n + i]), "round %d PE %d dst[%d] = %ld", loop, me, i, got[i]);
    }
    n_bytes += 1024;
  }
}

// clients/sos_tests/bcast_flood.cpp:145-170: back-to-back int broadcasts from root 0 of
// source[i] = i + 1 over target = -90.
static void bcast_flood() {
  current_case = "bcast_flood.cpp";
  const int elements = 4096, loops = 20;
  Sym<int> source(elements), target(elements);
  std::vector<int> pattern(elements);
  for (int i = 0; i < elements; ++i) pattern[i] = i + 1;
  for (int me = 0; me < npes; ++me) {
    source.store(me, pattern);
    target.fill(me, -90);
  }
  roc_shmem_barrier_all();
  for (int i = 0; i < loops; ++i)
    roc_shmem_ctx_int_broadcast(ROC_SHMEM_CTX_DEFAULT, target.ptr, source.ptr, elements, 0, 0, 0, npes, nullptr);
  roc_shmem_barrier_all();
  for (int me = 0; me < npes; ++me) {
    std::vector<int> got = target.load(me);
    for (int i = 0; i < elements; ++i)
      EXPECT(got[i] == (me == 0 ? -90 : i + 1), "PE %d target[%d] = %d", me, i, got[i]);
  }
}

// clients/sos_tests/broadcast_active_set.cpp:84-128: the active set shrinks from the front
// (PE_start = i, size = npes - i) and the root is its first member; members other than the root
// receive the root's value, everybody else keeps what it had.
static void broadcast_active_set() {
  current_case = "broadcast_active_set.cpp";
  const int N = 8;
  Sym<long> src(N), dst(N);
  for (int start = 0; start < npes; ++start) {
    for (int me = 0; me < npes; ++me) {
      src.fill(me, me + 100);
      dst.fill(me, -1);
    }
    roc_shmem_barrier_all();
    roc_shmem_ctx_long_broadcast(ROC_SHMEM_CTX_DEFAULT, dst.ptr, src.ptr, N, 0, start, 0, npes - start, nullptr);
    for (int me = 0; me < npes; ++me) {
      std::vector<long> got = dst.load(me);
      const long want = me > start ? start + 100 : -1;
      for (int i = 0; i < N; ++i) EXPECT(got[i] == want, "start %d PE %d [%d] = %ld", start, me, i, got[i]);
    }
  }
}

// ---- point-to-point synchronisation ---------------------------------------------------------

// clients/sos_tests/cxx_test_shmem_wait_until.cpp:42-60 and cxx_test_shmem_test.cpp:42-61: every PE
// puts (TYPE)me + 1 into its right-hand neighbour and waits on its own copy for a value other
// than zero, which must be that of its left-hand neighbour.  In one process all puts are made
// first; each PE's wait then finds its condition already true.
template <typename T, typename P, typename W, typename Tst>
static void wait_case(const char *name, P p, W wait_until, Tst test) {
  current_case = name;
  Sym<T> remote(1);
  for (int use_test = 0; use_test < 2; ++use_test) {
    for (int me = 0; me < npes; ++me) remote.fill(me, 0);
    roc_shmemx_set_pe(0);
    EXPECT(test(remote.ptr, ROC_SHMEM_CMP_NE, static_cast<T>(0)) == 0, "test true before any put");
    EXPECT(test(remote.ptr, ROC_SHMEM_CMP_EQ, static_cast<T>(0)) == 1, "test of the initial value");
    for (int me = 0; me < npes; ++me) {
      roc_shmemx_set_pe(me);
      p(remote.ptr, static_cast<T>(static_cast<T>(me) + 1), (me + 1) % npes);
    }
    for (int me = 0; me < npes; ++me) {
      roc_shmemx_set_pe(me);
      if (use_test) {
        int spins = 0;
        while (!test(remote.ptr, ROC_SHMEM_CMP_NE, static_cast<T>(0)) && ++spins < 1000000) {
        }
        EXPECT(spins < 1000000, "test never became true on PE %d", me);
      } else {
        wait_until(remote.ptr, ROC_SHMEM_CMP_NE, static_cast<T>(0));
      }
      const T want = static_cast<T>(static_cast<T>((me + npes - 1) % npes) + 1);
      EXPECT(remote.load(me)[0] == want, "PE %d holds the wrong value", me);
      // the remaining comparisons, on the value that is there now
      EXPECT(test(remote.ptr, ROC_SHMEM_CMP_EQ, want) == 1, "EQ on PE %d", me);
      EXPECT(test(remote.ptr, ROC_SHMEM_CMP_GE, want) == 1, "GE on PE %d", me);
      EXPECT(test(remote.ptr, ROC_SHMEM_CMP_LE, want) == 1, "LE on PE %d", me);
      EXPECT(test(remote.ptr, ROC_SHMEM_CMP_GT, want) == 0, "GT on PE %d", me);
      EXPECT(test(remote.ptr, ROC_SHMEM_CMP_LT, static_cast<T>(want + 1)) == 1, "LT on PE %d", me);
    }
  }
}

static void wait_until_and_test() {
#define WAIT_CASE(T, TNAME)                                                                    \
  wait_case<T>("cxx_test_shmem_wait_until.cpp / cxx_test_shmem_test.cpp " #TNAME,              \
               [](T *d, T v, int pe) { roc_shmem_##TNAME##_p(d, v, pe); },                      \
               [](T *ptr, roc_shmem_cmps c, T v) { roc_shmem_##TNAME##_wait_until(ptr, c, v); }, \
               [](T *ptr, roc_shmem_cmps c, T v) { return roc_shmem_##TNAME##_test(ptr, c, v); });
  WAIT_CASE(short, short)
  WAIT_CASE(int, int)
  WAIT_CASE(long, long)
  WAIT_CASE(long long, longlong)
  WAIT_CASE(unsigned short, ushort)
  WAIT_CASE(unsigned int, uint)
  WAIT_CASE(unsigned long, ulong)
  WAIT_CASE(unsigned long long, ulonglong)
#undef WAIT_CASE
}

// clients/sos_tests/waituntil.cpp:58-137: PE 0 clears `target` everywhere, puts 1..10 into every
// other PE, waits for pong > 666 (PE 1 sets it to 999 once its target[9] reads 10) and then puts
// 0xDD into t2[9] of the others, which wait for it.  The steps run here in an order in which every
// wait finds its condition met by a put made earlier.
static void waituntil() {
  current_case = "waituntil.cpp";
  long source[10] = {1, 2, 3, 4, 5, 6, 7, 8, 9, 10};
  Sym<long> target(10), pong(1), t2(10);
  for (int me = 0; me < npes; ++me) {
    pong.fill(me, 666);
    target.fill(me, 0xFF);
    t2.fill(me, 0xFF);
  }
  roc_shmem_barrier_all();
  roc_shmemx_set_pe(0);
  long zeros[10] = {0};
  for (int pe = 1; pe < npes; ++pe) roc_shmem_long_put(target.ptr, zeros, 10, pe);
  for (int pe = 1; pe < npes; ++pe) roc_shmem_long_put(target.ptr, source, 10, pe);
  for (int me = 1; me < npes; ++me) {
    roc_shmemx_set_pe(me);
    roc_shmem_long_wait_until(&target.ptr[9], ROC_SHMEM_CMP_NE, 0xFF);
    roc_shmem_long_wait_until(&target.ptr[9], ROC_SHMEM_CMP_EQ, 10);
    if (me == 1) {
      EXPECT(roc_shmem_long_g(pong.ptr, 0) == 666, "pong on PE 0 before the reply");
      roc_shmem_long_p(pong.ptr, 999, 0);
    }
  }
  roc_shmemx_set_pe(0);
  roc_shmem_long_wait_until(pong.ptr, ROC_SHMEM_CMP_GT, 666);
  EXPECT(pong.load(0)[0] == 999, "pong on PE 0 = %ld", pong.load(0)[0]);
  for (int pe = 1; pe < npes; ++pe) roc_shmem_long_p(&t2.ptr[9], 0xDD, pe);
  for (int me = 1; me < npes; ++me) {
    roc_shmemx_set_pe(me);
    roc_shmem_long_wait_until(&t2.ptr[9], ROC_SHMEM_CMP_NE, 0xFF);
    EXPECT(t2.load(me)[9] == 0xDD, "t2[9] on PE %d = %ld", me, t2.load(me)[9]);
    std::vector<long> got = target.load(me);
    for (int i = 0; i < 10; ++i) EXPECT(got[i] == i + 1, "target[%d] on PE %d = %ld", i, me, got[i]);
  }
  EXPECT(t2.load(0)[9] == 0xFF, "PE 0's own t2 was written");
}

// ---- small programs -------------------------------------------------------------------------

// clients/sos_tests/circular_shift.cpp:38-62: every PE stores its rank and gets its right-hand
// neighbour's; get1.cpp:44-80: PE 0 gets ten longs i + 1 from PE 1.
static void circular_shift_and_get1() {
  current_case = "circular_shift.cpp";
  Sym<int> bbb(1);
  for (int me = 0; me < npes; ++me) bbb.fill(me, me);
  roc_shmem_barrier_all();
  for (int me = 0; me < npes; ++me) {
    roc_shmemx_set_pe(me);
    const int neighbor = (me + 1) % npes;
    int aaa = -1;
    roc_shmem_int_get(&aaa, bbb.ptr, 1, neighbor);
    EXPECT(aaa == neighbor, "PE %d got %d from PE %d", me, aaa, neighbor);
  }
  current_case = "get1.cpp";
  Sym<long> source(10);
  std::vector<long> pattern(10);
  for (int i = 0; i < 10; ++i) pattern[i] = i + 1;
  for (int me = 0; me < npes; ++me) source.store(me, pattern);
  roc_shmem_barrier_all();
  roc_shmemx_set_pe(0);
  long target[10] = {0};
  roc_shmem_long_get(target, source.ptr, 10, 1);
  roc_shmem_barrier_all();
  EXPECT(memcmp(target, pattern.data(), sizeof(target)) == 0, "source and target differ");
}

// clients/sos_tests/pi.cpp:40-110: every PE counts the random points that fall inside the unit
// circle; PE 0 gets and adds the others' counters.  The reference checks |pi - estimate| < 0.1;
// here the gathered totals are also compared with the counts made on the host.
static void pi() {
  current_case = "pi.cpp";
  const long long points = 10000;
  Sym<long long> inside(1), total(1);
  long long want_inside = 0;
  for (int me = 0; me < npes; ++me) {
    srand(1 + me);
    long long in = 0;
    for (long long t = 0; t < points; ++t) {
      const double x = rand() / static_cast<double>(RAND_MAX), y = rand() / static_cast<double>(RAND_MAX);
      if (x * x + y * y < 1) ++in;
    }
    inside.fill(me, in);
    total.fill(me, points);
    want_inside += in;
  }
  roc_shmem_barrier_all();
  roc_shmemx_set_pe(0);
  long long sum_inside = inside.load(0)[0], sum_total = total.load(0)[0];
  for (int i = 1; i < npes; ++i) {
    long long remote_inside = 0, remote_total = 0;
    roc_shmem_longlong_get(&remote_inside, inside.ptr, 1, i);
    roc_shmem_longlong_get(&remote_total, total.ptr, 1, i);
    sum_inside += remote_inside;
    sum_total += remote_total;
  }
  EXPECT(sum_total == points * npes && sum_inside == want_inside, "gathered %lld of %lld", sum_inside, sum_total);
  const double approx = 4.0 * sum_inside / static_cast<double>(sum_total);
  EXPECT(approx > 3.04 && approx < 3.25, "pi estimate %f", approx);
}

// clients/sos_tests/many-ctx.cpp:36-80: every PE creates NUM_CTX contexts and increments a
// counter on its right-hand neighbour once through each; after quiet on every context and
// sync_all each counter holds NUM_CTX.
static void many_ctx() {
  current_case = "many-ctx.cpp";
  const int kNumCtx = 32;
  Sym<int64_t> data(1);
  for (int me = 0; me < npes; ++me) data.fill(me, 0);
  roc_shmem_barrier_all();
  for (int me = 0; me < npes; ++me) {
    roc_shmemx_set_pe(me);
    roc_shmem_ctx_t ctx[kNumCtx];
    for (int i = 0; i < kNumCtx; ++i) {
      if (roc_shmem_ctx_create(0, &ctx[i]) != 0) ctx[i] = ROC_SHMEM_CTX_DEFAULT;  // as the reference does
    }
    for (int i = 0; i < kNumCtx; ++i) roc_shmem_ctx_int64_atomic_inc(ctx[i], data.ptr, (me + 1) % npes);
    for (int i = 0; i < kNumCtx; ++i) roc_shmem_ctx_quiet(ctx[i]);
    for (int i = 0; i < kNumCtx; ++i)
      if (ctx[i].ctx_opaque != ROC_SHMEM_CTX_DEFAULT.ctx_opaque) roc_shmem_ctx_destroy(ctx[i]);
  }
  roc_shmem_sync_all();
  for (int me = 0; me < npes; ++me)
    EXPECT(data.load(me)[0] == kNumCtx, "PE %d counted %ld", me, static_cast<long>(data.load(me)[0]));
}

// ---- teams ------------------------------------------------------------------------------------

// clients/sos_tests/shmem_team_b2b_collectives.cpp:68-100: NITERS back-to-back broadcasts and then
// reductions on the world team with src = me, no barrier in between; the last results must be
// those of a single call.
static void team_b2b_collectives() {
  current_case = "shmem_team_b2b_collectives.cpp";
  const int kIters = 100, kElems = 10;
  Sym<long> dest(kElems), src(kElems);
  for (int me = 0; me < npes; ++me) {
    src.fill(me, me);
    dest.fill(me, -7);
  }
  for (int i = 0; i < kIters; ++i)
    roc_shmem_ctx_long_broadcast(ROC_SHMEM_CTX_DEFAULT, ROC_SHMEM_TEAM_WORLD, dest.ptr, src.ptr, kElems, 0);
  for (int me = 0; me < npes; ++me)
    for (long x : dest.load(me)) EXPECT(x == (me == 0 ? -7 : 0), "broadcast: PE %d holds %ld", me, x);
  for (int i = 0; i < kIters; ++i)
    roc_shmem_ctx_long_sum_to_all(ROC_SHMEM_CTX_DEFAULT, ROC_SHMEM_TEAM_WORLD, dest.ptr, src.ptr, kElems);
  const long want = static_cast<long>(npes) * (npes - 1) / 2;
  for (int me = 0; me < npes; ++me)
    for (long x : dest.load(me)) EXPECT(x == want, "reduce: PE %d holds %ld", me, x);
}

// clients/sos_tests/shmem_team_reuse_teams.cpp:35-75: npes - 1 rounds in which the team loses its
// first member (split (1, 1, n - 1) of the previous team) and the previous team is destroyed.
static void team_reuse_teams() {
  current_case = "shmem_team_reuse_teams.cpp";
  roc_shmem_team_t old_team, new_team;
  int ret = roc_shmem_team_split_strided(ROC_SHMEM_TEAM_WORLD, 0, 1, npes, nullptr, 0, &old_team);
  EXPECT(ret == 0, "first split returned %d", ret);
  for (int i = 1; i < npes; ++i) {
    EXPECT(roc_shmem_team_translate_pe(old_team, 1, ROC_SHMEM_TEAM_WORLD) == i,
           "round %d: second member is world PE %d", i,
           roc_shmem_team_translate_pe(old_team, 1, ROC_SHMEM_TEAM_WORLD));
    const int size = roc_shmem_team_n_pes(old_team);
    EXPECT(size == npes - i + 1, "round %d: team of %d", i, size);
    ret = roc_shmem_team_split_strided(old_team, 1, 1, size - 1, nullptr, 0, &new_team);
    EXPECT(ret == 0 && new_team != ROC_SHMEM_TEAM_INVALID, "round %d: split returned %d", i, ret);
    roc_shmem_team_destroy(old_team);
    old_team = new_team;
  }
  EXPECT(roc_shmem_team_n_pes(old_team) == 1, "last team has %d members", roc_shmem_team_n_pes(old_team));
  EXPECT(roc_shmem_team_translate_pe(old_team, 0, ROC_SHMEM_TEAM_WORLD) == npes - 1, "last team's member");
  roc_shmem_team_destroy(old_team);
}

// clients/sos_tests/shmem_team_translate.cpp:40-93: teams of every second and every third PE; a PE
// is in team_2s iff me % 2 == 0 and in team_3s iff me % 3 == 0, and its rank translates from one
// team to the other iff it is in both.  Beyond the reference's checks: the ranks themselves, and a
// sum reduction and a broadcast over the team of stride 3.
static void team_translate() {
  current_case = "shmem_team_translate.cpp";
  roc_shmem_team_t team_2s, team_3s;
  int ret = roc_shmem_team_split_strided(ROC_SHMEM_TEAM_WORLD, 0, 2, (npes - 1) / 2 + 1, nullptr, 0, &team_2s);
  EXPECT(ret == 0 && team_2s != ROC_SHMEM_TEAM_INVALID, "split of stride 2 returned %d", ret);
  ret = roc_shmem_team_split_strided(ROC_SHMEM_TEAM_WORLD, 0, 3, (npes - 1) / 3 + 1, nullptr, 0, &team_3s);
  EXPECT(ret == 0 && team_3s != ROC_SHMEM_TEAM_INVALID, "split of stride 3 returned %d", ret);
  if (team_2s == ROC_SHMEM_TEAM_INVALID || team_3s == ROC_SHMEM_TEAM_INVALID) return;
  for (int me = 0; me < npes; ++me) {
    roc_shmemx_set_pe(me);
    const int t_pe_3 = roc_shmem_team_my_pe(team_3s), t_pe_2 = roc_shmem_team_my_pe(team_2s);
    const int t_pe_3_to_2 = roc_shmem_team_translate_pe(team_3s, t_pe_3, team_2s);
    const int t_pe_2_to_3 = roc_shmem_team_translate_pe(team_2s, t_pe_2, team_3s);
    const bool in2 = me % 2 == 0, in3 = me % 3 == 0;
    EXPECT((t_pe_2 != -1) == in2 && (t_pe_3 != -1) == in3 && (t_pe_2_to_3 != -1) == (in2 && in3) &&
               (t_pe_3_to_2 != -1) == (in2 && in3),
           "PE %d: t_pe_2=%d t_pe_3=%d t_pe_3_to_2=%d t_pe_2_to_3=%d", me, t_pe_2, t_pe_3, t_pe_3_to_2,
           t_pe_2_to_3);
    if (in2) EXPECT(t_pe_2 == me / 2, "PE %d is member %d of team_2s", me, t_pe_2);
    if (in3) EXPECT(t_pe_3 == me / 3, "PE %d is member %d of team_3s", me, t_pe_3);
    if (in2 && in3)
      EXPECT(t_pe_3_to_2 == me / 2 && t_pe_2_to_3 == me / 3, "PE %d translates to %d and %d", me,
             t_pe_3_to_2, t_pe_2_to_3);
  }
  roc_shmemx_set_pe(0);
  const int N = 1000, members = (npes - 1) / 3 + 1;
  Sym<int> src(N), dst(N);
  for (int me = 0; me < npes; ++me) {
    std::vector<int> v(N);
    for (int i = 0; i < N; ++i) v[i] = (me + 1) * 1000 + i;
    src.store(me, v);
    dst.fill(me, -7);
  }
  roc_shmem_ctx_int_sum_to_all(ROC_SHMEM_CTX_DEFAULT, team_3s, dst.ptr, src.ptr, N);
  for (int me = 0; me < npes; ++me) {
    std::vector<int> got = dst.load(me);
    for (int i = 0; i < N; ++i) {
      int want = -7;
      if (me % 3 == 0) {
        want = 0;
        for (int k = 0; k < members; ++k) want += (3 * k + 1) * 1000 + i;
      }
      EXPECT(got[i] == want, "sum over team_3s: PE %d [%d] = %d, expected %d", me, i, got[i], want);
    }
    dst.fill(me, -7);
  }
  // root = last member of the team
  roc_shmem_ctx_int_broadcast(ROC_SHMEM_CTX_DEFAULT, team_3s, dst.ptr, src.ptr, N, members - 1);
  for (int me = 0; me < npes; ++me) {
    std::vector<int> got = dst.load(me);
    const int root_world = 3 * (members - 1);
    for (int i = 0; i < N; ++i) {
      const int want = (me % 3 == 0 && me != root_world) ? (root_world + 1) * 1000 + i : -7;
      EXPECT(got[i] == want, "broadcast over team_3s: PE %d [%d] = %d, expected %d", me, i, got[i], want);
    }
  }
  roc_shmem_team_destroy(team_3s);
  roc_shmem_team_destroy(team_2s);
}

// clients/sos_tests/barrier.cpp:92-103: thirty barrier_all calls in a row.
static void barrier_loop() {
  current_case = "barrier.cpp";
  for (int j = 0; j < 30; ++j) roc_shmem_barrier_all();
  EXPECT(roc_shmemx_take_status() == 0, "status word raised by thirty barriers");
}

// clients/sos_tests/shmem_test.cpp:38-75: every PE puts mype + 1 into wait_vars[mype] of every PE;
// each PE then polls the array with roc_shmem_long_test(!= 0) until it has seen npes messages,
// checks wait_vars[who] == who + 1 and clears the entry.
static void shmem_test_any() {
  current_case = "shmem_test.cpp";
  Sym<long> wait_vars(npes);
  for (int me = 0; me < npes; ++me) wait_vars.fill(me, 0);
  for (int me = 0; me < npes; ++me) {
    roc_shmemx_set_pe(me);
    for (int i = 0; i < npes; ++i) roc_shmem_long_p(&wait_vars.ptr[me], me + 1, i);
  }
  for (int me = 0; me < npes; ++me) {
    roc_shmemx_set_pe(me);
    int nrecv = 0, idx = 0, polls = 0;
    while (nrecv < npes && polls < 100 * npes) {
      ++polls;
      if (!roc_shmem_long_test(&wait_vars.ptr[idx], ROC_SHMEM_CMP_NE, 0)) {
        idx = (idx + 1) % npes;
        continue;
      }
      const long got = roc_shmem_long_g(&wait_vars.ptr[idx], me);
      EXPECT(got == idx + 1, "PE %d: wait_vars[%d] = %ld, expected %d", me, idx, got, idx + 1);
      roc_shmem_long_p(&wait_vars.ptr[idx], 0, me);
      ++nrecv;
    }
    EXPECT(nrecv == npes, "PE %d saw %d of %d messages", me, nrecv, npes);
  }
  roc_shmemx_set_pe(0);
}

int main() {
  if (!getenv("ROC_SHMEM_NUM_PES")) setenv("ROC_SHMEM_NUM_PES", "6", 1);
  setenv("ROC_SHMEM_HEAP_SIZE", "134217728", 0);
  roc_shmem_init();
  npes = roc_shmem_n_pes();
  struct {
    const char *name;
    void (*run)();
  } cases[] = {{"to_all", to_all_cases},
               {"max_reduction", max_reduction},
               {"big_reduction", big_and_in_place_reduction},
               {"reduce_active_set", reduce_active_set},
               {"team_reduce", team_reduce},
               {"put1", put1},
               {"get_nbi", get_nbi_put_nbi},
               {"bigput", bigput_bigget},
               {"p_g", p_and_g},
               {"atomics", atomics},
               {"lfinc", lfinc},
               {"mt_a2a", mt_a2a},
               {"bcast", bcast},
               {"bcast_flood", bcast_flood},
               {"broadcast_active_set", broadcast_active_set},
               {"wait_until_and_test", wait_until_and_test},
               {"waituntil", waituntil},
               {"circular_shift_get1", circular_shift_and_get1},
               {"pi", pi},
               {"many_ctx", many_ctx},
               {"team_b2b_collectives", team_b2b_collectives},
               {"team_reuse_teams", team_reuse_teams},
               {"team_translate", team_translate},
               {"barrier", barrier_loop},
               {"shmem_test", shmem_test_any}};
  for (auto &c : cases) {
    const int before = failures;
    c.run();
    roc_shmemx_set_pe(0);
    EXPECT(roc_shmemx_take_status() == 0, "device status word raised");
    printf("%-22s %s\n", c.name, failures == before ? "ok" : "FAILED");
    fflush(stdout);
  }
  roc_shmem_finalize();
  if (failures) {
    printf("SOS_CASES_FAILED %d\n", failures);
    return 1;
  }
  printf("SOS_CASES_OK\n");
  return 0;
}
