// Eight host threads on ONE context of libacchip's host code, built under ThreadSanitizer against the stand-in HIP
// runtime of mock_hip.cpp: what include/acc_hip.h promises ("every entry point may be called from any thread; one
// acc_skel may be executed from several threads") exercised where data races would sit -- the scratch pool (acquire,
// release, trim, blocks of several protocols and sizes), the lazily built second variant of a shared instance,
// instances created and destroyed while others run, the ordering of big scans across streams, guards set on and
// taken off streams, the status block, the memory table, the launch trace; a segmented fold that goes over to its
// variants with a table of jobs while it is being launched; instances whose compilation runs on the
// library's worker pool, used, waited for, polled and destroyed while it runs; a context's tuning table replaced
// while instances are created, and a thread that keeps changing the environment meanwhile (no driver call reads
// it).  Launches do nothing here; the checks are ThreadSanitizer's.  Exit status 0 and no report = pass.
#include <atomic>
#include <cstdio>
#include <cstdlib>
#include <cstring>
#include <thread>
#include <vector>

#include "../../include/acc_hip.h"

extern "C" long mock_hip_launches(void);
extern "C" void mock_hip_probe_finds(int argument);
extern "C" long mock_hip_sweeps(void);

#define OK(call)                                                                        \
  do {                                                                                  \
    int rc__ = (call);                                                                  \
    if (rc__ != ACC_OK) {                                                               \
      std::fprintf(stderr, "%s:%d: %s -> %d: %s\n", __FILE__, __LINE__, #call, rc__, acc_last_error()); \
      std::exit(2);                                                                     \
    }                                                                                   \
  } while (0)

static acc_array vec(uint64_t p, int64_t n)
{
  acc_array a;
  std::memset(&a, 0, sizeof(a));
  a.rank = 1;
  a.ncomp = 1;
  a.shape[0] = n;
  a.ptr[0] = p;
  return a;
}

static acc_skel make(acc_context ctx, int kind, const char *elt, const char *get, const char *combine, const char *seed,
                     const char *permutation, int hint, uint32_t flags, bool in_background = false)
{
  acc_env_sig env[1];
  std::memset(env, 0, sizeof(env));
  env[0].rank = 1;
  env[0].ncomp = 1;
  env[0].type[0] = "Int32";
  acc_skel_desc d;
  std::memset(&d, 0, sizeof(d));
  d.kind = kind;
  d.flags = flags;
  d.n_env = 1;
  d.env = env;
  d.elt_type = elt;
  d.out_rank = (kind == ACC_SKEL_FOLD) ? 0 : 1;
  d.get = get;
  d.combine = combine;
  d.seed = seed;
  d.permutation = permutation;
  d.combine_hint = hint;
  acc_skel s = nullptr;
  if (in_background) OK(acc_skel_create_async(ctx, &d, &s));
  else OK(acc_skel_create(ctx, &d, &s));
  return s;
}

int main(int argc, char **argv)
{
  const int threads = argc > 1 ? std::atoi(argv[1]) : 8, rounds = argc > 2 ? std::atoi(argv[2]) : 150;
  OK(acc_init());
  OK(acc_cache_set_dir(""));
  acc_context ctx = nullptr;
  OK(acc_context_create(0, &ctx));

  // shared instances
  acc_skel scan = make(ctx, ACC_SKEL_SCANL1, "Int32", "arrIn0_0[ix]", "x + y", nullptr, nullptr, 0, 0);
  acc_skel fold = make(ctx, ACC_SKEL_FOLD, "Int32", "arrIn0_0[ix]", "x + y", "0", nullptr, 0, 0);
  acc_skel hist = make(ctx, ACC_SKEL_PERMUTE, "Int32", "1", "x + y", nullptr, "arrIn0_0[ix]", ACC_COMBINE_ADD, 0);
  acc_skel locked = make(ctx, ACC_SKEL_PERMUTE, "Int16", "(Int16)1", "(Int16)(x + y)", nullptr, "arrIn0_0[ix]", 0, 0);
  // `permute const` (stores: a kernel of its own for the small element, the atomics template for the 4-byte one) and a
  // fold along the innermost dimension that gives a row to a lane (pieces in scratch memory where the rows are few)
  acc_skel scatter16 = make(ctx, ACC_SKEL_PERMUTE, "Int16", "(Int16)ix", "x", nullptr, "arrIn0_0[ix]", 0, 0);
  acc_skel scatter32 = make(ctx, ACC_SKEL_PERMUTE, "Int32", "(Int32)ix", "( x )", nullptr, "arrIn0_0[ix]", 0, 0);
  acc_skel across = make(ctx, ACC_SKEL_FOLD1, "Int32", "arrIn0_0[ix]", "x + y", nullptr, nullptr, 0, ACC_FLAG_TILED);
  acc_skel gmap = make(ctx, ACC_SKEL_MAP, "Int32", "arrIn0_0[ix] + 1", nullptr, nullptr, nullptr, 0, ACC_FLAG_GUARDED);
  acc_skel segs = make(ctx, ACC_SKEL_FOLDSEG, "Int32", "arrIn0_0[ix]", "x + y", "0", nullptr, 0, 0);
  acc_memtable table = nullptr;
  OK(acc_memtable_create(ctx, 0, &table));

  const int64_t n_max = int64_t(1) << 24;
  acc_devptr in = 0, out = 0, bins = 0, zeros = 0;
  OK(acc_malloc(ctx, (size_t)(n_max + 4) * 4, &in));
  OK(acc_malloc(ctx, (size_t)(n_max + 4) * 4, &out));
  OK(acc_malloc(ctx, (size_t)(1 << 20) * 4, &bins));
  OK(acc_malloc(ctx, (size_t)(1 << 20) * 4, &zeros));

  std::atomic<int> failures{0};
  std::vector<std::thread> pool;
  for (int t = 0; t < threads; ++t) {
    pool.emplace_back([&, t] {
      acc_stream st = nullptr;
      OK(acc_stream_create(ctx, &st));
      acc_guard guard = nullptr;
      OK(acc_guard_create(ctx, &guard));
      std::vector<char> host(1 << 16);
      for (int r = 0; r < rounds; ++r) {
        // sizes from one tile to thousands of them: small and big scans (the big ones are chained across streams),
        // folds with and without a second workgroup, so that scratch blocks of several sizes and protocols come and go
        const int64_t n = (r % 5 == 0) ? n_max : (int64_t(1) << (10 + (r * 7 + t * 3) % 12)) + t;
        // an unaligned operand every few rounds: the second variant of the shared instances is built on first need
        const uint64_t off = (r % 7 == 3) ? 4 : 0;
        acc_array a = vec(in + off, n), o = vec(out + off, n), total = vec(out, 1);
        total.rank = 0;
        OK(acc_exec_scan(scan, &a, n, &o, nullptr, st));
        OK(acc_exec_fold(fold, &a, 1, &n, &total, st));
        const int64_t nb = (r % 3 == 0) ? 256 : ((r % 3 == 1) ? 65536 : 200000);
        acc_array d = vec(zeros, nb), b = vec(bins, nb);
        OK(acc_exec_permute(hist, &a, n, &d, &b, st));
        {
          // a segmented fold, segments short or long on average; from a third of the way on its look at the segment
          // lengths "finds" a very long one (mock_hip.cpp), and the instance goes over to its variants with a table of
          // jobs -- compiled in the background, taken when they are there -- while all threads keep launching it
          if (t == 0 && r == rounds / 3) mock_hip_probe_finds(6);      // env (extent, pointer), result (extent, pointer), source extent, offsets: the word comes 7th
          const int64_t nseg = (r % 2 == 0) ? n / 8 + 1 : n / 700 + 1;
          acc_array offs = vec(in, nseg + 1), sums = vec(out, nseg);
          OK(acc_exec_foldseg(segs, &a, n, &offs, &sums, st));
        }
        if (r % 4 == 1) {
          acc_array d16 = vec(zeros, 3000), b16 = vec(bins, 3000), few = vec(in, 2000);
          OK(acc_exec_permute(locked, &few, 2000, &d16, &b16, st));
        }
        if (r % 5 == 2) {
          acc_array d16 = vec(zeros, 3000), b16 = vec(bins, 3000), few = vec(in, 2000);
          OK(acc_exec_permute(scatter16, &few, 2000, &d16, &b16, st));
          acc_array d32 = vec(zeros, 5000), b32 = vec(out, 5000);
          OK(acc_exec_permute(scatter32, &few, 2000, &d32, &b32, st));
          const int64_t few_rows[2] = {7, 3000}, many_rows[2] = {3000, 40};
          acc_array r7 = vec(out, 7), r3000 = vec(out, 3000);
          OK(acc_exec_fold(across, &a, 2, few_rows, &r7, st));
          OK(acc_exec_fold(across, &a, 2, many_rows, &r3000, st));
        }
        if (r % 6 == 2) {                       // a loop's kernels on this thread's stream, under its guard
          OK(acc_stream_set_guard(ctx, st, guard));
          OK(acc_guard_reset(guard, st));
          acc_array m = vec(out, 1000), mi = vec(in, 1000);
          OK(acc_exec_map(gmap, &mi, &m, st));
          int32_t alive = 0;
          int64_t count = 0;
          OK(acc_guard_read(guard, st, &alive, &count));
          OK(acc_stream_set_guard(ctx, st, nullptr));
        }
        if (r % 9 == 4) {                       // instances of this thread's own come and go
          acc_skel mine = make(ctx, ACC_SKEL_SCANL, "Int32", "arrIn0_0[ix] * 2", "x + y", "0", nullptr, 0, 0);
          acc_array o1 = vec(out, 1001), a1 = vec(in, 1000);
          OK(acc_exec_scan(mine, &a1, 1000, &o1, nullptr, st));
          acc_skel_info info;
          OK(acc_skel_get_info(mine, &info));
          OK(acc_skel_destroy(mine));
        }
        if (r % 10 == 3) {                      // compiled on the worker pool: used at once, or polled, or dropped while it compiles
          static const char *bodies[] = {"arrIn0_0[ix] * 3", "arrIn0_0[ix] - 7", "arrIn0_0[ix] ^ 5", "arrIn0_0[ix] + 11"};
          acc_skel bg = make(ctx, ACC_SKEL_MAP, "Int32", bodies[(r / 10 + t) % 4], nullptr, nullptr, nullptr, 0, 0, true);
          if ((r / 10) % 3 == 0) {
            acc_array m = vec(out, 1000), mi = vec(in, 1000);
            OK(acc_exec_map(bg, &mi, &m, st));            // the first use waits for the compilation
          } else if ((r / 10) % 3 == 1) {
            int ready = 0;
            OK(acc_skel_poll(bg, &ready));
            OK(acc_skel_wait(bg));
            OK(acc_skel_poll(bg, &ready));
            if (!ready) failures.fetch_add(1);
          }
          OK(acc_skel_destroy(bg));                       // ... possibly while it still compiles
        }
        if (r % 17 == 9 && t == 0) OK(acc_context_set_tuning(ctx, (r & 1) ? "map.oversub=4" : ""));
        if (r % 11 == 5) {                      // the pool gives back what is not lent, while the others borrow
          size_t freed = 0, held = 0;
          OK(acc_context_trim(ctx, &freed));
          OK(acc_context_scratch_bytes(ctx, &held));
        }
        if (r % 5 == 2) {                       // an array of the memory table, keyed by this thread and round
          const uint64_t key = (uint64_t(t) << 32) | uint64_t(r);
          int is_new = 0;
          acc_devptr p = 0;
          OK(acc_memtable_malloc(table, key, host.data(), host.size(), 1, &is_new));
          OK(acc_memtable_acquire(table, key, st, &p));
          OK(acc_memtable_release(table, key, st));
          OK(acc_memtable_free(table, key));
        }
        if (r % 25 == 8) {                      // copies large enough to be staged through the context's pinned buffers
          static thread_local std::vector<char> big(9u << 20, 1);
          OK(acc_memcpy_h2d(ctx, in, big.data(), big.size()));
          OK(acc_memcpy_d2h(ctx, big.data(), in, big.size()));
          const uint64_t key = (uint64_t(t) << 32) | uint64_t(r) | (1ull << 60);
          int is_new = 0;
          acc_devptr p = 0;
          OK(acc_memtable_malloc(table, key, big.data(), big.size(), 1, &is_new));
          OK(acc_memtable_acquire(table, key, st, &p));
          OK(acc_memtable_release(table, key, st));
          OK(acc_memtable_free(table, key));
        }
        if (r % 13 == 6) {
          OK(acc_trace_start(ctx));
          acc_array o2 = vec(out, 5000), a2 = vec(in, 5000);
          OK(acc_exec_scan(scan, &a2, 5000, &o2, nullptr, st));
          int32_t launches = 0;
          double ms = 0;
          OK(acc_trace_stop(ctx, &launches, &ms));
          if (launches != 1) failures.fetch_add(1);
        }
        if (r % 8 == 7) OK(acc_stream_sync(ctx, st));
      }
      OK(acc_stream_sync(ctx, st));
      OK(acc_guard_destroy(guard));
      OK(acc_stream_destroy(ctx, st));
    });
  }
  for (std::thread &th : pool) th.join();
  {
    // Driver calls while another thread keeps changing the environment: nothing on their path may read it.  (Only
    // calls whose variants exist by now: a compilation reads the environment inside the compiler's own library.)
    std::atomic<bool> stop_env{false};
    std::thread env_thread([&] {
      for (int k = 0; !stop_env.load(); ++k) {
        setenv("ACC_HIP_TUNE", (k & 1) ? "scan.rows=2" : "fold.unroll=2,map.unroll=2", 1);
        setenv("ACC_HIP_DEBUG", (k & 1) ? "" : "dump-exec", 1);
        std::this_thread::yield();
      }
    });
    std::vector<std::thread> callers;
    for (int t = 0; t < threads; ++t) {
      callers.emplace_back([&, t] {
        acc_stream st = nullptr;
        OK(acc_stream_create(ctx, &st));
        for (int r = 0; r < rounds; ++r) {
          const int64_t n = (int64_t(1) << (10 + (r * 7 + t * 3) % 12)) + t;
          const uint64_t off = (r % 7 == 3) ? 4 : 0;
          acc_array a = vec(in + off, n), o = vec(out + off, n), total = vec(out, 1);
          total.rank = 0;
          OK(acc_exec_scan(scan, &a, n, &o, nullptr, st));
          OK(acc_exec_fold(fold, &a, 1, &n, &total, st));
          acc_array d = vec(zeros, 256), b = vec(bins, 256);
          OK(acc_exec_permute(hist, &a, n, &d, &b, st));
        }
        OK(acc_stream_sync(ctx, st));
        OK(acc_stream_destroy(ctx, st));
      });
    }
    for (std::thread &th : callers) th.join();
    stop_env.store(true);
    env_thread.join();
  }
  {
    // a stream that goes away takes its guard entry with it: the next stream (often the same handle value) is free of it
    acc_stream s1 = nullptr, s2 = nullptr;
    acc_guard g = nullptr;
    OK(acc_stream_create(ctx, &s1));
    OK(acc_guard_create(ctx, &g));
    OK(acc_stream_set_guard(ctx, s1, g));
    OK(acc_stream_destroy(ctx, s1));
    OK(acc_stream_create(ctx, &s2));
    acc_array m = vec(out, 1000), mi = vec(in, 1000);
    acc_skel plain = make(ctx, ACC_SKEL_MAP, "Int32", "arrIn0_0[ix] + 2", nullptr, nullptr, nullptr, 0, 0);
    // (an idle stream that is given back is the next one handed out: the context keeps it)
    if (s2 != s1) { std::printf("a stream given back idle was not handed out again\n"); ++failures; }
    OK(acc_exec_map(plain, &mi, &m, s2));                  // was refused: "the stream is under a guard"
    acc_event e1 = nullptr, e2 = nullptr, e3 = nullptr;
    OK(acc_event_create(ctx, 1, &e1));
    OK(acc_event_record(ctx, e1, s2));
    OK(acc_event_destroy(ctx, e1));
    OK(acc_event_create(ctx, 0, &e3));                     // another kind: not the timed one that waits in the pool
    OK(acc_event_create(ctx, 1, &e2));
    if (e2 != e1 || e3 == e1) { std::printf("events are not pooled by kind\n"); ++failures; }
    OK(acc_event_destroy(ctx, e2));
    OK(acc_event_destroy(ctx, e3));
    OK(acc_skel_destroy(plain));
    OK(acc_guard_destroy(g));
    OK(acc_stream_destroy(ctx, s2));
  }
  OK(acc_context_sync(ctx));
  OK(acc_memtable_destroy(table));
  if (mock_hip_sweeps() == 0) {
    std::fprintf(stderr, "the segmented fold never went over to its variants with the table of jobs\n");
    return 3;
  }
  for (acc_skel s : {scan, fold, hist, locked, scatter16, scatter32, across, gmap, segs}) OK(acc_skel_destroy(s));
  for (acc_devptr p : {in, out, bins, zeros}) OK(acc_free(ctx, p));
  OK(acc_context_destroy(ctx));
  std::printf("threads %d rounds %d launches %ld failures %d\n", threads, rounds, mock_hip_launches(), failures.load());
  return failures.load() ? 1 : 0;
}
