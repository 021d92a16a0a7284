/*
 * skel_permute.h -- forward permutation with a combining function:
 *
 *     out = defaults;   for every source index ix:   j = permutation(ix);
 *     unless j is `ignore`:   out[j] = combine(get(ix), out[j])
 *
 * Takes the place of CodeGen/IndexSpace.hs:160-303.  The reference serialises
 * every update through a per-element spin lock (three atomics and a fence per
 * element, :285-303) and needs a lock array as large as the target
 * (Execute.hs:402-405).  Here
 *   - a combine the hardware can apply atomically (ACC_COMBINE_HINT: add, min,
 *     max, and, or, xor) is issued as one atomic; anything else is a
 *     compare-and-swap loop on the element's bits -- no locks either way;
 *   - target indices [0, lds_bins) are privatised in LDS: updates to them are
 *     LDS atomics and leave the block once, at the end, so hot targets (a
 *     256-bin histogram, the head of a skewed one) do not queue up on one
 *     memory-side atomic unit.  A target that fits entirely gets `lds_copies`
 *     replicas, one per group of waves, to thin out same-address collisions
 *     inside a block.  Privatisation needs an identity for the combine, so it
 *     is only used with a hint.
 *   - the privatised part leaves a block either as one global atomic per
 *     touched target (few blocks x few bins), or -- when that would again be
 *     millions of atomics, a thousand to the same address -- as a plain dump of
 *     the block's bins into a table that a second kernel, permute_merge, folds
 *     column by column into the result.
 *   - targets beyond the LDS window (the tail of a skewed histogram) are
 *     updated in one table row per XCD, shared by the workgroups running
 *     there: a few hundred KB that stay in that XCD's L2, where its atomics
 *     execute, instead of device-scope atomics that each travel to memory.
 *     permute_merge folds those rows into the result as well.
 * The new value is the FIRST operand of combine (IndexSpace.hs:207).  Updates
 * arrive in no particular order, as in the reference, so combine must be
 * associative and commutative.  Targets outside the result are dropped.
 *
 * Generated definitions expected: ACC_ELT, ACC_ENV_PARAMS, ACC_ENV_ASSUME,
 * ACC_OUT_PARAMS, ACC_OUT_SIZE, ACC_GET(ix), ACC_PERMUTATION(ix),
 * ACC_COMBINE(x,y), ACC_COMBINE_HINT, ACC_ELT_IS_INTEGER, ACC_BLOCK, ACC_VEC,
 * ACC_UNROLL.
 */

#define ACC_TILE (ACC_BLOCK * ACC_VEC * ACC_UNROLL)

#ifndef ACC_GATHER
#define ACC_GATHER 1                                     /* 0: for measuring what the combining of a hot target's lanes is worth */
#endif
#define ACC_GATHER_MIN 4                                 /* lanes that share the target, from which they combine first */
#if ACC_PERMUTE_LOCKED
/* a value and whether a run of equal targets begins at its lane: the inclusive scan of such pairs under
 * (a, b) -> b begins a run ? b : a (+) b  leaves in every lane the combination of its run up to that lane */
template <typename T> struct acc_run { T v; int head; };
#define ACC_DPP_WAVE_SHL1_ 0x130
/* An element no atomic instruction covers -- a tuple, or a scalar of another
 * size than 4 or 8 bytes -- is updated under a lock per target, which is how
 * the reference updates everything (IndexSpace.hs:285-303): locks[j] is 0 when
 * free.  Lanes of one wave may want the same target, and a lane that spins
 * for a lock held by another lane of its own wave never gets it: the holder
 * is masked off until the spinning lane leaves the loop.  So nobody spins: the
 * wave goes round a loop whose condition is a vote of the whole wave, every
 * lane that still has work tries its lock once per trip, and whoever gets it
 * updates the element and frees the lock within that trip.  The lock and the
 * element under it are only touched with relaxed device-scope atomics, which
 * go past the caches that are private to a compute die: the holder waits for
 * its stores to the element to be acknowledged before it stores the free lock,
 * and the next holder, on whichever die, loads the element after its exchange
 * has returned.  (A release/acquire pair would do as well and costs a
 * cache-wide write-back and invalidate per update: 40 times slower.)  `locks`
 * must be all zero on entry and is all zero again on exit, unless a lane gave
 * up (then the status block says so, and the host clears the locks).         */
/* When all targets fit, every workgroup combines its share of the source in a table of its own in LDS, under
 * LDS locks of the same kind (state per target: 0 nothing yet, 1 held, 2 holds a value), and leaves the table
 * in `dump_val` / `dump_ok` (one row per workgroup); permute_join then folds the rows into the result, one wave
 * per target, without any lock.  With few targets that turns millions of contended global lock rounds (1000
 * targets: 0.25 G updates/s at best) into LDS traffic.  Small tables are kept `lds_copies` times, the waves of
 * the workgroup spread over the copies.  More targets than one table holds are cut into windows of `lds_bins`:
 * `win_blocks` consecutive workgroups share a window, walk the whole source between them and take the elements
 * whose target lies in it (as many passes over the source as there are windows, still far cheaper than a round
 * of global locks per element while the windows are few).                                                 */
extern "C" __global__ void __launch_bounds__(ACC_BLOCK)
permute(ACC_ENV_PARAMS ACC_OUT_PARAMS, const Int64 shIn_0, int *__restrict__ locks, const int lds_bins, const int lds_copies,
        ACC_ELT *__restrict__ dump_val, int *__restrict__ dump_ok, const int win_blocks, unsigned int *acc_status ACC_GUARD_PARAM)
{
  ACC_GUARD_CHECK
  typedef ACC_ELT T;
  ACC_ENV_ASSUME
  extern __shared__ __attribute__((aligned(16))) unsigned char acc_lds_raw[];
  auto get  = [&](const Int64 ix) -> T { return (ACC_GET(ix)); };
  auto perm = [&](const Int64 ix) -> Int64 { return (Int64)(ACC_PERMUTATION(ix)); };
  auto f    = [&](const T &x, const T &y) -> T { return (ACC_COMBINE(x, y)); };
  const Int64 n = shIn_0;
  const Int64 ntarget = (ACC_OUT_SIZE);

  /* out[j] := f(x, out[j]) under the global lock of j, for the lanes that are `active`; every lane of the
   * wave comes here together.  Bounded, so that the kernel ends whatever `locks` held on entry: when every
   * element wants the same target the last lane waits for all the others, each of which holds the lock for
   * a few round trips to memory: hence the factor. */
  auto update_global = [&](const Int64 j, const T &x, const bool active) {
    bool done = !active;
    Int64 trips = 0;
    while (__ballot(!done) != 0 && trips < 64 * n + ACC_SPIN_LIMIT) {
      const bool got = !done && __hip_atomic_exchange(locks + j, 1, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT) == 0;
      /* failed exchanges queue at the lock's address in front of the store that frees it: a wave that keeps
       * getting nowhere steps back, for longer every time (up to a third of a millisecond: with the leaders of
       * eight thousand waves after one lock -- half of 2^22 pairs on one target of three million -- and an
       * exchange served every 0.1 us, each must stay away that long for the queue to stay short; stepping back for
       * a microsecond at most, such a launch took 6.8 s) */
      if (trips >= 4 && __ballot(got) == 0) {
        const int naps = (int)acc_min<Int64>(trips - 3, 96);
        for (int k = 0; k < naps; ++k) __builtin_amdgcn_s_sleep(127);
        trips += naps;                                               /* (they count: the bound below is one of time) */
      }
      if (got) {
        const T cur = ACC_READ_DEVICE(arrOut, j);
        ACC_SET_DEVICE(arrOut, j, f(x, cur));
        __asm__ volatile("s_waitcnt vmcnt(0)" ::: "memory");        /* the stores above are acknowledged ... */
        __hip_atomic_store(locks + j, 0, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);   /* ... before this one leaves */
        done = true;
      }
      ++trips;
    }
    if (!done) acc_report(acc_status, ACC_STATUS_PERMUTE_LOCK);      /* never in a healthy run: a lock that did not open; the update is lost */
  };

  /* Sorted or clustered sources send runs of consecutive elements to one target, and the lanes of a wave hold
   * consecutive elements: a whole run would queue at that target's lock (16 M sorted keys into 4096 targets: 7.6 ms
   * against 90 us for keys in random order).  Where a wave has such runs, each is combined first -- the scan of
   * (value, run begins here) pairs above -- and its last lane alone goes on to the lock, with the run's value. */
  const int lane = acc_lane();
  auto join_runs = [&](const Int64 j, T &x, bool &active) {
    const Int64 j_before = acc_dpp<ACC_DPP_WAVE_SHR1, 0xf>(j, j);
    auto continues_now = [&]() -> bool {
      const int active_before = acc_dpp<ACC_DPP_WAVE_SHR1, 0xf>((int)active, (int)active);
      return lane > 0 && active && active_before != 0 && j_before == j;
    };
    bool continues = continues_now();
    const unsigned long long runs = __ballot(continues);
    if (runs == 0) return;                                             /* the same in every lane */
#if ACC_GATHER
    /* A hot target among others, in no order (half of 2^22 sources on one target of 100 000: 4.3-6.9 ms against
     * 0.13-0.15 for uniform targets): its lanes stand all over the wave, a few of them side by side -- which is how
     * it is found.  The lanes that share the target of the first run combine, wherever they stand, and the first of
     * them goes on with the value. */
    {
      const Int64 hot = acc_readlane(j, (int)__builtin_ctzll(runs));
      const bool same = active && j == hot;
      const unsigned long long sharing = __ballot(same);
      if (__builtin_popcountll(sharing) >= ACC_GATHER_MIN) {
        const acc_opt<T> all = acc_wave_reduce(same ? acc_some(x) : acc_none<T>(), acc_lift<T>(f));
        if (lane == (int)__builtin_ctzll(sharing)) x = all.v;
        else if (same) active = false;
        continues = continues_now();
        if (__ballot(continues) == 0) return;
      }
    }
#endif
    acc_run<T> r;
    r.v = x;
    r.head = continues ? 0 : 1;
    r = acc_wave_scan(r, [&](const acc_run<T> &a, const acc_run<T> &b) -> acc_run<T> {
          acc_run<T> c;
          c.v = b.head ? b.v : f(a.v, b.v);
          c.head = a.head | b.head;
          return c;
        }, lane);
    const int next_continues = acc_dpp<ACC_DPP_WAVE_SHL1_, 0xf>((int)continues, (int)continues);
    x = r.v;
    active = active && (lane == ACC_WAVE - 1 || next_continues == 0);  /* the last lane of its run */
  };

  if (lds_bins <= 0) {
    /* every workgroup a stretch of the source of its own, not every gridDim.x-th block of it: under a sorted or
     * clustered source the workgroups that run at one time then work on targets far apart, instead of all on the
     * locks of one neighbourhood -- a few cache lines, whose atomics queue (16 M sorted keys into 300 000 targets:
     * 6.6 ms against 1.4 for keys in random order) */
    const Int64 rounds = (n + ACC_BLOCK - 1) / ACC_BLOCK;
    const Int64 mine_first = rounds * (Int64)blockIdx.x / gridDim.x, mine_past = rounds * ((Int64)blockIdx.x + 1) / gridDim.x;
    for (Int64 ix0 = mine_first * ACC_BLOCK; ix0 < mine_past * ACC_BLOCK; ix0 += ACC_BLOCK) {
      const Int64 ix = ix0 + threadIdx.x;
      const Int64 j = ix < n ? perm(ix) : -1;
      bool active = j >= 0 && j < ntarget;              /* else `ignore`, or outside the result */
      T x = T();
      if (active) x = get(ix);
      join_runs(j, x, active);
      update_global(j, x, active);
    }
    return;
  }

  const int slots = lds_bins * lds_copies;
  T *s_val = (T *)acc_lds_raw;
  int *s_state = (int *)(acc_lds_raw + (((size_t)slots * sizeof(T) + 15) & ~(size_t)15));
  for (int i = threadIdx.x; i < slots; i += ACC_BLOCK) s_state[i] = 0;
  __syncthreads();
  const int mine = (int)((threadIdx.x >> 6) % lds_copies) * lds_bins;     /* this wave's copy */
  const Int64 first = (Int64)(blockIdx.x / win_blocks) * lds_bins;          /* this workgroup's window of targets */
  const Int64 past = acc_min<Int64>(first + lds_bins, ntarget);
  for (Int64 ix0 = (Int64)(blockIdx.x % win_blocks) * ACC_BLOCK; ix0 < n; ix0 += (Int64)win_blocks * ACC_BLOCK) {
    const Int64 ix = ix0 + threadIdx.x;
    const Int64 j = ix < n ? perm(ix) - first : -1;
    bool active = j >= 0 && j < past - first;
    T x = T();
    if (active) x = get(ix);
    join_runs(j, x, active);
    bool done = !active;
    /* whoever holds an LDS lock frees it within the same trip, so every trip makes progress somewhere */
    while (__ballot(!done) != 0) {
      if (!done) {
        const int slot = mine + (int)j;
        const int was = __hip_atomic_exchange(s_state + slot, 1, __ATOMIC_ACQUIRE, __HIP_MEMORY_SCOPE_WORKGROUP);
        if (was != 1) {
          s_val[slot] = (was == 2) ? f(x, s_val[slot]) : x;
          __hip_atomic_store(s_state + slot, 2, __ATOMIC_RELEASE, __HIP_MEMORY_SCOPE_WORKGROUP);
          done = true;
        }
      }
    }
  }
  __syncthreads();
  /* what this workgroup gathered: its row of the table */
  for (int i = threadIdx.x; i < lds_bins; i += ACC_BLOCK) {
    bool have = false;
    T x = T();
    for (int c = 0; c < lds_copies; ++c) {
      if (s_state[c * lds_bins + i] != 2) continue;
      x = have ? f(s_val[c * lds_bins + i], x) : s_val[c * lds_bins + i];
      have = true;
    }
    dump_val[(Int64)blockIdx.x * lds_bins + i] = x;
    dump_ok[(Int64)blockIdx.x * lds_bins + i] = have ? 1 : 0;
  }
}

/* out[j] := f(everything the workgroups gathered for j, out[j]): one wave per target, its lanes spread over
 * the `rows` rows of the table that belong to the target's window of `bins` targets */
extern "C" __global__ void __launch_bounds__(256)
permute_join(ACC_ENV_PARAMS ACC_OUT_PARAMS, const ACC_ELT *__restrict__ dump_val, const int *__restrict__ dump_ok,
             const int rows, const int bins, const Int64 ntarget ACC_GUARD_PARAM)
{
  ACC_GUARD_CHECK
  typedef ACC_ELT T;
  ACC_ENV_ASSUME
  auto f  = [&](const T &x, const T &y) -> T { return (ACC_COMBINE(x, y)); };
  auto lf = acc_lift<T>(f);
  const int lane = acc_lane();
  const Int64 j = (Int64)blockIdx.x * 4 + (threadIdx.x >> 6);
  if (j >= ntarget) return;                           /* whole waves leave */
  const Int64 window = j / bins, col = j - window * bins;
  acc_opt<T> acc = acc_none<T>();
  for (int r = lane; r < rows; r += ACC_WAVE) {
    const Int64 at = (window * rows + r) * bins + col;
    acc_opt<T> p;
    p.v = dump_val[at];
    p.ok = dump_ok[at] != 0;
    acc = lf(acc, p);
  }
  acc = acc_wave_reduce(acc, lf);
  if (lane == 0 && acc.ok) ACC_SET(arrOut, j, f(acc.v, ACC_READ(arrOut, j)));
}

/* ---- permute const: the new value, whatever was there ----------------------
 * Where the combination is spelt as its first operand (the host says so by launching these two instead) nothing has
 * to be read or locked: the scatter of a stream compaction or of a sorting pass over pairs, whose targets are all
 * different.  A scalar of one or two bytes is simply stored (permute_place with winner == NULL).  A tuple's components
 * are arrays of their own, and of several sources on one target one must win whole: permute_claim stores every
 * source's index in its target's word of `winner` -- one of them stays -- and permute_place stores the components of
 * the sources that find their own index there.  (`winner` need not be cleared: what permute_place looks at,
 * permute_claim has written in the same call.)  2^24 pairs of Int32, half of them kept, in order: 277 us under
 * locks; a sorting pass by a 4-bit digit: 771 us. */
#define ACC_CONST_BATCH 4
extern "C" __global__ void __launch_bounds__(256)
permute_claim(ACC_ENV_PARAMS ACC_OUT_PARAMS, const Int64 shIn_0, unsigned int *__restrict__ winner ACC_GUARD_PARAM)
{
  ACC_GUARD_CHECK
  ACC_ENV_ASSUME
  auto perm = [&](const Int64 ix) -> Int64 { return (Int64)(ACC_PERMUTATION(ix)); };
  const Int64 n = shIn_0;
  const Int64 ntarget = (ACC_OUT_SIZE);
  for (Int64 ix0 = (Int64)blockIdx.x * (256 * ACC_CONST_BATCH) + threadIdx.x; ix0 < n; ix0 += (Int64)gridDim.x * (256 * ACC_CONST_BATCH)) {
    Int64 j[ACC_CONST_BATCH];
#pragma unroll
    for (int k = 0; k < ACC_CONST_BATCH; ++k) j[k] = ix0 + k * 256 < n ? perm(ix0 + k * 256) : -1;
#pragma unroll
    for (int k = 0; k < ACC_CONST_BATCH; ++k)
      if (j[k] >= 0 && j[k] < ntarget) winner[j[k]] = (unsigned int)(ix0 + k * 256);
  }
}

extern "C" __global__ void __launch_bounds__(256)
permute_place(ACC_ENV_PARAMS ACC_OUT_PARAMS, const Int64 shIn_0, const unsigned int *__restrict__ winner ACC_GUARD_PARAM)
{
  ACC_GUARD_CHECK
  typedef ACC_ELT T;
  ACC_ENV_ASSUME
  auto get  = [&](const Int64 ix) -> T { return (ACC_GET(ix)); };
  auto perm = [&](const Int64 ix) -> Int64 { return (Int64)(ACC_PERMUTATION(ix)); };
  const Int64 n = shIn_0;
  const Int64 ntarget = (ACC_OUT_SIZE);
  for (Int64 ix0 = (Int64)blockIdx.x * (256 * ACC_CONST_BATCH) + threadIdx.x; ix0 < n; ix0 += (Int64)gridDim.x * (256 * ACC_CONST_BATCH)) {
    Int64 j[ACC_CONST_BATCH];
    bool mine[ACC_CONST_BATCH];
#pragma unroll
    for (int k = 0; k < ACC_CONST_BATCH; ++k) {
      j[k] = ix0 + k * 256 < n ? perm(ix0 + k * 256) : -1;
      mine[k] = j[k] >= 0 && j[k] < ntarget;
    }
    if (winner) {
      unsigned int w[ACC_CONST_BATCH];
#pragma unroll
      for (int k = 0; k < ACC_CONST_BATCH; ++k) w[k] = mine[k] ? winner[j[k]] : 0u;
#pragma unroll
      for (int k = 0; k < ACC_CONST_BATCH; ++k) mine[k] = mine[k] && w[k] == (unsigned int)(ix0 + k * 256);
    }
#pragma unroll
    for (int k = 0; k < ACC_CONST_BATCH; ++k)
      if (mine[k]) ACC_SET(arrOut, j[k], get(ix0 + k * 256));
  }
}
#else /* atomics */

#ifndef ACC_RUNS
#define ACC_RUNS 1
#endif
#define ACC_HINT_GENERIC 0
#define ACC_HINT_ADD 1
#define ACC_HINT_MIN 2
#define ACC_HINT_MAX 3
#define ACC_HINT_AND 4
#define ACC_HINT_OR  5
#define ACC_HINT_XOR 6
/* (not a hint of the interface: the generator says so where the combination is spelt `x`, the new value whatever was
 * there -- `permute const`, the scatter of a stream compaction or of a sorting pass, whose targets are all different.
 * A plain store then: nothing is read, and of several sources on one target one wins whole, as under any order of
 * the combinations) */
#define ACC_HINT_REPLACE 7

/* identity of the hinted operator */
template <typename T>
ACC_DEV T acc_hint_identity()
{
#if ACC_COMBINE_HINT == ACC_HINT_MIN
#if ACC_ELT_IS_INTEGER
  return (T(-1) < T(0)) ? T((typename acc_bits<sizeof(T)>::type)(~(typename acc_bits<sizeof(T)>::type)0) >> 1) : T(~T(0));
#else
  return T(__builtin_inff());
#endif
#elif ACC_COMBINE_HINT == ACC_HINT_MAX
#if ACC_ELT_IS_INTEGER
  return (T(-1) < T(0)) ? T(~((typename acc_bits<sizeof(T)>::type)(~(typename acc_bits<sizeof(T)>::type)0) >> 1)) : T(0);
#else
  return T(-__builtin_inff());
#endif
#elif ACC_COMBINE_HINT == ACC_HINT_AND
  return T(~T(0));
#else
  return T(0);
#endif
}

/* one atomic application of the hinted operator at the given scope.  LDS and
 * a block's private table only need workgroup scope (the atomic is performed
 * in LDS, or in this compute die's L2); the shared result needs device scope,
 * which on this part is performed at the memory side and is far slower.      */
template <int SCOPE, typename T, typename F>
ACC_DEV void acc_hint_apply(T *p, const T &x, F combine)
{
#if ACC_COMBINE_HINT == ACC_HINT_REPLACE
  (void)combine;
  typedef typename acc_bits<sizeof(T)>::type B;
  B nb;
  __builtin_memcpy(&nb, &x, sizeof(T));
  __hip_atomic_store((B *)p, nb, __ATOMIC_RELAXED, SCOPE);
#elif ACC_ELT_IS_INTEGER && ACC_COMBINE_HINT != ACC_HINT_GENERIC
  (void)combine;
#if ACC_COMBINE_HINT == ACC_HINT_ADD
  (void)__hip_atomic_fetch_add(p, x, __ATOMIC_RELAXED, SCOPE);
#elif ACC_COMBINE_HINT == ACC_HINT_AND
  (void)__hip_atomic_fetch_and(p, x, __ATOMIC_RELAXED, SCOPE);
#elif ACC_COMBINE_HINT == ACC_HINT_OR
  (void)__hip_atomic_fetch_or(p, x, __ATOMIC_RELAXED, SCOPE);
#elif ACC_COMBINE_HINT == ACC_HINT_XOR
  (void)__hip_atomic_fetch_xor(p, x, __ATOMIC_RELAXED, SCOPE);
#elif ACC_COMBINE_HINT == ACC_HINT_MIN
  (void)__hip_atomic_fetch_min(p, x, __ATOMIC_RELAXED, SCOPE);
#elif ACC_COMBINE_HINT == ACC_HINT_MAX
  (void)__hip_atomic_fetch_max(p, x, __ATOMIC_RELAXED, SCOPE);
#endif
#elif !ACC_ELT_IS_INTEGER && ACC_COMBINE_HINT == ACC_HINT_ADD
  (void)combine;
  (void)__hip_atomic_fetch_add(p, x, __ATOMIC_RELAXED, SCOPE);
#else
  /* compare-and-swap on the bit pattern (cubits/accelerate_cuda_function.h:28-114) */
  typedef typename acc_bits<sizeof(T)>::type B;
  B *q = (B *)p;
  B old = __hip_atomic_load(q, __ATOMIC_RELAXED, SCOPE);
  for (;;) {
    T cur, nxt;
    __builtin_memcpy(&cur, &old, sizeof(T));
    nxt = combine(x, cur);
    B nb;
    __builtin_memcpy(&nb, &nxt, sizeof(T));
    if (__hip_atomic_compare_exchange_strong(q, &old, nb, __ATOMIC_RELAXED, __ATOMIC_RELAXED, SCOPE)) break;
  }
#endif
}

#define ACC_SCOPE_BLOCK  __HIP_MEMORY_SCOPE_WORKGROUP
#define ACC_SCOPE_DEVICE __HIP_MEMORY_SCOPE_AGENT

/* A combination applied by compare-and-swap gives way under a hot target: every lane that finds the word changed
 * tries again, and half of 2^22 sources on ONE target of 100 000 (in no order) took 4.3 ms against 0.13 for uniform
 * targets.  So the lanes of a wave that share a target combine first and one of them applies the result, wherever in
 * the wave they stand (neighbouring elements of one lane are taken care of by ACC_RUNS).  To find out, a lane looks
 * at its neighbour's target only: with a hot target some two neighbours share it, and where no two neighbours share
 * a target -- nearly always, for targets that are spread -- all this is five instructions an element.           */
#define ACC_PERMUTE_CAS (ACC_COMBINE_HINT == ACC_HINT_GENERIC || (!ACC_ELT_IS_INTEGER && ACC_COMBINE_HINT != ACC_HINT_ADD && ACC_COMBINE_HINT != ACC_HINT_REPLACE))
template <typename U, typename T, typename F>
ACC_DEV void acc_wave_gather(U &t, T &x, F f)
{
  const int lane = acc_lane();
  const U before = acc_wave_shift_up1(t);
  const unsigned long long pairs = __ballot(lane > 0 && t == before);
  if (pairs == 0) return;                                /* (the same in every lane) */
  const U hot = acc_readlane(t, (int)__builtin_ctzll(pairs));
  const bool same = t == hot;
  const unsigned long long sharing = __ballot(same);
  if (__builtin_popcountll(sharing) < ACC_GATHER_MIN) return;
  const acc_opt<T> all = acc_wave_reduce(same ? acc_some(x) : acc_none<T>(), acc_lift<T>(f));
  if (lane == (int)__builtin_ctzll(sharing)) x = all.v;
  else if (same) t = (U)~(U)0;                           /* (beyond every bound: dropped, like `ignore`) */
}

/* The XCD this workgroup runs on (hardware register XCC_ID, bits 3:0).  Every
 * XCD has an L2 of its own, and global atomics execute in the L2 of the XCD
 * that issues them. */
ACC_DEV int acc_xcd_id() { return (int)(__builtin_amdgcn_s_getreg(20 | (0 << 6) | (3 << 11)) & 15u); }
#define ACC_XCD_ROWS 16

/* dump == NULL : privatised bins are flushed into the result with atomics
 * dump         : privatised bins are dumped to row blockIdx.x of the table dump[gridDim.x][lds_bins]
 * far == NULL  : targets beyond the LDS window are updated in the result with device-scope atomics
 * far          : ... in row acc_xcd_id() of far[ACC_XCD_ROWS][target size] (filled with the combine's
 *                identity beforehand), shared by the workgroups of one XCD.  Their atomics meet in
 *                that XCD's L2, where the row stays resident, and need no wider scope than that
 *                cache; the rows reach memory when the kernel ends.                                */
/* ACC_PERMUTE_WINDOWS: more targets than one LDS table holds.  The targets are dealt out to 2^win_log windows
 * like cards (target t belongs to window t mod 2^win_log, so that hot targets that lie together spread over
 * the windows), `win_blocks` consecutive workgroups share a window, walk the whole source between them and take
 * the elements that belong to it; every workgroup dumps its table (row blockIdx.x of `dump`).  As many passes
 * over the source as windows -- 2^26 uniform keys into 2^18 targets: 8 passes, 0.25 ms, against 2.1 ms of
 * device-scope atomics -- and no worse for skewed keys than for uniform ones.                             */
/* ACC_PERMUTE_NARROW (integer addition): twice to four times the targets in one LDS table, for counting.  A
 * target's count is kept in 16 bits, two targets to a word (t and t + half the targets, so that neighbouring hot
 * targets do not meet on one word), and grows by additions of at most ACC_NARROW_MAX
 * (larger addends -- rare in a histogram, where they are all 1 -- go to the result directly).  The lane whose
 * addition takes a count from below 0x8000 to 0x8000 or above takes 0x8000 out again and adds it to the target's entry of
 * a table of carries in memory (`far`, all zero between launches), which permute_merge adds into the result;
 * so a count of 0x8000 or more always has such a correction on its way.  That the count cannot reach 0x10000
 * (and spill into its neighbour) before the correction lands is not left to timing: a lane that finds a count at
 * ACC_NARROW_STOP or above waits until it has dropped below that, and since a lane has at most ACC_VEC additions in flight
 * before it looks, the count ends below ACC_NARROW_STOP + ACC_NARROW_MAX * (1 + ACC_BLOCK * ACC_VEC) < 0x10000.
 * A wave applies the corrections of a batch before any of its lanes waits, so a lane never waits for its own wave.
 * What is left in the table at the end leaves as a row of words of `dump`.                                      */
#ifndef ACC_PERMUTE_NARROW
#define ACC_PERMUTE_NARROW 0
#endif
#if ACC_PERMUTE_NARROW
#define ACC_NARROW_MAX  3u
#define ACC_NARROW_HALF 0x8000u
#ifndef ACC_NARROW_DUMP_VEC
#define ACC_NARROW_DUMP_VEC 1
#endif
#ifndef ACC_NARROW_DUMP_NT
#define ACC_NARROW_DUMP_NT 0     /* the rows leave in plain stores: behind non-temporal ones the additions to the carries that follow them
                                    took 1.3 us of a launch instead of 0.4 (2^26 Zipf keys: 53.4 -> 52.5 us a step; uniform keys the same) */
#endif
#ifndef ACC_NARROW_STOP
#define ACC_NARROW_STOP 0xA000u
#endif
static_assert(ACC_NARROW_STOP > ACC_NARROW_HALF, "a lane would wait for a correction nobody owes");
static_assert(ACC_NARROW_STOP + ACC_NARROW_MAX * (1u + ACC_BLOCK * ACC_VEC) < 0x10000u, "a 16-bit count could spill into its neighbour");
static_assert(ACC_COMBINE_HINT == ACC_HINT_ADD && ACC_ELT_IS_INTEGER && !ACC_PERMUTE_WINDOWS, "narrow counts are for integer addition");
#endif

extern "C" __global__ void __launch_bounds__(ACC_BLOCK)
permute(ACC_ENV_PARAMS ACC_OUT_PARAMS, const Int64 shIn_0, const int lds_bins, const int lds_copies,
        ACC_ELT *__restrict__ dump, ACC_ELT *__restrict__ far
#if ACC_PERMUTE_WINDOWS
        , const int win_blocks, const int win_log
#endif
#if ACC_PERMUTE_NARROW
        , unsigned int *acc_status
#endif
#if !ACC_PERMUTE_NARROW && !ACC_PERMUTE_WINDOWS
        /* first_fill != NULL (only where every target has its bin in LDS and the bins leave by atomics): the
         * result starts as a copy of first_fill, made by workgroup 0 while the others read the source; `ready`
         * (a word that holds {epoch, 1} once the copy can be seen from every die) is what they look at before
         * their atomics.  One launch instead of two. */
        , const ACC_ELT *__restrict__ first_fill, unsigned long long *ready, const unsigned int epoch, unsigned int *acc_status
#endif
        ACC_GUARD_PARAM)
{
  ACC_GUARD_CHECK
  typedef ACC_ELT T;
  ACC_ENV_ASSUME
  extern __shared__ __attribute__((aligned(16))) unsigned char acc_lds_raw[];
  T *bins = (T *)acc_lds_raw;
#if !ACC_PERMUTE_NARROW && !ACC_PERMUTE_WINDOWS
  if (first_fill && blockIdx.x == 0) {
    /* Stores of device scope, which go through this die's L2 to memory, where the others' atomics are performed.
     * Every wave waits until its own have been acknowledged, the barrier until every wave has, and the word
     * follows them.  (A fence here, and an acquiring read on the other side, write back and invalidate whole L2s:
     * 9 us on a launch of 41; the barrier alone does not wait for stores to memory.) */
    const Int64 count = (ACC_OUT_SIZE);
    for (Int64 i = threadIdx.x; i < count; i += ACC_BLOCK)
      __hip_atomic_store(arrOut_0 + i, first_fill[i], __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
    asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
    __syncthreads();
    if (threadIdx.x == 0)
      __hip_atomic_store(ready, ((unsigned long long)epoch << 32) | 1ull, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
  }
#endif

  /* Target indices are handled as unsigned numbers of the width the
   * permutation produces (32 bits for Int32 keys): `ignore` (-1) and every
   * other negative index then lie beyond any bound, and each range test
   * lo <= t < hi is one subtraction and one comparison.  The update loop is
   * bound by instruction issue as much as by memory -- some twenty vector
   * instructions per element is all there is room for -- so this matters. */
  typedef decltype(ACC_PERMUTATION((Int64)0)) acc_perm_result;
  typedef typename acc_bits<(sizeof(acc_perm_result) <= 4 ? 4 : 8)>::type U;
  const Int64 n = shIn_0;
  const Int64 ntarget = (ACC_OUT_SIZE);
  /* what a non-negative index of that width can name */
  const Int64 reach = sizeof(U) == 4 ? acc_min<Int64>(ntarget, (Int64)1 << (acc_is_unsigned<acc_perm_result>::value ? 32 : 31)) : ntarget;
#if ACC_PERMUTE_WINDOWS
  const U u_window = (U)(blockIdx.x / win_blocks), u_mask = (U)((1u << win_log) - 1u);   /* this workgroup's window */
  const U u_reach = (U)reach;
#else
  const U u_bins = (U)acc_min<Int64>(lds_bins, reach), u_beyond = (U)(reach - acc_min<Int64>(lds_bins, reach));
#endif

  auto get  = [&](const Int64 ix) -> T { return (ACC_GET(ix)); };
  auto perm = [&](const Int64 ix) -> U { return (U)(ACC_PERMUTATION(ix)); };
  auto f    = [&](const T &x, const T &y) -> T { return (ACC_COMBINE(x, y)); };

  const T ident = acc_hint_identity<T>();
  T *row = dump ? dump + (Int64)blockIdx.x * lds_bins : (T *)0;
  T *far_row = far ? far + (Int64)acc_xcd_id() * ntarget : (T *)0;
  (void)far_row;

#if ACC_PERMUTE_NARROW
  unsigned *words = (unsigned *)acc_lds_raw;
  const int nwords = (lds_bins + 1) / 2;
  for (int i = threadIdx.x; i < nwords; i += ACC_BLOCK) words[i] = 0u;
  __syncthreads();
  typedef typename acc_bits<sizeof(T)>::type UT;
  const U u_half = (U)nwords;
  auto narrow_shift = [&](const U t) -> unsigned { return t < u_half ? 0u : 16u; };
  auto narrow_word  = [&](const U t) -> unsigned { return (unsigned)(t < u_half ? t : t - u_half); };
  /* the addition itself: what the count was before it, or 0 (which asks for neither a correction nor a wait) where
   * no count was touched */
  /* (Without a branch, so that the additions of a batch are issued one behind the other and waited for together:
   * a lane with nothing to add adds 0 to a word of its own.) */
  auto narrow_add = [&](const U t, const T &x, const unsigned most) -> unsigned {
    const UT ux = (UT)x;
    const bool in = t < u_bins, small = ux <= (UT)most;
    if (in && !small) acc_hint_apply<ACC_SCOPE_DEVICE>(arrOut_0 + t, x, f);
    const bool take = in && small;
    const unsigned sh = narrow_shift(t);
    const unsigned old = __hip_atomic_fetch_add(words + (take ? narrow_word(t) : (threadIdx.x & 63u)),
                                                take ? (unsigned)ux << sh : 0u, __ATOMIC_RELAXED, ACC_SCOPE_BLOCK);
    return take ? (old >> sh) & 0xFFFFu : 0u;
  };
  /* the lane that took the count over the half-way mark moves that half into the target's carry */
  auto narrow_carry = [&](const U t, const T &x, const unsigned before) {
    if (before < ACC_NARROW_HALF && before + (unsigned)(UT)x >= ACC_NARROW_HALF) {
      (void)__hip_atomic_fetch_sub(words + narrow_word(t), ACC_NARROW_HALF << narrow_shift(t), __ATOMIC_RELAXED, ACC_SCOPE_BLOCK);
      acc_hint_apply<ACC_SCOPE_DEVICE>(far + t, (T)ACC_NARROW_HALF, f);       /* `far` is the table of carries here */
    }
  };
  auto narrow_wait = [&](const U t, const unsigned before) {
    if (before >= ACC_NARROW_STOP) {
      const unsigned sh = narrow_shift(t);
      /* (the correction is a few instructions away in another wave; the bound only makes sure that every wave ends,
       * and a wait that does run out is reported: the count may then have spilt into its neighbour) */
      int polls = 0;
      while (((__hip_atomic_load(words + narrow_word(t), __ATOMIC_RELAXED, ACC_SCOPE_BLOCK) >> sh) & 0xFFFFu) >= ACC_NARROW_STOP &&
             polls < ACC_SPIN_LIMIT) {
        ++polls;
        __builtin_amdgcn_s_sleep(1);
      }
      if (polls >= ACC_SPIN_LIMIT) acc_report(acc_status, ACC_STATUS_PERMUTE_LOCK);
    }
  };
  (void)ident; (void)bins;
#else
  for (int i = threadIdx.x; i < lds_bins * lds_copies; i += ACC_BLOCK) bins[i] = ident;
  __syncthreads();
  T *mine = bins + ((threadIdx.x >> 6) % lds_copies) * lds_bins;
#endif

  /* two independent tests rather than a chain: each becomes a predicated
   * instruction, not a branch */
  auto update = [&](const U t, const T &x) {
#if ACC_PERMUTE_NARROW
    const unsigned before = narrow_add(t, x, ACC_NARROW_MAX);
    narrow_carry(t, x, before);
    narrow_wait(t, before);
#elif ACC_PERMUTE_WINDOWS
    if (t < u_reach && (t & u_mask) == u_window) acc_hint_apply<ACC_SCOPE_BLOCK>(mine + (t >> win_log), x, f);
#else
    if (t < u_bins) acc_hint_apply<ACC_SCOPE_BLOCK>(mine + t, x, f);
    if ((U)(t - u_bins) < u_beyond) {
      if (far_row) acc_hint_apply<ACC_SCOPE_BLOCK>(far_row + t, x, f);
      else         acc_hint_apply<ACC_SCOPE_DEVICE>(arrOut_0 + t, x, f);
    }
#endif
  };

  /* full tiles, software-pipelined: the next tile's indices and values are
   * requested before the current tile's updates are issued, so the atomics'
   * latency is spent under loads already in flight */
  const Int64 full_tiles = n / ACC_TILE;
  U j[ACC_UNROLL][ACC_VEC], jn[ACC_UNROLL][ACC_VEC];
  T x[ACC_UNROLL][ACC_VEC], xn[ACC_UNROLL][ACC_VEC];
  auto load = [&](const Int64 tile, U (&jj)[ACC_UNROLL][ACC_VEC], T (&xx)[ACC_UNROLL][ACC_VEC]) {
    const Int64 base = tile * (Int64)ACC_TILE + (Int64)threadIdx.x * ACC_VEC;
#pragma unroll
    for (int u = 0; u < ACC_UNROLL; ++u)
#pragma unroll
      for (int k = 0; k < ACC_VEC; ++k) {
        const Int64 ix = base + u * (ACC_BLOCK * ACC_VEC) + k;
        jj[u][k] = perm(ix);
        xx[u][k] = get(ix);
      }
  };
#if ACC_PERMUTE_WINDOWS
  const Int64 walkers = win_blocks, walker = blockIdx.x % win_blocks;         /* the workgroups that share the source */
#else
  const Int64 walkers = gridDim.x, walker = blockIdx.x;
#endif
  Int64 tile = walker;
  if (tile < full_tiles) load(tile, j, x);
  while (tile < full_tiles) {
    const Int64 next = tile + walkers;
    if (next < full_tiles) load(next, jn, xn);
#if ACC_PERMUTE_NARROW
#pragma unroll
    for (int u = 0; u < ACC_UNROLL; ++u) {           /* ACC_VEC additions, then their corrections, then the waits */
      unsigned before[ACC_VEC];
      T added[ACC_VEC];
      /* a lane's ACC_VEC consecutive elements on ONE target (sorted or clustered sources), each a small addend: one
       * addition of their sum -- no more than the lane would have had in flight anyway, so the bound above holds */
      bool one_target = ACC_RUNS && ACC_VEC > 1;
#pragma unroll
      for (int k = 0; k < ACC_VEC; ++k)
        one_target = one_target && j[u][k] == j[u][0] && (UT)x[u][k] <= (UT)ACC_NARROW_MAX;
      if (one_target) {
        T all = x[u][0];
#pragma unroll
        for (int k = 1; k < ACC_VEC; ++k) all = (T)(all + x[u][k]);
        before[0] = narrow_add(j[u][0], all, ACC_NARROW_MAX * ACC_VEC);
        added[0] = all;
#pragma unroll
        for (int k = 1; k < ACC_VEC; ++k) { before[k] = 0u; added[k] = T(0); }
      } else {
#pragma unroll
        for (int k = 0; k < ACC_VEC; ++k) { before[k] = narrow_add(j[u][k], x[u][k], ACC_NARROW_MAX); added[k] = x[u][k]; }
      }
      /* ONE test for the batch: a correction or a wait takes a count within an addend of ACC_NARROW_HALF or more, and
       * nearly no batch has one (a test and a branch per addition, skipped or not, were a third of the loop's
       * instructions; 2^26 Zipf keys into 65 536 targets: 54.2 -> 53.7 us) */
      unsigned top = before[0];
#pragma unroll
      for (int k = 1; k < ACC_VEC; ++k) top = acc_max(top, before[k]);
      if (top >= ACC_NARROW_HALF - ACC_NARROW_MAX * ACC_VEC) {
#pragma unroll
        for (int k = 0; k < ACC_VEC; ++k) narrow_carry(j[u][k], added[k], before[k]);
#pragma unroll
        for (int k = 0; k < ACC_VEC; ++k) narrow_wait(j[u][k], before[k]);
      }
    }
#else
#pragma unroll
    for (int u = 0; u < ACC_UNROLL; ++u) {
      /* a lane's ACC_VEC consecutive elements on ONE target (sorted or clustered sources, flat areas of an image):
       * combined first, one update instead of ACC_VEC on the same address */
      bool one_target = ACC_RUNS && ACC_VEC > 1;
#pragma unroll
      for (int k = 1; k < ACC_VEC; ++k) one_target = one_target && j[u][k] == j[u][0];
#if ACC_GATHER && ACC_PERMUTE_CAS
      if (one_target) {
#pragma unroll
        for (int k = 1; k < ACC_VEC; ++k) { x[u][0] = f(x[u][0], x[u][k]); j[u][k] = (U)~(U)0; }
      }
#pragma unroll
      for (int k = 0; k < ACC_VEC; ++k) acc_wave_gather(j[u][k], x[u][k], f);
#pragma unroll
      for (int k = 0; k < ACC_VEC; ++k) update(j[u][k], x[u][k]);
#else
      if (one_target) {
        T all = x[u][0];
#pragma unroll
        for (int k = 1; k < ACC_VEC; ++k) all = f(all, x[u][k]);
        update(j[u][0], all);
      } else {
#pragma unroll
        for (int k = 0; k < ACC_VEC; ++k) update(j[u][k], x[u][k]);
      }
#endif
    }
#endif
#pragma unroll
    for (int u = 0; u < ACC_UNROLL; ++u)
#pragma unroll
      for (int k = 0; k < ACC_VEC; ++k) { j[u][k] = jn[u][k]; x[u][k] = xn[u][k]; }
    tile = next;
  }

  /* the ragged last tile, taken by whichever block it falls to */
  if (full_tiles * (Int64)ACC_TILE < n && walker == full_tiles % walkers) {
    const Int64 base = full_tiles * (Int64)ACC_TILE + (Int64)threadIdx.x * ACC_VEC;
#pragma unroll
    for (int u = 0; u < ACC_UNROLL; ++u)
#pragma unroll
      for (int k = 0; k < ACC_VEC; ++k) {
        const Int64 ix = base + u * (ACC_BLOCK * ACC_VEC) + k;
        if (ix < n) update(perm(ix), get(ix));
      }
  }

  /* the privatised part leaves the block */
#if ACC_PERMUTE_NARROW
  __syncthreads();
  {
    /* A count leaves as its low byte: words i and i + nd of the table make one word of the row (bytes: targets
     * i, i + nwords, i + nd, i + nd + nwords), half of what whole counts would write here and the merge read again.
     * What a count holds above its low byte goes to the target's carry; few counts do (those of more than 255 of this
     * workgroup's share of the source), and nothing but speed depends on how few. */
    const int nd = (nwords + 1) / 2;
    unsigned *wrow = (unsigned *)dump + (Int64)blockIdx.x * nd;
    auto pack = [&](const unsigned a, const unsigned b) -> unsigned {
      return (a & 0xFFu) | ((a >> 8) & 0xFF00u) | ((b & 0xFFu) << 16) | ((b << 8) & 0xFF000000u);
    };
    int scalar_from = 0;
#if ACC_NARROW_DUMP_VEC
    if ((nd & 3) == 0 && nwords == 2 * nd) {
      /* Four words of the row a lane: two 128-bit reads of the table, one 128-bit store (uniform keys: 51.9 -> 50.5 us
       * a step).  Where a wave finds counts with something above their low byte among the 256 words it has just sent
       * out, it goes over those words once more, a word a lane, for the additions to the carries: one instruction
       * then covers a run of neighbouring carries once.  (Made from the 128-bit reads, four instructions a lane would
       * each cover every fourth carry of the same few cache lines, and the requests of 256 workgroups for those lines
       * queue at the memory side four times over: Zipf keys 65 us a step against 53.) */
      typedef unsigned acc_u4 __attribute__((ext_vector_type(4)));
      for (int i0 = (threadIdx.x & ~63) * 4; i0 < nd; i0 += ACC_BLOCK * 4) {          /* this wave's 256 words */
        const int i = i0 + (threadIdx.x & 63) * 4;
        unsigned high = 0u;
        if (i < nd) {                                  /* (a whole vector: nd is a multiple of 4) */
          const acc_u4 a = *(const acc_u4 *)(words + i), b = *(const acc_u4 *)(words + i + nd);
          high = (a.x | a.y | a.z | a.w | b.x | b.y | b.z | b.w) & 0xFF00FF00u;
          acc_u4 o;
          o.x = pack(a.x, b.x); o.y = pack(a.y, b.y); o.z = pack(a.z, b.z); o.w = pack(a.w, b.w);
#if ACC_NARROW_DUMP_NT
          __builtin_nontemporal_store(o, (acc_u4 *)(wrow + i));
#else
          *(acc_u4 *)(wrow + i) = o;
#endif
        }
        if (__ballot(high != 0u) != 0) {
          for (int q = 0; q < 4; ++q) {
            const int w = i0 + q * 64 + (threadIdx.x & 63);
            if (w >= nd) continue;
            const unsigned c = words[w], d = words[w + nd];
            if (c & 0x0000FF00u) acc_hint_apply<ACC_SCOPE_DEVICE>(far + w, (T)(c & 0xFF00u), f);
            if (c & 0xFF000000u) acc_hint_apply<ACC_SCOPE_DEVICE>(far + w + nwords, (T)((c >> 16) & 0xFF00u), f);
            if (d & 0x0000FF00u) acc_hint_apply<ACC_SCOPE_DEVICE>(far + w + nd, (T)(d & 0xFF00u), f);
            if (d & 0xFF000000u) acc_hint_apply<ACC_SCOPE_DEVICE>(far + w + nd + nwords, (T)((d >> 16) & 0xFF00u), f);
          }
        }
      }
      scalar_from = nd;
    }
#endif
    for (int i = scalar_from + threadIdx.x; i < nd; i += ACC_BLOCK) {
      const unsigned a = words[i];
      const unsigned b = i + nd < nwords ? words[i + nd] : 0u;
      if ((a | b) & 0xFF00FF00u) {
        if (a & 0x0000FF00u) acc_hint_apply<ACC_SCOPE_DEVICE>(far + i, (T)(a & 0xFF00u), f);
        if (a & 0xFF000000u) acc_hint_apply<ACC_SCOPE_DEVICE>(far + i + nwords, (T)((a >> 16) & 0xFF00u), f);
        if (b & 0x0000FF00u) acc_hint_apply<ACC_SCOPE_DEVICE>(far + i + nd, (T)(b & 0xFF00u), f);
        if (b & 0xFF000000u) acc_hint_apply<ACC_SCOPE_DEVICE>(far + i + nd + nwords, (T)((b >> 16) & 0xFF00u), f);
      }
      wrow[i] = pack(a, b);
    }
  }
  (void)row;
#else
  if (lds_bins > 0) {
#if !ACC_PERMUTE_WINDOWS
    if (first_fill && blockIdx.x != 0) {
      /* workgroup 0 made its copy tens of microseconds ago; the wait is bounded all the same, and one that runs
       * out is reported (the atomics below would then add to whatever the result held before) */
      if (threadIdx.x == 0) {
        int polls = 0;
        while ((__hip_atomic_load(ready, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT) >> 32) != (unsigned long long)epoch &&
               polls < ACC_SPIN_LIMIT) {
          ++polls;
          __builtin_amdgcn_s_sleep(4);
        }
        if (polls >= ACC_SPIN_LIMIT) acc_report(acc_status, ACC_STATUS_PERMUTE_LOCK);
      }
    }
#endif
    __syncthreads();
    for (int i = threadIdx.x; i < lds_bins; i += ACC_BLOCK) {
      T acc = bins[i];
      for (int c = 1; c < lds_copies; ++c) acc = f(bins[c * lds_bins + i], acc);
      if (row) {
        row[i] = acc;
      } else {
        typename acc_bits<sizeof(T)>::type a, b;
        __builtin_memcpy(&a, &acc, sizeof(T));
        __builtin_memcpy(&b, &ident, sizeof(T));
        if (a != b) acc_hint_apply<ACC_SCOPE_DEVICE>(arrOut_0 + i, acc, f);
      }
    }
  }
#endif
}

/* fills p[0 .. count) with the combine's identity and copies copy_count
 * elements from copy_src to copy_dst (the defaults into the result): the two
 * small jobs that precede the main kernel, in one launch */
extern "C" __global__ void __launch_bounds__(256)
permute_fill(ACC_ELT *__restrict__ p, const Int64 count, ACC_ELT *__restrict__ copy_dst,
             const ACC_ELT *__restrict__ copy_src, const Int64 copy_count ACC_GUARD_PARAM)
{
  ACC_GUARD_CHECK
  const ACC_ELT ident = acc_hint_identity<ACC_ELT>();
  const Int64 first = (Int64)blockIdx.x * 256 + threadIdx.x, step = (Int64)gridDim.x * 256;
  for (Int64 i = first; i < count; i += step) p[i] = ident;
  for (Int64 i = first; i < copy_count; i += step) copy_dst[i] = copy_src[i];
}

/* one table to fold: columns [first, first + cols) of dump[nrows][stride] go
 * into the same positions of the result.  The rows are split into `slices`
 * groups handled by different workgroups; with one slice the result is
 * written plainly, otherwise each group applies its share with one atomic per
 * target.                                                                    */
struct acc_merge_job {
  const ACC_ELT *dump;
  Int64 stride, first, cols;
  int nrows, slices;
  int window_log;         /* >= 0: the table is one block of `nrows` rows per window, target t in window
                             t mod 2^window_log at column t >> window_log; -1: one table, target t at column t */
};

#if ACC_PERMUTE_NARROW
/* result = base + carries + the sum of the workgroups' rows of packed 8-bit counts.  A row has nd = ceil(nwords / 2)
 * words; byte q of word `column` is the low byte of the count of target  column + (q & 2 ? nd : 0) + (q & 1 ? nwords : 0)
 * (the main kernel's table holds targets w and w + nwords in word w, and sends words w and w + nd out as one).  A
 * workgroup takes 64 consecutive words, each of its ACC_MERGE_WAVES waves its share of the rows, sixteen loads in flight a lane,
 * whose bytes are added two to a register (16 x 255 fits 16 bits) before they are widened; the waves' sums meet in
 * LDS and wave q writes the targets of byte q -- one thread per target, so no atomics and nothing that must be in
 * the result beforehand -- and clears the carries it has taken (the table is all zero between launches).  `base` is
 * the defaults array, or the result itself where that was filled from the defaults before the main kernel (which
 * then also added to it directly).                                                                          */
#ifndef ACC_MERGE_WAVES
#define ACC_MERGE_WAVES 4
#endif
static_assert(ACC_MERGE_WAVES >= 4 && ACC_MERGE_WAVES <= 16, "a wave for each byte of a row's word");
extern "C" __global__ void __launch_bounds__(64 * ACC_MERGE_WAVES)
permute_merge(ACC_ENV_PARAMS ACC_OUT_PARAMS, const unsigned *__restrict__ dump, const Int64 nwords, const int nrows,
              const Int64 ntarget, ACC_ELT *carry, const ACC_ELT *base ACC_GUARD_PARAM)
{
  ACC_GUARD_CHECK
  typedef ACC_ELT T;
  ACC_ENV_ASSUME
  __shared__ unsigned s_sum[ACC_MERGE_WAVES][4][64];   /* [wave][byte][lane] */
  auto f = [&](const T &x, const T &y) -> T { return (ACC_COMBINE(x, y)); };
  const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
  constexpr int waves = ACC_MERGE_WAVES;
  const Int64 nd = (nwords + 1) / 2;
  const Int64 column = (Int64)blockIdx.x * 64 + lane;
  const Int64 col_c = acc_min<Int64>(column, nd - 1);           /* lanes past the end read the last word and drop it */
  unsigned c0 = 0u, c1 = 0u, c2 = 0u, c3 = 0u;
  int r = wave;
#ifndef ACC_MERGE_BATCH
#define ACC_MERGE_BATCH 16                     /* loads in flight a lane (x 255 fits 16 bits up to 257) */
#endif
  for (; r + waves * (ACC_MERGE_BATCH - 1) < nrows; r += waves * ACC_MERGE_BATCH) {
    unsigned w[ACC_MERGE_BATCH];
#pragma unroll
    for (int k = 0; k < ACC_MERGE_BATCH; ++k) w[k] = __builtin_nontemporal_load(dump + (Int64)(r + waves * k) * nd + col_c);
    unsigned even = 0u, odd = 0u;
#pragma unroll
    for (int k = 0; k < ACC_MERGE_BATCH; ++k) { even += w[k] & 0x00FF00FFu; odd += (w[k] >> 8) & 0x00FF00FFu; }
    c0 += even & 0xFFFFu; c2 += even >> 16;
    c1 += odd & 0xFFFFu;  c3 += odd >> 16;
  }
  for (; r < nrows; r += waves) {
    const unsigned w = __builtin_nontemporal_load(dump + (Int64)r * nd + col_c);
    c0 += w & 0xFFu; c1 += (w >> 8) & 0xFFu; c2 += (w >> 16) & 0xFFu; c3 += w >> 24;
  }
  s_sum[wave][0][lane] = c0;
  s_sum[wave][1][lane] = c1;
  s_sum[wave][2][lane] = c2;
  s_sum[wave][3][lane] = c3;
  __syncthreads();
  if (wave >= 4) return;                                         /* wave q writes the targets of byte q */
  unsigned total = 0u;
  for (int w = 0; w < waves; ++w) total += s_sum[w][wave][lane];
  const Int64 word = column + ((wave & 2) ? nd : 0);             /* the word of the main kernel's table the count sat in */
  const Int64 t = word + ((wave & 1) ? nwords : 0);
  if (column < nd && word < nwords && t < ntarget) {
    const T c = carry[t];
    if (c != T(0)) carry[t] = T(0);
    arrOut_0[t] = f((T)((T)total + c), base[t]);
  }
}
#else
/* folds up to two tables in one launch: workgroups [0, blocks_a) take job a,
 * the rest job b */
extern "C" __global__ void __launch_bounds__(256)
permute_merge(ACC_ENV_PARAMS ACC_OUT_PARAMS, const acc_merge_job a, const int blocks_a, const acc_merge_job b ACC_GUARD_PARAM)
{
  ACC_GUARD_CHECK
  typedef ACC_ELT T;
  ACC_ENV_ASSUME
  auto f = [&](const T &x, const T &y) -> T { return (ACC_COMBINE(x, y)); };
  const bool second = (int)blockIdx.x >= blocks_a;
  const acc_merge_job job = second ? b : a;
  const int block = second ? (int)blockIdx.x - blocks_a : (int)blockIdx.x;
  const Int64 column = (Int64)(block / job.slices) * 256 + threadIdx.x;
  const int slice = block % job.slices;
  if (column >= job.cols) return;
  const int per = (job.nrows + job.slices - 1) / job.slices;
  const int r0 = slice * per, r1 = acc_min(job.nrows, r0 + per);
  if (r0 >= r1) return;
  const T *src = job.dump + job.first + column;
  if (job.window_log >= 0) {
    const Int64 window = column & (((Int64)1 << job.window_log) - 1);
    src = job.dump + window * job.nrows * job.stride + (column >> job.window_log);
  }
  T acc = src[(Int64)r0 * job.stride];
#pragma unroll 8
  for (int r = r0 + 1; r < r1; ++r) acc = f(src[(Int64)r * job.stride], acc);
  T *dst = arrOut_0 + job.first + column;
  if (job.slices == 1) {
    *dst = f(acc, *dst);
  } else {
    const T ident = acc_hint_identity<T>();
    typename acc_bits<sizeof(T)>::type x, y;
    __builtin_memcpy(&x, &acc, sizeof(T));
    __builtin_memcpy(&y, &ident, sizeof(T));
    if (x != y) acc_hint_apply<ACC_SCOPE_DEVICE>(dst, acc, f);
  }
}
#endif /* ACC_PERMUTE_NARROW */
#endif /* ACC_PERMUTE_LOCKED */
