/*
 * skel_foldseg.h -- foldSeg / fold1Seg: reduce every segment of a vector,
 * segment s being the index range [offset[s], offset[s+1]).
 *
 * Takes the place of CodeGen/Reduction.hs:399-574, which gives each segment a
 * 32-lane warp (one useful load per lane and a five-step shared-memory tree
 * for a 32-element row).  With 64-lane waves and short segments most of that
 * would idle, so the work is split the other way round:
 *   - a workgroup owns ACC_BLOCK consecutive segments, i.e. ONE contiguous
 *     range of the input;
 *   - all its lanes stream that range through LDS in chunks of ACC_CHUNK
 *     elements, evaluating the (fused) producer with fully coalesced, 128-bit
 *     reads whatever the segment lengths are;
 *   - lane i then folds the part of segment i that lies in the chunk, reading
 *     LDS sequentially, and carries its accumulator to the next chunk; the
 *     next chunk's loads are already in flight while it does so.
 * Every segment is thus combined strictly in index order, the order of a
 * sequential fold: the operator need only be associative for the result to
 * be independent of the schedule, and with ACC_FOLD_RIGHT the association is
 * x0 (+) (x1 (+) (... (+) (x_last (+) z))) instead of
 * ((x0 (+) x1) (+) ...) (+) z.  The seed is the second operand and an empty
 * segment yields the seed (Reduction.hs:567-574).
 *
 * Generated definitions expected: ACC_ENTRY (via kind), ACC_ELT,
 * ACC_ENV_PARAMS, ACC_ENV_ASSUME, ACC_GET(ix), ACC_COMBINE(x,y), ACC_HAS_SEED,
 * ACC_SEED, ACC_SEG_TYPE, ACC_FOLD_RIGHT, ACC_BLOCK, ACC_VEC, ACC_CHUNK.
 */

static_assert(ACC_CHUNK % (ACC_BLOCK * ACC_VEC) == 0, "chunk must be a whole number of block-wide vector loads");

/* ACC_SEG_UNIFORM: the segments are the rows of a rank > 1 array, all of the same length -- `fold` / `fold1` along
 * the innermost dimension (CodeGen/Reduction.hs:221-367, mkFoldDim) is this template with computed offsets.      */
#ifndef ACC_SEG_UNIFORM
#define ACC_SEG_UNIFORM 0
#endif
#if ACC_SEG_UNIFORM
#if ACC_HAS_SEED
#define ACC_FOLDSEG_ENTRY fold
#else
#define ACC_FOLDSEG_ENTRY fold1
#endif
/* (rows, row length) as the kernel parameters shIn_1, shIn_0 */
#define ACC_SEG_PARAMS const Int64 shIn_1, const Int64 shIn_0
#define ACC_SEG_TOTAL (shIn_1 * shIn_0)
#define ACC_SEG_AT(s) ((Int64)(s) * shIn_0)
/* The element function of such a fold may name acc_row and acc_col, the row of the folded array and the place within
 * it (ix == acc_row * row length + acc_col).  The entries that give a row to a lane know both as they stand; the
 * others divide, where the names are used at all. */
#define ACC_GET_AT_IX [&](const Int64 ix) -> T { const Int64 acc_row = ix / shIn_0, acc_col = ix - acc_row * shIn_0; (void)acc_row; (void)acc_col; return (ACC_GET(ix)); }
#define ACC_GET_AT_ROW_COL [&](const Int64 acc_row, const Int64 acc_col) -> T { const Int64 ix = acc_row * shIn_0 + acc_col; (void)ix; return (ACC_GET(ix)); }
#else
#define ACC_GET_AT_IX [&](const Int64 ix) -> T { return (ACC_GET(ix)); }
#if ACC_HAS_SEED
#define ACC_FOLDSEG_ENTRY foldSeg
#else
#define ACC_FOLDSEG_ENTRY fold1Seg
#endif
/* ACC_SEG_OUTER: foldSeg / fold1Seg of an array of rank > 1.  The segment descriptor cuts the innermost dimension of
 * every outer row alike (CodeGen/Reduction.hs:473-474: base = (seg / num_segments) * innerExtent): segment s of the
 * flattened result is segment s % seg_per_row of row s / seg_per_row, `seg_inner` elements a row.  What a row holds
 * beyond its last segment belongs to no segment.                                                                  */
#ifndef ACC_SEG_OUTER
#define ACC_SEG_OUTER 0
#endif
#if ACC_SEG_OUTER
#define ACC_SEG_PARAMS const Int64 shIn_0, const ACC_SEG_TYPE *__restrict__ arrSeg_0, const Int64 seg_inner, const Int64 seg_per_row
#define ACC_SEG_TOTAL shIn_0
#define ACC_SEG_AT(s)  (((Int64)(s) / seg_per_row) * seg_inner + (Int64)arrSeg_0[(Int64)(s) % seg_per_row])
#define ACC_SEG_END(s) (((Int64)(s) / seg_per_row) * seg_inner + (Int64)arrSeg_0[(Int64)(s) % seg_per_row + 1])
#else
#define ACC_SEG_PARAMS const Int64 shIn_0, const ACC_SEG_TYPE *__restrict__ arrSeg_0
#define ACC_SEG_TOTAL shIn_0
#define ACC_SEG_AT(s) ((Int64)arrSeg_0[s])
#endif
#endif
/* where segment s ends: where the next one begins, unless rows have tails */
#ifndef ACC_SEG_END
#define ACC_SEG_END(s) ACC_SEG_AT((s) + 1)
#endif

/* ACC_GIANTS: among many short segments a few may hold most of the source (the rows of a power-law graph).  The
 * workgroup that owns such a segment would stream it alone, chunk after chunk, long after the others have ended: one
 * segment of 2^23 elements among a million short ones took 6-12 ms.  So where a workgroup has folded a stretch of a
 * segment together (ACC_WIDE, below) and ACC_GIANT_FROM elements or more of that segment lie beyond the chunk, the
 * rest is handed over: the owner enters it in a table of jobs in scratch memory, with the value of what it has
 * folded of the segment so far, and goes on with the chunk in which the segment ends.  A second launch, <entry>_sweep
 * at the end of this file, takes the jobs in pieces of ACC_GIANT_PIECE elements, by ticket, until none is left; a
 * piece is folded in index order, all lanes together, and its value left as tagged words.  A job's tickets come
 * from ACC_GIANT_LINES counters, a cache line of their own each, every one for a run of consecutive pieces
 * (additions to one word, and to the words of one cache line, are performed one after the other).  Whoever draws
 * the ticket behind the last piece of the last line puts the owner's value and the pieces together, in order, and
 * writes the segment's result.  The only wait is that workgroup's, for pieces whose tickets were drawn before its
 * own -- by workgroups that are running, or done; it is bounded like every wait.  With no room in the table the
 * segment stays with its owner as if there were no table.  The table and the values carry the launch's tag
 * (nothing is cleared between launches).  Index order, another association than the sequential fold's: as for
 * every long segment.
 *   The teams of lanes that take segments which are long on average (<entry>_team, below) enter a segment that is
 * far longer than the rest in the same table, whole and with no value of their own.
 *   Variants 4 to 7 of an instance are built like this, and the host takes them once a look at the segment lengths
 * (<entry>_probe, at the end of this file) has found such a segment.  Not every instance, not from the start: the code
 * in this kernel lies behind the test for a stretch that the workgroup folds together, and yet, with it compiled in
 * and no such segment in the source, 2^25 elements in segments of 2 / 8 / 32 took 101 / 36 / 29 us instead of
 * 89 / 33 / 27 and the sparse matrix-vector product 193 instead of 190; the second launch costs a source without
 * such segments 2-3 us more.  (A test of every block of segments ahead of its first chunk, by way of a barrier that
 * carries the lanes' answers, made the segments of two elements 117 us: the block's first loads then wait for the
 * lanes' offsets.)                                                                                               */
#ifndef ACC_GIANTS
#define ACC_GIANTS 0
#endif
#if ACC_SEG_UNIFORM || ACC_SEG_OUTER
#undef ACC_GIANTS
#define ACC_GIANTS 0                                     /* (segments of one length; rows with segments of their own) */
#endif
#ifndef ACC_GIANT_CHUNKS
#define ACC_GIANT_CHUNKS 4
#endif
#define ACC_GIANT_PIECE ((Int64)ACC_GIANT_CHUNKS * ACC_CHUNK)
#define ACC_GIANT_FROM  (2 * ACC_GIANT_PIECE)
#define ACC_GIANT_TIMES 32                               /* ... and, for a team of lanes, so many times the average segment */
#if ACC_GIANTS
#define ACC_GIANT_PARAMS , unsigned long long *__restrict__ acc_jobs, const unsigned int acc_epoch, unsigned int *acc_status
#define ACC_GIANT_JOBS  32                               /* the host sizes the scratch block by these three */
#define ACC_GIANT_HEAD  8                                /* 64-bit words in front of the jobs */
#define ACC_GIANT_LINES 16                               /* ticket counters a job, each for a run of its pieces */
#define ACC_GIANT_SPREAD 32                              /* words between two counters: additions to one cache line queue like additions to one word */
#define ACC_GIANT_JOB   (8 + ACC_GIANT_LINES * ACC_GIANT_SPREAD)           /* 64-bit words a job: tag; the low halves of segment, first, end; lines that have run out; the high halves; the counters */
#else
#define ACC_GIANT_PARAMS
#endif

#define ACC_LOADS (ACC_CHUNK / (ACC_BLOCK * ACC_VEC))   /* vector loads per lane and chunk */
/* One word of padding per 32 elements of the staged chunk: lanes that fold segments whose starts are a multiple
 * of 32 elements apart (every segment 32, 64, 128 ... long) would otherwise all read the same LDS bank.  The padding
 * moves that worst case to starts 31, 62, 93 ... apart, so rows of ONE length (ACC_SEG_UNIFORM, where the length is
 * known) are padded only if the length is a multiple of 8: 2^25 Float32 in rows of 31 / 62 / 124 54 -> 25 / 31 / 34 us,
 * rows of 32 / 64 / 96 stay at 25 / 29 / 31 (68 / 67 / 76 without).                                              */
#ifndef ACC_PAD_ON
#define ACC_PAD_ON 1                                     /* 0: for measuring what the padding is worth */
#endif
#define ACC_PAD_SPACE(i) (ACC_PAD_ON ? ((i) + ((i) >> 5)) : (i))
#define ACC_PAD(i) ((i) + (((i) >> 5) & acc_pad_mask))
#define ACC_EAT 8                                        /* LDS reads kept in flight while folding */
#ifndef ACC_WIDE
#define ACC_WIDE 256                                     /* elements of one segment in a chunk from which the workgroup folds them together */
#endif

#if ACC_GIANTS
/* enter elements [a, b) of segment `seg` in the table of jobs; the job's number, or -1 if the table is full.
 * `with_value`: the owner has folded a part of the segment itself and leaves its value for whoever joins the pieces */
ACC_DEV int acc_giant_enter(unsigned long long *jobs, const unsigned int epoch, const Int64 seg, const Int64 a, const Int64 b, const bool with_value)
{
  unsigned long long h = __hip_atomic_load(jobs, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
  unsigned int at;
  for (;;) {                                     /* the head word: {tag of the launch, jobs entered so far} */
    at = (unsigned int)(h >> 32) == epoch ? (unsigned int)h : 0u;
    if (at >= ACC_GIANT_JOBS) return -1;
    const unsigned long long want = ((unsigned long long)epoch << 32) | (at + 1u);
    if (__hip_atomic_compare_exchange_strong(jobs, &h, want, __ATOMIC_RELAXED, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT)) break;
  }
  unsigned long long *j = jobs + ACC_GIANT_HEAD + (Int64)at * ACC_GIANT_JOB;
  /* (words whose upper half may be anything but zero carry the launch's tag there, like every word of this memory
   * that others read by its tag: an offset beyond 2^32 left as it is would read as a tag of some later launch) */
  const unsigned long long tag = (unsigned long long)epoch << 32;
  const unsigned long long what[3] = {(unsigned long long)seg, (unsigned long long)a, (unsigned long long)b};
#pragma unroll
  for (int k = 0; k < 3; ++k) {
    __hip_atomic_store(j + 1 + k, tag | (unsigned int)what[k], __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
    __hip_atomic_store(j + 5 + k, tag | (unsigned int)(what[k] >> 32), __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
  }
  __hip_atomic_store(j + 4, 0ull, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
  for (int k = 0; k < ACC_GIANT_LINES; ++k) __hip_atomic_store(j + 8 + k * ACC_GIANT_SPREAD, 0ull, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
  /* (nobody looks at a job before this launch has ended: no order among these stores is needed) */
  __hip_atomic_store(j, tag | (with_value ? 1u : 2u), __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
  return (int)at;
}

/* where the value that a job's owner has folded itself goes: behind the two values for every piece of the source */
ACC_DEV unsigned int acc_giant_edge_slot(const Int64 n, const int job) { return (unsigned int)(2 * (n / ACC_GIANT_PIECE + 2) + job); }

#endif

extern "C" __global__ void __launch_bounds__(ACC_BLOCK)
ACC_FOLDSEG_ENTRY(ACC_ENV_PARAMS
                  const Int64 shOut_0, ACC_OUT_ARRAY(arrOut),
                  ACC_SEG_PARAMS ACC_GIANT_PARAMS ACC_GUARD_PARAM)
{
  ACC_GUARD_CHECK
  typedef ACC_ELT T;
  ACC_ENV_ASSUME
  __shared__ __attribute__((aligned(16))) T s_val[ACC_PAD_SPACE(ACC_CHUNK)];
#if ACC_GIANTS
  __shared__ int s_skip;
#endif
  /* for the stretches the whole workgroup folds (below) */
  __shared__ int s_wide[ACC_BLOCK / ACC_WAVE];
  __shared__ int s_owner, s_from, s_to;
  __shared__ acc_opt<T> s_part[ACC_BLOCK / ACC_WAVE];

  auto get = ACC_GET_AT_IX;
  auto f   = [&](const T &x, const T &y) -> T { return (ACC_COMBINE(x, y)); };
  auto lf  = acc_lift<T>(f);

  const Int64 nseg = shOut_0;
  const Int64 n = ACC_SEG_TOTAL;
  const int tid = threadIdx.x;
#if ACC_HAS_SEED
  const T seed = (ACC_SEED);
#endif
  if (tid == 0) s_owner = ACC_BLOCK;
#if ACC_GIANTS
  if (tid == 0) s_skip = -1;
#endif
  /* (the loop over this workgroup's blocks of segments, compiled with and without the padding: an address that adds
   * the padding under a run-time mask costs the inner loop more than the bank conflicts it avoids) */
  auto blocks_of_segments = [&](auto padded_c) {
  constexpr int acc_pad_mask = decltype(padded_c)::value ? ~0 : 0;
  /* (seen by all at the first barrier of the first chunk) */

  for (Int64 first = (Int64)blockIdx.x * ACC_BLOCK; first < nseg; first += (Int64)gridDim.x * ACC_BLOCK) {
    const Int64 seg = first + tid;
    const bool live = seg < nseg;
    /* both ends of the lane's segment are asked for at once (a lane past the last segment asks for the last one's
     * and takes nothing) */
    const Int64 seg_c = acc_min<Int64>(seg, nseg - 1);
    const Int64 a_c = ACC_SEG_AT(seg_c), b_c = ACC_SEG_END(seg_c);
    Int64 a = live ? a_c : 0;
    Int64 b = live ? b_c : 0;
    const Int64 last = acc_min<Int64>(first + ACC_BLOCK, nseg);
    const Int64 lo = ACC_SEG_AT(first), hi = acc_min<Int64>(ACC_SEG_END(last - 1), n);
    bool handed = false;                             /* this lane's segment has been handed over (below) */

    T acc = T();
    bool have = false;
#if ACC_HAS_SEED && ACC_FOLD_RIGHT
    acc = seed;
    have = true;
#endif

    /* chunks start on a vector boundary so that the loads stay aligned */
    const Int64 lo_al = lo - (lo % ACC_VEC);
    const Int64 nchunks = hi > lo_al ? (hi - lo_al + ACC_CHUNK - 1) / ACC_CHUNK : 0;
    /* stage a chunk: every load is issued before any result is used, with no branch among them, so that all the
     * loads of a chunk -- and the gathers that may stand behind every element -- are in flight together.  Elements
     * of the chunk's first and last vector that belong to a neighbouring block are loaded too (they exist) and
     * never read back.  A vector that lies wholly beyond this block's segments is not wanted (short segments fill
     * a fraction of a chunk, and every element may cost a gather): its lane reads the block's last vector instead,
     * which all such lanes of a wave do with one request between them.  Only the block that holds the ragged end
     * of the array goes element by element. */
    T v[ACC_LOADS][ACC_VEC];
    auto chunk_start = [&](const Int64 q) -> Int64 { return lo_al + (ACC_FOLD_RIGHT ? (nchunks - 1 - q) : q) * (Int64)ACC_CHUNK; };
    const Int64 last_vec = hi > 0 ? (hi - 1) / ACC_VEC : 0;           /* index of the vector that holds element hi - 1 */
    const bool whole_vectors = (last_vec + 1) * ACC_VEC <= n;        /* uniform over the block */
    auto stage = [&](const Int64 cs) {
      if (whole_vectors) {
#pragma unroll
        for (int u = 0; u < ACC_LOADS; ++u) {
          const Int64 i0 = acc_min<Int64>(cs / ACC_VEC + (u * ACC_BLOCK + tid), last_vec) * ACC_VEC;
#pragma unroll
          for (int k = 0; k < ACC_VEC; ++k) v[u][k] = get(i0 + k);
        }
#pragma unroll
        for (int u = 0; u < ACC_LOADS; ++u)
#pragma unroll
          for (int k = 0; k < ACC_VEC; ++k) acc_pin(v[u][k]);
      } else {
#pragma unroll
        for (int u = 0; u < ACC_LOADS; ++u)
#pragma unroll
          for (int k = 0; k < ACC_VEC; ++k) {
            /* past the end of the array: its last element instead, which no segment reads back from there */
            const Int64 ix = acc_min<Int64>(acc_min<Int64>(cs / ACC_VEC + (u * ACC_BLOCK + tid), last_vec) * ACC_VEC + k, n - 1);
            v[u][k] = get(ix);
          }
      }
    };
    if (nchunks > 0) stage(chunk_start(0));
    for (Int64 q = 0; q < nchunks; ++q) {
      const Int64 cs = chunk_start(q);
      const Int64 ce = acc_min<Int64>(cs + ACC_CHUNK, hi);
      __syncthreads();                               /* the previous chunk has been consumed */
#pragma unroll
      for (int u = 0; u < ACC_LOADS; ++u)
        if (cs + (Int64)(u * ACC_BLOCK + tid) * ACC_VEC < hi) {
#pragma unroll
          for (int k = 0; k < ACC_VEC; ++k) s_val[ACC_PAD((u * ACC_BLOCK + tid) * ACC_VEC + k)] = v[u][k];
        }
      /* this lane's segment, as far as it lies in the chunk */
      int p0 = (int)(acc_max(a, cs) - cs), p1 = (int)(acc_min(b, ce) - cs);
      /* One lane a segment serialises a long segment on its lane while the rest of the workgroup waits: among a
       * million short segments a single one of 2^23 elements took 130-200 ms.  A stretch of ACC_WIDE elements or more
       * of one segment in a chunk is therefore folded by the whole workgroup: every lane a run of consecutive
       * elements, in order, the lanes joined in lane order and the waves in wave order, and the owner of the segment
       * puts the stretch's value on the proper side of what it holds -- index order still, another association, as
       * for the segments that teams of lanes fold (below).  Whether a chunk has such a stretch travels with the
       * barrier that every chunk has anyway, and is looked at after the lanes' own folds (the SMVM configuration:
       * 191.2 us with the look before them, 189.8 after, as with none of this). */
      constexpr bool wide_stretches = ACC_WIDE <= ACC_CHUNK;      /* (a larger ACC_WIDE switches all of this off) */
      const bool wide = wide_stretches && p1 - p0 >= ACC_WIDE;
      if (wide_stretches) {
        const bool wide_in_wave = __ballot(wide) != 0;
        if (acc_lane() == 0) s_wide[tid >> 6] = wide_in_wave ? 1 : 0;
      }
      __syncthreads();
      /* the next chunk's loads (and the gathers behind them) travel while this one is folded */
      if (q + 1 < nchunks) stage(chunk_start(q + 1));

      /* (the flags are asked for here and looked at after the lanes' own folds, which hide the wait for them; a lane
       * with a wide stretch leaves it to the workgroup) */
      int wide_flag[ACC_BLOCK / ACC_WAVE];
#pragma unroll
      for (int w = 0; w < ACC_BLOCK / ACC_WAVE; ++w) wide_flag[w] = wide_stretches ? s_wide[w] : 0;
      const int w0 = p0, w1 = p1;
      if (wide) p1 = p0;

      /* fold this lane's segment, as far as it lies in the chunk, in index order */
#if ACC_FOLD_RIGHT
      if (!have && p0 < p1) { --p1; acc = s_val[ACC_PAD(p1)]; have = true; }
      for (; p1 - ACC_EAT >= p0; p1 -= ACC_EAT) {
        T w[ACC_EAT];
#pragma unroll
        for (int k = 0; k < ACC_EAT; ++k) w[k] = s_val[ACC_PAD(p1 - 1 - k)];
#pragma unroll
        for (int k = 0; k < ACC_EAT; ++k) acc = f(w[k], acc);
      }
      for (; p1 > p0; --p1) acc = f(s_val[ACC_PAD(p1 - 1)], acc);
#else
      if (!have && p0 < p1) { acc = s_val[ACC_PAD(p0)]; ++p0; have = true; }
      for (; p0 + ACC_EAT <= p1; p0 += ACC_EAT) {
        T w[ACC_EAT];
#pragma unroll
        for (int k = 0; k < ACC_EAT; ++k) w[k] = s_val[ACC_PAD(p0 + k)];
#pragma unroll
        for (int k = 0; k < ACC_EAT; ++k) acc = f(acc, w[k]);
      }
      for (; p0 < p1; ++p0) acc = f(acc, s_val[ACC_PAD(p0)]);
#endif

      bool any_wide = false;
#pragma unroll
      for (int w = 0; w < ACC_BLOCK / ACC_WAVE; ++w) any_wide = any_wide || wide_flag[w] != 0;
      if (any_wide) {                                              /* the same in every lane */
        bool pending = wide;
        for (;;) {
          if (pending) (void)__hip_atomic_fetch_min(&s_owner, tid, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_WORKGROUP);   /* the owners take their turns in lane order */
          __syncthreads();
          const int owner = s_owner;
          if (owner >= ACC_BLOCK) break;                           /* nobody left */
          if (tid == owner) { s_from = w0; s_to = w1; }
          __syncthreads();
          const int from = s_from, to = s_to;
          const int per = (to - from + ACC_BLOCK - 1) / ACC_BLOCK;
          const int i0 = acc_min(from + tid * per, to), i1 = acc_min(i0 + per, to);
          acc_opt<T> m = acc_none<T>();
          for (int i = i0; i < i1; ++i) m = lf(m, acc_some(s_val[ACC_PAD(i)]));
          m = acc_wave_reduce(m, lf);
          if (acc_lane() == 0) s_part[tid >> 6] = m;
          if (tid == owner) s_owner = ACC_BLOCK;
          __syncthreads();
          if (tid == owner) {
            acc_opt<T> whole = s_part[0];
#pragma unroll
            for (int w = 1; w < ACC_BLOCK / ACC_WAVE; ++w) whole = lf(whole, s_part[w]);
#if ACC_FOLD_RIGHT
            acc = have ? f(whole.v, acc) : whole.v;
#else
            acc = have ? f(acc, whole.v) : whole.v;
#endif
            have = true;
            pending = false;
#if ACC_GIANTS
            /* What is left of the segment beyond this chunk, if that is ACC_GIANT_FROM elements or more, is handed
             * over: entered in the table of jobs, together with the value of what has been folded so far, and this
             * workgroup goes on with the chunk in which the segment ends. */
            const Int64 rest = ACC_FOLD_RIGHT ? cs - a : b - ce;
            if (acc_jobs && rest >= ACC_GIANT_FROM) {
              const int job = ACC_FOLD_RIGHT ? acc_giant_enter(acc_jobs, acc_epoch, seg, a, cs, true) : acc_giant_enter(acc_jobs, acc_epoch, seg, ce, b, true);
              if (job >= 0) {                                      /* (no room in the table: the segment stays here) */
                const acc_tagged<T> values_of = {acc_jobs + ACC_GIANT_HEAD + ACC_GIANT_JOBS * ACC_GIANT_JOB};
                values_of.put(acc_giant_edge_slot(n, job), acc_epoch, acc);
                s_skip = ACC_FOLD_RIGHT ? (int)(nchunks - 1 - (a - lo_al) / ACC_CHUNK) : (int)((b - lo_al) / ACC_CHUNK);
                handed = true;
#if ACC_FOLD_RIGHT
                a = b;                                             /* nothing of it is this lane's any more */
#else
                b = a;
#endif
              }
            }
#endif
          }
        }
#if ACC_GIANTS
        /* (the turns end with a barrier: what an owner has written is seen by all) */
        const int skip_to = s_skip;
        if (skip_to >= 0) {                                        /* the same in every lane */
          __syncthreads();
          if (tid == 0) s_skip = -1;
          if (skip_to < nchunks) stage(chunk_start(skip_to));      /* (in place of the chunk asked for above) */
          q = skip_to - 1;
        }
#endif
      }

    }

    if (live && !handed) {
#if ACC_HAS_SEED && !ACC_FOLD_RIGHT
      ACC_SET(arrOut, seg, have ? f(acc, seed) : seed);
#else
      ACC_SET(arrOut, seg, acc);      /* fold1Seg of an empty segment is undefined; T() is written */
#endif
    }
  }
  };   /* blocks_of_segments */
#if ACC_SEG_UNIFORM && ACC_PAD_ON
  if (shIn_0 % 8 == 0) blocks_of_segments(acc_bool<true>());
  else                 blocks_of_segments(acc_bool<false>());
#else
  blocks_of_segments(acc_bool<ACC_PAD_ON != 0>());
#endif
}

#if ACC_SEG_UNIFORM
/* ---- short rows: a lane per row, straight from memory ----------------------
 * Rows of up to ACC_ROWS_MAX elements (a fold over colour channels, small vectors, 4 x 4 blocks): a lane reads its
 * row with as few, as wide loads as the row length allows -- the lanes of a wave read one contiguous stretch
 * between them -- and folds it in index order, in the association of the entry above.  Nothing is staged: the
 * chunks of the entry above hold whole blocks of segments, which for rows this short leaves most of a chunk unused. */
#define ACC_ROWS_MAX 16
template <int W, typename T, typename F>
ACC_DEV T acc_fold_row(const T (&x)[W], F f, const T &seed)
{
  (void)seed;
#if ACC_FOLD_RIGHT
  /* x0 (+) (x1 (+) (... (x_last (+) z))) */
#if ACC_HAS_SEED
  T acc = f(x[W - 1], seed);
#else
  T acc = x[W - 1];
#endif
#pragma unroll
  for (int k = W - 2; k >= 0; --k) acc = f(x[k], acc);
#else
  /* ((x0 (+) x1) (+) ... x_last) (+) z */
  T acc = x[0];
#pragma unroll
  for (int k = 1; k < W; ++k) acc = f(acc, x[k]);
#if ACC_HAS_SEED
  acc = f(acc, seed);
#endif
#endif
  return acc;
}

/* A lane takes R consecutive rows -- 4 rows of 1, 2 rows of 2, so that its load is one 128-bit vector and the lanes'
 * vectors lie side by side; longer rows one at a time, lane after lane -- and U such groups a workgroup-width
 * apart, so that about 64 bytes per lane are requested before the first is used.  The host computes the same R
 * and U for the grid.                                                                                            */
template <int W, typename T, typename G, typename F, typename P>
ACC_DEV void acc_fold_rows(const Int64 nseg, G get, F f, const T &seed, P put)
{
  constexpr int R = W == 1 ? 4 : (W == 2 ? 2 : 1);
  constexpr int U = (R * W >= 16) ? 1 : 16 / (R * W);
  const Int64 per_block = (Int64)ACC_BLOCK * R * U;
  for (Int64 b0 = (Int64)blockIdx.x * per_block; b0 < nseg; b0 += (Int64)gridDim.x * per_block) {
    if (b0 + per_block <= nseg) {
      T x[U][R][W];
#pragma unroll
      for (int u = 0; u < U; ++u)
#pragma unroll
        for (int r = 0; r < R; ++r)
#pragma unroll
          for (int k = 0; k < W; ++k) x[u][r][k] = get(b0 + ((Int64)u * ACC_BLOCK + threadIdx.x) * R + r, k);
#pragma unroll
      for (int u = 0; u < U; ++u)
#pragma unroll
        for (int r = 0; r < R; ++r) put(b0 + ((Int64)u * ACC_BLOCK + threadIdx.x) * R + r, acc_fold_row<W, T>(x[u][r], f, seed));
    } else {
#pragma unroll
      for (int u = 0; u < U; ++u)
#pragma unroll
        for (int r = 0; r < R; ++r) {
          const Int64 seg = b0 + ((Int64)u * ACC_BLOCK + threadIdx.x) * R + r;
          if (seg < nseg) {
            T x[W];
#pragma unroll
            for (int k = 0; k < W; ++k) x[k] = get(seg, k);
            put(seg, acc_fold_row<W, T>(x, f, seed));
          }
        }
    }
  }
}

#define ACC_FS_CAT2_(a, b) a##b
#define ACC_FS_CAT_(a, b) ACC_FS_CAT2_(a, b)
extern "C" __global__ void __launch_bounds__(ACC_BLOCK)
ACC_FS_CAT_(ACC_FOLDSEG_ENTRY, _rows)(ACC_ENV_PARAMS
                                      const Int64 shOut_0, ACC_OUT_ARRAY(arrOut),
                                      ACC_SEG_PARAMS ACC_GUARD_PARAM)
{
  ACC_GUARD_CHECK
  typedef ACC_ELT T;
  ACC_ENV_ASSUME
  auto get = ACC_GET_AT_ROW_COL;
  auto f   = [&](const T &x, const T &y) -> T { return (ACC_COMBINE(x, y)); };
  auto put = [&](const Int64 seg, const T &v) { ACC_PUT(arrOut, seg, v); };       /* written once, not read again here */
  (void)shIn_1;
#if ACC_HAS_SEED
  const T seed = (ACC_SEED);
#else
  const T seed = T();
#endif
  switch ((int)shIn_0) {
#define ACC_ROW_CASE(W) case W: acc_fold_rows<W, T>(shOut_0, get, f, seed, put); break;
    ACC_ROW_CASE(1) ACC_ROW_CASE(2) ACC_ROW_CASE(3) ACC_ROW_CASE(4) ACC_ROW_CASE(5) ACC_ROW_CASE(6) ACC_ROW_CASE(7) ACC_ROW_CASE(8)
    ACC_ROW_CASE(9) ACC_ROW_CASE(10) ACC_ROW_CASE(11) ACC_ROW_CASE(12) ACC_ROW_CASE(13) ACC_ROW_CASE(14) ACC_ROW_CASE(15) ACC_ROW_CASE(16)
#undef ACC_ROW_CASE
    default: break;                                /* the host does not launch this entry for other lengths */
  }
}

/* ---- rows that lie across memory: a lane per row, whatever the length ------
 * <entry>_across, for an element function that, where the ROW index moves by one, reads neighbouring addresses --
 * the fold of a transposed matrix (sums down its columns), of a matrix product written as a fold over
 * `zipWith (*)` of two replicated operands, one of them transposed (ACC_FLAG_TILED says so: the host cannot see it).
 * A team of lanes along such a row asks for 64 cache lines with every load; a lane per row, neighbouring rows in
 * neighbouring lanes, asks for one.  Lane t takes piece t / rows of row t % rows: with fewer rows than the device
 * has lanes the rows are cut into `split` pieces of consecutive elements, whose values <entry>_join puts together in
 * order; with split == 1 the lane writes the row's result itself.  Every piece is folded in index order, eight
 * elements requested before the first is used.                                                                   */
#define ACC_ACROSS_UNROLL 8
extern "C" __global__ void __launch_bounds__(ACC_BLOCK)
ACC_FS_CAT_(ACC_FOLDSEG_ENTRY, _across)(ACC_ENV_PARAMS
                                        const Int64 shOut_0, ACC_OUT_ARRAY(arrOut),
                                        ACC_SEG_PARAMS,
                                        const Int64 split, ACC_ELT *__restrict__ part, int *__restrict__ part_ok ACC_GUARD_PARAM)
{
  ACC_GUARD_CHECK
  typedef ACC_ELT T;
  ACC_ENV_ASSUME
  auto get = ACC_GET_AT_ROW_COL;
  auto f   = [&](const T &x, const T &y) -> T { return (ACC_COMBINE(x, y)); };
  (void)shIn_1;
  const Int64 rows = shOut_0, len = shIn_0;
  const Int64 piece = (len + split - 1) / split;
  for (Int64 t = (Int64)blockIdx.x * ACC_BLOCK + threadIdx.x; t < rows * split; t += (Int64)gridDim.x * ACC_BLOCK) {
    const Int64 p = t / rows, row = t - p * rows;
    const Int64 k0 = acc_min<Int64>(p * piece, len), k1 = acc_min<Int64>(k0 + piece, len);
    if (k0 >= k1) {                                        /* (a last piece without elements; the host launches no empty rows) */
      if (split > 1) part_ok[row * split + p] = 0;
      continue;
    }
    T x[ACC_ACROSS_UNROLL];
#if ACC_HAS_SEED
    const T seed = (ACC_SEED);
#endif
#if ACC_FOLD_RIGHT
    /* x0 (+) (x1 (+) (... (x_last (+) z))), as the other entries associate a row */
    T acc = get(row, k1 - 1);
#if ACC_HAS_SEED
    if (split == 1) acc = f(acc, seed);
#endif
    Int64 k = k1 - 1;
    for (; k - ACC_ACROSS_UNROLL >= k0; k -= ACC_ACROSS_UNROLL) {
#pragma unroll
      for (int u = 0; u < ACC_ACROSS_UNROLL; ++u) x[u] = get(row, k - 1 - u);
#pragma unroll
      for (int u = 0; u < ACC_ACROSS_UNROLL; ++u) acc = f(x[u], acc);
    }
    for (; k > k0; --k) acc = f(get(row, k - 1), acc);
#else
    T acc = get(row, k0);
    Int64 k = k0 + 1;
    for (; k + ACC_ACROSS_UNROLL <= k1; k += ACC_ACROSS_UNROLL) {
#pragma unroll
      for (int u = 0; u < ACC_ACROSS_UNROLL; ++u) x[u] = get(row, k + u);
#pragma unroll
      for (int u = 0; u < ACC_ACROSS_UNROLL; ++u) acc = f(acc, x[u]);
    }
    for (; k < k1; ++k) acc = f(acc, get(row, k));
#endif
    if (split > 1) {
      part[row * split + p] = acc;
      part_ok[row * split + p] = 1;
    } else {
#if ACC_HAS_SEED && !ACC_FOLD_RIGHT
      ACC_PUT(arrOut, row, f(acc, seed));                  /* ((x0 (+) x1) (+) ... x_last) (+) z */
#else
      ACC_PUT(arrOut, row, acc);
#endif
    }
  }
}
#endif /* ACC_SEG_UNIFORM */

/* ---- long segments: a team of lanes per segment ---------------------------
 * One lane per segment serialises a long segment on that lane, so when the
 * segments are long on average the host launches this entry instead: a row
 * of 16 lanes (block_team == 2: four segments a wave side by side, for
 * segments of a few hundred elements, of which a whole wave would ask for
 * more than they hold), a whole wave (block_team == 0) or a whole workgroup
 * (block_team == 1) takes one segment at a time.  The team walks the segment in rounds of ACC_TVEC
 * consecutive elements per lane, each lane folds its own elements in order,
 * the lanes are combined in lane order (the wave reduction preserves order,
 * waves meet in LDS in wave order) and the round's value joins the running
 * one on the proper side: the segment is still combined in index order, only
 * the association differs from the one-lane-per-segment entry, as the
 * operator's associativity allows.  ACC_TROUNDS rounds of loads are issued
 * before the first is used.
 *
 * With fewer segments than the device has room for teams, every segment is
 * cut into `split` consecutive pieces of equal length, each piece goes to
 * a team that leaves its value (and whether the piece held anything) in
 * `part` / `part_ok`, and <entry>_join puts the pieces of every segment
 * together, in order.                                                        */
#define ACC_TVEC 4
#ifndef ACC_TROUNDS
#define ACC_TROUNDS 4
#endif
#define ACC_FS_WAVES (ACC_BLOCK / ACC_WAVE)
#define ACC_FS_CAT2(a, b) a##b
#define ACC_FS_CAT(a, b) ACC_FS_CAT2(a, b)

extern "C" __global__ void __launch_bounds__(ACC_BLOCK)
ACC_FS_CAT(ACC_FOLDSEG_ENTRY, _team)(ACC_ENV_PARAMS
                                     const Int64 shOut_0, ACC_OUT_ARRAY(arrOut),
                                     ACC_SEG_PARAMS,
                                     const int block_team, const Int64 split,
                                     ACC_ELT *__restrict__ part, int *__restrict__ part_ok ACC_GIANT_PARAMS ACC_GUARD_PARAM)
{
  ACC_GUARD_CHECK
  typedef ACC_ELT T;
  ACC_ENV_ASSUME
  __shared__ acc_opt<T> s_wave[ACC_FS_WAVES];
#if ACC_GIANTS
  __shared__ int s_entered;
#endif

  auto get = ACC_GET_AT_IX;
  auto f   = [&](const T &x, const T &y) -> T { return (ACC_COMBINE(x, y)); };
  auto lf  = acc_lift<T>(f);

  const Int64 nseg = shOut_0;
  const Int64 n = ACC_SEG_TOTAL;
  const int tid = threadIdx.x;
  const int wave = tid >> 6;
  const bool row_team = block_team == 2, whole_block = block_team == 1;
  const int me = whole_block ? tid : (row_team ? (acc_lane() & 15) : acc_lane());      /* place in the team */
  const Int64 team_lanes = whole_block ? ACC_BLOCK : (row_team ? 16 : ACC_WAVE);
  const Int64 wave0 = (Int64)blockIdx.x * ACC_FS_WAVES + wave;
  const Int64 team0 = whole_block ? (Int64)blockIdx.x : (row_team ? wave0 * 4 + (acc_lane() >> 4) : wave0);
  const Int64 nteams = whole_block ? (Int64)gridDim.x : (Int64)gridDim.x * ACC_FS_WAVES * (row_team ? 4 : 1);
  const Int64 round = team_lanes * ACC_TVEC;
#if ACC_HAS_SEED
  const T seed = (ACC_SEED);
#endif

  /* the values of round `r` of [a, b) that fall to this lane, folded in order */
  auto mine = [&](const Int64 a, const Int64 b, const Int64 r, const T (&v)[ACC_TVEC]) -> acc_opt<T> {
    const Int64 base = a + r * round + (Int64)me * ACC_TVEC;
    if (base + ACC_TVEC <= b) {                      /* all there: plain values */
      T t = v[0];
#pragma unroll
      for (int k = 1; k < ACC_TVEC; ++k) t = f(t, v[k]);
      return acc_some(t);
    }
    acc_opt<T> m = acc_none<T>();
#pragma unroll
    for (int k = 0; k < ACC_TVEC; ++k)
      if (base + k < b) m = lf(m, acc_some(v[k]));
    return m;
  };
  auto fetch = [&](const Int64 a, const Int64 b, const Int64 r, T (&v)[ACC_TVEC]) {
    const Int64 base = a + r * round + (Int64)me * ACC_TVEC;
    if (base + ACC_TVEC <= b) {
#pragma unroll
      for (int k = 0; k < ACC_TVEC; ++k) v[k] = get(base + k);
      return;
    }
#pragma unroll
    for (int k = 0; k < ACC_TVEC; ++k) {
      v[k] = T();
      if (base + k < b) v[k] = get(base + k);
    }
  };
  /* all lanes of the team, in order; uniform over the team (block teams: over the workgroup) */
  /* (a row team's value is in the row's first lane only, which is the lane that uses it) */
  auto team = [&](acc_opt<T> m) -> acc_opt<T> {
    if (row_team) return acc_row_reduce(m, lf);
    m = acc_wave_reduce(m, lf);
    if (!whole_block) return m;
    if (acc_lane() == 0) s_wave[wave] = m;
    __syncthreads();
    acc_opt<T> r = s_wave[0];
#pragma unroll
    for (int w = 1; w < ACC_FS_WAVES; ++w) r = lf(r, s_wave[w]);
    __syncthreads();
    return r;
  };

#if ACC_GIANTS
  const Int64 giant_from = acc_max<Int64>(ACC_GIANT_FROM, ACC_GIANT_TIMES * (n / acc_max<Int64>(nseg, 1)));
#endif
  for (Int64 job = team0; job < nseg * split; job += nteams) {
    const Int64 seg = job / split, part_no = job - seg * split;
    const Int64 sa = ACC_SEG_AT(seg);
    const Int64 sb = acc_min<Int64>(ACC_SEG_END(seg), n);
    /* `split` pieces of equal length, whole rounds each so that only a segment's last piece is ragged */
    const Int64 piece = (((sb - sa) + split - 1) / split + round - 1) / round * round;
    const Int64 a = split > 1 ? acc_min<Int64>(sa + part_no * piece, sb) : sa;
    const Int64 b = split > 1 ? acc_min<Int64>(a + piece, sb) : sb;
#if ACC_GIANTS
    /* A segment far longer than the rest -- a team would walk it alone long after the others have ended: one of 2^23
     * elements among segments of 256 to 4096 took 14-44 ms -- is entered in the table of jobs whole and left to the
     * launch that takes the jobs (ACC_GIANTS, above).  (Not where every segment is cut into pieces anyway.)  The
     * team's first lane enters it and tells the others. */
    if (acc_jobs && split == 1) {
      int entered = (me == 0 && sb - sa >= giant_from) ? (acc_giant_enter(acc_jobs, acc_epoch, seg, sa, sb, false) >= 0 ? 1 : 0) : 0;
      if (whole_block) {
        if (tid == 0) s_entered = entered;
        __syncthreads();
        entered = s_entered;
        __syncthreads();
      } else {
        entered = __shfl(entered, row_team ? (acc_lane() & ~15) : 0);
      }
      if (entered) continue;
    }
#endif
    const Int64 nrounds = b > a ? (b - a + round - 1) / round : 0;
    acc_opt<T> acc = acc_none<T>();
    for (Int64 r0 = 0; r0 < nrounds; r0 += ACC_TROUNDS) {
      T v[ACC_TROUNDS][ACC_TVEC];
#pragma unroll
      for (int u = 0; u < ACC_TROUNDS; ++u) {
        const Int64 r = ACC_FOLD_RIGHT ? nrounds - 1 - (r0 + u) : r0 + u;
        if (r0 + u < nrounds) fetch(a, b, r, v[u]);
      }
#pragma unroll
      for (int u = 0; u < ACC_TROUNDS; ++u) {
        const Int64 r = ACC_FOLD_RIGHT ? nrounds - 1 - (r0 + u) : r0 + u;
        if (r0 + u < nrounds) {                                  /* uniform over the team */
          const acc_opt<T> t = team(mine(a, b, r, v[u]));
#if ACC_FOLD_RIGHT
          acc = lf(t, acc);
#else
          acc = lf(acc, t);
#endif
        }
      }
    }
    if (me != 0) continue;
    if (split > 1) {
      part[job] = acc.v;
      part_ok[job] = acc.ok ? 1 : 0;
      continue;
    }
    /* (x0 (+) ... (+) x_last) (+) z in either association direction: the seed is the right operand */
#if ACC_HAS_SEED
    ACC_SET(arrOut, seg, acc.ok ? f(acc.v, seed) : seed);
#else
    ACC_SET(arrOut, seg, acc.v);        /* fold1Seg of an empty segment is undefined; T() is written */
#endif
  }
}

/* the pieces of every segment, in order, and the seed: one wave per segment, every lane a run of
 * consecutive pieces, the lanes combined in lane order */
extern "C" __global__ void __launch_bounds__(ACC_BLOCK)
ACC_FS_CAT(ACC_FOLDSEG_ENTRY, _join)(ACC_ENV_PARAMS
                                     const Int64 shOut_0, ACC_OUT_ARRAY(arrOut), const Int64 split,
                                     const ACC_ELT *__restrict__ part, const int *__restrict__ part_ok ACC_GUARD_PARAM)
{
  ACC_GUARD_CHECK
  typedef ACC_ELT T;
  ACC_ENV_ASSUME
  auto f  = [&](const T &x, const T &y) -> T { return (ACC_COMBINE(x, y)); };
  auto lf = acc_lift<T>(f);
  const int lane = acc_lane();
  const Int64 seg = (Int64)blockIdx.x * ACC_FS_WAVES + (threadIdx.x >> 6);
  if (seg >= shOut_0) return;                         /* whole waves leave */
  const Int64 per = (split + ACC_WAVE - 1) / ACC_WAVE;
  acc_opt<T> acc = acc_none<T>();
  for (Int64 k = lane * per; k < acc_min<Int64>((lane + 1) * per, split); ++k) {
    acc_opt<T> p;
    p.v = part[seg * split + k];
    p.ok = part_ok[seg * split + k] != 0;
    acc = lf(acc, p);
  }
  acc = acc_wave_reduce(acc, lf);
  if (lane != 0) return;
#if ACC_HAS_SEED
  const T seed = (ACC_SEED);
  ACC_SET(arrOut, seg, acc.ok ? f(acc.v, seed) : seed);
#else
  ACC_SET(arrOut, seg, acc.v);
#endif
}

#if !ACC_GIANTS && !ACC_SEG_UNIFORM && !ACC_SEG_OUTER
/* ---- is there a segment that a build with the table of jobs would hand over? ----
 * <entry>_probe, which the host launches behind <entry> on an instance's calls number 1, 2, 4, 8 ...: a look at the
 * segment lengths, and a word of host memory set if one of them is as long as that; the host then has variants 4 to
 * 7 built and takes them once they are there.  (The question asked inside <entry> -- a comparison a segment and a
 * store that never happens, wherever they stand -- costs the sparse matrix-vector product 1.1 us of 190.)  The
 * parameters of <entry>, and the word's address behind them. */
extern "C" __global__ void __launch_bounds__(ACC_BLOCK)
ACC_FS_CAT(ACC_FOLDSEG_ENTRY, _probe)(ACC_ENV_PARAMS
                                      const Int64 shOut_0, ACC_OUT_ARRAY(arrOut),
                                      ACC_SEG_PARAMS ACC_GUARD_PARAM, unsigned int *acc_hint)
{
  /* (what the kernels with the table take for such a segment: the staged one, and the teams of lanes) */
  const Int64 from = acc_max<Int64>(ACC_GIANT_FROM + 2 * ACC_CHUNK, ACC_GIANT_TIMES * (shIn_0 / acc_max<Int64>(shOut_0, 1)));
  for (Int64 s = (Int64)blockIdx.x * ACC_BLOCK + threadIdx.x; s < shOut_0; s += (Int64)gridDim.x * ACC_BLOCK)
    if ((Int64)arrSeg_0[s + 1] - (Int64)arrSeg_0[s] >= from) *acc_hint = 1u;
}
#endif

#if ACC_GIANTS
/* ---- the segments that were handed over -------------------------------------
 * <entry>_sweep, launched behind <entry> with as many workgroups as the device holds at once: they take the jobs'
 * pieces by ticket until none is left, and the workgroup that draws the ticket behind a job's last piece puts the
 * owner's value and the pieces together and writes the segment's result.  (As a part of <entry> -- every workgroup
 * looking at the table when its own segments were done -- this took 20 registers of it, and a segment met by the
 * workgroup that is started last found nobody left to take pieces.)  With an empty table the launch is a read of
 * 16 bytes a workgroup.  Same parameters as <entry>. */
extern "C" __global__ void __launch_bounds__(ACC_BLOCK)
ACC_FS_CAT(ACC_FOLDSEG_ENTRY, _sweep)(ACC_ENV_PARAMS
                                      const Int64 shOut_0, ACC_OUT_ARRAY(arrOut),
                                      ACC_SEG_PARAMS ACC_GIANT_PARAMS ACC_GUARD_PARAM)
{
  ACC_GUARD_CHECK
  typedef ACC_ELT T;
  ACC_ENV_ASSUME
  (void)shOut_0;
  (void)arrSeg_0;
  __shared__ __attribute__((aligned(16))) T s_val[ACC_PAD_SPACE(ACC_CHUNK)];
  __shared__ unsigned long long s_jobs[ACC_GIANT_JOBS][8 + ACC_GIANT_LINES], s_tick;
  __shared__ int s_pick;
  __shared__ acc_opt<T> s_part[ACC_BLOCK / ACC_WAVE];
  auto get = [&](const Int64 ix) -> T { return (ACC_GET(ix)); };
  auto f   = [&](const T &x, const T &y) -> T { return (ACC_COMBINE(x, y)); };
  auto lf  = acc_lift<T>(f);
  const Int64 n = ACC_SEG_TOTAL;
  const int tid = threadIdx.x;
#if ACC_HAS_SEED
  const T seed = (ACC_SEED);
#endif
  /* an ordered fold of s_val[from .. to) by all lanes: every lane a run of consecutive elements, the lanes joined in
   * lane order and the waves in wave order */
  auto together = [&](const int from, const int to) -> acc_opt<T> {
    constexpr int acc_pad_mask = ACC_PAD_ON ? ~0 : 0;
    const int per = (to - from + ACC_BLOCK - 1) / ACC_BLOCK;
    const int i0 = acc_min(from + tid * per, to), i1 = acc_min(i0 + per, to);
    acc_opt<T> m = acc_none<T>();
    for (int i = i0; i < i1; ++i) m = lf(m, acc_some(s_val[ACC_PAD(i)]));
    m = acc_wave_reduce(m, lf);
    if (acc_lane() == 0) s_part[tid >> 6] = m;
    __syncthreads();
    acc_opt<T> whole = s_part[0];
#pragma unroll
    for (int w = 1; w < ACC_BLOCK / ACC_WAVE; ++w) whole = lf(whole, s_part[w]);
    return whole;
  };
  /* elements [from, to) of the source folded by the whole workgroup, chunk by chunk in index order (to > from).
   * (The loads of two or four chunks in flight together make no piece faster: 36-39 us either way.) */
  auto fold_range = [&](const Int64 from, const Int64 to) -> acc_opt<T> {
    constexpr int acc_pad_mask = ACC_PAD_ON ? ~0 : 0;
    acc_opt<T> value = acc_none<T>();
    for (Int64 cs = from - from % ACC_VEC; cs < to; cs += ACC_CHUNK) {
      __syncthreads();                                              /* the chunk before has been read */
      {
        T w[ACC_LOADS][ACC_VEC];
        const bool whole = cs + ACC_CHUNK <= n;                     /* (the same in every lane) */
#pragma unroll
        for (int u = 0; u < ACC_LOADS; ++u)
#pragma unroll
          for (int k = 0; k < ACC_VEC; ++k) {
            const Int64 ix = cs + (u * ACC_BLOCK + tid) * ACC_VEC + k;
            w[u][k] = get(whole ? ix : acc_min<Int64>(ix, n - 1));  /* (what lies beyond `to` is never read back) */
          }
#pragma unroll
        for (int u = 0; u < ACC_LOADS; ++u)
#pragma unroll
          for (int k = 0; k < ACC_VEC; ++k) s_val[ACC_PAD((u * ACC_BLOCK + tid) * ACC_VEC + k)] = w[u][k];
      }
      __syncthreads();
      value = lf(value, together((int)(acc_max(from, cs) - cs), (int)(acc_min(to, cs + ACC_CHUNK) - cs)));
    }
    return value;
  };
  {
    const acc_tagged<T> pieces_of = {acc_jobs + ACC_GIANT_HEAD + ACC_GIANT_JOBS * ACC_GIANT_JOB};
    if (tid == 0) s_tick = __hip_atomic_load(acc_jobs, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
    __syncthreads();
    const unsigned long long head = s_tick;          /* {tag of the launch, jobs entered} */
    const int jobs_in = (unsigned int)(head >> 32) == acc_epoch ? (int)acc_min<unsigned int>((unsigned int)head, ACC_GIANT_JOBS) : 0;
    /* Tickets are drawn from ACC_GIANT_LINES counters a job, each for a run of `p_line` consecutive pieces: additions
     * to ONE word are performed one after the other, 0.1 us each, so that a thousand workgroups that ask for a ticket
     * at the same moment were handed theirs over 100 us.  A line has one ticket more than pieces: whoever draws it
     * knows that the line has run out, and a counter beyond it says so to everybody who looks.  And a look comes
     * before every ticket: a counter that has run out is not asked again -- thousands of workgroups that each drew a
     * ticket only to find the job done kept a launch busy for 200 us. */
    struct acc_job_shape { Int64 seg, a, b, p_first, p_count, p_line; };
    auto shape_of = [&](const unsigned long long *sj) -> acc_job_shape {
      auto whole_of = [&](const int k) -> Int64 { return (Int64)(((unsigned long long)(unsigned int)sj[5 + k] << 32) | (unsigned int)sj[1 + k]); };
      acc_job_shape g;
      g.seg = whole_of(0); g.a = whole_of(1); g.b = whole_of(2);
      g.p_first = g.a / ACC_GIANT_PIECE;
      g.p_count = (g.b - 1) / ACC_GIANT_PIECE - g.p_first + 1;
      g.p_line = (g.p_count + ACC_GIANT_LINES - 1) / ACC_GIANT_LINES;
      return g;
    };
    auto line_first = [&](const acc_job_shape &g, const int l) -> Int64 { return acc_min<Int64>((Int64)l * g.p_line, g.p_count); };
    auto line_count = [&](const acc_job_shape &g, const int l) -> Int64 { return acc_min<Int64>(line_first(g, l) + g.p_line, g.p_count) - line_first(g, l); };
    /* A round: a look at every job's words, all in one round trip; of the lines that have a ticket left the one
     * nearest to the job and the line that this workgroup's number names (so that the workgroups begin spread over
     * all of them); tickets of that line until it has run out.  Then the next round, until a look finds no line.
     * (Job after job, each looked at when its turn came, thirty segments of 2^18 elements took 240 us: most of a
     * workgroup's time went into finding out, one round trip a job, that the others had done it already.) */
    const int j0 = jobs_in > 0 ? (int)((blockIdx.x / ACC_GIANT_LINES) % (unsigned int)jobs_in) : 0, l0 = (int)(blockIdx.x % ACC_GIANT_LINES);
    for (int round = 0; round < 2 * ACC_GIANT_JOBS * ACC_GIANT_LINES && jobs_in > 0; ++round) {
      __syncthreads();                                              /* (the round before has read these words) */
      if (tid == 0) s_pick = 0x7fffffff;
      for (int i = tid; i < jobs_in * (8 + ACC_GIANT_LINES); i += ACC_BLOCK) {
        const int jn = i / (8 + ACC_GIANT_LINES), wn = i % (8 + ACC_GIANT_LINES);
        s_jobs[jn][wn] = __hip_atomic_load(acc_jobs + ACC_GIANT_HEAD + (Int64)jn * ACC_GIANT_JOB + (wn < 8 ? wn : 8 + (wn - 8) * ACC_GIANT_SPREAD),
                                           __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
      }
      __syncthreads();
      for (int c = tid; c < jobs_in * ACC_GIANT_LINES; c += ACC_BLOCK) {
        const int jn = c / ACC_GIANT_LINES, l = c % ACC_GIANT_LINES;
        const acc_job_shape g = shape_of(s_jobs[jn]);
        if ((unsigned int)(s_jobs[jn][0] >> 32) == acc_epoch && line_count(g, l) > 0 && (Int64)s_jobs[jn][8 + l] <= line_count(g, l))
          (void)__hip_atomic_fetch_min(&s_pick, ((jn - j0 + jobs_in) % jobs_in) * ACC_GIANT_LINES + (l - l0 + ACC_GIANT_LINES) % ACC_GIANT_LINES,
                                       __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_WORKGROUP);
      }
      __syncthreads();
      const int pick = s_pick;
      if (pick == 0x7fffffff) break;                                /* no line of any job has a ticket left */
      const int j = (j0 + pick / ACC_GIANT_LINES) % jobs_in, line = (l0 + pick % ACC_GIANT_LINES) % ACC_GIANT_LINES;
      unsigned long long *job = acc_jobs + ACC_GIANT_HEAD + (Int64)j * ACC_GIANT_JOB;
      const acc_job_shape g = shape_of(s_jobs[j]);
      const Int64 g_seg = g.seg, g_a = g.a, g_b = g.b, p_first = g.p_first, p_count = g.p_count;
      const Int64 lines_in_use = (p_count + g.p_line - 1) / g.p_line;
      /* Where a piece's value goes: two values for every piece of the source.  A handed-over segment is at least two
       * pieces long, so a piece of the source is shared by two of them at most -- one that ends in it and one that
       * begins in it -- and the one that begins there (its piece 0) takes the odd place. */
      auto slot_of = [&](const Int64 piece) -> unsigned int { return (unsigned int)(2 * (p_first + piece) + (piece == 0 ? 1 : 0)); };
      const Int64 l_first = line_first(g, line), l_count = line_count(g, line);
      for (;;) {
        __syncthreads();
        if (tid == 0) {
          unsigned long long t = __hip_atomic_fetch_add(job + 8 + line * ACC_GIANT_SPREAD, 1ull, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
          /* the ticket behind a line's last piece: one line more has run out; the last such line ends the job */
          if ((Int64)t == l_count &&
              (Int64)__hip_atomic_fetch_add(job + 4, 1ull, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT) + 1 == lines_in_use)
            t = ~0ull;
          s_tick = t;
        }
        __syncthreads();
        const Int64 ticket = s_tick == ~0ull ? -1 : (Int64)s_tick;
        if (ticket >= l_count) break;
        if (ticket < 0) {
          /* Every piece of every line has been drawn (whoever folds a piece asks for another ticket afterwards, so the
           * ticket behind a line's last piece is always drawn, and by one workgroup): the pieces are put together
           * here, in order.  Each is waited for by its tag -- the workgroups that drew them are running, or done. */
          const Int64 per = (p_count + ACC_BLOCK - 1) / ACC_BLOCK;
          const Int64 i0 = acc_min<Int64>((Int64)tid * per, p_count), i1 = acc_min<Int64>(i0 + per, p_count);
          acc_opt<T> m = acc_none<T>();
          for (Int64 i = i0; i < i1; ++i) m = lf(m, acc_some(pieces_of.wait(slot_of(i), acc_epoch, acc_status)));
          m = acc_wave_reduce(m, lf);
          if (acc_lane() == 0) s_part[tid >> 6] = m;
          __syncthreads();
          if (tid == 0) {
            acc_opt<T> whole = s_part[0];
#pragma unroll
            for (int w = 1; w < ACC_BLOCK / ACC_WAVE; ++w) whole = lf(whole, s_part[w]);
            /* and joined with what the owner folded itself before it handed the rest over, if it did */
            if ((unsigned int)s_jobs[j][0] == 1u) {
              const T edge = pieces_of.wait(acc_giant_edge_slot(n, j), acc_epoch, acc_status);
#if ACC_FOLD_RIGHT
              ACC_SET(arrOut, g_seg, f(whole.v, edge));             /* (a seed is in the owner's value already) */
#elif ACC_HAS_SEED
              ACC_SET(arrOut, g_seg, f(f(edge, whole.v), seed));
#else
              ACC_SET(arrOut, g_seg, f(edge, whole.v));
#endif
            } else {
#if ACC_HAS_SEED
              ACC_SET(arrOut, g_seg, f(whole.v, seed));             /* the seed is the last operand in either association */
#else
              ACC_SET(arrOut, g_seg, whole.v);
#endif
            }
          }
          break;
        }
        /* piece p_first + l_first + ticket of the source, as far as it belongs to the segment, chunk by chunk in index order */
        const Int64 piece = l_first + ticket;
        const Int64 from = acc_max(g_a, (p_first + piece) * ACC_GIANT_PIECE), to = acc_min(g_b, (p_first + piece + 1) * ACC_GIANT_PIECE);
        const acc_opt<T> value = fold_range(from, to);
        if (tid == 0) pieces_of.put(slot_of(piece), acc_epoch, value.v);
      }
    }   /* rounds */
  }
}
#endif
