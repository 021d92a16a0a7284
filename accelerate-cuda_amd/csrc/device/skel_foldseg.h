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

#if ACC_HAS_SEED
#define ACC_FOLDSEG_ENTRY foldSeg
#else
#define ACC_FOLDSEG_ENTRY fold1Seg
#endif

#define ACC_LOADS (ACC_CHUNK / (ACC_BLOCK * ACC_VEC))   /* vector loads per lane and chunk */
#define ACC_EAT 8                                        /* LDS reads kept in flight while folding */

extern "C" __global__ void __launch_bounds__(ACC_BLOCK)
ACC_FOLDSEG_ENTRY(ACC_ENV_PARAMS
                  const Int64 shOut_0, ACC_OUT_ARRAY(arrOut),
                  const Int64 shIn_0,
                  const ACC_SEG_TYPE *__restrict__ arrSeg_0)
{
  typedef ACC_ELT T;
  ACC_ENV_ASSUME
  __shared__ __attribute__((aligned(16))) T s_val[ACC_CHUNK];

  auto get = [&](const Int64 ix) -> T { return (ACC_GET(ix)); };
  auto f   = [&](const T &x, const T &y) -> T { return (ACC_COMBINE(x, y)); };

  const Int64 nseg = shOut_0;
  const Int64 n = shIn_0;
  const int tid = threadIdx.x;
#if ACC_HAS_SEED
  const T seed = (ACC_SEED);
#endif

  for (Int64 first = (Int64)blockIdx.x * ACC_BLOCK; first < nseg; first += (Int64)gridDim.x * ACC_BLOCK) {
    const Int64 seg = first + tid;
    const bool live = seg < nseg;
    const Int64 a = live ? (Int64)arrSeg_0[seg] : 0;
    const Int64 b = live ? (Int64)arrSeg_0[seg + 1] : 0;
    const Int64 last = acc_min<Int64>(first + ACC_BLOCK, nseg);
    const Int64 lo = (Int64)arrSeg_0[first], hi = acc_min<Int64>((Int64)arrSeg_0[last], n);

    T acc = T();
    bool have = false;
#if ACC_HAS_SEED && ACC_FOLD_RIGHT
    acc = seed;
    have = true;
#endif

    /* chunks start on a vector boundary so that the loads stay aligned */
    const Int64 lo_al = lo - (lo % ACC_VEC);
    const Int64 nchunks = hi > lo_al ? (hi - lo_al + ACC_CHUNK - 1) / ACC_CHUNK : 0;
    /* stage a chunk: every load is issued before any result is used.  Elements
     * of the chunk's first and last vector that belong to a neighbouring block
     * are loaded too (they exist) and never read back; only the very end of
     * the array needs a guard. */
    T v[ACC_LOADS][ACC_VEC];
    auto chunk_start = [&](const Int64 q) -> Int64 { return lo_al + (ACC_FOLD_RIGHT ? (nchunks - 1 - q) : q) * (Int64)ACC_CHUNK; };
    auto stage = [&](const Int64 cs) {
      if (cs + ACC_CHUNK <= n) {
#pragma unroll
        for (int u = 0; u < ACC_LOADS; ++u)
#pragma unroll
          for (int k = 0; k < ACC_VEC; ++k) v[u][k] = get(cs + (u * ACC_BLOCK + tid) * ACC_VEC + k);
      } else {
#pragma unroll
        for (int u = 0; u < ACC_LOADS; ++u)
#pragma unroll
          for (int k = 0; k < ACC_VEC; ++k) {
            const Int64 ix = cs + (u * ACC_BLOCK + tid) * ACC_VEC + k;
            v[u][k] = T();
            if (ix < n) v[u][k] = get(ix);
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
#pragma unroll
        for (int k = 0; k < ACC_VEC; ++k) s_val[(u * ACC_BLOCK + tid) * ACC_VEC + k] = v[u][k];
      __syncthreads();
      /* the next chunk's loads (and the gathers behind them) travel while this one is folded */
      if (q + 1 < nchunks) stage(chunk_start(q + 1));

      /* fold this lane's segment, as far as it lies in the chunk, in index order */
      int p0 = (int)(acc_max(a, cs) - cs), p1 = (int)(acc_min(b, ce) - cs);
#if ACC_FOLD_RIGHT
      if (!have && p0 < p1) { acc = s_val[--p1]; have = true; }
      for (; p1 - ACC_EAT >= p0; p1 -= ACC_EAT) {
        T w[ACC_EAT];
#pragma unroll
        for (int k = 0; k < ACC_EAT; ++k) w[k] = s_val[p1 - 1 - k];
#pragma unroll
        for (int k = 0; k < ACC_EAT; ++k) acc = f(w[k], acc);
      }
      for (; p1 > p0; --p1) acc = f(s_val[p1 - 1], acc);
#else
      if (!have && p0 < p1) { acc = s_val[p0++]; have = true; }
      for (; p0 + ACC_EAT <= p1; p0 += ACC_EAT) {
        T w[ACC_EAT];
#pragma unroll
        for (int k = 0; k < ACC_EAT; ++k) w[k] = s_val[p0 + k];
#pragma unroll
        for (int k = 0; k < ACC_EAT; ++k) acc = f(acc, w[k]);
      }
      for (; p0 < p1; ++p0) acc = f(acc, s_val[p0]);
#endif
    }

    if (live) {
#if ACC_HAS_SEED && !ACC_FOLD_RIGHT
      ACC_SET(arrOut, seg, have ? f(acc, seed) : seed);
#else
      ACC_SET(arrOut, seg, acc);      /* fold1Seg of an empty segment is undefined; T() is written */
#endif
    }
  }
}
