/*
 * skel_fold.h -- fold / fold1: reduction of a whole array to one value
 * (entry foldAll / fold1All).  Reduction along the innermost dimension of a
 * rank > 1 array is skel_foldseg.h with segments of one length.
 *
 * Takes the place of CodeGen/Reduction.hs:87-215 (mkFoldAll: a first kernel
 * plus a recursive second one, Execute.hs:291-318) and of the shared-memory
 * tree reducers at :616-699.
 *
 * foldAll: every block strides over tiles of the (fused) input, each lane
 * reading ACC_UNROLL independent groups of ACC_VEC consecutive elements per
 * tile; lanes are combined with a wave64 DPP reduction, waves through a few
 * words of LDS, and each block leaves one partial result in global memory.
 * With ACC_FOLD_SINGLE (the default) that is all one launch: the partial
 * travels as tagged 64-bit words and the last block collects the others'
 * and applies the seed; without it a second, single-block launch of
 * <entry>_finish does (a lone block finishes the job itself either way).
 * Blocks never meet on an atomic or behind a fence: same-address device-scope
 * atomics cost tens of nanoseconds each on this part and a release/acquire
 * pair a cache-wide write-back and invalidate; and with a fixed grid the
 * association order, hence the Float32 result, is reproducible from run to
 * run.  As in the reference
 * the operator must be associative AND commutative here (the striding
 * reorders elements, Reduction.hs:160-165), it needs no identity, the seed
 * enters once as the second operand (Reduction.hs:203-211) and an empty input
 * yields the seed (:212-214).
 *
 * Generated definitions expected: ACC_ENTRY, ACC_ELT, ACC_ENV_PARAMS,
 * ACC_ENV_ASSUME, ACC_GET(ix), ACC_COMBINE(x,y), ACC_HAS_SEED, ACC_SEED,
 * ACC_BLOCK, ACC_VEC, ACC_UNROLL, ACC_FOLD_SINGLE.
 */

#define ACC_TILE  (ACC_BLOCK * ACC_VEC * ACC_UNROLL)
#define ACC_WAVES (ACC_BLOCK / ACC_WAVE)

/* combine the optional per-thread values of a block; result valid in every thread */
template <typename T, typename F>
ACC_DEV acc_opt<T> acc_block_reduce(acc_opt<T> x, F f, acc_opt<T> *s_wave)
{
  auto lf = acc_lift<T>(f);
  const int lane = acc_lane();
  const int wave = (int)(threadIdx.x >> 6);
  x = acc_wave_reduce(x, lf);
  if (lane == 0) s_wave[wave] = x;
  __syncthreads();
  acc_opt<T> r = s_wave[0];
#pragma unroll
  for (int w = 1; w < ACC_WAVES; ++w) r = lf(r, s_wave[w]);
  __syncthreads();
  return r;
}

extern "C" __global__ void __launch_bounds__(ACC_BLOCK)
ACC_ENTRY(ACC_ENV_PARAMS
          ACC_OUT_ARRAY(arrOut),
          const Int64 shIn_0,
#if ACC_FOLD_SINGLE
          unsigned long long *partials, const unsigned int epoch, unsigned int *acc_status ACC_GUARD_PARAM)
#else
          ACC_ELT *__restrict__ partials ACC_GUARD_PARAM)
#endif
{
  ACC_GUARD_CHECK
  typedef ACC_ELT T;
  ACC_ENV_ASSUME
  __shared__ acc_opt<T> s_wave[ACC_WAVES];

  auto get = [&](const Int64 ix) -> T { return (ACC_GET(ix)); };
  auto f   = [&](const T &x, const T &y) -> T { return (ACC_COMBINE(x, y)); };
  auto lf  = acc_lift<T>(f);

  const Int64 n = shIn_0;
  const Int64 full_tiles = n / ACC_TILE;

  /* full tiles: no bounds checks, ACC_UNROLL independent accumulators */
  T a[ACC_UNROLL];
  bool have = false;
  Int64 tile = blockIdx.x;
  if (tile < full_tiles) {
    const Int64 base = tile * (Int64)ACC_TILE + (Int64)threadIdx.x * ACC_VEC;
#pragma unroll
    for (int u = 0; u < ACC_UNROLL; ++u) {
      T v = get(base + u * (ACC_BLOCK * ACC_VEC));
#pragma unroll
      for (int k = 1; k < ACC_VEC; ++k) v = f(v, get(base + u * (ACC_BLOCK * ACC_VEC) + k));
      a[u] = v;
    }
    have = true;
    for (tile += gridDim.x; tile < full_tiles; tile += gridDim.x) {
      const Int64 b2 = tile * (Int64)ACC_TILE + (Int64)threadIdx.x * ACC_VEC;
      T v[ACC_UNROLL][ACC_VEC];
#pragma unroll
      for (int u = 0; u < ACC_UNROLL; ++u)
#pragma unroll
        for (int k = 0; k < ACC_VEC; ++k) v[u][k] = get(b2 + u * (ACC_BLOCK * ACC_VEC) + k);
#pragma unroll
      for (int u = 0; u < ACC_UNROLL; ++u)
#pragma unroll
        for (int k = 0; k < ACC_VEC; ++k) a[u] = f(a[u], v[u][k]);
    }
  }

  acc_opt<T> mine = acc_none<T>();
  if (have) {
    T v = a[0];
#pragma unroll
    for (int u = 1; u < ACC_UNROLL; ++u) v = f(v, a[u]);
    mine = acc_some(v);
  }

  /* the ragged last tile, taken by whichever block it falls to ...
   * but not by the last block of a larger grid, which collects the partial results and should not be late */
  Int64 ragged_owner = full_tiles % gridDim.x;
  if (gridDim.x > 1 && ragged_owner == (Int64)gridDim.x - 1) ragged_owner = 0;
  if (full_tiles * (Int64)ACC_TILE < n && (Int64)blockIdx.x == ragged_owner) {
    const Int64 base = full_tiles * (Int64)ACC_TILE + (Int64)threadIdx.x * ACC_VEC;
    /* every load is issued before any value is used: positions past the end read the last element instead and are
     * left out below (a load under `if (ix < n)` waits for its result inside the branch, one round trip each) */
    T v[ACC_UNROLL][ACC_VEC];
#pragma unroll
    for (int u = 0; u < ACC_UNROLL; ++u)
#pragma unroll
      for (int k = 0; k < ACC_VEC; ++k) v[u][k] = get(acc_min<Int64>(base + u * (ACC_BLOCK * ACC_VEC) + k, n - 1));
#pragma unroll
    for (int u = 0; u < ACC_UNROLL; ++u)
#pragma unroll
      for (int k = 0; k < ACC_VEC; ++k) {
        const Int64 ix = base + u * (ACC_BLOCK * ACC_VEC) + k;
        if (ix < n) mine = lf(mine, acc_some(v[u][k]));
      }
  }

  acc_opt<T> total = acc_block_reduce(mine, f, s_wave);

#if ACC_FOLD_SINGLE
  /* One launch: every block but the last leaves its partial result, tagged with this launch's epoch
   * (whatever an earlier launch left carries an older one); the last block collects them.  The grid
   * never exceeds what is resident at once, so nobody waits for a place on the device meanwhile.   */
  if (gridDim.x > 1) {
    const acc_tagged<T> slots = {partials};
    const unsigned int last = gridDim.x - 1;
    if (blockIdx.x != last) {
      if (threadIdx.x == 0) slots.put(blockIdx.x, epoch, total.v);   /* the host guarantees every block owns >= 1 element */
      return;
    }
    acc_opt<T> p = threadIdx.x == 0 ? total : acc_none<T>();
    for (unsigned int i = threadIdx.x; i < last; i += ACC_BLOCK) p = lf(p, acc_some(slots.wait(i, epoch, acc_status)));
    total = acc_block_reduce(p, f, s_wave);
  }
  if (threadIdx.x != 0) return;
#else
  if (threadIdx.x != 0) return;
  if (gridDim.x > 1) {
    partials[blockIdx.x] = total.v;              /* the host guarantees every block owns >= 1 element */
    return;
  }
#endif
#if ACC_HAS_SEED
  const T seed = (ACC_SEED);
  ACC_SET(arrOut, 0, total.ok ? f(total.v, seed) : seed);
#else
  ACC_SET(arrOut, 0, total.v);
#endif
}

#define ACC_CAT2(a, b) a##b
#define ACC_CAT(a, b) ACC_CAT2(a, b)

/* second launch: one block folds the `count` partial results */
extern "C" __global__ void __launch_bounds__(ACC_BLOCK)
ACC_CAT(ACC_ENTRY, _finish)(ACC_ENV_PARAMS
                            ACC_OUT_ARRAY(arrOut),
                            const ACC_ELT *__restrict__ partials, const Int64 count ACC_GUARD_PARAM)
{
  ACC_GUARD_CHECK
  typedef ACC_ELT T;
  ACC_ENV_ASSUME
  __shared__ acc_opt<T> s_wave[ACC_WAVES];
  auto f  = [&](const T &x, const T &y) -> T { return (ACC_COMBINE(x, y)); };
  auto lf = acc_lift<T>(f);
  acc_opt<T> p = acc_none<T>();
  for (Int64 i = threadIdx.x; i < count; i += ACC_BLOCK) p = lf(p, acc_some(partials[i]));
  const acc_opt<T> total = acc_block_reduce(p, f, s_wave);
  if (threadIdx.x != 0) return;
#if ACC_HAS_SEED
  const T seed = (ACC_SEED);
  ACC_SET(arrOut, 0, total.ok ? f(total.v, seed) : seed);
#else
  ACC_SET(arrOut, 0, total.v);
#endif
}
