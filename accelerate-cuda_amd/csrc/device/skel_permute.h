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
 *     LDS atomics and reach global memory once per block, at the end, so hot
 *     targets (a 256-bin histogram, the head of a skewed one) do not queue up
 *     on one memory-side atomic unit.  A target that fits entirely gets
 *     `lds_copies` replicas, one per group of waves, to thin out same-address
 *     collisions inside a block.  Privatisation needs an identity for the
 *     combine, so it is only used with a hint.
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

#define ACC_HINT_GENERIC 0
#define ACC_HINT_ADD 1
#define ACC_HINT_MIN 2
#define ACC_HINT_MAX 3
#define ACC_HINT_AND 4
#define ACC_HINT_OR  5
#define ACC_HINT_XOR 6

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

/* one atomic application of the hinted operator; P is a global or LDS pointer */
template <typename T, typename F>
ACC_DEV void acc_hint_apply(T *p, const T &x, F combine)
{
#if ACC_ELT_IS_INTEGER && ACC_COMBINE_HINT != ACC_HINT_GENERIC
  typedef typename acc_bits<sizeof(T)>::type U;
  (void)combine;
#if ACC_COMBINE_HINT == ACC_HINT_ADD
  atomicAdd((U *)p, (U)x);
#elif ACC_COMBINE_HINT == ACC_HINT_AND
  atomicAnd((U *)p, (U)x);
#elif ACC_COMBINE_HINT == ACC_HINT_OR
  atomicOr((U *)p, (U)x);
#elif ACC_COMBINE_HINT == ACC_HINT_XOR
  atomicXor((U *)p, (U)x);
#elif ACC_COMBINE_HINT == ACC_HINT_MIN
  if (T(-1) < T(0)) { if (sizeof(T) == 4) atomicMin((int *)p, (int)x); else atomicMin((long long *)p, (long long)x); }
  else atomicMin((U *)p, (U)x);
#elif ACC_COMBINE_HINT == ACC_HINT_MAX
  if (T(-1) < T(0)) { if (sizeof(T) == 4) atomicMax((int *)p, (int)x); else atomicMax((long long *)p, (long long)x); }
  else atomicMax((U *)p, (U)x);
#endif
#elif !ACC_ELT_IS_INTEGER && ACC_COMBINE_HINT == ACC_HINT_ADD
  (void)combine;
  atomicAdd(p, x);
#else
  acc_atomic_rmw(p, x, combine);
#endif
}

extern "C" __global__ void __launch_bounds__(ACC_BLOCK)
permute(ACC_ENV_PARAMS ACC_OUT_PARAMS, const Int64 shIn_0, const int lds_bins, const int lds_copies)
{
  typedef ACC_ELT T;
  ACC_ENV_ASSUME
  extern __shared__ __attribute__((aligned(16))) unsigned char acc_lds_raw[];
  T *bins = (T *)acc_lds_raw;

  auto get  = [&](const Int64 ix) -> T { return (ACC_GET(ix)); };
  auto perm = [&](const Int64 ix) -> Int64 { return (Int64)(ACC_PERMUTATION(ix)); };
  auto f    = [&](const T &x, const T &y) -> T { return (ACC_COMBINE(x, y)); };

  const Int64 n = shIn_0;
  const Int64 ntarget = (ACC_OUT_SIZE);
  const T ident = acc_hint_identity<T>();

  for (int i = threadIdx.x; i < lds_bins * lds_copies; i += ACC_BLOCK) bins[i] = ident;
  __syncthreads();
  T *mine = bins + ((threadIdx.x >> 6) % lds_copies) * lds_bins;

  auto update = [&](const Int64 j, const T &x) {
    if (j < 0 || j >= ntarget) return;            /* `ignore`, or outside the result */
    if (j < lds_bins) acc_hint_apply(mine + j, x, f);
    else              acc_hint_apply(arrOut_0 + j, x, f);
  };

  const Int64 num_tiles = (n + ACC_TILE - 1) / ACC_TILE;
  for (Int64 tile = blockIdx.x; tile < num_tiles; tile += gridDim.x) {
    const Int64 base = tile * (Int64)ACC_TILE + (Int64)threadIdx.x * ACC_VEC;
    if ((tile + 1) * (Int64)ACC_TILE <= n) {
      Int64 j[ACC_UNROLL][ACC_VEC];
      T x[ACC_UNROLL][ACC_VEC];
#pragma unroll
      for (int u = 0; u < ACC_UNROLL; ++u)
#pragma unroll
        for (int k = 0; k < ACC_VEC; ++k) {
          const Int64 ix = base + u * (ACC_BLOCK * ACC_VEC) + k;
          j[u][k] = perm(ix);
          x[u][k] = get(ix);
        }
#pragma unroll
      for (int u = 0; u < ACC_UNROLL; ++u)
#pragma unroll
        for (int k = 0; k < ACC_VEC; ++k) update(j[u][k], x[u][k]);
    } else {
#pragma unroll
      for (int u = 0; u < ACC_UNROLL; ++u)
#pragma unroll
        for (int k = 0; k < ACC_VEC; ++k) {
          const Int64 ix = base + u * (ACC_BLOCK * ACC_VEC) + k;
          if (ix < n) update(perm(ix), get(ix));
        }
    }
  }

  /* flush the privatised part: one global atomic per touched target */
  if (lds_bins > 0) {
    __syncthreads();
    for (int i = threadIdx.x; i < lds_bins; i += ACC_BLOCK) {
      T acc = bins[i];
      for (int c = 1; c < lds_copies; ++c) acc = f(bins[c * lds_bins + i], acc);
      typename acc_bits<sizeof(T)>::type a, b;
      __builtin_memcpy(&a, &acc, sizeof(T));
      __builtin_memcpy(&b, &ident, sizeof(T));
      if (a != b) acc_hint_apply(arrOut_0 + i, acc, f);
    }
  }
}
