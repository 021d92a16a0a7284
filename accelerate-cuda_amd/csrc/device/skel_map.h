/*
 * skel_map.h -- map / zipWith / generate / transform / backpermute.
 *
 * Takes the place of CodeGen/Mapping.hs:39-78 (map), CodeGen/IndexSpace.hs:47-83
 * (generate) and :96-141 (transform; backpermute is transform with the identity
 * function, CodeGen.hs:101).  After fusion all of them are "for every linear
 * index ix of the result, out[ix] = get(ix)", where `get` is the generated
 * fragment (an element function applied to delayed inputs, an index
 * permutation followed by a read, or a pure function of the index), so one
 * template serves the three entry points.
 *
 * Each thread handles ACC_UNROLL groups of ACC_VEC consecutive elements; a
 * full tile runs without bounds checks so that reads of manifest arrays and
 * the writes merge into 128-bit accesses, and the ACC_UNROLL independent
 * groups keep several of them in flight per lane.
 *
 * Generated definitions expected: ACC_ENTRY, ACC_ELT, ACC_ENV_PARAMS,
 * ACC_ENV_ASSUME, ACC_OUT_PARAMS, ACC_OUT_SIZE, ACC_GET(ix), ACC_BLOCK, ACC_VEC,
 * ACC_UNROLL, ACC_ALIGNED.
 */

#define ACC_TILE (ACC_BLOCK * ACC_VEC * ACC_UNROLL)

extern "C" __global__ void __launch_bounds__(ACC_BLOCK)
ACC_ENTRY(ACC_ENV_PARAMS ACC_OUT_PARAMS ACC_GUARD_PARAM)
{
  ACC_GUARD_CHECK
  typedef ACC_ELT T;
  ACC_ENV_ASSUME
#if ACC_ALIGNED
  ACC_OUT_ASSUME(arrOut)
#endif
  auto get = [&](const Int64 ix) -> T { return (ACC_GET(ix)); };

  const Int64 n = (ACC_OUT_SIZE);
  const Int64 num_tiles = (n + ACC_TILE - 1) / ACC_TILE;

  for (Int64 tile = blockIdx.x; tile < num_tiles; tile += gridDim.x) {
    const Int64 base = tile * (Int64)ACC_TILE + (Int64)threadIdx.x * ACC_VEC;
    if ((tile + 1) * (Int64)ACC_TILE <= n) {
      T v[ACC_UNROLL][ACC_VEC];
#pragma unroll
      for (int u = 0; u < ACC_UNROLL; ++u)
#pragma unroll
        for (int k = 0; k < ACC_VEC; ++k) v[u][k] = get(base + u * (ACC_BLOCK * ACC_VEC) + k);
#pragma unroll
      for (int u = 0; u < ACC_UNROLL; ++u)
#pragma unroll
        for (int k = 0; k < ACC_VEC; ++k) ACC_PUT(arrOut, base + u * (ACC_BLOCK * ACC_VEC) + k, v[u][k]);
    } else {
#pragma unroll
      for (int u = 0; u < ACC_UNROLL; ++u)
#pragma unroll
        for (int k = 0; k < ACC_VEC; ++k) {
          const Int64 ix = base + u * (ACC_BLOCK * ACC_VEC) + k;
          if (ix < n) ACC_SET(arrOut, ix, get(ix));
        }
    }
  }
}
