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

#ifndef ACC_MAP_TILED
#define ACC_MAP_TILED 0
#endif

#if ACC_MAP_TILED
/*
 * The same result produced in square tiles of its two innermost dimensions (ACC_FLAG_TILED, rank >= 2), for element
 * functions that read their sources ACROSS rows -- a transposing backpermute above all, where a run of consecutive
 * result elements reads one element of as many source rows (IndexSpace.hs:96-141 evaluates in runs whatever the
 * index function does).  A wave takes a tile of 32 x 32 elements, its lanes 8 across and 8 down with a block of 4 x 4
 * each: a row of the tile is written in a run of 128 bytes (Float32), and a source read along the tile's columns is
 * read in runs of 128 bytes too (the four elements a lane reads down a column are consecutive there, and so are the
 * eight lanes below one another).  Tiles are numbered along the rows of the result, the waves of a workgroup side by
 * side.  (A workgroup that evaluates a tile of 64 x 64 down its columns, passes it through LDS and writes it along its
 * rows -- runs of 256 bytes both ways, but the direction of the source fixed -- transposes no faster: 8192 x 8192
 * Float32 in 123-130 us against 123-125, and 281 in runs.)
 */
#ifndef ACC_TT
#define ACC_TT 4                                      /* a lane's block is ACC_TT x ACC_TT */
#endif
#define ACC_TSIDE (8 * ACC_TT)                        /* a wave's tile is ACC_TSIDE x ACC_TSIDE */

extern "C" __global__ void __launch_bounds__(ACC_BLOCK)
ACC_ENTRY(ACC_ENV_PARAMS ACC_OUT_PARAMS ACC_GUARD_PARAM)
{
  ACC_GUARD_CHECK
  typedef ACC_ELT T;
  ACC_ENV_ASSUME
  auto get = [&](const Int64 ix) -> T { return (ACC_GET(ix)); };

  /* The tiles' second dimension is the second innermost one of the result, or one further out (ACC_TILE_H its
   * extent, ACC_TILE_STRIDE the elements between neighbours along it: a volume turned so that its innermost
   * dimension becomes its outermost reads its source along that one).  What lies between that dimension and the
   * innermost (`mids` rows for every place along it) and outside it (`outers`) is walked tile by tile. */
  const Int64 w = shOut_0, h = ACC_TILE_H, stride = ACC_TILE_STRIDE;
  const Int64 n = (ACC_OUT_SIZE);
  const Int64 mids = w > 0 ? stride / w : 0, outers = (h > 0 && stride > 0) ? n / (h * stride) : 0;
  const Int64 tiles_x = (w + ACC_TSIDE - 1) / ACC_TSIDE, tiles_y = (h + ACC_TSIDE - 1) / ACC_TSIDE;
  const Int64 tiles = tiles_x * tiles_y * mids * outers;
  const int lane = acc_lane();
  const int lx = lane & 7, ly = lane >> 3;
  const Int64 wave = (Int64)blockIdx.x * (ACC_BLOCK / ACC_WAVE) + (Int64)__builtin_amdgcn_readfirstlane((int)(threadIdx.x >> 6));
  const Int64 step = (Int64)gridDim.x * (ACC_BLOCK / ACC_WAVE);

  for (Int64 tile = wave; tile < tiles; tile += step) {
    const Int64 tx = tile % tiles_x, ty = (tile / tiles_x) % tiles_y, plane = tile / (tiles_x * tiles_y);
    const Int64 mid = plane % mids, outer = plane / mids;
    const Int64 x = tx * ACC_TSIDE + lx * ACC_TT, y = ty * ACC_TSIDE + ly * ACC_TT;
    const Int64 base = ((outer * h + y) * mids + mid) * w + x;
    if ((tx + 1) * ACC_TSIDE <= w && (ty + 1) * ACC_TSIDE <= h) {
      T v[ACC_TT][ACC_TT];
      /* down the columns first: what a transposed source holds side by side */
#pragma unroll
      for (int k = 0; k < ACC_TT; ++k)
#pragma unroll
        for (int i = 0; i < ACC_TT; ++i) v[i][k] = get(base + i * stride + k);
#pragma unroll
      for (int i = 0; i < ACC_TT; ++i)
#pragma unroll
        for (int k = 0; k < ACC_TT; ++k) ACC_SET(arrOut, base + i * stride + k, v[i][k]);
    } else {
#pragma unroll
      for (int i = 0; i < ACC_TT; ++i)
#pragma unroll
        for (int k = 0; k < ACC_TT; ++k)
          if (x + k < w && y + i < h) ACC_SET(arrOut, base + i * stride + k, get(base + i * stride + k));
    }
  }
}

#else

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

#endif   /* ACC_MAP_TILED */
