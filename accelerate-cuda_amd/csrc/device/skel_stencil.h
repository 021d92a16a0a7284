/*
 * skel_stencil.h -- 1-D and 2-D stencils: every element of the result is a
 * function of the elements of the source at fixed offsets from it.
 *
 * Takes the place of CodeGen/Stencil.hs:55-114 and the access generator of
 * CodeGen/Stencil/Extra.hs:53-128.  The reference reads every tap straight
 * from global memory (relying on the L1 cache, Context.hs:61-68), recovers the
 * multidimensional index with 64-bit divisions and tests a whole warp for
 * "interior" (Stencil.hs:103-110).  Here a workgroup stages a
 * (ACC_TILE_H + 2 ry) x (ACC_TILE_W + 2 rx) patch of the source in LDS once
 * -- 128-bit loads for the body of each row, a handful of scalar loads for the
 * halo columns -- and every tap is an LDS read.  Only tiles that touch the
 * array's edge apply the boundary condition, while they fill the patch; the
 * index maps are exactly those of Stencil/Extra.hs:191-226:
 *     clamp    max(0, min(i, sz-1))
 *     mirror   i < 0 ? -i : i >= sz ? sz - (i - sz + 2) : i
 *     wrap     i < 0 ? sz + i : i >= sz ? i - sz : i
 *     constant out-of-range taps read the constant
 * Each lane produces ACC_VEC consecutive results of a row and a workgroup
 * walks down its tile ACC_BLOCK / (ACC_TILE_W / ACC_VEC) rows at a time.
 *
 * Generated definitions expected: ACC_ELT, ACC_IN_ELT, ACC_ENV_PARAMS,
 * ACC_ENV_ASSUME, ACC_OUT_PARAMS, ACC_STENCIL_RANK (1|2), ACC_RADIUS_Y,
 * ACC_RADIUS_X, ACC_BOUNDARY, ACC_BOUNDARY_CONSTANT, ACC_STENCIL_TAPS(READ),
 * ACC_STENCIL_FN, ACC_TILE_W, ACC_TILE_H, ACC_BLOCK, ACC_ALIGNED.
 */

#define ACC_SVEC 4                                     /* results per lane and row */
#define ACC_TPR  (ACC_TILE_W / ACC_SVEC)               /* lanes per tile row */
#define ACC_RPP  (ACC_BLOCK / ACC_TPR)                 /* tile rows per pass */
#define ACC_LW   (ACC_TILE_W + 2 * ACC_RADIUS_X)
#define ACC_LH   (ACC_TILE_H + 2 * ACC_RADIUS_Y)
#define ACC_LPITCH (ACC_LW + ((4 - (ACC_LW & 3)) & 3) + 4)   /* keep rows 16-byte aligned, skew banks */
#define ACC_LX0  4                                     /* LDS column of tile column 0 (>= rx, multiple of 4) */

static_assert(ACC_TILE_W % ACC_SVEC == 0 && ACC_BLOCK % ACC_TPR == 0 && ACC_TILE_H % ACC_RPP == 0, "tile shape does not divide among the lanes");
static_assert(ACC_RADIUS_X <= ACC_LX0, "stencil too wide for the patch layout");

#define ACC_B_CLAMP 0
#define ACC_B_MIRROR 1
#define ACC_B_WRAP 2
#define ACC_B_CONSTANT 3

ACC_DEV Int64 acc_boundary_index(Int64 i, const Int64 sz)
{
#if ACC_BOUNDARY == ACC_B_CLAMP
  i = acc_max<Int64>(0, acc_min<Int64>(i, sz - 1));
#elif ACC_BOUNDARY == ACC_B_MIRROR
  i = i < 0 ? -i : (i >= sz ? sz - (i - sz + 2) : i);
#elif ACC_BOUNDARY == ACC_B_WRAP
  i = i < 0 ? sz + i : (i >= sz ? i - sz : i);
#endif
  /* positions of a ragged tile that no valid result reads may still lie
   * outside; keep the address legal */
  return acc_max<Int64>(0, acc_min<Int64>(i, sz - 1));
}

struct __attribute__((aligned(16))) acc_in_vec { ACC_IN_ELT v[ACC_SVEC]; };
struct __attribute__((aligned(16))) acc_out_vec { ACC_ELT v[ACC_SVEC]; };

extern "C" __global__ void __launch_bounds__(ACC_BLOCK)
stencil(ACC_ENV_PARAMS ACC_OUT_PARAMS, const ACC_IN_ELT *__restrict__ arrStencil_0)
{
  typedef ACC_ELT T;
  typedef ACC_IN_ELT S;
  ACC_ENV_ASSUME
  __shared__ __attribute__((aligned(16))) S patch[ACC_LH][ACC_LPITCH];

#if ACC_STENCIL_RANK == 2
  const Int64 h = shOut_1, w = shOut_0;
#else
  const Int64 h = 1, w = shOut_0;
#endif
  const Int64 tiles_x = (w + ACC_TILE_W - 1) / ACC_TILE_W;
  const Int64 ty = (Int64)blockIdx.x / tiles_x, tx = (Int64)blockIdx.x % tiles_x;
  const Int64 y0 = ty * ACC_TILE_H, x0 = tx * ACC_TILE_W;

  const int tid = threadIdx.x;
  const bool interior = (y0 - ACC_RADIUS_Y >= 0) && (y0 + ACC_TILE_H + ACC_RADIUS_Y <= h) &&
                        (x0 - ACC_RADIUS_X >= 0) && (x0 + ACC_TILE_W + ACC_RADIUS_X <= w);

  /* ---- stage the patch ---------------------------------------------------- */
  if (interior) {
    /* body of every patch row: one vector per lane */
    for (int i = tid; i < ACC_LH * ACC_TPR; i += ACC_BLOCK) {
      const int ly = i / ACC_TPR, c = i % ACC_TPR;
      const S *src = arrStencil_0 + (y0 - ACC_RADIUS_Y + ly) * w + x0 + c * ACC_SVEC;
#if ACC_ALIGNED
      *(acc_in_vec *)&patch[ly][ACC_LX0 + c * ACC_SVEC] = *(const acc_in_vec *)src;
#else
#pragma unroll
      for (int k = 0; k < ACC_SVEC; ++k) patch[ly][ACC_LX0 + c * ACC_SVEC + k] = src[k];
#endif
    }
    /* halo columns */
    if (ACC_RADIUS_X > 0) {
      for (int i = tid; i < ACC_LH * 2 * ACC_RADIUS_X; i += ACC_BLOCK) {
        const int ly = i / (2 * ACC_RADIUS_X), e = i % (2 * ACC_RADIUS_X);
        const int lx = (e < ACC_RADIUS_X) ? (e - ACC_RADIUS_X) : (ACC_TILE_W + e - ACC_RADIUS_X);   /* relative to tile column 0 */
        patch[ly][ACC_LX0 + lx] = arrStencil_0[(y0 - ACC_RADIUS_Y + ly) * w + x0 + lx];
      }
    }
  } else {
    for (int i = tid; i < ACC_LH * ACC_LW; i += ACC_BLOCK) {
      const int ly = i / ACC_LW, lx = i % ACC_LW - ACC_RADIUS_X;
      const Int64 gy = y0 - ACC_RADIUS_Y + ly, gx = x0 + lx;
#if ACC_BOUNDARY == ACC_B_CONSTANT
      const bool inside = gy >= 0 && gy < h && gx >= 0 && gx < w;
      const S v = inside ? arrStencil_0[gy * w + gx] : (S)(ACC_BOUNDARY_CONSTANT);
#else
      const S v = arrStencil_0[acc_boundary_index(gy, h) * w + acc_boundary_index(gx, w)];
#endif
      patch[ly][ACC_LX0 + lx] = v;
    }
  }
  __syncthreads();

  /* ---- evaluate ------------------------------------------------------------- */
  const int c = tid % ACC_TPR, r0 = tid / ACC_TPR;
#pragma unroll
  for (int p = 0; p < ACC_TILE_H / ACC_RPP; ++p) {
    const int r = r0 + p * ACC_RPP;
    const Int64 gy = y0 + r, gx = x0 + c * ACC_SVEC;
    acc_out_vec res;
#pragma unroll
    for (int k = 0; k < ACC_SVEC; ++k) {
#define ACC_PATCH_READ(dy, dx) patch[r + ACC_RADIUS_Y + (dy)][ACC_LX0 + c * ACC_SVEC + k + (dx)]
      ACC_STENCIL_TAPS(ACC_PATCH_READ)
#undef ACC_PATCH_READ
      res.v[k] = (T)(ACC_STENCIL_FN);
    }
    if (gy < h) {
      T *dst = arrOut_0 + gy * w + gx;
#if ACC_ALIGNED
      if (gx + ACC_SVEC <= w) *(acc_out_vec *)dst = res;
      else
#endif
      {
#pragma unroll
        for (int k = 0; k < ACC_SVEC; ++k)
          if (gx + k < w) dst[k] = res.v[k];
      }
    }
  }
}
