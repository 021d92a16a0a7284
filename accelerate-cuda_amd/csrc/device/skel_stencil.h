/*
 * skel_stencil.h -- 1-D and 2-D stencils: every element of the result is a
 * function of the elements of the source at fixed offsets from it.
 *
 * Takes the place of CodeGen/Stencil.hs:55-114 and the access generator of
 * CodeGen/Stencil/Extra.hs:53-128.  The reference reads every tap straight
 * from global memory (relying on the L1 cache, Context.hs:61-68), recovers the
 * multidimensional index with 64-bit divisions and tests a whole warp for
 * "interior" (Stencil.hs:103-110).  Here the work is cut into strips: one
 * 64-lane wave owns 256 columns (4 per lane) and walks down ACC_TILE_H rows,
 * keeping the 2 ry + 1 source rows it currently needs in registers:
 *   - every source row is fetched once per strip with one 128-bit load per
 *     lane, ACC_PREFETCH rows ahead of its use, so a wave always has several
 *     kilobytes in flight and never waits at a barrier;
 *   - taps to the left and right come from the neighbouring lanes' registers
 *     through DPP wave shifts; the rx elements just outside the strip, for
 *     all its rows, are fetched by one gather at the start and handed to the
 *     strip's first and last lane with readlane;
 *   - taps above and below are simply older and newer rows of the register
 *     window, which rotates by renaming (the row loop is unrolled by the
 *     window length).
 * The boundary condition is applied where rows and halo elements are fetched;
 * the index maps are exactly those of Stencil/Extra.hs:191-226:
 *     clamp    max(0, min(i, sz-1))
 *     mirror   i < 0 ? -i : i >= sz ? sz - (i - sz + 2) : i
 *     wrap     i < 0 ? sz + i : i >= sz ? i - sz : i
 *     constant out-of-range taps read the constant
 * Strips are kept short (ACC_TILE_H rows): the workgroups in flight then sweep
 * a compact window of the image, which DRAM serves far better than many
 * distant rows at once; the price is that neighbouring strips re-read each
 * other's boundary rows.  ACC_XCD_REMAP renumbers the workgroups so that such
 * neighbours run on the same compute die (acc_xcd_contiguous_block).
 * Strips that are cut by the right edge, and arrays whose rows are not
 * 16-byte aligned, take a slower path that maps every element on its own.
 *
 * Generated definitions expected: ACC_ELT, ACC_IN_ELT, ACC_ENV_PARAMS,
 * ACC_ENV_ASSUME, ACC_OUT_PARAMS, ACC_STENCIL_RANK (1|2), ACC_RADIUS_Y,
 * ACC_RADIUS_X, ACC_BOUNDARY, ACC_BOUNDARY_CONSTANT, ACC_STENCIL_TAPS(READ),
 * ACC_STENCIL_FN, ACC_TILE_H, ACC_PREFETCH, ACC_BLOCK, ACC_ALIGNED.
 */

#define ACC_SVEC  4                                   /* results per lane and row */
#define ACC_STRIP (ACC_WAVE * ACC_SVEC)               /* columns per wave */
#define ACC_NR    (2 * ACC_RADIUS_Y + 1)              /* rows a result depends on */
#define ACC_RING  (ACC_NR + ACC_PREFETCH)             /* rows held in registers */
#define ACC_WW    (ACC_SVEC + 2 * ACC_RADIUS_X)       /* row window of one lane */
#define ACC_WAVES (ACC_BLOCK / ACC_WAVE)
#define ACC_TOTAL_MAX  (ACC_TILE_H + 2 * ACC_RADIUS_Y)        /* source rows a strip touches */
#define ACC_HALO_COUNT (2 * ACC_RADIUS_X * ACC_TOTAL_MAX)     /* elements just outside the strip */
#define ACC_HALO_LOADS (ACC_HALO_COUNT > 0 ? (ACC_HALO_COUNT + ACC_WAVE - 1) / ACC_WAVE : 1)

static_assert(ACC_RADIUS_X <= ACC_SVEC, "stencil wider than one lane's neighbours can supply");

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
  /* the maps assume the array spans the stencil; keep the address legal if not */
  return acc_max<Int64>(0, acc_min<Int64>(i, sz - 1));
}

struct __attribute__((aligned(16))) acc_in_vec { ACC_IN_ELT v[ACC_SVEC]; };
struct __attribute__((aligned(16))) acc_out_vec { ACC_ELT v[ACC_SVEC]; };

/* value held by the next lane (the last lane keeps its own: caller masks it) */
#define ACC_DPP_WAVE_SHL1 0x130
template <typename T> ACC_DEV T acc_wave_shift_down1(const T &x) { return acc_dpp<ACC_DPP_WAVE_SHL1, 0xf>(x, x); }

/* one source row as a lane sees it: [rx left | ACC_SVEC own | rx right] */
struct acc_row { ACC_IN_ELT e[ACC_WW]; };

extern "C" __global__ void __launch_bounds__(ACC_BLOCK)
stencil(ACC_ENV_PARAMS ACC_OUT_PARAMS, const ACC_IN_ELT *__restrict__ arrStencil_0)
{
  typedef ACC_ELT T;
  typedef ACC_IN_ELT S;
  ACC_ENV_ASSUME
#if ACC_STENCIL_RANK == 2
  const Int64 h = shOut_1, w = shOut_0;
#else
  const Int64 h = 1, w = shOut_0;
#endif
  const int lane = acc_lane();
  const Int64 strips_x = (w + ACC_STRIP - 1) / ACC_STRIP;
  /* the wave's number within the workgroup, as a scalar: everything derived
   * from it (the strip's origin, which path it takes) is then uniform for the
   * compiler too, and the paths below become scalar branches */
  const int wave_in_block = __builtin_amdgcn_readfirstlane((int)(threadIdx.x >> 6));
#if ACC_XCD_REMAP
  const Int64 strip = acc_xcd_contiguous_block() * ACC_WAVES + wave_in_block;
#else
  const Int64 strip = (Int64)blockIdx.x * ACC_WAVES + wave_in_block;
#endif
#if ACC_STACK_WAVES
  /* the waves of a workgroup take vertically adjacent strips: the boundary
   * rows they share are then requested from the same compute unit, where the
   * second request merges with the first instead of going out to memory */
  const Int64 group = strip / ACC_WAVES, within = strip % ACC_WAVES;
  const Int64 y0 = ((group / strips_x) * ACC_WAVES + within) * ACC_TILE_H, x0 = (group % strips_x) * ACC_STRIP;
#else
  const Int64 y0 = (strip / strips_x) * ACC_TILE_H, x0 = (strip % strips_x) * ACC_STRIP;
#endif
  if (y0 >= h) return;                                   /* whole wave leaves together */
  const Int64 gx = x0 + lane * ACC_SVEC;
  const int rows_here = (int)acc_min<Int64>(ACC_TILE_H, h - y0);
#if ACC_ALIGNED
  const bool fast_here = (x0 + ACC_STRIP <= w);          /* every lane owns a full, aligned vector */
#else
  const bool fast_here = false;
#endif

  /* the strip, compiled three times: fast and ACC_TILE_H rows tall (all constants),
   * fast and cut by the bottom edge, and the element-wise path */
  auto run = [&](auto fast_c, auto full_c) {
  constexpr bool fast = decltype(fast_c)::value;
  const int rows = decltype(full_c)::value ? ACC_TILE_H : rows_here;

  const int total = rows + 2 * ACC_RADIUS_Y;              /* source rows this strip touches */

  /* fast path: the 2 rx elements just outside the strip, for every source row
   * the strip will touch, are requested in one go -- lane q takes element
   * q = (side * rx + j) * ACC_TOTAL_MAX + rho -- ahead of all row loads; finish()
   * hands them to the strip's first and last lane.  One instruction for the
   * strip instead of two per row. */
  S halo[ACC_HALO_LOADS];
  if (fast) {
#pragma unroll
    for (int g = 0; g < ACC_HALO_LOADS; ++g) {
      const int q = lane + ACC_WAVE * g;
      const int side = q / (ACC_RADIUS_X * ACC_TOTAL_MAX), rem = q % (ACC_RADIUS_X * ACC_TOTAL_MAX);
      const int j = rem / ACC_TOTAL_MAX, rho = rem % ACC_TOTAL_MAX;
      halo[g] = S();
      if (q < ACC_HALO_COUNT && rho < total) {
        const Int64 gy = y0 - ACC_RADIUS_Y + rho;
        const Int64 xx = side ? x0 + ACC_STRIP + j : x0 - ACC_RADIUS_X + j;
#if ACC_BOUNDARY == ACC_B_CONSTANT
        const bool inside = gy >= 0 && gy < h && xx >= 0 && xx < w;
        const Int64 my = acc_max<Int64>(0, acc_min<Int64>(gy, h - 1)), mx = acc_max<Int64>(0, acc_min<Int64>(xx, w - 1));
        halo[g] = inside ? arrStencil_0[my * w + mx] : (S)(ACC_BOUNDARY_CONSTANT);
#else
        halo[g] = arrStencil_0[acc_boundary_index(gy, h) * w + acc_boundary_index(xx, w)];
#endif
      }
    }
  }
  auto halo_of = [&](const int side, const int j, const int rho) -> S {
    const int q = (side * ACC_RADIUS_X + j) * ACC_TOTAL_MAX + rho;
    S v = acc_readlane(halo[0], q % ACC_WAVE);
#pragma unroll
    for (int g = 1; g < ACC_HALO_LOADS; ++g)
      if (q / ACC_WAVE == g) v = acc_readlane(halo[g], q % ACC_WAVE);
    return v;
  };

  /* fetch source row (y0 - ry + rho) into a window; in the fast path the left
   * and right parts are only valid once finish() has run */
  auto fetch = [&](const int rho, acc_row &r) {
    const Int64 gy = y0 - ACC_RADIUS_Y + rho;
#if ACC_BOUNDARY == ACC_B_CONSTANT
    const bool row_inside = gy >= 0 && gy < h;
    const Int64 my = acc_max<Int64>(0, acc_min<Int64>(gy, h - 1));
#else
    const bool row_inside = true;
    const Int64 my = acc_boundary_index(gy, h);
#endif
    const S *src = arrStencil_0 + my * w;
    if (fast) {
#if ACC_STENCIL_NT & 2
      typedef S acc_in_native __attribute__((ext_vector_type(ACC_SVEC)));
      const acc_in_native own = __builtin_nontemporal_load((const acc_in_native *)(src + gx));
#pragma unroll
      for (int k = 0; k < ACC_SVEC; ++k) r.e[ACC_RADIUS_X + k] = row_inside ? own[k] : (S)(ACC_BOUNDARY_CONSTANT);
#else
      const acc_in_vec own = *(const acc_in_vec *)(src + gx);
#pragma unroll
      for (int k = 0; k < ACC_SVEC; ++k) r.e[ACC_RADIUS_X + k] = row_inside ? own.v[k] : (S)(ACC_BOUNDARY_CONSTANT);
#endif
#pragma unroll
      for (int j = 0; j < ACC_RADIUS_X; ++j) {           /* filled in by finish() */
        r.e[j] = S();
        r.e[ACC_RADIUS_X + ACC_SVEC + j] = S();
      }
    } else {
#pragma unroll
      for (int e = 0; e < ACC_WW; ++e) {
        const Int64 xx = gx - ACC_RADIUS_X + e;
        r.e[e] = S();
        if (gx < w) {                                    /* lanes past the edge produce nothing */
#if ACC_BOUNDARY == ACC_B_CONSTANT
          const bool inside = row_inside && xx >= 0 && xx < w;
          r.e[e] = inside ? src[xx] : (S)(ACC_BOUNDARY_CONSTANT);
#else
          r.e[e] = src[acc_boundary_index(xx, w)];
#endif
        }
      }
    }
  };

  /* fast path only: complete the window with the neighbours' elements */
  auto finish = [&](const int rho, acc_row &r) {
    if (!fast) return;
#pragma unroll
    for (int j = 0; j < ACC_RADIUS_X; ++j) {
      const S from_left  = acc_wave_shift_up1(r.e[ACC_SVEC + j]);          /* neighbour's own[SVEC - rx + j] */
      const S from_right = acc_wave_shift_down1(r.e[ACC_RADIUS_X + j]);    /* neighbour's own[j] */
      r.e[j] = (lane != 0) ? from_left : halo_of(0, j, rho);
      r.e[ACC_RADIUS_X + ACC_SVEC + j] = (lane != ACC_WAVE - 1) ? from_right : halo_of(1, j, rho);
    }
  };

  acc_row ring[ACC_RING];

  /* prologue: the rows the first result needs, minus the newest, plus the prefetch */
#pragma unroll
  for (int rho = 0; rho < ACC_RING - 1; ++rho)
    if (rho < total) fetch(rho, ring[rho]);
#pragma unroll
  for (int rho = 0; rho < ACC_NR - 1; ++rho) finish(rho, ring[rho]);

  for (int yb = 0; yb < rows; yb += ACC_RING) {
#pragma unroll
    for (int s = 0; s < ACC_RING; ++s) {
      const int y = yb + s;                               /* row of the strip being produced */
      if (y < rows) {
        /* newest row needed now is rho = y + 2 ry, in slot (s + NR - 1) % RING; the
         * slot freed by the previous step takes the row PREFETCH further on */
        const int rho_new = y + ACC_NR - 1 + ACC_PREFETCH;
        if (rho_new < total) fetch(rho_new, ring[(s + ACC_RING - 1) % ACC_RING]);
        finish(y + ACC_NR - 1, ring[(s + ACC_NR - 1) % ACC_RING]);

        acc_out_vec res;
#pragma unroll
        for (int k = 0; k < ACC_SVEC; ++k) {
#define ACC_WINDOW_READ(dy, dx) ring[(s + ACC_RADIUS_Y + (dy)) % ACC_RING].e[ACC_RADIUS_X + k + (dx)]
          ACC_STENCIL_TAPS(ACC_WINDOW_READ)
#undef ACC_WINDOW_READ
          res.v[k] = (T)(ACC_STENCIL_FN);
        }
        T *dst = arrOut_0 + (y0 + y) * w + gx;
        if (fast) {
#if ACC_STENCIL_NT & 1
          typedef T acc_out_native __attribute__((ext_vector_type(ACC_SVEC)));
          acc_out_native nv;
#pragma unroll
          for (int k = 0; k < ACC_SVEC; ++k) nv[k] = res.v[k];
          __builtin_nontemporal_store(nv, (acc_out_native *)dst);
#else
          *(acc_out_vec *)dst = res;
#endif
        } else {
#pragma unroll
          for (int k = 0; k < ACC_SVEC; ++k)
            if (gx + k < w) dst[k] = res.v[k];
        }
      }
    }
  }
  };   /* run */

  if (fast_here) {
    if (rows_here == ACC_TILE_H) run(acc_bool<true>(), acc_bool<true>());
    else                         run(acc_bool<true>(), acc_bool<false>());
  } else {
    run(acc_bool<false>(), acc_bool<false>());
  }
}
