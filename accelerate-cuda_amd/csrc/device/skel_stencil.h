/*
 * skel_stencil.h -- 1-D, 2-D and 3-D stencils: every element of the result
 * is a function of the elements of the source at fixed offsets from it.
 *
 * Takes the place of CodeGen/Stencil.hs:55-114 and the access generator of
 * CodeGen/Stencil/Extra.hs:53-128.  The reference reads every tap straight
 * from global memory (relying on the L1 cache, Context.hs:61-68), recovers the
 * multidimensional index with 64-bit divisions and tests a whole warp for
 * "interior" (Stencil.hs:103-110).  Here the work is cut into strips: one
 * 64-lane wave owns 256 columns (ACC_SVEC = 4 per lane; 2 per lane, 128
 * columns, of 8-byte elements) and walks down ACC_TILE_H rows,
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
 * The last strip of a row of strips ends at the right edge (it overlaps its
 * neighbour rather than reach past the edge); only an array narrower than a
 * strip takes a slower path that maps every element on its own.  Rows that are
 * not 16-byte aligned are read with the same 128-bit accesses, element-aligned.
 *
 * A 3-D stencil keeps a register window per plane it reads.  Without taps in
 * other planes, or with ACC_ZMARCH 0, a strip lies in ACC_TZ planes and all its
 * windows advance down the rows together.  With ACC_ZMARCH the two axes change
 * places: a strip is ACC_TZ rows tall and walks through ACC_TILE_H planes (or
 * the fewer the driver asks for on a small volume, `acc_walk`), the
 * windows hold the 2 ry + ACC_TZ rows it reads of each of the 2 rz + 1 planes
 * in reach (plus the planes requested ahead), and a row fetched once serves
 * the results of every plane that reads it -- what a walk down the rows reads
 * 2 rz + ACC_TZ planes for, ACC_TZ at a time.  Everything below is written for
 * a "marching" axis (the ring) and a "static" axis (the windows side by side);
 * which of y and z is which is decided in a handful of places marked ACC_ZMARCH.
 *
 * With ACC_STENCIL_SOURCES == 2 the same kernel is stencil2
 * (CodeGen/Stencil.hs:118-237): two source arrays, each with its own taps,
 * element type, boundary condition and extents; the result covers the
 * intersection of the two extents and its element is a function of both
 * neighbourhoods (taps t0.. of the first source, u0.. of the second).
 *
 * A source of tuples (Stencil/Extra.hs:53-128 reads every component) is one
 * array per component: each gets its own register window, and a tap is a
 * struct of the components' values (t0.a1, t0.a0).
 *
 * Generated definitions expected: ACC_ELT, ACC_ENV_PARAMS, ACC_ENV_ASSUME,
 * ACC_OUT_PARAMS, ACC_STENCIL_RANK (1|2|3), ACC_RADIUS_Z, ACC_RADIUS_Y,
 * ACC_RADIUS_X (the larger of the two sources'), ACC_STENCIL_FN, ACC_TILE_H,
 * ACC_PREFETCH, ACC_BLOCK, ACC_ALIGNED, ACC_STENCIL_SOURCES (1|2) and per
 * source n = 1, 2: ACC_BOUNDARY (ACC_BOUNDARY2), ACC_SRC<n>_COMPONENTS(X, arg),
 * ACC_SRC<n>_PARAMS, ACC_IN<n>_ELT, ACC_STENCIL_TAPS<n>(READ) with
 * READ(component, dz, dy, dx).
 */

#ifndef ACC_SVEC
#define ACC_SVEC  4                                   /* results per lane and row */
#endif
#define ACC_STRIP (ACC_WAVE * ACC_SVEC)               /* columns per wave */
#ifndef ACC_ZMARCH
#define ACC_ZMARCH 0
#endif
#if ACC_ZMARCH
#define ACC_RADIUS_M ACC_RADIUS_Z                     /* reach along the axis the strip walks */
#define ACC_RADIUS_S ACC_RADIUS_Y                     /* reach along the axis its windows lie side by side on */
#else
#define ACC_RADIUS_M ACC_RADIUS_Y
#define ACC_RADIUS_S ACC_RADIUS_Z
#endif
#define ACC_NR    (2 * ACC_RADIUS_M + 1)              /* rows (planes) a result depends on */
#define ACC_RING  (ACC_NR + ACC_PREFETCH)             /* rows held in registers */
#define ACC_WW    (ACC_SVEC + 2 * ACC_RADIUS_X)       /* row window of one lane */
#define ACC_WAVES (ACC_BLOCK / ACC_WAVE)
#ifndef ACC_RADIUS_Z
#define ACC_RADIUS_Z 0
#endif
#ifndef ACC_TZ
#define ACC_TZ 1
#endif
/* a strip produces ACC_TZ consecutive planes of the result from one register window over
 * ACC_NZ source planes: a source row fetched once serves the results of up to 2 rz + 1 planes */
#define ACC_NZ    (2 * ACC_RADIUS_S + ACC_TZ)         /* planes (rows) held side by side */
#define ACC_TOTAL_MAX  (ACC_TILE_H + 2 * ACC_RADIUS_M)        /* source rows (planes) a strip touches, per window */
/* a strip cut by the right edge of the array gathers up to 2 rx + ACC_SVEC - 1 elements a row and window: where it walks
 * through planes, a lane each in one request; elsewhere all of a strip's at its start, held in registers and handed
 * out by readlane -- for no more than 512 of them (a stencil that reaches 4 columns and 4 rows in 3 planes has 792:
 * 677 us on 200^3 against 87 us element by element) */
#define ACC_CUT_OK (ACC_ZMARCH ? ACC_NZ * (2 * ACC_RADIUS_X + ACC_SVEC - 1) <= ACC_WAVE \
                               : (2 * ACC_RADIUS_X + ACC_SVEC - 1) * ACC_TOTAL_MAX * ACC_NZ <= 512)

static_assert(ACC_RADIUS_X <= ACC_SVEC, "stencil wider than one lane's neighbours can supply");

#define ACC_B_CLAMP 0
#define ACC_B_MIRROR 1
#define ACC_B_WRAP 2
#define ACC_B_CONSTANT 3

template <int MODE>
ACC_DEV Int64 acc_boundary_index(Int64 i, const Int64 sz)
{
  if (MODE == ACC_B_CLAMP)  i = acc_max<Int64>(0, acc_min<Int64>(i, sz - 1));
  if (MODE == ACC_B_MIRROR) i = i < 0 ? -i : (i >= sz ? sz - (i - sz + 2) : i);
  if (MODE == ACC_B_WRAP)   i = i < 0 ? sz + i : (i >= sz ? i - sz : i);
  /* the maps assume the array spans the stencil; keep the address legal if not */
  return acc_max<Int64>(0, acc_min<Int64>(i, sz - 1));
}

struct acc_out_vec { ACC_ELT v[ACC_SVEC]; };

/* value held by the next lane (the last lane keeps its own: caller masks it) */
#define ACC_DPP_WAVE_SHL1 0x130
template <typename T> ACC_DEV T acc_wave_shift_down1(const T &x) { return acc_dpp<ACC_DPP_WAVE_SHL1, 0xf>(x, x); }

/* One source array as a strip sees it: the register window of ACC_RING rows,
 * each row [rx left | ACC_SVEC own | rx right] per lane, and what fills it.
 * S element type, MODE boundary condition, FAST the aligned full-strip path. */
/* CUT (with FAST): the strip reaches past the right edge of the array.  The lanes whose four columns lie inside work as
 * in any strip; lane `last` holds the `rem` columns left over (all four if rem is 0), lanes beyond it nothing.  Every
 * lane still makes one 128-bit request -- from the edge on, for the last whole vector of the row, whose elements the
 * lane across the edge moves down to where its columns belong -- and what stands right of the array (the rest of that
 * lane's vector, then the rx elements its results reach for) is gathered like the elements outside a full strip. */
template <typename S, int MODE, bool FAST, bool CUT = false>
struct acc_strip_source {
  static_assert(FAST || !CUT, "a cut strip is a fast strip");
  static constexpr int RX = ACC_RADIUS_X;
  static constexpr int RIGHT = CUT ? RX + ACC_SVEC - 1 : RX;       /* gathered elements right of the strip, a row */
  static constexpr int PER_ROW = RX + RIGHT;                        /* ... either side */
  static constexpr int HALO_COUNT = PER_ROW * ACC_TOTAL_MAX * ACC_NZ;
  static constexpr int HALO_LOADS = HALO_COUNT > 0 ? (HALO_COUNT + ACC_WAVE - 1) / ACC_WAVE : 1;
  struct row { S e[ACC_WW]; };
  /* one lane's run of a row.  When rows start on 16-byte boundaries (ACC_ALIGNED) the type says so; otherwise
   * it is only element-aligned, which the memory instructions accept as well */
  struct __attribute__((aligned(ACC_ALIGNED ? ACC_SVEC * sizeof(S) : alignof(S)))) vec { S v[ACC_SVEC]; };

  const S *base;            /* the array, its extents, the value outside it (constant boundary) */
  Int64 d, h, w;
  S outside;
  Int64 z0, y0, x0, gx;     /* the strip's plane and origin, this lane's first column */
  int lane, total;          /* total = source rows the strip touches in each plane */
  int last, rem;            /* CUT: the lane across the right edge, and how many of its columns lie inside (0: all) */
  row ring[ACC_NZ][ACC_RING];
  S halo[HALO_LOADS];
#if ACC_ZMARCH
  S halo_ring[ACC_RING];    /* lane (p * 2 + side) * rx + j: the element outside the strip for window p of the slot's plane */
#endif
  /* window p, line rho of the strip's walk: which plane and row of the source that is */
  ACC_DEV Int64 plane_of(const int p, const int rho) const { return ACC_ZMARCH ? z0 - ACC_RADIUS_Z + rho : z0 - ACC_RADIUS_Z + p; }
  ACC_DEV Int64 row_of(const int p, const int rho) const   { return ACC_ZMARCH ? y0 - ACC_RADIUS_Y + p : y0 - ACC_RADIUS_Y + rho; }
  /* one element outside the strip: window p, line rho, `side` 0 left 1 right, the j-th of rx */
  ACC_DEV S outside_element(const int p, const int rho, const int side, const int j) const
  {
    const Int64 gz = plane_of(p, rho), gy = row_of(p, rho);
    const Int64 xx = side ? (CUT ? w : x0 + ACC_STRIP) + j : x0 - ACC_RADIUS_X + j;
    if (MODE == ACC_B_CONSTANT) {
      const bool inside = gz >= 0 && gz < d && gy >= 0 && gy < h && xx >= 0 && xx < w;
      const Int64 mz = acc_max<Int64>(0, acc_min<Int64>(gz, d - 1));
      const Int64 my = acc_max<Int64>(0, acc_min<Int64>(gy, h - 1)), mx = acc_max<Int64>(0, acc_min<Int64>(xx, w - 1));
      return inside ? base[(mz * h + my) * w + mx] : outside;
    }
    return base[(acc_boundary_index<MODE>(gz, d) * h + acc_boundary_index<MODE>(gy, h)) * w + acc_boundary_index<MODE>(xx, w)];
  }

  /* FAST: the 2 rx elements just outside the strip, for every source row the
   * strip will touch, are requested in one go -- lane q takes element
   * q = (side * rx + j) * ACC_TOTAL_MAX + rho -- ahead of all row loads;
   * finish() hands them to the strip's first and last lane.  One instruction
   * for the strip instead of two per row. */
  ACC_DEV void gather_halo()
  {
    if (!FAST || ACC_ZMARCH || RX == 0) return;            /* (a strip that walks through planes asks line by line: fetch) */
    constexpr int per_plane = PER_ROW * ACC_TOTAL_MAX > 0 ? PER_ROW * ACC_TOTAL_MAX : 1;
#pragma unroll
    for (int g = 0; g < HALO_LOADS; ++g) {
      const int q = lane + ACC_WAVE * g;
      const int p = q / per_plane, qq = q % per_plane;
      const int entry = qq / ACC_TOTAL_MAX, rho = qq % ACC_TOTAL_MAX;     /* entries 0 .. rx - 1 left, the others right */
      halo[g] = S();
      if (q < HALO_COUNT && rho < total) halo[g] = outside_element(p, rho, entry >= RX, entry >= RX ? entry - RX : entry);
    }
  }
  /* the j-th element left (side 0) or right of the strip, for window p and line rho (held in ring slot `slot`); j may be
   * a run-time value that is the same in every lane */
  ACC_DEV S halo_of(const int p, const int side, const int j, const int rho, const int slot) const
  {
    const int entry = side ? RX + j : j;
#if ACC_ZMARCH
    (void)rho;
    return acc_readlane(halo_ring[slot], p * PER_ROW + entry);
#endif
    (void)slot;
    const int q = p * (PER_ROW * ACC_TOTAL_MAX) + entry * ACC_TOTAL_MAX + rho;
    S v = acc_readlane(halo[0], q % ACC_WAVE);
#pragma unroll
    for (int g = 1; g < HALO_LOADS; ++g)
      if (q / ACC_WAVE == g) v = acc_readlane(halo[g], q % ACC_WAVE);
    return v;
  }

  /* fetch source row (y0 - ry + rho) of every plane into ring[.][slot]; on the FAST
   * path the left and right parts are only valid once finish() has run */
  ACC_DEV void fetch(const int rho, const int slot)
  {
#if ACC_ZMARCH
    /* the 2 rx elements outside the strip of all the windows' rows of this plane: one request, a lane each */
    static_assert(ACC_NZ * PER_ROW <= ACC_WAVE, "more elements outside the strip than lanes to ask for them");
    if (FAST && RX > 0) {
      constexpr int per_row = PER_ROW > 0 ? PER_ROW : 1;
      const int entry = lane % per_row;
      halo_ring[slot] = S();
      if (lane < ACC_NZ * per_row) halo_ring[slot] = outside_element(lane / per_row, rho, entry >= RX, entry >= RX ? entry - RX : entry);
    }
#endif
#pragma unroll
    for (int p = 0; p < ACC_NZ; ++p) fetch_plane(p, rho, slot);
  }
  ACC_DEV void fetch_plane(const int p, const int rho, const int slot)
  {
    row &r = ring[p][slot];
    const Int64 gz = plane_of(p, rho);
    const Int64 gy = row_of(p, rho);
    const bool row_inside = MODE != ACC_B_CONSTANT || (gy >= 0 && gy < h && gz >= 0 && gz < d);
    const Int64 my = MODE == ACC_B_CONSTANT ? acc_max<Int64>(0, acc_min<Int64>(gy, h - 1)) : acc_boundary_index<MODE>(gy, h);
    const Int64 mz = MODE == ACC_B_CONSTANT ? acc_max<Int64>(0, acc_min<Int64>(gz, d - 1)) : acc_boundary_index<MODE>(gz, d);
    const S *src = base + (mz * h + my) * w;
    if (FAST) {
      const Int64 from = CUT ? acc_min<Int64>(gx, w - ACC_SVEC) : gx;
      vec own = *(const vec *)(src + from);
      if (CUT && rem != 0) {                     /* (the same in every lane: a row that ends with a whole vector skips this) */
        /* the lane across the edge has asked `down` elements to the left of its own columns: move them down (lanes
         * beyond it move theirs anywhere: nothing of theirs is used) */
        const int down = (int)(gx - from);
        const vec asked = own;
#pragma unroll
        for (int k = 0; k + 1 < ACC_SVEC; ++k) {
#pragma unroll
          for (int m = 1; k + m < ACC_SVEC; ++m) own.v[k] = (down == m) ? asked.v[k + m] : own.v[k];
        }
      }
#pragma unroll
      for (int k = 0; k < ACC_SVEC; ++k) r.e[ACC_RADIUS_X + k] = row_inside ? own.v[k] : outside;
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
          if (MODE == ACC_B_CONSTANT) {
            const bool inside = row_inside && xx >= 0 && xx < w;
            r.e[e] = inside ? src[acc_max<Int64>(0, acc_min<Int64>(xx, w - 1))] : outside;
          } else {
            r.e[e] = src[acc_boundary_index<MODE>(xx, w)];
          }
        }
      }
    }
  }

  /* FAST only: complete ring[.][slot], which holds source row rho, with the neighbours' elements */
  ACC_DEV void finish(const int rho, const int slot)
  {
    if (!FAST) return;
#pragma unroll
    for (int p = 0; p < ACC_NZ; ++p) {
      row &r = ring[p][slot];
      if (CUT && RX > 0 && rem != 0) {
        /* first the columns of the lane across the edge that lie outside the array: its neighbour reads them below */
#pragma unroll
        for (int k = 1; k < ACC_SVEC; ++k) {
          const S outside_own = halo_of(p, 1, acc_max(0, k - rem), rho, slot);
          r.e[ACC_RADIUS_X + k] = (lane == last && rem != 0 && k >= rem) ? outside_own : r.e[ACC_RADIUS_X + k];
        }
      }
#pragma unroll
      for (int j = 0; j < ACC_RADIUS_X; ++j) {
        const S from_left  = acc_wave_shift_up1(r.e[ACC_SVEC + j]);          /* neighbour's own[SVEC - rx + j] */
        const S from_right = acc_wave_shift_down1(r.e[ACC_RADIUS_X + j]);    /* neighbour's own[j] */
        /* (read by every lane, before the choice: a read of another lane's register made under a condition sees
         * whatever that lane holds where only the lanes that pass the condition have worked the value out -- for
         * an element narrower than a register, its widening) */
        /* (a cut strip: right of the lane across the edge come the columns of its own vector that lie outside the
         * array, ACC_SVEC - rem of them if any, and then the elements asked for here) */
        const int beyond = CUT ? (rem ? ACC_SVEC - rem : 0) : 0;
        const S outside_left = halo_of(p, 0, j, rho, slot), outside_right = halo_of(p, 1, beyond + j, rho, slot);
        r.e[j] = (lane != 0) ? from_left : outside_left;
        r.e[ACC_RADIUS_X + ACC_SVEC + j] = (lane != (CUT ? last : ACC_WAVE - 1)) ? from_right : outside_right;
      }
    }
  }
};

/* A source is one array per component of its element type; the generator hands over, per source, the list of its
 * components ACC_SRC<n>_COMPONENTS(X, arg) = X(component, type, value outside, arg) ..., highest component first, and
 * its kernel parameters ACC_SRC<n>_PARAMS in the same order (for stencil2 each source with its own extents in front,
 * Stencil.hs:146-152).  Every component gets a register window of its own; they all move together. */
#if ACC_STENCIL_SOURCES == 2
#define ACC_STENCIL_ENTRY stencil2
#define ACC_SOURCE_PARAMS ACC_SRC1_PARAMS ACC_SRC2_PARAMS
#else
#define ACC_STENCIL_ENTRY stencil
#define ACC_SOURCE_PARAMS ACC_SRC1_PARAMS
#define ACC_SRC2_COMPONENTS(X, arg)
#endif

extern "C" __global__ void __launch_bounds__(ACC_BLOCK)
ACC_STENCIL_ENTRY(ACC_ENV_PARAMS ACC_OUT_PARAMS ACC_SOURCE_PARAMS, const int acc_walk ACC_GUARD_PARAM)
{
  ACC_GUARD_CHECK
  typedef ACC_ELT T;
  ACC_ENV_ASSUME
#if ACC_STENCIL_RANK == 3
  const Int64 d = shOut_2, h = shOut_1, w = shOut_0;
#elif ACC_STENCIL_RANK == 2
  const Int64 d = 1, h = shOut_1, w = shOut_0;
#else
  const Int64 d = 1, h = 1, w = shOut_0;
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
  /* strips are numbered row of strips after row of strips (band), plane after plane */
#if ACC_STACK_WAVES
  /* the waves of a workgroup take vertically adjacent strips: the boundary
   * rows they share are then requested from the same compute unit, where the
   * second request merges with the first instead of going out to memory */
  const Int64 group = strip / ACC_WAVES, within = strip % ACC_WAVES;
  const Int64 band = (group / strips_x) * ACC_WAVES + within, x0_across = (group % strips_x) * ACC_STRIP;
#else
  const Int64 band = strip / strips_x, x0_across = (strip % strips_x) * ACC_STRIP;
#endif
#if ACC_STENCIL_RANK == 3 && ACC_ZMARCH
  /* strips ACC_TZ rows tall, numbered DOWN a plane first (the waves of a workgroup are vertical neighbours: the rows
   * they share are asked for by one compute unit at about the same time), then across it, then run of ACC_TILE_H
   * planes after run */
  /* (`acc_walk` planes a run: ACC_TILE_H, or fewer where strips that long would be too few to fill the device) */
  const Int64 bands = (h + ACC_TZ - 1) / ACC_TZ;
  const Int64 across = strip / bands;
  const Int64 z0 = (across / strips_x) * acc_walk, y0 = (strip % bands) * ACC_TZ;
  if (z0 >= d) return;
#elif ACC_STENCIL_RANK == 3
  const Int64 bands = (h + ACC_TILE_H - 1) / ACC_TILE_H;
  const Int64 z0 = (band / bands) * ACC_TZ, y0 = (band % bands) * ACC_TILE_H;
  if (z0 >= d) return;
#else
  const Int64 z0 = 0, y0 = band * ACC_TILE_H;
#endif
  if (y0 >= h) return;                                   /* whole wave leaves together */
#if ACC_STENCIL_RANK == 3 && ACC_ZMARCH
  const Int64 x0_grid = (across % strips_x) * ACC_STRIP;
  (void)band; (void)x0_across;
#else
  const Int64 x0_grid = x0_across;
#endif
  /* The last strip of a row of strips is laid to END at the right edge: it overlaps its neighbour, whose columns it
   * produces a second time (the same values), instead of reaching past the edge, and every lane of it owns a whole
   * vector like in any other strip.  (An array narrower than a strip has the one strip, on the element-wise path.) */
  const Int64 x0 = (w >= ACC_STRIP && w - x0_grid >= ACC_SHIFT_MIN) ? acc_min<Int64>(x0_grid, w - ACC_STRIP) : x0_grid;
  const Int64 gx = x0 + lane * ACC_SVEC;
  /* how far the strip walks: rows, or planes */
  const int rows_here = (int)acc_min<Int64>(ACC_ZMARCH ? acc_walk : ACC_TILE_H, ACC_ZMARCH ? d - z0 : h - y0);
  (void)acc_walk;
  const bool fast_here = (x0 + ACC_STRIP <= w);          /* every lane owns a full vector */
  /* a strip cut by the right edge: the last of its lanes with columns inside the array, and how many it has if not all
   * (a row shorter than one vector is left to the element-wise path) */
#if ACC_STENCIL_SOURCES == 2
  const bool same_width = shStencil1_0 == w && shStencil2_0 == w;   /* (a wider source has elements where the result ends) */
#else
  const bool same_width = true;
#endif
  /* (with few columns inside, mapping each element on its own is cheaper: fewer than ACC_CUT_MIN take that path) */
  const bool cut_here = ACC_CUT_OK && !fast_here && w >= ACC_SVEC && w - x0 >= ACC_CUT_MIN && same_width;
  const int cut_last = (int)((w - x0 + ACC_SVEC - 1) / ACC_SVEC) - 1, cut_rem = (int)((w - x0) % ACC_SVEC);

  /* the strip, compiled four times: fast and ACC_TILE_H rows tall (all constants), fast and cut by the bottom edge,
   * fast and cut by the right edge, and the element-wise path */
  auto run = [&](auto fast_c, auto full_c, auto cut_c) {
  constexpr bool fast = decltype(fast_c)::value;
  constexpr bool cut = decltype(cut_c)::value;
  const int rows = decltype(full_c)::value ? ACC_TILE_H : rows_here;
  const int total = rows + 2 * ACC_RADIUS_M;              /* source rows (planes) this strip touches */

  /* one strip source per component of either source's element: a<c> for the first source, b<c> for the second */
#if ACC_STENCIL_SOURCES == 2
#if ACC_STENCIL_RANK == 3
#define ACC_SRC1_EXTENTS(o) o.d = shStencil1_2; o.h = shStencil1_1; o.w = shStencil1_0
#define ACC_SRC2_EXTENTS(o) o.d = shStencil2_2; o.h = shStencil2_1; o.w = shStencil2_0
#elif ACC_STENCIL_RANK == 2
#define ACC_SRC1_EXTENTS(o) o.d = 1; o.h = shStencil1_1; o.w = shStencil1_0
#define ACC_SRC2_EXTENTS(o) o.d = 1; o.h = shStencil2_1; o.w = shStencil2_0
#else
#define ACC_SRC1_EXTENTS(o) o.d = 1; o.h = 1; o.w = shStencil1_0
#define ACC_SRC2_EXTENTS(o) o.d = 1; o.h = 1; o.w = shStencil2_0
#endif
#define ACC_SRC1_ARRAY(c) arrStencil1_##c
#define ACC_SRC2_ARRAY(c) arrStencil2_##c
#else
#define ACC_SRC1_EXTENTS(o) o.d = d; o.h = h; o.w = w
#define ACC_SRC1_ARRAY(c) arrStencil_##c
#endif
#define ACC_DECLARE_A(c, CT, OUTSIDE, arg)                                         \
  acc_strip_source<CT, ACC_BOUNDARY, fast, cut> a##c;                             \
  a##c.last = cut_last; a##c.rem = cut_rem;                                       \
  a##c.base = ACC_SRC1_ARRAY(c);                                                  \
  ACC_SRC1_EXTENTS(a##c);                                                         \
  a##c.outside = (CT)OUTSIDE;                                                     \
  a##c.z0 = z0; a##c.y0 = y0; a##c.x0 = x0; a##c.gx = gx; a##c.lane = lane; a##c.total = total;
  ACC_SRC1_COMPONENTS(ACC_DECLARE_A, 0)
#undef ACC_DECLARE_A
#if ACC_STENCIL_SOURCES == 2
#define ACC_DECLARE_B(c, CT, OUTSIDE, arg)                                         \
  acc_strip_source<CT, ACC_BOUNDARY2, fast, cut> b##c;                            \
  b##c.last = cut_last; b##c.rem = cut_rem;                                       \
  b##c.base = ACC_SRC2_ARRAY(c);                                                  \
  ACC_SRC2_EXTENTS(b##c);                                                         \
  b##c.outside = (CT)OUTSIDE;                                                     \
  b##c.z0 = z0; b##c.y0 = y0; b##c.x0 = x0; b##c.gx = gx; b##c.lane = lane; b##c.total = total;
  ACC_SRC2_COMPONENTS(ACC_DECLARE_B, 0)
#undef ACC_DECLARE_B
#endif
  /* the same call on every component's window */
#define ACC_CALL_A(c, CT, OUTSIDE, call) a##c.call;
#define ACC_CALL_B(c, CT, OUTSIDE, call) b##c.call;
#define ACC_BOTH(call) do { ACC_SRC1_COMPONENTS(ACC_CALL_A, call) ACC_SRC2_COMPONENTS(ACC_CALL_B, call) } while (0)

  ACC_BOTH(gather_halo());

  /* prologue: the rows the first result needs, minus the newest, plus the prefetch */
#pragma unroll
  for (int rho = 0; rho < ACC_RING - 1; ++rho)
    if (rho < total) ACC_BOTH(fetch(rho, rho));
#if ACC_SCHED_BARRIER
  /* nothing that uses a row moves up between the requests for the rows: left to itself the compiler asks for two
   * rows, waits for the first to shift its elements between lanes, and only then asks for the others */
  __builtin_amdgcn_sched_barrier(0);
#endif
#pragma unroll
  for (int rho = 0; rho < ACC_NR - 1; ++rho) ACC_BOTH(finish(rho, rho));

  for (int yb = 0; yb < rows; yb += ACC_RING) {
#pragma unroll
    for (int s = 0; s < ACC_RING; ++s) {
      const int y = yb + s;                               /* row of the strip being produced */
      if (y < rows) {
        /* newest row needed now is rho = y + 2 ry, in slot (s + NR - 1) % RING; the
         * slot freed by the previous step takes the row PREFETCH further on */
        const int rho_new = y + ACC_NR - 1 + ACC_PREFETCH;
        if (decltype(full_c)::value) {
          if (rho_new < total) ACC_BOTH(fetch(rho_new, (s + ACC_RING - 1) % ACC_RING));
        } else {
          /* a strip of a length only known at run time asks without a test -- a load under a condition is waited
           * for on the spot, and with it every row requested ahead: past the strip's end it asks for its last row
           * again, into a slot nothing reads any more */
          ACC_BOTH(fetch(acc_min(rho_new, total - 1), (s + ACC_RING - 1) % ACC_RING));
        }
#if ACC_SCHED_BARRIER & 2
        __builtin_amdgcn_sched_barrier(0);                 /* the requests of this step before anything of the step's results */
#endif
        ACC_BOTH(finish(y + ACC_NR - 1, (s + ACC_NR - 1) % ACC_RING));

#pragma unroll
        for (int pz = 0; pz < ACC_TZ; ++pz) {
        if (ACC_TZ > 1 && (ACC_ZMARCH ? y0 + pz >= h : z0 + pz >= d)) break;   /* the last band of planes (rows) may be short */
        acc_out_vec res;
#pragma unroll
        for (int k = 0; k < ACC_SVEC; ++k) {
#if ACC_ZMARCH
#define ACC_WINDOW_AT(dz, dy) [pz + ACC_RADIUS_Y + (dy)][(s + ACC_RADIUS_Z + (dz)) % ACC_RING]
#else
#define ACC_WINDOW_AT(dz, dy) [pz + ACC_RADIUS_Z + (dz)][(s + ACC_RADIUS_Y + (dy)) % ACC_RING]
#endif
#define ACC_WINDOW_READ(c, dz, dy, dx) a##c.ring ACC_WINDOW_AT(dz, dy).e[ACC_RADIUS_X + k + (dx)]
          ACC_STENCIL_TAPS1(ACC_WINDOW_READ)
#undef ACC_WINDOW_READ
#if ACC_STENCIL_SOURCES == 2
#define ACC_WINDOW_READ(c, dz, dy, dx) b##c.ring ACC_WINDOW_AT(dz, dy).e[ACC_RADIUS_X + k + (dx)]
          ACC_STENCIL_TAPS2(ACC_WINDOW_READ)
#undef ACC_WINDOW_READ
#endif
#undef ACC_WINDOW_AT
          res.v[k] = (T)(ACC_STENCIL_FN);
        }
        /* one vector store per component of the result (a tuple result is one array per component) */
        const Int64 at = ACC_ZMARCH ? (((z0 + y) * h) + (y0 + pz)) * w + gx : (((z0 + pz) * h) + (y0 + y)) * w + gx;
#define ACC_STORE_COMPONENT(c, CT)                                                   \
        {                                                                            \
          CT *dst = arrOut_##c + at;                                                 \
          if (fast && (!cut || gx + ACC_SVEC <= w)) {                                \
            typedef CT acc_out_native __attribute__((ext_vector_type(ACC_SVEC)));    \
            typedef acc_out_native acc_out_stored __attribute__((aligned(ACC_ALIGNED ? ACC_SVEC * sizeof(CT) : alignof(CT)))); \
            acc_out_native nv;                                                       \
            _Pragma("unroll") for (int k = 0; k < ACC_SVEC; ++k) nv[k] = ACC_COMPONENT(res.v[k], c); \
            if (ACC_STENCIL_NT & 1) __builtin_nontemporal_store(nv, (acc_out_stored *)dst); \
            else                    *(acc_out_stored *)dst = nv;                     \
          } else {                                                                   \
            _Pragma("unroll") for (int k = 0; k < ACC_SVEC; ++k)                     \
              if (gx + k < w) dst[k] = ACC_COMPONENT(res.v[k], c);                   \
          }                                                                          \
        }
        ACC_FOR_COMPONENTS(ACC_STORE_COMPONENT)
#undef ACC_STORE_COMPONENT
        }   /* pz */
      }
    }
  }
#undef ACC_BOTH
#undef ACC_CALL_A
#undef ACC_CALL_B
  };   /* run */

  if (fast_here) {
    if (rows_here == ACC_TILE_H) run(acc_bool<true>(), acc_bool<true>(), acc_bool<false>());
    else                         run(acc_bool<true>(), acc_bool<false>(), acc_bool<false>());
  } else if (cut_here) {
    run(acc_bool<true>(), acc_bool<false>(), acc_bool<ACC_CUT_OK>());
  } else {
    run(acc_bool<false>(), acc_bool<false>(), acc_bool<false>());
  }
}
