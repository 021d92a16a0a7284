/*
 * skel_stencil_nd.h -- stencils of any rank and reach, an element of the result a thread.
 *
 * Takes the place of CodeGen/Stencil.hs:55-114 as it stands there: the linear index of the element is taken apart
 * into the index of every dimension (cfromIndex, CodeGen/Base.hs:207-218), every tap adds its offsets, the
 * boundary condition is applied dimension by dimension (Stencil/Extra.hs:158-226) and the source is read at the
 * row-major position of the result (ctoIndex, Base.hs:193-202).  skel_stencil.h keeps the rows a strip needs in
 * registers, which is written for up to three dimensions and for offsets a register window can hold; this template
 * serves what lies beyond that -- arrays of rank 4 and more, taps further than 2 planes or 4 rows or columns away --
 * and leaves the reuse of neighbouring elements to the caches, as the reference does.  Same entry names, same
 * parameters (the strip kernel's `acc_walk` is taken and ignored), same results.
 *
 * Generated definitions expected: ACC_ELT, ACC_ENV_PARAMS, ACC_ENV_ASSUME, ACC_OUT_PARAMS, ACC_STENCIL_RANK,
 * ACC_OUT_EXTENTS (shOut_<rank-1>, ..., shOut_0), ACC_STENCIL_SOURCES (1|2), ACC_STENCIL_FN, ACC_BLOCK and per
 * source n = 1, 2: ACC_BOUNDARY (ACC_BOUNDARY2), ACC_SRC<n>_COMPONENTS(X, arg), ACC_SRC<n>_PARAMS,
 * ACC_SRC<n>_EXTENTS (the source's own extents, outermost first), ACC_IN<n>_ELT, ACC_STENCIL_TAPS<n>_ND(READ) with
 * READ(component, offset of the outermost dimension, ..., offset of the innermost), ACC_SRC<n>_REACH_LO / _HI (how far
 * the taps reach towards the beginning and the end of every dimension, outermost first).
 */

#ifndef ACC_ND_INNER
#define ACC_ND_INNER 1                                   /* 0: every element takes the way of the elements at the boundary */
#endif
#define ACC_B_CLAMP 0
#define ACC_B_MIRROR 1
#define ACC_B_WRAP 2
#define ACC_B_CONSTANT 3

/* Indices are 32 bits wide where the arrays allow it (fewer than 2^31 elements each): the index of an element is
 * taken apart and the position of every tap put together with divisions, multiplications and comparisons, which cost
 * twice to five times as much on 64-bit numbers -- 3 x 3 on 2^24 x 3 elements: 200 us with 64-bit indices. */
template <typename I> struct acc_nd_index { I i[ACC_STENCIL_RANK]; };
struct acc_nd_offset { int o[ACC_STENCIL_RANK]; };

template <int MODE, typename I>
ACC_DEV I acc_nd_boundary(I i, const I sz)
{
  if (MODE == ACC_B_CLAMP)  i = acc_max<I>(0, acc_min<I>(i, sz - 1));
  if (MODE == ACC_B_MIRROR) i = i < 0 ? -i : (i >= sz ? sz - (i - sz + 2) : i);
  if (MODE == ACC_B_WRAP)   i = i < 0 ? sz + i : (i >= sz ? i - sz : i);
  /* the maps assume the array spans the stencil; keep the address legal if not */
  return acc_max<I>(0, acc_min<I>(i, sz - 1));
}

/* the element of `base` (extents `sh`) at `at` + `off`, under the boundary condition; `outside` beyond a constant boundary */
template <int MODE, typename S, typename I>
ACC_DEV S acc_nd_read(const S *__restrict__ base, const acc_nd_index<I> &sh, const acc_nd_index<I> &at, const acc_nd_offset &off, const S outside)
{
  I lin = 0;
  bool inside = true;
#pragma unroll
  for (int d = 0; d < ACC_STENCIL_RANK; ++d) {
    const I i = at.i[d] + (I)off.o[d];
    if (MODE == ACC_B_CONSTANT) inside = inside && i >= 0 && i < sh.i[d];
    lin = lin * sh.i[d] + acc_nd_boundary<MODE, I>(i, sh.i[d]);
  }
  const S v = base[lin];
  return (MODE == ACC_B_CONSTANT && !inside) ? outside : v;
}

/* the same where every dimension but the innermost is known to take the tap inside the array: `row` is the position of
 * the element's row (innermost index 0), `step` the elements between neighbours along every dimension */
template <int MODE, typename S, typename I>
ACC_DEV S acc_nd_read_row(const S *__restrict__ base, const acc_nd_index<I> &sh, const acc_nd_index<I> &step, const I row, const I x,
                          const acc_nd_offset &off, const S outside)
{
  I lin = row;
#pragma unroll
  for (int d = 0; d < ACC_STENCIL_RANK - 1; ++d) lin += (I)off.o[d] * step.i[d];
  const I i = x + (I)off.o[ACC_STENCIL_RANK - 1];
  const bool inside = i >= 0 && i < sh.i[ACC_STENCIL_RANK - 1];
  const S v = base[lin + acc_nd_boundary<MODE, I>(i, sh.i[ACC_STENCIL_RANK - 1])];
  return (MODE == ACC_B_CONSTANT && !inside) ? outside : v;
}

#if ACC_STENCIL_SOURCES == 2
#define ACC_STENCIL_ENTRY stencil2
#define ACC_SOURCE_PARAMS ACC_SRC1_PARAMS ACC_SRC2_PARAMS
#define ACC_SRC1_ARRAY(c) arrStencil1_##c
#define ACC_SRC2_ARRAY(c) arrStencil2_##c
#else
#define ACC_STENCIL_ENTRY stencil
#define ACC_SOURCE_PARAMS ACC_SRC1_PARAMS
#define ACC_SRC1_ARRAY(c) arrStencil_##c
#define ACC_SRC2_COMPONENTS(X, arg)
#endif

extern "C" __global__ void __launch_bounds__(ACC_BLOCK)
ACC_STENCIL_ENTRY(ACC_ENV_PARAMS ACC_OUT_PARAMS ACC_SOURCE_PARAMS, const int acc_walk ACC_GUARD_PARAM)
{
  ACC_GUARD_CHECK
  typedef ACC_ELT T;
  ACC_ENV_ASSUME
  (void)acc_walk;
  const Int64 acc_extents[ACC_STENCIL_RANK] = {ACC_OUT_EXTENTS};
  const Int64 acc_extents1[ACC_STENCIL_RANK] = {ACC_SRC1_EXTENTS};
#if ACC_STENCIL_SOURCES == 2
  const Int64 acc_extents2[ACC_STENCIL_RANK] = {ACC_SRC2_EXTENTS};
#endif
  Int64 n = 1, n1 = 1, n2 = 1;
#pragma unroll
  for (int d = 0; d < ACC_STENCIL_RANK; ++d) {
    n *= acc_extents[d];
    n1 *= acc_extents1[d];
#if ACC_STENCIL_SOURCES == 2
    n2 *= acc_extents2[d];
#endif
  }
  /* the value outside a constant boundary, component by component */
#define ACC_DECLARE_OUTSIDE1(c, CT, OUTSIDE, arg) const CT acc_outside1_##c = (CT)OUTSIDE;
#define ACC_DECLARE_OUTSIDE2(c, CT, OUTSIDE, arg) const CT acc_outside2_##c = (CT)OUTSIDE;
  ACC_SRC1_COMPONENTS(ACC_DECLARE_OUTSIDE1, 0)
  ACC_SRC2_COMPONENTS(ACC_DECLARE_OUTSIDE2, 0)
#undef ACC_DECLARE_OUTSIDE1
#undef ACC_DECLARE_OUTSIDE2

  auto elements = [&](auto width) {
    typedef decltype(width) I;
    acc_nd_index<I> sh, sh1, step1;
#pragma unroll
    for (int d = 0; d < ACC_STENCIL_RANK; ++d) { sh.i[d] = (I)acc_extents[d]; sh1.i[d] = (I)acc_extents1[d]; }
    /* (elements between neighbours along every dimension: the row-major position of an index is their inner product) */
    step1.i[ACC_STENCIL_RANK - 1] = 1;
#pragma unroll
    for (int d = ACC_STENCIL_RANK - 2; d >= 0; --d) step1.i[d] = step1.i[d + 1] * sh1.i[d + 1];
    constexpr int lo1[ACC_STENCIL_RANK] = ACC_SRC1_REACH_LO, hi1[ACC_STENCIL_RANK] = ACC_SRC1_REACH_HI;
#if ACC_STENCIL_SOURCES == 2
    acc_nd_index<I> sh2, step2;
#pragma unroll
    for (int d = 0; d < ACC_STENCIL_RANK; ++d) sh2.i[d] = (I)acc_extents2[d];
    step2.i[ACC_STENCIL_RANK - 1] = 1;
#pragma unroll
    for (int d = ACC_STENCIL_RANK - 2; d >= 0; --d) step2.i[d] = step2.i[d + 1] * sh2.i[d + 1];
    constexpr int lo2[ACC_STENCIL_RANK] = ACC_SRC2_REACH_LO, hi2[ACC_STENCIL_RANK] = ACC_SRC2_REACH_HI;
#endif
    auto inner_product = [&](const acc_nd_index<I> &a, const acc_nd_index<I> &b) -> I {
      I v = 0;
#pragma unroll
      for (int d = 0; d < ACC_STENCIL_RANK; ++d) v += a.i[d] * b.i[d];
      return v;
    };
    auto of_offset = [&](const acc_nd_offset &o, const acc_nd_index<I> &b) -> I {
      I v = 0;
#pragma unroll
      for (int d = 0; d < ACC_STENCIL_RANK; ++d) v += (I)o.o[d] * b.i[d];
      return v;
    };
    for (Int64 ix = (Int64)blockIdx.x * ACC_BLOCK + threadIdx.x; ix < n; ix += (Int64)gridDim.x * ACC_BLOCK) {
      acc_nd_index<I> at;
      I rest = (I)ix;
#pragma unroll
      for (int d = ACC_STENCIL_RANK - 1; d > 0; --d) {      /* innermost dimension last: Base.hs:207-218 */
        at.i[d] = rest % sh.i[d];
        rest /= sh.i[d];
      }
      at.i[0] = rest;
      /* An element whose taps all lie inside the source(s) -- nearly every element of an array that is not thin --
       * needs no boundary condition: a tap is then the element's own position plus a distance that is the same for
       * all elements (nine planes of 256^3 floats: 93 -> 50 us; 3 x 3 on 4096^2: 59 -> 40 us). */
      bool inside = ACC_ND_INNER != 0, rows_inside = ACC_ND_INNER != 0 && ACC_STENCIL_RANK > 1;
#pragma unroll
      for (int d = 0; d < ACC_STENCIL_RANK; ++d) {
        bool in_d = at.i[d] >= (I)lo1[d] && at.i[d] < sh1.i[d] - (I)hi1[d];
#if ACC_STENCIL_SOURCES == 2
        in_d = in_d && at.i[d] >= (I)lo2[d] && at.i[d] < sh2.i[d] - (I)hi2[d];
#endif
        inside = inside && in_d;
        if (d < ACC_STENCIL_RANK - 1) rows_inside = rows_inside && in_d;
      }
      /* (wave by wave: a wave with an element at the boundary among its 64 would go both ways, one after the other) */
      T r;
      if (__ballot(!inside) == 0) {
        const I here1 = inner_product(at, step1);
#define ACC_ND_READ1(c, ...) ACC_SRC1_ARRAY(c)[here1 + of_offset(acc_nd_offset{{__VA_ARGS__}}, step1)]
        ACC_STENCIL_TAPS1_ND(ACC_ND_READ1)
#undef ACC_ND_READ1
#if ACC_STENCIL_SOURCES == 2
        const I here2 = inner_product(at, step2);
#define ACC_ND_READ2(c, ...) ACC_SRC2_ARRAY(c)[here2 + of_offset(acc_nd_offset{{__VA_ARGS__}}, step2)]
        ACC_STENCIL_TAPS2_ND(ACC_ND_READ2)
#undef ACC_ND_READ2
#endif
        r = (T)(ACC_STENCIL_FN);
      } else if (__ballot(!rows_inside) == 0) {
        /* Only along the innermost dimension does a tap of this wave leave the array -- every wave of an array of a
         * few columns, and of one whose rows are no longer than a wave (3 x 3 x 3 x 3 on 64^4), but for the first and
         * last rows: the boundary condition is applied along that dimension alone. */
        const I x1 = at.i[ACC_STENCIL_RANK - 1], row1 = inner_product(at, step1) - x1;
#define ACC_ND_READ1(c, ...) acc_nd_read_row<ACC_BOUNDARY>(ACC_SRC1_ARRAY(c), sh1, step1, row1, x1, acc_nd_offset{{__VA_ARGS__}}, acc_outside1_##c)
        ACC_STENCIL_TAPS1_ND(ACC_ND_READ1)
#undef ACC_ND_READ1
#if ACC_STENCIL_SOURCES == 2
        const I row2 = inner_product(at, step2) - x1;
#define ACC_ND_READ2(c, ...) acc_nd_read_row<ACC_BOUNDARY2>(ACC_SRC2_ARRAY(c), sh2, step2, row2, x1, acc_nd_offset{{__VA_ARGS__}}, acc_outside2_##c)
        ACC_STENCIL_TAPS2_ND(ACC_ND_READ2)
#undef ACC_ND_READ2
#endif
        r = (T)(ACC_STENCIL_FN);
      } else {
#define ACC_ND_READ1(c, ...) acc_nd_read<ACC_BOUNDARY>(ACC_SRC1_ARRAY(c), sh1, at, acc_nd_offset{{__VA_ARGS__}}, acc_outside1_##c)
        ACC_STENCIL_TAPS1_ND(ACC_ND_READ1)
#undef ACC_ND_READ1
#if ACC_STENCIL_SOURCES == 2
#define ACC_ND_READ2(c, ...) acc_nd_read<ACC_BOUNDARY2>(ACC_SRC2_ARRAY(c), sh2, at, acc_nd_offset{{__VA_ARGS__}}, acc_outside2_##c)
        ACC_STENCIL_TAPS2_ND(ACC_ND_READ2)
#undef ACC_ND_READ2
#endif
        r = (T)(ACC_STENCIL_FN);
      }
      ACC_PUT(arrOut, ix, r);
    }
  };
  /* (the extents with a tap's offset added must fit as well: a stencil reaches 64 elements at most) */
  if (n < 0x7fff0000LL && n1 < 0x7fff0000LL && n2 < 0x7fff0000LL) elements((int)0);
  else elements((Int64)0);
}
