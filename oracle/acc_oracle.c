/*
 * acc_oracle.c -- TEST INFRASTRUCTURE, NOT PRODUCT CODE.
 *
 * A sequential, single-threaded CPU restatement of what each Accelerate
 * collective operation computes, used only as the checker for the HIP
 * skeletons (tests, the smoke check and the CPU-baseline leg of the bench).
 * Nothing in the shipped library links or calls this file.
 *
 * The semantics restated here are those of the Accelerate array language as
 * the reference backend documents and implements them:
 *
 *   scans      Data/Array/Accelerate/CUDA/CodeGen/PrefixSum.hs:137-198
 *              (Data.List-style scanl/scanl1/scanl' and right-handed duals),
 *              output lengths Data/Array/Accelerate/CUDA/Execute.hs:328-362
 *   folds      Data/Array/Accelerate/CUDA/CodeGen/Reduction.hs:37-55 (fold, fold1),
 *              :203-215 (seed combined as the SECOND operand; empty -> seed),
 *              Execute.hs:282-289 (fold1 of empty is an error; empty outer
 *              extents become 1)
 *   foldSeg    Reduction.hs:395-397 (segment i is [off[i], off[i+1])),
 *              :567-574 (empty segment -> seed), Execute.hs:320-324
 *              (#segments = length offsets - 1)
 *   permute    Data/Array/Accelerate/CUDA/CodeGen/IndexSpace.hs:144-158,197-210
 *              (out = defaults; out[p ix] = combine (src ix) (out[p ix]);
 *              `ignore` drops the element), Execute.hs:396-408 (defaults copy)
 *   stencil    Data/Array/Accelerate/CUDA/CodeGen/Stencil.hs:34-44 and the
 *              boundary index maps of CodeGen/Stencil/Extra.hs:191-226
 *   indexing   row-major, innermost dimension fastest: CodeGen/Base.hs:193-218
 *
 * PARITY PINNING.  The interpreter these semantics come from
 * (Data.Array.Accelerate.Interpreter, package accelerate-1.0.*, pinned by the
 * reference at stack-8.0.yaml:6-11) is not vendored and cannot run here.
 * Every function below is therefore pinned by independent means in
 * tests/test_oracle_*.py: the reference's doc-comment vectors
 * (PrefixSum.hs:149-166), numpy / scipy routines (cumsum, bincount,
 * ndimage.correlate, sparse CSR product, float64 dot), closed forms, algebraic
 * identities and a pure-Python brute force on tiny inputs.
 * Two points stay "parity unpinned" because only running the interpreter
 * could settle them:
 *   (1) the association direction of its sequential Float32 fold / foldSeg
 *       (both directions are provided: ORC_DIR_LEFT / ORC_DIR_RIGHT; integer
 *       results do not depend on it);
 *   (2) the operand order of scanr for a NON-commutative operator (the
 *       Data.List convention  out[i] = f x[i] out[i+1]  is used; the
 *       reference's kernel passes the carry first, PrefixSum.hs:263-266).
 *
 * Build: gcc -O2 -ffp-contract=off -fno-fast-math -shared -fPIC (see Makefile).
 * Float32 arithmetic is strict: every product and sum is rounded to float.
 */
#include <stdint.h>
#include <stddef.h>
#include <string.h>

#define ORC_OK            0
#define ORC_ERR_INVALID   1
#define ORC_ERR_EMPTY     2   /* fold1 / fold1Seg / scan1 over an empty range */

/* binary operators the tests exercise */
enum {
  ORC_OP_ADD = 0,
  ORC_OP_MUL = 1,
  ORC_OP_MIN = 2,
  ORC_OP_MAX = 3,
  ORC_OP_FIRST = 4,   /* f x y = x   (associative, not commutative) */
  ORC_OP_LAST  = 5,   /* f x y = y   (associative, not commutative) */
  ORC_OP_AFFINE16 = 6 /* integer types only: composition of the affine maps
                         t -> a*t+b over Z/2^16, packed as (a<<16)|b:
                         f x y = x . y  (associative, not commutative) */
};

enum { ORC_DIR_LEFT = 0, ORC_DIR_RIGHT = 1 };

/* scan variants (PrefixSum.hs:51-120) */
enum {
  ORC_SCANL = 0, ORC_SCANL1 = 1, ORC_SCANLP = 2,   /* scanl' */
  ORC_SCANR = 3, ORC_SCANR1 = 4, ORC_SCANRP = 5    /* scanr' */
};

/* stencil boundary modes (Stencil/Extra.hs:112-116) */
enum { ORC_CLAMP = 0, ORC_MIRROR = 1, ORC_WRAP = 2, ORC_CONSTANT = 3 };

/* ------------------------------------------------------------------------ */
/* operators                                                                */

static inline uint32_t affine16(uint32_t x, uint32_t y)
{
  /* (a1,b1).(a2,b2) = (a1*a2, a1*b2 + b1)  mod 2^16 */
  uint32_t a1 = x >> 16, b1 = x & 0xffffu, a2 = y >> 16, b2 = y & 0xffffu;
  return (((a1 * a2) & 0xffffu) << 16) | ((a1 * b2 + b1) & 0xffffu);
}

static inline int32_t op_i32(int op, int32_t x, int32_t y)
{
  switch (op) {
    case ORC_OP_ADD: return (int32_t)((uint32_t)x + (uint32_t)y);  /* wraps, as Int32 does */
    case ORC_OP_MUL: return (int32_t)((uint32_t)x * (uint32_t)y);
    case ORC_OP_MIN: return x < y ? x : y;
    case ORC_OP_MAX: return x > y ? x : y;
    case ORC_OP_FIRST: return x;
    case ORC_OP_LAST:  return y;
    case ORC_OP_AFFINE16: return (int32_t)affine16((uint32_t)x, (uint32_t)y);
  }
  return 0;
}

static inline int64_t op_i64(int op, int64_t x, int64_t y)
{
  switch (op) {
    case ORC_OP_ADD: return (int64_t)((uint64_t)x + (uint64_t)y);
    case ORC_OP_MUL: return (int64_t)((uint64_t)x * (uint64_t)y);
    case ORC_OP_MIN: return x < y ? x : y;
    case ORC_OP_MAX: return x > y ? x : y;
    case ORC_OP_FIRST: return x;
    case ORC_OP_LAST:  return y;
    case ORC_OP_AFFINE16: return (int64_t)affine16((uint32_t)x, (uint32_t)y);
  }
  return 0;
}

static inline float op_f32(int op, float x, float y)
{
  switch (op) {
    case ORC_OP_ADD: return x + y;
    case ORC_OP_MUL: return x * y;
    case ORC_OP_MIN: return x < y ? x : y;
    case ORC_OP_MAX: return x > y ? x : y;
    case ORC_OP_FIRST: return x;
    case ORC_OP_LAST:  return y;
  }
  return 0.0f;
}

static inline double op_f64(int op, double x, double y)
{
  switch (op) {
    case ORC_OP_ADD: return x + y;
    case ORC_OP_MUL: return x * y;
    case ORC_OP_MIN: return x < y ? x : y;
    case ORC_OP_MAX: return x > y ? x : y;
    case ORC_OP_FIRST: return x;
    case ORC_OP_LAST:  return y;
  }
  return 0.0;
}

static int op_valid(int op, int is_float)
{
  if (op < 0 || op > ORC_OP_AFFINE16) return 0;
  if (is_float && op == ORC_OP_AFFINE16) return 0;
  return 1;
}

/* ------------------------------------------------------------------------ */
/* fold / fold1 over one contiguous range (Reduction.hs:37-55,203-215).
 *
 *   LEFT :  ((x0 (+) x1) (+) ... (+) x_{n-1}) (+) z
 *   RIGHT:  x0 (+) (x1 (+) ( ... (x_{n-1} (+) z)))
 *
 * has_seed == 0 is fold1: n must be > 0 (Execute.hs:282-285).
 * An empty range with a seed yields the seed (Reduction.hs:212-214).       */

#define DEF_FOLD_RANGE(T, SUF)                                                 \
static int fold_range_##SUF(int op, int has_seed, T z, const T *x, int64_t n,  \
                            int dir, T *out)                                   \
{                                                                              \
  if (n <= 0) {                                                                \
    if (!has_seed) return ORC_ERR_EMPTY;                                       \
    *out = z;                                                                  \
    return ORC_OK;                                                             \
  }                                                                            \
  T acc;                                                                       \
  if (dir == ORC_DIR_LEFT) {                                                   \
    acc = x[0];                                                                \
    for (int64_t i = 1; i < n; ++i) acc = op_##SUF(op, acc, x[i]);             \
    if (has_seed) acc = op_##SUF(op, acc, z);                                  \
  } else {                                                                     \
    int64_t i = n - 1;                                                         \
    if (has_seed) acc = op_##SUF(op, x[i], z); else acc = x[i];                \
    for (--i; i >= 0; --i) acc = op_##SUF(op, x[i], acc);                      \
  }                                                                            \
  *out = acc;                                                                  \
  return ORC_OK;                                                               \
}

DEF_FOLD_RANGE(int32_t, i32)
DEF_FOLD_RANGE(int64_t, i64)
DEF_FOLD_RANGE(float,   f32)
DEF_FOLD_RANGE(double,  f64)

/* fold along the innermost dimension of an array of `outer` rows of `inner`
 * elements (row-major).  outer == 1 is the total reduction of a vector.
 * Execute.hs:287-289: an empty outer extent is treated as 1, so the caller
 * passes outer >= 1.                                                        */
#define DEF_FOLD(T, SUF, ISF)                                                  \
int orc_fold_##SUF(int op, int has_seed, T z, const T *x, int64_t outer,       \
                   int64_t inner, int dir, T *out)                             \
{                                                                              \
  if (!op_valid(op, ISF) || outer < 0 || inner < 0) return ORC_ERR_INVALID;    \
  for (int64_t r = 0; r < outer; ++r) {                                        \
    int rc = fold_range_##SUF(op, has_seed, z, x + r * inner, inner, dir,      \
                              out + r);                                        \
    if (rc) return rc;                                                         \
  }                                                                            \
  return ORC_OK;                                                               \
}

DEF_FOLD(int32_t, i32, 0)
DEF_FOLD(int64_t, i64, 0)
DEF_FOLD(float,   f32, 1)
DEF_FOLD(double,  f64, 1)

/* foldSeg / fold1Seg: segment s of the (single-row) input is
 * [off[s], off[s+1]); off has nseg+1 entries (Execute.hs:320-324).          */
#define DEF_FOLDSEG(T, SUF, ISF)                                               \
int orc_foldseg_##SUF(int op, int has_seed, T z, const T *x,                   \
                      const int32_t *off, int64_t nseg, int dir, T *out)       \
{                                                                              \
  if (!op_valid(op, ISF) || nseg < 0) return ORC_ERR_INVALID;                  \
  for (int64_t s = 0; s < nseg; ++s) {                                         \
    int64_t a = off[s], b = off[s + 1];                                        \
    if (b < a) return ORC_ERR_INVALID;                                         \
    int rc = fold_range_##SUF(op, has_seed, z, x + a, b - a, dir, out + s);    \
    if (rc) return rc;                                                         \
  }                                                                            \
  return ORC_OK;                                                               \
}

DEF_FOLDSEG(int32_t, i32, 0)
DEF_FOLDSEG(float,   f32, 1)
DEF_FOLDSEG(double,  f64, 1)

/* foldSeg / fold1Seg of an array of rank > 1 (`outer` rows of `inner`
 * elements): the descriptor segments the innermost dimension of every row
 * alike, segment s of row r being [r*inner + off[s], r*inner + off[s+1])
 * (CodeGen/Reduction.hs:473-474,485-486: base = (seg / num_segments) *
 * innerExtent, start = base + off[s], end = base + off[s+1]); the result is
 * outer x nseg, row-major (Execute.hs:323-324).  What a row holds beyond
 * off[nseg] belongs to no segment.                                          */
#define DEF_FOLDSEG_ND(T, SUF, ISF)                                            \
int orc_foldseg_nd_##SUF(int op, int has_seed, T z, const T *x, int64_t outer, \
                         int64_t inner, const int32_t *off, int64_t nseg,      \
                         int dir, T *out)                                      \
{                                                                              \
  if (!op_valid(op, ISF) || nseg < 0 || outer < 0 || inner < 0)                \
    return ORC_ERR_INVALID;                                                    \
  for (int64_t r = 0; r < outer; ++r)                                          \
    for (int64_t s = 0; s < nseg; ++s) {                                       \
      int64_t a = off[s], b = off[s + 1];                                      \
      if (b < a || a < 0 || b > inner) return ORC_ERR_INVALID;                 \
      int rc = fold_range_##SUF(op, has_seed, z, x + r * inner + a, b - a,     \
                                dir, out + r * nseg + s);                      \
      if (rc) return rc;                                                       \
    }                                                                          \
  return ORC_OK;                                                               \
}

DEF_FOLDSEG_ND(int32_t, i32, 0)
DEF_FOLDSEG_ND(float,   f32, 1)
DEF_FOLDSEG_ND(double,  f64, 1)

/* ------------------------------------------------------------------------ */
/* The two fused Float32 configurations, written out so that no temporary
 * array is needed at full size.                                             */

/* fold (+) 0 (zipWith (*) xs ys): each product is rounded to Float32 before
 * it is added (the interpreter evaluates (*) and (+) as separate Float32
 * operations).                                                              */
float orc_dot_f32(const float *x, const float *y, int64_t n, int dir)
{
  const float z = 0.0f;
  if (n <= 0) return z;
  float acc;
  if (dir == ORC_DIR_LEFT) {
    acc = x[0] * y[0];
    for (int64_t i = 1; i < n; ++i) { float p = x[i] * y[i]; acc = acc + p; }
    acc = acc + z;
  } else {
    float p = x[n - 1] * y[n - 1];
    acc = p + z;
    for (int64_t i = n - 2; i >= 0; --i) { p = x[i] * y[i]; acc = p + acc; }
  }
  return acc;
}

/* the same sum in Float64 with Float64 products of the Float32 inputs: the
 * ground truth both the oracle and the GPU result are reported against.     */
double orc_dot_f64(const float *x, const float *y, int64_t n)
{
  double acc = 0.0;
  for (int64_t i = 0; i < n; ++i) acc += (double)x[i] * (double)y[i];
  return acc;
}

/* sum_i |x_i y_i| in Float64: the condition-number denominator.             */
double orc_dot_abs_f64(const float *x, const float *y, int64_t n)
{
  double acc = 0.0;
  for (int64_t i = 0; i < n; ++i) {
    double p = (double)x[i] * (double)y[i];
    acc += p < 0 ? -p : p;
  }
  return acc;
}

/* CSR sparse matrix-vector product  y = A x  composed as
 * foldSeg (+) 0 (zipWith (*) vals (backpermute .. (x ! cols))) offsets.      */
int orc_smvm_f32(const float *vals, const int32_t *cols, const int32_t *off,
                 const float *x, int64_t nrows, int dir, float *y)
{
  for (int64_t r = 0; r < nrows; ++r) {
    int64_t a = off[r], b = off[r + 1];
    if (b < a) return ORC_ERR_INVALID;
    float acc = 0.0f;
    if (b > a) {
      if (dir == ORC_DIR_LEFT) {
        acc = vals[a] * x[cols[a]];
        for (int64_t i = a + 1; i < b; ++i) { float p = vals[i] * x[cols[i]]; acc = acc + p; }
        acc = acc + 0.0f;
      } else {
        float p = vals[b - 1] * x[cols[b - 1]];
        acc = p + 0.0f;
        for (int64_t i = b - 2; i >= a; --i) { p = vals[i] * x[cols[i]]; acc = p + acc; }
      }
    }
    y[r] = acc;
  }
  return ORC_OK;
}

int orc_smvm_f64(const float *vals, const int32_t *cols, const int32_t *off,
                 const float *x, int64_t nrows, double *y, double *yabs)
{
  for (int64_t r = 0; r < nrows; ++r) {
    double acc = 0.0, aacc = 0.0;
    for (int64_t i = off[r]; i < off[r + 1]; ++i) {
      double p = (double)vals[i] * (double)x[cols[i]];
      acc += p;
      aacc += p < 0 ? -p : p;
    }
    y[r] = acc;
    if (yabs) yabs[r] = aacc;
  }
  return ORC_OK;
}

/* ------------------------------------------------------------------------ */
/* scans (PrefixSum.hs:137-198; output shapes Execute.hs:328-362)
 *
 *   scanl  f z xs : n+1 outputs, out[0] = z,     out[i+1] = f out[i] x[i]
 *   scanl1 f   xs : n   outputs, out[0] = x[0],  out[i]   = f out[i-1] x[i]
 *   scanl' f z xs : (init r, last r) with r = scanl f z xs
 *   scanr  f z xs : n+1 outputs, out[n] = z,     out[i]   = f x[i] out[i+1]
 *   scanr1 f   xs : n   outputs, out[n-1]=x[n-1],out[i]   = f x[i] out[i+1]
 *   scanr' f z xs : (tail r, head r) with r = scanr f z xs
 *
 * `out` must hold n+1 elements for scanl/scanr and n otherwise; `total`
 * receives the reduction for the primed variants (may be NULL otherwise).   */
#define DEF_SCAN(T, SUF, ISF)                                                  \
int orc_scan_##SUF(int kind, int op, T z, const T *x, int64_t n, T *out,       \
                   T *total)                                                   \
{                                                                              \
  if (!op_valid(op, ISF) || n < 0) return ORC_ERR_INVALID;                     \
  T acc;                                                                       \
  switch (kind) {                                                              \
    case ORC_SCANL:                                                            \
      acc = z; out[0] = acc;                                                   \
      for (int64_t i = 0; i < n; ++i) { acc = op_##SUF(op, acc, x[i]); out[i + 1] = acc; } \
      return ORC_OK;                                                           \
    case ORC_SCANLP:                                                           \
      acc = z;                                                                 \
      for (int64_t i = 0; i < n; ++i) { out[i] = acc; acc = op_##SUF(op, acc, x[i]); } \
      if (total) *total = acc;                                                 \
      return ORC_OK;                                                           \
    case ORC_SCANL1:                                                           \
      if (n == 0) return ORC_OK;                                               \
      acc = x[0]; out[0] = acc;                                                \
      for (int64_t i = 1; i < n; ++i) { acc = op_##SUF(op, acc, x[i]); out[i] = acc; } \
      return ORC_OK;                                                           \
    case ORC_SCANR:                                                            \
      acc = z; out[n] = acc;                                                   \
      for (int64_t i = n - 1; i >= 0; --i) { acc = op_##SUF(op, x[i], acc); out[i] = acc; } \
      return ORC_OK;                                                           \
    case ORC_SCANRP:                                                           \
      acc = z;                                                                 \
      for (int64_t i = n - 1; i >= 0; --i) { out[i] = acc; acc = op_##SUF(op, x[i], acc); } \
      if (total) *total = acc;                                                 \
      return ORC_OK;                                                           \
    case ORC_SCANR1:                                                           \
      if (n == 0) return ORC_OK;                                               \
      acc = x[n - 1]; out[n - 1] = acc;                                        \
      for (int64_t i = n - 2; i >= 0; --i) { acc = op_##SUF(op, x[i], acc); out[i] = acc; } \
      return ORC_OK;                                                           \
  }                                                                            \
  return ORC_ERR_INVALID;                                                      \
}

DEF_SCAN(int32_t, i32, 0)
DEF_SCAN(int64_t, i64, 0)
DEF_SCAN(float,   f32, 1)
DEF_SCAN(double,  f64, 1)

/* ------------------------------------------------------------------------ */
/* permute (IndexSpace.hs:144-158,197-210; Execute.hs:396-408)
 *
 *   out = defaults
 *   for ix in source order:  j = dst[ix];  unless j == ignore (-1):
 *       out[j] = combine (src ix) (out[j])       -- new value FIRST
 *
 * `src` may be NULL, meaning the constant source array `fill 1`.            */
#define DEF_PERMUTE(T, SUF, ISF)                                               \
int orc_permute_##SUF(int op, const T *defaults, int64_t ntarget,              \
                      const int32_t *dst, const T *src, int64_t nsrc, T *out)  \
{                                                                              \
  if (!op_valid(op, ISF) || ntarget < 0 || nsrc < 0) return ORC_ERR_INVALID;   \
  if (out != defaults) memcpy(out, defaults, (size_t)ntarget * sizeof(T));     \
  for (int64_t ix = 0; ix < nsrc; ++ix) {                                      \
    int64_t j = dst[ix];                                                       \
    if (j == -1) continue;                                                     \
    if (j < 0 || j >= ntarget) return ORC_ERR_INVALID;                         \
    T v = src ? src[ix] : (T)1;                                                \
    out[j] = op_##SUF(op, v, out[j]);                                          \
  }                                                                            \
  return ORC_OK;                                                               \
}

DEF_PERMUTE(int32_t, i32, 0)
DEF_PERMUTE(float,   f32, 1)

/* ------------------------------------------------------------------------ */
/* index-space transforms: backpermute / gather (IndexSpace.hs:96-141)       */
int orc_backpermute_f32(const float *in, int64_t nin, const int32_t *idx,
                        int64_t nout, float *out)
{
  for (int64_t i = 0; i < nout; ++i) {
    int64_t j = idx[i];
    if (j < 0 || j >= nin) return ORC_ERR_INVALID;
    out[i] = in[j];
  }
  return ORC_OK;
}

int orc_backpermute_i32(const int32_t *in, int64_t nin, const int32_t *idx,
                        int64_t nout, int32_t *out)
{
  for (int64_t i = 0; i < nout; ++i) {
    int64_t j = idx[i];
    if (j < 0 || j >= nin) return ORC_ERR_INVALID;
    out[i] = in[j];
  }
  return ORC_OK;
}

/* ------------------------------------------------------------------------ */
/* stencils (Stencil.hs:34-44).  Boundary index maps exactly as
 * Stencil/Extra.hs:198-226:
 *   clamp : max(0, min(i, sz-1))
 *   mirror: i < 0 ? -i : i >= sz ? sz - (i - sz + 2) : i
 *   wrap  : i < 0 ? sz + i : i >= sz ? i - sz : i
 * constant: out-of-range taps read the constant (Extra.hs:122-128).         */
static inline int64_t bmap(int mode, int64_t i, int64_t sz)
{
  switch (mode) {
    case ORC_CLAMP:  { int64_t m = i < sz - 1 ? i : sz - 1; return m > 0 ? m : 0; }
    case ORC_MIRROR: return i < 0 ? -i : (i >= sz ? sz - (i - sz + 2) : i);
    case ORC_WRAP:   return i < 0 ? sz + i : (i >= sz ? i - sz : i);
  }
  return i;
}

/* A linear 2-D stencil: ntaps taps at offsets (dy[k], dx[k]) with
 * coefficients c[k], evaluated as the user expression
 *
 *     ((c0*t0 + c1*t1) + c2*t2 + ... ) / divisor
 *
 * left to right in Float32, every product and sum rounded; divisor == 1
 * skips the division.                                                       */
int orc_stencil2d_f32(const float *in, int64_t h, int64_t w, int ntaps,
                      const int32_t *dy, const int32_t *dx, const float *c,
                      float divisor, int mode, float constant, float *out)
{
  if (h < 0 || w < 0 || ntaps <= 0 || mode < 0 || mode > ORC_CONSTANT) return ORC_ERR_INVALID;
  for (int64_t y = 0; y < h; ++y) {
    for (int64_t x = 0; x < w; ++x) {
      float acc = 0.0f;
      for (int k = 0; k < ntaps; ++k) {
        int64_t yy = y + dy[k], xx = x + dx[k];
        float t;
        if (mode == ORC_CONSTANT) {
          t = (yy >= 0 && yy < h && xx >= 0 && xx < w) ? in[yy * w + xx] : constant;
        } else {
          t = in[bmap(mode, yy, h) * w + bmap(mode, xx, w)];
        }
        float p = c[k] * t;
        acc = (k == 0) ? p : acc + p;
      }
      out[y * w + x] = (divisor == 1.0f) ? acc : acc / divisor;
    }
  }
  return ORC_OK;
}

/* `iters` applications, ping-ponging between out and tmp; the result is
 * always left in `out`.                                                     */
int orc_stencil2d_iter_f32(const float *in, int64_t h, int64_t w, int ntaps,
                           const int32_t *dy, const int32_t *dx, const float *c,
                           float divisor, int mode, float constant, int iters,
                           float *out, float *tmp)
{
  if (iters <= 0) { memcpy(out, in, (size_t)(h * w) * sizeof(float)); return ORC_OK; }
  const float *src = in;
  /* arrange that the last write lands in `out` */
  float *dst = (iters & 1) ? out : tmp;
  for (int it = 0; it < iters; ++it) {
    int rc = orc_stencil2d_f32(src, h, w, ntaps, dy, dx, c, divisor, mode, constant, dst);
    if (rc) return rc;
    src = dst;
    dst = (dst == out) ? tmp : out;
  }
  return ORC_OK;
}

/* 1-D linear stencil, same conventions                                      */
int orc_stencil1d_f32(const float *in, int64_t n, int ntaps, const int32_t *dx,
                      const float *c, float divisor, int mode, float constant,
                      float *out)
{
  if (n < 0 || ntaps <= 0 || mode < 0 || mode > ORC_CONSTANT) return ORC_ERR_INVALID;
  for (int64_t x = 0; x < n; ++x) {
    float acc = 0.0f;
    for (int k = 0; k < ntaps; ++k) {
      int64_t xx = x + dx[k];
      float t;
      if (mode == ORC_CONSTANT) t = (xx >= 0 && xx < n) ? in[xx] : constant;
      else t = in[bmap(mode, xx, n)];
      float p = c[k] * t;
      acc = (k == 0) ? p : acc + p;
    }
    out[x] = (divisor == 1.0f) ? acc : acc / divisor;
  }
  return ORC_OK;
}

/* exposed for the boundary-map unit tests */
int64_t orc_boundary_index(int mode, int64_t i, int64_t sz) { return bmap(mode, i, sz); }

/* ------------------------------------------------------------------------ */
/* zipWith (*) xs ys (Mapping.hs:59-78: one element function application per
 * index): every product rounded to Float32.  The CPU side of the map-family
 * benchmark leg.                                                            */
void orc_zipwith_mul_f32(const float *x, const float *y, int64_t n, float *out)
{
  for (int64_t i = 0; i < n; ++i) out[i] = x[i] * y[i];
}
