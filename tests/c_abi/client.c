/*
 * A client of libacchip written in plain C99 against include/acc_hip.h alone:
 * what a foreign-function binding of another language sees.  It runs the
 * benchmark programs at small sizes (dot product, the three scans, a
 * histogram by permute, a 3x3 stencil, a sparse matrix-vector product by
 * foldSeg) and the memory table, checks every result against a loop written
 * here, and exercises the error statuses.
 *
 *   client            run everything on device 0; exit status 0 = all checks passed
 *   client --no-gpu   only what needs no device: generate and compile a skeleton for gfx950
 */
#include <math.h>
#include <stdio.h>
#include <stdlib.h>
#include <string.h>

#include "acc_hip.h"

static int failures = 0;

#define CHECK(cond, what)                                                        \
  do {                                                                           \
    if (!(cond)) { printf("FAILED: %s (%s:%d)\n", what, __FILE__, __LINE__); ++failures; } \
  } while (0)

#define OK(call)                                                                 \
  do {                                                                           \
    int rc_ = (call);                                                            \
    if (rc_ != ACC_OK) {                                                         \
      printf("FAILED: %s -> status %d: %s (%s:%d)\n", #call, rc_, acc_last_error(), __FILE__, __LINE__); \
      ++failures;                                                                \
      return;                                                                    \
    }                                                                            \
  } while (0)

static unsigned long long rng_state = 0x9E3779B97F4A7C15ull;
static unsigned int rnd(void)
{
  rng_state = rng_state * 6364136223846793005ull + 1442695040888963407ull;
  return (unsigned int)(rng_state >> 33);
}

static acc_array vector_of(acc_devptr p, int64_t n)
{
  acc_array a;
  memset(&a, 0, sizeof a);
  a.rank = 1;
  a.ncomp = 1;
  a.shape[0] = n;
  a.ptr[0] = p;
  return a;
}

static acc_env_sig sig(int rank, const char *type)
{
  acc_env_sig s;
  memset(&s, 0, sizeof s);
  s.rank = rank;
  s.ncomp = 1;
  s.type[0] = type;
  return s;
}

static acc_devptr upload(acc_context ctx, const void *host, size_t bytes)
{
  acc_devptr p = 0;
  if (acc_malloc(ctx, bytes, &p) != ACC_OK || acc_memcpy_h2d(ctx, p, host, bytes) != ACC_OK) {
    printf("FAILED: upload: %s\n", acc_last_error());
    ++failures;
  }
  return p;
}

/* ---- no device needed ---------------------------------------------------- */
static void compile_without_a_device(void)
{
  acc_env_sig env[2];
  acc_skel_desc d;
  size_t size = 0;
  const char *text = NULL, *entry = NULL;
  env[0] = sig(1, "float");
  env[1] = sig(1, "float");
  memset(&d, 0, sizeof d);
  d.kind = ACC_SKEL_FOLD;
  d.n_env = 2;
  d.env = env;
  d.elt_type = "float";
  d.get = "arrIn0_0[ix] * arrIn1_0[ix]";
  d.combine = "x + y";
  d.seed = "0.0f";
  OK(acc_skel_preview(&d, 0, &text, &entry));
  CHECK(strcmp(entry, "foldAll") == 0 && strstr(text, "arrIn0_0[ix] * arrIn1_0[ix]") != NULL, "generated text");
  OK(acc_skel_compile_only("gfx950", &d, &size));
  CHECK(size > 1000, "code object size");
  d.combine = "x +* y";
  CHECK(acc_skel_compile_only("gfx950", &d, &size) == ACC_ERR_COMPILE && strlen(acc_compile_log()) > 0, "compile error status and log");
  d.combine = NULL;
  CHECK(acc_skel_compile_only("gfx950", &d, &size) == ACC_ERR_INVALID, "missing fragment is refused");
}

/* ---- dot product: fold (+) 0 (zipWith (*) xs ys) -------------------------- */
static void dot_product(acc_context ctx)
{
  enum { N = 100003 };
  static float x[N], y[N];
  acc_env_sig env[2];
  acc_skel_desc d;
  acc_skel sk = NULL;
  acc_array in[2], out;
  acc_devptr dx, dy, dr;
  int64_t shape[1] = {N};
  double ref = 0.0;
  float got = 0.0f;
  int i;
  for (i = 0; i < N; ++i) {
    x[i] = (float)(rnd() % 17) - 8.0f;        /* small whole numbers: every order of summation gives the same float */
    y[i] = (float)(rnd() % 5) - 2.0f;
    ref += (double)x[i] * y[i];
  }
  env[0] = sig(1, "float");
  env[1] = sig(1, "float");
  memset(&d, 0, sizeof d);
  d.kind = ACC_SKEL_FOLD;
  d.n_env = 2;
  d.env = env;
  d.elt_type = "float";
  d.get = "arrIn0_0[ix] * arrIn1_0[ix]";
  d.combine = "x + y";
  d.seed = "0.0f";
  OK(acc_skel_create(ctx, &d, &sk));
  dx = upload(ctx, x, sizeof x);
  dy = upload(ctx, y, sizeof y);
  OK(acc_malloc(ctx, sizeof(float), &dr));
  in[0] = vector_of(dx, N);
  in[1] = vector_of(dy, N);
  memset(&out, 0, sizeof out);
  out.rank = 0;
  out.ncomp = 1;
  out.ptr[0] = dr;
  OK(acc_exec_fold(sk, in, 1, shape, &out, NULL));
  OK(acc_memcpy_d2h(ctx, &got, dr, sizeof got));
  CHECK((double)got == ref, "dot product");
  /* fold1 of nothing is an error, fold of nothing the seed (Execute.hs:282-285, Reduction.hs:212-214) */
  shape[0] = 0;
  OK(acc_exec_fold(sk, in, 1, shape, &out, NULL));
  OK(acc_memcpy_d2h(ctx, &got, dr, sizeof got));
  CHECK(got == 0.0f, "fold of an empty array is the seed");
  OK(acc_skel_destroy(sk));
  d.kind = ACC_SKEL_FOLD1;
  d.seed = NULL;
  OK(acc_skel_create(ctx, &d, &sk));
  CHECK(acc_exec_fold(sk, in, 1, shape, &out, NULL) == ACC_ERR_INVALID, "fold1 of an empty array is refused");
  OK(acc_skel_destroy(sk));
  acc_free(ctx, dx);
  acc_free(ctx, dy);
  acc_free(ctx, dr);
}

/* ---- scanl, scanl1, scanr (+) over Int32 ---------------------------------- */
static void prefix_sums(acc_context ctx)
{
  enum { N = 70001 };
  static int32_t x[N], got[N + 1], ref[N + 1];
  const int kinds[3] = {ACC_SKEL_SCANL, ACC_SKEL_SCANL1, ACC_SKEL_SCANR};
  acc_env_sig env[1];
  acc_devptr dx, dout;
  int k, i;
  for (i = 0; i < N; ++i) x[i] = (int32_t)(rnd() % 16);
  env[0] = sig(1, "Int32");
  dx = upload(ctx, x, sizeof x);
  OK(acc_malloc(ctx, sizeof got, &dout));
  for (k = 0; k < 3; ++k) {
    acc_skel_desc d;
    acc_skel sk = NULL;
    acc_array in = vector_of(dx, N), out;
    int64_t m = kinds[k] == ACC_SKEL_SCANL1 ? N : N + 1;
    memset(&d, 0, sizeof d);
    d.kind = kinds[k];
    d.n_env = 1;
    d.env = env;
    d.elt_type = "Int32";
    d.get = "arrIn0_0[ix]";
    d.combine = "x + y";
    d.seed = kinds[k] == ACC_SKEL_SCANL1 ? NULL : "7";
    OK(acc_skel_create(ctx, &d, &sk));
    out = vector_of(dout, m);
    OK(acc_exec_scan(sk, &in, N, &out, NULL, NULL));
    OK(acc_memcpy_d2h(ctx, got, dout, (size_t)m * sizeof(int32_t)));
    if (kinds[k] == ACC_SKEL_SCANL) {            /* [z, z+x0, ..., z+x0+..+x(n-1)] */
      ref[0] = 7;
      for (i = 0; i < N; ++i) ref[i + 1] = ref[i] + x[i];
    } else if (kinds[k] == ACC_SKEL_SCANL1) {
      ref[0] = x[0];
      for (i = 1; i < N; ++i) ref[i] = ref[i - 1] + x[i];
    } else {                                     /* scanr: [x0+..+z, ..., x(n-1)+z, z] */
      ref[N] = 7;
      for (i = N - 1; i >= 0; --i) ref[i] = ref[i + 1] + x[i];
    }
    CHECK(memcmp(got, ref, (size_t)m * sizeof(int32_t)) == 0, k == 0 ? "scanl" : k == 1 ? "scanl1" : "scanr");
    OK(acc_skel_destroy(sk));
  }
  acc_free(ctx, dx);
  acc_free(ctx, dout);
}

/* ---- histogram: permute (+) zeros (\i -> keys ! i) ones -------------------- */
static void histogram(acc_context ctx)
{
  enum { N = 200000, BINS = 256 };
  static int32_t keys[N], zeros[BINS], got[BINS], ref[BINS];
  acc_env_sig env[1];
  acc_skel_desc d;
  acc_skel sk = NULL;
  acc_array in, dfl, out;
  acc_devptr dk, dz, dout;
  int i;
  for (i = 0; i < N; ++i) {
    keys[i] = (int32_t)(rnd() % (BINS + 8)) - 4;  /* a few outside the result on both sides: dropped */
    if (keys[i] >= 0 && keys[i] < BINS) ref[keys[i]]++;
  }
  env[0] = sig(1, "Int32");
  memset(&d, 0, sizeof d);
  d.kind = ACC_SKEL_PERMUTE;
  d.n_env = 1;
  d.env = env;
  d.elt_type = "Int32";
  d.out_rank = 1;
  d.get = "1";
  d.combine = "x + y";
  d.permutation = "arrIn0_0[ix]";
  d.combine_hint = ACC_COMBINE_ADD;
  OK(acc_skel_create(ctx, &d, &sk));
  dk = upload(ctx, keys, sizeof keys);
  dz = upload(ctx, zeros, sizeof zeros);
  OK(acc_malloc(ctx, sizeof got, &dout));
  in = vector_of(dk, N);
  dfl = vector_of(dz, BINS);
  out = vector_of(dout, BINS);
  OK(acc_exec_permute(sk, &in, N, &dfl, &out, NULL));
  OK(acc_memcpy_d2h(ctx, got, dout, sizeof got));
  CHECK(memcmp(got, ref, sizeof ref) == 0, "histogram");
  OK(acc_skel_destroy(sk));
  acc_free(ctx, dk);
  acc_free(ctx, dz);
  acc_free(ctx, dout);
}

/* ---- 3x3 Gaussian with clamped edges --------------------------------------- */
static void gaussian(acc_context ctx)
{
  enum { H = 67, W = 301 };
  static float img[H][W], got[H][W];
  static const int32_t dy[9] = {-1, -1, -1, 0, 0, 0, 1, 1, 1}, dx[9] = {-1, 0, 1, -1, 0, 1, -1, 0, 1};
  static const float wt[9] = {1, 2, 1, 2, 4, 2, 1, 2, 1};
  acc_skel_desc d;
  acc_skel sk = NULL;
  acc_array in, out;
  acc_devptr din, dout;
  int y, x, k, bad = 0;
  for (y = 0; y < H; ++y)
    for (x = 0; x < W; ++x) img[y][x] = (float)(rnd() % 64);
  memset(&d, 0, sizeof d);
  d.kind = ACC_SKEL_STENCIL;
  d.elt_type = "float";
  d.out_rank = 2;
  d.boundary = ACC_BOUNDARY_CLAMP;
  d.n_taps = 9;
  d.tap_dy = dy;
  d.tap_dx = dx;
  d.stencil_fn = "(t0 + 2.0f * t1 + t2 + 2.0f * t3 + 4.0f * t4 + 2.0f * t5 + t6 + 2.0f * t7 + t8) / 16.0f";
  OK(acc_skel_create(ctx, &d, &sk));
  din = upload(ctx, img, sizeof img);
  OK(acc_malloc(ctx, sizeof got, &dout));
  memset(&in, 0, sizeof in);
  in.rank = 2;
  in.ncomp = 1;
  in.shape[0] = H;
  in.shape[1] = W;
  in.ptr[0] = din;
  out = in;
  out.ptr[0] = dout;
  OK(acc_exec_stencil(sk, NULL, &in, &out, NULL));
  OK(acc_memcpy_d2h(ctx, got, dout, sizeof got));
  for (y = 0; y < H; ++y)
    for (x = 0; x < W; ++x) {
      float s = 0.0f;                            /* whole numbers up to 64 * 16: exact in float in any order */
      for (k = 0; k < 9; ++k) {
        int yy = y + dy[k], xx = x + dx[k];
        yy = yy < 0 ? 0 : yy >= H ? H - 1 : yy;
        xx = xx < 0 ? 0 : xx >= W ? W - 1 : xx;
        s += wt[k] * img[yy][xx];
      }
      if (got[y][x] != s / 16.0f) ++bad;
    }
  CHECK(bad == 0, "3x3 gaussian, clamp");
  OK(acc_skel_destroy(sk));
  acc_free(ctx, din);
  acc_free(ctx, dout);
}

/* ---- sparse matrix-vector product: foldSeg (+) 0 (zipWith (*) vals (gather cols x)) */
static void smvm(acc_context ctx)
{
  enum { ROWS = 5000, COLS = 777, MAXNNZ = ROWS * 24 };
  static int32_t offs[ROWS + 1], cols[MAXNNZ];
  static float vals[MAXNNZ], xv[COLS], got[ROWS];
  acc_env_sig env[3];
  acc_skel_desc d;
  acc_skel sk = NULL;
  acc_array in[3], seg, out;
  acc_devptr dv, dc, dxv, doffs, dout;
  int r, i, nnz = 0, bad = 0;
  for (r = 0; r < ROWS; ++r) {
    int len = (int)(rnd() % 24);
    if (r % 11 == 0) len = 0;                    /* empty rows yield the seed */
    offs[r] = nnz;
    for (i = 0; i < len; ++i, ++nnz) {
      cols[nnz] = (int32_t)(rnd() % COLS);
      vals[nnz] = (float)(rnd() % 9) - 4.0f;
    }
  }
  offs[ROWS] = nnz;
  for (i = 0; i < COLS; ++i) xv[i] = (float)(rnd() % 7) - 3.0f;
  env[0] = sig(1, "float");
  env[1] = sig(1, "Int32");
  env[2] = sig(1, "float");
  memset(&d, 0, sizeof d);
  d.kind = ACC_SKEL_FOLDSEG;
  d.n_env = 3;
  d.env = env;
  d.elt_type = "float";
  d.get = "arrIn0_0[ix] * arrIn2_0[arrIn1_0[ix]]";
  d.combine = "x + y";
  d.seed = "0.0f";
  d.seg_type = "Int32";
  OK(acc_skel_create(ctx, &d, &sk));
  dv = upload(ctx, vals, sizeof vals);
  dc = upload(ctx, cols, sizeof cols);
  dxv = upload(ctx, xv, sizeof xv);
  doffs = upload(ctx, offs, sizeof offs);
  OK(acc_malloc(ctx, sizeof got, &dout));
  in[0] = vector_of(dv, nnz);
  in[1] = vector_of(dc, nnz);
  in[2] = vector_of(dxv, COLS);
  seg = vector_of(doffs, ROWS + 1);
  out = vector_of(dout, ROWS);
  OK(acc_exec_foldseg(sk, in, nnz, &seg, &out, NULL));
  OK(acc_memcpy_d2h(ctx, got, dout, sizeof got));
  for (r = 0; r < ROWS; ++r) {
    float s = 0.0f;
    for (i = offs[r]; i < offs[r + 1]; ++i) s += vals[i] * xv[cols[i]];
    if (got[r] != s) ++bad;
  }
  CHECK(bad == 0, "sparse matrix-vector product");
  OK(acc_skel_destroy(sk));
  acc_free(ctx, dv);
  acc_free(ctx, dc);
  acc_free(ctx, dxv);
  acc_free(ctx, doffs);
  acc_free(ctx, dout);
}

/* ---- foldSeg over the rows of a matrix: the same segments in every row ------------------------------------- */
static void segmented_rows(acc_context ctx)
{
  enum { ROWS = 300, W = 100, NSEG = 4 };
  static int32_t m[ROWS * W], got[ROWS * NSEG];
  static const int32_t offs[NSEG + 1] = {0, 10, 10, 55, 93};          /* an empty segment, and a tail nobody reads */
  acc_env_sig env[1];
  acc_skel_desc d;
  acc_skel sk = NULL;
  acc_array in, seg, out;
  acc_devptr dm, doffs, dout;
  int64_t shape[2] = {ROWS, W};
  int r, k, i, bad = 0;
  for (i = 0; i < ROWS * W; ++i) m[i] = (int32_t)(rnd() % 200) - 100;
  env[0] = sig(2, "Int32");
  memset(&d, 0, sizeof d);
  d.kind = ACC_SKEL_FOLDSEG;
  d.n_env = 1;
  d.env = env;
  d.elt_type = "Int32";
  d.out_rank = 2;                                /* the rank of the input and of the result */
  d.get = "arrIn0_0[ix]";
  d.combine = "x + y";
  d.seed = "7";
  OK(acc_skel_create(ctx, &d, &sk));
  dm = upload(ctx, m, sizeof m);
  doffs = upload(ctx, offs, sizeof offs);
  OK(acc_malloc(ctx, sizeof got, &dout));
  memset(&in, 0, sizeof in);
  in.rank = 2; in.ncomp = 1; in.shape[0] = ROWS; in.shape[1] = W; in.ptr[0] = dm;
  memset(&out, 0, sizeof out);
  out.rank = 2; out.ncomp = 1; out.shape[0] = ROWS; out.shape[1] = NSEG; out.ptr[0] = dout;
  seg = vector_of(doffs, NSEG + 1);
  OK(acc_exec_foldseg_nd(sk, &in, 2, shape, &seg, &out, NULL));
  OK(acc_memcpy_d2h(ctx, got, dout, sizeof got));
  for (r = 0; r < ROWS; ++r)
    for (k = 0; k < NSEG; ++k) {
      int32_t sum = 7;
      for (i = offs[k]; i < offs[k + 1]; ++i) sum += m[r * W + i];
      if (got[r * NSEG + k] != sum) ++bad;
    }
  CHECK(bad == 0, "segmented sums of every row of a matrix");
  CHECK(acc_exec_foldseg(sk, &in, ROWS * W, &seg, &out, NULL) == ACC_ERR_INVALID, "the vector entry refuses a rank-2 kernel");
  OK(acc_skel_destroy(sk));
  acc_free(ctx, dm);
  acc_free(ctx, doffs);
  acc_free(ctx, dout);
}

/* ---- awhile: double a vector until its largest element passes a bound, twelve iterations enqueued ahead -------- */
static void guarded_loop(acc_context ctx)
{
  enum { N = 50000, AHEAD = 12 };
  static int32_t x[N], got[N];
  acc_env_sig env[1], senv[1];
  acc_skel_desc d;
  acc_skel dbl = NULL, mx = NULL, below = NULL;
  acc_guard guard = NULL;
  acc_stream st = NULL;
  acc_devptr buf[AHEAD + 1], dtop, dflag;
  acc_array a, b, top, flag;
  int64_t n = N, count = -1;
  int32_t alive = -1;
  int i, k, steps = 0, top_now = 0;
  for (i = 0; i < N; ++i) { x[i] = (int32_t)(rnd() % 40) + 1; if (x[i] > top_now) top_now = x[i]; }
  while (top_now < 5000) { top_now *= 2; ++steps; }             /* what the loop should do: `steps` doublings */
  env[0] = sig(1, "Int32");
  memset(&d, 0, sizeof d);
  d.flags = ACC_FLAG_GUARDED;
  d.n_env = 1;
  d.env = env;
  d.elt_type = "Int32";
  d.kind = ACC_SKEL_MAP;  d.out_rank = 1;  d.get = "arrIn0_0[ix] * 2";
  OK(acc_skel_create(ctx, &d, &dbl));
  d.kind = ACC_SKEL_FOLD;  d.out_rank = 0;  d.get = "arrIn0_0[ix]";  d.combine = "acc_max(x, y)";  d.seed = "0";
  OK(acc_skel_create(ctx, &d, &mx));
  senv[0] = sig(0, "Int32");
  memset(&d, 0, sizeof d);
  d.flags = ACC_FLAG_GUARDED;
  d.kind = ACC_SKEL_MAP;  d.n_env = 1;  d.env = senv;  d.elt_type = "Word8";  d.out_rank = 0;  d.get = "(Word8)(arrIn0_0[0] < 5000)";
  OK(acc_skel_create(ctx, &d, &below));
  OK(acc_stream_create(ctx, &st));
  OK(acc_guard_create(ctx, &guard));
  buf[0] = upload(ctx, x, sizeof x);
  for (k = 1; k <= AHEAD; ++k) OK(acc_malloc(ctx, sizeof x, &buf[k]));
  OK(acc_malloc(ctx, 256, &dtop));
  dflag = dtop + 128;
  memset(&top, 0, sizeof top);   top.ncomp = 1;   top.ptr[0] = dtop;         /* rank 0 */
  memset(&flag, 0, sizeof flag); flag.ncomp = 1;  flag.ptr[0] = dflag;
  OK(acc_stream_set_guard(ctx, st, guard));
  OK(acc_guard_reset(guard, st));
  for (k = 0; k < AHEAD; ++k) {                  /* predicate; latch; body -- without looking at the device */
    a = vector_of(buf[k], N);
    b = vector_of(buf[k + 1], N);
    OK(acc_exec_fold(mx, &a, 1, &n, &top, st));
    OK(acc_exec_map(below, &top, &flag, st));
    OK(acc_guard_latch(guard, &flag, st));
    OK(acc_exec_map(dbl, &a, &b, st));
  }
  OK(acc_guard_read(guard, st, &alive, &count));
  CHECK(alive == 0 && count == steps && steps > 3 && steps < AHEAD, "the guard counts the iterations that were taken");
  OK(acc_memcpy_d2h(ctx, got, buf[count], sizeof got));
  for (i = 0, k = 0; i < N; ++i) k += got[i] != x[i] << steps;
  CHECK(k == 0, "the loop's value is what the last iteration taken produced");
  OK(acc_stream_set_guard(ctx, st, NULL));
  OK(acc_guard_destroy(guard));
  OK(acc_stream_destroy(ctx, st));
  OK(acc_skel_destroy(dbl));
  OK(acc_skel_destroy(mx));
  OK(acc_skel_destroy(below));
  for (k = 0; k <= AHEAD; ++k) acc_free(ctx, buf[k]);
  acc_free(ctx, dtop);
}

/* ---- the scratch the drivers pool can be had back ------------------------------------------------------------- */
static void scratch_pool(acc_context ctx)
{
  size_t held = 0, freed = 0;
  OK(acc_context_sync(ctx));
  OK(acc_context_scratch_bytes(ctx, &held));
  CHECK(held > 0, "the scans and folds above left scratch in the pool");
  OK(acc_context_trim(ctx, &freed));
  CHECK(freed == held, "all of it comes back when nothing is running");
  OK(acc_context_scratch_bytes(ctx, &held));
  CHECK(held == 0, "and the pool is empty");
}

/* ---- memory table: three arrays under a budget that holds two ---------------- */
static void memory_table(acc_context ctx)
{
  enum { N = 1 << 18 };                          /* 1 MiB each */
  static int32_t a[N], b[N], c[N], back[N];
  acc_memtable mt = NULL;
  acc_memtable_stats st;
  acc_devptr pa, pb, pc;
  int is_new = -1, i;
  for (i = 0; i < N; ++i) { a[i] = i; b[i] = -i; c[i] = 0; }
  OK(acc_memtable_create(ctx, 2u << 20, &mt));
  OK(acc_memtable_malloc(mt, 1, a, sizeof a, 1, &is_new));
  CHECK(is_new == 1, "first entry is new");
  OK(acc_memtable_malloc(mt, 1, a, sizeof a, 1, &is_new));
  CHECK(is_new == 0, "the same array again is not");
  OK(acc_memtable_malloc(mt, 2, b, sizeof b, 1, NULL));
  OK(acc_memtable_acquire(mt, 1, NULL, &pa));
  OK(acc_memtable_acquire(mt, 2, NULL, &pb));
  CHECK(acc_memtable_malloc(mt, 3, c, sizeof c, 0, NULL) == ACC_ERR_OOM, "everything resident is in use: out of memory");
  OK(acc_memtable_release(mt, 1, NULL));
  OK(acc_memtable_malloc(mt, 3, c, sizeof c, 0, NULL));     /* a leaves the device */
  OK(acc_memtable_acquire(mt, 3, NULL, &pc));
  OK(acc_memcpy_d2d(ctx, pc, pb, sizeof b));                /* c := b, on the device */
  OK(acc_memtable_release(mt, 2, NULL));
  OK(acc_memtable_release(mt, 3, NULL));
  OK(acc_memtable_acquire(mt, 1, NULL, &pa));                /* a comes back; b (clean) or c (written back) leaves */
  OK(acc_memcpy_d2h(ctx, back, pa, sizeof back));
  CHECK(memcmp(back, a, sizeof a) == 0, "an evicted input is uploaded again");
  OK(acc_memtable_release(mt, 1, NULL));
  OK(acc_memtable_acquire(mt, 3, NULL, &pc));
  OK(acc_memcpy_d2h(ctx, back, pc, sizeof back));
  CHECK(memcmp(back, b, sizeof b) == 0, "an array produced on the device survives eviction");
  OK(acc_memtable_release(mt, 3, NULL));
  OK(acc_memtable_get_stats(mt, &st));
  CHECK(st.evictions >= 2 && st.arrays == 3 && st.resident_bytes <= (2u << 20), "eviction statistics");
  CHECK(acc_memtable_acquire(mt, 99, NULL, &pa) == ACC_ERR_NOT_FOUND, "unknown key");
  OK(acc_memtable_destroy(mt));
}

/* ---- kernels compiled in the background, knobs per context, a stencil of rank 4 ------------------------------- */
static void background_compilation(acc_context ctx)
{
  enum { D = 6, N = D * D * D * D };
  static float v[N], got[N];
  static int32_t offsets[81 * 4];
  char fn[81 * 8];
  acc_skel_desc d;
  acc_skel_info info;
  acc_skel box = NULL, twice = NULL;
  acc_env_sig env[1];
  acc_array src, out;
  acc_devptr dsrc, dout;
  int ready = -1, i, k = 0, a, b, c, e, bad = 0;
  size_t at = 0;
  for (i = 0; i < N; ++i) v[i] = (float)(rnd() % 7);
  for (a = -1; a <= 1; ++a) for (b = -1; b <= 1; ++b) for (c = -1; c <= 1; ++c) for (e = -1; e <= 1; ++e) {
    offsets[4 * k] = a; offsets[4 * k + 1] = b; offsets[4 * k + 2] = c; offsets[4 * k + 3] = e;
    at += (size_t)sprintf(fn + at, k ? " + t%d" : "t%d", k);
    ++k;
  }
  CHECK(acc_compile_threads() >= 1, "the pool has room for a worker");
  OK(acc_context_set_tuning(ctx, "map.block=128"));            /* instances created from now on take the knob ... */
  memset(&d, 0, sizeof d);
  env[0] = sig(1, "float");
  d.kind = ACC_SKEL_MAP;  d.n_env = 1;  d.env = env;  d.elt_type = "float";  d.out_rank = 1;  d.get = "arrIn0_0[ix] * 2.0f";
  OK(acc_skel_create_async(ctx, &d, &twice));                   /* both handles at once: the kernels compile side by side */
  OK(acc_context_set_tuning(ctx, NULL));                        /* ... and the process's table is back for the next one */
  memset(&d, 0, sizeof d);
  d.kind = ACC_SKEL_STENCIL;  d.elt_type = "float";  d.out_rank = 4;  d.boundary = ACC_BOUNDARY_WRAP;
  d.n_taps = 81;  d.tap_offsets = offsets;  d.stencil_fn = fn;
  OK(acc_skel_create_async(ctx, &d, &box));
  OK(acc_skel_poll(box, &ready));
  CHECK(ready == 0 || ready == 1, "poll says whether the compilation has ended");
  OK(acc_skel_prefetch(twice, 1));                              /* the unaligned variant, ahead of any launch that wants it */
  OK(acc_skel_wait(twice));
  OK(acc_skel_get_info(twice, &info));
  CHECK(info.block == 128, "the instance took the knob its context had when it was created");
  dsrc = upload(ctx, v, sizeof v);
  OK(acc_malloc(ctx, sizeof v, &dout));
  memset(&src, 0, sizeof src);  src.rank = 4;  src.ncomp = 1;  src.ptr[0] = dsrc;
  for (i = 0; i < 4; ++i) src.shape[i] = D;
  out = src;  out.ptr[0] = dout;
  OK(acc_exec_stencil(box, NULL, &src, &out, NULL));            /* the first use waits for the kernel */
  OK(acc_memcpy_d2h(ctx, got, dout, sizeof got));
  for (a = 0; a < D; ++a) for (b = 0; b < D; ++b) for (c = 0; c < D; ++c) for (e = 0; e < D; ++e) {
    float sum = 0.0f;                                           /* small integers: exact in any order */
    for (k = 0; k < 81; ++k)
      sum += v[((((a + offsets[4 * k] + D) % D) * D + (b + offsets[4 * k + 1] + D) % D) * D + (c + offsets[4 * k + 2] + D) % D) * D +
               (e + offsets[4 * k + 3] + D) % D];
    bad += got[((a * D + b) * D + c) * D + e] != sum;
  }
  CHECK(bad == 0, "a 3 x 3 x 3 x 3 stencil that wraps round");
  OK(acc_skel_destroy(box));
  OK(acc_skel_destroy(twice));
  acc_free(ctx, dsrc);
  acc_free(ctx, dout);
}

int main(int argc, char **argv)
{
  acc_context ctx = NULL;
  acc_device_props props;
  int count = 0;
  printf("libacchip %s\n", acc_version());
  compile_without_a_device();
  if (argc > 1 && strcmp(argv[1], "--no-gpu") == 0) {
    printf(failures ? "%d check(s) FAILED\n" : "all checks passed (no device used)\n", failures);
    return failures ? 1 : 0;
  }
  if (acc_init() != ACC_OK || acc_device_count(&count) != ACC_OK || count < 1) {
    printf("no device: %s\n", acc_last_error());
    return 2;
  }
  if (acc_device_get_props(0, &props) != ACC_OK || acc_context_create(0, &ctx) != ACC_OK) {
    printf("cannot open device 0: %s\n", acc_last_error());
    return 2;
  }
  printf("device 0: %s, %d compute units\n", props.arch, props.compute_units);
  fflush(stdout);
  dot_product(ctx);
  prefix_sums(ctx);
  histogram(ctx);
  gaussian(ctx);
  smvm(ctx);
  segmented_rows(ctx);
  guarded_loop(ctx);
  scratch_pool(ctx);
  memory_table(ctx);
  background_compilation(ctx);
  CHECK(acc_context_sync(ctx) == ACC_OK, "device still healthy");
  acc_context_destroy(ctx);
  CHECK(acc_compile_drain() == ACC_OK, "nothing is compiling when the process ends");
  printf(failures ? "%d check(s) FAILED\n" : "all checks passed\n", failures);
  return failures ? 1 : 0;
}
