"""The embedded array language (accelerate_hip) against numpy: the benchmark programs written the way a user of
the reference writes them (accelerate-examples' dotp, scan, histogram via permute, stencil, smvm), plus the
delayed-array combinators.  Integer results are exact; floating-point sums carry the tolerance stated per test."""
import numpy as np
import pytest

import pyref

pytestmark = pytest.mark.gpu


@pytest.fixture(scope="module")
def acc():
    import accelerate_hip
    return accelerate_hip


def add(x, y):
    return x + y


def test_dotp_is_one_kernel(acc):
    rng = np.random.default_rng(1)
    x, y = rng.standard_normal(1000003).astype(np.float32), rng.standard_normal(1000003).astype(np.float32)
    cx = acc.Context.default()
    before = len(cx.skeletons)
    r = acc.run(acc.fold(add, 0.0, acc.zipWith(lambda a, b: a * b, acc.use(x), acc.use(y))))
    assert len(cx.skeletons) == before + 1                      # zipWith fused into the fold
    assert r.shape == () and abs(float(r) - float(np.dot(x.astype(np.float64), y.astype(np.float64)))) < 1e-3 * np.sqrt(x.size)
    xi, yi = rng.integers(-1000, 1000, 77777).astype(np.int32), rng.integers(-1000, 1000, 77777).astype(np.int32)
    r = acc.run(acc.fold(add, 0, acc.zipWith(lambda a, b: a * b, acc.use(xi), acc.use(yi))))
    assert int(r) == pyref.wrap(int(np.dot(xi.astype(np.int64), yi.astype(np.int64))), 32, True)


def test_saxpy_and_run1_reuses_kernels(acc):
    rng = np.random.default_rng(2)
    cx = acc.Context.default()
    saxpy = acc.run1(lambda xs, ys: acc.zipWith(lambda x, y: acc.constant(1.5, "float") * x + y, xs, ys))
    x, y = rng.standard_normal(4099).astype(np.float32), rng.standard_normal(4099).astype(np.float32)
    assert np.array_equal(saxpy(x, y), np.float32(1.5) * x + y)
    n = len(cx.skeletons)
    x2, y2 = rng.standard_normal(513).astype(np.float32), rng.standard_normal(513).astype(np.float32)
    assert np.array_equal(saxpy(x2, y2), np.float32(1.5) * x2 + y2)
    assert len(cx.skeletons) == n


def test_six_scans(acc):
    rng = np.random.default_rng(3)
    x = rng.integers(-50, 50, 100001).astype(np.int32)
    xs = acc.use(x)
    c = np.cumsum(x, dtype=np.int32)
    rc = np.cumsum(x[::-1], dtype=np.int32)[::-1]
    assert np.array_equal(acc.run(acc.scanl(add, 0, xs)), np.concatenate([[0], c]).astype(np.int32))
    assert np.array_equal(acc.run(acc.scanl1(add, xs)), c)
    body, total = acc.run(acc.scanl_(add, 0, xs))
    assert np.array_equal(body, np.concatenate([[0], c[:-1]]).astype(np.int32)) and int(total) == int(c[-1])
    assert np.array_equal(acc.run(acc.scanr(add, 0, xs)), np.concatenate([rc, [0]]).astype(np.int32))
    assert np.array_equal(acc.run(acc.scanr1(add, xs)), rc)
    body, total = acc.run(acc.scanr_(add, 0, xs))
    assert np.array_equal(body, np.concatenate([rc[1:], [0]]).astype(np.int32)) and int(total) == int(rc[0])
    # a scan of a delayed array with a non-commutative-looking operator: running maximum of squares
    m = acc.run(acc.scanl1(acc.max_, acc.map(lambda v: v * v, xs)))
    assert np.array_equal(m, np.maximum.accumulate(x * x))


def test_histogram_via_permute_reads_keys_inside_the_permutation(acc):
    rng = np.random.default_rng(4)
    bins, n = 256, 300007
    keys = rng.integers(0, bins, n).astype(np.int32)
    ks = acc.use(keys)
    zeros = acc.generate((bins,), lambda i: acc.constant(0, "Int32"))
    ones = acc.generate((n,), lambda i: acc.constant(1, "Int32"))
    h = acc.run(acc.permute(add, zeros, lambda i: (ks[i],), ones))
    assert np.array_equal(h, np.bincount(keys, minlength=bins).astype(np.int32))
    # weighted, with every odd key dropped
    w = rng.integers(1, 9, n).astype(np.int32)
    h = acc.run(acc.permute(add, zeros, lambda i: acc.index_if((ks[i] & 1).eq(0), (ks[i],)), acc.use(w)))
    even = (keys & 1) == 0
    assert np.array_equal(h, np.bincount(keys[even], weights=w[even], minlength=bins).astype(np.int32))
    # nothing lands anywhere
    h = acc.run(acc.permute(add, acc.use(np.arange(bins, dtype=np.int32)), lambda i: acc.ignore, acc.use(w)))
    assert np.array_equal(h, np.arange(bins, dtype=np.int32))
    # counting into 65536 targets: the constant source is what lets the driver keep 16-bit counts in LDS
    keys = np.minimum(rng.zipf(1.3, 1 << 20) - 1, 65535).astype(np.int32)
    ks = acc.use(keys)
    h = acc.run(acc.permute(add, acc.fill((65536,), 0, "Int32"), lambda i: (ks[i],), acc.fill((keys.size,), 1, "Int32")))
    assert np.array_equal(h, np.bincount(keys, minlength=65536).astype(np.int32))
    h = acc.run(acc.permute(add, acc.fill((65536,), 5, "Int64"), lambda i: (ks[i],), acc.fill((keys.size,), 2, "Int64")))
    assert np.array_equal(h, 5 + 2 * np.bincount(keys, minlength=65536).astype(np.int64))


def test_permute_with_a_generic_combination(acc):
    rng = np.random.default_rng(5)
    n, m = 50021, 97
    t = rng.integers(0, m, n).astype(np.int32)
    v = rng.integers(-10 ** 6, 10 ** 6, n).astype(np.int64)
    ts = acc.use(t)
    first = np.full(m, -2 ** 62, dtype=np.int64)
    out = acc.run(acc.permute(lambda x, y: acc.cond(x > y, x, y), acc.use(first), lambda i: (ts[i],), acc.use(v)))
    ref = first.copy()
    np.maximum.at(ref, t, v)
    assert np.array_equal(out, ref)


def test_stencils(acc):
    rng = np.random.default_rng(6)
    img = rng.standard_normal((301, 517)).astype(np.float32)
    pat = [(dy, dx) for dy in (-1, 0, 1) for dx in (-1, 0, 1)]
    wts = [1, 2, 1, 2, 4, 2, 1, 2, 1]

    def gauss(*t):
        s = t[0] * acc.constant(wts[0], "float")
        for k in range(1, 9):
            s = s + t[k] * acc.constant(wts[k], "float")
        return s / acc.constant(16, "float")
    for mode in ("clamp", "mirror", "wrap"):
        out = acc.run(acc.stencil(pat, gauss, mode, acc.use(img)))
        taps = pyref.tap_arrays(img, pat, mode, 0, img.shape)
        ref = taps[0] * np.float32(wts[0])
        for k in range(1, 9):
            ref = ref + taps[k] * np.float32(wts[k])
        assert np.array_equal(out, ref / np.float32(16)), mode
    # 1-D second difference of a delayed array (forced to a manifest array first), constant boundary
    x = rng.integers(-100, 100, 10007).astype(np.int32)
    out = acc.run(acc.stencil([(-1,), (0,), (1,)], lambda a, b, c: a - 2 * b + c, "constant",
                              acc.map(lambda v: v + 1, acc.use(x)), constant_value=7))
    p = np.concatenate([[7], x + 1, [7]]).astype(np.int32)
    assert np.array_equal(out, p[:-2] - 2 * p[1:-1] + p[2:])
    # stencil2: difference of a horizontal gradient of one image and a vertical gradient of another
    img2 = rng.standard_normal((301, 517)).astype(np.float32)
    out = acc.run(acc.stencil2([(0, -1), (0, 1)], [(-1, 0), (1, 0)], lambda t, u: (t[1] - t[0]) - (u[1] - u[0]),
                               "clamp", acc.use(img), "wrap", acc.use(img2)))
    t = pyref.tap_arrays(img, [(0, -1), (0, 1)], "clamp", 0, img.shape)
    u = pyref.tap_arrays(img2, [(-1, 0), (1, 0)], "wrap", 0, img.shape)
    assert np.array_equal(out, (t[1] - t[0]) - (u[1] - u[0]))


def test_smvm_by_foldseg(acc):
    rng = np.random.default_rng(7)
    rows, ncols = 4001, 3000
    lens = rng.integers(0, 40, rows).astype(np.int32)
    nnz = int(lens.sum())
    cols = rng.integers(0, ncols, nnz).astype(np.int32)
    vals = rng.integers(-9, 10, nnz).astype(np.float32)          # small integers: float sums are exact
    vec = rng.integers(-9, 10, ncols).astype(np.float32)
    v = acc.use(vec)
    products = acc.zipWith(lambda c, a: a * v[c], acc.use(cols), acc.use(vals))
    y = acc.run(acc.foldSeg(add, 0.0, products, acc.use(lens)))
    offs = np.concatenate([[0], np.cumsum(lens)])
    ref = np.array([np.sum(vals[offs[r]:offs[r + 1]] * vec[cols[offs[r]:offs[r + 1]]], dtype=np.float32) for r in range(rows)],
                   dtype=np.float32)
    assert np.array_equal(y, ref)


def test_foldseg_of_a_matrix_and_fold1seg(acc):
    """foldSeg over the rows of a matrix (the same segments in every row, Reduction.hs:473-474) fused with its
    producer, and fold1Seg"""
    rng = np.random.default_rng(17)
    m = rng.integers(-50, 50, (301, 64)).astype(np.int32)
    lens = np.array([5, 0, 20, 1, 30], np.int32)              # 56 of the 64 columns
    offs = np.concatenate([[0], np.cumsum(lens)])
    got = acc.run(acc.foldSeg(add, 10, acc.map(lambda v: v * 2, acc.use(m)), acc.use(lens)))
    ref = np.stack([(2 * m[:, offs[k]:offs[k + 1]]).sum(axis=1) + 10 for k in range(5)], axis=1).astype(np.int32)
    assert got.shape == (301, 5) and np.array_equal(got, ref)
    lens1 = np.array([5, 2, 20, 1, 30], np.int32)
    offs1 = np.concatenate([[0], np.cumsum(lens1)])
    got = acc.run(acc.fold1Seg(add, acc.use(m), acc.use(lens1)))
    ref = np.stack([m[:, offs1[k]:offs1[k + 1]].sum(axis=1) for k in range(5)], axis=1).astype(np.int32)
    assert np.array_equal(got, ref)
    v = rng.integers(-50, 50, 1000).astype(np.int32)
    lv = np.array([100, 0, 900], np.int32)
    assert np.array_equal(acc.run(acc.fold1Seg(add, acc.use(v), acc.use(np.array([100, 900], np.int32)))),
                          np.array([v[:100].sum(), v[100:].sum()], np.int32))
    assert np.array_equal(acc.run(acc.foldSeg(add, 0, acc.use(v), acc.use(lv))), np.array([v[:100].sum(), 0, v[100:].sum()], np.int32))


def test_index_transformations(acc):
    rng = np.random.default_rng(8)
    m = rng.integers(0, 1000, (37, 101)).astype(np.int32)
    assert np.array_equal(acc.run(acc.transpose(acc.use(m))), m.T)
    # a transpose is produced in square tiles, and so is what is fused on top of it
    big = rng.integers(0, 1000, (300, 517)).astype(np.int32)
    other = rng.integers(0, 1000, (517, 300)).astype(np.int32)
    tr = acc.transpose(acc.use(big))
    assert tr.across and acc.map(lambda v: v + 1, tr).across
    assert np.array_equal(acc.run(acc.map(lambda v: v * 2 + 1, tr)), big.T * 2 + 1)
    assert np.array_equal(acc.run(acc.zipWith(lambda a, b: a - b, acc.use(other), tr)), other - big.T)
    x = rng.integers(0, 1000, 1001).astype(np.int64)
    assert np.array_equal(acc.run(acc.reverse(acc.use(x))), x[::-1])
    # zipWith over different extents takes the intersection
    a, b = rng.integers(0, 9, (5, 9)).astype(np.int32), rng.integers(0, 9, (7, 4)).astype(np.int32)
    assert np.array_equal(acc.run(acc.zipWith(add, acc.use(a), acc.use(b))), a[:5, :4] + b[:5, :4])
    # generate over a rank-3 index, fold over the innermost dimension of it
    g = acc.generate((3, 5, 7), lambda z, y, x_: z * 100 + y * 10 + x_)
    zz, yy, xx = np.meshgrid(np.arange(3), np.arange(5), np.arange(7), indexing="ij")
    ref = (zz * 100 + yy * 10 + xx).astype(np.int64)
    assert np.array_equal(acc.run(g), ref)
    assert np.array_equal(acc.run(acc.fold(add, 0, g)), ref.sum(axis=2))
    assert np.array_equal(acc.run(acc.fold1(acc.min_, g)), ref.min(axis=2))


def test_integer_division_follows_haskell(acc):
    a = np.array([7, -7, 7, -7, 0, 5, -5, 2 ** 31 - 1, -2 ** 31], dtype=np.int32)
    b = np.array([2, 2, -2, -2, 3, 5, 5, -1, 1], dtype=np.int32)
    xs, ys = acc.use(a), acc.use(b)
    assert np.array_equal(acc.run(acc.zipWith(lambda x, y: x // y, xs, ys)), a // b)
    assert np.array_equal(acc.run(acc.zipWith(lambda x, y: x % y, xs, ys)), a % b)
    assert np.array_equal(acc.run(acc.zipWith(acc.quot, xs, ys)), np.array([pyref.wrap(pyref.quot(int(p), int(q)), 32, True) for p, q in zip(a, b)], dtype=np.int32))
    assert np.array_equal(acc.run(acc.zipWith(acc.rem, xs, ys)), np.array([pyref.wrap(pyref.rem(int(p), int(q)), 32, True) for p, q in zip(a, b)], dtype=np.int32))


def test_tuples_argmax_and_unzip(acc):
    rng = np.random.default_rng(9)
    n = 123457
    x = rng.permutation(n).astype(np.float32)
    idx = acc.generate((n,), lambda i: acc.fromIntegral(i, "Int32"))
    pairs = acc.zip_(acc.use(x), idx)
    best = acc.fold(lambda p, q: acc.cond(acc.fst(p) >= acc.fst(q), p, q), (-np.inf, -1), pairs)
    val, where = acc.run(best)
    assert float(val) == float(x.max()) and int(where) == int(np.argmax(x))
    # a manifest array of pairs read back, swapped
    ys = rng.integers(0, 100, 1000).astype(np.int16)
    zs = rng.standard_normal(1000)
    sw = acc.map(lambda p: acc.lift(acc.snd(p), acc.fst(p)), acc.use((ys, zs)))
    a, b = acc.run(sw)
    assert np.array_equal(a, zs) and np.array_equal(b, ys)
    f, s = acc.unzip(sw)
    assert np.array_equal(acc.run(s), ys)


def test_type_errors_are_reported_before_anything_is_compiled(acc):
    xs = acc.use(np.zeros(4, dtype=np.int32))
    with pytest.raises(TypeError):
        acc.zipWith(add, xs, acc.use(np.zeros(4, dtype=np.float32)))
    with pytest.raises(TypeError):
        acc.scanl(add, 0, acc.use(np.zeros((2, 2), dtype=np.int32)))
    with pytest.raises(TypeError):
        acc.map(lambda v: 1 if v > 0 else 0, xs)


def test_scalar_while_mandelbrot_and_collatz(acc):
    # Mandelbrot escape counts (accelerate-examples' mandelbrot): state (zr, zi, i) iterated per element
    h, w, limit = 96, 128, 64
    f32 = lambda v: acc.constant(v, "float")

    def pixel(y, x):
        cr = acc.fromIntegral(x, "float") * f32(3.0 / w) - f32(2.25)
        ci = acc.fromIntegral(y, "float") * f32(2.5 / h) - f32(1.25)

        def inside(s):
            zr, zi, i = s.comps
            return (zr * zr + zi * zi <= f32(4.0)).land(i < limit)

        def step(s):
            zr, zi, i = s.comps
            return (zr * zr - zi * zi + cr, f32(2.0) * zr * zi + ci, i + 1)
        return acc.while_(inside, step, acc.lift(f32(0.0), f32(0.0), acc.constant(0, "Int32"))).comps[2]
    counts = acc.run(acc.generate((h, w), pixel))
    yy, xx = np.meshgrid(np.arange(h), np.arange(w), indexing="ij")
    cr = xx.astype(np.float32) * np.float32(3.0 / w) - np.float32(2.25)
    ci = yy.astype(np.float32) * np.float32(2.5 / h) - np.float32(1.25)
    zr, zi, it = np.zeros_like(cr), np.zeros_like(cr), np.zeros((h, w), np.int32)
    for _ in range(limit):
        live = (zr * zr + zi * zi <= np.float32(4.0)) & (it < limit)
        nzr = zr * zr - zi * zi + cr
        nzi = np.float32(2.0) * zr * zi + ci
        zr, zi, it = np.where(live, nzr, zr), np.where(live, nzi, zi), np.where(live, it + 1, it)
    assert np.array_equal(counts, it) and 0 < it.min() < it.max() == limit
    # Collatz steps: a scalar loop state, the loop inside a fold's producer
    n = np.arange(1, 5001, dtype=np.int64)

    def steps(v):
        s = acc.while_(lambda t: t.comps[0] > 1,
                       lambda t: (acc.cond((t.comps[0] & 1).eq(0), t.comps[0] // 2, 3 * t.comps[0] + 1), t.comps[1] + 1),
                       acc.lift(v, acc.constant(0, "Int64")))
        return s.comps[1]
    ref = []
    for v in n:
        c = 0
        while v > 1:
            v, c = (v // 2 if v % 2 == 0 else 3 * v + 1), c + 1
        ref.append(c)
    assert np.array_equal(acc.run(acc.map(steps, acc.use(n))), np.array(ref, dtype=np.int64))
    assert int(acc.run(acc.fold1(acc.max_, acc.map(steps, acc.use(n))))) == max(ref)
    # a loop whose state is one scalar: integer square root by counting
    r = acc.run(acc.map(lambda v: acc.while_(lambda k: (k + 1) * (k + 1) <= v, lambda k: k + 1, acc.constant(0, "Int64")), acc.use(n)))
    assert np.array_equal(r, np.floor(np.sqrt(n)).astype(np.int64))


def test_a_working_set_larger_than_the_memory_budget(acc):
    """twelve 16 MiB arrays alive under a 64 MiB table: results leave the device for their host side and come back"""
    cx = acc.Context(0, budget_bytes=64 << 20)
    n = 4 << 20
    rng = np.random.default_rng(10)
    x = rng.integers(-100, 100, n).astype(np.int32)
    xs = acc.use(x, cx)
    assert acc.use(x, cx).manifest.key == xs.manifest.key                         # one entry, one upload
    stages = [xs]
    for k in range(1, 12):
        prev = stages[-1]
        stages.append(acc.compute(acc.map(lambda v, k=k: v * 3 + k, prev), cx))   # each stage is a manifest array that stays alive
    st = cx.table.stats()
    assert st["arrays"] == 12 and st["resident_bytes"] <= 64 << 20 and st["evictions"] >= 8 and st["writebacks"] >= 7
    assert st["uploads"] >= 1
    ref = x.copy()
    for k in range(1, 12):
        ref = ref * 3 + k
        assert np.array_equal(acc.run(stages[k], cx), ref), k                     # evicted stages are re-uploaded to be read
    total = acc.run(acc.fold(add, 0, acc.zipWith(add, stages[1], stages[11]), context=cx), cx)
    assert int(total) == pyref.wrap(int((x.astype(np.int64) * 3 + 1).sum() + ref.astype(np.int64).sum()), 32, True)
    del stages, xs
    import gc
    gc.collect()
    assert cx.table.stats()["arrays"] <= 2                                         # results die with their last reference


def test_independent_subcomputations_run_on_their_own_streams_and_meet_by_events(acc):
    cx = acc.Context(0)
    rng = np.random.default_rng(11)
    n = 1 << 22
    x, y = rng.integers(-9, 9, n).astype(np.int64), rng.integers(-9, 9, n).astype(np.int64)
    xs, ys = acc.use(x, cx), acc.use(y, cx)
    sx = acc.compute(acc.scanl1(add, xs, context=cx), cx)      # two independent scans (launched now, not when asked for) ...
    sy = acc.compute(acc.scanr1(add, ys, context=cx), cx)
    assert sx.manifest.stream is not sy.manifest.stream        # ... on two streams
    both = acc.compute(acc.zipWith(lambda a, b: a - b, sx, sy), cx)     # joins them: runs behind sx, waits for sy's event
    assert both.manifest.stream is sx.manifest.stream
    chain = both
    for k in range(5):                                          # a dependent chain stays on one stream
        chain = acc.compute(acc.map(lambda v, k=k: v + k, chain), cx)
        assert chain.manifest.stream is sx.manifest.stream
    ref = np.cumsum(x) - np.cumsum(y[::-1])[::-1]
    assert np.array_equal(acc.run(chain, cx), ref + 10)
    assert np.array_equal(acc.run(sy, cx), np.cumsum(y[::-1])[::-1])
    # the same input read from two streams right after its upload was queued on the first
    z = rng.integers(-9, 9, 1 << 24).astype(np.int32)
    zs = acc.use(z, cx)
    f1 = acc.compute(acc.fold(add, 0, zs, context=cx), cx)
    f2 = acc.compute(acc.fold(acc.max_, -100, acc.map(lambda v: v * 2, zs), context=cx), cx)
    assert f1.manifest.stream is not f2.manifest.stream and cx.table.stats()["uploads"] == 3
    assert int(acc.run(f1, cx)) == int(z.sum()) and int(acc.run(f2, cx)) == int(z.max() * 2)


def test_awhile_iterates_on_the_device_until_the_flag_clears(acc):
    cx = acc.Context(0)
    rng = np.random.default_rng(12)
    x = rng.integers(1, 50, 100003).astype(np.int64)
    # double every element until the largest passes a million
    big = lambda xs: acc.map(lambda m: m < 1000000, acc.fold(acc.max_, 0, xs, context=cx))
    out = acc.run(acc.awhile(big, lambda xs: acc.map(lambda v: v * 2, xs), acc.use(x, cx), context=cx), cx)
    ref = x.copy()
    while ref.max() < 1000000:
        ref = ref * 2
    assert np.array_equal(out, ref)
    # a pair of arrays as the state: Jacobi sweeps of a 1-D heat rod until the update is small, with a sweep counter
    u0 = np.zeros(4097, np.float64)
    u0[0], u0[-1] = 1.0, 3.0

    def sweep(u, k):
        nu = acc.stencil([(-1,), (0,), (1,)], lambda a, b, c: (a + c) / 2.0, "clamp", u, context=cx)
        n = u.shape[0]
        fixed = acc.zipWith(lambda new, old: new, nu, u)        # interior from the sweep ...
        ends = acc.generate((n,), lambda i: acc.cond(i.eq(0).lor(i.eq(n - 1)), acc.constant(1, "Word8"), acc.constant(0, "Word8")))
        fixed = acc.zipWith(lambda e, p: acc.cond(e, acc.snd(p), acc.fst(p)), ends, acc.zip_(nu, u))   # ... ends kept
        return fixed, acc.map(lambda c: c + 1, k)

    def moving(u, k):
        nu, _ = sweep(u, k)
        delta = acc.fold(acc.max_, 0.0, acc.zipWith(lambda a, b: acc.abs_(a - b), nu, u), context=cx)
        return acc.zipWith(lambda d, c: (d > 1e-3).land(c < 500), delta, k)
    u, k = acc.awhile(moving, sweep, (acc.use(u0, cx), acc.unit(0, "Int32", cx)), context=cx)
    ref, steps = u0.copy(), 0
    while True:
        nxt = ref.copy()
        nxt[1:-1] = (ref[:-2] + ref[2:]) / 2.0
        if not (np.abs(nxt - ref).max() > 1e-3 and steps < 500):
            break
        ref, steps = nxt, steps + 1
    assert int(acc.run(k, cx)) == steps and steps > 3
    assert np.array_equal(acc.run(u, cx), ref)
    with pytest.raises(TypeError):
        acc.awhile(lambda xs: xs, lambda xs: xs, acc.use(x, cx), context=cx)


def test_awhile_enqueued_ahead_agrees_with_one_iteration_at_a_time(acc):
    """the same loops with the flag read back every iteration (ahead=1), every 3 and every 8: identical values and
    iteration counts; the host reads the guard once per batch; bodies with every kind of skeleton in them; a body that
    needs the host falls back; limits; loops that never run"""
    import acchip as A
    cx = acc.Context(0)
    rng = np.random.default_rng(31)
    x = rng.integers(1, 50, 50021).astype(np.int64)
    reads = []
    real_read = A.Guard.read
    A.Guard.read = lambda self, stream=None: (reads.append(1), real_read(self, stream))[1]
    try:
        big = lambda xs, k: acc.map(lambda m: m < 3000000, acc.fold(acc.max_, 0, xs, context=cx))
        step = lambda xs, k: (acc.map(lambda v: v * 2, xs), acc.map(lambda c: c + 1, k))
        ref, steps = x.copy(), 0
        while ref.max() < 3000000:
            ref, steps = ref * 2, steps + 1
        assert steps > 10
        for ahead in (1, 3, 8, 64):
            del reads[:]
            out, k = acc.awhile(big, step, (acc.use(x, cx), acc.unit(0, "Int32", cx)), context=cx, ahead=ahead)
            assert np.array_equal(acc.run(out, cx), ref) and int(acc.run(k, cx)) == steps, ahead
            assert len(reads) == (0 if ahead == 1 else steps // ahead + 1), (ahead, len(reads))
        # a limit below and above the natural end; a loop that never runs
        for limit in (0, 1, 5, steps, steps + 7):
            out, k = acc.awhile(big, step, (acc.use(x, cx), acc.unit(0, "Int32", cx)), context=cx, limit=limit, ahead=4)
            took = min(limit, steps)
            assert int(acc.run(k, cx)) == took and np.array_equal(acc.run(out, cx), x * 2 ** took), limit
        never = lambda xs, k: acc.map(lambda m: m < 0, acc.fold(acc.max_, 0, xs, context=cx))
        out, k = acc.awhile(never, step, (acc.use(x, cx), acc.unit(0, "Int32", cx)), context=cx)
        assert int(acc.run(k, cx)) == 0 and np.array_equal(acc.run(out, cx), x)

        # scan, segmented fold, permute (its copy of the defaults included) and a stencil inside the body, an Int32 flag
        y = rng.integers(0, 7, 4096).astype(np.int32)
        lens = np.full(64, 64, np.int32)

        def body(v, k):
            sums = acc.foldSeg(add, 0, v, acc.use(lens, cx), context=cx)                       # 64 block sums
            hist = acc.permute(add, acc.fill((8,), 0, "Int32"), lambda i: (v[i] & 7,), acc.map(lambda t: t * 0 + 1, v), context=cx)
            run_ = acc.scanl1(add, v, context=cx)
            sm = acc.stencil([(-1,), (0,), (1,)], lambda a, b, c: acc.max_(a, acc.max_(b, c)), "clamp", v, context=cx)
            nv = acc.zipWith(lambda a, b: (a + b) & 1023, sm, run_)
            nv = acc.zipWith(lambda a, i: a + hist[i & 7] + sums[i & 63], nv, acc.generate((4096,), lambda i: acc.fromIntegral(i, "Int32")))
            return acc.map(lambda t: t & 4095, nv), acc.map(lambda c: c + 1, k)

        def ref_body(v):
            sums = v.reshape(64, 64).sum(axis=1).astype(np.int32)
            hist = np.bincount(v & 7, minlength=8).astype(np.int32)
            run_ = np.cumsum(v, dtype=np.int32)
            p = np.concatenate([v[:1], v, v[-1:]])
            sm = np.maximum(p[:-2], np.maximum(p[1:-1], p[2:]))
            nv = (sm + run_) & 1023
            i = np.arange(4096)
            return ((nv + hist[i & 7] + sums[i & 63]) & 4095).astype(np.int32)
        cont = lambda v, k: acc.map(lambda m: acc.cond((m % 5).ne(0), acc.constant(1, "Int32"), acc.constant(0, "Int32")),
                                    acc.fold(add, 0, v, context=cx))
        ry, rk = y.copy(), 0
        while int(ry.sum(dtype=np.int32)) % 5 != 0 and rk < 40:
            ry, rk = ref_body(ry), rk + 1
        for ahead in (1, 4):
            out, k = acc.awhile(cont, body, (acc.use(y, cx), acc.unit(0, "Int32", cx)), context=cx, limit=40, ahead=ahead)
            assert int(acc.run(k, cx)) == rk and np.array_equal(acc.run(out, cx), ry), ahead
        assert rk >= 1

        # a body that needs a value on the host (filter_ reads the count back): the loop goes on stepwise, same result
        z = rng.integers(0, 1000, 3001).astype(np.int32)

        def shrink(v):
            kept, _ = acc.filter_(lambda t: (t % 7).ne(0), v, context=cx)
            return acc.map(lambda t: t + 1, kept)
        many = lambda v: acc.map(lambda m: m > 3, acc.fold(acc.max_, 0, acc.map(lambda t: t % 7, v), context=cx))
        del reads[:]
        out = acc.run(acc.awhile(many, shrink, acc.use(z, cx), context=cx, limit=6), cx)
        rz, it = z.copy(), 0
        while it < 6 and (rz % 7).max() > 3:
            rz, it = rz[rz % 7 != 0] + 1, it + 1
        assert np.array_equal(out, rz) and it >= 2

        # a loop inside a loop: the inner one is enqueued ahead, the outer one steps
        def outer_body(v, k):
            inner = acc.awhile(lambda w: acc.map(lambda m: m < 100000, acc.fold(acc.max_, 0, w, context=cx)),
                               lambda w: acc.map(lambda t: t * 3, w), v, context=cx)
            return acc.map(lambda t: t % 1000 + 1, inner), acc.map(lambda c: c + 1, k)
        out, k = acc.awhile(lambda v, k: acc.map(lambda c: c < 3, k), outer_body, (acc.use(x, cx), acc.unit(0, "Int32", cx)), context=cx)
        r = x.copy()
        for _ in range(3):
            while r.max() < 100000:
                r = r * 3
            r = r % 1000 + 1
        assert int(acc.run(k, cx)) == 3 and np.array_equal(acc.run(out, cx), r)
    finally:
        A.Guard.read = real_read
        acc.destroy(cx)


def test_library_functions_built_from_the_primitives(acc):
    cx = acc.Context(0)
    rng = np.random.default_rng(13)
    x = rng.integers(-1000, 1000, 200003).astype(np.int32)
    xs = acc.use(x, cx)
    # filter: scan of the flags, then a permute into the places it gives
    kept, count = acc.filter_(lambda v: (v % 3).eq(0), xs, context=cx)
    assert int(acc.run(count, cx)) == int((x % 3 == 0).sum())
    assert np.array_equal(acc.run(kept, cx), x[x % 3 == 0])
    none, count = acc.filter_(lambda v: v > 5000, xs, context=cx)
    assert none.shape == (0,) and int(acc.run(count, cx)) == 0
    # whole-array reductions of a matrix
    m = rng.integers(-50, 50, (301, 77)).astype(np.int64)
    ms = acc.use(m, cx)
    assert int(acc.run(acc.sum_(ms, cx), cx)) == int(m.sum())
    assert int(acc.run(acc.maximum(ms, cx), cx)) == int(m.max()) and int(acc.run(acc.minimum(ms, cx), cx)) == int(m.min())
    assert int(acc.run(acc.all_(lambda v: v < 50, ms, cx), cx)) == 1 and int(acc.run(acc.any_(lambda v: v > 49, ms, cx), cx)) == 0
    f = rng.integers(1, 3, 40).astype(np.float64)
    assert float(acc.run(acc.product(acc.use(f, cx), cx), cx)) == float(np.prod(f))
    # index-space helpers
    assert np.array_equal(acc.run(acc.take(10, xs), cx), x[:10]) and np.array_equal(acc.run(acc.drop(199990, xs), cx), x[199990:])
    assert np.array_equal(acc.run(acc.init(xs), cx), x[:-1]) and np.array_equal(acc.run(acc.tail(xs), cx), x[1:])
    assert np.array_equal(acc.run(acc.enumFromN((3, 4), 5, "Int32"), cx), np.arange(5, 17, dtype=np.int32).reshape(3, 4))
    assert np.array_equal(acc.run(acc.fill((2, 3), 7, "Int16"), cx), np.full((2, 3), 7, np.int16))
    idx = rng.permutation(x.size).astype(np.int32)
    ids = acc.use(idx, cx)
    assert np.array_equal(acc.run(acc.gather(ids, xs), cx), x[idx])
    sc = acc.run(acc.scatter(ids, acc.fill((x.size,), 0, "Int32"), xs, context=cx), cx)       # a permutation: no collisions
    ref = np.zeros_like(x)
    ref[idx] = x
    assert np.array_equal(sc, ref)


def test_stencil_producing_pairs(acc):
    cx = acc.Context(0)
    rng = np.random.default_rng(14)
    img = rng.integers(-100, 100, (70, 333)).astype(np.float32)
    g = acc.stencil([(0, -1), (0, 1), (-1, 0), (1, 0)], lambda l, r, u, d: acc.lift(r - l, d - u), "clamp", acc.use(img, cx), context=cx)
    gx, gy = acc.run(g, cx)
    t = pyref.tap_arrays(img, [(0, -1), (0, 1), (-1, 0), (1, 0)], "clamp", 0, img.shape)
    assert np.array_equal(gx, t[1] - t[0]) and np.array_equal(gy, t[3] - t[2])
    mag = acc.run(acc.map(lambda p: acc.fst(p) * acc.fst(p) + acc.snd(p) * acc.snd(p), g), cx)
    assert np.array_equal(mag, (t[1] - t[0]) ** 2 + (t[3] - t[2]) ** 2)


def test_stencil_over_an_array_of_pairs(acc):
    """complex numbers as (re, im) pairs: a 3-point average along rows, the pairs kept together"""
    cx = acc.Context(0)
    rng = np.random.default_rng(15)
    re, im = rng.integers(-9, 9, (33, 260)).astype(np.float32), rng.integers(-9, 9, (33, 260)).astype(np.float32)
    z = acc.use((re, im), cx)

    def avg(a, b, c):
        return acc.lift(acc.fst(a) + acc.fst(b) + acc.fst(c), acc.snd(a) + acc.snd(b) + acc.snd(c))
    out_re, out_im = acc.run(acc.stencil([(0, -1), (0, 0), (0, 1)], avg, "wrap", z, context=cx), cx)
    tr = pyref.tap_arrays(re, [(0, -1), (0, 0), (0, 1)], "wrap", 0, re.shape)
    ti = pyref.tap_arrays(im, [(0, -1), (0, 0), (0, 1)], "wrap", 0, im.shape)
    assert np.array_equal(out_re, tr[0] + tr[1] + tr[2]) and np.array_equal(out_im, ti[0] + ti[1] + ti[2])
    # and of a delayed array of pairs, with a constant boundary given as a pair
    zz = acc.map(lambda p: acc.lift(acc.snd(p), acc.fst(p)), z)
    o1, o2 = acc.run(acc.stencil([(-1, 0), (1, 0)], lambda u, d: acc.lift(acc.fst(d) - acc.fst(u), acc.snd(d) - acc.snd(u)),
                                 "constant", zz, context=cx, constant_value=(1.0, -1.0)), cx)
    ti2 = pyref.tap_arrays(im, [(-1, 0), (1, 0)], "constant", 1.0, im.shape)
    tr2 = pyref.tap_arrays(re, [(-1, 0), (1, 0)], "constant", -1.0, re.shape)
    assert np.array_equal(o1, ti2[1] - ti2[0]) and np.array_equal(o2, tr2[1] - tr2[0])


def test_contexts_streams_of_inputs_and_asynchronous_runs(acc):
    """the rest of the reference module's export list (CUDA.hs:184-200): *With variants over a context made with
    `create`, `stream` over a sequence of inputs, `runAsync`/`run1Async` with `wait`/`poll`/`cancel`, `unsafeFree`
    and `performGC`"""
    rng = np.random.default_rng(40)
    cx = acc.create(0)
    try:
        x = rng.integers(-9, 9, 50001).astype(np.int32)
        assert np.array_equal(acc.runWith(cx, acc.scanl1(add, acc.use(x, cx), context=cx)), np.cumsum(x, dtype=np.int32))
        step = lambda xs: acc.map(lambda v: v * 3 + 1, xs)
        assert np.array_equal(acc.run1With(cx, step)(x), x * 3 + 1)
        inputs = [rng.integers(-9, 9, n).astype(np.int32) for n in (1, 1000, 77777)]
        n_kernels = None
        for a, r in zip(inputs, acc.streamWith(cx, step, inputs)):
            assert np.array_equal(r, a * 3 + 1)
            n_kernels = n_kernels or len(cx.skeletons)
        assert len(cx.skeletons) == n_kernels                     # built for the first input, reused for the rest
        # several computations in flight, in this context and the default one
        ys = [rng.standard_normal(200003).astype(np.float32) for _ in range(4)]
        dot = lambda a, b: acc.fold(add, 0.0, acc.zipWith(lambda p, q: p * q, a, b))
        jobs = [acc.runAsyncWith(cx if k % 2 else acc.Context.default(),
                                 dot(acc.use(y, cx if k % 2 else None), acc.use(ys[0], cx if k % 2 else None)))
                for k, y in enumerate(ys)]
        for y, j in zip(ys, jobs):
            r = acc.wait(j)
            assert abs(float(r) - float(np.dot(y.astype(np.float64), ys[0].astype(np.float64)))) < 1e-3 * np.sqrt(y.size)
            assert acc.poll(j) is not None
        go = acc.run1AsyncWith(cx, step)
        assert np.array_equal(acc.wait(go(x)), x * 3 + 1)
        # a cancelled computation stops at its next skeleton and says so
        import threading
        gate = threading.Event()

        def slow(xs):
            gate.wait()
            return acc.map(lambda v: v + 1, xs)
        j = acc.Async(lambda: acc.run(slow(acc.use(x, cx)), cx))
        stopper = threading.Thread(target=acc.cancel, args=(j,))
        stopper.start()
        while not j._cancelled:
            pass
        gate.set()
        stopper.join()
        with pytest.raises(acc.Cancelled):
            acc.wait(j)
        # unsafeFree gives the device copy back at once; performGC empties the pool of freed blocks
        big = rng.integers(0, 9, 1 << 20).astype(np.int32)
        xs = acc.use(big, cx)
        assert int(acc.runWith(cx, acc.fold(add, 0, xs, context=cx))) == int(big.sum())
        resident = cx.table.stats()["resident_arrays"]
        acc.unsafeFreeWith(cx, big)
        assert cx.table.stats()["resident_arrays"] == resident - 1
        with pytest.raises(Exception):
            acc.runWith(cx, acc.fold(add, 0, xs, context=cx))     # the computation still refers to it: it fails, loudly
        acc.performGCWith(cx)
        assert cx.table.stats()["nursery_bytes"] == 0
    finally:
        acc.destroy(cx)
    assert cx.ctx.handle is None


def test_reshape_replicate_slice_and_array_level_conditional(acc):
    rng = np.random.default_rng(41)
    m = rng.integers(-50, 50, (37, 53)).astype(np.int32)
    v = rng.integers(-50, 50, 53).astype(np.int32)
    ms, vs = acc.use(m), acc.use(v)
    # matrix-vector product the Accelerate way: replicate the vector over the rows, multiply, fold the rows
    mv = acc.fold(add, 0, acc.zipWith(lambda a, b: a * b, ms, acc.replicate((37, acc.All), vs)))
    assert np.array_equal(acc.run(mv), m @ v)
    # a new innermost dimension
    r = acc.run(acc.replicate((acc.All, 4), vs))
    assert r.shape == (53, 4) and np.array_equal(r, np.repeat(v[:, None], 4, axis=1))
    # slices: a row, a column
    assert np.array_equal(acc.run(acc.map(lambda x: x + 1, acc.slice_(ms, (5, acc.All)))), m[5] + 1)
    assert np.array_equal(acc.run(acc.map(lambda x: x + 1, acc.slice_(ms, (acc.All, 7)))), m[:, 7] + 1)
    # reshape of a manifest array (no kernel) and of a delayed one
    cx = acc.Context.default()
    n = len(cx.skeletons)
    flat = acc.flatten(ms)
    assert flat.manifest is ms.manifest and len(cx.skeletons) == n
    assert np.array_equal(acc.run(acc.scanl1(add, flat)), np.cumsum(m.reshape(-1), dtype=np.int32))
    d = acc.reshape((53, 37), acc.map(lambda x: x * 2, ms))
    assert np.array_equal(acc.run(acc.fold(add, 0, d)), (m * 2).reshape(53, 37).sum(axis=1, dtype=np.int32))
    with pytest.raises(ValueError):
        acc.reshape((10, 10), ms)
    # imap, zipWith3, iterate
    assert np.array_equal(acc.run(acc.imap(lambda ix, x: x + acc.fromIntegral(ix[0] * 100 + ix[1], "Int32"), ms)),
                          m + (np.arange(37)[:, None] * 100 + np.arange(53)[None, :]).astype(np.int32))
    assert np.array_equal(acc.run(acc.zipWith3(lambda a, b, c: a * b + c, vs, vs, vs)), v * v + v)
    assert np.array_equal(acc.run(acc.iterate(3, lambda a: acc.map(lambda x: x * 2 + 1, a), vs)), ((v * 2 + 1) * 2 + 1) * 2 + 1)
    # acond: only the branch taken is built
    built = []

    def branch(tag, k):
        def go():
            built.append(tag)
            return acc.map(lambda x: x + k, vs)
        return go
    big = acc.map(lambda s: s > 10 ** 6, acc.fold(add, 0, vs))
    assert np.array_equal(acc.run(acc.acond(big, branch("then", 1), branch("else", 2))), v + 2) and built == ["else"]


def test_the_rest_of_the_scalar_primitives(acc):
    """every PrimFun the reference's code generator knows (CodeGen.hs) is reachable from the language: the ones the
    other tests do not use, against numpy.  Transcendental results within 4 ulp of numpy's Float32 (the device's
    math library is not bit-identical to the host's); everything else exact."""
    rng = np.random.default_rng(42)
    x = (rng.random(5003) * 1.8 - 0.9).astype(np.float32)
    xs = acc.use(x)

    def close(got, ref, ulps=4):
        ref = ref.astype(np.float32)
        return np.all(np.abs(got - ref) <= ulps * np.spacing(np.abs(ref)) + 1e-37)
    for fn, ref in ((acc.asin, np.arcsin), (acc.acos, np.arccos), (acc.atan, np.arctan), (acc.sinh, np.sinh),
                    (acc.cosh, np.cosh), (acc.tanh, np.tanh), (acc.asinh, np.arcsinh), (acc.atanh, np.arctanh)):
        assert close(acc.run(acc.map(fn, xs)), ref(x)), fn.__name__
    assert close(acc.run(acc.map(lambda v: acc.acosh(v + 2.0), xs)), np.arccosh(x + np.float32(2)))
    assert close(acc.run(acc.map(lambda v: acc.atan2(v, v * v - 0.5), xs)), np.arctan2(x, x * x - np.float32(0.5)))
    assert close(acc.run(acc.map(lambda v: acc.pow_(v + 2.0, v), xs)), np.power(x + np.float32(2), x))
    assert close(acc.run(acc.map(lambda v: acc.logBase(acc.constant(3.0, "float"), v + 2.0), xs)),
                 np.log(x + np.float32(2)) / np.log(np.float32(3)), ulps=8)
    assert np.array_equal(acc.run(acc.map(acc.recip, xs)), np.float32(1) / x)
    nan = x.copy()
    nan[::7] = np.nan
    assert np.array_equal(acc.run(acc.map(acc.isNaN, acc.use(nan))), np.isnan(nan).astype(np.uint8))
    w = rng.integers(0, 2 ** 32, 4001, dtype=np.uint32)
    ws = acc.use(w)
    assert np.array_equal(acc.run(acc.map(lambda v: acc.rotateL(v, 7), ws)), (w << np.uint32(7)) | (w >> np.uint32(25)))
    assert np.array_equal(acc.run(acc.map(lambda v: acc.rotateR(v, 7), ws)), (w >> np.uint32(7)) | (w << np.uint32(25)))
    assert np.array_equal(acc.run(acc.map(lambda v: acc.boolToInt(v > 2 ** 31), ws)), (w > 2 ** 31).astype(np.int64))
    assert np.array_equal(acc.run(acc.map(lambda v: acc.ord_(acc.chr_(v)), ws)), w.astype(np.int64))
    a = rng.integers(-1000, 1000, 4001).astype(np.int32)
    b = rng.integers(1, 50, 4001).astype(np.int32) * rng.choice([-1, 1], 4001).astype(np.int32)
    q, r = acc.run(acc.unzip(acc.zipWith(acc.quotRem, acc.use(a), acc.use(b))))
    assert np.array_equal(q, np.trunc(a / b).astype(np.int32)) and np.array_equal(r, a - b * np.trunc(a / b).astype(np.int32))
    d, m = acc.run(acc.unzip(acc.zipWith(acc.divMod, acc.use(a), acc.use(b))))
    assert np.array_equal(d, a // b) and np.array_equal(m, a % b)


def test_empty_arrays_and_booleans(acc):
    """arrays without elements through every consumer (Reduction.hs:212-214, PrefixSum.hs:249-251, Execute.hs:282-289),
    and host arrays of booleans, which are Word8 on the device"""
    e = np.zeros(0, np.int32)
    assert acc.run(acc.map(lambda v: v + 1, acc.use(e))).shape == (0,)
    assert int(acc.run(acc.fold(add, 7, acc.use(e)))) == 7
    assert acc.run(acc.scanl(add, 3, acc.use(e))).tolist() == [3]
    assert acc.run(acc.scanl1(add, acc.use(e))).shape == (0,)
    body, total = acc.run(acc.scanl_(add, 3, acc.use(e)))
    assert body.shape == (0,) and int(total) == 3
    assert acc.run(acc.permute(add, acc.fill((5,), 1, "Int32"), lambda i: (i,), acc.use(e))).tolist() == [1] * 5
    with pytest.raises(Exception, match="empty array"):
        acc.run(acc.fold1(add, acc.use(e)))
    # rows without elements yield the seed; an empty OUTER extent counts as 1 in a seeded fold's result, and a fold1
    # over no rows is an empty array
    assert acc.run(acc.fold(add, 7, acc.use(np.zeros((5, 0), np.int32)))).tolist() == [7] * 5
    assert acc.run(acc.fold(add, 7, acc.use(np.zeros((0, 5), np.int32)))).tolist() == [7]
    assert acc.run(acc.fold1(add, acc.use(np.zeros((0, 5), np.int32)))).shape == (0,)
    assert acc.run(acc.foldSeg(add, 0, acc.use(e), acc.use(e))).shape == (0,)
    assert acc.run(acc.foldSeg(add, 0, acc.use(np.arange(6, dtype=np.int32)), acc.use(np.array([0, 3, 0, 3, 0], np.int32)))).tolist() == [0, 3, 0, 12, 0]
    kept, count = acc.run(acc.filter_(lambda v: v > 100, acc.use(np.arange(10, dtype=np.int32))))
    assert kept.shape == (0,) and int(count) == 0
    # an array `use`d inside the scalar function itself, Int64 indices
    h = acc.run(acc.permute(add, acc.fill((4,), 0, "Int64"), lambda i: (acc.use(np.array([0, 3, 3, 1], np.int64))[i],), acc.fill((4,), 5, "Int64")))
    assert h.tolist() == [5, 5, 0, 10]
    flags = np.array([True, False, True, True])
    assert acc.run(acc.map(lambda v: v.lnot(), acc.use(flags))).tolist() == [0, 1, 0, 0]
    assert int(acc.run(acc.sum_(acc.map(lambda v: acc.fromIntegral(v, "Int32"), acc.use(flags))))) == 3


def test_threads_building_computations_in_one_context(acc):
    """consumers launch as they are built, so threads that share a context meet in its launch path: eight threads,
    each with its own arrays and a few skeletons in common"""
    import threading
    cx = acc.create(0)
    errors = []

    def work(k):
        try:
            rng = np.random.default_rng(100 + k)
            for rep in range(5):
                x = rng.integers(-50, 50, 20000 + 37 * k + rep).astype(np.int32)
                xs = acc.use(x, cx)
                s = acc.run(acc.scanl1(add, acc.map(lambda v: v * 2, xs)), cx)
                assert np.array_equal(s, np.cumsum(x * 2, dtype=np.int32))
                h = acc.run(acc.permute(add, acc.fill((64,), 0, "Int32"), lambda i: (acc.use(np.abs(x) % 64, cx)[i],), acc.fill((x.size,), 1, "Int32")), cx)
                assert np.array_equal(h, np.bincount(np.abs(x) % 64, minlength=64).astype(np.int32))
        except Exception as e:                      # reported by the main thread
            errors.append((k, repr(e)))
    threads = [threading.Thread(target=work, args=(k,)) for k in range(8)]
    for t in threads:
        t.start()
    for t in threads:
        t.join()
    try:
        assert not errors, errors
    finally:
        acc.destroy(cx)


def test_results_of_a_repeated_call_come_in_page_locked_memory_that_is_used_again(acc):
    """`run` hands large results out in host memory that the device writes directly and that is used again when the
    program has dropped the array: not the first time a size is asked for, never beyond the pool's limit, and a buffer
    stays away from the pool for as long as any view of its array lives -- or its context does not."""
    rng = np.random.default_rng(12)
    cx = acc.create(0, result_pool_bytes=5 << 20)
    n = (1 << 19) + 3                                     # 2 MB and a little: a buffer of 3 MB
    inc = acc.run1(lambda a: acc.map(lambda v: v + acc.constant(1, "Int32"), a), cx)
    x = rng.integers(0, 1000, n).astype(np.int32)
    r1 = inc(x.copy())
    assert np.array_equal(r1, x + 1) and cx.results.held == 0        # an ordinary array the first time
    r2 = inc(x.copy())
    assert np.array_equal(r2, x + 1) and cx.results.held == 3 << 20
    where = r2.ctypes.data
    tail = r2[-5:]                                        # a view keeps the buffer out of the pool
    del r2
    r3 = inc(x.copy())
    assert r3.ctypes.data != where and cx.results.held == 3 << 20    # the limit: an ordinary array again
    assert np.array_equal(tail, x[-5:] + 1)
    del tail
    r4 = inc(x.copy())
    assert r4.ctypes.data == where and np.array_equal(r4, x + 1) and r4.flags.writeable
    r4 += 1                                               # the array is the program's to change
    assert np.array_equal(r4, x + 2)
    small = acc.run(acc.map(lambda v: v + acc.constant(1, "Int32"), acc.use(x[:100].copy(), cx)), cx)
    small = acc.run(acc.map(lambda v: v + acc.constant(1, "Int32"), acc.use(x[:100].copy(), cx)), cx)
    assert np.array_equal(small, x[:100] + 1) and cx.results.held == 3 << 20      # small results: ordinary arrays
    acc.performGC(cx)
    assert cx.results.held == 3 << 20                     # r4 still holds its buffer
    acc.destroy(cx)
    assert np.array_equal(r4, x + 2)                      # and keeps it when the context has gone
    del r4                                                # (given back to the system, not to the pool)


def test_pagerank_on_a_graph_with_hubs(acc):
    """PageRank as the reference's examples write it -- every edge carries rank[source] / outdegree[source] to its
    target, a segmented sum over the edges sorted by target, a damping map -- on a graph whose in-degrees follow a power
    law with three hubs that a third of all edges point to.  Two dozen iterations, each a `run1` call of the same
    computation (so the segmented fold's instance lives on, looks at its segment lengths, and takes its variants
    with a table of jobs once they are compiled); against Float64 numpy within 1e-4 of the largest rank."""
    rng = np.random.default_rng(21)
    nodes, edges = 60000, 1500000
    weight = 1.0 / np.arange(1, nodes + 1) ** 0.9
    target = rng.choice(nodes, edges, p=weight / weight.sum())
    hubs = rng.random(edges) < 0.33
    target[hubs] = rng.choice([5, 6, 40000], int(hubs.sum()))
    source = rng.integers(0, nodes, edges)
    order = np.argsort(target, kind="stable")
    target, source = target[order], source[order].astype(np.int32)
    indeg = np.bincount(target, minlength=nodes).astype(np.int32)
    outdeg = np.maximum(np.bincount(source, minlength=nodes), 1).astype(np.float32)
    assert indeg.max() > 150000

    src, seg, deg = acc.use(source), acc.use(indeg), acc.use(outdeg)

    def step(rank):
        share = acc.zipWith(lambda r, d: r / d, rank, deg)
        carried = acc.map(lambda s: share[s], src)
        inflow = acc.foldSeg(add, 0.0, carried, seg)
        return acc.map(lambda v: acc.constant(0.15 / nodes, "float") + acc.constant(0.85, "float") * v, inflow)
    one = acc.run1(step)
    rank = np.full(nodes, 1.0 / nodes, np.float32)
    ref = rank.astype(np.float64)
    import time
    for k in range(24):
        rank = one(rank)
        ref = 0.15 / nodes + 0.85 * np.bincount(target, weights=(ref / outdeg)[source], minlength=nodes)
        assert np.all(np.abs(rank - ref) <= 1e-4 * ref.max()), k
        if k == 11:
            time.sleep(1.0)                 # (the variants with the table are compiled by now: the second half takes them)


def test_column_sums_and_a_matrix_product_written_as_folds(acc):
    """`fold (+) 0 (transpose m)` and the matrix product of the reference's examples, `fold (+) 0 (zipWith (*)
    (replicate (Z :. All :. n :. All) a) (replicate (Z :. m :. All :. All) (transpose b)))`: the fold's rows lie
    across memory, which the front end knows and says (ACC_FLAG_TILED), so a lane takes a row.  One kernel each,
    integer results exact; a transpose of a transpose reads along the rows again."""
    rng = np.random.default_rng(31)
    cx = acc.Context.default()
    m = rng.integers(-50, 50, (3001, 257)).astype(np.int32)
    t = acc.transpose(acc.use(m))
    assert t.across and not acc.transpose(t).across
    before = len(cx.skeletons)
    got = acc.run(acc.fold(add, 0, t))
    assert len(cx.skeletons) == before + 1
    assert np.array_equal(got, m.sum(axis=0, dtype=np.int32))
    assert np.array_equal(acc.run(acc.fold(add, 0, acc.transpose(t))), m.sum(axis=1, dtype=np.int32))
    # an index function of the user's own that exchanges the two innermost dimensions of a rank-3 array: found out by
    # applying it to numbers
    c = rng.integers(-50, 50, (5, 60, 70)).astype(np.int32)
    swapped = acc.backpermute((5, 70, 60), lambda i, k, j: (i, j, k), acc.use(c))
    assert swapped.across and not acc.backpermute((60, 5, 70), lambda j, i, k: (i, j, k), acc.use(c)).across
    assert np.array_equal(acc.run(swapped), c.transpose(0, 2, 1))
    assert np.array_equal(acc.run(acc.fold(add, 0, swapped)), c.sum(axis=1, dtype=np.int32))
    # a volume turned so that its innermost dimension becomes the outermost: the source is read along the result's
    # outermost dimension, and the tiles pair that one with the innermost (ACC_FLAG_TILE_DIM)
    turned = acc.backpermute((70, 5, 60), lambda k, i, j: (i, j, k), acc.use(c))
    assert turned.across == 2
    assert np.array_equal(acc.run(turned), c.transpose(2, 0, 1))
    # its fold -- the sum over the volume's middle dimension -- goes through the fold of the volume with the two
    # dimensions exchanged, a lane a row, and comes back exchanged
    before = len(cx.skeletons)
    assert np.array_equal(acc.run(acc.fold(add, 0, turned)), c.sum(axis=1, dtype=np.int32).T)
    assert np.array_equal(acc.run(acc.fold1(lambda p, q: acc.cond(p > q, p, q), turned)), c.max(axis=1).T)
    c4 = rng.integers(-50, 50, (3, 40, 5, 70)).astype(np.int32)
    turned4 = acc.backpermute((3, 70, 5, 40), lambda a_, l, k, j: (a_, j, k, l), acc.use(c4))
    assert turned4.across == 2
    assert np.array_equal(acc.run(acc.map(lambda v: v + v, turned4)), 2 * c4.transpose(0, 3, 2, 1))
    assert np.array_equal(acc.run(acc.fold(add, 0, turned4)), c4.transpose(0, 3, 2, 1).sum(axis=3, dtype=np.int32))
    mm, kk, nn = 70, 333, 129
    a = rng.integers(-9, 9, (mm, kk)).astype(np.int32)
    b = rng.integers(-9, 9, (kk, nn)).astype(np.int32)

    def mmult(x, y):
        xr = acc.replicate((acc.All, nn, acc.All), x)
        yr = acc.replicate((mm, acc.All, acc.All), acc.transpose(y))
        assert yr.across and not xr.across
        return acc.fold(add, 0, acc.zipWith(lambda p, q: p * q, xr, yr))
    before = len(cx.skeletons)
    got = acc.run1(mmult)(a, b)
    assert len(cx.skeletons) == before + 1
    assert np.array_equal(got, a @ b)
    fa, fb = a.astype(np.float32) / 8, b.astype(np.float32) / 4            # exact in Float32 whatever the order
    def mmultf(x, y):
        xr = acc.replicate((acc.All, nn, acc.All), x)
        yr = acc.replicate((mm, acc.All, acc.All), acc.transpose(y))
        return acc.fold(add, 0.0, acc.zipWith(lambda p, q: p * q, xr, yr))
    assert np.array_equal(acc.run1(mmultf)(fa, fb), fa @ fb)
