"""Tuple element types (structure of arrays, one result pointer per component)
through map, fold, fold along a dimension, foldSeg and the scans.

What each case is checked against is independent of the kernels: numpy's
argmax / cumsum / reduceat / minimum / maximum, or a sequential Python loop
for the non-commutative operator.  Integer components are compared bit for
bit; the one Float64 sum states its tolerance.
"""
import sys

import numpy as np
import pytest

pytestmark = pytest.mark.gpu

F32, I32 = (1, "float"), (1, "Int32")
SIZES = [1, 63, 64, 65, 4097, 100003, (1 << 20) + 17]


def say(*a):
    print("[case]", *a)
    sys.stdout.flush()


@pytest.fixture(scope="module")
def A():
    import acchip
    return acchip


@pytest.fixture(scope="module")
def ctx(A):
    c = A.Context(0)
    yield c
    c.close()


def test_map_builds_and_takes_apart_pairs(A, ctx):
    rng = np.random.default_rng(3)
    zipk = ctx.skeleton(A.SKEL_MAP, "float, Int32", env=[F32, I32], out_rank=1, get="acc_elt{arrIn0_0[ix] * 2.0f, arrIn1_0[ix] + 1}")
    # a free array of pairs: component 1 is the first element, component 0 the second
    swap = ctx.skeleton(A.SKEL_MAP, "Int32, float", env=[(1, ["Int32", "float"])], out_rank=1,
                        get="acc_elt{arrIn0_0[ix], arrIn0_1[ix]}")
    for n in [0] + SIZES:
        say("zip / swap, n =", n)
        x = rng.random(n).astype(np.float32)
        k = rng.integers(-1000, 1000, n).astype(np.int32)
        out = ctx.empty_tuple(n, [np.float32, np.int32])
        zipk.map([ctx.array(x), ctx.array(k)], out)
        a, b = out.get()
        assert np.array_equal(a, x * np.float32(2)) and np.array_equal(b, k + 1)
        out2 = ctx.empty_tuple(n, [np.int32, np.float32])
        swap.map([out], out2)
        b2, a2 = out2.get()
        assert np.array_equal(a2, a) and np.array_equal(b2, b)


def test_fold_argmax_of_value_index_pairs(A, ctx):
    rng = np.random.default_rng(4)
    argmax = ctx.skeleton(A.SKEL_FOLD, "float, Int32", env=[F32], out_rank=0, get="acc_elt{arrIn0_0[ix], (Int32)ix}",
                          combine="(x.a1 > y.a1 || (x.a1 == y.a1 && x.a0 < y.a0)) ? x : y", seed="acc_elt{-1.0f, 2147483647}")
    for n in [0] + SIZES + [1 << 24]:
        say("argmax, n =", n)
        x = rng.integers(0, 1000, n).astype(np.float32)          # many ties: the smallest index must win
        out = ctx.empty_tuple((), [np.float32, np.int32])
        argmax.fold([ctx.array(x)], n, out)
        v, i = out.get()
        if n == 0:
            assert float(v) == -1.0 and int(i) == 2147483647      # the seed
        else:
            assert int(i) == int(np.argmax(x)) and float(v) == float(x.max())


def test_fold_along_rows_min_and_max(A, ctx):
    rng = np.random.default_rng(5)
    mm = ctx.skeleton(A.SKEL_FOLD, "Int32, Int32", env=[(2, "Int32")], out_rank=1, get="acc_elt{arrIn0_0[ix], arrIn0_0[ix]}",
                      combine="acc_elt{acc_pmin(x.a1, y.a1), acc_pmax(x.a0, y.a0)}", seed="acc_elt{2147483647, -2147483647 - 1}")
    for rows, cols in [(1, 1), (7, 100), (300, 65), (64, 4096), (1000, 1001)]:
        say("row-wise (min, max)", rows, "x", cols)
        x = rng.integers(-10 ** 9, 10 ** 9, (rows, cols)).astype(np.int32)
        out = ctx.empty_tuple(rows, [np.int32, np.int32])
        mm.fold([ctx.array(x)], (rows, cols), out)
        lo, hi = out.get()
        assert np.array_equal(lo, x.min(axis=1)) and np.array_equal(hi, x.max(axis=1))


def test_foldseg_sum_and_count(A, ctx):
    rng = np.random.default_rng(6)
    sc = ctx.skeleton(A.SKEL_FOLDSEG, "double, Int32", env=[F32], get="acc_elt{(double)arrIn0_0[ix], 1}",
                      combine="acc_elt{x.a1 + y.a1, x.a0 + y.a0}", seed="acc_elt{0.0, 0}")
    for nseg in [1, 5, 257, 10000]:
        say("foldSeg (sum, count), segments =", nseg)
        lens = rng.poisson(20, nseg).astype(np.int32)
        lens[::7] = 0
        offs = np.concatenate([[0], np.cumsum(lens)]).astype(np.int32)
        n = int(offs[-1])
        x = rng.random(n).astype(np.float32)
        out = ctx.empty_tuple(nseg, [np.float64, np.int32])
        sc.foldseg([ctx.array(x)], n, ctx.array(offs), out)
        s, c = out.get()
        assert np.array_equal(c, lens)
        exp = np.array([x[offs[i]:offs[i + 1]].astype(np.float64).sum() for i in range(nseg)])
        assert np.all(np.abs(s - exp) <= 1e-12 * np.maximum(1.0, np.abs(exp)))      # Float64 sums of <= ~50 Float32 values


def segmented_cumsum(flags, vals):
    out = np.empty_like(vals)
    run = 0
    for i in range(vals.size):
        run = int(vals[i]) if flags[i] else run + int(vals[i])
        out[i] = np.int32(run)
    return out


@pytest.mark.parametrize("kind", ["scanl1", "scanl", "scanl'", "scanr1"])
def test_segmented_scan_with_flag_value_pairs(A, ctx, kind):
    """(f1, v1) (+) (f2, v2) = (f1 | f2, f2 ? v2 : v1 + v2): associative, not commutative"""
    rng = np.random.default_rng(7)
    seeded = not kind.endswith("1")
    right = kind.startswith("scanr")
    # op(earlier, later) in logical order; the right-handed scans are handed f with its arguments as Data.List has them
    body = "acc_elt{E.a1 | L.a1, L.a1 ? L.a0 : E.a0 + L.a0}"
    combine = body.replace("E", "y").replace("L", "x") if right else body.replace("E", "x").replace("L", "y")
    sk = ctx.skeleton(A.SCAN_KINDS[kind], "Int32, Int32", env=[I32, I32], get="acc_elt{arrIn0_0[ix], arrIn1_0[ix]}",
                      combine=combine, seed="acc_elt{0, 0}" if seeded else None)
    for n in SIZES:
        say(kind, "segmented sum, n =", n)
        flags = (rng.random(n) < 0.01).astype(np.int32)
        vals = rng.integers(-100, 100, n).astype(np.int32)
        m = n + 1 if kind == "scanl" else n
        out = ctx.empty_tuple(m, [np.int32, np.int32])
        tot = ctx.empty_tuple((), [np.int32, np.int32]) if kind == "scanl'" else None
        sk.scan([ctx.array(flags), ctx.array(vals)], n, out, tot)
        gf, gv = out.get()
        if right:       # scanr1: the same recurrence walking from the end
            exp = segmented_cumsum(flags[::-1], vals[::-1])[::-1]
            assert np.array_equal(gv, exp) and np.array_equal(gf, np.maximum.accumulate(flags[::-1])[::-1])
            continue
        inc = segmented_cumsum(flags, vals)                       # inclusive results; the seed (0, 0) is an identity here
        incf = np.maximum.accumulate(flags)
        if kind == "scanl1":
            assert np.array_equal(gv, inc) and np.array_equal(gf, incf)
        elif kind == "scanl":
            assert gv[0] == 0 and gf[0] == 0 and np.array_equal(gv[1:], inc) and np.array_equal(gf[1:], incf)
        else:
            tf, tv = tot.get()
            assert gv[0] == 0 and np.array_equal(gv[1:], inc[:-1]) and np.array_equal(gf[1:], incf[:-1])
            assert int(tv) == int(inc[-1]) and int(tf) == int(incf[-1])


def test_permute_of_tuples_and_narrow_elements_under_locks(A, ctx):
    """elements no atomic instruction covers are combined under a lock per target (IndexSpace.hs:285-303)"""
    rng = np.random.default_rng(9)
    n, bins = 300000, 500
    keys = rng.integers(-3, bins + 3, n).astype(np.int32)            # a few strays on both sides, dropped
    keys[::19] = -1
    w = rng.integers(-50, 50, n).astype(np.float32)                  # whole numbers: Float32 sums are exact in any order
    ok = (keys >= 0) & (keys < bins)
    say("permute (sum, count) pairs")
    sk = ctx.skeleton(A.SKEL_PERMUTE, "float, Int32", env=[I32, F32], out_rank=1, get="acc_elt{arrIn1_0[ix], 1}",
                      combine="acc_elt{x.a1 + y.a1, x.a0 + y.a0}", permutation="arrIn0_0[ix]")
    d0 = rng.integers(-5, 5, bins).astype(np.float32)
    d1 = rng.integers(0, 3, bins).astype(np.int32)
    out = ctx.empty_tuple(bins, [np.float32, np.int32])
    sk.permute([ctx.array(keys), ctx.array(w)], n, ctx.tuple_array(d0, d1), out)
    s_, c_ = out.get()
    assert np.array_equal(c_, d1 + np.bincount(keys[ok], minlength=bins).astype(np.int32))
    assert np.array_equal(s_, d0 + np.bincount(keys[ok], weights=w[ok].astype(np.float64), minlength=bins).astype(np.float32))
    say("the same again: the locks were left open")
    sk.permute([ctx.array(keys), ctx.array(w)], n, ctx.tuple_array(d0, d1), out)
    assert np.array_equal(out.get()[1], c_)
    say("permute into Int16 and Word8 targets, every key the same target among them")
    h16 = ctx.skeleton(A.SKEL_PERMUTE, "Int16", env=[I32], out_rank=1, get="(Int16)1", combine="(Int16)(x + y)", permutation="arrIn0_0[ix]")
    few = rng.integers(0, 40, 20000).astype(np.int32)
    few[:3000] = 7
    o16 = ctx.empty(40, np.int16)
    h16.permute([ctx.array(few)], few.size, ctx.array(np.zeros(40, np.int16)), o16)
    assert np.array_equal(o16.get(), np.bincount(few, minlength=40).astype(np.int16))
    or8 = ctx.skeleton(A.SKEL_PERMUTE, "Word8", env=[I32, (1, "Word8")], out_rank=1, get="arrIn1_0[ix]", combine="(Word8)(x | y)",
                       permutation="arrIn0_0[ix]")
    bits = (1 << rng.integers(0, 8, few.size)).astype(np.uint8)
    o8 = ctx.empty(40, np.uint8)
    or8.permute([ctx.array(few), ctx.array(bits)], few.size, ctx.array(np.zeros(40, np.uint8)), o8)
    exp = np.zeros(40, np.uint8)
    np.bitwise_or.at(exp, few, bits)
    assert np.array_equal(o8.get(), exp)


def test_locked_permute_loses_no_update_at_scale(A, ctx):
    """4 M updates: on few targets (tables in LDS under LDS locks, joined by a second launch: 7 targets, where every
    lane of a workgroup wants the same few locks; 13 000, about the largest single table; 100 003, ten windows of
    targets) and on many (3 M: a lock per target in memory).  Integer sums and counts are exact, so one lost or torn
    update shows."""
    rng = np.random.default_rng(23)
    n = 1 << 22
    w = rng.integers(-1000, 1000, n).astype(np.int64)
    sk = ctx.skeleton(A.SKEL_PERMUTE, "Int64, Int32", env=[I32, (1, "Int64")], out_rank=1, get="acc_elt{arrIn1_0[ix], 1}",
                      combine="acc_elt{x.a1 + y.a1, x.a0 + y.a0}", permutation="arrIn0_0[ix]")
    for bins in (7, 1000, 13000, 100003, 3000017):
        say("locked permute, %d updates into %d targets" % (n, bins))
        keys = rng.integers(0, bins, n).astype(np.int32)
        out = ctx.empty_tuple(bins, [np.int64, np.int32])
        sk.permute([ctx.array(keys), ctx.array(w)], n, ctx.tuple_array(np.zeros(bins, np.int64), np.zeros(bins, np.int32)), out)
        s_, c_ = out.get()
        assert np.array_equal(c_, np.bincount(keys, minlength=bins).astype(np.int32))
        ref = np.zeros(bins, np.int64)
        np.add.at(ref, keys, w)
        assert np.array_equal(s_, ref)


def test_generic_combination_on_few_targets_goes_through_lds_tables(A, ctx):
    """a 4-byte element with a combination that is no hardware atomic: compare-and-swap loops on many targets,
    the locked template's tables in LDS on few -- same results"""
    rng = np.random.default_rng(29)
    n = 1 << 21
    v = rng.integers(-10 ** 6, 10 ** 6, n).astype(np.int32)
    sk = ctx.skeleton(A.SKEL_PERMUTE, "Int32", env=[I32, I32], out_rank=1, get="arrIn1_0[ix]",
                      combine="(x > y) ? x : y", permutation="arrIn0_0[ix]")        # max, spelt so that no hint applies
    for bins in (1, 5, 300, 20000, 200000, 1500000):
        say("generic permute (max) into", bins, "targets")
        keys = rng.integers(-2, bins + 2, n).astype(np.int32)
        d = rng.integers(-10 ** 6, 10 ** 6, bins).astype(np.int32)
        out = ctx.empty(bins, np.int32)
        sk.permute([ctx.array(keys), ctx.array(v)], n, ctx.array(d), out)
        ok = (keys >= 0) & (keys < bins)
        ref = d.copy()
        np.maximum.at(ref, keys[ok], v[ok])
        assert np.array_equal(out.get(), ref)


def test_stencils_with_tuple_results(A, ctx):
    """a stencil may produce a tuple per element (gradient pairs, magnitude and direction): one result array per
    component, in every boundary mode, on aligned and ragged widths, in 1, 2 and 3 dimensions, and from two sources"""
    import pyref
    rng = np.random.default_rng(31)
    taps = [(0, -1), (0, 1), (-1, 0), (1, 0)]
    for (h, w) in [(64, 256), (67, 301), (5, 1030)]:
        img = rng.integers(-100, 100, (h, w)).astype(np.float32)
        for mode in ("clamp", "mirror", "wrap", "constant"):
            say("gradient pairs", h, "x", w, mode)
            sk = ctx.skeleton(A.SKEL_STENCIL, "float, double, Int32", out_rank=2, taps=taps, boundary=mode, boundary_constant="2.0f",
                              stencil_in="float", stencil_fn="acc_elt{t1 - t0, (double)(t3 - t2) * 0.5, (Int32)(t0 + t1 + t2 + t3)}")
            out = ctx.empty_tuple((h, w), [np.float32, np.float64, np.int32])
            sk.stencil([], ctx.array(img), out)
            gx, gy, sm = out.get()
            t = pyref.tap_arrays(img, taps, mode, 2.0, (h, w))
            assert np.array_equal(gx, t[1] - t[0])
            assert np.array_equal(gy, (t[3] - t[2]).astype(np.float64) * 0.5)
            assert np.array_equal(sm, (t[0] + t[1] + t[2] + t[3]).astype(np.int32))
    say("1-D: value and index of the larger neighbour")
    v = rng.integers(-1000, 1000, 100003).astype(np.int32)
    sk = ctx.skeleton(A.SKEL_STENCIL, "Int32, Int8", out_rank=1, taps=[(0, -1), (0, 1)], boundary="clamp", stencil_in="Int32",
                      stencil_fn="acc_elt{acc_max(t0, t1), (Int8)(t1 > t0)}")
    out = ctx.empty_tuple((v.size,), [np.int32, np.int8])
    sk.stencil([], ctx.array(v), out)
    left, right = np.concatenate([v[:1], v[:-1]]), np.concatenate([v[1:], v[-1:]])
    big, which = out.get()
    assert np.array_equal(big, np.maximum(left, right)) and np.array_equal(which, (right > left).astype(np.int8))
    say("3-D: centre and sum of the two plane neighbours")
    vol = rng.integers(-9, 9, (9, 20, 260)).astype(np.float32)
    t3 = [(0, 0, 0), (-1, 0, 0), (1, 0, 0)]
    sk = ctx.skeleton(A.SKEL_STENCIL, "float, float", out_rank=3, taps=t3, boundary="wrap", stencil_in="float",
                      stencil_fn="acc_elt{t0, t1 + t2}")
    out = ctx.empty_tuple(vol.shape, [np.float32, np.float32])
    sk.stencil([], ctx.array(vol), out)
    c, nb = out.get()
    t = pyref.tap_arrays3(vol, t3, "wrap", 0, vol.shape)
    assert np.array_equal(c, t[0]) and np.array_equal(nb, t[1] + t[2])
    say("stencil2 with a pair result")
    a = rng.integers(-50, 50, (40, 300)).astype(np.float32)
    b = rng.integers(-50, 50, (40, 300)).astype(np.int32)
    sk = ctx.skeleton(A.SKEL_STENCIL2, "float, Int32", out_rank=2, taps=[(0, 0), (0, 1)], boundary="clamp", taps2=[(0, 0), (1, 0)],
                      boundary2="mirror", stencil_in="float", stencil_in2="Int32", stencil_fn="acc_elt{t1 - t0, u1 - u0}")
    out = ctx.empty_tuple(a.shape, [np.float32, np.int32])
    sk.stencil2([], ctx.array(a), ctx.array(b), out)
    da, db = out.get()
    ta, tb = pyref.tap_arrays(a, [(0, 0), (0, 1)], "clamp", 0, a.shape), pyref.tap_arrays(b, [(0, 0), (1, 0)], "mirror", 0, b.shape)
    assert np.array_equal(da, ta[1] - ta[0]) and np.array_equal(db, tb[1] - tb[0])


def test_tuple_results_need_tuple_arrays(A, ctx):
    say("misuse")
    zipk = ctx.skeleton(A.SKEL_MAP, "float, Int32", env=[F32], out_rank=1, get="acc_elt{arrIn0_0[ix], 0}")
    x = ctx.array(np.zeros(8, np.float32))
    with pytest.raises(A.AccError) as e:
        zipk.map([x], ctx.empty(8, np.float32))                  # one component offered, two needed
    assert e.value.code == A.ERR_INVALID
    with pytest.raises(A.AccError) as e:                         # a stencil with a tuple result must name its source's type
        ctx.skeleton(A.SKEL_STENCIL, "float, Int32", out_rank=1, taps=[(0, 0)], stencil_fn="acc_elt{t0, 1}")
    assert e.value.code == A.ERR_INVALID
    with pytest.raises(A.AccError) as e:
        ctx.skeleton(A.SKEL_MAP, "float, quux", env=[F32], out_rank=1, get="acc_elt{1.0f, 1}")
    assert e.value.code == A.ERR_INVALID


def test_stencils_over_sources_of_tuple_type(A, ctx):
    """the source of a stencil may be an array of tuples (Stencil/Extra.hs:53-128 reads every component): one array
    per component, a register window each, the taps structs of the components.  Components of different widths, a
    triple, every boundary mode (the constant one with a value per component), aligned and ragged widths, three
    dimensions, a result that is a tuple again, and a stencil2 with a tuple source and a scalar one"""
    import pyref
    rng = np.random.default_rng(47)
    taps = [(0, -1), (0, 0), (0, 1), (-1, 0), (1, 0)]
    for (h, w) in [(64, 256), (37, 301), (3, 1030)]:
        f = rng.integers(-50, 50, (h, w)).astype(np.float32)
        i = rng.integers(-50, 50, (h, w)).astype(np.int32)
        for mode in ("clamp", "mirror", "wrap", "constant"):
            say("5-point stencil over (float, Int32) pairs", h, "x", w, mode)
            sk = ctx.skeleton(A.SKEL_STENCIL, "float, Int32", out_rank=2, taps=taps, boundary=mode, boundary_constant="1.5f, -3",
                              stencil_in="float, Int32",
                              stencil_fn="acc_elt{t0.a1 + t2.a1 - 2.0f * t1.a1 + (float)t3.a0, t3.a0 + t4.a0 - t1.a0 + (Int32)t0.a1}")
            out = ctx.empty_tuple((h, w), [np.float32, np.int32])
            sk.stencil([], ctx.tuple_array(f, i), out)
            of, oi = out.get()
            tf = pyref.tap_arrays(f, taps, mode, 1.5, (h, w))
            ti = pyref.tap_arrays(i, taps, mode, -3, (h, w))
            assert np.array_equal(of, tf[0] + tf[2] - np.float32(2.0) * tf[1] + ti[3].astype(np.float32))
            assert np.array_equal(oi, ti[3] + ti[4] - ti[1] + tf[0].astype(np.int32))
            sk.destroy()
    say("a triple with components of 8, 1 and 2 bytes, scalar result")
    d = rng.integers(-9, 9, (20, 515)).astype(np.float64)
    b = rng.integers(0, 2, (20, 515)).astype(np.uint8)
    s16 = rng.integers(-300, 300, (20, 515)).astype(np.int16)
    sk = ctx.skeleton(A.SKEL_STENCIL, "double", out_rank=2, taps=[(0, -1), (0, 1)], boundary="mirror", stencil_in="double, Word8, Int16",
                      stencil_fn="(t0.a1 ? t0.a2 : t1.a2) + (double)(t1.a0 - t0.a0)")
    out = ctx.empty((20, 515), np.float64)
    sk.stencil([], ctx.tuple_array(d, b, s16), out)
    td = pyref.tap_arrays(d, [(0, -1), (0, 1)], "mirror", 0, d.shape)
    tb = pyref.tap_arrays(b, [(0, -1), (0, 1)], "mirror", 0, d.shape)
    ts = pyref.tap_arrays(s16, [(0, -1), (0, 1)], "mirror", 0, d.shape)
    assert np.array_equal(out.get(), np.where(tb[0] != 0, td[0], td[1]) + (ts[1].astype(np.int32) - ts[0].astype(np.int32)).astype(np.float64))
    sk.destroy()
    say("1-D and 3-D")
    x, y = rng.integers(-99, 99, 100003).astype(np.int32), rng.integers(-99, 99, 100003).astype(np.int64)
    sk = ctx.skeleton(A.SKEL_STENCIL, "Int64", out_rank=1, taps=[(0, -2), (0, 2)], boundary="wrap", stencil_in="Int32, Int64",
                      stencil_fn="(Int64)t0.a1 * t1.a0 - (Int64)t1.a1 * t0.a0")
    out = ctx.empty(x.size, np.int64)
    sk.stencil([], ctx.tuple_array(x, y), out)
    assert np.array_equal(out.get(), np.roll(x, 2).astype(np.int64) * np.roll(y, -2) - np.roll(x, -2).astype(np.int64) * np.roll(y, 2))
    sk.destroy()
    vf, vi = rng.integers(-9, 9, (7, 19, 260)).astype(np.float32), rng.integers(-9, 9, (7, 19, 260)).astype(np.int32)
    t3 = [(0, 0, 0), (-1, 0, 0), (1, 0, 0), (0, -1, 0), (0, 0, 1)]
    sk = ctx.skeleton(A.SKEL_STENCIL, "float", out_rank=3, taps=t3, boundary="clamp", stencil_in="float, Int32",
                      stencil_fn="t1.a1 + t2.a1 + t3.a1 + t4.a1 - 4.0f * t0.a1 + (float)(t1.a0 - t2.a0 + t3.a0 - t4.a0)")
    out = ctx.empty(vf.shape, np.float32)
    sk.stencil([], ctx.tuple_array(vf, vi), out)
    pf, pi = np.pad(vf, 1, mode="edge"), np.pad(vi, 1, mode="edge")
    c = lambda p, dz, dy, dx: p[1 + dz:p.shape[0] - 1 + dz, 1 + dy:p.shape[1] - 1 + dy, 1 + dx:p.shape[2] - 1 + dx]   # noqa: E731
    ref = (c(pf, -1, 0, 0) + c(pf, 1, 0, 0) + c(pf, 0, -1, 0) + c(pf, 0, 0, 1) - np.float32(4.0) * vf
           + (c(pi, -1, 0, 0) - c(pi, 1, 0, 0) + c(pi, 0, -1, 0) - c(pi, 0, 0, 1)).astype(np.float32))
    assert np.array_equal(out.get(), ref)
    sk.destroy()
    say("stencil2: a source of pairs and a scalar one, extents that differ")
    a1, a0 = rng.integers(-9, 9, (40, 300)).astype(np.float32), rng.integers(-9, 9, (40, 300)).astype(np.float32)
    m = rng.integers(-9, 9, (33, 310)).astype(np.int32)
    sk = ctx.skeleton(A.SKEL_STENCIL2, "float", out_rank=2, taps=[(0, -1), (0, 1)], boundary="clamp", taps2=[(-1, 0), (1, 0)], boundary2="constant",
                      boundary2_constant="5", stencil_in="float, float", stencil_in2="Int32",
                      stencil_fn="(t1.a1 - t0.a1) * (t1.a0 + t0.a0) + (float)(u1 - u0)")
    out = ctx.empty((33, 300), np.float32)
    sk.stencil2([], ctx.tuple_array(a1, a0), ctx.array(m), out)
    t1 = pyref.tap_arrays(a1, [(0, -1), (0, 1)], "clamp", 0, (33, 300))
    t0 = pyref.tap_arrays(a0, [(0, -1), (0, 1)], "clamp", 0, (33, 300))
    u = pyref.tap_arrays(m, [(-1, 0), (1, 0)], "constant", 5, (33, 300))
    assert np.array_equal(out.get(), (t1[1] - t1[0]) * (t0[1] + t0[0]) + (u[1] - u[0]).astype(np.float32))
    say("wrong use: a scalar array where the kernel was built for pairs; a constant with too few components")
    with pytest.raises(A.AccError) as e:
        sk.stencil2([], ctx.array(a1), ctx.array(m), out)
    assert e.value.code == A.ERR_INVALID
    sk.destroy()
    with pytest.raises(A.AccError) as e:
        ctx.skeleton(A.SKEL_STENCIL, "float", out_rank=1, taps=[(0, 0)], boundary="constant", boundary_constant="1.0f",
                     stencil_in="float, Int32", stencil_fn="t0.a1")
    assert e.value.code == A.ERR_INVALID



def test_tuples_of_twelve_components(A, ctx):
    """the kernel ABI names tuple components without a bound (CodeGen/Base.hs:69-79) and the array language's tuples have
    up to 15: a map that produces twelve components, a fold that reads an array of twelve"""
    n = 70001
    x = np.random.default_rng(12).integers(-1000, 1000, n).astype(np.int32)
    elt = ", ".join(["Int32"] * 12)
    make = ctx.skeleton(A.SKEL_MAP, elt, env=[I32], out_rank=1,
                        get="acc_elt{" + ", ".join("arrIn0_0[ix] * %d + %d" % (k + 1, k) for k in range(11, -1, -1)) + "}")
    out = ctx.empty_tuple(n, [np.int32] * 12)
    make.map([ctx.array(x)], out)
    got = out.get()                                           # components as the tuple reads: a11 first
    for i, g in enumerate(got):
        k = 11 - i
        assert np.array_equal(g, x * (k + 1) + k), k
    total = ctx.skeleton(A.SKEL_FOLD, "Int64", env=[(1, ["Int32"] * 12)], out_rank=0,
                         get=" + ".join("(Int64)arrIn0_%d[ix]" % k for k in range(12)), combine="x + y", seed="0")
    res = ctx.empty((), np.int64)
    total.fold([out], n, res)
    assert int(res.get()) == int(sum(int(g.astype(np.int64).sum()) for g in got))
    with pytest.raises(A.AccError) as e:                      # seventeen are too many
        ctx.skeleton(A.SKEL_MAP, ", ".join(["Int32"] * 17), env=[I32], out_rank=1, get="acc_elt{" + ", ".join(["0"] * 17) + "}")
    assert e.value.code == A.ERR_INVALID
