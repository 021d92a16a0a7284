"""Pins the CPU oracle (oracle/acc_oracle.c) by means independent of it.

The reference holds no tests, fixtures or golden vectors (its cabal file has a
Library stanza only), so the pins are: the doc-comment vectors the reference
does hold (CodeGen/PrefixSum.hs:149-166), numpy / scipy routines, closed
forms, algebraic identities and a pure-Python brute force (tests/pyref.py).
"""
import json
import os

import numpy as np
import pytest
import scipy.ndimage as ndi
import scipy.sparse as sp

import pyref

GOLDEN = os.path.join(os.path.dirname(__file__), "golden")
rng = np.random.default_rng(20251125)


def as_u32(a):
    return np.asarray(a, dtype=np.int32).view(np.uint32)


# --------------------------------------------------------------------------- scans

def test_scan_doc_vectors(orc):
    """The three worked examples in the reference: PrefixSum.hs:149-166."""
    ones = np.ones(10, dtype=np.int32)
    assert orc.scan("scanl", orc.OP_ADD, ones, seed=10).tolist() == list(range(10, 21))
    assert orc.scan("scanl1", orc.OP_ADD, ones).tolist() == list(range(1, 11))
    body, total = orc.scan("scanl'", orc.OP_ADD, ones, seed=10)
    full = orc.scan("scanl", orc.OP_ADD, ones, seed=10)
    assert body.tolist() == full[:-1].tolist() and total == full[-1]   # PrefixSum.hs:176-180


@pytest.mark.parametrize("n", [0, 1, 2, 63, 64, 65, 1000, 4097])
def test_scan_add_vs_numpy(orc, n):
    x = rng.integers(0, 16, n, dtype=np.int32)
    cs = np.cumsum(x, dtype=np.int32)
    assert np.array_equal(orc.scan("scanl1", orc.OP_ADD, x), cs)
    assert np.array_equal(orc.scan("scanl", orc.OP_ADD, x, seed=7), np.concatenate([[7], cs + 7]).astype(np.int32))
    rcs = np.cumsum(x[::-1], dtype=np.int32)[::-1]
    assert np.array_equal(orc.scan("scanr1", orc.OP_ADD, x), rcs)
    assert np.array_equal(orc.scan("scanr", orc.OP_ADD, x, seed=7), np.concatenate([rcs + 7, [7]]).astype(np.int32))
    body, tot = orc.scan("scanr'", orc.OP_ADD, x, seed=3)
    full = orc.scan("scanr", orc.OP_ADD, x, seed=3)
    assert np.array_equal(body, full[1:]) and tot == full[0]


def test_scan_wraps_like_int32(orc):
    x = np.full(5, 2**30, dtype=np.int32)
    expect = np.cumsum(x.astype(np.int64)).astype(np.int64)
    expect = ((expect + 2**31) % 2**32 - 2**31).astype(np.int32)
    assert np.array_equal(orc.scan("scanl1", orc.OP_ADD, x), expect)


@pytest.mark.parametrize("n", [0, 1, 5, 17])
def test_scan_noncommutative_vs_bruteforce(orc, n):
    """affine-map composition is associative but not commutative: pins the
    operand order of every variant (a swapped operand fails here)."""
    x = rng.integers(0, 2**32, n, dtype=np.uint32).view(np.int32)
    xs = [int(v) for v in as_u32(x)]
    z = 0x00030005
    f = pyref.affine16
    assert as_u32(orc.scan("scanl", orc.OP_AFFINE16, x, seed=z)).tolist() == pyref.scanl(f, z, xs)
    assert as_u32(orc.scan("scanl1", orc.OP_AFFINE16, x)).tolist() == pyref.scanl1(f, xs)
    assert as_u32(orc.scan("scanr", orc.OP_AFFINE16, x, seed=z)).tolist() == pyref.scanr(f, z, xs)
    assert as_u32(orc.scan("scanr1", orc.OP_AFFINE16, x)).tolist() == pyref.scanr1(f, xs)
    b, t = orc.scan("scanl'", orc.OP_AFFINE16, x, seed=z)
    pb, pt = pyref.scanl_p(f, z, xs)
    assert as_u32(b).tolist() == pb and int(as_u32([t])[0]) == pt
    b, t = orc.scan("scanr'", orc.OP_AFFINE16, x, seed=z)
    pb, pt = pyref.scanr_p(f, z, xs)
    assert as_u32(b).tolist() == pb and int(as_u32([t])[0]) == pt


def test_scan_identities(orc):
    x = rng.integers(-50, 50, 777, dtype=np.int32)
    l = orc.scan("scanl", orc.OP_ADD, x, seed=0)
    assert np.array_equal(l[1:], orc.scan("scanl1", orc.OP_ADD, x))            # scanl1 = tail . scanl, z identity
    assert l[-1] == orc.fold(orc.OP_ADD, x, seed=0)                            # last . scanl = fold
    r = orc.scan("scanr", orc.OP_ADD, x, seed=0)
    assert np.array_equal(r, orc.scan("scanl", orc.OP_ADD, x[::-1], seed=0)[::-1])  # scanr = reverse . scanl . reverse
    m = orc.scan("scanl1", orc.OP_MAX, x)
    assert np.array_equal(m, np.maximum.accumulate(x))
    assert np.array_equal(orc.scan("scanl1", orc.OP_MIN, x), np.minimum.accumulate(x))


def test_scan_empty(orc):
    e = np.zeros(0, dtype=np.int32)
    assert orc.scan("scanl", orc.OP_ADD, e, seed=9).tolist() == [9]            # PrefixSum.hs:249-251,330-334
    assert orc.scan("scanr", orc.OP_ADD, e, seed=9).tolist() == [9]
    assert orc.scan("scanl1", orc.OP_ADD, e).size == 0
    b, t = orc.scan("scanl'", orc.OP_ADD, e, seed=4)
    assert b.size == 0 and t == 4


def test_scan_f32_sequential_rounding(orc):
    x = rng.random(1000).astype(np.float32)
    acc = np.float32(0)
    exp = []
    for v in x:
        acc = np.float32(acc + v)
        exp.append(acc)
    assert np.array_equal(orc.scan("scanl1", orc.OP_ADD, x), np.array(exp, dtype=np.float32))


# --------------------------------------------------------------------------- folds

def test_fold_seed_and_empty(orc):
    e = np.zeros(0, dtype=np.int32)
    assert orc.fold(orc.OP_ADD, e, seed=42) == 42                              # Reduction.hs:212-214
    with pytest.raises(orc.OracleError):                                       # Execute.hs:282-285
        orc.fold(orc.OP_ADD, e)
    x = np.array([5], dtype=np.int32)
    assert orc.fold(orc.OP_ADD, x, seed=10) == 15
    assert orc.fold(orc.OP_ADD, x) == 5


def test_fold_dim_vs_numpy(orc):
    x = rng.integers(-100, 100, (7, 13, 31), dtype=np.int32)
    assert np.array_equal(orc.fold(orc.OP_ADD, x, seed=0), x.sum(axis=-1, dtype=np.int32))
    assert np.array_equal(orc.fold(orc.OP_MAX, x), x.max(axis=-1))
    assert np.array_equal(orc.fold(orc.OP_MIN, x), x.min(axis=-1))
    # empty innermost dimension: every output is the seed (Reduction.hs:351-362)
    z = np.zeros((3, 0), dtype=np.int32)
    assert orc.fold(orc.OP_ADD, z, seed=5).tolist() == [5, 5, 5]


def test_fold_direction_and_seed_position(orc):
    """FIRST/LAST expose where the seed and the ends go.
    left : ((x0.x1)...x_{n-1}).z     right: x0.(x1.(...(x_{n-1}.z)))"""
    x = np.array([10, 20, 30], dtype=np.int32)
    xs = x.tolist()
    for op, f in ((orc.OP_FIRST, lambda a, b: a), (orc.OP_LAST, lambda a, b: b)):
        assert orc.fold(op, x, seed=99, direction=orc.DIR_LEFT) == pyref.fold_left(f, 99, xs)
        assert orc.fold(op, x, seed=99, direction=orc.DIR_RIGHT) == pyref.fold_right(f, 99, xs)
    u = rng.integers(0, 2**32, 9, dtype=np.uint32).view(np.int32)
    us = [int(v) for v in as_u32(u)]
    z = 0x00070001
    for d, pf in ((orc.DIR_LEFT, pyref.fold_left), (orc.DIR_RIGHT, pyref.fold_right)):
        got = int(as_u32([orc.fold(orc.OP_AFFINE16, u, seed=z, direction=d)])[0])
        assert got == pf(pyref.affine16, z, us)     # associativity makes both equal, too
    assert pyref.fold_left(pyref.affine16, z, us) == pyref.fold_right(pyref.affine16, z, us)


def test_fold_f32_rounding_order(orc):
    x = (rng.random(4096) * 2 - 1).astype(np.float32)
    acc = np.float32(x[0])
    for v in x[1:]:
        acc = np.float32(acc + v)
    acc = np.float32(acc + np.float32(0))
    assert orc.fold(orc.OP_ADD, x, seed=0.0, direction=orc.DIR_LEFT) == acc
    acc = np.float32(0)
    for v in x[::-1]:
        acc = np.float32(v + acc)
    assert orc.fold(orc.OP_ADD, x, seed=0.0, direction=orc.DIR_RIGHT) == acc


def test_dot_against_float64_and_exact_inputs(orc):
    n = 50000
    x = (rng.random(n) * 2 - 1).astype(np.float32)
    y = (rng.random(n) * 2 - 1).astype(np.float32)
    truth = float(np.dot(x.astype(np.float64), y.astype(np.float64)))
    assert abs(orc.dot_f64(x, y) - truth) <= 1e-9 * max(1.0, abs(truth))
    bound = 2 * n * 2.0 ** -24 * orc.dot_abs_f64(x, y)          # classic recursive-summation bound
    for d in (orc.DIR_LEFT, orc.DIR_RIGHT):
        assert abs(float(orc.dot_f32(x, y, d)) - truth) <= bound
    # products rounded separately: equals fold over the rounded products
    prod = (x * y).astype(np.float32)
    assert orc.dot_f32(x, y, orc.DIR_LEFT) == orc.fold(orc.OP_ADD, prod, seed=0.0, direction=orc.DIR_LEFT)
    assert orc.dot_f32(x, y, orc.DIR_RIGHT) == orc.fold(orc.OP_ADD, prod, seed=0.0, direction=orc.DIR_RIGHT)
    # small integers: every order is exact, so all agree bit for bit
    xi = rng.integers(-8, 8, n).astype(np.float32)
    yi = rng.integers(-8, 8, n).astype(np.float32)
    exact = float(np.dot(xi.astype(np.int64), yi.astype(np.int64)))
    assert float(orc.dot_f32(xi, yi, orc.DIR_LEFT)) == exact == float(orc.dot_f32(xi, yi, orc.DIR_RIGHT))
    assert orc.dot_f32(x[:0], y[:0]) == 0.0


# --------------------------------------------------------------------------- foldSeg / SMVM

def _csr(nrows, ncols, mean, integer=False):
    lens = rng.poisson(mean, nrows).astype(np.int32)
    lens[rng.integers(0, nrows, max(1, nrows // 10))] = 0          # force empty rows
    offs = np.concatenate([[0], np.cumsum(lens)]).astype(np.int32)
    nnz = int(offs[-1])
    cols = rng.integers(0, ncols, nnz, dtype=np.int32)
    if integer:
        vals = rng.integers(-4, 5, nnz).astype(np.float32)
        x = rng.integers(-4, 5, ncols).astype(np.float32)
    else:
        vals = (rng.random(nnz) * 2 - 1).astype(np.float32)
        x = (rng.random(ncols) * 2 - 1).astype(np.float32)
    return vals, cols, offs, x


def test_zipwith_mul_rounds_every_product_to_float32(orc):
    rng = np.random.default_rng(33)
    x = (rng.standard_normal(10007) * 1e3).astype(np.float32)
    y = (rng.standard_normal(10007) * 1e-3).astype(np.float32)
    got = orc.zipwith_mul_f32(x, y)
    assert np.array_equal(got, x * y)                                         # numpy multiplies in Float32 as well
    assert np.array_equal(got, (x.astype(np.float64) * y.astype(np.float64)).astype(np.float32))   # = the rounded exact product
    assert orc.zipwith_mul_f32(x[:0], y[:0]).size == 0


def test_foldseg_vs_numpy_and_empty_segments(orc):
    vals, _, offs, _ = _csr(200, 50, 8, integer=True)
    vi = vals.astype(np.int32)
    exp = np.array([vi[offs[s]:offs[s + 1]].sum() + 3 for s in range(200)], dtype=np.int32)
    got = orc.foldseg(orc.OP_ADD, vi, offs, seed=3)
    assert np.array_equal(got, exp)
    empty = np.diff(offs) == 0
    assert empty.any() and np.all(got[empty] == 3)                            # Reduction.hs:567-574
    with pytest.raises(orc.OracleError):                                      # fold1Seg of an empty segment
        orc.foldseg(orc.OP_ADD, vi, offs)
    ps = pyref.foldseg(pyref.fold_left, lambda a, b: max(a, b), -999, vi.tolist(), offs.tolist())
    assert orc.foldseg(orc.OP_MAX, vi, offs, seed=-999).tolist() == ps


def test_foldseg_of_higher_rank_restarts_in_every_row(orc):
    """Reduction.hs:473-474: the descriptor cuts the innermost dimension of every outer row alike; pinned by numpy
    slicing per row (not by the oracle's own index arithmetic), a row tail that belongs to no segment, empty
    segments, a non-commutative operator against pure Python, and the rank-1 case against foldseg itself"""
    rng = np.random.default_rng(21)
    lens = np.array([3, 0, 5, 1, 0, 4], np.int32)
    offs = np.concatenate([[0], np.cumsum(lens)]).astype(np.int32)            # 13 of the 16 elements of a row
    x = rng.integers(-50, 50, (4, 3, 16)).astype(np.int32)
    got = orc.foldseg_nd(orc.OP_ADD, x, offs, seed=7)
    assert got.shape == (4, 3, 6)
    for i in range(4):
        for j in range(3):
            for s_ in range(6):
                assert got[i, j, s_] == x[i, j, offs[s_]:offs[s_ + 1]].sum() + 7
    # the tail x[..., 13:] reaches no result: changing it changes nothing
    y = x.copy()
    y[..., 13:] += 1000
    assert np.array_equal(orc.foldseg_nd(orc.OP_ADD, y, offs, seed=7), got)
    # segments of length 1 over the whole row without a seed: the array itself
    ones = np.arange(17, dtype=np.int32)
    assert np.array_equal(orc.foldseg_nd(orc.OP_ADD, x, ones), x)
    # a non-commutative operator: `first` keeps the segment's first element (the seed comes second), `last` the seed
    xf = rng.random((5, 16)).astype(np.float32)
    first = orc.foldseg_nd(orc.OP_FIRST, xf, offs, seed=-1.0)
    last = orc.foldseg_nd(orc.OP_LAST, xf, offs, seed=-1.0)
    for r in range(5):
        for s_ in range(6):
            assert first[r, s_] == (xf[r, offs[s_]] if lens[s_] else np.float32(-1.0))
            assert last[r, s_] == np.float32(-1.0)
    # composition of affine maps over Z/2^16 (associative, not commutative) against pure Python, both directions
    xa = rng.integers(0, 1 << 31, (3, 16)).astype(np.int32)
    z = int((5 << 16) | 9)
    for d, pf in ((orc.DIR_LEFT, pyref.fold_left), (orc.DIR_RIGHT, pyref.fold_right)):
        ps = [pyref.foldseg(pf, pyref.affine16, z, row.tolist(), offs.tolist()) for row in xa]
        got = orc.foldseg_nd(orc.OP_AFFINE16, xa, offs, seed=z, direction=d)
        assert (got.astype(np.int64) & 0xFFFFFFFF).tolist() == ps             # the same 32 bits, read as unsigned
    # rank 1 is foldseg
    v = x.reshape(-1)[:16]
    assert np.array_equal(orc.foldseg_nd(orc.OP_MAX, v, offs, seed=-999), orc.foldseg(orc.OP_MAX, v, offs, seed=-999))
    with pytest.raises(orc.OracleError):                                      # fold1Seg: an empty segment in some row
        orc.foldseg_nd(orc.OP_ADD, x, offs)
    with pytest.raises(orc.OracleError):                                      # a descriptor that runs past the row
        orc.foldseg_nd(orc.OP_ADD, x[..., :12], offs, seed=0)


def test_smvm_vs_scipy(orc):
    nrows, ncols = 300, 128
    vals, cols, offs, x = _csr(nrows, ncols, 12)
    A = sp.csr_matrix((vals.astype(np.float64), cols, offs), shape=(nrows, ncols))
    truth = A @ x.astype(np.float64)
    y64, yabs = orc.smvm_f64(vals, cols, offs, x)
    assert np.allclose(y64, truth, rtol=1e-12, atol=1e-12)
    for d in (orc.DIR_LEFT, orc.DIR_RIGHT):
        y = orc.smvm_f32(vals, cols, offs, x, d)
        assert np.all(np.abs(y - truth) <= 40 * 2.0 ** -24 * yabs + 1e-30)
        # composition law: smvm == foldSeg (+) 0 (zipWith (*) vals (gather x cols))
        prod = (vals * orc.backpermute(x, cols)).astype(np.float32)
        assert np.array_equal(y, orc.foldseg(orc.OP_ADD, prod, offs, seed=0.0, direction=d))
    assert np.all(orc.smvm_f32(vals, cols, offs, x)[np.diff(offs) == 0] == 0.0)
    # integer-valued matrix: exact in every order
    vals, cols, offs, x = _csr(nrows, ncols, 12, integer=True)
    A = sp.csr_matrix((vals.astype(np.float64), cols, offs), shape=(nrows, ncols))
    assert np.array_equal(orc.smvm_f32(vals, cols, offs, x).astype(np.float64), A @ x.astype(np.float64))


# --------------------------------------------------------------------------- permute

def test_permute_histogram_vs_bincount(orc):
    keys = rng.integers(0, 256, 100000, dtype=np.int32)
    zeros = np.zeros(256, dtype=np.int32)
    h = orc.permute(orc.OP_ADD, zeros, keys)
    assert np.array_equal(h, np.bincount(keys, minlength=256).astype(np.int32))
    assert h.sum() == keys.size
    # defaults are added in; ignored elements are dropped (IndexSpace.hs:150-151,226-233)
    dfl = rng.integers(0, 10, 256, dtype=np.int32)
    k2 = keys.copy()
    k2[::7] = -1
    h2 = orc.permute(orc.OP_ADD, dfl, k2)
    assert np.array_equal(h2, dfl + np.bincount(k2[k2 >= 0], minlength=256).astype(np.int32))
    assert h2.sum() - dfl.sum() == (k2 >= 0).sum()
    # weighted
    wts = rng.integers(-5, 6, keys.size, dtype=np.int32)
    h3 = orc.permute(orc.OP_ADD, zeros, keys, wts)
    assert np.array_equal(h3, np.bincount(keys, weights=wts, minlength=256).astype(np.int32))


def test_permute_argument_order(orc):
    """combine new old (IndexSpace.hs:207): FIRST keeps the last-arriving source
    value, LAST keeps the default."""
    dfl = np.array([100, 200, 300], dtype=np.int32)
    dst = np.array([2, 0, 2, -1, 0], dtype=np.int32)
    src = np.array([1, 2, 3, 4, 5], dtype=np.int32)
    assert orc.permute(orc.OP_FIRST, dfl, dst, src).tolist() == [5, 200, 3]
    assert orc.permute(orc.OP_LAST, dfl, dst, src).tolist() == [100, 200, 300]
    f = pyref.affine16
    d = [7, 8, 9]
    s = [0x00020003, 0x00050001, 0x00030004, 0x00010001, 0x00020002]
    got = orc.permute(orc.OP_AFFINE16, np.array(d, dtype=np.int32), dst, np.array(s, dtype=np.int32))
    assert as_u32(got).tolist() == pyref.permute(f, d, dst.tolist(), s)


def test_backpermute_vs_fancy_indexing(orc):
    a = rng.random(1000).astype(np.float32)
    idx = rng.integers(0, 1000, 5000, dtype=np.int32)
    assert np.array_equal(orc.backpermute(a, idx), a[idx])


# --------------------------------------------------------------------------- stencil

def test_boundary_maps_match_reference_formulas(orc):
    """Stencil/Extra.hs:198-226, spelt out value by value."""
    sz = 5
    assert [orc.boundary_index("clamp", i, sz) for i in range(-2, 8)] == [0, 0, 0, 1, 2, 3, 4, 4, 4, 4]
    assert [orc.boundary_index("mirror", i, sz) for i in range(-2, 7)] == [2, 1, 0, 1, 2, 3, 4, 3, 2]
    assert [orc.boundary_index("wrap", i, sz) for i in range(-2, 7)] == [3, 4, 0, 1, 2, 3, 4, 0, 1]
    for mode in ("clamp", "mirror", "wrap"):
        for i in range(-3, 9):
            assert orc.boundary_index(mode, i, 6) == pyref.bmap(mode, i, 6)


SCIPY_MODE = {"clamp": "nearest", "mirror": "mirror", "wrap": "wrap", "constant": "constant"}


@pytest.mark.parametrize("mode", ["clamp", "mirror", "wrap", "constant"])
@pytest.mark.parametrize("shape", [(5, 5), (7, 3), (33, 70), (3, 64)])
def test_stencil_vs_scipy(orc, mode, shape):
    img = rng.random(shape).astype(np.float32)
    for taps, div in ((orc.GAUSS3X3, 16.0), (orc.LAPLACE5, 1.0)):
        k = np.zeros((3, 3))
        for dy, dx, c in taps:
            k[dy + 1, dx + 1] = c
        truth = ndi.correlate(img.astype(np.float64), k / div, mode=SCIPY_MODE[mode], cval=0.25)
        got = orc.stencil2d(img, taps, divisor=div, mode=mode, constant=0.25)
        assert np.max(np.abs(got - truth)) <= 2e-6


def test_stencil_asymmetric_taps_vs_bruteforce(orc):
    """offsets that are not symmetric catch a transposed dy/dx or a flipped sign."""
    img = rng.integers(0, 50, (6, 9)).astype(np.float32)
    taps = [(-1, 1, 3.0), (0, -1, -2.0), (1, 0, 5.0)]
    offs = [(t[0], t[1]) for t in taps]
    fn = lambda t: 3.0 * t[0] - 2.0 * t[1] + 5.0 * t[2]
    for mode in ("clamp", "mirror", "wrap", "constant"):
        exp = pyref.stencil2d(fn, img.tolist(), offs, mode, constant=7.0)
        got = orc.stencil2d(img, taps, mode=mode, constant=7.0)
        assert np.array_equal(got, np.array(exp, dtype=np.float32)), mode


def test_stencil_fixed_points(orc):
    const = np.full((17, 23), 0.375, dtype=np.float32)
    for mode in ("clamp", "mirror", "wrap"):
        assert np.array_equal(orc.stencil2d(const, orc.GAUSS3X3, divisor=16.0, mode=mode, iters=3), const)
    yy, xx = np.mgrid[0:16, 0:20]
    ramp = (2 * yy + 3 * xx).astype(np.float32)
    lap = orc.stencil2d(ramp, orc.LAPLACE5, mode="mirror")
    assert np.all(lap[1:-1, 1:-1] == 0)           # Laplacian of an affine ramp vanishes inside
    # iterating k times equals applying once k times
    img = rng.random((12, 12)).astype(np.float32)
    a = img
    for _ in range(4):
        a = orc.stencil2d(a, orc.GAUSS3X3, divisor=16.0, mode="clamp")
    assert np.array_equal(a, orc.stencil2d(img, orc.GAUSS3X3, divisor=16.0, mode="clamp", iters=4))
    assert np.array_equal(img, orc.stencil2d(img, orc.GAUSS3X3, divisor=16.0, iters=0))


def test_stencil1d_vs_scipy(orc):
    v = rng.random(50).astype(np.float32)
    taps = [(-1, 1.0), (0, -2.0), (1, 1.0)]
    for mode in ("clamp", "mirror", "wrap", "constant"):
        truth = ndi.correlate1d(v.astype(np.float64), [1.0, -2.0, 1.0], mode=SCIPY_MODE[mode], cval=0.5)
        assert np.max(np.abs(orc.stencil1d(v, taps, mode=mode, constant=0.5) - truth)) <= 1e-6


# --------------------------------------------------------------------------- committed fixtures

def test_golden_fixtures(orc):
    """Small vectors written by tests/golden/make_golden.py from numpy / scipy
    (not from the oracle), committed so that the GPU box checks the same data."""
    with open(os.path.join(GOLDEN, "golden.json")) as fh:
        g = json.load(fh)
    x = np.array(g["scan"]["x"], dtype=np.int32)
    assert orc.scan("scanl", orc.OP_ADD, x, seed=g["scan"]["seed"]).tolist() == g["scan"]["scanl"]
    assert orc.scan("scanl1", orc.OP_ADD, x).tolist() == g["scan"]["scanl1"]
    assert orc.scan("scanr", orc.OP_ADD, x, seed=g["scan"]["seed"]).tolist() == g["scan"]["scanr"]
    keys = np.array(g["hist"]["keys"], dtype=np.int32)
    assert orc.permute(orc.OP_ADD, np.zeros(g["hist"]["bins"], dtype=np.int32), keys).tolist() == g["hist"]["counts"]
    img = np.array(g["stencil"]["img"], dtype=np.float32)
    for mode in ("clamp", "mirror", "wrap", "constant"):
        got = orc.stencil2d(img, orc.GAUSS3X3, divisor=16.0, mode=mode, constant=g["stencil"]["constant"])
        assert np.max(np.abs(got - np.array(g["stencil"]["gauss_" + mode]))) <= 1e-6
        got = orc.stencil2d(img, orc.LAPLACE5, mode=mode, constant=g["stencil"]["constant"])
        assert np.max(np.abs(got - np.array(g["stencil"]["laplace_" + mode]))) <= 2e-6
    s = g["smvm"]
    y = orc.smvm_f32(s["vals"], s["cols"], s["offsets"], s["x"])
    assert np.max(np.abs(y - np.array(s["y"]))) <= 1e-5
    d = g["dot"]
    assert abs(float(orc.dot_f32(d["x"], d["y"])) - d["dot"]) <= 1e-4 * abs(d["dot"])


def test_workload_generators_are_reproducible():
    import workloads as wl
    a = wl.uniform_pm1_f32(123, 1000)
    assert np.array_equal(a[100:200], wl.uniform_pm1_f32(123, 200)[100:200])
    assert a.min() >= -1 and a.max() < 1
    # SplitMix64 known answers for seed 0 (first outputs of the published generator)
    r = wl.splitmix64(0, 3)
    assert [hex(int(v)) for v in r] == ["0xe220a8397b1dcdaf", "0x6e789e6aa1b965f4", "0x6c45d188009454f"]
    k = wl.uniform_i32(5, 100000, 16)
    assert k.min() == 0 and k.max() == 15 and abs(k.mean() - 7.5) < 0.1
    z = wl.zipf_i32(7, 200000, 65536)
    c = np.bincount(z, minlength=65536)
    assert c[0] == c.max() and 0.10 < c[0] / z.size < 0.17        # p(rank 1) ~ 0.137 for s = 1.1
    p = wl.poisson_i32(9, 200000, 32)
    assert abs(p.mean() - 32) < 0.1 and abs(p.var() - 32) < 0.6
