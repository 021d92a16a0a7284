"""Rank-3 stencils (and a rank-3 stencil2) through the C ABI, against numpy
index maps (tests/pyref.py, tap_arrays3).  Sources hold small integers, so every
Float32 operation is exact and results are compared bit for bit whatever order
the sums are taken in; one case with fractional data states its tolerance."""
import sys

import numpy as np
import pytest

import pyref

pytestmark = pytest.mark.gpu

F = np.float32
SEVEN = [(0, 0, 0), (-1, 0, 0), (1, 0, 0), (0, -1, 0), (0, 1, 0), (0, 0, -1), (0, 0, 1)]
BOX = [(dz, dy, dx) for dz in (-1, 0, 1) for dy in (-1, 0, 1) for dx in (-1, 0, 1)]
# (the last two are deeper than one walk through the planes: strips that continue one another, the last one short)
SHAPES = [(1, 1, 1), (3, 3, 3), (5, 7, 9), (3, 33, 70), (4, 64, 256), (6, 37, 517), (2, 16, 1024), (17, 40, 260),
          (70, 10, 260), (131, 5, 512)]


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


@pytest.mark.parametrize("mode", ["clamp", "mirror", "wrap", "constant"])
def test_stencil_3d(A, ctx, mode):
    rng = np.random.default_rng(31)
    lap = ctx.skeleton(A.SKEL_STENCIL, "float", out_rank=3, taps=SEVEN, boundary=mode, boundary_constant="2.0f",
                       stencil_fn="t1 + t2 + t3 + t4 + t5 + t6 - 6.0f * t0")
    box = ctx.skeleton(A.SKEL_STENCIL, "float", out_rank=3, taps=BOX, boundary=mode, boundary_constant="2.0f",
                       stencil_fn=" + ".join("(float)%d * t%d" % (k % 5 - 2, k) for k in range(27)))
    lap.prefetch(range(1, 6))                          # the shapes below take every variant: they compile side by side
    box.prefetch(range(1, 6))
    for shape in SHAPES:
        if mode == "mirror" and min(shape) < 2:
            continue                                   # the index maps assume the array spans the stencil
        say("stencil 3-D", mode, shape)
        v = rng.integers(-9, 9, shape).astype(F)
        dv, out = ctx.array(v), ctx.empty(shape, F)
        lap.stencil([], dv, out)
        t = pyref.tap_arrays3(v, SEVEN, mode, 2.0, shape)
        assert np.array_equal(out.get(), t[1] + t[2] + t[3] + t[4] + t[5] + t[6] - F(6) * t[0])
        box.stencil([], dv, out)
        t = pyref.tap_arrays3(v, BOX, mode, 2.0, shape)
        assert np.array_equal(out.get(), sum(F(k % 5 - 2) * t[k] for k in range(27)))
    say("stencil 3-D fractional data", mode)
    v = rng.random((9, 50, 300)).astype(F)
    out = ctx.empty(v.shape, F)
    lap.stencil([], ctx.array(v), out)
    t = pyref.tap_arrays3(v, SEVEN, mode, 2.0, v.shape)
    exp = ((((t[1] + t[2]) + t[3]) + t[4]) + t[5]) + t[6] - F(6) * t[0]
    assert np.max(np.abs(out.get() - exp)) <= 1e-5                 # in fact the same operations in the same order:
    assert np.array_equal(out.get(), exp)


@pytest.mark.parametrize("tune", ["stencil.strips_per_cu=0", "stencil.walk_min=16", "stencil.walk_min=2"])
def test_stencil_3d_walks_of_every_length(A, ctx, tuned, tune):
    """the driver shortens a strip's walk through the planes on volumes as small as these (to 4 planes); here the
    full walk of 64 planes and walks of 16 and of 2 are forced on them: strips that continue one another, the last
    one short, and the narrow last strip of a row that ends at the right edge"""
    tuned(tune)
    rng = np.random.default_rng(32)
    for mode in ("clamp", "wrap", "constant"):
        lap = ctx.skeleton(A.SKEL_STENCIL, "float", out_rank=3, taps=SEVEN, boundary=mode, boundary_constant="2.0f",
                           stencil_fn="t1 + t2 + t3 + t4 + t5 + t6 - 6.0f * t0")
        for shape in [(3, 33, 70), (6, 37, 517), (17, 40, 260), (70, 10, 260), (131, 5, 512), (67, 9, 700)]:
            say("stencil 3-D", tune, mode, shape)
            v = rng.integers(-9, 9, shape).astype(F)
            dv, out = ctx.array(v), ctx.empty(shape, F)
            lap.stencil([], dv, out)
            t = pyref.tap_arrays3(v, SEVEN, mode, 2.0, shape)
            assert np.array_equal(out.get(), t[1] + t[2] + t[3] + t[4] + t[5] + t[6] - F(6) * t[0])


def test_stencil2_3d_and_iteration(A, ctx):
    rng = np.random.default_rng(32)
    say("stencil2 3-D, sources of different extents")
    sk = ctx.skeleton(A.SKEL_STENCIL2, "float", out_rank=3, taps=[(-1, 0, 0), (1, 0, 0)], boundary="wrap",
                      taps2=[(0, 0, -1), (0, 0, 1), (0, -1, 0)], boundary2="constant", boundary2_constant="1.0f",
                      stencil_fn="(t1 - t0) * (u0 + u1 + u2)")
    a = rng.integers(-5, 5, (6, 40, 300)).astype(F)
    b = rng.integers(-5, 5, (5, 44, 260)).astype(F)
    shape = (5, 40, 260)
    out = ctx.empty(shape, F)
    sk.stencil2([], ctx.array(a), ctx.array(b), out)
    t = pyref.tap_arrays3(a, [(-1, 0, 0), (1, 0, 0)], "wrap", 0, shape)
    u = pyref.tap_arrays3(b, [(0, 0, -1), (0, 0, 1), (0, -1, 0)], "constant", 1.0, shape)
    assert np.array_equal(out.get(), (t[1] - t[0]) * (u[0] + u[1] + u[2]))
    say("3-D stencil iterated on the device")
    avg = ctx.skeleton(A.SKEL_STENCIL, "float", out_rank=3, taps=SEVEN, boundary="clamp",
                       stencil_fn="(t0 + t0 + t1 + t2 + t3 + t4 + t5 + t6) * 0.125f")
    v = (rng.integers(0, 4, (8, 32, 256)) * 8 ** 4).astype(F)      # multiples of 8^4: four halvings by 8 stay exact
    a_, b_ = ctx.array(v), ctx.empty(v.shape, F)
    res = avg.stencil_iterate([], a_, b_, 4).get()
    exp = v
    for _ in range(4):
        t = pyref.tap_arrays3(exp, SEVEN, "clamp", 0, v.shape)
        exp = (t[0] + t[0] + t[1] + t[2] + t[3] + t[4] + t[5] + t[6]) * F(0.125)
    assert np.array_equal(res, exp)


@pytest.mark.parametrize("case", ["wide in x", "two planes either side", "Float64", "within the plane"])
def test_stencil_3d_window_shapes(A, ctx, case):
    """Neighbourhoods of other reaches: how many planes of the result a strip produces at once follows the
    registers its window takes, so each of these runs a different tiling of the depth."""
    rng = np.random.default_rng(33)
    taps, ctype, T = SEVEN, "float", F
    if case == "wide in x":
        taps = SEVEN + [(0, 0, -2), (0, 0, 2)]
    elif case == "two planes either side":
        taps = SEVEN + [(-2, 0, 0), (2, 0, 0)]
    elif case == "Float64":
        ctype, T = "double", np.float64
    else:
        taps = [(0, dy, dx) for dy in (-1, 0, 1) for dx in (-1, 0, 1)]
    fn = " + ".join("(%s)%d * t%d" % (ctype, k % 7 - 3, k) for k in range(len(taps)))
    sk = ctx.skeleton(A.SKEL_STENCIL, ctype, out_rank=3, taps=taps, boundary="mirror", stencil_fn=fn)
    for shape in [(3, 3, 3), (5, 7, 9), (7, 19, 300), (8, 16, 512), (11, 33, 257)]:
        say("stencil 3-D", case, shape)
        v = rng.integers(-9, 9, shape).astype(T)
        out = ctx.empty(shape, T)
        sk.stencil([], ctx.array(v), out)
        t = pyref.tap_arrays3(v, taps, "mirror", 0, shape)
        assert np.array_equal(out.get(), sum(T(k % 7 - 3) * t[k] for k in range(len(taps))))


def test_stencil_3d_strip_edges_of_narrow_elements(A, ctx):
    """what a strip reads just outside its 256 columns comes from another lane's register: elements narrower than
    a register (Int8, Word16) at widths of several strips, first plane included, every boundary mode"""
    rng = np.random.default_rng(34)
    sks = {}
    for ctype, T in (("Int8", np.int8), ("Word16", np.uint16)):     # the eight instances compile side by side
        for mode in ("clamp", "mirror", "wrap", "constant"):
            sks[ctype, mode] = ctx.skeleton(A.SKEL_STENCIL, ctype, out_rank=3, taps=BOX, boundary=mode, boundary_constant="(%s)3" % ctype,
                                            stencil_fn="(%s)(%s)" % (ctype, " + ".join("t%d" % k for k in range(27)))).prefetch([1])
    for ctype, T in (("Int8", np.int8), ("Word16", np.uint16)):
        for mode in ("clamp", "mirror", "wrap", "constant"):
            sk = sks[ctype, mode]
            for shape in ((2, 4, 256), (4, 9, 1031), (66, 6, 512)):
                say("stencil 3-D", ctype, mode, shape)
                v = rng.integers(0, 4, shape).astype(T)
                out = ctx.empty(shape, T)
                sk.stencil([], ctx.array(v), out)
                t = pyref.tap_arrays3(v, BOX, mode, 3, shape)
                assert np.array_equal(out.get(), sum(a.astype(np.int64) for a in t).astype(T))
