"""Stencils beyond what the strips of rows in registers take: arrays of rank 4 and more, taps further than 2 planes or
4 rows or columns away (CodeGen/Stencil.hs:55-114 serves every rank and every offset of the stencil patterns through
cfromIndex, Base.hs:207-218).  Checked against tests/pyref.py's index maps (Stencil/Extra.hs:198-226), and, where
both templates take a stencil, against each other."""
import itertools
import sys

import numpy as np
import pytest

import pyref

pytestmark = pytest.mark.gpu

MODES = ("clamp", "mirror", "wrap", "constant")


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


def test_rank_4_stencil_3x3x3x3(A, ctx):
    """all 81 neighbours in four dimensions, every boundary mode; integer weights, so the sums are exact in Float32"""
    rng = np.random.default_rng(4)
    taps = list(itertools.product((-1, 0, 1), repeat=4))
    coef = [int(rng.integers(-2, 3)) for _ in taps]
    fn = " + ".join("(float)(%d) * t%d" % (c, k) for k, c in enumerate(coef))
    sks = {m: ctx.skeleton(A.SKEL_STENCIL, "float", out_rank=4, taps=taps, boundary=m, boundary_constant="3.0f", stencil_fn=fn) for m in MODES}
    for mode in MODES:
        for shape in ((2, 3, 4, 5), (5, 4, 7, 66), (3, 2, 9, 257)):
            say("rank-4 stencil", mode, shape)
            v = rng.integers(-4, 5, shape).astype(np.float32)
            out = ctx.empty(shape, np.float32)
            sks[mode].stencil([], ctx.array(v), out)
            t = pyref.tap_arrays_nd(v, taps, mode, 3.0)
            ref = sum(np.float32(c) * a for c, a in zip(coef, t)).astype(np.float32)
            assert np.array_equal(out.get(), ref), (mode, shape)


def test_nine_planes_in_three_dimensions(A, ctx):
    """a 3-D stencil that reaches four planes either way (and four rows, four columns): the widest pattern of the array
    language along every axis"""
    rng = np.random.default_rng(5)
    taps = [(dz, 0, 0) for dz in range(-4, 5)] + [(0, dy, 0) for dy in (-4, -3, 3, 4)] + [(0, 0, dx) for dx in (-4, 4)] + [(-3, 2, -1), (4, -4, 4)]
    coef = [int(rng.integers(1, 4)) for _ in taps]
    for ctype, T in (("double", np.float64), ("Int16", np.int16)):
        fn = "(%s)(%s)" % (ctype, " + ".join("(%s)(%d) * t%d" % (ctype, c, k) for k, c in enumerate(coef)))
        sks = {m: ctx.skeleton(A.SKEL_STENCIL, ctype, out_rank=3, taps=taps, boundary=m, boundary_constant="(%s)2" % ctype, stencil_fn=fn) for m in MODES}
        for mode in MODES:
            for shape in ((5, 5, 5), (9, 6, 70), (12, 33, 131)):
                say("nine planes", ctype, mode, shape)
                v = rng.integers(0, 4, shape).astype(T)
                out = ctx.empty(shape, T)
                sks[mode].stencil([], ctx.array(v), out)
                t = pyref.tap_arrays_nd(v, taps, mode, 2)
                ref = sum(np.int64(c) * a.astype(np.int64) for c, a in zip(coef, t)).astype(T)
                assert np.array_equal(out.get(), ref), (ctype, mode, shape)


def test_both_templates_agree_where_both_apply(A, ctx):
    """a 2-D and a 3-D stencil within the strips' reach, run through the strips and (knob stencil.nd=1) an element a
    thread: the same bits, fractional data included"""
    rng = np.random.default_rng(6)
    five = [(-1, 0), (0, -1), (0, 0), (0, 1), (1, 0)]
    seven = [(0, 0, 0), (-1, 0, 0), (1, 0, 0), (0, -1, 0), (0, 1, 0), (0, 0, -1), (0, 0, 1)]
    for rank, taps, shape in ((2, five, (70, 300)), (3, seven, (6, 20, 131))):
        fn = " + ".join("(0.%df * t%d)" % (k + 1, k) for k in range(len(taps)))
        for mode in MODES:
            say("strips against an element a thread", rank, mode)
            strips = ctx.skeleton(A.SKEL_STENCIL, "float", out_rank=rank, taps=taps, boundary=mode, boundary_constant="0.5f", stencil_fn=fn)
            with A.tuning("stencil.nd=1", ctx):
                each = ctx.skeleton(A.SKEL_STENCIL, "float", out_rank=rank, taps=taps, boundary=mode, boundary_constant="0.5f", stencil_fn=fn)
            assert "skel_stencil_nd.h" in each.source() and "skel_stencil_nd.h" not in strips.source()
            v = rng.random(shape).astype(np.float32)
            dv, o1, o2 = ctx.array(v), ctx.empty(shape, np.float32), ctx.empty(shape, np.float32)
            strips.stencil([], dv, o1)
            each.stencil([], dv, o2)
            assert np.array_equal(o1.get(), o2.get())


def test_stencil2_of_rank_4_with_tuples(A, ctx):
    """two sources of different extents, the second one of pairs, a result of pairs; each source its own boundary"""
    rng = np.random.default_rng(7)
    t1 = [(0, 0, 0, 0), (1, 0, 0, -1), (0, -1, 2, 0)]
    t2 = [(0, 0, 0, 0), (0, -2, 0, 3)]
    sk = ctx.skeleton(A.SKEL_STENCIL2, "float, Int32", out_rank=4, taps=t1, taps2=t2, boundary="wrap", boundary2="constant",
                      boundary2_constant="7, -1", stencil_in="float", stencil_in2="Int32, Int32",
                      stencil_fn="acc_elt{t0 + 2.0f * t1 - t2, u0.a1 + u1.a0}")
    s1, s2 = (3, 4, 5, 40), (4, 3, 6, 37)
    shape = tuple(min(a, b) for a, b in zip(s1, s2))
    a = rng.integers(-5, 6, s1).astype(np.float32)
    b1, b0 = rng.integers(-5, 6, s2).astype(np.int32), rng.integers(-5, 6, s2).astype(np.int32)
    out = ctx.empty_tuple(shape, [np.float32, np.int32])
    sk.stencil2([], ctx.array(a), ctx.tuple_array(b1, b0), out)
    cut = tuple(slice(0, n) for n in shape)
    ta = [x[cut] for x in pyref.tap_arrays_nd(a, t1, "wrap", 0)]
    tb1 = [x[cut] for x in pyref.tap_arrays_nd(b1, t2, "constant", 7)]
    tb0 = [x[cut] for x in pyref.tap_arrays_nd(b0, t2, "constant", -1)]
    got = out.get()
    assert np.array_equal(got[0], ta[0] + np.float32(2) * ta[1] - ta[2])
    assert np.array_equal(got[1], tb1[0] + tb0[1])
