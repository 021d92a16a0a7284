"""stencil2 (two sources, Stencil.hs:118-237) through the C ABI.

Expected values come from numpy: each tap is the source array indexed through
the boundary's index map at the SOURCE's own edges (tests/pyref.py,
tap_arrays), and the stencil function is evaluated in Float32 in the order the
fragment spells it; contraction is off on the device, so results are compared
bit for bit.
"""
import sys

import numpy as np
import pytest

import pyref

pytestmark = pytest.mark.gpu

LAP = [(-1, 0), (0, -1), (0, 0), (0, 1), (1, 0)]
BOX3 = [(dy, dx) for dy in (-1, 0, 1) for dx in (-1, 0, 1)]


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


F = np.float32


def lap_times_box(t, u):
    """(laplacian of a) * (mean-ish of b), as the fragment below computes it"""
    lap = (((t[0] + t[1]) - F(4) * t[2]) + t[3]) + t[4]
    box = u[0]
    for k in range(1, 9):
        box = box + u[k]
    return lap * (box * F(0.125))


FRAG = "((((t0 + t1) - 4.0f * t2) + t3) + t4) * ((u0 + u1 + u2 + u3 + u4 + u5 + u6 + u7 + u8) * 0.125f)"


@pytest.mark.parametrize("mode1,mode2", [("clamp", "clamp"), ("mirror", "wrap"), ("constant", "clamp"), ("wrap", "constant")])
def test_stencil2_2d(A, ctx, mode1, mode2):
    rng = np.random.default_rng(21)
    sk = ctx.skeleton(A.SKEL_STENCIL2, "float", out_rank=2, taps=LAP, boundary=mode1, boundary_constant="0.5f",
                      taps2=BOX3, boundary2=mode2, boundary2_constant="-1.0f", stencil_fn=FRAG)
    # same extents, and extents that differ in one or both dimensions: the result covers the intersection
    for s1, s2 in [((5, 5), (5, 5)), ((33, 70), (33, 70)), ((64, 256), (64, 256)), ((300, 517), (300, 517)),
                   ((40, 300), (37, 300)), ((64, 512), (64, 260)), ((129, 1030), (140, 1024)), ((512, 1024), (512, 1024))]:
        say("stencil2", mode1, mode2, s1, s2)
        a = rng.integers(-8, 8, s1).astype(F)          # small integers: every Float32 operation is exact,
        b = rng.integers(-8, 8, s2).astype(F)          # so the association the compiler keeps cannot matter either
        shape = (min(s1[0], s2[0]), min(s1[1], s2[1]))
        out = ctx.empty(shape, F)
        sk.stencil2([], ctx.array(a), ctx.array(b), out)
        t = pyref.tap_arrays(a, LAP, mode1, 0.5, shape)
        u = pyref.tap_arrays(b, BOX3, mode2, -1.0, shape)
        assert np.array_equal(out.get(), lap_times_box(t, u))
    say("stencil2 with fractional data", mode1, mode2)
    a, b = rng.random((200, 260)).astype(F), rng.random((200, 260)).astype(F)
    out = ctx.empty(a.shape, F)
    sk.stencil2([], ctx.array(a), ctx.array(b), out)
    exp = lap_times_box(pyref.tap_arrays(a, LAP, mode1, 0.5, a.shape), pyref.tap_arrays(b, BOX3, mode2, -1.0, a.shape))
    assert np.max(np.abs(out.get() - exp)) <= 1e-5 * np.max(np.abs(exp))      # same operations in the same order
    assert np.array_equal(out.get(), exp)


def test_stencil2_mixed_types_and_1d(A, ctx):
    rng = np.random.default_rng(22)
    say("stencil2: Float32 source and Int32 source, Float64 result")
    sk = ctx.skeleton(A.SKEL_STENCIL2, "double", out_rank=2, taps=[(0, -1), (0, 1)], boundary="clamp", stencil_in="float",
                      taps2=[(-1, 0), (1, 0)], boundary2="mirror", stencil_in2="Int32",
                      stencil_fn="(double)(t1 - t0) * (double)(u1 - u0)")
    a = rng.random((70, 516)).astype(F)
    b = rng.integers(-1000, 1000, (70, 516)).astype(np.int32)
    out = ctx.empty(a.shape, np.float64)
    sk.stencil2([], ctx.array(a), ctx.array(b), out)
    t = pyref.tap_arrays(a, [(0, -1), (0, 1)], "clamp", 0, a.shape)
    u = pyref.tap_arrays(b, [(-1, 0), (1, 0)], "mirror", 0, a.shape)
    assert np.array_equal(out.get(), (t[1] - t[0]).astype(np.float64) * (u[1] - u[0]).astype(np.float64))
    say("stencil2 on vectors of different lengths")
    sk1 = ctx.skeleton(A.SKEL_STENCIL2, "float", out_rank=1, taps=[(0, -1), (0, 0), (0, 1)], boundary="wrap",
                       taps2=[(0, -2), (0, 2)], boundary2="constant", boundary2_constant="3.0f",
                       stencil_fn="(t0 + t1 + t2) - (u0 * u1)")
    for n1, n2 in [(5, 9), (1024, 1024), (100001, 70000), (1025, 5000)]:
        x = rng.integers(-5, 5, n1).astype(F)
        y = rng.integers(-5, 5, n2).astype(F)
        n = min(n1, n2)
        out = ctx.empty(n, F)
        sk1.stencil2([], ctx.array(x), ctx.array(y), out)
        t = pyref.tap_arrays(x, [(0, -1), (0, 0), (0, 1)], "wrap", 0, (n,))
        u = pyref.tap_arrays(y, [(0, -2), (0, 2)], "constant", 3.0, (n,))
        exp = ((t[0] + t[1]) + t[2]) - (u[0] * u[1])
        assert np.array_equal(out.get(), exp[0])
    say("stencil2 misuse")
    with pytest.raises(A.AccError) as e:       # result larger than the intersection
        sk1.stencil2([], ctx.array(np.zeros(8, F)), ctx.array(np.zeros(6, F)), ctx.empty(8, F))
    assert e.value.code == A.ERR_INVALID
    with pytest.raises(A.AccError) as e:       # a stencil2 skeleton is not a stencil
        sk1.stencil([], ctx.array(np.zeros(8, F)), ctx.empty(8, F))
    assert e.value.code == A.ERR_INVALID
