"""Stencils drawn at random (rank, reach in every dimension, which taps, coefficients, element type, boundary mode)
on shapes drawn around the strip width and the length of a walk through the planes, against numpy index maps
(tests/pyref.py).  Sources hold small integers, so every operation is exact in every element type and the results are
compared bit for bit.  The seed is fixed: the same instances every run."""
import itertools
import sys

import numpy as np
import pytest

import pyref

pytestmark = pytest.mark.gpu

TYPES = [("Int8", np.int8), ("Word16", np.uint16), ("Int32", np.int32), ("Int64", np.int64), ("float", np.float32),
         ("double", np.float64)]


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


def near(rng, mult, hi):
    return max(1, int(rng.integers(0, hi // mult + 1)) * mult + int(rng.choice([-3, -1, 0, 0, 1, 2, 5, 17, 100])))


@pytest.mark.parametrize("rank", [1, 2, 3])
def test_random_stencils(A, ctx, rank):
    rng = np.random.default_rng(1000 + rank)
    trials = []
    for trial in range(10 if rank < 3 else 14):          # every instance first: they compile side by side, variants included
        ctype, T = TYPES[int(rng.integers(0, len(TYPES)))]
        mode = str(rng.choice(["clamp", "mirror", "wrap", "constant"]))
        reach = [int(rng.integers(0, 3)) for _ in range(rank)]
        if rank < 3:
            reach[-1] = int(rng.integers(0, 5))
        box = list(itertools.product(*[range(-r, r + 1) for r in reach]))
        taps = [box[i] for i in rng.choice(len(box), int(rng.integers(1, min(len(box), 9) + 1)), replace=False)]
        for d in range(rank):                                  # the extremes, so that the reach is what was drawn
            for sign in (-1, 1):
                t = [0] * rank
                t[d] = sign * reach[d]
                if tuple(t) not in taps:
                    taps.append(tuple(t))
        coef = [int(rng.integers(-2, 3)) for _ in taps]
        whole = np.issubdtype(T, np.integer)
        fn = " + ".join("(%s)(%d) * t%d" % (ctype, c, k) for k, c in enumerate(coef))
        sk = ctx.skeleton(A.SKEL_STENCIL, ctype, out_rank=rank, taps=taps if rank > 1 else [(0, t[0]) for t in taps],
                          boundary=mode, boundary_constant="(%s)2" % ctype, stencil_fn="(%s)(%s)" % (ctype, fn) if whole else fn)
        sk.prefetch(range(1, 6))
        trials.append((ctype, T, mode, reach, taps, coef, whole, sk))
    for ctype, T, mode, reach, taps, coef, whole, sk in trials:
        for _ in range(2):
            shape = [near(rng, 256, 1100) if rng.random() < 0.7 else int(rng.integers(1, 80))]
            if rank >= 2:
                shape.insert(0, int(rng.integers(1, 70)))
            if rank == 3:
                shape.insert(0, near(rng, 64, 140) if rng.random() < 0.5 else int(rng.integers(1, 12)))
            shape = tuple(max(s, r + 1) for s, r in zip(shape, reach))      # the index maps assume the array spans the stencil
            say("stencil", ctype, mode, "taps", taps, "shape", shape)
            v = rng.integers(0, 4, shape).astype(T)
            out = ctx.empty(shape, T)
            sk.stencil([], ctx.array(v), out)
            if rank == 3:
                t = pyref.tap_arrays3(v, taps, mode, 2, shape)
            elif rank == 2:
                t = pyref.tap_arrays(v, taps, mode, 2, shape)
            else:
                t = [a[0] for a in pyref.tap_arrays(v.reshape(1, -1), [(0, x[0]) for x in taps], mode, 2, (1, shape[0]))]
            if whole:
                ref = sum(np.int64(c) * a.astype(np.int64) for c, a in zip(coef, t)).astype(T)
            else:
                ref = sum(T(c) * a for c, a in zip(coef, t)).astype(T)
            assert np.array_equal(out.get(), ref)


@pytest.mark.parametrize("rank", [2, 3])
def test_stencils_on_arrays_narrower_than_a_strip(A, ctx, rank):
    """a strip is 256 columns wide: on narrower arrays (and in the last strip of wider ones, where that is short) the
    lane across the right edge holds 1 to 4 columns, the lanes beyond it none.  Every width modulo 4, reaches of 1, 2
    and 4 columns, every boundary mode, elements of 1, 4 and 8 bytes.  Arrays of up to 36 columns (16 in three
    dimensions) take the variants that give a thread an element instead: both sides of that bound, and tall arrays of
    two and three columns."""
    rng = np.random.default_rng(2000 + rank)
    widths = [2, 3, 4, 5, 6, 7, 9, 16, 17, 36, 37, 63, 64, 66, 100, 129, 131, 202, 253, 254, 255, 256 + 65, 256 + 130, 512 + 70]
    cases = []
    for (ctype, T), mode, rx in itertools.product([("Int8", np.int8), ("float", np.float32), ("double", np.float64)],
                                                  ["clamp", "mirror", "wrap", "constant"], [1, 2, 4]):
        if rank == 3 and (rx == 4 or (ctype == "double" and (rx != 1 or mode in ("mirror", "wrap"))) or
                          (ctype == "Int8" and (rx != 2 or mode != "mirror"))):
            continue                                               # (rank 3 compiles slowly: a selection)
        if rank == 2:
            taps = [(0, 0), (0, -rx), (0, rx), (-1, 1), (1, -1), (1, rx - 1)]
        else:
            taps = [(0, 0, 0), (0, 0, -rx), (0, 0, rx), (-1, 0, 1), (1, 1, -1), (0, -1, rx - 1), (1, 0, 0)]
        coef = [int(rng.integers(-2, 3)) or 1 for _ in taps]
        whole = np.issubdtype(T, np.integer)
        fn = " + ".join("(%s)(%d) * t%d" % (ctype, c, k) for k, c in enumerate(coef))
        sk = ctx.skeleton(A.SKEL_STENCIL, ctype, out_rank=rank, taps=taps, boundary=mode, boundary_constant="(%s)2" % ctype,
                          stencil_fn="(%s)(%s)" % (ctype, fn) if whole else fn)
        sk.prefetch(range(1, 6))                                   # every width below: every variant is wanted
        cases.append((ctype, T, mode, rx, taps, coef, whole, sk))
    for ctype, T, mode, rx, taps, coef, whole, sk in cases:        # (the instances have been compiling side by side)
        for w in widths:
            if w < rx + 1:
                continue                                           # the index maps assume the array spans the stencil
            shape = (7, w) if rank == 2 else (6, 5, w)
            if w <= 3:                                             # (a few columns: an element a thread, many workgroups of them)
                shape = (20011, w) if rank == 2 else (3001, 3, w)
            say("narrow stencil", ctype, mode, "reach", rx, "shape", shape)
            v = rng.integers(0, 4, shape).astype(T)
            out = ctx.empty(shape, T)
            sk.stencil([], ctx.array(v), out)
            t = pyref.tap_arrays3(v, taps, mode, 2, shape) if rank == 3 else pyref.tap_arrays(v, taps, mode, 2, shape)
            if whole:
                ref = sum(np.int64(c) * a.astype(np.int64) for c, a in zip(coef, t)).astype(T)
            else:
                ref = sum(T(c) * a for c, a in zip(coef, t)).astype(T)
            assert np.array_equal(out.get(), ref), (ctype, mode, rx, shape)


def test_stencil2_on_narrow_sources_of_equal_and_unequal_width(A, ctx):
    """two sources as wide as the result take the cut strip; a wider source has elements where the result ends"""
    rng = np.random.default_rng(2100)
    taps = [(0, -1), (0, 0), (0, 1), (1, 1)]
    for mode1, mode2 in (("clamp", "wrap"), ("mirror", "constant")):
        sk = ctx.skeleton(A.SKEL_STENCIL2, "float", out_rank=2, taps=taps, taps2=taps, boundary=mode1, boundary2=mode2,
                          boundary_constant="2.0f", boundary2_constant="2.0f",
                          stencil_fn="t0 + 2.0f * t1 + t2 - t3 + u0 - 3.0f * u1 + u2 + u3")
        for (w1, w2) in ((101, 101), (131, 140), (140, 131), (70, 70), (255, 300), (7, 7)):
            h1, h2 = 9, 11
            say("narrow stencil2", mode1, mode2, "widths", w1, w2)
            a = rng.integers(0, 4, (h1, w1)).astype(np.float32)
            b = rng.integers(0, 4, (h2, w2)).astype(np.float32)
            shape = (min(h1, h2), min(w1, w2))
            out = ctx.empty(shape, np.float32)
            sk.stencil2([], ctx.array(a), ctx.array(b), out)
            t = pyref.tap_arrays(a, taps, mode1, 2.0, shape)
            u = pyref.tap_arrays(b, taps, mode2, 2.0, shape)
            ref = t[0] + 2 * t[1] + t[2] - t[3] + u[0] - 3 * u[1] + u[2] + u[3]
            assert np.array_equal(out.get(), ref.astype(np.float32)), (mode1, mode2, w1, w2)
