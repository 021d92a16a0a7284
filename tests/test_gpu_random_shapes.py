"""Scans, permutes and segmented and innermost folds on element types, sizes and key distributions drawn at random
(fixed seed: the same cases every run), against numpy.  Sources hold small integers, so every sum is exact in every
element type; results are compared bit for bit, and every result array carries two guard words past its end."""
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


class View(object):
    """a result that is the first part of a longer array"""
    def __init__(self, d):
        self.d = d

    def desc(self):
        return self.d


def near(rng, mult, hi):
    return max(1, int(rng.integers(0, hi // mult + 1)) * mult + int(rng.choice([-3, -1, 0, 0, 1, 2, 5, 17, 100])))


def test_random_scans(A, ctx):
    rng = np.random.default_rng(2001)
    kinds = ["scanl", "scanl1", "scanl'", "scanr", "scanr1", "scanr'"]
    for trial in range(18):
        kind = kinds[trial % 6]
        ctype, T = TYPES[int(rng.integers(0, len(TYPES)))]
        sk = ctx.skeleton(A.SCAN_KINDS[kind], ctype, env=[(1, ctype)], get="arrIn0_0[ix]", combine="(%s)(x + y)" % ctype,
                          seed=None if kind.endswith("1") else "(%s)3" % ctype)
        for _ in range(3):
            n = near(rng, 32768, 1 << 21) if rng.random() < 0.6 else int(rng.integers(1, 5000))
            say("scan", kind, ctype, "n", n)
            x = rng.integers(0, 3, n).astype(T)
            plus = 1 if kind in ("scanl", "scanr") else 0
            out = ctx.array(np.full(n + plus + 2, 77, T))
            tot = ctx.array(np.array(0, T))
            sk.scan([ctx.array(x)], n, out.desc(shape=(n + plus,)), tot if kind.endswith("'") else None)
            c = np.cumsum((x if kind.startswith("scanl") else x[::-1]).astype(np.int64))
            if plus:
                ref = np.concatenate([[3], 3 + c])
            elif kind.endswith("1"):
                ref = c
            else:
                ref = np.concatenate([[3], 3 + c[:-1]])
            if kind.startswith("scanr"):
                ref = ref[::-1]
            got = out.get()
            assert np.array_equal(got[:n + plus], ref.astype(T)) and np.all(got[n + plus:] == 77)
            if kind.endswith("'"):
                assert tot.get().reshape(-1)[0] == T(3 + c[-1])
        sk.destroy()


def test_random_permutes(A, ctx):
    rng = np.random.default_rng(2002)
    for trial in range(12):
        ctype, T = [("Int32", np.int32), ("Int64", np.int64), ("float", np.float32), ("Word32", np.uint32)][trial % 4]
        how = ["count", "weights", "max"][trial % 3]
        if how == "count":
            sk = ctx.skeleton(A.SKEL_PERMUTE, ctype, env=[(1, "Int32")], out_rank=1, get="(%s)1" % ctype, combine="x + y",
                              permutation="arrIn0_0[ix]", combine_hint=A.COMBINE_ADD)
        elif how == "weights":
            sk = ctx.skeleton(A.SKEL_PERMUTE, ctype, env=[(1, "Int32"), (1, ctype)], out_rank=1, get="arrIn1_0[ix]", combine="x + y",
                              permutation="arrIn0_0[ix]", combine_hint=A.COMBINE_ADD)
        else:
            sk = ctx.skeleton(A.SKEL_PERMUTE, ctype, env=[(1, "Int32"), (1, ctype)], out_rank=1, get="arrIn1_0[ix]",
                              combine="acc_max(x, y)", permutation="arrIn0_0[ix]")
        for _ in range(3):
            bins = int(rng.choice([1, 7, 256, 1000, 4097, 40960, 40961, 50001, 65536, 81920, 81921, 150000])) + int(rng.integers(0, 3))
            n = int(rng.choice([0, 1, 1000, 1 << 16, (1 << 20) + 3, 1 << 22]))
            skew = rng.random() < 0.5
            say("permute", how, ctype, "targets", bins, "n", n, "zipf keys" if skew else "uniform keys")
            keys = (np.minimum(rng.zipf(1.2, n) - 1, bins - 1) if skew else rng.integers(0, bins, n)).astype(np.int32)
            if n:
                keys[::11] = rng.integers(-3, bins + 3, keys[::11].size)
            src = rng.integers(0, 5, n).astype(T)
            dfl = rng.integers(0, 50, bins).astype(T)
            out = ctx.array(np.full(bins + 2, 99, T))
            env = [ctx.array(keys)] if how == "count" else [ctx.array(keys), ctx.array(src)]
            sk.permute(env, n, ctx.array(dfl), View(out.desc(shape=(bins,))))
            ok = (keys >= 0) & (keys < bins)
            ref = dfl.astype(np.int64)
            if how == "count":
                np.add.at(ref, keys[ok], 1)
            elif how == "weights":
                np.add.at(ref, keys[ok], src[ok].astype(np.int64))
            else:
                np.maximum.at(ref, keys[ok], src[ok].astype(np.int64))
            got = out.get()
            assert np.array_equal(got[:bins], ref.astype(T)) and np.all(got[bins:] == 99)
        sk.destroy()


def test_random_segmented_and_innermost_folds(A, ctx):
    rng = np.random.default_rng(2003)
    for trial in range(8):
        ctype, T = TYPES[int(rng.integers(0, len(TYPES)))]
        seg = ctx.skeleton(A.SKEL_FOLDSEG, ctype, env=[(1, ctype)], get="arrIn0_0[ix]", combine="(%s)(x + y)" % ctype, seed="(%s)1" % ctype)
        rows_ = ctx.skeleton(A.SKEL_FOLD, ctype, env=[(2, ctype)], out_rank=1, get="arrIn0_0[ix]", combine="(%s)(x + y)" % ctype,
                             seed="(%s)1" % ctype)
        for _ in range(3):
            nseg = int(rng.choice([1, 2, 255, 256, 257, 5000, 70001]))
            dist = str(rng.choice(["short", "mixed", "long", "mostly empty"]))
            if dist == "short":
                lens = rng.integers(0, 8, nseg)
            elif dist == "mixed":
                lens = rng.poisson(rng.choice([1, 4, 32, 100]), nseg)
            elif dist == "long":
                lens = rng.integers(0, max(2, (1 << 21) // nseg), nseg)
            else:
                lens = np.where(rng.random(nseg) < 0.8, 0, rng.integers(0, 3000, nseg))
            offs = np.concatenate([[0], np.cumsum(lens)]).astype(np.int32)
            n = int(offs[-1])
            say("foldSeg", ctype, nseg, "segments,", dist, "n", n)
            x = rng.integers(0, 3, n).astype(T)
            out = ctx.array(np.full(nseg + 2, 55, T))
            seg.foldseg([ctx.array(x)], n, ctx.array(offs), View(out.desc(shape=(nseg,))))
            c = np.concatenate([[0], np.cumsum(x.astype(np.int64))])
            got = out.get()
            assert np.array_equal(got[:nseg], (1 + c[offs[1:]] - c[offs[:-1]]).astype(T)) and np.all(got[nseg:] == 55)
        for _ in range(4):
            rows = int(rng.choice([1, 3, 255, 4096, 4097, 70001]))
            inner = int(rng.choice([1, 2, 3, 4, 5, 7, 8, 16, 31, 64, 191, 193, 1000, 16384, 100000]))
            while rows * inner > (1 << 23):
                rows = max(1, rows // 2)
            say("fold along rows", ctype, rows, "x", inner)
            x = rng.integers(0, 3, (rows, inner)).astype(T)
            out = ctx.array(np.full(rows + 2, 55, T))
            rows_.fold([ctx.array(x)], (rows, inner), out.desc(shape=(rows,)))
            got = out.get()
            assert np.array_equal(got[:rows], (1 + x.astype(np.int64).sum(axis=1)).astype(T)) and np.all(got[rows:] == 55)
        seg.destroy()
        rows_.destroy()


def test_segments_of_very_unequal_length(A, ctx):
    """the driver picks the kernel by the average length: among many short segments a few very long ones land on the
    kernel that gives every segment a lane, which folds their long stretches with the whole workgroup.  Integer sums
    are exact whatever the association; a non-commutative operator checks the order."""
    rng = np.random.default_rng(77)
    I32 = (1, "Int32")
    fs = ctx.skeleton(A.SKEL_FOLDSEG, "Int32", env=[I32], out_rank=1, get="arrIn0_0[ix]", combine="x + y", seed="5")
    aff = """
__device__ __forceinline__ Word32 affine16(Word32 x, Word32 y) {
  Word32 a1 = x >> 16, b1 = x & 0xffffu, a2 = y >> 16, b2 = y & 0xffffu;
  return (((a1 * a2) & 0xffffu) << 16) | ((a1 * b2 + b1) & 0xffffu);
}
"""
    f1 = ctx.skeleton(A.SKEL_FOLD1SEG, "Word32", env=[(1, "Word32")], out_rank=1, get="arrIn0_0[ix]", combine="affine16(x, y)", preamble=aff)
    fr = ctx.skeleton(A.SKEL_FOLDSEG, "Word32", env=[(1, "Word32")], out_rank=1, get="arrIn0_0[ix]", combine="affine16(x, y)", seed="0x00030005u",
                      preamble=aff, flags=A.FLAG_FOLD_RIGHT)
    for nseg, mean, longs in ((1000, 3, [(500, 100000)]), (5000, 1, [(0, 3000), (4999, 70001)]), (300, 20, [(7, 255), (8, 256), (9, 257), (200, 5000)]),
                              (2048, 2, [(k, 300 + k) for k in range(250, 262)]), (100000, 4, [(50000, 1 << 20)])):
        lens = rng.poisson(mean, nseg).astype(np.int64)
        for at, ln in longs:
            lens[at] = ln
        offs = np.concatenate([[0], np.cumsum(lens)]).astype(np.int32)
        n = int(offs[-1])
        say("segments of very unequal length: nseg", nseg, "n", n, "longs", longs[:3])
        x = rng.integers(-9, 9, n).astype(np.int32)
        out = ctx.empty(nseg, np.int32)
        fs.foldseg([ctx.array(x)], n, ctx.array(offs), out)
        want = np.add.reduceat(np.concatenate([x, [0]]).astype(np.int64), offs[:-1])
        want[lens == 0] = 0
        assert np.array_equal(out.get(), (want + 5).astype(np.int32))
        # composition of affine maps on 16-bit pairs: associative, not commutative -- the order must be the index order
        u = rng.integers(0, 2**32, n, dtype=np.uint64).astype(np.uint32)

        def chain(seg, right_seed=None):
            vals = [int(v) for v in seg] + ([right_seed] if right_seed is not None else [])
            acc = vals[0]
            for v in vals[1:]:
                acc = pyref.affine16(acc, v)
            return acc
        out1 = ctx.empty(nseg, np.uint32)
        f1.foldseg([ctx.array(u)], n, ctx.array(offs), out1)
        got = out1.get()
        picks = list(range(0, nseg, max(1, nseg // 40))) + [at for at, _ in longs]
        for s_ in picks:
            if lens[s_] > 0:
                assert int(got[s_]) == chain(u[offs[s_]:offs[s_ + 1]]), ("fold1Seg", s_, int(lens[s_]))
        outr = ctx.empty(nseg, np.uint32)
        fr.foldseg([ctx.array(u)], n, ctx.array(offs), outr)
        gotr = outr.get()
        for s_ in picks:
            assert int(gotr[s_]) == chain(u[offs[s_]:offs[s_ + 1]], 0x00030005), ("foldSeg right", s_, int(lens[s_]))


def test_segments_that_are_handed_over(A, ctx, tuned):
    """the variants of an instance with the table of jobs (`foldseg.giants=1`: always taken): among short segments, segments that go on for eight staged chunks or
    more beyond the chunk in which the workgroup first folds a stretch of them together.  Their owner enters the rest
    in a table of jobs and the workgroups take pieces of it when their own segments are done.  Several in one block of
    256 segments, next to one another, first and last of the array, more of them than the table has room for (the rest
    stay with their owners), the whole array one segment; sums of integers (exact), a non-commutative operator in both
    associations (the order of the pieces and of the owner's own part), pairs (a value of several tagged words), and
    the same inputs through the variants without the table (`foldseg.giants=0`)."""
    rng = np.random.default_rng(88)
    aff = """
__device__ __forceinline__ Word32 affine16(Word32 x, Word32 y) {
  Word32 a1 = x >> 16, b1 = x & 0xffffu, a2 = y >> 16, b2 = y & 0xffffu;
  return (((a1 * a2) & 0xffffu) << 16) | ((a1 * b2 + b1) & 0xffffu);
}
"""
    G = 30000                                        # above eight chunks of either staged length (2048, 3072)
    cases = [
        ("one in the middle", 3000, 3, {1500: 5 * G}),
        ("first and last", 2000, 5, {0: 2 * G + 1, 1999: 3 * G + 7}),
        ("three in one block, two of them neighbours", 1000, 2, {300: G, 301: 2 * G + 3, 420: G + 5}),
        ("behind empty segments", 700, 0, {5: 4 * G}),
        ("more than the table holds", 40 * 256, 1, {256 * k + 7: G + k for k in range(40)}),
        ("the whole array", 1, 0, {0: 6 * G + 11}),
        ("long ones that stay beside one that goes", 600, 4, {100: G - 5000, 101: 3 * G, 102: 12000, 103: 300}),
    ]

    def run_all(label):
        fs = ctx.skeleton(A.SKEL_FOLDSEG, "Int32", env=[(1, "Int32")], out_rank=1, get="arrIn0_0[ix]", combine="x + y", seed="5")
        f1 = ctx.skeleton(A.SKEL_FOLD1SEG, "Word32", env=[(1, "Word32")], out_rank=1, get="arrIn0_0[ix]", combine="affine16(x, y)", preamble=aff)
        fr = ctx.skeleton(A.SKEL_FOLDSEG, "Word32", env=[(1, "Word32")], out_rank=1, get="arrIn0_0[ix]", combine="affine16(x, y)",
                          seed="0x00030005u", preamble=aff, flags=A.FLAG_FOLD_RIGHT)
        fp = ctx.skeleton(A.SKEL_FOLDSEG, "Int64, Int32", env=[(1, "Int32")], out_rank=1, get="acc_elt{(Int64)arrIn0_0[ix], 1}",
                          combine="acc_elt{x.a1 + y.a1, x.a0 + y.a0}", seed="acc_elt{0, 0}")
        f1r = ctx.skeleton(A.SKEL_FOLD1SEG, "Word32", env=[(1, "Word32")], out_rank=1, get="arrIn0_0[ix]", combine="affine16(x, y)",
                           preamble=aff, flags=A.FLAG_FOLD_RIGHT)
        for name, nseg, mean, longs in cases:
            lens = rng.poisson(mean, nseg).astype(np.int64) if mean else np.zeros(nseg, np.int64)
            for at, ln in longs.items():
                lens[at] = ln
            offs = np.concatenate([[0], np.cumsum(lens)]).astype(np.int32)
            n = int(offs[-1])
            say("segments handed over:", label, name, "nseg", nseg, "n", n)
            x = rng.integers(-9, 9, n).astype(np.int32)
            c = np.concatenate([[0], np.cumsum(x.astype(np.int64))])
            sums = c[offs[1:]] - c[offs[:-1]]
            out = ctx.empty(nseg, np.int32)
            fs.foldseg([ctx.array(x)], n, ctx.array(offs), out)
            assert np.array_equal(out.get(), (sums + 5).astype(np.int32)), name
            pair = ctx.empty_tuple(nseg, [np.int64, np.int32])
            fp.foldseg([ctx.array(x)], n, ctx.array(offs), pair)
            got_sum, got_count = pair.get()
            assert np.array_equal(got_sum, sums) and np.array_equal(got_count, lens.astype(np.int32)), name
            u = rng.integers(0, 2**32, n, dtype=np.uint64).astype(np.uint32)

            def chain(seg, right_seed=None):
                vals = [int(v) for v in seg] + ([right_seed] if right_seed is not None else [])
                acc = vals[0]
                for v in vals[1:]:
                    acc = pyref.affine16(acc, v)
                return acc
            picks = sorted(set(list(range(0, nseg, max(1, nseg // 25))) + list(longs) + [k + 1 for k in longs if k + 1 < nseg]))
            g1, gr, g1r = ctx.empty(nseg, np.uint32), ctx.empty(nseg, np.uint32), ctx.empty(nseg, np.uint32)
            du, do = ctx.array(u), ctx.array(offs)
            f1.foldseg([du], n, do, g1)
            fr.foldseg([du], n, do, gr)
            f1r.foldseg([du], n, do, g1r)
            got1, gotr, got1r = g1.get(), gr.get(), g1r.get()
            for s_ in picks:
                if lens[s_] > 0:
                    assert int(got1[s_]) == chain(u[offs[s_]:offs[s_ + 1]]), (name, "fold1Seg", s_, int(lens[s_]))
                    assert int(got1r[s_]) == chain(u[offs[s_]:offs[s_ + 1]]), (name, "fold1Seg right", s_, int(lens[s_]))
                assert int(gotr[s_]) == chain(u[offs[s_]:offs[s_ + 1]], 0x00030005), (name, "foldSeg right", s_, int(lens[s_]))
        for sk_ in (fs, f1, fr, fp, f1r):
            sk_.destroy()
    tuned("foldseg.giants=0")
    run_all("(without the table)")
    tuned("foldseg.giants=1")
    run_all("")
    # the same under a loop's guard: both launches look at it, so an iteration past the loop's end writes nothing
    say("segments handed over: under a guard")
    fg = ctx.skeleton(A.SKEL_FOLDSEG, "Int32", env=[(1, "Int32")], out_rank=1, get="arrIn0_0[ix]", combine="x + y", seed="5", flags=A.FLAG_GUARDED)
    lens = rng.poisson(3, 3000).astype(np.int64)
    lens[1500] = 5 * G
    offs = np.concatenate([[0], np.cumsum(lens)]).astype(np.int32)
    n = int(offs[-1])
    x = rng.integers(-9, 9, n).astype(np.int32)
    c = np.concatenate([[0], np.cumsum(x.astype(np.int64))])
    want = (c[offs[1:]] - c[offs[:-1]] + 5).astype(np.int32)
    st, guard = ctx.stream(), A.Guard(ctx)
    dx, do = ctx.array(x), ctx.array(offs)
    first, second = ctx.array(np.full(3000, -1, np.int32)), ctx.array(np.full(3000, -1, np.int32))
    guard.attach(st)
    guard.reset(st)
    fg.foldseg([dx], n, do, first, stream=st)
    guard.latch(ctx.empty((), np.uint8).set(np.zeros(1, np.uint8)), st)      # the predicate says no: the loop has ended
    fg.foldseg([dx], n, do, second, stream=st)
    alive, count = guard.read(st)
    assert not alive and count == 0
    assert np.array_equal(first.get(), want) and np.all(second.get() == -1)
    guard.detach(st)
    guard.destroy()
    fg.destroy()


def test_an_instance_that_has_met_a_very_long_segment_takes_the_table(A, ctx):
    """as the knobs stand, an instance looks at its segment lengths behind calls number 1, 2, 4, 8 ... and, when it
    has found a segment that the variants with the table of jobs would hand over, has them compiled in the background
    and takes them when they are there: the same results before, while and after, and the launch trace names the
    second kernel from then on; an instance that sees no such segment never does"""
    import time
    rng = np.random.default_rng(89)

    def inputs(longest, mean, nseg):
        lens = rng.poisson(mean, nseg).astype(np.int64)
        lens[1234] = longest
        offs = np.concatenate([[0], np.cumsum(lens)]).astype(np.int32)
        x = rng.integers(-9, 9, int(offs[-1])).astype(np.int32)
        c = np.concatenate([[0], np.cumsum(x.astype(np.int64))])
        return ctx.array(x), ctx.array(offs), int(offs[-1]), (c[offs[1:]] - c[offs[:-1]] + 7).astype(np.int32)

    def kernels_of_a_call(sk, dx, do, n, nseg):
        out = ctx.empty(nseg, np.int32)
        ctx.trace_start()
        sk.foldseg([dx], n, do, out)
        ctx.sync()
        return ctx.trace_stop()[0], out.get()

    # (the last two: segments that rows of 16 lanes take, where "very long" is 32 times the average)
    for longest, switches, mean, nseg in ((200000, True, 6, 5000), (3000, False, 6, 5000), (300000, True, 300, 20000), (9000, False, 300, 20000)):
        sk = ctx.skeleton(A.SKEL_FOLDSEG, "Int32", env=[(1, "Int32")], out_rank=1, get="arrIn0_0[ix]", combine="x + y", seed="7")
        dx, do, n, want = inputs(longest, mean, nseg)
        say("segments of", mean, "elements on average and one of", longest, ": does the instance take the table?")
        launches, got = kernels_of_a_call(sk, dx, do, n, nseg)
        assert np.array_equal(got, want) and launches == 2          # the fold, and the look at the segment lengths
        deadline, taken = time.time() + 60, False
        for call in range(2, 4000):
            launches, got = kernels_of_a_call(sk, dx, do, n, nseg)
            assert np.array_equal(got, want), call
            if switches:                                            # (the first look has found the segment: no more of them)
                taken = taken or launches == 2                      # the fold and the launch that takes what it handed over
                assert launches == (2 if taken else 1), (call, launches)
            else:
                assert launches == (2 if (call & (call - 1)) == 0 else 1), (call, launches)
            if (taken and call > 100) or (not switches and call > 300) or time.time() > deadline:
                break
            if switches and not taken:
                time.sleep(0.005)                                   # (the compiler is at work meanwhile)
        assert taken == switches
        sk.destroy()


def test_sparse_matrix_with_a_few_very_long_rows(A, ctx, tuned):
    """the sparse matrix-vector product of a graph with a few hubs: rows of 40 000 to 200 000 non-zeros among rows of
    eight, with and without the table of jobs; Float32 sums in index order with another association than the
    sequential one, so against Float64 within 1e-5 of the sum of the magnitudes"""
    import scipy.sparse as sp
    rng = np.random.default_rng(90)
    rows, ncols = 6000, 50000
    lens = rng.poisson(8, rows).astype(np.int64)
    for at, ln in ((17, 200000), (18, 40000), (3000, 90001), (5999, 65536)):
        lens[at] = ln
    offs = np.concatenate([[0], np.cumsum(lens)]).astype(np.int32)
    nnz = int(offs[-1])
    vals = rng.standard_normal(nnz).astype(np.float32)
    cols = rng.integers(0, ncols, nnz).astype(np.int32)
    x = rng.standard_normal(ncols).astype(np.float32)
    m = sp.csr_matrix((vals.astype(np.float64), cols.copy(), offs.copy()), shape=(rows, ncols))     # (scipy may put its arrays in order)
    want = m @ x.astype(np.float64)
    size = abs(m) @ np.abs(x.astype(np.float64))
    dv, dc, dx, do = ctx.array(vals), ctx.array(cols), ctx.array(x), ctx.array(offs)
    for knobs in ("foldseg.giants=0", "foldseg.giants=1"):
        say("sparse matrix-vector product with four very long rows,", knobs)
        tuned(knobs)
        smvm = ctx.skeleton(A.SKEL_FOLDSEG, "float", env=[(1, "float"), (1, "Int32"), (1, "float")],
                            get="acc_stream(arrIn0_0, ix) * arrIn2_0[acc_stream(arrIn1_0, ix)]", combine="x + y", seed="0.0f")
        y = ctx.empty(rows, np.float32)
        smvm.foldseg([dv, dc, dx], nnz, do, y)
        got = y.get()
        assert np.all(np.abs(got - want) <= 1e-5 * size + 1e-30), knobs
        assert np.all(got[lens == 0] == 0.0)
        smvm.destroy()


def test_a_very_long_segment_among_segments_that_teams_of_lanes_fold(A, ctx, tuned):
    """segments of a few hundred to a few ten thousand elements on average go to rows of 16 lanes, waves or workgroups,
    a segment each; one that is far longer than the rest is entered in the table of jobs whole (`foldseg.giants=1`: the
    variants with the table, always) and folded in pieces by the launch behind.  Sums of integers, a non-commutative
    operator with and without a seed in both associations, and the same through the variants without the table."""
    rng = np.random.default_rng(91)
    aff = """
__device__ __forceinline__ Word32 affine16(Word32 x, Word32 y) {
  Word32 a1 = x >> 16, b1 = x & 0xffffu, a2 = y >> 16, b2 = y & 0xffffu;
  return (((a1 * a2) & 0xffffu) << 16) | ((a1 * b2 + b1) & 0xffffu);
}
"""
    cases = [("rows of 16 lanes", 300, 20000, {7000: 300000, 19999: 40000}), ("waves", 2000, 5000, {0: 250000, 2500: 2000 * 32 + 5}),
             ("workgroups", 20000, 1100, {550: 20000 * 32 + 1})]

    def chain(seg, right_seed=None):
        vals = [int(v) for v in seg] + ([right_seed] if right_seed is not None else [])
        acc = vals[0]
        for v in vals[1:]:
            acc = pyref.affine16(acc, v)
        return acc

    for knobs in ("foldseg.giants=1", "foldseg.giants=0"):
        tuned(knobs)
        fs = ctx.skeleton(A.SKEL_FOLDSEG, "Int32", env=[(1, "Int32")], out_rank=1, get="arrIn0_0[ix]", combine="x + y", seed="5")
        f1 = ctx.skeleton(A.SKEL_FOLD1SEG, "Word32", env=[(1, "Word32")], out_rank=1, get="arrIn0_0[ix]", combine="affine16(x, y)", preamble=aff)
        fr = ctx.skeleton(A.SKEL_FOLDSEG, "Word32", env=[(1, "Word32")], out_rank=1, get="arrIn0_0[ix]", combine="affine16(x, y)",
                          seed="0x00030005u", preamble=aff, flags=A.FLAG_FOLD_RIGHT)
        for name, mean, nseg, longs in cases:
            lens = rng.poisson(mean, nseg).astype(np.int64)
            lens[::97] = 0
            for at, ln in longs.items():
                lens[at] = ln
            offs = np.concatenate([[0], np.cumsum(lens)]).astype(np.int32)
            n = int(offs[-1])
            say("a very long segment among teams of lanes:", knobs, name, "nseg", nseg, "n", n)
            x = rng.integers(-9, 9, n).astype(np.int32)
            c = np.concatenate([[0], np.cumsum(x.astype(np.int64))])
            out = ctx.empty(nseg, np.int32)
            fs.foldseg([ctx.array(x)], n, ctx.array(offs), out)
            assert np.array_equal(out.get(), (c[offs[1:]] - c[offs[:-1]] + 5).astype(np.int32)), name
            u = rng.integers(0, 2**32, n, dtype=np.uint64).astype(np.uint32)
            g1, gr = ctx.empty(nseg, np.uint32), ctx.empty(nseg, np.uint32)
            du, do = ctx.array(u), ctx.array(offs)
            f1.foldseg([du], n, do, g1)
            fr.foldseg([du], n, do, gr)
            got1, gotr = g1.get(), gr.get()
            for s_ in sorted(set(list(range(1, nseg, max(1, nseg // 12))) + list(longs) + [k + 1 for k in longs if k + 1 < nseg])):
                if lens[s_] > 0:
                    assert int(got1[s_]) == chain(u[offs[s_]:offs[s_ + 1]]), (name, "fold1Seg", s_, int(lens[s_]))
                assert int(gotr[s_]) == chain(u[offs[s_]:offs[s_ + 1]], 0x00030005), (name, "foldSeg right", s_, int(lens[s_]))
        for sk_ in (fs, f1, fr):
            sk_.destroy()


def test_permute_with_a_hot_target_among_many(A, ctx, tuned):
    """a third to a half of the sources on one or two targets, the rest spread, in no order: the lanes of a wave that
    share the hot target combine first wherever they stand (tables under locks in LDS, locks in memory for tuples on
    more targets than the tables hold, compare-and-swap on the result for scalars there); with ignored elements among
    them; integer sums (exact), a maximum, pairs; and the same with `permute.gather=0`"""
    rng = np.random.default_rng(92)
    I32 = (1, "Int32")
    for knobs in ("", "permute.gather=0"):
        tuned(knobs)
        generic = ctx.skeleton(A.SKEL_PERMUTE, "Int32", env=[I32, I32], out_rank=1, get="arrIn1_0[ix]", combine="x + y",
                               permutation="arrIn0_0[ix]", combine_hint=A.COMBINE_GENERIC)
        biggest = ctx.skeleton(A.SKEL_PERMUTE, "float", env=[I32, I32], out_rank=1, get="(float)arrIn1_0[ix]", combine="acc_max(x, y)",
                               permutation="arrIn0_0[ix]", combine_hint=A.COMBINE_GENERIC)
        pair = ctx.skeleton(A.SKEL_PERMUTE, "Int32, Int32", env=[I32, I32], out_rank=1, get="acc_elt{arrIn1_0[ix], 1}",
                            combine="acc_elt{x.a1 + y.a1, x.a0 + y.a0}", permutation="arrIn0_0[ix]")
        # (targets: few enough for one table in LDS; for several; more than the tables are taken for, whatever the element)
        for n, bins, hot in ((200003, 900, (17,)), (500000, 100000, (7, 99999)), (1 << 18, 3000000, (123456,)), (70, 5, (2,))):
            if knobs and bins > 1000000:
                continue          # (a hundred thousand rounds on one lock in memory, one after the other: what the combining is there to avoid)
            keys = rng.integers(0, bins, n)
            for h in hot:
                keys[rng.random(n) < 0.45 / len(hot)] = h
            keys[rng.random(n) < 0.05] = -1
            keys = keys.astype(np.int32)
            w = rng.integers(-5, 6, n).astype(np.int32)
            say("permute with hot targets", hot, ": n", n, "targets", bins, knobs)
            valid = keys >= 0
            want = np.bincount(keys[valid], weights=w[valid], minlength=bins).astype(np.int64)
            count = np.bincount(keys[valid], minlength=bins)
            dk, dw = ctx.array(keys), ctx.array(w)
            out = ctx.empty(bins, np.int32)
            generic.permute([dk, dw], n, ctx.array(np.full(bins, 3, np.int32)), out)
            assert np.array_equal(out.get(), want + 3), ("generic", n, bins)
            top = np.full(bins, -100.0, np.float32)
            np.maximum.at(top, keys[valid], w[valid].astype(np.float32))
            outf = ctx.empty(bins, np.float32)
            biggest.permute([dk, dw], n, ctx.array(np.full(bins, -100.0, np.float32)), outf)
            assert np.array_equal(outf.get(), top), ("max", n, bins)
            outp, zero = ctx.empty_tuple(bins, [np.int32, np.int32]), ctx.empty_tuple(bins, [np.int32, np.int32])
            zero.comps[0].set(np.zeros(bins, np.int32)); zero.comps[1].set(np.zeros(bins, np.int32))
            pair.permute([dk, dw], n, zero, outp)
            assert np.array_equal(outp.comps[0].get(), want) and np.array_equal(outp.comps[1].get(), count), ("pairs", n, bins)
        for sk_ in (generic, biggest, pair):
            sk_.destroy()


def test_permute_of_sorted_and_clustered_keys(A, ctx):
    """runs of consecutive elements with one target: the kernels that update under a lock combine each run in its wave
    first (any combining function, floating-point addition on few targets, tuples); integer-valued sources, so every
    sum is exact"""
    rng = np.random.default_rng(78)
    I32 = (1, "Int32")
    generic = ctx.skeleton(A.SKEL_PERMUTE, "Int32", env=[I32, I32], out_rank=1, get="arrIn1_0[ix]", combine="x + y",
                           permutation="arrIn0_0[ix]", combine_hint=A.COMBINE_GENERIC)
    fadd = ctx.skeleton(A.SKEL_PERMUTE, "float", env=[I32, (1, "float")], out_rank=1, get="arrIn1_0[ix]", combine="x + y",
                        permutation="arrIn0_0[ix]", combine_hint=A.COMBINE_ADD)
    pair = ctx.skeleton(A.SKEL_PERMUTE, "Int32, Int32", env=[I32, I32], out_rank=1, get="acc_elt{arrIn1_0[ix], 1}",
                        combine="acc_elt{x.a1 + y.a1, x.a0 + y.a0}", permutation="arrIn0_0[ix]")
    for n, bins, how in ((100000, 7, "sorted"), (300001, 1000, "sorted"), (300001, 1000, "runs"), (200000, 5000, "runs with gaps"),
                         (65, 3, "sorted"), (1 << 20, 200000, "sorted")):
        if how == "sorted":
            keys = np.sort(rng.integers(0, bins, n))
        else:
            keys = np.repeat(rng.integers(0, bins, n // 37 + 1), 37)[:n]
        keys = keys.astype(np.int32)
        if how == "runs with gaps":
            keys[rng.random(n) < 0.1] = -1                       # ignored elements inside the runs
        w = rng.integers(-5, 6, n).astype(np.int32)
        say("permute of", how, "keys: n", n, "targets", bins)
        valid = keys >= 0
        want = np.bincount(keys[valid], weights=w[valid], minlength=bins).astype(np.int64)
        count = np.bincount(keys[valid], minlength=bins)
        dk, dw = ctx.array(keys), ctx.array(w)
        out = ctx.empty(bins, np.int32)
        generic.permute([dk, dw], n, ctx.array(np.full(bins, 3, np.int32)), out)
        assert np.array_equal(out.get(), want + 3), ("generic", how, n, bins)
        outf = ctx.empty(bins, np.float32)
        fadd.permute([dk, ctx.array(w.astype(np.float32))], n, ctx.array(np.zeros(bins, np.float32)), outf)
        assert np.array_equal(outf.get(), want.astype(np.float32)), ("float add", how, n, bins)
        outp = ctx.empty_tuple(bins, [np.int32, np.int32])
        zero = ctx.empty_tuple(bins, [np.int32, np.int32])
        zero.comps[0].set(np.zeros(bins, np.int32)); zero.comps[1].set(np.zeros(bins, np.int32))
        pair.permute([dk, dw], n, zero, outp)
        assert np.array_equal(outp.comps[0].get(), want) and np.array_equal(outp.comps[1].get(), count), ("pairs", how, n, bins)
    # counting into more targets than whole counts have room for in LDS (16-bit counts): sorted keys, runs of one key
    # long enough to take a count past its half-way mark many times over, and runs of 37
    count = ctx.skeleton(A.SKEL_PERMUTE, "Int32", env=[I32], out_rank=1, get="1", combine="x + y", permutation="arrIn0_0[ix]",
                         combine_hint=A.COMBINE_ADD)
    for n, bins, how in ((1 << 22, 65536, "sorted"), (1 << 22, 40000, "one key"), (1 << 21, 50001, "runs")):
        if how == "sorted":
            keys = np.sort(rng.integers(0, bins, n))
        elif how == "one key":
            keys = np.full(n, 12345)
            keys[::1000] = rng.integers(0, bins, keys[::1000].size)
        else:
            keys = np.repeat(rng.integers(0, bins, n // 37 + 1), 37)[:n]
        keys = keys.astype(np.int32)
        say("counting", how, "keys: n", n, "targets", bins)
        out = ctx.empty(bins, np.int32)
        count.permute([ctx.array(keys)], n, ctx.array(np.full(bins, 2, np.int32)), out)
        assert np.array_equal(out.get(), np.bincount(keys, minlength=bins) + 2), ("count", how, n, bins)


def test_fold_of_rows_that_lie_across_memory(A, ctx):
    """`ACC_FLAG_TILED` on a fold along the innermost dimension: the element function reads a matrix down its columns
    (the fold of a transposed matrix), and a lane takes a row.  Many short rows, rows just beyond what the
    one-lane-per-short-row entry takes, a few long rows (cut into pieces that a second launch joins) and one row;
    sums of integers, a non-commutative operator in both associations, fold1, pairs and Float64; the element function
    written over the kernel's names `acc_row` and `acc_col`; and `fold.across=1` on a plain row-major source, which
    takes the same kernels."""
    rng = np.random.default_rng(4711)
    aff = """
__device__ __forceinline__ Word32 affine16(Word32 x, Word32 y) {
  Word32 a1 = x >> 16, b1 = x & 0xffffu, a2 = y >> 16, b2 = y & 0xffffu;
  return (((a1 * a2) & 0xffffu) << 16) | ((a1 * b2 + b1) & 0xffffu);
}
"""
    def chain(vals):
        acc = int(vals[0])
        for v in vals[1:]:
            acc = pyref.affine16(acc, int(v))
        return acc

    # (h, w): the matrix in memory; the fold sees its transpose, w rows of h elements (the extents are read from the
    # source's descriptor, so that one instance serves every shape)
    across = "arrIn0_0[(ix % shIn0_1) * shIn0_0 + ix / shIn0_1]"
    fs = ctx.skeleton(A.SKEL_FOLD, "Int32", env=[(2, "Int32")], out_rank=1, get=across, combine="x + y", seed="5", flags=A.FLAG_TILED)
    fp = ctx.skeleton(A.SKEL_FOLD, "Int64, Int32", env=[(2, "Int32")], out_rank=1, get="acc_elt{(Int64)%s, 1}" % across,
                      combine="acc_elt{x.a1 + y.a1, x.a0 + y.a0}", seed="acc_elt{0, 0}", flags=A.FLAG_TILED)
    fd = ctx.skeleton(A.SKEL_FOLD1, "double", env=[(2, "double")], out_rank=1, get=across, combine="x + y", flags=A.FLAG_TILED)
    affine = [(flags, seed, ctx.skeleton(A.SKEL_FOLD if seed else A.SKEL_FOLD1, "Word32", env=[(2, "Word32")], out_rank=1, get=across,
                                         combine="affine16(x, y)", seed=seed, preamble=aff, flags=flags))
              for flags, seed in ((A.FLAG_TILED, "0x00030005u"), (A.FLAG_TILED | A.FLAG_FOLD_RIGHT, "0x00030005u"), (A.FLAG_TILED, None),
                                  (A.FLAG_TILED | A.FLAG_FOLD_RIGHT, None))]
    # the same element function written with the kernel's names for the row and the place within it, in an instance
    # that gives rows to lanes (which knows both) and in one that does not (which divides)
    by_name = "arrIn0_0[acc_col * shIn0_0 + acc_row]"
    named = [ctx.skeleton(A.SKEL_FOLD, "Int32", env=[(2, "Int32")], out_rank=1, get=by_name, combine="x + y", seed="5", flags=flags)
             for flags in (A.FLAG_TILED, 0)]
    for h, w in ((17, 70000), (40, 3000), (1000, 999), (5000, 33), (70000, 5), (300000, 1), (1, 4000), (129, 257), (5, 1000), (16, 300)):
        say("fold across", h, w)
        m = rng.integers(-9, 9, (h, w)).astype(np.int32)
        dm = ctx.array(m)
        for sk_ in [fs] + named:
            out = ctx.array(np.full(w + 2, 77, np.int32))
            sk_.fold([dm], (w, h), out.desc(shape=(w,)))
            got = out.get()
            assert np.array_equal(got[:w], m.sum(axis=0, dtype=np.int32) + 5), (h, w)
            assert np.array_equal(got[w:], [77, 77]), (h, w)
        # pairs: (sum as Int64, count)
        pair = ctx.empty_tuple(w, [np.int64, np.int32])
        fp.fold([dm], (w, h), pair)
        s_, c_ = pair.get()
        assert np.array_equal(s_, m.sum(axis=0, dtype=np.int64)) and np.array_equal(c_, np.full(w, h, np.int32)), (h, w)
        # Float64, small integers: exact
        md = ctx.array(m.astype(np.float64))
        od = ctx.empty(w, np.float64)
        fd.fold([md], (w, h), od)
        assert np.array_equal(od.get(), m.sum(axis=0).astype(np.float64)), (h, w)
        # a non-commutative operator, both associations, with and without a seed
        u = rng.integers(0, 2**32, (h, w), dtype=np.uint64).astype(np.uint32)
        du = ctx.array(u)
        picks = sorted(set([0, w - 1, w // 2] + [int(c) for c in rng.integers(0, w, 6)]))
        plain = {c: chain(u[:, c]) for c in picks}
        for flags, seed, fa in affine:
            oa = ctx.empty(w, np.uint32)
            fa.fold([du], (w, h), oa)
            ga = oa.get()
            for c in picks:
                want = pyref.affine16(plain[c], 0x00030005) if seed else plain[c]
                assert int(ga[c]) == want, ("affine", h, w, c, flags, seed)
    # a plain row-major source through the same kernels
    with A.tuning("fold.across=1", ctx):
        fs = ctx.skeleton(A.SKEL_FOLD, "Int32", env=[(2, "Int32")], out_rank=1, get="arrIn0_0[ix]", combine="x + y", seed="0")
    for rows, inner in ((3000, 40), (7, 100000), (100000, 17)):
        say("fold across, forced", rows, inner)
        m = rng.integers(-9, 9, (rows, inner)).astype(np.int32)
        out = ctx.empty(rows, np.int32)
        fs.fold([ctx.array(m)], (rows, inner), out)
        assert np.array_equal(out.get(), m.sum(axis=1, dtype=np.int32)), (rows, inner)


def test_permute_whose_combination_is_the_new_value(A, ctx):
    """`permute const`: the scatter of a stream compaction (targets in order, half of the sources ignored), of a
    stable sorting pass by a 4-bit digit and of a random permutation -- every target written once, so the result is
    exact -- for elements of 4 and 8 bytes, spelt `x` and `(x)`; with several sources on a target the result holds
    one of them whole; and the same through the compare-and-swap loop (`permute.replace=0`).  An instance whose
    combination is spelt so stores and reads nothing."""
    rng = np.random.default_rng(515)
    n = 300007
    keep = rng.random(n) < 0.5
    places = np.where(keep, np.cumsum(keep) - keep, -1).astype(np.int32)
    digit = rng.integers(0, 16, n)
    order = np.argsort(digit, kind="stable")
    dest = np.empty(n, np.int32)
    dest[order] = np.arange(n, dtype=np.int32)
    for knobs in ("", "permute.replace=0"):
        for ctype, dt in (("Int32", np.int32), ("float", np.float32), ("Int64", np.int64), ("double", np.float64)):
            for spelt in ("x", "( x )"):
                if knobs and spelt != "x":
                    continue
                say("permute const", knobs or "-", ctype, repr(spelt))
                with A.tuning(knobs, ctx):
                    sk = ctx.skeleton(A.SKEL_PERMUTE, ctype, env=[(1, "Int32"), (1, ctype)], out_rank=1, get="arrIn1_0[ix]",
                                      combine=spelt, permutation="(Int64)arrIn0_0[ix]")
                vals = rng.integers(-10**6, 10**6, n).astype(dt)
                dv = ctx.array(vals)
                for tgt, nt in ((places, int(keep.sum())), (dest, n), (rng.permutation(n).astype(np.int32), n)):
                    dfl = rng.integers(0, 100, nt + 2).astype(dt)
                    out = ctx.array(np.full(nt + 2, 77, dt))
                    dd = ctx.array(dfl)
                    sk.permute([ctx.array(tgt), dv], n, View(dd.desc(shape=(nt,))), View(out.desc(shape=(nt,))))
                    want = dfl[:nt].copy()
                    m = tgt >= 0
                    want[tgt[m]] = vals[m]
                    got = out.get()
                    assert np.array_equal(got[:nt], want) and np.all(got[nt:] == 77), (knobs, ctype, nt)
                # eight sources a target: one of them, whole
                many = (np.arange(n) // 8).astype(np.int32)
                nt = int(many[-1]) + 1
                wide = (vals.astype(np.int64) * 0x100000001).astype(dt) if dt == np.int64 else vals
                out = ctx.empty(nt, dt)
                sk.permute([ctx.array(many), ctx.array(wide)], n, ctx.array(np.zeros(nt, dt)), out)
                got = out.get()
                cand = np.full((nt, 8), wide[0], dt)
                cand.reshape(-1)[:n] = wide
                cand[-1, n - 8 * (nt - 1):] = wide[n - 1]
                assert np.all((cand == got[:, None]).any(axis=1)), (knobs, ctype)
    # pairs (components are arrays of their own: of several sources on a target one must win whole) and small scalars
    for knobs in ("", "permute.replace=0"):
        say("permute const, pairs and small scalars", knobs or "-")
        with A.tuning(knobs, ctx):
            sp = ctx.skeleton(A.SKEL_PERMUTE, "Int32, Int32", env=[(1, "Int32"), (1, "Int32")], out_rank=1,
                              get="acc_elt{arrIn1_0[ix], (Int32)ix}", combine="acc_elt{x.a1, x.a0}", permutation="(Int64)arrIn0_0[ix]")
            sb = ctx.skeleton(A.SKEL_PERMUTE, "Int8", env=[(1, "Int32"), (1, "Int32")], out_rank=1, get="(Int8)arrIn1_0[ix]",
                              combine="x", permutation="(Int64)arrIn0_0[ix]")
            sh = ctx.skeleton(A.SKEL_PERMUTE, "Word16", env=[(1, "Int32"), (1, "Int32")], out_rank=1, get="(Word16)arrIn1_0[ix]",
                              combine="x", permutation="(Int64)arrIn0_0[ix]")
        vals = rng.integers(-10**6, 10**6, n).astype(np.int32)
        dv = ctx.array(vals)
        for tgt, nt in ((places, int(keep.sum())), (dest, n)):
            m = tgt >= 0
            dk = ctx.array(tgt)
            out = ctx.empty_tuple(nt, [np.int32, np.int32])
            sp.permute([dk, dv], n, ctx.tuple_array(np.full(nt, 5, np.int32), np.full(nt, 6, np.int32)), out)
            a1, a0 = out.get()
            w1 = np.full(nt, 5, np.int32); w1[tgt[m]] = vals[m]
            w0 = np.full(nt, 6, np.int32); w0[tgt[m]] = np.arange(n, dtype=np.int32)[m]
            assert np.array_equal(a1, w1) and np.array_equal(a0, w0), (knobs, nt)
            for sk_, dt in ((sb, np.int8), (sh, np.uint16)):
                out = ctx.array(np.full(nt + 2, 77, dt))
                dd = ctx.array(np.full(nt, 9, dt))
                sk_.permute([dk, dv], n, dd, View(out.desc(shape=(nt,))))
                w = np.full(nt, 9, dt); w[tgt[m]] = vals[m].astype(dt)
                got = out.get()
                assert np.array_equal(got[:nt], w) and np.all(got[nt:] == 77), (knobs, dt, nt)
        many = (np.arange(n) // 8).astype(np.int32)
        many[::1000] = -1                                # (some are ignored)
        nt = n // 8 + 1
        out = ctx.empty_tuple(nt, [np.int32, np.int32])
        sp.permute([ctx.array(many), dv], n, ctx.tuple_array(np.zeros(nt, np.int32), np.full(nt, -1, np.int32)), out)
        a1, a0 = out.get()
        hit = a0 >= 0
        assert hit.sum() >= nt - 1
        assert np.array_equal(many[a0[hit]], np.arange(nt, dtype=np.int32)[hit]) and np.array_equal(vals[a0[hit]], a1[hit]), knobs
