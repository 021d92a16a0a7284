"""The five benchmark configurations at their full sizes, through the C ABI.

Checked against the CPU oracle where it runs in a second or two (the C
restatement handles 2^26 elements comfortably), and through size-independent
properties otherwise.  Tolerances are the configurations' own.

The fragments spell reads that are consumed once as acc_stream(array, ix), the
non-temporal load a code generator emits for the linear index of a delayed
array; indirect reads (the gathered vector of the SMVM) stay plain.
"""
import sys

import numpy as np
import pytest

pytestmark = pytest.mark.gpu

F32 = (1, "float")
I32 = (1, "Int32")


def say(*a):
    print("[case]", *a)
    sys.stdout.flush()


@pytest.fixture(scope="module")
def A():
    import acchip
    return acchip


@pytest.fixture(scope="module")
def wl():
    import workloads
    return workloads


@pytest.fixture(scope="module")
def ctx(A):
    c = A.Context(0)
    yield c
    c.close()


def test_config1_dot_product_2_24(A, ctx, wl, orc):
    say("dot 2^24")
    n = 1 << 24
    x, y = wl.dot_inputs(n)
    dot = ctx.skeleton(A.SKEL_FOLD, "float", env=[F32, F32], out_rank=0, get="acc_stream(arrIn0_0, ix) * acc_stream(arrIn1_0, ix)",
                       combine="x + y", seed="0.0f")
    out = ctx.empty((), np.float32)
    dx, dy = ctx.array(x), ctx.array(y)
    dot.fold([dx, dy], n, out)
    got = float(out.get())
    truth, cond = orc.dot_f64(x, y), orc.dot_abs_f64(x, y)
    left, right = float(orc.dot_f32(x, y, orc.DIR_LEFT)), float(orc.dot_f32(x, y, orc.DIR_RIGHT))
    say("gpu %.6f  f64 %.6f  seq-f32 left %.6f right %.6f  sum|xy| %.1f" % (got, truth, left, right, cond))
    # 1e-4 relative to the sequential Float32 result (either association), the denominator floored by
    # that sequential sum's own rounding noise n*eps*sum|x_i y_i| (the result itself can be near zero)
    floor = n * 2.0 ** -24 * cond
    assert min(abs(got - left), abs(got - right)) <= 1e-4 * max(abs(left), floor)
    # against the Float64 truth the blocked GPU sum is far more accurate than the sequential one
    assert abs(got - truth) <= 1e-6 * cond
    # reproducible: the grid and the association are fixed
    dot.fold([dx, dy], n, out)
    assert float(out.get()) == got


@pytest.mark.parametrize("kind", ["scanl", "scanl1", "scanr"])
def test_config2_prefix_sums_2_26(A, ctx, wl, orc, kind):
    say(kind, "2^26")
    n = 1 << 26
    x = wl.scan_input(n)
    sk = ctx.skeleton(A.SCAN_KINDS[kind], "Int32", env=[I32], get="acc_stream(arrIn0_0, ix)", combine="x + y",
                      seed=None if kind == "scanl1" else "0")
    m = n if kind == "scanl1" else n + 1
    out = ctx.empty(m, np.int32)
    sk.scan([ctx.array(x)], n, out)
    got = out.get()
    assert np.array_equal(got, orc.scan(kind, orc.OP_ADD, x, seed=0))          # bit-exact
    # and the properties that pin it without the oracle
    total = int(x.sum(dtype=np.int64))
    assert total < 2 ** 31
    if kind == "scanl":
        assert got[0] == 0 and got[-1] == total and np.array_equal(np.diff(got), x)
    elif kind == "scanl1":
        assert got[0] == x[0] and got[-1] == total and np.array_equal(np.diff(got), x[1:])
    else:
        assert got[-1] == 0 and got[0] == total and np.array_equal(got[:-1] - got[1:], x)


@pytest.mark.parametrize("case", ["uniform256", "zipf65536"])
def test_config3_histograms_2_26(A, ctx, wl, orc, case):
    say("histogram", case, "2^26 keys")
    n = 1 << 26
    bins = 256 if case == "uniform256" else 65536
    keys = wl.hist_uniform_keys(n, bins) if case == "uniform256" else wl.hist_zipf_keys(n, bins)
    hist = ctx.skeleton(A.SKEL_PERMUTE, "Int32", env=[I32], out_rank=1, get="1", combine="x + y",
                        permutation="acc_stream(arrIn0_0, ix)", combine_hint=A.COMBINE_ADD)
    zeros = np.zeros(bins, np.int32)
    out = ctx.empty(bins, np.int32)
    dk = ctx.array(keys)
    hist.permute([dk], n, ctx.array(zeros), out)
    got = out.get()
    assert int(got.sum(dtype=np.int64)) == n                                   # every key counted once
    assert np.array_equal(got, orc.permute(orc.OP_ADD, zeros, keys))            # bit-exact
    if case == "zipf65536":
        assert got[0] == got.max() and 0.12 < got[0] / n < 0.15                 # rank 1 carries ~13.7 %
    # a second launch on the same skeleton starts from the defaults again
    ones = np.ones(bins, np.int32)
    hist.permute([dk], n, ctx.array(ones), out)
    assert np.array_equal(out.get(), got + 1)


def test_config4_stencils_8192(A, ctx, wl, orc):
    h = w = 8192
    say("stencils on 8192 x 8192")
    img = wl.stencil_image(h, w)
    taps = [(dy, dx) for dy in (-1, 0, 1) for dx in (-1, 0, 1)]
    gauss = ctx.skeleton(A.SKEL_STENCIL, "float", out_rank=2, taps=taps, boundary="clamp",
                         stencil_fn=A.linear_stencil_fn([1, 2, 1, 2, 4, 2, 1, 2, 1], 16))
    a, b = ctx.array(img), ctx.empty((h, w), np.float32)
    res = gauss.stencil_iterate([], a, b, 10).get()
    # The oracle on full-width bands: ten applications contaminate ten rows inwards from an
    # artificial cut, so a band of 60 rows pins its middle 40 (and all 50 next to a true edge).
    for lo, hi, keep_lo, keep_hi in [(0, 60, 0, 50), (4000, 4060, 4010, 4050), (h - 60, h, h - 50, h)]:
        say("  gaussian x10 rows", keep_lo, "..", keep_hi)
        exp = orc.stencil2d(img[lo:hi], orc.GAUSS3X3, divisor=16.0, mode="clamp", iters=10)
        err = np.max(np.abs(res[keep_lo:keep_hi] - exp[keep_lo - lo:keep_hi - lo]))
        assert err <= 1e-5, err                                                 # the configuration's tolerance
        assert np.array_equal(res[keep_lo:keep_hi], exp[keep_lo - lo:keep_hi - lo])   # in fact the same bits
    assert 0.0 <= res.min() and res.max() < 1.0                                 # a convex combination stays in range
    say("  5-point laplacian, mirror")
    lap = ctx.skeleton(A.SKEL_STENCIL, "float", out_rank=2, taps=[(-1, 0), (0, -1), (0, 0), (0, 1), (1, 0)],
                       boundary="mirror", stencil_fn=A.linear_stencil_fn([1, 1, -4, 1, 1]))
    a.set(img)
    lap.stencil([], a, b)
    got = b.get()
    for lo, hi, keep_lo, keep_hi in [(0, 40, 0, 39), (5000, 5040, 5001, 5039), (h - 40, h, h - 39, h)]:
        exp = orc.stencil2d(img[lo:hi], orc.LAPLACE5, mode="mirror")
        assert np.max(np.abs(got[keep_lo:keep_hi] - exp[keep_lo - lo:keep_hi - lo])) <= 1e-5
    # the interior of the Laplacian sums to a boundary term only: sum over all = sum of edge differences
    inner = got[1:-1, 1:-1].astype(np.float64).sum()
    i64 = img.astype(np.float64)
    flux = (i64[0, 1:-1] - i64[1, 1:-1]).sum() + (i64[-1, 1:-1] - i64[-2, 1:-1]).sum() + \
           (i64[1:-1, 0] - i64[1:-1, 1]).sum() + (i64[1:-1, -1] - i64[1:-1, -2]).sum()
    assert abs(inner - flux) <= 1e-3 * max(1.0, abs(flux)) + 64.0               # telescoping sum, Float32 rounding


def test_config5_smvm_2_20_rows(A, ctx, wl, orc):
    say("smvm 2^20 rows")
    vals, cols, offs, lens, x = wl.smvm_inputs()
    nnz, rows = vals.size, offs.size - 1
    assert rows == 1 << 20 and abs(nnz / 2 ** 25 - 1) < 0.01
    # the front end turns segment lengths into offsets with an exclusive scan (CUDA.hs:402): do it on the device
    scan = ctx.skeleton(A.SKEL_SCANL, "Int32", env=[I32], get="arrIn0_0[ix]", combine="x + y", seed="0")
    doff = ctx.empty(rows + 1, np.int32)
    scan.scan([ctx.array(lens)], rows, doff)
    assert np.array_equal(doff.get(), offs)
    smvm = ctx.skeleton(A.SKEL_FOLDSEG, "float", env=[F32, I32, F32], get="acc_stream(arrIn0_0, ix) * arrIn2_0[acc_stream(arrIn1_0, ix)]",
                        combine="x + y", seed="0.0f")
    y = ctx.empty(rows, np.float32)
    smvm.foldseg([ctx.array(vals), ctx.array(cols), ctx.array(x)], nnz, doff, y)
    got = y.get()
    assert np.array_equal(got, orc.smvm_f32(vals, cols, offs, x, orc.DIR_LEFT))   # same order as a sequential fold
    y64, yabs = orc.smvm_f64(vals, cols, offs, x)
    # per row 1e-4 relative; rows that cancel to almost nothing are measured against their magnitude
    assert np.all(np.abs(got - y64) <= 1e-4 * np.maximum(np.abs(y64), 1e-3 * yabs) + 1e-30)
    assert np.all(got[lens == 0] == 0.0)


def test_more_than_2_31_elements(A, ctx):
    """indices are 64-bit throughout: map, fold, scan, permute and segmented fold over 2^31 + 1 000 003 bytes"""
    n = (1 << 31) + 1000003
    W8 = (1, "Word8")
    say("beyond 2^31 elements, n =", n)
    x = np.empty(n, np.uint8)
    blk = (np.arange(1 << 20, dtype=np.uint32) * 7 % 251).astype(np.uint8)
    for s in range(0, n, 1 << 20):
        e = min(n, s + (1 << 20))
        x[s:e] = blk[:e - s]
    dx, o = ctx.array(x), ctx.empty(n, np.uint8)
    say("map")
    A_map = ctx.skeleton(A.SKEL_MAP, "Word8", env=[W8], out_rank=1, get="(Word8)(arrIn0_0[ix] + 1)")
    A_map.map([dx], o)
    got = o.get()
    assert np.array_equal(got[-5000000:], (x[-5000000:] + 1).astype(np.uint8)) and np.array_equal(got[:1000], (x[:1000] + 1).astype(np.uint8))
    say("fold")
    f = ctx.skeleton(A.SKEL_FOLD, "Int64", env=[W8], out_rank=0, get="(Int64)arrIn0_0[ix]", combine="x + y", seed="0")
    s_ = ctx.empty((), np.int64)
    f.fold([dx], n, s_)
    assert int(s_.get().reshape(-1)[0]) == int(x.sum(dtype=np.int64))
    say("scanl1")
    sc = ctx.skeleton(A.SKEL_SCANL1, "Word8", env=[W8], get="arrIn0_0[ix]", combine="(Word8)(x ^ y)")
    sc.scan([dx], n, o)
    got = o.get()
    ref = np.bitwise_xor.accumulate(x)
    assert np.array_equal(got[:100000], ref[:100000]) and np.array_equal(got[-100000:], ref[-100000:])
    say("permute")
    p = ctx.skeleton(A.SKEL_PERMUTE, "Int64", env=[W8], out_rank=1, get="(Int64)1", combine="x + y", combine_hint=A.COMBINE_ADD,
                     permutation="(Int64)arrIn0_0[ix]")
    h = ctx.empty(256, np.int64)
    p.permute([dx], n, ctx.array(np.zeros(256, np.int64)), h)
    assert np.array_equal(h.get(), np.bincount(x, minlength=256).astype(np.int64))
    say("foldSeg, 64-bit offsets")
    rng = np.random.default_rng(31)
    lens = rng.integers(0, 129, 1 << 25).astype(np.int64)           # 64 elements a segment on average
    lens[12345] = 300000                                            # and one that the workgroup folds together
    offs = np.concatenate([[0], np.cumsum(lens)])
    offs = offs[offs <= n]
    nseg = offs.size - 1
    assert offs[-1] > (1 << 31)
    want = np.add.reduceat(x[:offs[-1]], offs[:-1].clip(max=offs[-1] - 1), dtype=np.int64)
    want[offs[1:] == offs[:-1]] = 0                                 # (reduceat gives an empty segment its neighbour's first element)
    doffs = ctx.array(offs)
    for knobs in ("", "foldseg.giants=1"):
        with A.tuning(knobs, ctx):
            fsg = ctx.skeleton(A.SKEL_FOLDSEG, "Int32", env=[W8], out_rank=1, get="(Int32)arrIn0_0[ix]", combine="x + y", seed="3", seg_type="Int64")
        sums = ctx.empty(nseg, np.int32)
        fsg.foldseg([dx], int(offs[-1]), doffs, sums)
        assert np.array_equal(sums.get(), (want + 3).astype(np.int32)), knobs
        fsg.destroy()


def test_stencil_over_more_than_2_31_elements(A, ctx):
    h, w = 65536, 33000
    say("5-point stencil over", h * w, "Int8 elements")
    img = np.empty((h, w), np.int8)
    row = (np.arange(w, dtype=np.int64) * 5 % 97).astype(np.int8)
    for y in range(h):
        img[y] = np.roll(row, y % 131)
    s = ctx.skeleton(A.SKEL_STENCIL, "Int8", out_rank=2, taps=[(-1, 0), (0, -1), (0, 0), (0, 1), (1, 0)], boundary="clamp",
                     stencil_fn="(Int8)(t0 + t1 + t2 + t3 + t4)", stencil_in="Int8")
    b = ctx.empty((h, w), np.int8)
    s.stencil([], ctx.array(img), b)
    got = b.get()
    for y in (0, 1, 777, 32768, 65000, 65534, 65535):          # the rows on both sides of index 2^31 among them
        up, dn = img[max(y - 1, 0)].astype(np.int32), img[min(y + 1, h - 1)].astype(np.int32)
        c = img[y].astype(np.int32)
        left, right = np.concatenate([c[:1], c[:-1]]), np.concatenate([c[1:], c[-1:]])
        assert np.array_equal(got[y], (up + left + c + right + dn).astype(np.int8)), y
    del img, got, b
    # the same on an array of three columns, which goes an element a thread (with 64-bit indices: too many for 32)
    h, w = (1 << 31) // 3 + 3000, 3
    say("5-point stencil over", h * w, "Int8 elements in three columns")
    img = (np.arange(h * w, dtype=np.int64) * 7 % 101).astype(np.int8).reshape(h, w)
    b = ctx.empty((h, w), np.int8)
    s.stencil([], ctx.array(img), b)
    got = b.get()
    for y0 in (0, 1 << 20, (1 << 31) // 3 - 500, h - 1000):    # (the rows on both sides of index 2^31 among them)
        rows = np.arange(y0, y0 + 1000)
        c = img[rows].astype(np.int32)
        up, dn = img[np.maximum(rows - 1, 0)].astype(np.int32), img[np.minimum(rows + 1, h - 1)].astype(np.int32)
        left, right = np.concatenate([c[:, :1], c[:, :-1]], axis=1), np.concatenate([c[:, 1:], c[:, -1:]], axis=1)
        assert np.array_equal(got[rows], (up + left + c + right + dn).astype(np.int8)), y0


def test_the_device_header_s_multi_index_of_a_linear_index(A, ctx):
    """`acc_from_index<R>({extents}, ix)` in an element function: ranks 2 to 4 with extents that are no powers of two,
    a result without elements, and an array of more than 2^31 elements (64-bit arithmetic; rows on both sides of
    index 2^31 are looked at)."""
    for shape in ((7, 11), (37, 1, 53), (3, 5, 7, 11), (1000, 999), (0, 5)):
        r = len(shape)
        ext = ", ".join("shOut_%d" % d for d in range(r - 1, -1, -1))
        parts = " + ".join("%d * acc_from_index<%d>({%s}, ix).i[%d]" % (10 ** (2 * (r - 1 - d)), r, ext, d) for d in range(r))
        say("acc_from_index", shape)
        sk = ctx.skeleton(A.SKEL_GENERATE, "Int64", out_rank=r, get="(Int64)(%s)" % parts)
        out = ctx.empty(shape, np.int64)
        sk.map([], out)
        idx = np.indices(shape, dtype=np.int64) if all(shape) else np.zeros((r,) + shape, np.int64)
        want = sum(idx[d] * 10 ** (2 * (r - 1 - d)) for d in range(r))
        assert np.array_equal(out.get(), want), shape
    h, w = 46400, 46400                                   # 2 152 960 000 elements
    say("acc_from_index beyond 2^31 elements", h, w)
    sk = ctx.skeleton(A.SKEL_GENERATE, "Word8", out_rank=2,
                      get="(Word8)(acc_from_index<2>({shOut_1, shOut_0}, ix).i[0] * 7 + acc_from_index<2>({shOut_1, shOut_0}, ix).i[1])")
    out = ctx.empty((h, w), np.uint8)
    sk.map([], out)
    got = out.get()
    xs = np.arange(w, dtype=np.int64)
    for y in (0, 1, 46280, 46281, 46282, h - 1):            # (index 2^31 lies in row 46 281)
        assert np.array_equal(got[y], ((y * 7 + xs) & 255).astype(np.uint8)), y
