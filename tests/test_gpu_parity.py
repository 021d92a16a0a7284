"""Parity of the HIP skeletons against the CPU oracle, through the C ABI.

Bit-exact for integer / index work; Float32 tolerances are written at each
assertion.  Every case prints its name before touching the GPU so that a
fault names its case.
"""
import json
import os
import sys

import numpy as np
import pytest

import pyref

pytestmark = pytest.mark.gpu

rng = np.random.default_rng(77)
GOLDEN = os.path.join(os.path.dirname(__file__), "golden")

F32 = (1, "float")
I32 = (1, "Int32")

AFFINE_PREAMBLE = """
__device__ __forceinline__ Word32 affine16(Word32 x, Word32 y) {
  Word32 a1 = x >> 16, b1 = x & 0xffffu, a2 = y >> 16, b2 = y & 0xffffu;
  return (((a1 * a2) & 0xffffu) << 16) | ((a1 * b2 + b1) & 0xffffu);
}
"""


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
    p = c.props()
    say("device", p.name.decode(), p.arch.decode(), "CUs", p.compute_units, "LDS/block", p.lds_per_block,
        "wave", p.wavefront_size)
    yield c
    c.close()


SIZES = [0, 1, 2, 3, 5, 63, 64, 65, 4095, 4096, 4097, 32766, 32767, 32768, 32769, 65535, 98306, 100003, (1 << 21) + 17]


# --------------------------------------------------------------------------- map family

def test_zipwith_saxpy_generate(A, ctx, orc):
    mul = ctx.skeleton(A.SKEL_MAP, "float", env=[F32, F32], out_rank=1, get="arrIn0_0[ix] * arrIn1_0[ix]")
    saxpy = ctx.skeleton(A.SKEL_MAP, "float", env=[F32, F32], out_rank=1, get="2.5f * arrIn0_0[ix] + arrIn1_0[ix]")
    for n in SIZES:
        say("zipWith/saxpy n =", n)
        x = (rng.random(n) * 2 - 1).astype(np.float32)
        y = (rng.random(n) * 2 - 1).astype(np.float32)
        dx, dy, do = ctx.array(x), ctx.array(y), ctx.empty(n, np.float32)
        mul.map([dx, dy], do)
        assert np.array_equal(do.get(), x * y)
        saxpy.map([dx, dy], do)
        exp = (np.float32(2.5) * x).astype(np.float32) + y          # two roundings: contraction is off
        assert np.array_equal(do.get(), exp)
    say("generate 2-D iota")
    gen = ctx.skeleton(A.SKEL_GENERATE, "Int32", out_rank=2, get="(Int32)((ix / shOut_0) * 1000 + ix % shOut_0)")
    out = ctx.empty((37, 211), np.int32)
    gen.map([], out)
    yy, xx = np.mgrid[0:37, 0:211]
    assert np.array_equal(out.get(), (yy * 1000 + xx).astype(np.int32))


def test_backpermute_and_unaligned(A, ctx, orc):
    gather = ctx.skeleton(A.SKEL_TRANSFORM, "float", env=[F32, I32], out_rank=1, get="arrIn0_0[arrIn1_0[ix]]")
    for n in (1, 1000, 262147):
        say("backpermute n =", n)
        src = rng.random(5000).astype(np.float32)
        idx = rng.integers(0, 5000, n, dtype=np.int32)
        out = ctx.empty(n, np.float32)
        gather.map([ctx.array(src), ctx.array(idx)], out)
        assert np.array_equal(out.get(), orc.backpermute(src, idx))
    say("map on pointers that are only 4-byte aligned")
    copy = ctx.skeleton(A.SKEL_MAP, "float", env=[F32], out_rank=1, get="arrIn0_0[ix] + 1.0f")
    n = 10001
    x = rng.random(n + 3).astype(np.float32)
    dx, do = ctx.array(x), ctx.array(np.zeros(n + 3, np.float32))
    copy.map([dx.desc(shape=(n,), offset_elems=1)], do.desc(shape=(n,), offset_elems=3))
    got = do.get()
    assert np.array_equal(got[3:], x[1:n + 1] + np.float32(1)) and np.all(got[:3] == 0)


# --------------------------------------------------------------------------- fold

def test_dot_product(A, ctx, orc):
    dot = ctx.skeleton(A.SKEL_FOLD, "float", env=[F32, F32], out_rank=0, get="arrIn0_0[ix] * arrIn1_0[ix]",
                       combine="x + y", seed="0.0f")
    out = ctx.empty((), np.float32)
    for n in SIZES + [1 << 22]:
        say("dot n =", n)
        x = (rng.random(n) * 2 - 1).astype(np.float32)
        y = (rng.random(n) * 2 - 1).astype(np.float32)
        dot.fold([ctx.array(x), ctx.array(y)], n, out)
        got = float(out.get())
        truth, cond = orc.dot_f64(x, y), orc.dot_abs_f64(x, y)
        # tolerance: 1e-4 relative to the interpreter's (sequential Float32) result, with the
        # denominator floored by the rounding noise of that sequential sum itself
        ref = float(orc.dot_f32(x, y))
        floor = n * 2.0 ** -24 * cond
        assert abs(got - ref) <= 1e-4 * max(abs(ref), floor) + 1e-30, (n, got, ref)
        # and against the Float64 truth the tree-shaped GPU sum is far inside the classic bound
        assert abs(got - truth) <= 64 * 2.0 ** -24 * cond + 1e-30
    say("dot of small integers is exact in any order")
    n = 1 << 20
    xi = rng.integers(-8, 8, n).astype(np.float32)
    yi = rng.integers(-8, 8, n).astype(np.float32)
    dot.fold([ctx.array(xi), ctx.array(yi)], n, out)
    assert float(out.get()) == float(orc.dot_f32(xi, yi))


def test_fold_integers_and_errors(A, ctx, orc):
    add = ctx.skeleton(A.SKEL_FOLD, "Int32", env=[I32], out_rank=0, get="arrIn0_0[ix]", combine="x + y", seed="42")
    mx = ctx.skeleton(A.SKEL_FOLD1, "Int32", env=[I32], out_rank=0, get="arrIn0_0[ix]", combine="acc_max(x, y)")
    add64 = ctx.skeleton(A.SKEL_FOLD, "Int64", env=[(1, "Int64")], out_rank=0, get="arrIn0_0[ix]", combine="x + y", seed="0")
    out = ctx.empty((), np.int32)
    out64 = ctx.empty((), np.int64)
    for n in SIZES:
        say("fold (+) / fold1 max n =", n)
        x = rng.integers(-1000, 1000, n, dtype=np.int32)
        dx = ctx.array(x)
        add.fold([dx], n, out)
        assert int(out.get()) == int(orc.fold(orc.OP_ADD, x, seed=42))
        if n > 0:
            mx.fold([dx], n, out)
            assert int(out.get()) == int(x.max())
        x64 = rng.integers(-2**40, 2**40, n, dtype=np.int64)
        add64.fold([ctx.array(x64)], n, out64)
        assert int(out64.get()) == int(x64.sum())
    say("fold1 of an empty array is an error")
    with pytest.raises(A.AccError) as e:
        mx.fold([ctx.array(np.zeros(0, np.int32))], 0, out)
    assert e.value.code == A.ERR_INVALID and "empty array" in e.value.message
    say("repeated launches reuse the ticket")
    x = rng.integers(-1000, 1000, 1 << 20, dtype=np.int32)
    dx = ctx.array(x)
    for _ in range(5):
        add.fold([dx], x.size, out)
        assert int(out.get()) == int(x.sum(dtype=np.int64)) + 42


def test_fold_innermost_dimension(A, ctx, orc):
    add = ctx.skeleton(A.SKEL_FOLD, "Int32", env=[(2, "Int32")], out_rank=1, get="arrIn0_0[ix]", combine="x + y", seed="7")
    mn = ctx.skeleton(A.SKEL_FOLD1, "float", env=[(2, "float")], out_rank=1, get="arrIn0_0[ix]", combine="acc_min(x, y)")
    for shape in [(1, 1), (3, 0), (17, 5), (300, 64), (33, 1000), (1000, 129)]:
        say("fold along rows", shape)
        x = rng.integers(-100, 100, shape, dtype=np.int32)
        out = ctx.empty(shape[0], np.int32)
        add.fold([ctx.array(x)], shape, out)
        assert np.array_equal(out.get(), orc.fold(orc.OP_ADD, x, seed=7))
        if shape[1] > 0:
            xf = rng.random(shape).astype(np.float32)
            outf = ctx.empty(shape[0], np.float32)
            mn.fold([ctx.array(xf)], shape, outf)
            assert np.array_equal(outf.get(), xf.min(axis=1))


# --------------------------------------------------------------------------- scans

def _run_scan(A, ctx, kind, elt, x, combine, seed, preamble=None, env_type=None):
    n = x.size
    sk = ctx.skeleton(A.SCAN_KINDS[kind], elt, env=[(1, env_type or elt)], get="arrIn0_0[ix]", combine=combine,
                      seed=seed, preamble=preamble)
    return sk


@pytest.mark.parametrize("kind", ["scanl", "scanl1", "scanl'", "scanr", "scanr1", "scanr'"])
def test_scan_int32_add(A, ctx, orc, kind):
    seeded = not kind.endswith("1")
    sk = ctx.skeleton(A.SCAN_KINDS[kind], "Int32", env=[I32], get="arrIn0_0[ix]", combine="x + y",
                      seed="5" if seeded else None)
    for n in SIZES + [(1 << 22) + 4099]:
        say(kind, "(+) Int32 n =", n)
        x = rng.integers(0, 16, n, dtype=np.int32)
        plus = 1 if kind in ("scanl", "scanr") else 0
        out = ctx.array(np.full(n + plus + 2, -777, np.int32))      # two guard words past the end
        tot = ctx.array(np.array(-1, np.int32))
        sk.scan([ctx.array(x)], n, out.desc(shape=(n + plus,)), tot if kind.endswith("'") else None)
        got = out.get()
        assert np.all(got[n + plus:] == -777), "wrote past the end"
        exp = orc.scan(kind, orc.OP_ADD, x, seed=5)
        if kind.endswith("'"):
            assert np.array_equal(got[:n], exp[0]) and int(tot.get().reshape(-1)[0]) == int(np.asarray(exp[1]).reshape(-1)[0])
        else:
            assert np.array_equal(got[:n + plus], exp)


@pytest.mark.parametrize("small_below_kb", ["0", "2000000"])
def test_scan_tiles_of_either_size_on_ragged_ends(A, ctx, orc, tuned, small_below_kb):
    """the driver takes small tiles for arrays up to 12 MB and large ones above: here each kind of tile is forced on
    sizes either side of that, with ends that fall anywhere in a vector, a row and a tile"""
    tuned("scan.small_below_kb=" + small_below_kb)
    sizes = [1, 3, 4, 5, 255, 1027, 4096, 4097, 32767, 32768, 32769, 32771, 65537, 98307, 5 * 32768 + 2, (1 << 21) + 4101]
    for kind in ("scanl", "scanl1", "scanr", "scanr1", "scanl'", "scanr'"):
        seeded = not kind.endswith("1")
        sk = ctx.skeleton(A.SCAN_KINDS[kind], "Int32", env=[I32], get="arrIn0_0[ix]", combine="x + y",
                          seed="5" if seeded else None)
        for n in sizes:
            say(kind, "(+) Int32, scan.small_below_kb =", small_below_kb, "n =", n)
            x = rng.integers(-9, 16, n, dtype=np.int32)
            plus = 1 if kind in ("scanl", "scanr") else 0
            out = ctx.array(np.full(n + plus + 2, -777, np.int32))
            tot = ctx.array(np.array(-1, np.int32))
            sk.scan([ctx.array(x)], n, out.desc(shape=(n + plus,)), tot if kind.endswith("'") else None)
            got = out.get()
            assert np.all(got[n + plus:] == -777), "wrote past the end"
            exp = orc.scan(kind, orc.OP_ADD, x, seed=5)
            if kind.endswith("'"):
                assert np.array_equal(got[:n], exp[0]) and int(tot.get().reshape(-1)[0]) == int(np.asarray(exp[1]).reshape(-1)[0])
            else:
                assert np.array_equal(got[:n + plus], exp)
    # elements of 1 and 8 bytes (16 and 2 a vector), from the left and from the right
    for kind, fn in (("scanl1", np.maximum.accumulate), ("scanr1", lambda v: np.maximum.accumulate(v[::-1])[::-1])):
        for ty, dt in (("Int8", np.int8), ("double", np.float64)):
            sk = ctx.skeleton(A.SCAN_KINDS[kind], ty, env=[(1, ty)], get="arrIn0_0[ix]", combine="acc_max(x, y)")
            for n in (1, 15, 17, 2049, 131071, 131073, 300001):
                say(kind, "max", ty, "scan.small_below_kb =", small_below_kb, "n =", n)
                x = (rng.standard_normal(n) * 40).astype(dt)
                out = ctx.empty(n, dt)
                sk.scan([ctx.array(x)], n, out)
                assert np.array_equal(out.get(), fn(x)), (kind, ty, n)
    # pairs (one array per component), from the left with a seed and from the right without
    for kind in ("scanl", "scanr1"):
        pr = ctx.skeleton(A.SCAN_KINDS[kind], "Int32, float", env=[(1, "Int32"), (1, "float")], get="acc_elt{arrIn0_0[ix], arrIn1_0[ix]}",
                          combine="acc_elt{x.a1 + y.a1, acc_max(x.a0, y.a0)}", seed="acc_elt{3, -1.0f}" if kind == "scanl" else None)
        for n in (5, 16385, 100003):
            say(kind, "of pairs, scan.small_below_kb =", small_below_kb, "n =", n)
            a, b = rng.integers(-9, 9, n).astype(np.int32), rng.random(n).astype(np.float32)
            plus = 1 if kind == "scanl" else 0
            out = A.TupleArray([ctx.empty(n + plus, np.int32), ctx.empty(n + plus, np.float32)])
            pr.scan([ctx.array(a), ctx.array(b)], n, out)
            if kind == "scanl":
                want_a = np.concatenate([[3], 3 + np.cumsum(a, dtype=np.int64)]).astype(np.int32)
                want_b = np.concatenate([[-1.0], np.maximum.accumulate(b)]).astype(np.float32)
            else:
                want_a = np.cumsum(a[::-1], dtype=np.int64)[::-1].astype(np.int32)
                want_b = np.maximum.accumulate(b[::-1])[::-1]
            assert np.array_equal(out.comps[0].get(), want_a) and np.array_equal(out.comps[1].get(), want_b), (kind, n)


def test_scan_repeated_launches_and_sizes_interleaved(A, ctx, orc):
    """the tile descriptors and the ticket counter are reused between launches"""
    sk = ctx.skeleton(A.SKEL_SCANL, "Int32", env=[I32], get="arrIn0_0[ix]", combine="x + y", seed="0")
    for n in [1 << 20, 1000, (1 << 21) + 3, 7, 1 << 20, 1 << 16]:
        say("scanl relaunch n =", n)
        x = rng.integers(0, 16, n, dtype=np.int32)
        out = ctx.empty(n + 1, np.int32)
        sk.scan([ctx.array(x)], n, out)
        assert np.array_equal(out.get(), orc.scan("scanl", orc.OP_ADD, x, seed=0))


@pytest.mark.parametrize("kind", ["scanl", "scanl1", "scanl'", "scanr", "scanr1", "scanr'"])
def test_scan_noncommutative(A, ctx, orc, kind):
    seeded = not kind.endswith("1")
    sk = ctx.skeleton(A.SCAN_KINDS[kind], "Word32", env=[(1, "Word32")], get="arrIn0_0[ix]",
                      combine="affine16(x, y)", seed="0x00030005u" if seeded else None, preamble=AFFINE_PREAMBLE)
    for n in [1, 2, 64, 1000, 4096, 4097, 50001]:
        say(kind, "affine16 n =", n)
        x = rng.integers(0, 2**32, n, dtype=np.uint32)
        plus = 1 if kind in ("scanl", "scanr") else 0
        out = ctx.empty(n + plus, np.uint32)
        tot = ctx.empty((), np.uint32)
        sk.scan([ctx.array(x)], n, out, tot if kind.endswith("'") else None)
        exp = orc.scan(kind, orc.OP_AFFINE16, x.view(np.int32), seed=0x00030005)
        if kind.endswith("'"):
            assert np.array_equal(out.get().view(np.int32), exp[0]) and int(tot.get().view(np.int32).reshape(-1)[0]) == int(np.asarray(exp[1]).reshape(-1)[0])
        else:
            assert np.array_equal(out.get().view(np.int32), exp)


def test_scan_wide_and_float_elements(A, ctx, orc):
    for kind in ("scanl", "scanr1", "scanl'"):
        seeded = not kind.endswith("1")
        sk = ctx.skeleton(A.SCAN_KINDS[kind], "Int64", env=[(1, "Int64")], get="arrIn0_0[ix]", combine="x + y",
                          seed="11" if seeded else None)
        for n in [1, 2047, 2048, 2049, 300001]:
            say(kind, "Int64 n =", n)
            x = rng.integers(-2**40, 2**40, n, dtype=np.int64)
            plus = 1 if kind in ("scanl", "scanr") else 0
            out = ctx.empty(n + plus, np.int64)
            tot = ctx.empty((), np.int64)
            sk.scan([ctx.array(x)], n, out, tot if kind.endswith("'") else None)
            exp = orc.scan(kind, orc.OP_ADD, x, seed=11)
            if kind.endswith("'"):
                assert np.array_equal(out.get(), exp[0]) and int(tot.get().reshape(-1)[0]) == int(np.asarray(exp[1]).reshape(-1)[0])
            else:
                assert np.array_equal(out.get(), exp)
    say("scanl1 (+) Float32: tolerance 1e-5 relative to the running magnitude")
    sk = ctx.skeleton(A.SKEL_SCANL1, "float", env=[F32], get="arrIn0_0[ix]", combine="x + y")
    n = 200000
    x = rng.random(n).astype(np.float32)
    out = ctx.empty(n, np.float32)
    sk.scan([ctx.array(x)], n, out)
    truth = np.cumsum(x.astype(np.float64))
    assert np.max(np.abs(out.get() - truth) / truth) <= 1e-5
    say("scanl1 max Float64")
    sk = ctx.skeleton(A.SKEL_SCANL1, "double", env=[(1, "double")], get="arrIn0_0[ix]", combine="acc_max(x, y)")
    xd = rng.random(70001)
    outd = ctx.empty(xd.size, np.float64)
    sk.scan([ctx.array(xd)], xd.size, outd)
    assert np.array_equal(outd.get(), np.maximum.accumulate(xd))


def test_scan_fused_producer(A, ctx, orc):
    """the input of a scan is a delayed array: here zipWith (*) fused in"""
    sk = ctx.skeleton(A.SKEL_SCANL, "Int32", env=[I32, I32], get="arrIn0_0[ix] * arrIn1_0[ix]", combine="x + y", seed="0")
    n = 123457
    a = rng.integers(-3, 4, n, dtype=np.int32)
    b = rng.integers(-3, 4, n, dtype=np.int32)
    out = ctx.empty(n + 1, np.int32)
    say("scanl over fused zipWith")
    sk.scan([ctx.array(a), ctx.array(b)], n, out)
    assert np.array_equal(out.get(), orc.scan("scanl", orc.OP_ADD, a * b, seed=0))


# --------------------------------------------------------------------------- permute

def test_histograms(A, ctx, orc):
    import workloads as wl
    hist = ctx.skeleton(A.SKEL_PERMUTE, "Int32", env=[I32], out_rank=1, get="1", combine="x + y",
                        permutation="arrIn0_0[ix]", combine_hint=A.COMBINE_ADD)
    for name, keys, bins in [("uniform 256", wl.uniform_i32(1, 1 << 22, 256), 256),
                             ("uniform 7", wl.uniform_i32(2, 100003, 7), 7),
                             ("zipf 65536", wl.zipf_i32(3, 1 << 22, 65536), 65536),
                             ("uniform 1M bins", wl.uniform_i32(4, 1 << 21, 1 << 20), 1 << 20),
                             ("empty source", np.zeros(0, np.int32), 16)]:
        say("histogram", name)
        dfl = rng.integers(0, 5, bins, dtype=np.int32)
        out = ctx.empty(bins, np.int32)
        hist.permute([ctx.array(keys)], keys.size, ctx.array(dfl), out)
        got = out.get()
        assert np.array_equal(got, orc.permute(orc.OP_ADD, dfl, keys))
        assert int(got.sum()) - int(dfl.sum()) == keys.size
    say("histogram with ignored and out-of-range targets, in place over the defaults")
    keys = wl.uniform_i32(5, 500000, 300)
    keys[::5] = -1
    dfl = rng.integers(0, 5, 300, dtype=np.int32)
    out = ctx.array(dfl)
    hist.permute([ctx.array(keys)], keys.size, out, out)
    assert np.array_equal(out.get(), orc.permute(orc.OP_ADD, dfl, keys))


def test_permute_other_combines(A, ctx, orc):
    n, bins = 300000, 1000
    dst = rng.integers(0, bins, n, dtype=np.int32)
    dst[::11] = -1
    src = rng.integers(-10**6, 10**6, n, dtype=np.int32)
    dd, ds = ctx.array(dst), ctx.array(src)
    for name, hint, comb, op in [("min", A.COMBINE_MIN, "acc_min(x, y)", orc.OP_MIN),
                                 ("max", A.COMBINE_MAX, "acc_max(x, y)", orc.OP_MAX),
                                 ("add generic (CAS loop)", A.COMBINE_GENERIC, "x + y", orc.OP_ADD),
                                 ("weighted add", A.COMBINE_ADD, "x + y", orc.OP_ADD)]:
        say("permute", name)
        sk = ctx.skeleton(A.SKEL_PERMUTE, "Int32", env=[I32, I32], out_rank=1, get="arrIn1_0[ix]", combine=comb,
                          permutation="arrIn0_0[ix]", combine_hint=hint)
        dfl = rng.integers(-100, 100, bins, dtype=np.int32)
        out = ctx.empty(bins, np.int32)
        sk.permute([dd, ds], n, ctx.array(dfl), out)
        assert np.array_equal(out.get(), orc.permute(op, dfl, dst, src))
    say("permute Float32 (+): order of arrival differs, tolerance 1e-4 of the absolute sum")
    sk = ctx.skeleton(A.SKEL_PERMUTE, "float", env=[I32, F32], out_rank=1, get="arrIn1_0[ix]", combine="x + y",
                      permutation="arrIn0_0[ix]", combine_hint=A.COMBINE_ADD)
    srcf = (rng.random(n) * 2 - 1).astype(np.float32)
    dfl = np.zeros(bins, np.float32)
    out = ctx.empty(bins, np.float32)
    sk.permute([dd, ctx.array(srcf)], n, ctx.array(dfl), out)
    ok = dst >= 0
    truth = np.bincount(dst[ok], weights=srcf[ok].astype(np.float64), minlength=bins)
    mag = np.bincount(dst[ok], weights=np.abs(srcf[ok]).astype(np.float64), minlength=bins)
    assert np.all(np.abs(out.get() - truth) <= 1e-4 * mag + 1e-30)
    say("permute with a unique target per element (a scatter): FIRST-style combine keeps the new value")
    perm = rng.permutation(5000).astype(np.int32)
    vals = rng.integers(0, 10**6, 5000, dtype=np.int32)
    sk = ctx.skeleton(A.SKEL_PERMUTE, "Int32", env=[I32, I32], out_rank=1, get="arrIn1_0[ix]", combine="x",
                      permutation="arrIn0_0[ix]")
    out = ctx.empty(5000, np.int32)
    sk.permute([ctx.array(perm), ctx.array(vals)], 5000, ctx.array(np.full(5000, -1, np.int32)), out)
    assert np.array_equal(out.get(), orc.permute(orc.OP_FIRST, np.full(5000, -1, np.int32), perm, vals))


def test_permute_whose_first_workgroup_copies_the_defaults(A, ctx):
    """few enough targets for one LDS table and few enough workgroups for atomics: one launch, workgroup 0 copies
    the defaults into the result while the others read the source, and they look at a word it leaves before they
    add their bins.  Defaults that are not the identity, several numbers of targets, Int32 / Int64 / Float32 sums
    and a maximum, launches that follow one another on one result (the word is tagged anew every time), a result
    that is its own defaults (no copy), and the same with the copy as a launch of its own."""
    import os
    rng_ = np.random.default_rng(77)
    for ctype, dt in (("Int32", np.int32), ("Int64", np.int64), ("float", np.float32)):
        for combine, hint, at in (("x + y", A.COMBINE_ADD, np.add.at), ("acc_max(x, y)", A.COMBINE_MAX, np.maximum.at)):
            for tune in ("", "permute.inline_fill=0"):
                knobs = A.tuning(tune, ctx)
                knobs.__enter__()
                try:
                    sk = ctx.skeleton(A.SKEL_PERMUTE, ctype, env=[I32, (1, ctype)], out_rank=1, get="arrIn1_0[ix]", combine=combine,
                                      permutation="arrIn0_0[ix]", combine_hint=hint)
                    for bins, n in ((1, 5000), (7, 1), (256, 1 << 22), (4097, 1 << 20), (40960, (1 << 21) + 3)):
                        say("permute, defaults copied inside the launch", ctype, combine, tune, "bins", bins, "n", n)
                        keys = rng_.integers(-2, bins + 2, n).astype(np.int32)
                        src = rng_.integers(0, 9, n).astype(dt)
                        dfl = rng_.integers(1, 5, bins).astype(dt)
                        ok = (keys >= 0) & (keys < bins)
                        ref = dfl.astype(np.int64)
                        at(ref, keys[ok], src[ok].astype(np.int64))
                        out = ctx.array(np.full(bins, 99, dt))
                        dk, ds_, dd = ctx.array(keys), ctx.array(src), ctx.array(dfl)
                        for _ in range(3):                             # the same result three times over
                            sk.permute([dk, ds_], n, dd, out)
                            assert np.array_equal(out.get(), ref.astype(dt))
                        acc = ctx.array(dfl)                           # the result is its own defaults: it accumulates
                        sk.permute([dk, ds_], n, acc, acc)
                        assert np.array_equal(acc.get(), ref.astype(dt))
                    sk.destroy()
                finally:
                    knobs.__exit__()


def test_permute_hinted_combines_over_windows_of_targets(A, ctx):
    """more targets than one LDS table holds: 2, 4 and 16 windows, every hinted operator, Int32 and Int64 elements,
    strays and `ignore` among the targets, a last window that is not full"""
    n = 1 << 21
    src = rng.integers(-10**6, 10**6, n, dtype=np.int32)
    ds = ctx.array(src)
    for bins in (50001, 150000, 500003):
        dst = rng.integers(-3, bins + 3, n).astype(np.int32)
        dst[::13] = -1
        dd = ctx.array(dst)
        ok = (dst >= 0) & (dst < bins)
        for name, hint, comb, ufunc in [("add", A.COMBINE_ADD, "x + y", np.add), ("min", A.COMBINE_MIN, "acc_min(x, y)", np.minimum),
                                        ("max", A.COMBINE_MAX, "acc_max(x, y)", np.maximum), ("xor", A.COMBINE_XOR, "x ^ y", np.bitwise_xor),
                                        ("and", A.COMBINE_AND, "x & y", np.bitwise_and), ("or", A.COMBINE_OR, "x | y", np.bitwise_or)]:
            say("hinted permute", name, "into", bins, "targets")
            sk = ctx.skeleton(A.SKEL_PERMUTE, "Int32", env=[I32, I32], out_rank=1, get="arrIn1_0[ix]", combine=comb,
                              permutation="arrIn0_0[ix]", combine_hint=hint)
            dfl = rng.integers(-100, 100, bins, dtype=np.int32)
            out = ctx.empty(bins, np.int32)
            sk.permute([dd, ds], n, ctx.array(dfl), out)
            ref = dfl.copy()
            ufunc.at(ref, dst[ok], src[ok])
            assert np.array_equal(out.get(), ref)
        say("Int64 sums into", bins, "targets")
        sk = ctx.skeleton(A.SKEL_PERMUTE, "Int64", env=[I32, I32], out_rank=1, get="(Int64)arrIn1_0[ix] * 1000003", combine="x + y",
                          permutation="arrIn0_0[ix]", combine_hint=A.COMBINE_ADD)
        out = ctx.empty(bins, np.int64)
        sk.permute([dd, ds], n, ctx.array(np.zeros(bins, np.int64)), out)
        ref = np.zeros(bins, np.int64)
        np.add.at(ref, dst[ok], src[ok].astype(np.int64) * 1000003)
        assert np.array_equal(out.get(), ref)


def test_counting_into_a_table_of_16_bit_counts(A, ctx):
    """a permute that counts (integer `+` over a source spelt as a small constant) into more targets than one LDS
    table of whole elements holds, but few enough for 16-bit counts: hot targets whose count passes 0x8000 in every
    workgroup many times over, odd numbers of targets, ignored and stray indices, defaults, Int64 and Word32 results,
    keys that are not 16-byte aligned"""
    import workloads as wl
    n = 1 << 24
    cases = [("zipf", wl.zipf_i32(7, n, 65536), 65536), ("uniform", wl.uniform_i32(8, n, 65535), 65535),
             ("one hot target", np.full(n, 4242, np.int32), 50001),
             ("four hot targets in two words", (rng.integers(0, 4, n) + 70000).astype(np.int32), 81919)]
    # (a table whose halves are whole 128-bit vectors but no whole number of a wave's 256 words: 65552 targets)
    cases.append(("hot targets at the ends of the table's quarters", rng.choice(np.array([0, 16387, 16388, 32775, 32776, 49163, 49164, 65551], np.int32), n), 65552))
    strays = rng.integers(-5, 65536 + 5, 1 << 22).astype(np.int32)
    strays[::7] = -1
    cases.append(("strays and ignore", strays, 65536))
    for ctype, dt, lit in (("Int32", np.int32, "1"), ("Int64", np.int64, "((Int64)(1))"), ("Word32", np.uint32, "3u")):
        sk = ctx.skeleton(A.SKEL_PERMUTE, ctype, env=[I32], out_rank=1, get=lit, combine="x + y",
                          permutation="arrIn0_0[ix]", combine_hint=A.COMBINE_ADD)
        w = 3 if lit == "3u" else 1
        for name, keys, bins in cases:
            say("counting", ctype, name, "into", bins)
            dfl = rng.integers(0, 1000, bins).astype(dt)
            out = ctx.empty(bins, dt)
            dk = ctx.array(np.concatenate([np.zeros(1, np.int32), keys]))
            for view in (dk.desc(shape=(keys.size,), offset_elems=1), ctx.array(keys)):   # 4 bytes off a 16-byte boundary, then on one
                sk.permute([view], keys.size, ctx.array(dfl), out)
                ok = (keys >= 0) & (keys < bins)
                ref = dfl + (np.bincount(keys[ok], minlength=bins) * w).astype(dt)
                assert np.array_equal(out.get(), ref)


def test_16_bit_counts_with_large_addends_and_with_lanes_made_to_wait(A, ctx):
    """the same table taken for a source that is not a constant (`permute.narrow=2`): addends above 3 and negative
    ones go to the result directly, the others through the counts; and with the mark at which a lane waits for a
    pending correction set as low as it goes, so that lanes do wait, on hot targets"""
    import os
    n, bins = 1 << 23, 60001
    dst = rng.integers(0, 40, n).astype(np.int32) * 1500           # 40 hot targets
    dst[::9] = rng.integers(-2, bins + 2, dst[::9].size)
    src = rng.integers(-2, 8, n).astype(np.int32)
    ok = (dst >= 0) & (dst < bins)
    knobs = A.tuning("permute.narrow=2,permute.narrow_stop=32769", ctx)
    knobs.__enter__()
    try:
        say("weighted sums through 16-bit counts, waits forced")
        sk = ctx.skeleton(A.SKEL_PERMUTE, "Int32", env=[I32, I32], out_rank=1, get="arrIn1_0[ix] ", combine="x + y",
                          permutation="arrIn0_0[ix]", combine_hint=A.COMBINE_ADD)
        dfl = rng.integers(-100, 100, bins, dtype=np.int32)
        out = ctx.empty(bins, np.int32)
        sk.permute([ctx.array(dst), ctx.array(src)], n, ctx.array(dfl), out)
        ref = dfl.copy()
        np.add.at(ref, dst[ok], src[ok])
        assert np.array_equal(out.get(), ref)
        say("counting with waits forced, one hot target")
        sk = ctx.skeleton(A.SKEL_PERMUTE, "Int32", env=[I32], out_rank=1, get="(1)", combine="x + y",
                          permutation="arrIn0_0[ix]", combine_hint=A.COMBINE_ADD)
        keys = np.full(1 << 24, 31, np.int32)
        keys[::3] = 30
        out = ctx.empty(bins, np.int32)
        sk.permute([ctx.array(keys)], keys.size, ctx.array(dfl), out)
        assert np.array_equal(out.get(), dfl + np.bincount(keys, minlength=bins).astype(np.int32))
    finally:
        knobs.__exit__()


# --------------------------------------------------------------------------- stencil

GAUSS_TAPS = [(dy, dx) for dy in (-1, 0, 1) for dx in (-1, 0, 1)]
LAPLACE_TAPS = [(-1, 0), (0, -1), (0, 0), (0, 1), (1, 0)]


@pytest.mark.parametrize("mode", ["clamp", "mirror", "wrap", "constant"])
def test_stencil_2d(A, ctx, orc, mode):
    gauss = ctx.skeleton(A.SKEL_STENCIL, "float", out_rank=2, taps=GAUSS_TAPS,
                         stencil_fn=A.linear_stencil_fn([1, 2, 1, 2, 4, 2, 1, 2, 1], 16), boundary=mode,
                         boundary_constant="0.25f")
    lap = ctx.skeleton(A.SKEL_STENCIL, "float", out_rank=2, taps=LAPLACE_TAPS,
                       stencil_fn=A.linear_stencil_fn([1, 1, -4, 1, 1]), boundary=mode, boundary_constant="0.25f")
    for shape in [(5, 5), (7, 3), (3, 64), (33, 70), (16, 256), (300, 517), (1024, 1024), (531, 1028)]:
        say("stencil", mode, shape)
        img = rng.random(shape).astype(np.float32)
        d, o = ctx.array(img), ctx.empty(shape, np.float32)
        gauss.stencil([], d, o)
        exp = orc.stencil2d(img, orc.GAUSS3X3, divisor=16.0, mode=mode, constant=0.25)
        assert np.max(np.abs(o.get() - exp)) <= 1e-5          # stated tolerance; in practice identical bits
        assert np.array_equal(o.get(), exp)
        lap.stencil([], d, o)
        exp = orc.stencil2d(img, orc.LAPLACE5, mode=mode, constant=0.25)
        assert np.max(np.abs(o.get() - exp)) <= 1e-5
        assert np.array_equal(o.get(), exp)


def test_stencil_iterated_and_asymmetric(A, ctx, orc):
    gauss = ctx.skeleton(A.SKEL_STENCIL, "float", out_rank=2, taps=GAUSS_TAPS,
                         stencil_fn=A.linear_stencil_fn([1, 2, 1, 2, 4, 2, 1, 2, 1], 16), boundary="clamp")
    for shape, iters in [((512, 768), 10), ((100, 260), 3), ((64, 256), 0)]:
        say("gaussian x", iters, shape)
        img = rng.random(shape).astype(np.float32)
        a, b = ctx.array(img), ctx.empty(shape, np.float32)
        res = gauss.stencil_iterate([], a, b, iters)
        exp = orc.stencil2d(img, orc.GAUSS3X3, divisor=16.0, mode="clamp", iters=iters)
        assert np.max(np.abs(res.get() - exp)) <= 1e-5
    say("asymmetric taps, radius 2")
    taps = [(-2, 1, 3.0), (0, -2, -2.0), (1, 0, 5.0), (2, 2, 1.0)]
    sk = ctx.skeleton(A.SKEL_STENCIL, "float", out_rank=2, taps=[(t[0], t[1]) for t in taps],
                      stencil_fn=A.linear_stencil_fn([t[2] for t in taps]), boundary="wrap")
    img = rng.integers(0, 50, (70, 300)).astype(np.float32)
    o = ctx.empty(img.shape, np.float32)
    sk.stencil([], ctx.array(img), o)
    assert np.array_equal(o.get(), orc.stencil2d(img, taps, mode="wrap"))


def test_stencil_1d(A, ctx, orc):
    for mode in ("clamp", "mirror", "wrap", "constant"):
        sk = ctx.skeleton(A.SKEL_STENCIL, "float", out_rank=1, taps=[(0, -1), (0, 0), (0, 1)],
                          stencil_fn=A.linear_stencil_fn([1, -2, 1]), boundary=mode, boundary_constant="0.5f")
        for n in (1, 2, 5, 1023, 1024, 1025, 100001):
            if n < 2 and mode in ("mirror",):
                continue                                        # the index maps assume the array spans the stencil
            say("stencil 1-D", mode, n)
            v = rng.random(n).astype(np.float32)
            o = ctx.empty(n, np.float32)
            sk.stencil([], ctx.array(v), o)
            exp = orc.stencil1d(v, [(-1, 1.0), (0, -2.0), (1, 1.0)], mode=mode, constant=0.5)
            assert np.array_equal(o.get(), exp)


# --------------------------------------------------------------------------- foldSeg / SMVM

def _csr(nrows, ncols, mean, empty_every=0):
    lens = rng.poisson(mean, nrows).astype(np.int32)
    if empty_every:
        lens[::empty_every] = 0
    offs = np.concatenate([[0], np.cumsum(lens)]).astype(np.int32)
    nnz = int(offs[-1])
    cols = rng.integers(0, ncols, nnz, dtype=np.int32)
    vals = (rng.random(nnz) * 2 - 1).astype(np.float32)
    x = (rng.random(ncols) * 2 - 1).astype(np.float32)
    return vals, cols, offs, x


@pytest.mark.parametrize("right", [False, True])
def test_smvm(A, ctx, orc, right):
    smvm = ctx.skeleton(A.SKEL_FOLDSEG, "float", env=[F32, I32, F32], get="arrIn0_0[ix] * arrIn2_0[arrIn1_0[ix]]",
                        combine="x + y", seed="0.0f", flags=A.FLAG_FOLD_RIGHT if right else 0)
    d = orc.DIR_RIGHT if right else orc.DIR_LEFT
    for nrows, ncols, mean, ee in [(1, 10, 3, 0), (255, 100, 8, 0), (256, 100, 32, 7), (257, 100, 32, 0),
                                   (50000, 4096, 32, 9), (3000, 512, 700, 4), (40, 64, 9000, 3), (100000, 1000, 1, 2)]:
        say("smvm right" if right else "smvm left", nrows, "rows, mean length", mean)
        vals, cols, offs, x = _csr(nrows, ncols, mean, ee)
        y = ctx.array(np.full(nrows, np.nan, np.float32))
        smvm.foldseg([ctx.array(vals), ctx.array(cols), ctx.array(x)], vals.size, ctx.array(offs), y)
        exp = orc.smvm_f32(vals, cols, offs, x, d)
        got = y.get()
        # short segments (one lane each) are folded in index order with the sequential association: identical bits.
        # Segments long on average go to a wave or a workgroup each: still index order, another association, so the
        # last bits may differ.  (Stated tolerance for this configuration, checked below for both: 1e-4 relative per row.)
        if vals.size // nrows < 128:
            assert np.array_equal(got, exp)
        y64, yabs = orc.smvm_f64(vals, cols, offs, x)
        assert np.all(np.abs(got - y64) <= 1e-4 * np.maximum(np.abs(y64), 1e-3 * yabs) + 1e-30)


def test_foldseg_integers(A, ctx, orc):
    add = ctx.skeleton(A.SKEL_FOLDSEG, "Int32", env=[I32], get="arrIn0_0[ix]", combine="x + y", seed="3")
    mx = ctx.skeleton(A.SKEL_FOLD1SEG, "Int32", env=[I32], get="arrIn0_0[ix]", combine="acc_max(x, y)")
    for nseg, mean in [(1, 5), (1000, 3), (70000, 20), (513, 1500)]:
        say("foldSeg Int32", nseg, "segments, mean", mean)
        lens = rng.poisson(mean, nseg).astype(np.int32)
        offs = np.concatenate([[0], np.cumsum(lens)]).astype(np.int32)
        x = rng.integers(-1000, 1000, int(offs[-1]), dtype=np.int32)
        out = ctx.empty(nseg, np.int32)
        add.foldseg([ctx.array(x)], x.size, ctx.array(offs), out)
        assert np.array_equal(out.get(), orc.foldseg(orc.OP_ADD, x, offs, seed=3))
        lens1 = np.maximum(lens, 1)
        offs1 = np.concatenate([[0], np.cumsum(lens1)]).astype(np.int32)
        x1 = rng.integers(-1000, 1000, int(offs1[-1]), dtype=np.int32)
        mx.foldseg([ctx.array(x1)], x1.size, ctx.array(offs1), out)
        assert np.array_equal(out.get(), orc.foldseg(orc.OP_MAX, x1, offs1))


def test_foldseg_long_segments_keep_index_order(A, ctx, orc):
    """segments long on average go to a wave or a workgroup each: same results as the sequential fold, also for an
    operator that is associative but not commutative, in both association directions, with empty segments between"""
    first = ctx.skeleton(A.SKEL_FOLDSEG, "Int32", env=[I32], get="arrIn0_0[ix]", combine="x != 0 ? x : y", seed="-7")
    last = ctx.skeleton(A.SKEL_FOLDSEG, "Int32", env=[I32], get="arrIn0_0[ix]", combine="y != 0 ? y : x", seed="0")
    last_r = ctx.skeleton(A.SKEL_FOLDSEG, "Int32", env=[I32], get="arrIn0_0[ix]", combine="y != 0 ? y : x", seed="0",
                          flags=A.FLAG_FOLD_RIGHT)
    add = ctx.skeleton(A.SKEL_FOLDSEG, "Int32", env=[I32], get="arrIn0_0[ix]", combine="x + y", seed="3")
    mx = ctx.skeleton(A.SKEL_FOLD1SEG, "Int32", env=[I32], get="arrIn0_0[ix]", combine="acc_max(x, y)")
    for nseg, mean in [(300, 200), (2000, 1000), (37, 20000), (5, 300000), (1, 1 << 21), (3, 5000), (100, 3000)]:
        say("foldSeg, long segments:", nseg, "of mean", mean)
        lens = rng.poisson(mean, nseg).astype(np.int64)
        lens[::7] = 0                                        # empty ones in between
        lens[-1] = mean + 3
        offs = np.concatenate([[0], np.cumsum(lens)]).astype(np.int32)
        n = int(offs[-1])
        x = rng.integers(-3, 4, n, dtype=np.int32)
        x[rng.random(n) < 0.9] = 0                          # mostly zeros: the first / last non-zero is somewhere inside
        dx, doffs, out = ctx.array(x), ctx.array(offs), ctx.empty(nseg, np.int32)
        exp_first = np.full(nseg, -7, np.int32)
        exp_last = np.zeros(nseg, np.int32)
        for k in range(nseg):
            nz = np.flatnonzero(x[offs[k]:offs[k + 1]])
            if nz.size:
                exp_first[k] = x[offs[k] + nz[0]]
                exp_last[k] = x[offs[k] + nz[-1]]
        first.foldseg([dx], n, doffs, out)
        assert np.array_equal(out.get(), exp_first)
        last.foldseg([dx], n, doffs, out)
        assert np.array_equal(out.get(), exp_last)
        last_r.foldseg([dx], n, doffs, out)                  # x0 (+) (x1 (+) (... (+) z)): the same value, associated the other way
        assert np.array_equal(out.get(), exp_last)
        add.foldseg([dx], n, doffs, out)
        assert np.array_equal(out.get(), orc.foldseg(orc.OP_ADD, x, offs, seed=3))
        lens1 = np.maximum(lens, 1)
        offs1 = np.concatenate([[0], np.cumsum(lens1)]).astype(np.int32)
        x1 = rng.integers(-1000, 1000, int(offs1[-1]), dtype=np.int32)
        mx.foldseg([ctx.array(x1)], x1.size, ctx.array(offs1), out)
        assert np.array_equal(out.get(), orc.foldseg(orc.OP_MAX, x1, offs1))


def test_foldseg_of_arrays_of_higher_rank(A, ctx, orc):
    """the descriptor segments the innermost dimension of every outer row alike (Reduction.hs:473-474): short
    segments (a lane each), long ones (a wave, a workgroup, several workgroups each), empty ones, a tail of every
    row that belongs to no segment, an operator that is not commutative, rank 2 and rank 3, a misaligned input"""
    I2, I3 = (2, "Int32"), (3, "Int32")
    add = ctx.skeleton(A.SKEL_FOLDSEG, "Int32", env=[I2], out_rank=2, get="arrIn0_0[ix]", combine="x + y", seed="3")
    first = ctx.skeleton(A.SKEL_FOLDSEG, "Int32", env=[I2], out_rank=2, get="arrIn0_0[ix]", combine="x != 0 ? x : y", seed="-7")
    last_r = ctx.skeleton(A.SKEL_FOLDSEG, "Int32", env=[I2], out_rank=2, get="arrIn0_0[ix]", combine="y != 0 ? y : x", seed="0",
                          flags=A.FLAG_FOLD_RIGHT)
    mx = ctx.skeleton(A.SKEL_FOLD1SEG, "Int32", env=[I2], out_rank=2, get="arrIn0_0[ix]", combine="acc_max(x, y)")
    add3 = ctx.skeleton(A.SKEL_FOLDSEG, "Int32", env=[I3], out_rank=3, get="arrIn0_0[ix]", combine="x + y", seed="0")
    for rows, nseg, mean, tail in [(1, 50, 4, 0), (7, 1, 9, 2), (300, 40, 6, 5), (4001, 33, 20, 0), (25, 12, 400, 17),
                                   (6, 5, 30000, 1), (3, 1, 700000, 3), (2000, 3, 0, 4)]:
        say("foldSeg of", rows, "rows x", nseg, "segments of mean", mean, "and a tail of", tail)
        lens = rng.poisson(mean, nseg).astype(np.int64)
        if nseg > 2:
            lens[::5] = 0
        offs = np.concatenate([[0], np.cumsum(lens)]).astype(np.int32)
        inner = int(offs[-1]) + tail
        x = rng.integers(-3, 4, (rows, inner), dtype=np.int32)
        x[rng.random((rows, inner)) < 0.8] = 0
        dx, doffs, out = ctx.array(x), ctx.array(offs), ctx.array(np.full((rows, nseg), 12345, np.int32))
        add.foldseg_nd([dx], x.shape, doffs, out)
        assert np.array_equal(out.get(), orc.foldseg_nd(orc.OP_ADD, x, offs, seed=3))
        exp_first, exp_last = np.full((rows, nseg), -7, np.int32), np.zeros((rows, nseg), np.int32)
        for r in range(min(rows, 64)):
            for k in range(nseg):
                nz = np.flatnonzero(x[r, offs[k]:offs[k + 1]])
                if nz.size:
                    exp_first[r, k] = x[r, offs[k] + nz[0]]
                    exp_last[r, k] = x[r, offs[k] + nz[-1]]
        first.foldseg_nd([dx], x.shape, doffs, out)
        assert np.array_equal(out.get()[:64], exp_first[:64])
        last_r.foldseg_nd([dx], x.shape, doffs, out)
        assert np.array_equal(out.get()[:64], exp_last[:64])
        if mean > 0:
            lens1 = np.maximum(lens, 1)
            offs1 = np.concatenate([[0], np.cumsum(lens1)]).astype(np.int32)
            x1 = rng.integers(-1000, 1000, (rows, int(offs1[-1]) + tail), dtype=np.int32)
            mx.foldseg_nd([ctx.array(x1)], x1.shape, ctx.array(offs1), out)
            assert np.array_equal(out.get(), orc.foldseg_nd(orc.OP_MAX, x1, offs1))
    say("rank 3, and an input that starts 4 bytes off a 16-byte boundary")
    lens = np.array([2, 0, 7, 1, 30, 0, 3], np.int64)
    offs = np.concatenate([[0], np.cumsum(lens)]).astype(np.int32)
    x = rng.integers(-100, 100, (5, 9, 45), dtype=np.int32)
    out3 = ctx.empty((5, 9, 7), np.int32)
    add3.foldseg_nd([ctx.array(x)], x.shape, ctx.array(offs), out3)
    assert np.array_equal(out3.get(), orc.foldseg_nd(orc.OP_ADD, x, offs, seed=0))
    buf = ctx.array(np.concatenate([[0], x.reshape(-1)]).astype(np.int32))
    add3.foldseg_nd([buf.desc(shape=x.shape, offset_elems=1)], x.shape, ctx.array(offs), out3)
    assert np.array_equal(out3.get(), orc.foldseg_nd(orc.OP_ADD, x, offs, seed=0))
    say("wrong use")
    with pytest.raises(A.AccError) as e:                     # the rank-1 entry on a rank-2 kernel
        add.foldseg([ctx.array(x.reshape(-1))], x.size, ctx.array(offs), ctx.empty(7, np.int32))
    assert e.value.code == A.ERR_INVALID
    with pytest.raises(A.AccError) as e:                     # a result whose rows are not the segments
        add.foldseg_nd([ctx.array(x.reshape(45, 45))], (45, 45), ctx.array(offs), ctx.empty((45, 8), np.int32))
    assert e.value.code == A.ERR_INVALID
    for s_ in (add, first, last_r, mx, add3):
        s_.destroy()


def test_fold_along_the_innermost_dimension_at_every_shape(A, ctx):
    """rows of 1 to 2^20 elements, 2^20 rows to one: a lane, a wave, a workgroup or several workgroups per row"""
    add = ctx.skeleton(A.SKEL_FOLD, "Int32", env=[(2, "Int32")], out_rank=1, get="arrIn0_0[ix]", combine="x + y", seed="5")
    first = ctx.skeleton(A.SKEL_FOLD1, "Int32", env=[(2, "Int32")], out_rank=1, get="arrIn0_0[ix]", combine="x != 0 ? x : y")
    add3 = ctx.skeleton(A.SKEL_FOLD, "Int64", env=[(3, "Int32")], out_rank=2, get="(Int64)arrIn0_0[ix]", combine="x + y", seed="0")
    for rows, inner in [(1 << 18, 1), (70001, 3), (40000, 31), (9999, 64), (3000, 191), (3000, 193), (700, 1000), (129, 16384),
                        (33, 40001), (7, 300007), (2, 1 << 20), (1, (1 << 21) + 5)]:
        say("fold of a", rows, "x", inner, "array")
        x = rng.integers(-5, 6, (rows, inner), dtype=np.int32)
        x[rng.random((rows, inner)) < 0.8] = 0
        dx, out = ctx.array(x), ctx.empty(rows, np.int32)
        add.fold([dx], (rows, inner), out)
        assert np.array_equal(out.get(), x.sum(axis=1, dtype=np.int32) + 5)
        first.fold([dx], (rows, inner), out)                    # associative, not commutative: index order must be kept
        nz = x != 0
        exp = np.where(nz.any(axis=1), x[np.arange(rows), nz.argmax(axis=1)], 0).astype(np.int32)
        assert np.array_equal(out.get(), exp)
    say("fold of a rank-3 array")
    x = rng.integers(-1000, 1000, (6, 50, 700), dtype=np.int32)
    out = ctx.empty((6, 50), np.int64)
    add3.fold([ctx.array(x)], x.shape, out)
    assert np.array_equal(out.get(), x.sum(axis=2, dtype=np.int64))
    say("rows without elements yield the seed")
    out = ctx.empty(17, np.int32)
    add.fold([ctx.empty((17, 0), np.int32)], (17, 0), out)
    assert np.array_equal(out.get(), np.full(17, 5, np.int32))
    say("an empty outer extent: no row exists to be read; a seeded fold gives the seed once (Execute.hs:287-289), fold1 nothing")
    out = ctx.array(np.full(1, -1, np.int32))
    add.fold([ctx.empty((0, 5), np.int32)], (0, 5), out)
    assert out.get().tolist() == [5]
    out = ctx.array(np.full(3, -1, np.int32))
    first.fold([ctx.empty((0, 5), np.int32)], (0, 5), out)
    assert out.get().tolist() == [-1, -1, -1]


def test_fold_of_short_rows(A, ctx, orc):
    """rows of 1 to 16 elements (a lane per row straight from memory up to 7, staged chunks beyond): row counts around
    the workgroup's share, an operator that is not commutative, Float32 sums bit for bit with the sequential left
    fold (the association is the same), a fused producer, a source that is not 16-byte aligned"""
    addf = ctx.skeleton(A.SKEL_FOLD, "float", env=[(2, "float")], out_rank=1, get="arrIn0_0[ix]", combine="x + y", seed="0.5f")
    sub1 = ctx.skeleton(A.SKEL_FOLD1, "Int32", env=[(2, "Int32")], out_rank=1, get="arrIn0_0[ix]", combine="2 * x - y")
    prod = ctx.skeleton(A.SKEL_FOLD, "Int64", env=[(2, "Int32"), (2, "Int32")], out_rank=1,
                        get="(Int64)arrIn0_0[ix] * (Int64)arrIn1_0[ix]", combine="x + y", seed="-3")
    for inner in range(1, 17):
        for rows in (1, 255, 4096, 4097, 70001):
            say("fold of", rows, "rows of", inner)
            xf = (rng.random((rows, inner)) * 2 - 1).astype(np.float32)
            out = ctx.empty(rows, np.float32)
            addf.fold([ctx.array(xf)], (rows, inner), out)
            ref = xf[:, 0].copy()
            for k in range(1, inner):
                ref = ref + xf[:, k]
            assert np.array_equal(out.get(), ref + np.float32(0.5))               # ((x0 + x1) + ...) + z, as written
            xi = rng.integers(-9, 10, (rows, inner), dtype=np.int32)
            outi = ctx.empty(rows, np.int32)
            sub1.fold([ctx.array(xi)], (rows, inner), outi)
            ref = xi[:, 0].copy()
            for k in range(1, inner):
                ref = 2 * ref - xi[:, k]
            assert np.array_equal(outi.get(), ref)
        rows = 30011
        a, b = rng.integers(-10**4, 10**4, (rows, inner), dtype=np.int32), rng.integers(-10**4, 10**4, (rows, inner), dtype=np.int32)
        flat = ctx.array(np.concatenate([np.zeros(1, np.int32), a.reshape(-1)]))   # the first source starts 4 bytes off
        out = ctx.empty(rows, np.int64)
        prod.fold([flat.desc(shape=(rows, inner), offset_elems=1), ctx.array(b)], (rows, inner), out)
        assert np.array_equal(out.get(), (a.astype(np.int64) * b).sum(axis=1) - 3)
    say("rows of pairs")
    pair = ctx.skeleton(A.SKEL_FOLD, "Int32, float", env=[(2, "Int32"), (2, "float")], out_rank=1,
                        get="acc_elt{arrIn0_0[ix], arrIn1_0[ix]}", combine="acc_elt{x.a1 + y.a1, acc_max(x.a0, y.a0)}",
                        seed="acc_elt{0, -1.0e30f}")
    rows, inner = 50001, 4
    a, b = rng.integers(-99, 99, (rows, inner), dtype=np.int32), rng.random((rows, inner)).astype(np.float32)
    out = A.TupleArray([ctx.empty(rows, np.int32), ctx.empty(rows, np.float32)])
    pair.fold([ctx.array(a), ctx.array(b)], (rows, inner), out)
    assert np.array_equal(out.comps[0].get(), a.sum(axis=1, dtype=np.int32)) and np.array_equal(out.comps[1].get(), b.max(axis=1))


# --------------------------------------------------------------------------- committed fixtures

def test_golden_fixtures_on_gpu(A, ctx):
    """the numpy/scipy-made vectors of tests/golden, through the HIP path"""
    with open(os.path.join(GOLDEN, "golden.json")) as fh:
        g = json.load(fh)
    say("golden scans")
    x = np.array(g["scan"]["x"], dtype=np.int32)
    dx = ctx.array(x)
    for kind, key in (("scanl", "scanl"), ("scanl1", "scanl1"), ("scanr", "scanr")):
        sk = ctx.skeleton(A.SCAN_KINDS[kind], "Int32", env=[I32], get="arrIn0_0[ix]", combine="x + y",
                          seed=str(g["scan"]["seed"]) if kind != "scanl1" else None)
        out = ctx.empty(len(g["scan"][key]), np.int32)
        sk.scan([dx], x.size, out)
        assert out.get().tolist() == g["scan"][key]
    say("golden histogram")
    keys = np.array(g["hist"]["keys"], dtype=np.int32)
    hist = ctx.skeleton(A.SKEL_PERMUTE, "Int32", env=[I32], out_rank=1, get="1", combine="x + y",
                        permutation="arrIn0_0[ix]", combine_hint=A.COMBINE_ADD)
    out = ctx.empty(g["hist"]["bins"], np.int32)
    hist.permute([ctx.array(keys)], keys.size, ctx.array(np.zeros(g["hist"]["bins"], np.int32)), out)
    assert out.get().tolist() == g["hist"]["counts"]
    say("golden stencils")
    img = np.array(g["stencil"]["img"], dtype=np.float32)
    for mode in ("clamp", "mirror", "wrap", "constant"):
        for name, taps, coef, div in (("gauss_", GAUSS_TAPS, [1, 2, 1, 2, 4, 2, 1, 2, 1], 16),
                                      ("laplace_", LAPLACE_TAPS, [1, 1, -4, 1, 1], None)):
            sk = ctx.skeleton(A.SKEL_STENCIL, "float", out_rank=2, taps=taps, stencil_fn=A.linear_stencil_fn(coef, div),
                              boundary=mode, boundary_constant="%rf" % g["stencil"]["constant"])
            o = ctx.empty(img.shape, np.float32)
            sk.stencil([], ctx.array(img), o)
            assert np.max(np.abs(o.get() - np.array(g["stencil"][name + mode]))) <= 1e-5
    say("golden smvm and dot")
    s = g["smvm"]
    smvm = ctx.skeleton(A.SKEL_FOLDSEG, "float", env=[F32, I32, F32], get="arrIn0_0[ix] * arrIn2_0[arrIn1_0[ix]]",
                        combine="x + y", seed="0.0f")
    y = ctx.empty(len(s["y"]), np.float32)
    smvm.foldseg([ctx.array(np.array(s["vals"], np.float32)), ctx.array(np.array(s["cols"], np.int32)),
                  ctx.array(np.array(s["x"], np.float32))], len(s["vals"]),
                 ctx.array(np.array(s["offsets"], np.int32)), y)
    ref = np.array(s["y"])
    assert np.max(np.abs(y.get() - ref)) <= 1e-5
    d = g["dot"]
    dot = ctx.skeleton(A.SKEL_FOLD, "float", env=[F32, F32], out_rank=0, get="arrIn0_0[ix] * arrIn1_0[ix]",
                       combine="x + y", seed="0.0f")
    out = ctx.empty((), np.float32)
    dot.fold([ctx.array(np.array(d["x"], np.float32)), ctx.array(np.array(d["y"], np.float32))], len(d["x"]), out)
    assert abs(float(out.get()) - d["dot"]) <= 1e-4 * abs(d["dot"])


def test_permute_index_types_and_stray_targets(A, ctx, orc):
    """targets of every width and signedness a permutation can produce; negative
    ones, `ignore` and those past the end of the result are dropped, in the LDS
    window, in the part of the target beyond it, and without any window"""
    n = 200000
    for bins in (300, 100000):                                   # inside one LDS window / larger than it
        base = rng.integers(-50, bins + 50, n)                   # ~ strays on both sides
        base[::17] = -1
        dfl = rng.integers(0, 5, bins, dtype=np.int32)
        keep = (base >= 0) & (base < bins)
        exp = dfl + np.bincount(base[keep], minlength=bins).astype(np.int32)
        for tname, dt, frag in (("Int32", np.int32, "arrIn0_0[ix]"), ("Int64", np.int64, "arrIn0_0[ix]"),
                                ("Int16 widened", np.int32, "(Int16)arrIn0_0[ix]"),
                                ("Int64 computed", np.int32, "(Int64)arrIn0_0[ix] * 1")):
            if tname.startswith("Int16") and bins > 30000:
                continue
            for hint in (A.COMBINE_ADD, A.COMBINE_GENERIC):
                say("permute targets as", tname, "bins", bins, "hint", hint)
                keys = base.astype(dt)
                sk = ctx.skeleton(A.SKEL_PERMUTE, "Int32", env=[(1, "Int64" if dt == np.int64 else "Int32")], out_rank=1,
                                  get="1", combine="x + y", permutation=frag, combine_hint=hint)
                out = ctx.empty(bins, np.int32)
                sk.permute([ctx.array(keys)], n, ctx.array(dfl), out)
                assert np.array_equal(out.get(), exp), (tname, bins, hint)
    say("unsigned 32-bit targets: values of 2^31 and more are simply past the end")
    keys = rng.integers(0, 400, n).astype(np.uint32)
    keys[::13] = np.uint32(0x80000005)
    keys[::29] = np.uint32(0xFFFFFFFF)
    sk = ctx.skeleton(A.SKEL_PERMUTE, "Int32", env=[(1, "Word32")], out_rank=1, get="1", combine="x + y",
                      permutation="arrIn0_0[ix]", combine_hint=A.COMBINE_ADD)
    out = ctx.empty(300, np.int32)
    sk.permute([ctx.array(keys)], n, ctx.array(np.zeros(300, np.int32)), out)
    assert np.array_equal(out.get(), np.bincount(keys[keys < 300], minlength=300).astype(np.int32))


def test_segmented_and_innermost_folds_of_narrow_elements(A, ctx):
    """1- and 2-byte elements: a lane loads 16 of them at once, so a workgroup's chunk is larger than for 4-byte ones"""
    for ctype, dt in (("Word8", np.uint8), ("Int16", np.int16)):
        seg = ctx.skeleton(A.SKEL_FOLDSEG, ctype, env=[(1, ctype)], get="arrIn0_0[ix]", combine="(%s)(x + y)" % ctype, seed="1")
        dim = ctx.skeleton(A.SKEL_FOLD, ctype, env=[(2, ctype)], out_rank=1, get="arrIn0_0[ix]", combine="(%s)(x + y)" % ctype, seed="1")
        for nseg, mean in ((1, 5), (1000, 3), (5000, 40), (300, 3000)):
            say("foldSeg of", ctype, nseg, "segments of about", mean)
            lens = rng.poisson(mean, nseg)
            offs = np.concatenate([[0], np.cumsum(lens)]).astype(np.int32)
            x = rng.integers(0, 7, int(offs[-1])).astype(dt)
            out = ctx.empty(nseg, dt)
            seg.foldseg([ctx.array(x) if x.size else ctx.empty(0, dt)], x.size, ctx.array(offs), out)
            ref = np.array([x[a:b].sum(dtype=np.int64) + 1 for a, b in zip(offs[:-1], offs[1:])]).astype(dt)
            assert np.array_equal(out.get(), ref)
        for rows, inner in ((7, 3), (1000, 16), (333, 1000), (4, 70001)):
            say("fold of a", rows, "x", inner, ctype, "array")
            x = rng.integers(0, 7, (rows, inner)).astype(dt)
            out = ctx.empty(rows, dt)
            dim.fold([ctx.array(x)], (rows, inner), out)
            assert np.array_equal(out.get(), (x.sum(axis=1, dtype=np.int64) + 1).astype(dt))


def test_stencils_of_every_element_width(A, ctx):
    """2-D stencils in the four boundary modes and a 3-D one over 1-, 2-, 4- and 8-byte elements (integer arithmetic
    wraps in the element type; Float64 on small integers is exact)"""
    five = [(-1, 0), (0, -1), (0, 0), (0, 1), (1, 0)]
    seven = [(0, 0, 0), (-1, 0, 0), (1, 0, 0), (0, -1, 0), (0, 1, 0), (0, 0, -1), (0, 0, 1)]
    types = (("Int8", np.int8), ("Word16", np.uint16), ("Int64", np.int64), ("double", np.float64))
    sks = {}
    for ctype, dt in types:                             # all twenty instances first: they compile side by side
        cast = "(%s)" % ctype
        for mode in ("clamp", "mirror", "wrap", "constant"):
            sks[ctype, mode] = ctx.skeleton(A.SKEL_STENCIL, ctype, out_rank=2, taps=five, boundary=mode, boundary_constant=cast + "2",
                                            stencil_fn=cast + "(t0 + 2 * t1 - t2 + t3 + t4)").prefetch(range(1, 6))
        sks[ctype, 3] = ctx.skeleton(A.SKEL_STENCIL, ctype, out_rank=3, taps=seven, boundary="mirror",
                                     stencil_fn=cast + "(t0 + t1 + t2 + t3 + t4 + t5 + 2 * t6)").prefetch(range(1, 6))
    for ctype, dt in types:
        cast = "(%s)" % ctype
        wide = (lambda a: a) if ctype == "double" else (lambda a: a.astype(np.int64))
        for mode in ("clamp", "mirror", "wrap", "constant"):
            sk = sks[ctype, mode]
            for shape in ((5, 7), (33, 300), (7, 1031)):
                say("stencil of", ctype, mode, shape)
                v = rng.integers(0, 5, shape).astype(dt)
                out = ctx.empty(shape, dt)
                sk.stencil([], ctx.array(v), out)
                t = [wide(a) for a in pyref.tap_arrays(v, five, mode, 2, shape)]
                assert np.array_equal(out.get(), (t[0] + 2 * t[1] - t[2] + t[3] + t[4]).astype(dt))
        sk = sks[ctype, 3]
        for shape in ((3, 5, 7), (4, 9, 1031)):
            say("3-D stencil of", ctype, shape)
            v = rng.integers(0, 5, shape).astype(dt)
            out = ctx.empty(shape, dt)
            sk.stencil([], ctx.array(v), out)
            t = [wide(a) for a in pyref.tap_arrays3(v, seven, "mirror", 0, shape)]
            assert np.array_equal(out.get(), (sum(t[:6]) + 2 * t[6]).astype(dt))


def test_right_handed_scans_of_every_element_width(A, ctx):
    """scanr, scanr1 and scanr' over 1-, 2-, 4- and 8-byte elements and over pairs, at sizes around the tile
    boundaries and sizes that are no multiple of a vector (the rounding positions of the first vector)"""
    def rscan(x):                                           # inclusive from the right, in the element type
        return np.cumsum(x[::-1], dtype=x.dtype)[::-1]
    types = (("Int8", np.int8), ("Word16", np.uint16), ("Int32", np.int32), ("Int64", np.int64), ("double", np.float64))
    sks = {}
    for ctype, dt in types:                             # all fifteen instances first, small tiles too: they compile side by side
        lit = "3.0" if ctype == "double" else "3"
        sks[ctype] = (ctx.skeleton(A.SKEL_SCANR, ctype, env=[(1, ctype)], get="arrIn0_0[ix]", combine="(%s)(x + y)" % ctype, seed=lit).prefetch([2]),
                      ctx.skeleton(A.SKEL_SCANR1, ctype, env=[(1, ctype)], get="arrIn0_0[ix]", combine="(%s)(x + y)" % ctype).prefetch([2]),
                      ctx.skeleton(A.SKEL_SCANRP, ctype, env=[(1, ctype)], get="arrIn0_0[ix]", combine="(%s)(x + y)" % ctype, seed=lit).prefetch([2]))
    for ctype, dt in types:
        r0, r1, rp = sks[ctype]
        tile = r1.info().elements_per_block
        for n in (1, 3, 17, tile - 1, tile, tile + 1, 3 * tile + 5, 300007):
            say("right-handed scans of", ctype, "n =", n)
            x = rng.integers(0, 9, n).astype(dt)
            inc = rscan(x)
            out = ctx.empty(n + 1, dt)
            r0.scan([ctx.array(x)], n, out)
            assert np.array_equal(out.get(), np.concatenate([inc + dt(3), [dt(3)]]).astype(dt))
            out = ctx.empty(n, dt)
            r1.scan([ctx.array(x)], n, out)
            assert np.array_equal(out.get(), inc)
            tot = ctx.empty((), dt)
            rp.scan([ctx.array(x)], n, out, total=tot)
            with np.errstate(over="ignore"):                       # narrow elements wrap around, here as on the device
                whole = dt(inc[0] + dt(3))
            assert np.array_equal(out.get(), np.concatenate([inc[1:] + dt(3), [dt(3)]]).astype(dt)) and tot.get()[()] == whole
    say("right-handed scan of pairs")
    pr = ctx.skeleton(A.SKEL_SCANR1, "Int32, float", env=[(1, "Int32"), (1, "float")], get="acc_elt{arrIn0_0[ix], arrIn1_0[ix]}",
                      combine="acc_elt{x.a1 + y.a1, acc_max(x.a0, y.a0)}")
    n = 100003
    a, b = rng.integers(-9, 9, n).astype(np.int32), rng.random(n).astype(np.float32)
    out = A.TupleArray([ctx.empty(n, np.int32), ctx.empty(n, np.float32)])
    pr.scan([ctx.array(a), ctx.array(b)], n, out)
    assert np.array_equal(out.comps[0].get(), rscan(a)) and np.array_equal(out.comps[1].get(), np.maximum.accumulate(b[::-1])[::-1])


def test_scan_tile_shape_follows_the_register_count(A, ctx):
    """the first build of a scan decides its tile shape: four waves with many rows a lane where that keeps within
    256 registers, else sixteen waves; tiles hold 128 KB either way, and the results do not depend on the shape"""
    for ctype, dt, comb in (("Int32", np.int32, "x + y"), ("double", np.float64, "acc_max(x, y)")):
        sk = ctx.skeleton(A.SKEL_SCANL1, ctype, env=[(1, ctype)], get="arrIn0_0[ix]", combine=comb)
        info = sk.info()
        say("scan of", ctype, "block", info.block, "registers", info.num_regs, "elements per tile", info.elements_per_block)
        assert info.block in (256, 1024) and (info.block == 1024 or info.num_regs <= 256)
        assert info.elements_per_block * np.dtype(dt).itemsize == 128 * 1024
        x = rng.integers(-1000, 1000, 3 * info.elements_per_block + 17).astype(dt)
        out = ctx.empty(x.size, dt)
        sk.scan([ctx.array(x)], x.size, out)
        ref = np.cumsum(x, dtype=dt) if ctype == "Int32" else np.maximum.accumulate(x)
        assert np.array_equal(out.get(), ref)


def test_map_in_tiles_gives_what_the_map_in_runs_gives(A, ctx):
    """ACC_FLAG_TILED changes the order the result is produced in (tiles of 32 x 32, for element functions that read
    across the rows of their source), never the result: transposes, ragged and narrow shapes, shapes too thin for
    tiles (which take the instance's variants in runs), rank 3, a function of the index alone, elements of 1 and 8 bytes"""
    rng = np.random.default_rng(9)
    for ctype, dt in (("float", np.float32), ("Int8", np.int8), ("double", np.float64)):
        tr = ctx.skeleton(A.SKEL_MAP, ctype, env=[(2, ctype)], out_rank=2, flags=A.FLAG_TILED,
                          get="arrIn0_0[(ix % shOut_0) * shIn0_0 + (ix / shOut_0)]")
        # (results of fewer than 10 rows or 33 columns are produced in runs after all: both sides of either bound)
        for (h, w) in ((1, 1), (3, 70), (64, 64), (65, 63), (64, 128), (100, 257), (257, 100), (1, 500), (500, 1), (1030, 515),
                       (40000, 5), (9, 70000), (10, 70000), (30011, 32), (30011, 33)):
            say("tiled transpose", ctype, (h, w))
            src = rng.integers(-100, 100, (w, h)).astype(dt)              # the source is w x h, the result h x w
            out = ctx.empty((h, w), dt)
            tr.map([ctx.array(src)], out)
            assert np.array_equal(out.get(), src.T)
    say("tiled map of rank 3, a function of the index")
    g = ctx.skeleton(A.SKEL_GENERATE, "Int32", env=[], out_rank=3, flags=A.FLAG_TILED, get="(Int32)(ix * 7 + 1)")
    for shape in ((1, 1, 1), (3, 40, 50), (2, 33, 65), (5, 1, 300)):
        out = ctx.empty(shape, np.int32)
        g.map([], out)
        assert np.array_equal(out.get().reshape(-1), (np.arange(int(np.prod(shape)), dtype=np.int64) * 7 + 1).astype(np.int32))
    say("tiles of the innermost dimension and one further out than the second innermost (ACC_FLAG_TILE_DIM)")
    for rank, dim, shapes in ((3, 2, ((1, 1, 1), (40, 3, 50), (33, 2, 65), (300, 1, 5), (70, 40, 33))), (4, 2, ((2, 40, 3, 50),)),
                              (4, 3, ((40, 2, 3, 50), (33, 1, 1, 65)))):
        g = ctx.skeleton(A.SKEL_GENERATE, "Int32", env=[], out_rank=rank, flags=A.FLAG_TILED | A.FLAG_TILE_DIM(dim), get="(Int32)(ix * 7 + 1)")
        for shape in shapes:
            out = ctx.array(np.full(int(np.prod(shape)) + 2, 77, np.int32))
            g.map([], out.desc(shape=shape))
            got = out.get()
            assert np.array_equal(got[:-2], (np.arange(int(np.prod(shape)), dtype=np.int64) * 7 + 1).astype(np.int32)), (rank, dim, shape)
            assert np.array_equal(got[-2:], [77, 77])
    vol = rng.integers(-100, 100, (30, 45, 70)).astype(np.int32)               # turned: result[k, i, j] = vol[i, j, k]
    tv = ctx.skeleton(A.SKEL_MAP, "Int32", env=[(3, "Int32")], out_rank=3, flags=A.FLAG_TILED | A.FLAG_TILE_DIM(2),
                      get="arrIn0_0[((ix / shOut_0) % shOut_1) * (shIn0_1 * shIn0_0) + (ix % shOut_0) * shIn0_0 + ix / (shOut_0 * shOut_1)]")
    out = ctx.empty((70, 30, 45), np.int32)
    tv.map([ctx.array(vol)], out)
    assert np.array_equal(out.get(), vol.transpose(2, 0, 1))
    with pytest.raises(A.AccError):
        ctx.skeleton(A.SKEL_GENERATE, "Int32", env=[], out_rank=2, flags=A.FLAG_TILED | A.FLAG_TILE_DIM(2), get="(Int32)ix", wait=True)
    say("tiled map producing pairs (one array per component)")
    pt = ctx.skeleton(A.SKEL_MAP, "float, Int32", env=[(2, "float"), (2, "Int32")], out_rank=2, flags=A.FLAG_TILED,
                      get="acc_elt{arrIn0_0[(ix % shOut_0) * shIn0_0 + (ix / shOut_0)] * 2.0f, arrIn1_0[ix] + 1}")
    for (h, w) in ((5, 7), (64, 96), (70, 131)):
        fa, ib = rng.integers(-9, 9, (w, h)).astype(np.float32), rng.integers(-9, 9, (h, w)).astype(np.int32)
        out = ctx.empty_tuple((h, w), [np.float32, np.int32])
        pt.map([ctx.array(fa), ctx.array(ib)], out)
        assert np.array_equal(out.comps[0].get(), fa.T * 2) and np.array_equal(out.comps[1].get(), ib + 1)
    say("the flag on a vector is ignored")
    v = ctx.skeleton(A.SKEL_MAP, "Int32", env=[I32], out_rank=1, flags=A.FLAG_TILED, get="arrIn0_0[ix] + 1")
    x = rng.integers(0, 9, 1000).astype(np.int32)
    out = ctx.empty(1000, np.int32)
    v.map([ctx.array(x)], out)
    assert np.array_equal(out.get(), x + 1)
