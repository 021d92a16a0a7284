"""The scalar primitives of the expression language (acc_prim.h), each run
through a map skeleton on the GPU and compared with an independent definition:
exact Python integer arithmetic for the Integral and Bits operators, numpy for
the floating ones.  Integer results are bit-exact; the tolerance of each
floating comparison is written at its assertion.
"""
import sys

import numpy as np
import pytest

import pyref

pytestmark = pytest.mark.gpu

INT_TYPES = [("Int8", np.int8), ("Int16", np.int16), ("Int32", np.int32), ("Int64", np.int64),
             ("Word8", np.uint8), ("Word16", np.uint16), ("Word32", np.uint32), ("Word64", np.uint64)]


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


def operands(dt, n=4096, seed=5):
    """pairs (x, y), y != 0, with the corners of the type among them; no (min, -1)"""
    info = np.iinfo(dt)
    rng = np.random.default_rng(seed)
    corners = [info.min, info.max, 0, 1, 2, 3, 7, info.max - 1, info.min + 1]
    if info.min < 0:
        corners += [-1, -2, -3, -7]
    x = rng.integers(info.min, info.max, n, dtype=dt, endpoint=True)
    y = rng.integers(info.min, info.max, n, dtype=dt, endpoint=True)
    small = rng.integers(max(info.min, -9), 9, n, dtype=dt, endpoint=True)
    y[::3] = small[::3]                                    # small divisors make interesting quotients
    k = 0
    for a in corners:
        for b in corners:
            x[k], y[k] = a, b
            k += 1
    y[y == 0] = 1
    if info.min < 0:
        y[(x == info.min) & (y == -1)] = 1                 # overflows in C and in Haskell alike
    return x, y


def run_map(A, ctx, tname, dt, get, x, y, out_t=None, out_dt=None):
    sk = ctx.skeleton(A.SKEL_MAP, out_t or tname, env=[(1, tname), (1, tname)], out_rank=1, get=get)
    out = ctx.empty(x.size, out_dt or dt)
    sk.map([ctx.array(x), ctx.array(y)], out)
    return out.get()


@pytest.mark.parametrize("tname,dt", INT_TYPES)
def test_integral_and_bits(A, ctx, tname, dt):
    bits = 8 * np.dtype(dt).itemsize
    signed = np.iinfo(dt).min < 0
    x, y = operands(dt)
    xs, ys = [int(v) for v in x], [int(v) for v in y]
    X, Y = "arrIn0_0[ix]", "arrIn1_0[ix]"
    cnt = "(Int64)(%s & %d)" % (Y, bits - 1)               # a legal shift count from y
    cs = [int(v) & (bits - 1) for v in y]

    def check(name, frag, expect):
        say(tname, name)
        got = run_map(A, ctx, tname, dt, frag, x, y)
        exp = np.array([pyref.wrap(e, bits, signed) for e in expect], dtype=dt)
        bad = np.nonzero(got != exp)[0]
        assert bad.size == 0, (name, tname, xs[bad[0]], ys[bad[0]], int(got[bad[0]]), int(exp[bad[0]]))

    check("quot", "acc_quot(%s, %s)" % (X, Y), [pyref.quot(a, b) for a, b in zip(xs, ys)])
    check("rem", "acc_rem(%s, %s)" % (X, Y), [pyref.rem(a, b) for a, b in zip(xs, ys)])
    check("idiv", "acc_idiv(%s, %s)" % (X, Y), [pyref.idiv(a, b) for a, b in zip(xs, ys)])
    check("mod", "acc_imod(%s, %s)" % (X, Y), [pyref.imod(a, b) for a, b in zip(xs, ys)])
    check("quotRem.fst", "acc_quot_rem(%s, %s).fst" % (X, Y), [pyref.quot(a, b) for a, b in zip(xs, ys)])
    check("quotRem.snd", "acc_quot_rem(%s, %s).snd" % (X, Y), [pyref.rem(a, b) for a, b in zip(xs, ys)])
    check("divMod.fst", "acc_div_mod(%s, %s).fst" % (X, Y), [pyref.idiv(a, b) for a, b in zip(xs, ys)])
    check("divMod.snd", "acc_div_mod(%s, %s).snd" % (X, Y), [pyref.imod(a, b) for a, b in zip(xs, ys)])
    check("abs", "acc_abs(%s)" % X, [abs(a) for a in xs])
    check("signum", "acc_signum(%s)" % X, [pyref.signum(a) for a in xs])
    check("max", "acc_pmax(%s, %s)" % (X, Y), [max(a, b) for a, b in zip(xs, ys)])
    check("min", "acc_pmin(%s, %s)" % (X, Y), [min(a, b) for a, b in zip(xs, ys)])
    check("shiftL", "acc_shift_l(%s, %s)" % (X, cnt), [a << c for a, c in zip(xs, cs)])
    check("shiftR (arithmetic)", "acc_shift_r(%s, %s)" % (X, cnt), [a >> c for a, c in zip(xs, cs)])
    check("shiftR (logical)", "acc_shift_rl(%s, %s)" % (X, cnt), [pyref.shift_rl(a, c, bits) for a, c in zip(xs, cs)])
    check("rotateL", "acc_rotate_l(%s, (Int64)%s)" % (X, Y), [pyref.rotate_l(a, b, bits) for a, b in zip(xs, ys)])
    check("rotateR", "acc_rotate_r(%s, (Int64)%s)" % (X, Y), [pyref.rotate_l(a, -b, bits) for a, b in zip(xs, ys)])
    check("band/bor/xor/complement", "(%s & %s) ^ (%s | ~%s)" % (X, Y, X, Y), [(a & b) ^ (a | ~b) for a, b in zip(xs, ys)])


@pytest.mark.parametrize("tname,dt", [("float", np.float32), ("double", np.float64)])
def test_floating(A, ctx, tname, dt):
    rng = np.random.default_rng(11)
    n = 4096
    x = ((rng.random(n) * 2 - 1) * 8).astype(dt)
    y = ((rng.random(n) * 2 - 1) * 8).astype(dt)
    special = [0.0, -0.0, 0.5, -0.5, 1.5, -1.5, 2.5, -2.5, 1.0, -1.0, np.inf, -np.inf, np.nan, 1e-30, 3.999999]
    x[:len(special)] = special
    y[:len(special)] = special[::-1]
    X, Y = "arrIn0_0[ix]", "arrIn1_0[ix]"
    ulp = float(np.finfo(dt).eps)

    def fl(name, frag, expect, tol):
        say(tname, name)
        got = run_map(A, ctx, tname, dt, frag, x, y)
        with np.errstate(all="ignore"):
            exp = expect.astype(dt)
        assert np.array_equal(np.isnan(got), np.isnan(exp)), name
        ok = ~np.isnan(exp)
        if tol == 0:
            assert np.array_equal(got[ok], exp[ok]), name
            assert np.array_equal(np.signbit(got[ok]), np.signbit(exp[ok])), name
        else:   # relative error of the library functions, in units of the type's epsilon
            fin = ok & np.isfinite(exp)
            assert np.array_equal(got[ok & ~fin], exp[ok & ~fin]), name
            assert np.all(np.abs(got[fin] - exp[fin]) <= tol * ulp * np.maximum(np.abs(exp[fin]), np.finfo(dt).tiny)), name

    with np.errstate(all="ignore"):
        one = dt(1)
        fl("recip", "acc_recip(%s)" % X, one / x, 0)
        fl("abs", "acc_abs(%s)" % X, np.abs(x), 0)
        sg = np.where(x == 0, dt(0), np.copysign(one, x))
        sg[np.isnan(x)] = np.nan        # copysign(1, NaN) is +-1 on the device; only its being set is compared below
        got = run_map(A, ctx, tname, dt, "acc_signum(%s)" % X, x, y)
        keep = ~np.isnan(x)
        assert np.array_equal(got[keep], sg[keep]) and np.all(np.abs(got[~keep]) == 1)
        fl("sqrt", "acc_sqrt(%s)" % X, np.sqrt(x), 0)                      # correctly rounded on both sides
        for name, f in (("sin", np.sin), ("cos", np.cos), ("tan", np.tan), ("atan", np.arctan), ("sinh", np.sinh),
                        ("cosh", np.cosh), ("tanh", np.tanh), ("asinh", np.arcsinh), ("exp", np.exp), ("log", np.log)):
            fl(name, "acc_%s(%s)" % (name, X), f(x.astype(np.float64)), 8)
        fl("asin", "acc_asin(%s / 8)" % X, np.arcsin((x / dt(8)).astype(np.float64)), 8)
        fl("acos", "acc_acos(%s / 8)" % X, np.arccos((x / dt(8)).astype(np.float64)), 8)
        fl("atanh", "acc_atanh(%s / 9)" % X, np.arctanh((x / dt(9)).astype(np.float64)), 16)
        fl("acosh", "acc_acosh(acc_abs(%s) + 1)" % X, np.arccosh((np.abs(x) + one).astype(np.float64)), 16)
        fl("pow", "acc_pow(acc_abs(%s), %s)" % (X, Y), np.power(np.abs(x).astype(np.float64), y.astype(np.float64)), 16)
        fl("atan2", "acc_atan2(%s, %s)" % (X, Y), np.arctan2(x.astype(np.float64), y.astype(np.float64)), 8)
        lb = (np.log(np.abs(y).astype(np.float64)).astype(dt) / np.log(np.abs(x).astype(np.float64)).astype(dt))
        fl("logBase", "acc_log_base(acc_abs(%s), acc_abs(%s))" % (X, Y), lb, 32)
        fl("max (fmax)", "acc_pmax(%s, %s)" % (X, Y), np.fmax(x, y), 0)
        fl("min (fmin)", "acc_pmin(%s, %s)" % (X, Y), np.fmin(x, y), 0)
    say(tname, "isNaN")
    got = run_map(A, ctx, tname, dt, "acc_is_nan(%s)" % X, x, y, out_t="Word8", out_dt=np.uint8)
    assert np.array_equal(got, np.isnan(x).astype(np.uint8))

    # RealFrac, on values an Int32 holds: round is C's (halves away from zero)
    xr = np.where(np.isfinite(x), x, dt(0)) * dt(1000)
    xr[:8] = [0.5, -0.5, 1.5, -1.5, 2.5, -2.5, 0.49999997, -0.49999997]
    for name, f in (("truncate", np.trunc), ("floor", np.floor), ("ceiling", np.ceil),
                    ("round", lambda v: np.copysign(np.floor(np.abs(v.astype(np.float64)) + 0.5), v))):
        say(tname, name)
        got = run_map(A, ctx, tname, dt, "acc_%s<Int32>(%s)" % (name, X), xr, y, out_t="Int32", out_dt=np.int32)
        assert np.array_equal(got, f(xr).astype(np.int32)), name


def test_conversions(A, ctx):
    say("fromIntegral, ord, chr, boolToInt")
    x = np.array([-5, -1, 0, 1, 65, 255, 256, 70000, -70000, 2 ** 31 - 1, -2 ** 31], np.int32)
    y = np.ones_like(x)
    for to, dt in (("Int8", np.int8), ("Word8", np.uint8), ("Word16", np.uint16), ("Int64", np.int64), ("Word64", np.uint64),
                   ("float", np.float32), ("double", np.float64)):
        got = run_map(A, ctx, "Int32", np.int32, "acc_from_integral<%s>(arrIn0_0[ix])" % to, x, y, out_t=to, out_dt=dt)
        assert np.array_equal(got, x.astype(dt)), to
    got = run_map(A, ctx, "Int32", np.int32, "acc_ord(acc_chr(arrIn0_0[ix])) + acc_bool_to_int((Word8)(arrIn0_0[ix] > 0))",
                  x, y, out_t="Int64", out_dt=np.int64)
    assert np.array_equal(got, x.astype(np.uint32).astype(np.int64) + (x > 0))
