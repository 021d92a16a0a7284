"""Waits inside kernels are bounded and a wait that runs out is reported: the kernel ends normally and the next
synchronising call returns ACC_ERR_STUCK, once.  The conditions are forced from the host -- a lock word left at 1, a
poll limit of zero -- so that every kernel here exits by itself.  Also: the scratch pool gives its memory back."""
import os
import sys

import numpy as np
import pytest

pytestmark = pytest.mark.gpu


def say(*a):
    print("[case]", *a)
    sys.stdout.flush()


@pytest.fixture(scope="module")
def A():
    import acchip
    return acchip


@pytest.fixture()
def ctx(A):
    c = A.Context(0)
    yield c
    c.close()


def tuned(text, ctx):
    """knobs for the skeletons created inside the block (they become part of the generated source)"""
    import acchip
    return acchip.tuning(text, ctx)


def test_a_lock_that_never_opens_is_reported_and_cleaned_up(A, ctx):
    I32 = (1, "Int32")
    bins, n = 1000, 2000          # fewer than four elements a target: per-target locks in memory, not tables in LDS
    rng = np.random.default_rng(3)
    keys = rng.integers(0, bins, n, dtype=np.int32)
    keys[:8] = 5
    want = np.bincount(keys, minlength=bins).astype(np.int16)
    with tuned("spin_limit=2000", ctx):
        sk = ctx.skeleton(A.SKEL_PERMUTE, "Int16", env=[I32], out_rank=1, get="(Int16)1", combine="(Int16)(x + y)",
                          permutation="arrIn0_0[ix]")
    dk, zero, out = ctx.array(keys), ctx.array(np.zeros(bins, np.int16)), ctx.empty(bins, np.int16)
    say("locked permute, healthy")
    sk.permute([dk], n, zero, out)
    ctx.sync()
    assert np.array_equal(out.get(), want)

    say("locked permute with the lock of target 5 held by nobody: the lanes for it give up")
    A.check(A.lib().acc_context_debug_poke_lock(ctx.handle, 5, 1))
    sk.permute([dk], n, zero, out)
    with pytest.raises(A.AccError) as e:
        ctx.sync()
    assert e.value.code == A.ERR_STUCK and "permute lock" in str(e.value)
    got = out.get()                                   # reported once: this copy is clean
    others = np.arange(bins) != 5
    assert np.array_equal(got[others], want[others]) and got[5] == 0

    say("the next locked permute starts from clean locks")
    sk.permute([dk], n, zero, out)
    ctx.sync()
    assert np.array_equal(out.get(), want)
    with pytest.raises(A.AccError) as e:
        A.check(A.lib().acc_context_debug_poke_lock(ctx.handle, 1 << 30, 1))
    assert e.value.code == A.ERR_INVALID
    sk.destroy()


def test_scan_and_fold_with_no_patience_still_end(A, ctx, orc):
    """poll limit zero: a tile whose predecessor has not posted yet gives up at once.  Whether any does is a matter of
    timing; the kernels end either way, a run that reports nothing is right, and the healthy instances are unharmed."""
    I32 = (1, "Int32")
    rng = np.random.default_rng(4)
    n = (1 << 22) + 123
    x = rng.integers(-8, 8, n, dtype=np.int32)
    dx = ctx.array(x)
    with tuned("spin_limit=0", ctx):
        scan0 = ctx.skeleton(A.SKEL_SCANL, "Int32", env=[I32], get="arrIn0_0[ix]", combine="x + y", seed="0")
        fold0 = ctx.skeleton(A.SKEL_FOLD, "Int32", env=[I32], out_rank=0, get="arrIn0_0[ix]", combine="x + y", seed="0")
    scan = ctx.skeleton(A.SKEL_SCANL, "Int32", env=[I32], get="arrIn0_0[ix]", combine="x + y", seed="0")
    fold = ctx.skeleton(A.SKEL_FOLD, "Int32", env=[I32], out_rank=0, get="arrIn0_0[ix]", combine="x + y", seed="0")
    want = orc.scan("scanl", orc.OP_ADD, x, seed=0)
    out, tot = ctx.empty(n + 1, np.int32), ctx.empty((), np.int32)
    for name, run, check in (("scan", lambda: scan0.scan([dx], n, out), lambda: np.array_equal(out.get(), want)),
                             ("fold", lambda: fold0.fold([dx], n, tot), lambda: int(tot.get()) == int(x.sum()))):
        say(name, "with a poll limit of zero")
        run()
        try:
            ctx.sync()
            stuck = False
        except A.AccError as e:
            assert e.code == A.ERR_STUCK
            stuck = True
        say(name, "gave up" if stuck else "needed no patience")
        if not stuck:
            assert check()
    say("the same operands through the patient instances")
    scan.scan([dx], n, out)
    fold.fold([dx], n, tot)
    ctx.sync()
    assert np.array_equal(out.get(), want) and int(tot.get()) == int(x.sum())
    for s in (scan0, fold0, scan, fold):
        s.destroy()


def test_the_scratch_pool_gives_its_memory_back(A, ctx, orc):
    I32 = (1, "Int32")
    n = (1 << 21) + 5
    x = np.random.default_rng(6).integers(0, 100000, n, dtype=np.int32)
    dx = ctx.array(x)
    scan = ctx.skeleton(A.SKEL_SCANL1, "Int32", env=[I32], get="arrIn0_0[ix]", combine="x + y")
    hist = ctx.skeleton(A.SKEL_PERMUTE, "Int32", env=[I32], out_rank=1, get="1", combine="x + y", permutation="arrIn0_0[ix]",
                        combine_hint=A.COMBINE_ADD)
    out, bins = ctx.empty(n, np.int32), ctx.empty(100000, np.int32)
    zero = ctx.array(np.zeros(100000, np.int32))
    assert ctx.scratch_bytes() == 0
    for rep in range(2):
        say("scan and a 100000-bin histogram, then trim: round", rep)
        scan.scan([dx], n, out)
        hist.permute([dx], n, zero, bins)
        ctx.sync()
        held = ctx.scratch_bytes()
        assert held > 0
        assert np.array_equal(out.get(), np.cumsum(x, dtype=np.int32))
        assert np.array_equal(bins.get(), np.bincount(x, minlength=100000).astype(np.int32))
        assert ctx.trim() == held and ctx.scratch_bytes() == 0
    scan.destroy()
    hist.destroy()
