"""The scan entry point that allocates nothing (acc_exec_scan_noalloc) against acc_exec_scan, through the C ABI.

Both run the same kernel; the one keeps its tile descriptors in a block of the context's pool, the other in the
library's file-scope device array.  Results must agree bit for bit, on calls in a row of which the later ones are
smaller (the array keeps what the earlier call left there), and limits must be refused with a clear error.
"""
import sys

import numpy as np
import pytest

pytestmark = pytest.mark.gpu

I32 = (1, "Int32")


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


def test_noalloc_scan_agrees_with_the_allocating_entry_point_on_two_calls_in_a_row(A, ctx, orc):
    rng = np.random.default_rng(5)
    for kind in ("scanl", "scanr1", "scanl'"):
        sk = ctx.skeleton(A.SCAN_KINDS[kind], "Int32", env=[I32], get="arrIn0_0[ix]", combine="x + y",
                          seed=None if kind.endswith("1") else "7")
        tile = sk.info().elements_per_block
        # the second and third call are smaller than the first: what the first left in the array must not be taken
        # for this call's descriptors
        for n in (5 * tile + 12345, 2 * tile + 1, 1000, 0, 3 * tile):
            say("noalloc", kind, "n =", n)
            x = rng.integers(-50, 50, size=n, dtype=np.int32)
            dx = ctx.array(x)
            extra = 1 if kind == "scanl" else 0
            ref_out, got_out = ctx.empty(n + extra, np.int32), ctx.empty(n + extra, np.int32)
            ref_tot, got_tot = ctx.empty((), np.int32), ctx.empty((), np.int32)
            primed = kind.endswith("'")
            sk.scan([dx], n, ref_out, total=ref_tot if primed else None)
            sk.scan([dx], n, got_out, total=got_tot if primed else None, noalloc=True)
            assert np.array_equal(got_out.get(), ref_out.get()), (kind, n)
            if primed:
                assert int(got_tot.get()) == int(ref_tot.get())
            # and both against the oracle
            want = orc.scan(kind, orc.OP_ADD, x, seed=0 if kind.endswith("1") else 7)
            assert np.array_equal(got_out.get(), want[0] if primed else want), (kind, n)


def test_noalloc_scan_of_wider_elements_and_pairs(A, ctx):
    rng = np.random.default_rng(6)
    sk = ctx.skeleton(A.SKEL_SCANL1, "double", env=[(1, "double")], get="arrIn0_0[ix]", combine="acc_max(x, y)")
    for n in (300001, 777):
        say("noalloc scanl1 max double n =", n)
        x = rng.standard_normal(n)
        dx = ctx.array(x)
        a, b = ctx.empty(n, np.float64), ctx.empty(n, np.float64)
        sk.scan([dx], n, a)
        sk.scan([dx], n, b, noalloc=True)
        assert np.array_equal(a.get(), b.get()) and np.array_equal(b.get(), np.maximum.accumulate(x))


def test_noalloc_scan_refuses_what_it_cannot_do_without_allocating(A, ctx):
    sk = ctx.skeleton(A.SKEL_SCANL1, "Int32", env=[I32], get="arrIn0_0[ix]", combine="x + y")
    tile = sk.info().elements_per_block
    n = 4096
    x = np.arange(n + 4, dtype=np.int32)
    dx = ctx.array(x)
    out = ctx.empty(n + 4, np.int32)
    # more tiles than the array has descriptors for: refused before anything is launched (the sizes are only named)
    big = out.desc(shape=(tile * 8193,))
    env = [dx.desc(shape=(tile * 8193,))]
    say("noalloc: too many tiles")
    with pytest.raises(A.AccError) as e:
        sk.scan(env, tile * 8193, big, noalloc=True)
    assert e.value.code == A.ERR_INVALID and "8192" in e.value.message
    # operands that need the unaligned variant, which nothing has loaded yet
    say("noalloc: unaligned variant not loaded")
    shifted_in = dx.desc(shape=(n,))
    shifted_in.ptr[0] += 4
    with pytest.raises(A.AccError) as e:
        sk.scan([shifted_in], n, out, noalloc=True)
    assert e.value.code == A.ERR_INVALID and "not loaded" in e.value.message
    # after one ordinary call on such operands it is there
    sk.scan([shifted_in], n, out)
    ref = out.get()[:n].copy()
    out2 = ctx.empty(n + 4, np.int32)
    sk.scan([shifted_in], n, out2, noalloc=True)
    assert np.array_equal(out2.get()[:n], ref) and np.array_equal(ref, np.cumsum(x[1:n + 1], dtype=np.int32))


def test_noalloc_scan_recorded_into_a_graph_and_replayed_on_changing_inputs(A, ctx, orc):
    """The entry point is for callers under HIP graph capture.  A recorded launch keeps its arguments, so the launch's
    tag is not among them: it is counted on the device by a kernel recorded in front of the scan.  Here one call is
    recorded and the graph replayed several times, the input changed between the replays (the second input is chosen
    so that tiles published by the first replay would give a wrong result if they were taken for this one's), eager
    scans and synchronisations of the program's own in between; every replay is checked against the eager result."""
    import ctypes as C
    hip = C.CDLL("libamdhip64.so")
    for name in ("hipStreamBeginCapture", "hipStreamEndCapture", "hipGraphInstantiate", "hipGraphLaunch", "hipGraphExecDestroy",
                 "hipGraphDestroy", "hipStreamSynchronize"):
        getattr(hip, name).restype = C.c_int
    hip.hipStreamBeginCapture.argtypes = [C.c_void_p, C.c_int]
    hip.hipStreamEndCapture.argtypes = [C.c_void_p, C.POINTER(C.c_void_p)]
    hip.hipGraphInstantiate.argtypes = [C.POINTER(C.c_void_p), C.c_void_p, C.c_void_p, C.c_void_p, C.c_size_t]
    hip.hipGraphLaunch.argtypes = [C.c_void_p, C.c_void_p]
    hip.hipGraphExecDestroy.argtypes = [C.c_void_p]
    hip.hipGraphDestroy.argtypes = [C.c_void_p]
    hip.hipStreamSynchronize.argtypes = [C.c_void_p]
    rng = np.random.default_rng(6)
    sk = ctx.skeleton(A.SKEL_SCANL, "Int32", env=[I32], get="arrIn0_0[ix]", combine="x + y", seed="0", wait=True)
    tile = sk.info().elements_per_block
    n = 700 * tile + 77                           # more tiles than are resident at once: the look-back really waits
    stream = ctx.stream()
    dx, got, ref = ctx.empty(n, np.int32), ctx.empty(n + 1, np.int32), ctx.empty(n + 1, np.int32)
    x0 = rng.integers(-50, 50, size=n, dtype=np.int32)
    dx.set(x0)
    sk.scan([dx], n, ref, stream=stream)          # the variant is loaded; and the eager result of the first input
    sk.scan([dx], n, got, stream=stream, noalloc=True)
    ctx.sync()
    assert np.array_equal(got.get(), ref.get())
    sk.scan([dx], 3 * tile + 1, ref, stream=stream)            # (loads the small-tile variant the calls between the replays take)
    graph, graph_exec = C.c_void_p(), C.c_void_p()
    assert hip.hipStreamBeginCapture(stream, 2) == 0          # hipStreamCaptureModeRelaxed
    try:
        sk.scan([dx], n, got, stream=stream, noalloc=True)
    finally:
        rc = hip.hipStreamEndCapture(stream, C.byref(graph))
    assert rc == 0 and graph.value
    assert hip.hipGraphInstantiate(C.byref(graph_exec), graph, None, None, 0) == 0
    try:
        for replay in range(5):
            x = rng.integers(-50, 50, size=n, dtype=np.int32) if replay != 1 else (x0 // 2).astype(np.int32)
            say("graph replay", replay)
            dx.set(x)
            got.set(np.full(n + 1, -1, np.int32))
            assert hip.hipGraphLaunch(graph_exec, stream) == 0
            assert hip.hipStreamSynchronize(stream) == 0
            want = orc.scan("scanl", orc.OP_ADD, x, seed=0)
            assert np.array_equal(got.get(), want), replay
            # the program's own eager work between the replays: an allocating scan and a smaller no-alloc one
            sk.scan([dx], n, ref, stream=stream)
            sk.scan([dx], 3 * tile + 1, ref, stream=stream, noalloc=True)
            ctx.sync()
    finally:
        hip.hipGraphExecDestroy(graph_exec)
        hip.hipGraphDestroy(graph)
