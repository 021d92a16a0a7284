"""Driver layer of the C ABI on a real device: memory, transfers, streams,
events, run-time compilation + module loading + raw launches, occupancy, and
the scratch pool under two streams."""
import ctypes as C
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


@pytest.fixture(scope="module")
def ctx(A):
    c = A.Context(0)
    yield c
    c.close()


def test_device_properties_and_memory(A, ctx):
    say("props / malloc / copies / memset")
    L = A.lib()
    n = C.c_int(0)
    A.check(L.acc_device_count(C.byref(n)))
    assert n.value >= 1
    p = ctx.props()
    assert p.arch.decode().startswith("gfx950") and p.wavefront_size == 64 and p.compute_units >= 64
    assert p.lds_per_block >= 65536 and p.total_mem > (1 << 33)
    free, total = C.c_size_t(), C.c_size_t()
    A.check(L.acc_mem_info(ctx.handle, C.byref(free), C.byref(total)))
    assert 0 < free.value <= total.value
    host = np.arange(100003, dtype=np.int32)
    a, b = ctx.array(host), ctx.empty(host.size, np.int32)
    A.check(L.acc_memcpy_d2d(ctx.handle, b.ptr, a.ptr, host.nbytes))
    assert np.array_equal(b.get(), host)
    A.check(L.acc_memset32_async(ctx.handle, b.ptr, 0xDEADBEEF, 1000, None))
    ctx.sync()
    got = b.get()
    assert np.all(got[:1000].view(np.uint32) == 0xDEADBEEF) and np.array_equal(got[1000:], host[1000:])
    # zero-sized arrays get a real pointer; freeing NULL is a no-op
    z = ctx.empty(0, np.float32)
    assert z.ptr != 0
    assert L.acc_free(ctx.handle, 0) == A.OK
    # an absurd request is the recoverable out-of-memory status, not a crash (Array/Remote.hs:63-67)
    ptr = C.c_uint64(0)
    rc = L.acc_malloc(ctx.handle, C.c_size_t(1 << 46), C.byref(ptr))
    assert rc == A.ERR_OOM and ptr.value == 0 and "memory" in L.acc_last_error().decode().lower()
    # and the device is still usable afterwards
    assert np.array_equal(ctx.array(host).get(), host)


def test_streams_events_and_pinned_transfers(A, ctx):
    say("streams / events / pinned async copies")
    L = A.lib()
    s = ctx.stream()
    e0, e1 = ctx.event(True), ctx.event(True)
    n = 1 << 22
    hp = C.c_void_p()
    A.check(L.acc_host_alloc(ctx.handle, n * 4, C.byref(hp)))
    src = np.ctypeslib.as_array(C.cast(hp, C.POINTER(C.c_int32)), shape=(n,))
    src[:] = np.arange(n, dtype=np.int32)
    d = ctx.empty(n, np.int32)
    hq = C.c_void_p()
    A.check(L.acc_host_alloc(ctx.handle, n * 4, C.byref(hq)))
    dst = np.ctypeslib.as_array(C.cast(hq, C.POINTER(C.c_int32)), shape=(n,))
    dst[:] = 0
    ctx.record(e0, s)
    A.check(L.acc_memcpy_h2d_async(ctx.handle, C.c_uint64(d.ptr), hp, C.c_size_t(n * 4), s))
    A.check(L.acc_memcpy_d2h_async(ctx.handle, hq, C.c_uint64(d.ptr), C.c_size_t(n * 4), s))
    ctx.record(e1, s)
    A.check(L.acc_stream_sync(ctx.handle, s))
    assert np.array_equal(dst, src)
    assert ctx.elapsed_ms(e0, e1) > 0
    done = C.c_int(0)
    A.check(L.acc_event_query(ctx.handle, e1, C.byref(done)))
    assert done.value == 1
    s2 = ctx.stream()
    A.check(L.acc_stream_wait_event(ctx.handle, s2, e1))
    A.check(L.acc_stream_sync(ctx.handle, s2))
    for ev in (e0, e1):
        A.check(L.acc_event_destroy(ctx.handle, ev))
    for st in (s, s2):
        A.check(L.acc_stream_destroy(ctx.handle, st))
    A.check(L.acc_host_free(ctx.handle, hp))
    A.check(L.acc_host_free(ctx.handle, hq))
    say("streams and events that are given back idle are handed out again")
    given = {st.value for st in (s, s2)}
    again = [ctx.stream(), ctx.stream()]
    assert {st.value for st in again} == given
    timed = {e0.value, e1.value}
    e2, e3 = ctx.event(False), ctx.event(True)
    assert e3.value in timed and e2.value not in timed              # pooled by kind: an untimed event is a new one
    # a stream that is given back with work pending is not kept: the work still completes
    busy = again[0]
    big = ctx.empty(1 << 26, np.int32)
    A.check(L.acc_memset32_async(ctx.handle, C.c_uint64(big.ptr), 7, C.c_size_t(1 << 26), busy))
    A.check(L.acc_stream_destroy(ctx.handle, busy))
    ctx.sync()
    assert int(big.get()[-1]) == 7
    A.check(L.acc_stream_destroy(ctx.handle, again[1]))
    for ev in (e2, e3):
        A.check(L.acc_event_destroy(ctx.handle, ev))


def test_compile_load_launch_a_raw_kernel(A, ctx):
    """acc_compile -> acc_module_load -> acc_module_get_function -> acc_launch: what
    Compile.hs:484-538 (link) and Execute.hs:958-978 (launch) do with the driver API"""
    say("raw kernel through the driver layer")
    L = A.lib()
    src = b"""
extern "C" __global__ void axpy(const float a, const float *x, float *y, const long long n)
{
  const long long i = (long long)blockIdx.x * blockDim.x + threadIdx.x;
  if (i < n) y[i] = a * x[i] + y[i];
}
"""
    opts = (C.c_char_p * 2)(b"-O3", b"-ffp-contract=off")
    code, size = C.c_void_p(), C.c_size_t()
    A.check(L.acc_compile(ctx.handle, None, src, opts, 2, C.byref(code), C.byref(size)))     # target = the context's device
    mod, fn = C.c_void_p(), C.c_void_p()
    L.acc_module_load.argtypes = [C.c_void_p, C.c_void_p, C.c_size_t, C.POINTER(C.c_void_p)]
    L.acc_module_get_function.argtypes = [C.c_void_p, C.c_void_p, C.c_char_p, C.POINTER(C.c_void_p)]
    L.acc_function_attr.argtypes = [C.c_void_p, C.c_void_p, C.c_int, C.POINTER(C.c_int)]
    L.acc_occupancy.argtypes = [C.c_void_p, C.c_void_p, C.c_int, C.c_size_t, C.POINTER(C.c_int)]
    L.acc_launch.argtypes = [C.c_void_p, C.c_void_p, C.c_uint32, C.c_uint32, C.c_uint32, C.c_void_p, C.POINTER(C.c_void_p)]
    L.acc_module_unload.argtypes = [C.c_void_p, C.c_void_p]
    A.check(L.acc_module_load(ctx.handle, code, size, C.byref(mod)))
    assert L.acc_module_get_function(ctx.handle, mod, b"nope", C.byref(fn)) == A.ERR_NOT_FOUND
    A.check(L.acc_module_get_function(ctx.handle, mod, b"axpy", C.byref(fn)))
    regs, occ = C.c_int(0), C.c_int(0)
    A.check(L.acc_function_attr(ctx.handle, fn, 0, C.byref(regs)))
    A.check(L.acc_occupancy(ctx.handle, fn, 256, 0, C.byref(occ)))
    assert regs.value > 0 and 1 <= occ.value <= 32
    n = 100001
    x = np.random.default_rng(0).random(n).astype(np.float32)
    y = np.random.default_rng(1).random(n).astype(np.float32)
    dx, dy = ctx.array(x), ctx.array(y)
    a_, px, py, n_ = C.c_float(3.0), C.c_uint64(dx.ptr), C.c_uint64(dy.ptr), C.c_longlong(n)
    args = (C.c_void_p * 4)(C.cast(C.byref(a_), C.c_void_p), C.cast(C.byref(px), C.c_void_p),
                            C.cast(C.byref(py), C.c_void_p), C.cast(C.byref(n_), C.c_void_p))
    grid = L.acc_launch_grid(n, 256, 1 << 30, 1)
    A.check(L.acc_launch(ctx.handle, fn, grid, 256, 0, None, args))
    ctx.sync()
    assert np.array_equal(dy.get(), (np.float32(3.0) * x).astype(np.float32) + y)
    assert L.acc_launch(ctx.handle, fn, 0, 256, 0, None, args) == A.ERR_INVALID          # shape is checked on the host
    assert L.acc_launch(ctx.handle, fn, 1, 4096, 0, None, args) == A.ERR_INVALID
    A.check(L.acc_module_unload(ctx.handle, mod))


def test_skeleton_info_source_and_wrong_use(A, ctx):
    say("kernel record, generated source, misuse is a status")
    I32 = (1, "Int32")
    sk = ctx.skeleton(A.SKEL_SCANL, "Int32", env=[I32], get="arrIn0_0[ix]", combine="x + y", seed="0")
    info = sk.info()
    assert info.entry == b"scanl" and info.block % 64 == 0 and info.blocks_per_cu >= 1 and info.num_regs > 0
    assert info.elements_per_block == info.block * 32 or info.elements_per_block > 0
    assert '#include "skel_scan.h"' in sk.source() and "#define ACC_COMBINE(x, y) x + y" in sk.source()
    x = ctx.array(np.ones(10, np.int32))
    out = ctx.empty(5, np.int32)
    with pytest.raises(A.AccError) as e:                      # result too small
        sk.scan([x], 10, out)
    assert e.value.code == A.ERR_INVALID
    with pytest.raises(A.AccError) as e:                      # wrong driver for this skeleton
        sk.map([x], out)
    assert e.value.code == A.ERR_INVALID
    with pytest.raises(A.AccError) as e:                      # env array of the wrong rank
        sk.scan([ctx.array(np.ones((2, 5), np.int32))], 10, ctx.empty(11, np.int32))
    assert e.value.code == A.ERR_INVALID
    sk.destroy()


def test_scratch_pool_with_two_streams(A, ctx, orc):
    """temporaries (tile descriptors, partials) are pooled per context; two streams must not
    trample each other's, and interleaved launches must still be right"""
    say("scans and folds interleaved on two streams")
    I32 = (1, "Int32")
    rng = np.random.default_rng(5)
    scan = ctx.skeleton(A.SKEL_SCANL, "Int32", env=[I32], get="arrIn0_0[ix]", combine="x + y", seed="0")
    fold = ctx.skeleton(A.SKEL_FOLD, "Int32", env=[I32], out_rank=0, get="arrIn0_0[ix]", combine="x + y", seed="0")
    s1, s2 = ctx.stream(), ctx.stream()
    n = (1 << 21) + 77
    xs = [rng.integers(0, 16, n, dtype=np.int32) for _ in range(4)]
    dxs = [ctx.array(x) for x in xs]
    outs = [ctx.empty(n + 1, np.int32) for _ in range(4)]
    sums = [ctx.empty((), np.int32) for _ in range(4)]
    for rep in range(3):
        for i in range(4):
            st = s1 if i % 2 == 0 else s2
            scan.scan([dxs[i]], n, outs[i], stream=st)
            fold.fold([dxs[i]], n, sums[i], stream=st)
    ctx.sync()
    for i in range(4):
        assert np.array_equal(outs[i].get(), orc.scan("scanl", orc.OP_ADD, xs[i], seed=0))
        assert int(sums[i].get()) == int(xs[i].sum())


def test_scans_larger_than_the_device_on_two_streams(A, ctx):
    """scans of many more tiles than the device holds at once, enqueued alternately on two streams and from two
    threads: the library keeps such scans from sharing the device (tiles of one must not wait for room that waiting
    tiles of the other hold), so the results are right and nothing is reported"""
    import threading
    I32 = (1, "Int32")
    scan = ctx.skeleton(A.SKEL_SCANL1, "Int32", env=[I32], get="arrIn0_0[ix]", combine="x + y")
    tile = scan.info().elements_per_block
    n = 1500 * tile + 11
    say("scanl1 of", n, "elements =", n // tile + 1, "tiles, twice on each of two streams")
    rng = np.random.default_rng(9)
    xs = [rng.integers(0, 16, n, dtype=np.int32) for _ in range(2)]
    dxs = [ctx.array(x) for x in xs]
    outs = [ctx.empty(n, np.int32) for _ in range(2)]
    streams = [ctx.stream(), ctx.stream()]
    for rep in range(2):
        for i in range(2):
            scan.scan([dxs[i]], n, outs[i], stream=streams[i])
    ctx.sync()
    for i in range(2):
        assert np.array_equal(outs[i].get(), np.cumsum(xs[i], dtype=np.int32))
    say("the same from two host threads")
    errors = []

    def work(i):
        try:
            for rep in range(3):
                scan.scan([dxs[i]], n, outs[i], stream=streams[i])
            A.check(A.lib().acc_stream_sync(ctx.handle, streams[i]))
        except Exception as e:                          # noqa: BLE001
            errors.append(e)
    threads = [threading.Thread(target=work, args=(i,)) for i in range(2)]
    for t in threads:
        t.start()
    for t in threads:
        t.join()
    assert not errors, errors
    for i in range(2):
        assert np.array_equal(outs[i].get(), np.cumsum(xs[i], dtype=np.int32))
    for st in streams:                                # a destroyed stream is not waited on by the next big scan
        A.check(A.lib().acc_stream_destroy(ctx.handle, st))
    scan.scan([dxs[0]], n, outs[0])
    ctx.sync()
    assert np.array_equal(outs[0].get(), np.cumsum(xs[0], dtype=np.int32))
    scan.destroy()


def test_a_loop_enqueued_ahead_under_a_guard(A, ctx):
    """awhile at the C ABI: twenty iterations of `predicate; latch; body` enqueued without looking at the device, the
    kernels past the loop's end do nothing, the guard says how many iterations were taken; an instance built
    without ACC_FLAG_GUARDED is refused on a stream that is under a guard"""
    I64 = (1, "Int64")
    n = 100003
    x = np.random.default_rng(10).integers(1, 50, n).astype(np.int64)
    G = A.FLAG_GUARDED
    dbl = ctx.skeleton(A.SKEL_MAP, "Int64", env=[I64], out_rank=1, get="arrIn0_0[ix] * 2", flags=G)
    mx = ctx.skeleton(A.SKEL_FOLD, "Int64", env=[I64], out_rank=0, get="arrIn0_0[ix]", combine="acc_max(x, y)", seed="0", flags=G)
    small = ctx.skeleton(A.SKEL_MAP, "Word8", env=[(0, "Int64")], out_rank=0, get="(Word8)(arrIn0_0[0] < 1000000)", flags=G)
    plain = ctx.skeleton(A.SKEL_MAP, "Int64", env=[I64], out_rank=1, get="arrIn0_0[ix] * 2")
    st = ctx.stream()
    guard = A.Guard(ctx)
    bufs = [ctx.array(x)] + [ctx.array(np.full(n, -1, np.int64)) for _ in range(20)]
    top, flag = ctx.empty((), np.int64), ctx.empty((), np.uint8)
    say("twenty iterations enqueued ahead; the doubling stops when the largest element passes a million")
    guard.attach(st)
    guard.reset(st)
    for k in range(20):
        mx.fold([bufs[k]], n, top, stream=st)
        small.map([top], flag, stream=st)
        guard.latch(flag, st)
        dbl.map([bufs[k]], bufs[k + 1], stream=st)
    with pytest.raises(A.AccError) as e:
        plain.map([bufs[0]], bufs[1], stream=st)
    assert e.value.code == A.ERR_INVALID and "ACC_FLAG_GUARDED" in str(e.value)
    alive, count = guard.read(st)
    ref, steps = x.copy(), 0
    while ref.max() < 1000000:
        ref, steps = ref * 2, steps + 1
    assert not alive and count == steps and 10 < steps < 20
    assert np.array_equal(bufs[count].get(), ref)
    assert np.all(bufs[count + 1].get() == -1) and np.all(bufs[20].get() == -1)       # the iterations past the end wrote nothing
    guard.detach(st)
    plain.map([bufs[0]], bufs[1], stream=st)              # the stream takes any instance again
    dbl.map([bufs[0]], bufs[2], stream=st)                # and a guarded instance runs unconditionally off a guard
    ctx.sync()
    assert np.array_equal(bufs[1].get(), x * 2) and np.array_equal(bufs[2].get(), x * 2)
    guard.destroy()
    for s_ in (dbl, mx, small, plain):
        s_.destroy()


def test_one_skeleton_launched_from_several_threads(A, ctx):
    """the reference runs every computation in a bound thread of its own (State.hs:84-92):
    threads sharing a context and a skeleton, each on its own stream, misaligned inputs so
    that the lazily built second variant is first needed by all of them at once"""
    import threading
    say("four host threads, one scan skeleton, one stream each")
    I32 = (1, "Int32")
    scan = ctx.skeleton(A.SKEL_SCANL1, "Int32", env=[I32], get="arrIn0_0[ix]", combine="x + y")
    n = (1 << 20) + 5
    rng = np.random.default_rng(8)
    results, errors = {}, []

    def work(k):
        try:
            st = ctx.stream()
            x = rng.integers(0, 16, n + 1, dtype=np.int32)
            dx = ctx.array(x)
            out = ctx.empty(n, np.int32)
            for rep in range(5):
                # a view that starts 4 bytes into the buffer: not 16-byte aligned
                scan.scan([dx.desc(shape=(n,), offset_elems=1)], n, out, stream=st)
            A.check(A.lib().acc_stream_sync(ctx.handle, st))
            results[k] = np.array_equal(out.get(), np.cumsum(x[1:], dtype=np.int32))
        except Exception as e:                          # noqa: BLE001
            errors.append(e)
    threads = [threading.Thread(target=work, args=(k,)) for k in range(4)]
    for t in threads:
        t.start()
    for t in threads:
        t.join()
    assert not errors, errors
    assert results == {0: True, 1: True, 2: True, 3: True}


def test_the_c_client_of_the_abi():
    """tests/c_abi/client.c: the benchmark programs and the memory table from plain C, checked against loops in C"""
    import os
    import subprocess
    exe = os.path.join(os.path.dirname(os.path.abspath(__file__)), "c_abi", "client")
    assert os.path.exists(exe), "build it first: make -C tests/c_abi (or __graft_entry__.build())"
    say("C client")
    out = subprocess.run([exe], capture_output=True, text=True, timeout=300)
    print(out.stdout)
    assert out.returncode == 0 and "all checks passed" in out.stdout, out.stdout + out.stderr
