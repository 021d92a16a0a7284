"""The memory table of the C ABI on a real device: host arrays entered once, blocks reused through the nursery,
least-recently-used eviction under a budget with write-back of arrays produced on the device, arrays in use never
evicted, unmanaged memory left alone.  The budget stands in for a full device: nothing here exhausts the GPU."""
import sys

import numpy as np
import pytest

pytestmark = pytest.mark.gpu

MB = 1 << 20
N = 4 * MB                    # elements of one 16 MiB float array


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


@pytest.fixture(scope="module")
def kernels(A, ctx):
    F = (1, "float")
    return {"double": ctx.skeleton(A.SKEL_MAP, "float", env=[F], out_rank=1, get="2.0f * arrIn0_0[ix]"),
            "add": ctx.skeleton(A.SKEL_MAP, "float", env=[F, F], out_rank=1, get="arrIn0_0[ix] + arrIn1_0[ix]")}


def host_arrays(k, seed):
    rng = np.random.default_rng(seed)
    return [rng.integers(-1000, 1000, N).astype(np.float32) for _ in range(k)]


def test_use_once_then_eviction_writes_back_only_what_the_device_produced(A, ctx, kernels):
    say("budget 64 MiB, five arrays of 16 MiB")
    mt = A.MemTable(ctx, budget_bytes=64 * MB)
    a, b, c = host_arrays(3, 1)
    r1, r2 = np.zeros(N, np.float32), np.zeros(N, np.float32)
    assert mt.malloc(a, frozen=True) and not mt.malloc(a, frozen=True)            # entered once
    assert mt.malloc(b, frozen=True) and mt.malloc(c, frozen=True)
    assert mt.stats()["resident_bytes"] == 0                                       # nothing uploaded before it is wanted
    da = mt.acquire(a)
    assert mt.acquire(a).ptr == da.ptr and mt.stats()["uploads"] == 1              # and uploaded once
    mt.release(a)
    assert mt.malloc(r1, frozen=False)
    d1 = mt.acquire(r1)
    assert mt.stats()["uploads"] == 1                                              # fresh device memory is not uploaded
    kernels["double"].map([da], d1)
    mt.release(a)
    mt.release(r1)
    db, dc = mt.acquire(b), mt.acquire(c)
    st = mt.stats()
    assert st["resident_bytes"] == 64 * MB and st["evictions"] == 0 and st["uploads"] == 3
    ctx.sync()                     # idle arrays are preferred as victims: with nothing running the order is by last use alone
    # a fifth array: the least recently used one, `a`, leaves; its host copy is authoritative, nothing is copied back
    assert mt.malloc(r2, frozen=False)
    st = mt.stats()
    assert st["evictions"] == 1 and st["writebacks"] == 0 and st["resident_bytes"] == 64 * MB
    d2 = mt.acquire(r2)
    kernels["add"].map([db, dc], d2)
    for h in (b, c, r2):
        mt.release(h)
    # `a` is wanted again: now r1 is the oldest, and it exists only on the device -> written back to its host array
    assert not r1.any()
    ctx.sync()
    da = mt.acquire(a)
    st = mt.stats()
    assert st["evictions"] == 2 and st["writebacks"] == 1 and st["writeback_bytes"] == r1.nbytes and st["uploads"] == 4
    assert np.array_equal(r1, 2 * a)
    assert np.array_equal(da.get(), a)
    mt.release(a)
    # r1 comes back from the host copy (evicting b, the oldest by now), r2 was never touched
    ctx.sync()
    d1 = mt.acquire(r1)
    assert np.array_equal(d1.get(), 2 * a) and mt.stats()["evictions"] == 3
    mt.release(r1)
    d2 = mt.acquire(r2)
    assert np.array_equal(d2.get(), b + c)
    mt.release(r2)
    assert mt.stats()["arrays"] == 5 and mt.stats()["resident_arrays"] == 4
    mt.destroy()


def test_arrays_in_use_are_never_evicted_and_oom_is_recoverable(A, ctx):
    say("every resident array acquired")
    mt = A.MemTable(ctx, budget_bytes=32 * MB)
    a, b, c = host_arrays(3, 2)
    for h in (a, b, c):
        mt.malloc(h, frozen=True)
    da, db = mt.acquire(a), mt.acquire(b)
    with pytest.raises(A.AccError) as e:
        mt.acquire(c)
    assert e.value.code == A.ERR_OOM and "in use" in str(e.value)
    assert np.array_equal(da.get(), a) and np.array_equal(db.get(), b)              # both untouched
    mt.release(b)
    dc = mt.acquire(c)                                                              # b may leave now
    assert np.array_equal(dc.get(), c) and mt.stats()["evictions"] == 1
    big = np.zeros(10 * N, np.float32)
    with pytest.raises(A.AccError) as e:
        mt.malloc(big, frozen=False)
    assert e.value.code == A.ERR_OOM and "budget" in str(e.value)
    # errors of use
    with pytest.raises(A.AccError) as e:
        mt.acquire(big)
    assert e.value.code == A.ERR_NOT_FOUND
    with pytest.raises(A.AccError):
        mt.release(b)                                                               # not acquired
    with pytest.raises(A.AccError):
        mt.free(a)                                                                  # still acquired
    with pytest.raises(A.AccError):
        A.check(A.lib().acc_memtable_malloc(mt.handle, mt.key(a), a.ctypes.data, 16, 1, None))   # same key, other size
    mt.release(a)
    mt.release(c)
    mt.destroy()


def test_nursery_reuses_blocks_of_the_same_rounded_size(A, ctx):
    say("nursery")
    mt = A.MemTable(ctx)                                                            # no budget
    x = np.arange(1000, dtype=np.int32)                                             # 4000 bytes -> one 4096-byte block
    y = np.arange(1001, dtype=np.int32)                                             # 4004 bytes -> the same size class
    z = np.arange(5000, dtype=np.int32)
    mt.malloc(x, frozen=False)
    px = mt.acquire(x).ptr
    mt.release(x)
    assert mt.stats()["resident_bytes"] == 4096 and mt.stats()["device_allocs"] == 1
    mt.free(x)
    mt.free(x)                                                                      # twice is harmless
    st = mt.stats()
    assert st["nursery_bytes"] == 4096 and st["resident_bytes"] == 0 and st["arrays"] == 0
    mt.malloc(y, frozen=True)
    dy = mt.acquire(y)
    assert dy.ptr == px and mt.stats()["nursery_hits"] == 1 and mt.stats()["device_allocs"] == 1
    assert np.array_equal(dy.get(), y)
    mt.release(y)
    mt.malloc(z, frozen=False)                                                      # another size: a new block
    assert mt.stats()["device_allocs"] == 2
    mt.free(z)
    assert mt.stats()["nursery_bytes"] == 20480
    mt.reclaim()
    assert mt.stats()["nursery_bytes"] == 0
    e = np.zeros(0, np.float32)                                                     # an empty array still gets a pointer
    mt.malloc(e, frozen=True)
    assert mt.acquire(e).ptr != 0
    mt.release(e)
    mt.destroy()


def test_unmanaged_memory_is_left_alone(A, ctx):
    say("unmanaged")
    mt = A.MemTable(ctx, budget_bytes=32 * MB)
    mine = np.arange(N, dtype=np.float32)
    dev = ctx.array(mine)
    mt.insert_unmanaged(mine, dev)
    a, b, c = host_arrays(3, 3)
    for h in (a, b, c):                                                             # churn through the budget
        mt.malloc(h, frozen=True)
        mt.acquire(h)
        mt.release(h)
    assert mt.stats()["evictions"] == 1
    assert mt.acquire(mine).ptr == dev.ptr
    mt.release(mine)
    mt.free(mine)
    mt.destroy()
    assert np.array_equal(dev.get(), mine)                                          # still the caller's, still valid


def test_eviction_waits_for_the_work_recorded_at_release(A, ctx, kernels):
    say("eviction behind a running stream")
    mt = A.MemTable(ctx, budget_bytes=32 * MB)
    a, = host_arrays(1, 4)
    r = np.zeros(N, np.float32)
    s = ctx.stream()
    mt.malloc(a, frozen=True)
    mt.malloc(r, frozen=False)
    da, dr = mt.acquire(a, s), mt.acquire(r, s)
    for _ in range(20):                                                             # a queue of work on the stream
        kernels["double"].map([da], dr, stream=s)
    mt.release(a, s)
    mt.release(r, s)
    filler = np.zeros(2 * N, np.float32)                                            # 32 MiB: both must leave
    mt.malloc(filler, frozen=False)
    assert mt.stats()["evictions"] == 2 and mt.stats()["writebacks"] == 1
    assert np.array_equal(r, 2 * a)
    mt.destroy()
    A.check(A.lib().acc_stream_destroy(ctx.handle, s))


def test_blocks_used_on_two_streams_wait_for_both(A, ctx, kernels):
    say("two streams, eviction and reuse behind running work")
    mt = A.MemTable(ctx, budget_bytes=48 * MB)
    a, = host_arrays(1, 5)
    r1, r2 = np.zeros(N, np.float32), np.zeros(N, np.float32)
    s1, s2 = ctx.stream(), ctx.stream()
    mt.malloc(a, frozen=True)
    mt.malloc(r1, frozen=False)
    mt.malloc(r2, frozen=False)
    da, d1 = mt.acquire(a, s1), mt.acquire(r1, s1)
    da2, d2 = mt.acquire(a, s2), mt.acquire(r2, s2)              # s2 is made to wait for the upload queued on s1
    assert da2.ptr == da.ptr and mt.stats()["uploads"] == 1
    for _ in range(10):
        kernels["double"].map([da], d1, stream=s1)
        kernels["add"].map([da2, da2], d2, stream=s2)
    mt.release(a, s1)
    mt.release(r1, s1)
    mt.release(a, s2)
    mt.release(r2, s2)
    # everything must leave for a 48 MiB array: each block waits for the streams it was released on
    filler = np.zeros(3 * N, np.float32)
    mt.malloc(filler, frozen=False)
    assert mt.stats()["evictions"] == 3 and mt.stats()["writebacks"] == 2
    assert np.array_equal(r1, 2 * a) and np.array_equal(r2, a + a)
    # a block freed while a kernel still writes it is reused only after that kernel
    mt.free(filler)
    mt.reclaim()
    t = np.zeros(N, np.float32)
    mt.malloc(t, frozen=False)
    da, dt = mt.acquire(a, s1), mt.acquire(t, s1)
    for _ in range(10):
        kernels["double"].map([da], dt, stream=s1)
    mt.release(a, s1)
    mt.release(t, s1)
    mt.free(t)                                                    # returns at once; the block carries s1's event
    u = (np.arange(N) % 7).astype(np.float32)
    mt.malloc(u, frozen=True)
    du = mt.acquire(u, s2)                                        # same size: the same block, uploaded on s2
    assert du.ptr == dt.ptr and mt.stats()["nursery_hits"] >= 1
    A.check(A.lib().acc_stream_sync(ctx.handle, s2))
    assert np.array_equal(du.get(), u)                            # not overwritten by the tail of s1's kernels
    mt.release(u, s2)
    mt.destroy()
    for s in (s1, s2):
        A.check(A.lib().acc_stream_destroy(ctx.handle, s))
