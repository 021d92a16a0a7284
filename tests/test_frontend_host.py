"""The embedded array language without a GPU: what text it generates for the benchmark programs, how it numbers the
free arrays, and that the generated skeleton instances compile for gfx950.  Device arrays are stood in for by objects
with a shape and a dtype; nothing is launched."""
import re

import numpy as np
import pytest

import acchip as A
import accelerate_hip as acc


class Resident(object):
    def __init__(self, shape, dt):
        self.shape, self.dtype = tuple(shape), np.dtype(dt)


def use(shape, dt):
    return acc.Acc(shape, acc.CTYPE[np.dtype(dt).type], manifest=Resident(shape, dt))


def add(x, y):
    return x + y


def test_dotp_fuses_into_one_fold_over_two_streamed_arrays():
    xs, ys = use((100,), np.float32), use((100,), np.float32)
    d = acc.zipWith(lambda a, b: a * b, xs, ys)
    arrays, sig, fr = acc._assemble(get=d.stream().text, combine=acc._combine(add, "float").text,
                                    seed=acc.Exp.of(0.0, "float").text)
    assert arrays == [xs.manifest, ys.manifest] and sig == [(1, "float"), (1, "float")]
    assert fr == {"get": "((float)(acc_stream(arrIn0_0, ix) * acc_stream(arrIn1_0, ix)))",
                  "combine": "((float)(x + y))", "seed": "0.0f"}
    assert A.compile_only(A.make_desc(A.SKEL_FOLD, "float", env=sig, **fr)) > 0
    # the same array twice is one environment slot
    sq = acc.zipWith(lambda a, b: a * b, xs, xs)
    arrays, sig, fr = acc._assemble(get=sq.stream().text)
    assert len(arrays) == 1 and fr["get"].count("arrIn0_0") == 2


def test_free_arrays_are_numbered_in_order_of_first_use_across_fragments():
    ks, ws = use((1000,), np.int32), use((1000,), np.int32)
    target = acc._linear((ks[acc.Exp("Int64", "ix")],), (256,))
    arrays, sig, fr = acc._assemble(get=ws.stream().text, combine=acc._combine(add, "Int32").text, permutation=target.text)
    assert arrays == [ws.manifest, ks.manifest]
    assert fr["permutation"] == "acc_from_integral<Int64>(acc_stream(arrIn1_0, ix))"
    desc = A.make_desc(A.SKEL_PERMUTE, "Int32", env=sig, out_rank=1, combine_hint=acc._hint(add, "Int32"), **fr)
    assert A.compile_only(desc) > 0


def test_combination_hints_are_read_off_the_generated_text():
    assert acc._hint(add, "Int32") == A.COMBINE_ADD
    assert acc._hint(lambda x, y: y + x, "float") == A.COMBINE_ADD
    assert acc._hint(acc.max_, "Int64") == A.COMBINE_MAX
    assert acc._hint(acc.min_, "Word32") == A.COMBINE_MIN
    assert acc._hint(acc.max_, "float") == A.COMBINE_GENERIC           # no floating-point atomic max is assumed
    assert acc._hint(lambda x, y: x ^ y, "Word64") == A.COMBINE_XOR
    assert acc._hint(lambda x, y: acc.cond(x > y, x, y), "Int32") == A.COMBINE_GENERIC
    assert acc._hint(add, "Int16") == A.COMBINE_GENERIC


def test_tuples_live_on_the_host_side_of_the_text():
    ps = acc.Acc((10,), ("Int16", "double"), manifest=Resident((10,), np.int16))
    sw = acc.map(lambda p: acc.lift(acc.snd(p), acc.fst(p)), ps)
    assert sw.ctype == ("double", "Int16")
    text = sw.stream().text
    assert text.startswith("acc_elt{") and text.index("_0[ix]") < text.index("_1[ix]")      # snd first: component 0
    c = acc._combine(lambda p, q: acc.cond(acc.fst(p) >= acc.fst(q), p, q), ("float", "Int32"))
    assert c.text == "acc_elt{(((Word8)(x.a1 >= y.a1)) ? x.a1 : y.a1), (((Word8)(x.a1 >= y.a1)) ? x.a0 : y.a0)}"
    seed = acc.Exp.of((-np.inf, -1), ("float", "Int32"))
    assert seed.text == "acc_elt{(-__builtin_inff()), ((Int32)-1)}"
    desc = A.make_desc(A.SKEL_FOLD, "float, Int32", env=[(1, ["Int32", "float"])],
                       get="acc_elt{arrIn0_1[ix], arrIn0_0[ix]}", combine=c.text, seed=seed.text)
    assert A.compile_only(desc) > 0


def test_components_nobody_uses_are_never_loaded():
    """dead-component elimination (CodeGen.hs:283-314): a fused producer's tuple is a list of component expressions on
    the host, so what a consumer does not use is not in the text -- neither the arithmetic nor the array read, and an
    array that only fed a dead component is not even a kernel parameter"""
    xs, ys = use((100,), np.float32), use((100,), np.int32)
    pairs = acc.zip_(xs, ys)
    firsts = acc.map(lambda p: acc.fst(p) * 2.0, pairs)
    arrays, sig, fr = acc._assemble(get=firsts.stream().text)
    assert arrays == [xs.manifest] and sig == [(1, "float")] and "arrIn1" not in fr["get"]
    # a producer that computes two things per element, a consumer that folds one of them
    both = acc.map(lambda v: acc.lift(acc.sqrt(v), acc.exp(v) + acc.sin(v)), xs)
    roots = acc.map(acc.fst, both)
    arrays, sig, fr = acc._assemble(get=roots.stream().text, combine=acc._combine(add, "float").text, seed=acc.Exp.of(0.0, "float").text)
    assert "acc_sqrt" in fr["get"] and "acc_exp" not in fr["get"] and "acc_sin" not in fr["get"]
    assert A.compile_only(A.make_desc(A.SKEL_FOLD, "float", env=sig, **fr)) > 0
    # a manifest array of pairs: only the component that is used is read (the other pointer is passed and left alone)
    ps = acc.Acc((10,), ("Int16", "double"), manifest=A.TupleArray.__new__(A.TupleArray))
    ps.manifest.comps = [Resident((10,), np.int16), Resident((10,), np.float64)]
    seconds = acc.map(acc.snd, ps)
    text = seconds.stream().text
    assert "_0" in text and "_1" not in text.replace("acc_stream", "")
    # through a conditional: each component selects for itself, so a dead component takes its test with it
    pick = acc.map(lambda p: acc.fst(acc.cond(acc.snd(p) > 0, p, acc.lift(acc.constant(0.0, "float"), acc.snd(p)))), pairs)
    arrays, sig, fr = acc._assemble(get=pick.stream().text)
    assert fr["get"].count("arrIn1_0") == 1                                    # the test, once; no select of the dead Int32 component


def test_index_arithmetic_of_the_delayed_combinators():
    m = use((3, 5), np.int32)
    t = acc.transpose(m)
    assert t.shape == (5, 3)
    arrays, sig, fr = acc._assemble(get=t.stream().text)
    assert sig == [(2, "Int32")]
    ix = np.arange(15)
    y, x = ix // 3, ix % 3                       # the result's (row, column)
    # (the text as Python reads it: casts and literal suffixes off -- the index of so small an array is taken apart in
    # 32 bits -- and the division a floor division)
    text = re.sub(r"\((Int64|Word32)\)", "", fr["get"].replace("arrIn0_0", "src")).replace("LL)", ")")
    text = re.sub(r"(\d)u\b", r"\1", text).replace("/", "//")
    src = eval(text, {"src": np.arange(15), "ix": ix})
    assert np.array_equal(src, x * 5 + y)
    with pytest.raises(TypeError):
        m[acc.Exp("Int64", "ix")]                # a rank-1 index into a matrix
    with pytest.raises(TypeError):
        acc.zipWith(add, m, use((3, 5), np.float32))
    with pytest.raises(TypeError):
        acc._combine(lambda x, y: x < y, "Int32")


def test_while_is_a_statement_ahead_of_the_expression_and_compiles():
    xs = use((64,), np.int64)
    r = acc.map(lambda v: acc.while_(lambda k: (k + 1) * (k + 1) <= v, lambda k: k + 1, acc.constant(0, "Int64")) + 1, xs)
    e = r.stream()
    assert len(e.binds) == 1 and " while (" in e.binds[0] and e.text.startswith("[&] { Int64 w")
    arrays, sig, fr = acc._assemble(get=e.text)
    assert A.compile_only(A.make_desc(A.SKEL_MAP, "Int64", env=sig, out_rank=1, **fr)) > 0
    # the same loop used twice is emitted once
    twice = acc.map(lambda v: (lambda s: s * s)(acc.while_(lambda k: k < v, lambda k: k + 2, acc.constant(0, "Int64"))), xs).stream()
    assert len(twice.binds) == 1
    # a tuple state: every component is a loop variable, components picked afterwards share the loop
    t = acc.while_(lambda s: s.comps[1] < 10, lambda s: (s.comps[0] * 2, s.comps[1] + 1), acc.lift(acc.constant(1, "Int64"), acc.constant(0, "Int64")))
    both = t.comps[0] + t.comps[1]
    assert len(both.binds) == 1
    with pytest.raises(TypeError):
        acc.while_(lambda k: k < 3, lambda k: acc.fromIntegral(k, "Int32"), acc.constant(0, "Int64"))


def test_async_wait_poll_cancel_without_a_device():
    """the thread-backed `Async` on its own: results and exceptions come out of `wait`, `poll` says None while the
    work runs, a cancelled computation raises `Cancelled`"""
    import threading
    gate = threading.Event()
    a = acc.Async(lambda: (gate.wait(), 42)[1])
    assert acc.poll(a) is None
    gate.set()
    assert acc.wait(a) == 42 and acc.poll(a) == 42

    def boom():
        raise ValueError("from the worker")
    with pytest.raises(ValueError, match="from the worker"):
        acc.wait(acc.Async(boom))

    gate2 = threading.Event()
    b = acc.Async(lambda: gate2.wait())
    stopper = threading.Thread(target=acc.cancel, args=(b,))
    stopper.start()                   # cancel waits for the thread to reach a stopping point: here, the end of its work
    gate2.set()
    stopper.join()
    with pytest.raises(acc.Cancelled):
        acc.wait(b)


def test_the_export_list_of_the_reference_module_is_there():
    for name in ("run run1 runWith run1With stream streamWith Async wait poll cancel runAsync run1Async runAsyncWith "
                 "run1AsyncWith Context create destroy unsafeFree unsafeFreeWith performGC performGCWith runN").split():
        assert callable(getattr(acc, name)), name
