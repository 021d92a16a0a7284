"""The embedded language's index arithmetic, which needs no device: what it writes for an index function applied to
the result of another, how it finds out that an index function reads its source across the rows, and the text of a
fold whose rows lie across memory."""
import os
import sys

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
sys.path[:0] = [os.path.join(ROOT, "accelerate-cuda_amd")]

import accelerate_hip as acc  # noqa: E402
from accelerate_hip import All  # noqa: E402


def source(name, shape, ctype="float"):
    """a stand-in for a manifest array: reads name[linear index]"""
    return acc.Acc(shape, ctype, at=lambda ix: acc.Exp(ctype, "%s[%s]" % (name, ix.term)))


def test_an_index_that_was_just_put_together_is_not_taken_apart_again():
    i, j, k = (acc.Exp("Int64", n) for n in "ijk")
    lin = acc._linear((i, j, k), (5, 6, 7))
    assert [e.term for e in acc._unlinear(lin, (5, 6, 7))] == ["i", "j", "k"]
    # another shape of the same size is another way of counting: divisions
    parts = acc._unlinear(lin, (5, 42))
    assert "%" in parts[1].term and "/" in parts[0].term
    # a vector's index is an object of its own (the note must not land on the caller's expression)
    one = acc._linear((i,), (9,))
    assert one is not i and not hasattr(i, "made_of") and acc._unlinear(one, (9,))[0].term == "i"


def test_transposes_and_replicates_of_transposes_read_without_divisions_once_the_index_is_known():
    b = source("B", (32, 48))
    t = acc.transpose(b)
    text = t.index(acc._linear((acc.Exp("Int64", "y"), acc.Exp("Int64", "x")), t.shape)).term
    assert "%" not in text and "/" not in text and "B[" in text
    r = acc.replicate((64, All, All), t)
    idx = tuple(acc.Exp("Int64", n) for n in "ijk")
    text = r.index(acc._linear(idx, r.shape)).term
    assert "%" not in text and "/" not in text
    # k walks down B's columns: B[k * 48 + j]
    assert text.replace(" ", "").replace("((Int64)", "(").count("k") == 1


def test_index_functions_are_asked_by_applying_them_to_numbers():
    m = source("M", (64, 32))
    c = source("C", (5, 6, 7))
    assert acc.transpose(m).across and not acc.transpose(acc.transpose(m)).across
    assert acc.backpermute((5, 7, 6), lambda i, k, j: (i, j, k), c).across
    assert not acc.backpermute((6, 5, 7), lambda j, i, k: (i, j, k), c).across
    assert not acc.backpermute((64, 32), lambda y, x: (y, 31 - x), m).across          # backwards along the rows
    assert not acc.backpermute((64, 16), lambda y, x: (y, 2 * x), m).across           # every other column
    assert not acc.replicate((All, All, 9), m).across                                 # the innermost dimension is new
    assert acc.replicate((9, All, All), acc.transpose(m)).across
    assert not acc.replicate((All, 9, All), m).across
    # an index function that is more than arithmetic cannot be asked: it counts as reading along the rows
    far = acc.backpermute((64, 32), lambda y, x: (acc.cond(y > acc.constant(3, "Int64"), y, y), x), m)
    assert not far.across
    # too small to take a step, a vector: not across
    assert not acc.transpose(source("T", (1, 9))).across
    assert not acc.backpermute((9,), lambda i: (8 - i,), source("V", (9,))).across
    # a volume turned: which dimension of the result, counted from the innermost, the source is read along
    assert acc.backpermute((7, 5, 6), lambda k, i, j: (i, j, k), c).across == 2
    assert acc.backpermute((5, 7, 6), lambda i, k, j: (i, j, k), c).across == 1
    # map and zipWith pass it on
    t = acc.transpose(m)
    assert acc.map(lambda v: v + v, t).across and acc.zipWith(lambda p, q: p * q, t, source("N", (32, 64))).across


def test_a_fold_whose_rows_lie_across_memory_is_written_over_the_row_and_the_place_within_it():
    a, b = source("A", (64, 32)), source("B", (32, 48))
    z = acc.zipWith(lambda p, q: p * q, acc.replicate((All, 48, All), a), acc.replicate((64, All, All), acc.transpose(b)))
    assert z.across and z.shape == (64, 48, 32)
    acc._building.rows_of = z.shape
    try:
        text = z.stream().text
    finally:
        acc._building.rows_of = None
    assert "acc_row" in text and "acc_col" in text and "ix" not in text.replace("acc_elt", "")
    # the place within the row is used as it stands; only the row is divided (by the literal 48)
    assert text.count("acc_col") == 2 and "%" in text
    plain = z.stream().text
    assert "acc_row" not in plain and "ix" in plain


def test_an_index_into_fewer_than_2_to_the_31_elements_is_taken_apart_in_32_bits():
    ix = acc.Exp("Int64", "ix")
    small = acc._unlinear(ix, (500, 500, 500))
    assert all(p.ctype == "Int64" for p in small)
    assert "(Word32)ix" in small[2].term and "500u" in small[2].term and "LL" not in small[2].term
    # 2^31 elements and more: 64-bit arithmetic throughout
    big = acc._unlinear(ix, (70000, 70000))
    assert all("Word32" not in p.term for p in big) and "70000LL" in big[1].term
    # an array without elements has no index to take apart (and no division by zero is written)
    none = acc._unlinear(ix, (0, 5))
    assert all("Word32" not in p.term for p in none)
    # a vector's index is the linear one
    assert acc._unlinear(ix, (9,))[0].term == "ix"
