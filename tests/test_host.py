"""Host-side logic of libacchip that needs no GPU: the C ABI surface, run-time
compilation for gfx950 (hiprtc works without a device), the kernel cache, the
skeleton generator's parameter ABI, launch arithmetic and error paths.
"""
import ctypes as C
import os
import re
import subprocess
import sys

import numpy as np
import pytest

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))


@pytest.fixture(scope="module")
def A():
    import acchip
    acchip.build()
    return acchip


def test_library_exports_every_declared_symbol(A):
    """every function include/acc_hip.h declares is exported by the shared library"""
    with open(os.path.join(ROOT, "include", "acc_hip.h")) as fh:
        text = fh.read()
    text = re.sub(r"/\*.*?\*/", "", text, flags=re.S)
    declared = set(re.findall(r"\b(acc_[a-z0-9_]+)\s*\(", text))
    assert len(declared) >= 50
    assert declared == set(A.SYMBOLS), declared ^ set(A.SYMBOLS)
    out = subprocess.check_output(["nm", "-D", "--defined-only", A.LIB_PATH]).decode()
    exported = set(re.findall(r" T (acc_[a-z0-9_]+)", out))
    assert declared <= exported, declared - exported
    L = A.lib()
    for name in declared:
        assert getattr(L, name) is not None
    assert L.acc_version().decode().count(".") == 2


def test_no_torch_types_and_no_oracle_in_the_product():
    """the boundary is plain C and the product never reaches into oracle/"""
    with open(os.path.join(ROOT, "include", "acc_hip.h")) as fh:
        hdr = re.sub(r"/\*.*?\*/", "", fh.read(), flags=re.S)
    assert "torch" not in hdr and "std::" not in hdr and "at::" not in hdr
    pkg = os.path.join(ROOT, "accelerate-cuda_amd")
    for dirpath, _, files in os.walk(pkg):
        for f in files:
            if f.endswith((".py", ".cpp", ".hpp", ".h")):
                with open(os.path.join(dirpath, f)) as fh:
                    assert "oracle" not in fh.read().lower(), os.path.join(dirpath, f)


def test_every_skeleton_instance_compiles_for_gfx950(A, tmp_path):
    import __graft_entry__ as g
    A.lib().acc_cache_set_dir(str(tmp_path).encode())
    inst = g.standard_instances(A)
    assert len(inst) >= 18
    for name, desc in inst.items():
        assert A.compile_only(desc, "gfx950") > 4000, name


def test_permute_variants_the_driver_chooses_between_all_compile(A, tmp_path):
    """tables under locks in LDS (+2), several LDS windows of targets (+4), 16-bit counts (+6): generated from the same
    description, each for aligned and unaligned operands"""
    A.lib().acc_cache_set_dir(str(tmp_path).encode())
    hist = A.make_desc(A.SKEL_PERMUTE, "Int32", env=[(1, "Int32")], out_rank=1, get="1", combine="x + y",
                       permutation="arrIn0_0[ix]", combine_hint=A.COMBINE_ADD)
    generic = A.make_desc(A.SKEL_PERMUTE, "float", env=[(1, "Int32"), (1, "float")], out_rank=1, get="arrIn1_0[ix]",
                          combine="acc_max(x, y)", permutation="arrIn0_0[ix]")
    for desc, variants in ((hist, (0, 1, 4, 5, 6, 7)), (generic, (0, 1, 2, 3))):
        for v in variants:
            name, src = A.preview(desc, v)
            assert name == "permute" and ("ACC_PERMUTE_NARROW 1" in src) == (v >= 6)
            assert A.compile_source(src) > 4000, v
    # and as a loop's body runs them (ACC_FLAG_GUARDED: one more parameter and a test on entry in every kernel)
    for desc, variants in ((hist, (4, 6)), (generic, (2,))):
        g = A.make_desc_copy(desc)
        g.flags |= A.FLAG_GUARDED
        for v in variants:
            name, src = A.preview(g, v)
            assert "#define ACC_GUARDED 1" in src
            assert A.compile_source(src) > 4000, v


def test_variants_by_shape_of_scans_stencils_and_maps_compile(A, tmp_path):
    """what the drivers take by the shape of a call: small tiles for scans of small arrays (+2), half and a quarter of
    the columns a lane for stencils on narrow arrays (+2, +4; two columns a lane of 8-byte elements to begin with), tiles
    for a map that reads across the rows of its source (ACC_FLAG_TILED, rank 2 or more only)"""
    A.lib().acc_cache_set_dir(str(tmp_path).encode())
    scan = A.make_desc(A.SKEL_SCANL, "Int32", env=[(1, "Int32")], get="arrIn0_0[ix]", combine="x + y", seed="0")
    rows = {}
    for v in (0, 1, 2, 3):
        name, src = A.preview(scan, v)
        assert name == "scanl" and A.compile_source(src) > 4000, v
        rows[v] = int([l for l in src.splitlines() if l.startswith("#define ACC_ROWS ")][0].split()[-1])
    assert rows[0] == rows[1] == 32 and rows[2] == rows[3] == 4
    seg = A.make_desc(A.SKEL_FOLDSEG, "float", env=[(1, "float")], out_rank=1, get="arrIn0_0[ix]", combine="x + y", seed="0.0f")
    chunks = {}
    for v in (0, 2, 3):                                            # a longer staged chunk for segments of 8 elements or more
        name, src = A.preview(seg, v)
        assert name == "foldSeg" and A.compile_source(src) > 4000, v
        chunks[v] = int([l for l in src.splitlines() if l.startswith("#define ACC_CHUNK ")][0].split()[-1])
    assert chunks[2] == chunks[3] > chunks[0]
    seven = [(0, 0, 0), (-1, 0, 0), (1, 0, 0), (0, -1, 0), (0, 1, 0), (0, 0, -1), (0, 0, 1)]
    nine = [(dy, dx) for dy in (-1, 0, 1) for dx in (-1, 0, 1)]
    for ctype, rank, taps, svecs in (("float", 2, nine, (4, 2, 1)), ("float", 3, seven, (4, 2, 1)), ("double", 3, seven, (2, 1, 1))):
        st = A.make_desc(A.SKEL_STENCIL, ctype, out_rank=rank, taps=taps, boundary="mirror",
                         stencil_fn=" + ".join("t%d" % k for k in range(len(taps))))
        for k, want in enumerate(svecs):
            for v in (2 * k, 2 * k + 1):
                name, src = A.preview(st, v)
                assert "#define ACC_SVEC %d\n" % want in src, (ctype, rank, v)
                assert A.compile_source(src) > 4000, (ctype, rank, v)
    wide = A.make_desc(A.SKEL_STENCIL, "float", out_rank=2, taps=[(0, -4), (0, 0), (0, 4)], boundary="clamp", stencil_fn="t0 + t1 + t2")
    assert "#define ACC_SVEC 4\n" in A.preview(wide, 0)[1]
    tr = "arrIn0_0[(ix % shOut_0) * shIn0_0 + (ix / shOut_0)]"
    tiled = A.make_desc(A.SKEL_MAP, "float", env=[(2, "float")], out_rank=2, get=tr, flags=A.FLAG_TILED)
    name, src = A.preview(tiled, 0)
    assert name == "map" and "#define ACC_MAP_TILED 1" in src and A.compile_source(src) > 2000
    vector = A.make_desc(A.SKEL_MAP, "float", env=[(1, "float")], out_rank=1, get="arrIn0_0[ix]", flags=A.FLAG_TILED)
    assert "#define ACC_MAP_TILED 0" in A.preview(vector, 0)[1]


def test_every_scalar_primitive_compiles_for_every_type(A, tmp_path):
    """acc_prim.h: one map per element type naming every primitive that type has
    (CodeGen.hs:406-476); what they compute is checked on the GPU"""
    A.lib().acc_cache_set_dir(str(tmp_path).encode())
    X, Y = "arrIn0_0[ix]", "arrIn1_0[ix]"
    integral = ["acc_quot(X, Y)", "acc_rem(X, Y)", "acc_idiv(X, Y)", "acc_imod(X, Y)", "acc_quot_rem(X, Y).snd",
                "acc_div_mod(X, Y).fst", "acc_abs(X)", "acc_signum(X)", "acc_pmax(X, Y)", "acc_pmin(X, Y)",
                "acc_shift_l(X, 1)", "acc_shift_r(X, 1)", "acc_shift_rl(X, 1)", "acc_rotate_l(X, (Int64)Y)",
                "acc_rotate_r(X, (Int64)Y)", "acc_from_integral<T>(acc_bool_to_int((Word8)(X > Y)))", "(T)acc_ord(acc_chr(X))"]
    floating = ["acc_recip(X)", "acc_abs(X)", "acc_signum(X)", "acc_pmax(X, Y)", "acc_pmin(X, Y)", "acc_pow(X, Y)",
                "acc_atan2(X, Y)", "acc_log_base(X, Y)", "(T)acc_is_nan(X)", "(T)acc_truncate<Int32>(X)",
                "(T)acc_round<Int64>(X)", "(T)acc_floor<Int16>(X)", "(T)acc_ceiling<Word32>(X)"] + \
               ["acc_%s(X)" % f for f in ("sin", "cos", "tan", "asin", "acos", "atan", "sinh", "cosh", "tanh", "asinh",
                                          "acosh", "atanh", "exp", "sqrt", "log")]
    for t in ("Int8", "Int16", "Int32", "Int64", "Word8", "Word16", "Word32", "Word64", "float", "double"):
        terms = floating if t in ("float", "double") else integral
        frag = " + ".join("(T)(%s)" % e for e in terms).replace("X", X).replace("Y", Y).replace("T", t)
        d = A.make_desc(A.SKEL_MAP, t, env=[(1, t), (1, t)], out_rank=1, get=frag)
        assert A.compile_only(d, "gfx950") > 4000, t


def test_kernel_cache_hit_miss_and_corruption(A, tmp_path):
    L = A.lib()
    d = str(tmp_path / "cache")
    L.acc_cache_set_dir(d.encode())
    assert L.acc_cache_dir().decode() == d
    src = b'extern "C" __global__ void k(float *p) { p[threadIdx.x] = 1.0f; }\n'
    opts = (C.c_char_p * 1)(b"-O3")
    code, size = C.c_void_p(), C.c_size_t()

    def compile_(source=src, options=opts, n=1, target=b"gfx950"):
        A.check(L.acc_compile(None, target, source, options, n, C.byref(code), C.byref(size)))
        return C.string_at(code, size.value)

    s0 = A.cache_stats()
    obj = compile_()
    assert obj[:4] == b"\x7fELF"
    s1 = A.cache_stats()
    assert s1["compiles"] == s0["compiles"] + 1
    files = [os.path.join(dp, f) for dp, _, fs in os.walk(d) for f in fs]
    assert len(files) == 1 and files[0].endswith(".co") and os.sep + "gfx950" + os.sep in files[0]
    # same text: found in memory
    assert compile_() == obj
    assert A.cache_stats()["ram_hits"] == s1["ram_hits"] + 1
    # memory table emptied: found on disk, not compiled again
    L.acc_cache_clear(0)
    assert compile_() == obj
    s2 = A.cache_stats()
    assert s2["disk_hits"] == s1["disk_hits"] + 1 and s2["compiles"] == s1["compiles"]
    # anything that decides the object changes the key: text, options, target
    compile_(source=src + b"// x\n")
    compile_(options=(C.c_char_p * 1)(b"-O2"))
    compile_(target=b"gfx942")
    s3 = A.cache_stats()
    assert s3["compiles"] == s2["compiles"] + 3
    assert len([f for dp, _, fs in os.walk(d) for f in fs]) == 4
    # a damaged entry (truncated, then bit-flipped) is detected, removed and rebuilt
    for damage in ("truncate", "flip"):
        L.acc_cache_clear(0)
        with open(files[0], "rb") as fh:
            blob = bytearray(fh.read())
        if damage == "truncate":
            blob = blob[:len(blob) // 2]
        else:
            blob[-10] ^= 0x40
        with open(files[0], "wb") as fh:
            fh.write(bytes(blob))
        before = A.cache_stats()
        assert compile_() == obj
        after = A.cache_stats()
        assert after["compiles"] == before["compiles"] + 1 and after["disk_errors"] == before["disk_errors"] + 1
        with open(files[0], "rb") as fh:
            assert fh.read(8) == b"ACCHIPCO"
    # an unusable directory degrades to memory only, it never fails a compile
    L.acc_cache_clear(0)
    L.acc_cache_set_dir(b"/proc/definitely/not/writable")
    assert compile_() == obj
    L.acc_cache_set_dir(b"")
    assert compile_(source=src + b"// y\n")[:4] == b"\x7fELF"
    # clear(also_disk) removes what this process put there
    L.acc_cache_set_dir(d.encode())
    compile_(source=src + b"// z\n")
    n_before = len([f for dp, _, fs in os.walk(d) for f in fs])
    L.acc_cache_clear(1)
    assert len([f for dp, _, fs in os.walk(d) for f in fs]) < n_before


def test_concurrent_compilation_from_many_threads(A, tmp_path):
    """the reference compiles on a pool of worker threads (Compile.hs:620-660): several
    threads asking for the same and for different kernels at once must all be served,
    and the disk entries they leave must be whole"""
    import threading
    L = A.lib()
    L.acc_cache_set_dir(str(tmp_path).encode())
    L.acc_cache_clear(0)
    before = A.cache_stats()
    descs = [A.make_desc(A.SKEL_MAP, "float", env=[(1, "float")], out_rank=1, get="arrIn0_0[ix] * %d.0f" % (k % 3))
             for k in range(12)]                        # 3 distinct kernels, each wanted by 4 threads
    sizes, errors = [0] * len(descs), []

    def work(k):
        try:
            sizes[k] = A.compile_only(descs[k], "gfx950")
        except Exception as e:                          # noqa: BLE001
            errors.append(e)
    threads = [threading.Thread(target=work, args=(k,)) for k in range(len(descs))]
    for t in threads:
        t.start()
    for t in threads:
        t.join()
    assert not errors and all(s > 4000 for s in sizes)
    assert len(set(sizes[k] for k in range(0, 12, 3))) == 1       # the same kernel gives the same object
    after = A.cache_stats()
    assert after["disk_errors"] == before["disk_errors"]
    files = [os.path.join(dp, f) for dp, _, fs in os.walk(str(tmp_path)) for f in fs]
    assert len(files) == 6 and not any(".tmp." in f for f in files)     # 3 kernels x 2 variants, no leftovers
    # every entry reads back: drop the RAM table and compile again without a single compiler run
    L.acc_cache_clear(0)
    mid = A.cache_stats()
    for d in descs[:3]:
        A.compile_only(d, "gfx950")
    end = A.cache_stats()
    assert end["compiles"] == mid["compiles"] and end["disk_hits"] == mid["disk_hits"] + 6
    assert end["disk_errors"] == mid["disk_errors"]


def test_compile_error_is_a_status_with_a_log(A):
    L = A.lib()
    L.acc_cache_set_dir(b"")
    code, size = C.c_void_p(), C.c_size_t()
    rc = L.acc_compile(None, b"gfx950", b"this is not HIP\n", None, 0, C.byref(code), C.byref(size))
    assert rc == A.ERR_COMPILE
    assert "error" in L.acc_compile_log().decode()
    assert "compilation failed" in L.acc_last_error().decode()
    # a bad scalar fragment surfaces the same way through the skeleton layer
    bad = A.make_desc(A.SKEL_MAP, "float", env=[(1, "float")], out_rank=1, get="arrIn0_0[ix] +* 2")
    with pytest.raises(A.AccError) as e:
        A.compile_only(bad)
    assert e.value.code == A.ERR_COMPILE and "error" in L.acc_compile_log().decode()
    assert L.acc_compile(None, None, b"x", None, 0, C.byref(code), C.byref(size)) == A.ERR_INVALID
    assert L.acc_compile(None, b"gfx950; rm -rf", b"x", None, 0, C.byref(code), C.byref(size)) == A.ERR_INVALID


def test_descriptions_are_validated(A):
    F32 = (1, "float")
    cases = [
        (dict(kind=A.SKEL_FOLD, elt="float", env=[F32], get="arrIn0_0[ix]", combine="x + y"), "seed"),            # fold needs a seed
        (dict(kind=A.SKEL_FOLD1, elt="float", env=[F32], get="arrIn0_0[ix]", combine="x + y", seed="0"), "no seed"),
        (dict(kind=A.SKEL_SCANL, elt="float", env=[F32], get="arrIn0_0[ix]", seed="0"), "combine"),
        (dict(kind=A.SKEL_MAP, elt="float", env=[F32], out_rank=1), "get"),
        (dict(kind=A.SKEL_MAP, elt="quaternion", env=[F32], out_rank=1, get="0"), "elt_size"),
        (dict(kind=A.SKEL_PERMUTE, elt="Int32", env=[], out_rank=0, get="1", combine="x+y", permutation="0"), "rank-0"),  # IndexSpace.hs:230
        (dict(kind=A.SKEL_PERMUTE, elt="Int16", env=[], out_rank=1, get="1", combine="x+y", permutation="0", combine_hint=A.COMBINE_ADD),
         "4- or 8-byte"),                                                                                        # no hardware atomic on 2 bytes
        (dict(kind=A.SKEL_PERMUTE, elt="float", env=[], out_rank=1, get="1", combine="x", permutation="0", combine_hint=A.COMBINE_XOR), "bitwise"),
        (dict(kind=A.SKEL_STENCIL, elt="float", out_rank=4, taps=[(0, 0)], stencil_fn="t0"), "tap_offsets"),     # rank 4: taps as rows of offsets
        (dict(kind=A.SKEL_STENCIL, elt="float", out_rank=3, taps=[(300, 0, 0)], stencil_fn="t0"), "elements away"),
        (dict(kind=A.SKEL_STENCIL2, elt="float", out_rank=2, taps=[(0, 0)], stencil_fn="t0"), "tap list"),       # second source missing
        (dict(kind=A.SKEL_STENCIL, elt="float", out_rank=2, taps=[(0, 99)], stencil_fn="t0"), "elements away"),
        (dict(kind=99, elt="float"), "unknown"),
    ]
    for kw, needle in cases:
        with pytest.raises(A.AccError) as e:
            A.compile_only(A.make_desc(**kw))
        assert e.value.code in (A.ERR_INVALID, A.ERR_UNSUPPORTED), kw
        assert needle in e.value.message, (needle, e.value.message)


def test_generated_parameter_abi_follows_the_reference(A):
    """free array variables first in Gamma order, per array the extents
    outermost first then the components highest first, then the result group
    (CodeGen/Base.hs:69-89,344-357,376-383); entry names as CodeGen builds them."""
    env = [(2, ["float", "Int32"]), (1, "double")]
    d = A.make_desc(A.SKEL_MAP, "float", env=env, out_rank=2, get="arrIn0_1[ix] + (float)arrIn1_0[0]")
    entry, src = A.preview(d)
    assert entry == "map"
    defs = dict(m.groups() for m in re.finditer(r"^#define (\w+)(?:\([^)]*\))? (.*)$", src, flags=re.M))
    assert defs["ACC_ENV_PARAMS"].strip() == (
        "const Int64 shIn0_1, const Int64 shIn0_0, const Int32 *__restrict__ arrIn0_1, "
        "const float *__restrict__ arrIn0_0, const Int64 shIn1_0, const double *__restrict__ arrIn1_0,")
    assert defs["ACC_OUT_PARAMS"].strip() == "const Int64 shOut_1, const Int64 shOut_0, ACC_OUT_ARRAY(arrOut)"
    assert defs["ACC_OUT_ARRAY"].strip() == "ACC_ELT *__restrict__ name##_0" and defs["ACC_ELT"].strip() == "float"
    # a tuple result: one pointer per component, highest component first, the element a struct with fields a<c>
    _, tsrc = A.preview(A.make_desc(A.SKEL_MAP, "float, Int32, double", env=env, out_rank=1, get="acc_elt{1.0f, 2, 3.0}"))
    tdefs = dict(m.groups() for m in re.finditer(r"^#define (\w+)(?:\([^)]*\))? (.*)$", tsrc, flags=re.M))
    assert tdefs["ACC_OUT_ARRAY"].strip() == "float *__restrict__ name##_2, Int32 *__restrict__ name##_1, double *__restrict__ name##_0"
    assert "struct acc_elt { float a2; Int32 a1; double a0; };" in tsrc and tdefs["ACC_ELT"].strip() == "acc_elt"
    assert defs["ACC_OUT_SIZE"].strip() == "(shOut_1 * shOut_0)"
    assert src.rstrip().endswith('#include "skel_map.h"') and '#include "acc_hip_device.h"' in src
    assert "__builtin_assume_aligned" in src and "__builtin_assume_aligned" not in A.preview(d, 1)[1]
    assert A.compile_only(d) > 0
    # entry names as the reference builds them: PrefixSum.hs:311, Reduction.hs:188,554, IndexSpace.hs:55,109,171, Mapping.hs:49
    I32 = (1, "Int32")
    expect = [(A.SKEL_SCANL, "0", "scanl"), (A.SKEL_SCANL1, None, "scanl1"), (A.SKEL_SCANLP, "0", "scanl"),
              (A.SKEL_SCANR, "0", "scanr"), (A.SKEL_SCANR1, None, "scanr1"), (A.SKEL_SCANRP, "0", "scanr"),
              (A.SKEL_FOLD, "0", "foldAll"), (A.SKEL_FOLD1, None, "fold1All"),
              (A.SKEL_FOLDSEG, "0", "foldSeg"), (A.SKEL_FOLD1SEG, None, "fold1Seg")]
    for kind, seed, name in expect:
        e, _ = A.preview(A.make_desc(kind, "Int32", env=[I32], get="arrIn0_0[ix]", combine="x + y", seed=seed))
        assert e == name
    assert A.preview(A.make_desc(A.SKEL_FOLD, "Int32", env=[(2, "Int32")], out_rank=1, get="arrIn0_0[ix]", combine="x+y", seed="0"))[0] == "fold"
    assert A.preview(A.make_desc(A.SKEL_GENERATE, "Int32", out_rank=1, get="0"))[0] == "generate"
    assert A.preview(A.make_desc(A.SKEL_TRANSFORM, "Int32", env=[I32], out_rank=1, get="arrIn0_0[ix]"))[0] == "transform"
    assert A.preview(A.make_desc(A.SKEL_PERMUTE, "Int32", env=[I32], out_rank=1, get="1", combine="x+y", permutation="arrIn0_0[ix]"))[0] == "permute"
    # multi-line fragments are flattened so that they fit a #define
    _, src = A.preview(A.make_desc(A.SKEL_MAP, "float", env=[(1, "float")], out_rank=1, get="({ const float a = arrIn0_0[ix];\n a * a; })"))
    assert "#define ACC_GET(ix) ({ const float a = arrIn0_0[ix];  a * a; })" in src
    # tuning knobs reach the text (and so the cache key)
    with A.tuning("scan.block=512,scan.rows=2"):
        _, src = A.preview(A.make_desc(A.SKEL_SCANL, "Int32", env=[I32], get="arrIn0_0[ix]", combine="x + y", seed="0"))
    # ... and what the environment held when the table was first wanted is what acc_tuning_set(NULL) reads again
    os.environ["ACC_HIP_TUNE"] = "scan.rows=3"
    try:
        A.check(A.lib().acc_tuning_set(None))
        assert A.lib().acc_tuning_text().decode() == "scan.rows=3"
        _, src3 = A.preview(A.make_desc(A.SKEL_SCANL, "Int32", env=[I32], get="arrIn0_0[ix]", combine="x + y", seed="0"))
        assert "#define ACC_ROWS 3" in src3
    finally:
        del os.environ["ACC_HIP_TUNE"]
        A.check(A.lib().acc_tuning_set(None))
    assert "#define ACC_BLOCK 512" in src and "#define ACC_ROWS 2" in src


def test_launch_arithmetic(A):
    """split / maxGrid of Analysis/Launch.hs:51-55,124-128"""
    g = A.lib().acc_launch_grid
    assert g(0, 256, 256, 8) == 1                 # at least one block, so that empty folds still write their seed
    assert g(1, 256, 256, 8) == 1
    assert g(256, 256, 256, 8) == 1
    assert g(257, 256, 256, 8) == 2
    assert g(1 << 26, 4096, 256, 8) == 2048       # capped at what is resident
    assert g(1 << 26, 4096, 256, 1 << 20) == 16384
    assert g(100, 0, 1, 1) == 1                   # degenerate arguments do not divide by zero


def test_without_a_gpu_the_runtime_reports_an_error_not_a_crash(A):
    import torch
    if torch.cuda.is_available():
        pytest.skip("a GPU is present")
    L = A.lib()
    n = C.c_int(-1)
    rc = L.acc_device_count(C.byref(n))
    h = C.c_void_p()
    rc2 = L.acc_context_create(0, C.byref(h))
    assert (rc != A.OK or n.value == 0) and rc2 != A.OK and not h.value
    assert len(L.acc_last_error()) > 0
    with pytest.raises(A.AccError):
        A.Context(0)


def test_workload_module_is_pure_numpy():
    import workloads as wl
    x, y = wl.dot_inputs(1000)
    assert x.dtype == np.float32 and x.shape == (1000,) and not np.array_equal(x, y)
    vals, cols, offs, lens, xv = wl.smvm_inputs(nrows=500, mean_len=8, ncols=64)
    assert offs[0] == 0 and offs[-1] == vals.size == cols.size and np.array_equal(np.diff(offs), lens)
    assert cols.min() >= 0 and cols.max() < 64 and xv.size == 64


def test_stencils_of_any_rank_and_reach_generate_and_compile(A):
    """rank 4 (taps as rows of offsets), and a tap five rows away in two dimensions: both take the template that maps an
    element a thread; a stencil within the strips' reach does not, unless the knob asks for it"""
    import itertools
    taps4 = list(itertools.product((-1, 0, 1), repeat=4))
    d4 = A.make_desc(A.SKEL_STENCIL, "float", out_rank=4, taps=taps4, boundary="mirror", stencil_fn=" + ".join("t%d" % k for k in range(81)))
    name, src = A.preview(d4, 0)
    assert name == "stencil" and '#include "skel_stencil_nd.h"' in src and "shOut_3" in src and "READ(0, -1, 0, 1, -1)" in src
    assert A.compile_only(d4) > 0
    far = A.make_desc(A.SKEL_STENCIL, "double", out_rank=2, taps=[(0, 0), (-5, 0), (0, 6)], boundary="constant", boundary_constant="1.0",
                      stencil_fn="t0 + t1 + t2")
    assert "skel_stencil_nd.h" in A.preview(far, 0)[1] and A.compile_only(far) > 0
    near = A.make_desc(A.SKEL_STENCIL, "double", out_rank=2, taps=[(0, 0), (-4, 0), (0, 4)], boundary="clamp", stencil_fn="t0 + t1 + t2")
    assert '#include "skel_stencil.h"' in A.preview(near, 0)[1]
    with A.tuning("stencil.nd=1"):
        assert "skel_stencil_nd.h" in A.preview(near, 0)[1]
    with pytest.raises(A.AccError) as e:                       # a rank-4 stencil cannot say its taps in three lists
        bad = A.make_desc(A.SKEL_STENCIL, "float", out_rank=4, taps=[(0, 0, 0)], stencil_fn="t0")
        A.preview(bad, 0)
    assert e.value.code == A.ERR_INVALID


def test_c_client_builds_as_c99_and_runs_its_deviceless_part():
    """include/acc_hip.h is a C header: a C99 program (-pedantic -Werror) includes it, links the library and drives
    generation and compilation through it"""
    import subprocess
    here = os.path.join(os.path.dirname(os.path.abspath(__file__)), "c_abi")
    subprocess.check_call(["make", "-C", here], stdout=subprocess.DEVNULL)
    out = subprocess.run([os.path.join(here, "client"), "--no-gpu"], capture_output=True, text=True, timeout=300)
    assert out.returncode == 0 and "all checks passed" in out.stdout, out.stdout + out.stderr


def test_haskell_bindings_cover_the_header():
    """the (uncompiled) Haskell FFI module imports every entry point the header declares, once, with as many
    arguments as the C declaration has; its structure accesses name fields the header has"""
    header = re.sub(r"/\*.*?\*/", "", open(os.path.join(ROOT, "include", "acc_hip.h")).read(), flags=re.S)
    hsc = open(os.path.join(ROOT, "accelerate-cuda_amd", "haskell", "Data", "Array", "Accelerate", "HIP", "FFI.hsc")).read()
    declared = {}
    for name, params in re.findall(r"^(?:const char \*|int64_t |int )\s*(acc_[a-z0-9_]+)\(([^;]*?)\);", header, flags=re.M | re.S):
        params = " ".join(params.split())
        declared[name] = 0 if params == "void" else params.count(",") + 1
    imported = {}
    for name, sig in re.findall(r'^foreign import ccall \w+\s+"(acc_\w+)"\s+\w+\s+::\s+(.*)$', hsc, flags=re.M):
        assert name not in imported, name
        depth, arrows = 0, 0
        for k, ch in enumerate(sig):                      # arrows outside parentheses separate the arguments
            depth += (ch == "(") - (ch == ")")
            arrows += depth == 0 and sig[k:k + 2] == "->"
        imported[name] = arrows
    assert imported == declared
    for struct, field in re.findall(r"#\{(?:peek|poke|ptr) (\w+), (\w+)\}", hsc):
        body = re.search(r"typedef struct %s \{(.*?)\} %s;" % (struct, struct), header, flags=re.S).group(1)
        assert re.search(r"\b%s\b" % field, body), (struct, field)
    for const in re.findall(r"#\{const (\w+)\}", hsc):
        assert re.search(r"#define %s\b|\b%s\s*=" % (const, const), header), const      # a macro, or a member of an enum


def test_haskell_modules_use_only_what_the_bindings_and_the_device_headers_have():
    """the (uncompiled) modules of the Haskell backend -- code generator, compile and execute traversals, front door --
    call only foreign imports and constants that FFI.hsc defines, and emit only device functions that the headers
    every generated unit includes define"""
    hdir = os.path.join(ROOT, "accelerate-cuda_amd", "haskell", "Data", "Array", "Accelerate")
    hsc = open(os.path.join(hdir, "HIP", "FFI.hsc")).read()
    bound = set(re.findall(r'^foreign import ccall \w+\s+"acc_\w+"\s+(c_\w+)', hsc, flags=re.M))
    constants = set(re.findall(r"^(acc[A-Z]\w+)\s+=", hsc, flags=re.M))
    device = ""
    for h in ("acc_prim.h", "acc_hip_device.h"):
        device += open(os.path.join(ROOT, "accelerate-cuda_amd", "csrc", "device", h)).read()
    defined = set(re.findall(r"\b(acc_[a-z0-9_]+)\s*\(", device)) | set(re.findall(r"#define (ACC_[A-Z_]+)", device))
    defined |= set(re.findall(r"^ACC_MATH\d\((acc_[a-z0-9_]+),", device, flags=re.M))       # defined through a macro
    modules = ["HIP.hs", "HIP/CodeGen.hs", "HIP/Compile.hs", "HIP/Execute.hs", "HIP/State.hs", "HIP/Array.hs"]
    for m in modules:
        text = open(os.path.join(hdir, m)).read()
        assert "UNCOMPILED" in text, m
        code = re.sub(r"--.*", "", text)
        for name in set(re.findall(r"\b(c_[a-zA-Z0-9]+)\b", code)):
            assert name in bound, (m, name)
        for name in set(re.findall(r"\b(acc(?:Skel|Combine|Flag|Err)[A-Za-z0-9]*)\b", code)):
            assert name in constants, (m, name)
        for name in set(re.findall(r'"(acc_[a-z0-9_]+)[<("]', code)):
            assert name in defined, (m, name)
        for name in set(re.findall(r"\b(ACC_[A-Z_]+)\b", code)) - {"ACC_FLAG_GUARDED", "ACC_ERR_INVALID", "ACC_ERR_STUCK", "ACC_COMBINE_ADD"}:
            assert name in defined, (m, name)


def test_haskell_modules_are_whole():
    """every Data.Array.Accelerate.HIP.* module that one of them imports is in the tree; no binding is left
    `undefined` (or an `error` that names what is missing); every name a module exports, and every name another
    module imports from it by name, has a definition in it; the front door exports what Data.Array.Accelerate.CUDA
    does (CUDA.hs:184-200) and the two names the task adds, runN and streamOut"""
    root = os.path.join(ROOT, "accelerate-cuda_amd", "haskell")
    paths = {}
    for d, _, files in os.walk(root):
        for f in files:
            if f.endswith((".hs", ".hsc")):
                rel = os.path.relpath(os.path.join(d, f), root)
                paths[rel.rsplit(".", 1)[0].replace(os.sep, ".")] = os.path.join(d, f)
    assert "Data.Array.Accelerate.HIP.Array" in paths

    def strip(text):
        text = re.sub(r"\{-.*?-\}", "", text, flags=re.S)
        return re.sub(r"--.*", "", text)

    def defined(code):
        names = set(re.findall(r"^([a-z_][A-Za-z0-9_']*)\s*(?:::|[^=\n]*=)", code, flags=re.M))            # bindings, signatures
        names |= set(re.findall(r"^(?:data|type|newtype|class)\s+([A-Z][A-Za-z0-9_']*)", code, flags=re.M))
        names |= set(re.findall(r'^foreign import ccall.*?"\s+(\w+)\s+::', code, flags=re.M))
        for body in re.findall(r"^data\s.*?(?=^\S)", code, flags=re.M | re.S):                        # constructors, fields
            names |= set(re.findall(r"[=|]\s*(?:forall [^.]*\.\s*)?(?:\([^)]*\)\s*=>\s*)?([A-Z][A-Za-z0-9_']*)", body))
            names |= set(re.findall(r"^\s+([A-Z][A-Za-z0-9_']*)\s*::", body, flags=re.M))              # GADT constructors
            names |= set(re.findall(r"[{,]\s*([a-z][A-Za-z0-9_']*)\s*::", body))
        return names

    codes = {m: strip(open(p).read()) for m, p in paths.items()}
    defs = {m: defined(c) for m, c in codes.items()}
    for m, code in codes.items():
        assert not re.search(r"=\s*undefined\b", code), m
        assert not re.search(r"^\w+\s*=\s*error\b", code, flags=re.M), m
        for line in re.findall(r"^import\s+(?:qualified\s+)?(Data\.Array\.Accelerate\.HIP[.\w]*)(.*)$", code, flags=re.M):
            mod, rest = line
            assert mod in paths, (m, "imports", mod)
            listed = re.search(r"\(\s*(.*)\)", rest)
            if listed and "hiding" not in rest:
                for name in re.findall(r"\b([A-Za-z_][A-Za-z0-9_']*)\b(?:\(\.\.\))?", listed.group(1)):
                    assert name in defs[mod], (m, "imports", name, "from", mod)
        head = re.search(r"^module\s+[\w.]+\s*\((.*?)\)\s*where", code, flags=re.M | re.S)
        if head:
            for name in re.findall(r"\b([A-Za-z_][A-Za-z0-9_']*)\b", re.sub(r"\(\.\.\)", "", head.group(1))):
                if name in ("module",):
                    continue
                imported = re.search(r"^import\s+.*\b%s\b" % re.escape(name), code, flags=re.M)           # re-exported
                assert name in defs[m] or imported, (m, "exports", name)
    front = re.search(r"^module\s+[\w.]+\s*\((.*?)\)\s*where", codes["Data.Array.Accelerate.HIP"], flags=re.M | re.S).group(1)
    exported = set(re.findall(r"\b([A-Za-z_][A-Za-z0-9_']*)\b", front))
    reference = """Arrays run run1 runWith run1With stream streamWith Async wait poll cancel runAsync run1Async runAsyncWith
                   run1AsyncWith Context create destroy unsafeFree unsafeFreeWith performGC performGCWith""".split()
    assert set(reference) | {"runN", "streamOut", "streamOutWith"} <= exported


def test_profile_summaries_were_measured_on_this_tree_s_kernel_sources():
    """every summary under profiles/ names the commit it was measured on and carries the SHA-256 of the kernel sources
    (csrc/device/*.h and skeleton.cpp) of that tree: a change to a kernel's source without collecting the counters
    again fails here, and bench.py marks the traffic figures it reads from them as stale"""
    import glob
    import re
    import bench
    now = bench.kernel_sources_hash()
    files = sorted(glob.glob(os.path.join(ROOT, "profiles", "*.txt")))
    assert len(files) >= 7
    for path in files:
        text = open(path).read()
        assert re.search(r"^git-head: [0-9a-f]{40}$", text, re.M), path
        assert bench.profile_hash(path) == now, "%s was measured on other kernel sources than this tree's" % os.path.basename(path)
        assert "rocprofv3" in text and "bench.py" in text, path      # the command that made it
    t = bench.profiled_traffic("scanl")
    assert t and t["stale"] is False and t["bytes"] > 2 * (1 << 26) * 4
