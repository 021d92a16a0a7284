"""ctypes binding of libacchip (include/acc_hip.h) for tests, the smoke check and
the bench.  It is a thin, faithful mirror of the C ABI -- the same thing a
Haskell `foreign import ccall` layer would be -- plus numpy conveniences for
moving arrays.  It computes nothing itself: every array operation goes through
the HIP skeletons in the shared library, and loading fails loudly if the
library has not been built.
"""
import ctypes as C
import os
import subprocess

import numpy as np

_HERE = os.path.dirname(os.path.abspath(__file__))
LIB_PATH = os.path.join(_HERE, "lib", "libacchip.so")
CSRC = os.path.join(_HERE, "csrc")

OK, ERR_INVALID, ERR_OOM, ERR_COMPILE, ERR_NOT_FOUND, ERR_HIP, ERR_UNSUPPORTED, ERR_IO, ERR_STUCK = range(9)
MAX_RANK, MAX_COMP = 8, 16

(SKEL_MAP, SKEL_GENERATE, SKEL_TRANSFORM, SKEL_FOLD, SKEL_FOLD1, SKEL_FOLDSEG, SKEL_FOLD1SEG,
 SKEL_SCANL, SKEL_SCANL1, SKEL_SCANLP, SKEL_SCANR, SKEL_SCANR1, SKEL_SCANRP, SKEL_PERMUTE,
 SKEL_STENCIL, SKEL_STENCIL2) = range(16)
SCAN_KINDS = {"scanl": SKEL_SCANL, "scanl1": SKEL_SCANL1, "scanl'": SKEL_SCANLP,
              "scanr": SKEL_SCANR, "scanr1": SKEL_SCANR1, "scanr'": SKEL_SCANRP}
COMBINE_GENERIC, COMBINE_ADD, COMBINE_MIN, COMBINE_MAX, COMBINE_AND, COMBINE_OR, COMBINE_XOR = range(7)
BOUNDARY = {"clamp": 0, "mirror": 1, "wrap": 2, "constant": 3}
FLAG_FOLD_RIGHT, FLAG_FAST_MATH, FLAG_GUARDED, FLAG_TILED = 1, 2, 4, 8


def FLAG_TILE_DIM(d):
    """with FLAG_TILED on a map of rank >= 3: the tiles' second dimension is the d-th above the innermost one"""
    return int(d) << 8

CTYPE = {np.dtype(np.float32): "float", np.dtype(np.float64): "double",
         np.dtype(np.int8): "Int8", np.dtype(np.int16): "Int16", np.dtype(np.int32): "Int32",
         np.dtype(np.int64): "Int64", np.dtype(np.uint8): "Word8", np.dtype(np.uint16): "Word16",
         np.dtype(np.uint32): "Word32", np.dtype(np.uint64): "Word64"}


class AccError(RuntimeError):
    def __init__(self, code, msg):
        RuntimeError.__init__(self, "libacchip status %d: %s" % (code, msg))
        self.code = code
        self.message = msg


class acc_array(C.Structure):
    _fields_ = [("rank", C.c_int32), ("ncomp", C.c_int32),
                ("shape", C.c_int64 * MAX_RANK), ("ptr", C.c_uint64 * MAX_COMP)]


class acc_env_sig(C.Structure):
    _fields_ = [("rank", C.c_int32), ("ncomp", C.c_int32), ("type", C.c_char_p * MAX_COMP)]


class acc_skel_desc(C.Structure):
    _fields_ = [("kind", C.c_int32), ("flags", C.c_uint32), ("n_env", C.c_int32),
                ("env", C.POINTER(acc_env_sig)), ("elt_type", C.c_char_p), ("elt_size", C.c_int32),
                ("out_rank", C.c_int32), ("preamble", C.c_char_p), ("get", C.c_char_p),
                ("combine", C.c_char_p), ("seed", C.c_char_p), ("permutation", C.c_char_p),
                ("combine_hint", C.c_int32), ("boundary", C.c_int32), ("boundary_constant", C.c_char_p),
                ("n_taps", C.c_int32), ("tap_dy", C.POINTER(C.c_int32)), ("tap_dx", C.POINTER(C.c_int32)),
                ("stencil_fn", C.c_char_p), ("stencil_in_type", C.c_char_p), ("seg_type", C.c_char_p),
                ("boundary2", C.c_int32), ("boundary2_constant", C.c_char_p), ("n_taps2", C.c_int32),
                ("tap2_dy", C.POINTER(C.c_int32)), ("tap2_dx", C.POINTER(C.c_int32)), ("stencil_in2_type", C.c_char_p),
                ("tap_dz", C.POINTER(C.c_int32)), ("tap2_dz", C.POINTER(C.c_int32)),
                ("tap_offsets", C.POINTER(C.c_int32)), ("tap2_offsets", C.POINTER(C.c_int32))]


class acc_device_props(C.Structure):
    _fields_ = [("name", C.c_char * 256), ("arch", C.c_char * 64), ("compute_units", C.c_int32),
                ("wavefront_size", C.c_int32), ("max_threads_per_block", C.c_int32), ("clock_khz", C.c_int32),
                ("lds_per_block", C.c_int64), ("lds_per_cu", C.c_int64), ("l2_bytes", C.c_int64),
                ("total_mem", C.c_int64), ("regs_per_block", C.c_int32), ("max_threads_per_cu", C.c_int32)]


class acc_cache_stats(C.Structure):
    _fields_ = [("ram_hits", C.c_uint64), ("disk_hits", C.c_uint64), ("compiles", C.c_uint64),
                ("disk_errors", C.c_uint64)]


class acc_skel_info(C.Structure):
    _fields_ = [("entry", C.c_char * 64), ("block", C.c_int32), ("blocks_per_cu", C.c_int32),
                ("num_regs", C.c_int32), ("static_lds", C.c_int32), ("elements_per_block", C.c_int32)]


# every symbol include/acc_hip.h declares (tests check that all are exported)
class acc_memtable_stats(C.Structure):
    _fields_ = [(n, C.c_uint64) for n in ("resident_bytes", "nursery_bytes", "arrays", "resident_arrays", "device_allocs",
                                          "nursery_hits", "uploads", "upload_bytes", "evictions", "writebacks",
                                          "writeback_bytes")]


SYMBOLS = """acc_last_error acc_version acc_init acc_device_count acc_device_get_props acc_context_create
acc_context_destroy acc_context_device acc_context_sync acc_context_trim acc_context_scratch_bytes
acc_context_debug_poke_lock acc_malloc acc_free acc_mem_info acc_host_alloc
acc_host_free acc_memcpy_h2d acc_memcpy_d2h acc_memcpy_d2d acc_memcpy_h2d_async acc_memcpy_d2h_async
acc_memcpy_d2d_async acc_memset32_async acc_stream_create acc_stream_destroy acc_stream_sync
acc_stream_wait_event acc_event_create acc_event_destroy acc_event_record acc_event_sync acc_event_query
acc_event_elapsed_ms acc_compile acc_compile_log acc_cache_set_dir acc_cache_dir acc_cache_get_stats
acc_cache_clear acc_module_load acc_module_unload acc_module_get_function acc_function_attr acc_occupancy
acc_launch acc_launch_grid acc_skel_create acc_skel_destroy acc_skel_source acc_skel_preview acc_skel_compile_only
acc_skel_get_info acc_exec_map acc_exec_fold acc_exec_foldseg acc_exec_foldseg_nd acc_exec_scan acc_exec_scan_noalloc acc_exec_permute
acc_exec_stencil acc_exec_stencil2 acc_exec_stencil_iterate acc_guard_create acc_guard_destroy acc_guard_reset
acc_guard_latch acc_guard_read acc_stream_set_guard acc_trace_start acc_trace_stop acc_memtable_create acc_memtable_destroy
acc_memtable_malloc acc_memtable_acquire acc_memtable_release acc_memtable_free acc_memtable_insert_unmanaged
acc_memtable_reclaim acc_memtable_get_stats acc_skel_create_async acc_skel_wait acc_skel_poll acc_skel_prefetch acc_compile_threads acc_compile_drain
acc_tuning_set acc_tuning_text acc_context_set_tuning""".split()


def build(force=False):
    """Compile libacchip.so in-tree with the committed Makefile."""
    if force or not os.path.exists(LIB_PATH):
        subprocess.check_call(["make", "-C", CSRC, "-j8"] + (["-B"] if force else []), stdout=subprocess.DEVNULL)
    return LIB_PATH


_lib = None


def lib():
    """The loaded library.  Raises if it has not been built: there is no fallback."""
    global _lib
    if _lib is None:
        if not os.path.exists(LIB_PATH):
            raise ImportError("libacchip.so is not built (%s); run `python -c 'import __graft_entry__ as g; g.build()'`"
                              % LIB_PATH)
        L = C.CDLL(LIB_PATH)
        for name in ("acc_last_error", "acc_version", "acc_compile_log", "acc_cache_dir", "acc_tuning_text"):
            getattr(L, name).restype = C.c_char_p
        L.acc_launch_grid.restype = C.c_int64
        L.acc_launch_grid.argtypes = [C.c_int64] * 4
        L.acc_malloc.argtypes = [C.c_void_p, C.c_size_t, C.POINTER(C.c_uint64)]
        L.acc_free.argtypes = [C.c_void_p, C.c_uint64]
        L.acc_host_alloc.argtypes = [C.c_void_p, C.c_size_t, C.POINTER(C.c_void_p)]
        L.acc_host_free.argtypes = [C.c_void_p, C.c_void_p]
        L.acc_memcpy_h2d.argtypes = [C.c_void_p, C.c_uint64, C.c_void_p, C.c_size_t]
        L.acc_memcpy_d2h.argtypes = [C.c_void_p, C.c_void_p, C.c_uint64, C.c_size_t]
        L.acc_memcpy_d2d.argtypes = [C.c_void_p, C.c_uint64, C.c_uint64, C.c_size_t]
        L.acc_memcpy_d2d_async.argtypes = [C.c_void_p, C.c_uint64, C.c_uint64, C.c_size_t, C.c_void_p]
        L.acc_memset32_async.argtypes = [C.c_void_p, C.c_uint64, C.c_uint32, C.c_size_t, C.c_void_p]
        L.acc_context_create.argtypes = [C.c_int, C.POINTER(C.c_void_p)]
        L.acc_context_destroy.argtypes = [C.c_void_p]
        L.acc_context_sync.argtypes = [C.c_void_p]
        L.acc_context_trim.argtypes = [C.c_void_p, C.POINTER(C.c_size_t)]
        L.acc_context_scratch_bytes.argtypes = [C.c_void_p, C.POINTER(C.c_size_t)]
        L.acc_context_debug_poke_lock.argtypes = [C.c_void_p, C.c_size_t, C.c_uint32]
        L.acc_stream_create.argtypes = [C.c_void_p, C.POINTER(C.c_void_p)]
        L.acc_stream_destroy.argtypes = [C.c_void_p, C.c_void_p]
        L.acc_stream_sync.argtypes = [C.c_void_p, C.c_void_p]
        L.acc_event_create.argtypes = [C.c_void_p, C.c_int, C.POINTER(C.c_void_p)]
        L.acc_event_destroy.argtypes = [C.c_void_p, C.c_void_p]
        L.acc_event_record.argtypes = [C.c_void_p, C.c_void_p, C.c_void_p]
        L.acc_event_sync.argtypes = [C.c_void_p, C.c_void_p]
        L.acc_stream_wait_event.argtypes = [C.c_void_p, C.c_void_p, C.c_void_p]
        L.acc_event_elapsed_ms.argtypes = [C.c_void_p, C.c_void_p, C.c_void_p, C.POINTER(C.c_float)]
        L.acc_compile.argtypes = [C.c_void_p, C.c_char_p, C.c_char_p, C.POINTER(C.c_char_p), C.c_int,
                                  C.POINTER(C.c_void_p), C.POINTER(C.c_size_t)]
        L.acc_cache_set_dir.argtypes = [C.c_char_p]
        L.acc_skel_create.argtypes = [C.c_void_p, C.POINTER(acc_skel_desc), C.POINTER(C.c_void_p)]
        L.acc_skel_destroy.argtypes = [C.c_void_p]
        L.acc_skel_create_async.argtypes = [C.c_void_p, C.POINTER(acc_skel_desc), C.POINTER(C.c_void_p)]
        L.acc_skel_wait.argtypes = [C.c_void_p]
        L.acc_skel_prefetch.argtypes = [C.c_void_p, C.c_int]
        L.acc_skel_poll.argtypes = [C.c_void_p, C.POINTER(C.c_int)]
        L.acc_tuning_set.argtypes = [C.c_char_p]
        L.acc_context_set_tuning.argtypes = [C.c_void_p, C.c_char_p]
        L.acc_skel_source.argtypes = [C.c_void_p, C.c_int, C.POINTER(C.c_char_p)]
        L.acc_skel_preview.argtypes = [C.POINTER(acc_skel_desc), C.c_int, C.POINTER(C.c_char_p), C.POINTER(C.c_char_p)]
        L.acc_skel_compile_only.argtypes = [C.c_char_p, C.POINTER(acc_skel_desc), C.POINTER(C.c_size_t)]
        L.acc_skel_get_info.argtypes = [C.c_void_p, C.POINTER(acc_skel_info)]
        AP = C.POINTER(acc_array)
        L.acc_exec_map.argtypes = [C.c_void_p, AP, AP, C.c_void_p]
        L.acc_exec_fold.argtypes = [C.c_void_p, AP, C.c_int32, C.POINTER(C.c_int64), AP, C.c_void_p]
        L.acc_exec_foldseg.argtypes = [C.c_void_p, AP, C.c_int64, AP, AP, C.c_void_p]
        L.acc_exec_foldseg_nd.argtypes = [C.c_void_p, AP, C.c_int32, C.POINTER(C.c_int64), AP, AP, C.c_void_p]
        L.acc_exec_scan.argtypes = [C.c_void_p, AP, C.c_int64, AP, AP, C.c_void_p]
        L.acc_exec_scan_noalloc.argtypes = [C.c_void_p, AP, C.c_int64, AP, AP, C.c_void_p]
        L.acc_exec_permute.argtypes = [C.c_void_p, AP, C.c_int64, AP, AP, C.c_void_p]
        L.acc_exec_stencil.argtypes = [C.c_void_p, AP, AP, AP, C.c_void_p]
        L.acc_exec_stencil2.argtypes = [C.c_void_p, AP, AP, AP, AP, C.c_void_p]
        L.acc_exec_stencil_iterate.argtypes = [C.c_void_p, AP, AP, AP, C.c_int32, C.c_void_p, C.POINTER(C.c_int32)]
        L.acc_guard_create.argtypes = [C.c_void_p, C.POINTER(C.c_void_p)]
        L.acc_guard_destroy.argtypes = [C.c_void_p]
        L.acc_guard_reset.argtypes = [C.c_void_p, C.c_void_p]
        L.acc_guard_latch.argtypes = [C.c_void_p, AP, C.c_void_p]
        L.acc_guard_read.argtypes = [C.c_void_p, C.c_void_p, C.POINTER(C.c_int32), C.POINTER(C.c_int64)]
        L.acc_stream_set_guard.argtypes = [C.c_void_p, C.c_void_p, C.c_void_p]
        L.acc_trace_start.argtypes = [C.c_void_p]
        L.acc_trace_stop.argtypes = [C.c_void_p, C.POINTER(C.c_int32), C.POINTER(C.c_double)]
        L.acc_memtable_create.argtypes = [C.c_void_p, C.c_uint64, C.POINTER(C.c_void_p)]
        L.acc_memtable_destroy.argtypes = [C.c_void_p]
        L.acc_memtable_malloc.argtypes = [C.c_void_p, C.c_uint64, C.c_void_p, C.c_uint64, C.c_int, C.POINTER(C.c_int)]
        L.acc_memtable_acquire.argtypes = [C.c_void_p, C.c_uint64, C.c_void_p, C.POINTER(C.c_uint64)]
        L.acc_memtable_release.argtypes = [C.c_void_p, C.c_uint64, C.c_void_p]
        L.acc_memtable_free.argtypes = [C.c_void_p, C.c_uint64]
        L.acc_memtable_insert_unmanaged.argtypes = [C.c_void_p, C.c_uint64, C.c_uint64, C.c_uint64]
        L.acc_memtable_reclaim.argtypes = [C.c_void_p]
        L.acc_memtable_get_stats.argtypes = [C.c_void_p, C.POINTER(acc_memtable_stats)]
        import atexit
        atexit.register(L.acc_compile_drain)     # no worker inside the compiler when exit() tears its static data down
        _lib = L
    return _lib


def check(rc):
    if rc != OK:
        raise AccError(rc, lib().acc_last_error().decode(errors="replace"))


def _b(s):
    return None if s is None else s.encode()


def make_desc(kind, elt, env=(), out_rank=0, get=None, combine=None, seed=None, permutation=None,
              combine_hint=COMBINE_GENERIC, flags=0, preamble=None, boundary="clamp", boundary_constant=None,
              taps=None, stencil_fn=None, stencil_in=None, seg_type=None, elt_size=0,
              taps2=None, boundary2="clamp", boundary2_constant=None, stencil_in2=None):
    """env: sequence of (rank, [ctype, ...]) or (rank, ctype).
    taps: [(dy, dx), ...] (1-D: [(0, dx)]; 3-D: [(dz, dy, dx), ...])."""
    keep = []
    sigs = (acc_env_sig * max(1, len(env)))()
    for k, (rank, types) in enumerate(env):
        if isinstance(types, str):
            types = [types]
        sigs[k].rank = rank
        sigs[k].ncomp = len(types)
        for c, t in enumerate(types):
            sigs[k].type[c] = t.encode()
    d = acc_skel_desc()
    d.kind, d.flags, d.n_env = kind, flags, len(env)
    d.env = C.cast(sigs, C.POINTER(acc_env_sig))
    d.elt_type, d.elt_size, d.out_rank = _b(elt), elt_size, out_rank
    d.preamble, d.get, d.combine, d.seed = _b(preamble), _b(get), _b(combine), _b(seed)
    d.permutation, d.combine_hint = _b(permutation), combine_hint
    d.boundary = BOUNDARY[boundary] if isinstance(boundary, str) else boundary
    d.boundary_constant = _b(boundary_constant)
    if taps is not None and len(taps[0]) > 3:          # any rank: rows of offsets, outermost dimension first
        flat = (C.c_int32 * (len(taps) * len(taps[0])))(*[o for t in taps for o in t])
        keep.append(flat)
        d.n_taps, d.tap_offsets = len(taps), flat
    elif taps is not None:
        dy = (C.c_int32 * len(taps))(*[t[-2] for t in taps])
        dx = (C.c_int32 * len(taps))(*[t[-1] for t in taps])
        keep += [dy, dx]
        d.n_taps, d.tap_dy, d.tap_dx = len(taps), dy, dx
        if len(taps[0]) == 3:
            dz = (C.c_int32 * len(taps))(*[t[0] for t in taps])
            keep.append(dz)
            d.tap_dz = dz
    d.stencil_fn, d.stencil_in_type, d.seg_type = _b(stencil_fn), _b(stencil_in), _b(seg_type)
    if taps2 is not None and len(taps2[0]) > 3:
        flat2 = (C.c_int32 * (len(taps2) * len(taps2[0])))(*[o for t in taps2 for o in t])
        keep.append(flat2)
        d.n_taps2, d.tap2_offsets = len(taps2), flat2
    elif taps2 is not None:       # stencil2: the second source
        dy2 = (C.c_int32 * len(taps2))(*[t[-2] for t in taps2])
        dx2 = (C.c_int32 * len(taps2))(*[t[-1] for t in taps2])
        keep += [dy2, dx2]
        d.n_taps2, d.tap2_dy, d.tap2_dx = len(taps2), dy2, dx2
        if len(taps2[0]) == 3:
            dz2 = (C.c_int32 * len(taps2))(*[t[0] for t in taps2])
            keep.append(dz2)
            d.tap2_dz = dz2
    d.boundary2 = BOUNDARY[boundary2] if isinstance(boundary2, str) else boundary2
    d.boundary2_constant, d.stencil_in2_type = _b(boundary2_constant), _b(stencil_in2)
    d._keep = (sigs, keep)
    return d


def make_desc_copy(d):
    """a description with the same fields (and the same storage behind its pointers), to vary a flag or a hint"""
    c = acc_skel_desc()
    C.memmove(C.byref(c), C.byref(d), C.sizeof(acc_skel_desc))
    c._keep = d._keep
    return c


def preview(desc, variant=0):
    """(entry name, generated translation unit) of a description; needs no GPU."""
    src, entry = C.c_char_p(), C.c_char_p()
    check(lib().acc_skel_preview(C.byref(desc), variant, C.byref(src), C.byref(entry)))
    return entry.value.decode(), src.value.decode()


def compile_only(desc, target="gfx950"):
    """hiprtc-compile both variants of a skeleton instance; needs no GPU."""
    size = C.c_size_t(0)
    check(lib().acc_skel_compile_only(target.encode(), C.byref(desc), C.byref(size)))
    return size.value


def compile_source(source, target="gfx950", options=("-O3", "-std=c++17", "-ffp-contract=off", "-Xclang", "-target-feature",
                                                      "-Xclang", "-packed-fp32-ops")):
    """hiprtc-compile one translation unit through the kernel cache; needs no GPU.  Returns the code size."""
    opts = (C.c_char_p * len(options))(*[o.encode() for o in options])
    code, size = C.c_void_p(), C.c_size_t(0)
    check(lib().acc_compile(None, target.encode(), source.encode(), opts, len(options), C.byref(code), C.byref(size)))
    return size.value


class tuning(object):
    """with tuning("scan.rows=2", ctx): ... -- the knobs as the process's table (what acc_skel_preview and
    acc_skel_compile_only read) and, if a context is given, as that context's, for the instances created inside the
    block; put back afterwards.  Nothing touches the environment."""

    def __init__(self, text, ctx=None):
        self.text, self.ctx = text, ctx

    def __enter__(self):
        self.old = lib().acc_tuning_text().decode()
        check(lib().acc_tuning_set(_b(self.text or "")))
        if self.ctx is not None:
            self.ctx.set_tuning(self.text or "")
        return self

    def __exit__(self, *exc):
        check(lib().acc_tuning_set(_b(self.old)))
        if self.ctx is not None:
            self.ctx.set_tuning(self.old)
        return False


def cache_stats():
    st = acc_cache_stats()
    check(lib().acc_cache_get_stats(C.byref(st)))
    return {"ram_hits": st.ram_hits, "disk_hits": st.disk_hits, "compiles": st.compiles, "disk_errors": st.disk_errors}


class DeviceArray(object):
    """A device-resident array: owner of one acc_malloc'd buffer."""

    def __init__(self, ctx, shape, dtype, ptr=None, owner=True):
        self.ctx, self.shape, self.dtype = ctx, tuple(int(s) for s in shape), np.dtype(dtype)
        self.size = int(np.prod(self.shape, dtype=np.int64)) if self.shape else 1
        self.nbytes = self.size * self.dtype.itemsize
        self.owner = owner
        if ptr is None:
            p = C.c_uint64(0)
            check(lib().acc_malloc(ctx.handle, self.nbytes, C.byref(p)))
            ptr = p.value
        self.ptr = ptr

    def desc(self, shape=None, offset_elems=0):
        a = acc_array()
        shape = self.shape if shape is None else tuple(shape)
        a.rank, a.ncomp = len(shape), 1
        for i, s in enumerate(shape):
            a.shape[i] = s
        a.ptr[0] = self.ptr + offset_elems * self.dtype.itemsize
        return a

    def get(self, out=None):
        """the array on the host; `out`: a C-contiguous array of the same shape and type to fill instead of a new one"""
        if out is None:
            out = np.empty(self.shape, dtype=self.dtype)
        assert out.flags.c_contiguous and out.dtype == self.dtype and out.size == self.size
        if self.nbytes:
            check(lib().acc_memcpy_d2h(self.ctx.handle, out.ctypes.data_as(C.c_void_p), self.ptr, self.nbytes))
        return out

    def set(self, host):
        host = np.ascontiguousarray(host, dtype=self.dtype)
        assert host.size == self.size
        if self.nbytes:
            check(lib().acc_memcpy_h2d(self.ctx.handle, self.ptr, host.ctypes.data_as(C.c_void_p), self.nbytes))
        return self

    def free(self):
        if self.owner and self.ptr:
            lib().acc_free(self.ctx.handle, self.ptr)
            self.ptr = 0

    def __del__(self):
        try:
            self.free()
        except Exception:
            pass


class TupleArray(object):
    """An array of tuples as the array language lays it out: one device array per
    component (structure of arrays).  `comps` lists the components as the tuple
    reads, left to right; the kernel ABI numbers them from the right, so the
    descriptor's ptr[c] is comps[n - 1 - c]."""

    def __init__(self, comps):
        comps = list(comps)
        assert comps and all(c.shape == comps[0].shape for c in comps)
        self.comps, self.shape, self.size = comps, comps[0].shape, comps[0].size

    def desc(self, shape=None, offset_elems=0):
        a = self.comps[0].desc(shape, offset_elems)
        n = len(self.comps)
        a.ncomp = n
        for c in range(n):
            comp = self.comps[n - 1 - c]
            a.ptr[c] = comp.ptr + offset_elems * comp.dtype.itemsize
        return a

    def ctypes_of(self):
        """component C types by component index (component 0 = the LAST element), for an env signature"""
        return [CTYPE_OF[c.dtype.type] for c in reversed(self.comps)]

    def get(self):
        return tuple(c.get() for c in self.comps)


CTYPE_OF = {np.float32: "float", np.float64: "double", np.int8: "Int8", np.int16: "Int16", np.int32: "Int32",
            np.int64: "Int64", np.uint8: "Word8", np.uint16: "Word16", np.uint32: "Word32", np.uint64: "Word64"}


class Context(object):
    def __init__(self, device=0):
        h = C.c_void_p()
        check(lib().acc_init())
        check(lib().acc_context_create(device, C.byref(h)))
        self.handle = h
        self.device = device

    def props(self):
        p = acc_device_props()
        check(lib().acc_device_get_props(self.device, C.byref(p)))
        return p

    def sync(self):
        check(lib().acc_context_sync(self.handle))

    def trace_start(self):
        check(lib().acc_trace_start(self.handle))

    def trace_stop(self):
        """(launches, milliseconds on the device) of what this thread launched since trace_start"""
        n, ms = C.c_int32(), C.c_double()
        check(lib().acc_trace_stop(self.handle, C.byref(n), C.byref(ms)))
        return n.value, ms.value

    def trim(self):
        """Free the scratch blocks that are not in use; returns the bytes given back."""
        freed = C.c_size_t()
        check(lib().acc_context_trim(self.handle, C.byref(freed)))
        return freed.value

    def scratch_bytes(self):
        held = C.c_size_t()
        check(lib().acc_context_scratch_bytes(self.handle, C.byref(held)))
        return held.value

    def empty(self, shape, dtype):
        if isinstance(shape, int):
            shape = (shape,)
        return DeviceArray(self, shape, dtype)

    def array(self, host):
        host = np.ascontiguousarray(host)
        return DeviceArray(self, host.shape, host.dtype).set(host)

    def tuple_array(self, *hosts):
        """an array of tuples from its component arrays, listed left to right"""
        return TupleArray([self.array(h) for h in hosts])

    def empty_tuple(self, shape, dtypes):
        return TupleArray([self.empty(shape, dt) for dt in dtypes])

    def stream(self):
        s = C.c_void_p()
        check(lib().acc_stream_create(self.handle, C.byref(s)))
        return s

    def event(self, timing=True):
        e = C.c_void_p()
        check(lib().acc_event_create(self.handle, 1 if timing else 0, C.byref(e)))
        return e

    def record(self, ev, stream=None):
        check(lib().acc_event_record(self.handle, ev, stream))

    def elapsed_ms(self, a, b):
        check(lib().acc_event_sync(self.handle, b))
        ms = C.c_float(0)
        check(lib().acc_event_elapsed_ms(self.handle, a, b, C.byref(ms)))
        return ms.value

    def skeleton(self, *args, **kw):
        """an instance whose compilation runs in the background: whatever first uses it waits for it (wait=True: now)"""
        wait = kw.pop("wait", False)
        return Skeleton(self, make_desc(*args, **kw), wait=wait)

    def set_tuning(self, text):
        """the knobs ("name=value,...") that instances created in this context from now on take; None: the process's"""
        check(lib().acc_context_set_tuning(self.handle, _b(text)))

    def close(self):
        if self.handle:
            lib().acc_context_destroy(self.handle)
            self.handle = None


class Guard(object):
    """acc_guard: the `alive` and `count` words of an array-level loop whose iterations are enqueued ahead"""

    def __init__(self, ctx):
        self.ctx = ctx
        h = C.c_void_p()
        check(lib().acc_guard_create(ctx.handle, C.byref(h)))
        self.handle = h

    def reset(self, stream=None):
        check(lib().acc_guard_reset(self.handle, stream))

    def latch(self, pred, stream=None):
        """`pred`: a rank-0 device array of one byte"""
        check(lib().acc_guard_latch(self.handle, C.byref(pred.desc()), stream))

    def read(self, stream=None):
        alive, count = C.c_int32(), C.c_int64()
        check(lib().acc_guard_read(self.handle, stream, C.byref(alive), C.byref(count)))
        return bool(alive.value), count.value

    def attach(self, stream):
        check(lib().acc_stream_set_guard(self.ctx.handle, stream, self.handle))

    def detach(self, stream):
        check(lib().acc_stream_set_guard(self.ctx.handle, stream, None))

    def destroy(self):
        if self.handle:
            lib().acc_guard_destroy(self.handle)
            self.handle = None


class MemTable(object):
    """acc_memtable: host numpy arrays (identified by the address of their storage) and their device copies."""

    def __init__(self, ctx, budget_bytes=0):
        self.ctx, self.hosts = ctx, {}
        h = C.c_void_p()
        check(lib().acc_memtable_create(ctx.handle, budget_bytes, C.byref(h)))
        self.handle = h

    @staticmethod
    def key(host):
        """address and length of the storage (a slice that starts where its parent starts is another array)"""
        return (host.ctypes.data ^ (host.nbytes * 0x9E3779B97F4A7C15)) & 0xFFFFFFFFFFFFFFFF

    def malloc(self, host, frozen):
        """enter a C-contiguous host array; returns True if it was not in the table yet"""
        assert host.flags.c_contiguous
        new = C.c_int()
        check(lib().acc_memtable_malloc(self.handle, self.key(host), host.ctypes.data, host.nbytes, int(frozen), C.byref(new)))
        self.hosts[self.key(host)] = host           # the table reads and writes this storage later
        return bool(new.value)

    def acquire(self, host, stream=None):
        p = C.c_uint64()
        check(lib().acc_memtable_acquire(self.handle, self.key(host), stream, C.byref(p)))
        return DeviceArray(self.ctx, host.shape, host.dtype, ptr=p.value, owner=False)

    def release(self, host, stream=None):
        check(lib().acc_memtable_release(self.handle, self.key(host), stream))

    def free(self, host):
        check(lib().acc_memtable_free(self.handle, self.key(host)))
        self.hosts.pop(self.key(host), None)

    def insert_unmanaged(self, host, dev):
        check(lib().acc_memtable_insert_unmanaged(self.handle, self.key(host), dev.ptr, host.nbytes))

    def reclaim(self):
        check(lib().acc_memtable_reclaim(self.handle))

    def stats(self):
        st = acc_memtable_stats()
        check(lib().acc_memtable_get_stats(self.handle, C.byref(st)))
        return {n: getattr(st, n) for n, _ in acc_memtable_stats._fields_}

    def destroy(self):
        if self.handle:
            check(lib().acc_memtable_destroy(self.handle))
            self.handle = None


def _env(arrays):
    if not arrays:
        return None
    env = (acc_array * len(arrays))()
    for k, a in enumerate(arrays):
        env[k] = a if isinstance(a, acc_array) else a.desc()
    return env


class Skeleton(object):
    """One compiled skeleton instance (acc_skel)."""

    def __init__(self, ctx, desc, wait=True):
        self.ctx, self.desc = ctx, desc
        h = C.c_void_p()
        check((lib().acc_skel_create if wait else lib().acc_skel_create_async)(ctx.handle, C.byref(desc), C.byref(h)))
        self.handle = h

    def wait(self):
        """block until the instance is compiled and loaded; raises what the compiler had to say"""
        check(lib().acc_skel_wait(self.handle))
        return self

    def prefetch(self, variants):
        """start compiling these variants in the background (the first launch that needs one would otherwise wait)"""
        for v in variants:
            check(lib().acc_skel_prefetch(self.handle, v))
        return self

    def ready(self):
        r = C.c_int(0)
        check(lib().acc_skel_poll(self.handle, C.byref(r)))
        return bool(r.value)

    def info(self):
        i = acc_skel_info()
        check(lib().acc_skel_get_info(self.handle, C.byref(i)))
        return i

    def source(self, variant=0):
        s = C.c_char_p()
        check(lib().acc_skel_source(self.handle, variant, C.byref(s)))
        return s.value.decode()

    def map(self, env, out, stream=None):
        check(lib().acc_exec_map(self.handle, _env(env), C.byref(out if isinstance(out, acc_array) else out.desc()), stream))

    def fold(self, env, in_shape, out, stream=None):
        if isinstance(in_shape, int):
            in_shape = (in_shape,)
        sh = (C.c_int64 * len(in_shape))(*in_shape)
        check(lib().acc_exec_fold(self.handle, _env(env), len(in_shape), sh,
                                  C.byref(out if isinstance(out, acc_array) else out.desc()), stream))

    def foldseg(self, env, n, offsets, out, stream=None):
        check(lib().acc_exec_foldseg(self.handle, _env(env), n, C.byref(offsets.desc()), C.byref(out.desc()), stream))

    def foldseg_nd(self, env, in_shape, offsets, out, stream=None):
        sh = (C.c_int64 * len(in_shape))(*in_shape)
        check(lib().acc_exec_foldseg_nd(self.handle, _env(env), len(in_shape), sh, C.byref(offsets.desc()), C.byref(out.desc()), stream))

    def scan(self, env, n, out, total=None, stream=None, noalloc=False):
        o = out if isinstance(out, acc_array) else out.desc()
        t = None if total is None else C.byref(total if isinstance(total, acc_array) else total.desc(shape=()))
        fn = lib().acc_exec_scan_noalloc if noalloc else lib().acc_exec_scan
        check(fn(self.handle, _env(env), n, C.byref(o), t, stream))

    def permute(self, env, n_src, defaults, out, stream=None):
        check(lib().acc_exec_permute(self.handle, _env(env), n_src, C.byref(defaults.desc()), C.byref(out.desc()), stream))

    def stencil(self, env, src, out, stream=None):
        check(lib().acc_exec_stencil(self.handle, _env(env), C.byref(src.desc()), C.byref(out.desc()), stream))

    def stencil2(self, env, src1, src2, out, stream=None):
        check(lib().acc_exec_stencil2(self.handle, _env(env), C.byref(src1.desc()), C.byref(src2.desc()),
                                      C.byref(out.desc()), stream))

    def stencil_iterate(self, env, a, b, iters, stream=None):
        r = C.c_int32(0)
        check(lib().acc_exec_stencil_iterate(self.handle, _env(env), C.byref(a.desc()), C.byref(b.desc()), iters, stream, C.byref(r)))
        return b if r.value else a

    def destroy(self):
        if self.handle:
            lib().acc_skel_destroy(self.handle)
            self.handle = None


# ---------------------------------------------------------------------------
# fragments for the benchmark configurations, as the Accelerate code generator
# would emit them after fusion (CodeGen.hs:714-747 names the array reads)

def linear_stencil_fn(coeffs, divisor=None, ctype="float"):
    """((c0*t0 + c1*t1) + ...) [/ divisor] with float literals, left to right."""
    def lit(v):
        s = repr(float(v))
        return ("(%sf)" % s) if ctype == "float" else "(%s)" % s
    e = "%s * t0" % lit(coeffs[0])
    for k, c in enumerate(coeffs[1:], 1):
        e = "(%s + %s * t%d)" % (e, lit(c), k)
    if divisor is not None:
        e = "(%s / %s)" % (e, lit(divisor))
    return e
