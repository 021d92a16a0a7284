"""An embedded array language over libacchip, shaped like the surface a user of
the reference programs against (Data.Array.Accelerate + Data.Array.Accelerate.CUDA:
`use`, `map`, `zipWith`, `generate`, `backpermute`, `fold`, `foldSeg`, the scans,
`permute`, `stencil`, and the whole export list of CUDA.hs:184-200: `run`, `run1`,
`runWith`, `run1With`, `stream`, `streamWith`, `Async`, `wait`, `poll`, `cancel`,
`runAsync`, `run1Async`, `runAsyncWith`, `run1AsyncWith`, `Context`, `create`,
`destroy`, `unsafeFree`, `unsafeFreeWith`, `performGC`, `performGCWith`; also `runN`).

    import accelerate_hip as acc
    def dotp(xs, ys):
        return acc.fold(lambda a, b: a + b, 0.0, acc.zipWith(lambda a, b: a * b, xs, ys))
    print(acc.run(dotp(acc.use(x), acc.use(y))))

What it does is what the reference's front end and code generator do for the
skeleton hot path, in miniature:
  * scalar functions are Python callables over `Exp` values; applying them builds
    HIP C++ expression text (the role of CodeGen.hs:338-821), with the primitive
    table of acc_prim.h behind the operators that are not plain C operators;
  * `map`, `zipWith`, `generate`, `backpermute` are DELAYED: they are index -> value
    functions that fuse into whatever consumes them, so `fold (+) 0 (zipWith (*) xs ys)`
    is one kernel reading two arrays (what the fusion of `convertAccWith` hands the
    reference's back end as `CUDelayed`, CodeGen/Base.hs:115-138);
  * consumers (`fold`, `foldSeg`, scans, `permute`, `stencil`, and forcing a delayed
    array) each become one skeleton instance, created once per distinct generated
    text and cached; free arrays are numbered in order of first use (the Gamma
    environment, AST.hs:87-112) and named arrIn<k>_0 in the text.
Everything runs on the GPU through the C ABI; there is no other execution path.
"""
import collections
import ctypes as C
import numbers
import re
import threading
import weakref

import numpy as np

import acchip as A

__all__ = ["Exp", "constant", "cond", "use", "unit", "map", "zipWith", "generate", "backpermute", "transpose", "reverse", "zip_", "unzip", "while_",
           "fold", "fold1", "foldSeg", "fold1Seg", "scanl", "scanl1", "scanl_", "scanr", "scanr1", "scanr_", "permute", "ignore",
           "stencil", "stencil2", "awhile", "run", "compute", "run1", "fill", "enumFromN", "take", "drop", "init", "tail", "gather",
           "scatter", "foldAll", "sum_", "product", "maximum", "minimum", "and_", "or_", "all_", "any_", "filter_", "fst", "snd", "lift", "index_if", "fromIntegral", "truncate", "round_", "floor",
           "ceiling", "idiv", "mod", "quot", "rem", "min_", "max_", "sqrt", "exp", "log", "sin", "cos", "tan", "abs_",
           "signum", "Context", "the", "runWith", "run1With", "runN", "stream", "streamWith", "Async", "wait", "poll",
           "cancel", "Cancelled", "streamOut", "streamOutWith", "runAsync", "run1Async", "runAsyncWith", "run1AsyncWith", "create", "destroy",
           "unsafeFree", "unsafeFreeWith", "performGC", "performGCWith", "acond", "reshape", "flatten", "replicate", "slice_", "All",
           "imap", "zipWith3", "iterate", "asin", "acos", "atan", "sinh", "cosh", "tanh", "asinh", "acosh", "atanh", "atan2",
           "pow_", "logBase", "recip", "isNaN", "rotateL", "rotateR", "boolToInt", "ord_", "chr_", "quotRem", "divMod"]

CTYPE = dict(A.CTYPE_OF)
NPTYPE = {v: k for k, v in CTYPE.items()}
FLOATS = ("float", "double")
RANK = {"Int8": 1, "Word8": 1, "Int16": 2, "Word16": 2, "Int32": 3, "Word32": 3, "Int64": 4, "Word64": 4, "float": 5, "double": 6}


# ------------------------------------------------------------------------------ scalar expressions

def _merge(exps):
    out = []
    for e in exps:
        for st in e.binds:
            if st not in out:
                out.append(st)
    return tuple(out)


class Exp(object):
    """A typed scalar expression: a C type name, the text of a pure expression (`term`) and the
    statements that must run before it (`binds`: the loops of `while_`; the local bindings of the
    reference's code generation monad, CodeGen/Monad.hs).  Of a tuple type it holds the component
    expressions instead: tuples exist only on the host side of the generated text, `fst`/`snd` pick a
    component, and the braces of the element struct are written where a tuple becomes a result.
    `text` is the closed form a skeleton fragment takes: the term alone, or an immediately applied
    lambda holding the statements."""

    def __init__(self, ctype, term=None, comps=None, binds=()):
        self.ctype, self.comps = ctype, comps
        if comps is not None:
            term = "acc_elt{%s}" % ", ".join(c.term for c in comps)
            binds = _merge(comps)
        self.term, self.binds = term, tuple(binds)

    @property
    def text(self):
        if not self.binds:
            return self.term
        return "[&] { %s return %s; }()" % (" ".join(self.binds), self.term)

    @staticmethod
    def mk(ctype, fmt, *args):
        """an expression whose text is `fmt` over the operands' terms and which runs their statements first"""
        return Exp(ctype, fmt % tuple(a.term for a in args), binds=_merge(args))

    # -- helpers
    @staticmethod
    def of(v, like=None):
        if isinstance(v, Exp):
            return v
        if isinstance(v, (tuple, list)):
            if isinstance(like, tuple):
                return lift(*[Exp.of(e, t) for e, t in zip(v, like)])
            return lift(*v)
        t = like if like is not None else ("double" if isinstance(v, float) else "Int64")
        return constant(v, t)

    def _bin(self, other, op, result=None):
        o = Exp.of(other, self.ctype)
        if o.ctype != self.ctype:
            raise TypeError("operands of %s differ in type: %s and %s (convert with fromIntegral)" % (op, self.ctype, o.ctype))
        return Exp.mk(result or self.ctype, "((%s)(%%s %s %%s))" % (result or self.ctype, op.replace("%", "%%")), self, o)

    def _rbin(self, other, op):
        return Exp.of(other, self.ctype)._bin(self, op)

    def _call(self, fn, *others):
        args = [self] + [Exp.of(o, self.ctype) for o in others]
        for a in args:
            if a.ctype != self.ctype:
                raise TypeError("operands of %s differ in type" % fn)
        return Exp.mk(self.ctype, "%s(%s)" % (fn, ", ".join(["%s"] * len(args))), *args)

    # -- Num
    def __add__(self, o): return self._bin(o, "+")
    def __radd__(self, o): return self._rbin(o, "+")
    def __sub__(self, o): return self._bin(o, "-")
    def __rsub__(self, o): return self._rbin(o, "-")
    def __mul__(self, o): return self._bin(o, "*")
    def __rmul__(self, o): return self._rbin(o, "*")
    def __neg__(self): return Exp.mk(self.ctype, "((%s)(-%%s))" % self.ctype, self)

    # -- Fractional / Integral: `/` is fdiv on floating types and Haskell's `div` (towards -inf) on integers
    def __truediv__(self, o):
        if self.ctype in FLOATS:
            return self._bin(o, "/")
        return self._call("acc_idiv", o)

    def __rtruediv__(self, o): return Exp.of(o, self.ctype).__truediv__(self)
    def __floordiv__(self, o): return self._call("acc_idiv", o)
    def __mod__(self, o): return self._call("acc_imod", o)

    # -- Bits
    def __and__(self, o): return self._bin(o, "&")
    def __or__(self, o): return self._bin(o, "|")
    def __xor__(self, o): return self._bin(o, "^")
    def __invert__(self): return Exp.mk(self.ctype, "((%s)(~%%s))" % self.ctype, self)
    def __lshift__(self, o): return Exp.mk(self.ctype, "acc_shift_l(%s, (Int64)%s)", self, Exp.of(o, "Int64"))
    def __rshift__(self, o): return Exp.mk(self.ctype, "acc_shift_r(%s, (Int64)%s)", self, Exp.of(o, "Int64"))

    # -- Eq / Ord: Bool is Word8 (CodeGen/Type.hs:139)
    def __lt__(self, o): return self._bin(o, "<", "Word8")
    def __le__(self, o): return self._bin(o, "<=", "Word8")
    def __gt__(self, o): return self._bin(o, ">", "Word8")
    def __ge__(self, o): return self._bin(o, ">=", "Word8")
    def eq(self, o): return self._bin(o, "==", "Word8")
    def ne(self, o): return self._bin(o, "!=", "Word8")
    def land(self, o): return self._bin(o, "&&", "Word8")
    def lor(self, o): return self._bin(o, "||", "Word8")
    def lnot(self): return Exp.mk("Word8", "((Word8)(!%s))", self)

    def __bool__(self):
        raise TypeError("an Exp has no truth value on the host: use cond(p, t, e)")


def _literal(v, ctype):
    if ctype == "float":
        f = np.float32(v)
        if np.isinf(f):
            return "(-__builtin_inff())" if f < 0 else "__builtin_inff()"
        return "%sf" % repr(float(f)) if "e" in repr(float(f)) or "." in repr(float(f)) else "%s.0f" % repr(float(f))
    if ctype == "double":
        f = float(v)
        if np.isinf(f):
            return "(-__builtin_inf())" if f < 0 else "__builtin_inf()"
        return repr(f)
    if ctype in ("Int64", "Word64"):
        i = int(v)
        if i == -2 ** 63:
            return "(-9223372036854775807LL - 1)"
        return "((%s)%d%s)" % (ctype, i, "LL" if ctype == "Int64" else "ULL")
    i = int(v)
    if i == -2 ** 31:
        return "((%s)(-2147483647 - 1))" % ctype
    return "((%s)%d)" % (ctype, i)


def constant(v, ctype):
    return Exp(ctype, _literal(v, ctype))


def lift(*es):
    """a tuple of expressions as one tuple-typed expression: brace initialiser of the generated struct"""
    es = [Exp.of(e) for e in es]
    return Exp(tuple(e.ctype for e in es), comps=es)


def _var(ctype, name):
    """a kernel-side variable of the given type; of a tuple type, its members (a<n-1> is the first component)"""
    if isinstance(ctype, tuple):
        n = len(ctype)
        return Exp(ctype, comps=[Exp(t, "%s.a%d" % (name, n - 1 - k)) for k, t in enumerate(ctype)])
    return Exp(ctype, name)


def _prj(e, k):
    if not isinstance(e.ctype, tuple):
        raise TypeError("not a tuple")
    return e.comps[k]


def fst(e): return _prj(e, 0)
def snd(e): return _prj(e, 1)


def cond(p, t, e):
    t = Exp.of(t, e.ctype if isinstance(e, Exp) else None)
    e = Exp.of(e, t.ctype)
    if t.ctype != e.ctype:
        raise TypeError("branches of cond differ in type")
    if isinstance(t.ctype, tuple):
        return lift(*[cond(p, a, b) for a, b in zip(t.comps, e.comps)])
    return Exp.mk(t.ctype, "(%s ? %s : %s)", Exp.of(p), t, e)


_FRESH = [0]


def while_(p, f, init):
    """iterate `f` from `init` while `p` holds (the scalar `While` of the expression language,
    CodeGen.hs:338-821): a loop statement ahead of the expression that uses its result.  Of a tuple,
    every component is a loop variable."""
    init = Exp.of(init)
    _FRESH[0] += 1
    tup = isinstance(init.ctype, tuple)
    types = list(init.ctype) if tup else [init.ctype]
    names = ["w%d_%d" % (_FRESH[0], k) for k in range(len(types))]
    inits = init.comps if tup else [init]
    var = lift(*[Exp(t, n) for t, n in zip(types, names)]) if tup else Exp(types[0], names[0])
    nxt = Exp.of(f(var), init.ctype)
    if nxt.ctype != init.ctype:
        raise TypeError("the body of while_ changes the type of its state: %s to %s" % (init.ctype, nxt.ctype))
    nxts = nxt.comps if tup else [nxt]
    # statements of the condition and of the body belong inside the loop: their closed forms are used there
    decl = " ".join("%s %s = %s;" % (t, n, e.term) for t, n, e in zip(types, names, inits))
    step = " ".join("const %s n%s = %s;" % (t, n, e.text) for t, n, e in zip(types, names, nxts))
    copy = " ".join("%s = n%s;" % (n, n) for n in names)
    loop = "%s while (%s) { %s %s }" % (decl, Exp.of(p(var)).text, step, copy)
    binds = _merge(inits) + (loop,)
    if tup:
        return Exp(init.ctype, comps=[Exp(t, n, binds=binds) for t, n in zip(types, names)])
    return Exp(types[0], names[0], binds=binds)


def fromIntegral(e, to): return Exp.mk(to, "acc_from_integral<%s>(%%s)" % to, e)
def truncate(e, to): return Exp.mk(to, "acc_truncate<%s>(%%s)" % to, e)
def round_(e, to): return Exp.mk(to, "acc_round<%s>(%%s)" % to, e)
def floor(e, to): return Exp.mk(to, "acc_floor<%s>(%%s)" % to, e)
def ceiling(e, to): return Exp.mk(to, "acc_ceiling<%s>(%%s)" % to, e)
def idiv(a, b): return Exp.of(a)._call("acc_idiv", b)
def mod(a, b): return Exp.of(a)._call("acc_imod", b)
def quot(a, b): return Exp.of(a)._call("acc_quot", b)
def rem(a, b): return Exp.of(a)._call("acc_rem", b)
def min_(a, b): return Exp.of(a)._call("acc_pmin", b)
def max_(a, b): return Exp.of(a)._call("acc_pmax", b)
def abs_(a): return a._call("acc_abs")
def signum(a): return a._call("acc_signum")
def sqrt(a): return a._call("acc_sqrt")
def exp(a): return a._call("acc_exp")
def log(a): return a._call("acc_log")
def sin(a): return a._call("acc_sin")
def cos(a): return a._call("acc_cos")
def tan(a): return a._call("acc_tan")
def asin(a): return a._call("acc_asin")
def acos(a): return a._call("acc_acos")
def atan(a): return a._call("acc_atan")
def sinh(a): return a._call("acc_sinh")
def cosh(a): return a._call("acc_cosh")
def tanh(a): return a._call("acc_tanh")
def asinh(a): return a._call("acc_asinh")
def acosh(a): return a._call("acc_acosh")
def atanh(a): return a._call("acc_atanh")
def atan2(y, x): return Exp.of(y)._call("acc_atan2", x)
def pow_(a, b): return Exp.of(a)._call("acc_pow", b)
def logBase(base, y): return Exp.of(base)._call("acc_log_base", y)
def recip(a): return a._call("acc_recip")
def isNaN(a): return Exp.mk("Word8", "acc_is_nan(%s)", a)
def rotateL(a, i): return Exp.mk(a.ctype, "acc_rotate_l(%s, (Int64)%s)", a, Exp.of(i, "Int64"))
def rotateR(a, i): return Exp.mk(a.ctype, "acc_rotate_r(%s, (Int64)%s)", a, Exp.of(i, "Int64"))
def boolToInt(b): return Exp.mk("Int64", "acc_bool_to_int(%s)", b)
def ord_(c): return Exp.mk("Int64", "acc_ord(%s)", c)
def chr_(i): return Exp.mk("Word32", "acc_chr(%s)", i)


def quotRem(a, b):
    """(quotient, remainder) truncated towards zero, as a pair (Arithmetic.hs:90-104)"""
    return lift(quot(a, b), rem(a, b))


def divMod(a, b):
    """(quotient, remainder) rounded towards minus infinity, as a pair (Arithmetic.hs:106-158)"""
    return lift(idiv(a, b), mod(a, b))


ignore = "ignore"        # the target index that drops an element (IndexSpace.hs:150-151)


# ------------------------------------------------------------------------------ arrays

class Acc(object):
    """An array-valued computation: its shape (outermost first), element type and either a device
    array (manifest) or an index -> value function (delayed)."""

    def __init__(self, shape, ctype, manifest=None, at=None, across=False):
        self.shape, self.ctype, self.manifest, self.at = tuple(int(s) for s in shape), ctype, manifest, at
        # a delayed array that reads a source across its rows (a transpose): the map kernel that makes it manifest
        # produces it in square tiles (ACC_FLAG_TILED).  The number of the result's dimension, counted from the
        # innermost, along which the source is read: 1 for a transpose, 2 and more for a volume that was turned
        # (ACC_FLAG_TILE_DIM); 0 for an array read along its rows.
        self.across = int(across) if (across and manifest is None and len(self.shape) >= 2) else 0

    @property
    def size(self):
        n = 1
        for s in self.shape:
            n *= s
        return n

    def index(self, ix):
        """value at linear index `ix` (an Exp of type Int64).  A manifest array is named by a tag that
        is replaced by its place in the kernel's environment when the kernel is assembled; read at the
        consuming skeleton's own index `ix` it is a streaming read (each element is wanted once)."""
        if self.manifest is not None:
            tag = _tag(self.manifest)
            if isinstance(self.ctype, tuple):
                n = len(self.ctype)
                return Exp(self.ctype, comps=[Exp.mk(t, "%s_%d[%%s]" % (tag, n - 1 - i), ix) for i, t in enumerate(self.ctype)])
            if ix.term == "ix":
                return Exp(self.ctype, "acc_stream(%s_0, ix)" % tag)
            return Exp.mk(self.ctype, "%s_0[%%s]" % tag, ix)
        return self.at(ix)

    def stream(self):
        """value at the consuming skeleton's own linear index"""
        return self.index(Exp("Int64", "ix"))

    def __getitem__(self, idx):
        """`arr ! ix` inside a scalar function: idx is a multi-index (a tuple of Exps) or, for a vector, one Exp"""
        return self.index(_linear(idx, self.shape))


_MANIFEST = weakref.WeakValueDictionary()        # tag number -> device array, while some computation still names it


_building = threading.local()     # .pending: arrays named in text that this thread has not assembled yet -- an array
                                  # `use`d inside a scalar function is referred to by nothing else until then


def _pending():
    q = getattr(_building, "pending", None)
    if q is None:
        q = _building.pending = collections.deque(maxlen=16)
    return q


def _tag(manifest):
    _MANIFEST[id(manifest)] = manifest
    q = _pending()
    if not any(m is manifest for m in q):
        q.append(manifest)
    return "@@%d@@" % id(manifest)


def _assemble(**fragments):
    """number the free arrays the fragments name, in order of first appearance (the Gamma environment of
    AST.hs:87-112), and spell them arrIn<k>: returns (arrays, signature, fragments)"""
    order = []
    for text in fragments.values():
        for m in re.finditer(r"@@(\d+)@@", text or ""):
            if int(m.group(1)) not in order:
                order.append(int(m.group(1)))
    arrays = [_MANIFEST[i] for i in order]
    q = _pending()
    for m in arrays:                                  # from here on the caller holds them
        for k in range(len(q) - 1, -1, -1):
            if q[k] is m:
                del q[k]
    out = {}
    for name, text in fragments.items():
        if text is not None:
            for k, i in enumerate(order):
                text = text.replace("@@%d@@" % i, "arrIn%d" % k)
        out[name] = text
    sig = []
    for m in arrays:
        if isinstance(m, A.TupleArray):
            sig.append((len(m.shape), m.ctypes_of()))
        else:
            sig.append((len(m.shape), CTYPE[m.dtype.type]))
    return arrays, sig, out


def _context(context, *operands):
    """where a skeleton runs: the context given, else the one its array operands live in (the context of
    `use ... context`), else the default one (CUDA.hs:205-206 `defaultContext`)"""
    if context is not None:
        return context
    found = None
    for a in operands:
        if isinstance(a, Acc) and a.manifest is not None:
            ms = [a.manifest]
        elif isinstance(a, (Acc, str)):          # a delayed array, or the text of a fragment: the arrays it names
            ms = [_MANIFEST[int(i)] for i in re.findall(r"@@(\d+)@@", a if isinstance(a, str) else a.stream().text)]
        else:
            continue
        for m in ms:
            for c in (m.comps if isinstance(m, A.TupleArray) else [m]):
                cx = getattr(c, "cx", None)
                if cx is not None and found is not None and cx is not found:
                    raise ValueError("the operands of one computation live in different contexts")
                found = found or cx
    return found or Context.default()


class _ResultPool(object):
    """Host memory for the results that `run` hands out, page-locked and used again.  A result of 256 MB in a new
    array costs 4 ms before a byte has arrived (the kernel clears every page when it is first touched) and comes
    through the library's staging buffers; into page-locked memory the device writes directly, at the link's rate,
    and a buffer whose array the program has dropped has its pages already.  Page-locking is dear (tens of ms for
    such a buffer), so a size is served from here from the second time it is asked for -- the program that calls a
    `run1` function over and over -- and the pool never holds more than `limit` bytes, handed out or not; everything
    else gets an ordinary array.  A buffer comes back when the last array (or view) on it is collected."""
    GRAIN = 1 << 20

    def __init__(self, ctx, limit):
        self.ctx, self.limit, self.held, self.closed = ctx, limit, 0, False
        self.spare, self.asked = {}, {}
        self.lock = threading.Lock()       # (collection may happen on any thread, at any time)

    def array(self, shape, dtype):
        dtype = np.dtype(dtype)
        size = int(np.prod(shape, dtype=np.int64))
        nbytes = size * dtype.itemsize
        if nbytes < self.GRAIN or self.closed:
            return None
        room = -(-nbytes // self.GRAIN) * self.GRAIN
        with self.lock:
            spare = self.spare.get(room)
            if spare:
                addr = spare.pop()
            else:
                self.asked[room] = self.asked.get(room, 0) + 1
                if self.asked[room] < 2 or self.held + room > self.limit:
                    return None
                p = C.c_void_p()
                if A.lib().acc_host_alloc(self.ctx.handle, room, C.byref(p)) != 0 or not p.value:
                    return None
                addr = p.value
                self.held += room
        buf = (C.c_ubyte * nbytes).from_address(addr)
        weakref.finalize(buf, self._back, room, addr).atexit = False
        return np.frombuffer(buf, dtype=dtype, count=size).reshape(shape)

    def _back(self, room, addr):
        with self.lock:
            if not self.closed:
                self.spare.setdefault(room, []).append(addr)
                return
        A.lib().acc_host_free(None, C.c_void_p(addr))      # its context has gone: the memory is the process's

    def trim(self, close=False):
        """give the buffers that nobody holds back to the system (and, closing, take no more back)"""
        with self.lock:
            addrs = [(room, a) for room, lst in self.spare.items() for a in lst]
            self.spare = {}
            self.held -= sum(room for room, _ in addrs)
            self.closed = self.closed or close
        for _, a in addrs:
            A.lib().acc_host_free(self.ctx.handle, C.c_void_p(a))


class _Resident(object):
    """A manifest array under the context's memory table: host storage (the array `use`d, or the place a result is
    written back to when the device is full) and the table entry keyed by it.  The device address is only known
    between acquire and release, which bracket every launch (Context.launch)."""

    def __init__(self, cx, host, frozen):
        self.cx, self.host, self.shape, self.dtype, self.size = cx, host, host.shape, host.dtype, host.size
        self.key = A.MemTable.key(host)
        self.stream, self.ready = None, None          # where it was produced, and the event recorded behind that
        self.pending = None                           # the launch that will produce it, while that is put off (_Pending)
        with cx.lock:
            cx.table.malloc(host, frozen)
            cx.live[self.key] = cx.live.get(self.key, 0) + 1

    def get(self):
        if self.cx.loop is not None:
            raise _HostReadInLoop()          # an iteration enqueued ahead cannot wait for the host
        if self.pending is not None:
            self.pending.force()
        if self.ready is not None:
            A.check(A.lib().acc_event_sync(self.cx.ctx.handle, self.ready))
        d = self.cx.table.acquire(self.host)
        try:
            return d.get(self.cx.results.array(self.shape, self.dtype))
        finally:
            self.cx.table.release(self.host)

    def __del__(self):
        try:
            cx = self.cx
            with cx.lock:
                if self.ready is not None:
                    cx.events.append(self.ready)
                cx.live[self.key] -= 1
                if cx.live[self.key] == 0:
                    del cx.live[self.key]
                    if cx.table.handle:
                        cx.table.free(self.host)
        except Exception:
            pass


def _parts(ms):
    for m in ms:
        if isinstance(m, A.TupleArray):
            for c in m.comps:
                yield c
        elif m is not None:
            yield m


class _Pending(object):
    """A skeleton launch that has been put off until its result is wanted.  The instance was created when the
    consumer was written down -- its compilation runs on the library's worker pool from then on -- and nothing waits
    for it before `run` (or `the`, or a loop) asks for a value that depends on it: the kernels of a program are
    compiling side by side while the program is still being built, and execution blocks where a kernel is first used
    (Compile.hs:451-457,484-538: the reference's compile phase forks every kernel's compilation before its execute
    phase starts).  The results hold the node; it goes away with them if nobody ever asks."""

    def __init__(self, cx, inputs, outputs, go):
        self.cx, self.inputs, self.outputs, self.go, self.done = cx, inputs, outputs, go, False
        for m in _parts(outputs):
            m.pending = self
        cx.pending.append(weakref.ref(self))

    def force(self):
        cx = self.cx
        with cx.lock:
            if self.done:
                return
            self.done = True
            inputs, outputs, go = self.inputs, self.outputs, self.go
            self.inputs = self.outputs = self.go = None
            for m in _parts(outputs):
                m.pending = None
            cx._launch(inputs, outputs, go)


class _HostReadInLoop(Exception):
    """raised where the body or the predicate of an `awhile` whose iterations are being enqueued ahead asks for a
    value on the host (`the`, a nested loop): that loop then goes on one iteration at a time"""


class _Loop(object):
    def __init__(self, stream, guard):
        self.stream, self.guard = stream, guard


class Cancelled(Exception):
    """raised inside, and by `wait` on, a computation that `cancel` stopped"""


_running = threading.local()     # .asy: the Async whose thread this is


class Context(object):
    """a device context, the table of skeleton instances built so far (the kernel table of State.hs:110-119) and the
    memory table every manifest array lives in (State.hs:120-122): `budget_bytes` bounds the device memory held,
    0 leaves that to the device.  Skeletons are launched asynchronously: a computation continues on the stream that
    produced its first operand, one whose operands are all `use`d arrays takes the next stream of a small reservoir
    (Execute/Stream.hs:66-74), and a stream waits for the events of operands produced on other streams
    (Execute.hs:104-105,183-184), so independent subcomputations overlap and the host never waits before `run`."""
    _default = None

    def __init__(self, device=0, budget_bytes=0, result_pool_bytes=1 << 30):
        self.ctx = A.Context(device)
        self.table = A.MemTable(self.ctx, budget_bytes)
        self.results = _ResultPool(self.ctx, result_pool_bytes)   # page-locked host memory for results, used again
        self.live = {}
        self.skeletons = {}
        self.streams, self.turn, self.events = [], 0, []
        self.lock = threading.RLock()      # one host thread at a time evaluates in a context (CUDA.hs:251-252)
        self.loop, self.guard = None, None # the `awhile` being enqueued ahead, if any, and the context's loop guard
        self.pending = []                  # weak references to the launches put off so far (_Pending), oldest first
        self.lazy = True                   # False: every consumer launches where it is written down

    @classmethod
    def default(cls):
        if cls._default is None:
            cls._default = Context(0)
        return cls._default

    def skeleton(self, kind, elt, env, **kw):
        key = (kind, elt, tuple((r, tuple(t) if isinstance(t, list) else t) for r, t in env),
               tuple(sorted((k, str(v)) for k, v in kw.items())))
        with self.lock:
            if self.loop is not None:          # kernels that look at the loop's guard: instances of their own
                kw = dict(kw, flags=kw.get("flags", 0) | A.FLAG_GUARDED)
                key = key + ("guarded",)
            sk = self.skeletons.get(key)
            if sk is None:
                sk = self.ctx.skeleton(kind, elt, env=env, **kw)
                self.skeletons[key] = sk
        return sk

    N_STREAMS = 4

    def _stream_for(self, inputs):
        if self.loop is not None:
            return self.loop.stream               # everything of a loop enqueued ahead is ordered by one stream
        for m in inputs:
            if m.stream is not None:
                return m.stream
        if len(self.streams) < self.N_STREAMS:
            self.streams.append(self.ctx.stream())
        self.turn = (self.turn + 1) % len(self.streams)
        return self.streams[self.turn]

    def launch(self, inputs, outputs, go):
        """run `go(input views, output views, stream)` with the arrays resident (None stays None), after what
        produced the inputs; the outputs carry the event recorded behind it"""
        with self.lock:
            # put off until a value is wanted, unless the launch belongs to a loop that is being enqueued ahead (its
            # kernels go onto the loop's stream now, in order) or produces nothing to wait for
            if self.lazy and self.loop is None and any(True for _ in _parts(outputs)):
                _Pending(self, inputs, outputs, go)
                return
            return self._launch(inputs, outputs, go)

    def flush(self):
        """launch everything that has been put off, oldest first (before a loop takes a stream under its guard,
        before arrays are freed by hand, before the context goes away)"""
        with self.lock:
            nodes, self.pending = self.pending, []
            for ref in nodes:
                node = ref()
                if node is not None:
                    node.force()

    def _launch(self, inputs, outputs, go):
        parts = _parts
        for m in list(parts(inputs)):                   # what produces an operand comes first
            if m.pending is not None:
                m.pending.force()
        if len(self.pending) > 256:                     # forget the nodes that are done or gone
            self.pending = [r for r in self.pending if r() is not None and not r().done]
        asy = getattr(_running, "asy", None)
        if asy is not None and asy._cancelled:
            raise Cancelled()                           # between two skeletons: a launch already made runs to its end
        stream = self._stream_for(list(parts(inputs)))
        L = A.lib()
        for m in parts(inputs):
            if m.ready is not None and m.stream is not stream:
                A.check(L.acc_stream_wait_event(self.ctx.handle, stream, m.ready))
        taken = []

        def view(m):
            if m is None:
                return None
            if isinstance(m, A.TupleArray):
                return A.TupleArray([view(c) for c in m.comps])
            d = self.table.acquire(m.host, stream)
            taken.append(m)
            return d
        try:
            go([view(m) for m in inputs], [view(m) for m in outputs], stream)
            for m in parts(outputs):
                if m.ready is None:
                    m.ready = self.events.pop() if self.events else self.ctx.event(timing=False)
                A.check(L.acc_event_record(self.ctx.handle, m.ready, stream))
                m.stream = stream
        finally:
            for m in taken:
                self.table.release(m.host, stream)


def _elt(ctype):
    return ", ".join(ctype) if isinstance(ctype, tuple) else ctype


def _dtype(ctype):
    return [NPTYPE[c] for c in ctype] if isinstance(ctype, tuple) else NPTYPE[ctype]


def _empty(cx, shape, ctype):
    """device memory for a result; its host side is untouched pages until the result is evicted or read"""
    if isinstance(ctype, tuple):
        return A.TupleArray([_Resident(cx, np.empty(shape, dtype=t), False) for t in _dtype(ctype)])
    return _Resident(cx, np.empty(shape, dtype=_dtype(ctype)), False)


def use(host, context=None):
    """a host array (or a tuple of equally shaped host arrays: an array of tuples) made available on the device.
    It is uploaded when first wanted there and once only, however often it is `use`d (Array/Prim.hs:177-192); it must
    not be changed afterwards."""
    cx = context or Context.default()
    as_word8 = lambda h: h.view(np.uint8) if h.dtype == np.bool_ else h      # Bool is Word8 on the device (CodeGen/Type.hs)
    if isinstance(host, tuple):
        hs = [as_word8(np.asarray(h, order="C")) for h in host]
        return Acc(hs[0].shape, tuple(CTYPE[h.dtype.type] for h in hs), manifest=A.TupleArray([_Resident(cx, h, True) for h in hs]))
    host = as_word8(np.asarray(host, order="C"))        # (ascontiguousarray would make a scalar array a vector)
    return Acc(host.shape, CTYPE[host.dtype.type], manifest=_Resident(cx, host, True))


def unit(value, ctype, context=None):
    return use(np.array(value, dtype=NPTYPE[ctype]), context)


def _unlinear(ix, shape):
    """multi-index (outermost first) of a linear index, as Exps; extents are literals, so the divisions are by constants"""
    if ix.term == "ix" and getattr(_building, "rows_of", None) == tuple(shape) and len(shape) >= 2:
        # inside a fold along the innermost dimension that gives every row to a lane: the row and the place within
        # it are names of the kernel, and what depends on the row alone leaves the lane's loop
        return _unlinear(Exp("Int64", "acc_row"), shape[:-1]) + (Exp("Int64", "acc_col"),)
    made_of = getattr(ix, "made_of", None)
    if made_of is not None and made_of[1] == tuple(shape):
        # the linear index of this very multi-index (an index function applied to the result of another, as where a
        # transposed array is replicated): taking it apart again gives the multi-index back, without a division
        return made_of[0]
    count = 1
    for ext in shape:
        count *= ext
    if 0 < count < 2 ** 31 and len(shape) > 1:
        # an index into fewer than 2^31 elements is taken apart in 32 bits: a division by a literal is then a
        # multiplication and a shift, where the 64-bit one is twenty instructions (generate over 500^3: 240 -> 100 us)
        out, rest = [], Exp.mk("Word32", "((Word32)%s)", ix)
        for d in range(len(shape) - 1, 0, -1):
            ext = Exp("Word32", "%du" % shape[d])
            out.append(Exp.mk("Int64", "((Int64)(%s %% %s))", rest, ext))
            rest = Exp.mk("Word32", "(%s / %s)", rest, ext)
        out.append(Exp.mk("Int64", "((Int64)%s)", rest))
        return tuple(reversed(out))
    out, rest = [], ix
    for d in range(len(shape) - 1, -1, -1):
        ext = constant(shape[d], "Int64")
        if d == 0:
            out.append(rest)
        else:
            out.append(Exp.mk("Int64", "(%s %% %s)", rest, ext))
            rest = Exp.mk("Int64", "(%s / %s)", rest, ext)
    return tuple(reversed(out))


def _linear(idx, shape):
    idx = [Exp.of(i, "Int64") for i in (idx if isinstance(idx, (tuple, list)) else (idx,))]
    idx = [i if i.ctype == "Int64" else fromIntegral(i, "Int64") for i in idx]
    if len(idx) != len(shape):
        raise TypeError("index of rank %d into an array of rank %d" % (len(idx), len(shape)))
    if not shape:
        return constant(0, "Int64")
    acc_ = idx[0]
    for d in range(1, len(shape)):
        acc_ = acc_ * constant(shape[d], "Int64") + idx[d]
    if acc_ is idx[0]:
        acc_ = Exp(acc_.ctype, acc_.term, binds=acc_.binds)     # (an object of its own to hang the note on)
    acc_.made_of = (tuple(idx), tuple(shape))
    return acc_


def _probe(f, *ctypes):
    """result type of a scalar function, found by applying it to dummy operands"""
    return Exp.of(f(*[_var(c, "_") for c in ctypes])).ctype


def map(f, a):
    t = _probe(f, a.ctype)
    return Acc(a.shape, t, at=lambda ix: Exp.of(f(a.index(ix))), across=a.across)


def _meet(s1, s2):
    return tuple(min(x, y) for x, y in zip(s1, s2))


def zipWith(f, a, b):
    """extent = intersection of the operands' extents (Accelerate's zipWith)"""
    if a.shape != b.shape:
        if len(a.shape) != len(b.shape):
            raise TypeError("zipWith of arrays of different rank")
        shape = _meet(a.shape, b.shape)
        a = a if a.shape == shape else backpermute(shape, lambda *i: i, a)
        b = b if b.shape == shape else backpermute(shape, lambda *i: i, b)
    t = _probe(f, a.ctype, b.ctype)
    return Acc(a.shape, t, at=lambda ix: Exp.of(f(a.index(ix), b.index(ix))), across=a.across or b.across)


def generate(shape, f):
    shape = (shape,) if isinstance(shape, numbers.Integral) else tuple(shape)
    t = _probe(f, *["Int64"] * len(shape))
    return Acc(shape, t, at=lambda ix: Exp.of(f(*_unlinear(ix, shape))))


def _steps_of(p, shape, src_shape):
    """how far `p` moves through the source (in elements of its row-major order) where the result's index moves by
    one along each of its dimensions, the innermost first: found by applying `p` to plain numbers, which an index
    function made of arithmetic alone accepts.  None where it does not, or where the result is too small to take a
    step along its two innermost dimensions."""
    if len(shape) < 2 or shape[-1] < 2 or shape[-2] < 2:
        return None

    def place(idx):
        r = p(*idx)
        r = tuple(r) if isinstance(r, (tuple, list)) else (r,)
        if len(r) != len(src_shape) or not all(isinstance(v, numbers.Integral) for v in r):
            raise TypeError
        at = 0
        for v, ext in zip(r, src_shape):
            at = at * ext + int(v)
        return at
    try:
        zero = [0] * len(shape)
        here = place(zero)
        steps = []
        for d in range(len(shape) - 1, -1, -1):               # innermost dimension first
            steps.append(place(zero[:d] + [1] + zero[d + 1:]) - here if shape[d] >= 2 else 0)
        return steps
    except Exception:
        return None


def backpermute(shape, p, a, across=None):
    """result[i] = a[p(i)]: p takes the result's multi-index and returns a multi-index of `a`.  `across`: p walks
    down a column of `a` where the result's index moves along a row (see transpose); where it is not given, an index
    function made of arithmetic alone is asked by applying it to numbers."""
    shape = (shape,) if isinstance(shape, numbers.Integral) else tuple(shape)
    if across is None:
        steps = _steps_of(p, shape, a.shape)
        across = 0
        if steps is None:
            pass
        elif abs(steps[0]) == 1:
            across = a.across if a.across <= 1 else 0    # along the rows of `a`: what `a` reads across, the result does
        elif steps[0] != 0 and a.across == 0:
            # the dimension of the result along which `a` is read side by side: the second innermost (a transpose),
            # or one further out (a volume turned so that its innermost dimension becomes an outer one)
            for d in range(1, len(steps)):
                if abs(steps[d]) == 1:
                    across = d
                    break
        # (an exchange of the two innermost dimensions of an array that is itself read across: along the rows again)
    return Acc(shape, a.ctype, at=lambda ix: a.index(_linear(p(*_unlinear(ix, shape)), a.shape)), across=across)


def transpose(a):
    h, w = a.shape
    return backpermute((w, h), lambda y, x: (x, y), a)


def zip_(a, b):
    """array of pairs over the intersection of the extents"""
    return zipWith(lambda x, y: lift(x, y), a, b)


def unzip(a):
    return map(fst, a), map(snd, a)


def reverse(a):
    n = a.shape[0]
    return backpermute((n,), lambda i: (constant(n - 1, "Int64") - i,), a)


# ------------------------------------------------------------------------------ execution

def _force(a, cx):
    """a manifest array holding `a` (one map kernel if it is delayed)"""
    if a.manifest is not None:
        return a
    arrays, sig, fr = _assemble(get=a.stream().text)
    sk = cx.skeleton(A.SKEL_MAP, _elt(a.ctype), sig, out_rank=len(a.shape),
                     flags=(A.FLAG_TILED | A.FLAG_TILE_DIM(a.across)) if a.across else 0, **fr)
    out = _empty(cx, a.shape, a.ctype)
    cx.launch(arrays, [out], lambda i, o, s: sk.map(i, o[0], stream=s))
    return Acc(a.shape, a.ctype, manifest=out)


def _combine(f, ctype):
    r = Exp.of(f(_var(ctype, "x"), _var(ctype, "y")), ctype)
    if r.ctype != ctype:
        raise TypeError("the combining function returns %s for elements of type %s" % (r.ctype, ctype))
    return r


def _fold(f, z, a, seedless, context):
    cx = _context(context, a)
    if a.across >= 2 and len(a.shape) > a.across:
        # The source is read side by side along a dimension of `a` further out than the second innermost (the sum
        # over the middle dimension of a volume, written as a fold of the volume turned): the fold of `a` with that
        # dimension and the second innermost exchanged gives a row to a lane with neighbouring rows side by side in
        # memory, and its result with the two exchanged back (delayed: whoever consumes it reads it across) is the
        # fold of `a`.
        r = len(a.shape)
        i1, id_ = r - 2, r - 1 - a.across

        def exchanged(ix):
            ix = list(ix)
            ix[i1], ix[id_] = ix[id_], ix[i1]
            return tuple(ix)
        turned = backpermute(exchanged(a.shape), lambda *ix: exchanged(ix), a, across=1)
        folded = _fold(f, z, turned, seedless, cx)
        return backpermute(exchanged(folded.shape), lambda *ix: exchanged(ix), folded)
    # an empty outer extent counts as 1 in the result of a seeded fold (Execute.hs:287-289)
    out_shape = a.shape[:-1] if seedless else tuple(max(1, d) for d in a.shape[:-1])
    _building.rows_of = tuple(a.shape) if a.across == 1 else None
    try:
        get = a.stream().text
    finally:
        _building.rows_of = None
    arrays, sig, fr = _assemble(get=get, combine=_combine(f, a.ctype).text, seed=None if seedless else Exp.of(z, a.ctype).text)
    # rows that lie across memory (the fold of a transposed matrix, of a product of replicated operands): a lane a row
    sk = cx.skeleton(A.SKEL_FOLD1 if seedless else A.SKEL_FOLD, _elt(a.ctype), sig, out_rank=len(out_shape),
                     flags=A.FLAG_TILED if a.across == 1 and len(out_shape) >= 1 else 0, **fr)
    out = _empty(cx, out_shape, a.ctype)
    cx.launch(arrays, [out], lambda i, o, s: sk.fold(i, a.shape, o[0], stream=s))
    return Acc(out_shape, a.ctype, manifest=out)


def fold(f, z, a, context=None):
    """reduce the innermost dimension with an associative f; z is combined in once (Reduction.hs:203-211)"""
    return _fold(f, z, a, False, context)


def fold1(f, a, context=None):
    return _fold(f, None, a, True, context)


def _foldseg(f, z, a, seg_lengths, seedless, context):
    cx = _context(context, a, seg_lengths)
    offs = scanl(lambda x, y: x + y, constant(0, seg_lengths.ctype), seg_lengths, context=cx)
    arrays, sig, fr = _assemble(get=a.stream().text, combine=_combine(f, a.ctype).text,
                                seed=None if seedless else Exp.of(z, a.ctype).text)
    rank = len(a.shape)
    sk = cx.skeleton(A.SKEL_FOLD1SEG if seedless else A.SKEL_FOLDSEG, _elt(a.ctype), sig, out_rank=rank,
                     seg_type=seg_lengths.ctype, **fr)
    nseg = seg_lengths.shape[0]
    out_shape = tuple(a.shape[:-1]) + (nseg,)
    out = _empty(cx, out_shape, a.ctype)
    cx.launch(arrays + [offs.manifest], [out], lambda i, o, s: sk.foldseg_nd(i[:-1], a.shape, i[-1], o[0], stream=s))
    return Acc(out_shape, a.ctype, manifest=out)


def foldSeg(f, z, a, seg_lengths, context=None):
    """reduce each segment of the innermost dimension -- of a vector, or of every outer row of an array of higher
    rank (Reduction.hs:473-474); `seg_lengths` is a vector of segment lengths (Int32), turned into offsets by an
    exclusive scan on the device as the front end does (CUDA.hs:402)"""
    return _foldseg(f, z, a, seg_lengths, False, context)


def fold1Seg(f, a, seg_lengths, context=None):
    """foldSeg without a seed: every segment must be non-empty"""
    return _foldseg(f, None, a, seg_lengths, True, context)


def _scan(kind, f, z, a, context):
    cx = _context(context, a)
    if len(a.shape) != 1:
        raise TypeError("scans are over vectors")
    arrays, sig, fr = _assemble(get=a.stream().text, combine=_combine(f, a.ctype).text,
                                seed=Exp.of(z, a.ctype).text if z is not None else None)
    sk = cx.skeleton(A.SCAN_KINDS[kind], _elt(a.ctype), sig, **fr)
    n = a.shape[0]
    m = n + 1 if kind in ("scanl", "scanr") else n
    out = _empty(cx, (m,), a.ctype)
    total = _empty(cx, (), a.ctype) if kind.endswith("'") else None
    cx.launch(arrays, [out, total], lambda i, o, s: sk.scan(i, n, o[0], o[1], stream=s))
    res = Acc((m,), a.ctype, manifest=out)
    return (res, Acc((), a.ctype, manifest=total)) if total is not None else res


def scanl(f, z, a, context=None): return _scan("scanl", f, z, a, context)
def scanl1(f, a, context=None): return _scan("scanl1", f, None, a, context)
def scanl_(f, z, a, context=None): return _scan("scanl'", f, z, a, context)      # scanl': (body, total)
def scanr(f, z, a, context=None): return _scan("scanr", f, z, a, context)
def scanr1(f, a, context=None): return _scan("scanr1", f, None, a, context)
def scanr_(f, z, a, context=None): return _scan("scanr'", f, z, a, context)


_HINTS = {"+": A.COMBINE_ADD, "min": A.COMBINE_MIN, "max": A.COMBINE_MAX, "&": A.COMBINE_AND, "|": A.COMBINE_OR, "^": A.COMBINE_XOR}


def _hint(f, ctype):
    """recognise a combining function the hardware applies atomically, by its generated text (the check a code
    generator makes on the expression tree)"""
    if isinstance(ctype, tuple) or ctype not in ("Int32", "Word32", "Int64", "Word64", "float", "double"):
        return A.COMBINE_GENERIC
    text = _combine(f, ctype).text
    for op, h in _HINTS.items():
        if len(op) == 1:
            forms = ("((%s)(x %s y))" % (ctype, op), "((%s)(y %s x))" % (ctype, op))
        else:
            forms = ("acc_p%s(x, y)" % op, "acc_p%s(y, x)" % op)
        if text in forms and (ctype not in FLOATS or op == "+"):
            return h
    return A.COMBINE_GENERIC


class _Maybe(object):
    def __init__(self, p, idx):
        self.p, self.idx = Exp.of(p), idx


def index_if(p, idx):
    """a permutation result that is `idx` where p holds and `ignore` elsewhere"""
    return _Maybe(p, idx)


def permute(f, defaults, p, a, context=None):
    """forward permutation: out = defaults; out[p(i)] = f(a[i], out[p(i)]) for every source index i;
    p(i) = ignore (or index_if with a false condition) drops the element"""
    t = p(*_unlinear(Exp("Int64", "ix"), a.shape))
    if isinstance(t, str) and t == ignore:
        perm_text = "ACC_IGNORE"
    elif isinstance(t, _Maybe):
        perm_text = Exp.mk("Int64", "(%s ? %s : ACC_IGNORE)", t.p, _linear(t.idx, defaults.shape)).text
    else:
        perm_text = _linear(t, defaults.shape).text
    cx = _context(context, defaults, a, perm_text)
    dfl = _force(defaults, cx)
    arrays, sig, fr = _assemble(get=a.stream().text, combine=_combine(f, a.ctype).text, permutation=perm_text)
    sk = cx.skeleton(A.SKEL_PERMUTE, _elt(a.ctype), sig, out_rank=len(dfl.shape), combine_hint=_hint(f, a.ctype), **fr)
    out = _empty(cx, dfl.shape, a.ctype)
    cx.launch(arrays + [dfl.manifest], [out], lambda i, o, s: sk.permute(i[:-1], a.size, i[-1], o[0], stream=s))
    return Acc(dfl.shape, a.ctype, manifest=out)


def the(a, context=None):
    """the value of a scalar array, on the host"""
    return run(a, context)[()]


def _taps(pattern, rank):
    offs = []
    for t in pattern:
        t = tuple(t) if isinstance(t, (tuple, list)) else (t,)
        offs.append((0,) * (max(2, rank) - len(t)) + t)
    return offs


def _boundary_constant(value, ctype):
    """the value outside the array under a constant boundary, as text: of a tuple source one literal per component"""
    if value is None:
        return None
    if isinstance(ctype, tuple):
        if not isinstance(value, (tuple, list)) or len(value) != len(ctype):
            raise TypeError("the boundary constant of a stencil over %d-tuples is a %d-tuple" % (len(ctype), len(ctype)))
        return ", ".join(_literal(v, t) for v, t in zip(value, ctype))
    return _literal(value, ctype)


def stencil(pattern, f, boundary, a, context=None, constant_value=None):
    """result[i] = f(a[i + o] for o in pattern); boundary is "clamp", "mirror", "wrap" or "constant"
    (Stencil/Extra.hs:112-116); the source is made manifest first, as in the reference (Execute.hs:413-425)"""
    cx = _context(context, a)
    src = _force(a, cx)
    rank = len(src.shape)
    taps = _taps(pattern, rank)
    res = Exp.of(f(*[_var(src.ctype, "t%d" % k) for k in range(len(taps))]))        # a tap of a tuple source: its members
    arrays, sig, fr = _assemble(stencil_fn=res.text)
    sk = cx.skeleton(A.SKEL_STENCIL, _elt(res.ctype), sig, out_rank=rank, taps=taps, boundary=boundary,
                     boundary_constant=_boundary_constant(constant_value, src.ctype), stencil_in=_elt(src.ctype), **fr)
    out = _empty(cx, src.shape, res.ctype)
    cx.launch(arrays + [src.manifest], [out], lambda i, o, s: sk.stencil(i[:-1], i[-1], o[0], stream=s))
    return Acc(src.shape, res.ctype, manifest=out)


def stencil2(pattern1, pattern2, f, boundary1, a, boundary2, b, context=None, constant1=None, constant2=None):
    """f receives the list of taps of the first source and the list of taps of the second"""
    cx = _context(context, a, b)
    s1, s2 = _force(a, cx), _force(b, cx)
    rank = len(s1.shape)
    t1, t2 = _taps(pattern1, rank), _taps(pattern2, rank)
    res = Exp.of(f([_var(s1.ctype, "t%d" % k) for k in range(len(t1))], [_var(s2.ctype, "u%d" % k) for k in range(len(t2))]))
    arrays, sig, fr = _assemble(stencil_fn=res.text)
    sk = cx.skeleton(A.SKEL_STENCIL2, _elt(res.ctype), sig, out_rank=rank, taps=t1, boundary=boundary1, taps2=t2, boundary2=boundary2,
                     boundary_constant=_boundary_constant(constant1, s1.ctype), boundary2_constant=_boundary_constant(constant2, s2.ctype),
                     stencil_in=_elt(s1.ctype), stencil_in2=_elt(s2.ctype), **fr)
    shape = _meet(s1.shape, s2.shape)
    out = _empty(cx, shape, res.ctype)
    cx.launch(arrays + [s1.manifest, s2.manifest], [out], lambda i, o, s: sk.stencil2(i[:-2], i[-2], i[-1], o[0], stream=s))
    return Acc(shape, res.ctype, manifest=out)


# ------------------------------------------------------------------------------ library functions
# What Data.Array.Accelerate.Prelude builds out of the primitive operations, built the same way.

def fill(shape, value, ctype):
    return generate(shape, lambda *ix: constant(value, ctype))


def enumFromN(shape, first, ctype="Int64"):
    """first, first + 1, ... in row-major order"""
    shape = (shape,) if isinstance(shape, numbers.Integral) else tuple(shape)
    def at(ix):
        i = ix if ctype == "Int64" else fromIntegral(ix, ctype)
        return i + constant(first, ctype)
    return Acc(shape, ctype, at=at)


def take(n, a):
    return backpermute((min(int(n), a.shape[0]),), lambda i: (i,), a)


def drop(n, a):
    n = min(int(n), a.shape[0])
    return backpermute((a.shape[0] - n,), lambda i: (i + n,), a)


def init(a):
    return take(a.shape[0] - 1, a)


def tail(a):
    return drop(1, a)


def gather(indices, a):
    """result[i] = a[indices[i]] (backpermute through an index vector)"""
    return Acc(indices.shape, a.ctype, at=lambda ix: a[indices.index(ix)])


def scatter(indices, defaults, a, context=None):
    """defaults overwritten at indices[i] by a[i]; which of several writers to one place wins is unspecified"""
    return permute(lambda new, old: new, defaults, lambda *i: (indices.index(_linear(i, indices.shape)),), a, context)


def foldAll(f, z, a, context=None):
    """reduce every dimension (Prelude's foldAll: a fold over the array seen as a vector)"""
    return fold(f, z, Acc((a.size,), a.ctype, at=lambda ix: a.index(ix)), context)


def _limit(ctype, low):
    if ctype == "float" or ctype == "double":
        return -np.inf if low else np.inf
    info = np.iinfo(NPTYPE[ctype])
    return info.min if low else info.max


def sum_(a, context=None): return foldAll(lambda x, y: x + y, constant(0, a.ctype), a, context)
def product(a, context=None): return foldAll(lambda x, y: x * y, constant(1, a.ctype), a, context)
def maximum(a, context=None): return foldAll(max_, constant(_limit(a.ctype, True), a.ctype), a, context)
def minimum(a, context=None): return foldAll(min_, constant(_limit(a.ctype, False), a.ctype), a, context)
def and_(a, context=None): return foldAll(lambda x, y: x.land(y), constant(1, "Word8"), a, context)
def or_(a, context=None): return foldAll(lambda x, y: x.lor(y), constant(0, "Word8"), a, context)
def all_(p, a, context=None): return and_(map(p, a), context)
def any_(p, a, context=None): return or_(map(p, a), context)


def filter_(p, a, context=None):
    """the elements of a vector that satisfy p, in order, and how many there are: the scan-then-permute
    compaction of the Prelude (an exclusive scan of the flags gives every kept element its place)"""
    cx = _context(context, a)
    a = _force(a, cx)
    flags = map(lambda v: cond(p(v), constant(1, "Int32"), constant(0, "Int32")), a)
    places, count = scanl_(lambda x, y: x + y, 0, flags, context=cx)
    n = int(the(count, cx))
    if n == 0:
        return Acc((0,), a.ctype, at=lambda ix: a.index(ix)), count
    keep = lambda i: index_if(p(a[i]), (places[i],))
    # every kept element has a place of its own, so the combination is never applied: defaults are overwritten
    out = permute(lambda new, old: new, generate((n,), lambda i: a[constant(0, "Int64")]), keep, a, context=cx)
    return out, count


def _awhile_stepwise(cx, p, f, a, tup, force, limit, n):
    """one iteration at a time, the flag read back before every one (as Execute.hs:236-244 does)"""
    while limit is None or n < limit:
        flag = p(*a) if tup else p(a)
        if flag.shape != ():
            raise TypeError("the predicate of awhile yields a scalar array")
        if not the(flag, cx):
            break
        a = force(f(*a) if tup else f(a))
        n += 1
    return a


def awhile(p, f, a, context=None, limit=None, ahead=8):
    """iterate the array function `f` from `a` while the scalar array `p(a)` holds a non-zero value
    (Execute.hs:236-244).  `a` is an Acc or a tuple of them; every iterate is made manifest.

    The reference reads the flag back before every iteration.  Here `ahead` iterations are enqueued at a time, on one
    stream, under a guard in device memory: a one-lane kernel behind each predicate folds its flag into the guard,
    every kernel of the loop looks at the guard and does nothing once it is down, and the host reads the guard --
    whether the loop still runs and how many iterations were taken -- once per batch.  A predicate or body that
    needs a value on the host itself (`the`, `filter_`, a loop of its own) makes the loop fall back to one
    iteration at a time."""
    cx = _context(context, *(a if isinstance(a, tuple) else (a,)))
    tup = isinstance(a, tuple)
    force = lambda v: tuple(_force(x, cx) for x in v) if tup else _force(v, cx)
    a = force(a)
    with cx.lock:
        if cx.loop is not None:
            raise _HostReadInLoop()              # a loop inside a loop: the outer one goes stepwise, this one ahead
        cx.flush()                               # what was put off so far is not the loop's: it runs before, unguarded
        if ahead < 2:
            return _awhile_stepwise(cx, p, f, a, tup, force, limit, 0)
        stream = cx._stream_for([m for x in (a if tup else (a,)) for m in
                                 (x.manifest.comps if isinstance(x.manifest, A.TupleArray) else [x.manifest])])
        if cx.guard is None:
            cx.guard = A.Guard(cx.ctx)
        guard = cx.guard
        guard.attach(stream)
        guard.reset(stream)
        cx.loop = _Loop(stream, guard)
        total, batch, stepwise = 0, [a], False
        try:
            while limit is None or total < limit:
                want = ahead if limit is None else min(ahead, limit - total)
                batch = [a]
                try:
                    for _ in range(want):
                        cur = batch[-1]
                        flag = p(*cur) if tup else p(cur)
                        if flag.shape != ():
                            raise TypeError("the predicate of awhile yields a scalar array")
                        if flag.ctype != "Word8":
                            flag = map(lambda v: v.ne(0), flag)
                        flag = _force(flag, cx)
                        cx.launch([flag.manifest], [], lambda i, o, s: guard.latch(i[0], s))
                        batch.append(force(f(*cur) if tup else f(cur)))
                except _HostReadInLoop:
                    stepwise = True
                alive, count = guard.read(stream)
                # (a batch cut short by the fall-back may have latched an iteration whose body was never enqueued whole)
                taken = min(count - total, len(batch) - 1)
                a = batch[taken]
                total += taken
                if stepwise or not alive:
                    break
        finally:
            cx.loop = None
            guard.detach(stream)
        del batch
        if stepwise:
            return _awhile_stepwise(cx, p, f, a, tup, force, limit, total)
        return a


def run(a, context=None):
    """evaluate and bring the result to the host (CUDA.hs:209-216); a tuple of Acc gives a tuple of results"""
    cx = _context(context, *(a if isinstance(a, tuple) else (a,)))
    with cx.lock:
        if isinstance(a, tuple):
            return tuple(run(x, cx) for x in a)
        return _force(a, cx).manifest.get()


def compute(a, context=None):
    """evaluate on the device without bringing anything to the host: every kernel the value depends on has been
    enqueued when this returns (none has been waited for); gives the manifest array, or a tuple of them"""
    cx = _context(context, *(a if isinstance(a, tuple) else (a,)))
    with cx.lock:
        if isinstance(a, tuple):
            return tuple(compute(x, cx) for x in a)
        m = _force(a, cx)
        for part in _parts([m.manifest]):
            if part.pending is not None:
                part.pending.force()
        return m


def run1(f, context=None):
    """a function from host arrays to host arrays whose kernels are built on the first call and reused afterwards
    (CUDA.hs:318-333: `run1 f` must be partially applied so that the compiled kernels are shared between calls)"""
    cx = context or Context.default()

    def go(*hosts):
        return run(f(*[use(h, cx) for h in hosts]), cx)
    return go


def acond(p, t, e, context=None):
    """array-level conditional: the scalar array `p` is read back and one of the two computations is returned
    (Execute.hs:187); `t` and `e` may be Acc values or functions of no argument, so that only the branch taken
    is built"""
    taken = t if the(p, context) else e
    return taken() if callable(taken) else taken


def reshape(shape, a):
    """the same elements in row-major order under another shape of the same size (Execute.hs:198: no kernel, a
    manifest array keeps its storage; a delayed one is re-indexed)"""
    shape = (shape,) if isinstance(shape, numbers.Integral) else tuple(int(x) for x in shape)
    n = 1
    for x in shape:
        n *= x
    if n != a.size:
        raise ValueError("reshape: %r has %d elements, the array %d" % (shape, n, a.size))
    if a.manifest is not None:
        return Acc(shape, a.ctype, manifest=a.manifest)          # device arrays are addressed linearly
    return Acc(shape, a.ctype, at=a.at)


def flatten(a):
    return reshape((a.size,), a)


All = slice(None)


def replicate(spec, a):
    """`replicate (Z :. 3 :. All) xs`: spec has `All` where a dimension of `a` goes and a number where a new
    dimension of that extent is inserted (fused into the consumer, Execute.hs:216)"""
    spec = tuple(spec)
    if sum(1 for x in spec if x is All or x == All) != len(a.shape):
        raise TypeError("replicate: as many All as the array has dimensions")
    dims = iter(a.shape)
    shape = tuple(next(dims) if (x is All or x == All) else int(x) for x in spec)
    keep = [k for k, x in enumerate(spec) if x is All or x == All]
    return backpermute(shape, lambda *ix: tuple(ix[k] for k in keep), a)


def slice_(a, spec):
    """`slice arr (Z :. 2 :. All)`: spec has `All` for a dimension that stays and an index (a number or an Exp)
    for one that is fixed (Execute.hs:217)"""
    spec = tuple(spec)
    if len(spec) != len(a.shape):
        raise TypeError("slice: one entry per dimension of the array")
    keep = [k for k, x in enumerate(spec) if x is All or (isinstance(x, slice) and x == All)]
    shape = tuple(a.shape[k] for k in keep)

    def at(*ix):
        it = iter(ix)
        return tuple(next(it) if k in keep else spec[k] for k in range(len(spec)))
    return backpermute(shape, at, a)


def imap(f, a):
    """map with the element's multi-index: f(index tuple, value)"""
    t = _probe(lambda v: f(tuple(constant(0, "Int64") for _ in a.shape), v), a.ctype)
    return Acc(a.shape, t, at=lambda ix: Exp.of(f(_unlinear(ix, a.shape), a.index(ix))))


def zipWith3(f, a, b, c):
    return zipWith(lambda xy, z: f(fst(xy), snd(xy), z), zip_(a, b), c)


def iterate(n, f, a):
    """f applied n times (n a host integer)"""
    for _ in range(int(n)):
        a = f(a)
    return a


def runN(f, context=None):
    """`run1` for a function of several arrays (`run1` over the uncurried argument tuple)"""
    return run1(f, context)


def runWith(context, a):
    """`run` in the given context instead of the default one (CUDA.hs:231-234)"""
    return run(a, context)


def run1With(context, f):
    """`run1` in the given context (CUDA.hs:306-309)"""
    return run1(f, context)


def stream(f, arrays, context=None):
    """the array function applied to each of a sequence of inputs, kernels built once; like the lazy list of
    CUDA.hs:338-344 an element is computed when it is asked for"""
    go = run1(f, context)
    for a in arrays:
        yield go(*a) if isinstance(a, tuple) else go(a)


def streamWith(context, f, arrays):
    return stream(f, arrays, context)


def streamOut(computations, context=None):
    """the results of a sequence of array computations as a lazy sequence of host arrays: a computation is built,
    run and collected when its element is asked for, never the whole sequence at once (the `streamOut` of
    CUDA.hs:349-372, which the reference keeps commented out together with its `Seq` execution; here the sequence is
    any iterable of Acc values, or of functions of no argument that build one)"""
    for c in computations:
        yield run(c() if callable(c) else c, context)


def streamOutWith(context, computations):
    return streamOut(computations, context)


class Async(object):
    """A computation running in a host thread of its own (the `Async` of the accelerate package that CUDA.hs:194-196
    re-exports with `wait`, `poll` and `cancel`; started by `asyncBound`, CUDA.hs:263,323).  Threads of one context
    take turns; computations in different contexts overlap."""

    def __init__(self, work):
        self._done, self._cancelled = threading.Event(), False
        self._value, self._error = None, None

        def body():
            _running.asy = self
            try:
                self._value = work()
            except BaseException as e:            # delivered to whoever waits
                self._error = e
            finally:
                self._done.set()
        self._thread = threading.Thread(target=body, daemon=True)
        self._thread.start()


def wait(asy):
    """block until the computation has finished; its result, or the exception that ended it"""
    asy._done.wait()
    if asy._cancelled:
        raise Cancelled()
    if asy._error is not None:
        raise asy._error
    return asy._value


def poll(asy):
    """None while the computation runs, afterwards what `wait` gives"""
    return wait(asy) if asy._done.is_set() else None


def cancel(asy):
    """stop the computation at its next skeleton (kernels already launched finish) and drop its result"""
    asy._cancelled = True
    asy._done.wait()


def runAsync(a, context=None):
    """`run` without waiting for the result (CUDA.hs:246-263)"""
    return Async(lambda: run(a, context))


def runAsyncWith(context, a):
    return runAsync(a, context)


def run1Async(f, context=None):
    """`run1` whose applications return at once (CUDA.hs:312-323)"""
    go = run1(f, context)
    return lambda *hosts: Async(lambda: go(*hosts))


def run1AsyncWith(context, f):
    return run1Async(f, context)


def create(device=0, budget_bytes=0, result_pool_bytes=1 << 30):
    """a new execution context on the given device (Context.hs:73-84); `result_pool_bytes`: how much page-locked host
    memory the context may keep for the results it hands out (0: none, every result in an ordinary array)"""
    return Context(device, budget_bytes, result_pool_bytes)


def destroy(context):
    """release the context's kernels, streams, events and device memory (Context.hs:100-103); arrays and
    computations made in it must not be used afterwards"""
    with context.lock:
        context.flush()
        context.ctx.sync()
        context.skeletons.clear()
        if context.guard is not None:
            context.guard.destroy()
            context.guard = None
        context.streams, context.events = [], []
        context.table.destroy()
        context.results.trim(close=True)
        context.ctx.close()
    if Context._default is context:
        Context._default = None


def unsafeFree(arrays, context=None):
    """give back the device copies of host arrays now instead of when their last `use` is dropped (CUDA.hs:421-432).
    Unsafe as there: a computation that still refers to one of them fails when it looks the array up."""
    cx = context or Context.default()
    with cx.lock:
        cx.flush()                               # launches put off may still want these arrays
        for h in (arrays if isinstance(arrays, (tuple, list)) else (arrays,)):
            cx.table.free(np.asarray(h, order="C"))


def unsafeFreeWith(context, arrays):
    unsafeFree(arrays, context)


def performGC(context=None):
    """return to the device the blocks the memory table keeps for reuse (CUDA.hs:436-441, Array/Remote.hs `cleanup`)"""
    cx = context or Context.default()
    with cx.lock:
        cx.table.reclaim()
    cx.results.trim()


def performGCWith(context):
    performGC(context)
