"""Pure-Python restatement of the collective operations for TINY inputs.

Written independently of oracle/acc_oracle.c (different language, arbitrary
Python callables as operators, list-based) so that a slip in either shows up
as a disagreement.  Definitions follow the same reference comments:
PrefixSum.hs:137-198 (scans), IndexSpace.hs:144-158 (permute),
Reduction.hs:37-55,203-215 (fold), Stencil/Extra.hs:198-226 (boundaries).
"""
from functools import reduce


def scanl(f, z, xs):
    out = [z]
    for x in xs:
        out.append(f(out[-1], x))
    return out


def scanl1(f, xs):
    out = []
    for x in xs:
        out.append(x if not out else f(out[-1], x))
    return out


def scanr(f, z, xs):
    out = [z]
    for x in reversed(xs):
        out.insert(0, f(x, out[0]))
    return out


def scanr1(f, xs):
    out = []
    for x in reversed(xs):
        out.insert(0, x if not out else f(x, out[0]))
    return out


def scanl_p(f, z, xs):
    r = scanl(f, z, xs)
    return r[:-1], r[-1]


def scanr_p(f, z, xs):
    r = scanr(f, z, xs)
    return r[1:], r[0]


def fold_left(f, z, xs):
    """((x0 . x1) . ... . x_{n-1}) . z ; empty -> z"""
    if not xs:
        return z
    return f(reduce(f, xs), z)


def fold_right(f, z, xs):
    """x0 . (x1 . (... (x_{n-1} . z)))"""
    acc = z
    for x in reversed(xs):
        acc = f(x, acc)
    return acc


def fold1_left(f, xs):
    if not xs:
        raise ValueError("empty array")
    return reduce(f, xs)


def foldseg(fold, f, z, xs, offsets):
    return [fold(f, z, xs[offsets[s]:offsets[s + 1]]) for s in range(len(offsets) - 1)]


def permute(f, defaults, dst, src, ignore=-1):
    out = list(defaults)
    for ix, j in enumerate(dst):
        if j == ignore:
            continue
        out[j] = f(src[ix], out[j])
    return out


def bmap(mode, i, sz):
    if mode == "clamp":
        return max(0, min(i, sz - 1))
    if mode == "mirror":
        return -i if i < 0 else (sz - (i - sz + 2) if i >= sz else i)
    if mode == "wrap":
        return sz + i if i < 0 else (i - sz if i >= sz else i)
    raise ValueError(mode)


def stencil2d(fn, img, offsets, mode, constant=0.0):
    """fn receives the list of taps in the order of `offsets` [(dy,dx)...]"""
    h, w = len(img), len(img[0])
    out = [[None] * w for _ in range(h)]
    for y in range(h):
        for x in range(w):
            taps = []
            for dy, dx in offsets:
                yy, xx = y + dy, x + dx
                if mode == "constant":
                    taps.append(img[yy][xx] if 0 <= yy < h and 0 <= xx < w else constant)
                else:
                    taps.append(img[bmap(mode, yy, h)][bmap(mode, xx, w)])
            out[y][x] = fn(taps)
    return out


def tap_arrays_nd(v, taps, mode, constant):
    """for every tap (a tuple of one offset per dimension, outermost first) the array of what that tap reads at
    every element of the numpy array `v`, under the boundary condition (Stencil/Extra.hs:198-226), dimension by
    dimension: index arrays made with `bmap`, one numpy take per dimension"""
    import numpy as np
    out = []
    for off in taps:
        a = v
        inside = np.ones(v.shape, bool)
        for d, o in enumerate(off):
            sz = v.shape[d]
            want = [i + o for i in range(sz)]
            idx = [max(0, min(i, sz - 1)) if mode == "constant" else max(0, min(bmap(mode, i, sz), sz - 1)) for i in want]
            a = np.take(a, idx, axis=d)
            if mode == "constant":
                ok = np.array([0 <= i < sz for i in want])
                shape = [1] * v.ndim
                shape[d] = sz
                inside &= ok.reshape(shape)
        out.append(np.where(inside, a, np.asarray(constant, dtype=v.dtype)) if mode == "constant" else a)
    return out


def affine16(x, y):
    a1, b1, a2, b2 = x >> 16, x & 0xFFFF, y >> 16, y & 0xFFFF
    return (((a1 * a2) & 0xFFFF) << 16) | ((a1 * b2 + b1) & 0xFFFF)


# ---- scalar primitives on fixed-width integers (exact, with Python integers) ---------------
# The definitions are Haskell's (quot/rem truncate, div/mod floor, rotate modulo the width),
# which the reference's generated C reproduces (CodeGen/Arithmetic.hs:90-217).

def wrap(v, bits, signed):
    v &= (1 << bits) - 1
    if signed and v >> (bits - 1):
        v -= 1 << bits
    return v


def quot(x, y):
    q = abs(x) // abs(y)
    return q if (x < 0) == (y < 0) else -q


def rem(x, y):
    return x - y * quot(x, y)


def idiv(x, y):
    return x // y


def imod(x, y):
    return x % y


def signum(x):
    return (x > 0) - (x < 0)


def shift_rl(x, i, bits):
    return (x & ((1 << bits) - 1)) >> i


def rotate_l(x, i, bits):
    u = x & ((1 << bits) - 1)
    k = i % bits
    return ((u << k) | (u >> (bits - k))) & ((1 << bits) - 1) if k else u


# ---- stencil taps as whole arrays (numpy index maps; the boundary rules of Stencil/Extra.hs:191-226) ----

def bmap_np(mode, i, sz):
    import numpy as np
    if mode == "clamp":
        return np.clip(i, 0, sz - 1)
    if mode == "mirror":
        return np.where(i < 0, -i, np.where(i >= sz, sz - (i - sz + 2), i))
    if mode == "wrap":
        return np.where(i < 0, sz + i, np.where(i >= sz, i - sz, i))
    raise ValueError(mode)


def tap_arrays(img, offsets, mode, constant, out_shape):
    """for each (dy, dx): the array, of the result's shape, of the source elements at that offset
    from every result position; the boundary applies at the SOURCE's own edges"""
    import numpy as np
    img = np.asarray(img)
    if img.ndim == 1:
        img = img[None, :]
        out_shape = (1, out_shape[-1])
    h, w = img.shape
    ys, xs = np.arange(out_shape[0])[:, None], np.arange(out_shape[1])[None, :]
    taps = []
    for dy, dx in offsets:
        yy, xx = ys + dy, xs + dx
        if mode == "constant":
            inside = (yy >= 0) & (yy < h) & (xx >= 0) & (xx < w)
            v = np.where(inside, img[np.clip(yy, 0, h - 1), np.clip(xx, 0, w - 1)], np.asarray(constant, img.dtype))
        else:
            v = img[bmap_np(mode, yy, h), bmap_np(mode, xx, w)]
        taps.append(v)
    return taps


def tap_arrays3(vol, offsets, mode, constant, out_shape):
    """tap_arrays for a rank-3 source and offsets (dz, dy, dx)"""
    import numpy as np
    vol = np.asarray(vol)
    d, h, w = vol.shape
    zs = np.arange(out_shape[0])[:, None, None]
    ys = np.arange(out_shape[1])[None, :, None]
    xs = np.arange(out_shape[2])[None, None, :]
    taps = []
    for dz, dy, dx in offsets:
        zz, yy, xx = zs + dz, ys + dy, xs + dx
        if mode == "constant":
            inside = (zz >= 0) & (zz < d) & (yy >= 0) & (yy < h) & (xx >= 0) & (xx < w)
            v = np.where(inside, vol[np.clip(zz, 0, d - 1), np.clip(yy, 0, h - 1), np.clip(xx, 0, w - 1)],
                         np.asarray(constant, vol.dtype))
        else:
            v = vol[bmap_np(mode, zz, d), bmap_np(mode, yy, h), bmap_np(mode, xx, w)]
        taps.append(v)
    return taps
