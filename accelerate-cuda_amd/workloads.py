"""Seeded synthetic inputs for the five benchmark configurations.

Every array is a pure function of (seed, index): a SplitMix64 counter-based
generator evaluated with numpy, so the CPU checker and the GPU run see the
same bits, and any slice can be regenerated without the rest.

    r(seed, i) = mix64(seed + (i + 1) * 0x9E3779B97F4A7C15)     (mod 2^64)

    Float32 uniform [-1,1):  k = r >> 40 (24 bits);  value = (2k - 2^24) / 2^24   (exact)
    Float32 uniform [0,1) :  value = k / 2^24                                      (exact)
    Int32 uniform [0,m)   :  (r >> 32) mod m
    Zipf(s) over ranks 1..N:  inverse-CDF table + binary search on u = (r >> 11) / 2^53;
                              rank k maps to bin k-1 (bin 0 is the hottest, no extra shuffle)
    Poisson(mean)         :  inversion: table of the CDF + binary search on the same u
"""
import numpy as np

GOLDEN = np.uint64(0x9E3779B97F4A7C15)

SEED_DOT_X = 0xACC00001
SEED_DOT_Y = 0xACC00002
SEED_SCAN = 0xACC00003
SEED_HIST_UNIFORM = 0xACC00004
SEED_HIST_ZIPF = 0xACC00005
SEED_STENCIL = 0xACC00006
SEED_SMVM_LEN = 0xACC00007
SEED_SMVM_COL = 0xACC00008
SEED_SMVM_VAL = 0xACC00009
SEED_SMVM_X = 0xACC0000A


def splitmix64(seed, n, start=0):
    """r(seed, start) .. r(seed, start + n - 1) as uint64."""
    with np.errstate(over="ignore"):
        i = np.arange(start + 1, start + n + 1, dtype=np.uint64)
        z = np.uint64(seed) + i * GOLDEN
        z = (z ^ (z >> np.uint64(30))) * np.uint64(0xBF58476D1CE4E5B9)
        z = (z ^ (z >> np.uint64(27))) * np.uint64(0x94D049BB133111EB)
        z = z ^ (z >> np.uint64(31))
    return z


def _chunks(n, step=1 << 22):
    s = 0
    while s < n:
        yield s, min(step, n - s)
        s += step


def uniform_pm1_f32(seed, n):
    out = np.empty(n, dtype=np.float32)
    for s, m in _chunks(n):
        k = (splitmix64(seed, m, s) >> np.uint64(40)).astype(np.int64)
        out[s:s + m] = ((2 * k - (1 << 24)).astype(np.float64) / float(1 << 24)).astype(np.float32)
    return out


def uniform_01_f32(seed, n):
    out = np.empty(n, dtype=np.float32)
    for s, m in _chunks(n):
        k = (splitmix64(seed, m, s) >> np.uint64(40)).astype(np.float64)
        out[s:s + m] = (k / float(1 << 24)).astype(np.float32)
    return out


def uniform_i32(seed, n, m):
    out = np.empty(n, dtype=np.int32)
    for s, c in _chunks(n):
        out[s:s + c] = ((splitmix64(seed, c, s) >> np.uint64(32)) % np.uint64(m)).astype(np.int32)
    return out


def _u53(seed, n, start):
    return (splitmix64(seed, n, start) >> np.uint64(11)).astype(np.float64) / float(1 << 53)


def zipf_i32(seed, n, nbins, s=1.1):
    ranks = np.arange(1, nbins + 1, dtype=np.float64)
    w = ranks ** (-s)
    cdf = np.cumsum(w)
    cdf /= cdf[-1]
    out = np.empty(n, dtype=np.int32)
    for st, c in _chunks(n):
        u = _u53(seed, c, st)
        out[st:st + c] = np.minimum(np.searchsorted(cdf, u, side="right"), nbins - 1).astype(np.int32)
    return out


def poisson_i32(seed, n, mean):
    kmax = int(mean + 12 * np.sqrt(mean) + 16)
    pmf = np.empty(kmax + 1, dtype=np.float64)
    pmf[0] = np.exp(-mean)
    for k in range(1, kmax + 1):
        pmf[k] = pmf[k - 1] * mean / k
    cdf = np.cumsum(pmf)
    out = np.empty(n, dtype=np.int32)
    for st, c in _chunks(n):
        u = _u53(seed, c, st)
        out[st:st + c] = np.minimum(np.searchsorted(cdf, u, side="right"), kmax).astype(np.int32)
    return out


# ---------------------------------------------------------------------------
# the five configurations

def dot_inputs(n=1 << 24):
    return uniform_pm1_f32(SEED_DOT_X, n), uniform_pm1_f32(SEED_DOT_Y, n)


def scan_input(n=1 << 26):
    return uniform_i32(SEED_SCAN, n, 16)


def hist_uniform_keys(n=1 << 26, nbins=256):
    return uniform_i32(SEED_HIST_UNIFORM, n, nbins)


def hist_zipf_keys(n=1 << 26, nbins=65536, s=1.1):
    return zipf_i32(SEED_HIST_ZIPF, n, nbins, s)


def stencil_image(h=8192, w=8192):
    return uniform_01_f32(SEED_STENCIL, h * w).reshape(h, w)


def smvm_inputs(nrows=1 << 20, mean_len=32, ncols=None):
    """CSR matrix (vals, cols, offsets, lengths) and dense vector x."""
    if ncols is None:
        ncols = nrows
    lengths = poisson_i32(SEED_SMVM_LEN, nrows, mean_len)
    offsets = np.zeros(nrows + 1, dtype=np.int64)
    np.cumsum(lengths, out=offsets[1:])
    nnz = int(offsets[-1])
    assert nnz < (1 << 31)
    cols = uniform_i32(SEED_SMVM_COL, nnz, ncols)
    vals = uniform_pm1_f32(SEED_SMVM_VAL, nnz)
    x = uniform_pm1_f32(SEED_SMVM_X, ncols)
    return vals, cols, offsets.astype(np.int32), lengths, x
