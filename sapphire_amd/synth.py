"""Seeded synthetic inputs for the five benchmark configurations.

Every value is a pure function of (seed, element index): a SplitMix64 finaliser
over a counter, so a tensor is identical on any machine, in any chunking, for
the CPU checker and for the GPU run.  No std/numpy distribution objects are
involved (their sequences are implementation-defined; the reference itself
seeds from random_device, Sources/Sapphire/compute/dense/naive/NaiveInitialize.cpp:15-16).

Seeds: BASE_SEED + configuration number, plus a sub-stream per tensor.
"""
import numpy as np

BASE_SEED = 0x5A990000
STREAM_A = 0x100
STREAM_B = 0x200
STREAM_C = 0x300
STREAM_W = 0x400   # + layer index
STREAM_BIAS = 0x500
STREAM_NNZ = 0x600
STREAM_COL = 0x700

_GOLDEN = np.uint64(0x9E3779B97F4A7C15)
_M1 = np.uint64(0xBF58476D1CE4E5B9)
_M2 = np.uint64(0x94D049BB133111EB)


def _mix(z):
    z = (z ^ (z >> np.uint64(30))) * _M1
    z = (z ^ (z >> np.uint64(27))) * _M2
    return z ^ (z >> np.uint64(31))


def bits64(seed, count, start=0):
    """count 64-bit words; word i depends only on (seed, start + i)."""
    with np.errstate(over="ignore"):
        idx = np.arange(start + 1, start + count + 1, dtype=np.uint64)
        base = _mix(np.uint64(seed) * _GOLDEN + np.uint64(0x1234567))
        return _mix(base + idx * _GOLDEN)


def uniform01(seed, count, start=0):
    """float32 in [0, 1) with 24 random mantissa bits (exactly representable)."""
    top = (bits64(seed, count, start) >> np.uint64(40)).astype(np.float32)
    return top * np.float32(1.0 / (1 << 24))


def uniform(seed, shape, lo=-1.0, hi=1.0):
    """float32 uniform in [lo, hi); for (-1, 1) every value is k / 2^23 exactly."""
    count = int(np.prod(shape))
    u = uniform01(seed, count)
    out = (u * np.float32(hi - lo) + np.float32(lo)).astype(np.float32)
    return out.reshape(shape)


def normal(seed, shape, sigma=1.0):
    """N(0, sigma) by Box-Muller in float64 on two counter streams, rounded to float32."""
    count = int(np.prod(shape))
    w1 = bits64(seed, count)
    w2 = bits64(seed ^ 0x5DEECE66D, count)
    u1 = ((w1 >> np.uint64(11)).astype(np.float64) + 1.0) * (1.0 / (1 << 53))  # (0, 1]
    u2 = (w2 >> np.uint64(11)).astype(np.float64) * (1.0 / (1 << 53))           # [0, 1)
    z = np.sqrt(-2.0 * np.log(u1)) * np.cos(2.0 * np.pi * u2)
    return (z * sigma).astype(np.float32).reshape(shape)


def small_integers(seed, shape, span=4):
    """float32 integers in [-span, span]: products and sums stay exact in fp16/fp32."""
    count = int(np.prod(shape))
    v = (bits64(seed, count) >> np.uint64(33)) % np.uint64(2 * span + 1)
    return (v.astype(np.int64) - span).astype(np.float32).reshape(shape)


def config_seed(config):
    return BASE_SEED + int(config)


# ---- the five configurations ------------------------------------------------

def config1():
    s = config_seed(1)
    return {"A": uniform(s + STREAM_A, (256, 256)), "B": uniform(s + STREAM_B, (256, 256)),
            "C": uniform(s + STREAM_C, (256, 256))}


def config2(batch=16, n=512):
    s = config_seed(2)
    return {"A": uniform(s + STREAM_A, (batch, n, n)), "B": uniform(s + STREAM_B, (1, n, n)),
            "C": uniform(s + STREAM_C, (batch, n, n))}


def config3(n=4096):
    """fp16 A, B ~ N(0, 1/sqrt(K)) rounded to nearest fp16; C zeros."""
    s = config_seed(3)
    sigma = 1.0 / np.sqrt(n)
    return {"A": normal(s + STREAM_A, (n, n), sigma).astype(np.float16),
            "B": normal(s + STREAM_B, (n, n), sigma).astype(np.float16),
            "C": np.zeros((n, n), dtype=np.float32)}


def config4(batch=1024, sizes=(784, 1024, 1024, 10)):
    """x U[0,1); W Xavier-uniform U(+-sqrt(6/(in+out))) stored [in, out]; b U[-0.1, 0.1)."""
    s = config_seed(4)
    out = {"x": uniform(s + STREAM_A, (batch, sizes[0]), 0.0, 1.0), "W": [], "b": []}
    for layer in range(len(sizes) - 1):
        fan_in, fan_out = sizes[layer], sizes[layer + 1]
        bound = float(np.sqrt(6.0 / (fan_in + fan_out)))
        out["W"].append(uniform(s + STREAM_W + layer, (fan_in, fan_out), -bound, bound))
        out["b"].append(uniform(s + STREAM_BIAS + layer, (fan_out,), -0.1, 0.1))
    return out


def _poisson_counts(seed, rows, mean, cap):
    """Inverse-CDF Poisson(mean) per row from one uniform each, clipped to [0, cap]."""
    ks = np.arange(0, cap + 1, dtype=np.float64)
    log_fact = np.concatenate([[0.0], np.cumsum(np.log(np.arange(1, cap + 1, dtype=np.float64)))])
    pmf = np.exp(ks * np.log(mean) - mean - log_fact)
    cdf = np.cumsum(pmf)
    u = (bits64(seed, rows) >> np.uint64(11)).astype(np.float64) * (1.0 / (1 << 53))
    return np.minimum(np.searchsorted(cdf, u, side="right"), cap).astype(np.int64)


def _row_columns(seed, row, count, ncols):
    """`count` distinct columns of a row: first distinct draws of a counter stream, sorted."""
    if count == 0:
        return np.empty(0, dtype=np.uint32)
    need = count
    draws = 2 * count + 16
    row_seed = (seed + 0x9E37 * (row + 1)) & 0xFFFFFFFFFFFF
    while True:
        cand = (bits64(row_seed, draws) % np.uint64(ncols)).astype(np.int64)
        _, first = np.unique(cand, return_index=True)
        if len(first) >= need:
            keep = np.sort(first)[:need]
            return np.sort(cand[keep]).astype(np.uint32)
        draws *= 2


def csr_matrix(seed, rows, cols, mean_nnz, forced=None, cap=1024):
    """CSR arrays (V fp32, COL uint32 ascending per row, ROW uint32 with rows+1 offsets).

    forced: {row: nnz} overrides the Poisson draw (e.g. an empty row, a full-length row);
    {row: ('cols', [..])} forces explicit columns.
    """
    counts = _poisson_counts(seed + STREAM_NNZ, rows, mean_nnz, min(cap, cols))
    explicit = {}
    for r, spec in (forced or {}).items():
        if isinstance(spec, tuple):
            explicit[r] = np.array(sorted(spec[1]), dtype=np.uint32)
            counts[r] = len(explicit[r])
        else:
            counts[r] = int(spec)
    row_off = np.zeros(rows + 1, dtype=np.uint32)
    np.cumsum(counts, out=row_off[1:])
    nnz = int(row_off[-1])
    col = np.empty(nnz, dtype=np.uint32)
    for r in range(rows):
        if counts[r]:
            col[row_off[r]:row_off[r + 1]] = explicit[r] if r in explicit else \
                _row_columns(seed + STREAM_COL, r, int(counts[r]), cols)
    val = uniform(seed + STREAM_A, (nnz,)) if nnz else np.empty(0, dtype=np.float32)
    return val, col, row_off


def config5(m=8192, k=8192, n=256, density=0.01, forced=None):
    s = config_seed(5)
    v, col, row = csr_matrix(s, m, k, density * k, forced=forced)
    return {"V": v, "COL": col, "ROW": row, "B": uniform(s + STREAM_B, (k, n)),
            "C": np.zeros((m, n), dtype=np.float32), "M": m, "K": k, "N": n}


def densify(v, col, row, m, k):
    dense = np.zeros((m, k), dtype=np.float32)
    for r in range(m):
        dense[r, col[row[r]:row[r + 1]]] = v[row[r]:row[r + 1]]
    return dense
