"""CSR x dense through the C ABI: bit-exact against the CPU checker.

Each output element is summed by one lane in storage order with separately rounded products
and sums, so values (not only structure) must match the oracle bit for bit.  Structure: rows
without entries are exactly zero (store mode) or untouched (accumulate mode), and nothing is
written outside out (guard values on both sides).
"""
import numpy as np
import pytest

from oracle import pyoracle as po
from sapphire_amd import capi, synth
from tests import helpers as h

pytestmark = pytest.mark.gpu


def _bits(x):
    return np.ascontiguousarray(x).view(np.uint32)


def test_config5_full_size_bit_exact(dev):
    forced = {0: 0, 1: 1, 2: 1024, 3: ("cols", [0, 8191]), 8191: 0}
    h.announce("sph_spmm_csr_f32 config5 8192x8192 1% x 8192x256 with forced rows")
    d = synth.config5(forced=forced)
    M, K, N = d["M"], d["K"], d["N"]
    row = d["ROW"]
    assert row[1] - row[0] == 0 and row[2] - row[1] == 1 and row[3] - row[2] == 1024
    assert 600000 < d["V"].size < 750000
    ref = po.spmm_csr(np.zeros((M, N), np.float32), d["V"], d["COL"], row, M, N, d["B"], threads=8)
    got = h.gpu_spmm(np.full((M, N), 7.0, np.float32), d["V"], d["COL"], row, M, K, N, d["B"],
                     accumulate=False, canary=4096)
    assert np.array_equal(_bits(got), _bits(ref))
    assert not got[0].any() and not got[8191].any()
    # accumulate mode adds into what is there
    C = synth.uniform(5, (M, N))
    ref2 = po.spmm_csr(C.copy(), d["V"], d["COL"], row, M, N, d["B"], threads=8)
    got2 = h.gpu_spmm(C, d["V"], d["COL"], row, M, K, N, d["B"], accumulate=True, canary=4096)
    assert np.array_equal(_bits(got2), _bits(ref2))
    assert np.array_equal(got2[0], C[0])


@pytest.mark.parametrize("N", [1, 3, 4, 10, 64, 100, 256, 260, 512, 1000])
def test_ragged_dense_widths(dev, N):
    h.announce("sph_spmm_csr_f32 N =", N)
    M, K = 300, 777
    v, col, row = synth.csr_matrix(900 + N, M, K, 20.0, forced={5: 0, 6: 700, 7: ("cols", [776])})
    B = synth.uniform(901 + N, (K, N))
    ref = po.spmm_csr(np.zeros((M, N), np.float32), v, col, row, M, N, B)
    got = h.gpu_spmm(np.ones((M, N), np.float32), v, col, row, M, K, N, B, False, canary=512)
    assert np.array_equal(_bits(got), _bits(ref))


def test_equals_dense_product_of_densified_matrix(dev):
    """Size-independent property: the sparse product equals the dense fp32 leaf applied to the
    densified matrix (adding the 0*b terms leaves every running sum unchanged)."""
    h.announce("sph_spmm_csr_f32 vs densified dense oracle")
    M, K, N = 128, 512, 64
    v, col, row = synth.csr_matrix(77, M, K, 12.0)
    B = synth.uniform(78, (K, N))
    dense = synth.densify(v, col, row, M, K)
    ref = po.naive_gemm(np.zeros((M, N), np.float32), dense, B, M, N, K)
    got = h.gpu_spmm(np.zeros((M, N), np.float32), v, col, row, M, K, N, B, False, canary=64)
    assert np.array_equal(_bits(got), _bits(ref))


def test_all_rows_empty(dev):
    M, K, N = 10, 10, 8
    row = np.zeros(M + 1, np.uint32)
    got = h.gpu_spmm(np.ones((M, N), np.float32), np.empty(0, np.float32),
                     np.empty(0, np.uint32), row, M, K, N, synth.uniform(1, (K, N)), False, 16)
    assert not got.any()


# ---- SPH_SPMM_FAST: values within rounding, structure exact -------------------------------
TOL_FAST = 1e-4


def _normalised(got, ref, V, COL, ROW, M, N, B):
    """max |got - ref| / sum_p |V[p] * B[COL[p]][n]| over the elements that have entries."""
    den = po.spmm_csr(np.zeros((M, N), np.float32), np.abs(V), COL, ROW, M, N, np.abs(B), threads=8)
    has = den > 0
    assert np.array_equal(got[~has], ref[~has])          # elements without entries: exact
    return float(np.max(np.abs(got[has].astype(np.float64) - ref[has]) / den[has])) if has.any() else 0.0


def test_fast_config5_full_size(dev):
    """The LDS-resident slab kernel at configuration 5's size: values within 1e-4 of the
    storage-order sum (normalised by the sum of the absolute products), rows without entries
    exactly zero, a 1024-entry row (more than is fetched ahead), guards intact, both modes."""
    forced = {0: 0, 1: 1, 2: 1024, 3: ("cols", [0, 8191]), 8191: 0, 4: 97, 5: 96, 6: 17}
    h.announce("sph_spmm_csr_f32_ex FAST config5 8192x8192 1% x 8192x256 with forced rows")
    d = synth.config5(forced=forced)
    M, K, N = d["M"], d["K"], d["N"]
    row = d["ROW"]
    ref = po.spmm_csr(np.zeros((M, N), np.float32), d["V"], d["COL"], row, M, N, d["B"], threads=8)
    got = h.gpu_spmm(np.full((M, N), 7.0, np.float32), d["V"], d["COL"], row, M, K, N, d["B"],
                     accumulate=False, canary=4096, fast=True)
    assert np.isfinite(got).all()
    err = _normalised(got, ref, d["V"], d["COL"], row, M, N, d["B"])
    assert err <= TOL_FAST, err
    assert not got[0].any() and not got[8191].any()
    # a row with a single entry is one product: exact
    assert np.array_equal(_bits(got[1]), _bits(ref[1]))
    C = synth.uniform(5, (M, N))
    ref2 = po.spmm_csr(C.copy(), d["V"], d["COL"], row, M, N, d["B"], threads=8)
    got2 = h.gpu_spmm(C, d["V"], d["COL"], row, M, K, N, d["B"], accumulate=True, canary=4096,
                      fast=True)
    den = po.spmm_csr(np.abs(C), np.abs(d["V"]), d["COL"], row, M, N, np.abs(d["B"]), threads=8)
    assert float(np.max(np.abs(got2.astype(np.float64) - ref2) / np.maximum(den, 1e-30))) <= TOL_FAST
    assert np.array_equal(got2[0], C[0]) and np.array_equal(got2[8191], C[8191])


# K not a multiple of 64, several row partitions per slab, widths from the first that takes
# the slab kernel (64) up, rows longer than the 96 entries fetched ahead, M not a multiple of 4
@pytest.mark.parametrize("shape", [(300, 777, 64), (1000, 1000, 100), (4099, 5000, 256),
                                   (37, 10000, 128), (2048, 64, 512), (513, 4096, 68)])
def test_fast_shapes(dev, shape):
    M, K, N = shape
    h.announce("sph_spmm_csr_f32_ex FAST M K N =", shape)
    per_row = min(40.0, K / 3)
    forced = {2: 0, 3: min(K, 700), 4: ("cols", [K - 1]), M - 1: min(K, 130)}
    v, col, row = synth.csr_matrix(3000 + M + N, M, K, per_row, forced=forced)
    B = synth.uniform(3001 + N, (K, N))
    for accumulate in (False, True):
        C = synth.uniform(3002, (M, N))
        ref = po.spmm_csr(C.copy() if accumulate else np.zeros((M, N), np.float32), v, col, row, M, N, B)
        got = h.gpu_spmm(C, v, col, row, M, K, N, B, accumulate, canary=512, fast=True)
        den = po.spmm_csr(np.abs(C) if accumulate else np.zeros((M, N), np.float32), np.abs(v), col,
                          row, M, N, np.abs(B))
        bad = np.abs(got.astype(np.float64) - ref) > TOL_FAST * den
        assert not bad.any(), (int(bad.sum()), accumulate)
        assert np.array_equal(got[2], C[2] if accumulate else np.zeros(N, np.float32))


@pytest.mark.parametrize("N", [1, 10, 32, 60])
def test_fast_falls_back_to_exact_kernels(dev, N):
    """Widths the slab kernel does not take run the exact kernels: same bits as without the flag."""
    M, K = 300, 777
    v, col, row = synth.csr_matrix(950 + N, M, K, 20.0)
    B = synth.uniform(951 + N, (K, N))
    ref = po.spmm_csr(np.zeros((M, N), np.float32), v, col, row, M, N, B)
    got = h.gpu_spmm(np.ones((M, N), np.float32), v, col, row, M, K, N, B, False, canary=64, fast=True)
    assert np.array_equal(_bits(got), _bits(ref))


def test_fast_integer_exact(dev):
    """Integer-valued operands make every product and partial sum exact whatever the
    association: the slab kernel must then agree bit for bit (indexing check)."""
    M, K, N = 2000, 8192, 256
    v, col, row = synth.csr_matrix(4100, M, K, 82.0, forced={7: 1024})
    v = np.round(v * 4).astype(np.float32)
    B = synth.small_integers(4101, (K, N))
    ref = po.spmm_csr(np.zeros((M, N), np.float32), v, col, row, M, N, B, threads=8)
    got = h.gpu_spmm(np.ones((M, N), np.float32), v, col, row, M, K, N, B, False, canary=256, fast=True)
    assert np.array_equal(got, ref)


@pytest.mark.parametrize("entries", [1, 2, 3])
def test_fast_tiny_entry_counts(dev, entries):
    """One, two and three entries in the whole matrix, the last one in the last row (the slab
    kernel reads entries in pairs and must not touch anything past the arrays)."""
    M, K, N = 70, 200, 64
    counts = np.zeros(M, np.uint32)
    counts[M - 1] = 1
    if entries > 1:
        counts[3] = entries - 1
    row = np.concatenate([[0], np.cumsum(counts)]).astype(np.uint32)
    col = np.array([5, 199, 7][:entries][::-1] if entries > 1 else [199], np.uint32)
    col = np.concatenate([np.sort(col[:entries - 1]), col[entries - 1:]]).astype(np.uint32)
    v = synth.uniform(77, (entries,))
    B = synth.uniform(78, (K, N))
    ref = po.spmm_csr(np.zeros((M, N), np.float32), v, col, row, M, N, B)
    got = h.gpu_spmm(np.ones((M, N), np.float32), v, col, row, M, K, N, B, False, canary=64, fast=True)
    assert np.allclose(got, ref, rtol=1e-6, atol=1e-7)
    assert not got[0].any()
