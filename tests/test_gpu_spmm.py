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


@pytest.mark.parametrize("N", [1, 3, 4, 5, 7, 10, 33, 64, 65, 67, 100, 255, 256, 260, 512, 1000, 1001])
def test_ragged_dense_widths(dev, N):
    h.announce("sph_spmm_csr_f32 N =", N)
    M, K = 300, 777
    v, col, row = synth.csr_matrix(900 + N, M, K, 20.0, forced={5: 0, 6: 700, 7: ("cols", [776])})
    B = synth.uniform(901 + N, (K, N))
    ref = po.spmm_csr(np.zeros((M, N), np.float32), v, col, row, M, N, B)
    got = h.gpu_spmm(np.ones((M, N), np.float32), v, col, row, M, K, N, B, False, canary=512)
    assert np.array_equal(_bits(got), _bits(ref))
    # and added to what out holds
    C = synth.uniform(902 + N, (M, N))
    ref = po.spmm_csr(C.copy(), v, col, row, M, N, B)
    got = h.gpu_spmm(C, v, col, row, M, K, N, B, True, canary=512)
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


@pytest.mark.parametrize("N", [1, 3, 6, 64, 65, 100, 255, 256])
def test_row_bias_form_equals_fill_bias_product_and_accumulate(dev, N):
    """sph_spmm_csr_bias_f32 against the CPU checker run the long way: out = 0, out += bias x
    ones (the K = 1 product of Linear's bias step, feature-major), out += A * B.  Rows without
    entries hold 0 + bias, a bias of -0 becomes +0, out's old contents (NaN) are not read."""
    h.announce("sph_spmm_csr_bias_f32 N =", N)
    M, K = 300, 777
    v, col, row = synth.csr_matrix(950 + N, M, K, 20.0, forced={5: 0, 6: 700, 7: ("cols", [776])})
    B = synth.uniform(951 + N, (K, N))
    bias = synth.uniform(952 + N, (M,))
    bias[5] = -0.0
    start = po.naive_gemm(np.zeros((M, N), np.float32), bias.reshape(M, 1).copy(),
                          np.ones((1, N), np.float32), M, N, 1)
    ref = po.spmm_csr(start, v, col, row, M, N, B)
    got = h.gpu_spmm_bias(np.full((M, N), np.float32(np.nan)), v, col, row, M, K, N, B, bias,
                          canary=512)
    assert np.array_equal(_bits(got), _bits(ref))
    assert np.array_equal(_bits(got[5]), _bits(np.zeros(N, np.float32)))     # 0 + (-0) = +0


def test_all_rows_empty(dev):
    M, K, N = 10, 10, 8
    row = np.zeros(M + 1, np.uint32)
    got = h.gpu_spmm(np.ones((M, N), np.float32), np.empty(0, np.float32),
                     np.empty(0, np.uint32), row, M, K, N, synth.uniform(1, (K, N)), False, 16)
    assert not got.any()

