"""CSR x CSR -> CSR on the device (C ABI and the C++ layer), bit-exact against the CPU checker."""
import ctypes

import numpy as np
import pytest

from oracle import pyoracle as po
from sapphire_amd import capi, synth
from tests import helpers as h
from tests import host_layer as hl

pytestmark = pytest.mark.gpu


def bits(x):
    return np.ascontiguousarray(x).view(np.uint32)


def sparse_dense(seed, shape, density):
    vals = synth.uniform(seed, shape)
    keep = synth.uniform(seed + 1, shape, 0.0, 1.0) < density
    return np.where(keep, vals, np.float32(0)).astype(np.float32)


def _dev(a, dtype):
    return capi.DeviceBuffer.from_array(a if a.size else np.zeros(1, dtype))


def gpu_spgemm(A, B, M, K, N):
    VA, CA, RA = A
    VB, CB, RB = B
    bufs = [_dev(VA, np.float32), _dev(CA, np.uint32), _dev(RA, np.uint32),
            _dev(VB, np.float32), _dev(CB, np.uint32), _dev(RB, np.uint32)]
    dRow = capi.DeviceBuffer(4 * (M + 1))
    nnz = ctypes.c_uint32(0xDEADBEEF)
    capi.call("sph_spgemm_row_offsets_f32", dRow.ptr, *[b.ptr for b in bufs], M, K, N,
              ctypes.byref(nnz))
    ROW = dRow.download(np.uint32, (M + 1,))
    assert ROW[M] == nnz.value
    guard = 4
    dV = capi.DeviceBuffer.from_array(np.full(nnz.value + guard, -77.0, np.float32))
    dCol = capi.DeviceBuffer.from_array(np.full(nnz.value + guard, 0xABCDEF, np.uint32))
    capi.call("sph_spgemm_fill_f32", dV.ptr, dCol.ptr, dRow.ptr, *[b.ptr for b in bufs], M, K, N)
    V = dV.download(np.float32, (nnz.value + guard,))
    COL = dCol.download(np.uint32, (nnz.value + guard,))
    assert np.all(V[nnz.value:] == -77.0) and np.all(COL[nnz.value:] == 0xABCDEF)
    for d in bufs + [dRow, dV, dCol]:
        d.release()
    return V[:nnz.value], COL[:nnz.value], ROW


def gpu_spgemm_one_call(A, B, M, K, N, capacity):
    """(V, COL, ROW, nnz) through sph_spgemm_f32 with room for `capacity` entries; the words past
    the capacity must come back untouched."""
    VA, CA, RA = A
    VB, CB, RB = B
    bufs = [_dev(VA, np.float32), _dev(CA, np.uint32), _dev(RA, np.uint32),
            _dev(VB, np.float32), _dev(CB, np.uint32), _dev(RB, np.uint32)]
    dRow = capi.DeviceBuffer.from_array(np.full(M + 1, 0xFFFFFFFF, np.uint32))
    guard = 8
    dV = capi.DeviceBuffer.from_array(np.full(capacity + guard, -77.0, np.float32))
    dCol = capi.DeviceBuffer.from_array(np.full(capacity + guard, 0xABCDEF, np.uint32))
    nnz = ctypes.c_uint32(0xDEADBEEF)
    capi.call("sph_spgemm_f32", dV.ptr, dCol.ptr, dRow.ptr, capacity, *[b.ptr for b in bufs],
              M, K, N, ctypes.byref(nnz))
    ROW = dRow.download(np.uint32, (M + 1,))
    V = dV.download(np.float32, (capacity + guard,))
    COL = dCol.download(np.uint32, (capacity + guard,))
    assert np.all(V[capacity:] == -77.0) and np.all(COL[capacity:] == 0xABCDEF)
    for d in bufs + [dRow, dV, dCol]:
        d.release()
    return V[:capacity], COL[:capacity], ROW, nnz.value


def check_one_call(A, B, M, K, N, want):
    """sph_spgemm_f32 against the result of the two calls: with room to spare, exactly enough,
    half of it (then the first half of the entries), and so little that the staging slots of
    the longer rows overflow and those rows are multiplied a second time."""
    wV, wC, wR = want
    total = int(wR[M])
    for capacity in (total + 3, total, total // 2, min(total, M)):
        V, COL, ROW, nnz = gpu_spgemm_one_call(A, B, M, K, N, capacity)
        assert nnz == total and np.array_equal(ROW, wR), capacity
        kept = min(capacity, total)
        assert np.array_equal(COL[:kept], wC[:kept]), capacity
        assert np.array_equal(bits(V[:kept]), bits(wV[:kept])), capacity
        if capacity > total:
            assert np.all(V[total:] == -77.0)


# M, K, N, density of A, density of B: single entries, rows of A and of B longer than 64
# entries, empty operands, a width that needs two strips, widths that are not multiples of 64
CASES = [(1, 1, 1, 1.0, 1.0), (5, 7, 3, 0.5, 0.5), (40, 60, 33, 0.1, 0.2), (64, 300, 200, 0.05, 0.05),
         (30, 200, 70, 1.0, 0.3), (20, 50, 700, 0.3, 0.5), (25, 25, 25, 0.0, 0.5),
         (25, 25, 25, 0.5, 0.0), (300, 400, 9000, 0.02, 0.01), (2000, 2000, 2000, 0.004, 0.004)]


@pytest.mark.parametrize("case", CASES)
def test_product_matches_checker(dev, case):
    M, K, N, da, db = case
    h.announce("sph_spgemm_* M K N dA dB =", case)
    dA = sparse_dense(3000 + M, (M, K), da)
    dB = sparse_dense(4000 + N, (K, N), db)
    A, B = po.csr_from_dense(dA), po.csr_from_dense(dB)
    wV, wC, wR = po.spgemm_csr(A, B, M, K, N)
    V, COL, ROW = gpu_spgemm(A, B, M, K, N)
    assert np.array_equal(ROW, wR)
    assert np.array_equal(COL, wC)
    assert np.array_equal(bits(V), bits(wV))
    check_one_call(A, B, M, K, N, (wV, wC, wR))


def test_cancelling_sums_are_dropped_and_unsorted_b_rows_are_accepted(dev):
    h.announce("sph_spgemm_* cancellation / unsorted rows of B")
    A = (np.array([1, -1, 3], np.float32), np.array([0, 1, 2], np.uint32),
         np.array([0, 2, 3], np.uint32))
    B = (np.array([2, 5, 2, 7, 4], np.float32), np.array([1, 3, 1, 0, 2], np.uint32),
         np.array([0, 2, 4, 5], np.uint32))
    V, COL, ROW = gpu_spgemm(A, B, 2, 3, 4)
    assert ROW.tolist() == [0, 2, 3] and COL.tolist() == [0, 3, 2]
    assert V.tolist() == [-7.0, 5.0, 12.0]


def test_equals_dense_product_of_the_densified_operands(dev):
    """Against the dense path of this library's own checker: densify, dense leaf, back to CSR."""
    M, K, N = 96, 128, 80
    h.announce("sph_spgemm_* against densify + dense leaf", (M, K, N))
    dA = sparse_dense(5000, (M, K), 0.08)
    dB = sparse_dense(5002, (K, N), 0.08)
    dense = po.naive_gemm(np.zeros((M, N), np.float32), dA, dB, M, N, K)
    wV, wC, wR = po.csr_from_dense(dense)
    V, COL, ROW = gpu_spgemm(po.csr_from_dense(dA), po.csr_from_dense(dB), M, K, N)
    assert np.array_equal(ROW, wR) and np.array_equal(COL, wC) and np.array_equal(bits(V), bits(wV))


@pytest.mark.parametrize("case", [(7, 9, 5, 0.5), (130, 90, 300, 0.05)])
def test_host_layer_sparse_sparse_gemm(dev, case):
    M, K, N, density = case
    h.announce("Sparse::Cuda::Gemm (sparse x sparse)", case)
    dA = sparse_dense(6000 + M, (M, K), density)
    dB = sparse_dense(6100 + N, (K, N), density)
    wV, wC, wR = po.spgemm_csr(po.csr_from_dense(dA), po.csr_from_dense(dB), M, K, N)
    V, COL, ROW = hl.sparse_sparse_gemm(dA, dB, capacity=wV.size + 16)
    assert np.array_equal(ROW, wR) and np.array_equal(COL, wC) and np.array_equal(bits(V), bits(wV))


@pytest.mark.parametrize("case", [(7, 9, 5, 0.5, 0.5), (130, 90, 300, 0.05, 0.2),
                                  (40, 33, 64, 0.0, 0.5), (64, 64, 64, 0.3, 0.0)])
def test_load_distribution_records(dev, case):
    """Per entry of A the number of entries in the row of B it selects (the reference's
    LoadDistMatrix), through GetLoadDist / CallLoadDist and every LoadDistMatrix copy overload of
    the C++ layer; the C ABI call with and without the load array."""
    M, K, N, da, db = case
    h.announce("load distribution M K N dA dB =", case)
    dA = sparse_dense(7100 + M, (M, K), da)
    dB = sparse_dense(7200 + N, (K, N), db)
    VA, CA, RA = po.csr_from_dense(dA)
    VB, CB, RB = po.csr_from_dense(dB)
    want = np.diff(RB.astype(np.int64))[CA].astype(np.uint32)
    load, col, row, products = hl.load_dist(dA, dB)
    assert np.array_equal(load, want) and np.array_equal(col, CA) and np.array_equal(row, RA)
    assert products == int(want.sum())
    # the products bound the entries of the product
    assert int(po.spgemm_csr((VA, CA, RA), (VB, CB, RB), M, K, N)[2][M]) <= products
    dCol, dRow = _dev(CA, np.uint32), _dev(RB, np.uint32)
    dLoad = capi.DeviceBuffer.from_array(np.full(max(len(CA), 1), 0xFFFFFFFF, np.uint32))
    total = ctypes.c_uint64(123)
    capi.call("sph_spgemm_load_u32", dLoad.ptr, dCol.ptr, dRow.ptr, len(CA), K, ctypes.byref(total))
    assert total.value == int(want.sum())
    assert np.array_equal(dLoad.download(np.uint32, (max(len(CA), 1),))[:len(CA)], want)
    total = ctypes.c_uint64(123)
    capi.call("sph_spgemm_load_u32", None, dCol.ptr, dRow.ptr, len(CA), K, ctypes.byref(total))
    assert total.value == int(want.sum())
    for d in (dCol, dRow, dLoad):
        d.release()


@pytest.mark.parametrize("block", range(4))
def test_random_shapes_and_densities(dev, block):
    """Widths on both sides of the bit-map word, run and strip boundaries (32, 64, 4096, several
    strips), short and long rows, empty results."""
    rng = np.random.default_rng(4200 + block)
    widths = [1, 7, 31, 32, 33, 63, 64, 65, 100, 127, 128, 129, 500, 2047, 2048, 2049, 4095, 4096,
              4097, 5000, 8191, 8193, 12289]
    for it in range(10):
        M, K = int(rng.integers(1, 300)), int(rng.integers(1, 300))
        N = int(rng.choice(widths))
        da = float(rng.choice([0.01, 0.05, 0.2, 0.6]))
        db = float(rng.choice([0.002, 0.01, 0.05] if N > 3000 else [0.002, 0.01, 0.05, 0.3]))
        h.announce("sph_spgemm_* random M K N dA dB =", (M, K, N, da, db))
        dA = sparse_dense(100000 + 100 * block + it, (M, K), da)
        dB = sparse_dense(200000 + 100 * block + it, (K, N), db)
        A, B = po.csr_from_dense(dA), po.csr_from_dense(dB)
        wV, wC, wR = po.spgemm_csr(A, B, M, K, N)
        V, COL, ROW = gpu_spgemm(A, B, M, K, N)
        assert np.array_equal(ROW, wR) and np.array_equal(COL, wC)
        assert np.array_equal(bits(V), bits(wV))
        check_one_call(A, B, M, K, N, (wV, wC, wR))


def test_wide_product_mixes_table_rows_and_strip_rows(dev):
    """More than two strips of columns: rows with few products are kept in the hash table,
    the others stay with the strips.  The operands mix both kinds: rows of A that select rows of
    B longer than 64 entries, rows of A with more than 64 entries, rows with more than 256
    products, empty rows, and a pair of entries whose contributions cancel exactly."""
    M, K, N = 260, 300, 20000
    h.announce("sph_spgemm_* wide product with light and heavy rows", (M, K, N))
    rng = np.random.default_rng(77)
    dB = np.zeros((K, N), np.float32)
    for k in range(K):
        count = 100 if k < 10 else 10
        cols = rng.choice(N, size=count, replace=False)
        dB[k, cols] = synth.uniform(9000 + k, (count,))
    dB[21] = dB[20]  # rows 20 and 21 of B are equal: +1 and -1 times them cancel
    dA = np.zeros((M, K), np.float32)
    for m in range(M):
        kind = m % 5
        if kind == 0:    # one or two long rows of B: light, with the 64-at-a-time tail
            ks = rng.choice(10, size=1 + m % 2, replace=False)
        elif kind == 1:  # a handful of short rows of B: light
            ks = 10 + rng.choice(K - 10, size=6, replace=False)
        elif kind == 2:  # more than 64 entries: the strips' row
            ks = rng.choice(K, size=150, replace=False)
        elif kind == 3:  # few entries, more than 256 products: the strips' row
            ks = rng.choice(10, size=6, replace=False)
        else:            # empty
            ks = np.zeros(0, np.int64)
        dA[m, ks] = synth.uniform(9500 + m, (len(ks),))
    dA[1, :] = 0
    dA[1, 20], dA[1, 21], dA[1, 30] = 1.0, -1.0, 0.5  # cancelling pair plus one survivor
    A, B = po.csr_from_dense(dA), po.csr_from_dense(dB)
    wV, wC, wR = po.spgemm_csr(A, B, M, K, N)
    assert wR[2] - wR[1] == np.count_nonzero(dB[30])  # the cancelled columns are not stored
    V, COL, ROW = gpu_spgemm(A, B, M, K, N)
    assert np.array_equal(ROW, wR) and np.array_equal(COL, wC)
    assert np.array_equal(bits(V), bits(wV))
    check_one_call(A, B, M, K, N, (wV, wC, wR))
