"""sph_csr_validate_u32: a CSR record is checked on the device before a product trusts it.

The products read B[COL[p]] and the entries ROW[i] .. ROW[i + 1] as given, so a bad record is
a device memory fault.  Every case here hands the bad record to the validator only; the
product kernels are never launched on it.
"""
import ctypes

import numpy as np
import pytest

from sapphire_amd import capi, synth
from tests import helpers as h

pytestmark = pytest.mark.gpu

ROW_START, ROW_ORDER, ROW_TOTAL, COL_RANGE, COL_UNSORTED = 1, 2, 4, 8, 16


def _validate(col, row, M, Kdim, nnz):
    d_col = capi.DeviceBuffer.from_array(col if col.size else np.zeros(1, np.uint32))
    d_row = capi.DeviceBuffer.from_array(row)
    assert d_row.nbytes >= 4 * (M + 1) and d_col.nbytes >= 4 * nnz
    problems = ctypes.c_uint32(0)
    status = capi.lib().sph_csr_validate_u32(d_col.ptr, d_row.ptr, M, Kdim, nnz,
                                             ctypes.byref(problems))
    text = capi.lib().sph_last_error().decode() if status else ""
    d_col.release()
    d_row.release()
    return status, problems.value, text


def test_good_records_pass(dev):
    h.announce("sph_csr_validate_u32 on well-formed records")
    for seed, M, K, per_row in ((1, 300, 777, 20.0), (2, 1, 5, 2.0), (3, 8192, 8192, 81.92)):
        v, col, row = synth.csr_matrix(5000 + seed, M, K, per_row)
        status, problems, _ = _validate(col, row, M, K, int(col.size))
        assert status == 0 and problems == 0
    # no entries at all, and no rows at all
    status, problems, _ = _validate(np.zeros(0, np.uint32), np.zeros(11, np.uint32), 10, 4, 0)
    assert status == 0 and problems == 0
    status, problems, _ = _validate(np.zeros(0, np.uint32), np.zeros(1, np.uint32), 0, 4, 0)
    assert status == 0 and problems == 0


def test_column_out_of_range_is_refused(dev):
    h.announce("sph_csr_validate_u32 column index == Kdim (validator only, no product launched)")
    M, K = 64, 100
    v, col, row = synth.csr_matrix(5100, M, K, 8.0)
    bad = col.copy()
    bad[bad.size // 2] = K          # one past the last valid column
    status, problems, text = _validate(bad, row, M, K, int(bad.size))
    assert status == 1              # SPH_ERR_INVALID
    assert problems & COL_RANGE
    assert "column index" in text
    bad[bad.size // 2] = 0xffffffff
    status, problems, _ = _validate(bad, row, M, K, int(bad.size))
    assert status == 1 and problems & COL_RANGE
    # the largest valid index passes
    ok = col.copy()
    ok[-1] = K - 1
    status, problems, _ = _validate(ok, row, M, K, int(ok.size))
    assert status == 0 and not problems & COL_RANGE


def test_row_offsets_are_checked(dev):
    h.announce("sph_csr_validate_u32 ROW rules")
    M, K = 50, 60
    v, col, row = synth.csr_matrix(5200, M, K, 6.0)
    nnz = int(col.size)
    r = row.copy()
    r[0] = 1
    status, problems, text = _validate(col, r, M, K, nnz)
    assert status == 1 and problems & ROW_START and "ROW[0]" in text
    r = row.copy()
    r[20], r[21] = r[21] + 3, r[20]            # a decreasing pair
    status, problems, _ = _validate(col, r, M, K, nnz)
    assert status == 1 and problems & ROW_ORDER
    r = row.copy()
    r[M] = nnz + 5                              # claims entries the arrays do not hold
    status, problems, text = _validate(col, r, M, K, nnz)
    assert status == 1 and problems & ROW_TOTAL and "entry count" in text
    # an offset far past the arrays is reported without anything being read there
    r = row.copy()
    r[10] = 0xfffffff0
    status, problems, _ = _validate(col, r, M, K, nnz)
    assert status == 1 and problems & ROW_ORDER


def test_unsorted_columns_are_reported_not_refused(dev):
    h.announce("sph_csr_validate_u32 unsorted row")
    row = np.array([0, 3, 5], np.uint32)
    col = np.array([4, 2, 7, 1, 3], np.uint32)
    status, problems, _ = _validate(col, row, 2, 8, 5)
    assert status == 0 and problems == COL_UNSORTED
    col = np.array([2, 2, 7, 1, 3], np.uint32)   # a repeated column is not strictly ascending
    status, problems, _ = _validate(col, row, 2, 8, 5)
    assert status == 0 and problems == COL_UNSORTED


def test_null_pointers(dev):
    assert capi.lib().sph_csr_validate_u32(None, None, 4, 4, 0, None) == 1
    d_row = capi.DeviceBuffer.from_array(np.zeros(5, np.uint32))
    assert capi.lib().sph_csr_validate_u32(None, d_row.ptr, 4, 4, 3, None) == 1
    assert capi.lib().sph_csr_validate_u32(None, d_row.ptr, 4, 4, 0, None) == 0
    d_row.release()


def test_helpers_refuse_a_bad_record_before_the_product(dev):
    """tests.helpers.gpu_spmm validates first: the product kernel is not launched."""
    M, K, N = 16, 32, 8
    v, col, row = synth.csr_matrix(5300, M, K, 4.0)
    bad = col.copy()
    bad[0] = K + 7
    with pytest.raises(capi.SphError):
        h.gpu_spmm(np.zeros((M, N), np.float32), v, bad, row, M, K, N, synth.uniform(1, (K, N)),
                   False)
    # and an operand smaller than its stated shape is refused on the host
    with pytest.raises(ValueError):
        h.gpu_spmm(np.zeros((M, N), np.float32), v, col, row, M, K, N, synth.uniform(1, (K - 1, N)),
                   False)
