"""sph_csr_row_offsets_noalloc_f32: the row-offset pass whose scan keeps its block totals in a
fixed array inside the library, against sph_csr_row_offsets_f32 (stream-ordered scratch block)
and the CPU checker, bit for bit; consecutive calls share the array, the later ones smaller."""
import ctypes

import numpy as np
import pytest

from oracle import pyoracle as po
from sapphire_amd import capi, synth
from tests import helpers as h

pytestmark = pytest.mark.gpu


def sparse_dense(seed, shape, density):
    vals = synth.uniform(seed, shape)
    keep = synth.uniform(seed + 1, shape, 0.0, 1.0) < density
    return np.where(keep, vals, np.float32(0)).astype(np.float32)


def row_offsets(entry, dDense, M, N, ld):
    # ROW is pre-filled with junk so that an entry the call leaves unwritten shows
    dRow = capi.DeviceBuffer.from_array(np.full(M + 1 + 8, 0xA5A5A5A5, np.uint32))
    if entry == "sph_csr_row_offsets_f32":
        capi.call(entry, dRow.ptr, dDense.ptr, M, N, ld, None)
    else:
        capi.call(entry, dRow.ptr, dDense.ptr, M, N, ld)
    got = dRow.download(np.uint32, (M + 1 + 8,))
    dRow.release()
    assert np.all(got[M + 1:] == 0xA5A5A5A5), "write past ROW[M]"
    return got[:M + 1]


def test_two_calls_in_a_row_second_smaller(dev):
    # both scans are longer than one workgroup's 65536 values, so both use the block totals;
    # the second has fewer blocks than the first and must not see what the first left behind;
    # the third and fourth fit one workgroup and one round and leave the array alone
    cases = [(300000, 24, 24, 0.30), (70001, 6, 8, 0.55), (5000, 24, 24, 0.1), (0, 4, 4, 0.0)]
    for idx, (M, N, ld, density) in enumerate(cases):
        h.announce("sph_csr_row_offsets_noalloc_f32 call", idx, "M N ld density =",
                   (M, N, ld, density))
        dense = sparse_dense(4200 + idx, (max(M, 1), ld), density)[:M]
        dense[:, N:] = 3.0
        want = po.csr_from_dense(dense, N=N)[2] if M else np.zeros(1, np.uint32)
        dD = capi.DeviceBuffer.from_array(dense if dense.size else np.zeros(1, np.float32))
        new = row_offsets("sph_csr_row_offsets_noalloc_f32", dD, M, N, ld)
        old = row_offsets("sph_csr_row_offsets_f32", dD, M, N, ld)
        dD.release()
        assert np.array_equal(new, old)
        assert np.array_equal(new, want)


def _allocations():
    count = ctypes.c_uint64(0)
    capi.call("sph_allocation_count", ctypes.byref(count))
    return count.value


def test_the_call_makes_no_allocation(dev):
    """The library counts every hipMalloc / hipMallocAsync / hipHostMalloc it makes.  Across the
    no-allocation entry the count stays put, for a scan that needs the block totals (more than
    65536 rows) and for one that does not; across the allocating entry on the same input it
    moves, which shows that the counter sees the scratch block."""
    M, N, ld = 200000, 12, 12
    dense = sparse_dense(4400, (M, ld), 0.2)
    dD = capi.DeviceBuffer.from_array(dense)
    dRow = capi.DeviceBuffer(4 * (M + 1))
    capi.sync()
    h.announce("sph_csr_row_offsets_noalloc_f32 allocation count", (M, N, ld))
    before = _allocations()
    capi.call("sph_csr_row_offsets_noalloc_f32", dRow.ptr, dD.ptr, M, N, ld)
    capi.call("sph_csr_row_offsets_noalloc_f32", dRow.ptr, dD.ptr, 5000, N, ld)
    capi.sync()
    assert _allocations() == before
    capi.call("sph_csr_row_offsets_f32", dRow.ptr, dD.ptr, M, N, ld, None)
    capi.sync()
    assert _allocations() == before + 1
    dD.release()
    dRow.release()


def test_rejects_more_rows_than_the_array_covers(dev):
    dRow = capi.DeviceBuffer(64)
    with pytest.raises(capi.SphError) as err:
        capi.call("sph_csr_row_offsets_noalloc_f32", dRow.ptr, dRow.ptr, 1 << 24, 1, 1)
    assert err.value.status == 1
    dRow.release()


def test_recordable_into_a_graph(dev):
    # the allocating entry refuses this size under capture; this one records and replays
    M, N, ld = 70001, 6, 8
    first = sparse_dense(4300, (M, ld), 0.4)
    second = sparse_dense(4301, (M, ld), 0.1)
    dD = capi.DeviceBuffer.from_array(first)
    dRow = capi.DeviceBuffer.from_array(np.zeros(M + 1, np.uint32))
    with capi.Graph() as g:
        with pytest.raises(capi.SphError):
            capi.call("sph_csr_row_offsets_f32", dRow.ptr, dD.ptr, M, N, ld, None)
        capi.call("sph_csr_row_offsets_noalloc_f32", dRow.ptr, dD.ptr, M, N, ld)
    for dense in (first, second, first):
        dD.upload(dense)
        g.launch()
        capi.sync()
        got = dRow.download(np.uint32, (M + 1,))
        assert np.array_equal(got, po.csr_from_dense(dense, N=N)[2])
        # eager work between the replays
        eager = row_offsets("sph_csr_row_offsets_f32", dD, M, N, ld)
        assert np.array_equal(got, eager)
    g.destroy()
    dD.release()
    dRow.release()
