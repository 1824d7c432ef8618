"""fp32 GEMM launches with more 64 x 64 tiles than resident workgroups: every workgroup takes
several tiles, fetches the next tile's first slabs during the current tile's last steps and
reads the old `out` values at the tile's first step.

Bars:
  * tolerance against the CPU checker (fp32 path, max_ij |gpu - cpu| / sum_k |a_ik b_kj| <= 1e-4);
  * bit for bit against the same product issued one unit (or one row band) per launch, which has
    few enough tiles to take one tile per workgroup - the arithmetic per element is the same.
"""
import numpy as np
import pytest

from oracle import pyoracle as po
from sapphire_amd import capi, synth
from tests import helpers as h

pytestmark = pytest.mark.gpu
TOL_F32 = 1e-4

TA, TB, OW = capi.SPH_GEMM_TRANS_A, capi.SPH_GEMM_TRANS_B, capi.SPH_GEMM_OVERWRITE


def bits(x):
    return np.ascontiguousarray(x).view(np.uint32)


def _stored(A, B, flags):
    As = np.ascontiguousarray(A.swapaxes(-1, -2)) if flags & TA else A
    Bs = np.ascontiguousarray(B.swapaxes(-1, -2)) if flags & TB else B
    return As, Bs


# (batch, M, N, K): 768 tiles (half of the workgroups take two), 1024 (two each), 1792 (three or
# four); one unit alone has 256 tiles, one per workgroup
@pytest.mark.parametrize("dims", [(3, 1024, 1024, 128), (4, 1024, 1024, 256), (7, 1024, 1024, 128)])
@pytest.mark.parametrize("flags", [0, TA, TB, TA | TB, OW, OW | TB])
def test_batched_launch_equals_one_launch_per_unit(dev, dims, flags):
    batch, M, N, K = dims
    h.announce("sph_gemm_f32_ex walk", dims, "flags", flags)
    A = synth.uniform(301, (batch, M, K))
    B = synth.uniform(302, (batch, K, N))
    C = synth.uniform(303, (batch, M, N))
    As, Bs = _stored(A, B, flags)
    got = h.gpu_gemm_f32_ex(C, As, Bs, M, N, K, flags, batch=batch)
    for b in range(batch):
        one = h.gpu_gemm_f32_ex(C[b], As[b], Bs[b], M, N, K, flags)
        assert np.array_equal(bits(got[b]), bits(one)), "unit %d" % b
    # the checker on the first 256 rows of the first and the last unit
    for b in (0, batch - 1):
        start = np.zeros((256, N), np.float32) if flags & OW else C[b, :256].copy()
        ref = po.gemm_rows(start, A[b, :256], B[b], 256, N, K)
        err = h.normalised_error(got[b, :256], ref, np.abs(A[b, :256]), np.abs(B[b]))
        assert err <= TOL_F32, (b, err)


def test_one_large_unit_equals_its_row_bands(dev):
    """2560 x 2560 output (1600 tiles, the band order of the tile walk in play) against the
    same product issued as ten launches of 256 rows each (160 tiles: one tile per workgroup)."""
    M = N = 2560
    K = 128
    h.announce("sph_gemm_f32 walk, one unit", (M, N, K))
    A = synth.uniform(311, (M, K))
    B = synth.uniform(312, (K, N))
    C = synth.uniform(313, (M, N))
    got = h.gpu_gemm_f32(C, A, B, M, N, K)
    for r in range(0, M, 256):
        band = h.gpu_gemm_f32(C[r:r + 256], A[r:r + 256], B, 256, N, K)
        assert np.array_equal(bits(got[r:r + 256]), bits(band)), "rows from %d" % r
    ref = po.gemm_rows(C[:256].copy(), A[:256], B, 256, N, K)
    assert h.normalised_error(got[:256], ref, np.abs(A[:256]), np.abs(B)) <= TOL_F32


@pytest.mark.parametrize("relu", [False, True])
def test_linear_forward_on_a_tile_walk(dev, relu):
    """Bias (and ReLU) epilogue of the walking kernel: 4096 x 640 outputs = 640 tiles, against the
    unfused device sequence bit for bit and the CPU layer within tolerance."""
    batch, fin, fout = 4096, 256, 640
    h.announce("sph_linear_forward_f32 walk", (batch, fin, fout), "relu", relu)
    x = synth.uniform(321, (batch, fin))
    W = synth.uniform(322, (fin, fout))
    bias = synth.uniform(323, (fout,))
    bias[0] = -0.0
    dX, dW, dB = (capi.DeviceBuffer.from_array(v) for v in (x, W, bias))
    dY = capi.DeviceBuffer.from_array(np.full((batch, fout), np.float32(np.nan)))
    flags = capi.SPH_LINEAR_RELU if relu else 0
    capi.call("sph_linear_forward_f32", dY.ptr, dX.ptr, dW.ptr, dB.ptr, batch, fin, fout, flags)
    got = dY.download(np.float32, (batch, fout))
    ones = capi.DeviceBuffer.from_array(np.ones(batch, np.float32))
    dZ = capi.DeviceBuffer(4 * batch * fout)
    capi.call("sph_fill_f32", dZ.ptr, 0.0, batch * fout)
    capi.call("sph_gemm_f32", dZ.ptr, ones.ptr, dB.ptr, batch, fout, 1, 1, batch * fout, batch, fout)
    # the product itself in bands of 1024 rows (160 tiles: one tile per workgroup)
    for r in range(0, batch, 1024):
        capi.call("sph_gemm_f32", dZ.ptr + 4 * r * fout, dX.ptr + 4 * r * fin, dW.ptr, 1024, fout,
                  fin, 1, 1024 * fout, 1024 * fin, fin * fout)
    if relu:
        capi.call("sph_relu_f32", dZ.ptr, dZ.ptr, batch * fout)
    want = dZ.download(np.float32, (batch, fout))
    assert np.array_equal(bits(got), bits(want))
    ref = po.linear_forward(x[:512], W, bias, threads=8)
    if relu:
        ref = po.relu(ref)
    den = np.abs(x[:512]).astype(np.float64) @ np.abs(W).astype(np.float64) + np.abs(bias)
    assert h.normalised_error(got[:512], ref, None, den, is_denominator=True) <= TOL_F32
    for d in (dX, dW, dB, dY, dZ, ones):
        d.release()


def test_grouped_table_on_a_tile_walk(dev):
    """Unit offsets from the device table (a broadcast B, outputs in reverse order) with enough
    units for the walk."""
    units, M, N, K = 3, 1024, 1024, 128
    h.announce("sph_gemm_f32_grouped walk", (units, M, N, K))
    A = synth.uniform(331, (units, M, K))
    B = synth.uniform(332, (2, K, N))
    C = synth.uniform(333, (units, M, N))
    triples = [((units - 1 - u) * M * N, u * M * K, (u % 2) * K * N) for u in range(units)]
    got = h.gpu_gemm_grouped(C, A, B, M, N, K, triples)
    for u in range(units):
        o = units - 1 - u
        one = h.gpu_gemm_f32(C[o], A[u], B[u % 2], M, N, K)
        assert np.array_equal(bits(got[o]), bits(one)), "unit %d" % u
    ref = po.gemm_rows(C[units - 1, :256].copy(), A[0, :256], B[0], 256, N, K)
    assert h.normalised_error(got[units - 1, :256], ref, np.abs(A[0, :256]), np.abs(B[0])) <= TOL_F32
