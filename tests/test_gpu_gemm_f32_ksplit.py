"""fp32 GEMM on 64 x 32 tiles with K split over two groups of wavefronts: the kernel for products
with more than a quarter and at most half as many 64 x 64 tiles as compute units (65 .. 128 on
this chip), where the few-tile kernel asks the caches for too many bytes and 64 x 64 tiles leave
half of the compute units idle.

Bars: the CPU loop within the fp32 tolerance (max_ij |gpu - cpu| / sum_k |a_ik b_kj| <= 1e-4);
a call with stored-transposed operands bit for bit equal to the plain call on the materialised
transposes; the fused epilogues bit for bit equal to their unfused sequences.
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


# (M, N, K, batch): whole tiles and whole steps; K = 32 q + r (partial last step, r % 4 != 0 too);
# ragged rows and columns; N % 4 != 0 (last columns on the few-tile kernel); M % 4 != 0 (an A
# stored K x M is cut into two launches); a batch; K = 64 (two steps, fewer than the LDS ring)
SHAPES = [(512, 1024, 1024, 1), (1024, 512, 256, 1), (512, 1024, 1000, 1), (512, 1024, 1001, 1),
          (640, 600, 72, 1), (500, 1000, 200, 1), (69, 65, 78, 19), (448, 1026, 64, 1),
          (1001, 512, 64, 1), (4096, 30, 100, 2), (384, 1024, 96, 1), (128, 128, 320, 20),
          (96, 160, 67, 11), (449, 1023, 129, 1)]


@pytest.mark.parametrize("flags", [0, TA, TB, TA | TB, OW, OW | TA | TB])
@pytest.mark.parametrize("shape", SHAPES)
def test_k_split_kernel_against_cpu_and_materialised_transposes(dev, shape, flags):
    M, N, K, batch = shape
    assert h.f32_k_split_range(M, N, K, batch)
    h.announce("sph_gemm_f32_ex K split on 64 x 32 tiles", shape, "flags", flags)
    A = synth.uniform(701, (batch, M, K))
    B = synth.uniform(702, (batch, K, N))
    C = synth.uniform(703, (batch, M, N))
    As, Bs = _stored(A, B, flags)
    got = h.gpu_gemm_f32_ex(C, As, Bs, M, N, K, flags, batch=batch)
    plain = h.gpu_gemm_f32_ex(C, A, B, M, N, K, flags & OW, batch=batch)
    assert np.array_equal(bits(got), bits(plain))
    rows = min(M, 192)
    for u in (0, batch - 1):
        start = np.zeros((rows, N), np.float32) if flags & OW else C[u, :rows].copy()
        ref = po.gemm_rows(start, A[u, :rows], B[u], rows, N, K)
        err = h.normalised_error(got[u, :rows], ref, np.abs(A[u, :rows]), np.abs(B[u]))
        assert err <= TOL_F32, (u, err)
    # the last rows too (row tiles past the first three)
    if M > rows:
        lo = M - min(M - rows, 70)
        start = np.zeros((M - lo, N), np.float32) if flags & OW else C[0, lo:].copy()
        ref = po.gemm_rows(start, A[0, lo:], B[0], M - lo, N, K)
        assert h.normalised_error(got[0, lo:], ref, np.abs(A[0, lo:]), np.abs(B[0])) <= TOL_F32


def test_k_split_kernel_writes_nothing_outside_out(dev):
    """Guard floats before and behind out, ragged M and N."""
    M, N, K = 450, 1000, 160
    assert h.f32_k_split_range(M, N, K)
    h.announce("sph_gemm_f32 K split, guards", (M, N, K))
    A, B, C = synth.uniform(711, (M, K)), synth.uniform(712, (K, N)), synth.uniform(713, (M, N))
    guard = np.full(1024, np.float32(-4321.25))
    padded = np.concatenate([guard, C.ravel(), guard]).astype(np.float32)
    dA, dB, dC = (capi.DeviceBuffer.from_array(x) for x in (A, B, padded))
    assert dC.nbytes >= 4 * (2048 + M * N) and dA.nbytes >= 4 * M * K and dB.nbytes >= 4 * K * N
    capi.call("sph_gemm_f32", dC.at(4096), dA.ptr, dB.ptr, M, N, K, 1, M * N, M * K, K * N)
    back = dC.download(np.float32, padded.shape)
    for d in (dA, dB, dC):
        d.release()
    assert np.array_equal(back[:1024], guard) and np.array_equal(back[-1024:], guard)
    got = back[1024:-1024].reshape(M, N)
    ref = po.gemm_rows(C.copy(), A, B, M, N, K, threads=8)
    assert h.normalised_error(got, ref, np.abs(A), np.abs(B)) <= TOL_F32


@pytest.mark.parametrize("relu", [False, True])
@pytest.mark.parametrize("dims", [(512, 1024, 1024), (1024, 784, 512), (500, 300, 1000)])
def test_linear_forward_in_the_k_split_range(dev, dims, relu):
    """Bias (and ReLU) epilogue: against the unfused device sequence bit for bit (same kernel,
    same order) and the CPU layer within tolerance."""
    batch, fin, fout = dims
    assert h.f32_k_split_range(batch, fout, fin)
    h.announce("sph_linear_forward_f32 K split", dims, "relu", relu)
    x, W = synth.uniform(721, (batch, fin)), synth.uniform(722, (fin, fout))
    bias = synth.uniform(723, (fout,))
    dX, dW, dB = (capi.DeviceBuffer.from_array(v) for v in (x, W, bias))
    dY = capi.DeviceBuffer.from_array(np.full((batch, fout), np.float32(np.nan)))
    capi.call("sph_linear_forward_f32", dY.ptr, dX.ptr, dW.ptr, dB.ptr, batch, fin, fout,
              capi.SPH_LINEAR_RELU if relu else 0)
    got = dY.download(np.float32, (batch, fout))
    ones = capi.DeviceBuffer.from_array(np.ones(batch, np.float32))
    dZ = capi.DeviceBuffer(4 * batch * fout)
    capi.call("sph_fill_f32", dZ.ptr, 0.0, batch * fout)
    capi.call("sph_gemm_f32", dZ.ptr, ones.ptr, dB.ptr, batch, fout, 1, 1, batch * fout, batch, fout)
    capi.call("sph_gemm_f32", dZ.ptr, dX.ptr, dW.ptr, batch, fout, fin, 1, batch * fout,
              batch * fin, fin * fout)
    if relu:
        capi.call("sph_relu_f32", dZ.ptr, dZ.ptr, batch * fout)
    want = dZ.download(np.float32, (batch, fout))
    for d in (dX, dW, dB, dY, dZ, ones):
        d.release()
    assert np.array_equal(bits(got), bits(want))
    ref = po.linear_forward(x[:256], W, bias, threads=8)
    if relu:
        ref = po.relu(ref)
    den = np.abs(x[:256]).astype(np.float64) @ np.abs(W).astype(np.float64) + np.abs(bias)
    assert h.normalised_error(got[:256], ref, None, den, is_denominator=True) <= TOL_F32


def test_grouped_units_in_the_k_split_range(dev):
    """Unit offsets from a table: 6 units of 256 x 256 (96 tiles), B shared by pairs of units."""
    units, M, N, K = 6, 256, 256, 192
    assert h.f32_k_split_range(M, N, K, units)
    h.announce("sph_gemm_f32_grouped K split", (units, M, N, K))
    A, B = synth.uniform(731, (units, M, K)), synth.uniform(732, (3, K, N))
    C = synth.uniform(733, (units, M, N))
    triples = [((units - 1 - u) * M * N, u * M * K, (u % 3) * K * N) for u in range(units)]
    got = h.gpu_gemm_grouped(C, A, B, M, N, K, triples)
    for u in range(units):
        o = units - 1 - u
        ref = po.gemm_rows(C[o].copy(), A[u], B[u % 3], M, N, K)
        assert h.normalised_error(got[o], ref, np.abs(A[u]), np.abs(B[u % 3])) <= TOL_F32


def test_integer_operands_are_exact(dev):
    """Small integers: every product and partial sum is exact, so any order gives the same bits
    as the CPU loop -- indexing and the hand-over between the two groups, not rounding."""
    M, N, K = 500, 1000, 264
    assert h.f32_k_split_range(M, N, K)
    h.announce("sph_gemm_f32 K split, integer operands", (M, N, K))
    A = np.round(synth.uniform(741, (M, K)) * 4).astype(np.float32)
    B = np.round(synth.uniform(742, (K, N)) * 4).astype(np.float32)
    C = np.round(synth.uniform(743, (M, N)) * 8).astype(np.float32)
    got = h.gpu_gemm_f32(C, A, B, M, N, K)
    ref = po.gemm_rows(C.copy(), A, B, M, N, K, threads=8)
    assert np.array_equal(bits(got), bits(ref))
