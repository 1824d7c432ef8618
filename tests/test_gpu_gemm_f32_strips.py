"""fp32 GEMM whose last rows and columns are cut off as thin strips: the last N % 4 columns, the
last M % 4 rows (from 68 rows up) and up to 16 rows or columns past a multiple of the tile edge
when that spares the busiest compute unit a tile.  The strips are computed by the few-tile
kernel's code inside the launch of the body (straight-to-LDS kernels) or by launches of their own
(register-staged kernel: operands that start off a 16-byte boundary).

Bars: the CPU loop within the fp32 tolerance (max_ij |gpu - cpu| / sum_k |a_ik b_kj| <= 1e-4);
a call with stored-transposed operands, and one on operands that start 4 bytes off a 16-byte
boundary, bit for bit equal to the plain call; nothing written outside out; exact on integers.
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


# (M, N, K, batch).  17 x 17 tiles of 64 cut down to 16 x 16; one row past 16 tile rows, 4 | N;
# 1 column past; rows and columns past by up to 16; M % 4 and N % 4 only (no tile spared);
# 128-tiles (33 x 33 of them cut to 32 x 32 would need 4225 rows: here 9 x 9 of 128 > 4 x 64-tile
# rounds); a batch whose units each lose a row and a column; K below one step of 32 and K = 16
SHAPES = [(1025, 1025, 40, 1), (1025, 1024, 70, 1), (1024, 1025, 33, 1), (1040, 1036, 48, 1),
          (1001, 1001, 36, 1), (1031, 1000, 64, 1), (2049, 2049, 32, 1), (8192, 65, 64, 1),
          (8192, 67, 17, 1), (513, 514, 24, 4), (321, 323, 50, 7), (1025, 1025, 16, 1),
          (2061, 1030, 20, 1), (1025, 1026, 20, 3)]


@pytest.mark.parametrize("flags", [0, TA, TB, TA | TB, OW, OW | TA | TB])
@pytest.mark.parametrize("shape", SHAPES)
def test_strips_against_cpu_and_materialised_transposes(dev, shape, flags):
    M, N, K, batch = shape
    h.announce("sph_gemm_f32_ex with edge strips", shape, "flags", flags)
    A = synth.uniform(801, (batch, M, K))
    B = synth.uniform(802, (batch, K, N))
    C = synth.uniform(803, (batch, M, N))
    As, Bs = _stored(A, B, flags)
    got = h.gpu_gemm_f32_ex(C, As, Bs, M, N, K, flags, batch=batch)
    plain = h.gpu_gemm_f32_ex(C, A, B, M, N, K, flags & OW, batch=batch)
    assert np.array_equal(bits(got), bits(plain))
    # the last rows (bottom strip and the body's last tile row), every column (right strip)
    lo = M - 80
    for u in (0, batch - 1):
        start = np.zeros((M - lo, N), np.float32) if flags & OW else C[u, lo:].copy()
        ref = po.gemm_rows(start, A[u, lo:], B[u], M - lo, N, K)
        err = h.normalised_error(got[u, lo:], ref, np.abs(A[u, lo:]), np.abs(B[u]))
        assert err <= TOL_F32, (u, err)
    # the last columns of every row
    cols = slice(max(0, N - 40), N)
    start = np.zeros((M, N), np.float32) if flags & OW else C[0].copy()
    width = cols.stop - cols.start
    Bc = np.ascontiguousarray(B[0][:, cols])
    ref = po.gemm_rows(np.ascontiguousarray(start[:, cols]), A[0], Bc, M, width, K, threads=8)
    assert h.normalised_error(got[0][:, cols], ref, np.abs(A[0]), np.abs(Bc)) <= TOL_F32


@pytest.mark.parametrize("shape", [(1025, 1025, 72), (1001, 1003, 40), (8192, 65, 64)])
def test_strips_do_not_depend_on_alignment(dev, shape):
    """Operands that start 4 bytes past a 16-byte boundary take the register-staged kernel and
    launches of their own for the strips: same cut, same kernels for the strips, same bits."""
    M, N, K = shape
    h.announce("sph_gemm_f32 strips, operands off a 16-byte boundary", shape)
    A, B, C = synth.uniform(811, (M, K)), synth.uniform(812, (K, N)), synth.uniform(813, (M, N))
    aligned = h.gpu_gemm_f32_ex(C[None], A[None], B[None], M, N, K, 0)[0]
    pad = np.zeros(1, np.float32)
    dA = capi.DeviceBuffer.from_array(np.concatenate([pad, A.ravel()]))
    dB = capi.DeviceBuffer.from_array(np.concatenate([pad, B.ravel()]))
    dC = capi.DeviceBuffer.from_array(C)
    assert dA.nbytes >= 4 * (M * K + 1) and dB.nbytes >= 4 * (K * N + 1) and dC.nbytes >= 4 * M * N
    capi.call("sph_gemm_f32", dC.ptr, dA.at(4), dB.at(4), M, N, K, 1, M * N, M * K, K * N)
    off = dC.download(np.float32, (M, N))
    for d in (dA, dB, dC):
        d.release()
    # the body's kernels differ (straight-to-LDS against register-staged) but sum in one order
    assert np.array_equal(bits(off), bits(aligned))


def test_strips_write_nothing_outside_out(dev):
    """Guard floats before and behind out."""
    M, N, K = 1025, 1027, 48
    h.announce("sph_gemm_f32 strips, guards", (M, N, K))
    A, B, C = synth.uniform(821, (M, K)), synth.uniform(822, (K, N)), synth.uniform(823, (M, N))
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


@pytest.mark.parametrize("flags", [0, TA, TB])
def test_integer_operands_are_exact(dev, flags):
    """Small integers: every product and partial sum is exact, so any order gives the CPU loop's
    bits -- the indexing of body and strips, not rounding."""
    M, N, K = 1025, 1026, 96
    h.announce("sph_gemm_f32_ex strips, integers", (M, N, K), "flags", flags)
    rng = np.random.default_rng(831)
    A = rng.integers(-4, 5, (M, K)).astype(np.float32)
    B = rng.integers(-4, 5, (K, N)).astype(np.float32)
    C = rng.integers(-100, 101, (M, N)).astype(np.float32)
    As, Bs = _stored(A, B, flags)
    got = h.gpu_gemm_f32_ex(C[None], As[None], Bs[None], M, N, K, flags)[0]
    want = (C.astype(np.float64) + A.astype(np.float64) @ B.astype(np.float64)).astype(np.float32)
    assert np.array_equal(got, want)


@pytest.mark.parametrize("relu", [False, True])
def test_linear_forward_with_strips(dev, relu):
    """Bias (and ReLU) epilogue in body and strips: against the unfused device sequence bit for
    bit and the CPU layer within tolerance."""
    batch, fin, fout = 1025, 48, 1026
    h.announce("sph_linear_forward_f32 with strips", (batch, fin, fout), "relu", relu)
    x, W = synth.uniform(841, (batch, fin)), synth.uniform(842, (fin, fout))
    bias = synth.uniform(843, (fout,))
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
    ref = po.linear_forward(x, W, bias, threads=8)
    if relu:
        ref = po.relu(ref)
    den = np.abs(x).astype(np.float64) @ np.abs(W).astype(np.float64) + np.abs(bias)
    assert h.normalised_error(got, ref, None, den, is_denominator=True) <= TOL_F32


def test_grouped_units_with_strips(dev):
    """Unit offsets from a table: 5 units of 321 x 323, out written in reverse order."""
    units, M, N, K = 5, 321, 323, 40
    h.announce("sph_gemm_f32_grouped with strips", (units, M, N, K))
    A, B = synth.uniform(851, (units, M, K)), synth.uniform(852, (2, K, N))
    C = synth.uniform(853, (units, M, N))
    triples = [((units - 1 - u) * M * N, u * M * K, (u % 2) * K * N) for u in range(units)]
    got = h.gpu_gemm_grouped(C, A, B, M, N, K, triples)
    for u in range(units):
        o = units - 1 - u
        ref = po.gemm_rows(C[o].copy(), A[u], B[u % 2], M, N, K)
        assert h.normalised_error(got[o], ref, np.abs(A[u]), np.abs(B[u % 2])) <= TOL_F32


@pytest.mark.parametrize("block", range(6))
def test_random_shapes_just_past_a_tile_grid(dev, block):
    """Seeded shapes a few rows and columns past multiples of 64 and 128 with about one tile per
    compute unit, where the cut depends on both remainders; all flag combinations, guard words."""
    rng = np.random.default_rng(9300 + block)
    for it in range(8):
        M = int(rng.choice([960, 1024, 1088, 2048])) + int(rng.integers(0, 19))
        N = int(rng.choice([960, 1024, 1088, 512])) + int(rng.integers(0, 19))
        K = int(rng.choice([16, 24, 33, 64, 100]))
        flags = int(rng.integers(0, 8))
        h.announce("sph_gemm_f32_ex random, past a tile grid", (M, N, K), "flags", flags)
        seed = 930000 + 100 * block + 3 * it
        A, B = synth.uniform(seed, (M, K)), synth.uniform(seed + 1, (K, N))
        C = synth.uniform(seed + 2, (M, N))
        As, Bs = _stored(A, B, flags)
        guard = np.full(64, np.float32(-777.25), np.float32)
        padded = np.concatenate([guard, C.ravel(), guard])
        dA, dB, dC = (capi.DeviceBuffer.from_array(x) for x in (As, Bs, padded))
        assert dC.nbytes >= 4 * (128 + M * N) and dA.nbytes >= 4 * M * K and dB.nbytes >= 4 * K * N
        capi.call("sph_gemm_f32_ex", dC.at(4 * 64), dA.ptr, dB.ptr, M, N, K, 1, M * N, M * K,
                  K * N, flags)
        back = dC.download(np.float32, padded.shape)
        for d in (dA, dB, dC):
            d.release()
        assert np.array_equal(back[:64], guard) and np.array_equal(back[-64:], guard)
        start = np.zeros_like(C) if flags & OW else C
        ref = po.gemm_rows(start.copy(), A, B, M, N, K, threads=8)
        err = h.normalised_error(back[64:-64].reshape(M, N), ref, np.abs(A), np.abs(B))
        assert err <= TOL_F32, (M, N, K, flags, err)
