"""Transposed-operand fp32 GEMM (sph_gemm_f32_ex) against the CPU checker.

Two bars:
  * against the checker on the explicitly transposed operands, tolerance (fp32 path)
    max_ij |gpu - cpu| / sum_k |a_ik * b_kj| <= 1e-4;
  * bit for bit against sph_transpose_f32 followed by sph_gemm_f32 on the device, which is
    what the flags replace.
"""
import numpy as np
import pytest

from oracle import pyoracle as po
from sapphire_amd import capi, synth
from tests import helpers as h

pytestmark = pytest.mark.gpu
TOL_F32 = 1e-4

FLAG_SETS = [capi.SPH_GEMM_TRANS_A, capi.SPH_GEMM_TRANS_B,
             capi.SPH_GEMM_TRANS_A | capi.SPH_GEMM_TRANS_B]

# shapes chosen to reach every kernel: 64-tiles, 128-tiles (two per compute unit: 4096 x 2048),
# the K-split kernel on 16 x 16 and 32 x 32 tiles (few tiles, long K), 16-byte and scalar load
# paths, ragged edges
SHAPES = [(1, 1, 1), (3, 5, 7), (64, 64, 64), (65, 33, 17), (128, 96, 40), (257, 130, 31),
          (512, 384, 100), (2048, 2048, 64), (4096, 2048, 32), (32, 32, 1024), (40, 24, 515),
          (8, 200, 4096), (1000, 10, 1000), (256, 256, 96), (640, 600, 72), (1, 200, 64),
          (1, 1000, 4096), (1, 64, 63),
          # M % 4 != 0 from 68 rows up: an A stored K x M is multiplied in two launches (the last 4
          # rows once more, of which only the new ones are stored)
          (1001, 512, 64), (301, 262, 100), (2049, 2048, 96), (69, 4096, 20), (1023, 1001, 1001)]


def bits(x):
    return np.ascontiguousarray(x).view(np.uint32)


def _stored(A, B, flags):
    """Operands as the caller holds them for these flags (A, B are M x K and K x N)."""
    As = np.ascontiguousarray(A.swapaxes(-1, -2)) if flags & capi.SPH_GEMM_TRANS_A else A
    Bs = np.ascontiguousarray(B.swapaxes(-1, -2)) if flags & capi.SPH_GEMM_TRANS_B else B
    return As, Bs


@pytest.mark.parametrize("flags", FLAG_SETS)
@pytest.mark.parametrize("shape", SHAPES)
def test_flags_match_checker_and_materialised_transpose(dev, shape, flags):
    M, N, K = shape
    h.announce("sph_gemm_f32_ex", shape, "flags", flags)
    A = synth.uniform(41, (M, K))
    B = synth.uniform(42, (K, N))
    C = synth.uniform(43, (M, N))
    As, Bs = _stored(A, B, flags)
    got = h.gpu_gemm_f32_ex(C, As, Bs, M, N, K, flags)
    ref = po.gemm_rows(C.copy(), A, B, M, N, K)
    err = h.normalised_error(got, ref, np.abs(A), np.abs(B))
    assert err <= TOL_F32, err
    # the same product with the transposes materialised on the device first
    Ad = h.gpu_transpose(As, K, M)[0] if flags & capi.SPH_GEMM_TRANS_A else A
    Bd = h.gpu_transpose(Bs, N, K)[0] if flags & capi.SPH_GEMM_TRANS_B else B
    assert np.array_equal(bits(Ad), bits(A)) and np.array_equal(bits(Bd), bits(B))
    plain = h.gpu_gemm_f32(C, Ad, Bd, M, N, K)
    if M == 1 and K >= 64 and flags & capi.SPH_GEMM_TRANS_B:
        # a single row of plain operands runs the row-reduction kernel (another summation
        # order than the matrix-core kernels the transposed B goes to): tolerance only
        assert h.normalised_error(got, plain, np.abs(A), np.abs(B)) <= TOL_F32
    else:
        assert np.array_equal(bits(got), bits(plain))


@pytest.mark.parametrize("flags", FLAG_SETS)
def test_batched_with_shared_operand(dev, flags):
    batch, M, N, K = 5, 70, 52, 36
    h.announce("sph_gemm_f32_ex batched, B shared, flags", flags)
    A = synth.uniform(51, (batch, M, K))
    B = synth.uniform(52, (1, K, N))
    C = synth.uniform(53, (batch, M, N))
    As, Bs = _stored(A, B, flags)
    got = h.gpu_gemm_f32_ex(C, As, Bs, M, N, K, flags, batch=batch, stride_b=0)
    ref = po.gemm_rows(C.copy(), A, B, M, N, K, batch=batch, stride_b=0)
    for b in range(batch):
        err = h.normalised_error(got[b], ref[b], np.abs(A[b]), np.abs(B[0]))
        assert err <= TOL_F32, (b, err)


@pytest.mark.parametrize("shape", [(5, 3, 9), (64, 64, 32), (130, 70, 200), (16, 16, 2048)])
@pytest.mark.parametrize("flags", [0] + FLAG_SETS)
def test_overwrite_ignores_old_contents(dev, shape, flags):
    M, N, K = shape
    h.announce("sph_gemm_f32_ex overwrite", shape, "flags", flags)
    A = synth.uniform(61, (M, K))
    B = synth.uniform(62, (K, N))
    As, Bs = _stored(A, B, flags)
    junk = np.full((M, N), np.float32(np.nan))
    got = h.gpu_gemm_f32_ex(junk, As, Bs, M, N, K, flags | capi.SPH_GEMM_OVERWRITE)
    acc = h.gpu_gemm_f32_ex(np.zeros((M, N), np.float32), As, Bs, M, N, K, flags)
    assert np.array_equal(bits(got), bits(acc))
    ref = po.gemm_rows(np.zeros((M, N), np.float32), A, B, M, N, K)
    assert h.normalised_error(got, ref, np.abs(A), np.abs(B)) <= TOL_F32


def test_overwrite_with_zero_k_stores_zeros_and_bad_flags_are_rejected(dev):
    h.announce("sph_gemm_f32_ex K = 0 / unknown flag")
    junk = np.full((3, 4), np.float32(7.0))
    one = np.zeros(1, np.float32)
    got = h.gpu_gemm_f32_ex(junk, one, one, 3, 4, 0, capi.SPH_GEMM_OVERWRITE)
    assert np.array_equal(got, np.zeros((3, 4), np.float32))
    kept = h.gpu_gemm_f32_ex(junk, one, one, 3, 4, 0, capi.SPH_GEMM_TRANS_A)
    assert np.array_equal(kept, junk)
    with pytest.raises(capi.SphError):
        # operands of the stated size: the helper checks extents before every raw-pointer call
        h.gpu_gemm_f32_ex(junk, np.zeros(3, np.float32), np.zeros(4, np.float32), 3, 4, 1, 64)


def test_backward_shapes_of_the_mlp(dev):
    """dx += dy W^T and dw = x^T dy at the sizes of the 784-1024-1024-10 network, batch 1024."""
    batch = 1024
    for fin, fout in [(784, 1024), (1024, 10)]:
        h.announce("backward GEMMs batch", batch, "in", fin, "out", fout)
        x = synth.uniform(71, (batch, fin))
        W = synth.uniform(72, (fin, fout))
        dy = synth.uniform(73, (batch, fout))
        dx = h.gpu_gemm_f32_ex(np.zeros((batch, fin), np.float32), dy, W, batch, fin, fout,
                               capi.SPH_GEMM_TRANS_B)
        Wt = np.ascontiguousarray(W.T)
        ref = po.gemm_rows(np.zeros((batch, fin), np.float32), dy, Wt, batch, fin, fout)
        assert h.normalised_error(dx, ref, np.abs(dy), np.abs(Wt)) <= TOL_F32
        dw = h.gpu_gemm_f32_ex(np.zeros((fin, fout), np.float32), x, dy, fin, fout, batch,
                               capi.SPH_GEMM_TRANS_A | capi.SPH_GEMM_OVERWRITE)
        xt = np.ascontiguousarray(x.T)
        ref = po.gemm_rows(np.zeros((fin, fout), np.float32), xt, dy, fin, fout, batch)
        assert h.normalised_error(dw, ref, np.abs(xt), np.abs(dy)) <= TOL_F32
