"""fp16-input / fp32-accumulate GEMM on 256 x 128 tiles (four wavefronts per workgroup): the form
of the 256-tile kernel for products with too few 256 x 256 tiles to fill the chip -- from 176 up to
256 tiles of 256 x 128, at least three quarters of the tiled area real output.

Integer-valued operands make every product and partial sum exact, so tiling, the copy plan, the
transposing reads and the old-contents mailbox are checked bit for bit against the CPU loop;
N(0, 1/sqrt(K)) operands are held to the fp16 tolerance 1e-2.
"""
import numpy as np
import pytest

from oracle import pyoracle as po
from sapphire_amd import capi, synth
from tests import helpers as h

pytestmark = pytest.mark.gpu
TOL_F16 = 1e-2
TA, TB, OW = capi.SPH_GEMM_TRANS_A, capi.SPH_GEMM_TRANS_B, capi.SPH_GEMM_OVERWRITE


def _in_range(M, N, batch):
    tiles = -(-M // 256) * -(-N // 128) * batch
    tiles256 = -(-M // 256) * -(-N // 256) * batch
    fills = 4 * M * N >= 3 * -(-M // 256) * -(-N // 128) * 256 * 128
    fills256 = 4 * M * N >= 3 * -(-M // 256) * -(-N // 256) * 256 * 256
    takes256 = tiles256 >= 192 and fills256       # the 256 x 256 kernel comes first
    return 176 <= tiles <= 256 and not takes256 and fills and N % 8 == 0


def _oracle(C, A16, B16, M, N, K, batch=1):
    return po.gemm_rows(C.copy(), A16.astype(np.float32), B16.astype(np.float32), M, N, K,
                        batch=batch, threads=8)


def _stored(A, B, flags):
    As = np.ascontiguousarray(A.swapaxes(-1, -2)) if flags & TA else A
    Bs = np.ascontiguousarray(B.swapaxes(-1, -2)) if flags & TB else B
    return As, Bs


# (M, N, K, batch).  K: a few steps; a partial last step (K = 32 q + r); 608 is the last K whose
# accumulating launch reads out in the epilogue, 640 .. 704 add it inside the loop every second
# step, 1152 .. 1280 every fourth.  Ragged M and N; a batch of small units.
SHAPES = [(3072, 2048, 64, 1), (2048, 4096, 96, 1), (4096, 2048, 200, 1), (3072, 2048, 608, 1),
          (2048, 4096, 640, 1), (3072, 2048, 672, 1), (4096, 2048, 704, 1), (3072, 2048, 1152, 1),
          (2816, 2048, 1184, 1), (2048, 4096, 1280, 1), (256, 128, 128, 200), (512, 256, 1216, 50),
          (3000, 1912, 96, 1), (2817, 2040, 160, 1), (250, 120, 72, 200), (3072, 2048, 1000, 1)]


# (an A stored K x M is copied 8 rows at a time: with M % 8 != 0 the product is cut up and its
# parts run other kernels, covered by the tests of those)
@pytest.mark.parametrize("shape,flags", [(shape, flags) for shape in SHAPES
                                         for flags in (0, TA, TB, TA | TB)
                                         if not (flags & TA and shape[0] % 8 != 0)])
def test_exact_on_integers(dev, shape, flags):
    M, N, K, batch = shape
    assert _in_range(M, N, batch), shape
    h.announce("sph_gemm_f16f32 256 x 128 tiles, integer exactness", shape, "flags", flags)
    span = 4 if K <= 256 else 3
    A = synth.small_integers(11, (batch, M, K), span=span).astype(np.float16)
    B = synth.small_integers(12, (batch, K, N), span=span).astype(np.float16)
    C = synth.small_integers(13, (batch, M, N), span=100)
    As, Bs = _stored(A, B, flags)
    ref = _oracle(C, A, B, M, N, K, batch=batch)
    got = h.gpu_gemm_f16(C, As, Bs, M, N, K, batch=batch, flags=flags)
    assert np.array_equal(got, ref)
    got = h.gpu_gemm_f16(C, As, Bs, M, N, K, batch=batch, flags=flags | OW)
    assert np.array_equal(got, ref - C)


@pytest.mark.parametrize("shape", [(3072, 2048, 2048), (2048, 4096, 1024), (3000, 1912, 520)])
def test_real_values_within_tolerance(dev, shape):
    M, N, K = shape
    assert _in_range(M, N, 1)
    h.announce("sph_gemm_f16f32 256 x 128 tiles, N(0, 1/sqrt(K)) operands", shape)
    A = synth.normal(21, (M, K), 1.0 / np.sqrt(K)).astype(np.float16)
    B = synth.normal(22, (K, N), 1.0 / np.sqrt(K)).astype(np.float16)
    C = synth.uniform(23, (M, N))
    got = h.gpu_gemm_f16(C, A, B, M, N, K)
    for lo in (0, M - 128):
        a32, b32 = A[lo:lo + 128].astype(np.float32), B.astype(np.float32)
        ref = po.gemm_rows(C[lo:lo + 128].copy(), a32, b32, 128, N, K, threads=8)
        assert h.normalised_error(got[lo:lo + 128], ref, np.abs(a32), np.abs(b32)) <= TOL_F16


def test_nothing_is_written_outside_out(dev):
    """Guard floats before and behind out, ragged M and N, accumulate and overwrite."""
    M, N, K = 2900, 2040, 128
    assert _in_range(M, N, 1)
    h.announce("sph_gemm_f16f32 256 x 128 tiles, guards", (M, N, K))
    A = synth.small_integers(31, (M, K), span=4).astype(np.float16)
    B = synth.small_integers(32, (K, N), span=4).astype(np.float16)
    C = synth.small_integers(33, (M, N), span=100)
    guard = np.full(2048, np.float32(-4321.25))
    for flags in (0, OW):
        padded = np.concatenate([guard, C.ravel(), guard]).astype(np.float32)
        dA, dB, dC = (capi.DeviceBuffer.from_array(x) for x in (A, B, padded))
        assert dC.nbytes >= 4 * (4096 + M * N) and dA.nbytes >= 2 * M * K and dB.nbytes >= 2 * K * N
        capi.call("sph_gemm_f16f32", dC.at(4 * 2048), dA.ptr, dB.ptr, M, N, K, 1, M * N, M * K, K * N,
                  flags)
        back = dC.download(np.float32, padded.shape)
        for d in (dA, dB, dC):
            d.release()
        assert np.array_equal(back[:2048], guard) and np.array_equal(back[-2048:], guard)
        ref = _oracle(C, A, B, M, N, K)
        want = ref - C if flags & OW else ref
        assert np.array_equal(back[2048:-2048].reshape(M, N), want)
