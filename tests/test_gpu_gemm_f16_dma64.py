"""fp16-input / fp32-accumulate GEMM on 64 x 64 tiles with K steps of 64: the straight-to-LDS
kernel for products with at most half as many 128 x 128 tiles as compute units (and more than
one 32 x 32 tile per compute unit, below which the few-tile kernel runs), K >= 64, N % 8 == 0.

Integer-valued operands make every product and partial sum exact, so the copy plan, both LDS
layouts, the transposing reads and the partial last step are checked bit for bit against the
CPU loop; N(0, 1/sqrt(K)) operands are held to the fp16 tolerance 1e-2.
"""
import numpy as np
import pytest

from oracle import pyoracle as po
from sapphire_amd import capi, synth
from tests import helpers as h

pytestmark = pytest.mark.gpu
TOL_F16 = 1e-2
TA, TB, OW = capi.SPH_GEMM_TRANS_A, capi.SPH_GEMM_TRANS_B, capi.SPH_GEMM_OVERWRITE
CUS = 256


def _in_range(M, N, K, batch):
    tiles128 = -(-M // 128) * -(-N // 128) * batch
    return tiles128 <= CUS // 2 and not h.f16_few_tiles(M, N, batch, K) and K >= 64 and N % 8 == 0


def _oracle(C, A16, B16, M, N, K, batch=1):
    return po.gemm_rows(C.copy(), A16.astype(np.float32), B16.astype(np.float32), M, N, K,
                        batch=batch, threads=8)


def _stored(A, B, flags):
    As = np.ascontiguousarray(A.swapaxes(-1, -2)) if flags & TA else A
    Bs = np.ascontiguousarray(B.swapaxes(-1, -2)) if flags & TB else B
    return As, Bs


# (M, N, K, batch): one step, two, fewer and more than the four LDS stages; K = 64 q + r with r a
# multiple of 8, odd r (rows of a K-contiguous operand then start at 2-byte-aligned addresses),
# r just below and above a step; ragged M and N; a batch of small units; the shapes of the MLP
SHAPES = [(1024, 1024, 64, 1), (1024, 1024, 128, 1), (1024, 1024, 192, 1), (1024, 1024, 1024, 1),
          (1024, 1024, 72, 1), (1024, 1024, 100, 1), (1024, 1024, 127, 1), (1024, 1024, 129, 1),
          (1024, 1024, 784, 1), (1024, 1024, 1000, 1), (1024, 1024, 999, 1), (600, 520, 200, 1),
          (1000, 1016, 328, 1), (128, 128, 256, 40), (120, 136, 77, 36), (1536, 1024, 320, 1),
          (600, 520, 65, 1), (520, 600, 1217, 1),
          # from half a 32 x 32 tile per compute unit up (below that: the few-tile kernel)
          (256, 512, 2048, 1), (128, 1024, 1024, 1), (256, 1024, 1024, 1), (512, 512, 515, 1)]


@pytest.mark.parametrize("flags", [0, TA, TB, TA | TB])
@pytest.mark.parametrize("shape", SHAPES)
def test_exact_on_integers(dev, shape, flags):
    M, N, K, batch = shape
    assert _in_range(M, N, K, batch), shape
    h.announce("sph_gemm_f16f32 64 x 64 tiles, integer exactness", shape, "flags", flags)
    span = 4 if K <= 256 else 3
    A = synth.small_integers(51, (batch, M, K), span=span).astype(np.float16)
    B = synth.small_integers(52, (batch, K, N), span=span).astype(np.float16)
    C = synth.small_integers(53, (batch, M, N), span=100)
    As, Bs = _stored(A, B, flags)
    ref = _oracle(C, A, B, M, N, K, batch=batch)
    got = h.gpu_gemm_f16(C, As, Bs, M, N, K, batch=batch, flags=flags)
    assert np.array_equal(got, ref)
    got = h.gpu_gemm_f16(C, As, Bs, M, N, K, batch=batch, flags=flags | OW)
    assert np.array_equal(got, ref - C)


@pytest.mark.parametrize("flags", [0, TA | TB])
@pytest.mark.parametrize("K", [72, 100, 127, 150, 190])
def test_partial_last_step_counts_an_infinity_once(dev, K, flags):
    """An infinity (and a 0 x Inf) at a k that lies in both of the last two step windows must come
    out exactly as in the CPU product: +Inf where the partner is positive, NaN where it is zero,
    and nothing else may change."""
    M, N = 1024, 1024
    assert _in_range(M, N, K, 1)
    h.announce("sph_gemm_f16f32 64 x 64 tiles, Inf inside the repeated window", K)
    A = synth.small_integers(61, (M, K), span=3).astype(np.float16)
    B = synth.small_integers(62, (K, N), span=3).astype(np.float16)
    C = synth.small_integers(63, (M, N), span=100)
    k = K - 64                      # the first position of the repeated window [K - 64, 64 q)
    assert K - 64 <= k < (K // 64) * 64
    A[5, k] = np.inf
    B[k, :] = 1
    B[k, 7] = 0                     # Inf x 0
    with np.errstate(invalid="ignore"):
        ref = _oracle(C, A, B, M, N, K)
    As, Bs = _stored(A, B, flags)
    got = h.gpu_gemm_f16(C, As, Bs, M, N, K, flags=flags)
    assert np.array_equal(got, ref, equal_nan=True)
    assert np.isnan(got[5, 7]) and np.isposinf(got[5, 8])


@pytest.mark.parametrize("shape", [(1024, 1024, 1024), (1024, 1024, 4096), (1000, 1016, 784)])
def test_real_values_within_tolerance(dev, shape):
    M, N, K = shape
    assert _in_range(M, N, K, 1)
    h.announce("sph_gemm_f16f32 64 x 64 tiles, N(0, 1/sqrt(K)) operands", shape)
    A = synth.normal(71, (M, K), 1.0 / np.sqrt(K)).astype(np.float16)
    B = synth.normal(72, (K, N), 1.0 / np.sqrt(K)).astype(np.float16)
    C = synth.uniform(73, (M, N))
    got = h.gpu_gemm_f16(C, A, B, M, N, K)
    for lo in (0, M - 128):
        a32, b32 = A[lo:lo + 128].astype(np.float32), B.astype(np.float32)
        ref = po.gemm_rows(C[lo:lo + 128].copy(), a32, b32, 128, N, K, threads=8)
        assert h.normalised_error(got[lo:lo + 128], ref, np.abs(a32), np.abs(b32)) <= TOL_F16


def test_nothing_is_written_outside_out(dev):
    """Guard floats before and behind out, ragged M and N, accumulate and overwrite."""
    M, N, K = 1000, 1016, 136
    assert _in_range(M, N, K, 1)
    h.announce("sph_gemm_f16f32 64 x 64 tiles, guards", (M, N, K))
    A = synth.small_integers(81, (M, K), span=4).astype(np.float16)
    B = synth.small_integers(82, (K, N), span=4).astype(np.float16)
    C = synth.small_integers(83, (M, N), span=100)
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
