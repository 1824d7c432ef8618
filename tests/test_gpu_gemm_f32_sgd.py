"""sph_gemm_f32_sgd: out = out - ((A * B) * scale) * rate in one launch.

Bar: bit for bit against the device sequence it replaces -- the gradient stored by an
overwriting GEMM, scaled, and applied by the one-pass SGD step (itself bit-exact against the
CPU checker's Scale + Sub) -- on shapes that reach every kernel and epilogue: the K-split
kernel on 16 x 16 and 32 x 32 tiles, 64- and 128-tiles of the straight-to-LDS kernel, the tile
walk, the register-staged kernel on unaligned shapes, and the single-row reduction (the bias
gradient ones x dy)."""
import numpy as np
import pytest

from oracle import pyoracle as po
from sapphire_amd import capi, synth
from tests import helpers as h

pytestmark = pytest.mark.gpu

TA, TB, OW = capi.SPH_GEMM_TRANS_A, capi.SPH_GEMM_TRANS_B, capi.SPH_GEMM_OVERWRITE


def bits(x):
    return np.ascontiguousarray(x).view(np.uint32)


def _stored(A, B, flags):
    As = np.ascontiguousarray(A.T) if flags & TA else A
    Bs = np.ascontiguousarray(B.T) if flags & TB else B
    return As, Bs


# (M, N, K, flags): the weight gradients of the 784-1024-1024-10 network at batch 1024 (x^T dy),
# its bias gradients (ones x dy), and shapes for the remaining kernels
CASES = [(784, 1024, 1024, TA), (1024, 1024, 1024, TA), (1024, 10, 1024, TA),
         (1, 1024, 1024, 0), (1, 10, 1024, 0), (1, 70, 300, 0),
         (2048, 2048, 256, 0), (2048, 2048, 128, TA), (4096, 2048, 64, TB),
         (130, 70, 200, 0), (65, 33, 17, TA | TB), (5, 3, 9, TB), (256, 256, 96, 0),
         (32, 32, 1024, 0), (40, 24, 515, TA),
         # ragged extents that the launcher splits: N % 4 != 0, M % 4 != 0 with A stored K x M, a
         # K that ends in a partial step
         (512, 1026, 100, 0), (301, 262, 1001, TA), (1000, 999, 77, TB), (1001, 130, 64, TA | TB)]


@pytest.mark.parametrize("case", CASES)
def test_update_equals_gradient_scale_and_step(dev, case):
    M, N, K, flags = case
    h.announce("sph_gemm_f32_sgd", case)
    A = synth.uniform(901, (M, K))
    B = synth.uniform(902, (K, N))
    W = synth.uniform(903, (M, N))
    W[0, 0] = -0.0
    As, Bs = _stored(A, B, flags)
    for scale, rate in ((1.0, 0.01), (1.0 / 1024.0, 0.37)):
        dA, dB, dW = (capi.DeviceBuffer.from_array(v) for v in (As, Bs, W))
        capi.call("sph_gemm_f32_sgd", dW.ptr, dA.ptr, dB.ptr, M, N, K, scale, rate, flags)
        got = dW.download(np.float32, (M, N))
        # the sequence it replaces, on the device
        dG = capi.DeviceBuffer.from_array(np.full((M, N), np.float32(np.nan)))
        dZ = capi.DeviceBuffer.from_array(W)
        capi.call("sph_gemm_f32_ex", dG.ptr, dA.ptr, dB.ptr, M, N, K, 1, M * N, M * K, K * N,
                  flags | OW)
        if scale != 1.0:
            capi.call("sph_scale_f32", dG.ptr, dG.ptr, scale, M * N)
        capi.call("sph_sgd_step_f32", dZ.ptr, dG.ptr, rate, M * N)
        want = dZ.download(np.float32, (M, N))
        grad = dG.download(np.float32, (M, N))
        assert np.array_equal(bits(got), bits(want)), (scale, rate)
        # and the step itself as the CPU checker takes it from that gradient
        cpu = po.sgd(W, np.ascontiguousarray(grad), rate)
        assert np.array_equal(bits(got), bits(cpu))
        for d in (dA, dB, dW, dG, dZ):
            d.release()


def test_zero_k_and_bad_flags(dev):
    h.announce("sph_gemm_f32_sgd K = 0 / unknown flag")
    W = synth.uniform(911, (3, 4))
    one = np.zeros(1, np.float32)
    dW, dO = capi.DeviceBuffer.from_array(W), capi.DeviceBuffer.from_array(one)
    capi.call("sph_gemm_f32_sgd", dW.ptr, dO.ptr, dO.ptr, 3, 4, 0, 1.0, 0.5, 0)
    assert np.array_equal(bits(dW.download(np.float32, (3, 4))), bits(W))
    with pytest.raises(capi.SphError):
        capi.call("sph_gemm_f32_sgd", dW.ptr, dO.ptr, dO.ptr, 3, 4, 1, 1.0, 0.5, OW)
    dW.release()
    dO.release()
