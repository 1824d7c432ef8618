"""Seeded random shapes through the dense entry points, with guard words round out.

The shape lists straddle every kernel boundary (tile edges 16 / 32 / 64 / 128 / 256, K steps of
16 and 32, 16-byte alignment of rows), so that a change of the kernel selection cannot leave a
shape class without a kernel that handles it.  fp32: all flag combinations, tolerance
max |gpu - cpu| / sum_k |a b| <= 1e-4.  fp16: small-integer operands, so every product and sum is
exact and the comparison is bit for bit.
"""
import numpy as np
import pytest

from oracle import pyoracle as po
from sapphire_amd import capi, synth
from tests import helpers as h

pytestmark = pytest.mark.gpu

DIMS = [1, 2, 7, 10, 15, 16, 17, 31, 32, 33, 48, 63, 64, 65, 69, 96, 100, 127, 128, 129, 137, 200,
        256, 257, 300, 511, 512, 640, 1000, 1001, 1024]
DEPTHS = [1, 3, 8, 15, 16, 17, 18, 32, 40, 63, 64, 65, 67, 72, 96, 100, 128, 200, 256, 500, 512,
          515, 1001, 1024, 2048]
GUARD = 64


def _guarded(C):
    guard = np.full(GUARD, np.float32(-777.25), np.float32)
    return guard, np.concatenate([guard, C.ravel(), guard])


def _check_guards(back, guard):
    assert np.array_equal(back[:GUARD], guard), "write before the start of out"
    assert np.array_equal(back[-GUARD:], guard), "write past the end of out"


@pytest.mark.parametrize("block", range(10))
def test_fp32_flags_on_random_shapes(dev, block):
    rng = np.random.default_rng(9000 + block)
    for it in range(16):
        M, N, K = int(rng.choice(DIMS)), int(rng.choice(DIMS)), int(rng.choice(DEPTHS))
        flags = int(rng.integers(0, 8))
        h.announce("sph_gemm_f32_ex random", (M, N, K), "flags", flags)
        seed = 100000 * block + 10 * it
        A, B, C = synth.uniform(seed, (M, K)), synth.uniform(seed + 1, (K, N)), synth.uniform(seed + 2, (M, N))
        As = np.ascontiguousarray(A.T) if flags & capi.SPH_GEMM_TRANS_A else A
        Bs = np.ascontiguousarray(B.T) if flags & capi.SPH_GEMM_TRANS_B else B
        guard, padded = _guarded(C)
        dA, dB, dC = (capi.DeviceBuffer.from_array(x) for x in (As, Bs, padded))
        capi.call("sph_gemm_f32_ex", dC.at(4 * GUARD), dA.ptr, dB.ptr, M, N, K, 1, M * N, M * K,
                  K * N, flags)
        back = dC.download(np.float32, padded.shape)
        for d in (dA, dB, dC):
            d.release()
        _check_guards(back, guard)
        start = np.zeros_like(C) if flags & capi.SPH_GEMM_OVERWRITE else C
        ref = po.gemm_rows(start.copy(), A, B, M, N, K)
        err = h.normalised_error(back[GUARD:-GUARD].reshape(M, N), ref, np.abs(A), np.abs(B))
        assert err <= 1e-4, (M, N, K, flags, err)


@pytest.mark.parametrize("block", range(8))
def test_fp16_exact_on_random_shapes(dev, block):
    rng = np.random.default_rng(9100 + block)
    for it in range(16):
        M = int(rng.choice(DIMS))
        N = int(rng.choice(DIMS + [264, 520, 1004]))
        K = int(rng.choice(DEPTHS + [24, 88, 168, 1000]))
        batch = int(rng.choice([1, 1, 2, 3]))
        if block % 2 == 1:
            # small products run on the few-tile kernel: every other block raises the batch
            # until the tiled kernels take the shape
            while h.f16_few_tiles(M, N, batch):
                batch += 1
        # the first four blocks as they always were; the others with the operands stored
        # either way
        flags = (int(rng.choice([0, capi.SPH_GEMM_OVERWRITE])) if block < 4
                 else int(rng.integers(0, 8)))
        h.announce("sph_gemm_f16f32 random", (M, N, K, batch), "flags", flags)
        seed = 200000 * (block + 1) + 10 * it
        A = synth.small_integers(seed, (batch, M, K), span=3).astype(np.float16)
        B = synth.small_integers(seed + 1, (batch, K, N), span=3).astype(np.float16)
        C = synth.small_integers(seed + 2, (batch, M, N), span=100)
        guard, padded = _guarded(C)
        As = np.ascontiguousarray(A.swapaxes(1, 2)) if flags & capi.SPH_GEMM_TRANS_A else A
        Bs = np.ascontiguousarray(B.swapaxes(1, 2)) if flags & capi.SPH_GEMM_TRANS_B else B
        dA, dB, dC = (capi.DeviceBuffer.from_array(x) for x in (As, Bs, padded))
        capi.call("sph_gemm_f16f32", dC.at(4 * GUARD), dA.ptr, dB.ptr, M, N, K, batch, M * N,
                  M * K, K * N, flags)
        back = dC.download(np.float32, padded.shape)
        for d in (dA, dB, dC):
            d.release()
        _check_guards(back, guard)
        ref = po.gemm_rows(C.copy(), A.astype(np.float32), B.astype(np.float32), M, N, K,
                           batch=batch, threads=8)
        want = ref - C if flags & capi.SPH_GEMM_OVERWRITE else ref
        assert np.array_equal(back[GUARD:-GUARD].reshape(C.shape), want), (M, N, K, batch, flags)
