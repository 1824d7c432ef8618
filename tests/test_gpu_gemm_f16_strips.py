"""fp16-input / fp32-accumulate GEMM whose last rows and columns are cut off as thin strips: the
last N % 8 columns (and, of an A stored K x M, the last M % 8 rows) that the straight-to-LDS
copies cannot take, and up to 16 rows or columns past a multiple of the tile edge when that
spares the busiest compute unit a tile.  The strips are computed by the few-tile kernel's code on
the last workgroups of the body's launch, whichever of the tiled kernels the body takes.

Integer-valued operands make every product and partial sum exact, so body, strips and the seam
between them are checked bit for bit against the CPU loop; N(0, 1/sqrt(K)) operands are held to
the fp16 tolerance 1e-2.  Odd K and odd N put the rows of the operands at odd halves (read as
aligned dwords and shifted).
"""
import numpy as np
import pytest

from oracle import pyoracle as po
from sapphire_amd import capi, synth
from tests import helpers as h

pytestmark = pytest.mark.gpu
TOL_F16 = 1e-2
TA, TB, OW = capi.SPH_GEMM_TRANS_A, capi.SPH_GEMM_TRANS_B, capi.SPH_GEMM_OVERWRITE


def _oracle(C, A16, B16, M, N, K, batch=1):
    return po.gemm_rows(C.copy(), A16.astype(np.float32), B16.astype(np.float32), M, N, K,
                        batch=batch, threads=8)


def _stored(A, B, flags):
    As = np.ascontiguousarray(A.swapaxes(-1, -2)) if flags & TA else A
    Bs = np.ascontiguousarray(B.swapaxes(-1, -2)) if flags & TB else B
    return As, Bs


# (M, N, K, batch), by the kernel the body takes.
# 64 x 64 tiles: 17 x 17 cut to 16 x 16, odd and even K; N % 8 only; a batch.
# 128 x 128 tiles: 1100 x 2052 (N % 8 = 4), 2049 x 2056 (one row past 16 tile rows).
# 256 x 128 tiles: 3073 x 2050.   256 x 256 tiles: 4097 x 4100 (one row past 16 tile rows, 4
# columns past 16 tile columns), whole tiles with the old out added inside the K loop
# (4097 x 4097 x 1280) and in the epilogue (x 96).
# general kernel (K below one step of the copies): 1025 x 1030 x 24.
SHAPES = [(1025, 1025, 65, 1), (1025, 1025, 128, 1), (1000, 1004, 200, 1), (1032, 1027, 77, 1),
          (321, 323, 96, 6), (1100, 2052, 64, 1), (2049, 2056, 72, 1), (3073, 2050, 64, 1),
          (4097, 4100, 64, 1), (4097, 4097, 96, 1), (1025, 1030, 24, 1),
          # a batch on 256 x 256 tiles: 4 x (9 x 9) tiles cut to 4 x (8 x 8)
          (2049, 2052, 64, 4)]


@pytest.mark.parametrize("flags", [0, TA, TB, TA | TB])
@pytest.mark.parametrize("shape", SHAPES)
def test_exact_on_integers(dev, shape, flags):
    M, N, K, batch = shape
    h.announce("sph_gemm_f16f32 with edge strips, integer exactness", shape, "flags", flags)
    A = synth.small_integers(851, (batch, M, K), span=4).astype(np.float16)
    B = synth.small_integers(852, (batch, K, N), span=4).astype(np.float16)
    C = synth.small_integers(853, (batch, M, N), span=100)
    As, Bs = _stored(A, B, flags)
    ref = _oracle(C, A, B, M, N, K, batch=batch)
    got = h.gpu_gemm_f16(C, As, Bs, M, N, K, batch=batch, flags=flags)
    assert np.array_equal(got, ref)
    got = h.gpu_gemm_f16(C, As, Bs, M, N, K, batch=batch, flags=flags | OW)
    assert np.array_equal(got, ref - C)


def test_old_out_added_inside_the_loop_with_strips(dev):
    """4097 x 4097 x 1280: 40 K steps, so the 256-tile kernel adds the old contents of out inside
    its loop (the form that uses all of a compute unit's LDS, which the strips' workgroups
    borrow)."""
    M, N, K = 4097, 4097, 1280
    h.announce("sph_gemm_f16f32 256-tile kernel with strips, out added in the loop", (M, N, K))
    A = synth.small_integers(861, (M, K), span=2).astype(np.float16)
    B = synth.small_integers(862, (K, N), span=2).astype(np.float16)
    C = synth.small_integers(863, (M, N), span=100)
    got = h.gpu_gemm_f16(C, A, B, M, N, K)
    # the last rows (bottom strip and the last tile row), then the last columns of every row
    lo = M - 40
    ref = _oracle(C[lo:], A[lo:], B, M - lo, N, K)
    assert np.array_equal(got[lo:], ref)
    Bc = np.ascontiguousarray(B[:, N - 24:])
    ref = _oracle(np.ascontiguousarray(C[:, N - 24:]), A, Bc, M, 24, K)
    assert np.array_equal(got[:, N - 24:], ref)
    # and a band from the middle of the body
    ref = _oracle(C[2000:2064], A[2000:2064], B, 64, N, K)
    assert np.array_equal(got[2000:2064], ref)


@pytest.mark.parametrize("shape", [(1025, 1025, 1025), (1001, 1001, 1001), (2048, 2052, 512)])
def test_real_values_within_tolerance(dev, shape):
    M, N, K = shape
    h.announce("sph_gemm_f16f32 with edge strips, N(0, 1/sqrt(K)) operands", shape)
    A = synth.normal(871, (M, K), 1.0 / np.sqrt(K)).astype(np.float16)
    B = synth.normal(872, (K, N), 1.0 / np.sqrt(K)).astype(np.float16)
    C = synth.uniform(873, (M, N))
    got = h.gpu_gemm_f16(C, A, B, M, N, K)
    b32 = B.astype(np.float32)
    for lo in (0, M - 128):
        a32 = A[lo:lo + 128].astype(np.float32)
        ref = po.gemm_rows(C[lo:lo + 128].copy(), a32, b32, 128, N, K, threads=8)
        assert h.normalised_error(got[lo:lo + 128], ref, np.abs(a32), np.abs(b32)) <= TOL_F16


def test_nothing_is_written_outside_out(dev):
    """Guard floats before and behind out, accumulate and overwrite."""
    M, N, K = 1025, 1027, 72
    h.announce("sph_gemm_f16f32 with edge strips, guards", (M, N, K))
    A = synth.small_integers(881, (M, K), span=4).astype(np.float16)
    B = synth.small_integers(882, (K, N), span=4).astype(np.float16)
    C = synth.small_integers(883, (M, N), span=100)
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


@pytest.mark.parametrize("flags", [0, TB, TA])
@pytest.mark.parametrize("shape", [(128, 128, 4095), (100, 60, 1023), (16, 512, 2049),
                                   (256, 256, 2047), (128, 128, 4094)])
def test_few_tile_kernel_with_rows_at_odd_halves(dev, shape, flags):
    """Odd K: every second row of an operand stored with K contiguous starts at an odd half."""
    M, N, K = shape
    assert h.f16_few_tiles(M, N, 1, K)
    h.announce("sph_gemm_f16f32 few-tile kernel, odd K", shape, "flags", flags)
    A = synth.small_integers(891, (M, K), span=2).astype(np.float16)
    B = synth.small_integers(892, (K, N), span=2).astype(np.float16)
    C = synth.small_integers(893, (M, N), span=100)
    As, Bs = _stored(A, B, flags)
    got = h.gpu_gemm_f16(C, As, Bs, M, N, K, flags=flags)
    assert np.array_equal(got, _oracle(C, A, B, M, N, K))


def test_operands_that_start_at_an_odd_half(dev):
    """Bases 2 bytes past a 4-byte boundary with even pitches: every row starts at an odd half."""
    M, N, K = 120, 136, 514
    h.announce("sph_gemm_f16f32 few-tile kernel, bases at odd halves", (M, N, K))
    A = synth.small_integers(895, (M, K), span=3).astype(np.float16)
    B = synth.small_integers(896, (N, K), span=3).astype(np.float16)   # stored N x K
    C = synth.small_integers(897, (M, N), span=100)
    pad = np.zeros(1, np.float16)
    dA = capi.DeviceBuffer.from_array(np.concatenate([pad, A.ravel()]))
    dB = capi.DeviceBuffer.from_array(np.concatenate([pad, B.ravel()]))
    dC = capi.DeviceBuffer.from_array(C)
    assert dA.nbytes >= 2 * (M * K + 1) and dB.nbytes >= 2 * (N * K + 1) and dC.nbytes >= 4 * M * N
    capi.call("sph_gemm_f16f32", dC.ptr, dA.at(2), dB.at(2), M, N, K, 1, M * N, M * K, K * N, TB)
    got = dC.download(np.float32, (M, N))
    for d in (dA, dB, dC):
        d.release()
    assert np.array_equal(got, _oracle(C, A, np.ascontiguousarray(B.T), M, N, K))


@pytest.mark.parametrize("block", range(6))
def test_random_shapes_just_past_a_tile_grid(dev, block):
    """Seeded shapes a few rows and columns past multiples of 64, 128 and 256 with about one tile
    per compute unit, where the cut depends on both remainders; all flag combinations, integer
    operands (bit for bit), guard words."""
    rng = np.random.default_rng(9400 + block)
    for it in range(8):
        M = int(rng.choice([960, 1024, 1088, 2048, 4096])) + int(rng.integers(0, 19))
        N = int(rng.choice([960, 1024, 1088, 2048, 4096])) + int(rng.integers(0, 19))
        K = int(rng.choice([24, 33, 64, 65, 96, 130]))
        flags = int(rng.integers(0, 8))
        h.announce("sph_gemm_f16f32 random, past a tile grid", (M, N, K), "flags", flags)
        seed = 940000 + 100 * block + 3 * it
        A = synth.small_integers(seed, (M, K), span=3).astype(np.float16)
        B = synth.small_integers(seed + 1, (K, N), span=3).astype(np.float16)
        C = synth.small_integers(seed + 2, (M, N), span=100)
        As, Bs = _stored(A, B, flags)
        guard = np.full(64, np.float32(-777.25), np.float32)
        padded = np.concatenate([guard, C.ravel(), guard]).astype(np.float32)
        dA, dB, dC = (capi.DeviceBuffer.from_array(x) for x in (As, Bs, padded))
        assert dC.nbytes >= 4 * (128 + M * N) and dA.nbytes >= 2 * M * K and dB.nbytes >= 2 * K * N
        capi.call("sph_gemm_f16f32", dC.at(4 * 64), dA.ptr, dB.ptr, M, N, K, 1, M * N, M * K,
                  K * N, flags)
        back = dC.download(np.float32, padded.shape)
        for d in (dA, dB, dC):
            d.release()
        assert np.array_equal(back[:64], guard) and np.array_equal(back[-64:], guard)
        ref = _oracle(C, A, B, M, N, K)
        want = ref - C if flags & OW else ref
        assert np.array_equal(back[64:-64].reshape(M, N), want), (M, N, K, flags)
