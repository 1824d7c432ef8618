"""fp16-input / fp32-accumulate GEMM through the C ABI.

Oracle: the reference's fp32 CPU loop run on the fp16 inputs exactly widened to fp32, so only
the summation order differs.  Tolerance (fp16-in path): max_ij |gpu - cpu| / sum_k|a_ik b_kj|
<= 1e-2.  Integer-valued inputs make every product and partial sum exact, so tiling and
indexing are additionally checked bit for bit.
"""
import numpy as np
import pytest

from oracle import pyoracle as po
from sapphire_amd import capi, synth
from tests import helpers as h

pytestmark = pytest.mark.gpu
TOL_F16 = 1e-2


_both_kernel_families = h.f16_both_kernel_families


def _oracle(C, A16, B16, M, N, K, batch=1, sa=None, sb=None):
    A = A16.astype(np.float32)
    B = B16.astype(np.float32)
    return po.gemm_rows(C.copy(), A, B, M, N, K, batch=batch, stride_a=sa, stride_b=sb, threads=8)


# the 256-tile kernel is chosen from 192 tiles up (three quarters of the compute units): the
# batch count brings these small shapes there
# from 20 K steps up (K >= 640) the accumulating launch adds the old contents of out during the
# first steps of the loop instead of in the epilogue, a block every second step (K = 640: no
# step after the written-out prefix, 672 and 704: one and two steps after it) and from 36 steps
# up (K >= 1152) every fourth step (1152, 1184, 1216, 1280 likewise); 608 is the last K that
# reads out in the epilogue
@pytest.mark.parametrize("shape", [(256, 256, 64, 192), (256, 512, 128, 96), (512, 256, 192, 96),
                                   (768, 1024, 256, 16), (4096, 3072, 32, 1), (256, 256, 640, 192),
                                   (4096, 3072, 672, 1), (512, 256, 704, 96), (1024, 768, 1280, 16),
                                   (256, 512, 608, 96), (256, 256, 1152, 192), (512, 512, 1184, 48),
                                   (256, 1024, 1216, 48), (256, 512, 1120, 96)])
def test_tile256_exact_on_integers(dev, shape):
    M, N, K, batch = shape
    h.announce("sph_gemm_f16f32 tile256 integer exactness", shape)
    span = 4 if K <= 256 else 3      # every partial sum stays an exact fp32 integer
    A = synth.small_integers(1, (batch, M, K), span=span).astype(np.float16)
    B = synth.small_integers(2, (batch, K, N), span=span).astype(np.float16)
    C = synth.small_integers(3, (batch, M, N), span=100)
    ref = _oracle(C, A, B, M, N, K, batch=batch)
    got = h.gpu_gemm_f16(C, A, B, M, N, K, batch=batch)
    assert np.array_equal(got, ref)
    got = h.gpu_gemm_f16(C, A, B, M, N, K, batch=batch, flags=capi.SPH_GEMM_OVERWRITE)
    assert np.array_equal(got, ref - C)


# the same kernel with M and N that are not multiples of 256 (rows and column chunks clamped
# when copied, guarded epilogue): at least 192 tiles and three quarters of the tiled area real
@pytest.mark.parametrize("shape", [(250, 248, 64, 192), (500, 504, 96, 48), (4000, 3592, 32, 1),
                                   (3841, 4096, 64, 1)])
def test_tile256_ragged_exact_on_integers(dev, shape):
    M, N, K, batch = shape
    h.announce("sph_gemm_f16f32 ragged tile256 integer exactness", shape)
    A = synth.small_integers(21, (batch, M, K)).astype(np.float16)
    B = synth.small_integers(22, (batch, K, N)).astype(np.float16)
    C = synth.small_integers(23, (batch, M, N), span=100)
    ref = _oracle(C, A, B, M, N, K, batch=batch)
    got = h.gpu_gemm_f16(C, A, B, M, N, K, batch=batch)
    assert np.array_equal(got, ref)
    got = h.gpu_gemm_f16(C, A, B, M, N, K, batch=batch, flags=capi.SPH_GEMM_OVERWRITE)
    assert np.array_equal(got, ref - C)


# K = 32 q + r, 0 < r < 32.  The 256-tile kernel takes the window [K - 32, K) as a last
# step and masks the 32 - r values of k it has already multiplied (shapes with 192 tiles: whole
# and ragged tiles, old contents added in the epilogue, every second step (20 steps and more:
# K = 632 ends inside the written-out prefix, 648 after it) and every fourth (36 and more: 1144,
# 1168, 1176)) and the 128-tile kernel, with the operands stored plainly or the other way round.
@pytest.mark.parametrize("shape", _both_kernel_families(
    [(256, 256, 72, 192), (250, 248, 80, 192), (4096, 3072, 88, 1), (256, 256, 632, 192),
     (256, 256, 648, 192), (512, 256, 1144, 96), (512, 256, 1168, 96), (256, 512, 1176, 96),
     (500, 504, 680, 48), (300, 520, 168, 1), (128, 128, 72, 3), (1000, 1000, 1000, 1),
     # K % 8 != 0: rows of A (of a B stored N x K) start at addresses that are no multiples of 16
     # bytes, positions cleared one by one
     (256, 256, 65, 192), (248, 256, 100, 192), (4096, 3072, 77, 1), (512, 256, 1145, 96),
     (256, 256, 667, 192), (304, 520, 171, 1), (128, 128, 95, 3), (1000, 1000, 999, 1),
     (304, 517, 77, 3)]))
@pytest.mark.parametrize("flags", [0, capi.SPH_GEMM_TRANS_A, capi.SPH_GEMM_TRANS_B,
                                   capi.SPH_GEMM_TRANS_A | capi.SPH_GEMM_TRANS_B])
def test_k_tail_exact_on_integers(dev, shape, flags):
    M, N, K, batch = shape
    h.announce("sph_gemm_f16f32 K tail integer exactness", shape, "flags", flags)
    A = synth.small_integers(31, (batch, M, K), span=3).astype(np.float16)
    B = synth.small_integers(32, (batch, K, N), span=3).astype(np.float16)
    C = synth.small_integers(33, (batch, M, N), span=100)
    As = np.ascontiguousarray(A.swapaxes(1, 2)) if flags & capi.SPH_GEMM_TRANS_A else A
    Bs = np.ascontiguousarray(B.swapaxes(1, 2)) if flags & capi.SPH_GEMM_TRANS_B else B
    ref = _oracle(C, A, B, M, N, K, batch=batch)
    got = h.gpu_gemm_f16(C, As, Bs, M, N, K, batch=batch, flags=flags)
    assert np.array_equal(got, ref)
    got = h.gpu_gemm_f16(C, As, Bs, M, N, K, batch=batch, flags=flags | capi.SPH_GEMM_OVERWRITE)
    assert np.array_equal(got, ref - C)


@pytest.mark.parametrize("flags", [0, capi.SPH_GEMM_TRANS_A | capi.SPH_GEMM_TRANS_B])
@pytest.mark.parametrize("K", [72, 80, 88, 73, 83])
def test_k_tail_window_counts_an_infinity_once(dev, K, flags):
    """An infinity (and a 0 x Inf) at a k that lies in both of the last two step windows must
    come out exactly as in the CPU product: +Inf where the partner is positive, NaN where it is
    zero, and nothing else in the matrix may change."""
    M, N, batch = 256, 256, 192
    h.announce("sph_gemm_f16f32 K tail, Inf inside the repeated window", K)
    A = synth.small_integers(41, (batch, M, K), span=3).astype(np.float16)
    B = synth.small_integers(42, (batch, K, N), span=3).astype(np.float16)
    C = synth.small_integers(43, (batch, M, N), span=100)
    k = K - 20                      # inside [K - 32, 32 q) for r < 20
    A[:, 5, k] = np.inf
    B[:, k, :] = 1
    B[:, k, 7] = 0                  # Inf x 0
    with np.errstate(invalid="ignore"):
        ref = _oracle(C, A, B, M, N, K, batch=batch)
    As = np.ascontiguousarray(A.swapaxes(1, 2)) if flags & capi.SPH_GEMM_TRANS_A else A
    Bs = np.ascontiguousarray(B.swapaxes(1, 2)) if flags & capi.SPH_GEMM_TRANS_B else B
    got = h.gpu_gemm_f16(C, As, Bs, M, N, K, batch=batch, flags=flags)
    assert np.array_equal(got, ref, equal_nan=True)
    assert np.isnan(got[:, 5, 7]).all() and np.isposinf(got[:, 5, 8]).all()


@pytest.mark.parametrize("shape", _both_kernel_families(
    [(1, 1, 1), (5, 3, 2), (31, 33, 17), (64, 64, 32), (100, 72, 40), (128, 128, 64), (130, 254, 96),
     (200, 8, 1000), (257, 255, 63), (100, 68, 44), (300, 132, 100), (64, 70, 34)]))
def test_general_exact_on_integers(dev, shape):
    M, N, K, batch = shape
    h.announce("sph_gemm_f16f32 general integer exactness", shape)
    A = synth.small_integers(4, (batch, M, K), span=3).astype(np.float16)
    B = synth.small_integers(5, (batch, K, N), span=3).astype(np.float16)
    C = synth.small_integers(6, (batch, M, N), span=100)
    ref = _oracle(C, A, B, M, N, K, batch=batch)
    got = h.gpu_gemm_f16(C, A, B, M, N, K, batch=batch)
    assert np.array_equal(got, ref)


# K % 32 == 0 and N % 8 == 0 without being whole 256-tiles: the straight-to-LDS 128-tile kernel,
# with clamped rows (M ragged) and clamped column chunks (N ragged), one and many tiles
@pytest.mark.parametrize("shape", _both_kernel_families(
    [(1, 8, 32), (64, 64, 32), (100, 136, 64), (130, 72, 96), (257, 264, 32), (128, 128, 512),
     (300, 520, 160), (1000, 1000, 992), (512, 384, 2048)]))
def test_dma128_exact_on_integers(dev, shape):
    M, N, K, batch = shape
    h.announce("sph_gemm_f16f32 128-tile integer exactness", shape)
    A = synth.small_integers(14, (batch, M, K), span=3).astype(np.float16)
    B = synth.small_integers(15, (batch, K, N), span=3).astype(np.float16)
    C = synth.small_integers(16, (batch, M, N), span=100)
    ref = _oracle(C, A, B, M, N, K, batch=batch)
    got = h.gpu_gemm_f16(C, A, B, M, N, K, batch=batch)
    assert np.array_equal(got, ref)
    got = h.gpu_gemm_f16(C, A, B, M, N, K, batch=batch, flags=capi.SPH_GEMM_OVERWRITE)
    assert np.array_equal(got, ref - C)


# the 128-tile kernel runs eight wavefronts per tile up to one tile per compute unit (all shapes
# above) and four beyond that: more than 256 tiles of 128 x 128 that are not 192 whole 256-tiles,
# plain, with a K tail, and with transposed operands
@pytest.mark.parametrize("flags", [0, capi.SPH_GEMM_TRANS_A, capi.SPH_GEMM_TRANS_B,
                                   capi.SPH_GEMM_TRANS_A | capi.SPH_GEMM_TRANS_B])
@pytest.mark.parametrize("shape", [(128, 128, 64, 300), (200, 136, 96, 80), (120, 256, 72, 160)])
def test_dma128_four_wavefront_form_exact_on_integers(dev, shape, flags):
    M, N, K, batch = shape     # (the K tail with transposed operands runs on the general kernel)
    h.announce("sph_gemm_f16f32 128-tile, many tiles, integer exactness", shape, "flags", flags)
    A = synth.small_integers(17, (batch, M, K), span=3).astype(np.float16)
    B = synth.small_integers(18, (batch, K, N), span=3).astype(np.float16)
    C = synth.small_integers(19, (batch, M, N), span=100)
    ref = _oracle(C, A, B, M, N, K, batch=batch)
    As = np.ascontiguousarray(A.swapaxes(1, 2)) if flags & capi.SPH_GEMM_TRANS_A else A
    Bs = np.ascontiguousarray(B.swapaxes(1, 2)) if flags & capi.SPH_GEMM_TRANS_B else B
    got = h.gpu_gemm_f16(C, As, Bs, M, N, K, batch=batch, flags=flags)
    assert np.array_equal(got, ref)


@pytest.mark.parametrize("flags", [capi.SPH_GEMM_TRANS_A, capi.SPH_GEMM_TRANS_B,
                                   capi.SPH_GEMM_TRANS_A | capi.SPH_GEMM_TRANS_B])
@pytest.mark.parametrize("shape", _both_kernel_families(
    [(1, 1, 1, 1), (5, 3, 2, 1), (64, 64, 32, 1), (100, 72, 40, 2), (130, 254, 96, 1),
     (257, 255, 63, 1), (256, 512, 128, 3), (300, 136, 1000, 1), (8, 8, 32, 1), (136, 264, 64, 2),
     (1000, 1000, 992, 1), (512, 384, 2048, 1), (129, 136, 96, 1), (256, 256, 64, 192),
     (512, 256, 1184, 96), (256, 512, 704, 96), (248, 256, 96, 192), (4096, 3072, 32, 1),
     (504, 496, 64, 48)]))
def test_transposed_operands_exact_on_integers(dev, shape, flags):
    """A stored K x M and / or B stored N x K: the same product as with the operands stored
    plainly, bit for bit on integer-valued inputs: the 256-tile kernel (whole and ragged tiles,
    with the old contents of out added in the loop or in the epilogue) from 192 tiles up, the
    straight-to-LDS 128-tile kernel below that when K is a multiple of 32, N of 8 (and M of 8
    for a transposed A), the general kernel otherwise."""
    M, N, K, batch = shape
    h.announce("sph_gemm_f16f32 transposed operands", shape, "flags", flags)
    A = synth.small_integers(41, (batch, M, K), span=3).astype(np.float16)
    B = synth.small_integers(42, (batch, K, N), span=3).astype(np.float16)
    C = synth.small_integers(43, (batch, M, N), span=100)
    As = np.ascontiguousarray(A.swapaxes(1, 2)) if flags & capi.SPH_GEMM_TRANS_A else A
    Bs = np.ascontiguousarray(B.swapaxes(1, 2)) if flags & capi.SPH_GEMM_TRANS_B else B
    ref = _oracle(C, A, B, M, N, K, batch=batch)
    got = h.gpu_gemm_f16(C, As, Bs, M, N, K, batch=batch, flags=flags)
    assert np.array_equal(got, ref)
    got = h.gpu_gemm_f16(C, As, Bs, M, N, K, batch=batch, flags=flags | capi.SPH_GEMM_OVERWRITE)
    assert np.array_equal(got, ref - C)


# N = 8 q + r, r != 0: the first 8 q
# columns on the straight-to-LDS kernels (rows of B and of out start at addresses that are no
# multiples of 16 bytes), the last r on the few-tile kernel.  (M, N, K, batch): 128-tile kernel
# with four and with eight wavefronts, ragged and whole 256-tiles (old values of out added in the
# epilogue, K = 64, or in the loop, K = 640), N % 4 == 0, N % 2 == 0 and odd N, a K tail on top.
@pytest.mark.parametrize("flags", [0, capi.SPH_GEMM_TRANS_A, capi.SPH_GEMM_TRANS_B,
                                   capi.SPH_GEMM_TRANS_A | capi.SPH_GEMM_TRANS_B])
@pytest.mark.parametrize("shape", _both_kernel_families(
    [(512, 132, 64, 1), (200, 1030, 96, 2), (304, 517, 64, 3), (128, 135, 32, 300),
     (4096, 3076, 64, 1), (256, 257, 64, 192), (256, 260, 640, 192), (1000, 999, 992, 1),
     (248, 250, 72, 3),
     # narrow products: 8 or 96 columns on the 128-tile kernel and the rest, or all of fewer than
     # 8 columns, on the few-tile kernel
     (1024, 10, 1024, 1), (304, 100, 96, 2), (512, 5, 64, 3), (1000, 7, 1001, 1), (40, 3, 32, 1)]))
def test_column_count_not_a_multiple_of_eight(dev, shape, flags):
    M, N, K, batch = shape
    h.announce("sph_gemm_f16f32, N % 8 != 0", shape, "flags", flags)
    span = 4 if K <= 256 else 3
    A = synth.small_integers(61, (batch, M, K), span=span).astype(np.float16)
    B = synth.small_integers(62, (batch, K, N), span=span).astype(np.float16)
    C = synth.small_integers(63, (batch, M, N), span=100)
    As = np.ascontiguousarray(A.swapaxes(1, 2)) if flags & capi.SPH_GEMM_TRANS_A else A
    Bs = np.ascontiguousarray(B.swapaxes(1, 2)) if flags & capi.SPH_GEMM_TRANS_B else B
    ref = _oracle(C, A, B, M, N, K, batch=batch)
    # 37 guard floats after every unit of out: nothing may be written past column N - 1
    pad = 37
    padded = np.full((batch, M * N + pad), np.float32(-777.25), np.float32)
    padded[:, :M * N] = C.reshape(batch, M * N)
    for extra in (0, capi.SPH_GEMM_OVERWRITE):
        got = h.gpu_gemm_f16(padded, As, Bs, M, N, K, batch=batch, stride_out=M * N + pad,
                             flags=flags | extra)
        assert np.array_equal(got[:, M * N:], padded[:, M * N:]), "guard floats overwritten"
        want = ref - C if extra else ref
        assert np.array_equal(got[:, :M * N].reshape(batch, M, N), want)


# A stored K x M with M = 8 q + r, r != 0 (and N % 8 != 0 on top): the first 8 q rows as before,
# the last r rows (columns) by a launch of the few-tile kernel over that strip.
# 257 x 256 x 640 x 192: the whole-tile kernel with the old values added in its loop on top, 8 rows
# below it; 4095 x 3077: ragged 256-tiles.
@pytest.mark.parametrize("flags", [capi.SPH_GEMM_TRANS_A, capi.SPH_GEMM_TRANS_A | capi.SPH_GEMM_TRANS_B])
@pytest.mark.parametrize("shape", _both_kernel_families(
    [(517, 304, 64, 3), (1001, 999, 96, 1), (4095, 3077, 77, 1), (143, 143, 64, 5),
     (257, 256, 640, 192), (137, 136, 32, 1)]))
def test_transposed_a_with_ragged_rows_and_columns(dev, shape, flags):
    M, N, K, batch = shape
    h.announce("sph_gemm_f16f32, A stored K x M, M % 8 != 0", shape, "flags", flags)
    span = 4 if K <= 256 else 3
    A = synth.small_integers(81, (batch, M, K), span=span).astype(np.float16)
    B = synth.small_integers(82, (batch, K, N), span=span).astype(np.float16)
    C = synth.small_integers(83, (batch, M, N), span=100)
    As = np.ascontiguousarray(A.swapaxes(1, 2))
    Bs = np.ascontiguousarray(B.swapaxes(1, 2)) if flags & capi.SPH_GEMM_TRANS_B else B
    ref = _oracle(C, A, B, M, N, K, batch=batch)
    pad = 37
    padded = np.full((batch, M * N + pad), np.float32(-777.25), np.float32)
    padded[:, :M * N] = C.reshape(batch, M * N)
    for extra in (0, capi.SPH_GEMM_OVERWRITE):
        got = h.gpu_gemm_f16(padded, As, Bs, M, N, K, batch=batch, stride_out=M * N + pad,
                             flags=flags | extra)
        assert np.array_equal(got[:, M * N:], padded[:, M * N:]), "guard floats overwritten"
        want = ref - C if extra else ref
        assert np.array_equal(got[:, :M * N].reshape(batch, M, N), want)


# The few-tile kernel: 32-wide tiles, 16-wide tiles with 4 and (K >= 1024, at most one tile per
# compute unit) 16 wavefronts, K that ends inside a group of 16 or 32 values of k or inside a
# fragment of 8, fewer values of k than one fragment, single rows and columns, every storage
# order, with guard floats behind every unit of out.
@pytest.mark.parametrize("flags", [0, capi.SPH_GEMM_TRANS_A, capi.SPH_GEMM_TRANS_B,
                                   capi.SPH_GEMM_TRANS_A | capi.SPH_GEMM_TRANS_B])
@pytest.mark.parametrize("shape", [(252, 1020, 1024, 1), (100, 1024, 784, 1), (300, 300, 300, 1),
                                   (500, 500, 300, 1), (96, 1024, 1024, 1),
                                   (128, 128, 4096, 1), (64, 64, 8203, 1), (33, 47, 5, 1),
                                   (17, 16, 31, 2), (1, 1000, 37, 1), (1000, 1, 1029, 1),
                                   (255, 257, 1031, 1), (508, 510, 515, 1), (96, 80, 1040, 3),
                                   (2048, 10, 300, 1), (16, 4000, 64, 1)])
def test_few_tile_kernel_exact_on_integers(dev, shape, flags):
    M, N, K, batch = shape
    assert h.f16_few_tiles(M, N, batch, K)
    h.announce("sph_gemm_f16f32 few-tile kernel", shape, "flags", flags)
    A = synth.small_integers(91, (batch, M, K), span=3).astype(np.float16)
    B = synth.small_integers(92, (batch, K, N), span=3).astype(np.float16)
    C = synth.small_integers(93, (batch, M, N), span=100)
    As = np.ascontiguousarray(A.swapaxes(1, 2)) if flags & capi.SPH_GEMM_TRANS_A else A
    Bs = np.ascontiguousarray(B.swapaxes(1, 2)) if flags & capi.SPH_GEMM_TRANS_B else B
    ref = _oracle(C, A, B, M, N, K, batch=batch)
    pad = 37
    padded = np.full((batch, M * N + pad), np.float32(-777.25), np.float32)
    padded[:, :M * N] = C.reshape(batch, M * N)
    for extra in (0, capi.SPH_GEMM_OVERWRITE):
        got = h.gpu_gemm_f16(padded, As, Bs, M, N, K, batch=batch, stride_out=M * N + pad,
                             flags=flags | extra)
        assert np.array_equal(got[:, M * N:], padded[:, M * N:]), "guard floats overwritten"
        want = ref - C if extra else ref
        assert np.array_equal(got[:, :M * N].reshape(batch, M, N), want)


@pytest.mark.parametrize("flags", [0, capi.SPH_GEMM_TRANS_A | capi.SPH_GEMM_TRANS_B])
def test_few_tile_kernel_operands_at_two_byte_aligned_addresses(dev, flags):
    M, N, K = 200, 264, 99
    h.announce("sph_gemm_f16f32 few-tile kernel, A and B 2 bytes past a 16-byte boundary", flags)
    A = synth.small_integers(94, (M, K)).astype(np.float16)
    B = synth.small_integers(95, (K, N)).astype(np.float16)
    C = synth.small_integers(96, (M, N), span=100)
    ref = _oracle(C, A, B, M, N, K)
    As = np.ascontiguousarray(A.T) if flags & capi.SPH_GEMM_TRANS_A else A
    Bs = np.ascontiguousarray(B.T) if flags & capi.SPH_GEMM_TRANS_B else B
    one = np.zeros(1, np.float16)
    dA = capi.DeviceBuffer.from_array(np.concatenate([one, As.ravel()]))
    dB = capi.DeviceBuffer.from_array(np.concatenate([one, Bs.ravel()]))
    dC = capi.DeviceBuffer.from_array(C)
    capi.call("sph_gemm_f16f32", dC.ptr, dA.ptr + 2, dB.ptr + 2, M, N, K, 1, M * N, M * K, K * N,
              flags)
    got = dC.download(np.float32, C.shape)
    for d in (dA, dB, dC):
        d.release()
    assert np.array_equal(got, ref)


def test_few_tile_kernel_real_values_within_tolerance(dev):
    """N(0, 0.1) operands, a shared A (stride 0) and a K that ends inside a fragment."""
    M, N, K, batch = 100, 520, 787, 3
    h.announce("sph_gemm_f16f32 few-tile kernel, real values", (M, N, K, batch))
    A = synth.normal(97, (1, M, K), 0.1).astype(np.float16)
    B = synth.normal(98, (batch, K, N), 0.1).astype(np.float16)
    C = synth.uniform(99, (batch, M, N))
    ref = _oracle(C, A, B, M, N, K, batch=batch, sa=0)
    got = h.gpu_gemm_f16(C, A, B, M, N, K, batch=batch, stride_a=0)
    for b in range(batch):
        err = h.normalised_error(got[b], ref[b], np.abs(A[0]).astype(np.float32),
                                 np.abs(B[b]).astype(np.float32))
        assert err <= TOL_F16


def test_rows_of_b_that_start_anywhere(dev):
    """A K x N matrix B that begins 2 bytes past a 16-byte boundary (and N % 8 == 0): its rows are
    copied straight into LDS from addresses that are only 2-byte aligned."""
    M, N, K = 1024, 264, 96     # enough tiles for the tiled kernels
    h.announce("sph_gemm_f16f32, B at a 2-byte-aligned address", (M, N, K))
    A = synth.small_integers(71, (M, K)).astype(np.float16)
    B = synth.small_integers(72, (K, N)).astype(np.float16)
    C = synth.small_integers(73, (M, N), span=100)
    ref = _oracle(C, A, B, M, N, K)
    shifted = np.concatenate([np.zeros(1, np.float16), B.ravel()])
    dA, dB, dC = (capi.DeviceBuffer.from_array(x) for x in (A, shifted, C))
    capi.call("sph_gemm_f16f32", dC.ptr, dA.ptr, dB.ptr + 2, M, N, K, 1, M * N, M * K, K * N, 0)
    got = dC.download(np.float32, C.shape)
    for d in (dA, dB, dC):
        d.release()
    assert np.array_equal(got, ref)


@pytest.mark.parametrize("batch", [3, 8])
def test_dma128_batched_with_shared_operand(dev, batch):
    # batch 3: few-tile kernel; batch 8: 128-tile kernel
    h.announce("sph_gemm_f16f32 batch", batch, "strideA = 0")
    M, N, K = 200, 136, 96
    A = synth.normal(17, (1, M, K), 0.1).astype(np.float16)
    B = synth.normal(18, (batch, K, N), 0.1).astype(np.float16)
    C = synth.uniform(19, (batch, M, N))
    ref = _oracle(C, A, B, M, N, K, batch=batch, sa=0)
    got = h.gpu_gemm_f16(C, A, B, M, N, K, batch=batch, stride_a=0)
    for b in range(batch):
        err = h.normalised_error(got[b], ref[b], np.abs(A[0]).astype(np.float32),
                                 np.abs(B[b]).astype(np.float32))
        assert err <= TOL_F16


def test_batched_and_broadcast(dev):
    h.announce("sph_gemm_f16f32 batch 192, strideB = 0, tile256 path")
    M, N, K, batch = 256, 256, 128, 192
    A = synth.normal(7, (batch, M, K), 0.1).astype(np.float16)
    B = synth.normal(8, (1, K, N), 0.1).astype(np.float16)
    C = synth.uniform(9, (batch, M, N))
    ref = _oracle(C, A, B, M, N, K, batch=batch, sb=0)
    got = h.gpu_gemm_f16(C, A, B, M, N, K, batch=batch, stride_b=0)
    for b in range(batch):
        err = h.normalised_error(got[b], ref[b], np.abs(A[b]).astype(np.float32),
                                 np.abs(B[0]).astype(np.float32))
        assert err <= TOL_F16
    for batch in (4, 30):     # few-tile kernel, general kernel
        h.announce("sph_gemm_f16f32 batch", batch, "K % 8 != 0, strideA = 0")
        M, N, K = 70, 90, 50
        A = synth.normal(10, (1, M, K), 0.1).astype(np.float16)
        B = synth.normal(11, (batch, K, N), 0.1).astype(np.float16)
        C = synth.uniform(12, (batch, M, N))
        ref = _oracle(C, A, B, M, N, K, batch=batch, sa=0)
        got = h.gpu_gemm_f16(C, A, B, M, N, K, batch=batch, stride_a=0)
        for b in range(batch):
            err = h.normalised_error(got[b], ref[b], np.abs(A[0]).astype(np.float32),
                                     np.abs(B[b]).astype(np.float32))
            assert err <= TOL_F16


def test_config3_4096_cubed(dev):
    """The headline shape: M = N = K = 4096, N(0, 1/sqrt(K)) fp16 inputs, C zeros."""
    h.announce("sph_gemm_f16f32 config3 4096^3")
    d = synth.config3()
    n = 4096
    ref = _oracle(d["C"], d["A"], d["B"], n, n, n)
    got = h.gpu_gemm_f16(d["C"], d["A"], d["B"], n, n, n)
    den = np.abs(d["A"]).astype(np.float32) @ np.abs(d["B"]).astype(np.float32)
    err = h.normalised_error(got, ref, None, den.astype(np.float64), True)
    assert np.isfinite(got).all()
    assert err <= TOL_F16, err
    # the same data with the overwrite flag must give the same bits (C is zero)
    got2 = h.gpu_gemm_f16(d["C"], d["A"], d["B"], n, n, n, flags=capi.SPH_GEMM_OVERWRITE)
    assert np.array_equal(got, got2)
    # linearity in the accumulator, size-independent: run again on top of the result
    dA, dB, dC = (capi.DeviceBuffer.from_array(x) for x in (d["A"], d["B"], got))
    capi.call("sph_gemm_f16f32", dC.ptr, dA.ptr, dB.ptr, n, n, n, 1, n * n, n * n, n * n, 0)
    twice = dC.download(np.float32, got.shape)
    for x in (dA, dB, dC):
        x.release()
    # the old contents join the sum during the first K steps, so out + A*B is associated
    # differently from "sum, then one add": equal within the accumulation error, not bit for bit
    assert h.normalised_error(twice, got + got, None, den.astype(np.float64), True) <= 1e-5
    # real-valued out of the size of the product
    C = synth.uniform(91, (n, n))
    ref = _oracle(C, d["A"], d["B"], n, n, n)
    got = h.gpu_gemm_f16(C, d["A"], d["B"], n, n, n)
    err = h.normalised_error(got, ref, None, den.astype(np.float64) + np.abs(C), True)
    assert err <= TOL_F16, err
    assert float(np.max(np.abs(got - ref))) <= 1e-4


def test_convert_f32_to_f16_matches_numpy_rounding(dev):
    h.announce("sph_convert_f32_to_f16")
    x = np.concatenate([synth.normal(13, (100003,), 3.0),
                        np.array([0.0, -0.0, 65504.0, 65520.0, 1e-8, 6e-8, -7e4, np.inf],
                                 np.float32)])
    dX = capi.DeviceBuffer.from_array(x)
    dY = capi.DeviceBuffer(2 * x.size)
    capi.call("sph_convert_f32_to_f16", dY.ptr, dX.ptr, x.size)
    got = dY.download(np.uint16, x.shape)
    with np.errstate(over="ignore"):
        want = x.astype(np.float16).view(np.uint16)
    assert np.array_equal(got, want)
    dX.release()
    dY.release()
