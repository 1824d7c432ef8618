"""Edge values through the GEMM and CSR x dense kernels against the CPU checker: fp16 and fp32
subnormal operands (a flush to zero anywhere on the way to or inside the matrix cores shows as
a wrong bit), and +-Inf / NaN in the operands and in out (propagation equal to the CPU loop's
element by element: the same elements are NaN, the same are +Inf or -Inf, the finite ones are
within the path's tolerance).  NaN payloads and signs are not compared: the host's invalid
operations produce the negative default NaN, the device's the positive one."""
import numpy as np
import pytest

from oracle import pyoracle as po
from sapphire_amd import capi, synth
from tests import helpers as h

pytestmark = pytest.mark.gpu


def bits(x):
    return np.ascontiguousarray(x).view(np.uint32)


def same_specials(got, ref, tol, den):
    """NaN and Inf patterns identical, finite elements within tol * den."""
    assert np.array_equal(np.isnan(got), np.isnan(ref)), "NaN pattern differs"
    assert np.array_equal(np.isposinf(got), np.isposinf(ref)), "+Inf pattern differs"
    assert np.array_equal(np.isneginf(got), np.isneginf(ref)), "-Inf pattern differs"
    fin = np.isfinite(ref)
    if fin.any():
        err = np.abs(got[fin].astype(np.float64) - ref[fin]) / np.maximum(den[fin], 1e-300)
        assert float(err.max()) <= tol, float(err.max())


# ---- subnormals -----------------------------------------------------------------------------

# every kernel of the fp16 entry: 256-tiles with and without the in-loop accumulate, few-tile
# (32- and 16-wide tiles), 128-tiles, general
F16_SHAPES = [(256, 256, 64, 192), (256, 256, 1152, 192), (128, 136, 96, 1), (70, 50, 44, 1),
              (128, 136, 96, 20), (70, 50, 44, 50), (300, 200, 1100, 1)]


@pytest.mark.parametrize("shape", F16_SHAPES)
def test_f16_subnormal_operands_are_not_flushed(dev, shape):
    """A and B hold only fp16 subnormals m * 2^-24 with |m| <= 15 (and zeros): every product
    m1*m2 * 2^-48 and every partial sum is exact in fp32, so the result must equal the CPU
    loop bit for bit; a flush to zero of the inputs would give all zeros."""
    M, N, K, batch = shape
    h.announce("sph_gemm_f16f32 subnormal operands", shape)
    A = (synth.small_integers(201, (batch, M, K), span=15) * np.float32(2.0 ** -24)).astype(np.float16)
    B = (synth.small_integers(202, (batch, K, N), span=15) * np.float32(2.0 ** -24)).astype(np.float16)
    assert np.all(np.abs(A.astype(np.float32)) < 6.2e-5) and np.any(A != 0)   # below 2^-14
    C = np.zeros((batch, M, N), np.float32)
    ref = po.gemm_rows(C.copy(), A.astype(np.float32), B.astype(np.float32), M, N, K, batch=batch,
                       threads=8)
    assert np.count_nonzero(ref) > ref.size // 2
    got = h.gpu_gemm_f16(C, A, B, M, N, K, batch=batch)
    assert np.array_equal(bits(got), bits(ref))


@pytest.mark.parametrize("shape", F16_SHAPES)
def test_f16_subnormal_times_normal(dev, shape):
    """Subnormal A (m * 2^-24) against small-integer B, old contents of out of the same scale:
    exact again, bit for bit."""
    M, N, K, batch = shape
    h.announce("sph_gemm_f16f32 subnormal x normal", shape)
    A = (synth.small_integers(203, (batch, M, K), span=7) * np.float32(2.0 ** -24)).astype(np.float16)
    B = synth.small_integers(204, (batch, K, N), span=3).astype(np.float16)
    C = synth.small_integers(205, (batch, M, N), span=50) * np.float32(2.0 ** -24)
    ref = po.gemm_rows(C.copy(), A.astype(np.float32), B.astype(np.float32), M, N, K, batch=batch,
                       threads=8)
    got = h.gpu_gemm_f16(C, A, B, M, N, K, batch=batch)
    assert np.array_equal(bits(got), bits(ref))


# every kernel of the fp32 entry: 128- and 64-tiles, K-split tiles, general, single row
F32_SHAPES = [(512, 512, 64), (256, 256, 256), (64, 64, 512), (70, 50, 44), (1, 300, 128)]


@pytest.mark.parametrize("shape", F32_SHAPES)
def test_f32_subnormal_operands_and_results(dev, shape):
    """A holds fp32 subnormals m * 2^-149, B small integers: products and sums are exact
    subnormals (or small normals after the scaled out is added); bit for bit."""
    M, N, K = shape
    h.announce("sph_gemm_f32 subnormal operands", shape)
    A = synth.small_integers(211, (M, K), span=7) * np.float32(2.0 ** -149)
    A = A.astype(np.float32)
    assert np.all(np.abs(A) < 1.2e-38) and np.any(A != 0)
    B = synth.small_integers(212, (K, N), span=3)
    C = (synth.small_integers(213, (M, N), span=50) * np.float32(2.0 ** -149)).astype(np.float32)
    ref = po.gemm_rows(C.copy(), A, B, M, N, K, threads=8)
    assert np.count_nonzero(ref) > ref.size // 2
    got = h.gpu_gemm_f32(C, A, B, M, N, K)
    assert np.array_equal(bits(got), bits(ref))


# ---- Inf and NaN ----------------------------------------------------------------------------

def _sprinkle(x, seed, what):
    """Puts `what` at a few fixed pseudo-random places of a copy of x."""
    y = x.copy().reshape(-1)
    idx = (synth.bits64(seed, 6) % np.uint64(y.size)).astype(np.int64)
    for i, v in zip(idx, what * 6):
        y[i] = v
    return y.reshape(x.shape)


SPECIALS = [np.inf, -np.inf, np.nan]


@pytest.mark.parametrize("shape", F32_SHAPES)
def test_f32_inf_nan_propagate_like_the_cpu_loop(dev, shape):
    M, N, K = shape
    h.announce("sph_gemm_f32 Inf / NaN", shape)
    A = _sprinkle(synth.uniform(221, (M, K)), 1, SPECIALS)
    B = _sprinkle(synth.uniform(222, (K, N)), 2, SPECIALS)
    B[0, :] = 0.0                                  # zeros meet the Inf of A: Inf * 0 = NaN
    C = _sprinkle(synth.uniform(223, (M, N)), 3, SPECIALS)
    with np.errstate(all="ignore"):
        ref = po.gemm_rows(C.copy(), A, B, M, N, K, threads=8)
        den = np.abs(np.nan_to_num(A, nan=0, posinf=0, neginf=0)).astype(np.float64) @ \
            np.abs(np.nan_to_num(B, nan=0, posinf=0, neginf=0)).astype(np.float64) + 1.0
    assert np.isnan(ref).any() and (M == 1 or np.isfinite(ref).any())   # one row: all NaN
    got = h.gpu_gemm_f32(C, A, B, M, N, K)
    same_specials(got, ref, 1e-4, den)


@pytest.mark.parametrize("shape", F16_SHAPES)
def test_f16_inf_nan_propagate_like_the_cpu_loop(dev, shape):
    M, N, K, batch = shape
    h.announce("sph_gemm_f16f32 Inf / NaN", shape)
    A = _sprinkle(synth.normal(231, (batch, M, K), 0.1), 4, SPECIALS).astype(np.float16)
    B = _sprinkle(synth.normal(232, (batch, K, N), 0.1), 5, SPECIALS).astype(np.float16)
    B[:, 0, :] = 0.0
    C = _sprinkle(synth.uniform(233, (batch, M, N)), 6, SPECIALS)
    A32, B32 = A.astype(np.float32), B.astype(np.float32)
    with np.errstate(all="ignore"):
        ref = po.gemm_rows(C.copy(), A32, B32, M, N, K, batch=batch, threads=8)
        den = np.abs(np.nan_to_num(A32, nan=0, posinf=0, neginf=0)).astype(np.float64) @ \
            np.abs(np.nan_to_num(B32, nan=0, posinf=0, neginf=0)).astype(np.float64) + 1.0
    assert np.isnan(ref).any() and np.isfinite(ref).any()
    got = h.gpu_gemm_f16(C, A, B, M, N, K, batch=batch)
    same_specials(got, ref, 1e-2, den)


def test_spmm_inf_nan_follow_the_storage_order_loop(dev):
    """Inf / NaN among the stored values and in rows of B that are referenced propagate as in
    the CPU loop; Inf / NaN in rows of B that no entry references do not reach the result --
    which is where the CSR product differs from the dense leaf on the densified matrix (that
    one adds 0 * Inf = NaN)."""
    M, K, N = 300, 500, 64
    h.announce("sph_spmm_csr_f32 Inf / NaN")
    v, col, row = synth.csr_matrix(241, M, K, 2.0)
    v = _sprinkle(v, 7, SPECIALS)
    B = synth.uniform(242, (K, N))
    used = np.zeros(K, bool)
    used[col] = True
    unused = np.flatnonzero(~used)
    assert unused.size >= 3 and used.sum() >= 3
    B[unused[0], :] = np.inf
    B[unused[1], 5] = np.nan
    hot = np.flatnonzero(used)[:3]
    B[hot[0], 3] = np.inf
    B[hot[1], 7] = -np.inf
    B[hot[2], 11] = np.nan
    with np.errstate(all="ignore"):
        ref = po.spmm_csr(np.zeros((M, N), np.float32), v, col, row, M, N, B)
    assert np.isnan(ref).any() and np.isinf(ref).any()
    got = h.gpu_spmm(np.ones((M, N), np.float32), v, col, row, M, K, N, B, False, canary=64)
    assert np.array_equal(np.isnan(got), np.isnan(ref))
    ok = ~np.isnan(ref)
    assert np.array_equal(bits(got)[ok], bits(ref)[ok])
    # the dense leaf on the densified matrix turns every row NaN in the columns where an
    # unreferenced row of B holds Inf or NaN; the CSR loop does not
    with np.errstate(all="ignore"):
        dense = po.naive_gemm(np.zeros((M, N), np.float32), synth.densify(v, col, row, M, K), B,
                              M, N, K)
    assert np.isnan(dense[:, 0]).all() and not np.isnan(got[:, 0]).all()
