"""fp32 GEMM through the C ABI against the CPU checker on identical seeded inputs.

Tolerance (fp32 path): max_ij |gpu - cpu| / sum_k |a_ik * b_kj| <= 1e-4.
"""
import numpy as np
import pytest

from oracle import pyoracle as po
from sapphire_amd import capi, synth
from tests import helpers as h

pytestmark = pytest.mark.gpu
TOL_F32 = 1e-4


def _check(got, ref, A2, B2, what):
    err = h.normalised_error(got, ref, np.abs(A2), np.abs(B2))
    assert np.isfinite(got).all(), what
    assert err <= TOL_F32, "%s: normalised error %.3e" % (what, err)
    return err


def test_config1_256_cubed(dev):
    h.announce("sph_gemm_f32 config1 256^3")
    d = synth.config1()
    ref = po.naive_gemm(d["C"].copy(), d["A"], d["B"], 256, 256, 256)
    got = h.gpu_gemm_f32(d["C"], d["A"], d["B"], 256, 256, 256)
    _check(got, ref, d["A"], d["B"], "config1")
    # C really takes part: result minus product of a zero-C run equals C up to rounding
    got0 = h.gpu_gemm_f32(np.zeros_like(d["C"]), d["A"], d["B"], 256, 256, 256)
    assert np.max(np.abs((got - got0) - d["C"])) < 1e-4


def test_config2_batch_broadcast_B(dev):
    h.announce("sph_gemm_f32 config2 A[16,512,512] B[1,512,512] strideB=0")
    d = synth.config2()
    ref = po.compute_gemm(d["C"].copy(), d["A"], d["B"], threads=8)
    got = h.gpu_gemm_f32(d["C"], d["A"], d["B"], 512, 512, 512, batch=16, stride_b=0)
    for b in range(16):
        _check(got[b], ref[b], d["A"][b], d["B"][0], "config2 unit %d" % b)


def test_broadcast_A(dev):
    h.announce("sph_gemm_f32 strideA=0")
    A = synth.uniform(11, (1, 96, 40))
    B = synth.uniform(12, (5, 40, 72))
    C = synth.uniform(13, (5, 96, 72))
    ref = po.compute_gemm(C.copy(), A, B)
    got = h.gpu_gemm_f32(C, A, B, 96, 72, 40, batch=5, stride_a=0)
    for b in range(5):
        _check(got[b], ref[b], A[0], B[b], "unit %d" % b)


@pytest.mark.parametrize("seed", range(12))
def test_reference_recipe_gemm1(dev, seed):
    """Tests/UnitTests/Sources/FunctionTest/GemmTest.cpp:20-84: M, N, K in [1,100], batch in
    [1,30], shapes {b,M,K} x {b,K,N} -> {b,M,N}, out zero.  Also meets that test's own bound
    (absolute difference <= 2.0 with inputs N(10,5))."""
    r = synth.bits64(0xC0FFEE + seed, 4)
    M, N, K = (int(x % 100) + 1 for x in r[:3])
    batch = int(r[3] % 100 + 1) % 30 + 1
    h.announce("Gemm1 recipe seed", seed, "M N K batch =", M, N, K, batch)
    A = (synth.normal(100 + seed, (batch, M, K), 5.0) + 10).astype(np.float32)
    B = (synth.normal(200 + seed, (batch, K, N), 5.0) + 10).astype(np.float32)
    C = np.zeros((batch, M, N), np.float32)
    ref = po.compute_gemm(C.copy(), A, B)
    got = h.gpu_gemm_f32(C, A, B, M, N, K, batch=batch)
    assert np.max(np.abs(got - ref)) <= 2.0
    assert np.any(got != 0)
    for b in range(batch):
        _check(got[b], ref[b], A[b], B[b], "unit %d" % b)


@pytest.mark.parametrize("shape", [(1, 1, 1), (1, 7, 3), (33, 1, 5), (64, 64, 16), (65, 63, 17),
                                   (128, 128, 15), (129, 257, 31), (300, 40, 1), (4, 4, 1000)])
def test_edges(dev, shape):
    M, N, K = shape
    h.announce("sph_gemm_f32 edge", shape)
    A = synth.uniform(21, (M, K))
    B = synth.uniform(22, (K, N))
    C = synth.uniform(23, (M, N))
    ref = po.naive_gemm(C.copy(), A, B, M, N, K)
    got = h.gpu_gemm_f32(C, A, B, M, N, K)
    _check(got, ref, A, B, str(shape))


def test_closed_forms(dev):
    h.announce("sph_gemm_f32 closed forms")
    n = 200
    B = synth.uniform(31, (n, n))
    C = synth.uniform(32, (n, n))
    eye = np.eye(n, dtype=np.float32)
    got = h.gpu_gemm_f32(C, eye, B, n, n, n)
    assert np.array_equal(got, C + B)          # identity: out = B + C exactly
    ones = np.ones((n, n), np.float32)
    got = h.gpu_gemm_f32(np.zeros((n, n), np.float32), ones, ones, n, n, n)
    assert np.array_equal(got, np.full((n, n), float(n), np.float32))
    # K = 1 outer product: how Linear adds its bias (Linear.cpp:134)
    col = np.ones((n, 1), np.float32)
    bias = synth.uniform(33, (1, n))
    got = h.gpu_gemm_f32(np.zeros((n, n), np.float32), col, bias, n, n, 1)
    assert np.array_equal(got, np.broadcast_to(bias, (n, n)))


def test_k_zero_leaves_out_untouched(dev):
    C = synth.uniform(41, (8, 8))
    got = h.gpu_gemm_f32(C, np.zeros(1, np.float32), np.zeros(1, np.float32), 8, 8, 0)
    assert np.array_equal(got, C)


def test_unaligned_bases(dev):
    """Operands that start 4 bytes into an allocation take the scalar load path."""
    h.announce("sph_gemm_f32 unaligned bases")
    M, N, K = 72, 64, 48
    A = synth.uniform(51, (M * K + 1,))
    B = synth.uniform(52, (K * N + 1,))
    C = synth.uniform(53, (M * N + 1,))
    ref = po.naive_gemm(C[1:].copy(), A[1:].copy(), B[1:].copy(), M, N, K)
    dA, dB, dC = (capi.DeviceBuffer.from_array(x) for x in (A, B, C))
    capi.call("sph_gemm_f32", dC.at(4), dA.at(4), dB.at(4), M, N, K, 1, M * N, M * K, K * N)
    got = dC.download(np.float32, C.shape)
    assert got[0] == C[0]
    _check(got[1:].reshape(M, N), ref.reshape(M, N), A[1:].reshape(M, K), B[1:].reshape(K, N),
           "unaligned")


# A K that is no multiple of 16 on the straight-to-LDS kernel: a last, partial step whose missing values
# of k count as zeros.  (M, N, K): one step only, 64-tiles with K steps of 32, 128-tiles with K
# steps of 16, ragged edges.  Bars: the CPU loop within tolerance, and bit for bit the same
# product from operands that start 4 bytes into their allocation, which the register-staged
# kernel multiplies (same order of the K products, zero padding included).
@pytest.mark.parametrize("flags", [0, capi.SPH_GEMM_TRANS_A, capi.SPH_GEMM_TRANS_B,
                                   capi.SPH_GEMM_TRANS_A | capi.SPH_GEMM_TRANS_B,
                                   capi.SPH_GEMM_OVERWRITE])
@pytest.mark.parametrize("dims", [(512, 512, 20), (1024, 1024, 1000), (640, 384, 36),
                                  (2048, 2048, 120), (300, 260, 44), (4096, 2048, 72),
                                  (1024, 1024, 28),
                                  # K % 4 != 0: rows of a K-contiguous operand start at 4-byte
                                  # aligned addresses, the chunk that ends at K is copied shifted
                                  (512, 512, 17), (1024, 1024, 1001), (640, 384, 35),
                                  (2048, 2048, 122), (300, 260, 47), (4096, 2048, 65),
                                  (1024, 1024, 33), (512, 768, 131)])
def test_partial_last_k_step(dev, dims, flags):
    M, N, K = dims
    h.announce("sph_gemm_f32_ex, K % 16 != 0", dims, "flags", flags)
    A = synth.uniform(401, (M, K))
    B = synth.uniform(402, (K, N))
    C = synth.uniform(403, (M, N))
    As = np.ascontiguousarray(A.T) if flags & capi.SPH_GEMM_TRANS_A else A
    Bs = np.ascontiguousarray(B.T) if flags & capi.SPH_GEMM_TRANS_B else B
    got = h.gpu_gemm_f32_ex(C, As, Bs, M, N, K, flags)
    start = np.zeros((256, N), np.float32) if flags & capi.SPH_GEMM_OVERWRITE else C[:256].copy()
    ref = po.gemm_rows(start, A[:256], B, 256, N, K)
    assert h.normalised_error(got[:256], ref, np.abs(A[:256]), np.abs(B)) <= TOL_F32
    shifted = [np.concatenate([np.zeros(1, np.float32), x.ravel()]) for x in (As, Bs, C)]
    dA, dB, dC = (capi.DeviceBuffer.from_array(x) for x in shifted)
    capi.call("sph_gemm_f32_ex", dC.at(4), dA.at(4), dB.at(4), M, N, K, 1, M * N, M * K, K * N,
              flags)
    other = dC.download(np.float32, (M * N + 1,))[1:].reshape(M, N)
    for d in (dA, dB, dC):
        d.release()
    if h.f32_k_split_range(M, N, K):
        # 65 .. 128 tiles of 64 x 64: aligned operands run the kernel that splits K over two groups
        # of wavefronts, misaligned ones the few-tile kernel: two orders of the K products, both
        # held to the tolerance
        assert h.normalised_error(other[:256], ref, np.abs(A[:256]), np.abs(B)) <= TOL_F32
    else:
        assert np.array_equal(got.view(np.uint32), other.view(np.uint32))


# N = 4 q + r, r != 0: the first 4 q columns on the tiled kernels with the
# row pitches left at N, the last r on the kernel for narrow products.  Guard floats behind
# every unit of out catch a store past column N - 1.
@pytest.mark.parametrize("flags", [0, capi.SPH_GEMM_TRANS_A, capi.SPH_GEMM_TRANS_B,
                                   capi.SPH_GEMM_OVERWRITE])
@pytest.mark.parametrize("dims", [(512, 1026, 64, 1), (1000, 999, 100, 1), (300, 70, 40, 3),
                                  (64, 69, 16, 5), (2048, 2049, 128, 1), (128, 1031, 2050, 1),
                                  # narrow products with enough rows for the tiled kernels
                                  (16384, 10, 64, 1), (9000, 5, 32, 1), (4096, 30, 100, 2)])
def test_column_count_not_a_multiple_of_four(dev, dims, flags):
    M, N, K, batch = dims
    h.announce("sph_gemm_f32_ex, N % 4 != 0", dims, "flags", flags)
    A = synth.uniform(411, (batch, M, K))
    B = synth.uniform(412, (batch, K, N))
    C = synth.uniform(413, (batch, M, N))
    As = np.ascontiguousarray(A.swapaxes(1, 2)) if flags & capi.SPH_GEMM_TRANS_A else A
    Bs = np.ascontiguousarray(B.swapaxes(1, 2)) if flags & capi.SPH_GEMM_TRANS_B else B
    pad = 29
    padded = np.full((batch, M * N + pad), np.float32(-777.25), np.float32)
    padded[:, :M * N] = C.reshape(batch, M * N)
    got = h.gpu_gemm_f32_ex(padded, As, Bs, M, N, K, flags, batch=batch, stride_out=M * N + pad)
    assert np.array_equal(got[:, M * N:], padded[:, M * N:]), "guard floats overwritten"
    got = got[:, :M * N].reshape(batch, M, N)
    rows = min(M, 128)
    for b in range(batch):
        start = (np.zeros((rows, N), np.float32) if flags & capi.SPH_GEMM_OVERWRITE
                 else C[b, :rows].copy())
        ref = po.gemm_rows(start, A[b, :rows], B[b], rows, N, K)
        err = h.normalised_error(got[b, :rows], ref, np.abs(A[b, :rows]), np.abs(B[b]))
        assert err <= TOL_F32, (b, err)
        # the last rows too: every row block writes the narrow part
        start = (np.zeros((rows, N), np.float32) if flags & capi.SPH_GEMM_OVERWRITE
                 else C[b, M - rows:].copy())
        ref = po.gemm_rows(start, A[b, M - rows:], B[b], rows, N, K)
        err = h.normalised_error(got[b, M - rows:], ref, np.abs(A[b, M - rows:]), np.abs(B[b]))
        assert err <= TOL_F32, (b, err)


def test_grouped_plan_with_modulo_quirk(dev):
    """{b,1,M,K} x {b,M,K,N} -> {b,M,M,N} (BroadcastTest.cpp:32-34): the walk picks
    A matrix i % b, which is not NumPy broadcasting; the leaves go out as one launch."""
    b, M, K, N = 2, 3, 2, 2
    ys, as_, bs = [b, M, M, N], [b, 1, M, K], [b, M, K, N]
    dims, leaves = po.gemm_plan(ys, as_, bs)
    assert [(o // (M * N), a // (M * K), bb // (K * N)) for o, a, bb, _ in leaves] == \
        [(0, 0, 0), (1, 1, 1), (2, 0, 2), (3, 1, 3), (4, 0, 4), (5, 1, 5)]
    h.announce("sph_gemm_f32_grouped modulo quirk")
    A = synth.uniform(61, as_)
    B = synth.uniform(62, bs)
    C = synth.uniform(63, ys)
    ref = po.compute_gemm(C.copy(), A, B)
    triples = []
    for o, a, bb, total in leaves:
        for u in range(total // (M * N)):
            triples.append((o + u * M * N, a + u * M * K, bb + u * K * N))
    got = h.gpu_gemm_grouped(C, A, B, M, N, K, triples)
    den = np.full(C.shape, 1e-30)
    flatA, flatB = A.reshape(-1, M, K), B.reshape(-1, K, N)
    den = den.reshape(-1, M, N)
    for i, (o, a, bb) in enumerate(triples):
        den[o // (M * N)] = np.abs(flatA[a // (M * K)]).astype(np.float64) @ np.abs(flatB[bb // (K * N)])
    err = h.normalised_error(got.reshape(-1, M, N), ref.reshape(-1, M, N), None, den, True)
    assert err <= TOL_F32


def test_grouped_repeated_output_is_applied_in_order(dev):
    """Two entries adding into one output unit are serialised, as the host walk would."""
    h.announce("sph_gemm_f32_grouped repeated outOff")
    M, N, K = 40, 24, 16
    A = synth.uniform(71, (3, M, K))
    B = synth.uniform(72, (3, K, N))
    C = synth.uniform(73, (2, M, N))
    triples = [(0, 0, 0), (M * N, M * K, K * N), (0, 2 * M * K, 2 * K * N)]
    ref = C.copy()
    for o, a, bb in triples:
        po.naive_gemm(ref.reshape(-1)[o:o + M * N], A.reshape(-1)[a:a + M * K].copy(),
                      B.reshape(-1)[bb:bb + K * N].copy(), M, N, K)
    got = h.gpu_gemm_grouped(C, A, B, M, N, K, triples)
    assert np.max(np.abs(got - ref)) < 1e-4


def test_errors_are_statuses_not_crashes(dev):
    with pytest.raises(capi.SphError) as e:
        capi.call("sph_gemm_f32", None, None, None, 4, 4, 4, 1, 16, 16, 16)
    assert e.value.status == 1 and "null" in str(e.value)
    with pytest.raises(capi.SphError):
        capi.call("sph_gemm_f32", 1, 1, 1, 0, 4, 4, 1, 0, 0, 0)
    with pytest.raises(capi.SphError) as e:
        capi.call("sph_set_device", 99)
    assert "exceeds number of available devices" in str(e.value)


@pytest.mark.parametrize("dims", [(1, 1, 1), (5, 0, 3), (7, 9, 5), (64, 64, 64), (100, 784, 130),
                                  (256, 1024, 10), (1024, 1024, 1024), (130, 100, 257)])
@pytest.mark.parametrize("relu", [False, True])
def test_linear_forward_one_launch(dev, dims, relu):
    """sph_linear_forward_f32 against the CPU layer (bias GEMM + GEMM on a zero y, then ReLU) and,
    bit for bit, against the unfused device sequence it replaces."""
    batch, fin, fout = dims
    h.announce("sph_linear_forward_f32", dims, "relu", relu)
    x = synth.uniform(31, (batch, max(fin, 1)))[:, :fin].copy()
    W = synth.uniform(32, (max(fin, 1), fout))[:fin].copy()
    bias = synth.uniform(33, (fout,))
    bias[0] = -0.0                                   # 0 + (-0) = +0 on the reference path
    dX = capi.DeviceBuffer.from_array(x if x.size else np.zeros(1, np.float32))
    dW = capi.DeviceBuffer.from_array(W if W.size else np.zeros(1, np.float32))
    dB = capi.DeviceBuffer.from_array(bias)
    dY = capi.DeviceBuffer.from_array(np.full((batch, fout), np.float32(np.nan)))
    flags = capi.SPH_LINEAR_RELU if relu else 0
    capi.call("sph_linear_forward_f32", dY.ptr, dX.ptr, dW.ptr, dB.ptr, batch, fin, fout, flags)
    got = dY.download(np.float32, (batch, fout))

    # the sequence it replaces, on the device
    ones = capi.DeviceBuffer.from_array(np.ones(batch, np.float32))
    dZ = capi.DeviceBuffer(4 * batch * fout)
    capi.call("sph_fill_f32", dZ.ptr, 0.0, batch * fout)
    capi.call("sph_gemm_f32", dZ.ptr, ones.ptr, dB.ptr, batch, fout, 1, 1, batch * fout, batch, fout)
    if fin:
        capi.call("sph_gemm_f32", dZ.ptr, dX.ptr, dW.ptr, batch, fout, fin, 1, batch * fout,
                  batch * fin, fin * fout)
    if relu:
        capi.call("sph_relu_f32", dZ.ptr, dZ.ptr, batch * fout)
    want_bits = dZ.download(np.float32, (batch, fout))
    assert np.array_equal(got.view(np.uint32), want_bits.view(np.uint32))

    ref = np.zeros((batch, fout), np.float32)
    if fin:
        ref = po.linear_forward(x, W, bias, threads=8)
    else:
        ref += (np.float32(0) + bias)[None, :]
    if relu:
        ref = po.relu(ref)
    den = np.abs(x).astype(np.float64) @ np.abs(W).astype(np.float64) + np.abs(bias)
    err = h.normalised_error(got, ref, None, np.maximum(den, 1e-30), is_denominator=True)
    assert err <= TOL_F32, err
    for d in (dX, dW, dB, dY, dZ, ones):
        d.release()


@pytest.mark.parametrize("case", [(1024, 1024, 1), (70, 300, 1), (10, 64, 1), (1000, 4099, 1),
                                  (96, 200, 5)])
def test_single_output_row(dev, case):
    """M = 1 with a long K (the ones x dy column sums of the bias gradient) runs on the row
    reduction kernel; accumulate, overwrite, the stored-transposed A flag and a batch."""
    N, K, batch = case
    h.announce("sph_gemm_f32 M = 1", case)
    A = synth.uniform(41, (batch, 1, K))
    B = synth.uniform(42, (batch, K, N))
    C = synth.uniform(43, (batch, 1, N))
    ref = po.gemm_rows(C.copy(), A, B, 1, N, K, batch=batch)
    got = h.gpu_gemm_f32(C, A, B, 1, N, K, batch=batch)
    for b in range(batch):
        _check(got[b], ref[b], A[b], B[b], "unit %d" % b)
    over = h.gpu_gemm_f32_ex(np.full_like(C, np.nan), A, B, 1, N, K, capi.SPH_GEMM_OVERWRITE,
                             batch=batch)
    for b in range(batch):
        _check(over[b], ref[b] - C[b], A[b], B[b], "overwrite unit %d" % b)
    # a 1 x K operand is its own transpose
    flagged = h.gpu_gemm_f32_ex(C, A, B, 1, N, K, capi.SPH_GEMM_TRANS_A, batch=batch)
    assert np.array_equal(flagged.view(np.uint32), got.view(np.uint32))


@pytest.mark.parametrize("dims", [(2, 64, 32, 48), (3, 160, 64, 136), (2, 96, 512, 8)])
def test_grouped_plan_on_aligned_shapes(dev, dims):
    """The same modulo walk at sizes that take the straight-to-LDS kernels (K a multiple of 16
    or 32, 16-byte aligned offsets) and, for the last one, the K-split kernel, with the unit
    offsets coming from the device table."""
    b, M, K, N = dims
    ys, as_, bs = [b, 2, M, N], [b, 1, M, K], [b, 2, K, N]
    _, leaves = po.gemm_plan(ys, as_, bs)
    h.announce("sph_gemm_f32_grouped aligned", dims, len(leaves), "leaves")
    A = synth.uniform(81, as_)
    B = synth.uniform(82, bs)
    C = synth.uniform(83, ys)
    ref = po.compute_gemm(C.copy(), A, B, threads=4)
    triples = []
    for o, a, bb, total in leaves:
        for u in range(total // (M * N)):
            triples.append((o + u * M * N, a + u * M * K, bb + u * K * N))
    got = h.gpu_gemm_grouped(C, A, B, M, N, K, triples)
    flatA, flatB = A.reshape(-1, M, K), B.reshape(-1, K, N)
    den = np.full((len(triples), M, N), 1e-30)
    for o, a, bb in triples:
        den[o // (M * N)] = np.abs(flatA[a // (M * K)]).astype(np.float64) @ np.abs(flatB[bb // (K * N)])
    err = h.normalised_error(got.reshape(-1, M, N), ref.reshape(-1, M, N), None, den, True)
    assert err <= TOL_F32
