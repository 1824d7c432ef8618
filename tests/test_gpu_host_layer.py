"""The C++ operator layer on the device, driven like the reference's own tests: build
TensorData, ToCuda, Compute::Gemm, ToHost, compare with the CPU result on the same data.

Tolerance (fp32 path): max |gpu - cpu| / sum_k |a b| <= 1e-4; the reference's own absolute
bounds (2.0 for Gemm1, 1.5 for the broadcast tests, inputs N(10, 5)) are asserted as well.
"""
import numpy as np
import pytest

from oracle import pyoracle as po
from sapphire_amd import synth
from tests import helpers as h
from tests import host_layer as hl

pytestmark = pytest.mark.gpu
TOL_F32 = 1e-4


def _n10_5(seed, shape):
    return (synth.normal(seed, shape, 5.0) + 10).astype(np.float32)


def _dims(seed, count, hi):
    return [int(x % hi) + 1 for x in synth.bits64(seed, count)]


def _assert_close_to_cpu(got, y0, a, b, abs_bound):
    ref = po.compute_gemm(y0.copy(), a, b)
    assert np.max(np.abs(got - ref)) <= abs_bound
    assert np.any(got != 0)
    # normalise by what the same walk gives for |a| |b|
    den = po.compute_gemm(np.zeros_like(y0), np.abs(a), np.abs(b))
    err = float(np.max(np.abs(got.astype(np.float64) - ref) / np.maximum(den, 1e-30)))
    assert err <= TOL_F32, err


@pytest.mark.parametrize("seed", range(6))
def test_gemm1_recipe(dev, seed):
    """GemmTest.cpp:20-84: {b,M,K} x {b,K,N} -> {b,M,N}, dims in [1,100], batch in [1,30]."""
    M, N, K, braw = _dims(0x100 + seed, 4, 100)
    batch = braw % 30 + 1
    h.announce("Compute::Gemm Gemm1 recipe", M, N, K, batch)
    a, b = _n10_5(1 + seed, (batch, M, K)), _n10_5(50 + seed, (batch, K, N))
    y0 = np.zeros((batch, M, N), np.float32)
    _assert_close_to_cpu(hl.compute_gemm(y0, a, b), y0, a, b, 2.0)


@pytest.mark.parametrize("seed", range(4))
def test_broadcast_with_one_dimension(dev, seed):
    """BroadcastTest.cpp:20-80: A{b,1,M,K} x B{b,M,K,N} -> {b,M,M,N}, dims in [1,10]."""
    M, N, K, braw = _dims(0x200 + seed, 4, 10)
    batch = braw % 3 + 1
    h.announce("Compute::Gemm BroadcastWithOneDimension", M, N, K, batch)
    a, b = _n10_5(2 + seed, (batch, 1, M, K)), _n10_5(60 + seed, (batch, M, K, N))
    y0 = np.zeros((batch, M, M, N), np.float32)
    _assert_close_to_cpu(hl.compute_gemm(y0, a, b), y0, a, b, 1.5)


@pytest.mark.parametrize("seed", range(4))
def test_broadcast_with_missing_dimension(dev, seed):
    """BroadcastTest.cpp:82-141: A{M,K} x B{M,K,N} -> {M,M,N}."""
    M, N, K = _dims(0x300 + seed, 3, 10)
    h.announce("Compute::Gemm BroadcastWithMissingDimension", M, N, K)
    a, b = _n10_5(3 + seed, (M, K)), _n10_5(70 + seed, (M, K, N))
    y0 = np.zeros((M, M, N), np.float32)
    _assert_close_to_cpu(hl.compute_gemm(y0, a, b), y0, a, b, 1.5)


@pytest.mark.parametrize("seed", range(4))
def test_broadcast_mixed(dev, seed):
    """BroadcastTest.cpp:143-202: A{M,K} x B{N,M,K,N} -> {N,M,M,N}."""
    M, N, K = _dims(0x400 + seed, 3, 10)
    h.announce("Compute::Gemm BroadcastMixed", M, N, K)
    a, b = _n10_5(4 + seed, (M, K)), _n10_5(80 + seed, (N, M, K, N))
    y0 = np.zeros((N, M, M, N), np.float32)
    _assert_close_to_cpu(hl.compute_gemm(y0, a, b), y0, a, b, 1.5)


def test_conv_style_broadcast_of_A_and_accumulation(dev):
    """Filter {1,C,K} shared by the batch (how the naive Conv2D calls Gemm), y not zero."""
    h.announce("Compute::Gemm A broadcast {1,6,9} x {5,9,8}")
    a, b = synth.uniform(5, (1, 6, 9)), synth.uniform(6, (5, 9, 8))
    y0 = synth.uniform(7, (5, 6, 8))
    _assert_close_to_cpu(hl.compute_gemm(y0, a, b), y0, a, b, 1e-3)


def test_repeated_outputs_accumulate_in_walk_order(dev):
    """y smaller than the operands: several leaves add into the same output unit."""
    h.announce("Compute::Gemm repeated outputs {2,4,5} <- {6,4,2} x {3,2,5}")
    a, b = synth.uniform(8, (6, 4, 2)), synth.uniform(9, (3, 2, 5))
    y0 = synth.uniform(10, (2, 4, 5))
    _assert_close_to_cpu(hl.compute_gemm(y0, a, b), y0, a, b, 1e-3)


@pytest.mark.parametrize("shapes", [
    ((64, 48), (64, 40), (40, 48)),                 # one product
    ((5, 6, 8), (5, 6, 9), (5, 9, 8)),              # equal batches
    ((5, 6, 8), (1, 6, 9), (5, 9, 8)),              # A shared by the batch
    ((16, 70, 33), (16, 70, 20), (1, 20, 33)),      # B shared by the batch, ragged widths
    ((300, 260), (300, 100), (100, 260)),           # tiled kernels
    ((2, 4, 5), (6, 4, 2), (3, 2, 5)),              # outputs hit several times: must NOT overwrite
    ((3,), (4,), (4, 3)),                           # 1-D operands
])
def test_fresh_y_is_stored_not_filled_and_read(dev, shapes):
    """A new TensorData reads as zeros but its fill is deferred; Compute::Gemm into it stores the
    product when the walk writes every element exactly once, and must give the bits of the
    accumulating call on an explicitly zeroed y in every case."""
    ys, as_, bs = shapes
    h.announce("Compute::Gemm fresh y", ys, as_, bs)
    a, b = synth.uniform(31, as_), synth.uniform(32, bs)
    # a dirty block of y's size goes back to the pool first, so that the fresh y reuses it
    hl.compute_gemm(np.full(ys, 9.0, np.float32), a, b)
    got = hl.compute_gemm_fresh_y(ys, a, b)
    on_zeros = hl.compute_gemm(np.zeros(ys, np.float32), a, b)
    assert np.array_equal(got.view(np.uint32), on_zeros.view(np.uint32))
    _assert_close_to_cpu(got, np.zeros(ys, np.float32), a, b, 1e-3)


@pytest.mark.parametrize("shape", [(512, 512, 512, 1), (256, 264, 96, 3), (100, 40, 70, 1),
                                   (4096, 4096, 4096, 1)])
def test_gemm_half_operator_fresh_y_equals_accumulating_on_zeros(dev, shape):
    """Compute::GemmHalf: the product stored into a fresh y has the bits of the product added
    to a zero y, and both are within 1e-2 of the CPU loop on the widened operands."""
    from sapphire_amd import capi
    M, N, K, batch = shape
    h.announce("Compute::GemmHalf fresh y", shape)
    A = synth.normal(41, (batch, M, K), 1.0 / np.sqrt(K)).astype(np.float16)
    B = synth.normal(42, (batch, K, N), 1.0 / np.sqrt(K)).astype(np.float16)
    dA, dB = capi.DeviceBuffer.from_array(A), capi.DeviceBuffer.from_array(B)
    assert dA.nbytes >= 2 * batch * M * K and dB.nbytes >= 2 * batch * K * N
    ys = (batch, M, N) if batch > 1 else (M, N)
    # leave a dirty block of y's size in the pool for the fresh y to pick up
    hl.gemm_half(np.full(ys, 5.0, np.float32), dA.ptr, dB.ptr, K, fresh_y=False)
    fresh = hl.gemm_half(np.full(ys, -3.0, np.float32), dA.ptr, dB.ptr, K, fresh_y=True)
    on_zeros = hl.gemm_half(np.zeros(ys, np.float32), dA.ptr, dB.ptr, K, fresh_y=False)
    dA.release()
    dB.release()
    assert np.array_equal(fresh.view(np.uint32), on_zeros.view(np.uint32))
    rows = M if M <= 512 else 64      # the CPU loop on a row slice of the large case
    for u in range(batch):
        a32 = A[u, :rows].astype(np.float32)
        b32 = B[u].astype(np.float32)
        ref = po.gemm_rows(np.zeros((rows, N), np.float32), a32, b32, rows, N, K, threads=4)
        got = fresh.reshape(batch, M, N)[u, :rows]
        assert h.normalised_error(got, ref, np.abs(a32), np.abs(b32)) <= 1e-2


def test_gemm_half_operator_accumulates_into_a_used_y(dev):
    from sapphire_amd import capi
    M, N, K = 130, 72, 64
    h.announce("Compute::GemmHalf accumulate", M, N, K)
    A = synth.normal(43, (M, K), 0.125).astype(np.float16)
    B = synth.normal(44, (K, N), 0.125).astype(np.float16)
    y0 = synth.uniform(45, (M, N))
    dA, dB = capi.DeviceBuffer.from_array(A), capi.DeviceBuffer.from_array(B)
    got = hl.gemm_half(y0, dA.ptr, dB.ptr, K, fresh_y=False)
    dA.release()
    dB.release()
    a32, b32 = A.astype(np.float32), B.astype(np.float32)
    ref = po.gemm_rows(y0.copy(), a32, b32, M, N, K, threads=2)
    assert h.normalised_error(got, ref, np.abs(a32), np.abs(b32)) <= 1e-2


def test_one_dimensional_operands(dev):
    h.announce("Compute::Gemm 1-D operands [4] x [4,3] -> [3]")
    a, b, y0 = synth.uniform(11, (4,)), synth.uniform(12, (4, 3)), synth.uniform(13, (3,))
    _assert_close_to_cpu(hl.compute_gemm(y0, a, b), y0, a, b, 1e-3)


def test_config2_through_the_operator(dev):
    h.announce("Compute::Gemm config2 through TensorData")
    d = synth.config2()
    got = hl.compute_gemm(d["C"], d["A"], d["B"])
    ref = po.compute_gemm(d["C"].copy(), d["A"], d["B"], threads=8)
    for b in range(16):
        err = h.normalised_error(got[b], ref[b], np.abs(d["A"][b]), np.abs(d["B"][0]))
        assert err <= TOL_F32


def test_config4_mlp_forward(dev):
    """3-layer MLP 784 -> 1024 -> 1024 -> 10, batch 1024, Linear = bias GEMM (K = 1) + GEMM,
    ReLU between layers; compared with the CPU composition layer by layer."""
    h.announce("config4 MLP forward through NN::LinearForward + Compute::ReLU")
    d = synth.config4()
    got = hl.mlp_forward(d["x"], d["W"], d["b"])
    act = d["x"]
    bound = np.abs(d["x"]).astype(np.float64)       # propagated sum_k |a b| bound
    for l in range(3):
        ref = po.linear_forward(act, d["W"][l], d["b"][l], threads=8)
        bound = bound @ np.abs(d["W"][l]).astype(np.float64) + np.abs(d["b"][l])
        act = po.relu(ref) if l < 2 else ref
    assert got.shape == (1024, 10) and np.isfinite(got).all()
    err = float(np.max(np.abs(got.astype(np.float64) - act) / bound))
    assert err <= TOL_F32, err
    # also against the plain magnitude of the output
    assert np.max(np.abs(got - act)) <= 1e-4 * max(1.0, float(np.max(np.abs(act))))
    # one launch per layer (bias row and ReLU applied where the product is stored): same bits
    h.announce("config4 MLP forward through NN::LinearForwardFused")
    fused = hl.mlp_forward(d["x"], d["W"], d["b"], fused=True)
    assert np.array_equal(fused.view(np.uint32), got.view(np.uint32))


def test_transpose(dev):
    h.announce("Compute::Transpose batched and broadcast")
    x = synth.uniform(14, (3, 37, 65))
    got = hl.transpose(x, (3, 65, 37))
    assert np.array_equal(got, np.transpose(x, (0, 2, 1)))
    assert np.array_equal(got.ravel(), po.transpose(x, 37, 65, 3))
    x2 = synth.uniform(15, (5, 9))
    got = hl.transpose(x2, (4, 9, 5))          # 2-D input repeated for every matrix of y
    assert np.array_equal(got, np.broadcast_to(x2.T, (4, 9, 5)))


def test_sparse_gemm_through_tensor_data(dev):
    h.announce("Compute::SparseGemm through SparseMatrix + TensorData")
    M, K, N = 200, 333, 48
    v, col, row = synth.csr_matrix(16, M, K, 9.0, forced={0: 0, 3: 200})
    B = synth.uniform(17, (K, N))
    y0 = synth.uniform(18, (M, N))
    ref = po.spmm_csr(y0.copy(), v, col, row, M, N, B)
    got = hl.sparse_gemm(y0, v, col, row, M, K, N, B, True)
    assert np.array_equal(got.view(np.uint32), ref.view(np.uint32))
    ref0 = po.spmm_csr(np.zeros((M, N), np.float32), v, col, row, M, N, B)
    got0 = hl.sparse_gemm(y0, v, col, row, M, K, N, B, False)
    assert np.array_equal(got0.view(np.uint32), ref0.view(np.uint32))


def test_tensor_data_life_cycle_on_device(dev):
    h.announce("TensorData / ResourceManager life cycle")
    lib = hl.lib()
    rc = lib.sphh_tensor_lifecycle()
    assert rc == 0, (rc, lib.sphh_last_error())


def test_pool_block_handed_to_another_threads_stream(dev):
    h.announce("ResourceManager: block reused by a second thread while the first stream still writes")
    lib = hl.lib()
    rc = lib.sphh_pool_handover()
    assert rc == 0, (rc, lib.sphh_last_error())


# ---- backward neighbours and the Linear backward pass -------------------------------------------

def _bits(x):
    return np.ascontiguousarray(x).view(np.uint32)


def test_compute_sub_matches_recorded_reference_outputs(dev):
    import os
    from tests.golden.cases import SUB_CASES
    kat = np.load(os.path.join(os.path.dirname(os.path.abspath(__file__)), "golden",
                               "backward_kat.npz"))
    for name, ys, as_, bs, seed in SUB_CASES:
        h.announce("Compute::Sub", name, ys, as_, bs)
        a = synth.uniform(seed + 1, as_)
        b = synth.uniform(seed + 2, bs)
        assert np.array_equal(_bits(hl.sub(ys, a, b)), _bits(kat["sub_" + name])), name


def test_compute_scale_and_relu_backward(dev):
    h.announce("Compute::Scale / Compute::ReLUBackward")
    x = synth.normal(5, (3001,))
    assert np.array_equal(_bits(hl.scale(x, 0.125)), _bits(po.scale(x, 0.125)))
    assert np.array_equal(_bits(hl.scale(x, -3.3, in_place=True)), _bits(po.scale(x, -3.3)))
    dx, dy = synth.uniform(6, (3001,)), synth.uniform(7, (3001,))
    assert np.array_equal(_bits(hl.relu_backward(dx, dy, x)), _bits(po.relu_backward(dx, dy, x)))


@pytest.mark.parametrize("dims", [(1, 1, 1), (4, 3, 2), (33, 20, 7), (128, 784, 64),
                                  (1024, 1024, 10), (256, 100, 300)])
def test_linear_backward(dev, dims):
    """Sources/Sapphire/operations/Backward/LinearBackward.cpp:27-99 + SGD on the device against
    the same call sequence on the CPU.  dx within the fp32 GEMM tolerance; the updated
    parameters within learningRate x that tolerance (plus one rounding of the parameter)."""
    batch, fin, fout = dims
    lr = 0.01
    h.announce("BackProp::LinearBackward", dims)
    x = synth.uniform(81, (batch, fin))
    W = synth.uniform(82, (fin, fout))
    bias = synth.uniform(83, (fout,))
    dy = synth.uniform(84, (batch, fout))
    dx0 = synth.uniform(85, (batch, fin))
    ref_dx, ref_W, ref_b = po.linear_backward(dx0, W, bias, dy, x, lr, threads=8)

    seq_ref = hl.linear_backward(dx0, W, bias, dy, x, lr, sequence=0, fused_sgd=False)
    direct = hl.linear_backward(dx0, W, bias, dy, x, lr, sequence=1, fused_sgd=True)
    # the direct sequence (transposed reads, overwrite, one-pass SGD) changes no bit
    for got, want in zip(direct, seq_ref):
        assert np.array_equal(_bits(got), _bits(want))

    dx, W2, b2 = seq_ref
    den = np.abs(dy).astype(np.float64) @ np.abs(W.T).astype(np.float64)
    assert h.normalised_error(dx, ref_dx, None, den, is_denominator=True) <= TOL_F32
    den = np.abs(x.T).astype(np.float64) @ np.abs(dy).astype(np.float64)
    slack = np.finfo(np.float32).eps * (np.abs(ref_W) + lr * den)
    assert np.all(np.abs(W2.astype(np.float64) - ref_W) <= lr * TOL_F32 * den + slack)
    den = np.abs(dy).astype(np.float64).sum(axis=0) / batch
    slack = np.finfo(np.float32).eps * (np.abs(ref_b) + lr * den)
    assert np.all(np.abs(b2.astype(np.float64) - ref_b) <= lr * TOL_F32 * den + slack)
    assert np.any(W2 != W) and np.any(b2 != bias) and np.any(dx != dx0)


@pytest.mark.parametrize("shapes", [((1, 3, 2), (1, 2, 4)), ((5, 33, 20), (5, 20, 17)),
                                    ((64, 48), (48, 80)), ((2, 3, 40, 64), (2, 3, 64, 24)),
                                    ((4, 9, 6), (6, 5))])
def test_matmul_backward(dev, shapes):
    """Sources/Sapphire/operations/Backward/MathBackward.cpp:35-51 (the reference's TestMatMul
    uses {1,3,2} x {1,2,4}): da += dy b^T, db += a^T dy against the same operator calls on the
    CPU; the last case has a 2-D b, which the direct sequence hands to the reference one."""
    sa, sb = shapes
    h.announce("BackProp::MatMulBackward", shapes)
    a = synth.uniform(101, sa)
    b = synth.uniform(102, sb)
    sy = tuple(sa[:-1]) + (sb[-1],)
    dy = synth.uniform(103, sy)
    da0 = synth.uniform(104, sa)
    db0 = synth.uniform(105, sb)
    # CPU: Transpose + Compute::Gemm as written in the reference
    rows_a, cols_a = sa[-2], sa[-1]
    rows_b, cols_b = sb[-2], sb[-1]
    nb_a = int(np.prod(sa[:-2])) if len(sa) > 2 else 1
    nb_b = int(np.prod(sb[:-2])) if len(sb) > 2 else 1
    ta = po.transpose(a, rows_a, cols_a, nb_a).reshape(tuple(sa[:-2]) + (cols_a, rows_a))
    tb = po.transpose(b, rows_b, cols_b, nb_b).reshape(tuple(sb[:-2]) + (cols_b, rows_b))
    ref_da = po.compute_gemm(da0.copy(), dy, tb)
    ref_db = po.compute_gemm(db0.copy(), ta, dy)
    seq_ref = hl.matmul_backward(da0, db0, dy, a, b, 0)
    direct = hl.matmul_backward(da0, db0, dy, a, b, 1)
    for got, want in zip(direct, seq_ref):
        assert np.array_equal(_bits(got), _bits(want))
    den_a = po.compute_gemm(np.zeros_like(da0), np.abs(dy), np.abs(tb))
    den_b = po.compute_gemm(np.zeros_like(db0), np.abs(ta), np.abs(dy))
    for got, ref, den in ((seq_ref[0], ref_da, den_a), (seq_ref[1], ref_db, den_b)):
        err = float(np.max(np.abs(got.astype(np.float64) - ref) / np.maximum(den, 1e-30)))
        assert err <= TOL_F32, err
