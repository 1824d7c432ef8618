"""Shared pieces of the parity tests: error metrics and device round trips."""
import sys

import numpy as np

from sapphire_amd import capi


def announce(*what):
    """Name the case on stdout before the GPU step runs."""
    print("[case]", *what)
    sys.stdout.flush()


def normalised_error(got, ref, absA, absB_or_denominator, is_denominator=False):
    """max_ij |got - ref| / sum_k |a_ik * b_kj|   (the K-length normalisation)."""
    if is_denominator:
        den = absB_or_denominator
    else:
        den = absA.astype(np.float64) @ absB_or_denominator.astype(np.float64)
    den = np.maximum(den, np.finfo(np.float32).tiny)
    return float(np.max(np.abs(got.astype(np.float64) - ref.astype(np.float64)) / den))


def gpu_gemm_f32(C, A, B, M, N, K, batch=1, stride_out=None, stride_a=None, stride_b=None):
    """C (numpy, any shape, float32) += A*B through sph_gemm_f32; returns the new C."""
    so = M * N if stride_out is None else stride_out
    sa = M * K if stride_a is None else stride_a
    sb = K * N if stride_b is None else stride_b
    dA, dB, dC = (capi.DeviceBuffer.from_array(x) for x in (A, B, C))
    capi.require_gemm_extents(dC, dA, dB, M, N, K, batch, so, sa, sb)
    capi.call("sph_gemm_f32", dC.ptr, dA.ptr, dB.ptr, M, N, K, batch, so, sa, sb)
    out = dC.download(np.float32, C.shape)
    for d in (dA, dB, dC):
        d.release()
    return out


def gpu_gemm_f16(C, A16, B16, M, N, K, batch=1, stride_out=None, stride_a=None, stride_b=None,
                 flags=0):
    so = M * N if stride_out is None else stride_out
    sa = M * K if stride_a is None else stride_a
    sb = K * N if stride_b is None else stride_b
    assert A16.dtype == np.float16 and B16.dtype == np.float16
    dA, dB, dC = (capi.DeviceBuffer.from_array(x) for x in (A16, B16, C))
    capi.require_gemm_extents(dC, dA, dB, M, N, K, batch, so, sa, sb, operand_bytes=2)
    capi.call("sph_gemm_f16f32", dC.ptr, dA.ptr, dB.ptr, M, N, K, batch, so, sa, sb, flags)
    out = dC.download(np.float32, C.shape)
    for d in (dA, dB, dC):
        d.release()
    return out


def gpu_gemm_grouped(C, A, B, M, N, K, triples):
    dA, dB, dC = (capi.DeviceBuffer.from_array(x) for x in (A, B, C))
    entries = capi.make_entries(triples)
    for o, a, b in triples:
        assert (o + M * N) * 4 <= dC.nbytes and (a + M * K) * 4 <= dA.nbytes \
            and (b + K * N) * 4 <= dB.nbytes, "a grouped unit lies outside its buffer"
    capi.call("sph_gemm_f32_grouped", entries, len(triples), dC.ptr, dA.ptr, dB.ptr, M, N, K)
    out = dC.download(np.float32, C.shape)
    for d in (dA, dB, dC):
        d.release()
    return out


def gpu_spmm(C, V, COL, ROW, M, Kdim, N, B, accumulate, canary=0):
    """Runs sph_spmm_csr_f32 with `canary` guard floats on both sides of out."""
    guard = np.full(canary, np.float32(-12345.5), dtype=np.float32)
    padded = np.concatenate([guard, C.ravel(), guard]).astype(np.float32)
    dC = capi.DeviceBuffer.from_array(padded)
    dV = capi.DeviceBuffer.from_array(V if V.size else np.zeros(1, np.float32))
    dCol = capi.DeviceBuffer.from_array(COL if COL.size else np.zeros(1, np.uint32))
    dRow = capi.DeviceBuffer.from_array(ROW)
    dB = capi.DeviceBuffer.from_array(B)
    assert padded.nbytes >= 4 * (2 * canary + M * N)
    capi.require_csr_extents(dC, dV, dCol, dRow, dB, M, Kdim, N, int(V.size))
    capi.validate_csr(dCol, dRow, M, Kdim, int(V.size))
    capi.call("sph_spmm_csr_f32", dC.at(4 * canary), dV.ptr, dCol.ptr, dRow.ptr, M, Kdim, N,
              dB.ptr, 1 if accumulate else 0)
    back = dC.download(np.float32, padded.shape)
    for d in (dC, dV, dCol, dRow, dB):
        d.release()
    if canary:
        assert np.array_equal(back[:canary], guard), "write before the start of out"
        assert np.array_equal(back[-canary:], guard), "write past the end of out"
    return back[canary:canary + C.size].reshape(C.shape)


def gpu_spmm_bias(junk, V, COL, ROW, M, Kdim, N, B, row_bias, canary=0):
    """Runs sph_spmm_csr_bias_f32 over an out that holds `junk`, with guard floats around it."""
    guard = np.full(canary, np.float32(-12345.5), dtype=np.float32)
    padded = np.concatenate([guard, junk.ravel(), guard]).astype(np.float32)
    dC = capi.DeviceBuffer.from_array(padded)
    dV = capi.DeviceBuffer.from_array(V if V.size else np.zeros(1, np.float32))
    dCol = capi.DeviceBuffer.from_array(COL if COL.size else np.zeros(1, np.uint32))
    dRow = capi.DeviceBuffer.from_array(ROW)
    dB = capi.DeviceBuffer.from_array(B)
    dBias = capi.DeviceBuffer.from_array(row_bias)
    assert padded.nbytes >= 4 * (2 * canary + M * N) and dBias.nbytes >= 4 * M
    capi.require_csr_extents(dC, dV, dCol, dRow, dB, M, Kdim, N, int(V.size))
    capi.validate_csr(dCol, dRow, M, Kdim, int(V.size))
    capi.call("sph_spmm_csr_bias_f32", dC.at(4 * canary), dV.ptr, dCol.ptr, dRow.ptr, M, Kdim, N,
              dB.ptr, dBias.ptr)
    back = dC.download(np.float32, padded.shape)
    for d in (dC, dV, dCol, dRow, dB, dBias):
        d.release()
    if canary:
        assert np.array_equal(back[:canary], guard), "write before the start of out"
        assert np.array_equal(back[-canary:], guard), "write past the end of out"
    return back[canary:canary + junk.size].reshape(junk.shape)


def gpu_gemm_f32_ex(C, A, B, M, N, K, flags, batch=1, stride_out=None, stride_a=None,
                    stride_b=None):
    """sph_gemm_f32_ex on numpy operands exactly as stored (A is K x M with SPH_GEMM_TRANS_A,
    B is N x K with SPH_GEMM_TRANS_B)."""
    so = M * N if stride_out is None else stride_out
    sa = M * K if stride_a is None else stride_a
    sb = K * N if stride_b is None else stride_b
    dA, dB, dC = (capi.DeviceBuffer.from_array(x) for x in (A, B, C))
    capi.require_gemm_extents(dC, dA, dB, M, N, K, batch, so, sa, sb)
    capi.call("sph_gemm_f32_ex", dC.ptr, dA.ptr, dB.ptr, M, N, K, batch, so, sa, sb, flags)
    out = dC.download(np.float32, C.shape)
    for d in (dA, dB, dC):
        d.release()
    return out


def gpu_transpose(x, rows, cols, batch=1):
    dX = capi.DeviceBuffer.from_array(x)
    dY = capi.DeviceBuffer(x.nbytes)
    capi.call("sph_transpose_f32", dY.ptr, dX.ptr, rows, cols, batch, 0)
    out = dY.download(np.float32, (batch, cols, rows))
    dX.release()
    dY.release()
    return out


# fp32: a product with more than a quarter and at most half as many 64 x 64 output tiles as the
# chip has compute units (K >= 64) runs on 64 x 32 tiles with K split over two groups of
# wavefronts when its operands allow the straight-to-LDS copies; the K products of an element
# are then summed in another order than by the other fp32 kernels.
F32_CUS = 256


def f32_k_split_range(M, N, K, batch=1):
    tiles64 = -(-M // 64) * -(-N // 64) * batch
    return (4 * tiles64 > F32_CUS and 2 * tiles64 <= F32_CUS and K >= 64 and M >= 4 and N >= 4
            and (M % 4 == 0 or M >= 68))


# Small products run on the few-tile kernel: at most one 32 x 32 output tile per compute unit
# (256 of them), or a matrix of at most 16 rows or columns with at most four 16 x 16 tiles per
# compute unit.  The tests of the tiled kernels' edges use small matrices, so each of those shapes
# is run twice: as given (few-tile kernel, where it qualifies) and with the batch raised until
# the tiled kernels take it.
F16_FEW_TILE_CUS = 256


def f16_few_tiles(M, N, batch, K=None):
    """Whether the few-tile kernel takes the product.  With K the exact rule; without it the
    wider one (every product this says no to runs on the tiled kernels whatever its K)."""
    b32 = -(-M // 32) * -(-N // 32) * batch
    b16 = -(-M // 16) * -(-N // 16) * batch
    limit = F16_FEW_TILE_CUS
    if K is not None and M % 8 == 0 and N % 8 == 0 and K >= 64:
        limit = F16_FEW_TILE_CUS // 2 - 1     # the 64 x 64-tile kernel takes these from here up
    return b32 <= limit or (min(M, N) <= 16 and b16 <= 4 * F16_FEW_TILE_CUS)


def f16_both_kernel_families(shapes):
    out = []
    for shape in shapes:
        M, N, K = shape[:3]
        batch = shape[3] if len(shape) > 3 else 1
        out.append((M, N, K, batch))
        if f16_few_tiles(M, N, batch):
            tiled = batch
            while f16_few_tiles(M, N, tiled):
                tiled += 1
            out.append((M, N, K, tiled))
    return out
