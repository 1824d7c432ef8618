"""One-pass neighbours of the path through the C ABI: fill, ReLU, transpose, and the backward /
SGD elementwise steps (bit-exact against the CPU checker)."""
import numpy as np
import pytest

from oracle import pyoracle as po
from sapphire_amd import capi, synth
from tests import helpers as h

pytestmark = pytest.mark.gpu


@pytest.mark.parametrize("n", [1, 3, 4, 1000, 4099, 1 << 20])
def test_fill_and_relu(dev, n):
    h.announce("sph_fill_f32 / sph_relu_f32 n =", n)
    x = synth.uniform(n, (n + 1,))
    dX = capi.DeviceBuffer.from_array(x)
    dY = capi.DeviceBuffer(4 * (n + 1))
    capi.call("sph_fill_f32", dY.ptr, -3.0, n + 1)
    capi.call("sph_relu_f32", dY.at(4), dX.at(4), n)       # unaligned start: scalar path
    got = dY.download(np.float32, (n + 1,))
    assert got[0] == -3.0
    assert np.array_equal(got[1:], po.relu(np.ascontiguousarray(x[1:])))
    capi.call("sph_relu_f32", dY.ptr, dX.ptr, n + 1)        # aligned: vector path
    assert np.array_equal(dY.download(np.float32, (n + 1,)), po.relu(x))
    capi.call("sph_fill_f32", dY.at(4), 2.5, n)
    got = dY.download(np.float32, (n + 1,))
    assert np.all(got[1:] == 2.5)
    dX.release()
    dY.release()


@pytest.mark.parametrize("shape", [(1, 1, 1), (2, 3, 5), (1, 64, 64), (3, 65, 129), (2, 1000, 7)])
def test_transpose_matches_cpu(dev, shape):
    batch, rows, cols = shape
    h.announce("sph_transpose_f32", shape)
    x = synth.uniform(99, shape)
    dX = capi.DeviceBuffer.from_array(x)
    dY = capi.DeviceBuffer(x.nbytes)
    capi.call("sph_transpose_f32", dY.ptr, dX.ptr, rows, cols, batch, 0)
    got = dY.download(np.float32, (batch * rows * cols,))
    assert np.array_equal(got, po.transpose(x, rows, cols, batch))
    dX.release()
    dY.release()


def bits(x):
    return np.ascontiguousarray(x).view(np.uint32)


@pytest.mark.parametrize("n", [1, 3, 4, 1000, 4099, 1 << 20])
def test_scale_sub_relu_backward_sgd_bit_exact(dev, n):
    h.announce("sph_scale_f32 / sph_sub_f32 / sph_relu_backward_f32 / sph_sgd_step_f32 n =", n)
    x = synth.normal(n + 1, (n + 1,))
    g = synth.uniform(n + 2, (n + 1,))
    z = synth.uniform(n + 3, (n + 1,))
    dX, dG, dZ = (capi.DeviceBuffer.from_array(v) for v in (x, g, z))
    dY = capi.DeviceBuffer(4 * (n + 1))
    for off in (0, 1):                       # aligned (16-byte path) and unaligned start
        cnt = n + 1 - off
        xs, gs, zs = (np.ascontiguousarray(v[off:]) for v in (x, g, z))
        capi.call("sph_scale_f32", dY.at(4 * off), dX.at(4 * off), 0.37, cnt)
        assert np.array_equal(bits(dY.download(np.float32, (n + 1,))[off:]),
                              bits(po.scale(xs, 0.37)))
        capi.call("sph_sub_f32", dY.at(4 * off), dX.at(4 * off), dG.at(4 * off), cnt, 0, 0, 0)
        assert np.array_equal(bits(dY.download(np.float32, (n + 1,))[off:]),
                              bits(po.sub_leaf(xs, gs, cnt)))
        dZ.upload(z)
        capi.call("sph_relu_backward_f32", dZ.at(4 * off), dG.at(4 * off), dX.at(4 * off), cnt)
        assert np.array_equal(bits(dZ.download(np.float32, (n + 1,))[off:]),
                              bits(po.relu_backward(zs, gs, xs)))
        dZ.upload(z)
        capi.call("sph_sgd_step_f32", dZ.at(4 * off), dG.at(4 * off), 0.0123, cnt)
        assert np.array_equal(bits(dZ.download(np.float32, (n + 1,))[off:]),
                              bits(po.sgd(zs, gs, 0.0123)))
    # in place: y = y * f and z = z - g, as Compute::Scale(dB, dB, ..) and Compute::Sub(z, z, ..) do
    dZ.upload(z)
    capi.call("sph_scale_f32", dZ.ptr, dZ.ptr, -2.5, n + 1)
    assert np.array_equal(bits(dZ.download(np.float32, (n + 1,))), bits(po.scale(z, -2.5)))
    dZ.upload(z)
    capi.call("sph_sub_f32", dZ.ptr, dZ.ptr, dG.ptr, n + 1, 0, 0, 0)
    assert np.array_equal(bits(dZ.download(np.float32, (n + 1,))), bits(po.sub_leaf(z, g, n + 1)))
    for d in (dX, dG, dZ, dY):
        d.release()


def test_sgd_step_keeps_the_two_roundings(dev):
    h.announce("sph_sgd_step_f32 rounding probe")
    z = np.array([1.9026086330413818] * 5, np.float32)
    dz = np.array([1.7237802743911743] * 5, np.float32)
    lr = float(np.float32(0.5041077733039856))
    dZ, dG = capi.DeviceBuffer.from_array(z), capi.DeviceBuffer.from_array(dz)
    capi.call("sph_sgd_step_f32", dZ.ptr, dG.ptr, lr, 5)
    got = dZ.download(np.float32, (5,))
    assert np.array_equal(bits(got), bits(po.sgd(z, dz, lr)))
    fused = np.float32(np.float64(z[0]) - np.float64(dz[0]) * np.float64(np.float32(lr)))
    assert got[0] != fused
    dZ.release()
    dG.release()


@pytest.mark.parametrize("case", [(60, 12, True, False), (60, 5, False, True),
                                  (64, 16, True, True), (100003, 1000, False, True)])
def test_sub_with_wrapping_operands(dev, case):
    count, stride, bca, bcb = case
    h.announce("sph_sub_f32 wrap", case)
    a = synth.uniform(7, (count,))
    b = synth.uniform(8, (count,))
    dA, dB = capi.DeviceBuffer.from_array(a), capi.DeviceBuffer.from_array(b)
    dY = capi.DeviceBuffer(4 * count)
    capi.call("sph_sub_f32", dY.ptr, dA.ptr, dB.ptr, count, stride, int(bca), int(bcb))
    assert np.array_equal(bits(dY.download(np.float32, (count,))),
                          bits(po.sub_leaf(a, b, count, stride, bca, bcb)))
    with pytest.raises(capi.SphError):
        capi.call("sph_sub_f32", dY.ptr, dA.ptr, dB.ptr, count, 0, 1, 0)
    for d in (dA, dB, dY):
        d.release()


def test_stream_ordered_allocation(dev):
    h.announce("sph_malloc_async / sph_free_async / sph_mem_pool_trim")
    import ctypes
    n = 1 << 16
    seen = set()
    for rep in range(5):
        ptr = capi._vp()
        capi.call("sph_malloc_async", ctypes.byref(ptr), 4 * n)
        assert ptr.value
        seen.add(ptr.value)
        capi.call("sph_fill_f32", ptr.value, float(rep), n)      # ordered after the allocation
        out = np.empty(n, np.float32)
        capi.call("sph_memcpy_d2h", out.ctypes.data, ptr.value, 4 * n)
        assert np.all(out == rep)
        capi.call("sph_free_async", ptr.value)
    assert len(seen) <= 5
    capi.call("sph_free_async", None)                             # a null pointer is accepted
    capi.sync()
    capi.call("sph_mem_pool_trim")
    empty = capi._vp()
    capi.call("sph_malloc_async", ctypes.byref(empty), 0)        # zero bytes still gives a block
    assert empty.value
    capi.call("sph_free_async", empty.value)
