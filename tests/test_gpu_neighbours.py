"""One-pass neighbours of the path through the C ABI: fill, ReLU, transpose."""
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
