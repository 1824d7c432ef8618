"""Recorded sequences (HIP graphs) against the same calls issued one by one.

Every replay is checked, with eager work and synchronisations between the replays, because a
graph that is right on its first replay can still be wrong on later ones."""
import numpy as np
import pytest

from sapphire_amd import capi, synth
from tests import helpers as h

pytestmark = pytest.mark.gpu


def bits(x):
    return np.ascontiguousarray(x).view(np.uint32)


class Mlp:
    """Buffers of a 3-layer network and its forward / backward call sequences."""

    def __init__(self, batch, sizes, seed):
        self.batch, self.sizes = batch, sizes
        self.W0 = [synth.uniform(seed + l, (sizes[l], sizes[l + 1])) for l in range(3)]
        self.b0 = [synth.uniform(seed + 10 + l, (sizes[l + 1],)) for l in range(3)]
        self.W = [capi.DeviceBuffer.from_array(w) for w in self.W0]
        self.b = [capi.DeviceBuffer.from_array(v) for v in self.b0]
        self.x = capi.DeviceBuffer(4 * batch * sizes[0])
        self.y = [capi.DeviceBuffer(4 * batch * n) for n in sizes[1:]]
        self.dy = capi.DeviceBuffer(4 * batch * sizes[3])
        self.grad = [capi.DeviceBuffer(4 * batch * n) for n in sizes]
        self.dpre = [capi.DeviceBuffer(4 * batch * n) for n in sizes[1:3]]
        big = max(sizes[l] * sizes[l + 1] for l in range(3))
        self.dw = capi.DeviceBuffer(4 * big)
        self.dB = capi.DeviceBuffer(4 * max(sizes))
        self.ones = capi.DeviceBuffer.from_array(np.ones(batch, np.float32))

    def reset_parameters(self):
        for d, w in zip(self.W, self.W0):
            d.upload(w)
        for d, v in zip(self.b, self.b0):
            d.upload(v)

    def forward(self):
        cur = self.x
        for l in range(3):
            capi.call("sph_linear_forward_f32", self.y[l].ptr, cur.ptr, self.W[l].ptr,
                      self.b[l].ptr, self.batch, self.sizes[l], self.sizes[l + 1],
                      capi.SPH_LINEAR_RELU if l < 2 else 0)
            cur = self.y[l]

    def backward(self, lr):
        """Direct sequence of the Linear backward + SGD update, ReLU backward between layers
        (y of a hidden layer is post-ReLU, and y > 0 exactly where its pre-activation was)."""
        TA, TB, OV = capi.SPH_GEMM_TRANS_A, capi.SPH_GEMM_TRANS_B, capi.SPH_GEMM_OVERWRITE
        batch, sizes = self.batch, self.sizes
        dy = self.dy
        for l in (2, 1, 0):
            n_in, n_out = sizes[l], sizes[l + 1]
            x = self.x if l == 0 else self.y[l - 1]
            capi.call("sph_gemm_f32_ex", self.grad[l].ptr, dy.ptr, self.W[l].ptr, batch, n_in,
                      n_out, 1, batch * n_in, batch * n_out, n_in * n_out, TB | OV)
            capi.call("sph_gemm_f32_ex", self.dw.ptr, x.ptr, dy.ptr, n_in, n_out, batch, 1,
                      n_in * n_out, n_in * batch, batch * n_out, TA | OV)
            capi.call("sph_sgd_step_f32", self.W[l].ptr, self.dw.ptr, lr, n_in * n_out)
            capi.call("sph_gemm_f32_ex", self.dB.ptr, self.ones.ptr, dy.ptr, 1, n_out, batch, 1,
                      n_out, batch, batch * n_out, OV)
            capi.call("sph_scale_f32", self.dB.ptr, self.dB.ptr, 1.0 / batch, n_out)
            capi.call("sph_sgd_step_f32", self.b[l].ptr, self.dB.ptr, lr, n_out)
            if l > 0:
                capi.call("sph_fill_f32", self.dpre[l - 1].ptr, 0.0, batch * n_in)
                capi.call("sph_relu_backward_f32", self.dpre[l - 1].ptr, self.grad[l].ptr,
                          self.y[l - 1].ptr, batch * n_in)
                dy = self.dpre[l - 1]

    def state(self):
        out = [self.y[2].download(np.float32, (self.batch, self.sizes[3]))]
        out += [d.download(np.float32, w.shape) for d, w in zip(self.W, self.W0)]
        out += [d.download(np.float32, v.shape) for d, v in zip(self.b, self.b0)]
        return out

    def release(self):
        for d in (self.W + self.b + self.y + self.grad + self.dpre +
                  [self.x, self.dy, self.dw, self.dB, self.ones]):
            d.release()


# the third network has ragged extents everywhere: its products are split by the launcher into
# several launches each (columns that are no multiple of 4, rows of a transposed operand)
@pytest.mark.parametrize("shape", [(64, [20, 48, 32, 10]), (1024, [784, 1024, 1024, 10]),
                                   (257, [301, 262, 131, 10])])
def test_training_step_replays_match_eager(dev, shape):
    batch, sizes = shape
    h.announce("graph of forward + backward + SGD", shape)
    net = Mlp(batch, sizes, 700)
    inputs = [(synth.uniform(800 + i, (batch, sizes[0])), synth.uniform(900 + i, (batch, sizes[3])))
              for i in range(4)]
    lr = 0.05

    # eager: four training steps from the initial parameters, state after each
    net.reset_parameters()
    eager = []
    for x, dy in inputs:
        net.x.upload(x)
        net.dy.upload(dy)
        net.forward()
        net.backward(lr)
        eager.append(net.state())

    # recorded once, replayed four times; uploads, downloads and syncs in between are eager
    net.reset_parameters()
    with capi.Graph() as graph:
        net.forward()
        net.backward(lr)
    after_capture = net.state()[1:]
    for got, want in zip(after_capture, net.W0 + net.b0):
        assert np.array_equal(bits(got), bits(want)), "recording must not run the work"
    for i, (x, dy) in enumerate(inputs):
        net.x.upload(x)
        net.dy.upload(dy)
        graph.launch()
        capi.sync()
        for got, want in zip(net.state(), eager[i]):
            assert np.array_equal(bits(got), bits(want)), "replay %d" % i
    graph.destroy()
    net.release()


def test_blocking_calls_are_refused_during_capture_and_capture_survives(dev):
    h.announce("graph capture: refused calls")
    n = 1000
    x = synth.uniform(5, (n,))
    dX = capi.DeviceBuffer.from_array(x)
    dY = capi.DeviceBuffer(4 * n)
    host = np.zeros(n, np.float32)
    words = capi.DeviceBuffer(4 * 64)
    with capi.Graph() as graph:
        capi.call("sph_scale_f32", dY.ptr, dX.ptr, 3.0, n)
        for name, args in [("sph_stream_sync", ()),
                           ("sph_memcpy_d2h", (host.ctypes.data, dY.ptr, 4 * n)),
                           ("sph_memcpy_h2d", (dY.ptr, host.ctypes.data, 4 * n))]:
            with pytest.raises(capi.SphError) as err:
                capi.call(name, *args)
            assert err.value.status == 3 and "captured" in str(err.value)
        # the one-call conversions and products take a scratch allocation: refused as well,
        # before anything of theirs is recorded
        for name, args in [("sph_csr_from_dense_f32", (words.ptr, words.ptr, words.ptr, 8, dX.ptr,
                                                       4, 128, 128, None)),
                           ("sph_spgemm_f32", (words.ptr, words.ptr, words.ptr, 8, dX.ptr, words.ptr,
                                               words.ptr, dX.ptr, words.ptr, words.ptr, 4, 4, 4,
                                               None)),
                           ("sph_spgemm_load_u32", (words.ptr, words.ptr, words.ptr, 4, 4,
                                                    capi.ctypes.byref(capi.ctypes.c_uint64(0))))]:
            with pytest.raises(capi.SphError) as err:
                capi.call(name, *args)
            assert err.value.status == 3 and "captured" in str(err.value)
        with pytest.raises(capi.SphError):
            capi.call("sph_graph_begin_capture")
        capi.call("sph_relu_f32", dY.ptr, dY.ptr, n)
    for _ in range(3):
        capi.call("sph_fill_f32", dY.ptr, -1.0, n)      # eager work between replays
        graph.launch()
        got = dY.download(np.float32, (n,))
        want = np.maximum(x * np.float32(3.0), 0)
        assert np.array_equal(bits(got), bits(want.astype(np.float32)))
    graph.destroy()
    with pytest.raises(capi.SphError):
        handle = capi._vp()
        capi.call("sph_graph_end_capture", capi.ctypes.byref(handle))   # nothing in progress
    dX.release()
    dY.release()
    words.release()


def test_non_affine_broadcast_walk_recorded_into_a_graph(dev):
    """The leaf list of a broadcast walk whose offsets are not affine (the reference's
    (chunk % size) * stride rule, here out[u] += A[u % 3] * B[(2 * u) % 5]) kept in a device
    table the caller owns and launched with sph_gemm_f32_grouped_device inside a recorded
    graph; every replay equals the eager grouped launch bit for bit."""
    from oracle import pyoracle as po
    M, N, K, units = 48, 40, 36, 10
    h.announce("sph_gemm_f32_grouped_device in a graph", (M, N, K, units))
    A = synth.uniform(9101, (3, M, K))
    B = synth.uniform(9102, (5, K, N))
    C0 = synth.uniform(9103, (units, M, N))
    triples = [(u * M * N, (u % 3) * M * K, ((2 * u) % 5) * K * N) for u in range(units)]
    table = np.array(triples, dtype=np.uint64)
    dTable = capi.DeviceBuffer.from_array(table)
    dA, dB = capi.DeviceBuffer.from_array(A), capi.DeviceBuffer.from_array(B)
    dC = capi.DeviceBuffer.from_array(C0)
    with capi.Graph() as g:
        with pytest.raises(capi.SphError):          # the uploading form refuses a capture
            capi.call("sph_gemm_f32_grouped", capi.make_entries(triples), units, dC.ptr, dA.ptr,
                      dB.ptr, M, N, K)
        capi.call("sph_gemm_f32_grouped_device", dTable.ptr, units, dC.ptr, dA.ptr, dB.ptr, M, N, K,
                  capi.SPH_GROUPED_OFFSETS_MULTIPLE_OF_4)
    ref = C0.copy()
    for rep in range(3):
        g.launch()
        capi.sync()
        got = dC.download(np.float32, C0.shape)
        for o, a, b in triples:
            u = o // (M * N)
            ref[u] = po.naive_gemm(ref[u], A[a // (M * K)], B[b // (K * N)], M, N, K)
        den = 1.0 + (rep + 1) * K
        assert float(np.max(np.abs(got - ref))) <= 1e-4 * den
        # eager work between the replays: the same walk through the uploading entry point on a copy
        eager = h.gpu_gemm_grouped(C0, A, B, M, N, K, triples)
        if rep == 0:
            assert np.array_equal(bits(eager), bits(got))
    g.destroy()
    for d in (dTable, dA, dB, dC):
        d.release()
