"""Several host threads driving the C ABI at once: every thread has its own stream, the shared
pieces (the offset table of grouped launches, the error text) must not mix their work up."""
import threading

import numpy as np
import pytest

from oracle import pyoracle as po
from sapphire_amd import capi, synth
from tests import helpers as h

pytestmark = pytest.mark.gpu
TOL_F32 = 1e-4


def test_threads_get_distinct_streams_and_independent_results(dev):
    h.announce("C ABI from 4 threads: plain, grouped and sparse launches interleaved")
    M, N, K = 96, 80, 64
    cases = []
    for t in range(4):
        A = synth.uniform(200 + t, (3, M, K))
        B = synth.uniform(300 + t, (3, K, N))
        C = synth.uniform(400 + t, (3, M, N))
        ref = po.gemm_rows(C.copy(), A, B, M, N, K, batch=3)
        v, col, row = synth.csr_matrix(500 + t, 64, 128, 6.0)
        D = synth.uniform(600 + t, (128, 32))
        sref = po.spmm_csr(np.zeros((64, 32), np.float32), v, col, row, 64, 32, D)
        cases.append((A, B, C, ref, v, col, row, D, sref))

    streams, errors = [None] * 4, []

    def worker(t):
        try:
            A, B, C, ref, v, col, row, D, sref = cases[t]
            capi.call("sph_set_device", 0)
            handle = capi._vp()
            capi.call("sph_get_stream", capi.ctypes.byref(handle))
            streams[t] = handle.value
            triples = [(u * M * N, u * M * K, u * K * N) for u in range(3)]
            den = np.stack([np.abs(A[u]).astype(np.float64) @ np.abs(B[u]) for u in range(3)])
            for rep in range(15):
                got = h.gpu_gemm_f32(C, A, B, M, N, K, batch=3)
                assert h.normalised_error(got, ref, None, den, True) <= TOL_F32
                got = h.gpu_gemm_grouped(C, A, B, M, N, K, triples)
                assert h.normalised_error(got, ref, None, den, True) <= TOL_F32
                got = h.gpu_spmm(np.zeros((64, 32), np.float32), v, col, row, 64, 128, 32, D, False)
                assert np.array_equal(got.view(np.uint32), sref.view(np.uint32))
            # an error raised in this thread carries this thread's text
            with pytest.raises(capi.SphError) as err:
                capi.call("sph_gemm_f32", 0, 0, 0, 0, 1, 1, 1, 0, 0, 0)
            assert "sph_gemm_f32" in str(err.value)
        except BaseException as exc:  # noqa: BLE001 - reported by the main thread
            errors.append((t, repr(exc)))

    threads = [threading.Thread(target=worker, args=(t,)) for t in range(4)]
    for th in threads:
        th.start()
    for th in threads:
        th.join()
    assert not errors, errors
    assert len(set(streams)) == 4 and all(streams), streams


def test_concurrent_grouped_launches_with_growing_tables(dev):
    """Grouped launches from 4 threads at once, each with its own offset tables of growing
    length (the tables are per thread: no thread waits for another, none sees another's
    offsets), including lists with repeated output units that are cut into ordered launches."""
    h.announce("sph_gemm_f32_grouped from 4 threads, tables of 3 .. 3000 entries")
    M, N, K = 16, 24, 8
    errors = []

    def worker(t):
        try:
            capi.call("sph_set_device", 0)
            for count in (3, 40, 1500, 3000, 7):
                units = count
                A = synth.uniform(700 + t, (units, M, K))
                B = synth.uniform(800 + t, (5, K, N))
                C = synth.uniform(900 + t, (max(units // 2, 1), M, N))
                # unit u: out[u % outs] += A[u] * B[(u * 7 + t) % 5]: non-affine, outputs repeat
                outs = C.shape[0]
                triples = [((u % outs) * M * N, u * M * K, ((u * 7 + t) % 5) * K * N)
                           for u in range(units)]
                ref = C.copy()
                for o, a, b in triples:
                    ref[o // (M * N)] = po.naive_gemm(ref[o // (M * N)], A[a // (M * K)],
                                                      B[b // (K * N)], M, N, K)
                got = h.gpu_gemm_grouped(C, A, B, M, N, K, triples)
                assert np.allclose(got, ref, rtol=1e-4, atol=1e-4), (t, count)
        except BaseException as exc:  # noqa: BLE001 - reported by the main thread
            errors.append((t, repr(exc)))

    threads = [threading.Thread(target=worker, args=(t,)) for t in range(4)]
    for th in threads:
        th.start()
    for th in threads:
        th.join()
    assert not errors, errors
