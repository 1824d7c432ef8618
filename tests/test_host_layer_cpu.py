"""The C++ operator layer without a GPU: Shape arithmetic and the broadcast plan must agree with
the reference's recorded answers and with the oracle; host-side life cycle and error paths."""
import json
import os

import pytest

from oracle import pyoracle as po
from sapphire_amd import synth
from tests import host_layer as hl
from tests.golden.cases import PLAN_CASES

GOLDEN = os.path.join(os.path.dirname(os.path.abspath(__file__)), "golden")


def test_shape_matches_recorded_reference_answers():
    for entry in json.load(open(os.path.join(GOLDEN, "shape_ops.json"))):
        dims = entry["dims"]
        assert hl.shape_query(dims, 0) == entry["rows"]
        assert hl.shape_query(dims, 1) == entry["cols"]
        assert hl.shape_query(dims, 2) == entry["size"]
        assert [hl.shape_query(dims, 3, k) for k in range(5)] == entry["units"]
        for k, want in enumerate(entry["expand"]):
            assert hl.shape_op(dims, 0, k) == want
        for k, want in zip(range(1, 7), entry["shrink"]):
            assert hl.shape_op(dims, 1, k) == want
    assert hl.shape_op([1, 4, 1, 5], 2) == [4, 5]           # Squeeze()
    assert hl.shape_op([3, 4, 5], 3) == [3, 5, 4]           # GetTranspose
    assert hl.shape_op([7], 3) == [7, 1]


def test_plan_matches_recorded_reference_walks():
    recorded = json.load(open(os.path.join(GOLDEN, "gemm_plans.json")))
    assert len(recorded) == len(PLAN_CASES)
    for rec in recorded:
        dims, leaves, _ = hl.gemm_plan(rec["y"], rec["a"], rec["b"])
        assert dims == rec["dims"], rec
        assert [list(l) for l in leaves] == rec["leaves"], rec


def test_plan_matches_oracle_on_random_shapes():
    rng = synth.bits64(0xBEEF, 6000)
    pos = 0
    for case in range(400):
        nd = int(rng[pos] % 4) + 2
        M, N, K = (int(rng[pos + 1 + i] % 5) + 1 for i in range(3))
        lead = [int(rng[pos + 4 + i] % 3) + 1 for i in range(nd - 2)]
        pos += 4 + nd - 2
        ys = lead + [M, N]

        def variant(tail):
            nonlocal pos
            keep = [(d if rng[pos + i] % 3 else 1) for i, d in enumerate(lead)]
            pos += len(lead)
            cut = int(rng[pos] % (len(keep) + 1))
            pos += 1
            return keep[cut:] + tail
        as_, bs = variant([M, K]), variant([K, N])
        want_dims, want_leaves = po.gemm_plan(ys, as_, bs)
        dims, leaves, strided = hl.gemm_plan(ys, as_, bs)
        assert (dims, leaves) == (want_dims, want_leaves), (ys, as_, bs)
        # when the plan claims to be one strided batch, expanding it must give the same units
        units = []
        for o, a, b, total in want_leaves:
            for u in range(total // (M * N)):
                units.append((o + u * M * N, a + u * M * K, b + u * K * N))
        if strided[0]:
            n, so, sa, sb = strided[1:]
            assert [(u * so, u * sa, u * sb) for u in range(n)] == units, (ys, as_, bs)


def test_strided_detection_on_known_cases():
    _, _, s = hl.gemm_plan([16, 512, 512], [16, 512, 512], [1, 512, 512])
    assert s == [1, 16, 512 * 512, 512 * 512, 0]
    _, _, s = hl.gemm_plan([7, 5, 3], [7, 5, 4], [7, 4, 3])
    assert s == [1, 7, 15, 20, 12]
    _, _, s = hl.gemm_plan([2, 3, 3, 2], [2, 1, 3, 2], [2, 3, 2, 2])     # modulo quirk: not affine
    assert s[0] == 0
    _, _, s = hl.gemm_plan([2, 4, 5], [6, 4, 2], [3, 2, 5])               # repeated outputs
    assert s[0] == 0


def test_host_life_cycle_and_error_paths():
    h = hl.lib()
    assert h.sphh_host_only_lifecycle() == 0, h.sphh_last_error()
    assert h.sphh_gemm_in_host_mode_throws() == 1
    assert b"Host mode is not provided" in h.sphh_last_error()
    with pytest.raises(RuntimeError, match="must be greater than zero"):
        hl.shape_op([2, 3], 0, -1)


def test_matching_dim_agrees_with_checker():
    cases = [[[3, 4], [3, 4], [3, 4]], [[2, 3, 4], [1, 3, 4], [2, 3, 4]], [[3, 4], [3, 5]],
             [[2, 3, 4], [3, 4]], [[5]], [[2, 3, 4], [2, 5, 4]], [[1, 1, 4, 5], [2, 3, 4, 5]]]
    for shapes in cases:
        assert hl.matching_dim(shapes) == po.matching_dim(shapes), shapes
    with pytest.raises(RuntimeError):
        hl.matching_dim([])


# ---- buffer pool bookkeeping: blocks are stream-affine ------------------------------------
def _pool_run(ops):
    import ctypes
    flat = (ctypes.c_int * (3 * len(ops)))(*[int(x) for op in ops for x in op])
    log = (ctypes.c_longlong * (3 * 64))()
    fn = hl.lib().sphh_block_pool_run
    fn.argtypes = [ctypes.POINTER(ctypes.c_int), ctypes.c_int, ctypes.POINTER(ctypes.c_longlong),
                   ctypes.c_int]
    n = fn(flat, len(ops), log, 64)
    assert 0 <= n <= 64, hl.lib().sphh_last_error()
    return [tuple(log[3 * i:3 * i + 3]) for i in range(n)]


GET, PRESERVE, CLEAN, FREE_PRESERVED, CLEAR_FREE, CLEAR_VOLATILE, CLEAR_PRESERVED = range(7)
HANDED, ALLOCATED, RELEASED, WAITS = range(4)


def test_pool_reuse_on_the_same_stream_needs_no_wait():
    log = _pool_run([(GET, 1, 1000), (CLEAN, 1, 0), (GET, 1, 1000)])
    # 1000 bytes round up to 1024; the second request takes the idle block of that size
    assert log == [(ALLOCATED, 1, 0), (HANDED, 1, 0), (HANDED, 1, 0)]


def test_pool_reuse_from_another_stream_waits_for_the_first():
    log = _pool_run([(GET, 1, 1000), (CLEAN, 1, 0), (GET, 2, 1024), (CLEAN, 2, 0), (GET, 2, 1024),
                     (GET, 2, 300)])
    assert log == [(ALLOCATED, 1, 0), (HANDED, 1, 0),
                   (WAITS, 2, 1), (HANDED, 1, 0),       # stream 2 takes over what stream 1 used
                   (HANDED, 1, 0),                      # now stream 2's own: no wait
                   (ALLOCATED, 2, 0), (HANDED, 2, 0)]   # another size: a fresh block


def test_pool_release_from_another_stream_waits_for_the_owner():
    log = _pool_run([(PRESERVE, 1, 512), (FREE_PRESERVED, 2, 1),
                     (GET, 1, 64), (CLEAN, 2, 0), (CLEAR_FREE, 2, 0),
                     (GET, 3, 64), (CLEAR_VOLATILE, 3, 0)])
    assert log == [(ALLOCATED, 1, 0), (HANDED, 1, 0),
                   (WAITS, 2, 1), (RELEASED, 1, 2),
                   (ALLOCATED, 2, 0), (HANDED, 2, 0),
                   (WAITS, 2, 1), (RELEASED, 2, 2),
                   (ALLOCATED, 3, 0), (HANDED, 3, 0), (RELEASED, 3, 3)]


def test_pool_unknown_block_is_refused():
    import ctypes
    flat = (ctypes.c_int * 3)(FREE_PRESERVED, 1, 77)
    log = (ctypes.c_longlong * 3)()
    fn = hl.lib().sphh_block_pool_run
    fn.argtypes = [ctypes.POINTER(ctypes.c_int), ctypes.c_int, ctypes.POINTER(ctypes.c_longlong),
                   ctypes.c_int]
    assert fn(flat, 1, log, 1) == -1
    assert b"Given ptr to free was not found" in hl.lib().sphh_last_error()
