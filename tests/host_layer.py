"""ctypes view of tests/host_harness/libhost_harness.so (the C++ operator layer)."""
import ctypes
import os

import numpy as np

HERE = os.path.dirname(os.path.abspath(__file__))
LIB_PATH = os.path.join(HERE, "host_harness", "libhost_harness.so")

_ip = ctypes.POINTER(ctypes.c_int)
_fp = ctypes.POINTER(ctypes.c_float)
_lib = None


def lib():
    global _lib
    if _lib is None:
        if not os.path.exists(LIB_PATH):
            raise RuntimeError("%s missing: python -m sapphire_amd.build host harness" % LIB_PATH)
        h = ctypes.CDLL(LIB_PATH)
        h.sphh_last_error.restype = ctypes.c_char_p
        h.sphh_gemm_plan.restype = ctypes.c_long
        h.sphh_gemm_plan.argtypes = [_ip, ctypes.c_int, _ip, ctypes.c_int, _ip, ctypes.c_int, _ip,
                                     ctypes.POINTER(ctypes.c_ulonglong), ctypes.c_long,
                                     ctypes.POINTER(ctypes.c_longlong)]
        h.sphh_compute_gemm.argtypes = [_fp, _ip, ctypes.c_int, _fp, _ip, ctypes.c_int, _fp, _ip,
                                        ctypes.c_int]
        h.sphh_compute_gemm_fresh_y.argtypes = h.sphh_compute_gemm.argtypes
        h.sphh_gemm_half.argtypes = [_fp, _ip, ctypes.c_int, ctypes.c_void_p, ctypes.c_void_p,
                                     ctypes.c_uint, ctypes.c_int]
        h.sphh_bench_gemm_half_fresh_y.argtypes = [ctypes.c_void_p, ctypes.c_void_p, ctypes.c_int,
                                                   ctypes.c_int, ctypes.c_int, ctypes.c_double,
                                                   _fp, ctypes.POINTER(ctypes.c_double)]
        h.sphh_k_partition.argtypes = [ctypes.c_uint] * 5 + [ctypes.POINTER(ctypes.c_uint)]
        h.sphh_k_partition_slot.argtypes = [ctypes.c_uint] * 7
        h.sphh_k_partition_slot.restype = ctypes.c_uint
        h.sphh_transpose.argtypes = [_fp, _ip, ctypes.c_int, _fp, _ip, ctypes.c_int]
        h.sphh_mlp_forward.argtypes = [_fp, ctypes.c_int, _ip, ctypes.c_int,
                                       ctypes.POINTER(_fp), ctypes.POINTER(_fp), _fp, ctypes.c_int]
        h.sphh_sparse_gemm.argtypes = [_fp, ctypes.c_int, ctypes.c_int, ctypes.c_int, _fp,
                                       ctypes.POINTER(ctypes.c_uint), ctypes.POINTER(ctypes.c_uint),
                                       _fp, ctypes.c_int]
        h.sphh_matching_dim.argtypes = [_ip, _ip, ctypes.c_int]
        h.sphh_sub.argtypes = [_fp, _ip, ctypes.c_int, _fp, _ip, ctypes.c_int, _fp, _ip,
                               ctypes.c_int]
        h.sphh_scale.argtypes = [_fp, _fp, ctypes.c_int, ctypes.c_float, ctypes.c_int]
        h.sphh_relu_backward.argtypes = [_fp, _fp, _fp, ctypes.c_int]
        h.sphh_linear_backward.argtypes = [_fp, _fp, _fp, _fp, _fp, ctypes.c_int, ctypes.c_int,
                                           ctypes.c_int, ctypes.c_float, ctypes.c_int,
                                           ctypes.c_int]
        up = ctypes.POINTER(ctypes.c_uint)
        h.sphh_csr_round_trip.argtypes = [_fp, ctypes.c_uint, ctypes.c_uint, ctypes.c_uint,
                                          ctypes.c_uint, up, _fp, up, up, ctypes.c_ulong, _fp,
                                          ctypes.c_float]
        h.sphh_sparse_sparse_gemm.argtypes = [_fp, _fp, ctypes.c_uint, ctypes.c_uint, ctypes.c_uint,
                                              up, up, _fp, up, ctypes.c_ulong]
        h.sphh_matmul_backward.argtypes = [_fp, _fp, _fp, _fp, _fp, _ip, ctypes.c_int, _ip,
                                           ctypes.c_int, _ip, ctypes.c_int, ctypes.c_int]
        h.sphh_sparse_linear_forward.argtypes = [_fp, ctypes.c_int, ctypes.c_int, ctypes.c_int,
                                                 _fp, _fp, _fp]
        h.sphh_shape_op.argtypes = [_ip, ctypes.c_int, ctypes.c_int, ctypes.c_int, _ip]
        h.sphh_shape_query.argtypes = [_ip, ctypes.c_int, ctypes.c_int, ctypes.c_int]
        _lib = h
    return _lib


def _ints(v):
    return (ctypes.c_int * max(len(v), 1))(*[int(x) for x in v])


def _f(a):
    assert a.dtype == np.float32 and a.flags["C_CONTIGUOUS"]
    return a.ctypes.data_as(_fp)


def _ok(rc):
    if rc != 0:
        raise RuntimeError(lib().sphh_last_error().decode())


def shape_op(dims, op, arg=0):
    out = (ctypes.c_int * 32)()
    n = lib().sphh_shape_op(_ints(dims), len(dims), op, arg, out)
    if n < 0:
        raise RuntimeError(lib().sphh_last_error().decode())
    return [out[i] for i in range(n)]


def shape_query(dims, what, arg=0):
    return lib().sphh_shape_query(_ints(dims), len(dims), what, arg)


def gemm_plan(ys, as_, bs):
    cap = 1 << 16
    leaves = (ctypes.c_ulonglong * (4 * cap))()
    dims = (ctypes.c_int * 7)()
    strided = (ctypes.c_longlong * 5)()
    n = lib().sphh_gemm_plan(_ints(ys), len(ys), _ints(as_), len(as_), _ints(bs), len(bs), dims,
                             leaves, cap, strided)
    if n < 0:
        raise RuntimeError(lib().sphh_last_error().decode())
    d = dict(M=dims[0], N=dims[1], K=dims[2], maxDim=dims[3], sizeOut=dims[4], sizeA=dims[5],
             sizeB=dims[6])
    out = [tuple(int(leaves[4 * i + j]) for j in range(4)) for i in range(n)]
    return d, out, [int(x) for x in strided]


def compute_gemm(y, a, b):
    """Compute::Gemm(y, a, b) in Cuda mode on numpy arrays; returns the new y."""
    out = np.ascontiguousarray(y.copy())
    _ok(lib().sphh_compute_gemm(_f(out), _ints(y.shape), y.ndim, _f(np.ascontiguousarray(a)),
                                _ints(a.shape), a.ndim, _f(np.ascontiguousarray(b)),
                                _ints(b.shape), b.ndim))
    return out


def compute_gemm_fresh_y(y_shape, a, b):
    """Compute::Gemm(y, a, b) with y a NEW TensorData of y_shape (never filled by the caller)."""
    out = np.full(y_shape, np.float32(-777.0))
    _ok(lib().sphh_compute_gemm_fresh_y(_f(out), _ints(y_shape), len(y_shape),
                                        _f(np.ascontiguousarray(a)), _ints(a.shape), a.ndim,
                                        _f(np.ascontiguousarray(b)), _ints(b.shape), b.ndim))
    return out


def gemm_half(y, a_dev_ptr, b_dev_ptr, K, fresh_y):
    """Compute::GemmHalf(y, a, b, K) on device arrays of binary16; y is a numpy array whose
    contents are uploaded unless fresh_y (then y is a new TensorData of that shape)."""
    out = np.ascontiguousarray(y.copy())
    _ok(lib().sphh_gemm_half(_f(out), _ints(y.shape), y.ndim, a_dev_ptr, b_dev_ptr, K,
                             1 if fresh_y else 0))
    return out


def bench_gemm_half_fresh_y(a_dev_ptr, b_dev_ptr, n, steps, warmup, settle_ms):
    """(event ms, wall ms) per pass of: fresh y from the pool, Compute::GemmHalf, Clean()."""
    ev = ctypes.c_float(0)
    wall = ctypes.c_double(0)
    _ok(lib().sphh_bench_gemm_half_fresh_y(a_dev_ptr, b_dev_ptr, n, steps, warmup, settle_ms,
                                           ctypes.byref(ev), ctypes.byref(wall)))
    return ev.value, wall.value


def k_partition(K, group_k, waves, wave, depth):
    """The few-tile kernels' K partition for one wavefront, from the kernels' own header."""
    out = (ctypes.c_uint * 7)()
    lib().sphh_k_partition(K, group_k, waves, wave, depth, out)
    keys = ("g_begin", "g_end", "whole", "whole_end", "last_whole", "rounds_end", "owns_partial")
    return dict(zip(keys, [int(v) for v in out]))


def k_partition_slot(K, group_k, waves, wave, depth, g, d):
    """Group held by slot d of the load pipeline: before the first round (g None) or the one
    loaded while the round that starts at group g is multiplied."""
    return int(lib().sphh_k_partition_slot(K, group_k, waves, wave, depth,
                                           0xffffffff if g is None else g, d))


def transpose(x, y_shape):
    out = np.zeros(y_shape, np.float32)
    _ok(lib().sphh_transpose(_f(out), _ints(y_shape), len(y_shape), _f(np.ascontiguousarray(x)),
                             _ints(x.shape), x.ndim))
    return out


def mlp_forward(x, weights, biases, fused=False):
    sizes = [x.shape[1]] + [w.shape[1] for w in weights]
    out = np.zeros((x.shape[0], sizes[-1]), np.float32)
    wp = (_fp * len(weights))(*[_f(w) for w in weights])
    bp = (_fp * len(biases))(*[_f(b) for b in biases])
    _ok(lib().sphh_mlp_forward(_f(x), x.shape[0], _ints(sizes), len(weights), wp, bp, _f(out),
                               1 if fused else 0))
    return out


def sparse_gemm(y, V, COL, ROW, M, K, N, B, accumulate):
    out = np.ascontiguousarray(y.copy())
    up = ctypes.POINTER(ctypes.c_uint)
    Vp = V if V.size else np.zeros(1, np.float32)
    Cp = COL if COL.size else np.zeros(1, np.uint32)
    _ok(lib().sphh_sparse_gemm(_f(out), M, K, N, _f(Vp), Cp.ctypes.data_as(up),
                               ROW.ctypes.data_as(up), _f(B), 1 if accumulate else 0))
    return out


def matching_dim(shapes):
    flat = [d for s in shapes for d in s]
    n = lib().sphh_matching_dim(_ints(flat), _ints([len(s) for s in shapes]), len(shapes))
    if n < 0:
        raise RuntimeError(lib().sphh_last_error().decode())
    return n


def sub(y_shape, a, b):
    out = np.zeros(y_shape, np.float32)
    _ok(lib().sphh_sub(_f(out), _ints(y_shape), len(y_shape), _f(np.ascontiguousarray(a)),
                       _ints(a.shape), a.ndim, _f(np.ascontiguousarray(b)), _ints(b.shape),
                       b.ndim))
    return out


def scale(x, factor, in_place=False):
    out = np.zeros_like(x)
    _ok(lib().sphh_scale(_f(out), _f(x), x.size, factor, 1 if in_place else 0))
    return out


def relu_backward(dx, dy, x):
    out = np.ascontiguousarray(dx.copy())
    _ok(lib().sphh_relu_backward(_f(out), _f(dy), _f(x), x.size))
    return out


def linear_backward(dx, W, bias, dy, x, lr, sequence, fused_sgd):
    """Returns the updated (dx, W, bias)."""
    dx, W, bias = (np.ascontiguousarray(v.copy()) for v in (dx, W, bias))
    batch, inputs = x.shape
    _ok(lib().sphh_linear_backward(_f(dx), _f(W), _f(bias), _f(dy), _f(x), batch, inputs,
                                   W.shape[1], lr, sequence, 1 if fused_sgd else 0))
    return dx, W, bias


def csr_round_trip(dense, n, fill=7.0):
    """dense: [numMatrices, m, paddedN].  Returns (nnz per matrix, V, COL, ROW [numMatrices, m+1],
    dense again) through the device-side conversion, copies and back-conversion."""
    num, m, padded = dense.shape
    up = ctypes.POINTER(ctypes.c_uint)
    cap = max(int(np.count_nonzero(dense)) + 8, 8)
    nnz = np.zeros(max(num, 1), np.uint32)
    V = np.zeros(cap, np.float32)
    COL = np.zeros(cap, np.uint32)
    ROW = np.zeros((max(num, 1), m + 1), np.uint32)
    back = np.zeros(dense.shape if dense.size else (1,), np.float32)
    src = np.ascontiguousarray(dense) if dense.size else np.zeros(1, np.float32)
    _ok(lib().sphh_csr_round_trip(_f(src), m, n, padded, num, nnz.ctypes.data_as(up), _f(V),
                                  COL.ctypes.data_as(up), ROW.ctypes.data_as(up), cap, _f(back),
                                  fill))
    total = int(nnz[:num].sum())
    return nnz[:num], V[:total], COL[:total], ROW[:num], back.reshape(dense.shape) if dense.size else back


def sparse_linear_forward(x, W, bias):
    batch, inputs = x.shape
    out = np.zeros((batch, W.shape[1]), np.float32)
    _ok(lib().sphh_sparse_linear_forward(_f(x), batch, inputs, W.shape[1],
                                         _f(np.ascontiguousarray(W)), _f(bias), _f(out)))
    return out


def sparse_sparse_gemm(dA, dB, capacity):
    """(V, COL, ROW) of the CSR x CSR product of two dense-given matrices."""
    m, k = dA.shape
    n = dB.shape[1]
    up = ctypes.POINTER(ctypes.c_uint)
    nnz = ctypes.c_uint(0)
    ROW = np.zeros(m + 1, np.uint32)
    V = np.zeros(max(capacity, 1), np.float32)
    COL = np.zeros(max(capacity, 1), np.uint32)
    _ok(lib().sphh_sparse_sparse_gemm(_f(np.ascontiguousarray(dA)), _f(np.ascontiguousarray(dB)),
                                      m, k, n, ctypes.byref(nnz), ROW.ctypes.data_as(up), _f(V),
                                      COL.ctypes.data_as(up), capacity))
    return V[:nnz.value], COL[:nnz.value], ROW


def load_dist(dA, dB):
    """(load, COL, ROW, products) of the load-distribution pre-pass for two dense-given matrices."""
    m, k = dA.shape
    n = dB.shape[1]
    up = ctypes.POINTER(ctypes.c_uint)
    h = lib()
    h.sphh_load_dist.argtypes = [_fp, _fp, ctypes.c_uint, ctypes.c_uint, ctypes.c_uint, up, up, up,
                                 up, up, ctypes.c_ulong]
    h.sphh_load_dist.restype = ctypes.c_int
    capacity = max(int(np.count_nonzero(dA)), 1)
    nnz = ctypes.c_uint(0)
    products = ctypes.c_uint(0)
    load = np.zeros(capacity, np.uint32)
    col = np.zeros(capacity, np.uint32)
    row = np.zeros(m + 1, np.uint32)
    _ok(h.sphh_load_dist(_f(np.ascontiguousarray(dA)), _f(np.ascontiguousarray(dB)), m, k, n,
                         ctypes.byref(nnz), load.ctypes.data_as(up), col.ctypes.data_as(up),
                         row.ctypes.data_as(up), ctypes.byref(products), capacity))
    return load[:nnz.value], col[:nnz.value], row, products.value


def matmul_backward(da, db, dy, a, b, sequence):
    """Returns the accumulated (da, db)."""
    da, db = np.ascontiguousarray(da.copy()), np.ascontiguousarray(db.copy())
    _ok(lib().sphh_matmul_backward(_f(da), _f(db), _f(np.ascontiguousarray(dy)),
                                   _f(np.ascontiguousarray(a)), _f(np.ascontiguousarray(b)),
                                   _ints(a.shape), a.ndim, _ints(b.shape), b.ndim,
                                   _ints(dy.shape), dy.ndim, sequence))
    return da, db
