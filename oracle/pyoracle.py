"""ctypes binding of the CPU checker -- TEST INFRASTRUCTURE ONLY.

Loads oracle/liboracle.so (the plain-C restatement) and, when it has been
built, oracle/_ref/libsapphire_ref.so (the reference's own host objects).
Only tests, the smoke check and the bench's cpu_baseline leg import this.
"""
import ctypes
import os

import numpy as np

_HERE = os.path.dirname(os.path.abspath(__file__))
ORACLE_PATH = os.path.join(_HERE, "liboracle.so")
REF_PATH = os.path.join(_HERE, "_ref", "libsapphire_ref.so")

ORC_MAX_DIM = 16


class OrcShape(ctypes.Structure):
    _fields_ = [("dim", ctypes.c_int), ("d", ctypes.c_int * ORC_MAX_DIM)]


class OrcLeaf(ctypes.Structure):
    _fields_ = [("outOff", ctypes.c_uint64), ("aOff", ctypes.c_uint64),
                ("bOff", ctypes.c_uint64), ("totalSizeOut", ctypes.c_uint32)]


class OrcGemmDims(ctypes.Structure):
    _fields_ = [("M", ctypes.c_uint), ("N", ctypes.c_uint), ("K", ctypes.c_uint),
                ("maxDim", ctypes.c_int), ("sizeOut", ctypes.c_int),
                ("sizeA", ctypes.c_int), ("sizeB", ctypes.c_int)]


_fp = ctypes.POINTER(ctypes.c_float)
_ip = ctypes.POINTER(ctypes.c_int)
_up = ctypes.POINTER(ctypes.c_uint32)
_u = ctypes.c_uint
_sz = ctypes.c_size_t


def _f(a):
    assert a.dtype == np.float32 and a.flags["C_CONTIGUOUS"]
    return a.ctypes.data_as(_fp)


def _ints(v):
    return (ctypes.c_int * max(len(v), 1))(*[int(x) for x in v])


_oracle = None
_ref = None


def oracle():
    global _oracle
    if _oracle is None:
        if not os.path.exists(ORACLE_PATH):
            raise RuntimeError("%s missing: run `make -C oracle`" % ORACLE_PATH)
        o = ctypes.CDLL(ORACLE_PATH)
        o.orc_naive_gemm.argtypes = [_u, _fp, _fp, _fp, _u, _u, _u]
        o.orc_naive_gemm.restype = None
        o.orc_gemm_rows.argtypes = [_fp, _fp, _fp, _u, _u, _u, _u, _sz, _sz, _sz, ctypes.c_int]
        o.orc_gemm_rows.restype = None
        o.orc_gemm_plan.argtypes = [_ip, ctypes.c_int, _ip, ctypes.c_int, _ip, ctypes.c_int,
                                    ctypes.POINTER(OrcGemmDims), ctypes.POINTER(OrcLeaf), _sz]
        o.orc_gemm_plan.restype = _sz
        o.orc_compute_gemm.argtypes = [_fp, _ip, ctypes.c_int, _fp, _ip, ctypes.c_int, _fp, _ip,
                                       ctypes.c_int, ctypes.c_int]
        o.orc_compute_gemm.restype = ctypes.c_int
        o.orc_relu.argtypes = [_fp, _fp, _u]
        o.orc_relu.restype = None
        o.orc_transpose.argtypes = [_fp, _fp, _u, _u, _u, ctypes.c_int]
        o.orc_transpose.restype = None
        o.orc_scale.argtypes = [_fp, _fp, ctypes.c_float, _u]
        o.orc_scale.restype = None
        o.orc_sub.argtypes = [_u, _fp, _fp, _fp, _u, ctypes.c_int, ctypes.c_int]
        o.orc_sub.restype = None
        o.orc_relu_backward.argtypes = [_fp, _fp, _fp, _u]
        o.orc_relu_backward.restype = None
        o.orc_get_matching_dim.argtypes = [ctypes.POINTER(OrcShape), ctypes.c_int]
        o.orc_get_matching_dim.restype = ctypes.c_int
        o.orc_compute_sub.argtypes = [_fp, _ip, ctypes.c_int, _fp, _ip, ctypes.c_int, _fp, _ip,
                                      ctypes.c_int]
        o.orc_compute_sub.restype = ctypes.c_int
        o.orc_sgd.argtypes = [_fp, _fp, ctypes.c_float, _u]
        o.orc_sgd.restype = None
        o.orc_linear_backward.argtypes = [_fp, _fp, _fp, _fp, _fp, _u, _u, _u, ctypes.c_float,
                                          ctypes.c_int]
        o.orc_linear_backward.restype = None
        o.orc_linear_forward.argtypes = [_fp, _fp, _fp, _fp, _u, _u, _u, ctypes.c_int]
        o.orc_linear_forward.restype = None
        o.orc_spmm_csr.argtypes = [_fp, _fp, _up, _up, ctypes.c_uint32, ctypes.c_uint32, _fp,
                                   ctypes.c_int]
        o.orc_spmm_csr.restype = None
        o.orc_csr_from_dense.argtypes = [_fp, _up, _up, _fp, ctypes.c_uint32, ctypes.c_uint32,
                                         ctypes.c_uint32]
        o.orc_csr_from_dense.restype = ctypes.c_uint32
        o.orc_csr_to_dense.argtypes = [_fp, ctypes.c_uint32, _fp, _up, _up, ctypes.c_uint32,
                                       ctypes.c_uint32]
        o.orc_csr_to_dense.restype = None
        o.orc_spgemm_csr.argtypes = [_fp, _up, _up, _fp, _up, _up, _fp, _up, _up,
                                     ctypes.c_uint32, ctypes.c_uint32, ctypes.c_uint32]
        o.orc_spgemm_csr.restype = ctypes.c_uint32
        for name in ("orc_shape_expand", "orc_shape_shrink"):
            getattr(o, name).argtypes = [ctypes.POINTER(OrcShape), ctypes.c_int]
            getattr(o, name).restype = ctypes.c_int
        for name in ("orc_shape_rows", "orc_shape_cols", "orc_shape_size"):
            getattr(o, name).argtypes = [ctypes.POINTER(OrcShape)]
            getattr(o, name).restype = ctypes.c_int
        o.orc_shape_num_units.argtypes = [ctypes.POINTER(OrcShape), ctypes.c_int]
        o.orc_shape_num_units.restype = ctypes.c_int
        _oracle = o
    return _oracle


def have_ref():
    return os.path.exists(REF_PATH)


def ref():
    """The reference's own objects; None when oracle/_ref has not been built."""
    global _ref
    if _ref is None and have_ref():
        r = ctypes.CDLL(REF_PATH)
        r.ref_naive_gemm.argtypes = [_u, _fp, _fp, _fp, _u, _u, _u]
        r.ref_naive_gemm.restype = None
        r.ref_relu.argtypes = [_fp, _fp, _u]
        r.ref_relu.restype = None
        r.ref_transpose.argtypes = [_fp, _fp, _u, _u, _u, ctypes.c_int]
        r.ref_transpose.restype = None
        r.ref_scale.argtypes = [_fp, _fp, ctypes.c_float, _u]
        r.ref_scale.restype = None
        r.ref_sub.argtypes = [_u, _fp, _fp, _fp, _u, ctypes.c_int, ctypes.c_int]
        r.ref_sub.restype = None
        r.ref_relu_backward.argtypes = [_fp, _fp, _fp, _u]
        r.ref_relu_backward.restype = None
        r.ref_compute_sub.argtypes = [_fp, _ip, ctypes.c_int, _fp, _ip, ctypes.c_int, _fp, _ip,
                                      ctypes.c_int, ctypes.c_int]
        r.ref_compute_sub.restype = None
        r.ref_shape_op.argtypes = [_ip, ctypes.c_int, ctypes.c_int, ctypes.c_int, _ip]
        r.ref_shape_op.restype = ctypes.c_int
        r.ref_shape_query.argtypes = [_ip, ctypes.c_int, ctypes.c_int, ctypes.c_int]
        r.ref_shape_query.restype = ctypes.c_int
        r.ref_gemm_plan.argtypes = [_ip, ctypes.c_int, _ip, ctypes.c_int, _ip, ctypes.c_int, _ip,
                                    ctypes.c_void_p, _sz]
        r.ref_gemm_plan.restype = _sz
        r.ref_compute_gemm.argtypes = [_fp, _ip, ctypes.c_int, _fp, _ip, ctypes.c_int, _fp, _ip,
                                       ctypes.c_int]
        r.ref_compute_gemm.restype = None
        _ref = r
    return _ref


# ---- numpy-level helpers -----------------------------------------------------

def make_shape(dims):
    s = OrcShape()
    s.dim = len(dims)
    for i, v in enumerate(dims):
        s.d[i] = int(v)
    return s


def shape_list(s):
    return [s.d[i] for i in range(s.dim)]


def naive_gemm(out, A, B, M, N, K):
    """out (float32, modified in place) += A*B over out.size/(M*N) chunks."""
    oracle().orc_naive_gemm(out.size, _f(out), _f(A), _f(B), M, N, K)
    return out


def gemm_rows(out, A, B, M, N, K, batch=1, stride_out=None, stride_a=None, stride_b=None,
              threads=8):
    so = M * N if stride_out is None else stride_out
    sa = M * K if stride_a is None else stride_a
    sb = K * N if stride_b is None else stride_b
    oracle().orc_gemm_rows(_f(out), _f(A), _f(B), M, N, K, batch, so, sa, sb, threads)
    return out


def gemm_plan(y_shape, a_shape, b_shape, lib=None):
    """(dims dict, [(outOff, aOff, bOff, totalSizeOut)]) from the oracle (or `lib`='ref')."""
    cap = 1 << 16
    leaves = (OrcLeaf * cap)()
    if lib == "ref":
        dims = (ctypes.c_int * 7)()
        n = ref().ref_gemm_plan(_ints(y_shape), len(y_shape), _ints(a_shape), len(a_shape),
                                _ints(b_shape), len(b_shape), dims, leaves, cap)
        d = dict(M=dims[0], N=dims[1], K=dims[2], maxDim=max(dims[3], 2), sizeOut=dims[4],
                 sizeA=dims[5], sizeB=dims[6])
    else:
        gd = OrcGemmDims()
        n = oracle().orc_gemm_plan(_ints(y_shape), len(y_shape), _ints(a_shape), len(a_shape),
                                   _ints(b_shape), len(b_shape), ctypes.byref(gd), leaves, cap)
        d = dict(M=gd.M, N=gd.N, K=gd.K, maxDim=gd.maxDim, sizeOut=gd.sizeOut, sizeA=gd.sizeA,
                 sizeB=gd.sizeB)
    assert n <= cap
    return d, [(leaves[i].outOff, leaves[i].aOff, leaves[i].bOff, leaves[i].totalSizeOut)
               for i in range(n)]


def compute_gemm(y, a, b, threads=1, y_shape=None, a_shape=None, b_shape=None, lib=None):
    """Compute::Gemm host branch on numpy arrays (y modified in place)."""
    ys = list(y.shape if y_shape is None else y_shape)
    as_ = list(a.shape if a_shape is None else a_shape)
    bs = list(b.shape if b_shape is None else b_shape)
    if lib == "ref":
        ref().ref_compute_gemm(_f(y), _ints(ys), len(ys), _f(a), _ints(as_), len(as_), _f(b),
                               _ints(bs), len(bs))
    else:
        rc = oracle().orc_compute_gemm(_f(y), _ints(ys), len(ys), _f(a), _ints(as_), len(as_),
                                       _f(b), _ints(bs), len(bs), threads)
        assert rc == 0
    return y


def relu(x):
    out = np.empty_like(x)
    oracle().orc_relu(_f(out), _f(x), x.size)
    return out


def transpose(x, rows, cols, batch, broadcast=False):
    out = np.zeros(batch * rows * cols, dtype=np.float32)
    oracle().orc_transpose(_f(out), _f(x), rows, cols, batch, 1 if broadcast else 0)
    return out


def scale(x, factor):
    out = np.empty_like(x)
    oracle().orc_scale(_f(out), _f(x), factor, x.size)
    return out


def sub_leaf(a, b, count, input_stride=0, broadcast_a=False, broadcast_b=False):
    out = np.empty(count, dtype=np.float32)
    oracle().orc_sub(count, _f(out), _f(a), _f(b), input_stride, int(broadcast_a),
                     int(broadcast_b))
    return out


def relu_backward(dx, dy, x):
    out = np.ascontiguousarray(dx.copy())
    oracle().orc_relu_backward(_f(out), _f(dy), _f(x), x.size)
    return out


def matching_dim(shapes):
    arr = (OrcShape * max(len(shapes), 1))()
    for i, dims in enumerate(shapes):
        arr[i] = make_shape(dims)
    return oracle().orc_get_matching_dim(arr, len(shapes))


def compute_sub(y_shape, a, b, lib=None):
    """Compute::Sub host branch; returns y (zeros where the walk writes nothing)."""
    y = np.zeros(y_shape, dtype=np.float32)
    ys, as_, bs = list(y_shape), list(a.shape), list(b.shape)
    if lib == "ref":
        dim = max(len(ys), len(as_), len(bs))
        pad = lambda v: [1] * (dim - len(v)) + v
        leaf_dim = matching_dim([pad(ys), pad(as_), pad(bs)])
        ref().ref_compute_sub(_f(y), _ints(ys), len(ys), _f(a), _ints(as_), len(as_), _f(b),
                              _ints(bs), len(bs), leaf_dim)
    else:
        rc = oracle().orc_compute_sub(_f(y), _ints(ys), len(ys), _f(a), _ints(as_), len(as_),
                                      _f(b), _ints(bs), len(bs))
        assert rc == 0
    return y


def sgd(z, dz, lr):
    out = np.ascontiguousarray(z.copy())
    oracle().orc_sgd(_f(out), _f(dz), lr, z.size)
    return out


def linear_backward(dx, W, bias, dy, x, lr, threads=1):
    """Returns the updated (dx, W, bias)."""
    dx, W, bias = (np.ascontiguousarray(v.copy()) for v in (dx, W, bias))
    batch, fin = x.shape
    oracle().orc_linear_backward(_f(dx), _f(W), _f(bias), _f(dy), _f(x), batch, fin, W.shape[1],
                                 lr, threads)
    return dx, W, bias


def linear_forward(x, W, bias, threads=1):
    batch, fin = x.shape
    fout = W.shape[1]
    y = np.zeros((batch, fout), dtype=np.float32)
    oracle().orc_linear_forward(_f(y), _f(x), _f(W), _f(bias), batch, fin, fout, threads)
    return y


def spmm_csr(out, V, COL, ROW, M, N, B, threads=1):
    assert COL.dtype == np.uint32 and ROW.dtype == np.uint32
    oracle().orc_spmm_csr(_f(out), _f(V) if V.size else _f(np.zeros(1, np.float32)),
                          COL.ctypes.data_as(_up) if COL.size else
                          np.zeros(1, np.uint32).ctypes.data_as(_up),
                          ROW.ctypes.data_as(_up), M, N, _f(B), threads)
    return out


def csr_from_dense(dense, N=None):
    """(V, COL, ROW) of a 2-D float32 array; N < dense.shape[1] treats the rest as pitch padding."""
    M, ld = dense.shape
    N = ld if N is None else N
    ROW = np.zeros(M + 1, np.uint32)
    nnz = oracle().orc_csr_from_dense(None, None, ROW.ctypes.data_as(_up), _f(dense), M, N, ld)
    V = np.zeros(max(nnz, 1), np.float32)
    COL = np.zeros(max(nnz, 1), np.uint32)
    oracle().orc_csr_from_dense(_f(V), COL.ctypes.data_as(_up), ROW.ctypes.data_as(_up),
                                _f(dense), M, N, ld)
    return V[:nnz], COL[:nnz], ROW


def csr_to_dense(V, COL, ROW, M, N, ld=None, fill=0.0):
    ld = N if ld is None else ld
    out = np.full((M, ld), np.float32(fill), np.float32)
    Vp = V if V.size else np.zeros(1, np.float32)
    Cp = COL if COL.size else np.zeros(1, np.uint32)
    oracle().orc_csr_to_dense(_f(out), ld, _f(Vp), Cp.ctypes.data_as(_up),
                              ROW.ctypes.data_as(_up), M, N)
    return out


def _u32p(a):
    a = a if a.size else np.zeros(1, np.uint32)
    assert a.dtype == np.uint32 and a.flags["C_CONTIGUOUS"]
    return a.ctypes.data_as(_up)


def spgemm_csr(A, B, M, K, N):
    """(V, COL, ROW) of A * B for CSR triples A = (V, COL, ROW), B likewise."""
    VA, CA, RA = A
    VB, CB, RB = B
    fa = VA if VA.size else np.zeros(1, np.float32)
    fb = VB if VB.size else np.zeros(1, np.float32)
    ROW = np.zeros(M + 1, np.uint32)
    nnz = oracle().orc_spgemm_csr(None, None, _u32p(ROW), _f(fa), _u32p(CA), _u32p(RA), _f(fb),
                                  _u32p(CB), _u32p(RB), M, K, N)
    V = np.zeros(max(nnz, 1), np.float32)
    COL = np.zeros(max(nnz, 1), np.uint32)
    oracle().orc_spgemm_csr(_f(V), _u32p(COL), _u32p(ROW), _f(fa), _u32p(CA), _u32p(RA), _f(fb),
                            _u32p(CB), _u32p(RB), M, K, N)
    return V[:nnz], COL[:nnz], ROW
