"""ctypes binding of the C ABI declared in include/sapphire_hip.h.

This is plumbing for the Python tests and the bench: it loads
sapphire_amd/libsapphire_hip.so, declares every entry point, turns non-zero
status codes into exceptions and moves numpy arrays to and from device
memory.  There is no other implementation behind it: if the library has not
been built the import of `lib()` raises.
"""
import ctypes
import os
import re

import numpy as np

_PKG = os.path.dirname(os.path.abspath(__file__))
LIB_PATH = os.path.join(_PKG, "libsapphire_hip.so")
HEADER_PATH = os.path.join(os.path.dirname(_PKG), "include", "sapphire_hip.h")

SPH_GEMM_ACCUMULATE = 0
SPH_GEMM_OVERWRITE = 1
SPH_GEMM_TRANS_A = 2
SPH_GEMM_TRANS_B = 4
SPH_LINEAR_RELU = 1
SPH_GROUPED_OFFSETS_MULTIPLE_OF_4 = 1


class SphError(RuntimeError):
    def __init__(self, status, text):
        super().__init__("status %d: %s" % (status, text))
        self.status = status


class SphDeviceInfo(ctypes.Structure):
    _fields_ = [
        ("name", ctypes.c_char * 128),
        ("arch", ctypes.c_char * 32),
        ("computeUnits", ctypes.c_int),
        ("clockMHz", ctypes.c_int),
        ("memoryClockMHz", ctypes.c_int),
        ("memoryBusWidthBits", ctypes.c_int),
        ("ldsBytesPerBlock", ctypes.c_int),
        ("l2Bytes", ctypes.c_int),
        ("totalMemoryBytes", ctypes.c_uint64),
        ("wavefrontSize", ctypes.c_int),
    ]


class SphGemmEntry(ctypes.Structure):
    _fields_ = [("outOff", ctypes.c_uint64), ("aOff", ctypes.c_uint64), ("bOff", ctypes.c_uint64)]


_vp = ctypes.c_void_p
_u32 = ctypes.c_uint32
_i64 = ctypes.c_int64
_sz = ctypes.c_size_t

# name -> argument types; every entry returns int except sph_last_error
SIGNATURES = {
    "sph_device_count": [ctypes.POINTER(ctypes.c_int)],
    "sph_set_device": [ctypes.c_int],
    "sph_get_device": [ctypes.POINTER(ctypes.c_int)],
    "sph_device_info": [ctypes.c_int, ctypes.POINTER(SphDeviceInfo)],
    "sph_malloc": [ctypes.POINTER(_vp), _sz],
    "sph_free": [_vp],
    "sph_malloc_async": [ctypes.POINTER(_vp), _sz],
    "sph_free_async": [_vp],
    "sph_mem_pool_trim": [],
    "sph_allocation_count": [ctypes.POINTER(ctypes.c_uint64)],
    "sph_memcpy_h2d": [_vp, _vp, _sz],
    "sph_memcpy_d2h": [_vp, _vp, _sz],
    "sph_memcpy_d2d": [_vp, _vp, _sz],
    "sph_memcpy_d2d_async": [_vp, _vp, _sz],
    "sph_host_malloc": [ctypes.POINTER(_vp), _sz],
    "sph_host_free": [_vp],
    "sph_stream_sync": [],
    "sph_device_sync": [],
    "sph_stream_wait_stream": [_vp],
    "sph_get_stream": [ctypes.POINTER(_vp)],
    "sph_set_stream": [_vp],
    "sph_event_create": [ctypes.POINTER(_vp)],
    "sph_event_record": [_vp],
    "sph_event_elapsed_ms": [_vp, _vp, ctypes.POINTER(ctypes.c_float)],
    "sph_event_destroy": [_vp],
    "sph_graph_begin_capture": [],
    "sph_graph_end_capture": [ctypes.POINTER(_vp)],
    "sph_graph_launch": [_vp],
    "sph_graph_destroy": [_vp],
    "sph_fill_f32": [_vp, ctypes.c_float, _sz],
    "sph_relu_f32": [_vp, _vp, _sz],
    "sph_transpose_f32": [_vp, _vp, _u32, _u32, _u32, ctypes.c_int],
    "sph_convert_f32_to_f16": [_vp, _vp, _sz],
    "sph_scale_f32": [_vp, _vp, ctypes.c_float, _sz],
    "sph_sub_f32": [_vp, _vp, _vp, _sz, _sz, ctypes.c_int, ctypes.c_int],
    "sph_relu_backward_f32": [_vp, _vp, _vp, _sz],
    "sph_sgd_step_f32": [_vp, _vp, ctypes.c_float, _sz],
    "sph_gemm_f32": [_vp, _vp, _vp, _u32, _u32, _u32, _u32, _i64, _i64, _i64],
    "sph_gemm_f32_ex": [_vp, _vp, _vp, _u32, _u32, _u32, _u32, _i64, _i64, _i64, _u32],
    "sph_gemm_f32_sgd": [_vp, _vp, _vp, _u32, _u32, _u32, ctypes.c_float, ctypes.c_float, _u32],
    "sph_linear_forward_f32": [_vp, _vp, _vp, _vp, _u32, _u32, _u32, _u32],
    "sph_gemm_f32_grouped": [ctypes.POINTER(SphGemmEntry), _u32, _vp, _vp, _vp, _u32, _u32, _u32],
    "sph_gemm_f32_grouped_device": [_vp, _u32, _vp, _vp, _vp, _u32, _u32, _u32, _u32],
    "sph_gemm_f16f32": [_vp, _vp, _vp, _u32, _u32, _u32, _u32, _i64, _i64, _i64, _u32],
    "sph_csr_row_offsets_f32": [_vp, _vp, _u32, _u32, _u32, ctypes.POINTER(ctypes.c_uint32)],
    "sph_csr_row_offsets_noalloc_f32": [_vp, _vp, _u32, _u32, _u32],
    "sph_csr_fill_f32": [_vp, _vp, _vp, _vp, _u32, _u32, _u32],
    "sph_csr_to_dense_f32": [_vp, _u32, _vp, _vp, _vp, _u32, _u32],
    "sph_csr_from_dense_f32": [_vp, _vp, _vp, _u32, _vp, _u32, _u32, _u32,
                               ctypes.POINTER(ctypes.c_uint32)],
    "sph_csr_validate_u32": [_vp, _vp, _u32, _u32, _u32, ctypes.POINTER(ctypes.c_uint32)],
    "sph_spgemm_row_offsets_f32": [_vp, _vp, _vp, _vp, _vp, _vp, _vp, _u32, _u32, _u32,
                                   ctypes.POINTER(ctypes.c_uint32)],
    "sph_spgemm_fill_f32": [_vp, _vp, _vp, _vp, _vp, _vp, _vp, _vp, _vp, _u32, _u32, _u32],
    "sph_spgemm_load_u32": [_vp, _vp, _vp, _u32, _u32, ctypes.POINTER(ctypes.c_uint64)],
    "sph_spgemm_f32": [_vp, _vp, _vp, _u32, _vp, _vp, _vp, _vp, _vp, _vp, _u32, _u32, _u32,
                       ctypes.POINTER(ctypes.c_uint32)],
    "sph_spmm_csr_f32": [_vp, _vp, _vp, _vp, _u32, _u32, _u32, _vp, ctypes.c_int],
    "sph_spmm_csr_bias_f32": [_vp, _vp, _vp, _vp, _u32, _u32, _u32, _vp, _vp],
}


def declared_symbols():
    """Names of the functions include/sapphire_hip.h declares."""
    text = open(HEADER_PATH).read()
    text = re.sub(r"/\*.*?\*/", "", text, flags=re.S)
    return sorted(set(re.findall(r"\b(sph_[a-z0-9_]+)\s*\(", text)))


_lib = None


def lib():
    """The loaded C ABI library; raises if it has not been built."""
    global _lib
    if _lib is None:
        if not os.path.exists(LIB_PATH):
            raise RuntimeError(
                "%s is missing: build it with `python -m sapphire_amd.build hip` "
                "(there is no fallback implementation)" % LIB_PATH)
        handle = ctypes.CDLL(LIB_PATH)
        handle.sph_last_error.restype = ctypes.c_char_p
        handle.sph_last_error.argtypes = []
        for name, argtypes in SIGNATURES.items():
            fn = getattr(handle, name)
            fn.restype = ctypes.c_int
            fn.argtypes = argtypes
        _lib = handle
    return _lib


def check(status):
    if status != 0:
        raise SphError(status, lib().sph_last_error().decode("utf-8", "replace"))


def call(name, *args):
    check(getattr(lib(), name)(*args))


class DeviceBuffer:
    """A hipMalloc'ed block owned by Python (freed on release()/garbage collection)."""

    def __init__(self, nbytes):
        self.nbytes = int(nbytes)
        ptr = _vp()
        call("sph_malloc", ctypes.byref(ptr), max(self.nbytes, 1))
        self.ptr = ptr.value

    @classmethod
    def from_array(cls, array):
        array = np.ascontiguousarray(array)
        buf = cls(array.nbytes)
        buf.upload(array)
        return buf

    def upload(self, array):
        array = np.ascontiguousarray(array)
        assert array.nbytes <= self.nbytes
        call("sph_memcpy_h2d", self.ptr, array.ctypes.data, array.nbytes)

    def download(self, dtype, shape):
        out = np.empty(shape, dtype=dtype)
        assert out.nbytes <= self.nbytes
        call("sph_memcpy_d2h", out.ctypes.data, self.ptr, out.nbytes)
        return out

    def at(self, byte_offset):
        return self.ptr + int(byte_offset)

    def release(self):
        if self.ptr:
            call("sph_free", self.ptr)
            self.ptr = 0

    def __del__(self):
        try:
            self.release()
        except Exception:
            pass


def require_gemm_extents(d_out, d_a, d_b, M, N, K, batch, stride_out, stride_a, stride_b,
                         operand_bytes=4):
    """Raises unless the three device buffers hold what a strided-batched product of this shape
    reads and writes.  The C ABI takes raw pointers and trusts the extents; a caller that owns
    DeviceBuffers checks them here before every such call, because an operand that is smaller
    than its stated shape is a device memory fault, not an error code."""
    last = max(int(batch), 1) - 1
    need = (("out", d_out, (last * stride_out + M * N) * 4),
            ("A", d_a, (last * stride_a + M * K) * operand_bytes),
            ("B", d_b, (last * stride_b + K * N) * operand_bytes))
    for name, buf, nbytes in need:
        if buf.nbytes < nbytes:
            raise ValueError("%s holds %d bytes, the %dx%dx%d x%d product needs %d"
                             % (name, buf.nbytes, M, N, K, batch, nbytes))


def require_csr_extents(d_out, d_v, d_col, d_row, d_b, M, Kdim, N, nnz):
    """The same for a CSR x dense product: V and COL of nnz entries, ROW of M + 1, B Kdim x N,
    out M x N."""
    need = (("out", d_out, M * N * 4), ("V", d_v, nnz * 4), ("COL", d_col, nnz * 4),
            ("ROW", d_row, (M + 1) * 4), ("B", d_b, Kdim * N * 4))
    for name, buf, nbytes in need:
        if buf.nbytes < nbytes:
            raise ValueError("%s holds %d bytes, the %dx%d CSR x %dx%d product needs %d"
                             % (name, buf.nbytes, M, Kdim, Kdim, N, nbytes))


def validate_csr(d_col, d_row, M, Kdim, nnz):
    """sph_csr_validate_u32 on device arrays; raises SphError when the record is unsafe."""
    problems = ctypes.c_uint32(0)
    call("sph_csr_validate_u32", d_col.ptr, d_row.ptr, M, Kdim, nnz, ctypes.byref(problems))
    return problems.value


def device_count():
    n = ctypes.c_int(0)
    status = lib().sph_device_count(ctypes.byref(n))
    return n.value if status == 0 else 0


def device_info(device=0):
    info = SphDeviceInfo()
    call("sph_device_info", device, ctypes.byref(info))
    return info


def sync():
    call("sph_stream_sync")


class Event:
    def __init__(self):
        ev = _vp()
        call("sph_event_create", ctypes.byref(ev))
        self.ptr = ev.value

    def record(self):
        call("sph_event_record", self.ptr)

    def elapsed_ms_since(self, start):
        ms = ctypes.c_float(0)
        call("sph_event_elapsed_ms", start.ptr, self.ptr, ctypes.byref(ms))
        return ms.value

    def destroy(self):
        if self.ptr:
            call("sph_event_destroy", self.ptr)
            self.ptr = 0


class Graph:
    """Records the calls made inside the `with` block; launch() replays them."""

    def __init__(self):
        self.ptr = None

    def __enter__(self):
        call("sph_graph_begin_capture")
        return self

    def __exit__(self, exc_type, exc, tb):
        handle = _vp()
        status = lib().sph_graph_end_capture(ctypes.byref(handle))
        if exc_type is None:
            check(status)
            self.ptr = handle.value
        elif status == 0 and handle.value:
            lib().sph_graph_destroy(handle.value)   # the block failed: drop what was recorded
        return False

    def launch(self):
        call("sph_graph_launch", self.ptr)

    def destroy(self):
        if self.ptr:
            call("sph_graph_destroy", self.ptr)
            self.ptr = None


def make_entries(triples):
    arr = (SphGemmEntry * len(triples))()
    for i, (o, a, b) in enumerate(triples):
        arr[i].outOff, arr[i].aOff, arr[i].bOff = int(o), int(a), int(b)
    return arr
