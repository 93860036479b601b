"""ctypes binding of the CPU oracle (oracle/libtfo_oracle.so) over numpy arrays.

TEST INFRASTRUCTURE ONLY: imported by tests/, by ``__graft_entry__.smoke`` and by the
``cpu_baseline`` leg of bench.py as the checker / CPU baseline -- never by the shipped package.
"""
import ctypes as C
import os
import subprocess

import numpy as np

MAX_RANK = 16
F32, F64, C64, C128 = 0, 1, 2, 3
SUM, MAX, MIN = 0, 1, 2
_HERE = os.path.dirname(os.path.abspath(__file__))
_LIB = os.path.join(_HERE, "libtfo_oracle.so")

DTYPES = {np.dtype(np.float32): F32, np.dtype(np.float64): F64,
          np.dtype(np.complex64): C64, np.dtype(np.complex128): C128}


class View(C.Structure):
    _fields_ = [("base", C.c_void_p), ("rank", C.c_int32), ("reserved", C.c_int32), ("offset", C.c_int64),
                ("dims", C.c_int64 * MAX_RANK), ("strides", C.c_int64 * MAX_RANK)]


def build():
    """Compile the oracle with its Makefile (g++, OpenMP)."""
    subprocess.check_call(["make", "-s", "-C", _HERE])


_lib = None


def lib():
    global _lib
    if _lib is None:
        if not os.path.exists(_LIB):
            build()
        _lib = C.CDLL(_LIB)
        _lib.tfo_last_message.restype = C.c_char_p
    return _lib


class OracleError(RuntimeError):
    def __init__(self, code, msg):
        super().__init__(f"oracle error {code}: {msg}")
        self.code = code


def _check(rc):
    if rc != 0:
        raise OracleError(rc, lib().tfo_last_message().decode())


def view_of(arr):
    """Strided view of a numpy array (element strides, offset 0 at arr's first element)."""
    v = View()
    v.base = arr.ctypes.data
    v.rank = arr.ndim
    v.offset = 0
    isz = arr.dtype.itemsize
    for d in range(arr.ndim):
        v.dims[d] = arr.shape[d]
        assert arr.strides[d] % isz == 0
        v.strides[d] = arr.strides[d] // isz
    return v


def _scalar(dt, x):
    x = complex(x)
    if dt in (F32, C64):
        return (C.c_float * 2)(x.real, x.imag)
    return (C.c_double * 2)(x.real, x.imag)


def _modes(m):
    m = list(m)
    return (C.c_uint32 * max(len(m), 1))(*m)


def _dt(arr):
    return DTYPES[arr.dtype]


def set_num_threads(n):
    lib().tfo_set_num_threads(int(n))


def num_threads():
    return lib().tfo_num_threads()


def permute(a, modes_a, b, modes_b, alpha=1.0, beta=0.0):
    dt = _dt(a)
    va, vb = view_of(a), view_of(b)
    _check(lib().tfo_permute(dt, _scalar(dt, alpha), C.byref(va), _modes(modes_a), _scalar(dt, beta),
                             C.byref(vb), _modes(modes_b)))


def reduce(a, modes_a, c, modes_c, op=SUM, alpha=1.0, beta=0.0):
    dt = _dt(a)
    va, vc = view_of(a), view_of(c)
    _check(lib().tfo_reduce(dt, _scalar(dt, alpha), C.byref(va), _modes(modes_a), _scalar(dt, beta),
                            C.byref(vc), _modes(modes_c), int(op)))


def contract(a, modes_a, b, modes_b, c, modes_c, alpha=1.0, beta=0.0, naive=False):
    dt = _dt(a)
    va, vb, vc = view_of(a), view_of(b), view_of(c)
    fn = lib().tfo_contract_naive if naive else lib().tfo_contract
    _check(fn(dt, _scalar(dt, alpha), C.byref(va), _modes(modes_a), C.byref(vb), _modes(modes_b),
              _scalar(dt, beta), C.byref(vc), _modes(modes_c)))


def batched_gemm(a, b, c, n_batch, alpha=1.0, beta=0.0):
    dt = _dt(a)
    va, vb, vc = view_of(a), view_of(b), view_of(c)
    _check(lib().tfo_batched_gemm(dt, int(n_batch), _scalar(dt, alpha), C.byref(va), C.byref(vb),
                                  _scalar(dt, beta), C.byref(vc)))


def elementwise_mul(a, b, c, alpha=1.0, beta=0.0):
    dt = _dt(a)
    va, vb, vc = view_of(a), view_of(b), view_of(c)
    _check(lib().tfo_elementwise_mul(dt, _scalar(dt, alpha), C.byref(va), C.byref(vb), _scalar(dt, beta),
                                     C.byref(vc)))


def conj(a, out):
    dt = _dt(a)
    va, vo = view_of(a), view_of(out)
    _check(lib().tfo_conj(dt, C.byref(va), C.byref(vo)))


def _paired(fn, a, modes_a, c, modes_c, pairs, alpha, beta):
    dt = _dt(a)
    va, vc = view_of(a), view_of(c)
    flat = [x for p in pairs for x in p]
    _check(fn(dt, _scalar(dt, alpha), C.byref(va), _modes(modes_a), _scalar(dt, beta), C.byref(vc),
              _modes(modes_c), _modes(flat), len(pairs)))


def trace(a, modes_a, c, modes_c, pairs, alpha=1.0, beta=0.0):
    _paired(lib().tfo_trace, a, modes_a, c, modes_c, pairs, alpha, beta)


def anti_trace(a, modes_a, c, modes_c, pairs, alpha=1.0, beta=0.0):
    _paired(lib().tfo_anti_trace, a, modes_a, c, modes_c, pairs, alpha, beta)


def anti_diag(a, modes_a, c, modes_c, pairs, alpha=1.0, beta=0.0):
    _paired(lib().tfo_anti_diag, a, modes_a, c, modes_c, pairs, alpha, beta)


def _einsum_args(operands, in_labels, out_labels):
    views = (View * len(operands))(*[view_of(o) for o in operands])
    flat = [l for ls in in_labels for l in ls]
    ranks = (C.c_int32 * len(operands))(*[len(ls) for ls in in_labels])
    return views, _modes(flat), ranks, _modes(out_labels)


def einsum_naive(operands, in_labels, out, out_labels, alpha=1.0, beta=0.0):
    dt = _dt(out)
    views, flat, ranks, ol = _einsum_args(operands, in_labels, out_labels)
    vo = view_of(out)
    _check(lib().tfo_einsum_naive(dt, len(operands), views, flat, ranks, ol, len(out_labels),
                                  _scalar(dt, alpha), _scalar(dt, beta), C.byref(vo)))


def einsum_pairs(operands, in_labels, out, out_labels, pairs, alpha=1.0, beta=0.0):
    dt = _dt(out)
    views, flat, ranks, ol = _einsum_args(operands, in_labels, out_labels)
    vo = view_of(out)
    fp = [x for p in pairs for x in p]
    _check(lib().tfo_einsum_pairs(dt, len(operands), views, flat, ranks, ol, len(out_labels),
                                  (C.c_int32 * max(len(fp), 1))(*fp), len(pairs),
                                  _scalar(dt, alpha), _scalar(dt, beta), C.byref(vo)))
