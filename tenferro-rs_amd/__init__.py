"""Host-side mirror of the tenferro interfaces this backend sits behind, over the C ABI of
libtenferro_hip.so (include/tenferro_hip.h).

Names, argument meaning and error behaviour follow the reference:
  HipBackend.plan / execute / has_extension_for   tenferro-prims/src/lib.rs:278-340 (TensorPrims<Standard>)
  PrimDescriptor, ReduceOp, Extension             tenferro-prims/src/lib.rs:100-245
  Subscripts, ContractionTree, einsum*            tenferro-einsum/src/lib.rs:239-621
  Tensor, MemoryOrder, CompletionEvent            tenferro-tensor/src/lib.rs:122-713
  LogicalMemorySpace, ComputeDevice, OpKind, Error  tenferro-device/src/lib.rs:30-162

PyTorch is used only to own device memory and to name the current HIP stream; every computation is
a call into the C ABI.  There is no CPU fallback: without the built library or without a HIP device
the calls raise.
"""
import ctypes as C
import os

import numpy as np

_HERE = os.path.dirname(os.path.abspath(__file__))
LIB_PATH = os.path.join(_HERE, "libtenferro_hip.so")
MAX_RANK = 16

F32, F64, C64, C128 = 0, 1, 2, 3
_NP_DTYPES = {np.dtype(np.float32): F32, np.dtype(np.float64): F64, np.dtype(np.complex64): C64, np.dtype(np.complex128): C128}
_DT_NP = {v: k for k, v in _NP_DTYPES.items()}


# ---------------------------------------------------------------------------------------------- C structs
class tfh_view(C.Structure):
    _fields_ = [("base", C.c_void_p), ("rank", C.c_int32), ("flags", C.c_int32), ("offset", C.c_int64),
                ("dims", C.c_int64 * MAX_RANK), ("strides", C.c_int64 * MAX_RANK)]


class tfh_desc(C.Structure):
    _fields_ = [("op", C.c_int32), ("reduce_op", C.c_int32),
                ("batch_dims", C.POINTER(C.c_int64)), ("n_batch_dims", C.c_int32), ("reserved", C.c_int32),
                ("m", C.c_int64), ("n", C.c_int64), ("k", C.c_int64),
                ("modes_a", C.POINTER(C.c_uint32)), ("n_modes_a", C.c_int32),
                ("modes_b", C.POINTER(C.c_uint32)), ("n_modes_b", C.c_int32),
                ("modes_c", C.POINTER(C.c_uint32)), ("n_modes_c", C.c_int32),
                ("paired", C.POINTER(C.c_uint32)), ("n_pairs", C.c_int32)]


class tfh_error_info(C.Structure):
    _fields_ = [("status", C.c_int32), ("n_expected", C.c_int32), ("n_got", C.c_int32), ("reserved", C.c_int32),
                ("expected", C.c_int64 * MAX_RANK), ("got", C.c_int64 * MAX_RANK), ("message", C.c_char * 512)]


class tfh_compute_device(C.Structure):
    _fields_ = [("kind", C.c_int32), ("device_id", C.c_int32)]


_lib = None


def lib():
    """The loaded C-ABI library.  Raises if it has not been built (python tenferro-rs_amd/build.py)."""
    global _lib
    if _lib is None:
        if not os.path.exists(LIB_PATH):
            raise RuntimeError(f"{LIB_PATH} is missing: build it with `python tenferro-rs_amd/build.py`")
        # GpuMemory tensors of this module live in torch CUDA tensors, so torch's HIP runtime must be the one in the
        # process: loaded after the system runtime that the library would otherwise pull in, torch finds no device.
        import torch  # noqa: F401
        L = C.CDLL(LIB_PATH)
        L.tfh_status_name.restype = C.c_char_p
        L.tfh_version.restype = C.c_char_p
        L.tfh_dtype_size.restype = C.c_size_t
        L.tfh_tree_mac_count.restype = C.c_double
        L.tfh_tree_peak_intermediate.restype = C.c_double
        L.tfh_plan_destroy.restype = None
        L.tfh_tree_destroy.restype = None
        L.tfh_subscripts_destroy.restype = None
        L.tfh_last_error.restype = None
        for name in ("tfh_plan_destroy", "tfh_tree_destroy", "tfh_subscripts_destroy", "tfh_free", "tfh_stream_destroy",
                     "tfh_stream_synchronize", "tfh_event_destroy", "tfh_event_synchronize"):
            getattr(L, name).argtypes = [C.c_void_p]
        L.tfh_execute.argtypes = [C.c_void_p, C.c_void_p, C.c_void_p, C.c_int32, C.c_void_p, C.c_void_p, C.c_void_p]
        L.tfh_execute_grouped.argtypes = [C.c_void_p, C.c_void_p, C.c_void_p, C.c_int32, C.c_void_p, C.c_void_p, C.c_void_p]
        L.tfh_execute_static.argtypes = L.tfh_execute.argtypes
        L.tfh_plan_cache_stats.argtypes = [C.c_void_p, C.c_void_p, C.c_void_p, C.c_void_p]
        L.tfh_static_scratch_bytes.restype = C.c_size_t
        L.tfh_static_scratch_bytes.argtypes = []
        L.tfh_einsum_execute.argtypes = [C.c_int32, C.c_void_p, C.c_void_p, C.c_int32, C.c_void_p, C.c_void_p, C.c_void_p,
                                         C.c_uint64, C.c_void_p]
        L.tfh_conj.argtypes = [C.c_int32, C.c_void_p, C.c_void_p, C.c_void_p]
        L.tfh_fill.argtypes = [C.c_int32, C.c_void_p, C.c_void_p, C.c_void_p]
        L.tfh_memcpy_h2d.argtypes = L.tfh_memcpy_d2h.argtypes = L.tfh_memcpy_d2d.argtypes = [C.c_void_p, C.c_void_p, C.c_size_t, C.c_void_p]
        L.tfh_host_malloc.argtypes = [C.c_size_t, C.POINTER(C.c_void_p)]
        L.tfh_host_free.argtypes = [C.c_void_p]
        L.tfh_malloc.argtypes = [C.c_size_t, C.POINTER(C.c_void_p)]
        L.tfh_event_record.argtypes = [C.c_void_p, C.c_void_p]
        L.tfh_stream_wait_event.argtypes = [C.c_void_p, C.c_void_p]
        L.tfh_event_query.argtypes = [C.c_void_p, C.POINTER(C.c_int32)]
        L.tfh_tree_step.argtypes = [C.c_void_p, C.c_int32, C.POINTER(C.c_int32), C.POINTER(C.c_int32)]
        L.tfh_tree_node.argtypes = [C.c_void_p, C.c_int32, C.c_void_p, C.c_void_p, C.c_int32]
        L.tfh_tree_output_dims.argtypes = [C.c_void_p, C.c_void_p, C.c_int32]
        for name in ("tfh_tree_n_inputs", "tfh_tree_n_steps", "tfh_tree_output_rank", "tfh_tree_mac_count",
                     "tfh_tree_peak_intermediate", "tfh_subscripts_n_inputs"):
            getattr(L, name).argtypes = [C.c_void_p]
        L.tfh_subscripts_input_rank.argtypes = [C.c_void_p, C.c_int32]
        L.tfh_tree_optimize.argtypes = [C.c_void_p, C.c_void_p, C.c_void_p, C.c_int32, C.c_void_p]
        L.tfh_tree_optimize_cached.argtypes = [C.c_void_p, C.c_void_p, C.c_void_p, C.c_int32, C.c_void_p]
        L.tfh_tree_cache_stats.argtypes = [C.POINTER(C.c_int64), C.POINTER(C.c_int64), C.POINTER(C.c_int64)]
        L.tfh_tree_from_pairs.argtypes = [C.c_void_p, C.c_void_p, C.c_void_p, C.c_int32, C.c_void_p, C.c_int32, C.c_void_p]
        L.tfh_plan_create.argtypes = [C.c_int32, C.c_void_p, C.c_void_p, C.c_void_p, C.c_int32, C.c_void_p]
        L.tfh_plan_create_grouped.argtypes = [C.c_int32, C.c_void_p, C.c_int32, C.c_void_p, C.c_void_p, C.c_int32, C.c_void_p]
        L.tfh_subscripts_new.argtypes = [C.c_void_p, C.c_void_p, C.c_int32, C.c_void_p, C.c_int32, C.c_void_p]
        L.tfh_subscripts_parse.argtypes = [C.c_char_p, C.c_void_p]
        L.tfh_last_error.argtypes = [C.c_void_p]
        L.tfh_event_create.argtypes = [C.c_void_p]
        L.tfh_stream_create.argtypes = [C.c_void_p]
        L.tfh_compute_device_format.argtypes = [C.c_int32, C.c_int64, C.c_char_p, C.c_size_t]
        L.tfh_preferred_compute_devices.argtypes = [C.c_int32, C.c_int64, C.c_int32, C.c_void_p, C.c_int32, C.c_void_p]
        L.tfh_has_extension.argtypes = [C.c_int32, C.c_int32]
        L.tfh_profile_enable.argtypes = [C.c_int32]
        L.tfh_profile_collect.argtypes = [C.c_int32, C.POINTER(C.c_double), C.POINTER(C.c_int32)]
        L.tfh_profile_kernel.argtypes = [C.c_int32, C.c_int32, C.c_char_p, C.c_size_t, C.POINTER(C.c_double), C.POINTER(C.c_int32)]
        L.tfh_last_kernel.restype = C.c_char_p
        L.tfh_last_kernel.argtypes = []
        L.tfh_subscripts_labels.argtypes = [C.c_void_p, C.c_int32, C.c_void_p, C.c_int32]
        L.tfh_subscripts_nesting.argtypes = [C.c_void_p, C.c_char_p, C.c_size_t]
        L.tfh_plan_describe.argtypes = [C.c_void_p, C.c_char_p, C.c_size_t]
        _lib = L
    return _lib


# ---------------------------------------------------------------------------------------------- errors
class Error(Exception):
    """tenferro_device::Error (tenferro-device/src/lib.rs:108-159)."""
    status = -1

    def __init__(self, message, expected=None, got=None):
        super().__init__(message)
        self.message = message
        self.expected = expected
        self.got = got


class ShapeMismatch(Error):
    status = 1


class RankMismatch(Error):
    status = 2


class DeviceError(Error):
    status = 3


class NoCompatibleComputeDevice(Error):
    """Fields `space` (LogicalMemorySpace) and `op` (an OpKind value), as in tenferro-device/src/lib.rs:134-140."""
    status = 4
    space = None
    op = None


class CrossMemorySpaceOperation(Error):
    status = 5


class InvalidArgument(Error):
    status = 6


class Strided(Error):
    status = 7


_ERRORS = {c.status: c for c in (ShapeMismatch, RankMismatch, DeviceError, NoCompatibleComputeDevice,
                                 CrossMemorySpaceOperation, InvalidArgument, Strided)}


def _check(status):
    if status == 0:
        return
    info = tfh_error_info()
    lib().tfh_last_error(C.byref(info))
    cls = _ERRORS.get(status, Error)
    expected = list(info.expected[:info.n_expected]) if info.n_expected else None
    got = list(info.got[:info.n_got]) if info.n_got else None
    if cls is RankMismatch and expected:
        expected, got = expected[0], got[0]
    err = cls(info.message.decode(errors="replace"), expected, got)
    if cls is NoCompatibleComputeDevice and expected and len(expected) == 2 and got:
        err.space, err.op = LogicalMemorySpace(int(expected[0]), int(expected[1])), int(got[0])
    raise err


# ---------------------------------------------------------------------------------------------- device model
class LogicalMemorySpace:
    """tenferro-device/src/lib.rs:30-38."""

    def __init__(self, kind, space_id=0):
        self.kind, self.space_id = kind, space_id

    def __eq__(self, o):
        return isinstance(o, LogicalMemorySpace) and (self.kind, self.space_id) == (o.kind, o.space_id)

    def __hash__(self):
        return hash((self.kind, self.space_id))

    def __repr__(self):
        return "MainMemory" if self.kind == 0 else f"GpuMemory {{ space_id: {self.space_id} }}"


MainMemory = LogicalMemorySpace(0)


def GpuMemory(space_id=0):
    return LogicalMemorySpace(1, space_id)


class ComputeDevice:
    """tenferro-device/src/lib.rs:46-72; str() gives "cpu:0" / "cuda:1" / "hip:0"."""
    CPU, CUDA, HIP = 0, 1, 2

    def __init__(self, kind, device_id=0):
        self.kind, self.device_id = kind, device_id

    @classmethod
    def Cpu(cls, device_id=0):
        return cls(cls.CPU, device_id)

    @classmethod
    def Cuda(cls, device_id=0):
        return cls(cls.CUDA, device_id)

    @classmethod
    def Hip(cls, device_id=0):
        return cls(cls.HIP, device_id)

    def __eq__(self, o):
        return isinstance(o, ComputeDevice) and (self.kind, self.device_id) == (o.kind, o.device_id)

    def __hash__(self):
        return hash((self.kind, self.device_id))

    def __str__(self):
        buf = C.create_string_buffer(64)
        _check(lib().tfh_compute_device_format(self.kind, C.c_int64(self.device_id), buf, 64))
        return buf.value.decode()

    __repr__ = __str__


class OpKind:
    """tenferro-device/src/lib.rs:77-90."""
    Contract, BatchedGemm, Reduce, Trace, Permute, ElementwiseMul = range(6)


def preferred_compute_devices(space, op_kind):
    """tenferro-device/src/lib.rs:92-105."""
    out = (tfh_compute_device * 8)()
    n = C.c_int32(0)
    _check(lib().tfh_preferred_compute_devices(space.kind, C.c_int64(space.space_id), op_kind, out, 8, C.byref(n)))
    return [ComputeDevice(out[i].kind, out[i].device_id) for i in range(n.value)]


# ---------------------------------------------------------------------------------------------- prims
class ReduceOp:
    """tenferro-prims/src/lib.rs:100-107."""
    Sum, Max, Min = 0, 1, 2


class Extension:
    """tenferro-prims/src/lib.rs:123-128."""
    Contract, ElementwiseMul = 0, 1


class PrimDescriptor:
    """tenferro-prims/src/lib.rs:152-245.  Build with the variant constructors below."""
    BATCHED_GEMM, REDUCE, TRACE, PERMUTE, ANTI_TRACE, ANTI_DIAG, CONTRACT, ELEMENTWISE_MUL = range(8)

    def __init__(self, op, **kw):
        self.op = op
        self.batch_dims = list(kw.get("batch_dims", []))
        self.m, self.n, self.k = kw.get("m", 0), kw.get("n", 0), kw.get("k", 0)
        self.modes_a = list(kw.get("modes_a", []))
        self.modes_b = list(kw.get("modes_b", []))
        self.modes_c = list(kw.get("modes_c", []))
        self.paired = [tuple(p) for p in kw.get("paired", [])]
        self.reduce_op = kw.get("op_", ReduceOp.Sum)

    @classmethod
    def BatchedGemm(cls, batch_dims, m, n, k):
        return cls(cls.BATCHED_GEMM, batch_dims=batch_dims, m=m, n=n, k=k)

    @classmethod
    def Reduce(cls, modes_a, modes_c, op):
        return cls(cls.REDUCE, modes_a=modes_a, modes_c=modes_c, op_=op)

    @classmethod
    def Trace(cls, modes_a, modes_c, paired):
        return cls(cls.TRACE, modes_a=modes_a, modes_c=modes_c, paired=paired)

    @classmethod
    def Permute(cls, modes_a, modes_b):
        return cls(cls.PERMUTE, modes_a=modes_a, modes_c=modes_b)

    @classmethod
    def AntiTrace(cls, modes_a, modes_c, paired):
        return cls(cls.ANTI_TRACE, modes_a=modes_a, modes_c=modes_c, paired=paired)

    @classmethod
    def AntiDiag(cls, modes_a, modes_c, paired):
        return cls(cls.ANTI_DIAG, modes_a=modes_a, modes_c=modes_c, paired=paired)

    @classmethod
    def Contract(cls, modes_a, modes_b, modes_c):
        return cls(cls.CONTRACT, modes_a=modes_a, modes_b=modes_b, modes_c=modes_c)

    @classmethod
    def ElementwiseMul(cls):
        return cls(cls.ELEMENTWISE_MUL)

    def _c(self):
        keep = []

        def arr(ctype, vals):
            a = (ctype * max(len(vals), 1))(*vals)
            keep.append(a)
            return C.cast(a, C.POINTER(ctype))

        d = tfh_desc()
        d.op, d.reduce_op = self.op, self.reduce_op
        d.batch_dims, d.n_batch_dims = arr(C.c_int64, self.batch_dims), len(self.batch_dims)
        d.m, d.n, d.k = self.m, self.n, self.k
        d.modes_a, d.n_modes_a = arr(C.c_uint32, self.modes_a), len(self.modes_a)
        d.modes_b, d.n_modes_b = arr(C.c_uint32, self.modes_b), len(self.modes_b)
        d.modes_c, d.n_modes_c = arr(C.c_uint32, self.modes_c), len(self.modes_c)
        flat = [x for p in self.paired for x in p]
        d.paired, d.n_pairs = arr(C.c_uint32, flat), len(self.paired)
        return d, keep


def _shapes_c(shapes):
    keep = [(C.c_int64 * max(len(s), 1))(*[int(x) for x in s]) for s in shapes]
    ptrs = (C.POINTER(C.c_int64) * max(len(shapes), 1))(*[C.cast(k, C.POINTER(C.c_int64)) for k in keep])
    ranks = (C.c_int32 * max(len(shapes), 1))(*[len(s) for s in shapes])
    return ptrs, ranks, keep


def _scalar_c(dtype, x):
    x = complex(x)
    return (C.c_float * 2)(x.real, x.imag) if dtype in (F32, C64) else (C.c_double * 2)(x.real, x.imag)


def dtype_code(dtype):
    """tfh_dtype of a numpy/torch dtype or an int code."""
    if isinstance(dtype, int):
        return dtype
    try:
        return _NP_DTYPES[np.dtype(dtype)]
    except TypeError:
        import torch
        return {torch.float32: F32, torch.float64: F64, torch.complex64: C64, torch.complex128: C128}[dtype]


def current_stream():
    import torch
    return torch.cuda.current_stream().cuda_stream


def view_of(t):
    """tfh_view of a Tensor, a torch CUDA tensor, or an existing tfh_view."""
    if isinstance(t, tfh_view):
        return t
    if isinstance(t, Tensor):
        return t._view()
    v = tfh_view()
    if not t.is_cuda:
        raise CrossMemorySpaceOperation(f"cross-memory-space operation between {MainMemory!r} and {GpuMemory(0)!r}")
    v.base = t.data_ptr()
    v.rank = t.dim()
    v.offset = 0
    for d in range(t.dim()):
        v.dims[d] = t.shape[d]
        v.strides[d] = t.stride(d)
    return v


_in_flight = []     # (event, buffers): device buffers that kernels on a stream other than torch's current one may still use


def _enqueue_on(tensors, st):
    """Stream-side prologue of a call that enqueues on stream `st`: pending completion events of the tensors become
    stream dependencies (tenferro-einsum/src/lib.rs:146-177), never host waits."""
    for t in tensors:
        if isinstance(t, Tensor) and t.event is not None:
            _check(lib().tfh_stream_wait_event(st, t.event._h))


def _completed_on(outputs, st, used=()):
    """The outputs of a call enqueued on `st` carry an event recorded behind it (tenferro-tensor/src/lib.rs:301-309).
    When `st` is not the stream torch's allocator ordered the buffers on, the buffers of every tensor the call used are
    held until that event has completed: dropping a tensor right after the call must not hand its memory to other work
    while the kernels enqueued here still run.  (Holding references rather than telling the allocator about the stream:
    the allocator would touch the stream again when the buffer is freed, and the caller may have destroyed it by then.)"""
    import torch
    ev = CompletionEvent(st)
    for t in outputs:
        if isinstance(t, Tensor):
            t.event = ev
    if st and st != torch.cuda.current_stream().cuda_stream:
        _in_flight[:] = [(e, bufs) for e, bufs in _in_flight if not e.ready()]
        _in_flight.append((ev, [t._buf for t in list(used) + list(outputs) if isinstance(t, Tensor)]))


class HipPlan:
    """Plan<T> of the Hip backend (tenferro-prims/src/lib.rs:279-280)."""

    def __init__(self, handle, dtype, n_inputs, grouped=0):
        self._h, self.dtype, self.n_inputs, self.n_groups = handle, dtype, n_inputs, grouped

    def cache_stats(self):
        """(executes that found their routed launch in the plan, executes that had to route, routes kept)."""
        h, m, e = C.c_int64(), C.c_int64(), C.c_int32()
        _check(lib().tfh_plan_cache_stats(self._h, C.byref(h), C.byref(m), C.byref(e)))
        return h.value, m.value, e.value

    def describe(self):
        buf = C.create_string_buffer(256)
        _check(lib().tfh_plan_describe(self._h, buf, 256))
        return buf.value.decode()

    def __del__(self):
        if getattr(self, "_h", None) and _lib is not None:
            _lib.tfh_plan_destroy(self._h)
            self._h = None


class HipBackend:
    """impl TensorPrims<Standard> for the HIP device (tenferro-prims/src/lib.rs:278-340).
    Associated functions, no instance state (:259-262)."""

    @staticmethod
    def plan(dtype, desc, shapes):
        dt = dtype_code(dtype)
        d, keep = desc._c()
        ptrs, ranks, keep2 = _shapes_c(shapes)
        out = C.c_void_p()
        _check(lib().tfh_plan_create(dt, C.byref(d), ptrs, ranks, len(shapes), C.byref(out)))
        return HipPlan(out.value, dt, len(shapes) - 1)

    @staticmethod
    def execute(plan, alpha, inputs, beta, output, stream=None):
        views = (tfh_view * max(len(inputs), 1))(*[view_of(t) for t in inputs])
        vo = view_of(output)
        st = current_stream() if stream is None else stream
        _enqueue_on(list(inputs) + [output], st)
        _check(lib().tfh_execute(plan._h, _scalar_c(plan.dtype, alpha), views, len(inputs), _scalar_c(plan.dtype, beta),
                                 C.byref(vo), st))
        _completed_on([output], st, inputs)

    @staticmethod
    def execute_static(plan, alpha, inputs, beta, output, stream=None):
        """execute() without device allocations: the scratch of the call comes from the library's fixed array
        (tfh_execute_static; no counterpart in the reference).  Calls that overlap on one device race on that array."""
        views = (tfh_view * max(len(inputs), 1))(*[view_of(t) for t in inputs])
        vo = view_of(output)
        st = current_stream() if stream is None else stream
        _enqueue_on(list(inputs) + [output], st)
        _check(lib().tfh_execute_static(plan._h, _scalar_c(plan.dtype, alpha), views, len(inputs), _scalar_c(plan.dtype, beta),
                                        C.byref(vo), st))
        _completed_on([output], st, inputs)

    @staticmethod
    def has_extension_for(dtype, ext):
        try:
            dt = dtype_code(dtype)
        except (KeyError, TypeError):
            return False
        return bool(lib().tfh_has_extension(dt, ext))

    @staticmethod
    def plan_grouped(dtype, desc, group_shapes):
        """group_shapes: one [shape_a, shape_b, shape_c] per group."""
        dt = dtype_code(dtype)
        d, keep = desc._c()
        flat = [s for g in group_shapes for s in g]
        ptrs, ranks, keep2 = _shapes_c(flat)
        out = C.c_void_p()
        _check(lib().tfh_plan_create_grouped(dt, C.byref(d), len(group_shapes), ptrs, ranks, 3, C.byref(out)))
        return HipPlan(out.value, dt, 2, grouped=len(group_shapes))

    @staticmethod
    def execute_grouped(plan, alpha, inputs, beta, outputs, stream=None):
        """inputs: [(a, b), ...] per group; outputs: [c, ...]."""
        flat = [view_of(t) for pair in inputs for t in pair]
        views = (tfh_view * len(flat))(*flat)
        outs = (tfh_view * len(outputs))(*[view_of(t) for t in outputs])
        st = current_stream() if stream is None else stream
        _enqueue_on([t for pair in inputs for t in pair] + list(outputs), st)
        _check(lib().tfh_execute_grouped(plan._h, _scalar_c(plan.dtype, alpha), views, 2, _scalar_c(plan.dtype, beta), outs, st))
        _completed_on(outputs, st, [t for pair in inputs for t in pair])


# ---------------------------------------------------------------------------------------------- einsum front end
class Subscripts:
    """tenferro-einsum/src/lib.rs:239-284."""

    def __init__(self, handle):
        self._h = handle
        L = lib()
        n = L.tfh_subscripts_n_inputs(handle)
        buf = (C.c_uint32 * 64)()
        self.inputs = []
        for i in range(n):
            r = L.tfh_subscripts_labels(handle, i, buf, 64)
            self.inputs.append(list(buf[:r]))
        r = L.tfh_subscripts_labels(handle, -1, buf, 64)
        self.output = list(buf[:r])

    @classmethod
    def new(cls, inputs, output):
        flat = [int(l) for ls in inputs for l in ls]
        ranks = (C.c_int32 * max(len(inputs), 1))(*[len(ls) for ls in inputs])
        out = C.c_void_p()
        _check(lib().tfh_subscripts_new((C.c_uint32 * max(len(flat), 1))(*flat), ranks, len(inputs),
                                        (C.c_uint32 * max(len(output), 1))(*[int(l) for l in output]), len(output), C.byref(out)))
        return cls(out.value)

    @classmethod
    def parse(cls, notation):
        out = C.c_void_p()
        _check(lib().tfh_subscripts_parse(notation.encode(), C.byref(out)))
        return cls(out.value)

    def nesting(self):
        buf = C.create_string_buffer(1024)
        _check(lib().tfh_subscripts_nesting(self._h, buf, 1024))
        return buf.value.decode()

    def __del__(self):
        if getattr(self, "_h", None) and _lib is not None:
            _lib.tfh_subscripts_destroy(self._h)
            self._h = None


class ContractionTree:
    """tenferro-einsum/src/lib.rs:297-356."""

    def __init__(self, handle):
        self._h = handle

    @classmethod
    def optimize(cls, subscripts, shapes):
        ptrs, ranks, keep = _shapes_c(shapes)
        out = C.c_void_p()
        _check(lib().tfh_tree_optimize(subscripts._h, ptrs, ranks, len(shapes), C.byref(out)))
        return cls(out.value)

    @classmethod
    def optimize_cached(cls, subscripts, shapes):
        """The tree `optimize` returns, shared through the library's cache of optimised networks (no counterpart in the
        reference: the einsum functions that take no plan use it so that a repeated call does not search again)."""
        ptrs, ranks, keep = _shapes_c(shapes)
        out = C.c_void_p()
        _check(lib().tfh_tree_optimize_cached(subscripts._h, ptrs, ranks, len(shapes), C.byref(out)))
        return cls(out.value)

    @classmethod
    def from_pairs(cls, subscripts, shapes, pairs):
        ptrs, ranks, keep = _shapes_c(shapes)
        flat = [int(x) for p in pairs for x in p]
        out = C.c_void_p()
        _check(lib().tfh_tree_from_pairs(subscripts._h, ptrs, ranks, len(shapes), (C.c_int32 * max(len(flat), 1))(*flat),
                                         len(pairs), C.byref(out)))
        return cls(out.value)

    @property
    def n_inputs(self):
        return lib().tfh_tree_n_inputs(self._h)

    @property
    def steps(self):
        L = lib()
        res = []
        for i in range(L.tfh_tree_n_steps(self._h)):
            a, b = C.c_int32(), C.c_int32()
            _check(L.tfh_tree_step(self._h, i, C.byref(a), C.byref(b)))
            res.append((a.value, b.value))
        return res

    def node(self, i):
        labels, dims = (C.c_uint32 * MAX_RANK)(), (C.c_int64 * MAX_RANK)()
        r = lib().tfh_tree_node(self._h, i, labels, dims, MAX_RANK)
        if r < 0:
            raise InvalidArgument(f"invalid argument: node {i} out of range")
        return list(labels[:r]), list(dims[:r])

    @property
    def output_dims(self):
        dims = (C.c_int64 * MAX_RANK)()
        r = lib().tfh_tree_output_dims(self._h, dims, MAX_RANK)
        return list(dims[:r])

    @property
    def mac_count(self):
        return lib().tfh_tree_mac_count(self._h)

    @property
    def peak_intermediate(self):
        return lib().tfh_tree_peak_intermediate(self._h)

    def __del__(self):
        if getattr(self, "_h", None) and _lib is not None:
            _lib.tfh_tree_destroy(self._h)
            self._h = None


# ---------------------------------------------------------------------------------------------- Tensor
class MemoryOrder:
    """tenferro-tensor/src/lib.rs:110-127."""
    ColumnMajor, RowMajor = 0, 1


def _contig_strides(dims, order):
    strides, n = [0] * len(dims), 1
    rng = range(len(dims)) if order == MemoryOrder.ColumnMajor else range(len(dims) - 1, -1, -1)
    for d in rng:
        strides[d] = n
        n *= dims[d]
    return strides


class CompletionEvent:
    """tenferro-tensor/src/lib.rs:301-309: a recorded hipEvent_t."""

    def __init__(self, stream):
        h = C.c_void_p()
        _check(lib().tfh_event_create(C.byref(h)))
        self._h = h.value
        _check(lib().tfh_event_record(self._h, stream))

    def synchronize(self):
        _check(lib().tfh_event_synchronize(self._h))

    def ready(self):
        r = C.c_int32()
        _check(lib().tfh_event_query(self._h, C.byref(r)))
        return bool(r.value)

    def __del__(self):
        if getattr(self, "_h", None) and _lib is not None:
            _lib.tfh_event_destroy(self._h)
            self._h = None


class Tensor:
    """Tensor<T> (tenferro-tensor/src/lib.rs:167-181): buffer + dims + strides (elements) + offset +
    logical memory space + preferred compute device + pending event.  MainMemory tensors hold a numpy
    array, GpuMemory tensors a flat torch CUDA tensor (DataBuffer::Hip)."""

    def __init__(self, buffer, dims, strides, offset, space, dtype, event=None, preferred=None):
        self._buf, self._dims, self._strides, self._offset = buffer, list(dims), list(strides), int(offset)
        self.logical_memory_space_, self.dtype, self.event = space, dtype, event
        self.preferred_compute_device_ = preferred
        self._lib_alloc = False     # the buffer was allocated by this module (not wrapped from the caller's tensor)
        self._conj = False          # conj_on_load(): operations read conj(element) (TFH_VIEW_CONJ)

    def _sole_owner(self):
        """No other Tensor (a permute/broadcast/diagonal view) and no caller-held object shares the buffer."""
        import sys
        return self._lib_alloc and sys.getrefcount(self._buf) <= 2      # the attribute + getrefcount's argument

    # ---- constructors (:336-371)
    @classmethod
    def _alloc(cls, dims, space, order, dtype, fill=None):
        dims = [int(d) for d in dims]
        n = int(np.prod(dims)) if dims else 1
        dt = dtype_code(dtype)
        if space.kind == 0:
            buf = np.zeros(n, _DT_NP[dt]) if fill is None else np.full(n, fill, _DT_NP[dt])
            return cls(buf, dims, _contig_strides(dims, order), 0, space, dt)
        import torch
        tdt = {F32: torch.float32, F64: torch.float64, C64: torch.complex64, C128: torch.complex128}[dt]
        buf = torch.empty(max(n, 1), dtype=tdt, device=f"cuda:{space.space_id}")
        t = cls(buf, dims, _contig_strides(dims, order), 0, space, dt)
        t._lib_alloc = True
        if fill is not None:
            v = t._view()
            st = current_stream()
            _check(lib().tfh_fill(dt, _scalar_c(dt, fill), C.byref(v), st))
            t.event = CompletionEvent(st)
        return t

    @classmethod
    def zeros(cls, dims, memory_space, order, dtype=np.float64):
        return cls._alloc(dims, memory_space, order, dtype, 0.0)

    @classmethod
    def ones(cls, dims, memory_space, order, dtype=np.float64):
        return cls._alloc(dims, memory_space, order, dtype, 1.0)

    @classmethod
    def empty(cls, dims, memory_space, order, dtype=np.float64):
        return cls._alloc(dims, memory_space, order, dtype, None)

    @classmethod
    def from_slice(cls, data, dims, order):
        """Data is laid out in `order`; memory space is MainMemory (:349-361)."""
        arr = np.ascontiguousarray(data).ravel()
        n = int(np.prod(dims)) if len(dims) else 1
        if arr.size != n:
            raise ShapeMismatch(f"shape mismatch: expected {[n]}, got {[arr.size]}", [n], [arr.size])
        return cls(arr.copy(), dims, _contig_strides(list(dims), order), 0, MainMemory, dtype_code(arr.dtype))

    @classmethod
    def from_torch(cls, t):
        """Zero-copy wrap of a torch CUDA tensor (any strides)."""
        if not t.is_cuda:
            raise InvalidArgument("invalid argument: from_torch takes a CUDA tensor")
        return cls(t, list(t.shape), [t.stride(d) for d in range(t.dim())], 0, GpuMemory(t.device.index or 0),
                   dtype_code(t.dtype))

    # ---- metadata (:378-420)
    def dims(self):
        return list(self._dims)

    def strides(self):
        return list(self._strides)

    def ndim(self):
        return len(self._dims)

    def len(self):
        return int(np.prod(self._dims)) if self._dims else 1

    def is_empty(self):
        return self.len() == 0

    def logical_memory_space(self):
        return self.logical_memory_space_

    def preferred_compute_device(self):
        return self.preferred_compute_device_

    def set_preferred_compute_device(self, device):
        self.preferred_compute_device_ = device

    def effective_compute_devices(self, op_kind):
        """:422-436: the override if set, else preferred_compute_devices(space, op)."""
        if self.preferred_compute_device_ is not None:
            return [self.preferred_compute_device_]
        return preferred_compute_devices(self.logical_memory_space_, op_kind)

    # ---- views (:502-542): metadata only, shared buffer
    def _like(self, dims, strides, offset=None):
        t = Tensor(self._buf, dims, strides, self._offset if offset is None else offset, self.logical_memory_space_,
                   self.dtype, self.event, self.preferred_compute_device_)
        t._lib_alloc = self._lib_alloc
        t._conj = self._conj
        return t

    def conj_on_load(self):
        """The lazy form of conj() (no counterpart in the reference, whose conj materialises): a view of the same buffer
        that contractions, permutes and einsum read as conj(element) -- the kernels flip the sign of the imaginary part
        while they stage the operand, so nothing is copied.  Real tensors come back unchanged.  The view and the views
        made of it (permute, broadcast, diagonal) keep the flag; conj() of such a view is a plain copy, into_conj() just
        drops the flag; it cannot be the output of an operation, and host access goes through conj() or to_numpy()."""
        t = self._like(self._dims, self._strides)
        if dtype_code(self.dtype) in (C64, C128):
            t._conj = not self._conj
        return t

    def permute(self, perm):
        if sorted(perm) != list(range(self.ndim())):
            raise InvalidArgument(f"invalid argument: {list(perm)} is not a permutation of 0..{self.ndim()}")
        return self._like([self._dims[p] for p in perm], [self._strides[p] for p in perm])

    def broadcast(self, target_dims):
        if len(target_dims) != self.ndim():
            raise RankMismatch(f"rank mismatch: expected {self.ndim()}, got {len(target_dims)}", self.ndim(), len(target_dims))
        strides = []
        for d, (have, want) in enumerate(zip(self._dims, target_dims)):
            if have == want:
                strides.append(self._strides[d])
            elif have == 1:
                strides.append(0)
            else:
                raise ShapeMismatch(f"shape mismatch: expected {self._dims}, got {list(target_dims)}", self._dims, list(target_dims))
        return self._like(list(target_dims), strides)

    def diagonal(self, axes):
        dims, strides = list(self._dims), list(self._strides)
        drop = []
        for i, j in axes:
            if not (0 <= i < self.ndim() and 0 <= j < self.ndim()) or i == j:
                raise InvalidArgument(f"invalid argument: diagonal axes ({i}, {j}) out of range")
            if dims[i] != dims[j]:
                raise ShapeMismatch(f"shape mismatch: expected {dims[i]}, got {dims[j]}", [dims[i]], [dims[j]])
            strides[i] += strides[j]
            drop.append(j)
        keep = [d for d in range(self.ndim()) if d not in drop]
        return self._like([dims[d] for d in keep], [strides[d] for d in keep])

    def is_contiguous(self):
        return self._strides in (_contig_strides(self._dims, MemoryOrder.ColumnMajor), _contig_strides(self._dims, MemoryOrder.RowMajor)) \
            or self.len() <= 1

    def reshape(self, new_dims):
        if int(np.prod(new_dims)) != self.len():
            raise ShapeMismatch(f"shape mismatch: expected {self._dims}, got {list(new_dims)}", self._dims, list(new_dims))
        if self._strides == _contig_strides(self._dims, MemoryOrder.ColumnMajor):
            return self._like(list(new_dims), _contig_strides(list(new_dims), MemoryOrder.ColumnMajor))
        if self._strides == _contig_strides(self._dims, MemoryOrder.RowMajor):
            return self._like(list(new_dims), _contig_strides(list(new_dims), MemoryOrder.RowMajor))
        raise InvalidArgument("invalid argument: reshape requires contiguous data")

    # ---- data operations (:552-671)
    def _view(self):
        if self.logical_memory_space_.kind == 0:
            raise NoCompatibleComputeDevice("no compatible compute device for this operation on MainMemory")
        v = tfh_view()
        v.base = self._buf.data_ptr()
        v.rank = len(self._dims)
        v.flags = 1 if self._conj else 0      # TFH_VIEW_CONJ
        v.offset = self._offset
        for d in range(len(self._dims)):
            v.dims[d], v.strides[d] = self._dims[d], self._strides[d]
        return v

    def contiguous(self, order):
        if self._strides == _contig_strides(self._dims, order):
            return self
        if self.logical_memory_space_.kind == 0:
            out = Tensor.from_slice(self.to_numpy().ravel(order="F" if order == MemoryOrder.ColumnMajor else "C"), self._dims, order)
            return out
        out = Tensor.empty(self._dims, self.logical_memory_space_, order, self.dtype)
        modes = list(range(self.ndim()))
        plan = HipBackend.plan(self.dtype, PrimDescriptor.Permute(modes, modes), [self._dims, self._dims])
        st = current_stream()
        HipBackend.execute(plan, 1.0, [self], 0.0, out, st)
        out.event = CompletionEvent(st)
        return out

    into_contiguous = contiguous

    def conj(self):
        """:622-647: conjugate every element, same layout.  Device tensors run tfh_conj."""
        if self.logical_memory_space_.kind == 0:
            return Tensor(np.conj(self._buf), self._dims, self._strides, self._offset, MainMemory, self.dtype)
        out = Tensor.empty(self._dims, self.logical_memory_space_, MemoryOrder.RowMajor, self.dtype)
        vi, vo = self._view(), out._view()
        st = current_stream()
        _check(lib().tfh_conj(self.dtype, C.byref(vi), C.byref(vo), st))
        out.event = CompletionEvent(st)
        return out

    def into_conj(self):
        """:653-658: in place when the tensor lives on the device."""
        if self.logical_memory_space_.kind == 0:
            return self.conj()
        if self._conj:                       # conj of a lazily conjugated view: the stored elements themselves
            self._conj = False
            return self
        vi = self._view()
        st = current_stream()
        _check(lib().tfh_conj(self.dtype, C.byref(vi), C.byref(vi), st))
        self.event = CompletionEvent(st)
        return self

    def view(self):
        """:445-449: the element view for host-side inspection.  Waits for pending work.  A main-memory tensor gives a
        numpy view with this tensor's dims and element strides over its buffer; device memory cannot back a host slice
        (use to_numpy, or to_memory_space_async, for a copy)."""
        self.wait()
        if self.logical_memory_space_.kind != 0:
            raise InvalidArgument("invalid argument: view() of a tensor in GPU memory; copy it with to_memory_space_async first")
        if self._conj:
            raise InvalidArgument("invalid argument: view() of a lazily conjugated tensor; materialise it with conj() first")
        return self._host_view(False)

    def _host_view(self, writeable):
        flat = np.asarray(self._buf).reshape(-1)
        isz = flat.dtype.itemsize
        return np.lib.stride_tricks.as_strided(flat[self._offset:], shape=self._dims, strides=[st * isz for st in self._strides],
                                               writeable=writeable and flat.flags.writeable)

    def view_mut(self):
        """:452-454"""
        self.view()
        return self._host_view(True)

    def tensor_view(self):
        """:455-470: waits, then a borrowed view (event None) sharing this tensor's buffer."""
        self.wait()
        return TensorView(self._like(self._dims, self._strides))

    def to_memory_space_async(self, target):
        """:660-671: same space -> self; Main->Gpu / Gpu->Main copy the underlying buffer."""
        if target == self.logical_memory_space_:
            return self
        if self._conj:
            raise InvalidArgument("invalid argument: a lazily conjugated tensor does not change memory space; materialise it with conj() first")
        import torch
        if target.kind == 1:
            buf = torch.from_numpy(np.ascontiguousarray(self._buf)).to(f"cuda:{target.space_id}", non_blocking=True)
            t = Tensor(buf, self._dims, self._strides, self._offset, target, self.dtype, CompletionEvent(current_stream()))
            t._lib_alloc = True
            return t
        self.wait()
        return Tensor(self._buf.cpu().numpy(), self._dims, self._strides, self._offset, target, self.dtype)

    def wait(self):
        """:677-704."""
        if self.event is not None:
            self.event.synchronize()
            self.event = None

    def is_ready(self):
        """:706-713."""
        return self.event is None or self.event.ready()

    def to_numpy(self):
        """Host copy with this tensor's dims (waits for pending work)."""
        self.wait()
        off = self._offset
        if self.logical_memory_space_.kind == 0:
            flat = self._buf
        else:
            # the elements as they lie in memory from the lowest to the highest address this view reaches (a wrapped
            # torch tensor may have any strides: its own .numpy() would hand back the logical order, not the memory order)
            import torch
            lo = off + sum((d - 1) * s for d, s in zip(self._dims, self._strides) if s < 0 and d > 0)
            hi = off + sum((d - 1) * s for d, s in zip(self._dims, self._strides) if s > 0 and d > 0)
            span = 0 if 0 in self._dims else hi - lo + 1
            flat = torch.as_strided(self._buf, (span,), (1,), self._buf.storage_offset() + lo).cpu().numpy()
            off -= lo
        isz = flat.dtype.itemsize
        out = np.lib.stride_tricks.as_strided(flat[off:], self._dims, [s * isz for s in self._strides]).copy()
        return np.conj(out) if self._conj else out


# ---------------------------------------------------------------------------------------------- einsum entry points
def _dispatch_check(operands, op_kind=OpKind.Contract):
    """Backend selection from the tensors' memory space (tenferro-einsum/src/lib.rs:16-20, 179-207)."""
    space = operands[0].logical_memory_space()
    for t in operands[1:]:
        if t.logical_memory_space() != space:
            raise CrossMemorySpaceOperation(f"cross-memory-space operation between {space!r} and {t.logical_memory_space()!r}",
                                            space, t.logical_memory_space())
    devices = None
    for t in operands:
        d = t.effective_compute_devices(op_kind)
        devices = d if devices is None else [x for x in devices if x in d]
    if not devices or devices[0].kind != ComputeDevice.HIP or space.kind != 1 or devices[0].device_id != space.space_id:
        raise NoCompatibleComputeDevice(f"no compatible compute device for Contract on {space!r}", space, op_kind)
    return space


class TensorView:
    """tenferro-tensor/src/lib.rs:183-300: the borrowed counterpart of Tensor.  It shares the source tensor's buffer,
    carries no pending event (tensor_view() has waited) and offers the zero-copy view operations plus the copying
    to_tensor / contiguous / conj."""

    def __init__(self, tensor):
        self._t = tensor
        self._t.event = None

    def dims(self):
        return self._t.dims()

    def strides(self):
        return self._t.strides()

    def ndim(self):
        return self._t.ndim()

    def logical_memory_space(self):
        return self._t.logical_memory_space()

    def preferred_compute_device(self):
        return self._t.preferred_compute_device()

    def permute(self, perm):
        """:250-252"""
        return TensorView(self._t.permute(perm))

    def broadcast(self, target_dims):
        """:262-264"""
        return TensorView(self._t.broadcast(target_dims))

    def diagonal(self, axes):
        """:272-274"""
        return TensorView(self._t.diagonal(axes))

    def to_tensor(self, order):
        """:281-283: always a fresh buffer, laid out in `order`."""
        t = self._t
        if t.logical_memory_space_.kind == 0:
            return Tensor.from_slice(t.to_numpy().ravel(order="F" if order == MemoryOrder.ColumnMajor else "C"), t._dims, order)
        out = Tensor.empty(t._dims, t.logical_memory_space_, order, t.dtype)
        modes = list(range(t.ndim()))
        st = current_stream()
        HipBackend.execute(HipBackend.plan(t.dtype, PrimDescriptor.Permute(modes, modes), [t._dims, t._dims]), 1.0, [t], 0.0, out, st)
        out.event = CompletionEvent(st)
        return out

    def contiguous(self, order):
        """:286-288: "a contiguous copy of this view's data"."""
        return self.to_tensor(order)

    def conj(self):
        """:293-299"""
        return self._t.conj()



def einsum_with_plan_into(tree, operands, alpha, beta, output, stream=None, _donate=0):
    """tenferro-einsum/src/lib.rs:584-621."""
    _dispatch_check(list(operands) + [output])
    dt = output.dtype
    views = (tfh_view * max(len(operands), 1))(*[t._view() for t in operands])
    vo = output._view()
    st = current_stream() if stream is None else stream
    # pending events of the operands are stream dependencies, never host waits (:146-177)
    _enqueue_on(list(operands) + [output], st)
    _check(lib().tfh_einsum_execute(dt, tree._h, views, len(operands), _scalar_c(dt, alpha), _scalar_c(dt, beta), C.byref(vo),
                                    C.c_uint64(_donate), st))
    _completed_on([output], st, operands)


def einsum_with_plan(tree, operands, stream=None, _donate=0):
    """:412-430"""
    space = _dispatch_check(operands)
    out = Tensor.empty(tree.output_dims, space, MemoryOrder.ColumnMajor, operands[0].dtype)
    einsum_with_plan_into(tree, operands, 1.0, 0.0, out, stream, _donate)
    return out


def einsum_with_subscripts(subscripts, operands, stream=None):
    """:397-412"""
    _dispatch_check(operands)
    tree = ContractionTree.optimize_cached(subscripts, [t.dims() for t in operands])
    return einsum_with_plan(tree, operands, stream)


def einsum(subscripts, operands, stream=None):
    """:393-398"""
    return einsum_with_subscripts(Subscripts.parse(subscripts), operands, stream)


def einsum_with_subscripts_into(subscripts, operands, alpha, beta, output, stream=None):
    """:578-582"""
    tree = ContractionTree.optimize_cached(subscripts, [t.dims() for t in operands])
    einsum_with_plan_into(tree, operands, alpha, beta, output, stream)


def einsum_into(subscripts, operands, alpha, beta, output, stream=None):
    """:541-549"""
    einsum_with_subscripts_into(Subscripts.parse(subscripts), operands, alpha, beta, output, stream)


def einsum_with_plan_owned(tree, operands, stream=None):
    """:493-498: operands are consumed: the executor may keep intermediates in the buffers that no other tensor
    shares, and they are released once the kernels are enqueued."""
    donate = sum(1 << i for i, t in enumerate(operands[:64]) if t._sole_owner())
    out = einsum_with_plan(tree, operands, stream, donate)
    operands.clear() if isinstance(operands, list) else None
    return out


def einsum_with_subscripts_owned(subscripts, operands, stream=None):
    """:474-480"""
    tree = ContractionTree.optimize_cached(subscripts, [t.dims() for t in operands])
    return einsum_with_plan_owned(tree, operands, stream)


def einsum_owned(subscripts, operands, stream=None):
    """:460-465"""
    return einsum_with_subscripts_owned(Subscripts.parse(subscripts), operands, stream)


# ---------------------------------------------------------------------------------------------- measurement aid
PROF_CONTRACT, PROF_COPY, PROF_REDUCE = 0, 1, 2


def profile_enable(on=True):
    """Bracket the dominant kernel of every launch with HIP events on its stream (tfh_profile_enable)."""
    _check(lib().tfh_profile_enable(1 if on else 0))


def tree_cache_stats():
    """(hits, misses, entries) of the library's cache of optimised einsum networks."""
    h, m, e = C.c_int64(), C.c_int64(), C.c_int64()
    _check(lib().tfh_tree_cache_stats(C.byref(h), C.byref(m), C.byref(e)))
    return h.value, m.value, e.value


def last_kernel():
    """Name of the dominant kernel the calling thread launched last (diagnostic)."""
    return lib().tfh_last_kernel().decode()


def profile_collect(kind):
    """(total milliseconds, launches) of one kernel kind since profile_enable."""
    ms, n = C.c_double(), C.c_int32()
    _check(lib().tfh_profile_collect(kind, C.byref(ms), C.byref(n)))
    return ms.value, n.value


def profile_kernels(kind):
    """[(kernel label, total milliseconds, launches)] of one kind since profile_enable, by kernel, in order of first
    launch (tfh_profile_kernel).  Call before profile_collect, which forgets the records."""
    out = []
    buf = C.create_string_buffer(512)
    while True:
        ms, n = C.c_double(), C.c_int32()
        _check(lib().tfh_profile_kernel(kind, len(out), buf, 512, C.byref(ms), C.byref(n)))
        if n.value == 0:
            return out
        out.append((buf.value.decode(), ms.value, n.value))
