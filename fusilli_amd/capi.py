"""ctypes binding of the C ABI declared in include/fusilli_hip.h.

This is the binding a non-C++ host would write; the tests and the benchmark
drive every kernel through it.  The library must have been built (see
``__graft_entry__.build``); a missing library is an error, never a fallback.
"""
from __future__ import annotations

import ctypes
import os
from ctypes import (POINTER, Structure, byref, c_char_p, c_double, c_float,
                    c_int, c_int32, c_int64, c_size_t, c_void_p)
from typing import Optional, Sequence

import numpy as np

MAX_RANK = 8
MAX_EPILOGUE = 4

# fhip_dtype
NOT_SET, HALF, BFLOAT16, FLOAT, DOUBLE, UINT8, INT4, INT8, INT16, INT32, INT64, \
    BOOLEAN, FP8E5M2, FP8E4M3 = range(14)

DTYPE_SIZE = {HALF: 2, BFLOAT16: 2, FLOAT: 4, DOUBLE: 8, UINT8: 1, INT8: 1,
              INT16: 2, INT32: 4, INT64: 8, BOOLEAN: 1, FP8E5M2: 1, FP8E4M3: 1}
DTYPE_NAME = {HALF: "f16", BFLOAT16: "bf16", FLOAT: "f32", DOUBLE: "f64",
              UINT8: "ui8", INT8: "si8", INT16: "si16", INT32: "si32",
              INT64: "si64", BOOLEAN: "i1", FP8E5M2: "f8E5M2",
              FP8E4M3: "f8E4M3FN"}

PW_NAMES = [
    "NOT_SET", "ABS", "ADD", "ADD_SQUARE", "BINARY_SELECT", "CEIL", "CMP_EQ",
    "CMP_GE", "CMP_GT", "CMP_LE", "CMP_LT", "CMP_NEQ", "DIV", "ELU_FWD", "ERF",
    "EXP", "FLOOR", "GELU_APPROX_TANH_BWD", "GELU_APPROX_TANH_FWD", "GELU_BWD",
    "GELU_FWD", "IDENTITY", "LOG", "LOGICAL_AND", "LOGICAL_NOT", "LOGICAL_OR",
    "MAX_OP", "MIN_OP", "MUL", "NEG", "RECIPROCAL", "RELU_BWD", "RELU_FWD",
    "RSQRT", "SIGMOID_FWD", "SIN", "SOFTPLUS_FWD", "SQRT", "SUB", "SWISH_BWD",
    "SWISH_FWD", "TAN", "TANH_BWD", "TANH_FWD",
]
PW = {n: i for i, n in enumerate(PW_NAMES)}
RED_NAMES = ["NOT_SET", "ADD", "SUM", "MUL", "MIN", "MAX", "AMAX", "AVG",
             "NORM1", "NORM2", "MUL_NO_ZEROS"]
RED = {n: i for i, n in enumerate(RED_NAMES)}

OPERAND_NONE, OPERAND_TENSOR, OPERAND_SCALAR = 0, 1, 2


class TensorDesc(Structure):
    _fields_ = [("rank", c_int32), ("dtype", c_int32),
                ("dim", c_int64 * MAX_RANK), ("stride", c_int64 * MAX_RANK)]

    @staticmethod
    def make(dims: Sequence[int], strides: Sequence[int], dtype: int) -> "TensorDesc":
        assert len(dims) == len(strides) <= MAX_RANK
        t = TensorDesc()
        t.rank = len(dims)
        t.dtype = dtype
        for i, (d, s) in enumerate(zip(dims, strides)):
            t.dim[i] = int(d)
            t.stride[i] = int(s)
        return t

    @staticmethod
    def absent() -> "TensorDesc":
        return TensorDesc()


class PointwiseParams(Structure):
    _fields_ = [("elu_alpha", c_float), ("softplus_beta", c_float),
                ("softplus_threshold", c_float), ("swish_beta", c_float)]

    @staticmethod
    def default() -> "PointwiseParams":
        return PointwiseParams(1.0, 1.0, 20.0, 1.0)


class EpilogueOp(Structure):
    _fields_ = [("mode", c_int32), ("operand_kind", c_int32),
                ("operand_index", c_int32), ("acc_is_in1", c_int32),
                ("result_dtype", c_int32), ("scalar", c_float),
                ("params", PointwiseParams), ("operand", TensorDesc)]


class Epilogue(Structure):
    _fields_ = [("count", c_int32), ("op", EpilogueOp * MAX_EPILOGUE)]


class MatmulDesc(Structure):
    _fields_ = [("a", TensorDesc), ("b", TensorDesc), ("c", TensorDesc),
                ("epilogue", Epilogue), ("out_dtype", c_int32),
                ("out", TensorDesc)]


class ConvDesc(Structure):
    _fields_ = [("x", TensorDesc), ("w", TensorDesc), ("y", TensorDesc),
                ("spatial_rank", c_int32), ("padding", c_int64 * 3),
                ("stride", c_int64 * 3), ("dilation", c_int64 * 3),
                ("epilogue", Epilogue), ("out_dtype", c_int32),
                ("out", TensorDesc)]


class SdpaDesc(Structure):
    _fields_ = [("q", TensorDesc), ("k", TensorDesc), ("v", TensorDesc),
                ("mask", TensorDesc), ("o", TensorDesc), ("is_causal", c_int32),
                ("has_scale", c_int32), ("scale", c_float)]


class NormDesc(Structure):
    _fields_ = [("x", TensorDesc), ("scale", TensorDesc), ("bias", TensorDesc),
                ("y", TensorDesc), ("epsilon", c_float),
                ("is_layernorm", c_int32), ("emit_stats", c_int32),
                ("stats_dtype", c_int32), ("epilogue", Epilogue),
                ("out_dtype", c_int32), ("out", TensorDesc)]


class BatchNormDesc(Structure):
    _fields_ = [("x", TensorDesc), ("y", TensorDesc), ("training", c_int32),
                ("has_scale", c_int32), ("has_bias", c_int32),
                ("scale_dtype", c_int32), ("bias_dtype", c_int32),
                ("running_dtype", c_int32), ("stats_dtype", c_int32),
                ("epsilon", c_float)]


class ReduceDesc(Structure):
    _fields_ = [("x", TensorDesc), ("y", TensorDesc), ("mode", c_int32)]


class PointwiseDesc(Structure):
    _fields_ = [("mode", c_int32), ("num_inputs", c_int32),
                ("in_", TensorDesc * 3), ("in_is_scalar", c_int32 * 3),
                ("in_scalar", c_double * 3), ("out", TensorDesc),
                ("params", PointwiseParams)]


def epilogue_op(mode: int, result_dtype: int, *, scalar: Optional[float] = None,
                operand: Optional[TensorDesc] = None, operand_index: int = 0,
                acc_is_in1: bool = False,
                params: Optional[PointwiseParams] = None) -> EpilogueOp:
    op = EpilogueOp()
    op.mode = mode
    op.result_dtype = result_dtype
    op.acc_is_in1 = 1 if acc_is_in1 else 0
    op.params = params or PointwiseParams.default()
    if operand is not None:
        op.operand_kind = OPERAND_TENSOR
        op.operand = operand
        op.operand_index = operand_index
    elif scalar is not None:
        op.operand_kind = OPERAND_SCALAR
        op.scalar = scalar
    else:
        op.operand_kind = OPERAND_NONE
    return op


def make_epilogue(ops: Sequence[EpilogueOp]) -> Epilogue:
    e = Epilogue()
    e.count = len(ops)
    for i, o in enumerate(ops):
        e.op[i] = o
    return e


# FUSILLI_HIP_LIBRARY names another build of the library (tuning runs that
# compare builds side by side); the default is the in-tree one.
_LIB_PATH = os.environ.get("FUSILLI_HIP_LIBRARY") or os.path.join(
    os.path.dirname(os.path.abspath(__file__)), "lib", "libfusilli_hip.so")

# name -> (restype, argtypes); every symbol include/fusilli_hip.h declares.
_P = c_void_p
SYMBOLS = {
    "fhip_abi_version": (c_int, []),
    "fhip_device_count": (c_int, [POINTER(c_int)]),
    "fhip_device_arch": (c_int, [c_int, c_char_p, c_size_t]),
    "fhip_tuning_reload": (c_int, []),
    "fhip_ctx_create": (c_int, [c_int, _P, POINTER(_P)]),
    "fhip_ctx_destroy": (c_int, [_P]),
    "fhip_last_error": (c_char_p, [_P]),
    "fhip_last_kernel": (c_char_p, [_P]),
    "fhip_ctx_stream": (_P, [_P]),
    "fhip_ctx_device": (c_int, [_P]),
    "fhip_malloc": (c_int, [_P, c_size_t, POINTER(_P)]),
    "fhip_free": (c_int, [_P, _P]),
    "fhip_memcpy_h2d": (c_int, [_P, _P, _P, c_size_t]),
    "fhip_memcpy_d2h": (c_int, [_P, _P, _P, c_size_t]),
    "fhip_memcpy_d2d": (c_int, [_P, _P, _P, c_size_t]),
    "fhip_memset": (c_int, [_P, _P, c_int, c_size_t]),
    "fhip_stream_sync": (c_int, [_P]),
    "fhip_event_create": (c_int, [_P, POINTER(_P)]),
    "fhip_event_record": (c_int, [_P, _P]),
    "fhip_event_elapsed_ms": (c_int, [_P, _P, _P, POINTER(c_float)]),
    "fhip_event_destroy": (c_int, [_P, _P]),
    "fhip_matmul_workspace_size": (c_int, [POINTER(MatmulDesc), POINTER(c_size_t)]),
    "fhip_matmul_supported": (c_int, [POINTER(MatmulDesc)]),
    "fhip_matmul": (c_int, [_P, POINTER(MatmulDesc), _P, _P, POINTER(_P), _P, _P, c_size_t]),
    "fhip_conv_fprop_workspace_size": (c_int, [POINTER(ConvDesc), POINTER(c_size_t)]),
    "fhip_conv_fprop_supported": (c_int, [POINTER(ConvDesc)]),
    "fhip_conv_fprop": (c_int, [_P, POINTER(ConvDesc), _P, _P, POINTER(_P), _P, _P, c_size_t]),
    "fhip_conv_dgrad_workspace_size": (c_int, [POINTER(ConvDesc), POINTER(c_size_t)]),
    "fhip_conv_dgrad_supported": (c_int, [POINTER(ConvDesc)]),
    "fhip_conv_dgrad": (c_int, [_P, POINTER(ConvDesc), _P, _P, _P, _P, c_size_t]),
    "fhip_conv_dgrad_static": (c_int, [_P, POINTER(ConvDesc), _P, _P, _P]),
    "fhip_conv_wgrad_workspace_size": (c_int, [POINTER(ConvDesc), POINTER(c_size_t)]),
    "fhip_conv_wgrad_supported": (c_int, [POINTER(ConvDesc)]),
    "fhip_conv_wgrad": (c_int, [_P, POINTER(ConvDesc), _P, _P, _P, _P, c_size_t]),
    "fhip_sdpa_fwd_workspace_size": (c_int, [POINTER(SdpaDesc), POINTER(c_size_t)]),
    "fhip_sdpa_fwd_supported": (c_int, [POINTER(SdpaDesc)]),
    "fhip_sdpa_fwd": (c_int, [_P, POINTER(SdpaDesc), _P, _P, _P, _P, _P, _P, c_size_t]),
    "fhip_norm_fwd_workspace_size": (c_int, [POINTER(NormDesc), POINTER(c_size_t)]),
    "fhip_norm_fwd_supported": (c_int, [POINTER(NormDesc)]),
    "fhip_norm_fwd": (c_int, [_P, POINTER(NormDesc), _P, _P, _P, POINTER(_P), _P, _P, _P, _P, c_size_t]),
    "fhip_batchnorm_fwd_workspace_size": (c_int, [POINTER(BatchNormDesc), POINTER(c_size_t)]),
    "fhip_batchnorm_fwd_supported": (c_int, [POINTER(BatchNormDesc)]),
    "fhip_batchnorm_fwd": (c_int, [_P, POINTER(BatchNormDesc), _P, _P, _P, _P, _P,
                                   _P, _P, _P, _P, c_size_t]),
    "fhip_reduce_workspace_size": (c_int, [POINTER(ReduceDesc), POINTER(c_size_t)]),
    "fhip_reduce_supported": (c_int, [POINTER(ReduceDesc)]),
    "fhip_reduce": (c_int, [_P, POINTER(ReduceDesc), _P, _P, _P, c_size_t]),
    "fhip_pointwise_supported": (c_int, [POINTER(PointwiseDesc)]),
    "fhip_pointwise": (c_int, [_P, POINTER(PointwiseDesc), _P, _P, _P, _P]),
}

_lib = None


class FusilliHipError(RuntimeError):
    pass


def library_path() -> str:
    return _LIB_PATH


def load() -> ctypes.CDLL:
    """Loads libfusilli_hip.so; raises if it has not been built."""
    global _lib
    if _lib is not None:
        return _lib
    if not os.path.exists(_LIB_PATH):
        raise FusilliHipError(
            f"{_LIB_PATH} is missing: build it with "
            "`python -c 'import __graft_entry__ as g; g.build()'` "
            "(there is no CPU fallback)")
    lib = ctypes.CDLL(_LIB_PATH)
    for name, (res, args) in SYMBOLS.items():
        fn = getattr(lib, name)
        fn.restype = res
        fn.argtypes = args
    _lib = lib
    return lib


class DeviceBuffer:
    """Device allocation owned through the C ABI."""

    def __init__(self, ctx: "Context", nbytes: int):
        self.ctx = ctx
        self.nbytes = int(nbytes)
        p = _P()
        ctx._check(ctx.lib.fhip_malloc(ctx.handle, self.nbytes, byref(p)))
        self.ptr = p.value

    def free(self):
        if self.ptr is not None and self.ctx.handle is not None:
            self.ctx.lib.fhip_free(self.ctx.handle, self.ptr)
        self.ptr = None

    def __del__(self):
        try:
            self.free()
        except Exception:
            pass

    def upload(self, host: np.ndarray):
        h = np.ascontiguousarray(host)
        assert h.nbytes <= self.nbytes
        self.ctx._check(self.ctx.lib.fhip_memcpy_h2d(
            self.ctx.handle, self.ptr, h.ctypes.data, h.nbytes))

    def download(self, np_dtype, count: Optional[int] = None) -> np.ndarray:
        item = np.dtype(np_dtype).itemsize
        n = self.nbytes // item if count is None else count
        out = np.empty(n, np_dtype)
        self.ctx._check(self.ctx.lib.fhip_memcpy_d2h(
            self.ctx.handle, out.ctypes.data, self.ptr, n * item))
        return out


class Event:
    def __init__(self, ctx: "Context"):
        self.ctx = ctx
        p = _P()
        ctx._check(ctx.lib.fhip_event_create(ctx.handle, byref(p)))
        self.ptr = p.value

    def record(self):
        self.ctx._check(self.ctx.lib.fhip_event_record(self.ctx.handle, self.ptr))

    def elapsed_ms_since(self, start: "Event") -> float:
        ms = c_float()
        self.ctx._check(self.ctx.lib.fhip_event_elapsed_ms(
            self.ctx.handle, start.ptr, self.ptr, byref(ms)))
        return ms.value

    def __del__(self):
        try:
            if self.ptr is not None and self.ctx.handle is not None:
                self.ctx.lib.fhip_event_destroy(self.ctx.handle, self.ptr)
        except Exception:
            pass


def _epi_ptrs(operands: Sequence[Optional[DeviceBuffer]]):
    arr = (_P * MAX_EPILOGUE)()
    for i, b in enumerate(operands):
        arr[i] = None if b is None else (b.ptr if isinstance(b, DeviceBuffer) else b)
    return arr


def _p(b):
    if b is None:
        return None
    return b.ptr if isinstance(b, DeviceBuffer) else b


class Context:
    """One fhip_ctx: a device plus the stream every call is ordered on."""

    def __init__(self, device: int = 0, stream: Optional[int] = None):
        self.lib = load()
        self.handle = None
        h = _P()
        rc = self.lib.fhip_ctx_create(device, stream, byref(h))
        if rc != 0:
            raise FusilliHipError(self.lib.fhip_last_error(None).decode())
        self.handle = h.value

    def close(self):
        if self.handle is not None:
            self.lib.fhip_ctx_destroy(self.handle)
            self.handle = None

    def __enter__(self):
        return self

    def __exit__(self, *exc):
        self.close()

    def _check(self, rc: int):
        if rc != 0:
            raise FusilliHipError(self.lib.fhip_last_error(self.handle).decode())

    def last_kernel(self) -> str:
        """Kernel variant the last operator call on this context launched."""
        return self.lib.fhip_last_kernel(self.handle).decode()

    def arch(self) -> str:
        buf = ctypes.create_string_buffer(256)
        self._check(self.lib.fhip_device_arch(
            self.lib.fhip_ctx_device(self.handle), buf, 256))
        return buf.value.decode()

    def alloc(self, nbytes: int) -> DeviceBuffer:
        return DeviceBuffer(self, nbytes)

    def to_device(self, host: np.ndarray) -> DeviceBuffer:
        b = DeviceBuffer(self, max(host.nbytes, 1))
        b.upload(host)
        return b

    def sync(self):
        self._check(self.lib.fhip_stream_sync(self.handle))

    def event(self) -> Event:
        return Event(self)

    def memset(self, buf: DeviceBuffer, value: int):
        self._check(self.lib.fhip_memset(self.handle, buf.ptr, value, buf.nbytes))

    # ---- ops -------------------------------------------------------------
    def matmul(self, d: MatmulDesc, a, b, out, epilogue_operands=()):
        self._check(self.lib.fhip_matmul(self.handle, byref(d), _p(a), _p(b),
                                         _epi_ptrs(epilogue_operands), _p(out),
                                         None, 0))

    def conv_fprop(self, d: ConvDesc, x, w, out, epilogue_operands=()):
        self._check(self.lib.fhip_conv_fprop(self.handle, byref(d), _p(x), _p(w),
                                             _epi_ptrs(epilogue_operands),
                                             _p(out), None, 0))

    def conv_dgrad(self, d: ConvDesc, dy, w, dx, workspace=None):
        """`workspace`: a DeviceBuffer of at least conv_dgrad_workspace(d)
        bytes; allocated here when omitted."""
        need = self.conv_dgrad_workspace(d)
        if need and workspace is None:
            workspace = self.alloc(need)
        self._check(self.lib.fhip_conv_dgrad(self.handle, byref(d), _p(dy),
                                             _p(w), _p(dx), _p(workspace),
                                             need))

    def conv_dgrad_static(self, d: ConvDesc, dy, w, dx):
        """The data gradient on the library's static scratch: no workspace
        argument and no allocation inside the call."""
        self._check(self.lib.fhip_conv_dgrad_static(self.handle, byref(d),
                                                    _p(dy), _p(w), _p(dx)))

    def conv_dgrad_workspace(self, d: ConvDesc) -> int:
        n = c_size_t(0)
        if self.lib.fhip_conv_dgrad_workspace_size(byref(d), byref(n)) != 0:
            # a query without a context reports through the process-wide slot
            raise FusilliHipError(self.lib.fhip_last_error(None).decode())
        return n.value

    def conv_wgrad(self, d: ConvDesc, dy, x, dw, workspace=None):
        """`workspace`: a DeviceBuffer of at least conv_wgrad_workspace(d)
        bytes; allocated here when omitted."""
        need = self.conv_wgrad_workspace(d)
        if need and workspace is None:
            workspace = self.alloc(need)
        self._check(self.lib.fhip_conv_wgrad(self.handle, byref(d), _p(dy),
                                             _p(x), _p(dw), _p(workspace),
                                             need))

    def conv_wgrad_workspace(self, d: ConvDesc) -> int:
        n = c_size_t(0)
        if self.lib.fhip_conv_wgrad_workspace_size(byref(d), byref(n)) != 0:
            raise FusilliHipError(self.lib.fhip_last_error(None).decode())
        return n.value

    def batchnorm_fwd(self, d: BatchNormDesc, x, y, scale=None, bias=None,
                      running_mean=None, running_var=None, saved_mean=None,
                      saved_inv_variance=None):
        self._check(self.lib.fhip_batchnorm_fwd(
            self.handle, byref(d), _p(x), _p(scale), _p(bias), _p(running_mean),
            _p(running_var), _p(y), _p(saved_mean), _p(saved_inv_variance),
            None, 0))

    def sdpa_fwd(self, d: SdpaDesc, q, k, v, o, mask=None):
        self._check(self.lib.fhip_sdpa_fwd(self.handle, byref(d), _p(q), _p(k),
                                           _p(v), _p(mask), _p(o), None, 0))

    def norm_fwd(self, d: NormDesc, x, scale, bias, out, mean=None, rstd=None,
                 epilogue_operands=()):
        self._check(self.lib.fhip_norm_fwd(self.handle, byref(d), _p(x),
                                           _p(scale), _p(bias),
                                           _epi_ptrs(epilogue_operands), _p(out),
                                           _p(mean), _p(rstd), None, 0))

    def reduce(self, d: ReduceDesc, x, y):
        self._check(self.lib.fhip_reduce(self.handle, byref(d), _p(x), _p(y),
                                         None, 0))

    def pointwise(self, d: PointwiseDesc, in0, in1, in2, out):
        self._check(self.lib.fhip_pointwise(self.handle, byref(d), _p(in0),
                                            _p(in1), _p(in2), _p(out)))
