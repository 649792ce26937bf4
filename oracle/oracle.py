"""CPU oracle: numpy front for oracle/fusilli_oracle.c.

TEST INFRASTRUCTURE ONLY — imported by tests/, by ``__graft_entry__.smoke()``
and by the ``cpu_baseline`` leg of ``bench.py``; never by the product package.

The reference holds no arithmetic of its own (every node lowers to one aten op
executed by IREE, which is not vendored), so this module restates the aten
semantics the reference's emitter selects (reference
``include/fusilli/support/asm_emitter.h``) together with the reference's
layout rules: a tensor is logical dims plus element strides
(``attributes/tensor_attributes.h:374-809``), ops work in a fixed logical dim
order, and the physical buffer is whatever the strides say.

Pinning status of each function (what independent evidence checks it) is
recorded next to it; the checks themselves live in
``tests/test_oracle_pinning.py``.
"""
from __future__ import annotations

import ctypes
import math
import os
import subprocess
from typing import Optional, Sequence

import numpy as np

_HERE = os.path.dirname(os.path.abspath(__file__))
_LIB_PATH = os.path.join(_HERE, "liboracle.so")

# Element type codes: the reference's DataType enum order
# (attributes/types.h:27-45) plus FP8E4M3 = 13.
NOT_SET, HALF, BFLOAT16, FLOAT, DOUBLE, UINT8, INT4, INT8, INT16, INT32, INT64, \
    BOOLEAN, FP8E5M2, FP8E4M3 = range(14)

_STORAGE = {
    HALF: np.float16, BFLOAT16: np.uint16, FLOAT: np.float32,
    DOUBLE: np.float64, UINT8: np.uint8, INT8: np.int8, INT16: np.int16,
    INT32: np.int32, INT64: np.int64, BOOLEAN: np.uint8, FP8E5M2: np.uint8,
    FP8E4M3: np.uint8,
}


def build(force: bool = False) -> str:
    """Compiles fusilli_oracle.c into liboracle.so (gcc, OpenMP)."""
    src = os.path.join(_HERE, "fusilli_oracle.c")
    if force or not os.path.exists(_LIB_PATH) or \
            os.path.getmtime(_LIB_PATH) < os.path.getmtime(src):
        subprocess.check_call(
            ["gcc", "-O2", "-fopenmp", "-fPIC", "-shared", "-std=c11",
             "-o", _LIB_PATH, src, "-lm"])
    return _LIB_PATH


_lib = None


def lib() -> ctypes.CDLL:
    global _lib
    if _lib is None:
        build()  # compiles only when the library is missing or stale
        _lib = ctypes.CDLL(_LIB_PATH)
    return _lib


def _ptr(a: Optional[np.ndarray]):
    return None if a is None else a.ctypes.data_as(ctypes.c_void_p)


def storage_dtype(dtype: int):
    return _STORAGE[dtype]


def is_float(dtype: int) -> bool:
    return dtype in (HALF, BFLOAT16, FLOAT, DOUBLE, FP8E5M2, FP8E4M3)


# --------------------------------------------------------------------------
# Element conversions.  Pinned by: exhaustive decode tables of both fp8
# formats against torch.float8_e4m3fn / float8_e5m2, bf16 against
# torch.bfloat16 on random and boundary values, round-trip identity over all
# 256 / 65536 codes.
# --------------------------------------------------------------------------
def quantize(values: np.ndarray, dtype: int) -> np.ndarray:
    """Rounds real values to the storage type (RNE; fp8 and integers saturate)."""
    v = np.ascontiguousarray(values)
    if dtype == BFLOAT16:
        f = v.astype(np.float32).ravel()
        out = np.empty(f.size, np.uint16)
        lib().oracle_f32_to_bf16_n(_ptr(f), _ptr(out), ctypes.c_int64(f.size))
        return out.reshape(v.shape)
    if dtype in (FP8E4M3, FP8E5M2):
        f = v.astype(np.float32).ravel()
        out = np.empty(f.size, np.uint8)
        lib().oracle_f32_to_fp8_n(_ptr(f), _ptr(out), ctypes.c_int64(f.size),
                                  ctypes.c_int(4 if dtype == FP8E4M3 else 5))
        return out.reshape(v.shape)
    if dtype == BOOLEAN:
        return (v != 0).astype(np.uint8)
    st = _STORAGE[dtype]
    if np.issubdtype(st, np.integer):
        info = np.iinfo(st)
        return np.clip(np.rint(v.astype(np.float64)), info.min, info.max).astype(st)
    return v.astype(st)


def dequantize(storage: np.ndarray, dtype: int) -> np.ndarray:
    """Exact widening of stored values: f32 for floats (f64 for Double), int64
    for integers."""
    s = np.ascontiguousarray(storage)
    if dtype == BFLOAT16:
        return (s.astype(np.uint32) << 16).view(np.float32).reshape(s.shape)
    if dtype in (FP8E4M3, FP8E5M2):
        flat = s.ravel()
        out = np.empty(flat.size, np.float32)
        lib().oracle_fp8_to_f32_n(_ptr(flat), _ptr(out),
                                  ctypes.c_int64(flat.size),
                                  ctypes.c_int(4 if dtype == FP8E4M3 else 5))
        return out.reshape(s.shape)
    if dtype == DOUBLE:
        return s.astype(np.float64)
    if dtype in (HALF, FLOAT):
        return s.astype(np.float32)
    return s.astype(np.int64)


# --------------------------------------------------------------------------
# Layout (reference attributes/tensor_attributes.h).  Pinned by the layout
# golden vectors of the reference's tests/test_tensor_attributes.cpp and by
# the transposed-add known answer of samples/pointwise/pointwise_add_transposed.cpp.
# --------------------------------------------------------------------------
def contiguous_strides(dims: Sequence[int]) -> list:
    """Row-major strides (tensor_attributes.h:159-176, 222-252)."""
    st, acc = [0] * len(dims), 1
    for i in range(len(dims) - 1, -1, -1):
        st[i] = acc
        acc *= dims[i]
    return st


def channels_last_strides(dims: Sequence[int]) -> list:
    """Channels-last strides for logical NC<spatial> dims
    (tensor_attributes.h:177-193): C innermost, then spatial right-to-left,
    N outermost."""
    n = len(dims)
    order = [1] + list(range(n - 1, 1, -1)) + [0]  # fastest -> slowest
    st, acc = [0] * n, 1
    for d in order:
        st[d] = acc
        acc *= dims[d]
    return st


def storage_extent(dims: Sequence[int], strides: Sequence[int]) -> int:
    """Number of storage elements a (dims, strides) view touches."""
    return 1 + sum((d - 1) * s for d, s in zip(dims, strides))


def logical_view(storage: np.ndarray, dims, strides) -> np.ndarray:
    """Strided logical view of a 1-D storage array."""
    flat = storage.reshape(-1)
    assert storage_extent(dims, strides) <= flat.size
    item = flat.itemsize
    return np.lib.stride_tricks.as_strided(
        flat, shape=tuple(dims), strides=tuple(int(s) * item for s in strides),
        writeable=False)


def to_storage(logical: np.ndarray, strides) -> np.ndarray:
    """Lays a logical array out in a fresh 1-D storage array with the given
    element strides (no broadcast strides)."""
    dims = logical.shape
    out = np.zeros(storage_extent(dims, strides), logical.dtype)
    view = np.lib.stride_tricks.as_strided(
        out, shape=tuple(dims),
        strides=tuple(int(s) * out.itemsize for s in strides))
    view[...] = logical
    return out


# --------------------------------------------------------------------------
# Ops on logical arrays.  Inputs: f32 (or int) logical ndarrays holding the
# exact stored values.  Outputs: f64 (int32 for the integer matmul).
# --------------------------------------------------------------------------
def matmul(a: np.ndarray, b: np.ndarray) -> np.ndarray:
    """aten.matmul with 1-to-N batch broadcast (asm_emitter.h:1669-1696,
    matmul_node.h:40-66).  Pinned by: all-ones => K (samples/matmul/
    matmul_basic.cpp:91-94), one-hot B selects columns, numpy float64 matmul
    on random inputs, brute-force triple loop on tiny shapes."""
    assert a.ndim == b.ndim >= 2 and a.shape[-1] == b.shape[-2]
    batch = np.broadcast_shapes(a.shape[:-2], b.shape[:-2])
    m, k, n = a.shape[-2], a.shape[-1], b.shape[-1]
    nb = int(np.prod(batch)) if batch else 1
    if np.issubdtype(a.dtype, np.integer) and np.issubdtype(b.dtype, np.integer):
        af = np.ascontiguousarray(np.broadcast_to(a, batch + (m, k))).astype(np.int8)
        bf = np.ascontiguousarray(np.broadcast_to(b, batch + (k, n))).astype(np.int8)
        assert np.array_equal(af, np.broadcast_to(a, batch + (m, k)))
        assert np.array_equal(bf, np.broadcast_to(b, batch + (k, n)))
        c = np.empty(batch + (m, n), np.int32)
        lib().oracle_matmul_i8_i32(_ptr(af), _ptr(bf), _ptr(c),
                                   *(ctypes.c_int64(x) for x in (nb, m, k, n)))
        return c
    af = np.ascontiguousarray(np.broadcast_to(a, batch + (m, k)), np.float32)
    bf = np.ascontiguousarray(np.broadcast_to(b, batch + (k, n)), np.float32)
    c = np.empty(batch + (m, n), np.float64)
    lib().oracle_matmul_f32(_ptr(af), _ptr(bf), _ptr(c),
                            *(ctypes.c_int64(x) for x in (nb, m, k, n)))
    return c


def matmul_rows(a: np.ndarray, b: np.ndarray, rows: np.ndarray) -> np.ndarray:
    """Rows ``rows`` of the 2-D product a @ b (full-size spot checks)."""
    assert a.ndim == 2 and b.ndim == 2
    rows = np.ascontiguousarray(rows, np.int64)
    k, n = a.shape[1], b.shape[1]
    if np.issubdtype(a.dtype, np.integer):
        a8, b8 = np.ascontiguousarray(a, np.int8), np.ascontiguousarray(b, np.int8)
        c = np.empty((rows.size, n), np.int32)
        lib().oracle_matmul_i8_i32_rows(_ptr(a8), _ptr(b8), _ptr(c), _ptr(rows),
                                        ctypes.c_int64(rows.size),
                                        ctypes.c_int64(k), ctypes.c_int64(n))
        return c
    af, bf = np.ascontiguousarray(a, np.float32), np.ascontiguousarray(b, np.float32)
    c = np.empty((rows.size, n), np.float64)
    lib().oracle_matmul_f32_rows(_ptr(af), _ptr(bf), _ptr(c), _ptr(rows),
                                 ctypes.c_int64(rows.size), ctypes.c_int64(k),
                                 ctypes.c_int64(n))
    return c


def conv_output_dims(x_dims, w_dims, padding, stride, dilation) -> list:
    """node/conv_node.h:38-56."""
    out = [x_dims[0], w_dims[0]]
    for i in range(len(x_dims) - 2):
        out.append(1 + (x_dims[2 + i] + 2 * padding[i]
                        - dilation[i] * (w_dims[2 + i] - 1) - 1) // stride[i])
    return out


def conv_fprop(x: np.ndarray, w: np.ndarray, padding, stride, dilation) -> np.ndarray:
    """aten.convolution forward, groups = C / fC (asm_emitter.h:690-701).
    Pinned by: all-ones known answers of the reference samples (1x1 => C,
    3x3 same-pad corner => 4*C, grouped => fC*R*S), delta filter = shifted
    copy, 1x1 filter = matmul, torch.nn.functional.conv{1,2,3}d on random
    inputs incl. stride/dilation/padding/groups."""
    sp = x.ndim - 2
    assert 1 <= sp <= 3 and w.ndim == x.ndim
    n, c = x.shape[:2]
    k, fc = w.shape[:2]
    assert c % fc == 0 and k % (c // fc) == 0
    od = conv_output_dims(x.shape, w.shape, padding, stride, dilation)
    lead = 3 - sp

    def pad3(v, fill):
        return (ctypes.c_int64 * 3)(*([fill] * lead + [int(t) for t in v]))

    xf = np.ascontiguousarray(x, np.float32)
    wf = np.ascontiguousarray(w, np.float32)
    y = np.empty(od, np.float64)
    lib().oracle_conv_fprop(
        _ptr(xf), _ptr(wf), _ptr(y), ctypes.c_int64(n), ctypes.c_int64(c),
        ctypes.c_int64(k), ctypes.c_int64(fc), pad3(x.shape[2:], 1),
        pad3(w.shape[2:], 1), pad3(od[2:], 1), pad3(padding, 0),
        pad3(stride, 1), pad3(dilation, 1))
    return y


def _conv_backward(fn, dy, other, x_dims, w_dims, padding, stride, dilation,
                   out_dims):
    sp = len(x_dims) - 2
    assert 1 <= sp <= 3
    n, c = x_dims[:2]
    k, fc = w_dims[:2]
    assert c % fc == 0 and k % (c // fc) == 0
    od = conv_output_dims(x_dims, w_dims, padding, stride, dilation)
    assert list(dy.shape) == od, (dy.shape, od)
    lead = 3 - sp

    def pad3(v, fill):
        return (ctypes.c_int64 * 3)(*([fill] * lead + [int(t) for t in v]))

    gy = np.ascontiguousarray(dy, np.float32)
    of = np.ascontiguousarray(other, np.float32)
    out = np.empty(out_dims, np.float64)
    fn(_ptr(gy), _ptr(of), _ptr(out), ctypes.c_int64(n), ctypes.c_int64(c),
       ctypes.c_int64(k), ctypes.c_int64(fc), pad3(x_dims[2:], 1),
       pad3(w_dims[2:], 1), pad3(od[2:], 1), pad3(padding, 0), pad3(stride, 1),
       pad3(dilation, 1))
    return out


def conv_dgrad(dy: np.ndarray, w: np.ndarray, x_dims, padding, stride,
               dilation) -> np.ndarray:
    """Data gradient of conv_fprop (node/conv_node.h:428-598, emitted as
    aten.convolution_backward).  Pinned by: the reference samples' all-ones
    answers (1x1 => K, grouped => K / groups), the adjoint identity
    <conv(x, w), dy> = <x, dgrad(dy, w)> on random inputs, torch autograd
    (float64) incl. stride/dilation/padding/groups, 1-D and 3-D."""
    assert dy.ndim == w.ndim == len(x_dims)
    return _conv_backward(lib().oracle_conv_dgrad, dy, w, list(x_dims),
                          list(w.shape), padding, stride, dilation,
                          list(x_dims))


def conv_wgrad(dy: np.ndarray, x: np.ndarray, w_dims, padding, stride,
               dilation) -> np.ndarray:
    """Weight gradient of conv_fprop (node/conv_node.h:255-426, emitted as
    aten.convolution_backward).  Pinned by: the reference samples' all-ones
    answers (1x1 => N*H*W, strided => N*Ho*Wo), the adjoint identity
    <conv(x, w), dy> = <w, wgrad(dy, x)>, torch autograd (float64)."""
    return _conv_backward(lib().oracle_conv_wgrad, dy, x, list(x.shape),
                          list(w_dims), padding, stride, dilation,
                          list(w_dims))


def sdpa(q, k, v, mask=None, is_causal=False, scale=None) -> np.ndarray:
    """aten.scaled_dot_product_attention (asm_emitter.h:2409-2468;
    samples/sdpa_utils.cpp:49-102).  ``mask``: additive float array or boolean
    array (True = attend), broadcastable to [B,Hq,Sq,Skv].  Pinned by:
    constant fill => V (reference samples), Skv = 1 => O = V, uniform scores
    under causal => prefix means of V, torch F.scaled_dot_product_attention on
    random inputs incl. GQA / cross-attention / masks."""
    B, Hq, Sq, D = q.shape
    _, Hkv, Skv, _ = k.shape
    Dv = v.shape[3]
    assert Hq % Hkv == 0
    if scale is None:
        scale = 1.0 / math.sqrt(D)
    m = None
    if mask is not None:
        mm = np.asarray(mask)
        if mm.dtype == np.bool_:
            mm = np.where(mm, 0.0, -np.inf)
        m = np.ascontiguousarray(np.broadcast_to(mm, (B, Hq, Sq, Skv)), np.float32)
    qf, kf, vf = (np.ascontiguousarray(t, np.float32) for t in (q, k, v))
    o = np.empty((B, Hq, Sq, Dv), np.float64)
    lib().oracle_sdpa(_ptr(qf), _ptr(kf), _ptr(vf), _ptr(m), _ptr(o),
                      *(ctypes.c_int64(t) for t in (B, Hq, Hkv, Sq, Skv, D, Dv)),
                      ctypes.c_int(1 if is_causal else 0), ctypes.c_double(scale))
    return o


def rmsnorm(x: np.ndarray, scale: Optional[np.ndarray], eps: float) -> np.ndarray:
    """aten.rms_norm over all dims but dim 0 (asm_emitter.h:1592-1626).
    ``scale`` has x's dims with dim 0 = 1.  Pinned by: the reference's
    two-value closed form (samples/rmsnorm/rmsnorm_utils.h:26-66), rms(y) = 1
    invariant, torch F.rms_norm."""
    rows = x.shape[0]
    inner = int(np.prod(x.shape[1:]))
    xf = np.ascontiguousarray(x, np.float32)
    sf = None if scale is None else np.ascontiguousarray(scale, np.float32).reshape(-1)
    assert sf is None or sf.size == inner
    y = np.empty(x.shape, np.float64)
    lib().oracle_rmsnorm(_ptr(xf), _ptr(sf), ctypes.c_double(eps), _ptr(y),
                         ctypes.c_int64(rows), ctypes.c_int64(inner))
    return y


def layernorm(x, scale, bias, eps):
    """aten.native_layer_norm over all dims but dim 0 (asm_emitter.h:1427-1503).
    Returns (y, mean, rstd) with mean/rstd of shape [B,1,...,1].  Pinned by:
    the reference's two-value closed form (samples/layernorm/
    layernorm_utils.h:25-82), torch F.layer_norm / native_layer_norm."""
    rows = x.shape[0]
    inner = int(np.prod(x.shape[1:]))
    xf = np.ascontiguousarray(x, np.float32)
    sf = None if scale is None else np.ascontiguousarray(scale, np.float32).reshape(-1)
    bf = None if bias is None else np.ascontiguousarray(bias, np.float32).reshape(-1)
    y = np.empty(x.shape, np.float64)
    mean = np.empty(rows, np.float64)
    rstd = np.empty(rows, np.float64)
    lib().oracle_layernorm(_ptr(xf), _ptr(sf), _ptr(bf), ctypes.c_double(eps),
                           _ptr(y), _ptr(mean), _ptr(rstd),
                           ctypes.c_int64(rows), ctypes.c_int64(inner))
    stat_shape = (rows,) + (1,) * (x.ndim - 1)
    return y, mean.reshape(stat_shape), rstd.reshape(stat_shape)


# Reduction modes (attributes/reduction_attributes.h:27-38).
RED_ADD, RED_SUM, RED_MUL, RED_MIN, RED_MAX, RED_AMAX, RED_AVG, RED_NORM1, \
    RED_NORM2, RED_MUL_NO_ZEROS = range(1, 11)


def batchnorm(x, scale, bias, running_mean, running_var, eps, training):
    """aten.native_batch_norm (asm_emitter.h:1066-1290, node/batchnorm_node.h):
    statistics per channel (dim 1) over batch and space.  Inference uses the
    running mean / variance; training the batch mean and BIASED variance, and
    also returns (mean, 1 / sqrt(var + eps)).  Returns (y, saved_mean,
    saved_inv_variance); the last two are None for inference.
    Pinned by: the reference samples' answers (samples/batchnorm/
    batchnorm_utils.h:22-107: x = c + 1 under mean 0 / var 1; a +-1 half / half
    pattern => mean 0, inv_variance 1/sqrt(1 + eps)), torch.native_batch_norm
    in float64, and the invariants mean_c(y) = bias, var_c(y) =
    scale^2 var / (var + eps)."""
    x = np.asarray(x, np.float32).astype(np.float64)
    c = x.shape[1]
    shape = [1, c] + [1] * (x.ndim - 2)
    axes = tuple(i for i in range(x.ndim) if i != 1)
    if training:
        mean = x.mean(axis=axes)
        var = ((x - mean.reshape(shape)) ** 2).mean(axis=axes)
    else:
        mean = np.asarray(running_mean, np.float32).astype(np.float64)
        var = np.asarray(running_var, np.float32).astype(np.float64)
    inv = 1.0 / np.sqrt(var + float(eps))
    y = (x - mean.reshape(shape)) * inv.reshape(shape)
    if scale is not None:
        y = y * np.asarray(scale, np.float32).astype(np.float64).reshape(shape)
    if bias is not None:
        y = y + np.asarray(bias, np.float32).astype(np.float64).reshape(shape)
    return (y, mean, inv) if training else (y, None, None)


def reduction(x: np.ndarray, out_dims, mode: int) -> np.ndarray:
    """Keep-dim reductions over dims where out == 1 < x
    (node/reduction_node.h:47-56; asm_emitter.h:2165-2322).  Pinned by the
    reference's table of known answers (samples/reduction/
    reduction_ops.cpp:150-217) and brute-force loops on tiny inputs."""
    axes = tuple(i for i, (xd, yd) in enumerate(zip(x.shape, out_dims))
                 if yd == 1 and xd > 1)
    v = x.astype(np.float64) if not np.issubdtype(x.dtype, np.integer) \
        else x.astype(np.int64)
    if mode in (RED_ADD, RED_SUM):
        r = v.sum(axis=axes, keepdims=True)
    elif mode == RED_MUL:
        r = v.prod(axis=axes, keepdims=True)
    elif mode == RED_MIN:
        r = v.min(axis=axes, keepdims=True)
    elif mode == RED_MAX:
        r = v.max(axis=axes, keepdims=True)
    elif mode == RED_AMAX:
        r = np.abs(v).max(axis=axes, keepdims=True)
    elif mode == RED_AVG:
        r = v.astype(np.float64).mean(axis=axes, keepdims=True)
    elif mode == RED_NORM1:
        r = np.abs(v).sum(axis=axes, keepdims=True)
    elif mode == RED_NORM2:
        r = np.sqrt((v.astype(np.float64) ** 2).sum(axis=axes, keepdims=True))
    elif mode == RED_MUL_NO_ZEROS:
        r = np.where(v == 0, 1, v).prod(axis=axes, keepdims=True)
    else:
        raise ValueError(mode)
    return r.reshape(tuple(out_dims))


# Pointwise modes (attributes/pointwise_attributes.h:27-74, NOT_SET = 0).
PW_NAMES = [
    "NOT_SET", "ABS", "ADD", "ADD_SQUARE", "BINARY_SELECT", "CEIL", "CMP_EQ",
    "CMP_GE", "CMP_GT", "CMP_LE", "CMP_LT", "CMP_NEQ", "DIV", "ELU_FWD", "ERF",
    "EXP", "FLOOR", "GELU_APPROX_TANH_BWD", "GELU_APPROX_TANH_FWD", "GELU_BWD",
    "GELU_FWD", "IDENTITY", "LOG", "LOGICAL_AND", "LOGICAL_NOT", "LOGICAL_OR",
    "MAX_OP", "MIN_OP", "MUL", "NEG", "RECIPROCAL", "RELU_BWD", "RELU_FWD",
    "RSQRT", "SIGMOID_FWD", "SIN", "SOFTPLUS_FWD", "SQRT", "SUB", "SWISH_BWD",
    "SWISH_FWD", "TAN", "TANH_BWD", "TANH_FWD",
]
PW = {name: i for i, name in enumerate(PW_NAMES)}


def _erf(x):
    from scipy.special import erf
    return erf(x)


def pointwise(mode: int, ins, elu_alpha=1.0, softplus_beta=1.0,
              softplus_threshold=20.0, swish_beta=1.0) -> np.ndarray:
    """Elementwise ops with right-aligned broadcasting (node/pointwise_node.h:
    108-168; formulas: asm_emitter.h:1806-2122 choose the aten op; the
    reference's samples/pointwise/pointwise_unary_ops.cpp:171-281 hold the
    matching std:: formulas).  Float math in f64; compare/logical results are
    0/1.  Pinned by the reference samples' formulas on their inputs and by
    torch elementwise ops."""
    name = PW_NAMES[mode]
    a = [np.asarray(t, np.float64) for t in ins]
    x = a[0]
    sig = lambda t: 1.0 / (1.0 + np.exp(-t))
    with np.errstate(all="ignore"):
        if name == "ABS":
            return np.abs(x)
        if name == "ADD":
            return x + a[1]
        if name == "ADD_SQUARE":
            return x + a[1] * a[1]
        if name == "BINARY_SELECT":
            return np.where(x != 0, a[1], a[2])
        if name == "CEIL":
            return np.ceil(x)
        if name == "CMP_EQ":
            return (x == a[1]).astype(np.float64)
        if name == "CMP_GE":
            return (x >= a[1]).astype(np.float64)
        if name == "CMP_GT":
            return (x > a[1]).astype(np.float64)
        if name == "CMP_LE":
            return (x <= a[1]).astype(np.float64)
        if name == "CMP_LT":
            return (x < a[1]).astype(np.float64)
        if name == "CMP_NEQ":
            return (x != a[1]).astype(np.float64)
        if name == "DIV":
            return x / a[1]
        if name == "ELU_FWD":
            return np.where(x > 0, x, elu_alpha * (np.exp(x) - 1.0))
        if name == "ERF":
            return _erf(x)
        if name == "EXP":
            return np.exp(x)
        if name == "FLOOR":
            return np.floor(x)
        if name == "GELU_FWD":
            return 0.5 * x * (1.0 + _erf(x / math.sqrt(2.0)))
        if name == "GELU_APPROX_TANH_FWD":
            return 0.5 * x * (1.0 + np.tanh(math.sqrt(2.0 / math.pi)
                                            * (x + 0.044715 * x ** 3)))
        if name == "GELU_BWD":
            g, t = x, a[1]
            cdf = 0.5 * (1.0 + _erf(t / math.sqrt(2.0)))
            pdf = np.exp(-0.5 * t * t) / math.sqrt(2.0 * math.pi)
            return g * (cdf + t * pdf)
        if name == "GELU_APPROX_TANH_BWD":
            g, t = x, a[1]
            kk = math.sqrt(2.0 / math.pi)
            inner = kk * (t + 0.044715 * t ** 3)
            th = np.tanh(inner)
            dinner = kk * (1.0 + 3 * 0.044715 * t * t)
            return g * (0.5 * (1 + th) + 0.5 * t * (1 - th * th) * dinner)
        if name == "IDENTITY":
            return x
        if name == "LOG":
            return np.log(x)
        if name == "LOGICAL_AND":
            return ((x != 0) & (a[1] != 0)).astype(np.float64)
        if name == "LOGICAL_NOT":
            return (x == 0).astype(np.float64)
        if name == "LOGICAL_OR":
            return ((x != 0) | (a[1] != 0)).astype(np.float64)
        if name == "MAX_OP":
            return np.maximum(x, a[1])
        if name == "MIN_OP":
            return np.minimum(x, a[1])
        if name == "MUL":
            return x * a[1]
        if name == "NEG":
            return -x
        if name == "RECIPROCAL":
            return 1.0 / x
        if name == "RELU_BWD":
            return np.where(a[1] > 0, x, 0.0)
        if name == "RELU_FWD":
            return np.maximum(x, 0.0)
        if name == "RSQRT":
            return 1.0 / np.sqrt(x)
        if name == "SIGMOID_FWD":
            return sig(x)
        if name == "SIN":
            return np.sin(x)
        if name == "SOFTPLUS_FWD":
            bx = x * softplus_beta
            return np.where(bx > softplus_threshold, x,
                            np.log1p(np.exp(bx)) / softplus_beta)
        if name == "SQRT":
            return np.sqrt(x)
        if name == "SUB":
            return x - a[1]
        if name == "SWISH_FWD":
            return x * sig(swish_beta * x)
        if name == "SWISH_BWD":
            g, t = x, a[1]
            s = sig(swish_beta * t)
            return g * (s + swish_beta * t * s * (1 - s))
        if name == "TAN":
            return np.tan(x)
        if name == "TANH_FWD":
            return np.tanh(x)
        if name == "TANH_BWD":
            y = np.tanh(a[1])
            return x * (1 - y * y)
    raise ValueError(name)


def rmsnorm_bf16_baseline(x_bits: np.ndarray, scale_bits: np.ndarray,
                          eps: float, mul: float) -> np.ndarray:
    """bf16 in / f32 accumulate / bf16 out RMSNorm * scalar on all host cores;
    the timed CPU-baseline body of the bandwidth benchmark."""
    rows, inner = x_bits.shape
    y = np.empty_like(x_bits)
    lib().oracle_rmsnorm_bf16_baseline(
        _ptr(x_bits), _ptr(scale_bits), ctypes.c_float(eps),
        ctypes.c_float(mul), _ptr(y), ctypes.c_int64(rows),
        ctypes.c_int64(inner))
    return y


def check_close(got: np.ndarray, ref: np.ndarray, rtol: float):
    """north-star criterion: |got - ref| <= rtol*|ref| + rtol*rms(ref).
    Returns (ok, report dict)."""
    g = np.asarray(got, np.float64)
    r = np.asarray(ref, np.float64)
    finite = np.isfinite(r)
    rms = float(np.sqrt(np.mean(r[finite] ** 2))) if finite.any() else 0.0
    err = np.abs(g - r)
    bound = rtol * np.abs(r) + rtol * rms
    same_nonfinite = (~finite) & ((g == r) | (np.isnan(g) & np.isnan(r)))
    bad = ~(same_nonfinite | (finite & (err <= bound)))
    rep = {
        "max_abs": float(np.nanmax(np.where(finite, err, 0.0))) if g.size else 0.0,
        "rms_ref": rms,
        "violations": int(bad.sum()),
        "count": int(g.size),
    }
    return not bad.any(), rep
