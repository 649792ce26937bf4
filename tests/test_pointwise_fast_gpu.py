"""Vector pointwise kernel (dense f32 / bf16 / f16 outputs; inputs of the same
dtype: dense, scalar, row-broadcast or column-broadcast) through the C ABI vs the oracle;
every case asserts that the tuned kernel is the one chosen."""
import numpy as np
import pytest

from fusilli_amd import capi
from oracle import oracle
from helpers import HT, assert_close, rand

pytestmark = pytest.mark.gpu

UNARY = ["ABS", "CEIL", "ELU_FWD", "ERF", "EXP", "FLOOR", "GELU_APPROX_TANH_FWD",
         "GELU_FWD", "IDENTITY", "LOG", "NEG", "RECIPROCAL", "RELU_FWD", "RSQRT",
         "SIGMOID_FWD", "SIN", "SOFTPLUS_FWD", "SQRT", "SWISH_FWD", "TAN",
         "TANH_FWD"]
BINARY = ["ADD", "ADD_SQUARE", "DIV", "MAX_OP", "MIN_OP", "MUL", "SUB",
          "RELU_BWD", "TANH_BWD", "GELU_BWD", "GELU_APPROX_TANH_BWD",
          "SWISH_BWD"]
RTOL = {capi.FLOAT: 1e-4, capi.HALF: 2e-2, capi.BFLOAT16: 2e-2}


def run(ctx, mode, ins, out_dtype, params=None, scalars=None, expect_tuned=True):
    scalars = scalars or {}
    shapes = [tuple(t.dims) for t in ins if t is not None]
    odims = list(np.broadcast_shapes(*shapes))
    out = HT.empty(odims, out_dtype)
    d = capi.PointwiseDesc()
    d.mode = capi.PW[mode]
    d.num_inputs = len(ins)
    d.params = params or capi.PointwiseParams.default()
    bufs = []
    for i, t in enumerate(ins):
        if t is None:
            d.in_is_scalar[i] = 1
            d.in_scalar[i] = scalars[i]
            bufs.append(None)
        else:
            d.in_[i] = t.desc()
            bufs.append(t.upload(ctx))
    d.out = out.desc()
    assert ctx.lib.fhip_pointwise_supported(d) == (2 if expect_tuned else 1)
    bufs += [None] * (3 - len(bufs))
    dout = out.upload(ctx)
    ctx.pointwise(d, bufs[0], bufs[1], bufs[2], dout)
    return out.fetch(ctx, dout)


@pytest.mark.parametrize("mode", UNARY)
@pytest.mark.parametrize("dtype", [capi.FLOAT, capi.HALF, capi.BFLOAT16])
def test_unary_vs_oracle(ctx, mode, dtype):
    vals = rand(71, 0, [24, 40], "uniform", lo=-3.0, hi=3.0)
    if mode in ("LOG", "RSQRT", "SQRT"):
        vals = np.abs(vals) + 0.1
    if mode in ("RECIPROCAL", "TAN"):
        vals = np.where(np.abs(vals) < 0.2, 0.7, vals) * (0.4 if mode == "TAN" else 1)
    x = HT.from_logical(vals, dtype)
    params = capi.PointwiseParams(1.5, 2.0, 3.0, 0.75)
    out = run(ctx, mode, [x], dtype, params=params)
    ref = oracle.pointwise(capi.PW[mode], [x.logical()], elu_alpha=1.5,
                           softplus_beta=2.0, softplus_threshold=3.0,
                           swish_beta=0.75)
    assert_close(out.logical(), ref, dtype, mode, rtol=RTOL[dtype])


@pytest.mark.parametrize("mode", BINARY)
@pytest.mark.parametrize("bdims", [[6, 5, 16], [16], [5, 16], [6, 1, 1], [6, 5, 1]],
                         ids=["full", "row1", "row2", "col1", "col2"])
@pytest.mark.parametrize("dtype", [capi.FLOAT, capi.BFLOAT16, capi.HALF])
def test_binary_broadcast_kinds_vs_oracle(ctx, mode, bdims, dtype):
    a = HT.from_logical(np.round(rand(72, 0, [6, 5, 16], "uniform", lo=-2, hi=2), 1),
                        dtype)
    b = HT.from_logical(np.round(rand(72, 1, bdims, "uniform", lo=-2, hi=2), 1) + 0.05,
                        dtype)
    out = run(ctx, mode, [a, b], dtype)
    ref = oracle.pointwise(capi.PW[mode], [a.logical(), b.logical()])
    assert_close(out.logical(), ref, dtype, mode, rtol=RTOL[dtype])
    # operands swapped: the broadcast input comes first
    out = run(ctx, mode, [b, a], dtype)
    ref = oracle.pointwise(capi.PW[mode], [b.logical(), a.logical()])
    assert_close(out.logical(), ref, dtype, mode + " swapped", rtol=RTOL[dtype])


@pytest.mark.parametrize("mode", ["ADD", "MUL", "SUB", "DIV", "MAX_OP"])
@pytest.mark.parametrize("which", [0, 1])
def test_binary_scalar_operand(ctx, mode, which):
    a = HT.from_logical(rand(73, 0, [8, 128]), capi.BFLOAT16)
    ins = [a, None] if which == 1 else [None, a]
    out = run(ctx, mode, ins, capi.BFLOAT16, scalars={which: 0.375})
    vals = [a.logical(), np.float32(0.375)]
    if which == 0:
        vals = vals[::-1]
    ref = oracle.pointwise(capi.PW[mode], vals)
    assert_close(out.logical(), np.broadcast_to(ref, out.logical().shape),
                 capi.BFLOAT16, mode)


@pytest.mark.parametrize("adt,bdt,odt", [
    (capi.BFLOAT16, capi.FLOAT, capi.FLOAT),
    (capi.HALF, capi.BFLOAT16, capi.BFLOAT16),
    (capi.FLOAT, capi.FLOAT, capi.HALF),
])
def test_mixed_dtypes_stay_on_strided_kernel(ctx, adt, bdt, odt):
    a = HT.from_logical(rand(74, 0, [32, 72]), adt)
    b = HT.from_logical(rand(74, 1, [1, 72]), bdt)
    out = run(ctx, "ADD", [a, b], odt, expect_tuned=False)
    ref = oracle.pointwise(capi.PW["ADD"], [a.logical(), b.logical()])
    assert_close(out.logical(), ref, odt, "mixed add", rtol=RTOL[odt])


def test_select_three_inputs(ctx):
    cond = HT.from_logical((rand(75, 0, [16, 64]) > 0).astype(np.float32), capi.FLOAT)
    a = HT.from_logical(rand(75, 1, [16, 64]), capi.FLOAT)
    b = HT.from_logical(rand(75, 2, [64]), capi.FLOAT)
    out = run(ctx, "BINARY_SELECT", [cond, a, b], capi.FLOAT).logical()
    want = np.where(cond.logical() != 0, a.logical(), b.logical()[None, :])
    assert np.array_equal(out, want)


def test_large_grid_stride_and_tail(ctx):
    # more vectors than one sweep of the grid covers, and a vector count that
    # is no multiple of the workgroup size
    n = 8 * (256 * 8 * 256 * 4 + 777)
    vals = rand(76, 0, [n // 8, 8])
    a = HT.from_logical(vals, capi.BFLOAT16)
    out = run(ctx, "RELU_FWD", [a], capi.BFLOAT16).logical()
    assert np.array_equal(out, np.maximum(a.logical(), 0))


def test_fallbacks_keep_working(ctx):
    # ragged volume, mixed broadcast and strided inputs stay on the strided
    # kernel and still match the oracle
    a = HT.from_logical(rand(77, 0, [4, 37]), capi.FLOAT)
    out = run(ctx, "NEG", [a], capi.FLOAT, expect_tuned=False)
    assert np.array_equal(out.logical(), -a.logical())
    a = HT.from_logical(rand(77, 1, [3, 1, 8]), capi.FLOAT)
    b = HT.from_logical(rand(77, 2, [5, 8]), capi.FLOAT)
    out = run(ctx, "ADD", [a, b], capi.FLOAT, expect_tuned=False)
    assert_close(out.logical(), a.logical() + b.logical(), capi.FLOAT, "mixed broadcast")
    t = HT.from_logical(rand(77, 3, [8, 16]), capi.FLOAT, strides=[1, 8])
    out = run(ctx, "ABS", [t], capi.FLOAT, expect_tuned=False)
    assert np.array_equal(out.logical(), np.abs(t.logical()))
