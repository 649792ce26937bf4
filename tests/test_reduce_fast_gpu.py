"""Row-reduction kernel (trailing dims of a dense tensor) through the C ABI vs
the oracle; every case asserts that the tuned kernel is the one chosen."""
import numpy as np
import pytest

from fusilli_amd import capi
from oracle import oracle
from helpers import HT, assert_close, rand

pytestmark = pytest.mark.gpu

MODES = ["ADD", "SUM", "MUL", "MIN", "MAX", "AMAX", "AVG", "NORM1", "NORM2",
         "MUL_NO_ZEROS"]


def run(ctx, x, odims, mode, y_dtype=None, expect_tuned=True):
    y = HT.empty(odims, x.dtype if y_dtype is None else y_dtype)
    d = capi.ReduceDesc()
    d.x, d.y, d.mode = x.desc(), y.desc(), capi.RED[mode]
    assert ctx.lib.fhip_reduce_supported(d) == (2 if expect_tuned else 1)
    dx, dy = x.upload(ctx), y.upload(ctx)
    ctx.reduce(d, dx, dy)
    return y.fetch(ctx, dy)


def make_x(seed, dims, dtype, mode):
    if mode in ("MUL", "MUL_NO_ZEROS"):
        v = 1.0 + 0.02 * rand(seed, 0, dims)  # products stay in range
        if mode == "MUL_NO_ZEROS":
            v.reshape(-1)[::7] = 0.0
    else:
        v = rand(seed, 0, dims)
    return HT.from_logical(v, dtype)


@pytest.mark.parametrize("mode", MODES)
@pytest.mark.parametrize("dtype", [capi.FLOAT, capi.BFLOAT16, capi.HALF])
@pytest.mark.parametrize("dims,odims", [
    ([2, 16, 8, 8], [2, 16, 1, 1]),      # the reference sample's shape: 64-element rows
    ([37, 1000], [37, 1]),               # one wavefront per row, ragged chunk count
    ([5, 3, 4096], [5, 3, 1]),           # one workgroup per row
    ([3, 1, 6000, 8], [3, 1, 1, 1]),     # long rows, odd number of chunk pairs
])
def test_reduce_rows_vs_oracle(ctx, mode, dtype, dims, odims):
    x = make_x(61, dims, dtype, mode)
    out = run(ctx, x, odims, mode, y_dtype=capi.FLOAT)
    ref = oracle.reduction(x.logical(), odims, capi.RED[mode])
    rtol = 1e-4 if dtype == capi.FLOAT else 2e-2
    assert_close(out.logical(), ref, capi.FLOAT, f"{mode} {dims}", rtol=rtol)


def test_reduce_reference_table_known_answers(ctx):
    # samples/reduction/reduction_ops.cpp: inputs i % 100 - 50 on [2,16,8,8]
    dims, odims = [2, 16, 8, 8], [2, 16, 1, 1]
    vals = (np.arange(int(np.prod(dims))) % 100 - 50).astype(np.float64).reshape(dims)
    x = HT.from_logical(vals, capi.FLOAT)
    g = vals.reshape(2, 16, 64)
    assert np.array_equal(run(ctx, x, odims, "SUM").logical().reshape(2, 16), g.sum(2))
    assert np.array_equal(run(ctx, x, odims, "MIN").logical().reshape(2, 16), g.min(2))
    assert np.array_equal(run(ctx, x, odims, "AMAX").logical().reshape(2, 16), np.abs(g).max(2))
    assert np.array_equal(run(ctx, x, odims, "NORM1").logical().reshape(2, 16), np.abs(g).sum(2))


def test_reduce_output_rounding_and_bf16_store(ctx):
    x = make_x(62, [64, 512], capi.BFLOAT16, "SUM")
    out = run(ctx, x, [64, 1], "SUM")  # bf16 result
    ref = oracle.reduction(x.logical(), [64, 1], capi.RED["SUM"])
    assert_close(out.logical(), ref, capi.BFLOAT16)


def test_reduce_not_chosen_outside_contract(ctx):
    # leading-dim reduction and int32 input keep the generic kernel
    x = make_x(63, [16, 64], capi.FLOAT, "SUM")
    out = run(ctx, x, [1, 64], "SUM", expect_tuned=False)
    assert_close(out.logical(), oracle.reduction(x.logical(), [1, 64], capi.RED["SUM"]),
                 capi.FLOAT)
    xi = HT.from_logical(np.arange(128).reshape(2, 64) - 60, capi.INT32)
    out = run(ctx, xi, [2, 1], "MAX", expect_tuned=False)
    assert np.array_equal(out.logical().reshape(-1), [3, 67])


def test_reduce_headline_size(ctx):
    # [8192, 4096] bf16 row sums and row maxima of |x| at full size
    x = make_x(64, [8192, 4096], capi.BFLOAT16, "SUM")
    xl = x.logical()
    out = run(ctx, x, [8192, 1], "SUM", y_dtype=capi.FLOAT).logical()
    assert_close(out, xl.sum(1, keepdims=True), capi.FLOAT, rtol=1e-4)
    out = run(ctx, x, [8192, 1], "AMAX", y_dtype=capi.FLOAT).logical()
    assert np.array_equal(out, np.abs(xl).max(1, keepdims=True))


@pytest.mark.parametrize("dtype", [capi.FLOAT, capi.BFLOAT16, capi.HALF])
@pytest.mark.parametrize("mode", ["MIN", "MAX", "AMAX"])
def test_reduce_min_max_propagate_nan_and_inf(ctx, mode, dtype):
    # aten.amin / amax semantics: a NaN anywhere in the row gives NaN; an
    # infinity is an ordinary extreme value
    v = rand(65, 0, [6, 640])
    v[1, 17] = np.nan
    v[2, 600] = -np.inf
    v[3, 5] = np.inf
    out = run(ctx, HT.from_logical(v, dtype), [6, 1], mode, y_dtype=capi.FLOAT).logical().reshape(-1)
    assert np.isnan(out[1]) and not np.isnan(out[[0, 2, 3, 4, 5]]).any()
    assert out[2] == (-np.inf if mode == "MIN" else np.inf if mode == "AMAX" else out[2])
    assert out[3] == (np.inf if mode in ("MAX", "AMAX") else out[3])
