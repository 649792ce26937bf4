"""Pins the CPU oracle (test infrastructure) before it is trusted as the
checker of the HIP kernels.

Each oracle function is checked against (a) the known answers the reference's
own samples and tests state, (b) closed forms and invariants, and (c) an
independent library routine (torch CPU in float64, numpy) on random inputs
chosen so that a dropped term, a wrong sign or index, or a transposed operand
fails.  Nothing here touches the GPU.
"""
import json
import math
import os

import numpy as np
import pytest
import torch
import torch.nn.functional as F

from fusilli_amd import capi, synth
from oracle import oracle

RNG = np.random.default_rng(1234)


def t64(a):
    return torch.from_numpy(np.ascontiguousarray(a, dtype=np.float64))


# ---- element conversions ----------------------------------------------------
@pytest.mark.parametrize("dtype,tdt", [
    (capi.BFLOAT16, torch.bfloat16), (capi.HALF, torch.float16),
    (capi.FP8E4M3, torch.float8_e4m3fn), (capi.FP8E5M2, torch.float8_e5m2)])
def test_quantize_round_trip_matches_torch(dtype, tdt):
    vals = np.concatenate([
        RNG.normal(0, 1, 4000), RNG.normal(0, 300, 2000), RNG.normal(0, 1e-3, 2000),
        np.array([0.0, -0.0, 1.0, -1.0, 0.5, 448.0, 57344.0, 65504.0, 3.0e38,
                  2.0 ** -9, 2.0 ** -10, 2.0 ** -16, 2.0 ** -17, 2.0 ** -24,
                  1.0 + 2.0 ** -8, 1.0 + 2.0 ** -9, 1.0 + 3 * 2.0 ** -9,
                  1.0625, 1.1875, 0.0009765625 * 1.5])]).astype(np.float32)
    if dtype in (capi.FP8E4M3, capi.FP8E5M2):
        lim = 448.0 if dtype == capi.FP8E4M3 else 57344.0
        vals = vals[np.abs(vals) <= lim]  # saturation is checked separately
    if dtype == capi.HALF:
        vals = vals[np.abs(vals) <= 65504.0]
    got = oracle.dequantize(oracle.quantize(vals, dtype), dtype)
    ref = torch.from_numpy(vals).to(tdt).to(torch.float32).numpy()
    assert np.array_equal(got.astype(np.float32), ref)


@pytest.mark.parametrize("dtype,tdt", [(capi.FP8E4M3, torch.float8_e4m3fn),
                                       (capi.FP8E5M2, torch.float8_e5m2)])
def test_fp8_decode_table_is_exhaustively_torchs(dtype, tdt):
    bits = np.arange(256, dtype=np.uint8)
    got = oracle.dequantize(bits, dtype).astype(np.float32)
    ref = torch.from_numpy(bits).view(tdt).to(torch.float32).numpy()
    ok = (got == ref) | (np.isnan(got) & np.isnan(ref))
    assert ok.all()


def test_fp8_and_int_saturate():
    assert oracle.dequantize(oracle.quantize(np.array([1e6, -1e6], np.float32),
                                             capi.FP8E4M3), capi.FP8E4M3).tolist() == [448.0, -448.0]
    assert oracle.dequantize(oracle.quantize(np.array([300.0, -300.0, 2.5, 3.5]),
                                             capi.INT8), capi.INT8).tolist() == [127, -128, 2, 4]


def test_synth_conversions_agree_with_oracle():
    v = RNG.normal(0, 2, 5000).astype(np.float32)
    assert np.array_equal(synth.f32_to_bf16_bits(v), oracle.quantize(v, capi.BFLOAT16))
    assert np.array_equal(synth.f32_to_fp8_bits(v, 4), oracle.quantize(v, capi.FP8E4M3))


# ---- layout -------------------------------------------------------------------
def test_layout_helpers_against_reference_vectors():
    # tests/golden/layout_vectors.json transcribes the expectations of the
    # reference's tests/test_tensor_attributes.cpp; contiguous and channels-last
    # strides must be among its valid (dim, stride) pairs.
    path = os.path.join(os.path.dirname(__file__), "golden", "layout_vectors.json")
    vec = json.load(open(path))
    for rec in vec["physical_dim"]:
        dims, strides = rec["dim"], rec["stride"]
        if min(dims) == 1:
            continue  # unit dims make the stride order ambiguous
        if strides == oracle.contiguous_strides(dims):
            assert rec["expect"] == dims
        if len(dims) >= 3 and strides == oracle.channels_last_strides(dims):
            assert rec["expect"] == [dims[0]] + dims[2:] + [dims[1]]
    assert oracle.contiguous_strides([2, 3, 4, 5]) == [60, 20, 5, 1]
    assert oracle.channels_last_strides([2, 3, 4, 5]) == [60, 1, 15, 3]
    x = RNG.normal(size=[2, 3, 4, 5])
    st = oracle.channels_last_strides(x.shape)
    flat = oracle.to_storage(x, st)
    assert np.array_equal(flat.reshape(2, 4, 5, 3), x.transpose(0, 2, 3, 1))
    assert np.array_equal(oracle.logical_view(flat, x.shape, st), x)


# ---- matmul ---------------------------------------------------------------------
def test_matmul_known_answers_and_torch():
    # samples/matmul: all-ones [M,K] x [K,N] => K
    assert np.all(oracle.matmul(np.ones([16, 64]), np.ones([64, 32])) == 64.0)
    a, b = RNG.normal(size=[3, 17, 29]), RNG.normal(size=[1, 29, 13])
    ref = torch.matmul(t64(a), t64(b)).numpy()
    assert np.allclose(oracle.matmul(a.astype(np.float32), b.astype(np.float32)),
                       np.matmul(a.astype(np.float32).astype(np.float64),
                                 b.astype(np.float32).astype(np.float64)), rtol=1e-12)
    assert np.allclose(oracle.matmul(a, b), ref, rtol=1e-5, atol=1e-5)
    # a transposed operand must fail: A is not symmetric
    assert not np.allclose(oracle.matmul(a[0, :17, :17], a[0, :17, :17]),
                           (t64(a[0, :17, :17]).T @ t64(a[0, :17, :17])).numpy())


def test_matmul_int8_is_exact():
    a = RNG.integers(-128, 128, [37, 300]).astype(np.int8)
    b = RNG.integers(-128, 128, [300, 21]).astype(np.int8)
    got = oracle.matmul(a, b)
    assert np.array_equal(got, a.astype(np.int64) @ b.astype(np.int64))
    rows = np.array([0, 5, 36])
    assert np.array_equal(oracle.matmul_rows(a, b, rows), got[rows])


# ---- convolution ----------------------------------------------------------------
def test_conv_known_answers():
    # samples/convolution: all-ones 1x1 => C; 3x3 same-pad corner => 4*C
    x, w = np.ones([4, 128, 8, 8]), np.ones([32, 128, 1, 1])
    assert np.all(oracle.conv_fprop(x, w, [0, 0], [1, 1], [1, 1]) == 128.0)
    y = oracle.conv_fprop(np.ones([2, 16, 8, 8]), np.ones([4, 16, 3, 3]),
                          [1, 1], [1, 1], [1, 1])
    assert y[0, 0, 0, 0] == 64.0 and y[0, 0, 0, 3] == 96.0 and y[1, 3, 4, 4] == 144.0
    # grouped: fC * R * S
    y = oracle.conv_fprop(np.ones([1, 16, 6, 6]), np.ones([8, 4, 3, 3]),
                          [0, 0], [1, 1], [1, 1])
    assert np.all(y == 36.0)
    # a delta filter is a shifted copy
    xs = RNG.normal(size=[1, 1, 5, 7])
    w = np.zeros([1, 1, 3, 3]); w[0, 0, 0, 2] = 1.0
    y = oracle.conv_fprop(xs, w, [1, 1], [1, 1], [1, 1])
    assert np.allclose(y[0, 0, 1:, :-1], xs[0, 0, :-1, 1:].astype(np.float32))


@pytest.mark.parametrize("case", [
    dict(x=[2, 6, 9, 11], w=[4, 6, 3, 3], pad=[1, 1], s=[1, 1], d=[1, 1]),
    dict(x=[2, 6, 9, 11], w=[4, 3, 3, 2], pad=[0, 1], s=[2, 1], d=[1, 2]),
    dict(x=[1, 8, 13], w=[8, 2, 4], pad=[2], s=[3], d=[2]),
    dict(x=[1, 4, 5, 6, 7], w=[2, 4, 2, 3, 3], pad=[1, 0, 1], s=[1, 2, 1], d=[1, 1, 1]),
])
def test_conv_matches_torch(case):
    x = RNG.normal(size=case["x"]).astype(np.float32)
    w = RNG.normal(size=case["w"]).astype(np.float32)
    groups = case["x"][1] // case["w"][1]
    fn = {1: F.conv1d, 2: F.conv2d, 3: F.conv3d}[len(case["pad"])]
    ref = fn(t64(x), t64(w), None, case["s"], case["pad"], case["d"], groups).numpy()
    got = oracle.conv_fprop(x, w, case["pad"], case["s"], case["d"])
    assert got.shape == ref.shape
    assert np.allclose(got, ref, rtol=1e-9, atol=1e-9)


def test_conv_backward_known_answers():
    # samples/convolution/conv_dgrad_nhwc_krsc.cpp:98: all-ones 1x1 => K
    dy, w = np.ones([4, 16, 8, 8]), np.ones([16, 8, 1, 1])
    assert np.all(oracle.conv_dgrad(dy, w, [4, 8, 8, 8], [0, 0], [1, 1], [1, 1]) == 16.0)
    # conv_dgrad_nhwc_krsc_grouped.cpp:99: grouped => K / groups
    dy, w = np.ones([4, 32, 8, 8]), np.ones([32, 4, 1, 1])
    assert np.all(oracle.conv_dgrad(dy, w, [4, 16, 8, 8], [0, 0], [1, 1], [1, 1]) == 8.0)
    # conv_wgrad_nhwc_krsc.cpp:99: all-ones 1x1 => N*H*W
    dy, x = np.ones([4, 16, 8, 8]), np.ones([4, 8, 8, 8])
    assert np.all(oracle.conv_wgrad(dy, x, [16, 8, 1, 1], [0, 0], [1, 1], [1, 1]) == 256.0)
    # conv_wgrad_nhwc_krsc_grouped.cpp:99 and ..._grouped_strided.cpp:103
    dy, x = np.ones([4, 32, 8, 8]), np.ones([4, 16, 8, 8])
    assert np.all(oracle.conv_wgrad(dy, x, [32, 4, 1, 1], [0, 0], [1, 1], [1, 1]) == 256.0)
    dy = np.ones([4, 32, 4, 4])
    assert np.all(oracle.conv_wgrad(dy, x, [32, 4, 1, 1], [0, 0], [2, 2], [1, 1]) == 64.0)
    # a delta gradient picks one filter-shaped window of X (wgrad) and writes
    # one filter-shaped stamp of W into DX (dgrad), at stride * o - pad
    x = RNG.normal(size=[1, 1, 7, 9]).astype(np.float32)
    w = RNG.normal(size=[1, 1, 3, 2]).astype(np.float32)
    od = oracle.conv_output_dims(x.shape, w.shape, [1, 0], [2, 1], [1, 1])
    dy = np.zeros(od); dy[0, 0, 2, 3] = 1.0
    dw = oracle.conv_wgrad(dy, x, w.shape, [1, 0], [2, 1], [1, 1])
    assert np.array_equal(dw[0, 0], x[0, 0, 3:6, 3:5].astype(np.float64))
    dx = oracle.conv_dgrad(dy, w, x.shape, [1, 0], [2, 1], [1, 1])
    want = np.zeros([7, 9]); want[3:6, 3:5] = w[0, 0]
    assert np.array_equal(dx[0, 0], want)


@pytest.mark.parametrize("case", [
    dict(x=[2, 6, 9, 11], w=[4, 6, 3, 3], pad=[1, 1], s=[1, 1], d=[1, 1]),
    dict(x=[2, 6, 9, 11], w=[4, 3, 3, 2], pad=[0, 1], s=[2, 1], d=[1, 2]),
    dict(x=[2, 6, 10, 11], w=[6, 2, 3, 3], pad=[1, 2], s=[3, 2], d=[1, 1]),
    dict(x=[1, 8, 13], w=[8, 2, 4], pad=[2], s=[3], d=[2]),
    dict(x=[1, 4, 5, 6, 7], w=[2, 4, 2, 3, 3], pad=[1, 0, 1], s=[1, 2, 1], d=[1, 1, 1]),
])
def test_conv_backward_matches_torch_autograd_and_adjoint(case):
    x = RNG.normal(size=case["x"]).astype(np.float32)
    w = RNG.normal(size=case["w"]).astype(np.float32)
    groups = case["x"][1] // case["w"][1]
    fn = {1: F.conv1d, 2: F.conv2d, 3: F.conv3d}[len(case["pad"])]
    tx, tw = t64(x).requires_grad_(True), t64(w).requires_grad_(True)
    y = fn(tx, tw, None, case["s"], case["pad"], case["d"], groups)
    dy = RNG.normal(size=list(y.shape)).astype(np.float32)
    y.backward(t64(dy))
    dx = oracle.conv_dgrad(dy, w, case["x"], case["pad"], case["s"], case["d"])
    dw = oracle.conv_wgrad(dy, x, case["w"], case["pad"], case["s"], case["d"])
    assert np.allclose(dx, tx.grad.numpy(), rtol=1e-9, atol=1e-9)
    assert np.allclose(dw, tw.grad.numpy(), rtol=1e-9, atol=1e-9)
    # adjoint identities against the (separately pinned) forward
    fwd = oracle.conv_fprop(x, w, case["pad"], case["s"], case["d"])
    lhs = float(np.sum(fwd * dy.astype(np.float64)))
    assert np.isclose(lhs, float(np.sum(dx * x.astype(np.float64))), rtol=1e-9)
    assert np.isclose(lhs, float(np.sum(dw * w.astype(np.float64))), rtol=1e-9)


# ---- batch norm -----------------------------------------------------------------
def test_batchnorm_known_answers():
    # samples/batchnorm/batchnorm_utils.h:22-47 (inference): x = c + 1, mean 0,
    # var 1 => scale * (c + 1) / sqrt(1 + eps) + bias
    n, c, h, w, eps = 2, 4, 8, 8, 1e-5
    x = np.broadcast_to(np.arange(1, c + 1, dtype=np.float64).reshape(1, c, 1, 1),
                        [n, c, h, w])
    y, m, v = oracle.batchnorm(x, None, None, np.zeros(c), np.ones(c), eps, False)
    assert m is None and v is None
    assert np.allclose(y, x / np.sqrt(1 + eps), rtol=1e-12)
    y, _, _ = oracle.batchnorm(x, np.full(c, 2.0), np.full(c, 0.5), np.zeros(c),
                               np.ones(c), eps, False)
    assert np.allclose(y, 2.0 * x / np.sqrt(1 + eps) + 0.5, rtol=1e-12)
    # batchnorm_utils.h:60-104 (training): -1 on the first half of (n, h, w),
    # +1 on the second => mean 0, biased var 1
    flat = np.where(np.arange(n * h * w) < n * h * w // 2, -1.0, 1.0)
    x = np.broadcast_to(flat.reshape(n, 1, h, w), [n, c, h, w])
    y, m, v = oracle.batchnorm(x, np.full(c, 2.0), np.full(c, 0.5), None, None,
                               eps, True)
    assert np.allclose(m, 0.0) and np.allclose(v, 1 / np.sqrt(1 + eps), rtol=1e-12)
    assert np.allclose(y, 2.0 * x / np.sqrt(1 + eps) + 0.5, rtol=1e-12)


@pytest.mark.parametrize("dims", [[3, 5, 7, 6], [4, 3, 9], [2, 6], [2, 3, 4, 5, 2]])
@pytest.mark.parametrize("training", [False, True])
@pytest.mark.parametrize("affine", [False, True])
def test_batchnorm_matches_torch_and_invariants(dims, training, affine):
    c, eps = dims[1], 1e-3
    x = (RNG.normal(size=dims) * 2 + 1).astype(np.float32)
    sc = RNG.normal(size=c).astype(np.float32) if affine else None
    b = RNG.normal(size=c).astype(np.float32) if affine else None
    rm = RNG.normal(size=c).astype(np.float32)
    rv = (RNG.uniform(size=c) + 0.5).astype(np.float32)
    ty, tm, tv = torch.native_batch_norm(
        t64(x), None if sc is None else t64(sc), None if b is None else t64(b),
        t64(rm), t64(rv), training, 0.1, eps)
    y, m, v = oracle.batchnorm(x, sc, b, rm, rv, eps, training)
    assert np.allclose(y, ty.numpy(), rtol=1e-9, atol=1e-9)
    if training:
        assert np.allclose(m, tm.numpy(), rtol=1e-9, atol=1e-12)
        assert np.allclose(v, tv.numpy(), rtol=1e-9)
        axes = tuple(i for i in range(len(dims)) if i != 1)
        var = x.astype(np.float64).var(axis=axes)
        s64 = np.ones(c) if sc is None else sc.astype(np.float64)
        b64 = np.zeros(c) if b is None else b.astype(np.float64)
        assert np.allclose(y.mean(axis=axes), b64, atol=1e-9)
        assert np.allclose(y.var(axis=axes), s64 ** 2 * var / (var + eps), rtol=1e-9)


# ---- attention ------------------------------------------------------------------
def torch_sdpa(q, k, v, mask=None, causal=False, scale=None):
    rep = q.shape[1] // k.shape[1]
    kt, vt = t64(k).repeat_interleave(rep, 1), t64(v).repeat_interleave(rep, 1)
    m = None
    if mask is not None:
        m = torch.from_numpy(mask) if mask.dtype == np.bool_ else t64(mask)
    return F.scaled_dot_product_attention(t64(q), kt, vt, attn_mask=m,
                                          is_causal=causal, scale=scale).numpy()


def test_sdpa_known_answers():
    # samples/sdpa: constant fill => V
    c = np.full([1, 8, 64, 64], 0.01)
    assert np.allclose(oracle.sdpa(c, c, c), 0.01)
    assert np.allclose(oracle.sdpa(c, c, c, is_causal=True), 0.01)
    # one key: O = V regardless of scores
    q, k, v = RNG.normal(size=[1, 2, 5, 8]), RNG.normal(size=[1, 2, 1, 8]), RNG.normal(size=[1, 2, 1, 6])
    assert np.allclose(oracle.sdpa(q, k, v), np.broadcast_to(v.astype(np.float32), [1, 2, 5, 6]))
    # uniform scores under a causal mask: prefix means
    v = RNG.normal(size=[1, 1, 9, 4])
    o = oracle.sdpa(np.zeros([1, 1, 9, 4]), RNG.normal(size=[1, 1, 9, 4]), v, is_causal=True)
    assert np.allclose(o[0, 0], np.cumsum(v[0, 0].astype(np.float32), 0) / np.arange(1, 10)[:, None])


@pytest.mark.parametrize("case", [
    dict(B=2, Hq=4, Hkv=4, Sq=7, Skv=7, D=8, Dv=8, causal=True),
    dict(B=1, Hq=6, Hkv=2, Sq=5, Skv=11, D=16, Dv=4, causal=False),
    dict(B=2, Hq=2, Hkv=1, Sq=6, Skv=9, D=8, Dv=8, causal=False, mask="float"),
    dict(B=1, Hq=2, Hkv=2, Sq=8, Skv=8, D=4, Dv=4, causal=False, mask="bool", scale=0.3),
])
def test_sdpa_matches_torch(case):
    c = case
    q = RNG.normal(size=[c["B"], c["Hq"], c["Sq"], c["D"]]).astype(np.float32)
    k = RNG.normal(size=[c["B"], c["Hkv"], c["Skv"], c["D"]]).astype(np.float32)
    v = RNG.normal(size=[c["B"], c["Hkv"], c["Skv"], c["Dv"]]).astype(np.float32)
    mask = None
    if c.get("mask") == "float":
        mask = RNG.normal(size=[c["B"], 1, c["Sq"], c["Skv"]]).astype(np.float32)
    elif c.get("mask") == "bool":
        mask = RNG.uniform(size=[1, 1, c["Sq"], c["Skv"]]) > 0.3
        mask[..., 0] = True
    got = oracle.sdpa(q, k, v, mask=mask, is_causal=c["causal"], scale=c.get("scale"))
    ref = torch_sdpa(q, k, v, mask, c["causal"], c.get("scale"))
    assert np.allclose(got, ref, rtol=1e-7, atol=1e-8)


# ---- norms ----------------------------------------------------------------------
def test_rmsnorm_closed_forms_and_torch():
    # constant row c: y = c / sqrt(c^2 + eps) * scale
    x = np.full([3, 16], 2.0)
    y = oracle.rmsnorm(x, np.full([1, 16], 1.5), 1e-5)
    assert np.allclose(y, 2.0 / math.sqrt(4.0 + 1e-5) * 1.5)
    # two-value rows (samples/rmsnorm/rmsnorm_utils.h): half +a, half -b
    x = np.tile(np.array([3.0, -1.0]), [4, 8])
    rms = math.sqrt((9.0 + 1.0) / 2 + 1e-5)
    assert np.allclose(oracle.rmsnorm(x, None, 1e-5), x / rms)
    xr = RNG.normal(size=[5, 3, 7]).astype(np.float32)
    sc = RNG.normal(size=[1, 3, 7]).astype(np.float32)
    ref = F.rms_norm(t64(xr), [3, 7], t64(sc[0]), 1e-6).numpy()
    assert np.allclose(oracle.rmsnorm(xr, sc, 1e-6), ref, rtol=1e-10, atol=1e-12)
    # invariant: rms(y) = 1 when eps -> 0 and no scale
    y = oracle.rmsnorm(xr, None, 0.0)
    assert np.allclose(np.sqrt((y.reshape(5, -1) ** 2).mean(1)), 1.0)


def test_layernorm_closed_forms_and_torch():
    # two-value rows (samples/layernorm/layernorm_utils.h): mean 1, var 4
    x = np.tile(np.array([3.0, -1.0]), [2, 6])
    y, mean, rstd = oracle.layernorm(x, None, None, 1e-5)
    assert np.allclose(mean, 1.0) and np.allclose(rstd, 1 / math.sqrt(4 + 1e-5))
    assert np.allclose(y, (x - 1.0) / math.sqrt(4 + 1e-5))
    xr = RNG.normal(2.0, 3.0, size=[4, 5, 6]).astype(np.float32)
    sc = RNG.normal(size=[1, 5, 6]).astype(np.float32)
    bi = RNG.normal(size=[1, 5, 6]).astype(np.float32)
    yt, mt, rt = torch.native_layer_norm(t64(xr), [5, 6], t64(sc[0]), t64(bi[0]), 1e-5)
    y, mean, rstd = oracle.layernorm(xr, sc, bi, 1e-5)
    assert np.allclose(y, yt.numpy(), rtol=1e-10, atol=1e-11)
    assert np.allclose(mean, mt.numpy()) and np.allclose(rstd, rt.numpy())
    assert mean.shape == (4, 1, 1)


# ---- reduction ------------------------------------------------------------------
def test_reduction_reference_table():
    # samples/reduction/reduction_ops.cpp:150-217 on [2,16,8,8] -> [2,16,1,1]
    dims, od = [2, 16, 8, 8], [2, 16, 1, 1]
    n = int(np.prod(dims))
    vals = (np.arange(n) % 100 - 50).astype(np.float64).reshape(dims)
    g = vals.reshape(2, 16, 64)
    R = capi.RED
    assert np.array_equal(oracle.reduction(vals, od, R["SUM"]).reshape(2, 16), g.sum(2))
    assert np.array_equal(oracle.reduction(vals, od, R["ADD"]).reshape(2, 16), g.sum(2))
    assert np.array_equal(oracle.reduction(vals, od, R["MIN"]).reshape(2, 16), g.min(2))
    assert np.array_equal(oracle.reduction(vals, od, R["MAX"]).reshape(2, 16), g.max(2))
    assert np.array_equal(oracle.reduction(vals, od, R["AMAX"]).reshape(2, 16), np.abs(g).max(2))
    assert np.allclose(oracle.reduction(vals, od, R["AVG"]).reshape(2, 16), g.mean(2))
    assert np.array_equal(oracle.reduction(vals, od, R["NORM1"]).reshape(2, 16), np.abs(g).sum(2))
    assert np.allclose(oracle.reduction(vals, od, R["NORM2"]).reshape(2, 16), np.sqrt((g * g).sum(2)))
    ones = np.ones(dims); ones.flat[0], ones.flat[1], ones.flat[2] = 2.0, 3.0, 0.0
    assert oracle.reduction(ones, od, R["MUL"]).flat[0] == 0.0
    assert oracle.reduction(ones, od, R["MUL_NO_ZEROS"]).flat[0] == 6.0
    # AMAX differs from MAX when the largest magnitude is negative
    neg = np.array([[-5.0, 2.0, 3.0]])
    assert oracle.reduction(neg, [1, 1], R["AMAX"]).item() == 5.0
    assert oracle.reduction(neg, [1, 1], R["MAX"]).item() == 3.0
    # reduced dims are exactly those where out == 1 < in
    x = RNG.normal(size=[3, 4, 5])
    assert np.allclose(oracle.reduction(x, [3, 1, 5], R["SUM"]), x.sum(1, keepdims=True))
    assert np.allclose(oracle.reduction(x, [1, 4, 1], R["SUM"]), x.sum((0, 2), keepdims=True))


# ---- pointwise ------------------------------------------------------------------
def test_pointwise_matches_torch():
    x = RNG.normal(0, 2, size=[64]).astype(np.float64)
    y = RNG.normal(0, 2, size=[64]).astype(np.float64)
    tx, ty = t64(x), t64(y)
    P = capi.PW
    checks = {
        "ABS": torch.abs(tx), "NEG": -tx, "CEIL": torch.ceil(tx), "FLOOR": torch.floor(tx),
        "EXP": torch.exp(tx), "ERF": torch.erf(tx), "SIN": torch.sin(tx), "TAN": torch.tan(tx),
        "TANH_FWD": torch.tanh(tx), "SIGMOID_FWD": torch.sigmoid(tx),
        "RELU_FWD": torch.relu(tx), "GELU_FWD": F.gelu(tx),
        "GELU_APPROX_TANH_FWD": F.gelu(tx, approximate="tanh"),
        "SWISH_FWD": F.silu(tx), "ELU_FWD": F.elu(tx, 1.0),
        "SOFTPLUS_FWD": F.softplus(tx, 1.0, 20.0), "RECIPROCAL": 1.0 / tx,
        "LOGICAL_NOT": (tx == 0).double(),
    }
    for name, ref in checks.items():
        assert np.allclose(oracle.pointwise(P[name], [x]), ref.numpy(), rtol=1e-6, atol=1e-7), name
    pos = np.abs(x) + 0.1
    assert np.allclose(oracle.pointwise(P["LOG"], [pos]), np.log(pos))
    assert np.allclose(oracle.pointwise(P["SQRT"], [pos]), np.sqrt(pos))
    assert np.allclose(oracle.pointwise(P["RSQRT"], [pos]), 1 / np.sqrt(pos))
    binary = {
        "ADD": tx + ty, "SUB": tx - ty, "MUL": tx * ty, "DIV": tx / ty,
        "MAX_OP": torch.maximum(tx, ty), "MIN_OP": torch.minimum(tx, ty),
        "ADD_SQUARE": tx + ty * ty, "CMP_GT": (tx > ty).double(), "CMP_LE": (tx <= ty).double(),
        "CMP_EQ": (tx == ty).double(), "CMP_NEQ": (tx != ty).double(),
        "CMP_GE": (tx >= ty).double(), "CMP_LT": (tx < ty).double(),
    }
    for name, ref in binary.items():
        assert np.allclose(oracle.pointwise(P[name], [x, y]), ref.numpy()), name
    # SUB and DIV are ordered: swapping operands must differ
    assert not np.allclose(oracle.pointwise(P["SUB"], [x, y]), oracle.pointwise(P["SUB"], [y, x]))
    # backward ops against autograd
    for name, fn in {"GELU_BWD": F.gelu, "TANH_BWD": torch.tanh, "SWISH_BWD": F.silu,
                     "GELU_APPROX_TANH_BWD": lambda t: F.gelu(t, approximate="tanh")}.items():
        tin = t64(y).requires_grad_(True)
        fn(tin).backward(tx)
        assert np.allclose(oracle.pointwise(P[name], [x, y]), tin.grad.numpy(), rtol=1e-6, atol=1e-8), name
    tin = t64(y).requires_grad_(True)
    torch.relu(tin).backward(tx)
    assert np.allclose(oracle.pointwise(P["RELU_BWD"], [x, y]), tin.grad.numpy())
    sel = oracle.pointwise(P["BINARY_SELECT"], [(x > 0).astype(np.float64), x, y])
    assert np.array_equal(sel, np.where(x > 0, x, y))
    # right-aligned broadcasting
    a, b = RNG.normal(size=[2, 3, 4]), RNG.normal(size=[4])
    assert np.allclose(oracle.pointwise(P["ADD"], [a, b]), a + b)


def test_check_close_criterion():
    ref = np.array([1.0, -2.0, 0.0, 4.0])
    rms = math.sqrt((ref ** 2).mean())
    ok, _ = oracle.check_close(ref + 0.9e-2 * rms, ref, 1e-2)
    assert ok
    bad = ref.copy(); bad[2] += 1.2e-2 * rms
    ok, rep = oracle.check_close(bad, ref, 1e-2)
    assert not ok and rep["violations"] == 1
