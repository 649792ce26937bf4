"""RMSNorm / LayerNorm through the C ABI vs the oracle and the reference's
closed-form known answers (samples/rmsnorm/rmsnorm_utils.h:26-66,
samples/layernorm/layernorm_utils.h:25-82)."""
import numpy as np
import pytest

from fusilli_amd import capi
from oracle import oracle
from helpers import HT, assert_close, rand

pytestmark = pytest.mark.gpu


def run_norm(ctx, x, scale, bias, *, eps, layernorm=False, stats=False,
             y_dtype=None, out_dtype=None, epilogue=(), epi_tensors=(),
             expect_path=None, out_strides=None):
    out_dtype = x.dtype if out_dtype is None else out_dtype
    out = HT.empty(x.dims, out_dtype, out_strides or x.strides)
    d = capi.NormDesc()
    d.x = x.desc()
    if scale is not None:
        d.scale = scale.desc()
    if bias is not None:
        d.bias = bias.desc()
    yd = out_dtype if y_dtype is None else y_dtype
    d.y = capi.TensorDesc.make(x.dims, x.strides, yd)
    d.out = out.desc()
    d.out_dtype = out_dtype
    d.epsilon = eps
    d.is_layernorm = int(layernorm)
    d.emit_stats = int(stats)
    d.stats_dtype = capi.FLOAT
    d.epilogue = capi.make_epilogue(list(epilogue))
    if expect_path is not None:
        assert ctx.lib.fhip_norm_fwd_supported(d) == expect_path
    bufs = [t.upload(ctx) for t in epi_tensors]
    dx = x.upload(ctx)
    ds = scale.upload(ctx) if scale is not None else None
    db = bias.upload(ctx) if bias is not None else None
    dout = out.upload(ctx)
    mean = HT.empty([x.dims[0]], capi.FLOAT)
    rstd = HT.empty([x.dims[0]], capi.FLOAT)
    dm, dr = (mean.upload(ctx), rstd.upload(ctx)) if stats else (None, None)
    ctx.norm_fwd(d, dx, ds, db, dout, dm, dr, epilogue_operands=bufs)
    out.fetch(ctx, dout)
    if stats:
        mean.fetch(ctx, dm)
        rstd.fetch(ctx, dr)
        return out, mean, rstd
    return out


@pytest.mark.parametrize("dtype", [capi.BFLOAT16, capi.HALF, capi.FLOAT])
@pytest.mark.parametrize("rows,cols", [(8, 4096), (5, 512), (3, 520), (7, 8192),
                                       (4, 16384), (2, 40000), (6, 24)])
def test_rmsnorm_rows_vs_oracle(ctx, dtype, rows, cols):
    x = HT.from_logical(rand(11, 0, [rows, cols]), dtype)
    s = HT.from_logical(rand(11, 1, [1, cols], mean=1.0, std=0.02), dtype)
    vec = 16 // capi.DTYPE_SIZE[dtype]
    fits = cols % vec == 0 and cols <= 64 * vec * 256
    out = run_norm(ctx, x, s, None, eps=1e-6, expect_path=2 if fits else 1)
    ref = oracle.rmsnorm(x.logical(), s.logical(), 1e-6)
    assert_close(out.logical(), ref, dtype, f"rmsnorm {rows}x{cols}")


def test_rmsnorm_config2_shape_slice_with_scalar_mul(ctx):
    # benchmark config 2 at reduced row count: bf16, eps 1e-6, learned scale,
    # followed by a pointwise MUL (scalar operand).
    rows, cols = 256, 4096
    x = HT.from_logical(rand(2, 0, [rows, cols]), capi.BFLOAT16)
    s = HT.from_logical(rand(2, 1, [1, cols], mean=1.0, std=0.02), capi.BFLOAT16)
    epi = [capi.epilogue_op(capi.PW["MUL"], capi.BFLOAT16, scalar=0.5)]
    out = run_norm(ctx, x, s, None, eps=1e-6, y_dtype=capi.FLOAT, epilogue=epi,
                   expect_path=2)
    ref = oracle.rmsnorm(x.logical(), s.logical(), 1e-6) * 0.5
    assert_close(out.logical(), ref, capi.BFLOAT16, "config2 slice")


@pytest.mark.parametrize("kind", ["full", "row_vector", "per_row"])
def test_rmsnorm_fused_mul_tensor_operands(ctx, kind):
    rows, cols = 33, 2048
    x = HT.from_logical(rand(3, 0, [rows, cols]), capi.BFLOAT16)
    s = HT.from_logical(rand(3, 1, [1, cols], mean=1.0, std=0.02), capi.BFLOAT16)
    gdims = {"full": [rows, cols], "row_vector": [1, cols], "per_row": [rows, 1]}[kind]
    g = HT.from_logical(rand(3, 2, gdims), capi.BFLOAT16)
    epi = [capi.epilogue_op(capi.PW["MUL"], capi.BFLOAT16, operand=g.desc(),
                            operand_index=0)]
    out = run_norm(ctx, x, s, None, eps=1e-6, y_dtype=capi.FLOAT, epilogue=epi,
                   epi_tensors=[g], expect_path=2)
    ref = oracle.rmsnorm(x.logical(), s.logical(), 1e-6) * g.logical()
    assert_close(out.logical(), ref, capi.BFLOAT16, f"fused mul {kind}")


def test_rmsnorm_intermediate_rounding_is_honoured(ctx):
    # With a bf16 virtual Y between the norm and the MUL, Y is rounded to bf16
    # before the multiply; with f32 it is not.
    rows, cols = 4, 1024
    x = HT.from_logical(rand(5, 0, [rows, cols]), capi.BFLOAT16)
    epi = [capi.epilogue_op(capi.PW["MUL"], capi.FLOAT, scalar=3.0)]
    out = run_norm(ctx, x, None, None, eps=1e-6, y_dtype=capi.BFLOAT16,
                   out_dtype=capi.BFLOAT16, epilogue=[
                       capi.epilogue_op(capi.PW["MUL"], capi.BFLOAT16, scalar=3.0)],
                   expect_path=2)
    y = oracle.rmsnorm(x.logical(), None, 1e-6)
    y_rounded = oracle.dequantize(oracle.quantize(y, capi.BFLOAT16), capi.BFLOAT16)
    expect = oracle.dequantize(
        oracle.quantize(y_rounded.astype(np.float64) * 3.0, capi.BFLOAT16),
        capi.BFLOAT16)
    mism = np.mean(out.logical() != expect)
    assert mism < 0.02, mism  # only f32-vs-f64 last-bit ties may differ


@pytest.mark.parametrize("layout", ["nchw", "nhwc"])
@pytest.mark.parametrize("with_scale", [False, True])
def test_rmsnorm_reference_two_value_pattern(ctx, layout, with_scale):
    # samples/rmsnorm/rmsnorm_infer_*.cpp: n2 c3 h32 w32, x0 = 2b+1, x1 = 2b+3,
    # scale 2.0, tol 1e-4.
    n, c, h, w, eps, sc = 2, 3, 32, 32, 1e-5, 2.0
    dims = [n, c, h, w]
    strides = oracle.contiguous_strides(dims) if layout == "nchw" \
        else oracle.channels_last_strides(dims)
    half = c * h * w // 2
    phys = np.zeros((n, c * h * w), np.float32)
    exp = np.zeros_like(phys)
    for b in range(n):
        x0, x1 = 2.0 * b + 1.0, 2.0 * b + 3.0
        rms = np.sqrt((x0 * x0 + x1 * x1) / 2.0 + eps)
        k = sc if with_scale else 1.0
        phys[b, :half], phys[b, half:] = x0, x1
        exp[b, :half], exp[b, half:] = k * x0 / rms, k * x1 / rms
    x = HT(dims, strides, capi.FLOAT, phys.reshape(-1).copy())
    sdims = [1, c, h, w]
    sstr = oracle.contiguous_strides(sdims) if layout == "nchw" \
        else oracle.channels_last_strides(sdims)
    s = HT(sdims, sstr, capi.FLOAT, np.full(c * h * w, sc, np.float32)) \
        if with_scale else None
    out = run_norm(ctx, x, s, None, eps=eps, expect_path=2)
    assert np.allclose(out.storage.reshape(n, -1), exp, atol=1e-4, rtol=0)


def test_rmsnorm_generic_layout_vs_oracle(ctx):
    # dim 0 innermost: rows are not dense -> generic strided kernel.
    dims = [6, 5, 7]
    strides = [1, 6 * 7, 6]
    x = HT.from_logical(rand(8, 0, dims), capi.FLOAT, strides)
    s = HT.from_logical(rand(8, 1, [1, 5, 7]), capi.FLOAT)
    out = run_norm(ctx, x, s, None, eps=1e-5, expect_path=1)
    assert_close(out.logical(), oracle.rmsnorm(x.logical(), s.logical(), 1e-5),
                 capi.FLOAT)


@pytest.mark.parametrize("dtype", [capi.BFLOAT16, capi.HALF, capi.FLOAT])
@pytest.mark.parametrize("train", [False, True])
def test_layernorm_vs_oracle(ctx, dtype, train):
    rows, dims = 9, [9, 4, 16, 24]
    x = HT.from_logical(rand(21, 0, dims, mean=0.5, std=2.0), dtype,
                        oracle.channels_last_strides(dims))
    sd = [1] + dims[1:]
    s = HT.from_logical(rand(21, 1, sd, mean=1.0, std=0.1), dtype,
                        oracle.channels_last_strides(sd))
    b = HT.from_logical(rand(21, 2, sd), dtype, oracle.channels_last_strides(sd))
    res = run_norm(ctx, x, s, b, eps=1e-5, layernorm=True, stats=train,
                   expect_path=2)
    y, mean, rstd = oracle.layernorm(x.logical(), s.logical(), b.logical(), 1e-5)
    out = res[0] if train else res
    assert_close(out.logical(), y, dtype, "layernorm y")
    if train:
        assert_close(res[1].logical(), mean.reshape(-1), capi.FLOAT, "mean")
        assert_close(res[2].logical(), rstd.reshape(-1), capi.FLOAT, "rstd")


@pytest.mark.parametrize("case", [
    # rows too long for the register-resident kernels (more than 16384 16-byte
    # chunks): segments of a row on many workgroups, two passes
    dict(dims=[3, 8, 64, 130], dtype=capi.FLOAT, nhwc=False, affine=False),
    dict(dims=[3, 8, 64, 130], dtype=capi.FLOAT, nhwc=True, affine=True),
    dict(dims=[2, 16, 96, 100], dtype=capi.BFLOAT16, nhwc=True, affine=True),
    dict(dims=[5, 16, 96, 100], dtype=capi.HALF, nhwc=False, affine=True),
    dict(dims=[1, 140000], dtype=capi.HALF, nhwc=False, affine=False),
    # the reference's benchmark shapes (benchmarks/CMakeLists.txt, layernorm)
    dict(dims=[16, 128, 64, 32], dtype=capi.FLOAT, nhwc=False, affine=False),
    dict(dims=[16, 128, 64, 32], dtype=capi.BFLOAT16, nhwc=True, affine=True),
])
@pytest.mark.parametrize("train", [False, True])
def test_layernorm_long_rows_vs_oracle(ctx, case, train):
    dims, dtype = case["dims"], case["dtype"]
    lay = oracle.channels_last_strides if case["nhwc"] else (lambda d: None)
    x = HT.from_logical(rand(23, 0, dims, mean=3.0, std=2.0), dtype, lay(dims))
    s = b = None
    if case["affine"]:
        sd = [1] + dims[1:]
        s = HT.from_logical(rand(23, 1, sd, mean=1.0, std=0.1), dtype, lay(sd))
        b = HT.from_logical(rand(23, 2, sd), dtype, lay(sd))
    res = run_norm(ctx, x, s, b, eps=1e-5, layernorm=True, stats=train,
                   expect_path=2)
    y, mean, rstd = oracle.layernorm(
        x.logical(), None if s is None else s.logical(),
        None if b is None else b.logical(), 1e-5)
    out = res[0] if train else res
    assert_close(out.logical(), y, dtype, f"long-row layernorm {case}")
    if train:
        assert_close(res[1].logical(), mean.reshape(-1), capi.FLOAT, "mean")
        assert_close(res[2].logical(), rstd.reshape(-1), capi.FLOAT, "rstd")


@pytest.mark.parametrize("dtype", [capi.BFLOAT16, capi.FLOAT])
def test_rmsnorm_long_rows_vs_oracle(ctx, dtype):
    rows, cols = 3, 150016
    x = HT.from_logical(rand(24, 0, [rows, cols]), dtype)
    s = HT.from_logical(rand(24, 1, [1, cols], mean=1.0, std=0.02), dtype)
    out = run_norm(ctx, x, s, None, eps=1e-6, expect_path=2)
    assert_close(out.logical(), oracle.rmsnorm(x.logical(), s.logical(), 1e-6),
                 dtype, "long-row rmsnorm")
    # a fused pointwise chain on such rows stays on the generic kernel
    out = run_norm(ctx, x, s, None, eps=1e-6, expect_path=1,
                   epilogue=[capi.epilogue_op(capi.PW["MUL"], dtype, scalar=0.5)])
    assert_close(out.logical(),
                 oracle.rmsnorm(x.logical(), s.logical(), 1e-6) * 0.5, dtype,
                 "long-row rmsnorm with a fused MUL", rtol=2e-2 if dtype == capi.BFLOAT16 else None)


def test_layernorm_reference_two_value_pattern(ctx):
    # samples/layernorm/layernorm_utils.h:25-82: x0 = 2b, x1 = 2b+2 =>
    # y = scale*(-/+ 1/sqrt(1+eps)) + bias, mean = 2b+1, rstd = 1/sqrt(1+eps).
    n, c, h, w, eps, sc, bi = 2, 4, 8, 8, 1e-5, 2.0, 1.0
    inner = c * h * w
    phys = np.zeros((n, inner), np.float32)
    exp = np.zeros_like(phys)
    for b in range(n):
        phys[b, :inner // 2], phys[b, inner // 2:] = 2.0 * b, 2.0 * b + 2.0
        r = 1.0 / np.sqrt(1.0 + eps)
        exp[b, :inner // 2], exp[b, inner // 2:] = -sc * r + bi, sc * r + bi
    dims = [n, c, h, w]
    x = HT(dims, oracle.contiguous_strides(dims), capi.FLOAT, phys.reshape(-1).copy())
    s = HT.from_logical(np.full([1, c, h, w], sc), capi.FLOAT)
    bb = HT.from_logical(np.full([1, c, h, w], bi), capi.FLOAT)
    out, mean, rstd = run_norm(ctx, x, s, bb, eps=eps, layernorm=True, stats=True)
    assert np.allclose(out.storage.reshape(n, -1), exp, atol=1e-4, rtol=0)
    assert np.allclose(mean.storage, [1.0, 3.0], atol=1e-4)
    assert np.allclose(rstd.storage, 1.0 / np.sqrt(1.0 + eps), atol=1e-4)


def test_norm_rejects_bad_descriptors(ctx):
    x = HT.from_logical(rand(1, 0, [4, 64]), capi.FLOAT)
    d = capi.NormDesc()
    d.x = x.desc()
    d.y = x.desc()
    d.out = capi.TensorDesc.make([4, 32], [32, 1], capi.FLOAT)
    d.out_dtype = capi.FLOAT
    dx = x.upload(ctx)
    with pytest.raises(capi.FusilliHipError, match="dims differ"):
        ctx.norm_fwd(d, dx, None, None, dx)


# ---- the benchmarked sizes: several row-blocks per workgroup ---------------
def test_rmsnorm_config2_full_size_all_rows(ctx):
    # benchmark config 2 exactly as bench.py launches it: bf16 X[8192, 4096],
    # learned scale, eps 1e-6, f32 Y, fused scalar MUL, bf16 output.  At this
    # size the grid is capped, so a workgroup walks more than one row-block
    # with the scale held in registers; every row is checked.
    rows, cols = 8192, 4096
    x = HT.from_logical(rand(2, 0, [rows, cols]), capi.BFLOAT16)
    s = HT.from_logical(rand(2, 1, [1, cols], mean=1.0, std=0.02), capi.BFLOAT16)
    epi = [capi.epilogue_op(capi.PW["MUL"], capi.BFLOAT16, scalar=0.5)]
    out = run_norm(ctx, x, s, None, eps=1e-6, y_dtype=capi.FLOAT, epilogue=epi,
                   expect_path=2)
    ref = oracle.rmsnorm(x.logical(), s.logical(), 1e-6) * 0.5
    assert_close(out.logical(), ref, capi.BFLOAT16, "config 2 full size")
    # rows held in registers, the variant with the scalar multiply compiled in
    assert ctx.last_kernel().startswith("rownorm chunks="), ctx.last_kernel()
    assert ctx.last_kernel().endswith("variant=2"), ctx.last_kernel()


def test_rmsnorm_config2_full_size_full_operand_mul(ctx):
    # the same with a full-size second operand G[8192, 4096]
    rows, cols = 8192, 4096
    x = HT.from_logical(rand(2, 0, [rows, cols]), capi.BFLOAT16)
    s = HT.from_logical(rand(2, 1, [1, cols], mean=1.0, std=0.02), capi.BFLOAT16)
    g = HT.from_logical(rand(2, 3, [rows, cols]), capi.BFLOAT16)
    epi = [capi.epilogue_op(capi.PW["MUL"], capi.BFLOAT16, operand=g.desc(),
                            operand_index=0)]
    out = run_norm(ctx, x, s, None, eps=1e-6, y_dtype=capi.FLOAT, epilogue=epi,
                   epi_tensors=[g], expect_path=2)
    ref = oracle.rmsnorm(x.logical(), s.logical(), 1e-6) * g.logical()
    assert_close(out.logical(), ref, capi.BFLOAT16, "config 2 full operand")


def test_layernorm_8192x4096_all_rows_with_stats(ctx):
    # the LayerNorm line of the benchmark (bf16, scale and bias, training
    # statistics), every row and both statistics against the oracle
    rows, cols = 8192, 4096
    x = HT.from_logical(rand(8, 0, [rows, cols], mean=0.3, std=1.5), capi.BFLOAT16)
    s = HT.from_logical(rand(8, 1, [1, cols], mean=1.0, std=0.1), capi.BFLOAT16)
    b = HT.from_logical(rand(8, 2, [1, cols], std=0.2), capi.BFLOAT16)
    out, mean, rstd = run_norm(ctx, x, s, b, eps=1e-5, layernorm=True,
                               stats=True, expect_path=2)
    ref, rmean, rrstd = oracle.layernorm(x.logical(), s.logical(), b.logical(),
                                         1e-5)
    assert_close(out.logical(), ref, capi.BFLOAT16, "layernorm full size")
    assert_close(mean.logical(), rmean.reshape(-1), capi.FLOAT, "mean", rtol=1e-4)
    assert_close(rstd.logical(), rrstd.reshape(-1), capi.FLOAT, "rstd", rtol=1e-4)


@pytest.mark.parametrize("rows,cols", [(4099, 512), (2051, 1024), (1029, 2048),
                                       (700, 4096), (600, 16384)])
@pytest.mark.parametrize("kind", ["rms_scalar", "rms_per_row", "rms_full", "ln"])
def test_rownorm_several_row_blocks_per_workgroup(ctx, knobs, rows, cols, kind):
    # One workgroup per compute unit (256 workgroups): every workgroup walks
    # two to five row-blocks, reusing the column parameters it fetched once.
    # At 512 / 1024 / 2048 columns a workgroup holds 4 / 4 / 2 rows at a time
    # and the row count is no multiple of that (ragged last block).
    knobs(ROWNORM_WGS_PER_CU=1)
    x = HT.from_logical(rand(9, 0, [rows, cols], mean=0.1), capi.BFLOAT16)
    s = HT.from_logical(rand(9, 1, [1, cols], mean=1.0, std=0.05), capi.BFLOAT16)
    if kind == "ln":
        b = HT.from_logical(rand(9, 2, [1, cols], std=0.2), capi.BFLOAT16)
        out, mean, rstd = run_norm(ctx, x, s, b, eps=1e-5, layernorm=True,
                                   stats=True, expect_path=2)
        ref, rmean, rrstd = oracle.layernorm(x.logical(), s.logical(),
                                             b.logical(), 1e-5)
        assert_close(mean.logical(), rmean.reshape(-1), capi.FLOAT, "mean", rtol=1e-4)
        assert_close(rstd.logical(), rrstd.reshape(-1), capi.FLOAT, "rstd", rtol=1e-4)
    else:
        ref = oracle.rmsnorm(x.logical(), s.logical(), 1e-6)
        if kind == "rms_scalar":
            epi, ops = [capi.epilogue_op(capi.PW["MUL"], capi.BFLOAT16, scalar=0.5)], []
            ref = ref * 0.5
        else:
            gd = [rows, 1] if kind == "rms_per_row" else [rows, cols]
            g = HT.from_logical(rand(9, 3, gd), capi.BFLOAT16)
            epi = [capi.epilogue_op(capi.PW["MUL"], capi.BFLOAT16,
                                    operand=g.desc(), operand_index=0)]
            ops = [g]
            ref = ref * g.logical()
        out = run_norm(ctx, x, s, None, eps=1e-6, y_dtype=capi.FLOAT,
                       epilogue=epi, epi_tensors=ops, expect_path=2)
    assert_close(out.logical(), ref, capi.BFLOAT16, f"{kind} {rows}x{cols}")
