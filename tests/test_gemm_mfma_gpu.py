"""MFMA GEMM (bf16 / f16 / int8 / fp8) through the C ABI vs the oracle: every
operand orientation, ragged edges, batches, fused epilogues, and the full-size
benchmark config-5 shapes checked on sampled rows plus a checksum identity."""
import numpy as np
import pytest

from fusilli_amd import capi
from oracle import oracle
from helpers import HT, assert_close, rand

pytestmark = pytest.mark.gpu


def make_operand(seed, tid, rows, cols, dtype, transposed, batch=None):
    """Logical [rows, cols] (optionally [batch, rows, cols]); `transposed`
    stores it column-major (the reference expresses transposes by strides)."""
    dims = ([batch] if batch else []) + [rows, cols]
    if dtype == capi.INT8:
        vals = rand(seed, tid, dims, "int", lo=-127, hi=127)
    elif dtype in (capi.FP8E4M3, capi.FP8E5M2):
        vals = rand(seed, tid, dims, "uniform", lo=-2.0, hi=2.0)
    else:
        vals = rand(seed, tid, dims)
    strides = oracle.contiguous_strides(dims)
    if transposed:
        strides[-2], strides[-1] = 1, rows
    return HT.from_logical(vals, dtype, strides)


def run(ctx, a, b, c_dtype, out_dtype=None, epilogue=(), epi_tensors=(),
        expect_fast=True):
    out_dtype = c_dtype if out_dtype is None else out_dtype
    batch = np.broadcast_shapes(tuple(a.dims[:-2]), tuple(b.dims[:-2]))
    cdims = list(batch) + [a.dims[-2], b.dims[-1]]
    out = HT.empty(cdims, out_dtype)
    d = capi.MatmulDesc()
    d.a, d.b = a.desc(), b.desc()
    d.c = capi.TensorDesc.make(cdims, out.strides, c_dtype)
    d.out, d.out_dtype = out.desc(), out_dtype
    d.epilogue = capi.make_epilogue(list(epilogue))
    assert ctx.lib.fhip_matmul_supported(d) == (2 if expect_fast else 1)
    bufs = [t.upload(ctx) for t in epi_tensors]
    da, db, do = a.upload(ctx), b.upload(ctx), out.upload(ctx)
    ctx.matmul(d, da, db, do, epilogue_operands=bufs)
    return out.fetch(ctx, do)


def ref_matmul(a, b):
    al, bl = a.logical(), b.logical()
    if a.dtype == capi.INT8:
        return oracle.matmul(al.astype(np.int8), bl.astype(np.int8))
    return oracle.matmul(al, bl)


@pytest.mark.parametrize("dtype", [capi.BFLOAT16, capi.HALF, capi.INT8,
                                   capi.FP8E4M3, capi.FP8E5M2])
@pytest.mark.parametrize("ta,tb", [(False, False), (False, True), (True, False),
                                   (True, True)])
@pytest.mark.parametrize("m,n,k", [(256, 256, 256), (384, 128, 512),
                                   (264, 400, 128), (128, 136, 384)])
def test_gemm_orientations_and_edges(ctx, dtype, ta, tb, m, n, k):
    a = make_operand(70, 0, m, k, dtype, ta)
    b = make_operand(70, 1, k, n, dtype, tb)
    cdt = capi.INT32 if dtype == capi.INT8 else capi.FLOAT
    elem = capi.DTYPE_SIZE[dtype]
    # M/N-contiguous operands move in 16-byte column chunks
    fast = (not ta or (m * elem) % 16 == 0) and (tb or (n * elem) % 16 == 0)
    out = run(ctx, a, b, cdt, expect_fast=fast)
    ref = ref_matmul(a, b)
    if dtype == capi.INT8:
        assert np.array_equal(out.logical(), ref)
    else:
        assert_close(out.logical(), ref, capi.FLOAT, rtol=1e-4)


@pytest.mark.parametrize("dtype", [capi.BFLOAT16, capi.INT8])
def test_gemm_batched_and_broadcast_b(ctx, dtype):
    a = make_operand(71, 0, 256, 128, dtype, False, batch=3)
    b = make_operand(71, 1, 128, 256, dtype, False, batch=3)
    cdt = capi.INT32 if dtype == capi.INT8 else capi.FLOAT
    out = run(ctx, a, b, cdt)
    assert_close(out.logical(), ref_matmul(a, b), capi.FLOAT, rtol=1e-4)
    b1 = make_operand(71, 2, 128, 256, dtype, False, batch=1)
    out = run(ctx, a, b1, cdt)
    assert_close(out.logical(), ref_matmul(a, b1), capi.FLOAT, rtol=1e-4)


@pytest.mark.parametrize("act", ["RELU_FWD", "GELU_FWD", "SWISH_FWD", None])
def test_gemm_bf16_bias_activation_epilogue(ctx, act):
    m, n, k = 300, 256, 192
    a = make_operand(72, 0, m, k, capi.BFLOAT16, False)
    b = make_operand(72, 1, k, n, capi.BFLOAT16, False)
    bias = HT.from_logical(rand(72, 2, [1, n]), capi.BFLOAT16)
    epi = [capi.epilogue_op(capi.PW["ADD"], capi.FLOAT, operand=bias.desc())]
    if act:
        epi.append(capi.epilogue_op(capi.PW[act], capi.FLOAT))
    out = run(ctx, a, b, capi.FLOAT, out_dtype=capi.BFLOAT16, epilogue=epi,
              epi_tensors=[bias])
    ref = ref_matmul(a, b) + bias.logical()
    if act:
        ref = oracle.pointwise(capi.PW[act], [ref])
    assert_close(out.logical(), ref, capi.BFLOAT16)


@pytest.mark.parametrize("dtype", [capi.BFLOAT16, capi.HALF, capi.FP8E4M3])
@pytest.mark.parametrize("ta,tb", [(False, False), (True, True)])
@pytest.mark.parametrize("m,n,k", [(256, 256, 8192), (300, 512, 4096), (512, 260, 16384),
                                   (128, 520, 8192)])
def test_gemm_split_reduction(ctx, dtype, ta, tb, m, n, k):
    # Few output tiles and a long K: the reduction is cut into parts on
    # workgroups of their own and a second kernel adds them, rounds to the C
    # type and applies the fused bias + GELU.
    a = make_operand(73, 0, m, k, dtype, ta)
    b = make_operand(73, 1, k, n, dtype, tb)
    bias = HT.from_logical(rand(73, 2, [1, n]), capi.BFLOAT16)
    epi = [capi.epilogue_op(capi.PW["ADD"], capi.FLOAT, operand=bias.desc()),
           capi.epilogue_op(capi.PW["GELU_FWD"], capi.FLOAT)]
    elem = capi.DTYPE_SIZE[dtype]
    fast = (not ta or (m * elem) % 16 == 0) and (tb or (n * elem) % 16 == 0)
    out = run(ctx, a, b, capi.FLOAT, out_dtype=capi.BFLOAT16, epilogue=epi,
              epi_tensors=[bias], expect_fast=fast)
    ref = oracle.pointwise(capi.PW["GELU_FWD"], [ref_matmul(a, b) + bias.logical()])
    assert_close(out.logical(), ref, capi.BFLOAT16)
    out = run(ctx, a, b, capi.FLOAT, expect_fast=fast)
    assert_close(out.logical(), ref_matmul(a, b), capi.FLOAT, rtol=1e-4)


@pytest.mark.parametrize("ta,tb", [(False, False), (True, True)])
@pytest.mark.parametrize("m,n,k", [(256, 256, 8192), (304, 512, 4096), (512, 260, 16384)])
def test_gemm_int8_split_reduction_bit_exact(ctx, ta, tb, m, n, k):
    # int8 operands: the parts are int32 sums and their sum is exact
    a = make_operand(75, 0, m, k, capi.INT8, ta)
    b = make_operand(75, 1, k, n, capi.INT8, tb)
    fast = tb or n % 16 == 0
    out = run(ctx, a, b, capi.INT32, expect_fast=fast)
    if fast:
        name = ctx.last_kernel()
        assert name.startswith("gemm_mfma i8") and "split=" in name and not name.endswith("split=1"), name
    assert np.array_equal(out.logical(), ref_matmul(a, b))


def test_gemm_split_reduction_benchmark_shape(ctx):
    # bf16 1024 x 1024 x 8192 -> bf16, as the benchmark line runs it
    a = make_operand(74, 0, 1024, 8192, capi.BFLOAT16, False)
    b = make_operand(74, 1, 8192, 1024, capi.BFLOAT16, False)
    out = run(ctx, a, b, capi.FLOAT, out_dtype=capi.BFLOAT16)
    assert_close(out.logical(), ref_matmul(a, b), capi.BFLOAT16)


def test_gemm_tile_shapes_agree_bit_for_bit(ctx, knobs):
    # 1024 x 2048 x 4096 bf16 with the reduction in one piece (a split adds
    # its parts in f32, another order).  Every output element accumulates its
    # K slices in the same order on every tile shape, so repeated runs and the
    # other tile shapes must give the same bits; a wavefront reading a stage
    # that another is still filling would not.
    knobs(GEMM_SPLIT="1")
    a = make_operand(75, 0, 1024, 4096, capi.BFLOAT16, False)
    b = make_operand(75, 1, 4096, 2048, capi.BFLOAT16, True)
    first = run(ctx, a, b, capi.FLOAT).logical()
    assert_close(first, ref_matmul(a, b), capi.FLOAT, rtol=1e-4)
    for _ in range(8):
        assert np.array_equal(run(ctx, a, b, capi.FLOAT).logical(), first)
    for tile in ("256,256", "256,128", "128,128"):
        knobs(GEMM_TILE=tile, GEMM_SPLIT="1")
        assert np.array_equal(run(ctx, a, b, capi.FLOAT).logical(), first), tile


def test_gemm_fp8_per_tensor_scales_bf16_out(ctx):
    # benchmark config 5b at reduced size: x ~ U[-1,1], per-tensor scale
    # s = max|x| / 448, saturating RNE cast, C = (A8 B8) * (sa * sb) -> bf16.
    m, n, k = 512, 384, 1024
    xa = rand(73, 0, [m, k], "uniform")
    xb = rand(73, 1, [k, n], "uniform")
    sa, sb = float(np.abs(xa).max() / 448.0), float(np.abs(xb).max() / 448.0)
    a = HT.from_logical(xa / sa, capi.FP8E4M3)
    b = HT.from_logical(xb / sb, capi.FP8E4M3)
    epi = [capi.epilogue_op(capi.PW["MUL"], capi.BFLOAT16, scalar=sa * sb)]
    out = run(ctx, a, b, capi.FLOAT, out_dtype=capi.BFLOAT16, epilogue=epi)
    ref = ref_matmul(a, b) * np.float32(sa * sb)
    assert_close(out.logical(), ref, capi.BFLOAT16)
    # and the quantised product tracks the unquantised one
    exact = xa.astype(np.float64) @ xb.astype(np.float64)
    assert np.abs(out.logical() - exact).max() < 0.06 * np.abs(exact).max()


def test_gemm_all_ones_f16_known_answer_large(ctx):
    # samples/matmul/matmul_basic.cpp pattern (all ones => K), at a size the
    # MFMA kernel takes; f16 compare with ==.
    a = HT.from_logical(np.ones([256, 512]), capi.HALF)
    b = HT.from_logical(np.ones([512, 256]), capi.HALF)
    out = run(ctx, a, b, capi.HALF)
    assert np.all(out.logical() == 512.0)


def test_gemm_small_shapes_use_generic_kernel(ctx):
    a = make_operand(74, 0, 64, 128, capi.BFLOAT16, False)
    b = make_operand(74, 1, 128, 96, capi.BFLOAT16, False)
    out = run(ctx, a, b, capi.FLOAT, expect_fast=False)
    assert_close(out.logical(), ref_matmul(a, b), capi.FLOAT, rtol=1e-4)


def _full_size_rows_check(ctx, dtype):
    m, k, n = 4096, 8192, 4096
    a = make_operand(5 if dtype == capi.INT8 else 6, 0, m, k, dtype, False)
    b = make_operand(5 if dtype == capi.INT8 else 6, 1, k, n, dtype, False)
    cdt = capi.INT32 if dtype == capi.INT8 else capi.FLOAT
    out = run(ctx, a, b, cdt).logical()
    # one 256 x 256 tile per compute unit on eight wavefronts
    kind = "i8" if dtype == capi.INT8 else "fp8e4m3"
    assert ctx.last_kernel() == f"gemm_mfma {kind} 256x256 waves=8 split=1", ctx.last_kernel()
    rows = np.array([0, 1, 31, 32, 255, 256, 1023, 2048, 2049, 3071, 4064, 4095])
    al, bl = a.logical(), b.logical()
    if dtype == capi.INT8:
        ref = oracle.matmul_rows(al.astype(np.int8), bl.astype(np.int8), rows)
        assert np.array_equal(out[rows], ref)
        # size-independent identity: column sums of C equal (1^T A) B, exactly
        colsum_a = al.sum(axis=0)
        expect = colsum_a @ bl
        assert np.array_equal(out.sum(axis=0), expect)
    else:
        ref = oracle.matmul_rows(al, bl, rows)
        assert_close(out[rows], ref, capi.FLOAT, rtol=1e-4)
        colsum_a = al.astype(np.float64).sum(axis=0)
        expect = colsum_a @ bl.astype(np.float64)
        assert np.allclose(out.astype(np.float64).sum(axis=0), expect,
                           rtol=1e-4, atol=1e-3 * np.abs(expect).max())


def test_gemm_config5a_int8_full_size_bit_exact(ctx):
    _full_size_rows_check(ctx, capi.INT8)


def test_gemm_config5b_fp8_full_size(ctx):
    _full_size_rows_check(ctx, capi.FP8E4M3)


def test_gemm_config5b_fp8_full_size_scaled_bf16_output(ctx):
    # benchmark config 5b as stated: fp8 e4m3 operands quantised with
    # per-tensor scales s = max|x| / 448, f32 accumulation, the product
    # multiplied by s_a * s_b (a fused scalar MUL) and stored as bf16;
    # rel 2e-2 against the oracle on sampled rows of the full-size result.
    m, k, n = 4096, 8192, 4096
    fa = rand(6, 0, [m, k], "uniform")
    fb = rand(6, 1, [k, n], "uniform")
    sa, sb = float(np.abs(fa).max()) / 448.0, float(np.abs(fb).max()) / 448.0
    a = HT.from_logical(fa / sa, capi.FP8E4M3)
    b = HT.from_logical(fb / sb, capi.FP8E4M3)
    epi = [capi.epilogue_op(capi.PW["MUL"], capi.BFLOAT16, scalar=sa * sb)]
    out = run(ctx, a, b, capi.FLOAT, out_dtype=capi.BFLOAT16, epilogue=epi).logical()
    rows = np.array([0, 1, 33, 255, 256, 1023, 2048, 3071, 4064, 4095])
    ref = oracle.matmul_rows(a.logical(), b.logical(), rows) * np.float32(sa * sb)
    assert_close(out[rows], ref, capi.BFLOAT16, "config 5b scaled bf16")
    # the dequantised product also tracks the unquantised one (fp8 has 3
    # mantissa bits: about 3 % per element, averaged down over K = 8192)
    exact = fa[rows].astype(np.float64) @ fb.astype(np.float64)
    assert np.abs(out[rows] - exact).max() < 0.05 * np.abs(exact).max()
