"""Matmul / conv / SDPA / reduction / pointwise through the C ABI vs the oracle
and the reference samples' known answers (strided generic kernels and
whichever tuned kernel the descriptor selects)."""
import numpy as np
import pytest

from fusilli_amd import capi
from oracle import oracle
from helpers import HT, assert_close, rand

pytestmark = pytest.mark.gpu


# ---- matmul ---------------------------------------------------------------
def run_matmul(ctx, a, b, c_dtype, *, out_dtype=None, epilogue=(),
               epi_tensors=(), out_strides=None):
    batch = np.broadcast_shapes(tuple(a.dims[:-2]), tuple(b.dims[:-2]))
    cdims = list(batch) + [a.dims[-2], b.dims[-1]]
    out_dtype = c_dtype if out_dtype is None else out_dtype
    out = HT.empty(cdims, out_dtype, out_strides)
    d = capi.MatmulDesc()
    d.a, d.b = a.desc(), b.desc()
    d.c = capi.TensorDesc.make(cdims, oracle.contiguous_strides(cdims), c_dtype)
    d.out = out.desc()
    d.out_dtype = out_dtype
    d.epilogue = capi.make_epilogue(list(epilogue))
    bufs = [t.upload(ctx) for t in epi_tensors]
    da, db, dout = a.upload(ctx), b.upload(ctx), out.upload(ctx)
    ctx.matmul(d, da, db, dout, epilogue_operands=bufs)
    return out.fetch(ctx, dout)


def test_matmul_config1_f32(ctx):
    # benchmark config 1: f32 A[1,256,512] x B[1,512,256], U[-1,1], rel 1e-4.
    a = HT.from_logical(rand(1, 0, [1, 256, 512], "uniform"), capi.FLOAT)
    b = HT.from_logical(rand(1, 1, [1, 512, 256], "uniform"), capi.FLOAT)
    out = run_matmul(ctx, a, b, capi.FLOAT)
    assert_close(out.logical(), oracle.matmul(a.logical(), b.logical()), capi.FLOAT)
    # 16 tiles of 64 x 64: the f32 matrix-instruction kernel that splits K
    # over the wavefronts of a 32 x 32 tile
    assert ctx.last_kernel() == "matmul_f32_splitk", ctx.last_kernel()


@pytest.mark.parametrize("transpose_b", [False, True])
def test_matmul_all_ones_f16_equals_k(ctx, transpose_b):
    # samples/matmul/matmul_basic.cpp:91-94,169-172: 64x128 * 128x256 => 128.
    m, k, n = 64, 128, 256
    a = HT.from_logical(np.ones([m, k]), capi.HALF)
    b = HT.from_logical(np.ones([k, n]), capi.HALF,
                        [1, k] if transpose_b else None)
    out = run_matmul(ctx, a, b, capi.HALF)
    assert np.all(out.logical() == 128.0)


def test_matmul_bias_known_answer(ctx):
    # samples/matmul/matmul_basic_with_bias.cpp:110-113: 128 + 2 = 130.
    m, k, n = 64, 128, 256
    a = HT.from_logical(np.ones([m, k]), capi.HALF)
    b = HT.from_logical(np.ones([k, n]), capi.HALF)
    bias = HT.from_logical(np.full([1, n], 2.0), capi.HALF)
    epi = [capi.epilogue_op(capi.PW["ADD"], capi.HALF, operand=bias.desc())]
    out = run_matmul(ctx, a, b, capi.HALF, epilogue=epi, epi_tensors=[bias])
    assert np.all(out.logical() == 130.0)


def test_matmul_batched_and_broadcast(ctx):
    # samples/matmul/matmul_batched.cpp: [16,16,M,K] x [1,1,K,N].
    a = HT.from_logical(rand(4, 0, [3, 4, 16, 24]), capi.FLOAT)
    b = HT.from_logical(rand(4, 1, [1, 1, 24, 8]), capi.FLOAT)
    out = run_matmul(ctx, a, b, capi.FLOAT)
    assert_close(out.logical(), oracle.matmul(a.logical(), b.logical()), capi.FLOAT)
    b2 = HT.from_logical(rand(4, 2, [3, 4, 24, 8]), capi.FLOAT)
    out2 = run_matmul(ctx, a, b2, capi.FLOAT)
    assert_close(out2.logical(), oracle.matmul(a.logical(), b2.logical()), capi.FLOAT)


@pytest.mark.parametrize("m,n,k", [(45, 70, 200), (33, 31, 129), (64, 64, 1000),
                                   (200, 300, 136), (130, 260, 64)])
@pytest.mark.parametrize("layout", ["nn", "tn", "nt"])
def test_matmul_f32_mfma_tiles(ctx, m, n, k, layout):
    # f32 operands run on the f32 matrix instruction: K split over the
    # wavefronts for small outputs, 64 x 64 tiles otherwise; ragged edges,
    # both operand orientations, batch broadcast and a fused bias + ReLU
    a_st = [m * k, 1, m] if layout == "tn" else None
    a = HT.from_logical(rand(8, 0, [2, m, k]), capi.FLOAT, a_st)
    bv = rand(8, 1, [1, k, n])
    b = HT.from_logical(bv, capi.FLOAT, [k * n, 1, k] if layout == "nt" else None)
    bias = HT.from_logical(rand(8, 2, [1, 1, n]), capi.FLOAT)
    epi = [capi.epilogue_op(capi.PW["ADD"], capi.FLOAT, operand=bias.desc()),
           capi.epilogue_op(capi.PW["RELU_FWD"], capi.FLOAT)]
    out = run_matmul(ctx, a, b, capi.FLOAT, epilogue=epi, epi_tensors=[bias])
    ref = np.maximum(oracle.matmul(a.logical(), b.logical()) + bias.logical(), 0.0)
    assert_close(out.logical(), ref, capi.FLOAT, f"{m}x{n}x{k} {layout}")


def test_matmul_strided_operands_and_output(ctx):
    a = HT.from_logical(rand(6, 0, [2, 33, 17]), capi.BFLOAT16, [33 * 17, 1, 33])
    b = HT.from_logical(rand(6, 1, [2, 17, 9]), capi.BFLOAT16, [17 * 9, 1, 17])
    out = run_matmul(ctx, a, b, capi.BFLOAT16, out_strides=[33 * 9, 1, 33])
    assert_close(out.logical(), oracle.matmul(a.logical(), b.logical()), capi.BFLOAT16)


def test_matmul_int8_exact_small(ctx):
    a = HT.from_logical(rand(5, 0, [70, 130], "int", lo=-127, hi=127), capi.INT8)
    b = HT.from_logical(rand(5, 1, [130, 50], "int", lo=-127, hi=127), capi.INT8)
    out = run_matmul(ctx, a, b, capi.INT32)
    ref = oracle.matmul(a.logical().astype(np.int8), b.logical().astype(np.int8))
    assert np.array_equal(out.logical(), ref)


def test_matmul_one_hot_selects_columns(ctx):
    a = HT.from_logical(rand(7, 0, [12, 10]), capi.FLOAT)
    sel = np.zeros([10, 4])
    for j, col in enumerate([7, 0, 3, 9]):
        sel[col, j] = 1.0
    out = run_matmul(ctx, a, HT.from_logical(sel, capi.FLOAT), capi.FLOAT)
    assert np.array_equal(out.logical(), a.logical()[:, [7, 0, 3, 9]])


# ---- conv -----------------------------------------------------------------
def run_conv(ctx, x, w, pad, stride, dil, y_dtype, *, out_dtype=None,
             epilogue=(), epi_tensors=(), channels_last_out=False):
    ydims = oracle.conv_output_dims(x.dims, w.dims, pad, stride, dil)
    out_dtype = y_dtype if out_dtype is None else out_dtype
    ostr = oracle.channels_last_strides(ydims) if channels_last_out else None
    out = HT.empty(ydims, out_dtype, ostr)
    d = capi.ConvDesc()
    d.x, d.w = x.desc(), w.desc()
    d.y = capi.TensorDesc.make(ydims, out.strides, y_dtype)
    d.out = out.desc()
    d.out_dtype = out_dtype
    d.spatial_rank = len(pad)
    for i in range(len(pad)):
        d.padding[i], d.stride[i], d.dilation[i] = pad[i], stride[i], dil[i]
    d.epilogue = capi.make_epilogue(list(epilogue))
    bufs = [t.upload(ctx) for t in epi_tensors]
    dx, dw, dout = x.upload(ctx), w.upload(ctx), out.upload(ctx)
    ctx.conv_fprop(d, dx, dw, dout, epilogue_operands=bufs)
    return out.fetch(ctx, dout)


@pytest.mark.parametrize("nhwc", [False, True])
def test_conv_all_ones_1x1_known_answer(ctx, nhwc):
    # tests/test_graph.cpp:198-223, samples/convolution/conv_fprop_nhwc_krsc.cpp:95:
    # all-ones f16, 1x1, C = 128 => 128.
    xd, wd = [4, 128, 8, 8], [32, 128, 1, 1]
    xs = oracle.channels_last_strides(xd) if nhwc else None
    ws = oracle.channels_last_strides(wd) if nhwc else None
    x = HT.from_logical(np.ones(xd), capi.HALF, xs)
    w = HT.from_logical(np.ones(wd), capi.HALF, ws)
    out = run_conv(ctx, x, w, [0, 0], [1, 1], [1, 1], capi.HALF,
                   channels_last_out=nhwc)
    assert np.all(out.logical() == 128.0)


def test_conv_bias_relu_known_answer(ctx):
    # samples/convolution/conv_fprop_with_relu_and_bias.cpp:112 => 129.
    xd, wd = [2, 128, 8, 8], [16, 128, 1, 1]
    x = HT.from_logical(np.ones(xd), capi.HALF, oracle.channels_last_strides(xd))
    w = HT.from_logical(np.ones(wd), capi.HALF, oracle.channels_last_strides(wd))
    bias = HT(list([1, 16, 1, 1]), [16, 1, 16, 16], capi.HALF,
              np.ones(16, np.float16))
    epi = [capi.epilogue_op(capi.PW["ADD"], capi.HALF, operand=bias.desc()),
           capi.epilogue_op(capi.PW["RELU_FWD"], capi.HALF)]
    out = run_conv(ctx, x, w, [0, 0], [1, 1], [1, 1], capi.HALF, epilogue=epi,
                   epi_tensors=[bias], channels_last_out=True)
    assert np.all(out.logical() == 129.0)


def test_conv_3x3_same_pad_corner_known_answer(ctx):
    # samples/convolution/conv_fprop_nhwc_krsc_with_pad.cpp:94: corner = 2*2*128.
    xd, wd = [2, 128, 8, 8], [16, 128, 3, 3]
    x = HT.from_logical(np.ones(xd), capi.HALF, oracle.channels_last_strides(xd))
    w = HT.from_logical(np.ones(wd), capi.HALF, oracle.channels_last_strides(wd))
    out = run_conv(ctx, x, w, [1, 1], [1, 1], [1, 1], capi.HALF,
                   channels_last_out=True)
    lg = out.logical()
    assert lg[0, 0, 0, 0] == 512.0 and lg[0, 0, 1, 1] == 1152.0 \
        and lg[1, 3, 0, 4] == 768.0


@pytest.mark.parametrize("case", [
    dict(x=[2, 6, 9, 11], w=[4, 6, 3, 3], pad=[1, 1], s=[1, 1], d=[1, 1]),
    dict(x=[2, 6, 9, 11], w=[4, 3, 3, 2], pad=[0, 1], s=[2, 1], d=[1, 2]),
    dict(x=[1, 8, 13], w=[8, 2, 4], pad=[2], s=[3], d=[2]),
    dict(x=[1, 4, 5, 6, 7], w=[2, 4, 2, 3, 3], pad=[1, 0, 1], s=[1, 2, 1], d=[1, 1, 1]),
])
@pytest.mark.parametrize("dtype", [capi.FLOAT, capi.BFLOAT16])
def test_conv_random_vs_oracle(ctx, case, dtype):
    x = HT.from_logical(rand(31, 0, case["x"]), dtype,
                        oracle.channels_last_strides(case["x"]))
    w = HT.from_logical(rand(31, 1, case["w"], std=0.2), dtype,
                        oracle.channels_last_strides(case["w"]))
    out = run_conv(ctx, x, w, case["pad"], case["s"], case["d"], dtype,
                   channels_last_out=True)
    ref = oracle.conv_fprop(x.logical(), w.logical(), case["pad"], case["s"],
                            case["d"])
    assert_close(out.logical(), ref, dtype, str(case))


# ---- conv backward --------------------------------------------------------
def conv_bwd_desc(x, w, dy, pad, stride, dil):
    d = capi.ConvDesc()
    d.x, d.w, d.y = x.desc(), w.desc(), dy.desc()
    d.spatial_rank = len(pad)
    for i in range(len(pad)):
        d.padding[i], d.stride[i], d.dilation[i] = pad[i], stride[i], dil[i]
    d.epilogue = capi.make_epilogue([])
    return d


def run_conv_dgrad(ctx, dy, w, x_dims, pad, stride, dil, dtype, nhwc=True,
                   tuned=False):
    dx = HT.empty(x_dims, dtype,
                  oracle.channels_last_strides(x_dims) if nhwc else None)
    d = conv_bwd_desc(dx, w, dy, pad, stride, dil)
    if tuned is not None:  # None: whichever kernel the library picks
        assert ctx.lib.fhip_conv_dgrad_supported(d) == (2 if tuned else 1)
        assert (ctx.conv_dgrad_workspace(d) > 0) == tuned
    bdy, bw, bdx = dy.upload(ctx), w.upload(ctx), dx.upload(ctx)
    ctx.conv_dgrad(d, bdy, bw, bdx)
    return dx.fetch(ctx, bdx)


def run_conv_wgrad(ctx, dy, x, w_dims, pad, stride, dil, dtype, nhwc=True,
                   tuned=False, w_dtype=None):
    dw = HT.empty(w_dims, dtype if w_dtype is None else w_dtype,
                  oracle.channels_last_strides(w_dims) if nhwc else None)
    d = conv_bwd_desc(x, dw, dy, pad, stride, dil)
    if tuned is not None:
        assert ctx.lib.fhip_conv_wgrad_supported(d) == (2 if tuned else 1)
        # (a tuned path may need none: 1 x 1 filters run as one matrix product)
        assert tuned or ctx.conv_wgrad_workspace(d) == 0
    bdy, bx, bdw = dy.upload(ctx), x.upload(ctx), dw.upload(ctx)
    ctx.conv_wgrad(d, bdy, bx, bdw)
    return dw.fetch(ctx, bdw)


@pytest.mark.parametrize("grouped", [False, True])
def test_conv_dgrad_all_ones_known_answer(ctx, grouped):
    # samples/convolution/conv_dgrad_nhwc_krsc.cpp:98 (=> K = 16) and
    # conv_dgrad_nhwc_krsc_grouped.cpp:99 (=> K / groups = 8); NHWC DY, KRSC
    # (contiguous) W, as the samples lay them out.
    n, c, k, fc = (4, 16, 32, 4) if grouped else (4, 8, 16, 8)
    dyd, wd = [n, k, 8, 8], [k, fc, 1, 1]
    dy = HT.from_logical(np.ones(dyd), capi.HALF, oracle.channels_last_strides(dyd))
    w = HT.from_logical(np.ones(wd), capi.HALF)
    # one group: the forward MFMA kernel on the mirrored filter (K = 16 channels
    # of DY, zero-padded to 64); grouped: the generic kernel
    dx = run_conv_dgrad(ctx, dy, w, [n, c, 8, 8], [0, 0], [1, 1], [1, 1], capi.HALF,
                        tuned=not grouped)
    assert np.all(dx.logical() == float(k // (c // fc)))


@pytest.mark.parametrize("variant", ["plain", "grouped", "grouped_strided"])
def test_conv_wgrad_all_ones_known_answer(ctx, variant):
    # samples/convolution/conv_wgrad_nhwc_krsc.cpp:99 (=> N*H*W = 256),
    # conv_wgrad_nhwc_krsc_grouped.cpp:99 (=> 256) and
    # conv_wgrad_nhwc_krsc_grouped_strided.cpp:103 (stride 2 => N*Ho*Wo = 64).
    n, c, k, fc = (4, 8, 16, 8) if variant == "plain" else (4, 16, 32, 4)
    st = 2 if variant == "grouped_strided" else 1
    dyd, xd = [n, k, 8 // st, 8 // st], [n, c, 8, 8]
    dy = HT.from_logical(np.ones(dyd), capi.HALF, oracle.channels_last_strides(dyd))
    x = HT.from_logical(np.ones(xd), capi.HALF, oracle.channels_last_strides(xd))
    dw = run_conv_wgrad(ctx, dy, x, [k, fc, 1, 1], [0, 0], [st, st], [1, 1],
                        capi.HALF)
    assert np.all(dw.logical() == float(n * (8 // st) ** 2))


@pytest.mark.parametrize("case", [
    dict(x=[2, 6, 9, 11], w=[4, 6, 3, 3], pad=[1, 1], s=[1, 1], d=[1, 1]),
    dict(x=[2, 6, 9, 11], w=[4, 3, 3, 2], pad=[0, 1], s=[2, 1], d=[1, 2]),
    dict(x=[2, 6, 10, 11], w=[6, 2, 3, 3], pad=[1, 2], s=[3, 2], d=[1, 1]),
    dict(x=[1, 8, 13], w=[8, 2, 4], pad=[2], s=[3], d=[2]),
    dict(x=[1, 4, 5, 6, 7], w=[2, 4, 2, 3, 3], pad=[1, 0, 1], s=[1, 2, 1], d=[1, 1, 1]),
    # channels-last 16-bit, one group, unit strides, K a multiple of 8: the data
    # gradient runs on the forward MFMA kernel (DY's 24 channels padded to 64)
    dict(x=[3, 16, 20, 20], w=[24, 16, 3, 3], pad=[1, 1], s=[1, 1], d=[1, 1],
         dgrad_mfma=True),
])
@pytest.mark.parametrize("dtype", [capi.FLOAT, capi.BFLOAT16])
@pytest.mark.parametrize("nhwc", [False, True])
def test_conv_backward_random_vs_oracle(ctx, case, dtype, nhwc):
    lay = oracle.channels_last_strides if nhwc else (lambda dims: None)
    yd = oracle.conv_output_dims(case["x"], case["w"], case["pad"], case["s"],
                                 case["d"])
    x = HT.from_logical(rand(32, 0, case["x"]), dtype, lay(case["x"]))
    w = HT.from_logical(rand(32, 1, case["w"], std=0.2), dtype, lay(case["w"]))
    dy = HT.from_logical(rand(32, 2, yd), dtype, lay(yd))
    dx = run_conv_dgrad(ctx, dy, w, case["x"], case["pad"], case["s"],
                        case["d"], dtype, nhwc,
                        tuned=case.get("dgrad_mfma", False) and nhwc
                        and dtype == capi.BFLOAT16)
    assert_close(dx.logical(),
                 oracle.conv_dgrad(dy.logical(), w.logical(), case["x"],
                                   case["pad"], case["s"], case["d"]),
                 dtype, f"dgrad {case}")
    dw = run_conv_wgrad(ctx, dy, x, case["w"], case["pad"], case["s"],
                        case["d"], dtype, nhwc)
    assert_close(dw.logical(),
                 oracle.conv_wgrad(dy.logical(), x.logical(), case["w"],
                                   case["pad"], case["s"], case["d"]),
                 dtype, f"wgrad {case}")


DIRECT_CASES = [
    # the reference benchmark's NCHW shape (reduced batch): 3 channels, 32 filters
    dict(x=[5, 3, 32, 32], w=[32, 3, 3, 3], pad=[0, 0], s=[1, 1], d=[1, 1]),
    # more filter channels than one staging pass holds (8192 / (9 * 8) = 113),
    # output channels no multiple of the blocks of 8 and 4
    dict(x=[1, 130, 6, 7], w=[13, 130, 3, 3], pad=[1, 1], s=[1, 1], d=[1, 1]),
    # groups whose channel counts are no multiple of the block sizes; stride
    dict(x=[2, 15, 9, 8], w=[21, 5, 2, 3], pad=[1, 0], s=[2, 1], d=[1, 2]),
    # more output channels than one staging pass of the data gradient holds
    dict(x=[1, 4, 5, 5], w=[300, 4, 2, 2], pad=[0, 1], s=[1, 1], d=[1, 1]),
    # 3-D, strided in depth; 1-D with dilation
    dict(x=[2, 3, 4, 9, 10], w=[6, 3, 2, 3, 3], pad=[0, 1, 1], s=[2, 1, 1], d=[1, 1, 1]),
    dict(x=[3, 2, 50], w=[5, 2, 7], pad=[3], s=[2], d=[3]),
]


@pytest.mark.parametrize("case", DIRECT_CASES)
@pytest.mark.parametrize("dtype", [capi.FLOAT, capi.HALF])
@pytest.mark.parametrize("nhwc", [False, True])
def test_conv_direct_kernels_vs_oracle(ctx, case, dtype, nhwc):
    # forward (+ per-channel bias), data gradient and weight gradient on the
    # register-blocked kernels, both layouts
    lay = oracle.channels_last_strides if nhwc else (lambda dims: None)
    yd = oracle.conv_output_dims(case["x"], case["w"], case["pad"], case["s"],
                                 case["d"])
    x = HT.from_logical(rand(33, 0, case["x"]), dtype, lay(case["x"]))
    w = HT.from_logical(rand(33, 1, case["w"], std=0.2), dtype, lay(case["w"]))
    dy = HT.from_logical(rand(33, 2, yd), dtype, lay(yd))
    k = case["w"][0]
    bdims = [1, k] + [1] * (len(yd) - 2)
    bias = HT.from_logical(rand(33, 3, bdims), dtype)
    epi = [capi.epilogue_op(capi.PW["ADD"], dtype, operand=bias.desc())]
    y = run_conv(ctx, x, w, case["pad"], case["s"], case["d"], dtype, epilogue=epi,
                 epi_tensors=[bias], channels_last_out=nhwc)
    ref = oracle.conv_fprop(x.logical(), w.logical(), case["pad"], case["s"],
                            case["d"]) + bias.logical()
    assert_close(y.logical(), ref, dtype, f"fprop {case}")
    # (channels-last 16-bit cases with unit strides and K % 8 == 0 qualify for
    # the MFMA data gradient; the other combinations run the direct kernel)
    dx = run_conv_dgrad(ctx, dy, w, case["x"], case["pad"], case["s"], case["d"],
                        dtype, nhwc, tuned=None)
    assert_close(dx.logical(),
                 oracle.conv_dgrad(dy.logical(), w.logical(), case["x"],
                                   case["pad"], case["s"], case["d"]),
                 dtype, f"dgrad {case}")
    dw = run_conv_wgrad(ctx, dy, x, case["w"], case["pad"], case["s"], case["d"],
                        dtype, nhwc, tuned=None)
    assert_close(dw.logical(),
                 oracle.conv_wgrad(dy.logical(), x.logical(), case["w"],
                                   case["pad"], case["s"], case["d"]),
                 dtype, f"wgrad {case}")


SMALL_GROUP_CASES = [
    # depthwise 3x3 (ConvNeXt / MobileNet style), ragged pixel count
    dict(x=[2, 40, 9, 7], w=[40, 1, 3, 3], pad=[1, 1], s=[1, 1], d=[1, 1]),
    # depthwise 7x7, more than one workgroup of channel blocks (136 channels)
    dict(x=[1, 136, 12, 10], w=[136, 1, 7, 7], pad=[3, 3], s=[1, 1], d=[1, 1]),
    # ResNeXt: 32 groups of 4 -> 4 channels; stride 2
    dict(x=[2, 128, 10, 11], w=[128, 4, 3, 3], pad=[1, 1], s=[2, 2], d=[1, 1]),
    # groups of 8 and of 2, dilation, asymmetric padding
    dict(x=[1, 64, 8, 9], w=[64, 8, 3, 2], pad=[2, 0], s=[1, 1], d=[2, 1]),
    dict(x=[3, 16, 6, 5], w=[16, 2, 1, 3], pad=[0, 1], s=[1, 2], d=[1, 1]),
    # 1-D depthwise
    dict(x=[2, 24, 50], w=[24, 1, 5], pad=[2], s=[1], d=[1]),
    # depthwise 3x3 strips: no padding (output narrower than a strip's reach),
    # padding 2 (output wider than the input), width a multiple of the strip
    dict(x=[1, 16, 6, 12], w=[16, 1, 3, 3], pad=[0, 0], s=[1, 1], d=[1, 1]),
    dict(x=[2, 24, 5, 9], w=[24, 1, 3, 3], pad=[2, 2], s=[1, 1], d=[1, 1]),
    dict(x=[3, 264, 4, 8], w=[264, 1, 3, 3], pad=[1, 0], s=[1, 1], d=[1, 1]),
]


@pytest.mark.parametrize("case", SMALL_GROUP_CASES)
@pytest.mark.parametrize("dtype", [capi.BFLOAT16, capi.HALF])
@pytest.mark.parametrize("out_dtype", ["same", "f32"])
def test_conv_small_groups_channels_last_vs_oracle(ctx, case, dtype, out_dtype):
    # Channels-last 16-bit convolutions whose groups have 1, 2, 4 or 8 input
    # and as many output channels: the kernel that owns whole groups per
    # thread (one 16-byte load per tap), with a per-channel bias and ReLU.
    lay = oracle.channels_last_strides
    x = HT.from_logical(rand(35, 0, case["x"]), dtype, lay(case["x"]))
    w = HT.from_logical(rand(35, 1, case["w"], std=0.3), dtype, lay(case["w"]))
    k = case["w"][0]
    bdims = [1, k] + [1] * len(case["pad"])
    bias = HT.from_logical(rand(35, 3, bdims), dtype)
    epi = [capi.epilogue_op(capi.PW["ADD"], capi.FLOAT, operand=bias.desc()),
           capi.epilogue_op(capi.PW["RELU_FWD"], capi.FLOAT)]
    od = dtype if out_dtype == "same" else capi.FLOAT
    ydims = oracle.conv_output_dims(case["x"], case["w"], case["pad"], case["s"], case["d"])
    d = capi.ConvDesc()
    d.x, d.w = x.desc(), w.desc()
    d.y = capi.TensorDesc.make(ydims, lay(ydims), capi.FLOAT)
    d.out = capi.TensorDesc.make(ydims, lay(ydims), od)
    d.out_dtype = od
    d.spatial_rank = len(case["pad"])
    for i in range(len(case["pad"])):
        d.padding[i], d.stride[i], d.dilation[i] = case["pad"][i], case["s"][i], case["d"][i]
    d.epilogue = capi.make_epilogue(epi)
    assert ctx.lib.fhip_conv_fprop_supported(d) == 2
    y = run_conv(ctx, x, w, case["pad"], case["s"], case["d"], capi.FLOAT, out_dtype=od,
                 epilogue=epi, epi_tensors=[bias], channels_last_out=True)
    ref = np.maximum(oracle.conv_fprop(x.logical(), w.logical(), case["pad"], case["s"],
                                       case["d"]) + bias.logical(), 0.0)
    assert_close(y.logical(), ref, od, f"{case}")


@pytest.mark.parametrize("dtype", [capi.BFLOAT16, capi.HALF])
def test_conv_depthwise_strip_kernel_matches_general_kernel(ctx, knobs, dtype):
    # depthwise 3x3 at unit stride runs on the strip kernel (4 output pixels
    # and 8 channels per thread, the filter in registers); with the switch off
    # the same call runs on the general small-group kernel.  Both add a pixel's
    # taps in filter order, so the results agree bit for bit.
    lay = oracle.channels_last_strides
    xd, wd = [2, 72, 11, 13], [72, 1, 3, 3]
    x = HT.from_logical(rand(36, 0, xd), dtype, lay(xd))
    w = HT.from_logical(rand(36, 1, wd, std=0.3), dtype, lay(wd))
    got = {}
    for strips in (1, 0):
        knobs(CONV_DEPTHWISE_STRIPS=strips)
        got[strips] = run_conv(ctx, x, w, [1, 1], [1, 1], [1, 1], capi.FLOAT, out_dtype=dtype,
                               channels_last_out=True).logical()
        name = ctx.last_kernel()
        assert name.startswith("conv_depthwise3x3" if strips else "conv_direct channels_last"), name
    assert np.array_equal(got[1], got[0])
    ref = oracle.conv_fprop(x.logical(), w.logical(), [1, 1], [1, 1], [1, 1])
    assert_close(got[1], ref, dtype, "depthwise strips")


def test_conv_direct_kernels_mixed_dtypes(ctx):
    # bf16 X against an f32 filter, f32 result: the run-time dtype path
    xd, wd = [2, 5, 8, 9], [7, 5, 3, 3]
    x = HT.from_logical(rand(34, 0, xd), capi.BFLOAT16)
    w = HT.from_logical(rand(34, 1, wd, std=0.2), capi.FLOAT)
    y = run_conv(ctx, x, w, [1, 1], [1, 1], [1, 1], capi.FLOAT)
    ref = oracle.conv_fprop(x.logical(), w.logical(), [1, 1], [1, 1], [1, 1])
    assert_close(y.logical(), ref, capi.FLOAT)
    dy = HT.from_logical(rand(34, 2, y.dims), capi.BFLOAT16)
    dw = run_conv_wgrad(ctx, dy, x, wd, [1, 1], [1, 1], [1, 1], capi.BFLOAT16,
                        nhwc=False, w_dtype=capi.FLOAT)
    assert_close(dw.logical(),
                 oracle.conv_wgrad(dy.logical(), x.logical(), wd, [1, 1], [1, 1],
                                   [1, 1]), capi.FLOAT)


@pytest.mark.parametrize("case", [
    # C % 64 == 0 is not needed: the reduction runs over K
    dict(x=[2, 24, 20, 20], w=[64, 24, 3, 3], pad=[1, 1], d=[1, 1]),
    dict(x=[3, 64, 17, 13], w=[128, 64, 3, 3], pad=[1, 1], d=[1, 1]),
    dict(x=[2, 40, 19, 23], w=[64, 40, 3, 2], pad=[2, 0], d=[2, 1]),
    dict(x=[1, 16, 30, 9], w=[192, 16, 1, 1], pad=[0, 0], d=[1, 1]),
    dict(x=[2, 72, 11, 11], w=[64, 72, 5, 5], pad=[0, 3], d=[1, 1]),
    dict(x=[4, 32, 150], w=[64, 32, 4], pad=[2], d=[3]),
    # strides above one: DY spread over a zero grid first
    dict(x=[2, 64, 15, 14], w=[128, 64, 3, 3], pad=[1, 1], d=[1, 1], s=[2, 2]),
    dict(x=[3, 24, 23, 31], w=[64, 24, 4, 3], pad=[2, 1], d=[2, 1], s=[3, 2]),
    dict(x=[2, 128, 16, 16], w=[256, 128, 1, 1], pad=[0, 0], d=[1, 1], s=[2, 2]),
    dict(x=[2, 16, 101], w=[64, 16, 5], pad=[2], d=[1], s=[4]),
    # groups whose K / groups is a multiple of 64: 2 groups of 24 <- 64
    # channels, 3 groups of 8 <- 128 with a stride, 1-D
    dict(x=[2, 48, 13, 12], w=[128, 24, 3, 3], pad=[1, 1], d=[1, 1]),
    dict(x=[1, 24, 15, 14], w=[384, 8, 3, 3], pad=[1, 1], d=[1, 1], s=[2, 2]),
    dict(x=[3, 32, 60], w=[128, 16, 5], pad=[2], d=[1]),
])
@pytest.mark.parametrize("dtype", [capi.BFLOAT16, capi.HALF])
@pytest.mark.parametrize("w_nhwc", [True, False])
def test_conv_dgrad_mfma_vs_oracle(ctx, case, dtype, w_nhwc):
    # 16-bit channels-last gradients: the forward MFMA kernel on the mirrored
    # filter (any filter layout), grouped when the convolution is
    sp = len(case["pad"])
    ones = case.get("s", [1] * sp)
    yd = oracle.conv_output_dims(case["x"], case["w"], case["pad"], ones, case["d"])
    w = HT.from_logical(rand(33, 1, case["w"], std=0.2), dtype,
                        oracle.channels_last_strides(case["w"]) if w_nhwc else None)
    dy = HT.from_logical(rand(33, 2, yd), dtype, oracle.channels_last_strides(yd))
    dx = run_conv_dgrad(ctx, dy, w, case["x"], case["pad"], ones, case["d"],
                        dtype, tuned=True)
    assert_close(dx.logical(),
                 oracle.conv_dgrad(dy.logical(), w.logical(), case["x"],
                                   case["pad"], ones, case["d"]),
                 dtype, f"dgrad {case}")


@pytest.mark.parametrize("case", [
    # [N, C, H, W] of DX, padding: 3 x 3 filters over K = 128 gradient channels,
    # C a multiple of 64 -- the kernel that keeps the filter in registers and
    # reads W as it lies
    dict(x=[2, 64, 12, 12], pad=1),     # small: the efficiency rule is overridden
    dict(x=[1, 64, 5, 7], pad=1),       # fewer pixel blocks than wavefronts
    dict(x=[3, 128, 17, 40], pad=1),    # two channel groups, ragged last tile
    dict(x=[2, 64, 9, 56], pad=0),      # widest slab row; DY smaller than DX
    dict(x=[2, 64, 11, 30], pad=2),     # DY larger than DX
    dict(x=[40, 64, 20, 20], pad=1),    # several tiles per workgroup
])
@pytest.mark.parametrize("dtype", [capi.BFLOAT16, capi.HALF])
@pytest.mark.parametrize("rows", [2, 5, 203, 407])
def test_conv_dgrad_register_filter_vs_oracle(ctx, case, dtype, rows, knobs):
    xd, wd, pad = case["x"], [128, case["x"][1], 3, 3], [case["pad"]] * 2
    yd = oracle.conv_output_dims(xd, wd, pad, [1, 1], [1, 1])
    cl = oracle.channels_last_strides
    dy = HT.from_logical(rand(36, 0, yd), dtype, cl(yd))
    w = HT.from_logical(rand(36, 1, wd, std=0.1), dtype, cl(wd))
    ref = oracle.conv_dgrad(dy.logical(), w.logical(), xd, pad, [1, 1], [1, 1])
    # rows per tile, + 100 x column tiles: forces the kernel and its tiling
    # (splits the width does not allow fall back to the kernel's own choice)
    knobs(DGRAD_ROWS=rows)
    dx = run_conv_dgrad(ctx, dy, w, xd, pad, [1, 1], [1, 1], dtype, tuned=True)
    assert_close(dx.logical(), ref, dtype, f"dgrad rf {case} rows {rows}")
    # the same call on the tiled kernel (mirrored filter in workspace)
    knobs(DGRAD_ROWS=0)
    dx2 = run_conv_dgrad(ctx, dy, w, xd, pad, [1, 1], [1, 1], dtype, tuned=True)
    assert_close(dx2.logical(), ref, dtype, f"dgrad tiled {case}")


def test_conv_dgrad_config3_shape_closed_form_and_oracle(ctx):
    # the data gradient of benchmark config 3 (N32 C64 56x56, K128 3x3 pad 1).
    # All-ones: DX = K * (taps whose output pixel exists) = 128 * {9, 6, 4}.
    xd, wd = [32, 64, 56, 56], [128, 64, 3, 3]
    yd = oracle.conv_output_dims(xd, wd, [1, 1], [1, 1], [1, 1])
    cl = oracle.channels_last_strides
    dy = HT.from_logical(np.ones(yd), capi.BFLOAT16, cl(yd))
    w = HT.from_logical(np.ones(wd), capi.BFLOAT16, cl(wd))
    dx = run_conv_dgrad(ctx, dy, w, xd, [1, 1], [1, 1], [1, 1], capi.BFLOAT16,
                        tuned=True).logical()
    edge = np.full(56, 3.0); edge[0] = edge[-1] = 2.0
    want = 128.0 * np.outer(edge, edge)
    assert np.array_equal(dx, np.broadcast_to(want, xd))
    # random values: the first two images against the oracle
    dy = HT.from_logical(rand(34, 0, yd), capi.BFLOAT16, cl(yd))
    w = HT.from_logical(rand(34, 1, wd, std=0.05), capi.BFLOAT16, cl(wd))
    dx = run_conv_dgrad(ctx, dy, w, xd, [1, 1], [1, 1], [1, 1], capi.BFLOAT16,
                        tuned=True).logical()
    ref = oracle.conv_dgrad(dy.logical()[:2], w.logical(), [2] + xd[1:],
                            [1, 1], [1, 1], [1, 1])
    assert_close(dx[:2], ref, capi.BFLOAT16, "config 3 dgrad")


@pytest.mark.parametrize("case", [
    dict(x=[2, 64, 12, 12], w=[128, 64, 3, 3], pad=[1, 1], d=[1, 1]),
    dict(x=[3, 32, 9, 21], w=[136, 32, 2, 5], pad=[0, 2], d=[1, 1]),
    dict(x=[1, 128, 7, 70], w=[192, 128, 3, 1], pad=[2, 0], d=[2, 1]),
    dict(x=[5, 24, 16, 16], w=[128, 24, 1, 7], pad=[0, 3], d=[1, 1]),
    dict(x=[2, 64, 15, 14], w=[128, 64, 3, 3], pad=[1, 1], d=[1, 1], s=2),
    dict(x=[3, 48, 23, 31], w=[160, 48, 4, 3], pad=[2, 1], d=[2, 1], s=3),
    dict(x=[2, 128, 16, 16], w=[256, 128, 1, 1], pad=[0, 0], d=[1, 1], s=2),
    # fewer than 128 output channels: DY is zero-padded to 128 (the shape class
    # of the reference's wgrad benchmark: C = K = 48, 3 x 3, padding 2)
    dict(x=[4, 48, 20, 16], w=[48, 48, 3, 3], pad=[2, 2], d=[1, 1]),
    dict(x=[3, 64, 9, 13], w=[8, 64, 3, 3], pad=[1, 1], d=[1, 1]),
    # 1 x 1, unit stride, no padding: the matrix product DY^T X over the pixels
    # (a multiple of 64 of them), its long reduction cut into parts
    dict(x=[4, 128, 16, 16], w=[256, 128, 1, 1], pad=[0, 0], d=[1, 1]),
    dict(x=[2, 136, 8, 40], w=[128, 136, 1, 1], pad=[0, 0], d=[1, 1]),
    dict(x=[3, 128, 320], w=[192, 128, 1], pad=[0], d=[1]),
])
@pytest.mark.parametrize("dtype", [capi.BFLOAT16, capi.HALF])
@pytest.mark.parametrize("w_nhwc", [True, False])
def test_conv_wgrad_mfma_vs_oracle(ctx, case, dtype, w_nhwc):
    # equal strides, one group, 16-bit channels-last X and DY, K >= 128 and
    # S * C >= 128: batched MFMA GEMMs over zero-padded grids
    st = [case.get("s", 1)] * len(case["pad"])
    yd = oracle.conv_output_dims(case["x"], case["w"], case["pad"], st, case["d"])
    cl = oracle.channels_last_strides
    x = HT.from_logical(rand(35, 0, case["x"]), dtype, cl(case["x"]))
    dy = HT.from_logical(rand(35, 2, yd), dtype, cl(yd))
    dw = run_conv_wgrad(ctx, dy, x, case["w"], case["pad"], st, case["d"],
                        dtype, nhwc=w_nhwc, tuned=True, w_dtype=capi.FLOAT)
    ref = oracle.conv_wgrad(dy.logical(), x.logical(), case["w"], case["pad"],
                            st, case["d"])
    assert_close(dw.logical(), ref, dtype, f"wgrad {case}")


@pytest.mark.parametrize("case", [
    # [N, C, H, W], K: 3 x 3 filters, padding 1, unit strides, images of up to
    # 56 columns, C and K multiples of 32 -- the kernel that reads X and DY in place
    dict(x=[2, 64, 12, 12], k=128),     # small batch: image rows cut into chunks
    dict(x=[1, 32, 5, 7], k=32),        # fewer rows than wavefronts
    dict(x=[3, 32, 17, 56], k=64),      # widest row, rows not a multiple of 8
    dict(x=[2, 96, 9, 33], k=32),       # three K-steps and a bit
    dict(x=[5, 32, 1, 1], k=32),        # one pixel per image
    dict(x=[70, 64, 10, 16], k=128),    # several images per workgroup, last group short
    dict(x=[40, 32, 23, 48], k=32),     # whole K-steps only
])
@pytest.mark.parametrize("dtype", [capi.BFLOAT16, capi.HALF])
def test_conv_wgrad_direct_kernel_vs_oracle(ctx, case, dtype, knobs):
    xd, wd = case["x"], [case["k"], case["x"][1], 3, 3]
    yd = [xd[0], case["k"], xd[2], xd[3]]
    cl = oracle.channels_last_strides
    x = HT.from_logical(rand(37, 0, xd), dtype, cl(xd))
    dy = HT.from_logical(rand(37, 1, yd), dtype, cl(yd))
    ref = oracle.conv_wgrad(dy.logical(), x.logical(), wd, [1, 1], [1, 1], [1, 1])
    dw = run_conv_wgrad(ctx, dy, x, wd, [1, 1], [1, 1], [1, 1], dtype, tuned=True,
                        w_dtype=capi.FLOAT)
    assert_close(dw.logical(), ref, dtype, f"direct wgrad {case}")
    # DW in the tensors' own dtype, filter laid out KCRS
    dw = run_conv_wgrad(ctx, dy, x, wd, [1, 1], [1, 1], [1, 1], dtype, nhwc=False,
                        tuned=True)
    assert_close(dw.logical(), ref, dtype, f"direct wgrad {case}, KCRS")
    # the workspace is only the partial sums: one 36 KB block per workgroup
    d = conv_bwd_desc(x, HT.empty(wd, dtype, cl(wd)), dy, [1, 1], [1, 1], [1, 1])
    assert ctx.conv_wgrad_workspace(d) % (9 * 16 * 64 * 4) == 0
    # switched off, the same descriptor runs on the batched-GEMM path or the
    # generic kernel and agrees
    knobs(WGRAD_DIRECT="0")
    assert ctx.conv_wgrad_workspace(d) % (9 * 16 * 64 * 4) != 0 or \
        ctx.conv_wgrad_workspace(d) == 0
    tuned = ctx.lib.fhip_conv_wgrad_supported(d) == 2
    dw = run_conv_wgrad(ctx, dy, x, wd, [1, 1], [1, 1], [1, 1], dtype, tuned=tuned,
                        w_dtype=capi.FLOAT)
    assert_close(dw.logical(), ref, dtype, f"wgrad without the direct kernel {case}")


def test_conv_wgrad_config3_shape_closed_form_and_oracle(ctx):
    # the weight gradient of benchmark config 3 (N32 C64 56x56, K128 3x3 pad 1).
    # All-ones: DW = N * (rows a tap sees) * (columns it sees) = 32 * {56, 55}^2.
    xd, wd = [32, 64, 56, 56], [128, 64, 3, 3]
    yd = [32, 128, 56, 56]
    cl = oracle.channels_last_strides
    x = HT.from_logical(np.ones(xd), capi.BFLOAT16, cl(xd))
    dy = HT.from_logical(np.ones(yd), capi.BFLOAT16, cl(yd))
    dw = run_conv_wgrad(ctx, dy, x, wd, [1, 1], [1, 1], [1, 1], capi.BFLOAT16,
                        tuned=True, w_dtype=capi.FLOAT).logical()
    span = np.array([55.0, 56.0, 55.0])
    assert np.array_equal(dw, np.broadcast_to(32.0 * np.outer(span, span), wd))
    # random values on four images against the oracle
    xd, yd = [4] + xd[1:], [4] + yd[1:]
    x = HT.from_logical(rand(36, 0, xd), capi.BFLOAT16, cl(xd))
    dy = HT.from_logical(rand(36, 1, yd), capi.BFLOAT16, cl(yd))
    dw = run_conv_wgrad(ctx, dy, x, wd, [1, 1], [1, 1], [1, 1], capi.BFLOAT16,
                        tuned=True).logical()
    ref = oracle.conv_wgrad(dy.logical(), x.logical(), wd, [1, 1], [1, 1], [1, 1])
    assert_close(dw, ref, capi.BFLOAT16, "config 3 wgrad")


def test_conv_dgrad_needs_its_workspace(ctx):
    xd, wd = [2, 24, 20, 20], [64, 24, 3, 3]
    cl = oracle.channels_last_strides
    dx = HT.empty(xd, capi.BFLOAT16, cl(xd))
    w = HT.empty(wd, capi.BFLOAT16, cl(wd))
    dy = HT.empty([2, 64, 20, 20], capi.BFLOAT16, cl([2, 64, 20, 20]))
    d = conv_bwd_desc(dx, w, dy, [1, 1], [1, 1], [1, 1])
    assert ctx.conv_dgrad_workspace(d) == 64 * 24 * 9 * 2
    with pytest.raises(Exception, match="workspace"):
        ctx._check(ctx.lib.fhip_conv_dgrad(ctx.handle, d, dy.upload(ctx).ptr,
                                           w.upload(ctx).ptr, dx.upload(ctx).ptr,
                                           None, 0))


def test_conv_backward_rejects_bad_descriptors(ctx):
    x = HT.empty([2, 6, 9, 11], capi.FLOAT)
    w = HT.empty([4, 6, 3, 3], capi.FLOAT)
    dy = HT.empty([2, 4, 9, 10], capi.FLOAT)  # Q should be 11
    d = conv_bwd_desc(x, w, dy, [1, 1], [1, 1], [1, 1])
    assert ctx.lib.fhip_conv_dgrad_supported(d) == 0
    assert ctx.lib.fhip_conv_wgrad_supported(d) == 0
    dy = HT.empty([2, 4, 9, 11], capi.FLOAT)
    d = conv_bwd_desc(x, w, dy, [1, 1], [1, 1], [1, 1])
    d.epilogue = capi.make_epilogue([capi.epilogue_op(capi.PW["RELU_FWD"], capi.FLOAT)])
    assert ctx.lib.fhip_conv_dgrad_supported(d) == 0
    with pytest.raises(Exception, match="gradient"):
        ctx.conv_dgrad(d, dy.upload(ctx), w.upload(ctx), x.upload(ctx))


# ---- batch norm -----------------------------------------------------------
def run_batchnorm(ctx, x, *, training, eps, scale=None, bias=None, mean=None,
                  var=None, y_dtype=None, stats_dtype=capi.FLOAT):
    """Returns (y, saved_mean, saved_inv_variance) as logical arrays."""
    c = x.dims[1]
    y = HT.empty(x.dims, x.dtype if y_dtype is None else y_dtype, x.strides)
    d = capi.BatchNormDesc()
    d.x, d.y = x.desc(), y.desc()
    d.training = int(training)
    d.has_scale, d.has_bias = int(scale is not None), int(bias is not None)
    d.scale_dtype = scale.dtype if scale is not None else capi.FLOAT
    d.bias_dtype = bias.dtype if bias is not None else capi.FLOAT
    d.running_dtype = mean.dtype if mean is not None else capi.FLOAT
    d.stats_dtype = stats_dtype
    d.epsilon = eps
    assert ctx.lib.fhip_batchnorm_fwd_supported(d) >= 1
    up = lambda t: None if t is None else t.upload(ctx)
    sm, sv = HT.empty([c], stats_dtype), HT.empty([c], stats_dtype)
    by, bsm, bsv = y.upload(ctx), sm.upload(ctx), sv.upload(ctx)
    ctx.batchnorm_fwd(d, x.upload(ctx), by, up(scale), up(bias), up(mean), up(var),
                      bsm if training else None, bsv if training else None)
    y.fetch(ctx, by)
    if not training:
        return y.logical(), None, None
    return y.logical(), sm.fetch(ctx, bsm).logical(), sv.fetch(ctx, bsv).logical()


@pytest.mark.parametrize("nhwc", [False, True])
@pytest.mark.parametrize("affine", [False, True])
def test_batchnorm_inference_known_answer(ctx, nhwc, affine):
    # samples/batchnorm/batchnorm_infer_{nchw,nchw_scale_bias,nhwc_scale_bias}.cpp
    # with batchnorm_utils.h:22-47: x = c + 1, mean 0, var 1.
    n, c, h, w, eps = 2, 4, 8, 8, 1e-5
    xd = [n, c, h, w]
    xv = np.broadcast_to(np.arange(1, c + 1, dtype=np.float64).reshape(1, c, 1, 1), xd)
    x = HT.from_logical(xv, capi.FLOAT, oracle.channels_last_strides(xd) if nhwc else None)
    vec = lambda v: HT.from_logical(np.full([c], v), capi.FLOAT)
    y, _, _ = run_batchnorm(ctx, x, training=False, eps=eps,
                            scale=vec(2.0) if affine else None,
                            bias=vec(0.5) if affine else None,
                            mean=vec(0.0), var=vec(1.0))
    want = xv / np.sqrt(np.float32(1 + eps))
    want = 2.0 * want + 0.5 if affine else want
    assert np.max(np.abs(y - want)) < 1e-4  # the samples' tolerance


@pytest.mark.parametrize("affine", [False, True])
def test_batchnorm_training_known_answer(ctx, affine):
    # samples/batchnorm/batchnorm_train_nchw{,_scale_bias}.cpp with
    # batchnorm_utils.h:60-104: +-1 halves => mean 0, inv_variance 1/sqrt(1+eps).
    n, c, h, w, eps = 2, 4, 8, 8, 1e-5
    flat = np.where(np.arange(n * h * w) < n * h * w // 2, -1.0, 1.0)
    xv = np.broadcast_to(flat.reshape(n, 1, h, w), [n, c, h, w])
    x = HT.from_logical(xv, capi.FLOAT)
    vec = lambda v: HT.from_logical(np.full([c], v), capi.FLOAT)
    y, m, v = run_batchnorm(ctx, x, training=True, eps=eps,
                            scale=vec(2.0) if affine else None,
                            bias=vec(0.5) if affine else None)
    inv = 1.0 / np.sqrt(1.0 + eps)
    want = xv * inv
    want = 2.0 * want + 0.5 if affine else want
    assert np.max(np.abs(y - want)) < 1e-4
    assert np.max(np.abs(m)) < 1e-4 and np.max(np.abs(v - inv)) < 1e-4


@pytest.mark.parametrize("dims", [[3, 5, 7, 6], [4, 3, 9], [2, 6], [2, 3, 4, 5, 2],
                                  [8, 64, 28, 28]])
@pytest.mark.parametrize("training", [False, True])
@pytest.mark.parametrize("dtype", [capi.FLOAT, capi.BFLOAT16, capi.HALF])
@pytest.mark.parametrize("nhwc", [False, True])
def test_batchnorm_random_vs_oracle(ctx, dims, training, dtype, nhwc):
    if nhwc and len(dims) < 3:
        pytest.skip("no spatial dims")
    c, eps = dims[1], 1e-3
    x = HT.from_logical(rand(41, 0, dims, std=2.0, mean=1.0), dtype,
                        oracle.channels_last_strides(dims) if nhwc else None)
    sc = HT.from_logical(rand(41, 1, [c], mean=1.0, std=0.3), dtype)
    b = HT.from_logical(rand(41, 2, [c]), dtype)
    rm = HT.from_logical(rand(41, 3, [c]), capi.FLOAT)
    rv = HT.from_logical(rand(41, 4, [c], "uniform", lo=0.5, hi=1.5), capi.FLOAT)
    y, m, v = run_batchnorm(ctx, x, training=training, eps=eps, scale=sc, bias=b,
                            mean=None if training else rm,
                            var=None if training else rv)
    ry, rmean, rinv = oracle.batchnorm(x.logical(), sc.logical(), b.logical(),
                                       rm.logical(), rv.logical(), eps, training)
    assert_close(y, ry, dtype, f"batchnorm {dims}")
    if training:
        assert_close(m, rmean, capi.FLOAT, "saved mean")
        assert_close(v, rinv, capi.FLOAT, "saved inv variance")


BN_CL_CASES = [
    # channels-last shapes of the column kernels: one chunk of channels (256 row
    # lanes), 17 chunks (15 row lanes, idle threads), fewer rows than row lanes,
    # 1-D and 3-D space, f32 chunks of 4
    ([64, 8, 5, 7], capi.BFLOAT16), ([3, 136, 9, 11], capi.HALF), ([2, 128, 1, 3], capi.BFLOAT16),
    ([5, 40, 33], capi.HALF), ([2, 16, 3, 4, 5], capi.BFLOAT16), ([6, 12, 10, 9], capi.FLOAT),
    ([16, 256, 28, 28], capi.BFLOAT16),
]


@pytest.mark.parametrize("dims,dtype", BN_CL_CASES)
@pytest.mark.parametrize("training", [False, True])
@pytest.mark.parametrize("affine", [False, True])
def test_batchnorm_channels_last_kernels_vs_oracle(ctx, dims, dtype, training, affine):
    c, eps = dims[1], 1e-3
    x = HT.from_logical(rand(43, 0, dims, std=1.5, mean=3.0), dtype,
                        oracle.channels_last_strides(dims))
    sc = HT.from_logical(rand(43, 1, [c], mean=1.0, std=0.3), capi.FLOAT) if affine else None
    b = HT.from_logical(rand(43, 2, [c]), dtype) if affine else None
    rm = HT.from_logical(rand(43, 3, [c], mean=3.0), capi.FLOAT)
    rv = HT.from_logical(rand(43, 4, [c], "uniform", lo=0.5, hi=3.0), capi.FLOAT)
    y, m, v = run_batchnorm(ctx, x, training=training, eps=eps, scale=sc, bias=b,
                            mean=None if training else rm, var=None if training else rv)
    assert ctx.last_kernel().startswith("batchnorm_channels_last"), ctx.last_kernel()
    ry, rmean, rinv = oracle.batchnorm(x.logical(), None if sc is None else sc.logical(),
                                       None if b is None else b.logical(),
                                       rm.logical(), rv.logical(), eps, training)
    assert_close(y, ry, dtype, f"batchnorm channels-last {dims}")
    if training:
        assert_close(m, rmean, capi.FLOAT, "saved mean")
        assert_close(v, rinv, capi.FLOAT, "saved inv variance")
        # moment invariants of the output: mean_c(y) = bias, var_c(y) = scale^2 var / (var + eps)
        axes = tuple(i for i in range(len(dims)) if i != 1)
        tol = 2e-2 if dtype != capi.FLOAT else 1e-4
        want_mean = 0.0 if b is None else b.logical()
        assert np.max(np.abs(y.mean(axis=axes) - want_mean)) < tol


def test_batchnorm_rejects_bad_descriptors(ctx):
    d = capi.BatchNormDesc()
    d.x = capi.TensorDesc.make([2, 4, 8, 8], [256, 64, 8, 1], capi.FLOAT)
    d.y = capi.TensorDesc.make([2, 4, 8, 7], [224, 56, 7, 1], capi.FLOAT)
    d.running_dtype = d.stats_dtype = d.scale_dtype = d.bias_dtype = capi.FLOAT
    d.epsilon = 1e-5
    assert ctx.lib.fhip_batchnorm_fwd_supported(d) == 0
    d.y = d.x
    assert ctx.lib.fhip_batchnorm_fwd_supported(d) == 1
    d.x = capi.TensorDesc.make([8], [1], capi.FLOAT)
    d.y = d.x
    assert ctx.lib.fhip_batchnorm_fwd_supported(d) == 0
    d.x = d.y = capi.TensorDesc.make([2, 4, 8, 8], [256, 64, 8, 1], capi.INT32)
    assert ctx.lib.fhip_batchnorm_fwd_supported(d) == 0


# ---- sdpa -----------------------------------------------------------------
def run_sdpa(ctx, q, k, v, *, mask=None, causal=False, scale=None, o_dtype=None):
    o_dtype = q.dtype if o_dtype is None else o_dtype
    out = HT.empty([q.dims[0], q.dims[1], q.dims[2], v.dims[3]], o_dtype)
    d = capi.SdpaDesc()
    d.q, d.k, d.v, d.o = q.desc(), k.desc(), v.desc(), out.desc()
    if mask is not None:
        d.mask = mask.desc()
    d.is_causal = int(causal)
    if scale is not None:
        d.has_scale, d.scale = 1, scale
    bufs = [t.upload(ctx) for t in (q, k, v)]
    dm = mask.upload(ctx) if mask is not None else None
    dout = out.upload(ctx)
    ctx.sdpa_fwd(d, bufs[0], bufs[1], bufs[2], dout, mask=dm)
    return out.fetch(ctx, dout)


@pytest.mark.parametrize("variant", ["mha", "causal", "mask", "gqa", "cross"])
def test_sdpa_constant_fill_equals_v(ctx, variant):
    # samples/sdpa/*.cpp via samples/sdpa_utils.cpp:184-247: q = k = v = 0.01
    # (mask -1) => output == v within 1e-2; B1 H8 S64 D64 f16.
    B, Hq, Hkv, Sq, Skv, D = 1, 8, 8, 64, 64, 64
    if variant == "gqa":
        Hkv = 2
    if variant == "cross":
        Sq, Skv = 32, 128
    q = HT.from_logical(np.full([B, Hq, Sq, D], 0.01), capi.HALF)
    k = HT.from_logical(np.full([B, Hkv, Skv, D], 0.01), capi.HALF)
    v = HT.from_logical(np.full([B, Hkv, Skv, D], 0.01), capi.HALF)
    mask = HT.from_logical(np.full([B, 1, Sq, Skv], -1.0), capi.HALF) \
        if variant == "mask" else None
    out = run_sdpa(ctx, q, k, v, mask=mask, causal=(variant == "causal"))
    assert np.allclose(out.logical(), v.logical()[0, 0, 0, 0], atol=1e-2)


@pytest.mark.parametrize("case", [
    dict(B=2, Hq=4, Hkv=4, Sq=70, Skv=70, D=32, Dv=32, causal=True),
    dict(B=1, Hq=6, Hkv=2, Sq=33, Skv=129, D=16, Dv=24, causal=False),
    dict(B=2, Hq=2, Hkv=1, Sq=17, Skv=65, D=64, Dv=64, causal=False, mask="float"),
    dict(B=1, Hq=2, Hkv=2, Sq=40, Skv=40, D=128, Dv=128, causal=False, mask="bool"),
])
@pytest.mark.parametrize("dtype", [capi.FLOAT, capi.BFLOAT16])
def test_sdpa_random_vs_oracle(ctx, case, dtype):
    c = case
    q = HT.from_logical(rand(41, 0, [c["B"], c["Hq"], c["Sq"], c["D"]]), dtype)
    k = HT.from_logical(rand(41, 1, [c["B"], c["Hkv"], c["Skv"], c["D"]]), dtype)
    v = HT.from_logical(rand(41, 2, [c["B"], c["Hkv"], c["Skv"], c["Dv"]]), dtype)
    mask, mref = None, None
    if c.get("mask") == "float":
        mask = HT.from_logical(rand(41, 3, [c["B"], 1, c["Sq"], c["Skv"]]), dtype)
        mref = mask.logical()
    elif c.get("mask") == "bool":
        keep = rand(41, 3, [1, 1, c["Sq"], c["Skv"]], "uniform") > -0.5
        keep[..., 0] = True
        mask = HT.from_logical(keep, capi.BOOLEAN)
        mref = keep
    out = run_sdpa(ctx, q, k, v, mask=mask, causal=c["causal"])
    ref = oracle.sdpa(q.logical(), k.logical(), v.logical(), mask=mref,
                      is_causal=c["causal"])
    assert_close(out.logical(), ref, dtype, str(case))


# ---- reduction ------------------------------------------------------------
@pytest.mark.parametrize("mode", ["ADD", "SUM", "MUL", "MIN", "MAX", "AMAX",
                                  "AVG", "NORM1", "NORM2", "MUL_NO_ZEROS"])
@pytest.mark.parametrize("dtype", [capi.INT32, capi.HALF, capi.FLOAT])
def test_reduction_reference_table(ctx, mode, dtype):
    # samples/reduction/reduction_ops.cpp:31-64, 83-273: [2,16,8,8] -> [2,16,1,1];
    # inputs i % 100 - 50 (sums) or ones with a 2 and a 3 (products).
    if mode == "AVG" and dtype == capi.INT32:
        pytest.skip("integer AVG is rejected at validation (reduction_node.h:122-127)")
    dims, odims = [2, 16, 8, 8], [2, 16, 1, 1]
    n = int(np.prod(dims))
    if mode in ("MUL", "MUL_NO_ZEROS"):
        vals = np.ones(n)
        vals[0], vals[1] = 2.0, 3.0
        if mode == "MUL_NO_ZEROS":
            vals[2] = 0.0
    else:
        vals = (np.arange(n) % 100 - 50).astype(np.float64)
    x = HT.from_logical(vals.reshape(dims), dtype)
    out = HT.empty(odims, dtype)
    d = capi.ReduceDesc()
    d.x, d.y, d.mode = x.desc(), out.desc(), capi.RED[mode]
    dx, dy = x.upload(ctx), out.upload(ctx)
    ctx.reduce(d, dx, dy)
    out.fetch(ctx, dy)
    ref = oracle.reduction(x.logical(), odims, capi.RED[mode])
    if dtype == capi.INT32:
        assert np.array_equal(out.logical(), ref.astype(np.int64))
    else:
        assert np.all(np.abs(out.logical() - ref) < max(0.01, 2e-3 * np.abs(ref).max()))


@pytest.mark.parametrize("mode", ["SUM", "MAX", "NORM2", "AVG"])
def test_reduction_few_outputs_long_ranges(ctx, mode):
    # the bias gradient of a convolution: [N, K, H, W] -> [1, K, 1, 1]; few
    # outputs, so the range of each is cut into slices on workgroups of their
    # own and combined by a second kernel
    x = HT.from_logical(rand(43, 0, [20, 6, 30, 31]), capi.FLOAT)
    d = capi.ReduceDesc()
    out = HT.empty([1, 6, 1, 1], capi.FLOAT)
    d.x, d.y, d.mode = x.desc(), out.desc(), capi.RED[mode]
    assert ctx.lib.fhip_reduce_supported(d) == 1
    bx, bo = x.upload(ctx), out.upload(ctx)
    ctx.reduce(d, bx, bo)
    got = out.fetch(ctx, bo).logical()
    ref = oracle.reduction(x.logical(), [1, 6, 1, 1], capi.RED[mode])
    assert_close(got, ref, capi.FLOAT, mode)


def test_reduction_middle_dim_strided(ctx):
    dims, odims = [3, 50, 7], [3, 1, 7]
    x = HT.from_logical(rand(51, 0, dims), capi.FLOAT, [7, 21, 1])
    out = HT.empty(odims, capi.FLOAT)
    d = capi.ReduceDesc()
    d.x, d.y, d.mode = x.desc(), out.desc(), capi.RED["NORM2"]
    dx, dy = x.upload(ctx), out.upload(ctx)
    ctx.reduce(d, dx, dy)
    assert_close(out.fetch(ctx, dy).logical(),
                 oracle.reduction(x.logical(), odims, capi.RED["NORM2"]), capi.FLOAT)


# ---- pointwise ------------------------------------------------------------
def run_pointwise(ctx, mode, ins, out_dtype, out_dims=None, params=None,
                  scalars=None):
    scalars = scalars or {}
    shapes = [tuple(t.dims) for t in ins if t is not None]
    odims = list(np.broadcast_shapes(*shapes)) if out_dims is None else out_dims
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
    bufs += [None] * (3 - len(bufs))
    dout = out.upload(ctx)
    ctx.pointwise(d, bufs[0], bufs[1], bufs[2], dout)
    return out.fetch(ctx, dout)


UNARY = ["ABS", "CEIL", "ELU_FWD", "ERF", "EXP", "FLOOR", "GELU_APPROX_TANH_FWD",
         "GELU_FWD", "IDENTITY", "LOG", "NEG", "RECIPROCAL", "RELU_FWD", "RSQRT",
         "SIGMOID_FWD", "SIN", "SOFTPLUS_FWD", "SQRT", "SWISH_FWD", "TAN",
         "TANH_FWD", "LOGICAL_NOT"]
BINARY = ["ADD", "ADD_SQUARE", "DIV", "MAX_OP", "MIN_OP", "MUL", "SUB", "CMP_EQ",
          "CMP_GE", "CMP_GT", "CMP_LE", "CMP_LT", "CMP_NEQ", "LOGICAL_AND",
          "LOGICAL_OR", "RELU_BWD", "TANH_BWD", "GELU_BWD",
          "GELU_APPROX_TANH_BWD", "SWISH_BWD"]


@pytest.mark.parametrize("mode", UNARY)
@pytest.mark.parametrize("dtype", [capi.FLOAT, capi.HALF])
def test_pointwise_unary_vs_oracle(ctx, mode, dtype):
    vals = rand(61, 0, [4, 37], "uniform", lo=-3.0, hi=3.0)
    if mode in ("LOG", "RSQRT", "SQRT"):
        vals = np.abs(vals) + 0.1
    if mode in ("RECIPROCAL", "TAN"):
        vals = np.where(np.abs(vals) < 0.2, 0.7, vals) * (0.4 if mode == "TAN" else 1)
    x = HT.from_logical(vals, dtype)
    params = capi.PointwiseParams(1.5, 2.0, 3.0, 0.75)
    odt = capi.BOOLEAN if mode == "LOGICAL_NOT" else dtype
    out = run_pointwise(ctx, mode, [x], odt, params=params)
    ref = oracle.pointwise(capi.PW[mode], [x.logical()], elu_alpha=1.5,
                           softplus_beta=2.0, softplus_threshold=3.0,
                           swish_beta=0.75)
    if odt == capi.BOOLEAN:
        assert np.array_equal(out.logical(), ref.astype(np.int64))
    else:
        assert_close(out.logical(), ref, dtype, mode,
                     rtol=1e-4 if dtype == capi.FLOAT else 2e-2)


@pytest.mark.parametrize("mode", BINARY)
def test_pointwise_binary_broadcast_vs_oracle(ctx, mode):
    a = HT.from_logical(np.round(rand(62, 0, [3, 1, 8], "uniform", lo=-2, hi=2), 1),
                        capi.FLOAT)
    b = HT.from_logical(np.round(rand(62, 1, [5, 8], "uniform", lo=-2, hi=2), 1) + 0.05,
                        capi.FLOAT)
    boolean = mode.startswith("CMP") or mode.startswith("LOGICAL")
    out = run_pointwise(ctx, mode, [a, b], capi.BOOLEAN if boolean else capi.FLOAT)
    ref = oracle.pointwise(capi.PW[mode], [a.logical(), b.logical()])
    if boolean:
        assert np.array_equal(out.logical(), ref.astype(np.int64))
    else:
        assert_close(out.logical(), ref, capi.FLOAT, mode)


def test_pointwise_add_transposed_known_answer(ctx):
    # samples/pointwise/pointwise_add_transposed.cpp:22-112: a = {1..6} as 3x2
    # row-major, b = same bytes viewed with dim {3,2} stride {1,3}.
    data = np.arange(1, 7, dtype=np.float32)
    a = HT([3, 2], [2, 1], capi.FLOAT, data.copy())
    b = HT([3, 2], [1, 3], capi.FLOAT, data.copy())
    out = run_pointwise(ctx, "ADD", [a, b], capi.FLOAT)
    assert out.storage.tolist() == [2, 6, 5, 9, 8, 12]


def test_pointwise_scalar_mul_known_answer(ctx):
    # samples/pointwise/pointwise_scalar_mul.cpp:22-78: 3 * 2 = 6, the scalar is
    # a constant, not a buffer.
    a = HT.from_logical(np.full([2, 5], 3.0), capi.FLOAT)
    out = run_pointwise(ctx, "MUL", [a, None], capi.FLOAT, scalars={1: 2.0})
    assert np.all(out.logical() == 6.0)


def test_pointwise_int32_add_and_select(ctx):
    # samples/aot/single_backend.cpp:52-110: int32 2 + 3 = 5.
    a = HT.from_logical(np.full([4, 4], 2), capi.INT32)
    b = HT.from_logical(np.full([4, 4], 3), capi.INT32)
    assert np.all(run_pointwise(ctx, "ADD", [a, b], capi.INT32).logical() == 5)
    big = HT.from_logical(np.full([4, 4], 2_000_000_011), capi.INT32)
    assert np.all(run_pointwise(ctx, "IDENTITY", [big], capi.INT32).logical()
                  == 2_000_000_011)
    cond = HT.from_logical(np.eye(4), capi.BOOLEAN)
    sel = run_pointwise(ctx, "BINARY_SELECT", [cond, a, b], capi.INT32).logical()
    assert np.array_equal(sel, np.where(np.eye(4) != 0, 2, 3))
