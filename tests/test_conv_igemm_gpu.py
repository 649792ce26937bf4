"""Implicit-GEMM convolution (MFMA kernel) through the C ABI vs the oracle.

Shapes here satisfy the tuned kernel's contract (channels-last bf16/f16,
C a multiple of 8 -- channel counts that are no multiple of 64 run on
zero-padded copies --, one group or groups of a multiple of 64 channels); each test asserts that the tuned kernel is
the one chosen, so a silent fall back to the generic kernel fails.
"""
import numpy as np
import pytest

from fusilli_amd import capi
from oracle import oracle
from helpers import HT, assert_close, rand

pytestmark = pytest.mark.gpu


def conv_desc(x, w, out, pad, stride, dil, y_dtype, epilogue=()):
    d = capi.ConvDesc()
    d.x, d.w = x.desc(), w.desc()
    d.y = capi.TensorDesc.make(out.dims, out.strides, y_dtype)
    d.out = out.desc()
    d.out_dtype = out.dtype
    d.spatial_rank = len(pad)
    for i in range(len(pad)):
        d.padding[i], d.stride[i], d.dilation[i] = pad[i], stride[i], dil[i]
    d.epilogue = capi.make_epilogue(list(epilogue))
    return d


def run(ctx, x, w, pad, stride, dil, y_dtype, out_dtype=None, epilogue=(),
        epi_tensors=(), expect_tuned=True):
    ydims = oracle.conv_output_dims(x.dims, w.dims, pad, stride, dil)
    out = HT.empty(ydims, y_dtype if out_dtype is None else out_dtype,
                   oracle.channels_last_strides(ydims))
    d = conv_desc(x, w, out, pad, stride, dil, y_dtype, epilogue)
    assert ctx.lib.fhip_conv_fprop_supported(d) == (2 if expect_tuned else 1)
    bufs = [t.upload(ctx) for t in epi_tensors]
    dx, dw, dout = x.upload(ctx), w.upload(ctx), out.upload(ctx)
    ctx.conv_fprop(d, dx, dw, dout, epilogue_operands=bufs)
    return out.fetch(ctx, dout)


def cl(dims, seed, tid, dtype, std=1.0):
    return HT.from_logical(rand(seed, tid, dims, std=std), dtype,
                           oracle.channels_last_strides(dims))


CASES = [
    # 3x3 same padding, the shape family of the headline conv config
    dict(x=[2, 64, 14, 14], w=[128, 64, 3, 3], pad=[1, 1], s=[1, 1], d=[1, 1]),
    # ragged M (2*7*5 = 70 pixels) and ragged K_out, stride 2
    dict(x=[2, 64, 13, 9], w=[40, 64, 3, 3], pad=[1, 1], s=[2, 2], d=[1, 1]),
    # dilation 2 with asymmetric padding / stride, C = 128 (two K slices per tap)
    dict(x=[1, 128, 17, 12], w=[136, 128, 3, 2], pad=[2, 1], s=[1, 2], d=[2, 2]),
    # 1x1 (pure GEMM), many pixels, > 256 output channels
    dict(x=[3, 192, 12, 12], w=[264, 192, 1, 1], pad=[0, 0], s=[1, 1], d=[1, 1]),
    # 5x5 filter larger than the padded border reach, no padding
    dict(x=[1, 64, 11, 11], w=[64, 64, 5, 5], pad=[0, 0], s=[1, 1], d=[1, 1]),
    # padding wider than the filter reach (all-zero taps at the border)
    dict(x=[1, 64, 6, 6], w=[32, 64, 3, 3], pad=[3, 3], s=[1, 1], d=[1, 1]),
    # 1-D convolution
    dict(x=[2, 64, 50], w=[48, 64, 5], pad=[2], s=[2], d=[1]),
]


RESHAPED_CASES = [
    # channel counts that are no multiple of 64 run on zero-padded copies: the
    # reference's NHWC benchmark shape (C = K = 48, 3 x 3, padding 2, dilation 2
    # or 1), a wider one with a ragged channel tail, 1-D
    dict(x=[3, 48, 20, 16], w=[48, 48, 3, 3], pad=[2, 2], s=[1, 1], d=[2, 2]),
    dict(x=[2, 48, 20, 16], w=[48, 48, 3, 3], pad=[2, 2], s=[1, 1], d=[1, 1]),
    # (that shape at full size, as the benchmark line runs it)
    dict(x=[16, 48, 48, 32], w=[48, 48, 3, 3], pad=[2, 2], s=[1, 1], d=[1, 1]),
    dict(x=[2, 200, 9, 7], w=[72, 200, 2, 3], pad=[1, 0], s=[2, 1], d=[1, 1]),
    dict(x=[2, 24, 70], w=[40, 24, 5], pad=[2], s=[1], d=[1]),
    # 3-D convolutions with a 1 x 1 filter in H and W fold into 2-D ones: the
    # reference's NDHWC benchmark shape class (depth filter 2, depth stride 2),
    # with and without a channel tail, with depth padding and dilation
    dict(x=[2, 288, 2, 12, 8], w=[96, 288, 2, 1, 1], pad=[0, 0, 0], s=[2, 1, 1], d=[1, 1, 1]),
    dict(x=[2, 64, 5, 6, 10], w=[136, 64, 3, 1, 1], pad=[1, 0, 0], s=[1, 1, 1], d=[1, 1, 1]),
    dict(x=[1, 40, 7, 5, 9], w=[24, 40, 2, 1, 1], pad=[2, 0, 0], s=[2, 1, 1], d=[2, 1, 1]),
]


@pytest.mark.parametrize("case", RESHAPED_CASES)
@pytest.mark.parametrize("dtype", [capi.BFLOAT16, capi.HALF])
@pytest.mark.parametrize("bias", [False, True])
def test_conv_padded_channels_and_folded_3d_vs_oracle(ctx, case, dtype, bias):
    x = cl(case["x"], 43, 0, dtype)
    w = cl(case["w"], 43, 1, dtype, std=0.1)
    ref = oracle.conv_fprop(x.logical(), w.logical(), case["pad"], case["s"],
                            case["d"])
    if not bias:
        out = run(ctx, x, w, case["pad"], case["s"], case["d"], dtype)
        assert_close(out.logical(), ref, dtype, str(case))
        return
    k = case["w"][0]
    bd = [1, k] + [1] * (len(case["x"]) - 2)
    b = HT.from_logical(rand(43, 2, bd), dtype)
    out = run(ctx, x, w, case["pad"], case["s"], case["d"], capi.FLOAT,
              out_dtype=dtype,
              epilogue=[capi.epilogue_op(capi.PW["ADD"], dtype, operand_index=0,
                                         operand=b.desc())],
              epi_tensors=[b])
    assert_close(out.logical(), ref + b.logical(), dtype, f"{case} + bias")


@pytest.mark.parametrize("case", CASES)
@pytest.mark.parametrize("dtype", [capi.BFLOAT16, capi.HALF])
def test_conv_igemm_random_vs_oracle(ctx, case, dtype):
    x = cl(case["x"], 41, 0, dtype)
    w = cl(case["w"], 41, 1, dtype, std=0.1)
    out = run(ctx, x, w, case["pad"], case["s"], case["d"], dtype)
    ref = oracle.conv_fprop(x.logical(), w.logical(), case["pad"], case["s"],
                            case["d"])
    assert_close(out.logical(), ref, dtype, str(case))


@pytest.mark.parametrize("tile", ["128,128", "256,128", "256,256", "512,128"])
def test_conv_igemm_every_tile_shape(ctx, tile, knobs):
    knobs(CONV_TILE=tile, CONV_HALO="0", CONV_ROWS="0")  # the gather kernel's tiles
    case = dict(x=[2, 64, 15, 17], w=[300, 64, 3, 3], pad=[1, 1], s=[1, 1], d=[1, 1])
    x = cl(case["x"], 42, 0, capi.BFLOAT16)
    w = cl(case["w"], 42, 1, capi.BFLOAT16, std=0.1)
    out = run(ctx, x, w, case["pad"], case["s"], case["d"], capi.FLOAT)
    ref = oracle.conv_fprop(x.logical(), w.logical(), case["pad"], case["s"],
                            case["d"])
    # f32 result of bf16 inputs: only the accumulation order differs
    assert_close(out.logical(), ref, capi.FLOAT, tile, rtol=1e-4)


SAME_CASES = [
    # unit stride, output extent == input extent: eligible for the halo kernel
    dict(x=[2, 64, 14, 14], w=[128, 64, 3, 3], pad=[1, 1], d=[1, 1]),
    # ragged M (3*9*11 = 297 pixels: 2 full tiles + 41 rows), ragged K_out > 128
    dict(x=[3, 64, 9, 11], w=[200, 64, 3, 3], pad=[1, 1], d=[1, 1]),
    # dilation 2 (reach 2 rows + 2 pixels either side)
    dict(x=[1, 64, 12, 10], w=[64, 64, 3, 3], pad=[2, 2], d=[2, 2]),
    # 5x5, C = 128 (two K slices per tap)
    dict(x=[1, 128, 9, 9], w=[48, 128, 5, 5], pad=[2, 2], d=[1, 1]),
    # asymmetric filter 1x3 and 3x1
    dict(x=[2, 64, 8, 16], w=[32, 64, 1, 3], pad=[0, 1], d=[1, 1]),
    dict(x=[2, 64, 16, 8], w=[32, 64, 3, 1], pad=[1, 0], d=[1, 1]),
    # 1x1 (no halo at all) and 1-D
    dict(x=[2, 64, 10, 13], w=[136, 64, 1, 1], pad=[0, 0], d=[1, 1]),
    dict(x=[3, 64, 70], w=[48, 64, 5], pad=[2], d=[1]),
    # image narrower than the filter reach
    dict(x=[4, 64, 2, 3], w=[16, 64, 3, 3], pad=[1, 1], d=[1, 1]),
]


@pytest.mark.parametrize("case", SAME_CASES)
@pytest.mark.parametrize("halo", ["128", "256", "0"])
@pytest.mark.parametrize("dtype", [capi.BFLOAT16, capi.HALF])
def test_conv_same_geometry_halo_and_gather(ctx, case, halo, dtype, knobs):
    knobs(CONV_HALO=halo, CONV_ROWS="0")
    st = [1] * len(case["pad"])
    x = cl(case["x"], 46, 0, dtype)
    w = cl(case["w"], 46, 1, dtype, std=0.1)
    out = run(ctx, x, w, case["pad"], st, case["d"], capi.FLOAT)
    ref = oracle.conv_fprop(x.logical(), w.logical(), case["pad"], st, case["d"])
    assert_close(out.logical(), ref, capi.FLOAT, f"halo={halo} {case}", rtol=1e-4)


@pytest.mark.parametrize("xd,wd,split", [
    ([2, 128, 10, 12], [136, 128, 1, 1], False),   # ragged columns, 240 pixels
    ([4, 2048, 7, 7], [256, 2048, 1, 1], True),    # long reduction: cut into parts
    ([3, 192, 60], [128, 192, 1], False),          # 1-D
])
def test_conv_single_tap_as_matrix_product_fused_operands(ctx, xd, wd, split):
    """1 x 1 filters at unit stride are handed to the GEMM entry; the fused
    per-channel and per-pixel operands keep their conv layouts (bias[K],
    residual[N, K, ...] channels-last), also through the split reduction."""
    sp = len(xd) - 2
    pad, one = [0] * sp, [1] * sp
    x = cl(xd, 48, 0, capi.BFLOAT16)
    w = cl(wd, 48, 1, capi.BFLOAT16, std=0.05)
    yd = oracle.conv_output_dims(xd, wd, pad, one, one)
    bd = [1, wd[0]] + one
    bias = HT.from_logical(rand(48, 2, bd), capi.BFLOAT16, oracle.channels_last_strides(bd))
    res = cl(yd, 48, 3, capi.BFLOAT16)
    epi = [capi.epilogue_op(capi.PW["ADD"], capi.FLOAT, operand_index=0, operand=bias.desc()),
           capi.epilogue_op(capi.PW["RELU_FWD"], capi.FLOAT),
           capi.epilogue_op(capi.PW["ADD"], capi.BFLOAT16, operand_index=1, operand=res.desc())]
    out = run(ctx, x, w, pad, one, one, capi.FLOAT, out_dtype=capi.BFLOAT16, epilogue=epi,
              epi_tensors=[bias, res])
    name = ctx.last_kernel()
    assert name.startswith("conv_igemm as gemm_mfma bf16"), name
    assert name.endswith("split=1") != split, name
    ref = oracle.conv_fprop(x.logical(), w.logical(), pad, one, one)
    ref = np.maximum(ref + bias.logical(), 0.0) + res.logical()
    assert_close(out.logical(), ref, capi.BFLOAT16)
    out = run(ctx, x, w, pad, one, one, capi.FLOAT)
    assert_close(out.logical(), oracle.conv_fprop(x.logical(), w.logical(), pad, one, one),
                 capi.FLOAT, rtol=1e-4)


def test_conv_igemm_bias_relu_residual(ctx):
    # conv -> +bias[K] -> relu -> +residual[N,K,P,Q] (channels-last) -> bf16
    xd, wd = [2, 64, 10, 12], [96, 64, 3, 3]
    x = cl(xd, 43, 0, capi.BFLOAT16)
    w = cl(wd, 43, 1, capi.BFLOAT16, std=0.1)
    yd = oracle.conv_output_dims(xd, wd, [1, 1], [1, 1], [1, 1])
    bias = HT.from_logical(rand(43, 2, [1, 96, 1, 1]), capi.BFLOAT16,
                           oracle.channels_last_strides([1, 96, 1, 1]))
    res = cl(yd, 43, 3, capi.BFLOAT16)
    epi = [capi.epilogue_op(capi.PW["ADD"], capi.FLOAT, operand_index=0,
                            operand=bias.desc()),
           capi.epilogue_op(capi.PW["RELU_FWD"], capi.FLOAT),
           capi.epilogue_op(capi.PW["ADD"], capi.BFLOAT16, operand_index=1,
                            operand=res.desc())]
    out = run(ctx, x, w, [1, 1], [1, 1], [1, 1], capi.FLOAT,
              out_dtype=capi.BFLOAT16, epilogue=epi, epi_tensors=[bias, res])
    ref = oracle.conv_fprop(x.logical(), w.logical(), [1, 1], [1, 1], [1, 1])
    ref = np.maximum(ref + bias.logical(), 0.0) + res.logical()
    assert_close(out.logical(), ref, capi.BFLOAT16)


GROUPED_CASES = [
    # two groups of 64 -> 64 channels, same geometry (halo tiles, 64 wide)
    dict(x=[2, 128, 9, 11], w=[128, 64, 3, 3], pad=[1, 1], s=[1, 1], d=[1, 1]),
    # four groups of 64 -> 24 channels (ragged columns), stride 2 (gather)
    dict(x=[2, 256, 8, 8], w=[96, 64, 3, 3], pad=[1, 1], s=[2, 2], d=[1, 1]),
    # three groups of 128 -> 136 channels (two column tiles per group), 1x1
    dict(x=[1, 384, 7, 6], w=[408, 128, 1, 1], pad=[0, 0], s=[1, 1], d=[1, 1]),
    # 1-D, two groups of 64 -> 16, dilation 2
    dict(x=[3, 128, 40], w=[32, 64, 5], pad=[4], s=[1], d=[2]),
    # many groups: 16 groups of 64 -> 8 channels
    dict(x=[1, 1024, 6, 5], w=[128, 64, 3, 3], pad=[1, 1], s=[1, 1], d=[1, 1]),
]


@pytest.mark.parametrize("case", GROUPED_CASES)
@pytest.mark.parametrize("halo", ["auto", "0"])
@pytest.mark.parametrize("dtype", [capi.BFLOAT16, capi.HALF])
def test_conv_grouped_vs_oracle(ctx, case, halo, dtype, knobs):
    # Reference: conv with groups = C / filter channels (aten.convolution's
    # groups operand, reference support/asm_emitter.h:690-701).  One GEMM per
    # group on the MFMA kernels; the fused bias is indexed by the channel of
    # the whole output, not of the group.
    if halo != "auto":
        knobs(CONV_HALO=halo)
    x = cl(case["x"], 48, 0, dtype)
    w = cl(case["w"], 48, 1, dtype, std=0.1)
    k = case["w"][0]
    bdims = [1, k] + [1] * len(case["pad"])
    bias = HT.from_logical(rand(48, 2, bdims), dtype, oracle.channels_last_strides(bdims))
    epi = [capi.epilogue_op(capi.PW["ADD"], capi.FLOAT, operand_index=0, operand=bias.desc()),
           capi.epilogue_op(capi.PW["RELU_FWD"], capi.FLOAT)]
    out = run(ctx, x, w, case["pad"], case["s"], case["d"], capi.FLOAT, out_dtype=dtype,
              epilogue=epi, epi_tensors=[bias])
    ref = oracle.conv_fprop(x.logical(), w.logical(), case["pad"], case["s"], case["d"])
    ref = np.maximum(ref + bias.logical(), 0.0)
    assert_close(out.logical(), ref, dtype, f"halo={halo} {case}")
    # no epilogue, f32 out
    out = run(ctx, x, w, case["pad"], case["s"], case["d"], capi.FLOAT)
    ref = oracle.conv_fprop(x.logical(), w.logical(), case["pad"], case["s"], case["d"])
    assert_close(out.logical(), ref, capi.FLOAT, f"halo={halo} {case}", rtol=1e-4)


SPLIT_CASES = [
    # few output pixels and a long reduction: the K slices are cut into parts
    # on workgroups of their own and a second kernel adds them
    dict(x=[2, 512, 7, 7], w=[512, 512, 3, 3], pad=[1, 1], s=[1, 1], d=[1, 1]),    # 8 parts
    dict(x=[2, 1024, 5, 5], w=[64, 1024, 1, 1], pad=[0, 0], s=[1, 1], d=[1, 1]),   # 2 parts
    dict(x=[3, 192, 9, 9], w=[40, 192, 3, 3], pad=[0, 0], s=[2, 2], d=[1, 1]),     # ragged tile, stride
    dict(x=[1, 256, 40], w=[72, 256, 5], pad=[2], s=[1], d=[1]),                   # 1-D
]


@pytest.mark.parametrize("case", SPLIT_CASES)
@pytest.mark.parametrize("dtype", [capi.BFLOAT16, capi.HALF])
def test_conv_split_reduction_vs_oracle(ctx, case, dtype, knobs):
    knobs(CONV_HALO="0")  # the gather kernel (the halo kernel does not split)
    x = cl(case["x"], 50, 0, dtype)
    w = cl(case["w"], 50, 1, dtype, std=0.05)
    k = case["w"][0]
    bdims = [1, k] + [1] * len(case["pad"])
    bias = HT.from_logical(rand(50, 2, bdims), dtype, oracle.channels_last_strides(bdims))
    epi = [capi.epilogue_op(capi.PW["ADD"], capi.FLOAT, operand_index=0, operand=bias.desc()),
           capi.epilogue_op(capi.PW["RELU_FWD"], capi.FLOAT)]
    out = run(ctx, x, w, case["pad"], case["s"], case["d"], capi.FLOAT, out_dtype=dtype,
              epilogue=epi, epi_tensors=[bias])
    ref = oracle.conv_fprop(x.logical(), w.logical(), case["pad"], case["s"], case["d"])
    assert_close(out.logical(), np.maximum(ref + bias.logical(), 0.0), dtype, f"{case}")
    out = run(ctx, x, w, case["pad"], case["s"], case["d"], capi.FLOAT)
    assert_close(out.logical(), ref, capi.FLOAT, f"{case}", rtol=1e-4)


SPLIT_OPERAND_CASES = [
    # 2-D, split reduction
    dict(x=[2, 512, 7, 7], w=[128, 512, 3, 3], pad=[1, 1], s=[1, 1], d=[1, 1]),
    # 3-D with a 1 x 1 filter in H and W (folded into 2-D) and a split reduction
    dict(x=[2, 512, 4, 7, 7], w=[128, 512, 3, 1, 1], pad=[1, 0, 0], s=[1, 1, 1], d=[1, 1, 1]),
    dict(x=[8, 512, 4, 7, 7], w=[512, 512, 3, 1, 1], pad=[1, 0, 0], s=[1, 1, 1], d=[1, 1, 1]),
]


@pytest.mark.parametrize("case", SPLIT_OPERAND_CASES)
@pytest.mark.parametrize("operand", ["bias", "residual", "bias_relu_residual"])
def test_conv_split_reduction_fused_operands(ctx, case, operand, knobs):
    """Fused operands on the split-reduction path, whose second kernel applies
    them: a per-channel vector, a tensor of the output's shape (residual add,
    addressed by pixel), and both around a ReLU; 2-D and folded 3-D problems.
    Reference: pointwise nodes consuming the convolution's output
    (reference samples/convolution/conv_fprop_with_relu_and_bias.cpp)."""
    knobs(CONV_HALO="0")
    dt = capi.BFLOAT16
    x = cl(case["x"], 61, 0, dt)
    w = cl(case["w"], 61, 1, dt, std=0.05)
    yd = oracle.conv_output_dims(case["x"], case["w"], case["pad"], case["s"], case["d"])
    bd = [1, case["w"][0]] + [1] * len(case["pad"])
    bias = HT.from_logical(rand(61, 2, bd), dt, oracle.channels_last_strides(bd))
    res = cl(yd, 61, 3, dt)
    ref = oracle.conv_fprop(x.logical(), w.logical(), case["pad"], case["s"], case["d"])
    add = lambda t, i, rd=capi.FLOAT: capi.epilogue_op(capi.PW["ADD"], rd, operand_index=i,
                                                       operand=t.desc())
    if operand == "bias":
        epi, tensors, ref = [add(bias, 0)], [bias], ref + bias.logical()
    elif operand == "residual":
        epi, tensors, ref = [add(res, 0)], [res], ref + res.logical()
    else:
        epi = [add(bias, 0), capi.epilogue_op(capi.PW["RELU_FWD"], capi.FLOAT), add(res, 1)]
        tensors = [bias, res]
        ref = np.maximum(ref + bias.logical(), 0.0) + res.logical()
    out = run(ctx, x, w, case["pad"], case["s"], case["d"], capi.FLOAT, out_dtype=dt,
              epilogue=epi, epi_tensors=tensors)
    assert "split=" in ctx.last_kernel() and "split=1" not in ctx.last_kernel(), ctx.last_kernel()
    assert_close(out.logical(), ref, dt, f"{operand} {case}")


def test_conv_split_reduction_benchmark_shape(ctx):
    """N32 C512 7x7 -> K512, 3x3, padding 1, bf16 at full size (the
    benchmark's late-layer line): closed form on all-ones tensors for every
    pixel, the oracle on the first and last image for random ones."""
    xd, wd = [32, 512, 7, 7], [512, 512, 3, 3]
    pad, st, dil = [1, 1], [1, 1], [1, 1]
    ones_x = HT.from_logical(np.ones(xd), capi.BFLOAT16, oracle.channels_last_strides(xd))
    ones_w = HT.from_logical(np.ones(wd), capi.BFLOAT16, oracle.channels_last_strides(wd))
    lg = run(ctx, ones_x, ones_w, pad, st, dil, capi.FLOAT, out_dtype=capi.BFLOAT16).logical()
    assert ctx.last_kernel().startswith("conv_igemm gather") and "split=8" in ctx.last_kernel(), \
        ctx.last_kernel()
    taps = np.full(7, 3.0); taps[[0, -1]] = 2.0
    assert np.array_equal(lg, np.broadcast_to(512.0 * taps[:, None] * taps[None, :], lg.shape))
    x = cl(xd, 51, 0, capi.BFLOAT16)
    w = cl(wd, 51, 1, capi.BFLOAT16, std=0.02)
    lg = run(ctx, x, w, pad, st, dil, capi.FLOAT, out_dtype=capi.BFLOAT16).logical()
    for img in (0, 31):
        ref = oracle.conv_fprop(x.logical()[img:img + 1], w.logical(), pad, st, dil)
        assert_close(lg[img:img + 1], ref, capi.BFLOAT16, f"image {img}")


def test_conv_igemm_not_chosen_outside_contract(ctx):
    # C = 44 (not whole 16-byte chunks per pixel) and groups of 32 channels
    # (half a K slice) keep the generic kernel
    x = cl([1, 44, 8, 8], 44, 0, capi.BFLOAT16)
    w = cl([16, 44, 3, 3], 44, 1, capi.BFLOAT16, std=0.1)
    out = run(ctx, x, w, [1, 1], [1, 1], [1, 1], capi.BFLOAT16, expect_tuned=False)
    ref = oracle.conv_fprop(x.logical(), w.logical(), [1, 1], [1, 1], [1, 1])
    assert_close(out.logical(), ref, capi.BFLOAT16)
    x = cl([1, 128, 8, 8], 44, 2, capi.BFLOAT16)
    w = cl([16, 32, 3, 3], 44, 3, capi.BFLOAT16, std=0.1)
    out = run(ctx, x, w, [1, 1], [1, 1], [1, 1], capi.BFLOAT16, expect_tuned=False)
    ref = oracle.conv_fprop(x.logical(), w.logical(), [1, 1], [1, 1], [1, 1])
    assert_close(out.logical(), ref, capi.BFLOAT16)


def test_conv_igemm_headline_shape(ctx):
    """N32 C64 56x56, K128 3x3 pad 1, bf16, + bias + ReLU at full size.

    All-ones input and filter give closed-form answers (64 channels times the
    number of in-image taps); random data is checked against the oracle on the
    first and last image (the convolution is independent per image)."""
    xd, wd = [32, 64, 56, 56], [128, 64, 3, 3]
    pad, st, dil = [1, 1], [1, 1], [1, 1]
    bias = HT.from_logical(rand(45, 2, [1, 128, 1, 1]), capi.BFLOAT16,
                           oracle.channels_last_strides([1, 128, 1, 1]))
    epi = [capi.epilogue_op(capi.PW["ADD"], capi.FLOAT, operand_index=0,
                            operand=bias.desc()),
           capi.epilogue_op(capi.PW["RELU_FWD"], capi.BFLOAT16)]
    ones_x = HT.from_logical(np.ones(xd), capi.BFLOAT16, oracle.channels_last_strides(xd))
    ones_w = HT.from_logical(np.ones(wd), capi.BFLOAT16, oracle.channels_last_strides(wd))
    out = run(ctx, ones_x, ones_w, pad, st, dil, capi.FLOAT, out_dtype=capi.BFLOAT16)
    lg = out.logical()
    taps_h = np.full(56, 3.0); taps_h[[0, -1]] = 2.0
    expect = 64.0 * taps_h[:, None] * taps_h[None, :]
    assert np.array_equal(lg, np.broadcast_to(expect, lg.shape))

    x = cl(xd, 45, 0, capi.BFLOAT16)
    w = cl(wd, 45, 1, capi.BFLOAT16, std=0.05)
    out = run(ctx, x, w, pad, st, dil, capi.FLOAT, out_dtype=capi.BFLOAT16,
              epilogue=epi, epi_tensors=[bias])
    # the kernel that the benchmark's headline convolution line times
    assert ctx.last_kernel().startswith("conv_rf c=64 r=3 s=3"), ctx.last_kernel()
    lg = out.logical()
    xl = x.logical()
    for img in (0, 31):
        ref = oracle.conv_fprop(xl[img:img + 1], w.logical(), pad, st, dil)
        ref = np.maximum(ref + bias.logical(), 0.0)
        assert_close(lg[img:img + 1], ref, capi.BFLOAT16, f"image {img}")

    # Every workgroup slot: the same random image in all 32 batch entries must
    # give 32 bit-identical outputs, and image 0's has just been compared with
    # the oracle's arithmetic on the same kernel.
    xs = np.broadcast_to(rand(45, 3, [1] + xd[1:]), xd)
    x = HT.from_logical(xs, capi.BFLOAT16, oracle.channels_last_strides(xd))
    out = run(ctx, x, w, pad, st, dil, capi.FLOAT, out_dtype=capi.BFLOAT16,
              epilogue=epi, epi_tensors=[bias])
    lg = out.logical()
    ref = oracle.conv_fprop(x.logical()[:1], w.logical(), pad, st, dil)
    assert_close(lg[:1], np.maximum(ref + bias.logical(), 0.0), capi.BFLOAT16, "shared image")
    for img in range(1, 32):
        assert np.array_equal(lg[img], lg[0]), f"image {img} differs from image 0"


LARGE_128_CASES = [
    # 784 tiles of 128 x 128: 3x3 (halo-eligible), 1x1 reduction, 1x1 stride 2
    dict(x=[32, 128, 56, 56], w=[128, 128, 3, 3], pad=[1, 1], s=[1, 1]),
    dict(x=[32, 256, 56, 56], w=[64, 256, 1, 1], pad=[0, 0], s=[1, 1]),
    dict(x=[32, 64, 112, 112], w=[64, 64, 1, 1], pad=[0, 0], s=[2, 2]),
    # 1x1 at unit stride with 128 output channels: a plain matrix product
    dict(x=[32, 256, 56, 56], w=[128, 256, 1, 1], pad=[0, 0], s=[1, 1]),
]


@pytest.mark.parametrize("case", LARGE_128_CASES)
def test_conv_many_128_wide_tiles_take_the_gather_tile(ctx, case):
    """The 56 x 56 layers with up to 128 output channels: 512 or more tiles of
    128 x 128 run on the gather kernel's eight-wavefront tile, also where the
    halo kernel could take them (1 x 1 filters at unit stride: the GEMM entry).  All-ones operands have closed-form answers at
    every output; random data is checked against the oracle on the first and
    the last image."""
    xd, wd, pad, st = case["x"], case["w"], case["pad"], case["s"]
    dil = [1, 1]
    ones_x = HT.from_logical(np.ones(xd), capi.BFLOAT16, oracle.channels_last_strides(xd))
    ones_w = HT.from_logical(np.ones(wd), capi.BFLOAT16, oracle.channels_last_strides(wd))
    out = run(ctx, ones_x, ones_w, pad, st, dil, capi.FLOAT, out_dtype=capi.BFLOAT16)
    # (a single tap at unit stride is handed to the GEMM entry as it lies)
    want = "conv_igemm as gemm_mfma bf16" if wd[2] == 1 and st == [1, 1] and wd[0] >= 128 \
        else "conv_igemm gather 128x128 split=1"
    assert ctx.last_kernel().startswith(want), ctx.last_kernel()
    lg = out.logical()
    if wd[2] == 3:
        taps = np.full(xd[2], 3.0); taps[[0, -1]] = 2.0
        expect = wd[1] * taps[:, None] * taps[None, :]
    else:
        expect = np.full(lg.shape[2:], float(wd[1]))
    assert np.array_equal(lg, np.broadcast_to(expect, lg.shape))

    x = cl(xd, 47, 0, capi.BFLOAT16)
    w = cl(wd, 47, 1, capi.BFLOAT16, std=0.05)
    out = run(ctx, x, w, pad, st, dil, capi.FLOAT, out_dtype=capi.BFLOAT16)
    lg, xl = out.logical(), x.logical()
    for img in (0, xd[0] - 1):
        ref = oracle.conv_fprop(xl[img:img + 1], w.logical(), pad, st, dil)
        assert_close(lg[img:img + 1], ref, capi.BFLOAT16, f"{case} image {img}")


@pytest.mark.parametrize("shape", ["groups4", "depthwise"])
def test_conv_grouped_benchmark_shapes(ctx, shape):
    """The two grouped lines of the benchmark at full size (N32 56x56, 3x3,
    padding 1, bf16): 4 groups of 64 -> 64 channels on the register-filter
    kernel (two groups per workgroup) and a
    depthwise convolution over 128 channels on the small-group kernel.
    All-ones tensors have closed-form answers (channels of a group times the
    taps inside the image) on every pixel; random data is checked against the
    oracle on the first and last image."""
    c, cg = (256, 64) if shape == "groups4" else (128, 1)
    xd, wd = [32, c, 56, 56], [c, cg, 3, 3]
    pad, st, dil = [1, 1], [1, 1], [1, 1]
    ones_x = HT.from_logical(np.ones(xd), capi.BFLOAT16, oracle.channels_last_strides(xd))
    ones_w = HT.from_logical(np.ones(wd), capi.BFLOAT16, oracle.channels_last_strides(wd))
    lg = run(ctx, ones_x, ones_w, pad, st, dil, capi.FLOAT, out_dtype=capi.BFLOAT16).logical()
    if shape == "groups4":
        assert ctx.last_kernel().startswith("conv_rf c=64 r=3 s=3") and \
            ctx.last_kernel().endswith("groups_per_wg=2"), ctx.last_kernel()
    taps = np.full(56, 3.0); taps[[0, -1]] = 2.0
    expect = float(cg) * taps[:, None] * taps[None, :]
    assert np.array_equal(lg, np.broadcast_to(expect, lg.shape))
    x = cl(xd, 49, 0, capi.BFLOAT16)
    w = cl(wd, 49, 1, capi.BFLOAT16, std=0.1)
    lg = run(ctx, x, w, pad, st, dil, capi.FLOAT, out_dtype=capi.BFLOAT16).logical()
    xl = x.logical()
    for img in (0, 31):
        ref = oracle.conv_fprop(xl[img:img + 1], w.logical(), pad, st, dil)
        assert_close(lg[img:img + 1], ref, capi.BFLOAT16, f"{shape} image {img}")


# ---- register-filter kernel (3 x 3 x 64 filters, unit stride, K % 128 == 0) -----
RF_CASES = [
    # rows per tile forced (CONV_ROWS): image geometry, channels
    # width not a multiple of 16, rows not a multiple of the tile height
    dict(x=[2, 64, 13, 21], k=128, pad=[1, 1], rows=4),
    # one row per tile (halo rows dominate), two channel groups
    dict(x=[1, 64, 9, 17], k=256, pad=[1, 1], rows=1),
    # no padding: output smaller than input
    dict(x=[3, 64, 12, 19], k=128, pad=[0, 0], rows=5),
    # padding 2: output larger than input, rows of zeros above and below
    dict(x=[2, 64, 7, 30], k=128, pad=[2, 2], rows=3),
    # asymmetric padding
    dict(x=[2, 64, 10, 16], k=128, pad=[0, 2], rows=8),
    # more tiles than compute units: workgroups walk several tiles
    dict(x=[40, 64, 16, 8], k=128, pad=[1, 1], rows=2),
    # whole image per tile, a single group of blocks and a ragged one
    dict(x=[2, 64, 6, 11], k=128, pad=[1, 1], rows=6),
    # wide image (several KB of slab per row)
    dict(x=[1, 64, 5, 100], k=128, pad=[1, 1], rows=2),
]


@pytest.mark.parametrize("case", RF_CASES)
@pytest.mark.parametrize("dtype", [capi.BFLOAT16, capi.HALF])
@pytest.mark.parametrize("epi_kind", ["bias_relu", "none", "scale_bias"])
@pytest.mark.parametrize("slices", [4, 2])
def test_conv_register_filter_kernel_vs_oracle(ctx, knobs, case, dtype, epi_kind, slices):
    # slices: 128 output channels per workgroup (two wavefronts per 32-channel
    # slice) or 64 (four per slice, the filter staged in the slab's place)
    xd, wd = case["x"], [case["k"], 64, 3, 3]
    pad, st, dil = case["pad"], [1, 1], [1, 1]
    x = cl(xd, 47, 0, dtype)
    w = cl(wd, 47, 1, dtype, std=0.05)
    bias = HT.from_logical(rand(47, 2, [1, case["k"], 1, 1]), dtype,
                           oracle.channels_last_strides([1, case["k"], 1, 1]))
    ref = oracle.conv_fprop(x.logical(), w.logical(), pad, st, dil)
    if epi_kind == "bias_relu":
        epi = [capi.epilogue_op(capi.PW["ADD"], capi.FLOAT, operand_index=0,
                                operand=bias.desc()),
               capi.epilogue_op(capi.PW["RELU_FWD"], dtype)]
        ops = [bias]
        ref = np.maximum(ref + bias.logical(), 0.0)
    elif epi_kind == "scale_bias":
        epi = [capi.epilogue_op(capi.PW["MUL"], capi.FLOAT, scalar=0.25),
               capi.epilogue_op(capi.PW["SUB"], dtype, operand_index=0,
                                operand=bias.desc())]
        ops = [bias]
        ref = ref * 0.25 - bias.logical()
    else:
        epi, ops = [], []
    got = {}
    for rows in (case["rows"], 0):  # the register-filter kernel, then the tiled one
        knobs(CONV_ROWS=rows, CONV_SLICES=slices)
        got[rows] = run(ctx, x, w, pad, st, dil, capi.FLOAT, out_dtype=dtype,
                        epilogue=epi, epi_tensors=ops).logical()
        if rows:
            name = ctx.last_kernel()
            assert name.startswith("conv_rf c=64 r=3 s=3") and \
                name.endswith("slices=2") == (slices == 2), name
        assert_close(got[rows], ref, dtype, f"rows={rows} slices={slices} {case} {epi_kind}")


def test_conv_register_filter_kernel_64_output_channels(ctx, knobs):
    # K = 64 (one pair of channel slices): only the two-slice variant applies;
    # workgroups walk runs of tiles that share halo rows in LDS
    xd, wd = [8, 64, 30, 24], [64, 64, 3, 3]
    x = cl(xd, 52, 0, capi.BFLOAT16)
    w = cl(wd, 52, 1, capi.BFLOAT16, std=0.05)
    ref = oracle.conv_fprop(x.logical(), w.logical(), [1, 1], [1, 1], [1, 1])
    for rows in (3, 7):
        knobs(CONV_ROWS=rows)
        got = run(ctx, x, w, [1, 1], [1, 1], [1, 1], capi.FLOAT, out_dtype=capi.BFLOAT16).logical()
        assert ctx.last_kernel().endswith("slices=2"), ctx.last_kernel()
        assert_close(got, ref, capi.BFLOAT16, f"rows={rows}")


RF_GROUPED_CASES = [
    # groups of 64 -> 64 channels, two per workgroup; rows per tile forced
    dict(x=[2, 128, 13, 21], pad=[1, 1], rows=4),   # one pair of groups
    dict(x=[1, 256, 9, 17], pad=[1, 1], rows=1),    # two pairs, one row per tile
    dict(x=[3, 384, 12, 19], pad=[0, 0], rows=5),   # three pairs, no padding
    dict(x=[40, 128, 16, 8], pad=[1, 1], rows=2),   # workgroups walk several tiles
    dict(x=[2, 256, 6, 50], pad=[1, 2], rows=2),    # wide rows, asymmetric padding
]


@pytest.mark.parametrize("case", RF_GROUPED_CASES)
@pytest.mark.parametrize("dtype", [capi.BFLOAT16, capi.HALF])
@pytest.mark.parametrize("epi_kind", ["bias_relu", "none"])
def test_conv_register_filter_kernel_grouped_vs_oracle(ctx, knobs, case, dtype, epi_kind):
    # Reference: aten.convolution's groups operand (reference
    # support/asm_emitter.h:690-701).  The same problem on the register-filter
    # kernel (two groups per workgroup) and on the tiled kernel (one GEMM per
    # group), both against the oracle; distinct random data per group, so a
    # slice reading the other group's half of a slab pixel cannot pass.
    xd = case["x"]
    k = xd[1]
    wd = [k, 64, 3, 3]
    pad, st, dil = case["pad"], [1, 1], [1, 1]
    x = cl(xd, 51, 0, dtype)
    w = cl(wd, 51, 1, dtype, std=0.05)
    bias = HT.from_logical(rand(51, 2, [1, k, 1, 1]), dtype,
                           oracle.channels_last_strides([1, k, 1, 1]))
    ref = oracle.conv_fprop(x.logical(), w.logical(), pad, st, dil)
    if epi_kind == "bias_relu":
        epi = [capi.epilogue_op(capi.PW["ADD"], capi.FLOAT, operand_index=0,
                                operand=bias.desc()),
               capi.epilogue_op(capi.PW["RELU_FWD"], dtype)]
        ops = [bias]
        ref = np.maximum(ref + bias.logical(), 0.0)
    else:
        epi, ops = [], []
    for rows in (case["rows"], 0):
        knobs(CONV_ROWS=rows)
        got = run(ctx, x, w, pad, st, dil, capi.FLOAT, out_dtype=dtype,
                  epilogue=epi, epi_tensors=ops).logical()
        name = ctx.last_kernel()
        assert ("groups_per_wg=2" in name) == (rows != 0), name
        assert_close(got, ref, dtype, f"rows={rows} {case} {epi_kind}")


def test_conv_register_filter_kernel_chosen_rows(ctx, knobs):
    # the planner's own tile height on a mid-sized problem (no knob), and the
    # all-ones closed form there: 64 channels x taps inside the image
    xd, wd = [16, 64, 28, 28], [256, 64, 3, 3]
    ones_x = HT.from_logical(np.ones(xd), capi.BFLOAT16, oracle.channels_last_strides(xd))
    ones_w = HT.from_logical(np.ones(wd), capi.BFLOAT16, oracle.channels_last_strides(wd))
    out = run(ctx, ones_x, ones_w, [1, 1], [1, 1], [1, 1], capi.FLOAT,
              out_dtype=capi.BFLOAT16).logical()
    taps = np.full(28, 3.0); taps[[0, -1]] = 2.0
    assert np.array_equal(out, np.broadcast_to(64.0 * taps[:, None] * taps[None, :],
                                               out.shape))
