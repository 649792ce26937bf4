"""The data gradient's entry point that allocates nothing
(fhip_conv_dgrad_static: scratch in a per-device static array inside the
library) against fhip_conv_dgrad with caller workspace: same kernels, so the
results must be identical bit for bit.  Two calls in a row, the second with a
smaller input, so stale scratch contents of the first call would show."""
import ctypes

import numpy as np
import pytest

from fusilli_amd import capi
from oracle import oracle
from helpers import HT, rand

pytestmark = pytest.mark.gpu

MAX_BYTES = 8 << 20  # FHIP_CONV_DGRAD_STATIC_MAX_BYTES


def _desc(dx, w, dy, pad, stride, dil):
    d = capi.ConvDesc()
    d.x, d.w, d.y = dx.desc(), w.desc(), dy.desc()
    d.spatial_rank = len(pad)
    for i in range(len(pad)):
        d.padding[i], d.stride[i], d.dilation[i] = pad[i], stride[i], dil[i]
    d.epilogue = capi.make_epilogue([])
    return d


def _both(ctx, case, dtype, seed):
    sp = len(case["pad"])
    st = case.get("s", [1] * sp)
    cl = oracle.channels_last_strides
    yd = oracle.conv_output_dims(case["x"], case["w"], case["pad"], st, case["d"])
    w = HT.from_logical(rand(seed, 1, case["w"], std=0.2), dtype, cl(case["w"]))
    dy = HT.from_logical(rand(seed, 2, yd), dtype, cl(yd))
    got = {}
    for which in ("workspace", "static"):
        dx = HT.empty(case["x"], dtype, cl(case["x"]))
        d = _desc(dx, w, dy, case["pad"], st, case["d"])
        assert ctx.lib.fhip_conv_dgrad_supported(d) == 2
        need = ctx.conv_dgrad_workspace(d)
        assert 0 < need <= MAX_BYTES
        bdy, bw, bdx = dy.upload(ctx), w.upload(ctx), dx.upload(ctx)
        if which == "workspace":
            ctx.conv_dgrad(d, bdy, bw, bdx)
        else:
            ctx.conv_dgrad_static(d, bdy, bw, bdx)
        got[which] = dx.fetch(ctx, bdx).logical()
    ref = oracle.conv_dgrad(dy.logical(), w.logical(), case["x"], case["pad"],
                            st, case["d"])
    return got, ref


def test_static_scratch_dgrad_matches_workspace_dgrad_twice(ctx):
    big = dict(x=[3, 64, 17, 13], w=[128, 64, 3, 3], pad=[1, 1], d=[1, 1])
    # smaller filter and image, strides above one: the zero grid of DY sits in
    # scratch that the first call filled with filter values
    small = dict(x=[2, 24, 11, 9], w=[64, 24, 2, 3], pad=[1, 1], d=[1, 1],
                 s=[2, 2])
    for seed, case in ((51, big), (52, small)):
        got, ref = _both(ctx, case, capi.BFLOAT16, seed)
        assert np.array_equal(got["static"], got["workspace"]), case
        ok, rep = oracle.check_close(got["static"], ref, 2e-2)
        assert ok, (case, rep)


def test_static_scratch_rejects_oversized_descriptor(ctx):
    # stride 2 over 8 x 128 x 127 x 127: the zero grid alone is far past 8 MiB
    case = dict(x=[8, 128, 127, 127], w=[128, 128, 3, 3], pad=[1, 1],
                d=[1, 1], s=[2, 2])
    cl = oracle.channels_last_strides
    yd = oracle.conv_output_dims(case["x"], case["w"], case["pad"], case["s"],
                                 case["d"])
    mk = lambda dims: capi.TensorDesc.make(dims, cl(dims), capi.BFLOAT16)
    d = capi.ConvDesc()
    d.x, d.w, d.y = mk(case["x"]), mk(case["w"]), mk(yd)
    d.spatial_rank = 2
    for i in range(2):
        d.padding[i], d.stride[i], d.dilation[i] = 1, 2, 1
    d.epilogue = capi.make_epilogue([])
    assert ctx.conv_dgrad_workspace(d) > MAX_BYTES
    one = ctx.alloc(256)  # never touched: the call fails before any launch
    rc = ctx.lib.fhip_conv_dgrad_static(ctx.handle, ctypes.byref(d), one.ptr,
                                        one.ptr, one.ptr)
    assert rc != 0
    assert b"static array holds" in ctx.lib.fhip_last_error(ctx.handle)
