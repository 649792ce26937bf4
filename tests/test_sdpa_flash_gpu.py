"""Flash-attention forward (MFMA kernel) through the C ABI vs the oracle.

Every case satisfies the tuned kernel's contract (bf16/f16, head dim 64 or 128;
mask tensors with unit key stride and extents that are multiples of 4) and
asserts that the tuned kernel is chosen, so a silent fall back to the generic
kernel fails the test.
"""
import numpy as np
import pytest

from fusilli_amd import capi
from oracle import oracle
from helpers import HT, assert_close, rand

pytestmark = pytest.mark.gpu


def run(ctx, q, k, v, causal=False, scale=None, o_strides=None, expect_tuned=True,
        mask=None):
    out = HT.empty([q.dims[0], q.dims[1], q.dims[2], v.dims[3]], q.dtype, o_strides)
    d = capi.SdpaDesc()
    d.q, d.k, d.v, d.o = q.desc(), k.desc(), v.desc(), out.desc()
    if mask is not None:
        d.mask = mask.desc()
    d.is_causal = int(causal)
    if scale is not None:
        d.has_scale, d.scale = 1, scale
    assert ctx.lib.fhip_sdpa_fwd_supported(d) == (2 if expect_tuned else 1)
    bufs = [t.upload(ctx) for t in (q, k, v)]
    dout = out.upload(ctx)
    dm = mask.upload(ctx) if mask is not None else None
    ctx.sdpa_fwd(d, bufs[0], bufs[1], bufs[2], dout, mask=dm)
    return out.fetch(ctx, dout)


def bshd_strides(dims):
    b, h, s, d = dims
    return [s * h * d, d, h * d, 1]


CASES = [
    dict(B=1, Hq=2, Hkv=2, Sq=256, Skv=256, causal=False),
    dict(B=1, Hq=2, Hkv=2, Sq=256, Skv=256, causal=True),
    # ragged: rows past Sq in the last query tile, keys past Skv in the last tile
    dict(B=2, Hq=3, Hkv=3, Sq=300, Skv=200, causal=False),
    dict(B=1, Hq=2, Hkv=2, Sq=333, Skv=333, causal=True),
    # GQA and cross attention; more than one query tile and many key tiles
    dict(B=1, Hq=4, Hkv=2, Sq=513, Skv=700, causal=False),
    dict(B=1, Hq=4, Hkv=1, Sq=520, Skv=520, causal=True),
    # causal with fewer keys than queries, and a single key
    dict(B=1, Hq=1, Hkv=1, Sq=300, Skv=70, causal=True),
    dict(B=1, Hq=2, Hkv=2, Sq=40, Skv=1, causal=False),
    dict(B=1, Hq=1, Hkv=1, Sq=1, Skv=129, causal=False),
]


@pytest.mark.parametrize("case", CASES)
@pytest.mark.parametrize("dtype", [capi.BFLOAT16, capi.HALF])
@pytest.mark.parametrize("hd", [128, 64])
def test_flash_random_vs_oracle(ctx, case, dtype, hd):
    c = case
    q = HT.from_logical(rand(51, 0, [c["B"], c["Hq"], c["Sq"], hd]), dtype)
    k = HT.from_logical(rand(51, 1, [c["B"], c["Hkv"], c["Skv"], hd]), dtype)
    v = HT.from_logical(rand(51, 2, [c["B"], c["Hkv"], c["Skv"], hd]), dtype)
    out = run(ctx, q, k, v, causal=c["causal"])
    ref = oracle.sdpa(q.logical(), k.logical(), v.logical(), is_causal=c["causal"])
    assert_close(out.logical(), ref, dtype, str(case))


@pytest.mark.parametrize("hd", [128, 64])
def test_flash_bshd_layout_and_scale(ctx, hd):
    # tensors stored [B, S, H, D] (heads interleaved per position), custom scale
    dims_q, dims_k = [2, 4, 200, hd], [2, 2, 300, hd]
    q = HT.from_logical(rand(52, 0, dims_q), capi.BFLOAT16, bshd_strides(dims_q))
    k = HT.from_logical(rand(52, 1, dims_k), capi.BFLOAT16, bshd_strides(dims_k))
    v = HT.from_logical(rand(52, 2, dims_k), capi.BFLOAT16, bshd_strides(dims_k))
    out = run(ctx, q, k, v, scale=0.05, o_strides=bshd_strides(dims_q))
    ref = oracle.sdpa(q.logical(), k.logical(), v.logical(), scale=0.05)
    assert_close(out.logical(), ref, capi.BFLOAT16)


@pytest.mark.parametrize("hd", [128, 64])
def test_flash_large_scores_are_stable(ctx, hd):
    # scores of magnitude ~1e3: the running maximum must keep exp() in range
    q = HT.from_logical(rand(53, 0, [1, 2, 300, hd]) * 8.0, capi.BFLOAT16)
    k = HT.from_logical(rand(53, 1, [1, 2, 300, hd]) * 8.0, capi.BFLOAT16)
    v = HT.from_logical(rand(53, 2, [1, 2, 300, hd]), capi.BFLOAT16)
    out = run(ctx, q, k, v, causal=True)
    assert np.all(np.isfinite(out.logical()))
    ref = oracle.sdpa(q.logical(), k.logical(), v.logical(), is_causal=True)
    assert_close(out.logical(), ref, capi.BFLOAT16)


@pytest.mark.parametrize("causal", [False, True])
@pytest.mark.parametrize("hd", [128, 64])
def test_flash_constant_fill_equals_v(ctx, causal, hd):
    # samples/sdpa_utils.cpp:184-247: q = k = v = 0.01 => output == v (1e-2)
    q = HT.from_logical(np.full([1, 8, 320, hd], 0.01), capi.HALF)
    out = run(ctx, q, q, q, causal=causal)
    assert np.allclose(out.logical(), 0.01, atol=1e-2)


@pytest.mark.parametrize("hd", [128, 64])
def test_flash_uniform_scores_causal_gives_prefix_means(ctx, hd):
    # q = 0 => uniform attention over the visible prefix: O[i] = mean(V[:i+1])
    S = 400
    q = HT.from_logical(np.zeros([1, 1, S, hd]), capi.BFLOAT16)
    k = HT.from_logical(rand(54, 1, [1, 1, S, hd]), capi.BFLOAT16)
    v = HT.from_logical(rand(54, 2, [1, 1, S, hd]), capi.BFLOAT16)
    out = run(ctx, q, k, v, causal=True)
    vl = v.logical()[0, 0]
    ref = np.cumsum(vl, axis=0) / np.arange(1, S + 1)[:, None]
    assert_close(out.logical()[0, 0], ref, capi.BFLOAT16)


MASK_CASES = [
    # the reference benchmark's shape: mask [B, 1, Sq, Skv] of the I/O type
    dict(B=1, Hq=8, Hkv=8, Sq=64, Skv=64, mdims="b1qk"),
    # ragged query tile, several key tiles with a partial last one
    dict(B=2, Hq=3, Hkv=3, Sq=300, Skv=200, mdims="b1qk"),
    # per-head masks, GQA, more than one query tile
    dict(B=1, Hq=4, Hkv=2, Sq=513, Skv=260, mdims="bhqk"),
    # one mask for every batch entry and head
    dict(B=2, Hq=2, Hkv=2, Sq=130, Skv=132, mdims="11qk"),
    # one mask row for every query (padding mask)
    dict(B=2, Hq=2, Hkv=1, Sq=70, Skv=324, mdims="b11k"),
]


def mask_dims(c):
    full = dict(b=c["B"], h=c["Hq"], q=c["Sq"], k=c["Skv"])
    return [1 if ch == "1" else full[ch] for ch in c["mdims"]]


@pytest.mark.parametrize("case", MASK_CASES)
@pytest.mark.parametrize("kind", ["same", "f32", "bool"])
@pytest.mark.parametrize("dtype,hd", [(capi.BFLOAT16, 128), (capi.HALF, 64),
                                      (capi.HALF, 128), (capi.BFLOAT16, 64)])
def test_flash_mask_vs_oracle(ctx, case, kind, dtype, hd):
    c = case
    q = HT.from_logical(rand(56, 0, [c["B"], c["Hq"], c["Sq"], hd]), dtype)
    k = HT.from_logical(rand(56, 1, [c["B"], c["Hkv"], c["Skv"], hd]), dtype)
    v = HT.from_logical(rand(56, 2, [c["B"], c["Hkv"], c["Skv"], hd]), dtype)
    md = mask_dims(c)
    if kind == "bool":
        keep = rand(56, 3, md, "uniform") > 0.2
        # whole key tiles masked at the front of some rows, no row without a key
        keep[..., ::3, :128] = False
        keep[..., -1] = True
        mask, mref = HT.from_logical(keep, capi.BOOLEAN), keep
    else:
        mask = HT.from_logical(rand(56, 3, md) * 3.0,
                               dtype if kind == "same" else capi.FLOAT)
        mref = mask.logical()
    out = run(ctx, q, k, v, mask=mask)
    ref = oracle.sdpa(q.logical(), k.logical(), v.logical(), mask=mref)
    assert_close(out.logical(), ref, dtype, f"{case} {kind}")


def test_flash_mask_minus_infinity_and_dead_rows(ctx):
    # additive -inf entries; a query with every key masked yields NaN, as
    # softmax over an empty set does in aten, and leaves its neighbours alone
    B, H, Sq, Skv, hd = 1, 2, 96, 128, 64
    q = HT.from_logical(rand(57, 0, [B, H, Sq, hd]), capi.HALF)
    k = HT.from_logical(rand(57, 1, [B, H, Skv, hd]), capi.HALF)
    v = HT.from_logical(rand(57, 2, [B, H, Skv, hd]), capi.HALF)
    m = rand(57, 3, [B, 1, Sq, Skv]).astype(np.float32)
    m[..., 5:40] = -np.inf
    m[0, 0, 17, :] = -np.inf
    mask = HT.from_logical(m, capi.FLOAT)
    out = run(ctx, q, k, v, mask=mask).logical()
    assert np.all(np.isnan(out[:, :, 17, :]))
    rows = np.arange(Sq) != 17
    ref = oracle.sdpa(q.logical(), k.logical(), v.logical(), mask=m)
    assert_close(out[:, :, rows, :], ref[:, :, rows, :], capi.HALF)


def test_flash_mask_outside_contract_runs_generic(ctx):
    # a key count that is no multiple of 4: mask rows are not 4-element aligned
    q = HT.from_logical(rand(58, 0, [1, 2, 40, 64]), capi.HALF)
    k = HT.from_logical(rand(58, 1, [1, 2, 66, 64]), capi.HALF)
    mask = HT.from_logical(rand(58, 3, [1, 1, 40, 66]), capi.HALF)
    out = run(ctx, q, k, k, mask=mask, expect_tuned=False)
    ref = oracle.sdpa(q.logical(), k.logical(), k.logical(), mask=mask.logical())
    assert_close(out.logical(), ref, capi.HALF)


def test_flash_not_chosen_outside_contract(ctx):
    # other head dims (and f32) keep the generic kernel
    q = HT.from_logical(rand(55, 0, [1, 2, 70, 96]), capi.BFLOAT16)
    out = run(ctx, q, q, q, expect_tuned=False)
    ref = oracle.sdpa(q.logical(), q.logical(), q.logical())
    assert_close(out.logical(), ref, capi.BFLOAT16)


def test_flash_headline_shape(ctx):
    """B4 H32 S2048 D128 bf16 causal at full size.

    Heads are independent, so the oracle is run on four (batch, head) slices
    picked across the grid; q = 0 in one further head gives the closed-form
    prefix means."""
    B, H, S, D = 4, 32, 2048, 128
    qv = rand(56, 0, [B, H, S, D])
    qv[2, 7] = 0.0
    q = HT.from_logical(qv, capi.BFLOAT16)
    k = HT.from_logical(rand(56, 1, [B, H, S, D]), capi.BFLOAT16)
    v = HT.from_logical(rand(56, 2, [B, H, S, D]), capi.BFLOAT16)
    out = run(ctx, q, k, v, causal=True).logical()
    assert np.all(np.isfinite(out))
    ql, kl, vl = q.logical(), k.logical(), v.logical()
    for b, h in [(0, 0), (1, 13), (3, 31), (2, 20)]:
        ref = oracle.sdpa(ql[b:b + 1, h:h + 1], kl[b:b + 1, h:h + 1],
                          vl[b:b + 1, h:h + 1], is_causal=True)
        assert_close(out[b:b + 1, h:h + 1], ref, capi.BFLOAT16, f"b{b} h{h}")
    ref = np.cumsum(vl[2, 7], axis=0) / np.arange(1, S + 1)[:, None]
    assert_close(out[2, 7], ref, capi.BFLOAT16, "uniform head")
    assert ctx.last_kernel() == "sdpa_fwd d=128 causal=1 mask=0", ctx.last_kernel()

    # Every workgroup slot: the same random head in all 128 (batch, head)
    # entries must give 128 bit-identical outputs; entry (0, 0) is compared
    # with the oracle.
    one = lambda tid: np.broadcast_to(rand(57, tid, [1, 1, S, D]), [B, H, S, D])
    q, k, v = (HT.from_logical(one(i), capi.BFLOAT16) for i in range(3))
    out = run(ctx, q, k, v, causal=True).logical()
    ref = oracle.sdpa(q.logical()[:1, :1], k.logical()[:1, :1], v.logical()[:1, :1],
                      is_causal=True)
    assert_close(out[:1, :1], ref, capi.BFLOAT16, "shared head")
    for b in range(B):
        for h in range(H):
            assert np.array_equal(out[b, h], out[0, 0]), f"b{b} h{h} differs from b0 h0"


def test_flash_benchmark_lines_mask_and_head_dim_64(ctx):
    """The two SDPA lines beside the headline at full size (B4 H32 S2048 bf16):
    head dim 64 under the causal flag, and head dim 128 under an additive bf16
    mask [B, 1, S, S] shared by the heads.  The oracle runs on three (batch,
    head) slices each; q = 0 in one head of the masked call gives the
    closed form softmax(mask row) . V."""
    B, H, S = 4, 32, 2048
    for D, masked in ((64, False), (128, True)):
        qv = rand(58, 0, [B, H, S, D])
        if masked:
            qv[1, 5] = 0.0
        q = HT.from_logical(qv, capi.BFLOAT16)
        k = HT.from_logical(rand(58, 1, [B, H, S, D]), capi.BFLOAT16)
        v = HT.from_logical(rand(58, 2, [B, H, S, D]), capi.BFLOAT16)
        mask = HT.from_logical(rand(58, 3, [B, 1, S, S]), capi.BFLOAT16) if masked else None
        out = run(ctx, q, k, v, causal=not masked, mask=mask).logical()
        assert np.all(np.isfinite(out))
        ql, kl, vl = q.logical(), k.logical(), v.logical()
        ml = mask.logical() if masked else None
        for b, h in [(0, 0), (2, 17), (3, 31)]:
            ref = oracle.sdpa(ql[b:b + 1, h:h + 1], kl[b:b + 1, h:h + 1], vl[b:b + 1, h:h + 1],
                              mask=ml[b:b + 1] if masked else None, is_causal=not masked)
            assert_close(out[b:b + 1, h:h + 1], ref, capi.BFLOAT16, f"D{D} b{b} h{h}")
        if masked:
            m = ml[1, 0].astype(np.float64)
            p = np.exp(m - m.max(axis=1, keepdims=True))
            p /= p.sum(axis=1, keepdims=True)
            assert_close(out[1, 5], p @ vl[1, 5].astype(np.float64), capi.BFLOAT16,
                         "uniform scores under the mask")


def test_flash_head_dim_64_many_tiles(ctx):
    """Head dim 64, causal, eight query tiles per head: every key-tile count
    from 1 to 32 occurs, and the paired query tiles (long + short) share one
    workgroup.  One head has q = 0 for the closed-form prefix means."""
    B, H, S, D = 1, 3, 2048, 64
    qv = rand(57, 0, [B, H, S, D])
    qv[0, 1] = 0.0
    q = HT.from_logical(qv, capi.BFLOAT16)
    k = HT.from_logical(rand(57, 1, [B, H, S, D]), capi.BFLOAT16)
    v = HT.from_logical(rand(57, 2, [B, H, S, D]), capi.BFLOAT16)
    out = run(ctx, q, k, v, causal=True).logical()
    ref = oracle.sdpa(q.logical(), k.logical(), v.logical(), is_causal=True)
    assert_close(out, ref, capi.BFLOAT16)
    vl = v.logical()[0, 1]
    assert_close(out[0, 1], np.cumsum(vl, axis=0) / np.arange(1, S + 1)[:, None],
                 capi.BFLOAT16, "uniform head")
