"""Shared test plumbing: host tensors with the reference's dims+strides
layout model, upload/download through the C ABI, comparison with the oracle."""
from __future__ import annotations

from typing import Optional, Sequence

import numpy as np

from fusilli_amd import capi
from oracle import oracle

RTOL = {capi.FLOAT: 1e-4, capi.DOUBLE: 1e-4, capi.HALF: 2e-2,
        capi.BFLOAT16: 2e-2}


class HT:
    """Host tensor: logical dims, element strides, dtype and 1-D storage."""

    def __init__(self, dims, strides, dtype, storage):
        self.dims = [int(d) for d in dims]
        self.strides = [int(s) for s in strides]
        self.dtype = dtype
        self.storage = storage

    @classmethod
    def from_logical(cls, values, dtype, strides: Optional[Sequence[int]] = None):
        values = np.asarray(values)
        dims = list(values.shape)
        if strides is None:
            strides = oracle.contiguous_strides(dims)
        q = oracle.quantize(values, dtype)
        if any(s == 0 and d > 1 for d, s in zip(dims, strides)):
            # broadcast input: storage holds only the non-broadcast part
            idx = tuple(slice(0, 1) if s == 0 else slice(None)
                        for s in strides)
            q = q[idx]
            st = oracle.to_storage(q, [s for s in strides])
        else:
            st = oracle.to_storage(q, strides)
        return cls(dims, strides, dtype, st)

    @classmethod
    def empty(cls, dims, dtype, strides=None, fill=0):
        if strides is None:
            strides = oracle.contiguous_strides(dims)
        n = oracle.storage_extent(dims, strides)
        return cls(dims, strides, dtype,
                   np.full(n, fill, oracle.storage_dtype(dtype)))

    def logical(self) -> np.ndarray:
        """Exact stored values in logical dim order (f32 / f64 / int64)."""
        return np.array(oracle.logical_view(
            oracle.dequantize(self.storage, self.dtype), self.dims, self.strides))

    def desc(self) -> capi.TensorDesc:
        return capi.TensorDesc.make(self.dims, self.strides, self.dtype)

    def upload(self, ctx) -> capi.DeviceBuffer:
        return ctx.to_device(self.storage)

    def fetch(self, ctx, buf) -> "HT":
        self.storage = buf.download(self.storage.dtype, self.storage.size)
        return self


def worst_violations(got, ref, rtol, limit=8):
    """Index, value and reference of the entries furthest outside the bar
    |got - ref| <= rtol |ref| + rtol rms(ref) (for the failure message: where
    a kernel went wrong says more than how far)."""
    g = np.asarray(got, np.float64)
    r = np.asarray(ref, np.float64)
    finite = np.isfinite(r)
    rms = float(np.sqrt(np.mean(r[finite] ** 2))) if finite.any() else 0.0
    excess = np.where(finite, np.abs(g - r) - (rtol * np.abs(r) + rtol * rms), 0.0)
    excess = np.nan_to_num(excess, nan=np.inf)
    order = np.argsort(excess, axis=None)[::-1][:limit]
    worst = [(tuple(int(i) for i in np.unravel_index(o, g.shape)), float(g.flat[o]), float(r.flat[o]))
             for o in order if excess.flat[o] > 0]
    # the extent of the damage: per dim the range of indices with a violation
    # and how many distinct ones (a tile, a row of a wavefront, one column ...)
    bad = np.argwhere(excess > 0)
    if len(bad):
        extent = [(int(bad[:, d].min()), int(bad[:, d].max()), int(len(np.unique(bad[:, d]))))
                  for d in range(bad.shape[1])]
        worst.append(("extent per dim (min, max, distinct)", extent))
    return worst


def assert_close(got, ref, dtype, what="", rtol=None):
    rtol = RTOL[dtype] if rtol is None else rtol
    ok, rep = oracle.check_close(got, ref, rtol)
    assert ok, (f"{what}: {rep} (rtol {rtol}); worst (index, got, ref): "
                f"{worst_violations(got, ref, rtol)}")


def rand(seed, tid, dims, kind="normal", **kw):
    from fusilli_amd import synth
    n = int(np.prod(dims))
    if kind == "normal":
        v = synth.normal(seed, tid, n, kw.get("mean", 0.0), kw.get("std", 1.0))
    elif kind == "uniform":
        v = synth.uniform(seed, tid, n, kw.get("lo", -1.0), kw.get("hi", 1.0))
    else:
        v = synth.integers(seed, tid, n, kw["lo"], kw["hi"])
    return v.reshape(dims)
