"""Seeded synthetic inputs and storage-type conversions (numpy, host side).

The reference has no random inputs (its samples fill constants), so the seeds
are ours: a counter-based generator — splitmix64 of (seed, tensor id, linear
index) — so any element can be regenerated anywhere without carrying state.
Values are quantised once on the host and the same bits go to the device and
to whatever checks them.
"""
from __future__ import annotations

import numpy as np

from . import capi

_M64 = np.uint64(0xFFFFFFFFFFFFFFFF)


def _splitmix64(x: np.ndarray) -> np.ndarray:
    with np.errstate(over="ignore"):
        x = (x + np.uint64(0x9E3779B97F4A7C15)) & _M64
        z = x
        z = ((z ^ (z >> np.uint64(30))) * np.uint64(0xBF58476D1CE4E5B9)) & _M64
        z = ((z ^ (z >> np.uint64(27))) * np.uint64(0x94D049BB133111EB)) & _M64
        return z ^ (z >> np.uint64(31))


def raw_bits(seed: int, tensor_id: int, count: int, stream: int = 0) -> np.ndarray:
    """64 random bits per element, a pure function of its arguments."""
    idx = np.arange(count, dtype=np.uint64)
    with np.errstate(over="ignore"):
        key = _splitmix64(np.uint64(seed) * np.uint64(0x100000001B3)
                          + np.uint64(tensor_id) * np.uint64(0x9E3779B1)
                          + np.uint64(stream) * np.uint64(0x85EBCA77))
        return _splitmix64(idx ^ key)


def uniform(seed: int, tensor_id: int, count: int, lo=-1.0, hi=1.0,
            stream: int = 0) -> np.ndarray:
    """Uniform [lo, hi) f32 from the top 24 bits."""
    u = (raw_bits(seed, tensor_id, count, stream) >> np.uint64(40)).astype(np.float64)
    return (lo + (hi - lo) * (u / float(1 << 24))).astype(np.float32)


def normal(seed: int, tensor_id: int, count: int, mean=0.0, std=1.0) -> np.ndarray:
    """N(mean, std) f32 by Box-Muller on two uniform streams."""
    u1 = ((raw_bits(seed, tensor_id, count, 1) >> np.uint64(40)).astype(np.float64)
          + 1.0) / float(1 << 24)  # (0, 1]
    u2 = (raw_bits(seed, tensor_id, count, 2) >> np.uint64(40)).astype(np.float64) \
        / float(1 << 24)
    z = np.sqrt(-2.0 * np.log(u1)) * np.cos(2.0 * np.pi * u2)
    return (mean + std * z).astype(np.float32)


def integers(seed: int, tensor_id: int, count: int, lo: int, hi: int) -> np.ndarray:
    """Integers uniform in [lo, hi] as int64."""
    span = np.uint64(hi - lo + 1)
    return (raw_bits(seed, tensor_id, count) % span).astype(np.int64) + lo


# ---- storage conversions --------------------------------------------------
def f32_to_bf16_bits(x: np.ndarray) -> np.ndarray:
    """Round-to-nearest-even f32 -> bf16, as uint16 bit patterns."""
    u = np.ascontiguousarray(x, np.float32).view(np.uint32)
    nan = (u & np.uint32(0x7FFFFFFF)) > np.uint32(0x7F800000)
    lsb = (u >> np.uint32(16)) & np.uint32(1)
    with np.errstate(over="ignore"):
        r = ((u + np.uint32(0x7FFF) + lsb) >> np.uint32(16)).astype(np.uint16)
    r[nan] = ((u[nan] >> np.uint32(16)) | np.uint32(0x40)).astype(np.uint16)
    return r


def bf16_bits_to_f32(b: np.ndarray) -> np.ndarray:
    return (np.ascontiguousarray(b, np.uint16).astype(np.uint32)
            << np.uint32(16)).view(np.float32)


def _fp8_table(ebits: int) -> np.ndarray:
    mbits = 7 - ebits
    bias = (1 << (ebits - 1)) - 1
    t = np.empty(256, np.float64)
    for v in range(256):
        sign = -1.0 if v & 0x80 else 1.0
        e = (v >> mbits) & ((1 << ebits) - 1)
        m = v & ((1 << mbits) - 1)
        if ebits == 4 and e == 15 and m == 7:
            val = np.nan
        elif ebits == 5 and e == 31:
            val = np.nan if m else np.inf
        elif e == 0:
            val = m * 2.0 ** (1 - bias - mbits)
        else:
            val = ((1 << mbits) | m) * 2.0 ** (e - bias - mbits)
        t[v] = sign * val
    return t


_FP8_TABLES = {4: _fp8_table(4), 5: _fp8_table(5)}


def fp8_bits_to_f32(b: np.ndarray, ebits: int = 4) -> np.ndarray:
    return _FP8_TABLES[ebits][np.ascontiguousarray(b, np.uint8)].astype(np.float32)


def f32_to_fp8_bits(x: np.ndarray, ebits: int = 4) -> np.ndarray:
    """Saturating round-to-nearest-even f32 -> OCP fp8 (e4m3fn or e5m2)."""
    table = _FP8_TABLES[ebits]
    maxcode = 0x7E if ebits == 4 else 0x7B
    pos = table[: maxcode + 1]  # ascending non-negative finite values
    a = np.abs(np.ascontiguousarray(x, np.float64))
    hi = np.clip(np.searchsorted(pos, a, side="left"), 0, maxcode)
    lo = np.clip(hi - 1, 0, maxcode)
    dlo, dhi = a - pos[lo], pos[hi] - a
    pick_hi = (dhi < dlo) | ((dhi == dlo) & (hi % 2 == 0))
    code = np.where(pick_hi, hi, lo).astype(np.uint8)
    code = np.where(a >= pos[maxcode], np.uint8(maxcode), code)
    out = code | (np.signbit(x).astype(np.uint8) << 7)
    nan_code = 0x7F if ebits == 4 else 0x7E
    return np.where(np.isnan(x), np.uint8(nan_code), out).astype(np.uint8)


def to_storage_bits(x: np.ndarray, dtype: int) -> np.ndarray:
    """Real values -> storage array of the given fhip dtype."""
    if dtype == capi.BFLOAT16:
        return f32_to_bf16_bits(x)
    if dtype == capi.HALF:
        return np.ascontiguousarray(x, np.float32).astype(np.float16)
    if dtype == capi.FLOAT:
        return np.ascontiguousarray(x, np.float32)
    if dtype == capi.DOUBLE:
        return np.ascontiguousarray(x, np.float64)
    if dtype == capi.FP8E4M3:
        return f32_to_fp8_bits(x, 4)
    if dtype == capi.FP8E5M2:
        return f32_to_fp8_bits(x, 5)
    if dtype == capi.BOOLEAN:
        return (np.asarray(x) != 0).astype(np.uint8)
    np_t = {capi.UINT8: np.uint8, capi.INT8: np.int8, capi.INT16: np.int16,
            capi.INT32: np.int32, capi.INT64: np.int64}[dtype]
    info = np.iinfo(np_t)
    return np.clip(np.rint(np.asarray(x, np.float64)), info.min, info.max).astype(np_t)


def from_storage_bits(b: np.ndarray, dtype: int) -> np.ndarray:
    """Storage array -> exact widened values (f32 / f64 / int64)."""
    if dtype == capi.BFLOAT16:
        return bf16_bits_to_f32(b)
    if dtype == capi.FP8E4M3:
        return fp8_bits_to_f32(b, 4)
    if dtype == capi.FP8E5M2:
        return fp8_bits_to_f32(b, 5)
    if dtype in (capi.HALF, capi.FLOAT):
        return np.asarray(b).astype(np.float32)
    if dtype == capi.DOUBLE:
        return np.asarray(b, np.float64)
    return np.asarray(b).astype(np.int64)


STORAGE_NP = {capi.HALF: np.float16, capi.BFLOAT16: np.uint16,
              capi.FLOAT: np.float32, capi.DOUBLE: np.float64,
              capi.UINT8: np.uint8, capi.INT8: np.int8, capi.INT16: np.int16,
              capi.INT32: np.int32, capi.INT64: np.int64,
              capi.BOOLEAN: np.uint8, capi.FP8E5M2: np.uint8,
              capi.FP8E4M3: np.uint8}
