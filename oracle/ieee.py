"""Bit-level binary32 helpers for the oracle (test infrastructure only).

Everything takes and returns ``numpy.float32`` arrays and performs exactly one
IEEE-754 rounding per named operation.
"""

from __future__ import annotations

import numpy as np

F32 = np.float32
LOG2E = F32(1.44269504088896340736)  # csrc/kernels/math.cuh:33
U8_OFFSET = F32(7.9943534)  # csrc/kernels/attention_types.cuh:42 (S_U8_OFFSET)
ROW_FLOOR = F32(-50000.0)  # csrc/kernels/attention_int8.cuh:286, attention_softmax.cuh:40


def f32(x) -> np.ndarray:
    return np.asarray(x, dtype=F32)


def fma32(a, b, c) -> np.ndarray:
    """round32(a*b + c) with a single rounding (CUDA ``fmaf``).

    The product of two binary32 numbers is exact in binary64.  The binary64 sum
    is then forced to round-to-odd (Boldo-Melquiond) so that the final
    conversion to binary32 cannot suffer a double rounding.
    """
    a64, b64, c64 = np.broadcast_arrays(
        np.asarray(a, dtype=np.float64),
        np.asarray(b, dtype=np.float64),
        np.asarray(c, dtype=np.float64),
    )
    shape = a64.shape
    a64, b64, c64 = a64.reshape(-1), b64.reshape(-1), c64.reshape(-1)
    with np.errstate(invalid="ignore", over="ignore"):
        p = a64 * b64
        s = p + c64
        # TwoSum error term of p + c.
        bb = s - p
        err = (p - (s - bb)) + (c64 - bb)
    fix = np.isfinite(s) & np.isfinite(err) & (err != 0.0) & ((s.view(np.int64) & 1) == 0)
    if np.any(fix):
        toward = np.where(err[fix] > 0.0, np.inf, -np.inf)
        s[fix] = np.nextafter(s[fix], toward)
    s = s.reshape(shape)
    return s.astype(F32)


def rni_sat(x, lo: int, hi: int) -> np.ndarray:
    """``cvt.rni.sat``: round to nearest even, clamp, NaN -> 0 (float_utils.cuh:23-27)."""
    x = np.asarray(x, dtype=F32)
    with np.errstate(invalid="ignore"):
        r = np.rint(x)
    r = np.where(np.isnan(r), F32(0), r)
    return np.clip(r, lo, hi)


def exp2_32(x) -> np.ndarray:
    """Correctly rounded 2**x with flush-to-zero of subnormal results.

    Stands in for ``ex2.approx.ftz.f32`` (csrc/kernels/math.cuh:35-39).
    """
    x = np.asarray(x, dtype=F32)
    with np.errstate(over="ignore", under="ignore", invalid="ignore"):
        y = np.exp2(x.astype(np.float64)).astype(F32)
    tiny = np.abs(y) < np.finfo(F32).tiny
    return np.where(tiny, F32(0), y)


def log2_32(x) -> np.ndarray:
    """Correctly rounded log2 (stands in for ``lg2.approx.ftz.f32``, math.cuh:49-53)."""
    x = np.asarray(x, dtype=F32)
    with np.errstate(divide="ignore", invalid="ignore"):
        return np.log2(x.astype(np.float64)).astype(F32)


def to_bf16_bits(x) -> np.ndarray:
    """binary32 -> bfloat16 bit patterns, round to nearest even, NaN kept quiet."""
    x = np.ascontiguousarray(x, dtype=F32)
    bits = x.view(np.uint32).astype(np.uint64)
    rounded = (bits + 0x7FFF + ((bits >> 16) & 1)) >> 16
    nan = np.isnan(x)
    rounded = np.where(nan, (bits >> 16) | 0x40, rounded)
    return rounded.astype(np.uint16)


def round_to_dtype(x, dtype_name: str) -> np.ndarray:
    """Round binary32 values to ``float16``/``bfloat16`` and return them as binary32."""
    x = np.asarray(x, dtype=F32)
    if dtype_name == "float16":
        with np.errstate(over="ignore"):
            return x.astype(np.float16).astype(F32)
    if dtype_name == "bfloat16":
        return (to_bf16_bits(x).astype(np.uint32) << 16).view(F32).reshape(x.shape)
    if dtype_name == "float32":
        return x
    raise ValueError(f"unsupported dtype {dtype_name}")
