"""bfloat16 host arrays without ``ml_dtypes``.

numpy has no bfloat16; the reference uses ``ml_dtypes.bfloat16`` when that
optional package is installed (``python/tessera/runtime.py:314-324``).  The lane
only needs the 16-bit patterns, so bf16 data travels as :class:`BF16Array` — a
``uint16`` ndarray subclass that marks its contents as bfloat16 bits.  An
``ml_dtypes.bfloat16`` array is accepted wherever a :class:`BF16Array` is.
"""
from __future__ import annotations

import numpy as np


class BF16Array(np.ndarray):
    """``uint16`` array whose elements are bfloat16 bit patterns."""

    def to_float32(self) -> np.ndarray:
        return (np.asarray(self, np.uint16).astype(np.uint32) << 16).view(np.float32)


def from_float32(x) -> BF16Array:
    """f32 -> bf16 bits, round-to-nearest-even (the rounding the reference's
    ``_round_to_storage`` fallback applies, ``compiler/fusion_core.py:358-361``)."""
    a = np.ascontiguousarray(x, np.float32)
    flat = a.reshape(-1)
    bits = np.empty(flat.shape, np.uint16)
    step = 1 << 22                                   # chunked: 32-bit temporaries stay cache-sized
    for i in range(0, flat.size, step):
        u = flat[i:i + step].view(np.uint32)
        r = (u >> 16) & np.uint32(1)
        r += np.uint32(0x7FFF)
        r += u                                       # wraps only for NaN patterns, fixed below
        r >>= 16
        nan = np.isnan(flat[i:i + step])
        if nan.any():
            r = np.where(nan, (u >> 16) | np.uint32(0x40), r)
        bits[i:i + step] = r
    bits = bits.reshape(a.shape)
    return bits.view(BF16Array)


def from_bits(bits) -> BF16Array:
    return np.ascontiguousarray(bits, np.uint16).view(BF16Array)


def is_bf16(a) -> bool:
    if isinstance(a, BF16Array):
        return True
    dt = getattr(a, "dtype", None)
    return dt is not None and getattr(dt, "name", "") == "bfloat16"


def as_bits(a) -> np.ndarray:
    """Contiguous ``uint16`` view of a bf16 array (BF16Array or ml_dtypes)."""
    if isinstance(a, BF16Array):
        return np.ascontiguousarray(np.asarray(a, np.uint16))
    return np.ascontiguousarray(a).view(np.uint16)
