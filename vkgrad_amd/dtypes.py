"""Host-side conversions between float32 and the 16-bit storage types.

numpy has float16 but no bfloat16; bf16 tensors are carried as uint16 bit
patterns everywhere in this package (Buffer.array(np.uint16)).
"""

import numpy as np


def f32_to_bf16_bits(x):
    """float32 -> bfloat16 bit patterns, round to nearest even (NaN -> 0x7FC0)."""
    x = np.ascontiguousarray(x, dtype=np.float32)
    u = x.view(np.uint32)
    r = ((u + np.uint32(0x7FFF) + ((u >> np.uint32(16)) & np.uint32(1))) >> np.uint32(16)).astype(np.uint16)
    nan = np.isnan(x)
    return np.where(nan, np.uint16(0x7FC0), r) if nan.any() else r


def bf16_bits_to_f32(b):
    """bfloat16 bit patterns -> float32, exact."""
    return (np.ascontiguousarray(b, dtype=np.uint16).astype(np.uint32) << np.uint32(16)).view(np.float32)


def to_storage(x, dtype):
    """float data -> the array to upload for `dtype` ('f16' or 'bf16')."""
    if dtype == "f16":
        return np.asarray(x, dtype=np.float32).astype(np.float16)
    if dtype == "bf16":
        return f32_to_bf16_bits(x)
    raise ValueError(f"unknown dtype {dtype!r}")


def from_storage(a, dtype):
    """Stored array -> float32, exact."""
    if dtype == "f16":
        return np.asarray(a, dtype=np.float16).astype(np.float32)
    if dtype == "bf16":
        return bf16_bits_to_f32(a)
    raise ValueError(f"unknown dtype {dtype!r}")
