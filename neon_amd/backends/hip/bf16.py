"""
bfloat16 storage on the host side.

numpy has no bfloat16, so the dtype that marks a tensor as bf16-stored is a
one-field record of 16 bits, ``bfloat16``: two bytes per element, distinct from
``uint16``, usable wherever a numpy dtype is expected (``be.empty(shape,
dtype=bfloat16)``).  Host arrays cross over as float32: ``set`` rounds to
nearest even (NaN stays NaN), ``get`` widens exactly.  On the device the type
is ``__bf16`` with fp32 arithmetic, like fp16 storage (the reference stops at
fp16: neon/backends/nervanagpu.py:99-100).
"""
import numpy as np

bfloat16 = np.dtype([("bf16", np.uint16)])


def is_bfloat16(dtype):
    return np.dtype(dtype) == bfloat16


def to_bits(values):
    """float array -> uint16 array of bf16 bit patterns, round to nearest even"""
    f = np.ascontiguousarray(values, dtype=np.float32)
    bits = f.view(np.uint32)
    rounded = ((bits.astype(np.uint64) + 0x7FFF + ((bits >> 16) & 1)) >> 16).astype(np.uint16)
    nan = np.isnan(f)
    if nan.any():
        rounded = np.where(nan, ((bits >> 16) | 0x40).astype(np.uint16), rounded)
    return rounded


def from_bits(bits):
    """uint16 array of bf16 bit patterns -> float32 array (exact)"""
    b = np.ascontiguousarray(bits).view(np.uint16) if np.dtype(getattr(bits, "dtype", np.uint16)) == bfloat16 \
        else np.ascontiguousarray(bits, dtype=np.uint16)
    return (b.astype(np.uint32) << 16).view(np.float32)


def quantise(values):
    """float32 values rounded to the nearest bf16 value"""
    return from_bits(to_bits(values)).reshape(np.shape(values))
