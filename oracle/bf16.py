"""
CPU ORACLE (test infrastructure): bfloat16 rounding.

The reference has no bfloat16 (its storage types end at fp16,
neon/backends/nervanagpu.py:99-100); the oracle for bf16-stored tensors is the
fp32 oracle on inputs that hold bf16 values exactly, with results rounded to
bf16 by ``round_to_bf16`` -- what the mathematics fixes: the nearer of the two
neighbouring bf16 values, ties to the one with an even last mantissa bit, NaN
stays NaN, magnitudes beyond the largest finite bf16 value's rounding range go
to infinity.  Written as a comparison of distances in float64 (exact for
float32 inputs), NOT as the add-and-shift bit trick the product uses;
tests/test_oracle.py pins it by exhaustive and brute-force checks.
"""
import numpy as np


def round_to_bf16(values):
    x = np.asarray(values, dtype=np.float32)
    bits = x.view(np.uint32) if x.flags.c_contiguous else np.ascontiguousarray(x).view(np.uint32)
    bits = bits.reshape(x.shape)
    down_bits = bits & np.uint32(0xFFFF0000)                     # toward zero
    up_bits = (down_bits.astype(np.uint64) + 0x10000).astype(np.uint32)   # next bf16 value away from zero
    with np.errstate(all="ignore"):
        down = down_bits.view(np.float32).astype(np.float64)
        # (the neighbour above the largest finite value is 2^128: infinity as a float32, finite here)
        up_is_inf = (up_bits & np.uint32(0x7FFFFFFF)) == np.uint32(0x7F800000)
        up = np.where(up_is_inf, np.copysign(2.0 ** 128, down), up_bits.view(np.float32).astype(np.float64))
        xd = x.astype(np.float64)
        d_down, d_up = np.abs(xd - down), np.abs(up - xd)
        even_down = ((down_bits >> 16) & 1) == 0
        take_up = (d_up < d_down) | ((d_up == d_down) & ~even_down)
        out = np.where(take_up, up_bits.view(np.float32), down_bits.view(np.float32)).astype(np.float32)
    out = np.where(np.isnan(x), np.float32(np.nan), out)
    out = np.where(np.isinf(x), x, out)
    return out.astype(np.float32)
