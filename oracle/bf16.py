"""bfloat16 helpers in numpy (test infrastructure).  bf16 values travel either as uint16 bit patterns or as FP32
arrays whose low 16 mantissa bits are zero.

Rounding is round-to-nearest-even on the FP32 bit pattern, the `sc_rbf` of e2e/fused_olmoe.py:34-40 and the
conversion every `static_cast<T>` in e2e/sc_kernels.py performs for T = bfloat16."""
import numpy as np


def to_bits(x):
    """FP32 array -> uint16 bf16 bit patterns (RNE; NaN stays NaN)."""
    x = np.ascontiguousarray(x, dtype=np.float32)
    u = x.view(np.uint32)
    r = (u + (np.uint32(0x7FFF) + ((u >> np.uint32(16)) & np.uint32(1)))) >> np.uint32(16)
    nan = np.isnan(x)
    if nan.any():
        r = np.where(nan, (u >> np.uint32(16)) | np.uint32(0x40), r)
    return r.astype(np.uint16)


def from_bits(b):
    """uint16 bf16 bit patterns -> FP32 array."""
    b = np.ascontiguousarray(b, dtype=np.uint16)
    return (b.astype(np.uint32) << np.uint32(16)).view(np.float32)


def rnd(x):
    """Round an FP32 array to the nearest bf16, returned as FP32."""
    return from_bits(to_bits(x))
