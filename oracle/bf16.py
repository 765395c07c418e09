"""Round-to-nearest-even bf16 / fp16 rounding in numpy (test infrastructure)."""
import numpy as np


def round_bf16(x):
    """fp32 array -> nearest bf16 value, returned as fp32 (ties to even, NaN kept)."""
    x = np.ascontiguousarray(x, dtype=np.float32)
    u = x.view(np.uint32)
    r = (u >> np.uint32(16)) & np.uint32(1)
    r += np.uint32(0x7FFF)
    r += u
    r &= np.uint32(0xFFFF0000)
    r = r.view(np.float32)
    nan = np.isnan(x)
    if nan.any():
        r[nan] = x[nan]
    return r


def round_f16(x):
    return np.asarray(x, dtype=np.float32).astype(np.float16).astype(np.float32)


def round_to(x, dtype_name):
    if dtype_name == "bf16":
        return round_bf16(x)
    if dtype_name == "f16":
        return round_f16(x)
    if dtype_name == "f32":
        return np.asarray(x, dtype=np.float32)
    raise ValueError(dtype_name)
