"""First Block Cache similarity test (src/para_attn/first_block_cache/utils.py:220-234)
and the gates in front of it (utils.py:269-286), restated with torch's rounding chain.
Test infrastructure only.
"""
import numpy as np

from .bf16 import round_to


def residual_diff_ratio(t1, t2, dtype_name="bf16"):
    """``(t1 - t2).abs().mean() / t1.abs().mean()`` (utils.py:228-233) for activations of
    ``dtype_name`` ("bf16", "f16" or "f32"), inputs given as fp32 arrays holding
    representable values.  Rounding, as torch's eager ops do it:
      * t1 - t2 is computed in fp32 and rounded to the dtype per element;
      * each mean accumulates wide; the mean (not the sum) is rounded to the dtype once;
      * the quotient of the two rounded means is rounded to the dtype.
    Returns (ratio, mean_diff, mean_t1) as Python floats.
    """
    a = np.asarray(t1, dtype=np.float32)
    b = np.asarray(t2, dtype=np.float32)
    assert a.shape == b.shape and a.size > 0
    d = np.abs(round_to(a - b, dtype_name))
    n = a.size
    mean_d = round_to(np.float32(np.sum(d, dtype=np.float64) / n), dtype_name)
    mean_a = round_to(np.float32(np.sum(np.abs(a), dtype=np.float64) / n), dtype_name)
    with np.errstate(divide="ignore", invalid="ignore"):
        ratio = round_to(np.float32(mean_d) / np.float32(mean_a), dtype_name)
    return float(np.asarray(ratio).reshape(())), float(np.asarray(mean_d).reshape(())), float(np.asarray(mean_a).reshape(()))


def are_two_tensors_similar(t1, t2, threshold, dtype_name="bf16"):
    """utils.py:220-234: threshold <= 0 -> False; shape mismatch -> False; strict ``<``."""
    if threshold <= 0.0:
        return False
    if np.shape(t1) != np.shape(t2):
        return False
    return residual_diff_ratio(t1, t2, dtype_name)[0] < threshold


def get_can_use_cache(prev, cur, threshold, *, in_warmup=False, downsample_factor=1, dtype_name="bf16"):
    """utils.py:269-286: warm-up gate (:271), threshold gate (:273-275), ``[..., ::k]`` on the
    fresh residual (:276-278), missing previous residual (:280), then the similarity test.
    ``prev`` is the stored residual (already down-sampled when k > 1, utils.py:289-295)."""
    if in_warmup:
        return False
    if threshold <= 0.0:
        return False
    if downsample_factor > 1:
        cur = np.asarray(cur)[..., ::downsample_factor]
    if prev is None:
        return False
    return are_two_tensors_similar(prev, cur, threshold, dtype_name)
