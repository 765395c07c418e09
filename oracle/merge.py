"""Merge of partial attention results: torch's ``_SDPAMerger``
(torch/distributed/tensor/experimental/_context_parallel/_attention.py:138-223),
which the reference constructs at src/para_attn/sparse_attn.py:174-176,212-214 and
reaches through ``_templated_ring_attention`` at
src/para_attn/para_attn_interface.py:182-193.  Test infrastructure only.
"""
import numpy as np


def _sigmoid(x):
    with np.errstate(over="ignore"):
        return 1.0 / (1.0 + np.exp(-x))


def _logsigmoid(x):
    # min(x, 0) - log1p(exp(-|x|)), the stable form torch uses
    with np.errstate(over="ignore"):
        return np.minimum(x, 0.0) - np.log1p(np.exp(-np.abs(x)))


def merge_step(acc_out, acc_lse, blk_out, blk_lse, dtype=np.float32):
    """One non-first ``_merge_one`` step (_attention.py:182-183):
        out = out - sigmoid(block_lse - lse) * (out - block_out)
        lse = lse - logsigmoid(lse - block_lse)
    acc_out/blk_out [..., Sq, D]; acc_lse/blk_lse [..., Sq].  Computed in ``dtype``
    (fp32 = the merger's convert_to_f32 mode, _attention.py:209-211).
    A row whose accumulator is still empty (lse = -inf) takes the block.
    """
    a = np.asarray(acc_out, dtype=dtype)
    b = np.asarray(blk_out, dtype=dtype)
    la = np.asarray(acc_lse, dtype=dtype)[..., None]
    lb = np.asarray(blk_lse, dtype=dtype)[..., None]
    with np.errstate(invalid="ignore"):
        w = _sigmoid(lb - la)
        out = a - w * (a - b)
        lse = la - _logsigmoid(la - lb)
    empty = np.isneginf(la)
    out = np.where(empty, b, out)
    lse = np.where(empty, lb, lse)
    return out.astype(dtype), lse[..., 0].astype(dtype)


def merge_all(outs, lses, dtype=np.float32):
    """``step`` over a list of partials, then ``results()`` (_attention.py:205-223) without the final cast."""
    acc_out = np.asarray(outs[0], dtype=dtype)
    acc_lse = np.asarray(lses[0], dtype=dtype)
    for o, l in zip(outs[1:], lses[1:]):
        acc_out, acc_lse = merge_step(acc_out, acc_lse, o, l, dtype)
    return acc_out, acc_lse
