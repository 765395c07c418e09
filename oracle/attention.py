"""Dense attention with log-sum-exp: what the aten kernels behind
``attention_forward_with_lse`` compute (src/para_attn/ops/__init__.py:48-157).
Test infrastructure only.
"""
import math

import numpy as np


def sdpa_lse_f64(q, k, v, scale=None, keep=None):
    """Closed form in fp64.

    q [..., Sq, D], k [..., Skv, D], v [..., Skv, Dv] (any float arrays).
    keep: optional bool array broadcastable to [..., Sq, Skv]; False = -inf.
    Returns (out [..., Sq, Dv], lse [..., Sq]) in fp64; lse is the natural-log
    sum of exp(scale * q.k) over kept keys (the logsumexp the flash kernels
    return, ops/__init__.py:58-65), -inf and out = 0 for a row that keeps nothing.
    """
    q = np.asarray(q, dtype=np.float64)
    k = np.asarray(k, dtype=np.float64)
    v = np.asarray(v, dtype=np.float64)
    if scale is None:
        scale = 1.0 / math.sqrt(q.shape[-1])
    s = np.matmul(q, np.swapaxes(k, -1, -2)) * scale
    if keep is not None:
        s = np.where(keep, s, -np.inf)
    m = np.max(s, axis=-1, keepdims=True)
    m_safe = np.where(np.isfinite(m), m, 0.0)
    p = np.exp(s - m_safe)
    l = np.sum(p, axis=-1, keepdims=True)
    with np.errstate(divide="ignore", invalid="ignore"):
        out = np.where(l > 0, np.matmul(p, v) / np.where(l > 0, l, 1.0), 0.0)
        lse = np.where(l[..., 0] > 0, m_safe[..., 0] + np.log(np.where(l[..., 0] > 0, l[..., 0], 1.0)), -np.inf)
    return out, lse


def causal_keep(Sq, Skv):
    """torch's is_causal mask (what the aten kernels apply for
    src/para_attn/ops/__init__.py:117, 138): query i keeps keys j <= i, the lower
    triangle aligned at the top-left corner, for any Sq and Skv."""
    return np.arange(Skv)[None, :] <= np.arange(Sq)[:, None]


def sdpa_lse_torch_cpu(q, k, v, scale=None, attn_mask=None, is_causal=False):
    """torch's CPU flash kernel: the library routine the reference's SDPA path reduces
    to off-GPU (bit-equal to F.scaled_dot_product_attention on CPU).

    q,k,v: CPU torch tensors [B,H,S,D].  attn_mask: None, or a bool / additive mask
    broadcastable to [B,H,Sq,Skv].  Returns (out in q.dtype, fp32 lse [B,H,Sq]).
    """
    import torch

    mask = attn_mask
    if mask is not None and mask.dtype == torch.bool:
        mask = torch.zeros(mask.shape, dtype=q.dtype).masked_fill_(~mask, float("-inf"))
    out, lse = torch.ops.aten._scaled_dot_product_flash_attention_for_cpu(
        q, k, v, dropout_p=0.0, is_causal=is_causal, attn_mask=mask, scale=scale
    )
    return out, lse
