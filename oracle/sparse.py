"""Block-sparse attention as the reference's ``StructuredSparseAttnFunc.forward`` does it
(src/para_attn/sparse_attn.py:74-278).  Test infrastructure only.
"""
import numpy as np

from .attention import sdpa_lse_f64
from .merge import merge_all


def mask_row_runs(mask_row):
    """Runs [start, end) of kept blocks in one mask row, found exactly as the reference's
    scan does (sparse_attn.py:215-234: skip False, extend while True, restart at end + 1)."""
    runs = []
    start = 0
    n = len(mask_row)
    while start < n:
        if not mask_row[start]:
            start += 1
            continue
        end = start + 1
        while end < n and mask_row[end]:
            end += 1
        runs.append((start, end))
        start = end + 1
    return runs


def expand_block_mask(block_mask, Sq, Skv, q_range=None, kv_range=None):
    """Element-level keep mask [..., Sq, Skv] of a block mask [..., nQ, nK]: rows outside
    q_range and keys outside kv_range are dense (sparse_attn.py:133-171, 178-189, 247-274)."""
    bm = np.asarray(block_mask, dtype=bool)
    nQ, nK = bm.shape[-2:]
    q_lo, q_hi = q_range if q_range is not None else (0, Sq)
    kv_lo, kv_hi = kv_range if kv_range is not None else (0, Skv)
    assert (q_hi - q_lo) % nQ == 0 and (kv_hi - kv_lo) % nK == 0  # sparse_attn.py:124-131
    qb, kb = (q_hi - q_lo) // nQ, (kv_hi - kv_lo) // nK
    keep = np.ones(bm.shape[:-2] + (Sq, Skv), dtype=bool)
    mid = np.repeat(np.repeat(bm, qb, axis=-2), kb, axis=-1)
    keep[..., q_lo:q_hi, kv_lo:kv_hi] = mid
    return keep


def struct_sparse_f64(q, k, v, block_mask, scale=None, q_range=None, kv_range=None):
    """The reference's algorithm, step for step, in fp64: per query chunk one dense
    attention per run of kept key blocks, merged by LSE (sparse_attn.py:209-243), the left
    and right key margins merged in (:178-189, :247-258), dense query margins (:158-171,
    :263-274).  block_mask is 2-D [nQ,nK] as in the reference (:107).
    Returns (out, lse) for q [B,H,Sq,D]."""
    q = np.asarray(q, dtype=np.float64)
    k = np.asarray(k, dtype=np.float64)
    v = np.asarray(v, dtype=np.float64)
    bm = np.asarray(block_mask, dtype=bool)
    assert bm.ndim == 2
    Sq, Skv = q.shape[2], k.shape[2]
    q_lo, q_hi = q_range if q_range is not None else (0, Sq)
    kv_lo, kv_hi = kv_range if kv_range is not None else (0, Skv)
    nQ, nK = bm.shape
    qb, kb = (q_hi - q_lo) // nQ, (kv_hi - kv_lo) // nK
    out = np.zeros(q.shape[:3] + (v.shape[3],))
    lse = np.full(q.shape[:3], -np.inf)
    if q_lo > 0:
        out[:, :, :q_lo], lse[:, :, :q_lo] = sdpa_lse_f64(q[:, :, :q_lo], k, v, scale)
    if q_hi < Sq:
        out[:, :, q_hi:], lse[:, :, q_hi:] = sdpa_lse_f64(q[:, :, q_hi:], k, v, scale)
    for i in range(nQ):
        rows = slice(q_lo + i * qb, q_lo + (i + 1) * qb)
        qc = q[:, :, rows]
        outs, lses = [], []
        if kv_lo > 0:
            o, l = sdpa_lse_f64(qc, k[:, :, :kv_lo], v[:, :, :kv_lo], scale)
            outs.append(o), lses.append(l)
        sub_o, sub_l = [], []
        for (s, e) in mask_row_runs(bm[i]):
            ks = slice(kv_lo + s * kb, kv_lo + e * kb)
            o, l = sdpa_lse_f64(qc, k[:, :, ks], v[:, :, ks], scale)
            sub_o.append(o), sub_l.append(l)
        if sub_o:
            o, l = merge_all(sub_o, sub_l, dtype=np.float64)
            outs.append(o), lses.append(l)
        if kv_hi < Skv:
            o, l = sdpa_lse_f64(qc, k[:, :, kv_hi:], v[:, :, kv_hi:], scale)
            outs.append(o), lses.append(l)
        if outs:
            out[:, :, rows], lse[:, :, rows] = merge_all(outs, lses, dtype=np.float64)
    return out, lse


def block_sparse_torch_cpu(q, k, v, block_mask, scale=None):
    """Block-sparse attention at sizes the fp64 form cannot hold: per (head, query block) gather
    the kept key blocks and run torch's CPU SDPA on them (the reference's own strategy,
    sparse_attn.py:223-233, with the runs concatenated instead of merged).
    q,k,v CPU tensors [1,H,S,D]; block_mask bool [H or 1, nQ, nK]; returns (out, fp32 lse)."""
    import torch

    from .attention import sdpa_lse_torch_cpu

    B, H, Sq, D = q.shape
    Skv = k.shape[2]
    if block_mask.ndim == 2:
        block_mask = block_mask[None]
    Hm, nQ, nK = block_mask.shape
    qb, kb = Sq // nQ, Skv // nK
    out = torch.zeros_like(q)
    lse = torch.full((B, H, Sq), float("-inf"), dtype=torch.float32)
    for h in range(H):
        bm = block_mask[h if Hm > 1 else 0]
        kh = k[:, h : h + 1].reshape(B, 1, nK, kb, D)
        vh = v[:, h : h + 1].reshape(B, 1, nK, kb, D)
        for i in range(nQ):
            idx = torch.nonzero(bm[i]).flatten()
            if idx.numel() == 0:
                continue
            ks = kh[:, :, idx].reshape(B, 1, -1, D)
            vs = vh[:, :, idx].reshape(B, 1, -1, D)
            o, l = sdpa_lse_torch_cpu(q[:, h : h + 1, i * qb : (i + 1) * qb], ks, vs, scale)
            out[:, h : h + 1, i * qb : (i + 1) * qb] = o
            lse[:, h : h + 1, i * qb : (i + 1) * qb] = l
    return out, lse
