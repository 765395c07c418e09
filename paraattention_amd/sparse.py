"""Block-sparse attention behind the reference's struct-sparse interface
(src/para_attn/sparse_attn.py:285-311, 643-693): same arguments, one kernel
launch instead of a Python loop of SDPA calls and merges.
"""
import weakref

import torch
import torch.nn.functional as F

from . import ops
from .interface import _SdpaMode

_RUNS_CACHE_ENTRIES = 4


def struct_sparse_attn_func(
    query,
    key,
    value,
    attn_mask=None,
    dropout_p=0.0,
    is_causal=False,
    *,
    scale=None,
    sparse_mask=None,
    sparse_range_query=None,
    sparse_range_key_value=None,
    print_attn_weight_means=False,
    runs_cache=None,
):
    """Signature of the reference's ``struct_sparse_attn_func`` (sparse_attn.py:285-311), plus ``runs_cache``:
    a dict in which the key ranges extracted from the mask are kept, so that a mask that serves many calls
    (``StructSparseAttnMode`` passes its own) is scanned once per key length and not once per call.

    ``sparse_mask`` is the reference's 2-D bool [nQ,nK]; a 3-D [H,nQ,nK] mask (one
    per head) is accepted as well.  Returns the output only, like the reference
    (the LSE is dropped at sparse_attn.py:260).
    """
    if sparse_mask is None:
        return F.scaled_dot_product_attention(
            query, key, value, attn_mask=attn_mask, dropout_p=dropout_p, is_causal=is_causal, scale=scale
        )
    assert query.ndim == 4, f"query must have 4 dimensions, got {query.ndim}"
    assert key.ndim == 4, f"key must have 4 dimensions, got {key.ndim}"
    assert value.ndim == 4, f"value must have 4 dimensions, got {value.ndim}"
    assert not is_causal, "is_causal is not supported in struct_sparse_attn_func"
    assert sparse_mask.ndim in (2, 3), f"sparse_mask must have 2 (or 3) dimensions, got {sparse_mask.ndim}"
    if attn_mask is not None or dropout_p != 0.0:
        raise NotImplementedError("attn_mask / dropout are not supported together with sparse_mask")
    if print_attn_weight_means:
        raise NotImplementedError("print_attn_weight_means is a debugging aid of the reference and is not provided")
    s_q, s_kv = query.shape[2], value.shape[2]
    q_lo, q_hi = sparse_range_query if sparse_range_query is not None else (0, s_q)
    kv_lo, kv_hi = sparse_range_key_value if sparse_range_key_value is not None else (0, s_kv)
    assert 0 <= q_lo <= q_hi <= s_q, f"sparse_range_query must be in [0, {s_q}], got {(q_lo, q_hi)}"
    assert 0 <= kv_lo <= kv_hi <= s_kv, f"sparse_range_key_value must be in [0, {s_kv}], got {(kv_lo, kv_hi)}"
    assert (q_hi - q_lo) % sparse_mask.shape[-2] == 0, "sparse_mask must divide the query dimension"
    assert (kv_hi - kv_lo) % sparse_mask.shape[-1] == 0, "sparse_mask must divide the key/value dimension"
    if runs_cache is None:
        mask = sparse_mask.to(device=query.device, dtype=torch.bool)
        out, _ = ops.attention_forward_block_sparse(query, key, value, mask, q_lo, q_hi, kv_lo, kv_hi, scale=scale)
        return out
    # An entry serves one (key length, sparse key range, device); it remembers which mask it was built from by a
    # weak reference (an id() alone could be a later tensor at a freed one's address) and by the mask's version
    # counter (in-place edits bump it).  A few entries are kept, so a model that sends two or three key lengths
    # through the mode in one step scans the mask once for each and not once per call.
    tag = (query.device, s_kv, kv_lo, kv_hi)
    entry = runs_cache.get(tag)
    if entry is not None and (entry[0]() is not sparse_mask or entry[1] != sparse_mask._version):
        entry = None
    if entry is None:
        mask = sparse_mask.to(device=query.device, dtype=torch.bool)
        runs = ops.block_sparse_key_runs(mask, s_kv, kv_lo, kv_hi)
        runs_cache.pop(tag, None)
        while len(runs_cache) >= _RUNS_CACHE_ENTRIES:
            runs_cache.pop(next(iter(runs_cache)))  # oldest first
        runs_cache[tag] = entry = (weakref.ref(sparse_mask), sparse_mask._version, runs)
    runs = entry[2]
    shape = (1, *sparse_mask.shape) if sparse_mask.ndim == 2 else tuple(sparse_mask.shape)
    out, _ = ops.attention_forward_block_sparse_runs(query, key, value, runs, shape[0], shape[1], shape[2], q_lo, q_hi, scale=scale)
    return out


class StructSparseAttnMode(_SdpaMode):
    """Reroutes ``F.scaled_dot_product_attention`` to the block-sparse kernel while active
    (the reference's mode of the same name, src/para_attn/sparse_attn.py:643-693), with the class-wide
    ``disabled`` switch and ``disable()`` context of the other modes (:679-692)."""

    disabled = False

    @torch.compiler.disable
    def __init__(self, *, sparse_mask=None, sparse_range_query=None, sparse_range_key_value=None,
                 print_attn_weight_means=False):
        super().__init__()
        self._sparse = dict(sparse_mask=sparse_mask, sparse_range_query=sparse_range_query,
                            sparse_range_key_value=sparse_range_key_value,
                            print_attn_weight_means=print_attn_weight_means,
                            runs_cache={} if sparse_mask is not None else None)

    def _call(self, *args, **kwargs):
        return struct_sparse_attn_func(*args, **kwargs, **self._sparse)
