"""Host side of the ring-attention merge: a merger object with the interface of
torch's ``_SDPAMerger`` (torch/distributed/tensor/experimental/_context_parallel/
_attention.py:138-223) whose steps run as one fused kernel each, and the
single-rank ring sweep that uses it (the loop of ``_templated_ring_attention``,
_attention.py:422-475, which the reference drives from
src/para_attn/para_attn_interface.py:164-197) with the key/value exchange
replaced by slicing.
"""
from typing import Optional, Tuple

import torch

from . import config, ops


class SDPAMerger:
    """Accumulates partial (out, lse) pairs.

    ``convert_to_f32`` keeps the running output in fp32 between steps, as the
    reference asks for unless ``allow_reduced_precision_compute`` is set
    (src/para_attn/para_attn_interface.py:132-137).  The first step's cast and
    the cast in ``results()`` never run as separate passes: the first partial
    is kept as it came and the second step reads it directly; ``results()`` of
    a single step returns it untouched.
    """

    def __init__(self, convert_to_f32: bool = True, seq_dim: int = 2):
        self._seq_dim = seq_dim
        self._convert_to_f32 = convert_to_f32
        self._out: Optional[torch.Tensor] = None
        self._lse: Optional[torch.Tensor] = None
        self._out_dtype = torch.float32
        self._lse_shape = None
        self._owned = False  # accumulators are private buffers (safe to update in place)

    def step(self, out: torch.Tensor, lse: torch.Tensor, partial: bool = False) -> None:
        if partial:
            raise NotImplementedError("partial (load-balanced causal) merging is not on the reference's path")
        self._out_dtype = out.dtype
        if self._lse_shape is None:
            self._lse_shape = lse.shape
        if lse.dtype != torch.float32:
            lse = lse.float()
        if self._out is None:
            self._out, self._lse = out, lse
            self._owned = False
            return
        acc_dtype = torch.float32 if self._convert_to_f32 else out.dtype
        if self._owned and self._out.dtype == acc_dtype:
            ops.merge_attention_lse_(self._out, self._lse, out, lse)
        else:
            self._out, self._lse = ops.merge_attention_lse(self._out, self._lse, out, lse, acc_dtype)
            self._owned = True

    def results(self) -> Tuple[torch.Tensor, torch.Tensor]:
        assert self._out is not None and self._lse is not None
        out = self._out if self._out.dtype == self._out_dtype else self._out.to(self._out_dtype)
        return out, self._lse.reshape(self._lse_shape)


def _sweepable(query, key_blocks, value_blocks):
    """Whether ``para_attn::attention_forward_sweep`` takes these blocks (head_dim 128, at most 16 blocks of one
    shape, dtype and device, each below 4 GiB per head)."""
    k0 = key_blocks[0]
    if query.shape[-1] != 128 or not 1 < len(key_blocks) <= 16 or k0.shape[2] == 0:
        return False
    if k0.shape[2] * max(k0.stride(2), value_blocks[0].stride(2), 128) * 2 >= (1 << 32) - 8192:
        return False
    return all(t.shape == k0.shape and t.dtype == query.dtype and t.device == query.device for t in list(key_blocks) + list(value_blocks))


def ring_sweep(query, key_blocks, value_blocks, *, scale=None, fused=None):
    """One rank's ring-attention pass: ``query`` against successive key/value blocks.

    Equals one SDPA of ``query`` over the concatenation of all blocks.  ``fused``:
      "sweep"  one launch walks all blocks and carries the softmax state across them in registers (the default
               where the blocks allow it: they are all resident on this GPU, which is what a one-rank sweep is);
      True     one launch per block, each folding its result into an fp32 running pair inside the attention
               kernel (what a rank of a real ring does as blocks arrive; the default otherwise when the
               accumulator is fp32 and head_dim is 128);
      False    attention and merge as two launches per block.
    The last step writes the activation dtype directly, so no separate cast pass runs.
    Returns (out in query.dtype, fp32 lse [B,H,Sq]).
    """
    assert len(key_blocks) == len(value_blocks) and len(key_blocks) > 0
    convert = not config.attention.allow_reduced_precision_compute
    acc_dtype = torch.float32 if convert else query.dtype
    n = len(key_blocks)
    if fused is None:
        fused = "sweep" if _sweepable(query, key_blocks, value_blocks) else (convert and n > 1 and query.shape[-1] == 128)
    if fused == "sweep":
        return ops.attention_forward_sweep(query, list(key_blocks), list(value_blocks), scale=scale)
    if fused:
        # attention and merge in one launch per block: the blocks' own outputs never exist
        B, H, Sq, D = query.shape
        acc_out = torch.empty((B, H, Sq, D), dtype=torch.float32, device=query.device)
        acc_lse = torch.empty((B, H, Sq), dtype=torch.float32, device=query.device)
        try:
            for i, (k, v) in enumerate(zip(key_blocks[:-1], value_blocks[:-1])):
                ops.attention_forward_accumulate_(acc_out, acc_lse, query, k, v, i == 0, scale=scale)
            out = ops.attention_forward_accumulate_final(acc_out, acc_lse, query, key_blocks[-1], value_blocks[-1], scale=scale)
            return out, acc_lse
        except NotImplementedError:
            pass  # a block the fused kernel does not take (K/V of 4 GiB per head): two launches per block below
    acc_out = acc_lse = None
    for i, (k, v) in enumerate(zip(key_blocks, value_blocks)):
        out, lse = ops.attention_forward_with_lse(query, k, v, scale=scale)
        if acc_out is None:
            acc_out, acc_lse = out, lse
        elif i == n - 1:
            acc_out, acc_lse = ops.merge_attention_lse(acc_out, acc_lse, out, lse, query.dtype)
        elif acc_out.dtype != acc_dtype or i == 1:
            acc_out, acc_lse = ops.merge_attention_lse(acc_out, acc_lse, out, lse, acc_dtype)
        else:
            ops.merge_attention_lse_(acc_out, acc_lse, out, lse)
    return acc_out, acc_lse
