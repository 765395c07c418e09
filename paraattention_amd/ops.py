"""The attention op layer: same op names and schemas as the reference's
``para_attn.ops`` (src/para_attn/ops/__init__.py:160-343), backed by the gfx950
kernels of libparaattn_hip.so instead of aten CUDA kernels.

Registered in the ``para_attn`` namespace so ``torch.ops.para_attn.<name>`` and
``torch.compile`` graphs resolve exactly as they do with the reference.  The ops
exist for device type "cuda" only (which is what ROCm devices report): a CPU
tensor raises from the dispatcher, as the reference's own assert does
(src/para_attn/ops/__init__.py:123).

Ops with a counterpart in the reference:
  attention_forward_with_lse   (ops/__init__.py:160-201)
  attention_forward            (ops/__init__.py:204-245)
  attention_forward_sparse_kv  (ops/__init__.py:248-343)
Ops the reference has no name for, because there the arithmetic is a chain of
torch elementwise calls:
  merge_attention_lse / merge_attention_lse_   (torch _SDPAMerger._merge_one)
  attention_forward_accumulate_ / _final       (attention + merge step in one launch)
  attention_forward_sweep                      (a whole ring sweep over resident key/value blocks in one launch)
  attention_forward_block_sparse               (sparse_attn.py:74-278)
  block_sparse_key_runs, attention_forward_block_sparse_runs  (the same with the mask's run scan done once)
  fbcache_residual_diff                        (first_block_cache/utils.py:228-233)
  fbcache_first_residual_diff, fbcache_apply_residual (utils.py:359, 237-259)
  taylorseer_derivatives, taylorseer_value     (first_block_cache/taylorseer.py:29-48)
"""
import ctypes
import math
from typing import List, Optional, Tuple

import torch

from . import _lib

_DTYPE_CODE = {torch.bfloat16: _lib.PA_DTYPE_BF16, torch.float16: _lib.PA_DTYPE_F16, torch.float32: _lib.PA_DTYPE_F32}


def _stream_ptr(device):
    return ctypes.c_void_p(torch.cuda.current_stream(device).cuda_stream)


def _ptr(t):
    return ctypes.c_void_p(t.data_ptr()) if t is not None else None


def _ptr_array(tensors):
    return (ctypes.c_void_p * len(tensors))(*[t.data_ptr() for t in tensors])


def _kernel_ready(t):
    """Rows must be unit-stride and 16-byte aligned for the kernels' vector loads."""
    if t.stride(-1) != 1 or any(t.shape[d] > 1 and t.stride(d) % 8 for d in range(t.ndim - 1)) or t.data_ptr() % 16:
        return t.contiguous()
    return t


def _native_head_dims(query, value):
    """The kernels are built for head_dim 64 and 128 with values as wide as the keys; anything else up to 128 runs
    through them zero-padded (``_pad_head_dims``)."""
    return query.shape[-1] == value.shape[-1] and query.shape[-1] in (64, 128)


def _pad_head_dims(query, key, value, scale):
    """q, k, v with head_dim zero-padded to 64 or 128 and the scale of the true head_dim.  Zero columns add nothing
    to q.k, and the padded columns of v give output columns that are dropped, so the result is that of the unpadded
    problem: head_dim 32, 40, 72, 80, 96 ... and values narrower or wider than the keys (which aten's kernels behind
    src/para_attn/ops/__init__.py:58-109 take directly) at the price of one copy of each operand."""
    D, Dv = query.shape[-1], value.shape[-1]
    to = 64 if max(D, Dv) <= 64 else 128
    if scale is None:
        scale = 1.0 / math.sqrt(D)
    pad = torch.nn.functional.pad
    return pad(query, (0, to - D)), pad(key, (0, to - D)), pad(value, (0, to - Dv)), scale


def _out_like(query, value=None):
    """The attention output for ``query``: the query's own memory layout (a [B,S,H,D]-memory view stays one, so the
    caller's transpose back is free) whenever the kernels can write it -- unit head_dim stride, 16-byte aligned rows
    -- and contiguous otherwise (also for the head_dims that run zero-padded).  Reads sizes and strides only, so
    the fake implementations allocate through it too and a compiled graph is planned against the strides the
    kernel really writes."""
    if value is not None and not _native_head_dims(query, value):
        return torch.empty((*query.shape[:3], value.shape[-1]), dtype=query.dtype, device=query.device)
    out = torch.empty_like(query)
    if out.stride(-1) != 1 or any(out.shape[d] > 1 and out.stride(d) % 8 for d in range(out.ndim - 1)):
        out = torch.empty(query.shape, dtype=query.dtype, device=query.device)
    return out


def _lse_like(query):
    B, H, Sq, _ = query.shape
    return torch.empty((B, H, Sq), dtype=torch.float32, device=query.device)


def _same_device(ref, **operands):
    """The kernels take raw pointers, so an operand on another device (a CPU mask beside GPU activations) must stop
    here with an error, as it does in the aten ops the reference calls, and not at a memory fault on the GPU.
    Every function below that hands a tensor's pointer to the library runs its tensors through this first."""
    for name, t in operands.items():
        if t is not None and t.device != ref.device:
            raise ValueError(f"{name} is on {t.device} but must be on {ref.device}: all operands must share one device")


def _check_sdpa_args(query, key, value, dropout_p, is_causal, attn_mask=None, causal_ok=False, any_head_dim=False):
    if query.ndim != 4 or key.ndim != 4 or value.ndim != 4:
        raise ValueError("query, key and value must be 4-D [batch, heads, seq, head_dim]")
    _same_device(query, key=key, value=value, attn_mask=attn_mask)
    if dropout_p != 0.0:
        raise NotImplementedError("dropout_p > 0 is not supported (the reference's hot path is inference only)")
    if is_causal and not causal_ok:
        raise NotImplementedError("is_causal=True is not supported by this op")
    if is_causal and attn_mask is not None:
        raise ValueError("an explicit attn_mask must not be set when is_causal=True")  # as torch's SDPA
    if query.dtype not in (torch.bfloat16, torch.float16):
        raise NotImplementedError(f"attention dtype {query.dtype} not supported (bf16 / fp16)")
    if key.dtype != query.dtype or value.dtype != query.dtype:
        raise ValueError("query, key and value must share one dtype")
    B, H, Sq, D = query.shape
    if key.shape[0] != B or key.shape[1] != H or key.shape[3] != D:
        raise ValueError(f"key shape {tuple(key.shape)} does not match query {tuple(query.shape)}")
    if value.shape[:3] != key.shape[:3]:
        raise ValueError(f"value shape {tuple(value.shape)} does not match key {tuple(key.shape)}")
    if (value.shape[3] != D or D not in (64, 128)) and not any_head_dim:
        raise NotImplementedError(f"head_dim {D} / value width {value.shape[3]}: this op takes 64 or 128 with values as wide as the keys")
    if max(D, value.shape[3]) > 128 or min(D, value.shape[3]) < 1:
        raise NotImplementedError(f"head_dim {D} / value width {value.shape[3]} not supported (1..128)")


def _dense_forward(query, key, value, scale, want_lse, kv_len=None, is_causal=False):
    B, H, Sq, D = query.shape
    Skv = key.shape[2]
    _same_device(query, key=key, value=value, kv_len=kv_len)
    q, k, v = _kernel_ready(query), _kernel_ready(key), _kernel_ready(value)
    out = _out_like(query)
    lse = _lse_like(query) if want_lse else None
    if scale is None:
        scale = 1.0 / math.sqrt(D)
    lib = _lib.load()
    with torch.cuda.device(q.device):
        # scratch for the score bound and the key-split tail of the launch (torch's caching allocator:
        # no hipMalloc in the steady state); its lifetime on the launch stream is the allocator's business
        ks, vs = _lib.strides3(k), _lib.strides3(v)
        ws_bytes = lib.pa_attn_fwd_call_workspace_bytes(B, H, Sq, Skv, D, ks, vs, 0 if kv_len is None else 1, 1 if is_causal else 0)
        ws = torch.empty(ws_bytes, dtype=torch.uint8, device=q.device) if ws_bytes else None
        rc = lib.pa_attn_fwd_lse_ws(
            _ptr(q), _ptr(k), _ptr(v), _ptr(out), _ptr(lse), _DTYPE_CODE[q.dtype], B, H, Sq, Skv, D,
            _lib.strides3(q), ks, vs, _lib.strides3(out),
            float(scale), _ptr(kv_len), 1 if is_causal else 0, _ptr(ws), ws_bytes, _stream_ptr(q.device),
        )
    _lib.check(rc, "pa_attn_fwd_lse_ws")
    return out, lse


def _accumulate_forward(acc_out, acc_lse, query, key, value, scale, first, final):
    """One fused ring step (pa_attn_fwd_accumulate); returns the 16-bit output if ``final``."""
    B, H, Sq, D = query.shape
    Skv = key.shape[2]
    if acc_out.dtype != torch.float32 or acc_lse.dtype != torch.float32:
        raise ValueError("accumulators must be fp32")
    if tuple(acc_out.shape) != (B, H, Sq, D) or tuple(acc_lse.shape) != (B, H, Sq):
        raise ValueError("accumulator shapes must be [B,H,Sq,D] and [B,H,Sq]")
    if not acc_out.is_contiguous() or not acc_lse.is_contiguous():
        raise ValueError("accumulators must be contiguous")
    _same_device(query, key=key, value=value, acc_out=acc_out, acc_lse=acc_lse)
    q, k, v = _kernel_ready(query), _kernel_ready(key), _kernel_ready(value)
    out = torch.empty(q.shape, dtype=q.dtype, device=q.device) if final else None
    if scale is None:
        scale = 1.0 / math.sqrt(D)
    lib = _lib.load()
    with torch.cuda.device(q.device):
        ks, vs = _lib.strides3(k), _lib.strides3(v)
        ws_bytes = lib.pa_attn_fwd_workspace_bytes(B, H, Sq, Skv, D, ks, vs)
        ws = torch.empty(ws_bytes, dtype=torch.uint8, device=q.device) if ws_bytes else None
        rc = lib.pa_attn_fwd_accumulate(
            _ptr(q), _ptr(k), _ptr(v), _ptr(acc_out), _ptr(acc_lse), _ptr(out), _DTYPE_CODE[q.dtype], B, H, Sq, Skv, D,
            _lib.strides3(q), ks, vs, _lib.strides3(out) if final else None,
            float(scale), None, 1 if first else 0, _ptr(ws), ws_bytes, _stream_ptr(q.device),
        )
    _lib.check(rc, "pa_attn_fwd_accumulate")
    return out


def _broadcast_mask(attn_mask, B, H, Sq, Skv, dtype):
    """The mask as torch's SDPA reads it: trailing dimensions aligned with [B,H,Sq,Skv], every dimension full or 1
    (src/para_attn/ops/__init__.py:215-223 hands it to F.scaled_dot_product_attention as it came).  Returns
    (tensor to pass, mask kind, (batch, head, query, key) strides in elements with 0 on broadcast dimensions)."""
    m = attn_mask
    if m.ndim > 4:
        raise ValueError(f"attn_mask has {m.ndim} dimensions; at most 4 ([B,H,Sq,Skv]) broadcast against the scores")
    while m.ndim < 4:
        m = m.unsqueeze(0)
    full = (B, H, Sq, Skv)
    for d in range(4):
        if m.shape[d] not in (1, full[d]):
            raise ValueError(f"attn_mask shape {tuple(attn_mask.shape)} does not broadcast to {full}")
    if m.dtype == torch.bool:
        kind = _lib.PA_MASK_BOOL
    elif m.dtype == torch.float32:
        kind = _lib.PA_MASK_F32
    elif m.dtype == dtype:
        kind = _lib.PA_MASK_ACT
    elif m.is_floating_point():
        m, kind = m.float(), _lib.PA_MASK_F32
    else:
        raise ValueError(f"attn_mask must be boolean or floating point, got {m.dtype}")
    strides = [0 if m.shape[d] == 1 else m.stride(d) for d in range(4)]
    return m, kind, (ctypes.c_int64 * 4)(*strides)


def _masked_forward(query, key, value, attn_mask, scale, want_lse, is_causal=False):
    """attn_mask / is_causal handling shared by the three SDPA-signature ops.  Nothing here reads the mask on
    the host: whether a key mask is a prefix is settled on the device (pa_attn_fwd_masked), so masked calls can
    be captured in a HIP graph like the unmasked ones."""
    if not _native_head_dims(query, value):
        q, k, v, scale = _pad_head_dims(query, key, value, scale)
        out, lse = _masked_forward(q, k, v, attn_mask, scale, want_lse, is_causal)
        return out[..., : value.shape[-1]].contiguous(), lse
    if attn_mask is None:
        return _dense_forward(query, key, value, scale, want_lse, is_causal=is_causal)
    B, H, Sq, D = query.shape
    Skv = key.shape[2]
    _same_device(query, key=key, value=value, attn_mask=attn_mask)
    mask, kind, mstrides = _broadcast_mask(attn_mask, B, H, Sq, Skv, query.dtype)
    q, k, v = _kernel_ready(query), _kernel_ready(key), _kernel_ready(value)
    out = _out_like(query)
    lse = _lse_like(query) if want_lse else None
    if scale is None:
        scale = 1.0 / math.sqrt(D)
    lib = _lib.load()
    with torch.cuda.device(q.device):
        ks, vs = _lib.strides3(k), _lib.strides3(v)
        ws_bytes = lib.pa_attn_fwd_masked_workspace_bytes(B, H, Sq, Skv, D, ks, vs)
        ws = torch.empty(ws_bytes, dtype=torch.uint8, device=q.device) if ws_bytes else None
        rc = lib.pa_attn_fwd_masked(
            _ptr(q), _ptr(k), _ptr(v), _ptr(out), _ptr(lse), _DTYPE_CODE[q.dtype], B, H, Sq, Skv, D,
            _lib.strides3(q), ks, vs, _lib.strides3(out), float(scale),
            _ptr(mask), kind, mstrides, _ptr(ws), ws_bytes, _stream_ptr(q.device),
        )
    _lib.check(rc, "pa_attn_fwd_masked")
    return out, lse


# ---------------------------------------------------------------------------------
# ops that exist in the reference
# ---------------------------------------------------------------------------------
@torch.library.custom_op("para_attn::attention_forward_with_lse", mutates_args=(), device_types=("cuda",))
def attention_forward_with_lse(
    query: torch.Tensor,
    key: torch.Tensor,
    value: torch.Tensor,
    attn_mask: Optional[torch.Tensor] = None,
    dropout_p: float = 0.0,
    is_causal: bool = False,
    *,
    scale: Optional[float] = None,
) -> Tuple[torch.Tensor, torch.Tensor]:
    """out [B,H,Sq,D] in query's dtype and natural-log LSE [B,H,Sq] in fp32
    (src/para_attn/ops/__init__.py:160-179)."""
    _check_sdpa_args(query, key, value, dropout_p, is_causal, attn_mask, causal_ok=True, any_head_dim=True)
    out, lse = _masked_forward(query, key, value, attn_mask, scale, True, is_causal)
    return out, lse


@torch.library.register_fake("para_attn::attention_forward_with_lse")
def _(query, key, value, attn_mask=None, dropout_p=0.0, is_causal=False, *, scale=None):
    return _out_like(query, value), _lse_like(query)


@torch.library.custom_op("para_attn::attention_forward", mutates_args=(), device_types=("cuda",))
def attention_forward(
    query: torch.Tensor,
    key: torch.Tensor,
    value: torch.Tensor,
    attn_mask: Optional[torch.Tensor] = None,
    dropout_p: float = 0.0,
    is_causal: bool = False,
    *,
    scale: Optional[float] = None,
) -> torch.Tensor:
    """Plain SDPA forward, no LSE (src/para_attn/ops/__init__.py:204-223)."""
    _check_sdpa_args(query, key, value, dropout_p, is_causal, attn_mask, causal_ok=True, any_head_dim=True)
    out, _ = _masked_forward(query, key, value, attn_mask, scale, False, is_causal)
    return out


@torch.library.register_fake("para_attn::attention_forward")
def _(query, key, value, attn_mask=None, dropout_p=0.0, is_causal=False, *, scale=None):
    return _out_like(query, value)


@torch.library.custom_op("para_attn::attention_forward_sparse_kv", mutates_args=(), device_types=("cuda",))
def attention_forward_sparse_kv(
    query: torch.Tensor,
    key: torch.Tensor,
    value: torch.Tensor,
    attn_mask: Optional[torch.Tensor] = None,
    dropout_p: float = 0.0,
    is_causal: bool = False,
    *,
    scale: Optional[float] = None,
) -> torch.Tensor:
    """SDPA over the keys a boolean mask keeps (src/para_attn/ops/__init__.py:248-321).

    As in the reference the mask is reduced to its first head and first query
    row per batch element (ops/__init__.py:280-282), must be boolean (:269) and
    excludes is_causal (:270).  A prefix mask (valid text length) costs nothing:
    the kernel just stops at the per-batch key count.
    """
    _check_sdpa_args(query, key, value, dropout_p, is_causal, attn_mask, any_head_dim=True)
    if attn_mask is None:
        return _masked_forward(query, key, value, None, scale, False)[0]
    if attn_mask.dtype != torch.bool:
        raise AssertionError("attn_mask must be a boolean tensor")
    m = attn_mask
    if m.shape[-1] != key.shape[2]:
        raise ValueError(f"attn_mask's last dimension {m.shape[-1]} is not the key length {key.shape[2]}")
    if m.shape[0] != query.shape[0]:
        m = m.expand(query.shape[0], *m.shape[1:])
    while m.ndim > 2:
        m = m[:, 0]
    out, _ = _masked_forward(query, key, value, m[:, None, None, :], scale, False)
    return out


@torch.library.register_fake("para_attn::attention_forward_sparse_kv")
def _(query, key, value, attn_mask=None, dropout_p=0.0, is_causal=False, *, scale=None):
    return _out_like(query, value)


# ---------------------------------------------------------------------------------
# merge of partial attention results
# ---------------------------------------------------------------------------------
def _merge_launch(acc_out, acc_lse, blk_out, blk_lse, out, lse_out):
    D = acc_out.shape[-1]
    rows = acc_out.numel() // D if D else 0
    lib = _lib.load()
    with torch.cuda.device(acc_out.device):
        rc = lib.pa_merge_lse(
            _ptr(acc_out), _DTYPE_CODE[acc_out.dtype], _ptr(acc_lse),
            _ptr(blk_out), _DTYPE_CODE[blk_out.dtype], _ptr(blk_lse),
            _ptr(out), _DTYPE_CODE[out.dtype], _ptr(lse_out), rows, D, _stream_ptr(acc_out.device),
        )
    _lib.check(rc, "pa_merge_lse")


def _check_merge_args(acc_out, acc_lse, blk_out, blk_lse):
    _same_device(acc_out, acc_lse=acc_lse, blk_out=blk_out, blk_lse=blk_lse)
    if acc_out.shape != blk_out.shape:
        raise ValueError(f"partial outputs differ in shape: {tuple(acc_out.shape)} vs {tuple(blk_out.shape)}")
    rows = acc_out.numel() // max(acc_out.shape[-1], 1)
    if acc_lse.numel() != rows or blk_lse.numel() != rows:
        raise ValueError("LSE must have one value per output row ([...,Sq] or [...,Sq,1])")
    if acc_lse.dtype != torch.float32 or blk_lse.dtype != torch.float32:
        raise NotImplementedError("LSE must be fp32")
    for t in (acc_out, blk_out):
        if t.dtype not in _DTYPE_CODE:
            raise NotImplementedError(f"dtype {t.dtype} not supported by the merge kernel")


@torch.library.custom_op("para_attn::merge_attention_lse", mutates_args=(), device_types=("cuda",))
def merge_attention_lse(
    acc_out: torch.Tensor,
    acc_lse: torch.Tensor,
    blk_out: torch.Tensor,
    blk_lse: torch.Tensor,
    out_dtype: Optional[torch.dtype] = None,
) -> Tuple[torch.Tensor, torch.Tensor]:
    """One functional merge step: returns (out, lse) of the two partial results combined.

    out = acc_out - sigmoid(blk_lse - acc_lse) * (acc_out - blk_out)
    lse = acc_lse - logsigmoid(acc_lse - blk_lse)
    (torch _SDPAMerger._merge_one, _context_parallel/_attention.py:182-183), in
    fp32.  ``out_dtype`` defaults to fp32 (the merger's convert_to_f32 mode);
    pass the activation dtype on the last step to fold results()'s cast.
    The returned lse has acc_lse's shape.
    """
    _check_merge_args(acc_out, acc_lse, blk_out, blk_lse)
    a, b = acc_out.contiguous(), blk_out.contiguous()
    la, lb = acc_lse.contiguous(), blk_lse.contiguous()
    out = torch.empty(a.shape, dtype=out_dtype or torch.float32, device=a.device)
    lse = torch.empty(la.shape, dtype=torch.float32, device=a.device)
    _merge_launch(a, la, b, lb, out, lse)
    return out, lse


@torch.library.register_fake("para_attn::merge_attention_lse")
def _(acc_out, acc_lse, blk_out, blk_lse, out_dtype=None):
    return (
        acc_out.new_empty(acc_out.shape, dtype=out_dtype or torch.float32),
        acc_lse.new_empty(acc_lse.shape, dtype=torch.float32),
    )


@torch.library.custom_op("para_attn::merge_attention_lse_", mutates_args=("acc_out", "acc_lse"), device_types=("cuda",))
def merge_attention_lse_(
    acc_out: torch.Tensor, acc_lse: torch.Tensor, blk_out: torch.Tensor, blk_lse: torch.Tensor
) -> None:
    """In-place merge step: folds (blk_out, blk_lse) into the contiguous accumulators."""
    _check_merge_args(acc_out, acc_lse, blk_out, blk_lse)
    if not acc_out.is_contiguous() or not acc_lse.is_contiguous():
        raise ValueError("in-place merge needs contiguous accumulators")
    _merge_launch(acc_out, acc_lse, blk_out.contiguous(), blk_lse.contiguous(), acc_out, acc_lse)


@torch.library.register_fake("para_attn::merge_attention_lse_")
def _(acc_out, acc_lse, blk_out, blk_lse):
    return None


@torch.library.custom_op(
    "para_attn::attention_forward_accumulate_", mutates_args=("acc_out", "acc_lse"), device_types=("cuda",)
)
def attention_forward_accumulate_(
    acc_out: torch.Tensor,
    acc_lse: torch.Tensor,
    query: torch.Tensor,
    key: torch.Tensor,
    value: torch.Tensor,
    first: bool = False,
    *,
    scale: Optional[float] = None,
) -> None:
    """Fused ring step: SDPA of ``query`` over one key/value block, merged into the fp32 running
    pair inside the attention kernel (what attention_forward_with_lse + _SDPAMerger.step do in
    two passes, src/para_attn/para_attn_interface.py:164-197).  ``first``: the pair is
    uninitialised.  head_dim 128 only (NotImplementedError otherwise)."""
    _check_sdpa_args(query, key, value, 0.0, False)
    _accumulate_forward(acc_out, acc_lse, query, key, value, scale, first, False)


@torch.library.register_fake("para_attn::attention_forward_accumulate_")
def _(acc_out, acc_lse, query, key, value, first=False, *, scale=None):
    return None


@torch.library.custom_op(
    "para_attn::attention_forward_accumulate_final", mutates_args=("acc_lse",), device_types=("cuda",)
)
def attention_forward_accumulate_final(
    acc_out: torch.Tensor,
    acc_lse: torch.Tensor,
    query: torch.Tensor,
    key: torch.Tensor,
    value: torch.Tensor,
    *,
    scale: Optional[float] = None,
) -> torch.Tensor:
    """Last fused ring step: returns the merged output in query's dtype (the cast of
    _SDPAMerger.results() folded in); ``acc_lse`` becomes the final LSE, ``acc_out`` is only read."""
    _check_sdpa_args(query, key, value, 0.0, False)
    return _accumulate_forward(acc_out, acc_lse, query, key, value, scale, False, True)


@torch.library.register_fake("para_attn::attention_forward_accumulate_final")
def _(acc_out, acc_lse, query, key, value, *, scale=None):
    return query.new_empty(query.shape)


@torch.library.custom_op("para_attn::attention_forward_sweep", mutates_args=(), device_types=("cuda",))
def attention_forward_sweep(
    query: torch.Tensor,
    key_blocks: List[torch.Tensor],
    value_blocks: List[torch.Tensor],
    *,
    scale: Optional[float] = None,
) -> Tuple[torch.Tensor, torch.Tensor]:
    """A whole same-GPU ring sweep in one launch: SDPA of ``query`` over the concatenation of the key/value
    blocks, which stay where they are (what the loop of src/para_attn/para_attn_interface.py:164-197 computes with
    one attention call and one merge per block).  Returns (out in query's dtype, fp32 LSE [B,H,Sq]).
    Blocks must share shape, dtype and strides; head_dim 128; at most 16 blocks (NotImplementedError otherwise)."""
    n = len(key_blocks)
    if n == 0 or len(value_blocks) != n:
        raise ValueError("key_blocks and value_blocks must be non-empty lists of equal length")
    _check_sdpa_args(query, key_blocks[0], value_blocks[0], 0.0, False)
    B, H, Sq, D = query.shape
    ks = [_kernel_ready(t) for t in key_blocks]
    vs = [_kernel_ready(t) for t in value_blocks]
    for t in ks + vs:
        if t.shape != ks[0].shape or t.dtype != query.dtype or t.device != query.device:
            raise ValueError("all key/value blocks must share the first key block's shape, and the query's dtype and device")
    if any(t.stride() != ks[0].stride() for t in ks) or any(t.stride() != vs[0].stride() for t in vs):
        ks = [t.contiguous() for t in ks]
        vs = [t.contiguous() for t in vs]
    blk = ks[0].shape[2]
    q = _kernel_ready(query)
    out = _out_like(query)
    lse = _lse_like(query)
    if scale is None:
        scale = 1.0 / math.sqrt(D)
    lib = _lib.load()
    with torch.cuda.device(q.device):
        kst, vst = _lib.strides3(ks[0]), _lib.strides3(vs[0])
        ws_bytes = lib.pa_attn_fwd_sweep_workspace_bytes(B, H, Sq, n, blk, D, kst, vst)
        ws = torch.empty(ws_bytes, dtype=torch.uint8, device=q.device) if ws_bytes else None
        rc = lib.pa_attn_fwd_sweep(
            _ptr(q), _ptr_array(ks), _ptr_array(vs), n, blk, _ptr(out), _ptr(lse), _DTYPE_CODE[q.dtype], B, H, Sq, D,
            _lib.strides3(q), kst, vst, _lib.strides3(out), float(scale), _ptr(ws), ws_bytes, _stream_ptr(q.device),
        )
    _lib.check(rc, "pa_attn_fwd_sweep")
    return out, lse


@torch.library.register_fake("para_attn::attention_forward_sweep")
def _(query, key_blocks, value_blocks, *, scale=None):
    return _out_like(query), _lse_like(query)


# ---------------------------------------------------------------------------------
# block-sparse attention
# ---------------------------------------------------------------------------------
def _sparse_geometry(query, key, block_mask_shape, q_lo, q_hi, kv_lo, kv_hi):
    """Checks the block-mask geometry against the tensors (src/para_attn/sparse_attn.py:112-131) and returns
    (Hm, nQ, nK, q_lo, q_hi, kv_lo, kv_hi, q_block, kv_block)."""
    B, H, Sq, D = query.shape
    Skv = key.shape[2]
    q_hi = Sq if q_hi < 0 else q_hi
    kv_hi = Skv if kv_hi < 0 else kv_hi
    if len(block_mask_shape) != 3 or block_mask_shape[0] not in (1, H):
        raise ValueError(f"block_mask must be [nQ,nK] or [H,nQ,nK], got {tuple(block_mask_shape)}")
    Hm, nQ, nK = block_mask_shape
    if not (0 <= q_lo <= q_hi <= Sq):
        raise ValueError(f"sparse query range must be in [0, {Sq}], got {(q_lo, q_hi)}")
    if not (0 <= kv_lo <= kv_hi <= Skv):
        raise ValueError(f"sparse key/value range must be in [0, {Skv}], got {(kv_lo, kv_hi)}")
    if nQ == 0 or nK == 0 or (q_hi - q_lo) % nQ or (kv_hi - kv_lo) % nK:
        raise ValueError("block_mask must divide the sparse query and key/value ranges")
    q_block = (q_hi - q_lo) // nQ
    kv_block = (kv_hi - kv_lo) // nK
    if q_block == 0 or kv_block == 0:
        raise ValueError("empty sparse range")
    return Hm, nQ, nK, q_lo, q_hi, kv_lo, kv_hi, q_block, kv_block


def _sparse_outputs(query):
    return _kernel_ready(query), _out_like(query), _lse_like(query)


@torch.library.custom_op("para_attn::attention_forward_block_sparse", mutates_args=(), device_types=("cuda",))
def attention_forward_block_sparse(
    query: torch.Tensor,
    key: torch.Tensor,
    value: torch.Tensor,
    block_mask: torch.Tensor,
    q_lo: int = 0,
    q_hi: int = -1,
    kv_lo: int = 0,
    kv_hi: int = -1,
    *,
    scale: Optional[float] = None,
) -> Tuple[torch.Tensor, torch.Tensor]:
    """Attention restricted to the kept tiles of ``block_mask``; returns (out, fp32 LSE).

    block_mask: bool [nQ,nK] (shared by batch and heads, the reference's form,
    src/para_attn/sparse_attn.py:107) or [H,nQ,nK].  Query rows [q_lo,q_hi) are
    cut into nQ equal blocks and keys [kv_lo,kv_hi) into nK equal blocks
    (sparse_range_query / sparse_range_key_value, sparse_attn.py:112-131);
    rows and keys outside those ranges are dense (:158-171, :178-189, :247-274).
    Identical to dense SDPA with -inf on the dropped tiles.
    """
    _check_sdpa_args(query, key, value, 0.0, False)
    B, H, Sq, D = query.shape
    Skv = key.shape[2]
    if block_mask.dtype != torch.bool:
        raise ValueError("block_mask must be boolean")
    _same_device(query, block_mask=block_mask)
    if block_mask.ndim == 2:
        block_mask = block_mask.unsqueeze(0)
    Hm, nQ, nK, q_lo, q_hi, kv_lo, kv_hi, q_block, kv_block = _sparse_geometry(query, key, block_mask.shape, q_lo, q_hi, kv_lo, kv_hi)
    k, v = _kernel_ready(key), _kernel_ready(value)
    q, out, lse = _sparse_outputs(query)
    mask_u8 = block_mask.contiguous().view(torch.uint8)
    lib = _lib.load()
    ws_bytes = lib.pa_blocksparse_workspace_bytes(Hm, nQ, nK)
    ws = torch.empty((ws_bytes + 3) // 4, dtype=torch.int32, device=q.device)
    if scale is None:
        scale = 1.0 / math.sqrt(D)
    with torch.cuda.device(q.device):
        rc = lib.pa_attn_fwd_blocksparse(
            _ptr(q), _ptr(k), _ptr(v), _ptr(out), _ptr(lse), _DTYPE_CODE[q.dtype], B, H, Sq, Skv, D,
            _lib.strides3(q), _lib.strides3(k), _lib.strides3(v), _lib.strides3(out), float(scale),
            _ptr(mask_u8), Hm, nQ, nK, q_lo, q_block, kv_lo, kv_block, _ptr(ws), ws_bytes,
            _stream_ptr(q.device),
        )
    _lib.check(rc, "pa_attn_fwd_blocksparse")
    return out, lse


@torch.library.register_fake("para_attn::attention_forward_block_sparse")
def _(query, key, value, block_mask, q_lo=0, q_hi=-1, kv_lo=0, kv_hi=-1, *, scale=None):
    return _out_like(query), _lse_like(query)


def _runs_words(Hm, nQ, nK):
    """Length in int32 words of the key-range buffer of a [Hm,nQ,nK] mask: the library's own figure (host
    arithmetic, no device call), so the op and its fake implementation cannot disagree."""
    return (_lib.load().pa_blocksparse_workspace_bytes(Hm, nQ, nK) + 3) // 4


@torch.library.custom_op("para_attn::block_sparse_key_runs", mutates_args=(), device_types=("cuda",))
def block_sparse_key_runs(block_mask: torch.Tensor, seq_kv: int, kv_lo: int = 0, kv_hi: int = -1) -> torch.Tensor:
    """The key ranges of a block mask, as the block-sparse kernel walks them: the mask's runs of kept blocks per
    (mask head, query block), merged with the dense key margins (the scan of src/para_attn/sparse_attn.py:215-234).
    Returns the int32 buffer ``attention_forward_block_sparse_runs`` takes; build it once for a mask that serves
    many calls.  ``block_sparse_runs`` gives a structured view of it."""
    if block_mask.dtype != torch.bool:
        raise ValueError("block_mask must be boolean")
    if block_mask.ndim == 2:
        block_mask = block_mask.unsqueeze(0)
    if block_mask.ndim != 3 or 0 in block_mask.shape:
        raise ValueError(f"block_mask must be [nQ,nK] or [H,nQ,nK], got {tuple(block_mask.shape)}")
    Hm, nQ, nK = block_mask.shape
    kv_hi = seq_kv if kv_hi < 0 else kv_hi
    if not (0 <= kv_lo <= kv_hi <= seq_kv) or (kv_hi - kv_lo) % nK or kv_hi == kv_lo:
        raise ValueError("block_mask must divide a non-empty sparse key/value range inside the keys")
    kv_block = (kv_hi - kv_lo) // nK
    lib = _lib.load()
    ws = torch.zeros(_runs_words(Hm, nQ, nK), dtype=torch.int32, device=block_mask.device)
    ws_bytes = ws.numel() * 4
    mask_u8 = block_mask.contiguous().view(torch.uint8)
    with torch.cuda.device(block_mask.device):
        rc = lib.pa_blocksparse_build_runs(
            _ptr(mask_u8), Hm, nQ, nK, seq_kv, kv_lo, kv_block, _ptr(ws), ws_bytes, _stream_ptr(block_mask.device)
        )
    _lib.check(rc, "pa_blocksparse_build_runs")
    return ws


@torch.library.register_fake("para_attn::block_sparse_key_runs")
def _(block_mask, seq_kv, kv_lo=0, kv_hi=-1):
    Hm, nQ, nK = block_mask.shape if block_mask.ndim == 3 else (1, *block_mask.shape)
    return block_mask.new_empty((_runs_words(Hm, nQ, nK),), dtype=torch.int32)


@torch.library.custom_op("para_attn::attention_forward_block_sparse_runs", mutates_args=(), device_types=("cuda",))
def attention_forward_block_sparse_runs(
    query: torch.Tensor,
    key: torch.Tensor,
    value: torch.Tensor,
    runs: torch.Tensor,
    mask_heads: int,
    n_q: int,
    n_k: int,
    q_lo: int = 0,
    q_hi: int = -1,
    *,
    scale: Optional[float] = None,
) -> Tuple[torch.Tensor, torch.Tensor]:
    """``attention_forward_block_sparse`` with the key ranges already extracted: ``runs`` is the result of
    ``block_sparse_key_runs`` for a [mask_heads, n_q, n_k] mask over keys of the same length (and the same
    sparse key range).  Saves the extraction on every call after the first."""
    _check_sdpa_args(query, key, value, 0.0, False)
    B, H, Sq, D = query.shape
    Skv = key.shape[2]
    if runs.dtype != torch.int32 or not runs.is_contiguous() or runs.device != query.device:
        raise ValueError("runs must be the contiguous int32 tensor block_sparse_key_runs returned, on the query's device")
    Hm, nQ, nK, q_lo, q_hi, _, _, q_block, _ = _sparse_geometry(query, key, (mask_heads, n_q, n_k), q_lo, q_hi, 0, n_k)
    lib = _lib.load()
    if runs.numel() * 4 < lib.pa_blocksparse_workspace_bytes(Hm, nQ, nK):
        raise ValueError(f"runs holds {runs.numel()} words, too few for a [{Hm},{nQ},{nK}] mask: not the result of block_sparse_key_runs for it")
    k, v = _kernel_ready(key), _kernel_ready(value)
    q, out, lse = _sparse_outputs(query)
    if scale is None:
        scale = 1.0 / math.sqrt(D)
    with torch.cuda.device(q.device):
        rc = lib.pa_attn_fwd_blocksparse_runs(
            _ptr(q), _ptr(k), _ptr(v), _ptr(out), _ptr(lse), _DTYPE_CODE[q.dtype], B, H, Sq, Skv, D,
            _lib.strides3(q), _lib.strides3(k), _lib.strides3(v), _lib.strides3(out), float(scale),
            Hm, nQ, nK, q_lo, q_block, _ptr(runs), runs.numel() * 4, _stream_ptr(q.device),
        )
    _lib.check(rc, "pa_attn_fwd_blocksparse_runs")
    return out, lse


@torch.library.register_fake("para_attn::attention_forward_block_sparse_runs")
def _(query, key, value, runs, mask_heads, n_q, n_k, q_lo=0, q_hi=-1, *, scale=None):
    return _out_like(query), _lse_like(query)


def block_sparse_runs(block_mask, Skv, kv_lo=0, kv_hi=-1):
    """Key ranges the block-sparse kernel walks, per (mask head, query segment), as the device built them.

    Returns (count [Hm, nQ+2] int32, ranges [Hm, nQ+2, cap, 2] int32) on the mask's device.
    """
    if block_mask.ndim == 2:
        block_mask = block_mask.unsqueeze(0)
    Hm, nQ, nK = block_mask.shape
    ws = block_sparse_key_runs(block_mask, Skv, kv_lo, kv_hi)
    nseg, cap = nQ + 2, nK // 2 + 3
    count = ws[: Hm * nseg].view(Hm, nseg)
    ranges = ws[Hm * nseg : Hm * nseg + Hm * nseg * cap * 2].view(Hm, nseg, cap, 2)
    return count, ranges


def block_sparse_launch_order(block_mask, Skv, kv_lo=0, kv_hi=-1):
    """[Hm, nQ] int32: the query blocks of each mask head in the order a launch starts them (the block that keeps most
    key blocks first, ties by block number), as the device built it; None beyond 2048 blocks per head, where the
    launch keeps the blocks' own order."""
    if block_mask.ndim == 2:
        block_mask = block_mask.unsqueeze(0)
    Hm, nQ, nK = block_mask.shape
    if nQ > 2048:
        return None
    ws = block_sparse_key_runs(block_mask, Skv, kv_lo, kv_hi)
    nseg, cap = nQ + 2, nK // 2 + 3
    first = Hm * nseg + Hm * nseg * cap * 2
    return ws[first : first + Hm * nQ].view(Hm, nQ)


# ---------------------------------------------------------------------------------
# First Block Cache reductions
# ---------------------------------------------------------------------------------
_fb_workspaces = {}


def _fb_workspace(device):
    """Zero-initialised ticket/partials buffer, one per (device, stream)."""
    key = (device.index, torch.cuda.current_stream(device).cuda_stream)
    ws = _fb_workspaces.get(key)
    if ws is None:
        nbytes = _lib.load().pa_fbcache_workspace_bytes()
        ws = torch.zeros((nbytes + 7) // 8, dtype=torch.int64, device=device)
        _fb_workspaces[key] = ws
    return ws


def _as_rows(t):
    """View a tensor as [rows, row_len] with (row_stride, col_stride) without copying, or None."""
    if t.ndim == 0:
        return 1, 1, 1, 1
    row_len = t.shape[-1]
    col_stride = t.stride(-1) if row_len > 1 else 1
    lead = t.shape[:-1]
    rows = 1
    for s in lead:
        rows *= s
    if rows <= 1:
        return max(rows, 0), row_len, row_len * col_stride, col_stride
    # leading dims must collapse to one stride
    expect = None
    for d in range(t.ndim - 2, -1, -1):
        if t.shape[d] == 1:
            continue
        if expect is None:
            row_stride = t.stride(d)
            expect = t.stride(d) * t.shape[d]
        else:
            if t.stride(d) != expect:
                return None
            expect = t.stride(d) * t.shape[d]
    return rows, row_len, row_stride, col_stride


@torch.library.custom_op("para_attn::fbcache_residual_diff", mutates_args=(), device_types=("cuda",))
def fbcache_residual_diff(prev: torch.Tensor, cur: torch.Tensor) -> torch.Tensor:
    """0-d tensor ``(prev - cur).abs().mean() / prev.abs().mean()`` in the activation dtype,
    with torch's rounding of every intermediate (src/para_attn/first_block_cache/utils.py:228-233).
    ``cur`` may be a strided view such as ``x[..., ::k]`` (utils.py:276-278)."""
    if prev.shape != cur.shape:
        raise ValueError(f"shape mismatch {tuple(prev.shape)} vs {tuple(cur.shape)}")
    if prev.dtype != cur.dtype or prev.dtype not in _DTYPE_CODE:
        raise NotImplementedError(f"dtypes {prev.dtype}/{cur.dtype} not supported")
    if prev.numel() == 0:
        raise ValueError("mean of an empty tensor")
    _same_device(prev, cur=cur)
    pr, cr = _as_rows(prev), _as_rows(cur)
    if pr is None:
        prev = prev.contiguous()
        pr = _as_rows(prev)
    if cr is None:
        cur = cur.contiguous()
        cr = _as_rows(cur)
    ratio = torch.empty((), dtype=prev.dtype, device=prev.device)
    ws = _fb_workspace(prev.device)
    lib = _lib.load()
    with torch.cuda.device(prev.device):
        rc = lib.pa_fbcache_absdiff_ratio(
            _ptr(prev), _ptr(cur), _DTYPE_CODE[prev.dtype], pr[0], pr[1], pr[2], pr[3], cr[2], cr[3],
            _ptr(ratio), None, _ptr(ws), ws.numel() * 8, _stream_ptr(prev.device),
        )
    _lib.check(rc, "pa_fbcache_absdiff_ratio")
    return ratio


@torch.library.register_fake("para_attn::fbcache_residual_diff")
def _(prev, cur):
    return prev.new_empty(())


@torch.library.custom_op("para_attn::fbcache_first_residual_diff", mutates_args=(), device_types=("cuda",))
def fbcache_first_residual_diff(
    hidden: torch.Tensor, hidden0: torch.Tensor, prev: Optional[torch.Tensor] = None
) -> Tuple[torch.Tensor, torch.Tensor]:
    """(residual, ratio): residual = hidden - hidden0 (src/para_attn/first_block_cache/utils.py:359)
    and, in the same pass, the reduction of ``fbcache_residual_diff(prev, residual)``.
    Without ``prev`` the ratio is +inf (never similar)."""
    if hidden.shape != hidden0.shape or hidden.dtype != hidden0.dtype or hidden.dtype not in _DTYPE_CODE:
        raise ValueError("hidden and hidden0 must share shape and a supported dtype")
    if prev is not None and (prev.shape != hidden.shape or prev.dtype != hidden.dtype):
        raise ValueError("prev must match hidden in shape and dtype")
    _same_device(hidden, hidden0=hidden0, prev=prev)
    h, h0 = hidden.contiguous(), hidden0.contiguous()
    pv = prev.contiguous() if prev is not None else None
    resid = torch.empty(h.shape, dtype=h.dtype, device=h.device)
    ratio = torch.full((), float("inf"), dtype=h.dtype, device=h.device)
    ws = _fb_workspace(h.device)
    lib = _lib.load()
    with torch.cuda.device(h.device):
        rc = lib.pa_fbcache_residual_ratio(
            _ptr(h), _ptr(h0), _ptr(pv), _ptr(resid), _DTYPE_CODE[h.dtype], h.numel(), _ptr(ratio), None,
            _ptr(ws), ws.numel() * 8, _stream_ptr(h.device),
        )
    _lib.check(rc, "pa_fbcache_residual_ratio")
    return resid, ratio


@torch.library.register_fake("para_attn::fbcache_first_residual_diff")
def _(hidden, hidden0, prev=None):
    return hidden.new_empty(hidden.shape), hidden.new_empty(())


@torch.library.custom_op("para_attn::fbcache_apply_residual", mutates_args=(), device_types=("cuda",))
def fbcache_apply_residual(residual: torch.Tensor, hidden: torch.Tensor) -> torch.Tensor:
    """``residual + hidden``, contiguous (src/para_attn/first_block_cache/utils.py:237-259)."""
    if residual.shape != hidden.shape or residual.dtype != hidden.dtype or hidden.dtype not in _DTYPE_CODE:
        raise ValueError("residual and hidden must share shape and a supported dtype")
    _same_device(hidden, residual=residual)
    r, h = residual.contiguous(), hidden.contiguous()
    out = torch.empty(h.shape, dtype=h.dtype, device=h.device)
    lib = _lib.load()
    with torch.cuda.device(h.device):
        rc = lib.pa_fbcache_apply_residual(_ptr(r), _ptr(h), _ptr(out), _DTYPE_CODE[h.dtype], h.numel(), _stream_ptr(h.device))
    _lib.check(rc, "pa_fbcache_apply_residual")
    return out


@torch.library.register_fake("para_attn::fbcache_apply_residual")
def _(residual, hidden):
    return hidden.new_empty(hidden.shape)


# ---------------------------------------------------------------------------------
# TaylorSeer
# ---------------------------------------------------------------------------------
def _flat_same(tensors, what):
    t0 = tensors[0]
    if t0.dtype not in _DTYPE_CODE:
        raise NotImplementedError(f"{what}: dtype {t0.dtype} not supported")
    out = []
    for t in tensors:
        if t.shape != t0.shape or t.dtype != t0.dtype or t.device != t0.device:
            raise ValueError(f"{what}: tensors must share shape, dtype and device")
        out.append(t if t.is_contiguous() and t.data_ptr() % 16 == 0 else t.contiguous().clone())
    return out


@torch.library.custom_op("para_attn::taylorseer_derivatives", mutates_args=(), device_types=("cuda",))
def taylorseer_derivatives(y: torch.Tensor, prev: List[torch.Tensor], window: float) -> List[torch.Tensor]:
    """The finite differences of TaylorSeer.approximate_derivative
    (src/para_attn/first_block_cache/taylorseer.py:29-38) in one pass: with x0 = y,
    returns [x1, ..., xn] where x_{i+1} = (x_i - prev[i]) / window, rounded as torch's
    eager ops round (difference, then quotient)."""
    n = len(prev)
    if n == 0:
        return []
    ts = _flat_same([y] + list(prev), "taylorseer_derivatives")
    cur = [torch.empty(y.shape, dtype=y.dtype, device=y.device) for _ in range(n)]
    lib = _lib.load()
    with torch.cuda.device(y.device):
        rc = lib.pa_taylorseer_update(
            _ptr(ts[0]), _ptr_array(ts[1:]), _ptr_array(cur), n, _DTYPE_CODE[y.dtype], y.numel(), float(window),
            _stream_ptr(y.device),
        )
    _lib.check(rc, "pa_taylorseer_update")
    return cur


@torch.library.register_fake("para_attn::taylorseer_derivatives")
def _(y, prev, window):
    return [y.new_empty(y.shape) for _ in prev]


@torch.library.custom_op("para_attn::taylorseer_value", mutates_args=(), device_types=("cuda",))
def taylorseer_value(derivs: List[torch.Tensor], elapsed: int, hidden: Optional[torch.Tensor] = None) -> torch.Tensor:
    """TaylorSeer.approximate_value (taylorseer.py:40-48): sum over the stored orders of
    (1 / i!) * derivs[i] * elapsed**i, each product and partial sum rounded as torch's eager
    ops round; with ``hidden``, the cache-hit add ``value + hidden`` of
    src/para_attn/first_block_cache/utils.py:239-243 in the same pass."""
    m = len(derivs)
    if m == 0:
        raise ValueError("taylorseer_value: no stored derivative")
    ts = _flat_same(list(derivs) + ([hidden] if hidden is not None else []), "taylorseer_value")
    d0 = ts[0]
    out = torch.empty(d0.shape, dtype=d0.dtype, device=d0.device)
    coef = (ctypes.c_float * m)(*[1 / math.factorial(i) for i in range(m)])
    pw = (ctypes.c_float * m)(*[float(elapsed**i) for i in range(m)])
    lib = _lib.load()
    with torch.cuda.device(d0.device):
        rc = lib.pa_taylorseer_value(
            _ptr_array(ts[:m]), m, coef, pw, _ptr(ts[m]) if hidden is not None else None, _ptr(out),
            _DTYPE_CODE[d0.dtype], d0.numel(), _stream_ptr(d0.device),
        )
    _lib.check(rc, "pa_taylorseer_value")
    return out


@torch.library.register_fake("para_attn::taylorseer_value")
def _(derivs, elapsed, hidden=None):
    return derivs[0].new_empty(derivs[0].shape)
