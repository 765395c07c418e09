"""The reference's interception mode for plain attention calls, for one GPU
(src/para_attn/para_attn_interface.py:395-479).

``with UnifiedAttnMode(): F.scaled_dot_product_attention(q, k, v)`` walks the reference's three
stages (ulysses, ring, none).  On one GPU the first two pass through
(para_attn_interface.py:62-63, 217-226), and the last one ends in ``attn_func`` if given, in
``para_attn::attention_forward`` when ``config.attention.force_dispatch_to_custom_ops`` is set
(:468-470) or -- where the reference would call aten's SDPA, which has no kernel of its own on
this GPU -- when the call is one the HIP kernel takes; any other call goes to
``F.scaled_dot_product_attention`` untouched.  A mesh of more than one rank is refused.
"""
import contextlib

import torch
import torch.nn.functional as F
from torch.overrides import TorchFunctionMode

from . import config, ops

_SDPA_ARGS = ("query", "key", "value", "attn_mask", "dropout_p", "is_causal", "scale", "enable_gqa")


def _bind(args, kwargs):
    bound = dict(zip(_SDPA_ARGS, args))
    bound.update(kwargs)
    return bound


def kernel_takes(query, key, value, attn_mask=None, dropout_p=0.0, is_causal=False, scale=None, enable_gqa=False):
    """Whether ``para_attn::attention_forward`` computes this SDPA call on the GPU."""
    if not (isinstance(query, torch.Tensor) and query.is_cuda and query.ndim == 4 and key.ndim == 4 and value.ndim == 4):
        return False
    if query.dtype not in (torch.bfloat16, torch.float16) or key.dtype != query.dtype or value.dtype != query.dtype:
        return False
    if dropout_p != 0.0 or enable_gqa or query.shape[1] != key.shape[1]:
        return False
    if is_causal and attn_mask is not None:
        return False
    if not (1 <= query.shape[-1] <= 128 and 1 <= value.shape[-1] <= 128) or key.shape[-1] != query.shape[-1]:
        return False  # 64 and 128 natively, other head_dims up to 128 zero-padded (ops._pad_head_dims)
    if query.requires_grad or key.requires_grad or value.requires_grad:
        return False  # forward only, like the reference's ops (src/para_attn/ops/__init__.py:203-211)
    if attn_mask is not None:
        # boolean or additive, broadcastable to the scores as torch's SDPA reads it (trailing dimensions aligned)
        if not isinstance(attn_mask, torch.Tensor) or attn_mask.ndim > 4 or attn_mask.device != query.device:
            return False
        if attn_mask.dtype != torch.bool and not attn_mask.is_floating_point():
            return False
        full = (query.shape[0], query.shape[1], query.shape[2], key.shape[2])
        shape = (1,) * (4 - attn_mask.ndim) + tuple(attn_mask.shape)
        if any(s not in (1, f) for s, f in zip(shape, full)):
            return False
    return True


def _world_size(mesh):
    if mesh is None:
        return 1
    if hasattr(mesh, "size"):
        return mesh.size() if callable(mesh.size) else mesh.size
    raise TypeError("mesh must be a ProcessGroup or DeviceMesh")


def _sdpa(*args, **kwargs):
    """The last stage on this GPU: the HIP kernel for the calls it takes, aten's SDPA for the rest."""
    b = _bind(args, kwargs)
    if kernel_takes(**b):
        b.pop("enable_gqa", None)
        return ops.attention_forward(**b)
    return F.scaled_dot_product_attention(*args, **kwargs)


def _one_rank(mesh, what):
    if _world_size(mesh) > 1:
        raise NotImplementedError(f"this build runs on one GPU: {what} over a mesh of more than one rank is not provided")


def ulysses_attn_func(query, key, value, attn_mask=None, dropout_p=0.0, is_causal=False, *, scale=None, mesh=None,
                      attn_func=None):
    """para_attn_interface.py:88-117 on one rank: the all-to-alls are identities, the attention remains."""
    assert query.ndim == 4, "query must have 4 dimensions, got {}".format(query.ndim)
    assert key.ndim == 4, "key must have 4 dimensions, got {}".format(key.ndim)
    assert value.ndim == 4, "value must have 4 dimensions, got {}".format(value.ndim)
    _one_rank(mesh, "ulysses attention")
    fn = attn_func if attn_func is not None else _sdpa
    return fn(query, key, value, attn_mask=attn_mask, dropout_p=dropout_p, is_causal=is_causal, scale=scale)


def ring_attn_func(query, key, value, attn_mask=None, dropout_p=0.0, is_causal=False, *, scale=None, mesh=None):
    """para_attn_interface.py:200-239 on one rank (world size <= 1 is plain attention there too, :213-222)."""
    _one_rank(mesh, "ring attention")
    return _sdpa(query, key, value, attn_mask=attn_mask, dropout_p=dropout_p, is_causal=is_causal, scale=scale)


def in_batch_attn_func(query, key, value, attn_mask=None, dropout_p=0.0, is_causal=False, *, scale=None):
    """para_attn_interface.py:242-276: the batch is folded into the sequence, so every image of the batch
    attends the keys of all of them.  With [B,S,H,D] memory behind the [B,H,S,D] view (what diffusers hands
    over) the fold is a view and the kernel reads it through its strides; otherwise torch copies once."""
    assert query.ndim == 4, "query must have 4 dimensions, got {}".format(query.ndim)
    assert key.ndim == 4, "key must have 4 dimensions, got {}".format(key.ndim)
    assert value.ndim == 4, "value must have 4 dimensions, got {}".format(value.ndim)
    assert attn_mask is None, "attn_mask is not supported in in_batch_attn_func"
    assert not is_causal, "is_causal is not supported in in_batch_attn_func"
    b, h, s_q, _ = query.shape
    s_kv = value.shape[2]
    query = query.permute(1, 0, 2, 3).reshape(1, h, b * s_q, -1)
    key = key.permute(1, 0, 2, 3).reshape(1, h, b * s_kv, -1)
    value = value.permute(1, 0, 2, 3).reshape(1, h, b * s_kv, -1)
    out = _sdpa(query, key, value, attn_mask=None, dropout_p=dropout_p, is_causal=False, scale=scale)
    return out.reshape(h, b, s_q, -1).permute(1, 0, 2, 3)


class _SdpaMode(TorchFunctionMode):
    """What the reference's modes share (src/para_attn/utils.py:19-32 and the class bodies): interception of
    F.scaled_dot_product_attention, a class-wide ``disabled`` switch with ``disable()``."""

    disabled = False

    @torch.compiler.disable
    def __init__(self, *, skip_small_kv=False):
        super().__init__()
        self._skip_small_kv = skip_small_kv

    def _call(self, *args, **kwargs):
        raise NotImplementedError

    def __torch_function__(self, func, types, args=(), kwargs=None):
        kwargs = {} if kwargs is None else kwargs
        if type(self).disabled or func is not F.scaled_dot_product_attention:
            return func(*args, **kwargs)
        if self._skip_small_kv:
            b = _bind(args, kwargs)
            if b["query"].shape[-2] > b["key"].shape[-2]:  # more queries than keys: a cross-attention, left alone
                return func(*args, **kwargs)
        return self._call(*args, **kwargs)

    @classmethod
    @contextlib.contextmanager
    def disable(cls):
        old = cls._set_disabled(True)
        try:
            yield
        finally:
            cls._set_disabled(old)

    @classmethod
    @torch.compiler.disable
    def _set_disabled(cls, value):
        old = cls.disabled
        cls.disabled = value
        return old


class UnifiedAttnMode(_SdpaMode):
    disabled = False

    @torch.compiler.disable
    def __init__(self, mesh=None, *, skip_small_kv=False, attn_func=None):
        super().__init__(skip_small_kv=skip_small_kv)
        _one_rank(mesh, "ulysses / ring attention")
        self._parallel_method = "ulysses"
        self._attn_func = attn_func

    def _call(self, *args, **kwargs):
        func = F.scaled_dot_product_attention
        method = self._parallel_method
        if method in ("ulysses", "ring"):  # world size 1: both stages pass the call on
            self._parallel_method = "ring" if method == "ulysses" else "none"
            try:
                with self:
                    return func(*args, **kwargs)
            finally:
                self._parallel_method = method
        if method != "none":
            raise ValueError(f"Unknown parallel method: {method}")
        if config.attention.force_dispatch_to_custom_ops:
            return ops.attention_forward(*args, **kwargs)
        if self._attn_func is not None:
            return self._attn_func(*args, **kwargs)
        return _sdpa(*args, **kwargs)


class RingAttnMode(_SdpaMode):
    """para_attn_interface.py:303-350."""

    disabled = False

    @torch.compiler.disable
    def __init__(self, mesh=None, *, skip_small_kv=False):
        super().__init__(skip_small_kv=skip_small_kv)
        _one_rank(mesh, "ring attention")

    def _call(self, *args, **kwargs):
        return ring_attn_func(*args, **kwargs)


class UlyssesAttnMode(_SdpaMode):
    """para_attn_interface.py:353-392."""

    disabled = False

    @torch.compiler.disable
    def __init__(self, mesh=None, *, skip_small_kv=False):
        super().__init__(skip_small_kv=skip_small_kv)
        _one_rank(mesh, "ulysses attention")

    def _call(self, *args, **kwargs):
        return ulysses_attn_func(*args, **kwargs)


class InBatchAttnMode(_SdpaMode):
    """para_attn_interface.py:498-530."""

    disabled = False

    @torch.compiler.disable
    def __init__(self):
        super().__init__()

    def _call(self, *args, **kwargs):
        return in_batch_attn_func(*args, **kwargs)


def sparse_kv_attn_func(query, key, value, attn_mask=None, dropout_p=0.0, is_causal=False, *, scale=None,
                        dispatch_to_custom_ops=True):
    """src/para_attn/sparse_attn.py:49-69: SDPA that drops the keys a boolean mask switches off.
    Both settings of ``dispatch_to_custom_ops`` end in the same kernel here."""
    return ops.attention_forward_sparse_kv(query, key, value, attn_mask=attn_mask, dropout_p=dropout_p,
                                           is_causal=is_causal, scale=scale)


class SparseKVAttnMode(_SdpaMode):
    """src/para_attn/sparse_attn.py:607-640."""

    disabled = False

    @torch.compiler.disable
    def __init__(self, *, dispatch_to_custom_ops=True):
        super().__init__()
        self._dispatch_to_custom_ops = dispatch_to_custom_ops

    def _call(self, *args, **kwargs):
        return sparse_kv_attn_func(*args, **kwargs, dispatch_to_custom_ops=self._dispatch_to_custom_ops)
