"""First Block Cache decision path with the reference's function names
(src/para_attn/first_block_cache/utils.py:12-120, 193-295): the cache context,
the gates of ``get_can_use_cache`` and ``are_two_tensors_similar``, whose
seven-launch reduction is one kernel here, and the TaylorSeer variant of the
cached residual (utils.py:297-312), and ``CachedTransformerBlocks``, the module the
reference's adapters swap in for a model's block list (utils.py:333-451).  The
diffusers adapters themselves are not part of this package.
"""
import contextlib
import dataclasses
from collections import defaultdict
from typing import Any, DefaultDict, Dict, List, Optional, Union

import torch

from . import ops
from .taylorseer import TaylorSeer


@dataclasses.dataclass
class CacheContext:
    """State of one pipeline call (reference fields of the same names, utils.py:12-37)."""

    residual_diff_threshold: Union[torch.Tensor, float] = 0.0
    alter_residual_diff_threshold: Optional[Union[torch.Tensor, float]] = None
    downsample_factor: int = 1
    enable_alter_cache: bool = False
    num_inference_steps: int = -1
    warmup_steps: int = 0
    enable_taylorseer: bool = False
    taylorseer_kwargs: Dict[str, Any] = dataclasses.field(default_factory=dict)
    slg_layers: Optional[List[int]] = None
    slg_start: float = 0.0
    slg_end: float = 0.1
    taylorseer: Optional[TaylorSeer] = None
    alter_taylorseer: Optional[TaylorSeer] = None
    buffers: Dict[str, Any] = dataclasses.field(default_factory=dict)
    incremental_name_counters: DefaultDict[str, int] = dataclasses.field(default_factory=lambda: defaultdict(int))
    executed_steps: int = 0
    is_alter_cache: bool = True

    def __post_init__(self):
        if self.enable_taylorseer:
            self.taylorseer = TaylorSeer(**self.taylorseer_kwargs)
            if self.enable_alter_cache:
                self.alter_taylorseer = TaylorSeer(**self.taylorseer_kwargs)

    def get_incremental_name(self, name=None):
        """utils.py:45-50: "<name>_<count>", counting per name from 0."""
        name = "default" if name is None else name
        idx = self.incremental_name_counters[name]
        self.incremental_name_counters[name] += 1
        return f"{name}_{idx}"

    def reset_incremental_names(self):
        self.incremental_name_counters.clear()

    def get_taylorseer(self):
        if self.enable_alter_cache and self.is_alter_cache:
            return self.alter_taylorseer
        return self.taylorseer

    def get_residual_diff_threshold(self):
        if self.enable_alter_cache and self.is_alter_cache and self.alter_residual_diff_threshold is not None:
            thr = self.alter_residual_diff_threshold
        else:
            thr = self.residual_diff_threshold
        if isinstance(thr, torch.Tensor):
            thr = thr.item()
        return thr

    def _name(self, name):
        return f"{name}_alter" if self.enable_alter_cache and self.is_alter_cache else name

    def get_buffer(self, name):
        return self.buffers.get(self._name(name))

    def set_buffer(self, name, buffer):
        self.buffers[self._name(name)] = buffer

    def remove_buffer(self, name):
        self.buffers.pop(self._name(name), None)

    def clear_buffers(self):
        self.buffers.clear()

    def mark_step_begin(self):
        if not self.enable_alter_cache:
            self.executed_steps += 1
        else:
            self.is_alter_cache = not self.is_alter_cache
            if not self.is_alter_cache:
                self.executed_steps += 1
        if self.enable_taylorseer:
            self.get_taylorseer().mark_step_begin()

    def is_slg_enabled(self):
        return self.slg_layers is not None

    def slg_should_skip_block(self, block_idx):
        """utils.py:102-114: skip-layer guidance drops the listed blocks on the alternating pass, inside
        the step window [slg_start, slg_end) of the schedule."""
        if not self.enable_alter_cache or not self.is_alter_cache:
            return False
        if self.slg_layers is None:
            return False
        if self.slg_start <= 0.0 and self.slg_end >= 1.0:
            return False
        assert self.num_inference_steps >= 0, "num_inference_steps must be non-negative"
        n = self.num_inference_steps
        return block_idx in self.slg_layers and n * self.slg_start <= self.get_current_step() < n * self.slg_end

    def get_current_step(self):
        return self.executed_steps - 1

    def is_in_warmup(self):
        return self.get_current_step() < self.warmup_steps


_current_cache_context = None


def create_cache_context(*args, **kwargs):
    return CacheContext(*args, **kwargs)


def get_current_cache_context():
    return _current_cache_context


def set_current_cache_context(cache_context=None):
    global _current_cache_context
    _current_cache_context = cache_context


@contextlib.contextmanager
def cache_context(cache_context):
    global _current_cache_context
    old = _current_cache_context
    _current_cache_context = cache_context
    try:
        yield
    finally:
        _current_cache_context = old


def _ctx():
    ctx = get_current_cache_context()
    assert ctx is not None, "cache_context must be set before"
    return ctx


def get_residual_diff_threshold():
    return _ctx().get_residual_diff_threshold()


def get_buffer(name):
    return _ctx().get_buffer(name)


def set_buffer(name, buffer):
    _ctx().set_buffer(name, buffer)


def remove_buffer(name):
    _ctx().remove_buffer(name)


def is_in_warmup():
    return _ctx().is_in_warmup()


def get_downsample_factor():
    return _ctx().downsample_factor


def residual_diff(t1, t2):
    """The 0-d ratio tensor ``mean|t1 - t2| / mean|t1|`` of utils.py:228-233, one kernel."""
    return ops.fbcache_residual_diff(t1, t2)


@torch.compiler.disable
def are_two_tensors_similar(t1, t2, *, threshold, parallelized=False):
    """utils.py:220-234.  ``parallelized`` would average the two means over ranks;
    this build runs on one GPU and refuses it."""
    if threshold <= 0.0:
        return False
    if t1.shape != t2.shape:
        return False
    if parallelized:
        raise NotImplementedError("cross-rank averaging of the means needs more than one GPU")
    diff = residual_diff(t1, t2)
    return diff.item() < threshold


@torch.compiler.disable
def get_first_hidden_states_residual():
    return _ctx().get_buffer("first_hidden_states_residual")


@torch.compiler.disable
def set_first_hidden_states_residual(first_hidden_states_residual):
    """utils.py:289-295: the stored copy is the down-sampled, contiguous one."""
    k = _ctx().downsample_factor
    if k > 1:
        first_hidden_states_residual = first_hidden_states_residual[..., ::k].contiguous()
    _ctx().set_buffer("first_hidden_states_residual", first_hidden_states_residual)


@torch.compiler.disable
def get_can_use_cache(first_hidden_states_residual, parallelized=False):
    """utils.py:269-286: warm-up gate, threshold gate, down-sampling, missing-previous gate, then the reduction."""
    ctx = _ctx()
    if ctx.is_in_warmup():
        return False
    threshold = ctx.get_residual_diff_threshold()
    if threshold <= 0.0:
        return False
    k = ctx.downsample_factor
    if k > 1:
        first_hidden_states_residual = first_hidden_states_residual[..., ::k]
    prev = get_first_hidden_states_residual()
    return prev is not None and are_two_tensors_similar(
        prev, first_hidden_states_residual, threshold=threshold, parallelized=parallelized
    )


@torch.compiler.disable
def first_block_step(hidden_states, original_hidden_states, parallelized=False):
    """Residual of the first block plus the cache decision in one pass over memory
    (utils.py:359-366: ``hidden - original``, ``mark_step_begin``, ``get_can_use_cache``).

    Returns (first_hidden_states_residual, can_use_cache).  Falls back to the
    two-step form when down-sampling is on, since the stored residual then has
    another shape than the fresh one.
    """
    ctx = _ctx()
    ctx.mark_step_begin()
    threshold = ctx.get_residual_diff_threshold()
    gated = ctx.is_in_warmup() or threshold <= 0.0
    prev = None if gated else get_first_hidden_states_residual()
    if ctx.downsample_factor > 1 or (prev is not None and prev.shape != hidden_states.shape):
        resid, _ = ops.fbcache_first_residual_diff(hidden_states, original_hidden_states, None)
        return resid, (not gated) and get_can_use_cache(resid, parallelized=parallelized)
    if parallelized and prev is not None:
        raise NotImplementedError("cross-rank averaging of the means needs more than one GPU")
    resid, ratio = ops.fbcache_first_residual_diff(hidden_states, original_hidden_states, prev)
    can_use = prev is not None and ratio.item() < threshold
    return resid, can_use


@torch.compiler.disable
def apply_prev_hidden_states_residual(hidden_states, encoder_hidden_states=None):
    """Cache hit (utils.py:237-259): add the stored residuals back."""
    ctx = _ctx()
    if ctx.enable_taylorseer:
        # utils.py:239-243: the extrapolated residual plus the hidden states, one pass; the
        # encoder residual is not kept in this mode (utils.py:314-317) and stays untouched
        return ctx.get_taylorseer().approximate_value_plus(hidden_states), encoder_hidden_states
    res = ctx.get_buffer("hidden_states_residual")
    assert res is not None, "hidden_states_residual must be set before"
    hidden_states = ops.fbcache_apply_residual(res, hidden_states)
    if encoder_hidden_states is not None:
        eres = ctx.get_buffer("encoder_hidden_states_residual")
        assert eres is not None, "encoder_hidden_states_residual must be set before"
        encoder_hidden_states = ops.fbcache_apply_residual(eres, encoder_hidden_states)
    return hidden_states, encoder_hidden_states


@torch.compiler.disable
def is_taylorseer_enabled():
    return _ctx().enable_taylorseer


@torch.compiler.disable
def get_taylorseer():
    return _ctx().get_taylorseer()


@torch.compiler.disable
def set_hidden_states_residual(hidden_states_residual):
    """utils.py:297-303."""
    ctx = _ctx()
    if ctx.enable_taylorseer:
        ctx.get_taylorseer().update(hidden_states_residual)
    else:
        ctx.set_buffer("hidden_states_residual", hidden_states_residual)


@torch.compiler.disable
def get_hidden_states_residual():
    """utils.py:306-312."""
    ctx = _ctx()
    if ctx.enable_taylorseer:
        return ctx.get_taylorseer().approximate_value()
    return ctx.get_buffer("hidden_states_residual")


@torch.compiler.disable
def set_encoder_hidden_states_residual(encoder_hidden_states_residual):
    """utils.py:314-318."""
    ctx = _ctx()
    if ctx.enable_taylorseer:
        return
    ctx.set_buffer("encoder_hidden_states_residual", encoder_hidden_states_residual)


@torch.compiler.disable
def get_encoder_hidden_states_residual():
    return _ctx().get_buffer("encoder_hidden_states_residual")


@torch.compiler.disable
def mark_step_begin():
    _ctx().mark_step_begin()


@torch.compiler.disable
def is_slg_enabled():
    return _ctx().is_slg_enabled()


@torch.compiler.disable
def slg_should_skip_block(block_idx):
    return _ctx().slg_should_skip_block(block_idx)


def _residual(after, before):
    """``after - before`` as one kernel, contiguous (utils.py:443-449)."""
    return ops.fbcache_first_residual_diff(after, before, None)[0]


class CachedTransformerBlocks(torch.nn.Module):
    """The caller of the First Block Cache path (src/para_attn/first_block_cache/utils.py:333-451): run the
    first block, decide from its residual whether the rest may be skipped, then either add the cached
    residuals back or run the remaining blocks and cache theirs.  Constructor and return conventions are
    the reference's; the residual, the reduction and the decision are one kernel (``first_block_step``),
    the cache hit another, the residuals of the remaining blocks one each."""

    def __init__(self, transformer_blocks, single_transformer_blocks=None, *, transformer=None,
                 return_hidden_states_first=True, return_hidden_states_only=False):
        super().__init__()
        self.transformer = transformer
        self.transformer_blocks = transformer_blocks
        self.single_transformer_blocks = single_transformer_blocks
        self.return_hidden_states_first = return_hidden_states_first
        self.return_hidden_states_only = return_hidden_states_only

    def _dual(self, block, hidden_states, encoder_hidden_states, *args, **kwargs):
        """A block returns the hidden states alone, or both streams in the order the model uses."""
        out = block(hidden_states, encoder_hidden_states, *args, **kwargs)
        if isinstance(out, torch.Tensor):
            return out, encoder_hidden_states
        first, second = out
        return (first, second) if self.return_hidden_states_first else (second, first)

    def forward(self, hidden_states, encoder_hidden_states, *args, **kwargs):
        original_hidden_states = hidden_states
        hidden_states, encoder_hidden_states = self._dual(
            self.transformer_blocks[0], hidden_states, encoder_hidden_states, *args, **kwargs)
        parallelized = self.transformer is not None and getattr(self.transformer, "_is_parallelized", False)
        first_residual, can_use_cache = first_block_step(hidden_states, original_hidden_states, parallelized)
        del original_hidden_states

        torch._dynamo.graph_break()
        if can_use_cache:
            del first_residual
            hidden_states, encoder_hidden_states = apply_prev_hidden_states_residual(hidden_states, encoder_hidden_states)
        else:
            set_first_hidden_states_residual(first_residual)
            del first_residual
            hidden_states, encoder_hidden_states, res, enc_res = self.call_remaining_transformer_blocks(
                hidden_states, encoder_hidden_states, *args, **kwargs)
            set_hidden_states_residual(res)
            set_encoder_hidden_states_residual(enc_res)
        torch._dynamo.graph_break()

        if self.return_hidden_states_only:
            return hidden_states
        if self.return_hidden_states_first:
            return hidden_states, encoder_hidden_states
        return encoder_hidden_states, hidden_states

    def call_remaining_transformer_blocks(self, hidden_states, encoder_hidden_states, *args, **kwargs):
        """utils.py:396-451: blocks 1.. of the dual-stream stack, then the single-stream stack on the
        concatenated sequence; blocks named by skip-layer guidance are left out."""
        original_hidden_states = hidden_states
        original_encoder_hidden_states = encoder_hidden_states
        slg = is_slg_enabled()
        for i, block in enumerate(self.transformer_blocks[1:]):
            if slg and slg_should_skip_block(i + 1):
                continue
            hidden_states, encoder_hidden_states = self._dual(block, hidden_states, encoder_hidden_states, *args, **kwargs)
        if self.single_transformer_blocks is not None:
            n_enc = encoder_hidden_states.shape[1]
            hidden_states = torch.cat([encoder_hidden_states, hidden_states], dim=1)
            for i, block in enumerate(self.single_transformer_blocks):
                if slg and slg_should_skip_block(len(self.transformer_blocks) + i):
                    continue
                hidden_states = block(hidden_states, *args, **kwargs)
            encoder_hidden_states, hidden_states = hidden_states.split([n_enc, hidden_states.shape[1] - n_enc], dim=1)

        hidden_states = hidden_states.contiguous().reshape(original_hidden_states.shape)
        res = _residual(hidden_states, original_hidden_states)
        enc_res = None
        if encoder_hidden_states is not None:
            encoder_hidden_states = encoder_hidden_states.contiguous().reshape(original_encoder_hidden_states.shape)
            enc_res = _residual(encoder_hidden_states, original_encoder_hidden_states)
        return hidden_states, encoder_hidden_states, res, enc_res
