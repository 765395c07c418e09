"""First Block Cache decision path with the reference's function names
(src/para_attn/first_block_cache/utils.py:12-120, 193-295): the cache context,
the gates of ``get_can_use_cache`` and ``are_two_tensors_similar``, whose
seven-launch reduction is one kernel here, and the TaylorSeer variant of the
cached residual (utils.py:297-312), and ``CachedTransformerBlocks``, the module the
reference's adapters swap in for a model's block list (utils.py:333-451).  The
diffusers adapters themselves are not part of this package.
"""
import contextlib
import itertools

import torch

from . import ops
from .taylorseer import TaylorSeer


class _Lane:
    """What one of the two passes of a step owns: its buffers, its TaylorSeer, its threshold.  A
    pipeline without an alternating pass (classifier-free guidance run as a second forward) only
    ever uses the main lane."""

    __slots__ = ("suffix", "threshold", "store", "seer")

    def __init__(self, suffix, threshold, seer):
        self.suffix = suffix
        self.threshold = threshold
        self.store = {}
        self.seer = seer


def _as_float(x):
    return x.item() if isinstance(x, torch.Tensor) else x


class CacheContext:
    """State of one pipeline call.  Constructor arguments are the reference's fields of the same
    names and order (src/para_attn/first_block_cache/utils.py:12-28); the bookkeeping is kept as one
    count of ``mark_step_begin`` calls, from which the running step and the pass (main or
    alternating) follow, and one lane of buffers per pass.

    With ``enable_alter_cache`` the calls alternate main, alter, main, ... and a step is one such
    pair; before the first call the context stands on the alternating pass (utils.py:37, 80-88).
    Without it every call is a step of the main pass.
    """

    def __init__(self, residual_diff_threshold=0.0, alter_residual_diff_threshold=None, downsample_factor=1,
                 enable_alter_cache=False, num_inference_steps=-1, warmup_steps=0, enable_taylorseer=False,
                 taylorseer_kwargs=None, slg_layers=None, slg_start=0.0, slg_end=0.1):
        self.downsample_factor = downsample_factor
        self.enable_alter_cache = enable_alter_cache
        self.num_inference_steps = num_inference_steps
        self.warmup_steps = warmup_steps
        self.enable_taylorseer = enable_taylorseer
        self.taylorseer_kwargs = dict(taylorseer_kwargs or {})
        self.slg_layers = slg_layers
        self.slg_start = slg_start
        self.slg_end = slg_end
        seer = lambda wanted: TaylorSeer(**self.taylorseer_kwargs) if wanted else None  # noqa: E731
        self._main = _Lane("", residual_diff_threshold, seer(enable_taylorseer))
        self._alter = _Lane("_alter", alter_residual_diff_threshold, seer(enable_taylorseer and enable_alter_cache))
        self._marks = 0        # mark_step_begin calls so far
        self._serials = {}     # name -> iterator of its serial numbers

    # -- where the context stands --------------------------------------------------------------------
    @property
    def is_alter_cache(self):
        """True on the alternating pass; stays True when there is none (the reference's flag, utils.py:37)."""
        return not self.enable_alter_cache or self._marks % 2 == 0

    @property
    def executed_steps(self):
        return (self._marks + 1) // 2 if self.enable_alter_cache else self._marks

    def get_current_step(self):
        return self.executed_steps - 1

    def is_in_warmup(self):
        return self.get_current_step() < self.warmup_steps

    def _lane(self):
        return self._alter if self.enable_alter_cache and self._marks % 2 == 0 else self._main

    def mark_step_begin(self):
        """One forward pass of the model begins (utils.py:80-90)."""
        self._marks += 1
        seer = self._lane().seer
        if seer is not None:
            seer.mark_step_begin()

    # -- per-pass settings -----------------------------------------------------------------------------
    @property
    def residual_diff_threshold(self):
        return self._main.threshold

    @property
    def alter_residual_diff_threshold(self):
        return self._alter.threshold

    def get_residual_diff_threshold(self):
        """Python number; the alternating pass has its own if one was given (utils.py:55-62)."""
        own = self._lane().threshold
        return _as_float(self._main.threshold if own is None else own)

    @property
    def taylorseer(self):
        return self._main.seer

    @property
    def alter_taylorseer(self):
        return self._alter.seer

    def get_taylorseer(self):
        return self._lane().seer

    # -- buffers ----------------------------------------------------------------------------------------
    def get_buffer(self, name):
        return self._lane().store.get(name)

    def set_buffer(self, name, buffer):
        self._lane().store[name] = buffer

    def remove_buffer(self, name):
        self._lane().store.pop(name, None)

    def clear_buffers(self):
        self._main.store.clear()
        self._alter.store.clear()

    @property
    def buffers(self):
        """All buffers under the reference's names: those of the alternating pass carry "_alter" (utils.py:64-72)."""
        return {name + lane.suffix: buf for lane in (self._main, self._alter) for name, buf in lane.store.items()}

    # -- serial names -----------------------------------------------------------------------------------
    def get_incremental_name(self, name=None):
        """"<name>_<n>" with n = 0, 1, ... per name (utils.py:45-50)."""
        stem = "default" if name is None else name
        return f"{stem}_{next(self._serials.setdefault(stem, itertools.count()))}"

    def reset_incremental_names(self):
        self._serials = {}

    # -- skip-layer guidance ------------------------------------------------------------------------------
    def is_slg_enabled(self):
        return self.slg_layers is not None

    def slg_should_skip_block(self, block_idx):
        """Skip-layer guidance (utils.py:102-114) drops the listed blocks on the alternating pass while
        the running step lies in [slg_start, slg_end) of the schedule; a window that covers the whole
        schedule switches it off."""
        if not (self.enable_alter_cache and self._marks % 2 == 0) or self.slg_layers is None:
            return False
        if self.slg_start <= 0.0 and self.slg_end >= 1.0:
            return False
        assert self.num_inference_steps >= 0, "num_inference_steps must be non-negative"
        lo, hi = self.num_inference_steps * self.slg_start, self.num_inference_steps * self.slg_end
        return lo <= self.get_current_step() < hi and block_idx in self.slg_layers


# The context in force, innermost last.  set_current_cache_context() replaces the innermost one,
# cache_context() nests (src/para_attn/first_block_cache/utils.py:193-217: one module-wide context,
# not per thread).
_contexts = [None]


def create_cache_context(*args, **kwargs):
    return CacheContext(*args, **kwargs)


def get_current_cache_context():
    return _contexts[-1]


def set_current_cache_context(cache_context=None):
    _contexts[-1] = cache_context


@contextlib.contextmanager
def cache_context(cache_context):
    _contexts.append(cache_context)
    try:
        yield
    finally:
        _contexts.pop()


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
