"""TaylorSeer: cached residuals extrapolated along the denoising schedule, behind the class name and
method names of the reference (src/para_attn/first_block_cache/taylorseer.py:4-64).

The predictor keeps a *ladder*: rung 0 is the residual of the last fully computed step, rung i its
i-th backward finite difference.  A full step climbs the ladder as far as the previous ladder
reaches (one kernel for all rungs, ``para_attn::taylorseer_derivatives``); a skipped step evaluates
the truncated Taylor polynomial over the ladder (one kernel, ``para_attn::taylorseer_value``).  The
reference does the same arithmetic with one torch launch per operation.
"""
from . import ops

MAX_RUNGS = 4  # finite-difference orders the kernels take


class _Clock:
    """Step counter of one predictor: ``now`` is the running step (-1 before the first), ``anchor`` the
    last step whose value was computed in full."""

    __slots__ = ("now", "anchor")

    def __init__(self):
        self.now = -1
        self.anchor = -1

    @property
    def gap(self):
        return self.now - self.anchor


class TaylorSeer:
    def __init__(self, n_derivatives=2, warmup_steps=1, skip_interval_steps=1, compute_step_map=None):
        if n_derivatives > MAX_RUNGS:
            raise NotImplementedError(f"at most {MAX_RUNGS} finite-difference orders")
        self.n_derivatives = n_derivatives
        self.warmup_steps = warmup_steps
        self.skip_interval_steps = skip_interval_steps
        self.compute_step_map = compute_step_map
        self.reset_cache()

    # -- state -------------------------------------------------------------------------------------
    def reset_cache(self):
        self._clock = _Clock()
        self._ladder = ()       # rungs of the last full step, lowest order first, no gaps
        self._older = ()        # the ladder before that

    @property
    def ORDER(self):
        """Slots of the reference's state lists: the value plus ``n_derivatives`` differences."""
        return self.n_derivatives + 1

    @property
    def current_step(self):
        return self._clock.now

    @property
    def last_non_approximated_step(self):
        return self._clock.anchor

    @property
    def state(self):
        """The reference's view of the state (taylorseer.py:13-17): two lists of ORDER slots, empty
        slots as None.  Read-only; the ladders are what the predictor works on."""
        pad = lambda rungs: list(rungs) + [None] * (self.ORDER - len(rungs))  # noqa: E731
        return {"dY_prev": pad(self._older), "dY_current": pad(self._ladder)}

    # -- schedule ----------------------------------------------------------------------------------
    def should_compute_full(self, step=None):
        """Whether ``step`` (default: the running one) is computed in full (taylorseer.py:21-27): a step map
        decides alone if given; otherwise all warm-up steps and then every ``skip_interval_steps``-th."""
        at = self._clock.now if step is None else step
        if self.compute_step_map is not None:
            return self.compute_step_map[at]
        past_warmup = at - self.warmup_steps
        return past_warmup < 0 or (past_warmup + 1) % self.skip_interval_steps == 0

    def mark_step_begin(self):
        self._clock.now += 1

    # -- arithmetic --------------------------------------------------------------------------------
    def _climb(self, Y, below):
        """The ladder over the value ``Y`` with ``below`` as the older ladder (taylorseer.py:29-38): one rung
        per rung of ``below``, capped by ``n_derivatives``, and none before the third step; each rung is the
        difference to the rung below's older value over the steps since the anchor."""
        n = min(len(below), self.n_derivatives) if self._clock.now > 1 else 0
        if n == 0:
            return (Y,)
        return (Y, *ops.taylorseer_derivatives(Y, list(below[:n]), float(self._clock.gap)))

    def approximate_derivative(self, Y):
        """The ladder for ``Y`` against the older stored one, in the reference's padded list form."""
        rungs = self._climb(Y, self._older)
        return list(rungs) + [None] * (self.ORDER - len(rungs))

    def approximate_value(self):
        """Taylor polynomial over the ladder at the running step (taylorseer.py:40-48); the reference's
        empty sum, the integer 0, when nothing has been stored yet."""
        if not self._ladder:
            return 0
        return ops.taylorseer_value(list(self._ladder), self._clock.gap)

    def approximate_value_plus(self, hidden_states):
        """``approximate_value() + hidden_states`` in one pass (the cache-hit path of
        src/para_attn/first_block_cache/utils.py:239-243)."""
        return ops.taylorseer_value(list(self._ladder), self._clock.gap, hidden_states)

    # -- stepping ----------------------------------------------------------------------------------
    def update(self, Y):
        """Record a fully computed value: the current ladder becomes the older one, the new ladder is
        climbed against it, and the anchor moves to the running step (taylorseer.py:53-56)."""
        self._older = self._ladder
        self._ladder = self._climb(Y, self._older)
        self._clock.anchor = self._clock.now

    def step(self, Y):
        self.mark_step_begin()
        if not self.should_compute_full():
            return self.approximate_value()
        self.update(Y)
        return Y
